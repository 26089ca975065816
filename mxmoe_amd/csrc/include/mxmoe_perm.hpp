// Pieces of the stable token permutation that more than one translation unit uses: the wave helpers and the single-workgroup
// permutation of decode-sized batches, which also runs as one workgroup of the launch that plans a layer's two GroupGEMMs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mxmoe {

constexpr int kPermChunk = 256;  // flattened (token, slot) entries per single-wave workgroup

// lanes of the wave that hold the same expert id as this lane (ids < 2^16)
__device__ __forceinline__ uint64_t match_same(int e, int nbits) {
  uint64_t m = ~0ull;
  for (int b = 0; b < nbits; ++b) {
    const uint64_t bal = __ballot((e >> b) & 1);
    m &= ((e >> b) & 1) ? bal : ~bal;
  }
  return m;
}

// inclusive scan of one value per lane across the wave
__device__ __forceinline__ int wave_inclusive_scan(int v, int lane) {
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(v, o);
    if (lane >= o) v += t;
  }
  return v;
}

// Stable permutation by expert of at most kPermChunk (token, slot) entries by the first wave of a workgroup: count, scan the experts,
// scatter (ref_bind.cu:47-64, 449-453 with a stable order).  `run` is LDS for E counters.  Every thread of the workgroup must call
// this (it holds workgroup barriers); threads with `active` false (the other waves of a wider workgroup) only pass the barriers.
__device__ __forceinline__ void perm_small_body(const int32_t* __restrict__ ids, int total, int E, int topk, int nbits, int64_t* __restrict__ recv,
                                                int32_t* __restrict__ dst_exp_sorted, int64_t* __restrict__ perm, int64_t* __restrict__ src_slot,
                                                int32_t* __restrict__ row_of_slot, int32_t* run, bool active) {
  const int lane = threadIdx.x & 63;
  if (active)
    for (int e = lane; e < E; e += 64) run[e] = 0;
  __syncthreads();
  if (active)
    for (int idx = lane; idx < total; idx += 64) {
      const int e = ids[idx];
      if (e >= 0 && e < E) atomicAdd(&run[e], 1);
    }
  __syncthreads();
  if (active) {
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const int v = e < E ? run[e] : 0;
      const int inc = wave_inclusive_scan(v, lane);
      if (e < E) {
        recv[e] = v;
        run[e] = carry + inc - v;
      }
      carry += __shfl(inc, 63);
    }
  }
  __syncthreads();
  for (int i = 0; i < total; i += 64) {  // sub-chunks in order keep the sort stable
    const int idx = i + lane;
    const bool ok = active && idx < total;
    int e = ok ? ids[idx] : -1;
    if (e < 0 || e >= E) e = E;
    const uint64_t same = match_same(e, nbits);
    const int before = __popcll(same & ((1ull << lane) - 1));
    int first = 0;
    if (e < E) first = run[e];
    __syncthreads();
    if (e < E) {
      const int pos = first + before;
      dst_exp_sorted[pos] = e;
      perm[pos] = idx / topk;
      if (src_slot) src_slot[pos] = idx;
      if (before == 0) run[e] = first + __popcll(same);
    }
    if (row_of_slot && ok) row_of_slot[idx] = e < E ? first + before : -1;
    __syncthreads();
  }
}

}  // namespace mxmoe
