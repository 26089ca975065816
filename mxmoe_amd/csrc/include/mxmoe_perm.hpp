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

// Scatter step of the permutation of a larger batch: workgroup `block` of `blocks` places its kPermChunk entries.  `hist` holds the
// per-expert counts of every workgroup's chunk (perm_hist_kernel).  With `raw` false it is laid out [blocks][E] and a scan kernel has
// already turned the rows into exclusive prefixes over the workgroups and written the totals to `recv`; with `raw` true it is laid
// out [E][perm_hist_stride(blocks)] and still holds plain counts: every workgroup sums what it needs itself (the counts before it,
// and all counts for the experts' first rows; workgroup 0 also writes `recv`) with 16-byte loads along its experts' rows, which saves
// a launch as long as blocks * E is small (kPermFusedScanMax).
// Called by every thread of the workgroup; only the first wave (`active`) works, the others pass the barriers.
constexpr int kPermFusedScanMax = 16384;
// row length of the expert-major histogram: the workgroup count rounded up to whole 16-byte loads (the padding is never written and
// its contents are masked out by the readers)
__host__ __device__ __forceinline__ int perm_hist_stride(int blocks) { return (blocks + 3) & ~3; }
// sum of an expert's counts over all workgroups, and over the workgroups before `block`
__device__ __forceinline__ void perm_hist_row_sums(const int32_t* __restrict__ row, int blocks, int block, int* total, int* before) {
  typedef int v4i_t __attribute__((ext_vector_type(4)));
  const v4i_t* r4 = reinterpret_cast<const v4i_t*>(row);
  int v = 0, bf = 0;
  const int n4 = perm_hist_stride(blocks) >> 2;
#pragma unroll 16
  for (int j = 0; j < n4; ++j) {
    const v4i_t h = r4[j];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int b = 4 * j + i;
      v += b < blocks ? h[i] : 0;
      bf += b < block ? h[i] : 0;
    }
  }
  *total = v;
  *before = bf;
}
__device__ __forceinline__ void perm_scatter_body(const int32_t* __restrict__ ids, int total, int E, int topk, int nbits, const int32_t* __restrict__ hist, int blocks, int block,
                                                  bool raw, int64_t* __restrict__ recv, int32_t* __restrict__ dst_exp_sorted, int64_t* __restrict__ perm,
                                                  int64_t* __restrict__ src_slot, int32_t* __restrict__ row_of_slot, int32_t* run, bool active) {
  const int lane = threadIdx.x & 63;
  if (active) {  // first row of every expert = exclusive scan of the per-expert totals, plus this workgroup's offset inside the expert
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      int v = 0, before = 0;
      if (e < E) {
        if (raw) {
          perm_hist_row_sums(hist + (long)e * perm_hist_stride(blocks), blocks, block, &v, &before);
          if (block == 0) recv[e] = v;
        } else {
          v = (int)recv[e];
          before = hist[block * E + e];
        }
      }
      const int inc = wave_inclusive_scan(v, lane);
      if (e < E) run[e] = carry + inc - v + before;
      carry += __shfl(inc, 63);
    }
  }
  __syncthreads();
  const int base = block * kPermChunk;
  for (int i = 0; i < kPermChunk; i += 64) {  // sub-chunks in order keep the sort stable
    const int idx = base + i + lane;
    const bool ok = active && idx < total;
    int e = ok ? ids[idx] : -1;
    if (e < 0 || e >= E) e = E;  // parked on a dummy id, never written
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
    // the inverse map (sorted row of every (token, slot); -1 where the expert id was out of range), for the combine
    if (row_of_slot && ok) row_of_slot[idx] = e < E ? first + before : -1;
    __syncthreads();
  }
}

// perm_hist_kernel on `stream`: entries of expert e among the kPermChunk entries of workgroup b, at hist[b * E + e], or with
// `expert_major` at hist[e * perm_hist_stride(blocks) + b] (act_kernels.hip)
void launch_perm_hist(const int32_t* ids, int total, int E, int32_t* hist, bool expert_major, hipStream_t stream);

}  // namespace mxmoe
