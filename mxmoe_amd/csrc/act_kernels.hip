// Prologue kernels of the MoE layer on gfx950:
//   * stable token permutation by expert (histogram -> scan -> ranked scatter);
//   * gather + online Hadamard rotation + per-token quantisation + packing      (quant_act);
//   * SiLU(gate) * up + online Hadamard rotation + per-token quantisation + packing (silu_mul_then_quant).
//
// The reference launches `quant_act_kernel` / `silu_mul_then_quant_kernel` (mxmoe/kernels/src/ref_bind.cu:531-544,
// 701-716) whose source file (act_kernel.cuh) is absent from the reference; the contracts implemented here are the
// launch arguments and the host offset builder of ref_bind.cu:461-505, 635-671: one workgroup per destination row,
// rows grouped by expert, per-expert tag {0 fp16 copy, 1 int8, 2 int4, 3 int4 with a scale per 128 values}, row strides K, K/2, K/4 halves, one fp16
// scale per row.  The permutation replaces torch::sort + bincount of ref_bind.cu:47-64,449-453 with a STABLE order.
//
// Arithmetic is the exact operation sequence of the fp16 quantiser (mxmoe/quant/quant.py:68-84: absmax / upper,
// x / scale, clamp, round-half-even, all rounded to fp16) and of a fixed-order fp32 Hadamard transform, so integer
// codes are reproducible bit for bit on a CPU; this file must be compiled with FMA contraction off.
#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

#include <cmath>
#include <string>

#include "../../include/mxmoe_amd.h"
#include "include/mxmoe_launch.hpp"
#include "include/mxmoe_plan.hpp"
#include "include/mxmoe_perm.hpp"

namespace mxmoe {

// ------------------------------------------------------------------------------------------------------------
// Stable permutation by expert
// ------------------------------------------------------------------------------------------------------------

__global__ void __launch_bounds__(64) perm_hist_kernel(const int32_t* __restrict__ ids, int total, int E, int32_t* __restrict__ hist, int stride /*0: [blocks][E]; else [E][stride]*/) {
  extern __shared__ int32_t cnt[];
  for (int e = threadIdx.x; e < E; e += 64) cnt[e] = 0;
  __syncthreads();
  const int base = blockIdx.x * kPermChunk;
  for (int i = threadIdx.x; i < kPermChunk; i += 64) {
    const int idx = base + i;
    if (idx < total) {
      const int e = ids[idx];
      if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < E; e += 64) hist[stride ? (long)e * stride + blockIdx.x : (long)blockIdx.x * E + e] = cnt[e];
}

// one single-wave workgroup per expert: exclusive scan of the expert's per-block counts (64 blocks per step); total -> recv
__global__ void __launch_bounds__(64) perm_scan_kernel(int32_t* __restrict__ hist, int blocks, int E, int64_t* __restrict__ recv) {
  const int e = blockIdx.x, lane = threadIdx.x;
  int carry = 0;
  for (int b0 = 0; b0 < blocks; b0 += 64) {
    const int b = b0 + lane;
    const int v = b < blocks ? hist[b * E + e] : 0;
    const int inc = wave_inclusive_scan(v, lane);
    if (b < blocks) hist[b * E + e] = carry + inc - v;
    carry += __shfl(inc, 63);
  }
  if (lane == 0) recv[e] = carry;
}

__global__ void __launch_bounds__(64) perm_scatter_kernel(const int32_t* __restrict__ ids, int total, int E, int topk, int nbits, const int32_t* __restrict__ hist,
                                                          int raw, int64_t* __restrict__ recv, int32_t* __restrict__ dst_exp_sorted, int64_t* __restrict__ perm,
                                                          int64_t* __restrict__ src_slot, int32_t* __restrict__ row_of_slot) {
  extern __shared__ int32_t run[];  // next free rank per expert for this block
  perm_scatter_body(ids, total, E, topk, nbits, hist, (int)gridDim.x, (int)blockIdx.x, raw != 0, recv, dst_exp_sorted, perm, src_slot, row_of_slot, run, true);
}

void launch_perm_hist(const int32_t* ids, int total, int E, int32_t* hist, bool expert_major, hipStream_t stream) {
  const int blocks = (total + kPermChunk - 1) / kPermChunk;
  hipLaunchKernelGGL(perm_hist_kernel, dim3(blocks), dim3(64), (size_t)E * sizeof(int32_t), stream, ids, total, E, hist, expert_major ? perm_hist_stride(blocks) : 0);
}

// The three kernels above in one, for at most kPermChunk (token, slot) entries (decode-sized batches): one single-wave workgroup
// counts, scans the experts and scatters, where three launches would cost more than their work (body: mxmoe_perm.hpp).
__global__ void __launch_bounds__(64) perm_small_kernel(const int32_t* __restrict__ ids, int total, int E, int topk, int nbits, int64_t* __restrict__ recv,
                                                        int32_t* __restrict__ dst_exp_sorted, int64_t* __restrict__ perm, int64_t* __restrict__ src_slot,
                                                        int32_t* __restrict__ row_of_slot) {
  extern __shared__ int32_t run[];  // [E] counts, then next free rank per expert
  perm_small_body(ids, total, E, topk, nbits, recv, dst_exp_sorted, perm, src_slot, row_of_slot, run, true);
}

// ------------------------------------------------------------------------------------------------------------
// Routing: router logits -> (top-k expert ids, top-k weights)
// ------------------------------------------------------------------------------------------------------------
// What the models' gates compute in front of the layer (mxmoe/quant/moe_tracer.py:79-86: softmax over the experts in fp32, top-k of
// the probabilities, optionally divided by their sum).  One wave per token, four tokens per workgroup; a token's probabilities sit in
// the wave's slice of LDS (entry e belongs to lane e mod 64: no lane reads what another wrote), and every one of the k rounds takes
// the largest remaining (probability, lowest index first) by a wave-wide maximum of a 64-bit key.
struct RouteArgs {
  const void* logits;  // [T][E]
  int dtype;           // 0 fp16, 1 fp32, 2 bf16
  int T, E, topk, renorm;
  int32_t* ids;        // [T][topk]
  float* weights;      // [T][topk]
};

__device__ __forceinline__ float route_logit(const RouteArgs& a, long i) {
  if (a.dtype == 1) return reinterpret_cast<const float*>(a.logits)[i];
  if (a.dtype == 0) return (float)reinterpret_cast<const _Float16*>(a.logits)[i];
  return __uint_as_float((unsigned)reinterpret_cast<const uint16_t*>(a.logits)[i] << 16);
}

__global__ void __launch_bounds__(256) route_topk_kernel(const RouteArgs a) {
  extern __shared__ float route_lds[];  // [4][E]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int t = blockIdx.x * 4 + wave;
  if (t >= a.T) return;  // (no workgroup barrier below)
  float* p = route_lds + wave * a.E;
  const long base = (long)t * a.E;
  float mx = -INFINITY;
  for (int e = lane; e < a.E; e += 64) {
    const float x = route_logit(a, base + e);
    p[e] = x;
    mx = fmaxf(mx, x);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  float sum = 0.0f;
  for (int e = lane; e < a.E; e += 64) {
    const float v = expf(p[e] - mx);
    p[e] = v;
    sum += v;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
  for (int e = lane; e < a.E; e += 64) p[e] = p[e] / sum;
  int my_id = 0;
  float my_w = 0.0f, wsum = 0.0f;
  for (int r = 0; r < a.topk; ++r) {
    // key = (probability bits, ~index): probabilities are not negative, so their bit patterns order like the values (a NaN sorts
    // above every number); a taken entry holds -1 and gets the key 0, which loses against every live entry
    unsigned long long key = 0;
    for (int e = lane; e < a.E; e += 64) {
      const float v = p[e];
      const unsigned long long k = v == -1.0f ? 0ull : ((unsigned long long)(__float_as_uint(v) & 0x7FFFFFFFu) << 32) | (0xFFFFFFFFu - (unsigned)e);
      key = k > key ? k : key;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const unsigned lo = __shfl_xor((unsigned)key, o), hi = __shfl_xor((unsigned)(key >> 32), o);
      const unsigned long long other = ((unsigned long long)hi << 32) | lo;
      key = other > key ? other : key;
    }
    const int idx = (int)(0xFFFFFFFFu - (unsigned)key);
    const float val = p[idx];  // (read before the owner's write below: the same value for every lane)
    __builtin_amdgcn_wave_barrier();
    if ((idx & 63) == lane) p[idx] = -1.0f;
    __builtin_amdgcn_wave_barrier();
    wsum += val;
    if (lane == r) {
      my_id = idx;
      my_w = val;
    }
  }
  if (lane < a.topk) {
    a.ids[(long)t * a.topk + lane] = my_id;
    a.weights[(long)t * a.topk + lane] = a.renorm ? my_w / wsum : my_w;
  }
}

// ------------------------------------------------------------------------------------------------------------
// Row kernels
// ------------------------------------------------------------------------------------------------------------
struct RotPlan {
  int n;        // row length
  int m;        // length of the Sylvester part (n = K * m), power of two >= 8
  int f;        // H_K = S_f kron B
  int kb;       // order of B (1 when K == 1)
  float scale;  // 1 / sqrt(n), computed in fp32 on the host
};

struct RowArgs {
  const _Float16* src;
  const _Float16* src_shared;
  uint8_t* inp_store;
  _Float16* scale_store;
  const int32_t* dst_exp;
  const int64_t* perm;
  const int64_t* table;  // [4][Et]: tag, start_row, inp_off, scale_off (offsets in fp16 elements)
  const float* signs;    // B as +-1.0f, [kb][kb], or null
  int R, T, E, Et;
  int rows;
  int rotate;  // 0 never, 1 rows of quantised experts, 2 every row
  RotPlan plan, plan_shared;
  // Planned mode (the tables were written by the device-side planner, the host never saw the counts): R is then the CAPACITY of the
  // routed part (tokens x top-k), rows routed .. R-1 do not exist when expert ids were dropped, and the shared expert's source rows
  // are wherever the planner put them.  Both null otherwise.
  const int64_t* routed_ptr;       // rows that were routed
  const int64_t* shared_src_addr;  // address of the shared expert's source rows
};

// rows [routed, R) of a planned launch do not exist
__device__ __forceinline__ bool row_exists(const RowArgs& a, int row) { return !a.routed_ptr || row >= a.R || row < (int)*a.routed_ptr; }
__device__ __forceinline__ const _Float16* shared_src(const RowArgs& a) {
  return a.shared_src_addr ? reinterpret_cast<const _Float16*>(*a.shared_src_addr) : a.src_shared;
}
// Load of a value that no kernel of this launch writes (routing arrays, expert table), through the constant address space: with a
// wave-uniform address it is a scalar load into scalar registers, off the vector register budget.
template <class T>
__device__ __forceinline__ T const_load(const T* p) {
  return *(const __attribute__((address_space(4))) T*)(p);
}

// silu(g) = g / (1 + exp(-g)) as a fixed sequence of correctly rounded fp32 operations and exact integer ones, identical to the CPU
// restatement (every multiply-add is fused: one rounding): exp(-g) = 2^t with t = clamp(-g log2(e), +-100) split into k = rint(t) and
// f = t - k (exact), 2^f by a degree-4 Horner polynomial (relative error 3.7e-6), 2^k added to the exponent field (the result stays a
// normal number); the reciprocal of d = 1 + exp(-g) from an integer-subtraction seed (within 5.06 %) and two Newton steps (7e-6).
// silu(g) * u rounded to fp16 lies within 0.52 fp16 ulp of the exact value for every fp16 g.
__device__ __forceinline__ float silu_fixed(float g) {
  float t = g * -1.4426950408889634f;
  t = fminf(fmaxf(t, -100.0f), 100.0f);
  const float k = rintf(t);
  const float f = t - k;
  float p = 0.00967604f;
  p = __builtin_fmaf(p, f, 0.05592204f);
  p = __builtin_fmaf(p, f, 0.24022107f);
  p = __builtin_fmaf(p, f, 0.693121f);
  p = __builtin_fmaf(p, f, 1.0000001f);
  const float e = __int_as_float(__float_as_int(p) + (int)((unsigned)(int)k << 23));
  const float d = 1.0f + e;
  float r = __int_as_float(0x7EF31000 - __float_as_int(d));
  r = __builtin_fmaf(r, __builtin_fmaf(-d, r, 1.0f), r);
  r = __builtin_fmaf(r, __builtin_fmaf(-d, r, 1.0f), r);
  return g * r;
}

__device__ __forceinline__ float round_h(float v) { return (float)(_Float16)v; }

// Integer code of a value already clamped to the code range, as the low bits of a word: the addition of 1.5 * 2^23 rounds to an
// integer by itself (to nearest, ties to even: rintf) and leaves its two's complement in the low mantissa bits.  push_code<BITS>
// shifts a word of codes right by BITS and puts the new code on top: after 32 / BITS pushes the first code sits in the lowest bits.
__device__ __forceinline__ unsigned code_word(float clamped) { return __float_as_uint(clamped + 12582912.0f); }
template <int BITS>
__device__ __forceinline__ unsigned push_code(unsigned w, unsigned code) {
  return __builtin_amdgcn_alignbit(code, w, BITS);
}

// v / s in fp32 for fp16-valued v and s, given r = 1.0f / s: the rounded product v * r corrected once with its exact remainder.
// With r the correctly rounded reciprocal this is the correctly rounded quotient, i.e. bit for bit what the division instruction
// sequence returns, for every pair of fp16 values (checked with exact integer arithmetic over all 2^20 mantissa pairs in
// tests/test_oracle_quant.py); a row's elements share one scale, so the division proper is done once per row.
// An infinite scale (a row that already holds an infinity) keeps the plain result: finite / inf = 0.
struct ScaleDiv {
  float r, s;
  __device__ __forceinline__ explicit ScaleDiv(float scale) : r(1.0f / scale), s(__builtin_isinf(scale) ? 0.0f : scale) {}
  __device__ __forceinline__ float operator()(float v) const {
    const float q0 = v * r;
    const float e = __builtin_fmaf(-s, q0, v);
    return __builtin_fmaf(e, r, q0);
  }
};

// Power-of-two factors of the dense stage of the non-power-of-two rotations for a row whose largest magnitude is mx (an fp16
// value held in fp32): with mx < 2^E, to_grid = 2^(17-E) turns the row into integers of magnitude <= 2^17 and from_grid = 2^(E-17)
// turns sums of them back.  Taken from the exponent field of mx; an all-zero row gets 1 and 1.
struct DenseGrid {
  float to_grid, from_grid;
  __device__ __forceinline__ explicit DenseGrid(float mx) {
    const int e_field = __float_as_int(mx) >> 23;  // mx >= 0
    to_grid = e_field == 0 ? 1.0f : __int_as_float((270 - e_field) << 23);
    from_grid = e_field == 0 ? 1.0f : __int_as_float(max(e_field - 16, 1) << 23);
  }
};

// Value of lane (l ^ M).  Distances 1 .. 8 stay inside a row of 16 lanes and are data-parallel-primitive moves in the vector ALU
// (quad permutations; l ^ 4 = mirror of 8 lanes, then of 4; l ^ 8 = a rotation of the row by 8); 16 and 32 go through the LDS
// crossbar, whose throughput is what bounds this kernel once the arithmetic is trimmed.
template <int M>
__device__ __forceinline__ float lane_xor(float v) {
  int x = __float_as_int(v);
  if constexpr (M == 1) {
    x = __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
  } else if constexpr (M == 2) {
    x = __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
  } else if constexpr (M == 4) {
    x = __builtin_amdgcn_update_dpp(0, x, 0x141, 0xF, 0xF, true);  // row_half_mirror: l ^ 7
    x = __builtin_amdgcn_update_dpp(0, x, 0x1B, 0xF, 0xF, true);   // quad_perm [3,2,1,0]: l ^ 3
  } else if constexpr (M == 8) {
    x = __builtin_amdgcn_update_dpp(0, x, 0x128, 0xF, 0xF, true);  // row_ror:8: lane (l + 8) mod 16 = l ^ 8
  } else {
    return __shfl_xor(v, M);
  }
  return __int_as_float(x);
}

// ---- tag 4: per-token int4 codes written as bf6 fragments, the operand layout of the w4a4 tiles on the 6-bit float matrix path
// (mxmoe_bf6_tiles.hpp).  Scale and codes are those of tag 2; only the storage differs: an expert's region holds ceil(rows / 32) row
// blocks of n / 64 fragments of 1536 bytes, row block major, and local row r of the expert is lane (r % 32) + 32 (k half) of its
// block's fragments.  Every row kernel leaves the row's codes in LDS as fp16 integers in natural order; a thread then turns 32
// consecutive codes into one lane's 192 bits with one conversion instruction and stores them as 16 + 8 bytes.
typedef _Float16 v32h __attribute__((ext_vector_type(32)));
typedef unsigned v6u __attribute__((ext_vector_type(6)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef unsigned v2u __attribute__((ext_vector_type(2)));

// the eight codes of a chunk: v / scale rounded to fp16, clamped to +-7, rounded to the nearest integer (ties to even)
template <class Div>
__device__ __forceinline__ v8h bf6_chunk_codes(const float (&v)[8], const Div& div) {
  v8h o;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = (_Float16)rintf(fminf(fmaxf(round_h(div(v[j])), -7.0f), 7.0f));
  return o;
}

// ---- tag 5: per-token fp8 (OCP e4m3) codes for the kernels whose w8a8 tiles run the fp8 matrix instruction.  scale = max|x| / 448
// (the largest e4m3 number) in fp16 like the integer scales; code = e4m3(clamp(fp16(x / scale), +-448)), round to nearest even; rows
// are stored like int8 rows, one byte per value.
template <class Div>
__device__ __forceinline__ uint2 fp8_chunk_codes(const float (&v)[8], const Div& div) {
  float r[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = fminf(fmaxf(round_h(div(v[j])), -448.0f), 448.0f);
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(r[0], r[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(r[2], r[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(r[4], r[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(r[6], r[7], hi, true);
  return make_uint2((unsigned)lo, (unsigned)hi);
}

// Codes of one row in LDS (fp16; value k at byte (k / row_elems) * pitch + (k % row_elems) * 2) -> the row's place in its expert's
// fragment region.  Thread t of nt takes the groups of 32 codes t, t + nt, ...
__device__ __forceinline__ void bf6_emit_row(const uint8_t* codes, int row_elems, int pitch, int n, uint8_t* region, long lrow, int t, int nt) {
  const int KS = n >> 6;
  uint8_t* blk = region + (lrow >> 5) * (long)KS * kBf6Frag;
  const int r = (int)(lrow & 31);
  for (int hf = t; hf < (n >> 5); hf += nt) {
    const int k0 = hf << 5;
    const uint8_t* src = codes + (k0 / row_elems) * pitch + (k0 % row_elems) * 2;
    v32h c;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v8h part = *reinterpret_cast<const v8h*>(src + q * 16);
#pragma unroll
      for (int j = 0; j < 8; ++j) c[q * 8 + j] = part[j];
    }
    const v6u w = __builtin_amdgcn_cvt_scalef32_pk32_bf6_f16(c, 1.0f);
    uint8_t* frag = blk + (hf >> 1) * kBf6Frag;
    const int l = ((hf & 1) << 5) | r;
    gstore<v4u>(frag + 16 * l, v4u{w[0], w[1], w[2], w[3]});
    gstore<v2u>(frag + 1024 + 8 * l, v2u{w[4], w[5]});
  }
}

// Workgroup -> group of four rows for the kernels that run one row per wave: the eight workgroups that share an XCD (workgroup id
// modulo 8) within a run of 64 take eight consecutive groups, i.e. 32 consecutive rows.  Rows of one 32-row block of a fragment
// region share cache lines (16 or 8 bytes per row side by side); written through one L2 they leave it as whole lines.  Needs a grid
// that is a multiple of 64.
__device__ __forceinline__ int xcd_row_group(int wg) { return (wg & ~63) | ((wg & 7) << 3) | ((wg >> 3) & 7); }

// NT threads per workgroup (256, or 192 when that wastes fewer lanes: a 1408-element row is 176 chunks of 8).
template <int MAXC, bool SILU, int NT, bool EXT>
__global__ void __launch_bounds__(NT) row_quant_kernel(const RowArgs a) {
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x;
  const int nmax = max(a.plan.n, a.plan_shared.n);
  float* x = lds;                  // [nmax]
  float* sg = lds + nmax;          // [kb*kb]
  float* red = sg + a.plan.kb * a.plan.kb;  // [16]: one slot per wave
  // A chunk of 8 values lives in two planes of 16 bytes (values 0-3, values 4-7): consecutive lanes then touch consecutive 16-byte
  // words and a wave's 128-bit accesses spread over all banks (32-byte lane strides would hit every bank twice).
  float4* xlo = reinterpret_cast<float4*>(x);
  float4* xhi = xlo + (nmax >> 3);
  auto put = [&](int c, const float (&w)[8]) {
    xlo[c] = make_float4(w[0], w[1], w[2], w[3]);
    xhi[c] = make_float4(w[4], w[5], w[6], w[7]);
  };
  auto get = [&](int c, float (&w)[8]) {
    const float4 l = xlo[c], h = xhi[c];
    w[0] = l.x; w[1] = l.y; w[2] = l.z; w[3] = l.w;
    w[4] = h.x; w[5] = h.y; w[6] = h.z; w[7] = h.w;
  };
  if (a.signs) {
    for (int i = tid; i < a.plan.kb * a.plan.kb; i += NT) sg[i] = a.signs[i];
  }

  // Row bookkeeping (expert, tag, offsets, source pointer) and the row's data are fetched one row ahead: each is a chain of
  // dependent global loads, several microseconds long, that must not sit in front of every row's arithmetic.
  struct RowMeta {
    int e, tag;
    long start_row, inp_off, scale_off;
    const _Float16* srow;
    bool shared_row, exists;
  };
  const _Float16* const src_shared = shared_src(a);
  auto load_meta = [&](int row) {
    RowMeta m;
    m.shared_row = row >= a.R;
    m.exists = row_exists(a, row);
    m.e = m.shared_row ? a.E : (m.exists ? a.dst_exp[row] : 0);
    m.tag = (int)a.table[m.e];
    m.start_row = a.table[a.Et + m.e];
    m.inp_off = a.table[2 * a.Et + m.e];
    m.scale_off = a.table[3 * a.Et + m.e];
    const int n = (m.shared_row ? a.plan_shared : a.plan).n;
    if (SILU) {
      m.srow = m.shared_row ? src_shared + (long)(row - a.R) * 2 * n : a.src + (long)row * 2 * n;
    } else {
      m.srow = (m.shared_row ? src_shared : a.src) + (m.shared_row ? (long)(row - a.R) : (m.exists ? (long)a.perm[row] : 0l)) * n;
    }
    return m;
  };
  auto load_data = [&](const RowMeta& m, v8h (&g)[MAXC], v8h (&u)[MAXC]) {
    const int n = (m.shared_row ? a.plan_shared : a.plan).n;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = tid + i * NT;
      if (c < (n >> 3)) {
        g[i] = *reinterpret_cast<const v8h*>(m.srow + c * 8);
        if (SILU) u[i] = *reinterpret_cast<const v8h*>(m.srow + n + c * 8);
      }
    }
  };
  RowMeta next_meta;
  v8h next_g[MAXC], next_u[MAXC];
  if ((int)blockIdx.x < a.rows) {
    next_meta = load_meta(blockIdx.x);
    load_data(next_meta, next_g, next_u);
  }

  for (int row = blockIdx.x; row < a.rows; row += gridDim.x) {
    const RowMeta cur = next_meta;
    v8h cur_g[MAXC], cur_u[MAXC];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      cur_g[i] = next_g[i];
      if (SILU) cur_u[i] = next_u[i];
    }
    if (row + (int)gridDim.x < a.rows) {
      next_meta = load_meta(row + gridDim.x);
      load_data(next_meta, next_g, next_u);
    }
    if (!cur.exists) continue;  // (the whole workgroup: a row belongs to one workgroup)
    const bool shared_row = cur.shared_row;
    const RotPlan pl = shared_row ? a.plan_shared : a.plan;
    const int n = pl.n;
    const int nchunks = n >> 3;
    const int tag = cur.tag;
    const long inp_off = cur.inp_off;
    const long scale_off = cur.scale_off;
    const long lrow = shared_row ? row - a.R : row - cur.start_row;  // (the shared expert's first row is R only when every row was routed)
    const bool rot = a.rotate == 2 || (a.rotate == 1 && tag != 0);

    float v[MAXC][8];
    __syncthreads();  // previous row fully consumed (and the sign table staged)
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = tid + i * NT;
      if (c < nchunks) {
        const v8h g = cur_g[i];
        if (SILU) {
          const v8h u = cur_u[i];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float gf = (float)g[j];
            const float s = silu_fixed(gf);
            v[i][j] = round_h(keep_f32(s * (float)u[j]));
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) v[i][j] = (float)g[j];
        }
        if (rot) {
          // Sylvester strides 1, 2, 4 inside the chunk
#pragma unroll
          for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              if (!(j & h)) {
                const float p = v[i][j], q = v[i][j + h];
                v[i][j] = p + q;
                v[i][j + h] = p - q;
              }
            }
          }
          put(c, v[i]);
        }
      }
    }

    if (rot) {
      // Sylvester strides 8 .. m/2 through LDS (ascending)
      bool lds_stale = false;  // registers ahead of the copy in LDS
      for (int h = 8; h < pl.m; h <<= 1) {
        const int hc = h >> 3;
        if (hc < 64) {
          // the partner chunk c ^ hc sits in the same wave, hc lanes away (NT is a multiple of 64): exchange in registers
          const float sgn = (tid & hc) ? -1.0f : 1.0f;
          auto stage = [&](auto mc) {
#pragma unroll
            for (int i = 0; i < MAXC; ++i)
#pragma unroll
              for (int j = 0; j < 8; ++j) v[i][j] = __builtin_fmaf(sgn, v[i][j], lane_xor<decltype(mc)::value>(v[i][j]));
          };
          switch (hc) {
            case 1: stage(std::integral_constant<int, 1>{}); break;
            case 2: stage(std::integral_constant<int, 2>{}); break;
            case 4: stage(std::integral_constant<int, 4>{}); break;
            case 8: stage(std::integral_constant<int, 8>{}); break;
            case 16: stage(std::integral_constant<int, 16>{}); break;
            default: stage(std::integral_constant<int, 32>{}); break;
          }
          lds_stale = true;
          continue;
        }
        if (lds_stale) {  // every thread rewrites its own chunks only, which nobody reads before the barrier below
#pragma unroll
          for (int i = 0; i < MAXC; ++i) {
            const int c = tid + i * NT;
            if (c < nchunks) put(c, v[i]);
          }
          lds_stale = false;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          const int c = tid + i * NT;
          if (c < nchunks) {
            float o[8];
            get(c ^ hc, o);
            const float sgn = (c & hc) ? -1.0f : 1.0f;  // upper half of a pair: other - own, lower half: own + other
#pragma unroll
            for (int j = 0; j < 8; ++j) v[i][j] = __builtin_fmaf(sgn, v[i][j], o[j]);  // +-own is exact, so this is the plain sum / difference
          }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          const int c = tid + i * NT;
          if (c < nchunks) {
            put(c, v[i]);
          }
        }
      }
      // scale, round to fp16
#pragma unroll
      for (int i = 0; i < MAXC; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = round_h(keep_f32(v[i][j] * pl.scale));

      if (pl.kb > 1) {
        const int mc = pl.m >> 3;  // chunks per k row
        // snap the row to the grid of step 2^(E-17), max|v| < 2^E: the sums of the dense stage are then sums of integers below
        // 2^17, exact in fp32 in any order
        float mx = 0.0f;
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          if (tid + i * NT < nchunks) {
#pragma unroll
            for (int j = 0; j < 8; ++j) mx = fmaxf(mx, fabsf(v[i][j]));
          }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        if ((tid & 63) == 0) red[tid >> 6] = mx;
        __syncthreads();
        mx = red[0];
#pragma unroll
        for (int w = 1; w < NT / 64; ++w) mx = fmaxf(mx, red[w]);
        const DenseGrid grid(mx);
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          const int c = tid + i * NT;
          if (c < nchunks) {
#pragma unroll
            for (int j = 0; j < 8; ++j) v[i][j] = rintf(v[i][j] * grid.to_grid);
            put(c, v[i]);
          }
        }
        __syncthreads();
        // dense B stage: t[b] = sum_{b'} B[b][b'] v[b'], b' ascending, starting from 0
#pragma unroll
        for (int i = 0; i < MAXC; ++i) {
          const int c = tid + i * NT;
          if (c < nchunks) {
            const int k = c / mc, jc = c - k * mc;
            const int blk = k / pl.kb, b = k - blk * pl.kb;
            const int vb = blk * pl.kb * mc + jc;
            const float* sr = sg + b * pl.kb;
            float acc[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
            for (int bp = 0; bp < pl.kb; ++bp) {
              const float s = sr[bp];
              float vv[8];
              get(vb + bp * mc, vv);
#pragma unroll
              for (int j = 0; j < 8; ++j) acc[j] = __builtin_fmaf(s, vv[j], acc[j]);  // s = +-1: the product is exact, so this is acc + s*v
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) v[i][j] = acc[j] * grid.from_grid;  // exact: an integer below 2^24 times a power of two
          }
        }
        // S_f butterflies across blocks of kb rows (ascending)
        for (int hh = 1; hh < pl.f; hh <<= 1) {
          const int hc = hh * pl.kb * mc;
          __syncthreads();
#pragma unroll
          for (int i = 0; i < MAXC; ++i) {
            const int c = tid + i * NT;
            if (c < nchunks) {
              put(c, v[i]);
            }
          }
          __syncthreads();
#pragma unroll
          for (int i = 0; i < MAXC; ++i) {
            const int c = tid + i * NT;
            if (c < nchunks) {
              const bool upper = ((c / (pl.kb * mc)) & hh) != 0;
              float o[8];
              get(upper ? c - hc : c + hc, o);
              const float sgn = upper ? -1.0f : 1.0f;
#pragma unroll
              for (int j = 0; j < 8; ++j) v[i][j] = __builtin_fmaf(sgn, v[i][j], o[j]);
            }
          }
        }
#pragma unroll
        for (int i = 0; i < MAXC; ++i)
#pragma unroll
          for (int j = 0; j < 8; ++j) v[i][j] = round_h(v[i][j]);
      }
    }

    // ---- store: fp16 copy or per-token symmetric quantisation ----
    if (tag == 0) {
      _Float16* out = reinterpret_cast<_Float16*>(a.inp_store) + inp_off + lrow * n;
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * NT;
        if (c < nchunks) {
          v8h o;
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = (_Float16)v[i][j];
          *reinterpret_cast<v8h*>(out + c * 8) = o;
        }
      }
      continue;
    }
    if (tag == 3) {
      // int4 with one scale per 128 values: a group is 16 consecutive chunks, i.e. the 16 lanes of an aligned lane group (the chunk
      // index and the lane index agree modulo 16), so its absmax is a 4-step exchange inside those lanes.  Row: n / 2 bytes of codes,
      // n / 128 scales.
      uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (n / 4));
      _Float16* sout = a.scale_store + scale_off + lrow * (n >> 7);
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * NT;
        const bool live = c < nchunks;  // whole lane groups are live or not: n is a multiple of 128
        float gmax = 0.0f;
        if (live) {
#pragma unroll
          for (int j = 0; j < 8; ++j) gmax = fmaxf(gmax, fabsf(v[i][j]));
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o));
        float scale = round_h(gmax / 7.0f);
        if (scale == 0.0f) scale = 1.0f;
        const ScaleDiv div(scale);
        if (live) {
          if ((c & 15) == 0) sout[c >> 4] = (_Float16)scale;
          unsigned w = 0;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float r = round_h(div(v[i][j]));
            w = push_code<4>(w, code_word(fminf(fmaxf(r, -7.0f), 7.0f)));
          }
          *reinterpret_cast<unsigned*>(out + c * 4) = w;
        }
      }
      continue;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = tid + i * NT;
      if (c < nchunks) {
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = red[0];
#pragma unroll
    for (int w = 1; w < NT / 64; ++w) amax = fmaxf(amax, red[w]);
    const float upper = tag == 1 ? 127.0f : (EXT && tag == 5 ? 448.0f : 7.0f);
    float scale = round_h(amax / upper);   // fp16 division: fp32 quotient of two fp16 values, rounded to fp16
    if (scale == 0.0f) scale = 1.0f;       // quantize.cuh:258
    const ScaleDiv div(scale);
    if (tid == 0) a.scale_store[scale_off + lrow] = (_Float16)scale;
    if (EXT && tag == 4) {  // the row's codes as fp16 in LDS (in place of the row itself, which every thread is done reading), then fragments
      uint8_t* codes = reinterpret_cast<uint8_t*>(x);
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = tid + i * NT;
        if (c < nchunks) *reinterpret_cast<v8h*>(codes + c * 16) = bf6_chunk_codes(v[i], div);
      }
      __syncthreads();
      bf6_emit_row(codes, n, 0, n, a.inp_store + 2 * inp_off, lrow, tid, NT);
      continue;  // (the next row begins with a barrier before it touches LDS)
    }
    uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (tag == 1 || (EXT && tag == 5) ? n / 2 : n / 4));
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = tid + i * NT;
      if (c < nchunks) {
        if (EXT && tag == 5) {
          *reinterpret_cast<uint2*>(out + c * 8) = fp8_chunk_codes(v[i], div);
          continue;
        }
        unsigned q[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float r = round_h(div(v[i][j]));
          q[j] = code_word(fminf(fmaxf(r, -upper), upper));
        }
        if (tag == 1) {
          uint2 w{0, 0};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            w.x = push_code<8>(w.x, q[j]);
            w.y = push_code<8>(w.y, q[j + 4]);
          }
          *reinterpret_cast<uint2*>(out + c * 8) = w;
        } else {
          unsigned w = 0;
#pragma unroll
          for (int j = 0; j < 8; ++j) w = push_code<4>(w, q[j]);
          *reinterpret_cast<unsigned*>(out + c * 4) = w;
        }
      }
    }
  }
}

// H_n x * scale for a row of n = 512 * NI values held by one wave (lane l: the NI chunks l + 64 i of 8 values), every level rounded
// to fp32 in ascending order of stride and the scaled result rounded to fp16: strides 1, 2, 4 inside a chunk, 8 .. 256 across
// lanes, 512 and up across the chunks of a lane.
template <int NI>
__device__ __forceinline__ void wave_rotate(float (&v)[NI][8], int lane, float scale) {
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int h = 1; h < 8; h <<= 1)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (!(j & h)) {
          const float p = v[i][j], q = v[i][j + h];
          v[i][j] = p + q;
          v[i][j + h] = p - q;
        }
  auto lane_stage = [&](auto mc) {
    constexpr int m = decltype(mc)::value;
    // upper half of a pair: other - own, lower half: own + other; one fused multiply-add with own's sign, which rounds once
    // exactly like the sum / difference (the product with +-1 is exact)
    const float sgn = (lane & m) ? -1.0f : 1.0f;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) v[i][j] = __builtin_fmaf(sgn, v[i][j], lane_xor<m>(v[i][j]));
  };
  lane_stage(std::integral_constant<int, 1>{});
  lane_stage(std::integral_constant<int, 2>{});
  lane_stage(std::integral_constant<int, 4>{});
  lane_stage(std::integral_constant<int, 8>{});
  lane_stage(std::integral_constant<int, 16>{});
  lane_stage(std::integral_constant<int, 32>{});
#pragma unroll
  for (int hi = 1; hi < NI; hi <<= 1)
#pragma unroll
    for (int i = 0; i < NI; ++i)
      if (!(i & hi)) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float p = v[i][j], q = v[i + hi][j];
          v[i][j] = p + q;
          v[i + hi][j] = p - q;
        }
      }
#pragma unroll
  for (int i = 0; i < NI; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) v[i][j] = round_h(keep_f32(v[i][j] * scale));
}

// One row per WAVE, for rows whose rotation is a pure Sylvester transform (n = 512 * NI, NI a power of two): lane l holds the NI
// 8-element chunks l + 64*i.  The butterfly strides map to three levels, taken in the same ascending order as everywhere else:
// 1, 2, 4 inside a chunk (registers), 8 .. 256 across the lanes (cross-lane exchange, no LDS staging, no barrier),
// 512 .. n/2 between a lane's own chunks (registers).  Four independent rows per workgroup, nothing shared between them.
template <int NI, bool SILU, bool EXT>
__global__ void __launch_bounds__(256) row_quant_wave_kernel(const RowArgs a) {
  extern __shared__ __align__(16) uint8_t wave_codes[];  // [4 waves][n] fp16: a row's codes on their way to bf6 fragments (tag 4)
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n = a.plan.n;  // == a.plan_shared.n == 512 * NI
  const int stride_rows = gridDim.x * 4;
  const _Float16* const src_shared = shared_src(a);
  for (int row = xcd_row_group(blockIdx.x) * 4 + wave; row < a.rows; row += stride_rows) {
    if (!row_exists(a, row)) continue;
    const bool shared_row = row >= a.R;
    const int e = shared_row ? a.E : a.dst_exp[row];
    const int tag = (int)a.table[e];
    const long lrow = shared_row ? row - a.R : row - a.table[a.Et + e];
    const long inp_off = a.table[2 * a.Et + e];
    const long scale_off = a.table[3 * a.Et + e];
    const bool rot = a.rotate == 2 || (a.rotate == 1 && tag != 0);
    const _Float16* srow;
    if (SILU) {
      srow = shared_row ? src_shared + (long)(row - a.R) * 2 * n : a.src + (long)row * 2 * n;
    } else {
      srow = (shared_row ? src_shared : a.src) + (shared_row ? (long)(row - a.R) : (long)a.perm[row]) * n;
    }
    float v[NI][8];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int c = lane + 64 * i;
      const v8h g = *reinterpret_cast<const v8h*>(srow + c * 8);
      if (SILU) {
        const v8h u = *reinterpret_cast<const v8h*>(srow + n + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float gf = (float)g[j];
          const float s = silu_fixed(gf);
          v[i][j] = round_h(keep_f32(s * (float)u[j]));
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = (float)g[j];
      }
    }
    if (rot) wave_rotate<NI>(v, lane, a.plan.scale);
    if (tag == 0) {
      _Float16* out = reinterpret_cast<_Float16*>(a.inp_store) + inp_off + lrow * n;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        v8h o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (_Float16)v[i][j];
        *reinterpret_cast<v8h*>(out + (lane + 64 * i) * 8) = o;
      }
      continue;
    }
    if (tag == 3) {  // int4, one scale per 128 values = the 16 chunks held by an aligned group of 16 lanes
      uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (n / 4));
      _Float16* sout = a.scale_store + scale_off + lrow * (n >> 7);
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int c = lane + 64 * i;
        float gmax = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) gmax = fmaxf(gmax, fabsf(v[i][j]));
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o));
        float scale = round_h(gmax / 7.0f);
        if (scale == 0.0f) scale = 1.0f;
        const ScaleDiv div(scale);
        if ((c & 15) == 0) sout[c >> 4] = (_Float16)scale;
        unsigned w = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float r = round_h(div(v[i][j]));
          w = push_code<4>(w, code_word(fminf(fmaxf(r, -7.0f), 7.0f)));
        }
        *reinterpret_cast<unsigned*>(out + c * 4) = w;
      }
      continue;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    const float upper = tag == 1 ? 127.0f : (EXT && tag == 5 ? 448.0f : 7.0f);
    float scale = round_h(amax / upper);   // fp16 division: fp32 quotient of two fp16 values, rounded to fp16
    if (scale == 0.0f) scale = 1.0f;       // quantize.cuh:258
    const ScaleDiv div(scale);
    if (lane == 0) a.scale_store[scale_off + lrow] = (_Float16)scale;
    if (EXT && tag == 4) {
      uint8_t* codes = wave_codes + wave * (n * 2);
#pragma unroll
      for (int i = 0; i < NI; ++i) *reinterpret_cast<v8h*>(codes + (lane + 64 * i) * 16) = bf6_chunk_codes(v[i], div);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      bf6_emit_row(codes, n, 0, n, a.inp_store + 2 * inp_off, lrow, lane, 64);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();  // the next row's codes come after these reads
      continue;
    }
    uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (tag == 1 || (EXT && tag == 5) ? n / 2 : n / 4));
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int c = lane + 64 * i;
      if (EXT && tag == 5) {
        *reinterpret_cast<uint2*>(out + c * 8) = fp8_chunk_codes(v[i], div);
        continue;
      }
      unsigned q[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float r = round_h(div(v[i][j]));
        q[j] = code_word(fminf(fmaxf(r, -upper), upper));
      }
      if (tag == 1) {
        uint2 w{0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w.x = push_code<8>(w.x, q[j]);
          w.y = push_code<8>(w.y, q[j + 4]);
        }
        *reinterpret_cast<uint2*>(out + c * 8) = w;
      } else {
        unsigned w = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) w = push_code<4>(w, q[j]);
        *reinterpret_cast<unsigned*>(out + c * 4) = w;
      }
    }
  }
}

// One TOKEN per wave, for the prologue of power-of-two rows (n = 512 * NI): a token's row is read, rotated and quantised once per
// format among its destinations and stored to each of them, instead of once per destination row as in row_quant_wave_kernel
// (top-k destinations of one format cost one rotation and one quantisation, not k).  Destinations: slot k of the token is sorted
// row row_of_slot[t * topk + k] (negative: the slot's expert id was out of range) of expert ids[t * topk + k], plus, with a shared
// expert, row t of expert E.  Same arithmetic per destination as the row kernels: the stored bytes are identical.  Tags 0 - 3.
struct TokenArgs {
  const _Float16* src;  // [T][n]
  uint8_t* inp_store;
  _Float16* scale_store;
  const int32_t* ids;
  const int32_t* row_of_slot;
  const int64_t* table;  // [4][Et]: tag, start_row, inp_off, scale_off (offsets in fp16 elements)
  int T, E, Et, topk, has_shared;
  int rotate;  // 0 never, 1 rows of quantised experts, 2 every row
  float scale;
};
constexpr int kTokenMaxTopk = 8;

template <int NI>
__global__ void __launch_bounds__(256) token_quant_wave_kernel(const TokenArgs a) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int n = 512 * NI;
  constexpr int KD = kTokenMaxTopk + 1;  // destinations at most: the slots, then the shared expert
  const int ndst = a.topk + (a.has_shared ? 1 : 0);
  const int stride = gridDim.x * 4;
  for (int t = xcd_row_group(blockIdx.x) * 4 + wave; t < a.T; t += stride) {
    // the destinations (wave-uniform: scalar loads, scalar registers)
    int e_of[KD], tag_of[KD];
    long lrow_of[KD];
    unsigned present = 0;  // bit per tag among the destinations
#pragma unroll
    for (int k = 0; k < KD; ++k) {
      e_of[k] = 0, tag_of[k] = -1, lrow_of[k] = 0;
      if (k < ndst) {
        const bool shared = k == a.topk;
        const int r = shared ? t : const_load(a.row_of_slot + t * a.topk + k);
        if (r >= 0) {
          const int e = shared ? a.E : const_load(a.ids + t * a.topk + k);
          e_of[k] = e;
          tag_of[k] = (int)const_load(a.table + e);
          lrow_of[k] = shared ? (long)t : (long)r - const_load(a.table + a.Et + e);
          present |= 1u << tag_of[k];
        }
      }
    }
    if (present == 0) continue;
    const _Float16* srow = a.src + (long)t * n;
    float v[NI][8];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const v8h g = *reinterpret_cast<const v8h*>(srow + (lane + 64 * i) * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[i][j] = (float)g[j];
    }
    // fp16 copies (tag 0): of the row as it is unless every row is rotated
    auto store_copies = [&]() {
#pragma unroll
      for (int k = 0; k < KD; ++k) {
        if (k < ndst && tag_of[k] == 0) {
          _Float16* out = reinterpret_cast<_Float16*>(a.inp_store) + const_load(a.table + 2 * a.Et + e_of[k]) + lrow_of[k] * n;
#pragma unroll
          for (int i = 0; i < NI; ++i) {
            v8h o;
#pragma unroll
            for (int j = 0; j < 8; ++j) o[j] = (_Float16)v[i][j];
            *reinterpret_cast<v8h*>(out + (lane + 64 * i) * 8) = o;
          }
        }
      }
    };
    if ((present & 1u) && a.rotate != 2) store_copies();
    if ((present & ~1u) == 0 && a.rotate != 2) continue;
    if (a.rotate != 0) wave_rotate<NI>(v, lane, a.scale);
    if ((present & 1u) && a.rotate == 2) store_copies();
    if (present & 0x8u) {  // tag 3: int4, one scale per 128 values = the 16 chunks held by an aligned group of 16 lanes
      unsigned w[NI];
      float gscale[NI];
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        float gmax = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) gmax = fmaxf(gmax, fabsf(v[i][j]));
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o));
        float scale = round_h(gmax / 7.0f);
        if (scale == 0.0f) scale = 1.0f;
        const ScaleDiv div(scale);
        gscale[i] = scale;
        w[i] = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float r = round_h(div(v[i][j]));
          w[i] = push_code<4>(w[i], code_word(fminf(fmaxf(r, -7.0f), 7.0f)));
        }
      }
#pragma unroll
      for (int k = 0; k < KD; ++k) {
        if (k < ndst && tag_of[k] == 3) {
          uint8_t* out = a.inp_store + 2 * (const_load(a.table + 2 * a.Et + e_of[k]) + lrow_of[k] * (n / 4));
          _Float16* sout = a.scale_store + const_load(a.table + 3 * a.Et + e_of[k]) + lrow_of[k] * (n >> 7);
#pragma unroll
          for (int i = 0; i < NI; ++i) {
            const int c = lane + 64 * i;
            if ((c & 15) == 0) sout[c >> 4] = (_Float16)gscale[i];
            *reinterpret_cast<unsigned*>(out + c * 4) = w[i];
          }
        }
      }
    }
    if ((present & 0x6u) == 0) continue;
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    if (present & 0x2u) {  // tag 1: int8 per token
      float scale = round_h(amax / 127.0f);  // fp16 division: fp32 quotient of two fp16 values, rounded to fp16
      if (scale == 0.0f) scale = 1.0f;       // quantize.cuh:258
      const ScaleDiv div(scale);
      uint2 w[NI];
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        w[i] = uint2{0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w[i].x = push_code<8>(w[i].x, code_word(fminf(fmaxf(round_h(div(v[i][j])), -127.0f), 127.0f)));
          w[i].y = push_code<8>(w[i].y, code_word(fminf(fmaxf(round_h(div(v[i][j + 4])), -127.0f), 127.0f)));
        }
      }
#pragma unroll
      for (int k = 0; k < KD; ++k) {
        if (k < ndst && tag_of[k] == 1) {
          uint8_t* out = a.inp_store + 2 * (const_load(a.table + 2 * a.Et + e_of[k]) + lrow_of[k] * (n / 2));
          if (lane == 0) a.scale_store[const_load(a.table + 3 * a.Et + e_of[k]) + lrow_of[k]] = (_Float16)scale;
#pragma unroll
          for (int i = 0; i < NI; ++i) *reinterpret_cast<uint2*>(out + (lane + 64 * i) * 8) = w[i];
        }
      }
    }
    if (present & 0x4u) {  // tag 2: int4 per token
      float scale = round_h(amax / 7.0f);
      if (scale == 0.0f) scale = 1.0f;
      const ScaleDiv div(scale);
      unsigned w[NI];
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        w[i] = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) w[i] = push_code<4>(w[i], code_word(fminf(fmaxf(round_h(div(v[i][j])), -7.0f), 7.0f)));
      }
#pragma unroll
      for (int k = 0; k < KD; ++k) {
        if (k < ndst && tag_of[k] == 2) {
          uint8_t* out = a.inp_store + 2 * (const_load(a.table + 2 * a.Et + e_of[k]) + lrow_of[k] * (n / 4));
          if (lane == 0) a.scale_store[const_load(a.table + 3 * a.Et + e_of[k]) + lrow_of[k]] = (_Float16)scale;
#pragma unroll
          for (int i = 0; i < NI; ++i) *reinterpret_cast<unsigned*>(out + (lane + 64 * i) * 4) = w[i];
        }
      }
    }
  }
}

// One row per WAVE for rotations H_K kron H_8 with a table-driven factor (K = f * kb, H_K = S_f kron B, f <= 4, kb <= 64; a 1408-value
// row is 176 x 8 with f = 4, kb = 44): lane l holds the chunks l + 64 i, a chunk being the 8 values of one k.  The Sylvester part
// (H_8) stays inside a chunk.  The dense stage t[b][col] = sum_b' B[b][b'] q[b'][col] over the 8 f columns col = blk * 8 + j runs on the
// matrix cores: the row, snapped to integers of at most 18 bits (DenseGrid) and divided by 16 so that every value is an fp16 number,
// is written to LDS transposed ([col][b'], b' contiguous), B (+-1, zero padded) is the first operand, kept in LDS in operand order
// and read block by block, and the fp32 results are exact whatever order the hardware adds in.  Results return through LDS in row order, so
// the quantise / pack / store code sees the same chunk-per-lane layout as in the other kernels and writes 16 bytes per lane.
// Four independent rows per workgroup; no barrier (each wave owns its piece of LDS).
constexpr int kDensePitch = 144;             // bytes per column of the transposed row: 64 fp16 + 16 (16 lanes read 16 distinct bank groups)
// LDS of a workgroup: B as matrix operands (one KiB per 16 x 32 block), then per wave the transposed row and the rotated row in row
// order (+ a slot of 8 values for discarded ones)
__host__ __device__ constexpr int dense_wave_lds(int n) { return 32 * kDensePitch + (n + 8) * 2; }
__host__ __device__ constexpr int dense_lds(int n, int kb) { return ((kb + 15) >> 4) * ((kb + 31) >> 5) * 1024 + 4 * dense_wave_lds(n); }
template <int MAXC, bool SILU, bool EXT>
__global__ void __launch_bounds__(256) row_quant_dense_kernel(const RowArgs a) {
  extern __shared__ __align__(16) uint8_t dlds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lm = lane & 15, lg = lane >> 4;
  const RotPlan pl = a.plan;
  const int n = pl.n, nchunks = n >> 3, kb = pl.kb;
  const int ksteps = (kb + 31) >> 5, mblocks = (kb + 15) >> 4;
  uint8_t* xt = dlds + mblocks * ksteps * 1024 + wave * dense_wave_lds(n);  // [32 columns][kDensePitch]
  uint8_t* yrow = xt + 32 * kDensePitch;                                      // [n] fp16, then the discard slot
  // B as the first operand of v_mfma_f32_16x16x32_f16: lane holds row 16 mb + (lane & 15), k = 32 ks + 8 (lane >> 4) + 0..7.  Kept in
  // LDS (block (mb, ks) at (mb * ksteps + ks) KiB, 16 bytes per lane) and read per row: 32 registers fewer per lane.
  for (int blkid = wave; blkid < mblocks * ksteps; blkid += 4) {
    const int mb = blkid / ksteps, ks = blkid - mb * ksteps;
    const int b = 16 * mb + lm;
    v8h bs;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // unconditional loads (index clamped into the table, the value dropped afterwards): all of them are in flight together
      const int bp = 32 * ks + 8 * lg + i;
      const float sv = a.signs[min(b, kb - 1) * kb + min(bp, kb - 1)];
      bs[i] = (b < kb && bp < kb) ? (_Float16)sv : (_Float16)0.0f;
    }
    *reinterpret_cast<v8h*>(dlds + blkid * 1024 + lane * 16) = bs;
  }
  // columns and k positions that no row ever writes must read as zero
  for (int i = lane; i < 32 * kDensePitch / 16; i += 64) reinterpret_cast<v4i*>(xt)[i] = v4i{0, 0, 0, 0};
  __syncthreads();

  struct RowMeta {
    int tag;
    long lrow, inp_off, scale_off;
    const _Float16* srow;
    bool exists;
  };
  const _Float16* const src_shared = shared_src(a);
  const int routed = a.routed_ptr ? (int)const_load(a.routed_ptr) : a.R;  // rows [routed, R) of a planned launch do not exist
  auto load_meta = [&](int row) {
    RowMeta m;
    const bool shared_row = row >= a.R;
    m.exists = row < routed || shared_row;
    const int e = shared_row ? a.E : (m.exists ? const_load(a.dst_exp + row) : 0);
    m.tag = (int)const_load(a.table + e);
    m.lrow = shared_row ? row - a.R : row - const_load(a.table + a.Et + e);
    m.inp_off = const_load(a.table + 2 * a.Et + e);
    m.scale_off = const_load(a.table + 3 * a.Et + e);
    if (SILU) {
      m.srow = shared_row ? src_shared + (long)(row - a.R) * 2 * n : a.src + (long)row * 2 * n;
    } else {
      m.srow = (shared_row ? src_shared : a.src) + (shared_row ? (long)(row - a.R) : (m.exists ? (long)const_load(a.perm + row) : 0l)) * n;
    }
    return m;
  };
  auto load_data = [&](const RowMeta& m, v8h (&g)[MAXC], v8h (&u)[MAXC]) {
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = min(lane + 64 * i, nchunks - 1);  // lanes past the row re-read its last chunk (never used)
      g[i] = *reinterpret_cast<const v8h*>(m.srow + c * 8);
      if (SILU) u[i] = *reinterpret_cast<const v8h*>(m.srow + n + c * 8);
    }
  };
  const int stride_rows = gridDim.x * 4;
  // One row ahead: the bookkeeping of the next row (a chain of dependent loads) is fetched at the top of a row, its data as soon as
  // this row's data has been turned into values, so the same registers hold both and the loads fly under the rotation and the stores.
  RowMeta next_meta;
  v8h row_g[MAXC], row_u[MAXC];
  const int row0 = xcd_row_group(blockIdx.x) * 4 + wave;
  if (row0 < a.rows) {
    next_meta = load_meta(row0);
    load_data(next_meta, row_g, row_u);
  }
  for (int row = row0; row < a.rows; row += stride_rows) {
    const RowMeta cur = next_meta;
    const bool has_next = row + stride_rows < a.rows;
    if (has_next) next_meta = load_meta(row + stride_rows);
    float v[MAXC][8];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const bool live = lane + 64 * i < nchunks;
      const v8h g = row_g[i];
      if (SILU) {
        const v8h u = row_u[i];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float gf = (float)g[j];
          const float sl = silu_fixed(gf);
          v[i][j] = round_h(keep_f32(sl * (float)u[j]));
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = (float)g[j];
      }
      if (!live) {  // chunks past the row count as zeros (in the row's maxima) and are never stored
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = 0.0f;
      }
    }
    if (has_next) load_data(next_meta, row_g, row_u);
    if (!cur.exists) continue;
    const int tag = cur.tag;
    const bool rot = a.rotate == 2 || (a.rotate == 1 && tag != 0);

    if (rot) {
      // H_8 inside the chunk (strides 1, 2, 4), scale, round to fp16
      float mx = 0.0f;
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
#pragma unroll
        for (int h = 1; h < 8; h <<= 1)
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (!(j & h)) {
              const float p = v[i][j], q = v[i][j + h];
              v[i][j] = p + q;
              v[i][j + h] = p - q;
            }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          v[i][j] = round_h(keep_f32(v[i][j] * pl.scale));
          mx = fmaxf(mx, fabsf(v[i][j]));
        }
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
      const DenseGrid grid(mx);
      const float to16 = grid.to_grid * 0.0625f;  // exact (a power of two well inside the range); rint(v * to_grid) / 16 below
      // transposed write: chunk c = blk * kb + b' -> columns blk * 8 + j, position b'
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunks) {
          const int blk = c / kb, bp = c - blk * kb;
          uint8_t* dst = xt + (blk * 8) * kDensePitch + bp * 2;
#pragma unroll
          for (int j = 0; j < 8; ++j) *reinterpret_cast<_Float16*>(dst + j * kDensePitch) = (_Float16)(rintf(v[i][j] * grid.to_grid) * 0.0625f);
        }
      }
      (void)to16;
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      // lane holds column col = 16 nb + (lane & 15), i.e. blk = 2 nb + ((lane >> 3) & 1), j = lane & 7, and rows b = 16 mb + 4 (lane >> 4) + r
      // of every 16 x 16 block.  One block of 16 rows of B at a time (8 accumulator registers live, the second operand re-read
      // from LDS), each followed by its way back: S_f butterflies across blk (bit 0 = lane bit 3, bit 1 = the column block;
      // ascending), back to the row's scale (a power of two: exact wherever it is applied) with the one rounding to fp16, and the
      // value goes to its place in the row (values of rows or blocks that do not exist go to the discard slot).  Compiled once per
      // order f of the Sylvester factor, so that nothing in it branches on f.
      const float back = grid.from_grid * 16.0f;
      // (positions from a lane number the compiler must take as changing from row to row: otherwise it keeps every position of
      // every row block in a register of its own for the whole kernel)
      int lane_now = lane;
      asm volatile("" : "+v"(lane_now));
      auto dense_stage = [&](auto f_const) {
        constexpr int F = decltype(f_const)::value;
        constexpr int NCOLS = F > 2 ? 2 : 1;
        const float sgn8 = (lane_now & 8) ? -1.0f : 1.0f;
        const int blk0 = (lane_now >> 3) & 1, jj = lane_now & 7;
        // row 16 mb + 4 (lane >> 4) + r of B exists, and the lane's column block too, when 16 mb + r < lim
        const int lim = blk0 < F ? kb - 4 * (lane_now >> 4) : 0;
        uint8_t* const y0 = yrow + 2 * (((blk0 * kb + 4 * (lane_now >> 4)) << 3) + jj);  // place of row block 0, r = 0, in the row
        uint8_t* const y1 = y0 + 2 * ((2 * kb) << 3);                                      // the same, two column blocks on
        uint8_t* const ydiscard = yrow + 2 * n;
        constexpr int kStep = 2 * 8;  // bytes between the places of consecutive rows of B
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
          if (mb < mblocks) {
            v4f acc[NCOLS];
#pragma unroll
            for (int nb = 0; nb < NCOLS; ++nb) acc[nb] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
              if (ks < ksteps) {
                const v8h bs = *reinterpret_cast<const v8h*>(dlds + (mb * ksteps + ks) * 1024 + lane * 16);
#pragma unroll
                for (int nb = 0; nb < NCOLS; ++nb) {
                  const v8h xf = *reinterpret_cast<const v8h*>(xt + (nb * 16 + lm) * kDensePitch + ks * 64 + lg * 16);
                  acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bs, xf, acc[nb], 0, 0, 0);
                }
              }
            }
            // a block whose 16 rows all exist, in a column block that exists for every lane, needs no test per value
            const bool whole = F > 1 && 16 * mb + 16 <= kb;
            auto emit = [&](auto whole_const) {
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                constexpr bool kWhole = decltype(whole_const)::value;
                const int off = (16 * mb + r) * kStep;
                const bool ok = kWhole || 16 * mb + r < lim;
                float t0 = acc[0][r], t1 = 0.0f;
                if constexpr (F > 1) t0 = __builtin_fmaf(sgn8, t0, lane_xor<8>(t0));
                if constexpr (F > 2) {
                  t1 = acc[NCOLS - 1][r];
                  t1 = __builtin_fmaf(sgn8, t1, lane_xor<8>(t1));
                  const float p = t0, q = t1;
                  t0 = p + q;
                  t1 = p - q;
                }
                *reinterpret_cast<_Float16*>((ok ? y0 : ydiscard - off) + off) = (_Float16)(t0 * back);
                if constexpr (F > 2) *reinterpret_cast<_Float16*>((ok ? y1 : ydiscard - off) + off) = (_Float16)(t1 * back);
              }
            };
            if (whole) {
              emit(std::true_type{});
            } else {
              emit(std::false_type{});
            }
          }
        }
      };
      switch (pl.f) {
        case 1: dense_stage(std::integral_constant<int, 1>{}); break;
        case 2: dense_stage(std::integral_constant<int, 2>{}); break;
        default: dense_stage(std::integral_constant<int, 4>{}); break;
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = min(lane + 64 * i, nchunks - 1);
        const bool live = lane + 64 * i < nchunks;
        const v8h y = *reinterpret_cast<const v8h*>(yrow + c * 16);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = live ? (float)y[j] : 0.0f;
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();  // the next row's writes come after these reads
    }

    // ---- store: fp16 copy or symmetric quantisation (as in the other row kernels) ----
    const long lrow = cur.lrow, inp_off = cur.inp_off, scale_off = cur.scale_off;
    if (tag == 0) {
      _Float16* out = reinterpret_cast<_Float16*>(a.inp_store) + inp_off + lrow * n;
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunks) {
          v8h o;
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = (_Float16)v[i][j];
          *reinterpret_cast<v8h*>(out + c * 8) = o;
        }
      }
      continue;
    }
    if (tag == 3) {  // int4, one scale per 128 values = the 16 chunks held by an aligned group of 16 lanes
      uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (n / 4));
      _Float16* sout = a.scale_store + scale_off + lrow * (n >> 7);
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = lane + 64 * i;
        const bool live = c < nchunks;  // whole lane groups are live or not: n is a multiple of 128
        float gmax = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) gmax = fmaxf(gmax, fabsf(v[i][j]));
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o));
        float scale = round_h(gmax / 7.0f);
        if (scale == 0.0f) scale = 1.0f;
        const ScaleDiv div(scale);
        if (live) {
          if ((c & 15) == 0) sout[c >> 4] = (_Float16)scale;
          unsigned w = 0;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float r = round_h(div(v[i][j]));
            w = push_code<4>(w, code_word(fminf(fmaxf(r, -7.0f), 7.0f)));
          }
          *reinterpret_cast<unsigned*>(out + c * 4) = w;
        }
      }
      continue;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));  // chunks past the row hold zeros
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    const float upper = tag == 1 ? 127.0f : (EXT && tag == 5 ? 448.0f : 7.0f);
    float scale = round_h(amax / upper);   // fp16 division: fp32 quotient of two fp16 values, rounded to fp16
    if (scale == 0.0f) scale = 1.0f;       // quantize.cuh:258
    const ScaleDiv div(scale);
    if (lane == 0) a.scale_store[scale_off + lrow] = (_Float16)scale;
    if (EXT && tag == 4) {  // codes into the wave's row buffer (its reads of the rotated row are behind a wave barrier), then fragments
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int c = lane + 64 * i;
        if (c < nchunks) *reinterpret_cast<v8h*>(yrow + c * 16) = bf6_chunk_codes(v[i], div);
      }
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();
      bf6_emit_row(yrow, n, 0, n, a.inp_store + 2 * inp_off, lrow, lane, 64);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_wave_barrier();  // the next row's writes come after these reads
      continue;
    }
    uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (tag == 1 || (EXT && tag == 5) ? n / 2 : n / 4));
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = lane + 64 * i;
      if (c < nchunks) {
        if (EXT && tag == 5) {
          *reinterpret_cast<uint2*>(out + c * 8) = fp8_chunk_codes(v[i], div);
          continue;
        }
        unsigned q[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float r = round_h(div(v[i][j]));
          q[j] = code_word(fminf(fmaxf(r, -upper), upper));
        }
        if (tag == 1) {
          uint2 w{0, 0};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            w.x = push_code<8>(w.x, q[j]);
            w.y = push_code<8>(w.y, q[j + 4]);
          }
          *reinterpret_cast<uint2*>(out + c * 8) = w;
        } else {
          unsigned w = 0;
#pragma unroll
          for (int j = 0; j < 8; ++j) w = push_code<4>(w, q[j]);
          *reinterpret_cast<unsigned*>(out + c * 4) = w;
        }
      }
    }
  }
}

// One row per WORKGROUP of 8 waves for rotations B_kb kron H_512 (kb <= 32, no Sylvester factor in the table: a 14336-value row is
// 28 x 512).  Wave w holds the k rows w, w + 8, w + 16, w + 24 of the [kb][512] view, lane l the chunk l of each, so the whole
// Sylvester part runs inside a wave: strides 1, 2, 4 in a chunk, 8 .. 256 across lanes, no LDS and no barrier.  The dense stage is the
// same exact integer sum as in row_quant_dense_kernel, on the matrix cores: the snapped row goes to LDS as it is ([k][column], one
// 16-byte write per chunk), every wave gathers the second operand of its 64 columns from there (two bytes per read, each landing in
// its half of the operand register) and multiplies B (first operand, in registers) into them, and the results return through LDS in
// row order for the quantise / pack / store code.  Four barriers per row; two workgroups share a CU.
constexpr int kWidePitch = 1024 + 8;                                 // bytes per k row of 512 fp16 in LDS: the 4 k groups (or row groups) that the
                                                                     // lanes of a wave touch together land 8 or 16 banks apart
constexpr int kWideLds = 2 * 32 * kWidePitch + 64;                   // snapped row, rotated row, reduction slots
template <bool SILU, bool EXT>
__global__ void __launch_bounds__(512) row_quant_wide_kernel(const RowArgs a) {
  extern __shared__ __align__(16) uint8_t wlds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register: "is k row wave + 8 i live" is then a scalar branch
  const int lm = lane & 15, lg = lane >> 4;
  uint8_t* xt = wlds;                                   // [32 k rows][kWidePitch]: the snapped row
  uint8_t* yrow = xt + 32 * kWidePitch;                 // [32 rows][kWidePitch]: the rotated row
  float* red = reinterpret_cast<float*>(yrow + 32 * kWidePitch);  // [8] + [8]
  const RotPlan pl = a.plan;
  const int n = pl.n, kb = pl.kb;
  constexpr int MAXC = 4;
  // B as the first operand of v_mfma_f32_16x16x32_f16: lane holds row 16 mb + (lane & 15), k = 8 (lane >> 4) + 0..7
  v8h bsign[2];
#pragma unroll
  for (int mb = 0; mb < 2; ++mb) {
    const int b = 16 * mb + lm;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int bp = 8 * lg + i;
      const float sv = a.signs[min(b, kb - 1) * kb + min(bp, kb - 1)];
      bsign[mb][i] = (b < kb && bp < kb) ? (_Float16)sv : (_Float16)0.0f;
    }
  }
  // k rows kb .. 31 are never written and must read as zero
  for (int i = tid; i < 32 * kWidePitch / 8; i += 512) reinterpret_cast<uint2*>(xt)[i] = make_uint2(0, 0);
  const _Float16* const src_shared = shared_src(a);
  for (int row = blockIdx.x; row < a.rows; row += gridDim.x) {
    if (!row_exists(a, row)) continue;
    const bool shared_row = row >= a.R;
    const int e = shared_row ? a.E : a.dst_exp[row];
    const int tag = (int)a.table[e];
    const long lrow = shared_row ? row - a.R : row - a.table[a.Et + e];
    const long inp_off = a.table[2 * a.Et + e];
    const long scale_off = a.table[3 * a.Et + e];
    const bool rot = a.rotate == 2 || (a.rotate == 1 && tag != 0);
    const _Float16* srow;
    if (SILU) {
      srow = shared_row ? src_shared + (long)(row - a.R) * 2 * n : a.src + (long)row * 2 * n;
    } else {
      srow = (shared_row ? src_shared : a.src) + (shared_row ? (long)(row - a.R) : (long)a.perm[row]) * n;
    }
    // A k row past kb (the last of a wave's four when kb is not a multiple of 8: waves 4 .. 7 of a 28-row view) costs nothing: the
    // whole wave skips its loads, its SiLU and its butterflies, and the slot holds zeros.
    float v[MAXC][8];
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int kr = wave + 8 * i;
      if (kr < kb) {
        const int c = kr * 64 + lane;  // chunk index in the row
        const v8h g = *reinterpret_cast<const v8h*>(srow + c * 8);
        if (SILU) {
          const v8h u = *reinterpret_cast<const v8h*>(srow + n + c * 8);
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float gf = (float)g[j];
            const float sl = silu_fixed(gf);
            v[i][j] = round_h(keep_f32(sl * (float)u[j]));
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) v[i][j] = (float)g[j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = 0.0f;
      }
    }
    if (rot) {
      // H_512 along each k row: strides 1, 2, 4 inside the chunk, 8 .. 256 across the lanes (ascending)
      float mx = 0.0f;
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        if (wave + 8 * i >= kb) continue;
#pragma unroll
        for (int h = 1; h < 8; h <<= 1)
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (!(j & h)) {
              const float p = v[i][j], q = v[i][j + h];
              v[i][j] = p + q;
              v[i][j + h] = p - q;
            }
        auto lane_stage = [&](auto mc) {
          constexpr int m = decltype(mc)::value;
          const float sgn = (lane & m) ? -1.0f : 1.0f;
#pragma unroll
          for (int j = 0; j < 8; ++j) v[i][j] = __builtin_fmaf(sgn, v[i][j], lane_xor<m>(v[i][j]));
        };
        lane_stage(std::integral_constant<int, 1>{});
        lane_stage(std::integral_constant<int, 2>{});
        lane_stage(std::integral_constant<int, 4>{});
        lane_stage(std::integral_constant<int, 8>{});
        lane_stage(std::integral_constant<int, 16>{});
        lane_stage(std::integral_constant<int, 32>{});
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          v[i][j] = round_h(keep_f32(v[i][j] * pl.scale));
          mx = fmaxf(mx, fabsf(v[i][j]));
        }
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
      if (lane == 0) red[wave] = mx;
      __syncthreads();  // (also: the previous row's readers of xt / yrow are done)
      mx = red[0];
#pragma unroll
      for (int w = 1; w < 8; ++w) mx = fmaxf(mx, red[w]);
      const DenseGrid grid(mx);
      // the snapped row, k row kr / chunk lane at its place
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int kr = wave + 8 * i;
        if (kr < kb) {
          v8h q;
#pragma unroll
          for (int j = 0; j < 8; ++j) q[j] = (_Float16)(rintf(v[i][j] * grid.to_grid) * 0.0625f);
          *reinterpret_cast<v8h*>(xt + kr * kWidePitch + lane * 16) = q;
        }
      }
      __syncthreads();
      // this wave's 64 columns: 4 column blocks x 2 row blocks; the second operand of a lane is column col, k = 8 (lane >> 4) + 0..7
      const float back = grid.from_grid * 16.0f;
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        const int col = wave * 64 + nb * 16 + lm;
        v8h xf;
#pragma unroll
        for (int i = 0; i < 8; ++i) xf[i] = *reinterpret_cast<const _Float16*>(xt + (8 * lg + i) * kWidePitch + col * 2);
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          v4f acc = {0.f, 0.f, 0.f, 0.f};
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(bsign[mb], xf, acc, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int b = 16 * mb + 4 * lg + r;  // lane holds column col and rows b of the block (rows kb .. 31 are never read back)
            *reinterpret_cast<_Float16*>(yrow + b * kWidePitch + col * 2) = (_Float16)(acc[r] * back);
          }
        }
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int kr = wave + 8 * i;
        if (kr >= kb) continue;  // (still zeros)
        const v8h y = *reinterpret_cast<const v8h*>(yrow + kr * kWidePitch + lane * 16);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = (float)y[j];
      }
    }

    // ---- store: fp16 copy or symmetric quantisation (as in the other row kernels); chunk c = kr * 64 + lane ----
    if (tag == 0) {
      _Float16* out = reinterpret_cast<_Float16*>(a.inp_store) + inp_off + lrow * n;
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int kr = wave + 8 * i;
        if (kr < kb) {
          v8h o;
#pragma unroll
          for (int j = 0; j < 8; ++j) o[j] = (_Float16)v[i][j];
          *reinterpret_cast<v8h*>(out + (kr * 64 + lane) * 8) = o;
        }
      }
      continue;
    }
    if (tag == 3) {  // int4, one scale per 128 values = the 16 chunks held by an aligned group of 16 lanes
      uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (n / 4));
      _Float16* sout = a.scale_store + scale_off + lrow * (n >> 7);
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int kr = wave + 8 * i;
        if (kr >= kb) continue;
        const int c = kr * 64 + lane;
        float gmax = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) gmax = fmaxf(gmax, fabsf(v[i][j]));
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, o));
        float scale = round_h(gmax / 7.0f);
        if (scale == 0.0f) scale = 1.0f;
        const ScaleDiv div(scale);
        if ((c & 15) == 0) sout[c >> 4] = (_Float16)scale;
        unsigned w = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float r = round_h(div(v[i][j]));
          w = push_code<4>(w, code_word(fminf(fmaxf(r, -7.0f), 7.0f)));
        }
        *reinterpret_cast<unsigned*>(out + c * 4) = w;
      }
      continue;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
    if (lane == 0) red[8 + wave] = amax;
    __syncthreads();
    amax = red[8];
#pragma unroll
    for (int w = 1; w < 8; ++w) amax = fmaxf(amax, red[8 + w]);
    const float upper = tag == 1 ? 127.0f : (EXT && tag == 5 ? 448.0f : 7.0f);
    float scale = round_h(amax / upper);   // fp16 division: fp32 quotient of two fp16 values, rounded to fp16
    if (scale == 0.0f) scale = 1.0f;       // quantize.cuh:258
    const ScaleDiv div(scale);
    if (tid == 0) a.scale_store[scale_off + lrow] = (_Float16)scale;
    if (EXT && tag == 4) {  // codes into the rotated row's buffer, each wave over its own k rows, then fragments by the whole workgroup
      __syncthreads();  // (a row that was not rotated did not pass the barriers that order the previous row's readers of this buffer)
#pragma unroll
      for (int i = 0; i < MAXC; ++i) {
        const int kr = wave + 8 * i;
        if (kr < kb) *reinterpret_cast<v8h*>(yrow + kr * kWidePitch + lane * 16) = bf6_chunk_codes(v[i], div);
      }
      __syncthreads();
      bf6_emit_row(yrow, 512, kWidePitch, n, a.inp_store + 2 * inp_off, lrow, tid, 512);
      __syncthreads();
      continue;
    }
    uint8_t* out = a.inp_store + 2 * (inp_off + lrow * (tag == 1 || (EXT && tag == 5) ? n / 2 : n / 4));
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int kr = wave + 8 * i;
      if (kr < kb) {
        const int c = kr * 64 + lane;
        if (EXT && tag == 5) {
          *reinterpret_cast<uint2*>(out + c * 8) = fp8_chunk_codes(v[i], div);
          continue;
        }
        unsigned q[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float r = round_h(div(v[i][j]));
          q[j] = code_word(fminf(fmaxf(r, -upper), upper));
        }
        if (tag == 1) {
          uint2 w{0, 0};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            w.x = push_code<8>(w.x, q[j]);
            w.y = push_code<8>(w.y, q[j + 4]);
          }
          *reinterpret_cast<uint2*>(out + c * 8) = w;
        } else {
          unsigned w = 0;
#pragma unroll
          for (int j = 0; j < 8; ++j) w = push_code<4>(w, q[j]);
          *reinterpret_cast<unsigned*>(out + c * 4) = w;
        }
      }
    }
  }
}

static int make_plan(int n, int had_k, int had_f, bool rotate, RotPlan* p) {
  p->n = n;
  p->scale = 1.0f / sqrtf((float)n);
  p->kb = 1;
  p->f = 1;
  p->m = n;
  if (had_k > 1) {
    if (n % had_k) return 1;
    p->m = n / had_k;
    p->f = had_f;
    p->kb = had_k / had_f;
  }
  if (rotate && (p->m < 8 || (p->m & (p->m - 1)))) return 1;
  return 0;
}

template <bool SILU, bool EXT>
static int launch_rows_as(const RowArgs& a, int lds_bytes, hipStream_t s) {
  const int nmax = a.plan.n > a.plan_shared.n ? a.plan.n : a.plan_shared.n;
  int dev = 0, cus = 256;
  (void)hipGetDevice(&dev);
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  const int grid = a.rows < cus * 8 ? a.rows : cus * 8;
  if (lds_bytes > 64 * 1024) {
    last_error() = "row too long for the activation kernels";
    return 3;
  }
  // pure power-of-two rows (no table-driven Hadamard factor): one row per wave
  const int n = a.plan.n;
  if (a.plan.kb == 1 && a.plan_shared.kb == 1 && a.plan_shared.n == n && n % 512 == 0 && n <= 4096 && (n & (n - 1)) == 0) {
    // (a multiple of 64 workgroups: xcd_row_group permutes within runs of 64)
    const int wgrid = ((a.rows + 3) / 4 < cus * 8 ? (a.rows + 3) / 4 : cus * 8) + 63 & ~63;
    const int wlds = EXT ? 4 * n * 2 : 0;  // the waves' code rows (tag 4)
    switch (n / 512) {
      case 1: hipLaunchKernelGGL((row_quant_wave_kernel<1, SILU, EXT>), dim3(wgrid), dim3(256), wlds, s, a); break;
      case 2: hipLaunchKernelGGL((row_quant_wave_kernel<2, SILU, EXT>), dim3(wgrid), dim3(256), wlds, s, a); break;
      case 4: hipLaunchKernelGGL((row_quant_wave_kernel<4, SILU, EXT>), dim3(wgrid), dim3(256), wlds, s, a); break;
      default: hipLaunchKernelGGL((row_quant_wave_kernel<8, SILU, EXT>), dim3(wgrid), dim3(256), wlds, s, a); break;
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
      return 4;
    }
    return 0;
  }
  // table-driven factor times H_8, one size of row: one row per wave, dense stage on the matrix cores
  if (a.plan.kb > 1 && a.plan.m == 8 && a.plan.f <= 4 && a.plan.kb <= 64 && n <= 2048 && a.plan_shared.n == n && a.plan_shared.kb == a.plan.kb && a.rotate != 0) {
    const int dlds = dense_lds(n, a.plan.kb);
    // as many workgroups as stay resident together (registers and LDS decide how many share a CU), each looping over its rows
    auto launch = [&](auto kernel, int which) {
      static int asked_lds[4][64] = {}, answer[4][64] = {};  // per kernel size and device: the last LDS size asked about
      int per_cu = 0;
      if (dev >= 0 && dev < 64 && asked_lds[which][dev] == dlds) {
        per_cu = answer[which][dev];
      } else {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, dlds) != hipSuccess || per_cu < 1) per_cu = 2;
        if (dev >= 0 && dev < 64) asked_lds[which][dev] = dlds, answer[which][dev] = per_cu;
      }
      const int wgrid = ((a.rows + 3) / 4 < cus * per_cu ? (a.rows + 3) / 4 : cus * per_cu) + 63 & ~63;  // (xcd_row_group: runs of 64)
      hipLaunchKernelGGL(kernel, dim3(wgrid), dim3(256), dlds, s, a);
    };
    switch ((n / 8 + 63) / 64) {
      case 1: launch(row_quant_dense_kernel<1, SILU, EXT>, 0); break;
      case 2: launch(row_quant_dense_kernel<2, SILU, EXT>, 1); break;
      case 3: launch(row_quant_dense_kernel<3, SILU, EXT>, 2); break;
      default: launch(row_quant_dense_kernel<4, SILU, EXT>, 3); break;
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
      return 4;
    }
    return 0;
  }
  // table-driven order times H_512, one size of row: one row per 512-thread workgroup, Sylvester part inside the waves, dense stage on
  // the matrix cores
  if (a.plan.kb > 1 && a.plan.kb <= 32 && a.plan.m == 512 && a.plan.f == 1 && a.plan_shared.n == n && a.plan_shared.kb == a.plan.kb && a.rotate != 0) {
    static bool opted_in[64] = {};
    if (dev >= 0 && dev < 64 && !opted_in[dev]) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(&row_quant_wide_kernel<SILU, EXT>), hipFuncAttributeMaxDynamicSharedMemorySize, kWideLds) != hipSuccess) {
        last_error() = "could not reserve LDS for the wide-row quantiser";
        return 4;
      }
      opted_in[dev] = true;
    }
    const int wgrid = a.rows < cus * 8 ? a.rows : cus * 8;
    hipLaunchKernelGGL((row_quant_wide_kernel<SILU, EXT>), dim3(wgrid), dim3(512), kWideLds, s, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
      return 4;
    }
    return 0;
  }
  // workgroup size and chunks per thread with the fewest idle lanes
  const int nchunks = nmax / 8;
  // long rows take 512 threads rather than more chunks per thread: a thread's chunks live in registers (with the next row's
  // already on their way), and seven of them leave room for one wave per SIMD only
  static const int kShapes[][2] = {{192, 1}, {256, 1}, {192, 2}, {256, 2}, {192, 3}, {256, 3}, {512, 2}, {512, 3}, {512, 4}};
  int pick = -1;
  for (int i = 0; i < 9 && pick < 0; ++i)
    if (kShapes[i][0] * kShapes[i][1] >= nchunks) pick = i;
  switch (pick) {
    case 0: hipLaunchKernelGGL((row_quant_kernel<1, SILU, 192, EXT>), dim3(grid), dim3(192), lds_bytes, s, a); break;
    case 1: hipLaunchKernelGGL((row_quant_kernel<1, SILU, 256, EXT>), dim3(grid), dim3(256), lds_bytes, s, a); break;
    case 2: hipLaunchKernelGGL((row_quant_kernel<2, SILU, 192, EXT>), dim3(grid), dim3(192), lds_bytes, s, a); break;
    case 3: hipLaunchKernelGGL((row_quant_kernel<2, SILU, 256, EXT>), dim3(grid), dim3(256), lds_bytes, s, a); break;
    case 4: hipLaunchKernelGGL((row_quant_kernel<3, SILU, 192, EXT>), dim3(grid), dim3(192), lds_bytes, s, a); break;
    case 5: hipLaunchKernelGGL((row_quant_kernel<3, SILU, 256, EXT>), dim3(grid), dim3(256), lds_bytes, s, a); break;
    case 6: hipLaunchKernelGGL((row_quant_kernel<2, SILU, 512, EXT>), dim3(grid), dim3(512), lds_bytes, s, a); break;
    case 7: hipLaunchKernelGGL((row_quant_kernel<3, SILU, 512, EXT>), dim3(grid), dim3(512), lds_bytes, s, a); break;
    case 8: hipLaunchKernelGGL((row_quant_kernel<4, SILU, 512, EXT>), dim3(grid), dim3(512), lds_bytes, s, a); break;
    default:
      last_error() = "row too long for the activation kernels";
      return 3;
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

// Tags 4 and 5 (operand variants of the bf6 and fp8 matrix paths) are compiled into a second set of the kernels: their code raises every
// kernel's register budget (the 512-thread kernel's past the two-workgroups-per-CU limit), and the host, which never reads the table,
// is told by bit 2 of the entry points' `rotate` argument whether a table may hold them.
template <bool SILU>
static int launch_rows(const RowArgs& a, int lds_bytes, hipStream_t s, bool variants) {
  return variants ? launch_rows_as<SILU, true>(a, lds_bytes, s) : launch_rows_as<SILU, false>(a, lds_bytes, s);
}

}  // namespace mxmoe

using namespace mxmoe;

// ---- un-permute + top-k weighted combine: the step after the down launch (the reference leaves it as the empty stub
// gg_unpermute_out, mxmoe/kernels/src/ref_bind.cu:66) ----
//
// row_of_slot[t * topk + k] = sorted row that holds (token t, slot k), or -1 when that slot's expert id was dropped.
__global__ void combine_fill_kernel(int32_t* __restrict__ row_of_slot, int slots) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < slots) row_of_slot[i] = -1;
}
__global__ void combine_invert_kernel(const int64_t* __restrict__ src_slot, int rows, int slots, int32_t* __restrict__ row_of_slot,
                                      const int64_t* __restrict__ rows_ptr) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (rows_ptr) rows = min(rows, (int)*rows_ptr);  // planned mode: `rows` is the capacity, the routed rows are counted on the device
  if (r < rows) {
    const int64_t sl = src_slot[r];
    if (sl >= 0 && sl < slots) row_of_slot[sl] = r;
  }
}
// One workgroup per token: out[t] = half( sum_k w[t,k] * float(down[row(t,k)])  (k ascending, fp32: product rounded, then the
// sum rounded)  + float(shared[t]) ).  Pure streaming: every down row is read once, 16 bytes per lane.
__global__ void __launch_bounds__(256) combine_kernel(const _Float16* __restrict__ down, const _Float16* __restrict__ shared, const float* __restrict__ weights,
                                                      const int32_t* __restrict__ row_of_slot, int topk, int K, _Float16* __restrict__ out,
                                                      const int64_t* __restrict__ shared_addr) {
  const int t = blockIdx.x;
  if (shared_addr) shared = reinterpret_cast<const _Float16*>(*shared_addr);  // planned mode: where the planner put the shared expert's rows (0: none)
  for (int c = threadIdx.x * 8; c < K; c += 256 * 8) {
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
    for (int k = 0; k < topk; ++k) {
      const int r = row_of_slot[t * topk + k];
      if (r < 0) continue;
      const float w = weights[t * topk + k];
      const v8h v = *reinterpret_cast<const v8h*>(down + (size_t)r * K + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = acc[e] + w * (float)v[e];
    }
    v8h o;
    if (shared) {
      const v8h v = *reinterpret_cast<const v8h*>(shared + (size_t)t * K + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = acc[e] + (float)v[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (_Float16)keep_f32(acc[e]);
    *reinterpret_cast<v8h*>(out + (size_t)t * K + c) = o;
  }
}

extern "C" {

size_t mxmoe_permute_workspace_bytes(int total, int num_experts) {
  const size_t blocks = (size_t)(total + kPermChunk - 1) / kPermChunk;
  return ((size_t)perm_hist_stride((int)blocks) * num_experts + num_experts) * sizeof(int32_t);
}

static int build_permutation_impl(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices,
                                  int64_t* src_slot, int64_t* recv_tokens_per_exp, int32_t* hist, hipStream_t s, int32_t* row_of_slot = nullptr) {
  const int total = num_tokens * topk;
  const int blocks = (total + kPermChunk - 1) / kPermChunk;
  int nbits = 1;
  while ((1 << nbits) <= num_experts) ++nbits;  // ids 0..E (E = parked lanes)
  const size_t lds = (size_t)num_experts * sizeof(int32_t);
  if (blocks == 1) {
    hipLaunchKernelGGL(perm_small_kernel, dim3(1), dim3(64), lds, s, topk_ids, total, num_experts, topk, nbits, recv_tokens_per_exp, dst_exp_sorted, perm_indices, src_slot,
                       row_of_slot);
  } else {
    // few workgroups and experts: the scatter workgroups sum the counts they need themselves, which saves the scan launch
    // (the 16-byte loads of that path need an aligned workspace; any other goes the three-launch way)
    const int raw = (long)blocks * num_experts <= kPermFusedScanMax && (reinterpret_cast<uintptr_t>(hist) & 15) == 0;
    launch_perm_hist(topk_ids, total, num_experts, hist, raw != 0, s);
    if (!raw) hipLaunchKernelGGL(perm_scan_kernel, dim3(num_experts), dim3(64), 0, s, hist, blocks, num_experts, recv_tokens_per_exp);
    hipLaunchKernelGGL(perm_scatter_kernel, dim3(blocks), dim3(64), lds, s, topk_ids, total, num_experts, topk, nbits, hist, raw, recv_tokens_per_exp, dst_exp_sorted,
                       perm_indices, src_slot, row_of_slot);
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

static int check_permutation_args(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, const int32_t* dst_exp_sorted, const int64_t* perm_indices,
                                  const int64_t* src_slot, const int64_t* recv_tokens_per_exp) {
  if (num_tokens <= 0 || topk <= 0 || (long)num_tokens * topk > (1l << 30) || num_experts <= 0 || num_experts > 4096) {
    last_error() = "bad permutation size";
    return 3;
  }
  if (!topk_ids || !dst_exp_sorted || !perm_indices || !src_slot || !recv_tokens_per_exp) {
    last_error() = "null pointer";
    return 5;
  }
  return 0;
}

int mxmoe_route_topk(const void* router_logits, int logits_dtype, int num_tokens, int num_experts, int topk, int renormalise, int32_t* topk_ids,
                     float* topk_weights, void* stream) {
  if (num_tokens < 0 || num_experts <= 0 || num_experts > 4096 || topk <= 0 || topk > num_experts || topk > 64 || logits_dtype < 0 || logits_dtype > 2) {
    last_error() = "routing takes 1..4096 experts, top-k of at most min(experts, 64), logits as fp16 (0), fp32 (1) or bf16 (2)";
    return 3;
  }
  if (num_tokens == 0) return 0;
  if (!router_logits || !topk_ids || !topk_weights) {
    last_error() = "null pointer";
    return 5;
  }
  RouteArgs a;
  a.logits = router_logits;
  a.dtype = logits_dtype;
  a.T = num_tokens;
  a.E = num_experts;
  a.topk = topk;
  a.renorm = renormalise != 0;
  a.ids = topk_ids;
  a.weights = topk_weights;
  hipLaunchKernelGGL(route_topk_kernel, dim3((num_tokens + 3) / 4), dim3(256), (size_t)4 * num_experts * sizeof(float), (hipStream_t)stream, a);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

int mxmoe_build_permutation(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices,
                            int64_t* src_slot, int64_t* recv_tokens_per_exp, void* workspace, void* stream) {
  if (const int rc = check_permutation_args(topk_ids, num_tokens, topk, num_experts, dst_exp_sorted, perm_indices, src_slot, recv_tokens_per_exp)) return rc;
  if (!workspace) {
    last_error() = "null pointer";
    return 5;
  }
  return build_permutation_impl(topk_ids, num_tokens, topk, num_experts, dst_exp_sorted, perm_indices, src_slot, recv_tokens_per_exp,
                                reinterpret_cast<int32_t*>(workspace), (hipStream_t)stream);
}

int mxmoe_build_permutation_inv(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices,
                                int64_t* src_slot, int64_t* recv_tokens_per_exp, int32_t* row_of_slot, void* workspace, void* stream) {
  if (const int rc = check_permutation_args(topk_ids, num_tokens, topk, num_experts, dst_exp_sorted, perm_indices, src_slot, recv_tokens_per_exp)) return rc;
  if (!workspace || !row_of_slot) {
    last_error() = "null pointer";
    return 5;
  }
  return build_permutation_impl(topk_ids, num_tokens, topk, num_experts, dst_exp_sorted, perm_indices, src_slot, recv_tokens_per_exp,
                                reinterpret_cast<int32_t*>(workspace), (hipStream_t)stream, row_of_slot);
}

// ---- the permutation for callers that may not allocate: the per-block histograms live in a static device array ----
constexpr size_t kStaticScratchInts = 256 * 1024;  // 1 MiB per device, held until the process ends
static __device__ __align__(256) int32_t scratch[kStaticScratchInts];

size_t mxmoe_static_scratch_bytes(void) { return kStaticScratchInts * sizeof(int32_t); }

int mxmoe_build_permutation_static(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices,
                                   int64_t* src_slot, int64_t* recv_tokens_per_exp, void* stream) {
  if (const int rc = check_permutation_args(topk_ids, num_tokens, topk, num_experts, dst_exp_sorted, perm_indices, src_slot, recv_tokens_per_exp)) return rc;
  const size_t need = mxmoe_permute_workspace_bytes(num_tokens * topk, num_experts);
  if (need > mxmoe_static_scratch_bytes()) {
    char buf[200];
    snprintf(buf, sizeof buf, "permutation of %d rows over %d experts needs %zu bytes of scratch, the static buffer holds %zu: use mxmoe_build_permutation with a workspace",
             num_tokens * topk, num_experts, need, mxmoe_static_scratch_bytes());
    last_error() = buf;
    return 3;
  }
  // every device has its own copy of the array at its own address; `scratch` itself is only a host-side handle for the lookup
  static int32_t* device_ptr[64] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    last_error() = "no current HIP device";
    return 4;
  }
  if (!device_ptr[dev]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      last_error() = std::string("hipGetSymbolAddress(scratch) failed: ") + hipGetErrorString(e);
      return 4;
    }
    device_ptr[dev] = reinterpret_cast<int32_t*>(p);
  }
  // nothing needs clearing: perm_hist_kernel writes every counter the later kernels read
  return build_permutation_impl(topk_ids, num_tokens, topk, num_experts, dst_exp_sorted, perm_indices, src_slot, recv_tokens_per_exp, device_ptr[dev], (hipStream_t)stream);
}

static int fill_common(RowArgs& a, int n, int n_shared, int had_k, int had_f, const float* signs) {
  const bool rot = a.rotate != 0;
  if (n % 8 || (n_shared % 8)) {
    last_error() = "row length must be a multiple of 8";
    return 3;
  }
  if (make_plan(n, had_k, had_f, rot, &a.plan) || make_plan(n_shared > 0 ? n_shared : n, had_k, had_f, rot, &a.plan_shared)) {
    last_error() = "row length is not (Hadamard order) x (power of two >= 8)";
    return 3;
  }
  a.signs = a.plan.kb > 1 ? signs : nullptr;
  if (a.plan.kb > 1 && !signs) {
    last_error() = "missing Hadamard sign table";
    return 3;
  }
  return 0;
}

int mxmoe_quant_act(const void* hidden, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const int64_t* perm_indices, const int64_t* exp_table,
                    int K, int rows_routed, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f, const float* had_signs, void* stream) {
  const bool variants = (rotate & 4) != 0;
  rotate &= 3;
  if (rows_routed < 0 || num_tokens < 0 || num_experts <= 0) {
    last_error() = "bad row or expert count";
    return 3;
  }
  if (!hidden || !inp_store || !exp_table || (rows_routed > 0 && (!dst_exp_sorted || !perm_indices))) {
    last_error() = "null pointer";
    return 5;
  }
  RowArgs a{};
  a.src = a.src_shared = reinterpret_cast<const _Float16*>(hidden);
  a.inp_store = reinterpret_cast<uint8_t*>(inp_store);
  a.scale_store = reinterpret_cast<_Float16*>(scale_store);
  a.dst_exp = dst_exp_sorted;
  a.perm = perm_indices;
  a.table = exp_table;
  a.R = rows_routed;
  a.T = num_tokens;
  a.E = num_experts;
  a.Et = num_experts + (has_shared ? 1 : 0);
  a.rows = rows_routed + (has_shared ? num_tokens : 0);
  a.rotate = rotate;
  if (a.rows == 0) return 0;
  if (const int rc = fill_common(a, K, K, rotate ? had_k : 1, rotate ? had_f : 1, had_signs)) return rc;
  const int lds = (K + a.plan.kb * a.plan.kb + 16) * (int)sizeof(float);
  return launch_rows<false>(a, lds, (hipStream_t)stream, variants);
}

int mxmoe_silu_mul_quant(const void* gate_up, const void* gate_up_shared, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const int64_t* exp_table,
                         int N, int N_shared, int rows_routed, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f,
                         const float* had_signs, void* stream) {
  const bool variants = (rotate & 4) != 0;
  rotate &= 3;
  if (rows_routed < 0 || num_tokens < 0 || num_experts <= 0) {
    last_error() = "bad row or expert count";
    return 3;
  }
  if (!gate_up || !inp_store || !exp_table || (rows_routed > 0 && !dst_exp_sorted) || (has_shared && !gate_up_shared)) {
    last_error() = "null pointer";
    return 5;
  }
  RowArgs a{};
  a.src = reinterpret_cast<const _Float16*>(gate_up);
  a.src_shared = reinterpret_cast<const _Float16*>(gate_up_shared);
  a.inp_store = reinterpret_cast<uint8_t*>(inp_store);
  a.scale_store = reinterpret_cast<_Float16*>(scale_store);
  a.dst_exp = dst_exp_sorted;
  a.perm = nullptr;
  a.table = exp_table;
  a.R = rows_routed;
  a.T = num_tokens;
  a.E = num_experts;
  a.Et = num_experts + (has_shared ? 1 : 0);
  a.rows = rows_routed + (has_shared ? num_tokens : 0);
  a.rotate = rotate;
  if (a.rows == 0) return 0;
  if (const int rc = fill_common(a, N, has_shared ? N_shared : N, rotate ? had_k : 1, rotate ? had_f : 1, had_signs)) return rc;
  const int nmax = N > a.plan_shared.n ? N : a.plan_shared.n;
  const int lds = (nmax + a.plan.kb * a.plan.kb + 16) * (int)sizeof(float);
  return launch_rows<true>(a, lds, (hipStream_t)stream, variants);
}

int mxmoe_quant_act_tokens(const void* hidden, void* inp_store, void* scale_store, const int32_t* topk_ids, const int32_t* row_of_slot, const int64_t* exp_table,
                           int K, int num_tokens, int topk, int num_experts, int has_shared, int rotate, void* stream) {
  if (num_tokens < 0 || num_experts <= 0 || topk < 0 || topk > kTokenMaxTopk) {
    last_error() = "bad token or expert count, or more than 8 slots per token";
    return 3;
  }
  if (K < 512 || K > 4096 || (K & (K - 1))) {
    last_error() = "the per-token prologue takes rows of 512, 1024, 2048 or 4096 values";
    return 3;
  }
  if (rotate < 0 || rotate > 2) {
    last_error() = "rotate is 0, 1 or 2 (tables with operand-variant tags go through mxmoe_quant_act)";
    return 3;
  }
  if (!hidden || !inp_store || !exp_table || (topk > 0 && (!topk_ids || !row_of_slot))) {
    last_error() = "null pointer";
    return 5;
  }
  if (num_tokens == 0 || topk + has_shared == 0) return 0;
  TokenArgs a{};
  a.src = reinterpret_cast<const _Float16*>(hidden);
  a.inp_store = reinterpret_cast<uint8_t*>(inp_store);
  a.scale_store = reinterpret_cast<_Float16*>(scale_store);
  a.ids = topk_ids;
  a.row_of_slot = row_of_slot;
  a.table = exp_table;
  a.T = num_tokens;
  a.E = num_experts;
  a.Et = num_experts + (has_shared ? 1 : 0);
  a.topk = topk;
  a.has_shared = has_shared ? 1 : 0;
  a.rotate = rotate;
  a.scale = 1.0f / sqrtf((float)K);
  int dev = 0, cus = 256;
  (void)hipGetDevice(&dev);
  (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  // (a multiple of 64 workgroups: xcd_row_group permutes within runs of 64)
  const int grid = ((num_tokens + 3) / 4 < cus * 8 ? (num_tokens + 3) / 4 : cus * 8) + 63 & ~63;
  hipStream_t s = (hipStream_t)stream;
  switch (K / 512) {
    case 1: hipLaunchKernelGGL((token_quant_wave_kernel<1>), dim3(grid), dim3(256), 0, s, a); break;
    case 2: hipLaunchKernelGGL((token_quant_wave_kernel<2>), dim3(grid), dim3(256), 0, s, a); break;
    case 4: hipLaunchKernelGGL((token_quant_wave_kernel<4>), dim3(grid), dim3(256), 0, s, a); break;
    default: hipLaunchKernelGGL((token_quant_wave_kernel<8>), dim3(grid), dim3(256), 0, s, a); break;
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

// ---- the same three steps behind a device-side plan (mxmoe_plan_block): nothing here depends on the routing ----
int mxmoe_quant_act_planned(const void* hidden, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const int64_t* perm_indices, const void* d_plan,
                            int K, int rows_capacity, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f, const float* had_signs,
                            void* stream) {
  const bool variants = (rotate & 4) != 0;
  rotate &= 3;
  if (rows_capacity <= 0 || num_tokens < 0 || num_experts <= 0) {
    last_error() = "bad row or expert count";
    return 3;
  }
  if (!hidden || !inp_store || !d_plan || !dst_exp_sorted || !perm_indices) {
    last_error() = "null pointer";
    return 5;
  }
  const int et = num_experts + (has_shared ? 1 : 0);
  const PlanLayout lay(et);
  const uint8_t* plan = reinterpret_cast<const uint8_t*>(d_plan);
  RowArgs a{};
  a.src = a.src_shared = reinterpret_cast<const _Float16*>(hidden);
  a.inp_store = reinterpret_cast<uint8_t*>(inp_store);
  a.scale_store = reinterpret_cast<_Float16*>(scale_store);
  a.dst_exp = dst_exp_sorted;
  a.perm = perm_indices;
  a.table = reinterpret_cast<const int64_t*>(plan + lay.table);
  a.routed_ptr = reinterpret_cast<const int64_t*>(plan + lay.misc);
  a.R = rows_capacity;
  a.T = num_tokens;
  a.E = num_experts;
  a.Et = et;
  a.rows = rows_capacity + (has_shared ? num_tokens : 0);
  a.rotate = rotate;
  if (const int rc = fill_common(a, K, K, rotate ? had_k : 1, rotate ? had_f : 1, had_signs)) return rc;
  const int lds = (K + a.plan.kb * a.plan.kb + 16) * (int)sizeof(float);
  return launch_rows<false>(a, lds, (hipStream_t)stream, variants);
}

int mxmoe_silu_mul_quant_planned(const void* gate_up, const void* d_plan_gate_up, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const void* d_plan,
                                 int N, int N_shared, int rows_capacity, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f,
                                 const float* had_signs, void* stream) {
  const bool variants = (rotate & 4) != 0;
  rotate &= 3;
  if (rows_capacity <= 0 || num_tokens < 0 || num_experts <= 0) {
    last_error() = "bad row or expert count";
    return 3;
  }
  if (!gate_up || !inp_store || !d_plan || !dst_exp_sorted || !d_plan_gate_up) {
    last_error() = "null pointer";
    return 5;
  }
  const int et = num_experts + (has_shared ? 1 : 0);
  const PlanLayout lay(et);
  const uint8_t* plan = reinterpret_cast<const uint8_t*>(d_plan);
  RowArgs a{};
  a.src = reinterpret_cast<const _Float16*>(gate_up);
  a.src_shared = nullptr;
  // the shared expert's gate_up rows are the output of problem E of the first launch: the planner of that launch left their address
  a.shared_src_addr = has_shared ? reinterpret_cast<const int64_t*>(reinterpret_cast<const uint8_t*>(d_plan_gate_up) + lay.misc) + 1 : nullptr;
  a.inp_store = reinterpret_cast<uint8_t*>(inp_store);
  a.scale_store = reinterpret_cast<_Float16*>(scale_store);
  a.dst_exp = dst_exp_sorted;
  a.perm = nullptr;
  a.table = reinterpret_cast<const int64_t*>(plan + lay.table);
  a.routed_ptr = reinterpret_cast<const int64_t*>(plan + lay.misc);
  a.R = rows_capacity;
  a.T = num_tokens;
  a.E = num_experts;
  a.Et = et;
  a.rows = rows_capacity + (has_shared ? num_tokens : 0);
  a.rotate = rotate;
  if (const int rc = fill_common(a, N, has_shared ? N_shared : N, rotate ? had_k : 1, rotate ? had_f : 1, had_signs)) return rc;
  const int nmax = N > a.plan_shared.n ? N : a.plan_shared.n;
  const int lds = (nmax + a.plan.kb * a.plan.kb + 16) * (int)sizeof(float);
  return launch_rows<true>(a, lds, (hipStream_t)stream, variants);
}

size_t mxmoe_combine_workspace_bytes(int num_tokens, int topk) { return (size_t)num_tokens * topk * sizeof(int32_t); }

int mxmoe_unpermute_combine(const void* down_out, const void* shared_out, const float* topk_weights, const int64_t* src_slot, int rows, int num_tokens, int topk,
                            int K, void* out, void* workspace, void* stream) {
  if (num_tokens <= 0 || topk <= 0 || K <= 0 || K % 8 || rows < 0 || rows > num_tokens * topk) {
    last_error() = "bad combine size (K must be a multiple of 8, rows <= tokens * topk)";
    return 3;
  }
  if (!down_out || !topk_weights || !src_slot || !out || !workspace) {
    last_error() = "null pointer";
    return 5;
  }
  hipStream_t s = (hipStream_t)stream;
  const int slots = num_tokens * topk;
  int32_t* row_of_slot = reinterpret_cast<int32_t*>(workspace);
  hipLaunchKernelGGL(combine_fill_kernel, dim3((slots + 255) / 256), dim3(256), 0, s, row_of_slot, slots);
  if (rows > 0) hipLaunchKernelGGL(combine_invert_kernel, dim3((rows + 255) / 256), dim3(256), 0, s, src_slot, rows, slots, row_of_slot, (const int64_t*)nullptr);
  hipLaunchKernelGGL(combine_kernel, dim3(num_tokens), dim3(256), 0, s, reinterpret_cast<const _Float16*>(down_out), reinterpret_cast<const _Float16*>(shared_out),
                     topk_weights, row_of_slot, topk, K, reinterpret_cast<_Float16*>(out), (const int64_t*)nullptr);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

int mxmoe_combine_planned(const void* down_out, const void* d_plan_down, int num_problems, const float* topk_weights, const int32_t* row_of_slot, int num_tokens,
                          int topk, int K, void* out, void* stream) {
  if (num_tokens <= 0 || topk <= 0 || K <= 0 || K % 8 || num_problems <= 0) {
    last_error() = "bad combine size (K must be a multiple of 8)";
    return 3;
  }
  if (!down_out || !d_plan_down || !topk_weights || !row_of_slot || !out) {
    last_error() = "null pointer";
    return 5;
  }
  const int64_t* misc = reinterpret_cast<const int64_t*>(reinterpret_cast<const uint8_t*>(d_plan_down) + mxmoe::PlanLayout(num_problems).misc);
  hipLaunchKernelGGL(combine_kernel, dim3(num_tokens), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<const _Float16*>(down_out), (const _Float16*)nullptr, topk_weights,
                     row_of_slot, topk, K, reinterpret_cast<_Float16*>(out), misc + 1);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

int mxmoe_unpermute_combine_planned(const void* down_out, const void* d_plan_down, int num_problems, const float* topk_weights, const int64_t* src_slot, int num_tokens,
                                    int topk, int K, void* out, void* workspace, void* stream) {
  if (num_tokens <= 0 || topk <= 0 || K <= 0 || K % 8 || num_problems <= 0) {
    last_error() = "bad combine size (K must be a multiple of 8)";
    return 3;
  }
  if (!down_out || !d_plan_down || !topk_weights || !src_slot || !out || !workspace) {
    last_error() = "null pointer";
    return 5;
  }
  hipStream_t s = (hipStream_t)stream;
  const int slots = num_tokens * topk;
  const int64_t* misc = reinterpret_cast<const int64_t*>(reinterpret_cast<const uint8_t*>(d_plan_down) + PlanLayout(num_problems).misc);
  int32_t* row_of_slot = reinterpret_cast<int32_t*>(workspace);
  hipLaunchKernelGGL(combine_fill_kernel, dim3((slots + 255) / 256), dim3(256), 0, s, row_of_slot, slots);
  hipLaunchKernelGGL(combine_invert_kernel, dim3((slots + 255) / 256), dim3(256), 0, s, src_slot, slots, slots, row_of_slot, misc);
  hipLaunchKernelGGL(combine_kernel, dim3(num_tokens), dim3(256), 0, s, reinterpret_cast<const _Float16*>(down_out), (const _Float16*)nullptr, topk_weights, row_of_slot,
                     topk, K, reinterpret_cast<_Float16*>(out), misc + 1);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

}  // extern "C"
