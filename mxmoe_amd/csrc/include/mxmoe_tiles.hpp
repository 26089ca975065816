// gfx950 (CDNA4) workgroup-level GEMM tiles for the fused mixed-precision MoE GroupGEMM.
//
// Every tile is a 256-thread workgroup (4 wavefronts of 64 lanes) so that tiles of different formats can
// share one launch, the way the reference requires equal warp counts across fused branches
// (mxmoe/kernels/compose_kernel.py:69-71).  The MFMA tiles here play the role of the reference's
// cta_gemm_multistage_qab_v2 / cta_gemm_multistage_v2 (mxmoe/kernels/src/include/cta_gemm.cuh:424-608, 8-107)
// but are laid out for 64-wide waves:
//
//  * weights [N,K] are the MFMA "A" operand (rows = output channels) and activations [M,K] the "B"
//    operand (columns = tokens), so each lane ends up with 4 consecutive output channels per
//    accumulator quad and the epilogue stores 8 contiguous bytes per lane;
//  * both operands are staged through LDS in 64-byte row slices, 16-byte chunks XOR-swizzled so that
//    the 8 lanes served together by a ds_read_b128 / ds_write_b128 hit 8 distinct 16-byte bank groups;
//  * int4 operands stay packed in HBM and LDS (two values per byte, even element in the low nibble)
//    and are widened in registers to int8 holding 16*v (one shift + two ANDs per dword); the int32
//    accumulator then holds 256 * sum(a*b) exactly and the epilogue shifts it back down.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxmoe_types.h"

namespace mxmoe {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;  // workgroup size shared by every fused branch
constexpr int kWaves = 4;
constexpr int kRowBytes = 64;  // bytes of one operand row held in LDS per pipeline stage

enum class Op { I8, I4, F16 };

// What one problem looks like to a tile.
struct TileArgs {
  const uint8_t* A;      // activations  [M, K]  (int8 / packed int4 / fp16), K contiguous
  const uint8_t* B;      // weights      [N, K]
  const _Float16* sa;    // per-token scales   [M]   (w-a formats)
  const _Float16* sb;    // per-channel scales [N]   (w-a formats) or group scale/zero table (weight-only)
  _Float16* C;           // output [M, N] fp16 row-major
  int32_t* acc_dump;     // optional [M, N] int32 / fp32-bits accumulator dump (tests), may be null
  int M, N, K;
  int tile_m, tile_n;
};

// Keeps a freshly computed fp32 value opaque to the optimiser.  Without it the compiler folds "fp32 multiply, then convert to
// fp16" into one v_fma_mixlo_f16, which rounds the exact product once; the reference arithmetic (and its CPU restatement) rounds
// to fp32 first and to fp16 second, and the two differ on ties.
__device__ __forceinline__ float keep_f32(float v) {
  asm volatile("" : "+v"(v));
  return v;
}

// LDS byte offset of 16-byte chunk `c` (0..3) of tile row `r`.  Rows are 64 bytes; the chunk index is XORed with
// bits 1..2 of the row so rows r, r+1 (which share a 128-byte bank line) and the next three row pairs all land
// on different 16-byte groups.
__device__ __forceinline__ int lds_chunk_off(int r, int c) { return r * kRowBytes + ((c ^ ((r >> 1) & 3)) << 4); }

template <Op OP>
struct OpTraits;
template <>
struct OpTraits<Op::I8> {
  using Acc = v16i;
  static constexpr int kBitsPerElem = 8;
};
template <>
struct OpTraits<Op::I4> {
  using Acc = v16i;
  static constexpr int kBitsPerElem = 4;
};
template <>
struct OpTraits<Op::F16> {
  using Acc = v16f;
  static constexpr int kBitsPerElem = 16;
};

// A BM x BN output tile computed by WGM x WGN waves with 32x32 MFMA blocks.
template <Op OP, int BM_, int BN_, int WGM_, int WGN_>
struct MfmaTile {
  static constexpr Op kOp = OP;
  static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
  static_assert(WGM * WGN == kWaves, "a tile is always 4 waves");
  static constexpr int TM = BM / WGM, TN = BN / WGN;  // per-wave output
  static constexpr int FM = TM / 32, FN = TN / 32;    // 32x32 MFMA blocks per wave
  static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA block");
  static constexpr int kBits = OpTraits<OP>::kBitsPerElem;
  static constexpr int BK = kRowBytes * 8 / kBits;  // K elements per pipeline stage: 64 (int8), 128 (int4), 32 (fp16)
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static constexpr int A_CHUNKS = BM * 4, B_CHUNKS = BN * 4;
  static constexpr int A_IT = (A_CHUNKS + kThreads - 1) / kThreads, B_IT = (B_CHUNKS + kThreads - 1) / kThreads;
  using Acc = typename OpTraits<OP>::Acc;

  __device__ static __forceinline__ void run(const TileArgs& t, uint8_t* __restrict__ smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int M = t.M, N = t.N;
    const long row_bytes = (long)t.K * kBits / 8;
    const int KT = (int)(row_bytes / kRowBytes);
    const int m0 = t.tile_m * BM, n0 = t.tile_n * BN;

    // ---- global -> register -> LDS staging plan: thread owns 16-byte chunk (row = idx/4, chunk = idx%4) ----
    const uint8_t* ga[A_IT];
    const uint8_t* gb[B_IT];
    int la[A_IT], lb[B_IT];
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
      const int idx = tid + i * kThreads;
      const int r = idx >> 2, c = idx & 3;
      const int gr = min(m0 + r, M - 1);  // tail rows re-read the last valid row; their results are never stored
      ga[i] = t.A + (long)gr * row_bytes + c * 16;
      la[i] = lds_chunk_off(r, c);
    }
#pragma unroll
    for (int i = 0; i < B_IT; ++i) {
      const int idx = tid + i * kThreads;
      const int r = idx >> 2, c = idx & 3;
      const int gr = min(n0 + r, N - 1);
      gb[i] = t.B + (long)gr * row_bytes + c * 16;
      lb[i] = BM * kRowBytes + lds_chunk_off(r, c);
    }
    v4i ra[A_IT], rb[B_IT];

    auto g_load = [&](int kt) {
#pragma unroll
      for (int i = 0; i < A_IT; ++i)
        if (A_CHUNKS % kThreads == 0 || tid + i * kThreads < A_CHUNKS) ra[i] = *reinterpret_cast<const v4i*>(ga[i] + (long)kt * kRowBytes);
#pragma unroll
      for (int i = 0; i < B_IT; ++i)
        if (B_CHUNKS % kThreads == 0 || tid + i * kThreads < B_CHUNKS) rb[i] = *reinterpret_cast<const v4i*>(gb[i] + (long)kt * kRowBytes);
    };
    auto s_store = [&](int stage) {
      uint8_t* s = smem + stage * kStageBytes;
#pragma unroll
      for (int i = 0; i < A_IT; ++i)
        if (A_CHUNKS % kThreads == 0 || tid + i * kThreads < A_CHUNKS) *reinterpret_cast<v4i*>(s + la[i]) = ra[i];
#pragma unroll
      for (int i = 0; i < B_IT; ++i)
        if (B_CHUNKS % kThreads == 0 || tid + i * kThreads < B_CHUNKS) *reinterpret_cast<v4i*>(s + lb[i]) = rb[i];
    };

    // ---- LDS -> MFMA fragment plan: lane reads row (lane & 31) of a 32-row block, chunk 2*ks + (lane >> 5) ----
    const int lrow = lane & 31;
    const int swz = (lrow >> 1) & 3;
    const int c0 = (((lane >> 5) ^ swz) << 4);  // k-step 0; k-step 1 is c0 ^ 32
    const int fa = (wm * TM + lrow) * kRowBytes + c0;
    const int fb = BM * kRowBytes + (wn * TN + lrow) * kRowBytes + c0;

    Acc acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    g_load(0);
    s_store(0);
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
      const bool more = kt + 1 < KT;
      if (more) g_load(kt + 1);
      const uint8_t* s = smem + (kt & 1) * kStageBytes;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        v4i af[FM], bf[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) af[i] = *reinterpret_cast<const v4i*>(s + ((fa + i * 32 * kRowBytes) ^ (ks << 5)));
#pragma unroll
        for (int j = 0; j < FN; ++j) bf[j] = *reinterpret_cast<const v4i*>(s + ((fb + j * 32 * kRowBytes) ^ (ks << 5)));
        if constexpr (OP == Op::I8) {
#pragma unroll
          for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], acc[i][j], 0, 0, 0);
        } else if constexpr (OP == Op::I4) {
          // nibble n of a byte -> int8 holding 16 * signed(n): even elements via (x << 4), odd via x, both masked to the high nibbles
          v4i alo[FM], ahi[FM], blo[FN], bhi[FN];
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            alo[i] = (af[i] << 4) & (int)0xF0F0F0F0;
            ahi[i] = af[i] & (int)0xF0F0F0F0;
          }
#pragma unroll
          for (int j = 0; j < FN; ++j) {
            blo[j] = (bf[j] << 4) & (int)0xF0F0F0F0;
            bhi[j] = bf[j] & (int)0xF0F0F0F0;
          }
#pragma unroll
          for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) {
              acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(blo[j], alo[i], acc[i][j], 0, 0, 0);
              acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bhi[j], ahi[i], acc[i][j], 0, 0, 0);
            }
        } else {
#pragma unroll
          for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, bf[j]), __builtin_bit_cast(v8h, af[i]), acc[i][j], 0, 0, 0);
        }
      }
      if (more) s_store((kt + 1) & 1);
      __syncthreads();
    }

    // ---- epilogue.  Lane holds token m = lane & 31 and channels 8*(r/4) + 4*(lane >> 5) + (r & 3) of each 32x32 block ----
    const int nq = (lane >> 5) * 4;
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = m0 + wm * TM + i * 32 + lrow;
      if (m >= M) continue;
      _Float16 s_a = (_Float16)1.0f;
      if constexpr (OP != Op::F16) s_a = t.sa[m];
#pragma unroll
      for (int j = 0; j < FN; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * TN + j * 32 + q * 8 + nq;
          if (n >= N) continue;  // N is a multiple of 4, so a quad is all-in or all-out
          v4h o;
          if constexpr (OP == Op::F16) {
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (_Float16)acc[i][j][q * 4 + e];
          } else {
            const v4h s_b = *reinterpret_cast<const v4h*>(t.sb + n);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              int a = acc[i][j][q * 4 + e];
              if constexpr (OP == Op::I4) a >>= 8;  // exact: the accumulator is 256 * sum
              // float(acc) * (sa * sb) rounded to half, as the reference epilogue (mm_tile.cuh:490-493, 642-646) except that the
              // scale product stays in fp32, where it is exact: the reference rounds it to fp16 first, which turns subnormal
              // (a few significant bits) for typical int8 scales and breaks the 1e-2 agreement with the fake-quant path.
              const float s = (float)s_a * (float)s_b[e];
              o[e] = (_Float16)keep_f32((float)a * s);
              if (t.acc_dump) t.acc_dump[(long)m * N + n + e] = a;
            }
          }
          if constexpr (OP == Op::F16) {
            if (t.acc_dump) {
#pragma unroll
              for (int e = 0; e < 4; ++e) t.acc_dump[(long)m * N + n + e] = __builtin_bit_cast(int, acc[i][j][q * 4 + e]);
            }
          }
          *reinterpret_cast<v4h*>(t.C + (long)m * N + n) = o;
        }
      }
    }
  }
};

}  // namespace mxmoe
