// WxAxGTile: w4a4 with group-128 symmetric scales on both operands (w4a4_g128_sym).
//
// Every K slice of the int4 tiles is 128 values = one quantisation group, so the integer accumulators of a slice are complete
// per-group sums: after each slice they are converted, multiplied by the product of the token's and the channel's scale of that
// group and added to fp32 accumulators, groups in ascending order (the reference rescales each group's integer fragment into an
// fp32 fragment the same way, mxmoe/kernels/src/include/cta_gemm.cuh:613-772).
//
// Operands: activations int4 rows [M, K/2] with scales [M, K/128]; weights in MFMA fragment order as for w4a4 (mxmoe_tiles.hpp,
// WxAxTile) with scales stored group-major [K/128, N], so that the scales of a tile's channels for one group are contiguous.
// BM x 256 outputs per workgroup, 4 waves x 64 channels.  Activations go global -> registers -> LDS (3-stage ring, one barrier
// per slice), weights global -> registers two slices ahead, a group's scales global -> registers at the start of its slice; every load is an ordinary
// load whose waits the compiler places.  Indices past the ends (rows past M, channel blocks past N, slices past K) are clamped
// to the last valid one: such results are computed and never stored.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxmoe_tiles.hpp"

namespace mxmoe {

template <int BM_>
struct WxAxGTile {
  static constexpr int BM = BM_, BN = 256, BK = 128;
  static constexpr int FM = BM / 32, FN = 2;
  static_assert(BM == 32 || BM == 64, "two sets of accumulators (int32 per group, fp32 running sum) must fit 256 registers");
  static constexpr int kStageBytes = BM * kRowBytes, kStages = 3;
  static constexpr int kLdsBytes = kStages * kStageBytes;
  static constexpr int kAccRegs = 2 * FM * FN * 16;
  static constexpr int kWavesWanted = 2;  // waves per SIMD a kernel of such tiles is compiled for
  static constexpr int kABits = 4, kWBits = 4;  // bits per activation / weight element
  static constexpr int kPieces = BM / 16;                       // 1 KB pieces (16 rows) of one activation slice
  static constexpr int kQ = (kPieces + kWaves - 1) / kWaves;    // pieces a wave copies per slice

  __device__ static __forceinline__ void run(const TileArgs& t, uint8_t* __restrict__ smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = t.M, N = t.N;
    const int G = t.K / 128;  // K slices = quantisation groups
    const long row_bytes = t.K / 2;
    const int m0 = t.row0 + t.tile_m * BM, n0 = t.tile_n * BN;
    const int lrow = lane & 31, nq = (lane >> 5) * 4;

    // ---- activations: global -> registers -> LDS ----
    const uint8_t* a_src[kQ];
    int a_lds[kQ];
    bool a_mine[kQ];
#pragma unroll
    for (int q = 0; q < kQ; ++q) {
      const int piece = wave + kWaves * q;
      a_mine[q] = piece < kPieces;
      const int row = (a_mine[q] ? piece : 0) * 16 + (lane >> 2);
      a_src[q] = t.A + (long)min(m0 + row, M - 1) * row_bytes + (lane & 3) * 16;
      a_lds[q] = row * kRowBytes + (((lane & 3) ^ lds_swizzle(row)) << 4);
    }
    auto a_gload = [&](int kt, v4i (&r)[kQ]) {
#pragma unroll
      for (int q = 0; q < kQ; ++q) r[q] = gload<v4i>(a_src[q] + (long)min(kt, G - 1) * kRowBytes);
    };
    auto a_swrite = [&](int stage, const v4i (&r)[kQ]) {
#pragma unroll
      for (int q = 0; q < kQ; ++q)
        if (a_mine[q]) *reinterpret_cast<v4i*>(smem + stage * kStageBytes + a_lds[q]) = r[q];
    };
    const int fa = lrow * kRowBytes;
    const int sw = lds_swizzle(lrow);
    auto a_sread = [&](int stage, int step, int i) {
      return *reinterpret_cast<const v4i*>(smem + stage * kStageBytes + fa + i * 32 * kRowBytes + ((((lane >> 5) + 2 * step) ^ sw) << 4));
    };

    // ---- weights: fragment (block j, k-step s) of slice kt at ((nb * G + kt) * 2 + s) * 1 KB ----
    const int nblk = (N + 31) / 32;
    const uint8_t* bptr[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) bptr[j] = t.B + (long)min(n0 / 32 + wave * FN + j, nblk - 1) * G * 2048 + lane * 16;
    auto b_gload = [&](int j, int s, int kt) { return gload<v4i>(bptr[j] + ((long)min(kt, G - 1) * 2 + s) * 1024); };

    // ---- scales of one group: token scales of the lane's rows, channel scales of its 4-channel runs ----
    const _Float16* sa_ptr[FM];
#pragma unroll
    for (int i = 0; i < FM; ++i) sa_ptr[i] = t.sa + (long)min(m0 + i * 32 + lrow, M - 1) * G;
    // channel scales: the lane's first run of 4 channels; the others sit 8 channels (16 bytes) apart and are clamped one by one
    const int nbase = n0 + wave * 64 + nq;
    auto s_gload = [&](int kt, _Float16 (&sa_h)[FM], v4h (&sb_h)[FN][4]) {
      const int g = min(kt, G - 1);
#pragma unroll
      for (int i = 0; i < FM; ++i) sa_h[i] = gload<_Float16>(sa_ptr[i] + g);
      const _Float16* sbg = t.sb + (long)g * N;
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) sb_h[j][q] = gload<v4h>(sbg + min(nbase + j * 32 + q * 8, N - 4));
    };

    v16f facc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) facc[i][j][r] = 0.0f;

    v4i stg[2][kQ];       // activation slices kt+1 / kt+2 on their way to LDS
    v4i wb[2][FN][2];     // packed weight fragments of slices kt, kt+1 (slot = slice parity)

    a_gload(0, stg[0]);
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int s = 0; s < 2; ++s) wb[d][j][s] = b_gload(j, s, d);
    a_swrite(0, stg[0]);
    a_gload(1, stg[1]);
    __syncthreads();

    auto slice = [&](auto dc, int kt, int stage) {
      constexpr int d = decltype(dc)::value;
      const int nstage = stage == kStages - 1 ? 0 : stage + 1;
      a_swrite(nstage, stg[(d + 1) & 1]);  // slice kt+1, fetched during the previous slice
      a_gload(kt + 2, stg[d & 1]);
      // this group's scales: used after the slice's MFMAs, which cover the load
      _Float16 sa_c[FM];
      v4h sb_c[FN][4];
      s_gload(kt, sa_c, sb_c);
      v16i iacc[FM][FN];
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) iacc[i][j][r] = 0;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        v4i alo[FM], ahi[FM];
#pragma unroll
        for (int i = 0; i < FM; ++i) {
          const v4i p = a_sread(stage, s, i);
          alo[i] = (p << 4) & (int)0xF0F0F0F0;
          ahi[i] = p & (int)0xF0F0F0F0;
        }
#pragma unroll
        for (int j = 0; j < FN; ++j) {
          const v4i p = wb[d][j][s];
          const v4i blo = (p << 4) & (int)0xF0F0F0F0, bhi = p & (int)0xF0F0F0F0;
          wb[d][j][s] = b_gload(j, s, kt + 2);
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            iacc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(blo, alo[i], iacc[i][j], 0, 0, 0);
            iacc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bhi, ahi[i], iacc[i][j], 0, 0, 0);
          }
        }
      }
      // this group's contribution: float(acc) * (sa * sb), the accumulator holding 256 * sum (2^-8 folded into sa, exact)
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const float sa_f = (float)sa_c[i] * 0.00390625f;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float sc = sa_f * (float)sb_c[j][q][e];
              facc[i][j][q * 4 + e] = facc[i][j][q * 4 + e] + keep_f32((float)iacc[i][j][q * 4 + e] * sc);
            }
      }
      __syncthreads();  // slice kt+1 is in LDS for everybody, and everybody is done with the stage that slice kt+2 will overwrite
    };

    int stage = 0;
#pragma unroll 1
    for (int kt0 = 0; kt0 < G; kt0 += 2) {
      slice(std::integral_constant<int, 0>{}, kt0, stage);
      stage = stage == kStages - 1 ? 0 : stage + 1;
      if (kt0 + 1 < G) {
        slice(std::integral_constant<int, 1>{}, kt0 + 1, stage);
        stage = stage == kStages - 1 ? 0 : stage + 1;
      }
    }

    // ---- epilogue: lane holds token lane & 31 and channels 8*(r/4) + 4*(lane >> 5) + (r & 3) of each 32 x 32 block ----
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = m0 + i * 32 + lrow;
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wave * 64 + j * 32 + q * 8 + nq;
          if (m < M && n < N) {
            v4h o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (_Float16)facc[i][j][q * 4 + e];
            gstore(t.C + (long)m * N + n, o);
            if (t.acc_dump) {  // parity tests only: the fp32 sums as bit patterns
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float f = facc[i][j][q * 4 + e];  // a copy: a bit cast applied to a vector element reads element 0
                gstore(t.acc_dump + (long)m * N + n + e, __float_as_int(f));
              }
            }
          }
        }
    }
  }
};

}  // namespace mxmoe
