// Skinny weight-only tiles (w4a16 / w3a16, group 128) for experts that receive a handful of tokens.
//
// These problems are HBM-bound: every packed weight is read exactly once and the work is arranged around that
// stream.  Counterpart of the reference's cta_gemm_wxa16g128 with BM = 16 tiles
// (mxmoe/kernels/src/include/cta_gemm.cuh:292-421, dequant mxmoe/kernels/src/include/quantize.cuh:134-214).
//
// Packed weight layout (own format, produced by mxmoe_amd.pack): [N/16][K/128][64 lanes][WBITS dwords].
// Lane l of block (nb, kb) holds the 32 weights of output channel nb*16 + (l & 15) for k = kb*128 + (l >> 4)*32 + 0..31,
// so one wave-wide load instruction reads one contiguous 1024-byte (w4) / 768-byte (w3) run and a whole
// expert streams linearly.  Within a dword, element e of its 8 values sits in nibble (e >> 1) + 4*(e & 1), which
// lets two masks and one shift produce four fp16 pairs in k order (magic-number conversion, no per-element shifts).
// w3 stores 24 values in the low 3 bits of the 24 nibbles of three dwords; the 24 spare top bits hold values 24..31.
//
// The group scale is applied to the fp32 partial sum of each 128-wide group instead of to every weight:
//   sum_k x[k]*(q[k]*s + z) = s * sum_k x[k]*q[k] + z * sum_k x[k]
// with sum_k x[k] produced by one extra MFMA against an all-ones operand.  The integer-valued weights are exact
// in fp16, so this differs from dequantise-then-multiply only by the fp16 rounding of each dequantised weight.
//
// Scale / zero table layout: [N/16][K/128][16 channels][2] fp16 = (scale, zero) — symmetric formats are packed
// offset-binary with zero = -2^(b-1) * scale, which is exact.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxmoe_tiles.hpp"

namespace mxmoe {

template <int WBITS_, int BN_, int KC_ = 1024>
struct SkinnyWoTile {
  static constexpr int WBITS = WBITS_, BM = 16, BN = BN_, KC = KC_;
  static_assert(WBITS == 4 || WBITS == 3, "w4 / w3 only");
  static_assert(BN % 64 == 0, "BN rows are dealt to 4 waves in 16-row blocks");
  static constexpr int R = BN / 64;                  // 16-row blocks per wave
  static constexpr int kXStride = KC * 2 + 16;       // bytes per activation row in LDS (+16 so 8 rows cover 8 bank groups)
  static constexpr int kLdsBytes = 16 * kXStride;
  static constexpr int kAccRegs = R * 4;
  static constexpr int kLaneBytes = WBITS * 4;       // packed bytes per lane per (row block, k block)
  static constexpr int kBlockBytes = 64 * kLaneBytes;

  struct WReg {
    int d[WBITS];
  };

  __device__ static __forceinline__ WReg load_w(const uint8_t* p) {
    WReg w;
    if constexpr (WBITS == 4) {
      const v4i v = gload<v4i>(p);
      w.d[0] = v[0]; w.d[1] = v[1]; w.d[2] = v[2]; w.d[3] = v[3];
    } else {
      // three dword loads (4-byte aligned); a 16-byte vector load would read past the end of the last block
      w.d[0] = gload<int>(p); w.d[1] = gload<int>(p + 4); w.d[2] = gload<int>(p + 8);
    }
    return w;
  }

  // 8 packed values of one dword -> 8 fp16 integers in k order.
  template <int MASK_LO, int MASK_HI>
  __device__ static __forceinline__ v8h cvt8(int d) {
    const v2h k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
    const v2h k64 = {(_Float16)64.0f, (_Float16)64.0f};
    const int d8 = (int)((unsigned)d >> 8);
    const v2h h0 = __builtin_bit_cast(v2h, (d & MASK_LO) | 0x64006400) - k1024;
    const v2h h1 = __builtin_bit_cast(v2h, (d & MASK_HI) | 0x54005400) - k64;
    const v2h h2 = __builtin_bit_cast(v2h, (d8 & MASK_LO) | 0x64006400) - k1024;
    const v2h h3 = __builtin_bit_cast(v2h, (d8 & MASK_HI) | 0x54005400) - k64;
    v8h o;
    o[0] = h0[0]; o[1] = h0[1]; o[2] = h1[0]; o[3] = h1[1];
    o[4] = h2[0]; o[5] = h2[1]; o[6] = h3[0]; o[7] = h3[1];
    return o;
  }

  // The four 8-value MFMA operands (k sub-blocks j = 0..3) of one lane's 32 weights.
  __device__ static __forceinline__ void unpack(const WReg& w, v8h out[4]) {
    if constexpr (WBITS == 4) {
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = cvt8<0x000F000F, 0x00F000F0>(w.d[j]);
    } else {
#pragma unroll
      for (int j = 0; j < 3; ++j) out[j] = cvt8<0x00070007, 0x00700070>(w.d[j]);
      const int t = (int)(((unsigned)w.d[0] >> 3) & 0x11111111u) | (int)(((unsigned)w.d[1] >> 2) & 0x22222222u) | (int)(((unsigned)w.d[2] >> 1) & 0x44444444u);
      out[3] = cvt8<0x00070007, 0x00700070>(t);
    }
  }

  __device__ static __forceinline__ void run(const TileArgs& t, uint8_t* __restrict__ smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int M = t.M, N = t.N, K = t.K;
    const int m0 = t.row0 + t.tile_m * BM, n0 = t.tile_n * BN;
    const int KB = K / 128;  // k blocks (= quantisation groups) per row
    const int lm = lane & 15, lg = lane >> 4;

    const _Float16* X = reinterpret_cast<const _Float16*>(t.A);
    const v8h ones = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};

    // row blocks of this wave: nb = n0/16 + wave + 4*r
    const uint8_t* wp[R];
    const uint8_t* sp[R];
    bool live[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int nb = n0 / 16 + wave + 4 * r;
      live[r] = nb * 16 < N;
      const int nbc = live[r] ? nb : 0;
      wp[r] = t.B + ((long)nbc * KB) * kBlockBytes + lane * kLaneBytes;
      sp[r] = reinterpret_cast<const uint8_t*>(t.sb) + ((long)nbc * KB) * 64 + lg * 16;  // 16 channels * (scale, zero) * 2 B per block
    }

    v4f acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = v4f{0.f, 0.f, 0.f, 0.f};

    for (int kc0 = 0; kc0 < K; kc0 += KC) {
      const int kcur = min(KC, K - kc0);
      if (kc0) __syncthreads();  // previous chunk fully consumed before it is overwritten
      // stage activation rows m0..m0+15, columns kc0..kc0+kcur, zero-filling rows past M
      for (int idx = tid; idx < 16 * (KC / 8); idx += kThreads) {
        const int row = idx / (KC / 8), ch = idx % (KC / 8);
        if (ch * 8 < kcur) {
          v4i v = {0, 0, 0, 0};
          if (m0 + row < M) v = gload<v4i>(X + (long)(m0 + row) * K + kc0 + ch * 8);
          *reinterpret_cast<v4i*>(smem + row * kXStride + ch * 16) = v;
        }
      }
      __syncthreads();

      const int kb0 = kc0 / 128, nkb = kcur / 128;
      WReg wq[R];
      v4i sz[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        wq[r] = load_w(wp[r] + (long)kb0 * kBlockBytes);
        sz[r] = gload<v4i>(sp[r] + (long)kb0 * 64);
      }
      for (int kb = 0; kb < nkb; ++kb) {
        WReg wn[R];
        v4i szn[R];
        const int kbn = kb0 + min(kb + 1, nkb - 1);  // last iteration re-loads its own block (harmless, keeps the loop branch-free)
#pragma unroll
        for (int r = 0; r < R; ++r) {
          wn[r] = load_w(wp[r] + (long)kbn * kBlockBytes);
          szn[r] = gload<v4i>(sp[r] + (long)kbn * 64);
        }
        v8h xf[4];
        const uint8_t* xs = smem + lm * kXStride + (kb * 128 + lg * 32) * 2;
#pragma unroll
        for (int j = 0; j < 4; ++j) xf[j] = *reinterpret_cast<const v8h*>(xs + j * 16);
        v4f sx = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) sx = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, xf[j], sx, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          v8h wf[4];
          unpack(wq[r], wf);
          v4f part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < 4; ++j) part = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[j], xf[j], part, 0, 0, 0);
          const v8h s8 = __builtin_bit_cast(v8h, sz[r]);  // (scale, zero) of channels 4*lg .. 4*lg+3
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[r][e] += part[e] * (float)s8[2 * e] + sx[e] * (float)s8[2 * e + 1];
          wq[r] = wn[r];
          sz[r] = szn[r];
        }
      }
    }

    const int m = m0 + lm;
    if (m < M) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (!live[r]) continue;
        const int n = n0 + (wave + 4 * r) * 16 + lg * 4;
        v4h o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (_Float16)acc[r][e];
        gstore<v4h>(t.C + (long)m * N + n, o);
        if (t.acc_dump) {
#pragma unroll
          for (int e = 0; e < 4; ++e) gstore<int>(t.acc_dump + (long)m * N + n + e, __builtin_bit_cast(int, acc[r][e]));
        }
      }
    }
  }
};

}  // namespace mxmoe
