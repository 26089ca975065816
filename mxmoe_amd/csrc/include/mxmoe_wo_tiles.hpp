// Skinny weight-only tiles (w8a16 / w4a16 / w3a16 / w2a16, one (scale, zero) pair per channel and 128-wide K group) for experts that
// receive a handful of tokens.  Per-channel formats (group size -1, the reference's cta_gemm_multistage_qb_v2 with GSIZE = -1,
// mxmoe/kernels/src/include/cta_gemm.cuh:113-286) use the same tiles: their packer repeats the channel's pair for every group.
//
// These problems are HBM-bound: every packed weight is read exactly once and the work is arranged around that
// stream.  A workgroup owns 16 tokens x BN channels; its 4 waves split K into contiguous quarters, keep their quarter of the
// activations in registers and stream the packed weights through a deep register ring (no LDS and no barrier in the loop);
// the four partial sums meet in LDS at the end and are added in a fixed order.  Counterpart of the reference's cta_gemm_wxa16g128 with BM = 16 tiles
// (mxmoe/kernels/src/include/cta_gemm.cuh:292-421, dequant mxmoe/kernels/src/include/quantize.cuh:134-214).
//
// Packed weight layout (own format, produced by mxmoe_amd.pack): [N/16][K/128][64 lanes][WBITS dwords].
// Lane l of block (nb, kb) holds the 32 weights of output channel nb*16 + (l & 15) for k = kb*128 + (l >> 4)*32 + 0..31,
// so one wave-wide load instruction reads one contiguous 1024-byte (w4) / 768-byte (w3) run and a whole
// expert streams linearly.  Within a dword, element e of its 8 values sits in nibble (e >> 1) + 4*(e & 1), which
// lets two masks and one shift produce four fp16 pairs in k order (magic-number conversion, no per-element shifts).
// w3 stores 24 values in the low 3 bits of the 24 nibbles of three dwords; the 24 spare top bits hold values 24..31.
// w2 stores values 16d..16d+7 in the low two bits of the nibbles of dword d and values 16d+8..16d+15 in the high two.
// w8 stores one byte per value in k order (8 dwords per lane).
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

// KP: k blocks (128 wide) per pass of a wave, whose activations live in registers; RING: packed weight blocks in flight per wave;
// WAVES: waves per SIMD a kernel made of such tiles alone is compiled for (fewer registers per wave, more workgroups per CU);
// MB: blocks of 16 tokens per tile.  Every unpacked weight operand is multiplied into all MB token blocks, so an expert with 17 .. 32
// tokens still streams its weights once (two 16-token tiles stream them twice, the second time out of L2 at best, and take nearly
// twice as long); the activations of a pass and the partial sums take MB times the registers, which is why KP shrinks as MB grows.
template <int WBITS_, int BN_, int KP_ = 4, int RING_ = (WBITS_ == 8 ? 6 : 12), int WAVES_ = 2, int MB_ = 1>
struct SkinnyWoTile {
  static constexpr int WBITS = WBITS_, MB = MB_, BM = 16 * MB_, BN = BN_;
  static_assert(WBITS == 8 || WBITS == 4 || WBITS == 3 || WBITS == 2, "w8 / w4 / w3 / w2");
  static_assert(BN % 64 == 0, "the final reduction deals 16-channel blocks to 4 waves");
  static constexpr int NB = BN / 16;                 // 16-channel blocks per tile
  static constexpr int KP = KP_;                     // k blocks (128 wide) per pass of a wave: their activations live in registers
  static constexpr int kRedBytes = kWaves * NB * MB * 64 * 16;  // per-wave partial sums for the final reduction
  static constexpr int kScaleBytes = NB * KP * 64;         // per-wave patch of (scale, zero) pairs of one pass
  static constexpr int kLdsBytes = kRedBytes + kWaves * kScaleBytes;
  static constexpr int kAccRegs = NB * MB * 4;
  static constexpr int kWavesWanted = WAVES_;
  static constexpr int kABits = 16, kWBits = WBITS;  // fp16 activations, packed weights
  static constexpr int kLaneBytes = WBITS * 4;       // packed bytes per lane per (channel block, k block)
  static constexpr int kBlockBytes = 64 * kLaneBytes;
  static constexpr int kRing = RING_;                // packed blocks in flight per wave (12 KB by default)

  struct WReg {
    int d[WBITS];
  };

  __device__ static __forceinline__ WReg load_w(const uint8_t* p) {
    WReg w;
    if constexpr (WBITS == 8) {
      const v4i a = gload<v4i>(p), b = gload<v4i>(p + 16);
      w.d[0] = a[0]; w.d[1] = a[1]; w.d[2] = a[2]; w.d[3] = a[3];
      w.d[4] = b[0]; w.d[5] = b[1]; w.d[6] = b[2]; w.d[7] = b[3];
    } else if constexpr (WBITS == 4) {
      const v4i v = gload<v4i>(p);
      w.d[0] = v[0]; w.d[1] = v[1]; w.d[2] = v[2]; w.d[3] = v[3];
    } else if constexpr (WBITS == 3) {
      typedef int v3i __attribute__((ext_vector_type(3)));
      const v3i v = gload<v3i>(p);  // 12 bytes: a 16-byte load would read past the end of the last block
      w.d[0] = v[0]; w.d[1] = v[1]; w.d[2] = v[2];
    } else {
      typedef int v2i __attribute__((ext_vector_type(2)));
      const v2i v = gload<v2i>(p);
      w.d[0] = v[0]; w.d[1] = v[1];
    }
    return w;
  }

  // 8 packed values of one dword -> 8 fp16 numbers in k order, each still carrying the bias of its magic constant:
  // 0x6400 | q is the fp16 number 1024 + q (elements 0, 1, 4, 5), 0x5400 | (q << 4) is 64 + q (elements 2, 3, 6, 7).
  // The biases are taken out of the 128-wide partial sum instead of out of every weight (see pass()).
  template <int MASK_LO, int MASK_HI>
  __device__ static __forceinline__ v8h cvt8(int d) {
    const int d8 = (int)((unsigned)d >> 8);
    v4i o;
    o[0] = (d & MASK_LO) | 0x64006400;
    o[1] = (d & MASK_HI) | 0x54005400;
    o[2] = (d8 & MASK_LO) | 0x64006400;
    o[3] = (d8 & MASK_HI) | 0x54005400;
    return __builtin_bit_cast(v8h, o);
  }

  // The bias each of the 8 values of an operand still carries after unpack(): 1024 for values placed by the 0x6400 constant, 64 for
  // those placed by 0x5400 (8-bit codes are all placed by the first).
  __device__ static __forceinline__ v8h bias8() {
    constexpr float hi = WBITS == 8 ? 1024.0f : 64.0f;
    return v8h{(_Float16)1024.0f, (_Float16)1024.0f, (_Float16)hi, (_Float16)hi, (_Float16)1024.0f, (_Float16)1024.0f, (_Float16)hi, (_Float16)hi};
  }

  // The four 8-value MFMA operands (k sub-blocks j = 0..3) of one lane's 32 weights.
  __device__ static __forceinline__ void unpack(const WReg& w, v8h out[4]) {
    if constexpr (WBITS == 8) {
      // one byte per value, k order: byte b of a dword next to the constant byte 0x64 is the fp16 number 1024 + b
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v4i o;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          o[2 * h] = (int)__builtin_amdgcn_perm(0x64646464u, (unsigned)w.d[2 * j + h], 0x04010400u);
          o[2 * h + 1] = (int)__builtin_amdgcn_perm(0x64646464u, (unsigned)w.d[2 * j + h], 0x04030402u);
        }
        out[j] = __builtin_bit_cast(v8h, o);
      }
    } else if constexpr (WBITS == 4) {
#pragma unroll
      for (int j = 0; j < 4; ++j) out[j] = cvt8<0x000F000F, 0x00F000F0>(w.d[j]);
    } else if constexpr (WBITS == 3) {
#pragma unroll
      for (int j = 0; j < 3; ++j) out[j] = cvt8<0x00070007, 0x00700070>(w.d[j]);
      const int t = (int)(((unsigned)w.d[0] >> 3) & 0x11111111u) | (int)(((unsigned)w.d[1] >> 2) & 0x22222222u) | (int)(((unsigned)w.d[2] >> 1) & 0x44444444u);
      out[3] = cvt8<0x00070007, 0x00700070>(t);
    } else {
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        out[2 * d] = cvt8<0x00030003, 0x00300030>(w.d[d]);
        out[2 * d + 1] = cvt8<0x00030003, 0x00300030>((int)((unsigned)w.d[d] >> 2));
      }
    }
  }

  // One pass of a wave: NKB (<= KP) consecutive k blocks starting at kb0, against all NB channel blocks of the tile.
  // The wave's activations of these k blocks are loaded once into registers and its (scale, zero) pairs into a private LDS
  // patch; the packed weight blocks then stream through a ring of kRing register buffers with no barrier in the loop, so
  // kRing KB per wave are always in flight.  Per 128-wide group g and channel n the pass adds
  //   s * (sum_k x[k] * (q[k] + bias[k])  -  sum_k x[k] * bias[k])  +  z * sum_k x[k]
  // where the first sum comes from 4 MFMAs on the biased weights and the other two from MFMAs of x against constant operands.
  template <int NKB>
  __device__ static __forceinline__ void pass(const TileArgs& t, int kb0, int m0, int n0, int nbv, int lane, uint8_t* __restrict__ spatch, v4f (&acc)[NB][MB]) {
    const int K = t.K, KB = K / 128;
    const int lm = lane & 15, lg = lane >> 4;
    const v8h ones = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};
    const v8h bias = bias8();
    constexpr int Q = NB * NKB;  // blocks of this pass, channel block major

    // Everything the pass needs from memory is requested before anything is waited for, the weight ring first: the first blocks of
    // the stream, the activations and the (scale, zero) pairs then arrive together, one memory latency after the pass began
    // (waiting for the scales before requesting the weights costs a second one, which is a third of a short tile's life).
    const uint8_t* wb = t.B + ((long)(n0 / 16) * KB + kb0) * kBlockBytes + lane * kLaneBytes;
    auto w_of = [&](int q) { const int nb = q / NKB < nbv ? q / NKB : 0; return load_w(wb + ((long)nb * KB + q % NKB) * kBlockBytes); };
    WReg wr[kRing];
#pragma unroll
    for (int q = 0; q < kRing && q < Q; ++q) wr[q] = w_of(q);
    __builtin_amdgcn_sched_barrier(0);
    // activations: lane holds row lm of each token block, k = 128*(kb0 + s) + 32*lg + 8*j + 0..7
    v8h xf[MB][NKB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = m0 + mb * 16 + lm;
      const _Float16* xr = reinterpret_cast<const _Float16*>(t.A) + (long)(m < t.M ? m : 0) * K + kb0 * 128 + lg * 32;
#pragma unroll
      for (int s = 0; s < NKB; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const v4i v = gload<v4i>(xr + s * 128 + j * 8);
          xf[mb][s][j] = m < t.M ? __builtin_bit_cast(v8h, v) : v8h{};
        }
    }
    // (scale, zero) pairs of the pass: 64 bytes per block, NKB consecutive blocks per channel block -> LDS [nb][s][64 B]
    const uint8_t* sb = reinterpret_cast<const uint8_t*>(t.sb) + ((long)(n0 / 16) * KB + kb0) * 64;
    constexpr int kPieces = (Q * 4 + 63) / 64;  // 16-byte pieces per lane
    v4i sv[kPieces];
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int c = min(lane + 64 * i, Q * 4 - 1);
      const int nb = c / (NKB * 4), rest = c % (NKB * 4);
      sv[i] = gload<v4i>(sb + ((long)(nb < nbv ? nb : 0) * KB) * 64 + rest * 16);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kPieces; ++i) {
      const int c = lane + 64 * i;
      if (c < Q * 4) *reinterpret_cast<v4i*>(spatch + c * 16) = sv[i];
    }

    v4f sx[MB][NKB], sxb[MB][NKB];  // per token block and k block: sum of x, sum of x * bias  (row = any channel, column = token)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int s = 0; s < NKB; ++s) {
        sx[mb][s] = sxb[mb][s] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          sx[mb][s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, xf[mb][s][j], sx[mb][s], 0, 0, 0);
          sxb[mb][s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bias, xf[mb][s][j], sxb[mb][s], 0, 0, 0);
        }
      }
    static_for<Q>([&](auto qc) {
      constexpr int q = decltype(qc)::value;
      constexpr int nb = q / NKB, s = q % NKB;
      v8h wf[4];
      unpack(wr[q % kRing], wf);
      if constexpr (q + kRing < Q) wr[q % kRing] = w_of(q + kRing);
      const v8h s8 = __builtin_bit_cast(v8h, *reinterpret_cast<const v4i*>(spatch + q * 64 + lg * 16));  // (scale, zero) of channels 4*lg .. 4*lg+3
      __builtin_amdgcn_sched_barrier(0);  // the refill is issued here, kRing blocks ahead of its use, not where the scheduler likes it
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        v4f part = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) part = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[j], xf[mb][s][j], part, 0, 0, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc[nb][mb][e] = __builtin_fmaf(part[e] - sxb[mb][s][e], (float)s8[2 * e], __builtin_fmaf(sx[mb][s][e], (float)s8[2 * e + 1], acc[nb][mb][e]));
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  }

  __device__ static __forceinline__ void run(const TileArgs& t, uint8_t* __restrict__ smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = t.M, N = t.N, K = t.K;
    const int m0 = t.row0 + t.tile_m * BM, n0 = t.tile_n * BN;
    const int KB = K / 128;  // k blocks (= quantisation groups) per row
    const int lm = lane & 15, lg = lane >> 4;
    const int nbv = min(NB, (N - n0) / 16);  // channel blocks of this tile that exist

    // the K range is dealt to the 4 waves in contiguous quarters; each wave sums its quarter for every channel of the tile
    const int KW = (KB + kWaves - 1) / kWaves;
    const int kb_lo = min(KB, wave * KW), kb_hi = min(KB, kb_lo + KW);
    uint8_t* spatch = smem + kRedBytes + wave * kScaleBytes;
    v4f acc[NB][MB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int kb = kb_lo; kb < kb_hi; kb += KP) {
      const int nk = min(KP, kb_hi - kb);
      if constexpr (KP >= 4) {
        if (nk == 4) { pass<4>(t, kb, m0, n0, nbv, lane, spatch, acc); continue; }
      }
      if constexpr (KP >= 3) {
        if (nk == 3) { pass<3>(t, kb, m0, n0, nbv, lane, spatch, acc); continue; }
      }
      if constexpr (KP >= 2) {
        if (nk == 2) { pass<2>(t, kb, m0, n0, nbv, lane, spatch, acc); continue; }
      }
      pass<1>(t, kb, m0, n0, nbv, lane, spatch, acc);
    }

    // reduction over the 4 waves in a fixed order (wave 0 + 1 + 2 + 3), 16-channel blocks dealt round-robin to the waves
    v4f* red = reinterpret_cast<v4f*>(smem);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) red[((wave * NB + nb) * MB + mb) * 64 + lane] = acc[nb][mb];
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NB / kWaves; ++r) {
      const int nb = wave + kWaves * r;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = m0 + mb * 16 + lm;
        v4f sum = red[(nb * MB + mb) * 64 + lane];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) {
          const v4f p = red[((w * NB + nb) * MB + mb) * 64 + lane];
#pragma unroll
          for (int e = 0; e < 4; ++e) sum[e] += p[e];
        }
        if (m < M && nb < nbv) {
          const int n = n0 + nb * 16 + lg * 4;
          v4h o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (_Float16)sum[e];
          gstore<v4h>(t.C + (long)m * N + n, o);
          if (t.acc_dump) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float f = sum[e];  // a copy: a bit cast applied to a vector element reads element 0
              gstore<int>(t.acc_dump + (long)m * N + n + e, __float_as_int(f));
            }
          }
        }
      }
    }
  }
};

// Weight-only tile for experts with many tokens (w4a16 / w3a16 / w2a16, group 128): 128 tokens x 256 channels per workgroup as four
// waves side by side, each with all 128 tokens against its own 64 channels (BN = 128: 2 x 2 waves of 64 x 64, the shape with
// half the token reuse per unpacked weight).  Counterpart of the reference's cta_gemm_multistage_qb_v2 with its larger tiles
// (mxmoe/kernels/src/include/cta_gemm.cuh:113-286) and of Converter::dequant_frag (quantize.cuh:134-214): every packed weight
// becomes fp16 as fma(q, scale, zero) in fp16, one rounding, exactly like the reference's __hfma2, and the products are summed in
// fp32 by the fp16 MFMA over the whole of K, in the same order for both shapes.
// Same packed weight and (scale, zero) layouts as the skinny tile: a wave streams its 4 channel blocks of each 128-wide k block
// straight from global memory through a register ring and reuses each dequantised 8-weight operand for all of its token blocks
// (8, or 4 in the 2 x 2 shape): the unpack work per MFMA, about 3 vector instructions in the 2 x 2 shape, is what bounds the tile.
// The k block is walked in four 32-wide sub-blocks so that only one sub-block's token fragments are live beside the accumulators.
// Activations go global -> LDS (direct loads, two stages of 128 rows x 256 B, 16-byte chunks XOR-swizzled with the row so that
// the 16 rows a read touches hit 16 different bank groups).
template <int WBITS_, int BM_ = 128, int BN_ = 128>
struct WoMfmaTile {
  static constexpr int WBITS = WBITS_, BM = BM_, BN = BN_;
  static_assert(BM == 128 && (BN == 128 || BN == 256), "2 x 2 waves of 64 tokens x 64 channels, or 4 waves of 128 x 64 side by side");
  static constexpr int WM = BN == 128 ? 2 : 1;  // waves along the tokens
  static constexpr int TM = BM / WM;            // tokens per wave
  static constexpr int MB = TM / 16;            // token blocks per wave
  using Sk = SkinnyWoTile<WBITS, 128>;  // (its packed-block loader and unpacker)
  static constexpr int kStageBytes = BM * 256;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static constexpr int kAccRegs = 16 * MB;
  static constexpr int kWavesWanted = 2;
  static constexpr int kABits = 16, kWBits = WBITS;  // fp16 activations, packed weights
  static constexpr int kLaneBytes = Sk::kLaneBytes, kBlockBytes = Sk::kBlockBytes;
  static constexpr int kDma = kStageBytes / 1024 / kWaves;  // direct-to-LDS loads per wave per stage

  __device__ static __forceinline__ void run(const TileArgs& t, uint8_t* __restrict__ smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = WM == 2 ? wave >> 1 : 0, wn = WM == 2 ? wave & 1 : wave;
    const int M = t.M, N = t.N, K = t.K;
    const int m0 = t.row0 + t.tile_m * BM, n0 = t.tile_n * BN;
    const int KB = K / 128;
    const int lm = lane & 15, lg = lane >> 4;
    // channel blocks of this wave that exist; a wave whose 64 channels all lie past N runs on the tile's first blocks instead
    // (every wave must take part in the barriers) and stores nothing
    const int nbv = max(0, min(4, (N - n0) / 16 - wn * 4));
    const int nb0 = n0 / 16 + (nbv > 0 ? wn * 4 : 0);

    // activations: buffer resource over the valid rows of the tile (rows past M read as zeros)
    const int a_rows = min(BM, M - m0);
    const v4i rs_x = make_rsrc(t.A + (long)m0 * K * 2, (unsigned)((long)a_rows * K * 2));
    const int lds_base = (int)(uintptr_t)smem;
    int dma_voff[kDma], dma_lds[kDma];
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
      const int ii = wave * kDma + i;             // 1 KB piece = 4 rows
      const int row = 4 * ii + (lane >> 4);
      dma_voff[i] = row * K * 2 + (((lane & 15) ^ (row & 15)) << 4);
      dma_lds[i] = ii * 1024;
    }
    auto dma_x = [&](int kb, int stage) {
      const int koff = __builtin_amdgcn_readfirstlane(kb * 256);
#pragma unroll
      for (int i = 0; i < kDma; ++i) dma16_to_lds(rs_x, __builtin_amdgcn_readfirstlane(lds_base + stage * kStageBytes + dma_lds[i]), dma_voff[i], koff);
    };
    // fragment reads: token row wm*TM + mb*16 + lm, chunk lg*4 + j
    const int xrow = wm * TM + lm;
    auto lds_x = [&](int stage, int mb, int j) {
      const int row = xrow + mb * 16;
      return *reinterpret_cast<const v4i*>(smem + stage * kStageBytes + row * 256 + (((lg * 4 + j) ^ (row & 15)) << 4));
    };

    // weights: blocks (n0/16 + wn*4 + nb, kb); ring of 8 = two k blocks ahead.  Loads past the end of K re-read the last k block
    // (never used) so that every iteration issues the same number of loads, which the wait for the activation stage relies on.
    const uint8_t* wb = t.B + ((long)nb0 * KB) * kBlockBytes + lane * kLaneBytes;
    const uint8_t* sb = reinterpret_cast<const uint8_t*>(t.sb) + ((long)nb0 * KB) * 64 + lm * 4;
    auto w_of = [&](int nb, int kb) { return Sk::load_w(wb + ((long)(nb < nbv ? nb : 0) * KB + min(kb, KB - 1)) * kBlockBytes); };
    auto s_of = [&](int nb, int kb) { return gload<int>(sb + ((long)(nb < nbv ? nb : 0) * KB + min(kb, KB - 1)) * 64); };
    typename Sk::WReg wr[8];
    int sr[8];

    v4f acc[4][MB];  // [channel block][token block]
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[nb][mb] = v4f{0.f, 0.f, 0.f, 0.f};

    {
      // prologue: exactly 8 ring loads are younger than the loads of the first activation stage, as in every later iteration
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        wr[q] = w_of(q, 0);
        sr[q] = s_of(q, 0);
      }
      asm volatile("" ::: "memory");
      dma_x(0, 0);
#pragma unroll
      for (int q = 4; q < 8; ++q) {
        wr[q] = w_of(q - 4, 1);
        sr[q] = s_of(q - 4, 1);
      }
      asm volatile("" ::: "memory");
      const v8h bias = Sk::bias8();
      // token blocks of this wave that hold rows of the problem: a tile of a problem with at most half of BM rows left (an expert
      // with a few dozen tokens, a short last row tile) runs a second copy of the loop that leaves out the fragment reads and
      // matrix instructions of the upper half, which would only multiply zeros; such a tile is then bound by its weight stream
      // rather than by 128 rows of arithmetic
      const int mbv = __builtin_amdgcn_readfirstlane(max(0, min(MB, (a_rows - wm * TM + 15) / 16)));
      // one k block; PAR = parity of kb, a compile-time constant so that the ring slots are fixed registers; LIVE: token blocks computed
      auto step = [&](auto parc, int kb, auto livec) {
        constexpr int st = decltype(parc)::value;
        constexpr int LIVE = decltype(livec)::value;
        // the activation stage of this k block has landed: the only younger loads are the 8 ring refills of the last iteration
        // (or the 8 ring loads of the prologue)
        vm_wait<8>();
        __syncthreads();  // ... for every wave; and every wave holds the previous stage's fragments in registers by now
        if (kb + 1 < KB) dma_x(kb + 1, st ^ 1);
        constexpr int base = st * 4;
        // k sub-block by k sub-block: its token fragments, then every channel block's 8 weights per lane against all of them
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v8h xf[MB];
#pragma unroll
          for (int mb = 0; mb < LIVE; ++mb) xf[mb] = __builtin_bit_cast(v8h, lds_x(st, mb, j));
#pragma unroll
          for (int nb = 0; nb < 4; ++nb) {
            v8h wf[4];
            Sk::unpack(wr[base + nb], wf);  // only wf[j] is used: the rest folds away
            const v2h sz = __builtin_bit_cast(v2h, sr[base + nb]);
            const v8h s8 = {sz[0], sz[0], sz[0], sz[0], sz[0], sz[0], sz[0], sz[0]};
            const v8h z8 = {sz[1], sz[1], sz[1], sz[1], sz[1], sz[1], sz[1], sz[1]};
            const v8h w8 = __builtin_elementwise_fma(wf[j] - bias, s8, z8);  // exact q, then fma(q, scale, zero) in fp16
#pragma unroll
            for (int mb = 0; mb < LIVE; ++mb) acc[nb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(w8, xf[mb], acc[nb][mb], 0, 0, 0);
          }
          // keeps the scheduler from starting the next sub-block's unpacking and fragment reads early: that costs no time (the
          // other wave of the SIMD fills the gap) and without it the 3-bit tile runs out of registers
          __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
          wr[base + nb] = w_of(nb, kb + 2);
          sr[base + nb] = s_of(nb, kb + 2);
        }
      };
      if (mbv > MB / 2) {
#pragma unroll 1
        for (int kb = 0; kb < KB; kb += 2) {
          step(std::integral_constant<int, 0>{}, kb, std::integral_constant<int, MB>{});
          if (kb + 1 < KB) step(std::integral_constant<int, 1>{}, kb + 1, std::integral_constant<int, MB>{});
        }
      } else {
#pragma unroll 1
        for (int kb = 0; kb < KB; kb += 2) {
          step(std::integral_constant<int, 0>{}, kb, std::integral_constant<int, MB / 2>{});
          if (kb + 1 < KB) step(std::integral_constant<int, 1>{}, kb + 1, std::integral_constant<int, MB / 2>{});
        }
      }
    }
    vm_wait<0>();
    __syncthreads();  // LDS is reused for the output patch

    // epilogue, 64 tokens at a time: [token][channel] fp16 patch per wave (64 x 64, row pitch 136 B), then 16-byte
    // row-contiguous stores
    constexpr int kPitch = 64 * 2 + 8;
    uint8_t* patch = smem + wave * (64 * kPitch);
    const int pr = lane >> 3, pc = lane & 7;  // 8 lanes x 16 B per 64-channel row, 8 rows per pass
#pragma unroll
    for (int h = 0; h < TM / 64; ++h) {
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
          const v4f a = acc[nb][h * 4 + mb];
          v4h o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (_Float16)a[e];
          *reinterpret_cast<v4h*>(patch + (mb * 16 + lm) * kPitch + (nb * 16 + lg * 4) * 2) = o;
          if (t.acc_dump) {
            const int m = m0 + wm * TM + h * 64 + mb * 16 + lm, n = n0 + wn * 64 + nb * 16 + lg * 4;
            if (m < M && n < N) {
#pragma unroll
              for (int e = 0; e < 4; ++e) gstore<int>(t.acc_dump + (long)m * N + n + e, __float_as_int(a[e]));
            }
          }
        }
#pragma unroll
      for (int r0 = 0; r0 < 64; r0 += 8) {
        const int ml = r0 + pr;
        const int m = m0 + wm * TM + h * 64 + ml, n = n0 + wn * 64 + pc * 8;
        const v4i v = *reinterpret_cast<const v4i*>(patch + ml * kPitch + pc * 16);
        if (m < M && n < N) gstore_stream<v4i>(t.C + (long)m * N + n, v);
      }
    }
  }
};

}  // namespace mxmoe
