// Bf6Tile: w4a4_g-1_sym on the 6-bit float matrix path.
//
// Every integer -8 .. 8 is a bf6 (e3m2) number, a product of two of them is at most 64 and fp32 adds such integers exactly up to
// 2^24, so v_mfma_scale_f32_32x32x64_f8f6f4 on bf6 operands with unit scales returns the int32 accumulators of the integer tiles
// (cta_gemm_multistage_qab_v2 of the reference, mxmoe/kernels/src/include/cta_gemm.cuh:424-608, accumulates the same sums with
// mma.s4) as fp32 integers, bit for bit, at twice the operations per cycle of the int8 instruction.  The price is storage: both
// operands are held as 6-bit codes, 0.75 bytes per value.  The activation quantisers write them directly (tag 4); the weights are
// re-encoded when they are packed (mxmoe_amd.pack.pack_bf6_fragments).
//
// Operand layout, the same for activations (rows = tokens of one expert, local row 0 first) and weights (rows = channels):
// fragments of 32 rows x 64 k, 1536 bytes each, row block major:
//   offset(row block rb, k step ks) = (rb * K / 64 + ks) * 1536.
// A fragment is what one matrix instruction takes from a wave: lane l (row l % 32, k = 64 ks + 32 (l / 32) + i, i = 0 .. 31) holds
// 32 codes = 192 bits, value i at bit 6 i; its first 128 bits lie at byte 16 l of the fragment, its last 64 bits at byte 1024 + 8 l,
// so that a wave reads a fragment with one 16-byte and one 8-byte access per lane, both contiguous across the wave.  An expert's
// activation region holds ceil(rows / 32) row blocks; rows past the last one of a block are never written and never used.
//
// Workgroup = BM tokens x 256 channels, four waves side by side with all BM tokens against 64 channels each.  Per 64-wide k step a
// wave takes its BM / 32 token fragments from LDS, where direct-to-LDS loads put the workgroup's token fragments three steps
// ahead (4-stage ring), and its two channel fragments straight from global memory through a register ring two steps ahead.
// Every load of the loop is inline assembly and is awaited by one hand-counted wait per step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxmoe_tiles.hpp"

namespace mxmoe {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr int kBf6Frag = 1536;  // bytes of one 32 x 64 fragment

struct Bf6Frag {
  v4i lo;
  v2i hi;
};
__device__ __forceinline__ v8i bf6_operand(const Bf6Frag& f) { return v8i{f.lo[0], f.lo[1], f.lo[2], f.lo[3], f.hi[0], f.hi[1], 0, 0}; }

// Loads whose completion is tracked by hand, like the direct-to-LDS loads they share the counter with (a compiler-placed wait
// would not know of those and would end up waiting for loads issued moments ago).  Address = scalar base + 32-bit lane offset.
__device__ __forceinline__ Bf6Frag bf6_load_untracked(const uint8_t* sbase, int off_lo, int off_hi) {
  Bf6Frag f;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(f.lo) : "v"(off_lo), "s"(sbase) : "memory");
  asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(f.hi) : "v"(off_hi), "s"(sbase) : "memory");
  return f;
}
// wait until at most N vector-memory loads are outstanding; the comment names the registers that have landed by then
template <int N>
__device__ __forceinline__ void bf6_wait(Bf6Frag (&f)[2]) {
  asm volatile("s_waitcnt vmcnt(%4) ; landed %0 %1 %2 %3" : "+v"(f[0].lo), "+v"(f[0].hi), "+v"(f[1].lo), "+v"(f[1].hi) : "n"(N) : "memory");
}

template <int BM_>
struct Bf6Tile {
  static constexpr Op kOp = Op::I4;
  static constexpr int BM = BM_, BN = 256, BK = 64, WGM = 1, WGN = 4;
  static_assert(BM == 32 || BM == 64 || BM == 128, "BM x 256 tiles, BM = 32 / 64 / 128");
  static constexpr int TF = BM / 32;                 // token fragments per k step (every wave uses all of them)
  static constexpr int CA = 2;                       // channel fragments per wave
  static constexpr int kStageData = TF * kBf6Frag;   // the workgroup's token fragments of one k step
  static constexpr int kPieces = (kStageData + 1023) / 1024;  // direct-to-LDS loads of 1 KB that fill a stage
  static constexpr int kStage = kPieces * 1024;      // a stage in LDS (the last piece of a 32-row tile is half empty)
  static constexpr int kStages = 4;
  // Every wave issues the same number of loads per stage, because the hand-placed waits count them: with fewer pieces than wave
  // slots some pieces are brought twice (same bytes to the same place).
  static constexpr int kDma = (kPieces + kWaves - 1) / kWaves;
  static constexpr int kYounger = kDma + 2 * CA;     // loads issued after a step's channel fragments and before the step begins
  static constexpr int kChan = CA * 32;              // channels of a wave
  static constexpr int kPitch = kChan * 2 + 16;      // bytes per token row of the epilogue patch
  static constexpr int kPatchBytes = kWaves * 32 * kPitch;
  static constexpr int kLdsBytes = kStages * kStage > kPatchBytes ? kStages * kStage : kPatchBytes;
  static constexpr int kAccRegs = TF * CA * 16;
  static constexpr int kWavesWanted = 2;  // waves per SIMD a kernel of such tiles is compiled for
  static constexpr int kABits = 6, kWBits = 6;       // bits per activation / weight element as stored

  __device__ static __forceinline__ void run(const TileArgs& t, uint8_t* __restrict__ smem) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int M = t.M, N = t.N;
    const int KS = t.K / 64;  // k steps; even (K is a multiple of 128): the ring below runs whole rounds of two
    const int m0 = t.row0 + t.tile_m * BM, n0 = t.tile_n * BN;
    const int rb0 = m0 >> 5;  // first row block of the tile (segments start at multiples of 32 rows)

    // token fragments: global -> LDS.  The buffer covers the row blocks that exist from rb0 on; fragments past them read as zero.
    const int blocks = min(TF, ((M + 31) >> 5) - rb0);
    const long frag_row = (long)KS * kBf6Frag;  // bytes of one row block
    const v4i rs_a = make_rsrc(t.A + rb0 * frag_row, (unsigned)(blocks * frag_row));
    const int lds_base = (int)(uintptr_t)smem;
    int dma_voff[kDma], dma_lds[kDma];
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
      const int piece = (wave * kDma + i) % kPieces;
      const int b = piece * 1024 + lane * 16;           // byte of the stage this lane fills
      const int f = b / kBf6Frag, w = b - f * kBf6Frag;  // fragment and place inside it
      dma_voff[i] = f < TF ? f * (int)frag_row + w : 0x7FFFFFF0;  // (past the stage's data: out of range, zeros land in the padding)
      dma_lds[i] = __builtin_amdgcn_readfirstlane(piece * 1024);
    }
    auto dma_a = [&](int ks) {
      const int st = __builtin_amdgcn_readfirstlane((ks & (kStages - 1)) * kStage);
      const int soff = __builtin_amdgcn_readfirstlane(ks * kBf6Frag);
#pragma unroll
      for (int i = 0; i < kDma; ++i) dma16_to_lds(rs_a, lds_base + st + dma_lds[i], dma_voff[i], soff);
    };
    auto lds_a = [&](int ks, int j) {
      const uint8_t* f = smem + (ks & (kStages - 1)) * kStage + j * kBf6Frag;
      Bf6Frag r;
      r.lo = *reinterpret_cast<const v4i*>(f + lane * 16);
      r.hi = *reinterpret_cast<const v2i*>(f + 1024 + lane * 8);
      return r;
    };
    // channel fragments: global -> registers, scalar fragment address plus one lane offset per plane.  Blocks past N re-read the
    // last one (their results are never stored); steps past the end of K re-read the last step (never used), so that the number
    // of loads per step stays fixed.
    const int nblk = (N + 31) >> 5;
    const uint8_t* bbase[CA];
#pragma unroll
    for (int j = 0; j < CA; ++j) bbase[j] = t.B + (long)min((n0 >> 5) + wave * CA + j, nblk - 1) * frag_row;
    const int b_lo = lane * 16, b_hi = 1024 + lane * 8;
    auto load_b = [&](int ks, int j) {
      const long off = (long)__builtin_amdgcn_readfirstlane(ks < KS ? ks : KS - 1) * kBf6Frag;
      return bf6_load_untracked(bbase[j] + off, b_lo, b_hi);
    };

    v16f acc[CA][TF];  // [channel fragment][token fragment]
#pragma unroll
    for (int c = 0; c < CA; ++c)
#pragma unroll
      for (int f = 0; f < TF; ++f)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[c][f][r] = 0.f;

    // Order of the loads within step ks: after the barrier the kDma direct-to-LDS loads of stage ks + 3, and after the matrix
    // instructions the 2 CA ring loads of step ks + 2's channel fragments.  When step ks begins, the loads younger than its channel
    // fragments (issued in step ks - 2) are the kDma + 2 CA of step ks - 1, and its stage (issued in step ks - 3) is older still:
    // one wait for "at most that many outstanding" covers both operands.  The prologue issues its loads in the order the steps
    // before ks = 0 would have.
    Bf6Frag br[2][CA];
    dma_a(0);
    dma_a(1);
#pragma unroll
    for (int j = 0; j < CA; ++j) br[0][j] = load_b(0, j);
    dma_a(2);
#pragma unroll
    for (int j = 0; j < CA; ++j) br[1][j] = load_b(1, j);

    auto step = [&](auto parc, int ks) {
      constexpr int par = decltype(parc)::value;
      bf6_wait<kYounger>(br[par]);
      __syncthreads();  // the stage is complete for every wave, and no wave still reads the stage that is overwritten next
      dma_a(ks + 3 < KS ? ks + 3 : ks);  // (past the end: the stage being read is loaded once more with the same bytes; the count stays fixed)
      Bf6Frag af[TF];
#pragma unroll
      for (int f = 0; f < TF; ++f) af[f] = lds_a(ks, f);
#pragma unroll
      for (int c = 0; c < CA; ++c) {
        const v8i w = bf6_operand(br[par][c]);
#pragma unroll
        for (int f = 0; f < TF; ++f)
          acc[c][f] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, bf6_operand(af[f]), acc[c][f], 3, 3, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
      }
      __builtin_amdgcn_sched_barrier(0);  // the ring registers are free only after the last instruction that reads them
#pragma unroll
      for (int j = 0; j < CA; ++j) br[par][j] = load_b(ks + 2, j);
    };
#pragma unroll 1
    for (int ks = 0; ks < KS; ks += 2) {
      step(std::integral_constant<int, 0>{}, ks);
      step(std::integral_constant<int, 1>{}, ks + 1);
    }
    bf6_wait<0>(br[0]);  // everything has landed (vmcnt(0)), the loads past the end of K included
    bf6_wait<0>(br[1]);

    // ---- epilogue: lane l holds, of fragment pair (c, f), token l % 32 and channels 8 (r / 4) + 4 (l / 32) + r % 4, r = 0 .. 15.  32 tokens
    // at a time go through a [token][channel] patch in LDS and leave as 16-byte pieces of whole rows of the wave's channels.
    const int tok_l = lane & 31, ch_l = (lane >> 5) * 4;
    float s_a[TF];
    v4h s_b[CA][4];
#pragma unroll
    for (int f = 0; f < TF; ++f) s_a[f] = (float)gload<_Float16>(t.sa + min(m0 + f * 32 + tok_l, M - 1));
#pragma unroll
    for (int c = 0; c < CA; ++c)
#pragma unroll
      for (int g = 0; g < 4; ++g) s_b[c][g] = gload<v4h>(t.sb + min(n0 + wave * kChan + c * 32 + 8 * g + ch_l, N - 4));
    if (t.acc_dump) {  // parity tests only
#pragma unroll
      for (int f = 0; f < TF; ++f)
#pragma unroll
        for (int c = 0; c < CA; ++c)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = m0 + f * 32 + tok_l, n = n0 + wave * kChan + c * 32 + (r / 4) * 8 + ch_l + (r & 3);
            if (m < M && n < N) gstore<int>(t.acc_dump + (long)m * N + n, (int)acc[c][f][r]);
          }
    }
    __syncthreads();  // every wave is done with the stages
    uint8_t* patch = smem + wave * (32 * kPitch);
    constexpr int kRowLanes = kChan * 2 / 16;  // lanes per row of 16-byte pieces
    const int pr = lane / kRowLanes, pc = lane % kRowLanes;
#pragma unroll
    for (int f = 0; f < TF; ++f) {
#pragma unroll
      for (int c = 0; c < CA; ++c)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          v4h o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            // float(acc) * (sa * sb) rounded once to half, the scale product kept in fp32: the arithmetic of the integer tiles
            const float sc = s_a[f] * (float)s_b[c][g][e];
            o[e] = (_Float16)keep_f32(acc[c][f][4 * g + e] * sc);
          }
          *reinterpret_cast<v4h*>(patch + tok_l * kPitch + (c * 32 + 8 * g + ch_l) * 2) = o;
        }
      // same-wave LDS traffic is ordered: no barrier between the patch writes above and the reads below, nor before the next round
#pragma unroll
      for (int r0 = 0; r0 < 32; r0 += 64 / kRowLanes) {
        const int row = r0 + pr;
        const v4i v = *reinterpret_cast<const v4i*>(patch + row * kPitch + pc * 16);
        const int m = m0 + f * 32 + row, n = n0 + wave * kChan + pc * 8;
        if (m < M && n < N) gstore_stream<v4i>(t.C + (long)m * N + n, v);
      }
    }
  }
};

}  // namespace mxmoe
