// Diagnostic: one int4 x int4 GEMM on the 6-bit float matrix path, C[M][N] = (A . B^T) * sa[m] * sb[n].
// Every integer -8 .. 8 is a bf6 (e3m2) number and fp32 adds their products exactly (see mfma_probe.hip), so
// v_mfma_scale_f32_32x32x64_f8f6f4 on bf6 operands with unit scales yields the int32 accumulators of the integer tiles as fp32
// integers, at twice the int8 instruction's operations per cycle.  This kernel measures what a tile built on that instruction
// sustains with its operands coming from memory; it is not part of the fused GroupGEMM.
//
// Operand layout (both operands, rows = tokens of A or channels of B): fragments of 32 rows x 64 k, k step major,
//   offset(row block rb, k step ks) = (ks * R/32 + rb) * 1536 bytes,
// a fragment being what one matrix instruction takes from 64 lanes: lane l (row l % 32, k = 64*ks + 32*(l / 32) + i, i = 0..31)
// holds 32 codes = 192 bits, value i at bit 6*i; its first 128 bits lie at byte 16*l of the fragment and its last 64 bits at byte
// 1024 + 8*l, so that a wave reads a fragment with one 16-byte and one 8-byte access per lane, both contiguous across the wave.
//
// Two shapes.  CA = 4: workgroup = 256 tokens x 256 channels, 2 x 2 waves of 128 x 128 (256 accumulator registers per lane: one wave
// per SIMD with the full register budget; every fragment feeds 4 instructions).  CA = 2: workgroup = 128 tokens x 256 channels, four
// waves side by side of 128 x 64 (128 accumulator registers, two workgroups per CU that hide each other's barriers, latencies and
// epilogues; channel fragments feed 4 instructions, token fragments 2, so LDS is read twice as much per instruction).
// Per 64-wide k step a wave takes its 4 token fragments from LDS, where direct-to-LDS loads put the workgroup's token fragments
// (contiguous in memory thanks to the k-step-major order) three steps ahead, and its CA channel fragments straight from global
// memory through a register ring four steps ahead.  All loads of the loop are inline assembly awaited by one hand-counted wait
// per step.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxmoe_tiles.hpp"

namespace {

using namespace mxmoe;
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v2i __attribute__((ext_vector_type(2)));

constexpr int kFrag = 1536;          // bytes of one 32 x 64 fragment
constexpr int kStages = 4;

struct Frag {
  v4i lo;
  v2i hi;
};
__device__ __forceinline__ v8i operand(const Frag& f) { return v8i{f.lo[0], f.lo[1], f.lo[2], f.lo[3], f.hi[0], f.hi[1], 0, 0}; }

// Loads whose completion is tracked by hand, like the direct-to-LDS loads they share the counter with (a compiler-placed wait
// would not know of those and would end up waiting for loads issued moments ago).  Address = scalar base + 32-bit lane offset.
__device__ __forceinline__ Frag load_frag_untracked(const uint8_t* sbase, int off_lo, int off_hi) {
  Frag f;
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(f.lo) : "v"(off_lo), "s"(sbase) : "memory");
  asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(f.hi) : "v"(off_hi), "s"(sbase) : "memory");
  return f;
}
// wait until at most N vector-memory loads are outstanding; the comment names the registers that have landed by then
template <int N>
__device__ __forceinline__ void wait_frags(Frag (&f)[4]) {
  asm volatile("s_waitcnt vmcnt(%8) ; landed %0 %1 %2 %3 %4 %5 %6 %7"
               : "+v"(f[0].lo), "+v"(f[0].hi), "+v"(f[1].lo), "+v"(f[1].hi), "+v"(f[2].lo), "+v"(f[2].hi), "+v"(f[3].lo), "+v"(f[3].hi)
               : "n"(N)
               : "memory");
}
template <int N>
__device__ __forceinline__ void wait_frags(Frag (&f)[2]) {
  asm volatile("s_waitcnt vmcnt(%4) ; landed %0 %1 %2 %3" : "+v"(f[0].lo), "+v"(f[0].hi), "+v"(f[1].lo), "+v"(f[1].hi) : "n"(N) : "memory");
}

template <bool DUMP, int CA>
__global__ void __launch_bounds__(256, CA == 4 ? 1 : 2) bf6_gemm_kernel(const uint8_t* __restrict__ A6, const uint8_t* __restrict__ B6, const _Float16* __restrict__ sa,
                                                          const _Float16* __restrict__ sb, _Float16* __restrict__ C, int32_t* __restrict__ Cint, int M, int N, int K) {
  constexpr int WROWS = CA == 4 ? 2 : 1;    // waves along the tokens
  constexpr int TM = 128 * WROWS;           // tokens per workgroup (channels: 256 either way)
  constexpr int kStage = 4 * WROWS * kFrag; // the workgroup's token fragments of one k step
  constexpr int kDma = CA == 4 ? 3 : 2;     // direct-to-LDS loads per wave and stage (1 KB each)
  constexpr int kPieces = kStage / 1024;    // 12 or 6; with 6 pieces two of the eight loads bring a piece a second time
  constexpr int RD = CA == 4 ? 4 : 2;       // steps the channel-fragment ring runs ahead (alone on its SIMD a wave needs the longer one)
  constexpr int kYounger = RD == 4 ? 2 * CA + 2 * (kDma + 2 * CA) : kDma + 2 * CA;  // outstanding loads a step may begin with, see below
  __shared__ __align__(16) uint8_t smem[kStages * kStage];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = CA == 4 ? wave >> 1 : 0, wn = CA == 4 ? wave & 1 : wave;
  const int KS = K / 64, RB = M / 32, CB = N / 32;
  // workgroup -> tile: each XCD (workgroup id modulo 8) walks a contiguous range of tiles, token tile fastest, so that the
  // workgroups it runs at a time share channel fragments in its L2
  const int tiles_m = M / TM, ntiles = tiles_m * (N / 256);
  const int chunk = (ntiles + 7) / 8;
  const int pt = ((int)blockIdx.x % 8) * chunk + (int)blockIdx.x / 8;
  if (pt >= ntiles) return;
  const int tile_m = pt % tiles_m, tile_n = pt / tiles_m;

  // token fragments: global -> LDS in pieces of 1 KB, kDma per wave and stage
  const v4i rs_a = make_rsrc(A6, (unsigned)((long)RB * KS * kFrag));
  const int lds_base = (int)(uintptr_t)smem;
  const int a_lane = lane * 16;
  auto dma_a = [&](int ks) {
    const int st = ks % kStages;
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
      const int piece = (wave * kDma + i) % kPieces;
      const int soff = __builtin_amdgcn_readfirstlane((ks * RB + tile_m * (TM / 32)) * kFrag + piece * 1024);
      dma16_to_lds(rs_a, __builtin_amdgcn_readfirstlane(lds_base + st * kStage + piece * 1024), a_lane, soff);
    }
  };
  auto lds_a = [&](int ks, int j) {
    const uint8_t* f = smem + (ks % kStages) * kStage + (wm * 4 + j) * kFrag;
    Frag r;
    r.lo = *reinterpret_cast<const v4i*>(f + lane * 16);
    r.hi = *reinterpret_cast<const v2i*>(f + 1024 + lane * 8);
    return r;
  };
  // channel fragments: global -> registers, scalar fragment address plus one lane offset per plane
  const int b_lo = lane * 16, b_hi = 1024 + lane * 8;
  auto load_b = [&](int ks, int j) {
    const int ksc = ks < KS ? ks : KS - 1;  // past the end: re-read the last step (never used), the load count per step stays fixed
    const long off = (long)__builtin_amdgcn_readfirstlane(ksc * CB + tile_n * 8 + wn * CA + j) * kFrag;
    return load_frag_untracked(B6 + off, b_lo, b_hi);
  };

  v16f acc[CA][4];  // [channel fragment][token fragment]
#pragma unroll
  for (int c = 0; c < CA; ++c)
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[c][t][r] = 0.f;

  // Every vector-memory load of the loop is issued and awaited by hand.  Order within step ks: after the barrier the kDma
  // direct-to-LDS loads of stage ks + 3, and after the matrix instructions the 2 CA ring loads of step ks + RD's channel fragments.
  // Ring four steps ahead (one wave per SIMD: nothing else hides a load's latency): when step ks begins, the loads younger than
  // its stage (issued in step ks - 3) are 2 CA + 2 (kDma + 2 CA) = 30, and its channel fragments (issued in step ks - 4) are older
  // still.  Ring two steps ahead: the loads younger than its channel fragments (issued in step ks - 2) are the kDma + 2 CA = 6 of
  // step ks - 1, and its stage is older still.  One wait for "at most that many outstanding" covers both operands either way, and
  // the prologue issues its loads in the order the steps before ks = 0 would have.
  Frag br[RD][CA];
  if constexpr (RD == 4) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
#pragma unroll
      for (int j = 0; j < CA; ++j) br[p][j] = load_b(p, j);
      if (p < 3) dma_a(p);
    }
  } else {
    dma_a(0);
    dma_a(1);
#pragma unroll
    for (int j = 0; j < CA; ++j) br[0][j] = load_b(0, j);
    dma_a(2);
#pragma unroll
    for (int j = 0; j < CA; ++j) br[1][j] = load_b(1, j);
  }

  auto step = [&](auto parc, int ks) {
    constexpr int par = decltype(parc)::value;
    wait_frags<kYounger>(br[par]);
    __syncthreads();  // the stage is complete for every wave, and no wave still reads the stage that is overwritten next
    dma_a(ks + 3 < KS ? ks + 3 : ks);  // (past the end: the stage being read is loaded once more with the same bytes; the count stays fixed)
    Frag af[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) af[t] = lds_a(ks, t);
#pragma unroll
    for (int c = 0; c < CA; ++c) {
      const v8i w = operand(br[par][c]);
#pragma unroll
      for (int t = 0; t < 4; ++t)
        acc[c][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(w, operand(af[t]), acc[c][t], 3, 3, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
    }
    __builtin_amdgcn_sched_barrier(0);  // the ring registers are free only after the last instruction that reads them
#pragma unroll
    for (int j = 0; j < CA; ++j) br[par][j] = load_b(ks + RD, j);
  };
#pragma unroll 1
  for (int ks = 0; ks < KS; ks += RD) {  // K is a multiple of 64 RD: whole rounds of the ring
    step(std::integral_constant<int, 0>{}, ks);
    step(std::integral_constant<int, 1>{}, ks + 1);
    if constexpr (RD == 4) {
      step(std::integral_constant<int, 2>{}, ks + 2);
      step(std::integral_constant<int, 3>{}, ks + 3);
    }
  }
#pragma unroll
  for (int p = 0; p < RD; ++p) wait_frags<0>(br[p]);  // everything has landed (vmcnt(0)), the loads past the end of K included

  // epilogue: lane l holds, of fragment pair (c, t), token l % 32 and channels 8*(r/4) + 4*(l/32) + r%4, r = 0..15.  32 tokens at a
  // time go through a [token][channel] patch in LDS and leave as 16-byte pieces of whole rows of the wave's channels: stores of
  // 8 bytes scattered over 32 rows took longer than the whole K loop.
  __syncthreads();  // every wave is done with the stages
  constexpr int kChan = CA * 32;             // channels of a wave
  constexpr int kPitch = kChan * 2 + 16;
  constexpr int kRowLanes = kChan * 2 / 16;  // lanes per row of 16-byte pieces
  uint8_t* patch = smem + wave * (32 * kPitch);
  const int tok_l = lane & 31, ch_l = (lane >> 5) * 4;
  const int pr = lane / kRowLanes, pc = lane % kRowLanes;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int m_l = tile_m * TM + wm * 128 + t * 32 + tok_l;
    const float sam = (float)sa[m_l];
#pragma unroll
    for (int c = 0; c < CA; ++c) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int nl = c * 32 + 8 * g + ch_l;  // channel within the wave's
        const int n = tile_n * 256 + wn * kChan + nl;
        const v4h s4 = *reinterpret_cast<const v4h*>(sb + n);
        v4h o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (_Float16)(acc[c][t][4 * g + e] * (sam * (float)s4[e]));
        *reinterpret_cast<v4h*>(patch + tok_l * kPitch + nl * 2) = o;
        if (DUMP) {
#pragma unroll
          for (int e = 0; e < 4; ++e) Cint[(long)m_l * N + n + e] = (int)acc[c][t][4 * g + e];
        }
      }
    }
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += 64 / kRowLanes) {
      const int row = r0 + pr;
      const v4i v = *reinterpret_cast<const v4i*>(patch + row * kPitch + pc * 16);
      const int m = tile_m * TM + wm * 128 + t * 32 + row, n = tile_n * 256 + wn * kChan + pc * 8;
      gstore_stream<v4i>(C + (long)m * N + n, v);
    }
  }
}

}  // namespace

// C[M][N] (fp16) = half(acc * (float(sa[m]) * float(sb[n]))) with acc = sum_k a[m][k] * b[n][k] over int4 values stored as bf6
// fragments (layout above; mxmoe_amd.bf6.pack_fragments), and the accumulators themselves as int32 into d_cint when it is given.
// shape 0: workgroups of 256 x 256 (one wave per SIMD), M and K multiples of 256; shape 1: workgroups of 128 x 256 (two per CU), M
// and K multiples of 128 (K >= 256).  N a multiple of 256.  Returns 0, 3 for bad arguments, 4 for a launch error.
extern "C" int mxmoe_bf6_gemm_probe(const void* d_a6, const void* d_b6, const void* d_sa, const void* d_sb, void* d_c, void* d_cint, int M, int N, int K,
                                    int shape, void* stream) {
  const int tm = shape == 0 ? 256 : 128, km = shape == 0 ? 256 : 128;  // rows of a workgroup; k covered by one round of the ring
  if (!d_a6 || !d_b6 || !d_sa || !d_sb || !d_c || shape < 0 || shape > 1 || M < tm || N < 256 || K < 256 || M % tm || N % 256 || K % km) return 3;
  if ((long)M * K / 64 * 48 >= (1L << 32) || (long)N * K / 64 * 48 >= (1L << 31)) return 3;  // operands addressed with 32-bit offsets
  const int ntiles = (M / tm) * (N / 256);
  const int grid = (ntiles + 7) / 8 * 8;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const uint8_t* a6 = static_cast<const uint8_t*>(d_a6);
  const uint8_t* b6 = static_cast<const uint8_t*>(d_b6);
  const _Float16* sa = static_cast<const _Float16*>(d_sa);
  const _Float16* sb = static_cast<const _Float16*>(d_sb);
  _Float16* c = static_cast<_Float16*>(d_c);
  int32_t* ci = static_cast<int32_t*>(d_cint);
  if (shape == 0) {
    if (ci) hipLaunchKernelGGL((bf6_gemm_kernel<true, 4>), dim3(grid), dim3(256), 0, st, a6, b6, sa, sb, c, ci, M, N, K);
    else hipLaunchKernelGGL((bf6_gemm_kernel<false, 4>), dim3(grid), dim3(256), 0, st, a6, b6, sa, sb, c, ci, M, N, K);
  } else {
    if (ci) hipLaunchKernelGGL((bf6_gemm_kernel<true, 2>), dim3(grid), dim3(256), 0, st, a6, b6, sa, sb, c, ci, M, N, K);
    else hipLaunchKernelGGL((bf6_gemm_kernel<false, 2>), dim3(grid), dim3(256), 0, st, a6, b6, sa, sb, c, ci, M, N, K);
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}
