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

#include <utility>

#include <type_traits>

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

enum class Op { I8, I4, F16, F8, BF16 };  // F8: OCP e4m3 codes on the fp8 matrix instruction, fp32 accumulators; BF16: bfloat16 operands and outputs

// What one problem looks like to a tile.
struct TileArgs {
  const uint8_t* A;      // activations  [M, K]  (int8 / packed int4 / fp16), K contiguous
  const uint8_t* B;      // weights      [N, K]
  const _Float16* sa;    // per-token scales   [M]   (w-a formats)
  const _Float16* sb;    // per-channel scales [N]   (w-a formats) or group scale/zero table (weight-only)
  _Float16* C;           // output [M, N] fp16 row-major
  int32_t* acc_dump;     // optional [M, N] int32 / fp32-bits accumulator dump (tests), may be null
  int M, N, K;           // M = end row of the segment this tile belongs to (rows at or past M are not computed)
  int row0;              // first row of the segment: tile_m counts BM-row tiles from here
  int tile_m, tile_n;
};

// Keeps a freshly computed fp32 value opaque to the optimiser.  Without it the compiler folds "fp32 multiply, then convert to
// fp16" into one v_fma_mixlo_f16, which rounds the exact product once; the reference arithmetic (and its CPU restatement) rounds
// to fp32 first and to fp16 second, and the two differ on ties.
__device__ __forceinline__ float keep_f32(float v) {
  asm("" : "+v"(v));  // not volatile: it may be scheduled freely, it just cannot be looked through
  return v;
}

// Loads / stores through pointers known to be global memory.  Pointers fetched from the per-problem pointer arrays are
// generic to the compiler, which would emit flat_* instructions; those also count on the LDS counter, so every wait for an
// LDS read would wait for the global prefetch as well.
#define MXMOE_GLOBAL __attribute__((address_space(1)))
template <class T>
__device__ __forceinline__ T gload(const void* p) {
  return *(const MXMOE_GLOBAL T*)(p);
}
template <class T>
__device__ __forceinline__ void gstore(void* p, const T& v) {
  *(MXMOE_GLOBAL T*)(p) = v;
}
// Output rows are written once and read by a later kernel: a streaming store keeps them from displacing the operands that the
// workgroups of the launch still share in L2.
template <class T>
__device__ __forceinline__ void gstore_stream(void* p, const T& v) {
  __builtin_nontemporal_store(v, (MXMOE_GLOBAL T*)(p));
}

// Raw buffer resource over `bytes` bytes at `p` (stride 0: offsets are plain byte offsets, loads past the end return zero).
__device__ __forceinline__ v4i make_rsrc(const void* p, unsigned bytes) {
  const uint64_t a = (uint64_t)p;
  v4i r;
  r[0] = (int)(uint32_t)a;
  r[1] = (int)((uint32_t)(a >> 32) & 0xFFFFu);
  r[2] = (int)bytes;
  r[3] = 0x00020000;
  return r;
}

// One wave-wide 16-byte-per-lane load from a buffer straight into LDS (no register staging): lane l's 16 bytes land at
// lds_addr + 16*l.  Issued as inline assembly so that the compiler does not serialise later LDS reads behind it; completion is
// tracked by hand with vm_wait<N>() (loads retire in order).
__device__ __forceinline__ void dma16_to_lds(const v4i& rsrc, int lds_addr, int voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" : : "s"(lds_addr), "v"(voffset), "s"(rsrc), "s"(soffset) : "memory", "m0");
}
// 16-byte-per-lane global load whose completion the caller tracks itself (the compiler's own bookkeeping knows nothing of the
// direct-to-LDS loads that share the counter and would drain the queue far too early).  The value may only be used after
// vm_wait_for<N>(v) with N = number of vector-memory loads issued after this one; a value that is never used must still be
// passed to vm_wait_for before its register may die (the load writes the register whenever it completes).
__device__ __forceinline__ v4i gload16_untracked(const uint8_t* p) {
  v4i v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
  return v;
}
template <int N>
__device__ __forceinline__ void vm_wait_for(v4i& v) {
  asm volatile("s_waitcnt vmcnt(%1) ; landed %0" : "+v"(v) : "n"(N) : "memory");  // the comment names the register for the build's ISA check
}
template <int N>
__device__ __forceinline__ void vm_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// Swizzle of the four 16-byte chunks of a 64-byte LDS row.  A wave-wide 16-byte read is served 16 lanes (256 bytes, all 64
// banks) per cycle; lanes 0..15 read the same chunk of 16 consecutive rows, so rows r, r+4, r+8, r+12 (same position inside
// a 256-byte bank line) must store that chunk at four different places.  XORing the chunk index with row bits 1..2 separates
// every second row, bit 3 on top separates the two halves of the 16 rows; the same map is conflict-free if the hardware
// serves 8 lanes (128 bytes) per cycle.
__device__ __forceinline__ int lds_swizzle(int r) { return ((r >> 1) & 3) ^ ((r >> 3) & 1); }

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>): a loop whose index is a compile-time constant in the body
template <int... Is, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// Scheduling pattern of one pipeline unit: KMF times (one MFMA, then an even share of the unit's NV VALU instructions).
template <int NV, int KMF, int M>
__device__ __forceinline__ void sched_mfma_valu() {
  if constexpr (M < KMF) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (NV > 0) __builtin_amdgcn_sched_group_barrier(0x002, (NV + KMF - 1 - M) / KMF, 0);
    sched_mfma_valu<NV, KMF, M + 1>();
  }
}

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
template <>
struct OpTraits<Op::F8> {
  using Acc = v16f;
  static constexpr int kBitsPerElem = 8;
};
template <>
struct OpTraits<Op::BF16> {
  using Acc = v16f;
  static constexpr int kBitsPerElem = 16;
};
// operands and outputs are floating-point numbers of 16 bits (no scales, fp32 accumulators written out after one rounding)
template <Op OP>
constexpr bool kFloat16Op = OP == Op::F16 || OP == Op::BF16;

// fp32 -> bfloat16 bits, round to nearest even (NaN stays a quiet NaN)
__device__ __forceinline__ unsigned short bf16_bits(float x) {
  unsigned u = __float_as_uint(x);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return x != x ? (unsigned short)0x7FC0 : (unsigned short)(u >> 16);
}

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
  static constexpr int kStages = 3;
  static constexpr int kLdsBytes = kStages * kStageBytes;
  static constexpr int kAccRegs = FM * FN * 16;
  static constexpr int kWavesWanted = 2;  // waves per SIMD a kernel of such tiles is compiled for
  static constexpr int kABits = OpTraits<OP>::kBitsPerElem, kWBits = kABits;  // bits per activation / weight element
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
    const int m0 = t.row0 + t.tile_m * BM, n0 = t.tile_n * BN;

    // ---- global -> LDS staging plan.  A K slice of the tile is (BM + BN) rows of 64 bytes = (BM + BN) / 16 wave-wide loads of
    // 1 KB, dealt round-robin to the 4 waves.  Each load writes 16 consecutive LDS rows; lane l fills 16-byte slot (row l/4, slot
    // l%4) and therefore fetches the chunk the swizzle maps there.  The buffer resources cover exactly the valid rows of the
    // tile, so rows past M (or N) arrive as zeros.
    const int a_rows = min(BM, M - m0), b_rows = min(BN, N - n0);
    const v4i rs_a = make_rsrc(t.A + (long)m0 * row_bytes, (unsigned)(a_rows * row_bytes));
    const v4i rs_b = make_rsrc(t.B + (long)n0 * row_bytes, (unsigned)(b_rows * row_bytes));
    constexpr int kDmaTotal = (BM + BN) / 16, kDmaA = BM / 16;
    constexpr int kDma = (kDmaTotal + kWaves - 1) / kWaves;  // loads per wave per slice
    const int uwave = __builtin_amdgcn_readfirstlane(wave);
    const int lds_base = (int)(uintptr_t)smem;
    int dma_voff[kDma];
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
      const int ii = uwave + kWaves * i;
      const int r = (ii < kDmaA ? ii : ii - kDmaA) * 16 + (lane >> 2);
      dma_voff[i] = r * (int)row_bytes + (((lane & 3) ^ lds_swizzle(r)) << 4);
    }
    // load i of this wave (i < kDma) of the slice at byte offset koff, into stage `stage`; `live` = false turns it into a load of
    // zero bytes (nothing is fetched, nothing lands in LDS, the load still counts for s_waitcnt like any other)
    auto dma_one = [&](int i, int koff, int stage, bool live) {
      const int ii = uwave + kWaves * i;
      if (kDmaTotal % kWaves == 0 || ii < kDmaTotal) {
        v4i rs = ii < kDmaA ? rs_a : rs_b;
        if (!live) rs[2] = 0;
        dma16_to_lds(rs, lds_base + stage * kStageBytes + ii * 1024, dma_voff[i], koff);
      }
    };
    // whether this wave has a load number kDma-1 (the 1 KB pieces of a slice do not always divide evenly among the waves)
    const bool has_last = kDmaTotal % kWaves == 0 || uwave + kWaves * (kDma - 1) < kDmaTotal;

    // ---- LDS -> MFMA fragment plan: lane reads row (lane & 31) of a 32-row block, chunk 2*ks + (lane >> 5) ----
    const int lrow = lane & 31;
    const int swz = lds_swizzle(lrow);
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

    // The main loop is software-pipelined by hand at the granularity of one "unit" = one k-step of one 32-channel block
    // (FM or 2*FM MFMAs).  While the MFMAs of unit u run, the packed fragment of unit u+LA is read from LDS and the fragment of
    // unit u+1 is widened to MFMA operands (int4 only); the activation-side operands of the next k-step are read at the first
    // unit of a k-step and widened, a few registers per unit, into a second operand buffer during its last units.  So LDS
    // latency (which grows well beyond its idle value while direct-to-LDS loads are landing) and the unpack VALU work hide
    // under the matrix pipe, and the VALU work is spread evenly between the MFMAs.
    // Three LDS stages let the read-ahead run into the next K slice:
    //   iteration kt:  the loads of slice kt+2 into stage (kt+2)%3 are issued one or two per unit (a burst of them delays the
    //   LDS reads of every wave on the CU); units 0..UB-1 touch stage kt%3 only; at unit UB the wave waits for its loads of
    //   slice kt+1 and passes the barrier; the remaining units also read stage (kt+1)%3.
    // The loop body is branch-free: past the end of K the loads are zero-length (they fetch nothing) and the read-ahead touches
    // a stage whose contents are never used.
    constexpr int U = 2 * FN;  // units per K slice
    static_assert(FN == 2 || FN == 4, "the fragment ring below assumes 4 or 8 units per K slice");
    constexpr int LA = U == 8 ? 5 : 3;               // units of read-ahead of the packed B fragments
    constexpr int RB = LA > 3 ? 8 : 4;               // ring slots for them (slot = unit % RB)
    constexpr int UB = (U - LA < FN) ? U - LA : FN;  // unit that holds the barrier
    constexpr int NW = FN >= 4 ? 2 : 1;              // units over which the next k-step's A operands are widened
    constexpr int kAPiece = FM * 4 / NW;             // dwords of packed A widened per such unit
    constexpr int kOps = OP == Op::I4 ? 2 : 1;       // operand registers per fragment (low / high nibbles)
    // load i of a slice is issued at the top of unit i * U / kDma; at the barrier unit the loads of the current iteration issued
    // so far are the only ones that may still be in flight
    constexpr int kIssuedAtBarrier = ((UB + 1) * kDma + U - 1) / U;
    constexpr bool kLastBeforeBarrier = (kDma - 1) * U / kDma <= UB;
    auto lds_a = [&](const uint8_t* st, int step, int i) { return *reinterpret_cast<const v4i*>(st + ((fa + i * 32 * kRowBytes) ^ (step << 5))); };
    auto lds_b = [&](const uint8_t* st, int step, int j) { return *reinterpret_cast<const v4i*>(st + ((fb + j * 32 * kRowBytes) ^ (step << 5))); };
    // nibble n of a byte -> int8 holding 16 * signed(n): even elements via (x << 4), odd via x, both masked to the high nibbles
    auto widen = [&](const v4i& p, v4i* o) {
      if constexpr (OP == Op::I4) {
        o[0] = (p << 4) & (int)0xF0F0F0F0;
        o[1] = p & (int)0xF0F0F0F0;
      } else {
        o[0] = p;
      }
    };
    auto mma = [&](Acc& c, const v4i* a, const v4i* b) {
      if constexpr (OP == Op::I8) {
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[0], a[0], c, 0, 0, 0);
      } else if constexpr (OP == Op::I4) {
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[0], a[0], c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[1], a[1], c, 0, 0, 0);
      } else if constexpr (OP == Op::BF16) {
        typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, b[0]), __builtin_bit_cast(v8bf, a[0]), c, 0, 0, 0);
      } else {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, b[0]), __builtin_bit_cast(v8h, a[0]), c, 0, 0, 0);
      }
    };

    v4i aop[2][FM][kOps];  // A operands of the current k-step (buffer = k-step parity) and of the next one
    v4i pa[FM];            // packed A fragments of the next k-step (int4 only)
    v4i pb[RB];            // packed B fragments of units u+1 .. u+LA
    v4i bop[2][kOps];      // B operands of units u, u+1

    // prologue: slices 0 and 1 in flight, wait for slice 0 (loads retire in order), prime the fragment pipeline
#pragma unroll
    for (int i = 0; i < kDma; ++i) dma_one(i, 0, 0, true);
#pragma unroll
    for (int i = 0; i < kDma; ++i) dma_one(i, kRowBytes, 1, KT > 1);
    if (has_last) vm_wait<kDma>(); else vm_wait<kDma - 1>();
    __syncthreads();
#pragma unroll
    for (int i = 0; i < FM; ++i) widen(lds_a(smem, 0, i), aop[0][i]);
#pragma unroll
    for (int u = 1; u < LA; ++u) pb[u] = lds_b(smem, u / FN, u % FN);
    widen(lds_b(smem, 0, 0), bop[0]);

    int sidx = 0;
#pragma unroll 1
    for (int kt = 0; kt < KT; ++kt) {
      const uint8_t* sc = smem + sidx * kStageBytes;
      const int nidx = sidx == 2 ? 0 : sidx + 1;
      const uint8_t* sn = smem + nidx * kStageBytes;
      // slice kt+2 goes into the stage that was last read before the previous iteration's barrier
      const int nstage = nidx == 2 ? 0 : nidx + 1;
      const int nkoff = __builtin_amdgcn_readfirstlane((kt + 2) * kRowBytes);
      const bool nlive = kt + 2 < KT;
      static_for<U>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        constexpr int step = u / FN, j = u % FN;
        static_for<kDma>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          if constexpr (i * U / kDma == u) dma_one(i, nkoff, nstage, nlive);
        });
        // reads of this slice's stage: packed B fragment of unit u+LA, A fragments of k-step 1
        if (u + LA < U) pb[(u + LA) % RB] = lds_b(sc, (u + LA) / FN, (u + LA) % FN);
        if (u == 0) {
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            if constexpr (OP == Op::I4) pa[i] = lds_a(sc, 1, i); else aop[1][i][0] = lds_a(sc, 1, i);
          }
        }
        if (u == UB) {
          // this wave's part of slice kt+1 is in LDS (only its loads of slice kt+2 may be in flight); after the barrier
          // everybody's part is, and everybody is done reading the stage that the next iteration's loads overwrite
          if (!kLastBeforeBarrier || has_last) vm_wait<kIssuedAtBarrier>(); else vm_wait<kIssuedAtBarrier - 1>();
          __syncthreads();
        }
        // reads of the next slice's stage
        if (u + LA >= U) pb[(u + LA) % RB] = lds_b(sn, (u + LA - U) / FN, (u + LA - U) % FN);
        if (u == FN) {
#pragma unroll
          for (int i = 0; i < FM; ++i) {
            if constexpr (OP == Op::I4) pa[i] = lds_a(sn, 0, i); else aop[0][i][0] = lds_a(sn, 0, i);
          }
        }
        // operands of unit u+1, and this unit's share of the next k-step's A operands
        widen(pb[(u + 1) % RB], bop[(u + 1) & 1]);
        if constexpr (OP == Op::I4) {
          if (j >= FN - NW) {
#pragma unroll
            for (int d = (j - (FN - NW)) * kAPiece; d < (j - (FN - NW) + 1) * kAPiece; ++d) {
              aop[step ^ 1][d / 4][0][d % 4] = (pa[d / 4][d % 4] << 4) & (int)0xF0F0F0F0;
              aop[step ^ 1][d / 4][1][d % 4] = pa[d / 4][d % 4] & (int)0xF0F0F0F0;
            }
          }
        }
#pragma unroll
        for (int i = 0; i < FM; ++i) mma(acc[i][j], aop[step][i], bop[u & 1]);
        // issue order inside the unit: LDS reads first, then the VALU work dealt evenly between the MFMAs
        __builtin_amdgcn_sched_group_barrier(0x100, 1 + FM, 0);
        sched_mfma_valu<(OP == Op::I4 ? 12 + (j >= FN - NW ? 3 * kAPiece : 0) : 0), kOps * FM, 0>();
        __builtin_amdgcn_sched_barrier(0);  // keep the units in program order: the pipeline above is the schedule
      });
      sidx = nidx;
    }
    vm_wait<0>();  // nothing may still land in LDS once the epilogue reuses it

    // ---- epilogue.  Lane holds token m = lane & 31 and channels 8*(r/4) + 4*(lane >> 5) + (r & 3) of each 32x32 block.
    // The scaled fp16 results go through a per-wave LDS patch laid out [token][channel] so that the global stores are 16 bytes
    // per lane along a row (TN*2 contiguous bytes per token) instead of 8-byte pieces scattered over 32 rows.
    const int nq = (lane >> 5) * 4;
    // all scales of this lane are fetched in one batch of independent, unconditional loads (indices clamped into the tensor;
    // rows / channels past the edge are never stored), issued before the barrier so that their latency overlaps the wait for
    // the slowest wave
    float s_a[FM];
    v4h s_b[FN][4];
    if constexpr (!kFloat16Op<OP>) {
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        const int m = min(m0 + wm * TM + i * 32 + lrow, M - 1);
        s_a[i] = (float)gload<_Float16>(t.sa + m);
        // the int4 accumulator holds 256 * sum; 2^-8 folded into the (exact) scale product gives bit-identical results to
        // shifting first: float(256 * x) == 256 * float(x), and scaling by a power of two commutes with rounding
        if constexpr (OP == Op::I4) s_a[i] *= 0.00390625f;
      }
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = min(n0 + wn * TN + j * 32 + q * 8 + nq, N - 4);  // N is a multiple of 8, so a quad is all-in or all-out
          s_b[j][q] = gload<v4h>(t.sb + n);
        }
    }
    if (t.acc_dump) {  // parity tests only
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm * TM + i * 32 + lrow, n = n0 + wn * TN + j * 32 + (r / 4) * 8 + nq + (r & 3);
            const auto v = acc[i][j][r];
            int a;
            if constexpr (kFloat16Op<OP>) a = __builtin_bit_cast(int, (float)v); else a = (int)v;
            if constexpr (OP == Op::I4) a >>= 8;  // exact
            if (m < M && n < N) gstore<int>(t.acc_dump + (long)m * N + n, a);
          }
    }
    __syncthreads();  // every wave is done reading the pipeline stages: LDS can be reused
    constexpr int kPitch = TN * 2 + 8;  // bytes per token row of the patch; the odd multiple of 8 spreads rows over banks
    // the patch holds FI of the wave's FM 32-row blocks at a time (all of them when the pipeline's LDS is large enough)
    constexpr int FI = kWaves * TM * kPitch <= kLdsBytes ? FM : (kWaves * (TM / 2) * kPitch <= kLdsBytes ? FM / 2 : 1);
    static_assert(kWaves * FI * 32 * kPitch <= kLdsBytes && FM % FI == 0, "epilogue patch must fit the pipeline's LDS");
    uint8_t* patch = smem + wave * (FI * 32 * kPitch);
    constexpr int kLanesPerRow = TN / 8;           // 16-byte pieces per token row
    constexpr int kRowsPerPass = 64 / kLanesPerRow;
    const int pr = lane / kLanesPerRow, pc = lane % kLanesPerRow;
#pragma unroll
    for (int i0 = 0; i0 < FM; i0 += FI) {
#pragma unroll
      for (int ii = 0; ii < FI; ++ii) {
        const int i = i0 + ii;
        const int ml = ii * 32 + lrow;
#pragma unroll
        for (int j = 0; j < FN; ++j) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int nl = j * 32 + q * 8 + nq;
            v4h o;
            if constexpr (OP == Op::F16) {
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = (_Float16)acc[i][j][q * 4 + e];
            } else if constexpr (OP == Op::BF16) {
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = __builtin_bit_cast(_Float16, bf16_bits(acc[i][j][q * 4 + e]));
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                // float(acc) * (sa * sb) rounded to half, as the reference epilogue (mm_tile.cuh:490-493, 642-646) except that the
                // scale product stays in fp32, where it is exact: the reference rounds it to fp16 first, which turns subnormal
                // (a few significant bits) for typical int8 scales and breaks the 1e-2 agreement with the fake-quant path.
                const float sc = s_a[i] * (float)s_b[j][q][e];
                o[e] = (_Float16)keep_f32((float)acc[i][j][q * 4 + e] * sc);
              }
            }
            *reinterpret_cast<v4h*>(patch + ml * kPitch + nl * 2) = o;
          }
        }
      }
      // same-wave LDS traffic is ordered, so no barrier is needed between the patch writes above and the reads below, nor before
      // the next round of writes
#pragma unroll
      for (int r0 = 0; r0 < FI * 32; r0 += kRowsPerPass) {
        const int ml = r0 + pr;
        const int m = m0 + wm * TM + i0 * 32 + ml;
        const int n = n0 + wn * TN + pc * 8;
        const v4i v = *reinterpret_cast<const v4i*>(patch + ml * kPitch + pc * 16);
        if (m < M && n < N) gstore_stream<v4i>(t.C + (long)m * N + n, v);
      }
    }
  }
};

// ---------------------------------------------------------------------------------------------------------------------------------
// WxAxTile: w4a4 / w8a8 tile whose WEIGHTS never touch LDS.
//
// Expert weights are static, so they are stored in HBM in MFMA fragment order (mxmoe_amd.pack.pack_wxax_fragments):
//   [N/32 channel blocks][K slices of 64 B][2 k-steps][64 lanes][16 B],  lane l = 16-byte k-group (l >> 5) of channel (l & 31).
// A wave's operand of one k-step of one 32-channel block is then a single coalesced 1 KB load straight into registers.  The 4
// waves of a workgroup each own BN/4 = 64 channels (no weight is loaded twice) and all BM token rows; only the activations
// (BM x 64 B per slice) go through LDS (direct-to-LDS loads, 3-stage ring, swizzled as in MfmaTile).  Compared with staging
// both operands, LDS carries a third of the write traffic and two thirds of the read traffic of a w8a8 slice, and the reads
// no longer queue behind landing weight data.
//
// Pipeline unit = one k-step of one 32-channel block (2*FM or FM MFMAs), 4 units per K slice.  At unit u the wave
//   - issues this unit's share of the activation loads of slice kt+2 and re-loads the weight fragment used by unit u-1 for
//     slice kt+kDepth (its registers are free again): kDepth * 4 KB of weights per wave are always in flight;
//   - at the first unit of a k-step reads the activation fragments of the next k-step from LDS;
//   - int4: widens the weight fragment of unit u+1, and on the last unit of a k-step the activation fragments of the next
//     k-step, each right after its last use.
// Waits: vmcnt counts the direct-to-LDS loads and the weight loads together, in issue order; the barrier unit (2) waits until
// only the loads issued after this wave's activation loads of slice kt+1 are outstanding (a fixed count, see kYounger).
template <Op OP, int BM_, int BN_>
struct WxAxTile {
  static_assert(OP == Op::I4 || OP == Op::I8 || OP == Op::F8, "one byte or half a byte per value");
  static constexpr Op kOp = OP;
  static constexpr int BM = BM_, BN = BN_, WGM = 1, WGN = 4;
  static constexpr int TM = BM, TN = BN / 4;
  static constexpr int FM = TM / 32, FN = TN / 32;
  static_assert(BM % 32 == 0 && FN == 2, "BM x 256 tiles: 4 waves x 64 channels");
  static constexpr int kBits = OpTraits<OP>::kBitsPerElem;
  static constexpr int BK = kRowBytes * 8 / kBits;
  static constexpr int kStageBytes = BM * kRowBytes;
  static constexpr int kStages = 3;
  static constexpr int kPitch = TN * 2 + 8;                      // bytes per token row of the epilogue patch
  static constexpr int FI = FM >= 2 ? 2 : 1;                     // 32-row blocks of the patch written per round
  static constexpr int kPatchBytes = kWaves * FI * 32 * kPitch;
  static constexpr int kLdsBytes = kStages * kStageBytes > kPatchBytes ? kStages * kStageBytes : kPatchBytes;
  static constexpr int kAccRegs = FM * FN * 16;
  static constexpr int kWavesWanted = 2;  // waves per SIMD a kernel of such tiles is compiled for
  static constexpr int kABits = OpTraits<OP>::kBitsPerElem, kWBits = kABits;  // bits per activation / weight element
  static constexpr int kOps = OP == Op::I4 ? 2 : 1;
  static constexpr int U = 4;                                    // units per K slice
  static constexpr int kDmaTotal = BM / 16;                      // 1 KB pieces of one activation slice
  // Activation loads per wave and slice.  Every wave issues the same number of loads, because the hand-placed waits count them: a
  // tile with fewer pieces than waves (BM = 32) has the spare waves fetch a piece a second time (same bytes to the same LDS
  // address) rather than branch on "does this wave load" around the waits - a value that is live across such a branch gets
  // copied between registers, and a copy of a fragment register whose load is still in flight copies stale data.
  static constexpr int kDma = (kDmaTotal + kWaves - 1) / kWaves;
  static_assert(kDmaTotal % kWaves == 0 || kDma == 1, "fewer pieces than waves: one (possibly repeated) piece per wave");
  static_assert(kDma <= U, "one activation load per unit");
  // loads issued after a wave's last activation load of a slice and before the barrier unit of the next iteration
  static constexpr int kYounger = (U - (kDma - 1)) + (kDma < 2 ? kDma : 2) + 2;
  // K slices of weight fragments in flight per wave: int8 slices are half as long in time, so they are fetched further ahead
  static constexpr int kDepth = OP == Op::I4 ? 2 : 4;
  using Acc = typename OpTraits<OP>::Acc;

  // One 16-byte fragment pair of the byte formats.  int8: one instruction over the 32 k of the pair.  fp8 (e4m3): two instructions of
  // 16 k, the first on the low 8 bytes of both lanes' fragments, the second on the high 8; which k a byte stands for is the same on
  // both sides, and the sum runs over all of them either way (w8a8_g-1_sym_E4M3 of the reference: MMA_E4M3_K32,
  // mxmoe/kernels/src/include/mm_tile.cuh:696-697).
  __device__ static __forceinline__ void mma_bytes(Acc& c, const v4i& w, const v4i& a) {
    if constexpr (OP == Op::F8) {
      typedef long v2l __attribute__((ext_vector_type(2)));
      const v2l wl = __builtin_bit_cast(v2l, w), al = __builtin_bit_cast(v2l, a);
      c = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(wl[0], al[0], c, 0, 0, 0);
      c = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(wl[1], al[1], c, 0, 0, 0);
    } else {
      c = __builtin_amdgcn_mfma_i32_32x32x32_i8(w, a, c, 0, 0, 0);
    }
  }

  // Vector-memory loads a wave issues in units a..b of one iteration: one weight fragment per unit, plus one activation load in
  // each of the first nd units (before the fragment).
  static constexpr int ops_in(int a, int b, int nd) {
    int n = 0;
    for (int u = a; u <= b; ++u) n += 1 + (u < nd ? 1 : 0);
    return n;
  }
  // Loads issued after the load of fragment `uf` (= k-step * FN + block) of a slice, up to and including the unit that first
  // uses it: the fragment of unit uf is (re)loaded at unit uf+1 kDepth slices earlier and first used at unit uf-1 (int4: widened
  // one unit ahead) or uf (int8).
  static constexpr int younger_than_fragment(int uf, int nd) {
    const int ul = (uf + 1) % U, kl = -kDepth + (uf == U - 1 ? 1 : 0);
    const int uc = OP == Op::I4 ? (uf + U - 1) % U : uf, kc = OP == Op::I4 && uf == 0 ? -1 : 0;
    return ops_in(ul + 1, U - 1, nd) + ops_in(0, U - 1, nd) * (kc - kl - 1) + ops_in(0, uc, nd);
  }

  __device__ static __forceinline__ void widen(const v4i& p, v4i* o) {
    if constexpr (OP == Op::I4) {
      o[0] = (p << 4) & (int)0xF0F0F0F0;
      o[1] = p & (int)0xF0F0F0F0;
    } else {
      o[0] = p;
    }
  }

  __device__ static __forceinline__ void run(const TileArgs& t, uint8_t* __restrict__ smem) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = t.M, N = t.N;
    const long row_bytes = (long)t.K * kBits / 8;
    const int KT = (int)(row_bytes / kRowBytes);
    const int m0 = t.row0 + t.tile_m * BM, n0 = t.tile_n * BN;

    // activations: global -> LDS
    const int a_rows = min(BM, M - m0);
    const v4i rs_a = make_rsrc(t.A + (long)m0 * row_bytes, (unsigned)(a_rows * row_bytes));
    const int lds_base = (int)(uintptr_t)smem;
    int dma_voff[kDma];
#pragma unroll
    for (int i = 0; i < kDma; ++i) {
      const int r = ((wave + kWaves * i) % kDmaTotal) * 16 + (lane >> 2);
      dma_voff[i] = r * (int)row_bytes + (((lane & 3) ^ lds_swizzle(r)) << 4);
    }
    auto dma_a = [&](int i, int kt, int stage) {
      const int ii = (wave + kWaves * i) % kDmaTotal;
      v4i rs = rs_a;
      if (kt >= KT) rs[2] = 0;  // past the end of K: a load of zero bytes, still counted by vmcnt
      dma16_to_lds(rs, lds_base + stage * kStageBytes + ii * 1024, dma_voff[i], __builtin_amdgcn_readfirstlane(kt * kRowBytes));
    };
    // wait until the weight fragment `uf` of the current slice has arrived (see younger_than_fragment), then hand it out
    auto ready = [&](auto ufc, v4i& frag) {
      constexpr int uf = decltype(ufc)::value;
      vm_wait_for<younger_than_fragment(uf, kDma)>(frag);
    };
    const int lrow = lane & 31;
    const int fa = lrow * kRowBytes + (((lane >> 5) ^ lds_swizzle(lrow)) << 4);
    auto lds_a = [&](const uint8_t* st, int step, int i) { return *reinterpret_cast<const v4i*>(st + ((fa + i * 32 * kRowBytes) ^ (step << 5))); };

    // weights: global -> registers, fragment (j, step) of slice kt at ((nb * KT + kt) * 2 + step) * 1 KB
    const int nblk = (N + 31) / 32;
    const uint8_t* bptr[FN];
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const int nb = min(n0 / 32 + wave * FN + j, nblk - 1);  // blocks past N re-read the last one; their results are never stored
      bptr[j] = t.B + (long)nb * KT * 2048 + lane * 16;
    }
    auto load_b = [&](int j, int step, int kt) { return gload16_untracked(bptr[j] + ((long)min(kt, KT - 1) * 2 + step) * 1024); };

    Acc acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    v4i pbq[kDepth][FN][2];  // packed weight fragments [slice % kDepth][block][k-step]
    v4i bop[2][kOps];        // int4: widened weight operands of units u, u+1
    v4i aop[2][FM][kOps];    // activation operands; int8 double-buffers them by k-step parity, int4 widens in place (buffer 0)
    v4i pa[FM];              // int4: packed activation fragments of the next k-step

    auto mma = [&](Acc& c, const v4i* a, const v4i* b) {
      mma_bytes(c, b[0], a[0]);
      if constexpr (OP == Op::I4) mma_bytes(c, b[1], a[1]);
    };

    // ---- prologue: slices 0 .. kDepth-2 complete, then the load pattern of one (virtual) iteration for slice kDepth-1, so that
    // the counts below hold from kt = 0
#pragma unroll
    for (int i = 0; i < kDma; ++i) dma_a(i, 0, 0);
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int s = 0; s < 2; ++s) pbq[d][j][s] = load_b(j, s, d);
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int s = 0; s < 2; ++s) vm_wait_for<0>(pbq[d][j][s]);
    __syncthreads();
    static_for<U>([&](auto uc) {
      constexpr int u = decltype(uc)::value;
      if constexpr (u < kDma) dma_a(u, 1, 1);
      asm volatile("" ::: "memory");
      if constexpr (u == 0) pbq[kDepth - 2][1][1] = load_b(1, 1, kDepth - 2);  // in place of "fragment of the previous iteration's last unit"
      else pbq[kDepth - 1][(u - 1) % FN][(u - 1) / FN] = load_b((u - 1) % FN, (u - 1) / FN, kDepth - 1);
      asm volatile("" ::: "memory");
    });
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      if constexpr (OP == Op::I4) {
        const v4i p = lds_a(smem, 0, i);
        widen(p, aop[0][i]);
      } else {
        aop[0][i][0] = lds_a(smem, 0, i);
      }
    }
    if constexpr (OP == Op::I4) widen(pbq[0][0][0], bop[0]);

    // ---- one K slice; P = kt % kDepth (compile-time, so the ring slots are fixed registers).  The loop below always runs whole
    // groups of kDepth slices.  A slice past the end of K (`live` false) issues the same loads and passes the same waits and
    // barriers as any other (its activation loads have zero length, its weight loads re-read the last slice), so the hand-computed
    // counts hold on every path through the loop; it only skips the LDS reads, the widening and the matrix instructions.
    auto slice = [&](auto parc, int kt, const uint8_t* sc, const uint8_t* sn, int nstage) {
      constexpr int P = decltype(parc)::value;
      constexpr int Pprev = (P + kDepth - 1) % kDepth, Pnext = (P + 1) % kDepth;
      const bool live = kt < KT;
      static_for<U>([&](auto uc) {
        constexpr int u = decltype(uc)::value;
        constexpr int step = u / FN, j = u % FN;
        if (u == 2) {
          // this wave's activation loads of slice kt+1 have landed; after the barrier everybody's have, and everybody is done
          // reading the stage that the loads of the next iteration overwrite
          vm_wait<kYounger>();
          __syncthreads();
        }
        if constexpr (u < kDma) dma_a(u, kt + 2, nstage);
        asm volatile("" ::: "memory");
        // re-load the fragment that unit u-1 used, kDepth slices ahead
        if constexpr (u == 0) pbq[Pprev][1][1] = load_b(1, 1, kt - 1 + kDepth);
        else pbq[P][(u - 1) % FN][(u - 1) / FN] = load_b((u - 1) % FN, (u - 1) / FN, kt + kDepth);
        asm volatile("" ::: "memory");
        if constexpr (OP == Op::I4) {
          // weight operands of unit u+1
          if constexpr (u + 1 < U) ready(std::integral_constant<int, u + 1>{}, pbq[P][(u + 1) % FN][(u + 1) / FN]);
          else ready(std::integral_constant<int, 0>{}, pbq[Pnext][0][0]);
        } else {
          ready(uc, pbq[P][j][step]);
        }
        if (live) {
          // activation fragments of the next k-step
          if (j == 0) {
#pragma unroll
            for (int i = 0; i < FM; ++i) {
              const v4i p = step == 0 ? lds_a(sc, 1, i) : lds_a(sn, 0, i);
              if constexpr (OP == Op::I4) pa[i] = p; else aop[step ^ 1][i][0] = p;
            }
          }
          if constexpr (OP == Op::I4) {
            if constexpr (u + 1 < U) widen(pbq[P][(u + 1) % FN][(u + 1) / FN], bop[(u + 1) & 1]);
            else widen(pbq[Pnext][0][0], bop[0]);
#pragma unroll
            for (int i = 0; i < FM; ++i) {
              mma(acc[i][j], aop[0][i], bop[u & 1]);
              if (j == FN - 1) widen(pa[i], aop[0][i]);  // next k-step's operand, right after the last use of this one
            }
            __builtin_amdgcn_sched_group_barrier(0x100, FM, 0);
            sched_mfma_valu<12 + (j == FN - 1 ? 12 * FM : 0), 2 * FM, 0>();
          } else {
#pragma unroll
            for (int i = 0; i < FM; ++i) mma_bytes(acc[i][j], pbq[P][j][step], aop[step][i][0]);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    };

    int sidx = 0;
#pragma unroll 1
    for (int kt0 = 0; kt0 < KT; kt0 += kDepth) {
      static_for<kDepth>([&](auto dc) {
        constexpr int d = decltype(dc)::value;
        const int nidx = sidx == 2 ? 0 : sidx + 1;
        const int nn = nidx == 2 ? 0 : nidx + 1;
        slice(dc, kt0 + d, smem + sidx * kStageBytes, smem + nidx * kStageBytes, nn);
        sidx = nidx;
      });
    }
    // Nothing may still land in LDS once the epilogue reuses it, and nothing in registers either: the fragments fetched past the
    // end of K are never used, so without this tie the compiler would hand their registers to the epilogue while the loads are
    // still in flight.
#pragma unroll
    for (int d = 0; d < kDepth; ++d)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int s = 0; s < 2; ++s) vm_wait_for<0>(pbq[d][j][s]);

    // ---- epilogue (as MfmaTile): lane holds token lane & 31 and channels 8*(r/4) + 4*(lane >> 5) + (r & 3) of each 32x32 block
    const int nq = (lane >> 5) * 4;
    float s_a[FM];
    v4h s_b[FN][4];
#pragma unroll
    for (int i = 0; i < FM; ++i) {
      const int m = min(m0 + i * 32 + lrow, M - 1);
      s_a[i] = (float)gload<_Float16>(t.sa + m);
      if constexpr (OP == Op::I4) s_a[i] *= 0.00390625f;  // the int4 accumulator holds 256 * sum (exact power of two)
    }
#pragma unroll
    for (int j = 0; j < FN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = min(n0 + wave * TN + j * 32 + q * 8 + nq, N - 4);
        s_b[j][q] = gload<v4h>(t.sb + n);
      }
    if (t.acc_dump) {  // parity tests only
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int m = m0 + i * 32 + lrow, n = n0 + wave * TN + j * 32 + (r / 4) * 8 + nq + (r & 3);
            const auto v = acc[i][j][r];
            int a;
            if constexpr (OP == Op::F8) a = __builtin_bit_cast(int, (float)v); else a = (int)v;  // fp8: the fp32 sum's bit pattern
            if constexpr (OP == Op::I4) a >>= 8;  // exact
            if (m < M && n < N) gstore<int>(t.acc_dump + (long)m * N + n, a);
          }
    }
    __syncthreads();  // every wave is done reading the activation stages: LDS can be reused
    uint8_t* patch = smem + wave * (FI * 32 * kPitch);
    constexpr int kLanesPerRow = TN / 8, kRowsPerPass = 64 / kLanesPerRow;
    const int pr = lane / kLanesPerRow, pc = lane % kLanesPerRow;
#pragma unroll
    for (int i0 = 0; i0 < FM; i0 += FI) {
#pragma unroll
      for (int ii = 0; ii < FI; ++ii) {
        const int i = i0 + ii;
        const int ml = ii * 32 + lrow;
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            v4h o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              // float(acc) * (sa * sb) rounded once to half; the scale product stays in fp32 (see MfmaTile)
              const float sc = s_a[i] * (float)s_b[j][q][e];
              o[e] = (_Float16)keep_f32((float)acc[i][j][q * 4 + e] * sc);
            }
            *reinterpret_cast<v4h*>(patch + ml * kPitch + (j * 32 + q * 8 + nq) * 2) = o;
          }
      }
#pragma unroll
      for (int r0 = 0; r0 < FI * 32; r0 += kRowsPerPass) {
        const int ml = r0 + pr;
        const int m = m0 + i0 * 32 + ml;
        const int n = n0 + wave * TN + pc * 8;
        const v4i v = *reinterpret_cast<const v4i*>(patch + ml * kPitch + pc * 16);
        if (m < M && n < N) gstore_stream<v4i>(t.C + (long)m * N + n, v);
      }
    }
  }
};

}  // namespace mxmoe
