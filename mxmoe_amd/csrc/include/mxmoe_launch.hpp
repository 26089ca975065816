// Fused one-launch GroupGEMM: tile scheduler, per-problem branch dispatch, host launcher and kernel registry.
//
// Mirrors the reference's generated `groupgemm_hz_fused_<i>` pair (kernel + host launcher,
// mxmoe/kernels/compose_kernel.py:150-295, mxmoe/kernels/kernel_sketch.py:82-145) with these differences:
//  * one workgroup per tile instead of a persistent grid: the hardware dispatcher hands out tiles as
//    workgroups retire, which balances the mixed tile costs of a mixed-precision launch;
//  * the tile prefix sum and the per-problem branch index travel in the kernel-argument segment, so a launch
//    performs no allocation, no host-to-device copy and no synchronisation (the reference does
//    cudaMalloc + cudaMemcpy + cudaFree per call, kernel_sketch.py:102-104,142-143);
//  * workgroup ids are remapped so that each of the 8 XCDs (one L2 each; workgroups are dealt round-robin)
//    receives one contiguous run of the tile list, i.e. whole experts, and re-reads of an expert's weights
//    and activations by neighbouring tiles stay inside one L2;
//  * a qcfg may own several tile shapes; the host picks one per problem from its row count.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "mxmoe_tiles.hpp"
#include "mxmoe_grp_tiles.hpp"
#include "mxmoe_bf6_tiles.hpp"
#include "mxmoe_wo_tiles.hpp"

namespace mxmoe {

constexpr int kMaxProblems = 120;  // per launch (the tables ride in the 4 KB kernel argument block); longer problem lists are split into several launches
constexpr int kMaxEntries = 2 * kMaxProblems;  // a problem is run as at most two row segments, each with its own tile shape
constexpr int kNumXcd = 8;
constexpr int kMaxPhases = 8;

struct FusedArgs {
  const uint8_t* const* As;
  const uint8_t* const* Bs;
  const _Float16* const* sa;
  const _Float16* const* sb;
  _Float16* const* Cs;
  int32_t* const* acc;  // optional accumulator dumps (null, or per-problem pointers which may themselves be null)
  const mxmoe_dim3* sizes;
  int problem_offset;   // first problem of this launch inside the arrays above
  int num_entries;
  int total_tiles;
  // Phases: the entries are sorted so that the most expensive tile shapes come first (workgroups are dispatched in index order,
  // so the cheap tiles fill the tail of the launch).  Phase p covers tiles [phase_tile0[p], phase_tile0[p+1]) and workgroups
  // [phase_wg0[p], phase_wg0[p+1]); inside a phase, workgroup v maps to tile (v % 8) * chunk + v / 8 so that each XCD (one L2)
  // works on a contiguous run of tiles.
  int num_phases;
  int phase_tile0[kMaxPhases + 1];
  int phase_wg0[kMaxPhases + 1];
  // Bit p set: phase p maps workgroup v to tile v.  For the skinny weight-only tiles, which share no operand with their neighbours
  // (every tile streams its own weights once): dealing them round-robin to the XCDs balances the memory traffic tile by tile,
  // where contiguous runs would leave the XCD that holds a few long problems behind.
  int phase_flat;
  // One entry per row segment of a problem, 16 bytes so that a workgroup fetches its entry with one scalar load: first tile of the
  // entry (exclusive prefix sum of tiles), first row of the segment inside its problem, rows of the segment, and
  // problem (relative to problem_offset) | tile type << 16.
  struct Entry {
    int first, row0, rows, problem_branch;
  };
  Entry entry[kMaxEntries];
};
static_assert(sizeof(FusedArgs) <= 4096, "kernel arguments are limited to 4 KB");

// Activation bytes that a group of row tiles may hold (see Dispatch::go): half of an XCD's 4 MB L2.
#ifndef MXMOE_GROUP_BYTES
#define MXMOE_GROUP_BYTES (2 << 20)
#endif

template <int I, class... Tiles>
struct Dispatch;
template <int I>
struct Dispatch<I> {
  __device__ static __forceinline__ void go(int, TileArgs&, int, uint8_t*) {}
};
template <int I, class T, class... Rest>
struct Dispatch<I, T, Rest...> {
  __device__ static __forceinline__ void go(int branch, TileArgs& t, int local, uint8_t* smem) {
    if (branch == I) {
      // local index -> (row tile, column tile) as tile_scheduler.cuh:40-49, but row tile fastest: neighbouring workgroups then share
      // one block of weight rows and sweep the problem's activations.  The 64 workgroups that an XCD runs at a time only share
      // what its 4 MB L2 still holds, and they drift apart along K, so a problem whose activations exceed the L2 ends up
      // streaming them once per column tile.  Such a problem is walked in groups of row tiles holding at most 2 MB of
      // activations, each group against all column tiles: the group's activations stay resident whatever the drift, and a block
      // of weights is fetched once per group by row tiles that start together.  The plain order is kept where the estimate of
      // its traffic (activations once per 64 / grid_m column tiles, weights once) is below half of the grouped order's (weights
      // once per group, activations once): very long rows, of which only one or two row tiles fit.
      const int grid_m = (t.M - t.row0 + T::BM - 1) / T::BM;
      const int grid_n = (t.N + T::BN - 1) / T::BN;
      const int tile_bytes = max(T::BM * (t.K / 8) * T::kABits, 1);
      int rg = min(max(MXMOE_GROUP_BYTES / tile_bytes, 1), grid_m);  // row tiles per group
      if (rg < grid_m) {
        const float a_bytes = (float)grid_m * (float)tile_bytes;
        const float b_bytes = (float)t.N * (float)(t.K / 8) * (float)T::kWBits;
        const float grouped = (float)((grid_m + rg - 1) / rg) * b_bytes + a_bytes;
        const float plain = fmaxf((float)grid_n * (float)grid_m * (1.0f / 64.0f), 1.0f) * a_bytes + b_bytes;
        if (grouped >= 2.0f * plain || tile_bytes > MXMOE_GROUP_BYTES) rg = grid_m;  // (a single row tile beyond the budget cannot stay resident either)
      }
      const int per_group = rg * grid_n;
      const int g = local / per_group, r = local - g * per_group;
      const int rows_g = min(rg, grid_m - g * rg);
      t.tile_n = r / rows_g;
      t.tile_m = g * rg + (r - t.tile_n * rows_g);
      T::run(t, smem);
    } else {
      Dispatch<I + 1, Rest...>::go(branch, t, local, smem);
    }
  }
};

// Waves per SIMD the register allocator should aim for: 2 (two co-resident workgroups per CU, 256 registers per lane) unless a
// tile keeps more than 128 accumulator registers per lane, which needs the full 512-register budget of a lone wave.
// A kernel made only of tiles that ask for more waves (the few-token weight-only tiles: latency-bound streams that gain from every
// further workgroup in flight) is compiled for the smallest number any of its tiles asks for.
constexpr int min_of(int a) { return a; }
template <class... R>
constexpr int min_of(int a, R... r) { return a < min_of(r...) ? a : min_of(r...); }
template <class... Tiles>
constexpr int kWavesPerSimd = ((Tiles::kAccRegs > 128) || ...) ? 1 : min_of(Tiles::kWavesWanted...);

// Tables are read through the constant address space: what a workgroup reads from them is the same for all lanes and is not
// written while the kernel runs (a planned launch's tables were written by the planning kernel before it), so every read is a
// scalar load, whether the table came in the kernel arguments or lies in device memory.
#define MXMOE_CONST __attribute__((address_space(4)))
template <class T>
__device__ __forceinline__ T cload(const T* p) {
  return *(const MXMOE_CONST T*)(p);
}
__host__ __device__ __forceinline__ int uni(int v) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __builtin_amdgcn_readfirstlane(v);
#else
  return v;
#endif
}

// Tile that workgroup `wg` of a launch runs, or -1 when it has none (tile_scheduler.cuh:25-37 maps a persistent block's linear
// index the same way; here the index is the workgroup id).  Compiled for the host as well: the scheduler tests replay a whole grid
// through this very function.
template <class ArgsPtr>
__host__ __device__ __forceinline__ int tile_of_workgroup(ArgsPtr args, int wg) {
  const int num_phases = uni(args->num_phases);
  // A planned launch is sized for the worst routing: workgroups past the last phase have no tile (without this test they would
  // be folded back into the last phase by the XCD remap below and run one of its tiles a second time), and a launch whose plan
  // holds no tile at all has nothing else in its tables that may be read.
  if (num_phases <= 0 || wg >= uni(args->phase_wg0[num_phases])) return -1;
  int ph = 0;
  while (ph + 1 < num_phases && wg >= uni(args->phase_wg0[ph + 1])) ++ph;
  const int v = wg - uni(args->phase_wg0[ph]);
  const int tile0 = uni(args->phase_tile0[ph]);
  const int ntiles = uni(args->phase_tile0[ph + 1]) - tile0;
  const int chunk = (ntiles + kNumXcd - 1) / kNumXcd;
  const int pt = (uni(args->phase_flat) >> ph & 1) ? v : (v % kNumXcd) * chunk + v / kNumXcd;
  return pt < ntiles ? tile0 + pt : -1;
}

template <class ArgsPtr, class... Tiles>
__device__ __forceinline__ void fused_body(ArgsPtr args, uint8_t* smem) {
  const int tile = tile_of_workgroup(args, (int)blockIdx.x);
  if (tile < 0) return;
  // tile_scheduler.cuh:25-37 — the entry that holds the tile: last entry whose first tile is <= tile (binary search here; all
  // indices are wave-uniform, so these are scalar loads)
  int lo = 0, hi = uni(args->num_entries) - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (uni(args->entry[mid].first) <= tile) lo = mid; else hi = mid - 1;
  }
  const int en_first = uni(args->entry[lo].first), en_row0 = uni(args->entry[lo].row0), en_rows = uni(args->entry[lo].rows), en_pb = uni(args->entry[lo].problem_branch);
  const int local = tile - en_first;
  const int gp = uni(args->problem_offset) + (en_pb & 0xFFFF);
  const mxmoe_dim3* sizes = args->sizes;
  const uint8_t* const* As = args->As;
  const uint8_t* const* Bs = args->Bs;
  const _Float16* const* sa = args->sa;
  const _Float16* const* sb = args->sb;
  _Float16* const* Cs = args->Cs;
  int32_t* const* acc = args->acc;
  TileArgs t;
  t.A = cload(As + gp);
  t.B = cload(Bs + gp);
  t.sa = sa ? cload(sa + gp) : nullptr;
  t.sb = sb ? cload(sb + gp) : nullptr;
  t.C = cload(Cs + gp);
  t.acc_dump = acc ? cload(acc + gp) : nullptr;
  t.row0 = en_row0;
  t.M = t.row0 + en_rows;  // rows past the segment are treated like rows past the problem
  t.N = uni((int)cload(&sizes[gp].y));
  t.K = uni((int)cload(&sizes[gp].z));
  t.tile_m = t.tile_n = 0;
  Dispatch<0, Tiles...>::go(en_pb >> 16, t, local, smem);
}

template <class... Tiles>
__global__ void __launch_bounds__(kThreads, kWavesPerSimd<Tiles...>) fused_group_gemm_kernel(const FusedArgs args) {
  extern __shared__ __align__(16) uint8_t smem[];
  fused_body<const FusedArgs*, Tiles...>(&args, smem);
}

// The same kernel with its tables in device memory, where a planning kernel wrote them from the tokens-per-expert counts: the
// host then needs no copy of the counts, so a layer forward neither synchronises nor depends on its routing when it is enqueued
// (or captured into a graph).  The grid is sized for the worst case; workgroups past the planned tiles leave at once.
template <class... Tiles>
__global__ void __launch_bounds__(kThreads, kWavesPerSimd<Tiles...>) fused_group_gemm_planned_kernel(const FusedArgs* __restrict__ args) {
  extern __shared__ __align__(16) uint8_t smem[];
  fused_body<const MXMOE_CONST FusedArgs*, Tiles...>((const MXMOE_CONST FusedArgs*)args, smem);
}

// ------------------------------------------------------------------ host side ------------------------------------------------------------------

enum class Fmt { FP16, W8A8, W4A4, W4A16, W3A16, W2A16, W4A4G128, W8A16, UNSUPPORTED };

// Format of a problem from its QParams.  Weight-only formats come with one (scale, zero) pair per channel and 128-wide K group or
// per channel (group size -1): the tiles are the same, the packer repeats a per-channel pair for every group.
__host__ __device__ inline Fmt classify(const mxmoe_qparams& q) {
  if (q.a_bits >= 16 && q.w_bits >= 16) return Fmt::FP16;
  if (q.a_bits == 8 && q.w_bits == 8 && q.gsize == -1 && q.sym) return Fmt::W8A8;
  if (q.a_bits == 4 && q.w_bits == 4 && q.gsize == -1 && q.sym) return Fmt::W4A4;
  if (q.a_bits == 4 && q.w_bits == 4 && q.gsize == 128 && q.sym) return Fmt::W4A4G128;
  if (q.a_bits >= 16 && (q.gsize == 128 || q.gsize == -1)) {
    if (q.w_bits == 8) return Fmt::W8A16;
    if (q.w_bits == 4) return Fmt::W4A16;
    if (q.w_bits == 3) return Fmt::W3A16;
    if (q.w_bits == 2) return Fmt::W2A16;
  }
  return Fmt::UNSUPPORTED;
}
__host__ __device__ inline bool is_weight_only(Fmt f) { return f == Fmt::W8A16 || f == Fmt::W4A16 || f == Fmt::W3A16 || f == Fmt::W2A16; }

inline const char* fmt_name(Fmt f, bool sym) {
  switch (f) {
    case Fmt::FP16: return "fp16";
    case Fmt::W8A8: return "w8a8_g-1_sym";
    case Fmt::W4A4: return "w4a4_g-1_sym";
    case Fmt::W8A16: return sym ? "w8a16_g128_sym" : "w8a16_g128_asym";
    case Fmt::W4A16: return sym ? "w4a16_g128_sym" : "w4a16_g128_asym";
    case Fmt::W3A16: return sym ? "w3a16_g128_sym" : "w3a16_g128_asym";
    case Fmt::W2A16: return sym ? "w2a16_g128_sym" : "w2a16_g128_asym";
    case Fmt::W4A4G128: return "w4a4_g128_sym";
    default: return "unsupported";
  }
}

struct BranchInfo {
  Fmt fmt;
  int BM, BN, BK, WGM, WGN;
  int lds_bytes;
  int k_multiple;  // K must be a multiple of this
  int max_m;       // largest M this branch accepts (skinny weight-only tiles), or 0 = any
  int k_min = 0;   // smallest K this branch accepts, or 0 = one k_multiple
  // What QParams cannot say about the operands a branch takes: 0 as the format's table in the header says; 1 both operands of w4a4 as
  // bf6 fragments (the tiles on the 6-bit float matrix path); 2 both operands of w8a8 as fp8 e4m3 codes with fp32 accumulation
  // (w8a8_g-1_sym_E4M3, mxmoe/kernels/tile_config.py:45: QParams (8, 8, -1, sym) there as well).  A kernel with such a branch is
  // never chosen automatically: the caller names it, because only the caller knows what its operands hold.
  int variant = 0;
};
constexpr int kVariantBf6 = 1, kVariantFp8 = 2, kVariantBf16 = 3;

template <class T>
struct BranchOf;
template <Op OP, int BM, int BN, int WGM, int WGN>
struct BranchOf<MfmaTile<OP, BM, BN, WGM, WGN>> {
  static BranchInfo get() {
    using T = MfmaTile<OP, BM, BN, WGM, WGN>;
    const Fmt f = OP == Op::I8 ? Fmt::W8A8 : (OP == Op::I4 ? Fmt::W4A4 : Fmt::FP16);
    // bfloat16 problems carry the QParams of fp16 ones (16 / 16 bits): which of the two a kernel computes is the kernel's variant
    return BranchInfo{f, BM, BN, T::BK, WGM, WGN, T::kLdsBytes, T::BK, 0, 0, OP == Op::BF16 ? kVariantBf16 : 0};
  }
};
template <int BM>
struct BranchOf<WxAxGTile<BM>> {
  static BranchInfo get() {
    using T = WxAxGTile<BM>;
    return BranchInfo{Fmt::W4A4G128, BM, T::BN, T::BK, 1, 4, T::kLdsBytes, T::BK, 0};
  }
};
template <Op OP, int BM, int BN>
struct BranchOf<WxAxTile<OP, BM, BN>> {
  static BranchInfo get() {
    using T = WxAxTile<OP, BM, BN>;
    return BranchInfo{OP == Op::I4 ? Fmt::W4A4 : Fmt::W8A8, BM, BN, T::BK, 1, 4, T::kLdsBytes, T::BK, 0, 0, OP == Op::F8 ? kVariantFp8 : 0};
  }
};
template <int BM>
struct BranchOf<Bf6Tile<BM>> {
  // same format as the int4 tiles on the int8 instruction; what differs is the layout both operands are handed over in (6-bit
  // fragments), so the two kinds never share a kernel: the kernel a caller picks says which layout its operands have
  static BranchInfo get() {
    using T = Bf6Tile<BM>;
    return BranchInfo{Fmt::W4A4, BM, T::BN, T::BK, 1, 4, T::kLdsBytes, 128, 0, 256, kVariantBf6};
  }
};
template <int WBITS, int BN, int KP, int RING, int WAVES, int MB>
struct BranchOf<SkinnyWoTile<WBITS, BN, KP, RING, WAVES, MB>> {
  static BranchInfo get() {
    using T = SkinnyWoTile<WBITS, BN, KP, RING, WAVES, MB>;
    return BranchInfo{WBITS == 8 ? Fmt::W8A16 : WBITS == 4 ? Fmt::W4A16 : WBITS == 3 ? Fmt::W3A16 : Fmt::W2A16, T::BM, BN, 128, 1, 4, T::kLdsBytes, 128, 0};
  }
};

using LaunchFn = hipError_t (*)(const FusedArgs&, int grid, int lds, hipStream_t);
using LaunchPlannedFn = hipError_t (*)(const FusedArgs* d_args, int grid, int lds, hipStream_t);

// How a registered kernel walks a problem list (the reference generates one host launcher per policy, kernel_sketch.py:82-145
// fused, :148-274 sequential, :277-406 multi-stream):
//   Fused       one launch over all problems;
//   Sequential  one launch per run of consecutive problems of equal format, all on the caller's stream;
//   MultiStream the same launches dealt round-robin to side streams that fork from and join the caller's stream.
enum class Policy { Fused = 0, Sequential = 1, MultiStream = 2 };

struct FusedKernel {
  std::string name;  // "[qcfg: (BM,BN,BK) (WGM,WGN,1) 2], ...<fn name>" — same shape as registry.cuh:42-70
  std::vector<BranchInfo> branches;
  int lds_bytes;
  LaunchFn launch;
  Policy policy;
  mxmoe_func_t func;  // the kernel as a function of the reference's FuncType (registry.cuh:28-39)
  LaunchPlannedFn launch_planned;  // the same kernel reading its tables from device memory (device-side planning)
  int plan_index;                  // index into plan_infos()
  // Largest row count per problem this kernel is meant for, 0 = any.  A kernel with a limit is preferred by the automatic choice when
  // every problem of the list stays within it (the few-token kernels: same results, more workgroups per CU).
  int max_rows_hint;
};

inline std::vector<FusedKernel>& registry() {
  static std::vector<FusedKernel> r;
  return r;
}

inline std::string& last_error() {
  static thread_local std::string e;
  return e;
}

template <int WBITS, int BM, int BN>
struct BranchOf<WoMfmaTile<WBITS, BM, BN>> {
  static BranchInfo get() {
    using T = WoMfmaTile<WBITS, BM, BN>;
    return BranchInfo{WBITS == 8 ? Fmt::W8A16 : WBITS == 4 ? Fmt::W4A16 : WBITS == 3 ? Fmt::W3A16 : Fmt::W2A16, BM, BN, 128, T::WM, 4 / T::WM, T::kLdsBytes, 128, 0};
  }
};

// Run time of one tile of a branch relative to the 128 x 256 tile of the same format (same K), from the kernel-profile table
// measured on MI355X (ms per 256 tiles at K = 2048).  Small tiles pay a fixed prologue / epilogue and use the matrix pipe less
// well; the weight-only entries compare the skinny streaming tile with the 128 x 128 dequantise-to-fp16 tile (the 128 x 256
// one, four waves side by side with twice the tokens each, does twice the work in 1.5 times the time).
// The 32-token few-token tile costs the same for every bit width (it waits for memory, not for bytes), and two of them must not
// look cheaper than one 128 x 256 tile, which runs half its loop for a problem of 33 .. 64 rows.
inline double tile_cost(const BranchInfo& b) {
  struct Row { Fmt f; int bm, bn; double c; };
  static const Row table[] = {
      // (inside a fused kernel the small integer tiles run at the occupancy of the largest one, which costs them part of the
      // advantage they show as single-tile kernels in the profile table)
      {Fmt::W4A4, 128, 256, 1.00}, {Fmt::W4A4, 64, 256, 0.58}, {Fmt::W4A4, 32, 256, 0.48},
      {Fmt::W8A8, 128, 256, 1.00}, {Fmt::W8A8, 64, 256, 0.74}, {Fmt::W8A8, 32, 256, 0.56},
      {Fmt::FP16, 128, 256, 1.00}, {Fmt::FP16, 64, 256, 0.69}, {Fmt::FP16, 32, 256, 0.53}, {Fmt::FP16, 128, 128, 0.57}, {Fmt::FP16, 256, 128, 1.09},
      {Fmt::W4A16, 16, 128, 0.37}, {Fmt::W4A16, 16, 64, 0.20}, {Fmt::W4A16, 32, 128, 0.50}, {Fmt::W4A16, 128, 128, 1.00}, {Fmt::W4A16, 128, 256, 1.50},
      {Fmt::W3A16, 16, 128, 0.31}, {Fmt::W3A16, 16, 64, 0.20}, {Fmt::W3A16, 32, 128, 0.50}, {Fmt::W3A16, 128, 128, 1.00}, {Fmt::W3A16, 128, 256, 1.50},
      {Fmt::W2A16, 16, 128, 0.25}, {Fmt::W2A16, 16, 64, 0.20}, {Fmt::W2A16, 32, 128, 0.50}, {Fmt::W2A16, 128, 128, 1.00}, {Fmt::W2A16, 128, 256, 1.50},
      {Fmt::W8A16, 16, 128, 0.60}, {Fmt::W8A16, 16, 64, 0.35}, {Fmt::W8A16, 32, 128, 0.66}, {Fmt::W8A16, 128, 128, 1.00},
      {Fmt::W4A4G128, 64, 256, 1.00}, {Fmt::W4A4G128, 32, 256, 0.60},
  };
  for (const Row& r : table)
    if (r.f == b.fmt && r.bm == b.BM && r.bn == b.BN) return r.c;
  return (0.22 + 0.78 * b.BM / 128.0) * b.BN / 256.0;  // shapes without a measurement
}

// Rough run time of one tile across formats, used only to order the tile list (expensive shapes first): the matrix pipe runs
// fp16 at half the int8 rate, and int4 operands are widened to int8.
inline double branch_cost(const BranchInfo& b) {
  const double per_k = b.fmt == Fmt::FP16 ? 2.0 : is_weight_only(b.fmt) ? 1.2 : (b.fmt == Fmt::W8A8 ? 1.25 : 1.0);
  return tile_cost(b) * per_k;
}

// What the planners (the host launcher and the device-side planning kernel) need to know of a kernel's branches, as plain data.
constexpr int kMaxBranches = 32;
struct PlanBranch {
  int fmt, BM, BN, k_multiple;
  int bm_log2, bn_log2;  // of a tile dimension that is a power of two (the usual case: the planners shift instead of dividing), else -1
  double cost;           // tile_cost
  double cost_per_row;   // tile_cost / BM
};
// A phase of such tiles keeps the plain workgroup order (no XCD remap): the few-token weight-only tiles stream their own weights
// and share nothing but a few rows of activations with their neighbours.
__host__ __device__ inline bool flat_phase(const PlanBranch& b) { return b.BM <= 16 || (is_weight_only((Fmt)b.fmt) && b.BM < 128); }
// Tiles of size `dim` (2^`lg` when lg >= 0) that cover `x`.
__host__ __device__ inline int tiles_over(int x, int dim, int lg) { return lg >= 0 ? (x + dim - 1) >> lg : (x + dim - 1) / dim; }
constexpr int kNumFmts = (int)Fmt::UNSUPPORTED;
struct PlanInfo {
  int nb;                    // branches
  int order[kMaxBranches];   // branch indices, most expensive tile first (branch_cost); ties keep the registration order
  // the branches of one format as a list in registration order (-1 ends it): the planners look at no other branch
  int first_of_fmt[kNumFmts];
  int next_of_fmt[kMaxBranches];
  PlanBranch b[kMaxBranches];
};

// Cheapest branch of format `f` for a block of `rows` x `N` run with one tile shape: cost = row tiles * column tiles * tile_cost.
__host__ __device__ inline int pick_branch(const PlanInfo& k, int f, int rows, int N) {
  int best = -1;
  double best_cost = 0;
  if (f < 0 || f >= kNumFmts) return -1;
  for (int i = k.first_of_fmt[f]; i >= 0; i = k.next_of_fmt[i]) {
    const PlanBranch& b = k.b[i];
    const double c = (double)tiles_over(rows, b.BM, b.bm_log2) * tiles_over(N, b.BN, b.bn_log2) * b.cost;
    if (best < 0 || c < best_cost - 1e-9 || (c < best_cost + 1e-9 && b.BM > k.b[best].BM)) {
      best = i;
      best_cost = c;
    }
  }
  return best;
}

struct Segment {
  int row0, rows, branch;
};

// Split the M rows of an M x N problem into at most two segments: whole tiles of the shape that is cheapest per output element,
// then the remainder with the shape that covers it most cheaply.  Returns the number of segments (0 for M == 0), or -1 when
// the kernel has no tile for `f`.
__host__ __device__ inline int plan_segments(const PlanInfo& k, int f, int M, int N, Segment out[2]) {
  int big = -1;
  double big_unit = 0;
  if (f < 0 || f >= kNumFmts) return -1;
  for (int i = k.first_of_fmt[f]; i >= 0; i = k.next_of_fmt[i]) {
    const PlanBranch& b = k.b[i];
    const double unit = b.cost_per_row * tiles_over(N, b.BN, b.bn_log2);  // cost per row of the problem
    if (big < 0 || unit < big_unit - 1e-12 || (unit < big_unit + 1e-12 && b.BM > k.b[big].BM)) {
      big = i;
      big_unit = unit;
    }
  }
  if (big < 0) return -1;
  if (M <= 0) return 0;
  auto cost_of = [&](int branch, int rows) {
    const PlanBranch& b = k.b[branch];
    return (double)tiles_over(rows, b.BM, b.bm_log2) * tiles_over(N, b.BN, b.bn_log2) * b.cost;
  };
  const int bm = k.b[big].BM, bm_lg = k.b[big].bm_log2;
  const int full = bm_lg >= 0 ? (M >> bm_lg) << bm_lg : (M / bm) * bm, rem = M - full;
  const int whole = pick_branch(k, f, M, N);
  if (rem == 0 || full == 0) {
    out[0] = Segment{0, M, whole};
    return 1;
  }
  const int rb = pick_branch(k, f, rem, N);
  if (cost_of(whole, M) <= cost_of(big, full) + cost_of(rb, rem) + 1e-9 || rb == big) {
    out[0] = Segment{0, M, rb == big ? big : whole};
    return 1;
  }
  out[0] = Segment{0, full, big};
  out[1] = Segment{full, rem, rb};
  return 2;
}

__host__ __device__ inline int segment_tiles(const PlanInfo& k, const Segment& sg, int N) {
  const PlanBranch& b = k.b[sg.branch];
  return tiles_over(sg.rows, b.BM, b.bm_log2) * tiles_over(N, b.BN, b.bn_log2);
}

inline PlanInfo make_plan_info(const std::vector<BranchInfo>& branches) {
  PlanInfo k;
  std::memset(&k, 0, sizeof k);
  k.nb = std::min((int)branches.size(), kMaxBranches);
  for (int i = 0; i < k.nb; ++i) {
    auto log2_of = [](int v) {
      int lg = -1;
      if (v > 0 && (v & (v - 1)) == 0)
        for (lg = 0; (1 << lg) < v; ++lg) {}
      return lg;
    };
    const double cost = tile_cost(branches[i]);
    k.b[i] = PlanBranch{(int)branches[i].fmt, branches[i].BM, branches[i].BN, branches[i].k_multiple, log2_of(branches[i].BM), log2_of(branches[i].BN), cost,
                        cost / branches[i].BM};
    k.order[i] = i;
  }
  std::stable_sort(k.order, k.order + k.nb, [&](int x, int y) { return branch_cost(branches[x]) > branch_cost(branches[y]); });
  for (int f = 0; f < kNumFmts; ++f) k.first_of_fmt[f] = -1;
  for (int i = k.nb - 1; i >= 0; --i) {
    const int f = k.b[i].fmt;
    k.next_of_fmt[i] = -1;
    if (f < 0 || f >= kNumFmts) continue;
    k.next_of_fmt[i] = k.first_of_fmt[f];
    k.first_of_fmt[f] = i;
  }
  return k;
}

inline std::vector<PlanInfo>& plan_infos() {
  static std::vector<PlanInfo> v;
  return v;
}
inline const PlanInfo& plan_of(const FusedKernel& k) { return plan_infos()[k.plan_index]; }

template <class... Tiles>
hipError_t launch_fused(const FusedArgs& a, int grid, int lds, hipStream_t s) {
  // more than 64 KB of dynamic LDS must be opted into, once per device (kept out of library load time: no HIP call before first use)
  static bool lds_opted_in[64] = {};
  if (lds > 64 * 1024) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return hipGetLastError();
    if (dev >= 0 && dev < 64 && !lds_opted_in[dev]) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&fused_group_gemm_kernel<Tiles...>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      if (e != hipSuccess) return e;
      lds_opted_in[dev] = true;
    }
  }
  hipLaunchKernelGGL((fused_group_gemm_kernel<Tiles...>), dim3(grid), dim3(kThreads), lds, s, a);
  return hipGetLastError();
}

template <class... Tiles>
hipError_t launch_fused_planned(const FusedArgs* d_args, int grid, int lds, hipStream_t s) {
  static bool lds_opted_in[64] = {};
  if (lds > 64 * 1024) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return hipGetLastError();
    if (dev >= 0 && dev < 64 && !lds_opted_in[dev]) {
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&fused_group_gemm_planned_kernel<Tiles...>), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
      if (e != hipSuccess) return e;
      lds_opted_in[dev] = true;
    }
  }
  hipLaunchKernelGGL((fused_group_gemm_planned_kernel<Tiles...>), dim3(grid), dim3(kThreads), lds, s, d_args);
  return hipGetLastError();
}

inline int group_gemm(int kernel_id, const void* const* As, const void* const* Bs, const void* const* sa, const void* const* sb, void* const* Cs,
                      int32_t* const* acc, const mxmoe_dim3* d_sizes, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int count, hipStream_t stream);

// Stream the FuncType functions launch on (that type has no stream argument; the reference launches on stream 0,
// kernel_sketch.py:123), and the status of the calling thread's last FuncType call (that type returns void).
inline hipStream_t& func_stream() {
  static thread_local hipStream_t s = nullptr;
  return s;
}
inline int& func_status() {
  static thread_local int rc = 0;
  return rc;
}

inline int checked_group_gemm(int kernel_id, const void* const* As, const void* const* Bs, const void* const* sa, const void* const* sb, void* const* Cs,
                              void* const* Ds, int32_t* const* acc, const mxmoe_dim3* d_sizes, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int count,
                              hipStream_t stream) {
  if (count < 0 || (count > 0 && (!As || !Bs || !Cs || !d_sizes || !h_sizes || !h_q))) {
    last_error() = "null argument";
    return 5;
  }
  // Ds is accepted and never read, as in the reference's kernels (hz_fused.cuh:89,110 store through ptr_Cs only; its own caller
  // passes a second array with the same entries, test.cu:446-459): results go to Cs.
  (void)Ds;
  return group_gemm(kernel_id, As, Bs, sa, sb, Cs, acc, d_sizes, h_sizes, h_q, count, stream);
}

// One C function of the reference's FuncType per registered kernel: the template instance is the function, its static member the
// registry index it launches.  A failure is reported like the reference's launcher reports CUDA errors (message on stderr,
// helper.h:186-193) but the process is left alive; mxmoe_last_status() returns the code.
template <int POLICY, class... Tiles>
struct FuncThunk {
  static inline int kernel_id = -1;
  static void call(mxmoe_half** As, mxmoe_half** Bs, mxmoe_half** sa, mxmoe_half** sb, mxmoe_half** Cs, mxmoe_half** Ds, int64_t*, int64_t*, int64_t*, int64_t*,
                   mxmoe_dim3* d_sizes, mxmoe_dim3* h_sizes, mxmoe_qparams*, mxmoe_qparams* h_q, int problem_count) {
    const int rc = checked_group_gemm(kernel_id, (const void* const*)As, (const void* const*)Bs, (const void* const*)sa, (const void* const*)sb, (void* const*)Cs,
                                      (void* const*)Ds, nullptr, d_sizes, h_sizes, h_q, problem_count, func_stream());
    func_status() = rc;
    if (rc != 0) fprintf(stderr, "mxmoe: %s\n", last_error().c_str());
  }
};

template <class... Tiles>
int register_fused(const char* fn_name, Policy policy = Policy::Fused, int max_rows_hint = 0) {
  static_assert(sizeof...(Tiles) <= kMaxBranches, "the planners' branch table holds kMaxBranches tile shapes per kernel");
  FusedKernel k;
  k.policy = policy;
  k.max_rows_hint = max_rows_hint;
  k.branches = {BranchOf<Tiles>::get()...};
  k.lds_bytes = 0;
  std::string n;
  for (const auto& b : k.branches) {
    char buf[160];
    snprintf(buf, sizeof buf, "[%s%s: (%d,%d,%d) (%d,%d,1) 2], ", b.variant == kVariantBf16 ? "bf16" : fmt_name(b.fmt, b.fmt == Fmt::W8A8 || b.fmt == Fmt::W4A4),
             b.variant == kVariantFp8 ? "_E4M3" : "", b.BM, b.BN,
             b.BK, b.WGM, b.WGN);
    n += buf;
    k.lds_bytes = std::max(k.lds_bytes, b.lds_bytes);
  }
  k.name = n + fn_name;
  k.launch = &launch_fused<Tiles...>;
  k.launch_planned = &launch_fused_planned<Tiles...>;
  k.plan_index = (int)plan_infos().size();
  plan_infos().push_back(make_plan_info(k.branches));
  const int id = (int)registry().size();
  switch (policy) {
    case Policy::Fused: FuncThunk<0, Tiles...>::kernel_id = id; k.func = &FuncThunk<0, Tiles...>::call; break;
    case Policy::Sequential: FuncThunk<1, Tiles...>::kernel_id = id; k.func = &FuncThunk<1, Tiles...>::call; break;
    default: FuncThunk<2, Tiles...>::kernel_id = id; k.func = &FuncThunk<2, Tiles...>::call; break;
  }
  registry().push_back(k);
  return id;
}

// Operand variant (BranchInfo::variant) of the kernel's tiles for format `f`, 0 when it has none or the plain ones.
inline int kernel_variant(const FusedKernel& k, Fmt f) {
  for (const BranchInfo& b : k.branches)
    if (b.fmt == f && b.variant) return b.variant;
  return 0;
}
inline bool kernel_takes_bf6(const FusedKernel& k) { return kernel_variant(k, Fmt::W4A4) == kVariantBf6; }
inline bool kernel_has_variants(const FusedKernel& k) {
  for (const BranchInfo& b : k.branches)
    if (b.variant) return true;
  return false;
}

// A kernel can run a problem list when it has a branch for every format in it.  The automatic choice (kernel_id = -1) never
// falls on a kernel with operand variants (bf6 fragments, fp8 codes): QParams do not say what the operands hold, so those kernels
// are asked for by id.
inline bool kernel_covers(const FusedKernel& k, const mxmoe_qparams* q, int count) {
  for (int i = 0; i < count; ++i) {
    const Fmt f = classify(q[i]);
    Segment sg[2];
    if (f == Fmt::UNSUPPORTED || plan_segments(plan_of(k), (int)f, 1, 256, sg) < 0) return false;
  }
  return true;
}

// The kernel the launcher picks when the caller names none: the first fused kernel without operand variants that has a tile for every
// format; a kernel made for few rows per problem wins when no problem has more (`max_rows` < 0: row counts unknown, none of those).
inline int auto_kernel_for(const mxmoe_qparams* h_q, int count, long max_rows) {
  auto& reg = registry();
  int plain = -1;
  for (int i = 0; i < (int)reg.size(); ++i) {
    if (reg[i].policy != Policy::Fused || kernel_has_variants(reg[i]) || !kernel_covers(reg[i], h_q, count)) continue;
    if (reg[i].max_rows_hint > 0) {
      if (max_rows >= 0 && max_rows <= reg[i].max_rows_hint) return i;
    } else if (plain < 0) {
      plain = i;
    }
  }
  return plain;
}
// (A few-row kernel runs 16-row tiles: it is meant for lists whose problems mostly fit one such tile.  When more than a quarter of
// the non-empty problems need several, the kernels that also hold the 32-row few-token tile do better, whatever the largest count.)
inline int auto_kernel(const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int count) {
  long max_rows = 0;
  int live = 0, over = 0;
  for (int i = 0; i < count; ++i) {
    max_rows = std::max(max_rows, (long)h_sizes[i].x);
    live += h_sizes[i].x > 0;
    over += h_sizes[i].x > 16;
  }
  return auto_kernel_for(h_q, count, 4 * over > live ? -1 : max_rows);
}

// K a multiple of the tile's K step, N a multiple of 8 (16 for the weight-only layouts)
inline bool shape_ok(const BranchInfo& bi, const mxmoe_dim3& sz) {
  const bool wo = is_weight_only(bi.fmt);
  return sz.z != 0 && sz.z % bi.k_multiple == 0 && (int)sz.z >= bi.k_min && sz.y % 8 == 0 && !(wo && sz.y % 16 != 0);
}

// Tile tables of one launch over problems [base, base + n) (n <= kMaxProblems): entries, phases, totals of `a`; *grid receives the
// workgroups to launch.  Host-only arithmetic.
inline int build_fused_tables(const FusedKernel& k, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int base, int n, FusedArgs& a, int* grid) {
  a.problem_offset = base;
  a.phase_flat = 0;
  const PlanInfo& pi = plan_of(k);
  struct Entry {
    int row0, rows, problem, branch, tiles;
  };
  Entry entries[kMaxEntries];
  int nent = 0;
  for (int i = 0; i < n; ++i) {
    const mxmoe_dim3& sz = h_sizes[base + i];
    const Fmt f = classify(h_q[base + i]);
    Segment sg[2];
    const int ns = f == Fmt::UNSUPPORTED ? -1 : plan_segments(pi, (int)f, (int)sz.x, (int)sz.y, sg);
    if (ns < 0) {
      last_error() = "quant type not supported";
      return 1;
    }
    for (int j = 0; j < ns; ++j) {
      const BranchInfo& bi = k.branches[sg[j].branch];
      if (!shape_ok(bi, sz)) {
        char buf[200];
        snprintf(buf, sizeof buf, "problem %d: shape [%u,%u,%u] not supported by tile %s (K %% %d, N %% 8)", base + i, sz.x, sz.y, sz.z, fmt_name(bi.fmt, true), bi.k_multiple);
        last_error() = buf;
        return 3;
      }
      entries[nent++] = Entry{sg[j].row0, sg[j].rows, i, sg[j].branch, segment_tiles(pi, sg[j], (int)sz.y)};
    }
  }
  // Most expensive tile shape first.  Inside a shape, the problems whose K is above the launch's smallest K go first (their tiles
  // run longest: a shared expert with a wider intermediate, say; workgroups are dispatched in index order, and the longest
  // jobs first is what keeps the tail of the launch short), then the others; problems keep their order otherwise (neighbouring tiles
  // share operands).
  uint32_t kmin = ~0u;
  for (int i = 0; i < n; ++i) kmin = std::min(kmin, h_sizes[base + i].z);
  int total = 0, ne = 0, wg = 0, np = 0;
  for (int oi = 0; oi < pi.nb; ++oi) {
    const int b = pi.order[oi];
    const int tile0 = total;
    for (int pass = 0; pass < 2; ++pass)
      for (int ei = 0; ei < nent; ++ei) {
        const Entry& en = entries[ei];
        if (en.branch != b || en.tiles == 0 || (h_sizes[base + en.problem].z > kmin) != (pass == 0)) continue;
        a.entry[ne] = FusedArgs::Entry{total, en.row0, en.rows, en.problem | (en.branch << 16)};
        total += en.tiles;
        ++ne;
      }
    if (total == tile0) continue;
    // shapes beyond the phase table share the last phase (their relative order is kept)
    if (np < kMaxPhases) {
      a.phase_tile0[np] = tile0;
      a.phase_wg0[np] = wg;
      if (flat_phase(pi.b[b])) a.phase_flat |= 1 << np;
      ++np;
    }
    const int p0 = a.phase_tile0[np - 1];
    wg = a.phase_wg0[np - 1] + (total - p0 + kNumXcd - 1) / kNumXcd * kNumXcd;
  }
  a.num_entries = ne;
  a.total_tiles = total;
  a.num_phases = np;
  a.phase_tile0[np] = total;
  a.phase_wg0[np] = wg;
  *grid = wg;
  return 0;
}

// One launch over problems [base, base + n) of the caller's arrays with kernel `k` (n <= kMaxProblems).
inline int launch_range(const FusedKernel& k, const void* const* As, const void* const* Bs, const void* const* sa, const void* const* sb, void* const* Cs,
                        int32_t* const* acc, const mxmoe_dim3* d_sizes, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int base, int n, hipStream_t stream) {
  FusedArgs a;
  std::memset(&a, 0, sizeof a);
  a.As = reinterpret_cast<const uint8_t* const*>(As);
  a.Bs = reinterpret_cast<const uint8_t* const*>(Bs);
  a.sa = reinterpret_cast<const _Float16* const*>(sa);
  a.sb = reinterpret_cast<const _Float16* const*>(sb);
  a.Cs = reinterpret_cast<_Float16* const*>(Cs);
  a.acc = acc;
  a.sizes = d_sizes;
  int grid = 0;
  if (const int rc = build_fused_tables(k, h_sizes, h_q, base, n, a, &grid)) return rc;
  if (a.total_tiles == 0) return 0;
  const hipError_t e = k.launch(a, grid, k.lds_bytes, stream);
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

// Side streams of the multi-stream policy, created on first use per device (default priority, non-blocking) and kept for the
// life of the process, with the events that fork them from and join them to the caller's stream.
constexpr int kSideStreams = 4;
struct SideStreams {
  hipStream_t stream[kSideStreams];
  hipEvent_t fork, join[kSideStreams];
  bool ready;
};
inline SideStreams* side_streams() {
  static SideStreams pool[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  SideStreams& p = pool[dev];
  if (!p.ready) {
    if (hipEventCreateWithFlags(&p.fork, hipEventDisableTiming) != hipSuccess) return nullptr;
    for (int i = 0; i < kSideStreams; ++i)
      if (hipStreamCreateWithFlags(&p.stream[i], hipStreamNonBlocking) != hipSuccess || hipEventCreateWithFlags(&p.join[i], hipEventDisableTiming) != hipSuccess) return nullptr;
    p.ready = true;
  }
  return &p;
}

// Host launcher.  Array arguments as in the reference FuncType (registry.cuh:28-39): every pointer array and
// d_sizes / d_q live in device memory, h_sizes / h_q are their host mirrors.  ld* and d_q are accepted and unused.
inline int group_gemm(int kernel_id, const void* const* As, const void* const* Bs, const void* const* sa, const void* const* sb, void* const* Cs,
                      int32_t* const* acc, const mxmoe_dim3* d_sizes, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int count, hipStream_t stream) {
  if (count <= 0) return 0;
  auto& reg = registry();
  if (kernel_id < 0) {
    kernel_id = auto_kernel(h_sizes, h_q, count);
    if (kernel_id < 0) {
      last_error() = "quant type not supported";  // same message as the reference launcher (compose_kernel.py:433)
      return 1;
    }
  }
  if (kernel_id >= (int)reg.size()) {
    last_error() = "kernel id out of range";
    return 2;
  }
  const FusedKernel& k = reg[kernel_id];
  for (int i = 0; i < count; ++i) {  // the tiles read the scales unconditionally: refuse a launch whose scale arrays are missing
    const Fmt f = classify(h_q[i]);
    const bool wa = f == Fmt::W8A8 || f == Fmt::W4A4 || f == Fmt::W4A4G128;
    const bool wo = is_weight_only(f);
    if (h_sizes[i].x != 0 && ((wa && (!sa || !sb)) || (wo && !sb))) {
      last_error() = "scale arrays are required for quantised formats";
      return 5;
    }
  }
  auto run = [&](int base, int n, hipStream_t s) { return launch_range(k, As, Bs, sa, sb, Cs, acc, d_sizes, h_sizes, h_q, base, n, s); };
  if (k.policy == Policy::Fused) {
    for (int base = 0; base < count; base += kMaxProblems)
      if (const int rc = run(base, std::min(kMaxProblems, count - base), stream)) return rc;
    return 0;
  }
  // runs of consecutive problems of equal format (kernel_sketch.py:192-246 compares the QParams of neighbours the same way)
  auto same = [&](int x, int y) { return h_q[x].a_bits == h_q[y].a_bits && h_q[x].w_bits == h_q[y].w_bits && h_q[x].gsize == h_q[y].gsize && h_q[x].sym == h_q[y].sym; };
  SideStreams* side = nullptr;
  if (k.policy == Policy::MultiStream) {
    side = side_streams();
    if (!side || hipEventRecord(side->fork, stream) != hipSuccess) {
      last_error() = "could not set up the side streams of the multi-stream policy";
      return 4;
    }
  }
  int nrun = 0, rc = 0;
  unsigned used = 0;
  for (int base = 0; base < count && rc == 0;) {
    int n = 1;
    while (base + n < count && n < kMaxProblems && same(base, base + n)) ++n;
    hipStream_t s = stream;
    if (side) {
      const int si = nrun % kSideStreams;
      s = side->stream[si];
      if (!(used >> si & 1) && hipStreamWaitEvent(s, side->fork, 0) != hipSuccess) rc = 4;
      used |= 1u << si;
    }
    if (rc == 0) rc = run(base, n, s);
    base += n;
    ++nrun;
  }
  if (side) {  // join whatever was forked, also after a failure, so that the caller's stream stays ordered after the side work
    for (int si = 0; si < kSideStreams; ++si)
      if (used >> si & 1)
        if (hipEventRecord(side->join[si], side->stream[si]) != hipSuccess || hipStreamWaitEvent(stream, side->join[si], 0) != hipSuccess) rc = rc ? rc : 4;
    if (rc == 4 && last_error().empty()) last_error() = "stream fork / join failed";
  }
  return rc;
}

}  // namespace mxmoe
