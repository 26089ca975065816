// Device-side planning of the two fused launches of a layer forward.
//
// The reference's operators read the tokens-per-expert counts back to the host (`.cpu()`, mxmoe/kernels/src/ref_bind.cu:451) and
// build every table there: the per-expert {tag, first row, offsets} table of the quantisers (ref_bind.cu:475-505), the five pointer
// arrays and sizes of the launch (ref_bind.cu:362-404) and, in the generated launcher, the tile prefix sums
// (mxmoe/kernels/kernel_sketch.py:89-104).  Here one small kernel derives all of them from the counts where they are, in device
// memory, so that the host enqueues the whole forward without waiting for the routing: no synchronisation, nothing that depends
// on the counts in any launch argument, and therefore a sequence that a HIP graph can hold.
#include <hip/hip_runtime.h>

#include "../../include/mxmoe_amd.h"
#include "include/mxmoe_launch.hpp"
#include "include/mxmoe_plan.hpp"
#include "include/mxmoe_perm.hpp"

namespace mxmoe {

// A block descriptor (not the QParams arrays of the launcher, whose padding bytes belong to the caller) may name an operand variant
// in q._pad[0]: 1 = the int4 codes of per-token activations as bf6 fragments (for the kernels whose w4a4 tiles run on the 6-bit float
// matrix path), 2 = per-token fp8 e4m3 codes instead of int8 ones (for the kernels whose w8a8 tiles run the fp8 instruction).
__host__ __device__ inline bool wants_bf6(const mxmoe_qparams& q) { return q._pad[0] == 1 && q.a_bits == 4 && q.w_bits == 4 && q.gsize == -1; }
__host__ __device__ inline bool wants_fp8(const mxmoe_qparams& q) { return q._pad[0] == 2 && q.a_bits == 8 && q.w_bits == 8 && q.gsize == -1; }

__host__ __device__ inline int act_tag_of(const mxmoe_qparams& q) {  // ref_bind.cu:461-473
  if (q.a_bits >= 16) return 0;
  if (wants_fp8(q)) return 5;
  if (q.a_bits == 8 && q.gsize == -1) return 1;
  if (wants_bf6(q)) return 4;
  if (q.a_bits == 4 && q.gsize == -1) return 2;
  if (q.a_bits == 4 && q.gsize == 128) return 3;
  return -1;
}

__host__ __device__ inline int fmt_of(const mxmoe_qparams& q) { return (int)classify(q); }

struct PlanParams {
  const int64_t* recv;
  const mxmoe_block_desc* desc;
  const uint8_t* inp;
  const uint8_t* scale;
  uint8_t* out;
  uint8_t* plan;
  int E, Et, shared_rows;
  PlanInfo info;
};

constexpr int kPlanThreads = 128;
constexpr int kMaxPlannedProblems = 4096;  // experts of a planned block (run as launches of kMaxProblems experts each)
static_assert(kMaxProblems <= kPlanThreads, "one thread per problem");

__device__ __forceinline__ long wave_excl_scan(long v, int lane, long* total) {
  long inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const long t = __shfl_up(inc, o);
    if (lane >= o) inc += t;
  }
  *total = __shfl(inc, 63);
  return inc - v;
}

// One workgroup of two waves per launch, thread e = expert e0 + e of the launch's chunk of experts [e0, e0 + kMaxProblems) (the shared
// expert, if any, is expert E with `shared_rows` rows).  Everything the host launcher computes (launch_range), with the same
// functions and in the same order, so the two produce identical tables; prefix sums over experts are wave scans (a later chunk
// first sums what the experts before it occupy), and an entry finds its place from per-branch counts instead of a sequential walk.
struct PlanPair {
  PlanParams p[2];
  int chunks;  // launches per block
};

// `recv`: the tokens-per-expert counts (device memory, or LDS when the planning workgroup counted them itself).
__device__ __forceinline__ void plan_block_body(const PlanParams& p, const int chunk, const int chunks, const int64_t* recv) {
  const int e0 = chunk * kMaxProblems;                       // first expert of this launch
  const int ecnt = min(kMaxProblems, p.Et - e0);             // experts of this launch
  __shared__ long s_tot[4][2];                       // per wave: rows, packed input, scales, output elements
  __shared__ long s_base[5][2];                      // the same four, and the routed rows, summed over the experts before this launch
  __shared__ int s_cnt[kMaxBranches][2], s_til[kMaxBranches][2];  // per run-order rank and wave: entries, tiles
  __shared__ int s_cnt_long[kMaxBranches][2], s_til_long[kMaxBranches][2];  // ... of which belong to long-K problems
  // the kernel's branch table, from the kernel arguments into LDS: the planning functions walk it entry by entry, and each step of
  // such a walk through the argument segment costs a trip to the scalar cache
  __shared__ PlanInfo info;
  static_assert(sizeof(PlanInfo) % 4 == 0, "copied word by word");
  for (int i = threadIdx.x; i < (int)(sizeof(PlanInfo) / 4); i += kPlanThreads) reinterpret_cast<int*>(&info)[i] = reinterpret_cast<const int*>(&p.info)[i];
  const int e = threadIdx.x, lane = e & 63, wave = e >> 6;
  const int ge = e0 + e;                             // this thread's expert
  __shared__ unsigned s_used[2];                     // per wave: branches in use
  if (e < kMaxBranches) {
    s_cnt[e][0] = s_cnt[e][1] = s_til[e][0] = s_til[e][1] = 0;
    s_cnt_long[e][0] = s_cnt_long[e][1] = s_til_long[e][0] = s_til_long[e][1] = 0;
  }
  if (e < 2) s_used[e] = 0;
  const bool mine = e < ecnt;
  const PlanLayout lay(p.Et);
  FusedArgs* fa = reinterpret_cast<FusedArgs*>(p.plan + chunk * kFusedArgsStride);
  int64_t* table = reinterpret_cast<int64_t*>(p.plan + lay.table);
  const void** ptrs = reinterpret_cast<const void**>(p.plan + lay.ptrs);
  int64_t* misc = reinterpret_cast<int64_t*>(p.plan + lay.misc);
  mxmoe_dim3* sizes = reinterpret_cast<mxmoe_dim3*>(p.plan + lay.sizes);

  // what one expert occupies: rows, packed activation elements, scales, output elements (all in fp16 elements but the rows)
  auto footprint = [&](int x, long (&f)[4], int* tag_out, mxmoe_block_desc* d_out) {
    const mxmoe_block_desc d = p.desc[x];
    const long rows = x < p.E ? (long)recv[x] : (long)p.shared_rows;
    const int tag = act_tag_of(d.q), K = (int)d.K;
    const long qld = tag == 0 ? K : (tag == 1 || tag == 5 ? K / 2 : K / 4);  // fp16 elements per packed activation row (ref_bind.cu:491)
    const long sld = tag == 0 ? 0 : (tag == 3 ? K / 128 : 1);                // scales per row (ref_bind.cu:492)
    f[0] = rows;
    // packed activations: rows of qld elements, or (tag 4) whole blocks of 32 rows of K / 64 fragments
    f[1] = tag == 4 ? ((rows + 31) >> 5) * (long)(K >> 6) * (kBf6Frag / 2) : qld * rows;
    f[2] = sld * rows;
    f[3] = (long)d.N * rows;
    if (tag_out) *tag_out = tag;
    if (d_out) *d_out = d;
  };
  // experts before this launch (none for the first: most blocks are one launch)
  if (e0 > 0) {
    long base[5] = {0, 0, 0, 0, 0};
    for (int x = e; x < e0; x += kPlanThreads) {
      long f[4];
      footprint(x, f, nullptr, nullptr);
#pragma unroll
      for (int i = 0; i < 4; ++i) base[i] += f[i];
      if (x < p.E) base[4] += f[0];
    }
#pragma unroll
    for (int i = 0; i < 5; ++i) {
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) base[i] += __shfl_xor(base[i], o);
      if (lane == 0) s_base[i][wave] = base[i];
    }
  } else if (lane == 0) {
#pragma unroll
    for (int i = 0; i < 5; ++i) s_base[i][wave] = 0;
  }

  long rows = 0, sld = 0;
  long foot[4] = {0, 0, 0, 0};
  int tag = 0, fmt = 0, N = 0, K = 0;
  mxmoe_block_desc d{};
  if (mine) {
    footprint(ge, foot, &tag, &d);
    rows = foot[0];
    fmt = fmt_of(d.q);
    N = (int)d.N;
    K = (int)d.K;
    sld = tag == 0 ? 0 : (tag == 3 ? K / 128 : 1);
  }
  // exclusive sums over the experts of this launch before this one
  long tot[4], routed_tot;
  long first_row = wave_excl_scan(foot[0], lane, &tot[0]);
  long inp_off = wave_excl_scan(foot[1], lane, &tot[1]);
  long sc_off = wave_excl_scan(foot[2], lane, &tot[2]);
  long out_off = wave_excl_scan(foot[3], lane, &tot[3]);
  wave_excl_scan(mine && ge < p.E ? rows : 0, lane, &routed_tot);
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) s_tot[i][wave] = tot[i];
  }
  // smallest K of the launch: problems above it run first inside their branch (see launch_range)
  __shared__ int s_kmin[2];
  __shared__ long s_routed[2];
  {
    int km = mine ? K : 0x7fffffff;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) km = min(km, __shfl_xor(km, o));
    if (lane == 0) {
      s_kmin[wave] = km;
      s_routed[wave] = routed_tot;
    }
  }
  __syncthreads();
  const bool long_k = mine && K > min(s_kmin[0], s_kmin[1]);
  // segments of this problem and, per branch in run order, this wave's entries and tiles
  Segment sg[2];
  const int ns = mine ? plan_segments(info, fmt, (int)rows, N, sg) : 0;
  int seg_tiles[2], seg_rank[2], seg_pos[2], seg_first[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    seg_tiles[j] = j < ns ? segment_tiles(info, sg[j], N) : 0;
    seg_rank[j] = -1;
    seg_pos[j] = seg_first[j] = 0;
  }
  // branches that this wave's problems use at all (most branches of a kernel are not used by a given launch: their counters stay zero)
  {
    unsigned mask = 0;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      if (j < ns && seg_tiles[j] > 0) mask |= 1u << sg[j].branch;
    if (mask) atomicOr(&s_used[wave], mask);
  }
  __builtin_amdgcn_wave_barrier();
  const unsigned used = (unsigned)__builtin_amdgcn_readfirstlane((int)*(volatile unsigned*)&s_used[wave]);
  for (int r = 0; r < info.nb; ++r) {
    const int b = info.order[r];
    if (!(used >> b & 1)) continue;
    int mine_tiles = 0, which = -1;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      if (j < ns && sg[j].branch == b && seg_tiles[j] > 0) {
        mine_tiles = seg_tiles[j];
        which = j;
      }
    // entries of this branch in this wave, long-K problems first: position = matching lanes that run earlier, first tile = their tiles
    const uint64_t has = __ballot(which >= 0);
    int tc = 0, tt = 0, tc_long = 0, tt_long = 0;
    if (has != 0) {  // (wave-uniform: most branches of a kernel are not used by a given launch)
      const uint64_t has_long = __ballot(which >= 0 && long_k);
      tc = __popcll(has);
      tc_long = __popcll(has_long);
      int inc_long = long_k ? mine_tiles : 0, inc_rest = long_k ? 0 : mine_tiles;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t0 = __shfl_up(inc_long, o), t1 = __shfl_up(inc_rest, o);
        if (lane >= o) {
          inc_long += t0;
          inc_rest += t1;
        }
      }
      tt_long = __shfl(inc_long, 63);
      tt = tt_long + __shfl(inc_rest, 63);
      const uint64_t before = (1ull << lane) - 1;
#pragma unroll
      for (int j = 0; j < 2; ++j)
        if (which == j) {
          seg_rank[j] = r;
          // position / first tile inside this wave's entries of its own class; the other wave's and the other class's are added below
          seg_pos[j] = long_k ? __popcll(has_long & before) : __popcll(has & ~has_long & before);
          seg_first[j] = long_k ? inc_long - mine_tiles : inc_rest - mine_tiles;
        }
    }
    if (lane == 0) {
      s_cnt[r][wave] = tc;
      s_til[r][wave] = tt;
      s_cnt_long[r][wave] = tc_long;
      s_til_long[r][wave] = tt_long;
    }
  }
  __syncthreads();
  if (wave == 1) {
    first_row += s_tot[0][0];
    inp_off += s_tot[1][0];
    sc_off += s_tot[2][0];
    out_off += s_tot[3][0];
  }
  first_row += s_base[0][0] + s_base[0][1];
  inp_off += s_base[1][0] + s_base[1][1];
  sc_off += s_base[2][0] + s_base[2][1];
  out_off += s_base[3][0] + s_base[3][1];
  if (mine) {
    table[ge] = tag;
    table[p.Et + ge] = first_row;
    table[2 * p.Et + ge] = inp_off;
    table[3 * p.Et + ge] = sc_off;
    ptrs[ge] = p.inp + 2 * inp_off;
    ptrs[p.Et + ge] = d.B;
    ptrs[2 * p.Et + ge] = sld > 0 ? p.scale + 2 * sc_off : nullptr;
    ptrs[3 * p.Et + ge] = d.scale_b;
    ptrs[4 * p.Et + ge] = p.out + 2 * out_off;
    sizes[ge] = mxmoe_dim3{(uint32_t)rows, (uint32_t)N, (uint32_t)K};
    if (ge == p.E) misc[1] = (int64_t)(p.out + 2 * out_off);
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    if (seg_rank[j] >= 0) {
      int pos = seg_pos[j], first = seg_first[j];
      for (int r = 0; r < seg_rank[j]; ++r) {
        pos += s_cnt[r][0] + s_cnt[r][1];
        first += s_til[r][0] + s_til[r][1];
      }
      // inside the branch: [long-K entries of wave 0][of wave 1][other entries of wave 0][of wave 1]
      const int r = seg_rank[j];
      if (long_k) {
        if (wave == 1) {
          pos += s_cnt_long[r][0];
          first += s_til_long[r][0];
        }
      } else {
        pos += s_cnt_long[r][0] + s_cnt_long[r][1];
        first += s_til_long[r][0] + s_til_long[r][1];
        if (wave == 1) {
          pos += s_cnt[r][0] - s_cnt_long[r][0];
          first += s_til[r][0] - s_til_long[r][0];
        }
      }
      fa->entry[pos] = FusedArgs::Entry{first, sg[j].row0, sg[j].rows, e | (sg[j].branch << 16)};  // problem index relative to the launch's first
    }
  }
  if (e == 0) {
    // rows routed = sum over the routed experts of every launch: the last launch knows them all
    if (chunk == chunks - 1) misc[0] = s_base[4][0] + s_base[4][1] + s_routed[0] + s_routed[1];
    if (chunk == 0 && p.Et == p.E) misc[1] = 0;
    int total = 0, wg = 0, np = 0, ne = 0, flat = 0;
    int last_tile0 = 0, last_wg0 = 0;  // of the phase being filled (kept here: reading them back from the table would wait for the store)
    for (int r = 0; r < info.nb; ++r) {
      const int tile0 = total;
      total += s_til[r][0] + s_til[r][1];
      ne += s_cnt[r][0] + s_cnt[r][1];
      if (total == tile0) continue;
      if (np < kMaxPhases) {  // shapes beyond the phase table share the last phase
        fa->phase_tile0[np] = last_tile0 = tile0;
        fa->phase_wg0[np] = last_wg0 = wg;
        if (flat_phase(info.b[info.order[r]])) flat |= 1 << np;
        ++np;
      }
      wg = last_wg0 + (total - last_tile0 + kNumXcd - 1) / kNumXcd * kNumXcd;
    }
    fa->phase_tile0[np] = total;
    fa->phase_wg0[np] = wg;
    if (np == 0) fa->phase_tile0[1] = fa->phase_wg0[1] = 0;  // a plan without tiles still holds one (empty) phase range
    fa->num_phases = np;
    fa->phase_flat = flat;
    fa->num_entries = ne;
    fa->total_tiles = total;
    fa->problem_offset = e0;
    fa->As = reinterpret_cast<const uint8_t* const*>(ptrs);
    fa->Bs = reinterpret_cast<const uint8_t* const*>(ptrs + p.Et);
    fa->sa = reinterpret_cast<const _Float16* const*>(ptrs + 2 * p.Et);
    fa->sb = reinterpret_cast<const _Float16* const*>(ptrs + 3 * p.Et);
    fa->Cs = reinterpret_cast<_Float16* const*>(const_cast<void**>(ptrs + 4 * p.Et));
    fa->acc = nullptr;
    fa->sizes = sizes;
  }
}

__global__ void __launch_bounds__(kPlanThreads) plan_block_kernel(const PlanPair pair) {
  // one workgroup per launch of each block of the layer (gate_up, down): all only read the counts
  plan_block_body(pair.p[blockIdx.x / pair.chunks], blockIdx.x % pair.chunks, pair.chunks, pair.p[0].recv);
}

// Permutation and planning of a decode-sized batch (at most kPermChunk (token, slot) entries) in ONE launch: workgroup 0 builds the
// permutation, the others plan the layer's launches from counts they take from the routed ids themselves (a few hundred ids: cheaper
// than waiting for workgroup 0 in a second launch).  A forward of some tens of microseconds feels every launch it saves.
struct PermSmallArgs {
  const int32_t* ids;
  int total, E, topk, nbits;
  int64_t* recv;
  int32_t* dst;
  int64_t* perm;
  int64_t* slot;
  int32_t* row_of_slot;
};
__global__ void __launch_bounds__(kPlanThreads) perm_plan_small_kernel(const PermSmallArgs a, const PlanPair pair) {
  extern __shared__ __align__(8) uint8_t pp_lds[];  // E int32 counters (workgroup 0) or E int64 counts (planning workgroups)
  if (blockIdx.x == 0) {
    perm_small_body(a.ids, a.total, a.E, a.topk, a.nbits, a.recv, a.dst, a.perm, a.slot, a.row_of_slot, reinterpret_cast<int32_t*>(pp_lds), threadIdx.x < 64);
    return;
  }
  int64_t* counts = reinterpret_cast<int64_t*>(pp_lds);
  unsigned long long* cnt = reinterpret_cast<unsigned long long*>(pp_lds);
  for (int e = threadIdx.x; e < a.E; e += kPlanThreads) counts[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < a.total; i += kPlanThreads) {
    const int e = a.ids[i];
    if (e >= 0 && e < a.E) atomicAdd(&cnt[e], 1ull);
  }
  __syncthreads();
  const int b = blockIdx.x - 1;
  plan_block_body(pair.p[b / pair.chunks], b % pair.chunks, pair.chunks, counts);
}

// The same for larger batches, after perm_hist_kernel has counted the experts per chunk of kPermChunk entries: the first `blocks`
// workgroups scatter their chunk (each summing the counts it needs: perm_scatter_body with raw counts), the others plan the
// layer's launches from the column sums of the same histogram.  Neither waits for the other, so the forward's serial head is two
// launches (count, scatter + plan) instead of four (count, scan, scatter, plan).
struct PermScatterArgs {
  const int32_t* ids;
  int total, E, topk, nbits, blocks;
  const int32_t* hist;
  int64_t* recv;
  int32_t* dst;
  int64_t* perm;
  int64_t* slot;
  int32_t* row_of_slot;
};
__global__ void __launch_bounds__(kPlanThreads) perm_scatter_plan_kernel(const PermScatterArgs a, const PlanPair pair) {
  extern __shared__ __align__(8) uint8_t pp_lds[];  // E int32 ranks (scatter workgroups) or E int64 counts (planning workgroups)
  if ((int)blockIdx.x < a.blocks) {
    perm_scatter_body(a.ids, a.total, a.E, a.topk, a.nbits, a.hist, a.blocks, (int)blockIdx.x, true, a.recv, a.dst, a.perm, a.slot, a.row_of_slot,
                      reinterpret_cast<int32_t*>(pp_lds), threadIdx.x < 64);
    return;
  }
  int64_t* counts = reinterpret_cast<int64_t*>(pp_lds);
  for (int e = threadIdx.x; e < a.E; e += kPlanThreads) {
    int v, before;
    perm_hist_row_sums(a.hist + (long)e * perm_hist_stride(a.blocks), a.blocks, 0, &v, &before);
    counts[e] = v;
  }
  __syncthreads();
  const int b = blockIdx.x - a.blocks;
  plan_block_body(pair.p[b / pair.chunks], b % pair.chunks, pair.chunks, counts);
}

// Kernel for the formats of `h_desc`, checked once on the host: every problem's format has a branch and its shape fits it.
static int resolve_kernel(int kernel_id, const mxmoe_block_desc* h_desc, int et) {
  auto& reg = registry();
  auto covers = [&](const FusedKernel& k) {
    for (int i = 0; i < et; ++i) {
      Segment sg[2];
      const int f = fmt_of(h_desc[i].q);
      if (f == (int)Fmt::UNSUPPORTED || plan_segments(plan_of(k), f, 1, 256, sg) < 0) return false;
      // a kernel's w4a4 tiles take packed int4 rows or bf6 fragments, never both: the descriptor says which the block will get
      if (f == (int)Fmt::W4A4 && kernel_takes_bf6(k) != wants_bf6(h_desc[i].q)) return false;
      if (f == (int)Fmt::W8A8 && (kernel_variant(k, Fmt::W8A8) == kVariantFp8) != wants_fp8(h_desc[i].q)) return false;
      // 16-bit float blocks of a layer are fp16 (the activation step between the launches computes in fp16): no bfloat16 kernel here
      if (f == (int)Fmt::FP16 && kernel_variant(k, Fmt::FP16) != 0) return false;
    }
    return true;
  };
  if (kernel_id < 0) {
    for (int i = 0; i < (int)reg.size() && kernel_id < 0; ++i)
      if (reg[i].policy == Policy::Fused && reg[i].max_rows_hint == 0 && covers(reg[i])) kernel_id = i;  // (row counts are not known here: no few-row kernel)
    if (kernel_id < 0) {
      last_error() = "quant type not supported";
      return -1;
    }
  }
  if (kernel_id >= (int)reg.size()) {
    last_error() = "kernel id out of range";
    return -2;
  }
  const FusedKernel& k = reg[kernel_id];
  if (!covers(k)) {
    last_error() = "quant type not supported";
    return -1;
  }
  for (int i = 0; i < et; ++i) {
    const mxmoe_dim3 sz{1, h_desc[i].N, h_desc[i].K};
    for (const BranchInfo& bi : k.branches)
      if ((int)bi.fmt == fmt_of(h_desc[i].q) && !shape_ok(bi, sz)) {
        char buf[200];
        snprintf(buf, sizeof buf, "problem %d: shape [N %u, K %u] not supported by tile %s (K %% %d, N %% 8)", i, sz.y, sz.z, fmt_name(bi.fmt, true), bi.k_multiple);
        last_error() = buf;
        return -3;
      }
    const int tag = act_tag_of(h_desc[i].q);
    if (tag < 0 || (tag == 3 && h_desc[i].K % 128)) {
      last_error() = tag < 0 ? "quant type not supported" : "group-128 activations need a row length that is a multiple of 128";
      return tag < 0 ? -1 : -3;
    }
  }
  return kernel_id;
}

}  // namespace mxmoe

using namespace mxmoe;

extern "C" {

size_t mxmoe_plan_bytes(int num_problems) { return PlanLayout(num_problems).total; }

size_t mxmoe_plan_offset(int which, int num_problems) {
  const PlanLayout lay(num_problems);
  switch (which) {
    case 0: return 0;
    case 1: return lay.table;
    case 2: return lay.ptrs;
    case 3: return lay.misc;
    case 4: return lay.sizes;
    default: return lay.total;
  }
}

int mxmoe_plan_select_kernel(int kernel_id, const mxmoe_block_desc* h_desc, int num_problems) {
  if (!h_desc || num_problems <= 0 || num_problems > kMaxPlannedProblems) {
    last_error() = "a planned block holds 1 to 4096 problems";
    return -3;
  }
  return resolve_kernel(kernel_id, h_desc, num_problems);
}

int mxmoe_plan_grid_bound(int kernel_id, const mxmoe_block_desc* h_desc, int num_experts, int routed_rows_max, int shared_rows) {
  const int et = num_experts + (shared_rows > 0 ? 1 : 0);
  const int kid = mxmoe_plan_select_kernel(kernel_id, h_desc, et);
  if (kid < 0) return kid;
  const PlanInfo& pi = plan_of(registry()[kid]);
  // For every routed expert tiles(M) <= first + slope * (M - 1) for all M >= 1, with first = tiles(1) and slope the steepest rise
  // found by walking M over 64 rows of the format's largest tile (the planner's decisions repeat with that tile's period).  With at
  // most n = min(experts, rows) experts non-empty, the launch has at most (sum of the n largest `first`) + max slope * (rows - n) tiles.
  auto tiles_of = [&](int f, int m, int n) {
    Segment sg[2];
    const int ns = plan_segments(pi, f, m, n, sg);
    int t = 0;
    for (int j = 0; j < ns; ++j) t += segment_tiles(pi, sg[j], n);
    return t;
  };
  // And tiles(M) <= extra + per_row * M, with per_row the columns per row of the shape that very long problems run on and extra the
  // largest excess over it: the smaller of the two sums holds.
  long shared_tiles = 0;
  double slope = 0, per_row = 0;
  long extras = 0;
  std::vector<int> firsts;
  struct Seen { int f, n, first, extra; double slope, per_row; };
  std::vector<Seen> seen;
  for (int e = 0; e < et; ++e) {
    const int f = fmt_of(h_desc[e].q), n = (int)h_desc[e].N;
    if (e >= num_experts) {  // the shared expert's row count is known
      shared_tiles += tiles_of(f, shared_rows, n);
      continue;
    }
    const Seen* hit = nullptr;
    for (const Seen& sn : seen)
      if (sn.f == f && sn.n == n) hit = &sn;
    if (!hit) {
      Segment sg[2];
      plan_segments(pi, f, 1 << 20, n, sg);
      const int bm = pi.b[sg[0].branch].BM, cols = (n + pi.b[sg[0].branch].BN - 1) / pi.b[sg[0].branch].BN;
      Seen sn{f, n, tiles_of(f, 1, n), 0, 0.0, (double)cols / bm};
      const int limit = std::min(std::max(routed_rows_max, 2), 64 * bm);
      for (int m = 1; m <= limit; ++m) {
        const int t = tiles_of(f, m, n);
        if (m > 1) sn.slope = std::max(sn.slope, (double)(t - sn.first) / (m - 1));
        sn.extra = std::max(sn.extra, t - (m / bm) * cols);
      }
      seen.push_back(sn);
      hit = &seen.back();
    }
    firsts.push_back(hit->first);
    slope = std::max(slope, hit->slope);
    per_row = std::max(per_row, hit->per_row);
    extras += hit->extra;
  }
  std::sort(firsts.begin(), firsts.end(), [](int x, int y) { return x > y; });
  const int nonempty = std::min((int)firsts.size(), routed_rows_max);
  long by_first = (long)(slope * (routed_rows_max - nonempty)) + 1;
  for (int i = 0; i < nonempty; ++i) by_first += firsts[i];
  const long by_rows = extras + (long)(per_row * routed_rows_max) + 1;
  long bound = shared_tiles + std::min(by_first, by_rows);
  bound += (long)kNumXcd * (kMaxPhases + 1);  // every phase is padded to a multiple of the XCD count
  bound = (bound + kNumXcd - 1) / kNumXcd * kNumXcd;
  if (bound > (1l << 30)) {
    last_error() = "planned grid too large";
    return -3;
  }
  return (int)bound;
}

static int fill_plan_params(PlanParams& p, int kernel_id, const int64_t* d_recv, int num_experts, int shared_rows, const mxmoe_block_desc* d_desc,
                            const mxmoe_block_desc* h_desc, const void* inp_store, const void* scale_store, void* out_store, void* d_plan) {
  const int et = num_experts + (shared_rows > 0 ? 1 : 0);
  if (!d_recv || !d_desc || !h_desc || !inp_store || !out_store || !d_plan) {
    last_error() = "null pointer";
    return 5;
  }
  const int kid = mxmoe_plan_select_kernel(kernel_id, h_desc, et);
  if (kid < 0) return kid == -1 ? 1 : (kid == -2 ? 2 : 3);
  p.recv = d_recv;
  p.desc = d_desc;
  p.inp = reinterpret_cast<const uint8_t*>(inp_store);
  p.scale = reinterpret_cast<const uint8_t*>(scale_store);
  p.out = reinterpret_cast<uint8_t*>(out_store);
  p.plan = reinterpret_cast<uint8_t*>(d_plan);
  p.E = num_experts;
  p.Et = et;
  p.shared_rows = shared_rows;
  p.info = plan_of(registry()[kid]);
  return 0;
}

static int launch_plan(PlanPair& pair, int blocks, void* stream) {
  pair.chunks = PlanLayout(pair.p[0].Et).chunks;
  hipLaunchKernelGGL(plan_block_kernel, dim3(blocks * pair.chunks), dim3(kPlanThreads), 0, (hipStream_t)stream, pair);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

int mxmoe_plan_block(int kernel_id, const int64_t* d_recv, int num_experts, int shared_rows, const mxmoe_block_desc* d_desc, const mxmoe_block_desc* h_desc,
                     const void* inp_store, const void* scale_store, void* out_store, void* d_plan, void* stream) {
  PlanPair pair;
  const int rc = fill_plan_params(pair.p[0], kernel_id, d_recv, num_experts, shared_rows, d_desc, h_desc, inp_store, scale_store, out_store, d_plan);
  if (rc) return rc;
  pair.p[1] = pair.p[0];
  return launch_plan(pair, 1, stream);
}

int mxmoe_plan_layer(const mxmoe_plan_call* gate_up, const mxmoe_plan_call* down, const int64_t* d_recv, int num_experts, int shared_rows, void* stream) {
  if (!gate_up || !down) {
    last_error() = "null pointer";
    return 5;
  }
  PlanPair pair;
  const mxmoe_plan_call* c[2] = {gate_up, down};
  for (int i = 0; i < 2; ++i) {
    const int rc = fill_plan_params(pair.p[i], c[i]->kernel_id, d_recv, num_experts, shared_rows, c[i]->d_desc, c[i]->h_desc, c[i]->inp_store, c[i]->scale_store,
                                    c[i]->out_store, c[i]->d_plan);
    if (rc) return rc;
  }
  return launch_plan(pair, 2, stream);
}

int mxmoe_permute_plan_layer(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices, int64_t* src_slot,
                             int64_t* recv_tokens_per_exp, int32_t* row_of_slot, const mxmoe_plan_call* gate_up, const mxmoe_plan_call* down, int shared_rows, void* stream) {
  if (num_tokens <= 0 || topk <= 0 || num_experts <= 0 || num_experts > kMaxPlannedProblems || (long)num_tokens * topk > kPermChunk) {
    last_error() = "the one-launch permutation + planning takes at most 256 (token, slot) entries: use mxmoe_build_permutation_inv and mxmoe_plan_layer";
    return 3;
  }
  if (!topk_ids || !dst_exp_sorted || !perm_indices || !src_slot || !recv_tokens_per_exp || !gate_up || !down) {
    last_error() = "null pointer";
    return 5;
  }
  PlanPair pair;
  const mxmoe_plan_call* c[2] = {gate_up, down};
  for (int i = 0; i < 2; ++i) {
    const int rc = fill_plan_params(pair.p[i], c[i]->kernel_id, recv_tokens_per_exp, num_experts, shared_rows, c[i]->d_desc, c[i]->h_desc, c[i]->inp_store, c[i]->scale_store,
                                    c[i]->out_store, c[i]->d_plan);
    if (rc) return rc;
  }
  pair.chunks = PlanLayout(pair.p[0].Et).chunks;
  PermSmallArgs a;
  a.ids = topk_ids;
  a.total = num_tokens * topk;
  a.E = num_experts;
  a.topk = topk;
  a.nbits = 1;
  while ((1 << a.nbits) <= num_experts) ++a.nbits;  // ids 0..E (E = parked lanes)
  a.recv = recv_tokens_per_exp;
  a.dst = dst_exp_sorted;
  a.perm = perm_indices;
  a.slot = src_slot;
  a.row_of_slot = row_of_slot;
  hipLaunchKernelGGL(perm_plan_small_kernel, dim3(1 + 2 * pair.chunks), dim3(kPlanThreads), (size_t)num_experts * 8, (hipStream_t)stream, a, pair);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

int mxmoe_permute_plan_layer_ws(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices, int64_t* src_slot,
                                int64_t* recv_tokens_per_exp, int32_t* row_of_slot, const mxmoe_plan_call* gate_up, const mxmoe_plan_call* down, int shared_rows,
                                void* workspace, void* stream) {
  if (num_tokens > 0 && topk > 0 && (long)num_tokens * topk <= kPermChunk)
    return mxmoe_permute_plan_layer(topk_ids, num_tokens, topk, num_experts, dst_exp_sorted, perm_indices, src_slot, recv_tokens_per_exp, row_of_slot, gate_up, down,
                                    shared_rows, stream);
  const long total = (long)num_tokens * topk;
  const long blocks = (total + kPermChunk - 1) / kPermChunk;
  if (num_tokens <= 0 || topk <= 0 || num_experts <= 0 || num_experts > kMaxPlannedProblems || blocks * num_experts > kPermFusedScanMax) {
    last_error() = "the two-launch permutation + planning takes batches whose (chunks of 256 entries) x experts is at most 16384: use mxmoe_build_permutation_inv and mxmoe_plan_layer";
    return 3;
  }
  if (!topk_ids || !dst_exp_sorted || !perm_indices || !src_slot || !recv_tokens_per_exp || !gate_up || !down || !workspace) {
    last_error() = "null pointer";
    return 5;
  }
  if (reinterpret_cast<uintptr_t>(workspace) & 15) {
    last_error() = "the workspace of the two-launch permutation + planning must be 16-byte aligned";
    return 3;
  }
  PlanPair pair;
  const mxmoe_plan_call* c[2] = {gate_up, down};
  for (int i = 0; i < 2; ++i) {
    const int rc = fill_plan_params(pair.p[i], c[i]->kernel_id, recv_tokens_per_exp, num_experts, shared_rows, c[i]->d_desc, c[i]->h_desc, c[i]->inp_store, c[i]->scale_store,
                                    c[i]->out_store, c[i]->d_plan);
    if (rc) return rc;
  }
  pair.chunks = PlanLayout(pair.p[0].Et).chunks;
  PermScatterArgs a;
  a.ids = topk_ids;
  a.total = (int)total;
  a.E = num_experts;
  a.topk = topk;
  a.nbits = 1;
  while ((1 << a.nbits) <= num_experts) ++a.nbits;  // ids 0..E (E = parked lanes)
  a.blocks = (int)blocks;
  a.hist = reinterpret_cast<const int32_t*>(workspace);
  a.recv = recv_tokens_per_exp;
  a.dst = dst_exp_sorted;
  a.perm = perm_indices;
  a.slot = src_slot;
  a.row_of_slot = row_of_slot;
  launch_perm_hist(topk_ids, a.total, num_experts, reinterpret_cast<int32_t*>(workspace), true, (hipStream_t)stream);
  hipLaunchKernelGGL(perm_scatter_plan_kernel, dim3(a.blocks + 2 * pair.chunks), dim3(kPlanThreads), (size_t)num_experts * 8, (hipStream_t)stream, a, pair);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
    return 4;
  }
  return 0;
}

int mxmoe_group_gemm_planned(int kernel_id, const void* d_plan, int num_problems, int grid, void* stream) {
  auto& reg = registry();
  if (kernel_id < 0 || kernel_id >= (int)reg.size()) {
    last_error() = "kernel id out of range";
    return 2;
  }
  if (!d_plan || grid <= 0 || num_problems <= 0 || num_problems > kMaxPlannedProblems) {
    last_error() = "null plan, empty grid or bad problem count";
    return 5;
  }
  const FusedKernel& k = reg[kernel_id];
  // one launch per chunk of kMaxProblems experts, each reading its own tables (workgroups past a launch's tiles leave at once)
  const int chunks = PlanLayout(num_problems).chunks;
  for (int c = 0; c < chunks; ++c) {
    const hipError_t e = k.launch_planned(reinterpret_cast<const FusedArgs*>(reinterpret_cast<const uint8_t*>(d_plan) + c * kFusedArgsStride), grid, k.lds_bytes, (hipStream_t)stream);
    if (e != hipSuccess) {
      last_error() = std::string("kernel launch failed: ") + hipGetErrorString(e);
      return 4;
    }
  }
  return 0;
}

}  // extern "C"
