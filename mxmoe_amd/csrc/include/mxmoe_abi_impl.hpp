// extern "C" entry points over the per-library kernel registry.  Included by exactly one translation unit of each shared
// library (the default library and every generated one), so each library answers with its own set of fused kernels.
#pragma once
#include "../../../include/mxmoe_amd.h"
#include "mxmoe_launch.hpp"

using namespace mxmoe;

extern "C" {

const char* mxmoe_last_error(void) { return last_error().c_str(); }

int mxmoe_num_kernels(void) { return (int)registry().size(); }

const char* mxmoe_kernel_name(int kernel_id) {
  if (kernel_id < 0 || kernel_id >= (int)registry().size()) return "";
  return registry()[kernel_id].name.c_str();
}

int mxmoe_find_kernel(const char* name) {
  const std::string n(name ? name : "");
  for (int i = 0; i < (int)registry().size(); ++i) {
    const std::string& k = registry()[i].name;
    if (k == n || (k.size() >= n.size() && !n.empty() && k.compare(k.size() - n.size(), n.size(), n) == 0)) return i;
  }
  return -1;
}

int mxmoe_kernel_num_branches(int kernel_id) {
  if (kernel_id < 0 || kernel_id >= (int)registry().size()) return -1;
  return (int)registry()[kernel_id].branches.size();
}

int mxmoe_kernel_branch(int kernel_id, int branch, int32_t out[8]) {
  if (kernel_id < 0 || kernel_id >= (int)registry().size()) { last_error() = "kernel id out of range"; return 2; }
  const auto& k = registry()[kernel_id];
  if (branch < 0 || branch >= (int)k.branches.size()) { last_error() = "branch out of range"; return 2; }
  const BranchInfo& b = k.branches[branch];
  out[0] = (int)b.fmt + 256 * b.variant; out[1] = b.BM; out[2] = b.BN; out[3] = b.BK; out[4] = b.WGM; out[5] = b.WGN; out[6] = b.lds_bytes; out[7] = b.k_multiple;
  return 0;
}

int mxmoe_group_gemm(int kernel_id, const void* const* As, const void* const* Bs, const void* const* scale_a, const void* const* scale_b,
                     void* const* Cs, void* const* Ds, const int64_t* lda, const int64_t* ldb, const int64_t* ldc, const int64_t* ldd,
                     const mxmoe_dim3* d_sizes, const mxmoe_dim3* h_sizes, const mxmoe_qparams* d_q, const mxmoe_qparams* h_q, int problem_count,
                     int32_t* const* acc_dump, void* stream) {
  // lda..ldd and d_q are device arrays the kernels never read (as in the reference, whose callers pass nullptr, ref_bind.cu:413):
  // leading dimensions are K, K, N
  (void)lda; (void)ldb; (void)ldc; (void)ldd; (void)d_q;
  return checked_group_gemm(kernel_id, As, Bs, scale_a, scale_b, Cs, Ds, acc_dump, d_sizes, h_sizes, h_q, problem_count, (hipStream_t)stream);
}

mxmoe_func_t mxmoe_kernel_func(int kernel_id) {
  if (kernel_id < 0 || kernel_id >= (int)registry().size()) { last_error() = "kernel id out of range"; return nullptr; }
  return registry()[kernel_id].func;
}

mxmoe_func_t mxmoe_get_kernel(const char* name) {
  const int id = mxmoe_find_kernel(name);
  if (id < 0) { last_error() = std::string("no kernel named ") + (name ? name : "(null)"); return nullptr; }
  return registry()[id].func;
}

int mxmoe_kernel_policy(int kernel_id) {
  if (kernel_id < 0 || kernel_id >= (int)registry().size()) return -1;
  return (int)registry()[kernel_id].policy;
}

void mxmoe_set_stream(void* stream) { func_stream() = (hipStream_t)stream; }
void* mxmoe_get_stream(void) { return (void*)func_stream(); }
int mxmoe_last_status(void) { return func_status(); }

int mxmoe_group_gemm_plan(int kernel_id, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int problem_count, int32_t* branch_out, int32_t* tiles_out) {
  auto& reg = registry();
  if (problem_count < 0 || (problem_count > 0 && (!h_sizes || !h_q))) {
    last_error() = "null argument";
    return 5;
  }
  if (kernel_id < 0) {
    kernel_id = auto_kernel(h_sizes, h_q, problem_count);
    if (kernel_id < 0) { last_error() = "quant type not supported"; return 1; }
  }
  if (kernel_id >= (int)reg.size()) { last_error() = "kernel id out of range"; return 2; }
  const FusedKernel& k = reg[kernel_id];
  int total = 0;
  for (int i = 0; i < problem_count; ++i) {
    const Fmt f = classify(h_q[i]);
    Segment sg[2];
    const int ns = f == Fmt::UNSUPPORTED ? -1 : plan_segments(plan_of(k), (int)f, (int)h_sizes[i].x, (int)h_sizes[i].y, sg);
    if (ns < 0) { last_error() = "quant type not supported"; return 1; }
    if (branch_out) branch_out[i] = ns ? sg[0].branch : pick_branch(plan_of(k), (int)f, 1, (int)h_sizes[i].y);
    for (int j = 0; j < ns; ++j) {
      const BranchInfo& bi = k.branches[sg[j].branch];
      if (!shape_ok(bi, h_sizes[i])) {  // what the launch itself would refuse
        char buf[200];
        snprintf(buf, sizeof buf, "problem %d: shape [%u,%u,%u] not supported by tile %s (K %% %d, N %% 8)", i, h_sizes[i].x, h_sizes[i].y, h_sizes[i].z, fmt_name(bi.fmt, true), bi.k_multiple);
        last_error() = buf;
        return 3;
      }
      total += ((sg[j].rows + bi.BM - 1) / bi.BM) * (int)((h_sizes[i].y + bi.BN - 1) / bi.BN);
    }
  }
  if (tiles_out) *tiles_out = total;
  return kernel_id + 1000;  // plan succeeded: 1000 + the kernel that would run
}

int mxmoe_group_gemm_plan_tables(int kernel_id, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int problem_count, int32_t* out, int out_ints) {
  auto& reg = registry();
  if (problem_count <= 0 || problem_count > kMaxProblems || !h_sizes || !h_q || !out || kernel_id < 0 || kernel_id >= (int)reg.size()) {
    last_error() = "bad argument";
    return 5;
  }
  FusedArgs a;
  std::memset(&a, 0, sizeof a);
  int grid = 0;
  if (const int rc = build_fused_tables(reg[kernel_id], h_sizes, h_q, 0, problem_count, a, &grid)) return rc;
  const int need = 4 + 2 * (kMaxPhases + 1) + 4 * a.num_entries;
  if (out_ints < need) {
    last_error() = "output too small";
    return 3;
  }
  int o = 0;
  out[o++] = a.num_entries; out[o++] = a.total_tiles; out[o++] = a.num_phases; out[o++] = grid;
  for (int i = 0; i <= kMaxPhases; ++i) out[o++] = a.phase_tile0[i];
  for (int i = 0; i <= kMaxPhases; ++i) out[o++] = a.phase_wg0[i];
  for (int i = 0; i < a.num_entries; ++i) {
    out[o++] = a.entry[i].first; out[o++] = a.entry[i].row0; out[o++] = a.entry[i].rows; out[o++] = a.entry[i].problem_branch;
  }
  return 0;
}

int mxmoe_group_gemm_plan_tile_map(int kernel_id, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int problem_count, int grid, int32_t* tile_of_wg) {
  auto& reg = registry();
  if (problem_count <= 0 || problem_count > kMaxProblems || !h_sizes || !h_q || !tile_of_wg || grid < 0 || kernel_id < 0 || kernel_id >= (int)reg.size()) {
    last_error() = "bad argument";
    return 5;
  }
  FusedArgs a;
  std::memset(&a, 0, sizeof a);
  int planned = 0;
  if (const int rc = build_fused_tables(reg[kernel_id], h_sizes, h_q, 0, problem_count, a, &planned)) return rc;
  for (int wg = 0; wg < grid; ++wg) tile_of_wg[wg] = tile_of_workgroup(&a, wg);
  return 0;
}

}  // extern "C"
