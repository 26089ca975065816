/* C-ABI of the MI355X-native mixed-precision MoE GroupGEMM library (libmxmoe_amd.so).
 *
 * Plain pointers and sizes only.  Every function returns 0 on success and a non-zero code on failure;
 * mxmoe_last_error() then returns a message for the calling thread.  All device pointers must belong to the
 * current HIP device; `stream` is a hipStream_t passed as void* (NULL = the default stream).  Nothing here
 * allocates device memory or synchronises the stream.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference repository).
 */
#pragma once
#include <stdint.h>

#include "../mxmoe_amd/csrc/include/mxmoe_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Message of the last failing call on this thread ("" if none). */
const char* mxmoe_last_error(void);

/* ---- kernel registry: replaces KernelRegistry / GetGlobalRegistry (mxmoe/kernels/src/include/registry.cuh:72-107) ---- */

/* Number of fused kernels compiled into this library. */
int mxmoe_num_kernels(void);
/* "[qcfg: (BM,BN,BK) (WGM,WGN,1) STAGE], ...fn_name" — the registry key format of registry.cuh:42-70,83-88. */
const char* mxmoe_kernel_name(int kernel_id);
/* Index of the kernel whose name equals or ends with `name`, or -1. */
int mxmoe_find_kernel(const char* name);
/* Number of tile branches of a kernel, and the description of one:
 * out[0..7] = {format (0 fp16, 1 w8a8, 2 w4a4, 3 w4a16 g128, 4 w3a16 g128), BM, BN, BK, WGM, WGN, lds_bytes, k_multiple}. */
int mxmoe_kernel_num_branches(int kernel_id);
int mxmoe_kernel_branch(int kernel_id, int branch, int32_t out[8]);

/* ---- the fused GroupGEMM launch: replaces FuncType / the generated groupgemm_hz_fused_<i>() host launcher
 *      (mxmoe/kernels/src/include/registry.cuh:28-39, mxmoe/kernels/kernel_sketch.py:25-43,82-145) ----
 *
 * One launch computes Cs[p][M,N] = As[p][M,K] * Bs[p][N,K]^T for every problem p in its own format.
 * As, Bs, scale_a, scale_b, Cs, Ds, d_sizes and d_q are DEVICE arrays of `problem_count` entries; h_sizes and h_q are
 * their HOST mirrors (as in the reference).  Ds must alias Cs; lda/ldb/ldc/ldd and d_q are accepted for signature
 * compatibility and ignored (leading dimensions are K, K, N; the reference passes nullptr, ref_bind.cu:413).
 *
 *   format            As[p]                      Bs[p]                               scale_a[p]      scale_b[p]
 *   fp16              fp16 [M,K]                 fp16 [N,K]                          -               -
 *   w8a8_g-1_sym      int8 [M,K]                 int8 [N,K]                          fp16 [M]        fp16 [N]
 *   w4a4_g-1_sym      int4 [M,K/2] (even k low)  int4 [N,K/2]                        fp16 [M]        fp16 [N]
 *   w{4,3}a16_g128    fp16 [M,K]                 packed [N/16][K/128][64][w dwords]  -               fp16 [N/16][K/128][16][2]
 *
 * kernel_id = -1 selects the first registered kernel that has a tile for every format in h_q.
 * acc_dump (optional, may be NULL) is a DEVICE array of per-problem int32 [M,N] buffers (entries may be NULL) that
 * receive the raw accumulators (int32 for w8a8 / w4a4, fp32 bit patterns otherwise); used by the parity tests.
 * Errors: 1 "quant type not supported" (same text as the reference launcher, compose_kernel.py:433), 2 bad kernel id,
 * 3 unsupported shape (K not a multiple of the tile's K step, N not a multiple of 4), 4 launch failure. */
int mxmoe_group_gemm(int kernel_id, const void* const* As, const void* const* Bs, const void* const* scale_a, const void* const* scale_b,
                     void* const* Cs, void* const* Ds, const int64_t* lda, const int64_t* ldb, const int64_t* ldc, const int64_t* ldd,
                     const mxmoe_dim3* d_sizes, const mxmoe_dim3* h_sizes, const mxmoe_qparams* d_q, const mxmoe_qparams* h_q, int problem_count,
                     int32_t* const* acc_dump, void* stream);

/* Tile count and branch choice the launcher would make, without launching: fills branch_out[p] and returns the total
 * number of tiles through *tiles_out.  Host-only; used by the scheduler tests and the kernel-profile table. */
int mxmoe_group_gemm_plan(int kernel_id, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int problem_count, int32_t* branch_out, int32_t* tiles_out);

#ifdef __cplusplus
}
#endif
