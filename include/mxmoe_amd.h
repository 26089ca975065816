/* C-ABI of the MI355X-native mixed-precision MoE GroupGEMM library (libmxmoe_amd.so).
 *
 * Plain pointers and sizes only.  Every function returns 0 on success and a non-zero code on failure
 * (1 format not supported, 2 bad kernel or branch id, 3 bad size or shape, 4 the launch failed, 5 a required pointer is NULL);
 * mxmoe_last_error() then returns a message for the calling thread.  All device pointers must belong to the
 * current HIP device; `stream` is a hipStream_t passed as void* (NULL = the default stream).  Nothing here
 * allocates device memory or synchronises the stream.
 *
 * Each entry point names the reference interface it replaces (paths relative to the reference repository).
 */
#pragma once
#include <stddef.h>
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
 * out[0..7] = {format (0 fp16, 1 w8a8, 2 w4a4, 3 w4a16 g128, 4 w3a16 g128, 5 w2a16 g128, 6 w4a4 g128), BM, BN, BK, WGM, WGN, lds_bytes, k_multiple}. */
int mxmoe_kernel_num_branches(int kernel_id);
int mxmoe_kernel_branch(int kernel_id, int branch, int32_t out[8]);

/* ---- the fused GroupGEMM launch: replaces FuncType / the generated groupgemm_hz_fused_<i>() host launcher
 *      (mxmoe/kernels/src/include/registry.cuh:28-39, mxmoe/kernels/kernel_sketch.py:25-43,82-145) ----
 *
 * One launch computes Cs[p][M,N] = As[p][M,K] * Bs[p][N,K]^T for every problem p in its own format.
 * As, Bs, scale_a, scale_b, Cs, Ds, d_sizes and d_q are DEVICE arrays of `problem_count` entries; h_sizes and h_q are
 * their HOST mirrors (as in the reference).  Ds is accepted and never read: results are written to Cs only, as by the reference's kernels
 * (hz_fused.cuh:89,110; its caller passes a second array with the same entries, test.cu:446-459); lda/ldb/ldc/ldd and d_q are DEVICE arrays accepted for signature compatibility and never read (leading dimensions are
 * K, K, N; the reference's kernels ignore them as well and its caller passes nullptr, ref_bind.cu:413).
 * A kernel registered with the sequential or the multi-stream policy (mxmoe_kernel_policy) runs the same problem list as one launch
 * per run of consecutive problems of equal format, on `stream` or on up to 4 library-owned side streams that fork from and join
 * `stream` (the reference's ablation launchers, kernel_sketch.py:148-274, 277-406); kernel_id = -1 only ever selects a fused kernel.
 *
 *   format            As[p]                      Bs[p]                               scale_a[p]      scale_b[p]
 *   fp16              fp16 [M,K]                 fp16 [N,K]                          -               -
 *   w8a8_g-1_sym      int8 [M,K]                 fragment blocks of int8 [N,K]  (*)  fp16 [M]        fp16 [N]
 *   w4a4_g-1_sym      int4 [M,K/2] (even k low)  fragment blocks of int4 [N,K/2] (*) fp16 [M]        fp16 [N]
 *   w4a4_g128_sym     int4 [M,K/2] (even k low)  fragment blocks of int4 [N,K/2] (*) fp16 [M,K/128]  fp16 [K/128,N] (group-major)
 *   w{4,3,2}a16_g128  fp16 [M,K]                 packed [N/16][K/128][64][w dwords]  -               fp16 [N/16][K/128][16][2]
 *   w8a16_g128        fp16 [M,K]                 packed [N/16][K/128][64][8 dwords]  -               fp16 [N/16][K/128][16][2]
 *   w{8,4,3,2}a16_g-1 as the g128 rows: a channel's one (scale, zero) pair is stored once per group of 128
 *
 * Operand variants (kernels whose mxmoe_kernel_branch reports a variant in out[0] >> 8; chosen by name, never by kernel_id = -1):
 *   w4a4_g-1_sym, variant 1 (bf6): As[p] = the int4 codes as 6-bit floats (e3m2) in fragments of 32 rows x 64 values, 1536 bytes each,
 *     ceil(M/32) * (K/64) of them, row-block-major; Bs[p] = fragment blocks of the same 6-bit codes; scales as w4a4_g-1_sym; K a
 *     multiple of 128, at least 256.  Results equal the integer kernels' bit for bit.
 *   w8a8_g-1_sym, variant 2 (fp8, the reference's w8a8_g-1_sym_E4M3, mm_tile.cuh:696-697): As[p], Bs[p] = OCP e4m3 codes in the int8
 *     layouts, scale = max|x| / 448.
 *   fp16, variant 3 (bfloat16, the reference's bf16, tile_config.py:42): As[p], Bs[p] and Cs[p] hold bfloat16 numbers in the fp16
 *     layouts; fp32 accumulation, one rounding (to nearest even) to bfloat16.  GroupGEMM entry points only: the layer forward's
 *     activation step computes in fp16.
 *
 * (*) weights of the integer formats are stored in MFMA fragment order: uint8 [ceil(N/32)][KB/64][2][64 lanes][16], KB = bytes per
 *     row; lane l of block (nb, ks, step) holds bytes ks*64 + (2*step + (l >> 5))*16 .. +16 of channel nb*32 + (l & 31), channels past N
 *     are zero (mxmoe_amd.pack.pack_wxax_fragments; the role of the reference's pack_wxax / permute_weight, quantize.cuh:318-381,424-475).
 *
 * kernel_id = -1 selects the first registered kernel that has a tile for every format in h_q.
 * acc_dump (optional, may be NULL) is a DEVICE array of per-problem int32 [M,N] buffers (entries may be NULL) that
 * receive the raw accumulators (int32 for w8a8 / w4a4 per channel, fp32 bit patterns otherwise: for w4a4_g128 the fp32 sum over the
 * groups of float(group's int32 sum) * (scale_a * scale_b), groups in ascending order); used by the parity tests.
 * Errors: 1 "quant type not supported" (same text as the reference launcher, compose_kernel.py:433), 2 bad kernel id,
 * 3 unsupported shape (K not a multiple of the tile's K step, N not a multiple of 8), 4 launch failure, 5 a required array is NULL
 * (the scale arrays are required as soon as one non-empty problem is quantised). */
int mxmoe_group_gemm(int kernel_id, const void* const* As, const void* const* Bs, const void* const* scale_a, const void* const* scale_b,
                     void* const* Cs, void* const* Ds, const int64_t* lda, const int64_t* ldb, const int64_t* ldc, const int64_t* ldd,
                     const mxmoe_dim3* d_sizes, const mxmoe_dim3* h_sizes, const mxmoe_qparams* d_q, const mxmoe_qparams* h_q, int problem_count,
                     int32_t* const* acc_dump, void* stream);

/* ---- the kernels as functions of the reference's own type: replaces KernelRegistry::Kernel::func and the registry loop of
 *      mxmoe/kernels/src/test.cu:793-815 (FuncType, mxmoe/kernels/src/include/registry.cuh:28-39,72-107) ----
 *
 * mxmoe_kernel_func(i) / mxmoe_get_kernel(name) return kernel i (the kernel whose registry name equals or ends with `name`) as a
 * function taking exactly FuncType's 15 arguments, or NULL.  Such a call launches on the stream last given to mxmoe_set_stream by
 * the calling thread (initially the default stream, where the reference launches, kernel_sketch.py:123).  FuncType returns void:
 * a failing call prints its message to stderr (the reference's launcher does the same and then exits, helper.h:186-193; here the
 * process lives on) and mxmoe_last_status() returns the code of the calling thread's last FuncType call (0 = launched).
 * mxmoe_kernel_policy: 0 fused, 1 sequential, 2 multi-stream (-1 bad id). */
mxmoe_func_t mxmoe_kernel_func(int kernel_id);
mxmoe_func_t mxmoe_get_kernel(const char* name);
int mxmoe_kernel_policy(int kernel_id);
void mxmoe_set_stream(void* stream);
void* mxmoe_get_stream(void);
int mxmoe_last_status(void);

/* Tile count and branch choice the launcher would make, without launching.  The launcher runs the rows of a problem as at
 * most two segments (whole tiles of the largest shape, then the remainder with the cheapest shape that covers it):
 * branch_out[p] receives the branch of the first segment and *tiles_out the total number of tiles over all segments.
 * Host-only; used by the scheduler tests and the kernel-profile table.  Returns 1000 + kernel id on success. */
int mxmoe_group_gemm_plan(int kernel_id, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int problem_count, int32_t* branch_out, int32_t* tiles_out);

/* The tile tables themselves (host-only; what the generated launcher keeps in its prefix-sum array, kernel_sketch.py:89-104): out receives
 * {entries, tiles, phases, workgroups}, phase_tile0[9], phase_wg0[9], then per entry {first tile, first row, rows, problem | branch << 16}.
 * At most 120 problems; used by the tests that compare the device-side planner with the host launcher. */
int mxmoe_group_gemm_plan_tables(int kernel_id, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int problem_count, int32_t* out, int out_ints);

/* The tile each workgroup of such a launch runs when the grid holds `grid` workgroups (host-only; the role of the block -> tile walk of
 * mxmoe/kernels/src/include/tile_scheduler.cuh:25-49): tile_of_wg[w] = tile index, or -1 for a workgroup without a tile.  A planned
 * launch is enqueued with a grid sized for the worst routing, so `grid` may exceed the workgroups the tables need; the function the
 * kernels call to find their tile is the one evaluated here. */
int mxmoe_group_gemm_plan_tile_map(int kernel_id, const mxmoe_dim3* h_sizes, const mxmoe_qparams* h_q, int problem_count, int grid, int32_t* tile_of_wg);

/* ---- routing: what the models' gates compute between the router's logits and this layer (mxmoe/quant/moe_tracer.py:79-86:
 *      F.softmax(router_logits, dim=1, dtype=float) -> torch.topk -> optional division by the sum of the k weights) ----
 *
 * router_logits [num_tokens, num_experts] (device) as fp16 (logits_dtype 0), fp32 (1) or bf16 (2).  Writes topk_ids [num_tokens, topk]
 * int32 and topk_weights [num_tokens, topk] fp32 in order of decreasing probability; equal probabilities go to the lower expert id
 * first (torch.topk leaves that order open).  probability = exp(x - max) / sum in fp32; renormalise != 0 divides the k weights by
 * their sum (Mixtral; Qwen-MoE and DeepSeek-V2-Lite keep the plain probabilities).  1 <= topk <= min(num_experts, 64),
 * num_experts <= 4096, error 3 otherwise; num_tokens = 0 is a no-op. */
int mxmoe_route_topk(const void* router_logits, int logits_dtype, int num_tokens, int num_experts, int topk, int renormalise, int32_t* topk_ids,
                     float* topk_weights, void* stream);

/* ---- token permutation: replaces gg_permute_inp and the sort / bincount prologue of quant_inp_act
 *      (mxmoe/kernels/src/ref_bind.cu:47-64, 449-453) ----
 *
 * topk_ids [num_tokens, topk] int32 (device).  Writes, in STABLE order (by expert, then by flattened (token, slot) index):
 * dst_exp_sorted [R] int32, perm_indices [R] int64 (source token of each sorted row), src_slot [R] int64 (flattened
 * (token, slot) index; may be NULL) and recv_tokens_per_exp [E] int64 (device), R = num_tokens * topk.
 * `workspace` is device scratch of mxmoe_permute_workspace_bytes(R, E) bytes.  Ids outside [0, E) are dropped. */
size_t mxmoe_permute_workspace_bytes(int total_rows, int num_experts);
int mxmoe_build_permutation(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices,
                            int64_t* src_slot, int64_t* recv_tokens_per_exp, void* workspace, void* stream);

/* The same, and also the inverse map: row_of_slot[t * topk + k] = sorted row of token t's k-th expert, -1 where that expert id was out of
 * range (int32 [num_tokens * topk]).  With it the combine needs no preparation pass (mxmoe_combine_planned).  No counterpart in the
 * reference, whose un-permute op is an empty stub (ref_bind.cu:66). */
int mxmoe_build_permutation_inv(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices,
                                int64_t* src_slot, int64_t* recv_tokens_per_exp, int32_t* row_of_slot, void* workspace, void* stream);

/* The same permutation for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  The per-block histograms that the `workspace` argument
 * above brings in live in a static device array of mxmoe_static_scratch_bytes() bytes (1 MiB per GPU, held until the process
 * ends) instead; the call allocates and frees nothing.  Sizes whose mxmoe_permute_workspace_bytes() exceeds it (more than
 * 262144 / num_experts - 1 blocks of 256 rows) are refused with error 3.  All calls on one GPU share that array: calls that overlap
 * in time on one GPU (different streams or threads) race and must be serialised by the caller.  Same outputs as above. */
size_t mxmoe_static_scratch_bytes(void);
int mxmoe_build_permutation_static(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices,
                                   int64_t* src_slot, int64_t* recv_tokens_per_exp, void* stream);

/* ---- activation quantisers: replace the launches of quant_act_kernel and silu_mul_then_quant_kernel
 *      (mxmoe/kernels/src/ref_bind.cu:524-544 and 691-716; their source, act_kernel.cuh, is absent from the reference) ----
 *
 * One workgroup per destination row; rows 0..R-1 are the routed rows in sorted order, rows R..R+T-1 (when has_shared) the
 * always-on shared expert, stored as expert index E.  exp_table is a DEVICE int64 [4][E(+1)] table: tag (0 fp16 copy,
 * 1 int8 per token, 2 int4 per token, 3 int4 with one scale per 128 values), first row, offset into inp_store and offset into
 * scale_store, both offsets in fp16 elements exactly as ref_bind.cu:475-505 computes them (row strides K, K/2, K/4, K/4 halves; one
 * scale per row, K/128 scales per row for tag 3).
 * Two more tags write the operands of the kernels whose branches carry a variant (mxmoe_kernel_branch): 4 = the int4 codes of
 * tag 2 as 6-bit floats in fragments of 32 rows x 64 values (1536 bytes; an expert's region holds ceil(rows / 32) * (K / 64) of them,
 * row-block-major, so its offset into inp_store is counted in fragments of 768 halves; K a multiple of 128), 5 = fp8 (OCP e4m3) codes
 * with scale = max|x| / 448, stored like tag 1.  Neither exists in the reference's prologue (its fp8 kernels take operands
 * converted on the host).
 * rotate: bits 0-1: 0 no rotation, 1 rotate rows of quantised experts, 2 rotate every row; bit 2 (value 4): the table may hold tags 4
 * and 5 (they live in a second set of kernels with a larger register budget; without the bit such an expert is quantised as tag 2).
 * The rotation is y = (H_k kron H_{n/k}) x / sqrt(n)
 * (mxmoe/quant/hadamard_utils.py:96-106).  had_k = 1 for power-of-two rows; otherwise H_k = S_f kron B and had_signs is a
 * DEVICE float [(k/f)^2] array holding B as +-1.0 (mxmoe/quant/hadamard_utils.py:162-4379 tables).
 *
 * mxmoe_quant_act gathers row perm_indices[r] of hidden [T, K] (shared rows read token r - R).
 * mxmoe_silu_mul_quant reads gate_up [R, 2N] (first half gate, second half up; shared rows from gate_up_shared [T, 2*N_shared]),
 * computes silu(gate) * up in fp32 rounded once to fp16, then rotates / quantises / packs like mxmoe_quant_act.
 * scale_store may be NULL when every tag is 0 (no expert quantises its activations). */
int mxmoe_quant_act(const void* hidden, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const int64_t* perm_indices, const int64_t* exp_table,
                    int K, int rows_routed, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f, const float* had_signs, void* stream);
int mxmoe_silu_mul_quant(const void* gate_up, const void* gate_up_shared, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const int64_t* exp_table,
                         int N, int N_shared, int rows_routed, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f,
                         const float* had_signs, void* stream);

/* ---- un-permute + top-k weighted combine: the step after the down launch.  The reference declares it as an empty stub
 *      (gg_unpermute_out, mxmoe/kernels/src/ref_bind.cu:66); the contract here is the one its callers need ----
 *
 * out[t, :] = half( sum_{k ascending} topk_weights[t, k] * float(down_out[row(t, k), :])  + float(shared_out[t, :]) ), accumulated in fp32
 * (each product rounded, then each sum), where row(t, k) is the sorted row whose src_slot equals t * topk + k; slots whose
 * expert id was dropped contribute nothing.  down_out [rows, K] fp16 are the rows of the down launch in sorted order,
 * shared_out [num_tokens, K] fp16 or NULL, topk_weights [num_tokens, topk] fp32, src_slot [rows] int64 as written by
 * mxmoe_build_permutation, out [num_tokens, K] fp16, all DEVICE pointers.  workspace: mxmoe_combine_workspace_bytes() bytes. */
/* mxmoe_quant_act for power-of-two rows (K = 512, 1024, 2048 or 4096; error 3 otherwise), one token at a time instead of one
 * destination row at a time: a token's row is read, rotated and quantised once per format among its destinations and stored to each,
 * so top-k destinations of one format cost one rotation and one quantisation.  Same bytes in inp_store / scale_store as
 * mxmoe_quant_act.  row_of_slot[t * topk + k] is the sorted row of slot k of token t, negative when that slot was dropped
 * (mxmoe_build_permutation_inv, mxmoe_permute_plan_layer); exp_table as above, tags 0 - 3 (a planned block's table sits at
 * mxmoe_plan_offset(1, problems) of its plan); topk <= 8; rotate 0, 1 or 2.  The reference quantises per destination row
 * (ref_bind.cu:524-544). */
int mxmoe_quant_act_tokens(const void* hidden, void* inp_store, void* scale_store, const int32_t* topk_ids, const int32_t* row_of_slot, const int64_t* exp_table,
                           int K, int num_tokens, int topk, int num_experts, int has_shared, int rotate, void* stream);

size_t mxmoe_combine_workspace_bytes(int num_tokens, int topk);
int mxmoe_unpermute_combine(const void* down_out, const void* shared_out, const float* topk_weights, const int64_t* src_slot, int rows, int num_tokens, int topk,
                            int K, void* out, void* workspace, void* stream);

/* ---- a layer forward that never waits for its routing (no counterpart in the reference, whose operators copy the tokens-per-expert
 *      counts to the host and build every table there: mxmoe/kernels/src/ref_bind.cu:451, 475-505, 362-404, kernel_sketch.py:89-104) ----
 *
 * For callers that cannot synchronise or must not let launch arguments depend on the data (HIP graph capture, serving loops): one
 * small kernel per linear block derives, from recv_tokens_per_exp in DEVICE memory, everything the host launcher computes from its
 * host copy (per-expert {tag, first row, offsets} table of the quantisers, the five pointer arrays, the sizes, the tile tables of the
 * fused launch) into a plan buffer; the *_planned entry points read their tables from it.  Same kernels, same results.
 *
 * A block is described per expert by mxmoe_block_desc {QParams, N, K, packed weights, weight scales} (d_desc in device memory, h_desc
 * its host mirror; the shared expert, when shared_rows > 0, is entry num_experts and has shared_rows rows).  At most 4096 problems; a
 * block of more than 120 is planned and run as launches of 120 consecutive experts each (one FusedArgs per launch at the head of
 * the plan buffer).
 * Stores are laid out as the host path lays them out (experts in order, rows packed), so they must be sized for the worst case:
 * capacity rows x the widest row of any expert.
 *
 *   mxmoe_plan_bytes(P)            size of a plan buffer for P problems (device memory, owned by the caller, reusable);
 *   mxmoe_plan_offset(which, P)    byte offset inside it of: 1 the quantisers' int64 [4][P] table, 2 the pointer arrays void* [5][P]
 *                                  (A, B, scale_a, scale_b, C), 3 two int64 {rows routed, address of the shared expert's output rows},
 *                                  4 the sizes mxmoe_dim3 [P];
 *   mxmoe_plan_select_kernel       the kernel (>= 0) that mxmoe_plan_block / mxmoe_plan_grid_bound use for these formats when given -1, after
 *                                  checking formats and shapes; negative on error;
 *   mxmoe_plan_grid_bound          workgroups that cover the launch whatever the routing, for at most routed_rows_max routed rows
 *                                  (tokens x top-k): per expert tiles(M) <= tiles(1) + slope * (M - 1), summed over the non-empty experts
 *                                  (workgroups past the planned tiles cost about 10 - 20 ns each, so the bound is kept tight);
 *   mxmoe_plan_block               enqueue the planning kernel for one block (inp_store / scale_store: the packed activations and
 *                                  their scales that the block reads, out_store: where its output rows go);
 *   mxmoe_plan_layer               the same for the two blocks of a layer (gate_up, down) in one launch: both plans depend on nothing
 *                                  but the tokens-per-expert counts, and a forward of a few dozen microseconds feels every launch;
 *   mxmoe_group_gemm_planned       the fused launch(es) of a block of num_problems experts, grid from mxmoe_plan_grid_bound (workgroups past
 *                                  the planned tiles exit at once);
 *   mxmoe_quant_act_planned, mxmoe_silu_mul_quant_planned, mxmoe_unpermute_combine_planned
 *                                  as their namesakes, with d_plan in place of exp_table / row counts / shared-expert pointers;
 *                                  rows_capacity = tokens x top-k (rows that were not routed because their expert id was out of
 *                                  range are skipped on the device); d_plan_gate_up is the first launch's plan, whose output the
 *                                  SiLU step reads. */
size_t mxmoe_plan_bytes(int num_problems);
size_t mxmoe_plan_offset(int which, int num_problems);
int mxmoe_plan_select_kernel(int kernel_id, const mxmoe_block_desc* h_desc, int num_problems);
int mxmoe_plan_grid_bound(int kernel_id, const mxmoe_block_desc* h_desc, int num_experts, int routed_rows_max, int shared_rows);
int mxmoe_plan_block(int kernel_id, const int64_t* d_recv_tokens_per_exp, int num_experts, int shared_rows, const mxmoe_block_desc* d_desc,
                     const mxmoe_block_desc* h_desc, const void* inp_store, const void* scale_store, void* out_store, void* d_plan, void* stream);
int mxmoe_plan_layer(const mxmoe_plan_call* gate_up, const mxmoe_plan_call* down, const int64_t* d_recv_tokens_per_exp, int num_experts, int shared_rows, void* stream);
/* mxmoe_build_permutation_inv and mxmoe_plan_layer in ONE launch, for decode-sized batches (num_tokens * topk <= 256, error 3 beyond):
 * one workgroup builds the permutation while the others plan both blocks from counts they take from topk_ids themselves.  Same
 * outputs as the two calls (no workspace is needed at this size). */
int mxmoe_permute_plan_layer(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices, int64_t* src_slot,
                             int64_t* recv_tokens_per_exp, int32_t* row_of_slot, const mxmoe_plan_call* gate_up, const mxmoe_plan_call* down, int shared_rows,
                             void* stream);
/* The same pair of calls in TWO launches for larger batches: the experts are counted per chunk of 256 (token, slot) entries, then one
 * launch scatters the chunks and, in further workgroups that do not wait for them, plans both blocks from the same counts (the two
 * separate calls take four launches).  `workspace`: mxmoe_permute_workspace_bytes(num_tokens * topk, num_experts) bytes of device
 * scratch.  Takes batches with ceil(num_tokens * topk / 256) * num_experts <= 16384 (8192 tokens x top-4 over 60 experts: 7680),
 * error 3 beyond; at most 256 entries it is mxmoe_permute_plan_layer. */
int mxmoe_permute_plan_layer_ws(const int32_t* topk_ids, int num_tokens, int topk, int num_experts, int32_t* dst_exp_sorted, int64_t* perm_indices, int64_t* src_slot,
                                int64_t* recv_tokens_per_exp, int32_t* row_of_slot, const mxmoe_plan_call* gate_up, const mxmoe_plan_call* down, int shared_rows,
                                void* workspace, void* stream);
int mxmoe_group_gemm_planned(int kernel_id, const void* d_plan, int num_problems, int grid, void* stream);
int mxmoe_quant_act_planned(const void* hidden, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const int64_t* perm_indices, const void* d_plan,
                            int K, int rows_capacity, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f, const float* had_signs,
                            void* stream);
int mxmoe_silu_mul_quant_planned(const void* gate_up, const void* d_plan_gate_up, void* inp_store, void* scale_store, const int32_t* dst_exp_sorted, const void* d_plan,
                                 int N, int N_shared, int rows_capacity, int num_tokens, int num_experts, int has_shared, int rotate, int had_k, int had_f,
                                 const float* had_signs, void* stream);
int mxmoe_unpermute_combine_planned(const void* down_out, const void* d_plan_down, int num_problems, const float* topk_weights, const int64_t* src_slot, int num_tokens,
                                    int topk, int K, void* out, void* workspace, void* stream);

/* The combine of the planned forward when the permutation already delivered the inverse map (mxmoe_build_permutation_inv): one
 * launch, no workspace. */
int mxmoe_combine_planned(const void* down_out, const void* d_plan_down, int num_problems, const float* topk_weights, const int32_t* row_of_slot, int num_tokens,
                          int topk, int K, void* out, void* stream);

#ifdef __cplusplus
}
#endif
