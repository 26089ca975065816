// Plain-old-data types shared by the C-ABI, the host launchers and the gfx950 kernels.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

// One GEMM problem C[M,N] = A[M,K] * B[N,K]^T; x = M (rows / tokens), y = N (out channels), z = K.
// Stands in for CUDA's dim3 in the reference launcher signature (mxmoe/kernels/src/include/registry.cuh:28-39).
typedef struct mxmoe_dim3 {
  uint32_t x, y, z;
} mxmoe_dim3;

// Per-problem quantisation descriptor, 16 bytes: {a_bits, w_bits}, gsize (-1 = per token / per channel), sym.
// Same fields and size as the reference QParams (mxmoe/kernels/src/include/quantize.cuh:14-25).
typedef struct mxmoe_qparams {
  int32_t a_bits;
  int32_t w_bits;
  int32_t gsize;
  uint8_t sym;
  uint8_t _pad[3];
} mxmoe_qparams;

// One linear block (gate_up or down) of one expert as the device-side planner sees it: format, output channels N, reduction
// length K, packed weights and weight scales.  40 bytes.
typedef struct mxmoe_block_desc {
  mxmoe_qparams q;
  uint32_t N, K;
  const void* B;
  const void* scale_b;
} mxmoe_block_desc;

// fp16 storage as the C-ABI names it (the reference's `half`); only ever used behind pointers.
typedef uint16_t mxmoe_half;

// The reference's kernel function type (`FuncType`, mxmoe/kernels/src/include/registry.cuh:28-39) with this library's plain-C
// stand-ins for half, dim3 and QParams (same sizes and layouts, so a caller may cast between the two pointer types).
typedef void (*mxmoe_func_t)(mxmoe_half** ptr_As, mxmoe_half** ptr_Bs, mxmoe_half** ptr_scale_a, mxmoe_half** ptr_scale_b, mxmoe_half** ptr_Cs, mxmoe_half** ptr_Ds,
                             int64_t* ldas, int64_t* ldbs, int64_t* ldcs, int64_t* ldds, mxmoe_dim3* device_problem_sizes, mxmoe_dim3* host_problem_sizes,
                             mxmoe_qparams* device_qbits_list, mxmoe_qparams* host_qbits_list, int problem_count);

// One block (gate_up or down) of a layer for mxmoe_plan_layer: the arguments mxmoe_plan_block takes per block.
typedef struct {
  int kernel_id;                    // -1: chosen from the formats, as mxmoe_plan_select_kernel does
  const mxmoe_block_desc* d_desc;   // device copy of the block descriptors [experts (+ 1 shared)]
  const mxmoe_block_desc* h_desc;   // host copy of the same
  const void* inp_store;            // packed activations the block reads
  const void* scale_store;          // their scales (may be NULL for fp16 activations)
  void* out_store;                  // where the block's output rows go
  void* d_plan;                     // plan buffer of mxmoe_plan_bytes() bytes
} mxmoe_plan_call;

#ifdef __cplusplus
}
#endif
