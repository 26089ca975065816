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

#ifdef __cplusplus
}
#endif
