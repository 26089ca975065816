// Diagnostic: what the int8 matrix pipes of this GPU sustain on their own, as a function of the operand data.
// A bare loop of v_mfma_i32_32x32x32_i8 (8 independent accumulators per wave, two waves per SIMD, no memory traffic inside the loop)
// is the ceiling any GroupGEMM tile can approach; it depends on how many operand bits toggle, because the chip lowers its clock under
// the matrix pipes' power draw.  bench.py --mfma-probe launches it per operand mode and reports rate and shader clock.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

// mode 0: all-zero operands; 1: one constant byte pattern; 2: random bytes of the form 16 * v (widened int4 codes, what the w4a4 tiles
// feed); 3: random int8 bytes; 4: random bytes 0 .. 15 (int4 codes kept offset-binary); 5: random sign-extended int4 (-8 .. 7).  src: 4096 random 16-byte words.  out: one int per thread (keeps the accumulators live), then for
// workgroup 0 the shader-clock cycles and the 100 MHz real-time ticks its loop took (two uint64 after the per-thread ints).
template <int MODE>
__global__ void __launch_bounds__(256, 2) mfma_probe_kernel(const v4i* __restrict__ src, int* __restrict__ out, int iters, int threads_total) {
  v16i acc[8];
  for (int i = 0; i < 8; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0;
  v4i a[8], b[8];
  for (int i = 0; i < 8; ++i) {
    if (MODE == 0) {
      a[i] = v4i{0, 0, 0, 0};
      b[i] = v4i{0, 0, 0, 0};
    } else if (MODE == 1) {
      a[i] = v4i{0x37373737, 0x37373737, 0x37373737, 0x37373737};
      b[i] = v4i{0x5a5a5a5a, 0x5a5a5a5a, 0x5a5a5a5a, 0x5a5a5a5a};
    } else {
      const int mask = MODE == 2 ? (int)0xF0F0F0F0 : MODE >= 4 ? 0x0F0F0F0F : -1;
      a[i] = src[(threadIdx.x * 16 + i) & 4095] & mask;
      b[i] = src[(threadIdx.x * 16 + 8 + i) & 4095] & mask;
      if (MODE == 5) {   // byte-wise sign extension of the low nibble: bit 3 copied into bits 4..7
        a[i] = a[i] | ((a[i] & 0x08080808) * 0x1E);
        b[i] = b[i] | ((b[i] & 0x08080808) * 0x1E);
      }
    }
  }
  const uint64_t c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[i], acc[i], 0, 0, 0);
  }
  int s = 0;
  for (int i = 0; i < 8; ++i)
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[blockIdx.x * 256 + threadIdx.x] = s;
  const uint64_t c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    uint64_t* rec = reinterpret_cast<uint64_t*>(out + threadIdx.x + threads_total + (s & 0));   // after the per-thread ints; s keeps the order
    rec[0] = c1 - c0;
    rec[1] = r1 - r0;
  }
}

// ---- the same question for int4 x int4 on the 6-bit float path ----
// Every integer -8 .. 8 is a bf6 (e3m2, bias 3) number, products of two of them are at most 64, and the fp32 accumulator adds
// integers exactly up to 2^24: v_mfma_scale_f32_32x32x64_f8f6f4 with both operands in bf6 and unit scales therefore computes int4
// dot products exactly (K up to 262144), at twice the int8 instruction's operations per cycle.  Operands must already be stored as
// 6-bit codes: there is no cheap way from a two's-complement nibble to sign, exponent and mantissa inside a tile.
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ unsigned bf6_of_int(int v) {  // -8 .. 8 -> sign | exponent | mantissa
  const unsigned m = v < 0 ? -v : v;  // magnitudes 0 .. 8 -> 0, 12, 16, 18, 20, 21, 22, 23, 24 (five bits each, in one constant)
  return (v < 0 ? 0x20u : 0u) | (unsigned)((0x18bdab494180ull >> (5 * m)) & 31u);
}

// 32 values (one lane's share of an operand: row lane % 32, k = 32 * (lane / 32) + i) -> 192 bits, value i at bit 6 * i
__device__ __forceinline__ v8i bf6_pack32(const int8_t* vals) {
  unsigned w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const uint64_t c = (uint64_t)bf6_of_int(vals[i]) << ((6 * i) & 31);
    w[(6 * i) >> 5] |= (unsigned)c;
    w[((6 * i) >> 5) + 1] |= (unsigned)(c >> 32);
  }
  return v8i{(int)w[0], (int)w[1], (int)w[2], (int)w[3], (int)w[4], (int)w[5], 0, 0};
}

// D[m][n] = sum_k A[m][k] * B[n][k] for A, B of 32 x 64 int8 values in -8 .. 8, by one matrix instruction of one wave.
__global__ void __launch_bounds__(64) bf6_dot_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ B, float* __restrict__ D) {
  const int l = threadIdx.x;
  const v8i a = bf6_pack32(A + (l % 32) * 64 + (l / 32) * 32), b = bf6_pack32(B + (l % 32) * 64 + (l / 32) * 32);
  v16f c;
  for (int r = 0; r < 16; ++r) c[r] = 0.f;
  c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 3, 3, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);  // 3 = bf6; scale 2^0
  for (int j = 0; j < 16; ++j) D[((j / 4) * 8 + (l / 32) * 4 + (j % 4)) * 32 + l % 32] = c[j];
}

// mode 6: operands = random integers -8 .. 7 as bf6 codes; mode 7: zeros.  Same shape of loop and records as mfma_probe_kernel.
template <int MODE>
__global__ void __launch_bounds__(256, 2) mfma_bf6_probe_kernel(const v4i* __restrict__ src, int* __restrict__ out, int iters, int threads_total) {
  v16f acc[8];
  for (int i = 0; i < 8; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  v8i a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = b[i] = v8i{0, 0, 0, 0, 0, 0, 0, 0};
    if (MODE == 6) {
      int8_t va[32], vb[32];
      const v4i ra = src[(threadIdx.x * 16 + i) & 4095], rb = src[(threadIdx.x * 16 + 8 + i) & 4095];  // 128 random bits = 32 nibbles each
#pragma unroll
      for (int q = 0; q < 32; ++q) {
        va[q] = (int8_t)(((ra[q >> 3] >> (4 * (q & 7))) & 15) - 8);
        vb[q] = (int8_t)(((rb[q >> 3] >> (4 * (q & 7))) & 15) - 8);
      }
      a[i] = bf6_pack32(va);
      b[i] = bf6_pack32(vb);
    }
  }
  const uint64_t c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i], b[i], acc[i], 3, 3, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
  }
  float s = 0.f;
  for (int i = 0; i < 8; ++i)
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  out[blockIdx.x * 256 + threadIdx.x] = (int)s;
  const uint64_t c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    uint64_t* rec = reinterpret_cast<uint64_t*>(out + threadIdx.x + threads_total + ((int)s & 0));
    rec[0] = c1 - c0;
    rec[1] = r1 - r0;
  }
}

}  // namespace

// One launch of the bare matrix-instruction loop: `workgroups` x 256 threads, `iters` x 8 instructions per wave.
// d_src: 65536 bytes of random data; d_out: (workgroups * 256 + 4) * 4 bytes.  Returns 0, or 3 for bad arguments, 4 for a launch error.
// Operations per launch: 2 * 32 * 32 * 32 * 8 * iters * 4 * workgroups for modes 0 .. 5 (v_mfma_i32_32x32x32_i8), twice that for
// modes 6 and 7 (v_mfma_scale_f32_32x32x64_f8f6f4 on bf6 operands).
extern "C" int mxmoe_mfma_probe(int mode, int iters, int workgroups, const void* d_src, void* d_out, void* stream) {
  if (mode < 0 || mode > 7 || iters < 1 || workgroups < 1 || !d_src || !d_out) return 3;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const v4i* src = static_cast<const v4i*>(d_src);
  int* out = static_cast<int*>(d_out);
  const int total = workgroups * 256;
  switch (mode) {
    case 0: hipLaunchKernelGGL(mfma_probe_kernel<0>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
    case 1: hipLaunchKernelGGL(mfma_probe_kernel<1>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
    case 2: hipLaunchKernelGGL(mfma_probe_kernel<2>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
    case 3: hipLaunchKernelGGL(mfma_probe_kernel<3>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
    case 4: hipLaunchKernelGGL(mfma_probe_kernel<4>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
    case 5: hipLaunchKernelGGL(mfma_probe_kernel<5>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
    case 6: hipLaunchKernelGGL(mfma_bf6_probe_kernel<6>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
    default: hipLaunchKernelGGL(mfma_bf6_probe_kernel<7>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// Diagnostic: D[32][32] (fp32) = A . B^T for A, B of 32 x 64 int8 values in -8 .. 8 (device pointers), computed by one
// v_mfma_scale_f32_32x32x64_f8f6f4 on bf6 operands.  Returns 0, or 3 for a null pointer, 4 for a launch error.
extern "C" int mxmoe_bf6_dot_probe(const void* d_a, const void* d_b, void* d_out, void* stream) {
  if (!d_a || !d_b || !d_out) return 3;
  hipLaunchKernelGGL(bf6_dot_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), static_cast<const int8_t*>(d_a), static_cast<const int8_t*>(d_b), static_cast<float*>(d_out));
  return hipGetLastError() == hipSuccess ? 0 : 4;
}
