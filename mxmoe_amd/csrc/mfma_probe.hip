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

}  // namespace

// One launch of the bare matrix-instruction loop: `workgroups` x 256 threads, `iters` x 8 instructions per wave.
// d_src: 65536 bytes of random data; d_out: (workgroups * 256 + 4) * 4 bytes.  Returns 0, or 3 for bad arguments, 4 for a launch error.
// Operations per launch: 2 * 32 * 32 * 32 * 8 * iters * 4 * workgroups.
extern "C" int mxmoe_mfma_probe(int mode, int iters, int workgroups, const void* d_src, void* d_out, void* stream) {
  if (mode < 0 || mode > 5 || iters < 1 || workgroups < 1 || !d_src || !d_out) return 3;
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
    default: hipLaunchKernelGGL(mfma_probe_kernel<5>, dim3(workgroups), dim3(256), 0, st, src, out, iters, total); break;
  }
  return hipGetLastError() == hipSuccess ? 0 : 4;
}
