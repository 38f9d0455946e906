// Measurement aid, not part of the quantized-matmul path: a loop of 32x32x16 float16 MFMAs on
// operands that stay in registers (no memory, LDS or other VALU work inside the loop).  What it
// sustains depends only on the operand values, which is how the matrix-pipe rate that the GEMM
// kernels can be held against on real data (as opposed to zeros) is measured.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// operands: per workgroup 8 vectors of 256 lanes x 8 float16 (4 A fragments, then 4 B fragments)
__global__ __launch_bounds__(256) void probe_mfma_kernel(const half8_t* __restrict__ operands,
                                                         float* __restrict__ out, int iters,
                                                         unsigned long long* __restrict__ clocks) {
  half8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = operands[(blockIdx.x * 8 + i) * 256 + threadIdx.x];
    b[i] = operands[(blockIdx.x * 8 + 4 + i) * 256 + threadIdx.x];
  }
  float16_t acc[4];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
  // shader-clock cycles and 100 MHz reference ticks around the loop: cycles per MFMA and the clock
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int t = 0; t < 4; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(t + u) & 3], b[u], acc[t], 0, 0, 0);
  }
  const unsigned long long c1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
  float s = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) s += acc[t][v];
  out[blockIdx.x * 256 + threadIdx.x] = s;
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    clocks[0] = c1 - c0;
    clocks[1] = r1 - r0;
  }
}

}  // namespace

// Launches `blocks` workgroups of four wavefronts (one workgroup per CU fills every SIMD with one
// wavefront), each wavefront issuing 16 * iters MFMAs
// (32768 flops each).  `operands` holds blocks * 8 * 256 * 16 bytes, `out` blocks * 256 floats;
// `clocks` receives two 64-bit counts taken by the first wavefront around its loop: shader-clock
// cycles and 100 MHz reference ticks.  Returns 0, or the HIP error code of the launch.
extern "C" __attribute__((visibility("default"))) int mi355x_probe_mfma_f16(const void* operands, void* out,
                                                                          int blocks, int iters, void* clocks,
                                                                          void* stream) {
  if (operands == nullptr || out == nullptr || clocks == nullptr || blocks <= 0 || iters <= 0) return -1;
  hipLaunchKernelGGL(probe_mfma_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const half8_t*>(operands), static_cast<float*>(out), iters,
                     static_cast<unsigned long long*>(clocks));
  return (int)hipGetLastError();
}
