// Measurement aids, not part of the quantized-matmul path.
//
// (1) A loop of 32x32x16 float16 MFMAs on
// operands that stay in registers (no memory, LDS or other VALU work inside the loop).  What it
// sustains depends only on the operand values, which is how the matrix-pipe rate that the GEMM
// kernels can be held against on real data (as opposed to zeros) is measured.
//
// (2) A kernel that only reads: two buffers streamed once with 16-byte loads, four in flight per lane,
// and folded into one word per thread.  Launched like a decode GEMV (one launch per weight matrix), it
// gives the time that launch, ramp and tail take for a given byte count on this part with no arithmetic,
// staging or reduction at all -- the floor the decode kernels are held against.
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

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(512) void probe_stream_read_kernel(const u32x4_t* __restrict__ a, long long na,
                                                                const u32x4_t* __restrict__ b, long long nb,
                                                                unsigned int* __restrict__ out) {
  const long long stride = (long long)gridDim.x * 512, t = (long long)blockIdx.x * 512 + threadIdx.x;
  u32x4_t f = {0u, 0u, 0u, 0u};
  auto sweep = [&](const u32x4_t* __restrict__ p, long long n) {
    long long i = t;
    for (; i + 3 * stride < n; i += 4 * stride) {
      const u32x4_t v0 = __builtin_nontemporal_load(p + i), v1 = __builtin_nontemporal_load(p + i + stride),
                    v2 = __builtin_nontemporal_load(p + i + 2 * stride),
                    v3 = __builtin_nontemporal_load(p + i + 3 * stride);
      f ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < n; i += stride) f ^= __builtin_nontemporal_load(p + i);
  };
  sweep(a, na);
  sweep(b, nb);
  out[t] = f[0] ^ f[1] ^ f[2] ^ f[3];
}

}  // namespace

// Reads `bytes_a` bytes at `a` and `bytes_b` at `b` (16-byte aligned, multiples of 16) once, with
// `blocks` workgroups of eight wavefronts; `out` receives blocks * 512 words.  Returns 0 or the HIP
// error code of the launch.
extern "C" __attribute__((visibility("default"))) int mi355x_probe_stream_read(const void* a, long long bytes_a,
                                                                             const void* b, long long bytes_b,
                                                                             void* out, int blocks, void* stream) {
  if (a == nullptr || out == nullptr || blocks <= 0 || bytes_a < 0 || bytes_b < 0 || (bytes_a | bytes_b) % 16 != 0)
    return -1;
  hipLaunchKernelGGL(probe_stream_read_kernel, dim3((unsigned)blocks), dim3(512), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4_t*>(a), bytes_a / 16, static_cast<const u32x4_t*>(b), bytes_b / 16,
                     static_cast<unsigned int*>(out));
  return (int)hipGetLastError();
}

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
