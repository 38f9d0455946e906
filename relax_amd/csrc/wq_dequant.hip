// Bit-exact dequantization kernel: wd[N,K] float16 from packed int4/int8 + group
// scales.  HBM-bound (write dominated: 2 bytes out per 0.5 or 1 byte in); every
// lane converts one 16-byte packed chunk and issues 16-byte stores.
#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

template <int BITS>
__global__ __launch_bounds__(256) void wq_dequant_kernel(const uint32_t* __restrict__ wq,
                                                         const half_t* __restrict__ scales,
                                                         half_t* __restrict__ wd, uint32_t n_rows,
                                                         uint32_t k, uint32_t group, int zero_point) {
  constexpr uint32_t CH = 128 / BITS;  // k per 16-byte chunk: 32 (int4) / 16 (int8)
  const uint32_t chunks_per_row = k / CH;
  const uint64_t total = (uint64_t)n_rows * chunks_per_row;
  const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const uint32_t n = (uint32_t)(idx / chunks_per_row);
  const uint32_t c = (uint32_t)(idx - (uint64_t)n * chunks_per_row);
  const u32x4 w = *reinterpret_cast<const u32x4*>(wq + idx * 4);
  const half_t s = scales[(uint64_t)n * (k / group) + (c * CH) / group];
  const half2_t s2 = bcast_h2(s);
  u32x4* out = reinterpret_cast<u32x4*>(wd + ((uint64_t)n * k + (uint64_t)c * CH));
  if constexpr (BITS == 4) {
    const Q4Consts cs = make_q4_consts(zero_point);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      half2_t h[4];
      q4_word_natural(w[j], s2, cs, h);
      out[j] = u32x4{as_u32(h[0]), as_u32(h[1]), as_u32(h[2]), as_u32(h[3])};
    }
  } else {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      half2_t a[2], b[2];
      q8_word_natural(w[2 * j], s2, a);
      q8_word_natural(w[2 * j + 1], s2, b);
      out[j] = u32x4{as_u32(a[0]), as_u32(a[1]), as_u32(b[0]), as_u32(b[1])};
    }
  }
}

int launch_dequant(const Problem& p, void* wd) {
  const uint32_t ch = 128 / p.bits;
  const uint64_t total = (uint64_t)p.n * (p.k / ch);
  const uint64_t blocks = (total + 255) / 256;
  if (blocks == 0) return 0;
  if (blocks > 0x7FFFFFFFull) {
    set_error("dequantize: %lld x %lld is too large for one launch", (long long)p.n, (long long)p.k);
    return -1;
  }
  dim3 grid((uint32_t)blocks), block(256);
  if (p.bits == 4)
    hipLaunchKernelGGL(wq_dequant_kernel<4>, grid, block, 0, p.stream, (const uint32_t*)p.wq,
                       (const half_t*)p.scales, (half_t*)wd, (uint32_t)p.n, (uint32_t)p.k,
                       (uint32_t)p.group, p.zero_point);
  else
    hipLaunchKernelGGL(wq_dequant_kernel<8>, grid, block, 0, p.stream, (const uint32_t*)p.wq,
                       (const half_t*)p.scales, (half_t*)wd, (uint32_t)p.n, (uint32_t)p.k,
                       (uint32_t)p.group, p.zero_point);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("dequantize launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

}  // namespace wq
