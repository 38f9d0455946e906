// Tile-major weight layout: the one-off transform between the canonical layout (rows of packed
// words, rows of group scales) and the stream the decode kernel reads fastest.
//
// Canonical (the interchange format): wq[N][K*bits/32] uint32, scales[N][K/group] float16.
// A chunk is 16 bytes of a weight row (32 int4 or 16 int8 weights); a super step is eight chunks
// (128 bytes of a row); a tile is 16 consecutive rows.  Tile-major:
//
//   wq_t    : for tile t, super step s, d in {0,1}, lane l = kq*16 + col (kq in 0..3, col in 0..15)
//             the 16 bytes at ((t*S + s)*2 + d)*1024 + l*16 are chunk s*8 + kq*2 + d of row t*16 + col
//             (S = super steps per row; rows past N are zero)
//   scales_t: int4 / group 32 (one scale per chunk): the 4 bytes at ((t*S + s)*64 + l)*4 are the
//             scales of chunks s*8 + kq*2 and s*8 + kq*2 + 1 of row t*16 + col;
//             int8 / group 128 (one scale per super step): the float16 at ((t*S + s)*16 + col)*2.
//
// Both buffers have the size of the canonical ones with N rounded up to a multiple of 16.  The
// transform only moves bytes: tiling followed by untiling returns the input bit for bit, and every
// kernel computes the same values in the same order from either layout.
#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

// One thread per 16-byte chunk of the tile-major weight buffer.
template <bool FORWARD>
__global__ __launch_bounds__(256) void wq_tile_weights_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                              uint32_t n, uint32_t tiles, uint32_t nsuper) {
  const uint32_t idx = blockIdx.x * 256u + threadIdx.x;  // index in the tile-major buffer
  if (idx >= tiles * nsuper * 128u) return;
  const uint32_t lane = idx & 63u, d = (idx >> 6) & 1u, item = idx >> 7;
  const uint32_t s = item % nsuper, t = item / nsuper;
  const uint32_t row = t * 16u + (lane & 15u), chunk = s * 8u + (lane >> 4) * 2u + d;
  const size_t canonical = (size_t)row * (nsuper * 8u) + chunk;
  if constexpr (FORWARD) {
    dst[idx] = row < n ? src[canonical] : u32x4{0u, 0u, 0u, 0u};
  } else {
    if (row < n) dst[canonical] = src[idx];
  }
}

// One thread per scale of the tile-major scale buffer.  PER_CHUNK: int4 / group 32, else one per
// super step (int8 / group 128).
template <bool FORWARD, bool PER_CHUNK>
__global__ __launch_bounds__(256) void wq_tile_scales_kernel(const half_t* __restrict__ src, half_t* __restrict__ dst,
                                                             uint32_t n, uint32_t tiles, uint32_t nsuper) {
  const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
  uint32_t row, group;
  if constexpr (PER_CHUNK) {
    if (idx >= tiles * nsuper * 128u) return;
    const uint32_t e = idx & 1u, lane = (idx >> 1) & 63u, item = idx >> 7;
    row = (item / nsuper) * 16u + (lane & 15u);
    group = (item % nsuper) * 8u + (lane >> 4) * 2u + e;
  } else {
    if (idx >= tiles * nsuper * 16u) return;
    const uint32_t col = idx & 15u, item = idx >> 4;
    row = (item / nsuper) * 16u + col;
    group = item % nsuper;
  }
  const size_t canonical = (size_t)row * (PER_CHUNK ? nsuper * 8u : nsuper) + group;
  if constexpr (FORWARD) {
    dst[idx] = row < n ? src[canonical] : (half_t)0;
  } else {
    if (row < n) dst[canonical] = src[idx];
  }
}

bool tiled_layout_defined(int bits, int group, int64_t k) {
  return (bits == 4 && group == 32 && k % 256 == 0) || (bits == 8 && group == 128 && k % 128 == 0);
}

int launch_tile_weights(const Problem& p, void* wq_out, void* scales_out, bool forward) {
  if (!tiled_layout_defined(p.bits, p.group, p.k)) {
    set_error("tile-major layout: needs int4 / group 32 with K %% 256 == 0 or int8 / group 128 with K %% 128 == 0, "
              "got bits=%d group=%d K=%lld", p.bits, p.group, (long long)p.k);
    return -1;
  }
  const uint32_t tiles = (uint32_t)((p.n + 15) / 16), nsuper = (uint32_t)(p.k * p.bits / 8 / 128);
  const uint64_t chunks = (uint64_t)tiles * nsuper * 128u;
  if (chunks * 16u > 0x7FFFFFF0ull) {
    set_error("tile-major layout: weight buffer of %llu bytes exceeds the 2 GiB the kernels address",
              (unsigned long long)(chunks * 16u));
    return -1;
  }
  const dim3 block(256), wgrid((unsigned)((chunks + 255) / 256));
  const u32x4* ws = static_cast<const u32x4*>(p.wq);
  const half_t* ss = static_cast<const half_t*>(p.scales);
  if (forward)
    hipLaunchKernelGGL(wq_tile_weights_kernel<true>, wgrid, block, 0, p.stream, ws, static_cast<u32x4*>(wq_out),
                       (uint32_t)p.n, tiles, nsuper);
  else
    hipLaunchKernelGGL(wq_tile_weights_kernel<false>, wgrid, block, 0, p.stream, ws, static_cast<u32x4*>(wq_out),
                       (uint32_t)p.n, tiles, nsuper);
  const bool per_chunk = p.bits == 4;
  const uint64_t nscales = (uint64_t)tiles * nsuper * (per_chunk ? 128u : 16u);
  const dim3 sgrid((unsigned)((nscales + 255) / 256));
  half_t* so = static_cast<half_t*>(scales_out);
  if (per_chunk) {
    if (forward) hipLaunchKernelGGL((wq_tile_scales_kernel<true, true>), sgrid, block, 0, p.stream, ss, so, (uint32_t)p.n, tiles, nsuper);
    else hipLaunchKernelGGL((wq_tile_scales_kernel<false, true>), sgrid, block, 0, p.stream, ss, so, (uint32_t)p.n, tiles, nsuper);
  } else {
    if (forward) hipLaunchKernelGGL((wq_tile_scales_kernel<true, false>), sgrid, block, 0, p.stream, ss, so, (uint32_t)p.n, tiles, nsuper);
    else hipLaunchKernelGGL((wq_tile_scales_kernel<false, false>), sgrid, block, 0, p.stream, ss, so, (uint32_t)p.n, tiles, nsuper);
  }
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("tile-major layout transform launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

}  // namespace wq
