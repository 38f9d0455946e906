// Bit-exact dequantization kernel: wd[N,K] float16 from packed int4/int8 + group
// scales.  HBM-bound (write dominated: 2 bytes out per 0.5 or 1 byte in).
#include <type_traits>

#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

// One lane converts 8 weights -- one packed int4 word or two int8 words -- per round (one round at int4, two at int8):
// consecutive lanes read consecutive words and write consecutive 16-byte pieces, so every
// load and every store instruction of a wavefront covers one contiguous span.  (K is a
// multiple of the group size, at least 16, so 8 weights never straddle a row or a group.)
// The (row, column) of a unit is needed for its scale only.  It comes from one division per thread -- 32-bit
// unless the matrix has 2^32 units or more (WIDE) -- and, for rows of at least 256 units (K >= 2048), an
// add and a compare per round: a 64-bit division per round is a couple of hundred instructions, several
// times the conversion itself.
template <int BITS, bool WIDE>
__global__ __launch_bounds__(256) void wq_dequant_kernel(const uint32_t* __restrict__ wq,
                                                         const half_t* __restrict__ scales,
                                                         half_t* __restrict__ wd, uint32_t n_rows,
                                                         uint32_t k, uint32_t group, int zero_point) {
  using idx_t = std::conditional_t<WIDE, uint64_t, uint32_t>;
  constexpr int WPL = BITS / 4;  // packed words per lane and round: 1 (int4), 2 (int8)
  constexpr int ROUNDS = BITS == 4 ? 1 : 2;  // (measured: 4 and 8 rounds are 3 - 10 % slower; many short workgroups stream best)
  const uint32_t units_per_row = k / 8;  // 8 weights = 16 bytes of output
  const idx_t total = (idx_t)n_rows * units_per_row;
  const uint32_t groups_per_row = k / group;
  const Q4Consts cs = make_q4_consts(zero_point);
  const idx_t base = (idx_t)blockIdx.x * (256 * ROUNDS) + threadIdx.x;
  const bool long_rows = units_per_row >= 256;
  uint32_t n = (uint32_t)(base / units_per_row);
  uint32_t c = (uint32_t)(base - (idx_t)n * units_per_row);
  uint32_t w[ROUNDS][WPL];
  half_t s[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const idx_t idx = base + (idx_t)r * 256;
    if (r > 0) {
      if (long_rows) {
        c += 256;
        if (c >= units_per_row) {
          c -= units_per_row;
          ++n;
        }
      } else {
        n = (uint32_t)(idx / units_per_row);
        c = (uint32_t)(idx - (idx_t)n * units_per_row);
      }
    }
    if (idx < total) {
      if constexpr (WPL == 1) {
        w[r][0] = wq[idx];
      } else {
        const u32x2 v = reinterpret_cast<const u32x2*>(wq)[idx];
        w[r][0] = v[0];
        w[r][1] = v[1];
      }
      s[r] = scales[(uint64_t)n * groups_per_row + (c * 8) / group];
    }
  }
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const idx_t idx = base + (idx_t)r * 256;
    if (idx >= total) continue;
    const half2_t s2 = bcast_h2(s[r]);
    half2_t h[4];
    if constexpr (BITS == 4) {
      q4_word_natural(w[r][0], s2, cs, h);
    } else {
      q8_word_natural(w[r][0], s2, h);
      q8_word_natural(w[r][WPL - 1], s2, h + 2);
    }
    // non-temporal: the output is two thirds to four fifths of the traffic and is not read again here.  Over
    // matrices rotated through 2 GB: 0.51 - 0.67 of the HBM peak with ordinary stores, 0.54 - 0.72 this way
    // (int8 +8 - 13 %, int4 +4 - 5 %).  The same hint on the packed loads costs a third on int4.
    __builtin_nontemporal_store(u32x4{as_u32(h[0]), as_u32(h[1]), as_u32(h[2]), as_u32(h[3])}, reinterpret_cast<u32x4*>(wd) + idx);
  }
}

// The two benchmark quantizations, int4 with group 32 and int8 with group 128: a quad of packed words (16 bytes:
// 32 or 16 weights) with flat index q takes the scale with flat index q (int4) or q / 8 (int8), so no
// (row, column) is needed.  A lane loads one quad (a wavefront 1 KB), the wavefront's scales come with one
// more load, both are handed to the lanes that write through a wavefront-private 1 KB + 128 B of LDS, and the
// wavefront stores contiguous kilobytes: 6 memory instructions per 4 KB of output instead of 12 at int4
// (0.55 - 0.63 -> 0.70 - 0.73 of the HBM peak), 4 instead of 6 per 2 KB at int8.
template <int BITS, bool WIDE>
__global__ __launch_bounds__(256) void wq_dequant_quad_kernel(const uint32_t* __restrict__ wq,
                                                              const half_t* __restrict__ scales,
                                                              half_t* __restrict__ wd, uint64_t quads,
                                                              int zero_point) {
  using idx_t = std::conditional_t<WIDE, uint64_t, uint32_t>;
  constexpr int UPQ = BITS == 4 ? 4 : 2;   // 16-byte output units per quad
  constexpr int QPS = BITS == 4 ? 1 : 8;   // quads per scale
  __shared__ __attribute__((aligned(16))) uint32_t words[4][256];
  __shared__ uint16_t sc[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const Q4Consts cs = make_q4_consts(zero_point);
  const idx_t q0 = ((idx_t)blockIdx.x * 4 + wave) * 64;  // first quad of this wavefront (a multiple of 64)
  const idx_t q = q0 + lane;
  if (q < (idx_t)quads) *reinterpret_cast<u32x4*>(&words[wave][lane * 4]) = reinterpret_cast<const u32x4*>(wq)[q];
  if (lane < 64 / QPS && q0 + (idx_t)lane * QPS < (idx_t)quads)
    sc[wave][lane] = reinterpret_cast<const uint16_t*>(scales)[q0 / QPS + lane];
  // (the loads below read other lanes' entries: the hardware runs a wavefront's LDS instructions in order, the
  // fences keep the compiler from moving them across the stores)
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
  for (int r = 0; r < UPQ; ++r) {
    const int u = 64 * r + lane;  // unit among this wavefront's 64 * UPQ
    if (q0 + u / UPQ >= (idx_t)quads) continue;
    const half2_t s2 = bcast_h2(__builtin_bit_cast(half_t, sc[wave][u / (UPQ * QPS)]));
    half2_t h[4];
    if constexpr (BITS == 4) {
      q4_word_natural(words[wave][u], s2, cs, h);
    } else {
      const u32x2 v = *reinterpret_cast<const u32x2*>(&words[wave][2 * u]);
      q8_word_natural(v[0], s2, h);
      q8_word_natural(v[1], s2, h + 2);
    }
    __builtin_nontemporal_store(u32x4{as_u32(h[0]), as_u32(h[1]), as_u32(h[2]), as_u32(h[3])},
                                reinterpret_cast<u32x4*>(wd) + (q0 * UPQ + u));
  }
}

namespace {
template <int BITS, bool WIDE>
void launch_dequant_as(const Problem& p, void* wd, dim3 grid) {
  hipLaunchKernelGGL((wq_dequant_kernel<BITS, WIDE>), grid, dim3(256), 0, p.stream, (const uint32_t*)p.wq,
                     (const half_t*)p.scales, (half_t*)wd, (uint32_t)p.n, (uint32_t)p.k, (uint32_t)p.group,
                     p.zero_point);
}
}  // namespace

int launch_dequant(const Problem& p, void* wd) {
  const uint64_t total = (uint64_t)p.n * (p.k / 8);  // units of 8 weights
  if (p.group == (p.bits == 4 ? 32 : 128)) {
    const uint64_t quads = total / (p.bits == 4 ? 4 : 2), qblocks = (quads + 255) / 256;
    if (qblocks == 0) return 0;
    if (qblocks > 0x7FFFFFFFull) {
      set_error("dequantize: %lld x %lld is too large for one launch", (long long)p.n, (long long)p.k);
      return -1;
    }
    const bool wide = total + 1024 > 0xFFFFFFFFull;
    auto go = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3((uint32_t)qblocks), dim3(256), 0, p.stream, (const uint32_t*)p.wq,
                         (const half_t*)p.scales, (half_t*)wd, quads, p.zero_point);
    };
    if (p.bits == 4) wide ? go(wq_dequant_quad_kernel<4, true>) : go(wq_dequant_quad_kernel<4, false>);
    else wide ? go(wq_dequant_quad_kernel<8, true>) : go(wq_dequant_quad_kernel<8, false>);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
      set_error("dequantize launch failed: %s", hipGetErrorString(e));
      return -1;
    }
    return 0;
  }
  const uint64_t per_block = 256 * (p.bits == 4 ? 1 : 2);  // 256 threads x the kernel's rounds
  const uint64_t blocks = (total + per_block - 1) / per_block;
  if (blocks == 0) return 0;
  if (blocks > 0x7FFFFFFFull) {
    set_error("dequantize: %lld x %lld is too large for one launch", (long long)p.n, (long long)p.k);
    return -1;
  }
  const dim3 grid((uint32_t)blocks);
  const bool wide = total + 2048 > 0xFFFFFFFFull;  // (a block's last index must not wrap either)
  if (p.bits == 4) wide ? launch_dequant_as<4, true>(p, wd, grid) : launch_dequant_as<4, false>(p, wd, grid);
  else wide ? launch_dequant_as<8, true>(p, wd, grid) : launch_dequant_as<8, false>(p, wd, grid);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("dequantize launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

}  // namespace wq
