// Bit-exact dequantization kernel: wd[N,K] float16 from packed int4/int8 + group
// scales.  HBM-bound (write dominated: 2 bytes out per 0.5 or 1 byte in).
#include <type_traits>

#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

// One lane converts 8 weights -- one packed int4 word or two int8 words -- per round:
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
  constexpr int ROUNDS = 4;
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
  const uint64_t blocks = (total + 1023) / 1024;     // 256 threads x 4 units
  if (blocks == 0) return 0;
  if (blocks > 0x7FFFFFFFull) {
    set_error("dequantize: %lld x %lld is too large for one launch", (long long)p.n, (long long)p.k);
    return -1;
  }
  const dim3 grid((uint32_t)blocks);
  const bool wide = total + 1024 > 0xFFFFFFFFull;  // (a block's last index must not wrap either)
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
