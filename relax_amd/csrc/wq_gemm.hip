// LDS-tiled MFMA GEMM for M > 64: y[M,N] = x[M,K] @ dequant(Wq,S)^T.
//
// Bound: dense float16 MFMA.  A workgroup owns a BM x BN output tile and walks K
// in steps of BK.  Per step the packed weight tile (BN x BK int4/int8) is loaded
// with 16-byte buffer loads, dequantized in registers to exactly the float16
// values the CPU path materialises and written to LDS next to the activation
// tile; the wavefronts then run v_mfma_f32_32x32x16_f16 from LDS with float32
// accumulators.  LDS is double buffered: global loads for step t+1 are issued
// before the MFMAs of step t and written to the other buffer afterwards, one
// barrier per step.
//
// LDS rows are padded by 16 bytes (row stride 144 B) so that the 16-byte operand
// reads of 8 consecutive lanes cover all banks once.
#include <algorithm>
#include <atomic>
#include "wq_device.h"
#include "wq_internal.h"

namespace wq {

template <int BITS, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM * WN * 64) void wq_gemm_kernel(
    const half_t* __restrict__ x, const uint32_t* __restrict__ wq, const half_t* __restrict__ scales,
    half_t* y, int M, int N, int K, int group_shift, int zero_point, int tiles_m, int tiles_n,
    const Epilogue ep) {
  constexpr int BK = 64;
  constexpr int LDK = BK + 8;          // halves per LDS row
  constexpr int NT = WM * WN * 64;     // threads
  constexpr int CH = 128 / BITS;       // k per 16-byte packed chunk
  constexpr int TM = BM / WM / 32;     // 32x32 MFMA tiles per wave along M
  constexpr int TN = BN / WN / 32;
  constexpr int XL = BM * BK / 8 / NT;   // 16-byte activation loads per thread per step
  constexpr int WL = BN * BK / CH / NT;  // 16-byte weight loads per thread per step
  static_assert(XL >= 1 && WL >= 1, "tile too small for the thread count");
  static_assert(BM * BK / 8 % NT == 0 && BN * BK / CH % NT == 0, "uneven tile split");

  // dynamic LDS: As[2][BM][LDK] followed by Bs[2][BN][LDK] (over the 64 KB static limit)
  extern __shared__ __attribute__((aligned(16))) unsigned char wq_gemm_smem[];
  half_t(*As)[BM][LDK] = reinterpret_cast<half_t(*)[BM][LDK]>(wq_gemm_smem);
  half_t(*Bs)[BN][LDK] = reinterpret_cast<half_t(*)[BN][LDK]>(wq_gemm_smem + 2 * BM * LDK * sizeof(half_t));

  // XCD-aware tile order: consecutive workgroup ids land on different XCDs, so
  // regroup them to keep the tiles that share a weight column block on one L2.
  const int nblocks = tiles_m * tiles_n;
  int bid = blockIdx.x;
  if ((nblocks & 7) == 0) bid = (bid & 7) * (nblocks >> 3) + (bid >> 3);
  const int tile_m = bid % tiles_m;
  const int tile_n = bid / tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  const uint32_t row_bytes = (uint32_t)K * BITS / 8;
  const uint32_t groups_per_row = ((uint32_t)K / CH) >> group_shift;
  const rsrc_t rw = make_rsrc(wq, (uint32_t)N * row_bytes);
  const rsrc_t rs = make_rsrc(scales, (uint32_t)N * groups_per_row * 2u);
  const rsrc_t rx = make_rsrc(x, (uint32_t)M * (uint32_t)K * 2u);

  // per-thread load coordinates
  int x_row[XL], x_kc[XL];
  uint32_t x_base[XL];
  bool x_ok[XL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int c = tid + i * NT;
    x_row[i] = c / (BK / 8);
    x_kc[i] = c % (BK / 8);
    const int m = m0 + x_row[i];
    x_ok[i] = m < M;
    x_base[i] = (uint32_t)m * (uint32_t)K * 2u + (uint32_t)x_kc[i] * 16u;
  }
  int w_row[WL], w_q[WL];
  uint32_t w_base[WL], s_base[WL];
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int c = tid + i * NT;
    w_row[i] = c / (BK / CH);
    w_q[i] = c % (BK / CH);
    const int n = min(n0 + w_row[i], N - 1);  // rows past N are computed but never stored
    w_base[i] = (uint32_t)n * row_bytes + (uint32_t)w_q[i] * 16u;
    s_base[i] = (uint32_t)n * groups_per_row * 2u;
  }

  const Q4Consts qc = make_q4_consts(zero_point);

  u32x4 xreg[XL];
  u32x4 wreg[WL];
  uint32_t sreg[WL];

  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < XL; ++i) {
      const bool ok = x_ok[i] && (k0 + x_kc[i] * 8 < K);
      xreg[i] = load_b128(rx, ok ? x_base[i] + (uint32_t)k0 * 2u : kOobOffset);
    }
#pragma unroll
    for (int i = 0; i < WL; ++i) {
      const int kk = k0 + w_q[i] * CH;
      const bool ok = kk < K;
      wreg[i] = load_b128(rw, ok ? w_base[i] + (uint32_t)k0 * BITS / 8 : kOobOffset);
      sreg[i] = load_b16(rs, ok ? s_base[i] + (((uint32_t)kk / CH) >> group_shift) * 2u : kOobOffset);
    }
  };

  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < XL; ++i)
      *reinterpret_cast<u32x4*>(&As[buf][x_row[i]][x_kc[i] * 8]) = xreg[i];
#pragma unroll
    for (int i = 0; i < WL; ++i) {
      const half2_t s2 = bcast_h2(__builtin_bit_cast(half_t, (uint16_t)sreg[i]));
      half_t* dst = &Bs[buf][w_row[i]][w_q[i] * CH];
      if constexpr (BITS == 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          half2_t h[4];
          q4_word_natural(wreg[i][j], s2, qc, h);
          *reinterpret_cast<u32x4*>(dst + j * 8) =
              u32x4{as_u32(h[0]), as_u32(h[1]), as_u32(h[2]), as_u32(h[3])};
        }
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          half2_t a[2], b[2];
          q8_word_natural(wreg[i][2 * j], s2, a);
          q8_word_natural(wreg[i][2 * j + 1], s2, b);
          *reinterpret_cast<u32x4*>(dst + j * 8) =
              u32x4{as_u32(a[0]), as_u32(a[1]), as_u32(b[0]), as_u32(b[1])};
        }
      }
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int ksteps = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();

  const int lrow = lane & 31;
  const int lk = (lane >> 5) * 8;
  for (int kt = 0; kt < ksteps; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < ksteps) load_global((kt + 1) * BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      half8_t a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[i] = *reinterpret_cast<const half8_t*>(&As[buf][wm * (BM / WM) + i * 32 + lrow][kk * 16 + lk]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = *reinterpret_cast<const half8_t*>(&Bs[buf][wn * (BN / WN) + j * 32 + lrow][kk * 16 + lk]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < ksteps) store_lds(buf ^ 1);
    __syncthreads();
  }

  // epilogue: lane holds column (lane % 32) and rows 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 tile
  // the tail's shape is tested once, not per element
  const bool plain = ep.bias == nullptr && ep.residual == nullptr && ep.activation == 0;
  auto store_tiles = [&](auto plain_c) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn * (BN / WN) + j * 32 + lrow;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wm * (BM / WM) + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
          if (m < M && n < N) {
            if constexpr (decltype(plain_c)::value) y[(size_t)m * N + n] = (half_t)acc[i][j][v];
            else store_out(ep, y, m, n, N, acc[i][j][v]);
          }
        }
      }
  };
  if (plain) store_tiles(std::true_type{});
  else store_tiles(std::false_type{});
}

namespace {

template <int BITS, int BM, int BN, int WM, int WN>
bool launch_one(const Problem& p, int group_shift) {
  const int tiles_m = (int)((p.m + BM - 1) / BM);
  const int tiles_n = (int)((p.n + BN - 1) / BN);
  dim3 grid(tiles_m * tiles_n), block(WM * WN * 64);
  constexpr size_t lds_bytes = 2 * (size_t)(BM + BN) * (64 + 8) * sizeof(half_t);
  static std::atomic<bool> lds_ok[kMaxDevices];
  if (!ensure_dynamic_lds((const void*)wq_gemm_kernel<BITS, BM, BN, WM, WN>, (int)lds_bytes, lds_ok)) return false;
  hipLaunchKernelGGL((wq_gemm_kernel<BITS, BM, BN, WM, WN>), grid, block, lds_bytes, p.stream,
                     (const half_t*)p.x, (const uint32_t*)p.wq, (const half_t*)p.scales,
                     (half_t*)p.y, (int)p.m, (int)p.n, (int)p.k, group_shift, p.zero_point, tiles_m,
                     tiles_n, Epilogue{(const half_t*)p.bias, (const half_t*)p.residual, p.activation});
  return true;
}

}  // namespace

namespace {

// y = gelu(y) [+ residual], element by element: the second pass of a gelu tail behind the direct-weight
// kernel, which is built without the gelu branch (its 128 accumulator registers leave no room for it).
// The float16 value the first pass stored is the value the fused form would have handed to gelu.
__global__ __launch_bounds__(256) void wq_gelu_tail_kernel(half_t* __restrict__ y, const half_t* __restrict__ residual,
                                                           int64_t count) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
    half_t h = gelu_f16(y[i]);
    if (residual != nullptr) h = h + residual[i];
    y[i] = h;
  }
}

int launch_gemm_any(const Problem& p, int variant, bool direct_ok);

}  // namespace

int launch_gemm(const Problem& p, int variant) {
  if (p.activation != kActGelu) return launch_gemm_any(p, variant, true);
  // gelu: fused by the LDS-staged kernels; behind the direct-weight kernel as a pass of its own -- unless the
  // residual is the output buffer itself, which the first pass would overwrite: then the fused kernels run.
  if (p.residual == p.y) {
    // On tile-major weights only the direct-weight kernel and the register-activation kernel read the layout;
    // the latter fuses gelu, so it runs the rows here, in blocks of as many rows as it takes (rows of the
    // output are independent; an in-place residual is read by the thread that then writes the element).
    if (p.tiled && variant == 0) {
      for (int64_t m0 = 0; m0 < p.m; m0 += kSkinnyMaxM) {
        Problem part = p;
        part.m = std::min<int64_t>(kSkinnyMaxM, p.m - m0);
        part.x = static_cast<const half_t*>(p.x) + m0 * p.k;
        part.y = static_cast<half_t*>(p.y) + m0 * p.n;
        part.residual = part.y;
        const int rc = launch_skinny(part, 0);
        if (rc != 0) return rc;
      }
      return 0;
    }
    return launch_gemm_any(p, variant, false);
  }
  Problem first = p;
  first.activation = 0;
  first.residual = nullptr;
  const int rc = launch_gemm_any(first, variant, true);
  if (rc != 0) return rc;
  const int64_t count = p.m * p.n;
  const int blocks = (int)std::min<int64_t>((count + 255) / 256, (int64_t)cu_count() * 8);
  hipLaunchKernelGGL(wq_gelu_tail_kernel, dim3(blocks), dim3(256), 0, p.stream, (half_t*)p.y, (const half_t*)p.residual, count);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("gelu tail kernel launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

namespace {

int launch_gemm_any(const Problem& p, int variant, bool direct_ok) {
  const int ch = 128 / p.bits;
  int ratio = p.group / ch, group_shift = 0;
  while ((1 << group_shift) < ratio) ++group_shift;
  if (ratio < 1 || (1 << group_shift) != ratio || p.group % ch != 0) {
    set_error("gemm kernel: group %d must be %d times a power of two", p.group, ch);
    return -1;
  }
  if (!direct_ok && (p.tiled || variant >= 21)) {
    set_error("gemm kernel: gelu with the residual in the output buffer is not available on the direct-weight kernel "
              "(tile-major weights, variants 21..29); pass the residual in a buffer of its own");
    return -1;
  }
  if (p.tiled) {
    // only the direct-weight kernel addresses the tile-major layout
    const int64_t tiles128 = ((p.m + 127) / 128) * ((p.n + 255) / 256);
    const int64_t tiles64x128 = ((p.m + 63) / 64) * ((p.n + 127) / 128);
    const int first = tiles128 <= cu_count() / 2 ? 4 : 2;
    bool ok = false;
    if (variant == 0)
      ok = (tiles64x128 <= cu_count() && launch_gemm_direct(p, group_shift, 5)) ||
           (first == 2 && launch_gemm_direct(p, group_shift, 6)) ||
           launch_gemm_direct(p, group_shift, first) || launch_gemm_direct(p, group_shift, first - 1);
    else if (variant >= 21)
      ok = launch_gemm_direct(p, group_shift, variant - 20);
    if (!ok) {
      set_error("gemm kernel: tile-major weights need the direct-weight kernel (K %% 256 == 0, operands below "
                "1 GiB; variant 0 or 21..29), got M=%lld N=%lld K=%lld variant=%d", (long long)p.m,
                (long long)p.n, (long long)p.k, variant);
      return -1;
    }
    variant = -1;
  } else if (variant == 0 && gemm_pipe_applicable(p) && !direct_ok) {
    variant = p.m >= 1024 ? 11 : 12;
  } else if (variant == 0 && gemm_pipe_applicable(p)) {
    // Measured on MI355X, M = 128 .. 4096 on the Llama shapes: the direct-weight kernel with two
    // K groups wins wherever it applies -- with 64-row tiles while 128-row tiles would leave
    // half of the CUs without one; next the same kernel with one group (K below 512), then the
    // LDS-staged pipeline (256x128 tile once M fills it a few times over, else 128x128).
    const int64_t tiles128 = ((p.m + 127) / 128) * ((p.n + 255) / 256);
    const int64_t tiles64x128 = ((p.m + 63) / 64) * ((p.n + 127) / 128);
    const int first = tiles128 <= cu_count() / 2 ? 4 : 2;
    // (and 64x128 tiles with four K groups while even those fit the CUs in one round)
    // (a last round of 128-row tiles that is at most half full runs as 64-row tiles in a launch of its
    // own: 2048 x 22016, 372 -> 346 us in isolation, unchanged under sustained load; never slower)
    if ((tiles64x128 <= cu_count() && launch_gemm_direct(p, group_shift, 5)) ||
        (first == 2 && launch_gemm_direct(p, group_shift, 6)) ||
        launch_gemm_direct(p, group_shift, first) || launch_gemm_direct(p, group_shift, first - 1))
      variant = -1;
    else variant = p.m >= 1024 ? 11 : 12;
  }
  if (p.activation == kActGated && variant != -1 && variant < 21) {
    // only the direct-weight kernel walks the rows in the interleaved gate / up order
    set_error("gemm kernel: the gated tail (silu_mul) needs the direct-weight kernel: K %% 256 == 0, group %d, operands "
              "below 1 GiB; got M=%lld N=%lld K=%lld group=%d variant=%d", p.bits == 4 ? 32 : 128, (long long)p.m,
              (long long)p.n, (long long)p.k, p.group, variant);
    return -1;
  }
  if (variant == -1) {
    // launched above
  } else if (variant >= 21) {
    if (!launch_gemm_direct(p, group_shift, variant - 20)) {
      set_error("gemm kernel: direct-weight variant %d does not apply to M=%lld N=%lld K=%lld group=%d",
                variant, (long long)p.m, (long long)p.n, (long long)p.k, p.group);
      return -1;
    }
    variant = -1;
  } else if (variant >= 11) {
    if (!launch_gemm_pipe(p, group_shift, variant - 10)) {
      set_error("gemm kernel: pipelined variant %d does not apply to M=%lld N=%lld K=%lld", variant,
                (long long)p.m, (long long)p.n, (long long)p.k);
      return -1;
    }
    variant = -1;
  }
  if (variant == 0) variant = 1;
  bool launched = true;
#define WQ_GEMM_CASE(ID, BM, BN, WM, WN)                                  \
  case ID:                                                                \
    launched = p.bits == 4 ? launch_one<4, BM, BN, WM, WN>(p, group_shift) \
                           : launch_one<8, BM, BN, WM, WN>(p, group_shift); \
    break;
  switch (variant) {
    case -1: break;  // already launched above
    WQ_GEMM_CASE(1, 128, 128, 2, 2)
    WQ_GEMM_CASE(2, 256, 128, 2, 2)
    WQ_GEMM_CASE(3, 128, 256, 2, 2)
    WQ_GEMM_CASE(4, 256, 256, 2, 2)
    WQ_GEMM_CASE(5, 256, 256, 2, 4)
    WQ_GEMM_CASE(6, 256, 256, 4, 2)
    default:
      set_error("gemm kernel: unknown variant %d", variant);
      return -1;
  }
#undef WQ_GEMM_CASE
  if (!launched) return -1;  // the error is already set
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("gemm kernel launch failed: %s", hipGetErrorString(e));
    return -1;
  }
  return 0;
}

}  // namespace

}  // namespace wq
