// C ABI of the library (include/mi355x_wq.h): argument validation, kernel-family
// dispatch and the thread-local error string.  No kernel is launched unless every
// shape, size and alignment assumption of the kernels has been checked here.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "../../include/mi355x_wq.h"
#include "wq_internal.h"

namespace wq {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int current_device_slot() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return dev >= 0 && dev < kMaxDevices ? dev : kMaxDevices - 1;
}

bool ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<bool>* done) {
  const int slot = current_device_slot();
  if (done[slot].load(std::memory_order_acquire)) return true;  // a race only repeats the same idempotent call
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    set_error("cannot reserve %d bytes of LDS for a kernel on this device: %s", bytes, hipGetErrorString(e));
    return false;
  }
  done[slot].store(true, std::memory_order_release);
  return true;
}

int cu_count() {
  static std::atomic<int> cached[kMaxDevices];  // same value for every caller of a device
  const int slot = current_device_slot();
  if (cached[slot].load(std::memory_order_relaxed) == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        prop.multiProcessorCount > 0)
      cached[slot].store(prop.multiProcessorCount, std::memory_order_relaxed);
    else
      return 256;
  }
  return cached[slot].load(std::memory_order_relaxed);
}

namespace {

constexpr int64_t kMaxBufferBytes = 0x7FFFFFF0ll;  // kernels address buffers with 32-bit offsets

bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

bool check_desc(const mi355x_wq_desc* d, int64_t m) {
  if (d == nullptr) {
    set_error("descriptor is NULL");
    return false;
  }
  if (d->bits != 4 && d->bits != 8) {
    set_error("bits must be 4 or 8, got %d", d->bits);
    return false;
  }
  if (d->reserved != 0) {
    set_error("descriptor.reserved must be 0, got %d", d->reserved);
    return false;
  }
  const int ch = 128 / d->bits;
  if (d->group <= 0 || d->group % ch != 0 || !is_pow2(d->group / ch)) {
    set_error("group must be %d times a power of two for %d-bit weights, got %d", ch, d->bits,
              d->group);
    return false;
  }
  if (d->bits == 4 && (d->zero_point < 0 || d->zero_point > 15)) {
    set_error("zero_point must be in 0..15 for 4-bit weights, got %d", d->zero_point);
    return false;
  }
  if (d->bits == 8 && d->zero_point != 0) {
    set_error("zero_point must be 0 for 8-bit weights, got %d", d->zero_point);
    return false;
  }
  if (d->n < 0 || d->k < 0 || m < 0) {
    set_error("negative extent: M=%lld N=%lld K=%lld", (long long)m, (long long)d->n,
              (long long)d->k);
    return false;
  }
  if (d->k % d->group != 0) {
    set_error("K=%lld is not a multiple of the group size %d", (long long)d->k, d->group);
    return false;
  }
  const int64_t w_bytes = d->n * (d->k * d->bits / 8);
  const int64_t s_bytes = d->n * (d->k / d->group) * 2;
  const int64_t x_bytes = m * d->k * 2;
  if (d->n > 0x7FFFFFFF || d->k > 0x7FFFFFFF || m > 0x7FFFFFFF || w_bytes > kMaxBufferBytes ||
      s_bytes > kMaxBufferBytes || x_bytes > kMaxBufferBytes) {
    set_error("operand too large (each of x, wq, scales must stay below 2 GiB): M=%lld N=%lld K=%lld",
              (long long)m, (long long)d->n, (long long)d->k);
    return false;
  }
  return true;
}

bool check_ptr(const void* p, const char* name, size_t align) {
  if (p == nullptr) {
    set_error("%s is NULL", name);
    return false;
  }
  if (reinterpret_cast<uintptr_t>(p) % align != 0) {
    set_error("%s (%p) is not %zu-byte aligned", name, p, align);
    return false;
  }
  return true;
}

int select_kernel(const mi355x_wq_desc* d, int64_t m, bool tiled = false) {
  Problem p{nullptr, nullptr, nullptr, nullptr, m, d->n, d->k, d->bits, d->group, d->zero_point, nullptr};
  if (gemv_applicable(p)) {
    // The GEMV kernel stages the activations in LDS, in K phases when they do not fit in one piece.
    const int64_t tiles = (d->n + 15) / 16;
    // (with at most 2048 columns of K and 256 row tiles the matrix is so small -- 4 MB -- that the
    // staging kernel's start-up costs more than it saves: 4096 x 2048, 5.6 against 4.9 us)
    const bool tiny = tiles <= 256 && d->k <= 2048;
    // Tile-major weights, at most two row tiles per CU (N <= 8192): the staging is spread over so few
    // tiles that the register-activation kernel, whose loads are as contiguous on this layout, wins for
    // int8 from 4 rows on, from 2 with more than one tile per CU (5120 x 5120: 7.9 - 10.7 us against
    // 8.7 - 11.6 us; 5120 x 13824 at 8 rows: 19.3 against 22.7 us), and for int4 with rows of at least
    // 4 KB at 8 rows and more with more than one tile per CU (5120 x 11008 at 8 rows: 13.7 against
    // 14.7 us).  Everywhere else the staging kernel is ahead or level since its start-up was shortened
    // (int4 4096 x 4096: 4.2 - 5.4 us against 4.3 - 6.5 us; from 640 tiles on always).
    bool few_tiles = false;
    if (tiled && tiles <= 2 * cu_count() && d->k < 16384) {
      const bool long_rows = d->k * d->bits / 8 >= 4096, over_one = tiles > cu_count();
      few_tiles = (d->bits == 8 && (m >= 4 || (m >= 2 && over_one))) || (d->bits == 4 && long_rows && m >= 8 && over_one);
    }
    // (rows of 16384 and more, one tile per CU: the staging kernel at batch 1 - 4, 17.7 against 19.8 us, the
    // other at 8 - 12 rows, 14.7 against 16.7 us)
    if (tiled && d->k >= 16384 && tiles <= cu_count() && m >= 8 && m <= 12) few_tiles = true;
    // int4 from 9 rows on with activations beyond the LDS (K phases in the staging kernel) and at most two row
    // tiles per CU: the register-activation kernel with its staged loads, on both layouts (4096 x 11008 at
    // 9 - 16 rows: 13.0 - 14.3 against 14.7 - 15.6 us, tile-major 11.9 - 12.8 against 13.2 - 14.0;
    // 5120 x 13824: 21 - 22 against 24 - 25 us)
    if (d->bits == 4 && m >= 9 && m * d->k * 2 > 144 * 1024 && tiles <= 2 * cu_count() && d->k < 16384) few_tiles = true;
    if (!tiny && !few_tiles) return MI355X_WQ_KERNEL_GEMV;
  }
  if (m > 64) {
    // 65..128 rows: the GEMM's tiles leave most CUs idle on narrow projections (5120 x 5120 at 65 rows: 40 column
    // tiles of 128, 43 us; 4096 x 11008 int4: 54 us), where the register-activation kernel runs the rows as two
    // grid slices (23 and 30 us).  Measured on both layouts: ahead or level with up to 64 column tiles at int4
    // (8192 x 8192: 31 - 40 against 43 us) and up to 80 at int8 (10240 x 5120: 34 - 41 against 45 us), behind
    // from 96 (12288 x 4096: 29 - 42 against 26 - 28 us) and 120 (15360 x 5120) on.
    const int64_t t128 = (d->n + 127) / 128;
    if (m <= 128 && t128 <= (d->bits == 8 ? 80 : 64)) return MI355X_WQ_KERNEL_SKINNY;
    // and with three or four slices on the narrowest ones: int8 up to 48 column tiles up to 192 rows (5120 x 5120:
    // 26 against 43 us; at 256 rows 38 against 43, and a workspace call takes 34), int4 up to 16 tiles up to 256
    // rows (2048 x 8192: 23 - 26 against 40 us)
    if (m <= kSkinnyMaxM && (d->bits == 8 ? (t128 <= 48 && m <= 192) : t128 <= 16)) return MI355X_WQ_KERNEL_SKINNY;
    return MI355X_WQ_KERNEL_GEMM;
  }
  // 17..64 rows.  The skinny kernel re-reads the activations from L2 once per 16-row weight tile, so
  // its time grows with M and N; the direct-weight GEMM with its 64x128 tile and four K groups costs
  // the same from 1 to 64 rows.  Measured crossovers on MI355X (q4f16 and q8f16, K = 4096 ... 13824, with
  // the skinny kernel's activations, canonical weights and scales staged through LDS): the GEMM takes over only
  // with 160 or more 128-column tiles, and there from the skinny kernel's third row block on (below); with fewer
  // tiles the skinny kernel stays ahead up to 64 rows (12288 x 4096 at 64 rows: 24.7 against 25.7 us,
  // 8192 x 8192: 28 against 43 us).
  const int64_t tiles128 = (d->n + 127) / 128;
  const bool direct_small_tile = d->k % 256 == 0 && d->k >= 1024 && tiles128 <= cu_count() &&
                                 ((d->bits == 4 && d->group == 32) || (d->bits == 8 && d->group == 128));
  if (tiled) {
    // On tile-major weights the skinny kernel's loads are contiguous and it holds out longer
    // (N = 12288: 12.9 - 23.9 us from 17 to 64 rows against the GEMM's 23 - 25 us): with 160 or more column
    // tiles the GEMM takes over from 40 rows at int4 (22016 x 4096: 27.4 against 27.1 us) and from 49 rows
    // at int8 (27648 x 5120: 44.0 against 48.7 us at 48 rows, 48.2 against 47.7 at 64).
    if (direct_small_tile && tiles128 >= 160 && m >= (d->bits == 8 ? 49 : 40)) return MI355X_WQ_KERNEL_GEMM;
    return MI355X_WQ_KERNEL_SKINNY;
  }
  // canonical weights: with 160 or more column tiles the GEMM from 33 rows on (22016 x 4096: 29 us from 1 to 64
  // rows against 26 - 27 us up to 32 rows and 33 - 45 us above; int8 27648 x 5120: 53 against 48 - 49 and 56 - 59)
  if (direct_small_tile && tiles128 >= 160 && m >= 33) return MI355X_WQ_KERNEL_GEMM;
  return MI355X_WQ_KERNEL_SKINNY;
}

}  // namespace
}  // namespace wq

extern "C" {

const char* mi355x_wq_last_error(void) { return wq::g_error; }

int mi355x_wq_version(void) { return 0 * 10000 + 1 * 100 + 0; }

int mi355x_wq_check(const mi355x_wq_desc* desc, int64_t m) {
  return wq::check_desc(desc, m) ? 0 : -1;
}

int mi355x_wq_select_kernel(const mi355x_wq_desc* desc, int64_t m) {
  if (!wq::check_desc(desc, m)) return -1;
  return wq::select_kernel(desc, m);
}

namespace {

int matmul_any_layout(const mi355x_wq_desc* desc, const void* x, const void* wq_, const void* scales,
                      const mi355x_wq_epilogue* ep, void* y, int64_t m, void* stream, int kernel, bool tiled,
                      void* workspace = nullptr, int64_t workspace_bytes = 0, bool library_scratch = false);

}  // namespace

int mi355x_wq_matmul_fused_ex(const mi355x_wq_desc* desc, const void* x, const void* wq_,
                              const void* scales, const mi355x_wq_epilogue* ep, void* y, int64_t m,
                              void* stream, int kernel) {
  return matmul_any_layout(desc, x, wq_, scales, ep, y, m, stream, kernel, false);
}

int mi355x_wq_matmul_tiled(const mi355x_wq_desc* desc, const void* x, const void* wq_tiled,
                           const void* scales_tiled, const mi355x_wq_epilogue* ep, void* y, int64_t m,
                           void* stream) {
  return matmul_any_layout(desc, x, wq_tiled, scales_tiled, ep, y, m, stream, MI355X_WQ_KERNEL_AUTO, true);
}

int64_t mi355x_wq_workspace_bytes(const mi355x_wq_desc* desc, int64_t m, int tiled) {
  using namespace wq;
  if (!check_desc(desc, m)) return -1;
  if (tiled != 0 && !tiled_layout_defined(desc->bits, desc->group, desc->k)) return 0;
  if (m == 0 || desc->n == 0 || desc->k == 0) return 0;
  Problem p{nullptr, nullptr, nullptr, nullptr, m, desc->n, desc->k, desc->bits, desc->group, desc->zero_point, nullptr};
  p.tiled = tiled != 0;
  if (m > 64 && select_kernel(desc, m, tiled != 0) == MI355X_WQ_KERNEL_SKINNY) return 0;  // (see mi355x_wq_matmul_ws)
  return m <= 16 ? gemv_split_workspace_bytes(p) : gemm_split_workspace_bytes(p);
}

int mi355x_wq_matmul_ws(const mi355x_wq_desc* desc, const void* x, const void* wq_, const void* scales,
                        const mi355x_wq_epilogue* ep, void* y, int64_t m, void* stream, int tiled, void* workspace,
                        int64_t workspace_bytes) {
  return matmul_any_layout(desc, x, wq_, scales, ep, y, m, stream, MI355X_WQ_KERNEL_AUTO, tiled != 0, workspace,
                           workspace_bytes);
}

int mi355x_wq_matmul_static_ws(const mi355x_wq_desc* desc, const void* x, const void* wq_, const void* scales,
                               const mi355x_wq_epilogue* ep, void* y, int64_t m, void* stream, int tiled) {
  return matmul_any_layout(desc, x, wq_, scales, ep, y, m, stream, MI355X_WQ_KERNEL_AUTO, tiled != 0, nullptr, 0,
                           true);
}

int64_t mi355x_wq_static_ws_bytes(void) { return wq::gemv_static_scratch_bytes(); }

int mi355x_wq_matmul_tiled_ex(const mi355x_wq_desc* desc, const void* x, const void* wq_tiled,
                              const void* scales_tiled, const mi355x_wq_epilogue* ep, void* y, int64_t m,
                              void* stream, int kernel) {
  return matmul_any_layout(desc, x, wq_tiled, scales_tiled, ep, y, m, stream, kernel, true);
}

int mi355x_wq_tiled_sizes(const mi355x_wq_desc* desc, int64_t* wq_bytes, int64_t* scales_bytes) {
  using namespace wq;
  if (!check_desc(desc, 0)) return -1;
  if (!tiled_layout_defined(desc->bits, desc->group, desc->k)) {
    set_error("tile-major layout: needs int4 / group 32 with K %% 256 == 0 or int8 / group 128 with K %% 128 == 0, "
              "got bits=%d group=%d K=%lld", desc->bits, desc->group, (long long)desc->k);
    return -1;
  }
  const int64_t rows = (desc->n + 15) / 16 * 16;
  if (wq_bytes != nullptr) *wq_bytes = rows * (desc->k * desc->bits / 8);
  if (scales_bytes != nullptr) *scales_bytes = rows * (desc->k / desc->group) * 2;
  return 0;
}

namespace {

int tile_or_untile(const mi355x_wq_desc* desc, const void* wq_src, const void* scales_src, void* wq_dst,
                   void* scales_dst, void* stream, bool forward) {
  using namespace wq;
  if (!check_desc(desc, 0)) return -1;
  if (desc->n == 0 || desc->k == 0) return 0;
  if (!check_ptr(wq_src, forward ? "wq" : "wq_tiled", 16) || !check_ptr(scales_src, forward ? "scales" : "scales_tiled", 16) ||
      !check_ptr(wq_dst, forward ? "wq_tiled" : "wq", 16) || !check_ptr(scales_dst, forward ? "scales_tiled" : "scales", 16))
    return -1;
  if (wq_dst == wq_src || scales_dst == scales_src) {
    set_error("the layout transform is not an in-place operation: source and destination must differ");
    return -1;
  }
  Problem p{nullptr, wq_src, scales_src, nullptr, 0, desc->n, desc->k, desc->bits, desc->group,
            desc->zero_point, static_cast<hipStream_t>(stream)};
  return launch_tile_weights(p, wq_dst, scales_dst, forward);
}

}  // namespace

int mi355x_wq_tile_weights(const mi355x_wq_desc* desc, const void* wq_, const void* scales, void* wq_tiled,
                           void* scales_tiled, void* stream) {
  return tile_or_untile(desc, wq_, scales, wq_tiled, scales_tiled, stream, true);
}

int mi355x_wq_untile_weights(const mi355x_wq_desc* desc, const void* wq_tiled, const void* scales_tiled, void* wq_,
                             void* scales, void* stream) {
  return tile_or_untile(desc, wq_tiled, scales_tiled, wq_, scales, stream, false);
}

namespace {

int matmul_any_layout(const mi355x_wq_desc* desc, const void* x, const void* wq_, const void* scales,
                      const mi355x_wq_epilogue* ep, void* y, int64_t m, void* stream, int kernel, bool tiled,
                      void* workspace, int64_t workspace_bytes, bool library_scratch) {
  using namespace wq;
  if (!check_desc(desc, m)) return -1;
  if (ep != nullptr) {
    if (ep->reserved != 0) {
      set_error("epilogue.reserved must be 0, got %d", ep->reserved);
      return -1;
    }
    if (ep->activation != MI355X_WQ_ACT_NONE && ep->activation != MI355X_WQ_ACT_RELU &&
        ep->activation != MI355X_WQ_ACT_SILU_MUL && ep->activation != MI355X_WQ_ACT_GELU) {
      set_error("unknown epilogue activation %d", ep->activation);
      return -1;
    }
    if (ep->activation == MI355X_WQ_ACT_SILU_MUL) {
      // y[M, N/2] = multiply(nn.silu(acc[:, :N/2]), acc[:, N/2:]): the whole tail of a gate+up projection
      if (ep->bias != nullptr || ep->residual != nullptr) {
        set_error("the gated tail (silu_mul) takes no bias and no residual");
        return -1;
      }
      if (desc->n % 2 != 0) {
        set_error("the gated tail (silu_mul) needs an even N (gate rows, then as many up rows), got N=%lld", (long long)desc->n);
        return -1;
      }
      if (tiled) {
        set_error("the gated tail (silu_mul) is computed on canonical weights only");
        return -1;
      }
    }
  }
  if (m == 0 || desc->n == 0) return 0;  // empty output
  if (desc->k == 0) {
    set_error("K = 0 is not supported (the output would be all zeros)");
    return -1;
  }
  // scales are fetched with up to 16-byte vector loads (rows of scales are 16-byte multiples
  // whenever a kernel does so), hence the same alignment as the other operands
  if (!check_ptr(x, "x", 16) || !check_ptr(wq_, "wq", 16) || !check_ptr(scales, "scales", 16) ||
      !check_ptr(y, "y", 2))
    return -1;
  if (ep != nullptr && ep->bias != nullptr && !check_ptr(ep->bias, "bias", 2)) return -1;
  if (ep != nullptr && ep->residual != nullptr && !check_ptr(ep->residual, "residual", 2)) return -1;
  const int family = kernel & 0xFF, variant = (kernel >> 8) & 0xFFFF;
  Problem p{x, wq_, scales, y, m, desc->n, desc->k, desc->bits, desc->group, desc->zero_point,
            static_cast<hipStream_t>(stream)};
  if (ep != nullptr) {
    p.bias = ep->bias;
    p.residual = ep->residual;
    p.activation = ep->activation;
  }
  if (tiled) {
    if (!tiled_layout_defined(desc->bits, desc->group, desc->k)) {
      set_error("tile-major layout: needs int4 / group 32 with K %% 256 == 0 or int8 / group 128 with "
                "K %% 128 == 0, got bits=%d group=%d K=%lld", desc->bits, desc->group, (long long)desc->k);
      return -1;
    }
    p.tiled = true;
  }
  if (p.activation == MI355X_WQ_ACT_SILU_MUL) {
    // Gated tail: the decode kernel (M <= 16, any of its variants) and the direct-weight GEMM walk the weight
    // rows in the interleaved gate / up order; the K split, the skinny kernel and the LDS-staged GEMMs do not.
    if (family == MI355X_WQ_KERNEL_SKINNY) {
      set_error("the gated tail (silu_mul) is not implemented by the skinny kernel");
      return -1;
    }
    const bool decode = family == MI355X_WQ_KERNEL_GEMV || (family == MI355X_WQ_KERNEL_AUTO && m <= 16 && gemv_applicable(p));
    return decode ? launch_gemv(p, variant) : launch_gemm(p, variant);
  }
  if (workspace != nullptr && family == MI355X_WQ_KERNEL_AUTO) {
    // a caller workspace allows the decode kernel's K split where it pays; everything else is as without
    if (!check_ptr(workspace, "workspace", 16)) return -1;
    // (above 64 rows, where the plain call runs row slices of the register-activation kernel, that is the faster
    // one -- 5120 x 5120 int8 at 192 rows: 26 us against 34 us split -- and the workspace stays unused)
    const bool sliced = m > 64 && select_kernel(desc, m, tiled) == MI355X_WQ_KERNEL_SKINNY;
    const int rc = sliced ? 0 : m <= 16 ? launch_gemv_split(p, workspace, workspace_bytes) : launch_gemm_split(p, workspace, workspace_bytes);
    if (rc != 0) return rc < 0 ? -1 : 0;
  }
  if (library_scratch) {
    // the same split on the library's own device array: nothing is allocated, sizes beyond it are refused
    const int rc = launch_gemv_split_static(p);
    if (rc != 0) return rc < 0 ? -1 : 0;
  }
  if (tiled) {
    // the same choice as for canonical weights; the kernels that read the layout are the decode
    // kernel, the skinny kernel and the direct-weight GEMM (which needs K % 256 == 0)
    switch (family == MI355X_WQ_KERNEL_AUTO ? select_kernel(desc, m, true) : family) {
      case MI355X_WQ_KERNEL_GEMV: return launch_gemv(p, variant);
      case MI355X_WQ_KERNEL_SKINNY: return launch_skinny(p, variant);
      case MI355X_WQ_KERNEL_GEMM: return launch_gemm(p, variant);
      default: set_error("unknown kernel family %d", family); return -1;
    }
  }
  int chosen = family == MI355X_WQ_KERNEL_AUTO ? select_kernel(desc, m) : family;
  switch (chosen) {
    case MI355X_WQ_KERNEL_GEMV: return launch_gemv(p, variant);
    case MI355X_WQ_KERNEL_SKINNY: return launch_skinny(p, variant);
    case MI355X_WQ_KERNEL_GEMM: return launch_gemm(p, variant);
    default: set_error("unknown kernel family %d", family); return -1;
  }
}

}  // namespace

int mi355x_wq_matmul_fused(const mi355x_wq_desc* desc, const void* x, const void* wq_,
                           const void* scales, const mi355x_wq_epilogue* ep, void* y, int64_t m,
                           void* stream) {
  return mi355x_wq_matmul_fused_ex(desc, x, wq_, scales, ep, y, m, stream, MI355X_WQ_KERNEL_AUTO);
}

int mi355x_wq_matmul_ex(const mi355x_wq_desc* desc, const void* x, const void* wq_, const void* scales,
                        void* y, int64_t m, void* stream, int kernel) {
  return mi355x_wq_matmul_fused_ex(desc, x, wq_, scales, nullptr, y, m, stream, kernel);
}

int mi355x_wq_matmul(const mi355x_wq_desc* desc, const void* x, const void* wq_, const void* scales,
                     void* y, int64_t m, void* stream) {
  return mi355x_wq_matmul_fused_ex(desc, x, wq_, scales, nullptr, y, m, stream, MI355X_WQ_KERNEL_AUTO);
}

int mi355x_wq_dequantize(const mi355x_wq_desc* desc, const void* wq_, const void* scales, void* wd,
                         void* stream) {
  using namespace wq;
  if (!check_desc(desc, 0)) return -1;
  if (desc->n == 0 || desc->k == 0) return 0;
  if (!check_ptr(wq_, "wq", 16) || !check_ptr(scales, "scales", 2) || !check_ptr(wd, "wd", 16))
    return -1;
  Problem p{nullptr, wq_, scales, nullptr, 0, desc->n, desc->k, desc->bits, desc->group,
            desc->zero_point, static_cast<hipStream_t>(stream)};
  return launch_dequant(p, wd);
}

}  // extern "C"
