// Host-side contract between the C ABI (wq_capi.cpp) and the kernel launchers.
#pragma once
#include <atomic>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wq {

struct Problem {
  const void* x;
  const void* wq;
  const void* scales;
  void* y;
  int64_t m, n, k;
  int bits, group, zero_point;
  hipStream_t stream;
  // fused epilogue (all optional): y = f16add(act(f16add(f16(acc), bias[n])), residual[m,n])
  const void* bias = nullptr;
  const void* residual = nullptr;
  int activation = 0;  // 0 none, 1 relu
  // wq / scales are in the tile-major layout written by launch_tile_weights (see wq_tiled.hip)
  bool tiled = false;
};

// Tuning variant: 0 = library default for the shape, >0 = explicit choice
// (only reachable through mi355x_wq_matmul_ex; used by sweeps).
int launch_gemv(const Problem& p, int variant);
bool gemv_applicable(const Problem& p);  // M <= 16 and a default variant's LDS plan (slots + activations) fits
// Cross-workgroup K split of the decode kernel (M <= 16): bytes of caller workspace it needs for `p`
// (0 = no split for this problem), and the launch (1 launched, 0 not applicable / workspace too small,
// -1 failure).  The workspace holds float32 partial tiles and per-tile arrival counters; the counters
// must be zero before the first use and are zero again when the kernel has finished.
int64_t gemv_split_workspace_bytes(const Problem& p);
int launch_gemv_split(const Problem& p, void* workspace, int64_t workspace_bytes);
// The same split on the library's own file-scope device array (no caller workspace, no allocation):
// 1 launched, 0 the split does not apply, -1 failure (also when the problem needs more than the array holds).
int launch_gemv_split_static(const Problem& p);
int64_t gemv_static_scratch_bytes();
// The same for the direct-weight GEMM (M > 64): 128 x 256 tiles whose K range is split over workgroups where
// those tiles alone would leave half of the CUs idle.
int64_t gemm_split_workspace_bytes(const Problem& p);
int launch_gemm_split(const Problem& p, void* workspace, int64_t workspace_bytes);
int launch_skinny(const Problem& p, int variant);
int launch_gemm(const Problem& p, int variant);
bool gemm_pipe_applicable(const Problem& p);  // K % 64 == 0, operands below 1 GiB
bool launch_gemm_pipe(const Problem& p, int group_shift, int variant);
bool launch_gemm_direct(const Problem& p, int group_shift, int variant);
int launch_dequant(const Problem& p, void* wd);
// canonical -> tile-major (forward) or back; p.wq / p.scales are the source, p.y is unused
int launch_tile_weights(const Problem& p, void* wq_out, void* scales_out, bool forward);
// K and (bits, group) for which the tile-major layout is defined: int4 / group 32 with K % 256 == 0,
// int8 / group 128 with K % 128 == 0
bool tiled_layout_defined(int bits, int group, int64_t k);

// Upper bound of rows the skinny family accepts.
constexpr int64_t kSkinnyMaxM = 256;  // (above 64 rows as grid slices)

void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// Index of the current HIP device, clamped to the size of the per-device caches below.
constexpr int kMaxDevices = 64;
int current_device_slot();

// Raises a kernel's dynamic-LDS limit on the current device, once per device and kernel
// (the attribute is per device; `done` is the kernel's own flag array of kMaxDevices
// entries).  Returns false with the error set if the runtime refuses.
bool ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<bool>* done);

// Compute units of the current device (cached per device).
int cu_count();

}  // namespace wq

// The packed boundary's pieces that the subgraph module (wq_module.cpp) shares.
struct mi355x_wq_callspec;
union mi355x_tvm_value;
namespace wq {
// mi355x_wq_packed_call; when `wq_tiled` is given, a matmul reads these tile-major copies instead of
// the canonical tensors in the wq / scales slots (which are still validated and give N, K and group).
// `library_scratch`: decode matmuls go through mi355x_wq_matmul_static_ws (K split on the library's scratch array).
// `workspace`: device memory of the caller for the K split (mi355x_wq_matmul_ws); it takes precedence over the
// library's scratch array.
int packed_call_with_weights(const mi355x_wq_callspec* spec, mi355x_tvm_value* args, int* type_codes, int num_args,
                             const void* wq_tiled, const void* scales_tiled, bool library_scratch = false,
                             void* workspace = nullptr, int64_t workspace_bytes = 0);
// Forwards the recorded error to TVM's error slot when the process has one; returns -1.
int packed_fail();
}  // namespace wq
