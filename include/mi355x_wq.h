/*
 * mi355x_wq.h -- C ABI of the MI355X (gfx950) weight-only-quantized
 * dequantize + matmul library.  Plain pointers and sizes only: no TVM, DLPack or
 * torch types appear below this line.  The TVM PackedFunc entries that Relax's VM
 * calls are declared in mi355x_wq_packed.h and forward to the functions here.
 *
 * Data layout (row-major, compact):
 *   x       [M, K]            float16 activations
 *   wq      [N, K*bits/32]    uint32; element k of row n is the field at bit
 *                             (k % (32/bits)) * bits of word k / (32/bits)
 *                             (least-significant field first)
 *   scales  [N, K/group]      float16, one scale per `group` consecutive k
 *   wd      [N, K]            float16 dequantized weights
 *   y       [M, N]            float16 = f16( sum_k f32(x[m,k]) * f32(wd[n,k]) )
 *
 *   bits = 4: wd = (f16(field) - f16(zero_point)) * scale   (one float16 rounding)
 *   bits = 8: wd = f16(int8(field)) * scale                 (zero_point must be 0)
 *
 * Every pointer is device memory of the current HIP device; x, wq, scales and wd must be
 * 16-byte aligned (y, bias and residual: 2 bytes).  All launches are
 * asynchronous on `stream` (a hipStream_t passed as void*; NULL = the null
 * stream); synchronisation is the caller's.  Functions return 0 on success and
 * -1 on failure, in which case nothing was launched and
 * mi355x_wq_last_error() describes the reason (thread-local string).
 */
#ifndef MI355X_WQ_H_
#define MI355X_WQ_H_

#include <stdint.h>

#ifndef MI355X_WQ_API
#define MI355X_WQ_API __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* Describes one quantized weight matrix.  Counterpart of the per-kernel
 * attributes the reference attaches to a partitioned function before codegen
 * (arg shapes, dtypes, leading dimensions):
 * python/tvm/contrib/cutlass/build.py:623-672 (handle_matmul). */
typedef struct mi355x_wq_desc {
  int32_t bits;       /* 4 or 8 */
  int32_t group;      /* k per scale: multiple of 32 (bits=4) or 16 (bits=8), divides K */
  int32_t zero_point; /* bits=4: 0..15 (7 for q4f16); bits=8: 0 */
  int32_t reserved;   /* must be 0 */
  int64_t n;          /* rows of the weight matrix = output features */
  int64_t k;          /* reduction length; multiple of `group` */
} mi355x_wq_desc;

/* Kernel families; MI355X_WQ_KERNEL_AUTO picks by M and K. */
enum {
  MI355X_WQ_KERNEL_AUTO = 0,
  MI355X_WQ_KERNEL_GEMV = 1,  /* HBM-bound decode path: M <= 16, activations staged in LDS */
  MI355X_WQ_KERNEL_GEMM = 2,  /* LDS-tiled MFMA GEMM, any M */
  MI355X_WQ_KERNEL_SKINNY = 3 /* HBM-bound path for M <= 64, activations in registers */
};

/* y[M,N] = f16( x[M,K] @ dequant(wq, scales)^T ), float32 accumulation.
 * Replaces the generated CUTLASS host glue `<sym>_(DLTensor* x, DLTensor* w,
 * DLTensor* out)`: python/tvm/contrib/cutlass/gemm_operation.py:265-303
 * (pointer/shape extraction, launch on the current stream, no host sync). */
MI355X_WQ_API int mi355x_wq_matmul(const mi355x_wq_desc* desc, const void* x, const void* wq, const void* scales,
                     void* y, int64_t m, void* stream);

/* Same, with the kernel family forced (tests and benchmarks). */
MI355X_WQ_API int mi355x_wq_matmul_ex(const mi355x_wq_desc* desc, const void* x, const void* wq,
                        const void* scales, void* y, int64_t m, void* stream, int kernel);

/* Element-wise operations fused behind the matmul, in the order a composite applies them to
 * t0 = f16(accumulator): t1 = t0 + bias[n]; t2 = act(t1); y = t2 + residual[m,n].  Every
 * step is one float16 operation with one rounding, as the CPU path executes `relax.add` /
 * `relax.nn.relu` on float16 tensors (python/tvm/relax/transform/legalize_ops.py:632;
 * relu = max(t, 0): python/tvm/topi/nn/elemwise.py:26-39, lowered to select(t > 0, t, 0):
 * src/target/llvm/codegen_llvm.cc:1500-1504).  This is the
 * `matmul_bias` / `matmul_bias_relu` family of the reference's pattern helpers
 * (python/tvm/relax/dpl/pattern.py:1049-1095) and of its CUTLASS epilogues
 * (python/tvm/contrib/cutlass/gen_tensor_op.py:377-380), plus the residual add that follows
 * the O and down projections of a decoder layer. */
enum {
  MI355X_WQ_ACT_NONE = 0,
  MI355X_WQ_ACT_RELU = 1,
  /* Gated tail of a fused gate+up projection (rows 0 .. N/2-1 of the weights: gate, rows N/2 .. N-1: up):
   *   y[M, N/2] = multiply(nn.silu(h[:, :N/2]), h[:, N/2:]),  h = f16(accumulator)
   * with the float16 operation sequence of the CPU path -- nn.silu(x) = multiply(x, sigmoid(x))
   * (python/tvm/relax/transform/legalize_ops.py:506-510), sigmoid(x) = 1 / (1 + exp(-x))
   * (src/target/intrin_rule.cc:135-141), exp evaluated in float32 and rounded: five float16 roundings.
   * Identical to the CPU result except where the last bit of the float32 exp differs between the two
   * math libraries and survives the rounding to float16 (about one output in a few thousand, then a few
   * float16 ulp).  The reference's counterpart is the activation member of its fused matmul patterns
   * (python/tvm/relax/dpl/pattern.py:1049-1095, python/tvm/contrib/cutlass/gen_tensor_op.py:377-380).
   * `y` is [M, N/2]; no bias, no residual, canonical weights, N even; M <= 16 runs the decode kernel,
   * larger M needs K % 256 == 0 with group 32 (int4) / 128 (int8). */
  MI355X_WQ_ACT_SILU_MUL = 2,
  /* nn.gelu behind the bias add (python/tvm/contrib/cutlass/gen_tensor_op.py:375-380, the *_bias_gelu members),
   * as the float16 operation sequence of its legalized form x * (0.5 + erf(x * sqrt(0.5)) * 0.5)
   * (python/tvm/relax/transform/legalize_ops.py:495-503): the constants rounded to float16, four float16
   * roundings, erf evaluated in float32 and rounded to float16.  The reference's CPU path has no float16 erf
   * to compare with (src/target/intrin_rule.h:39-48 gives it no extern name), so this member is checked
   * against that sequence restated on the host and, in closed form, against x * Phi(x) in float64: within
   * 4 float16 ulp wherever |x| <= 3.5 and the result is a normal number. */
  MI355X_WQ_ACT_GELU = 3
};
typedef struct mi355x_wq_epilogue {
  const void* bias;     /* float16 [N] (device), or NULL */
  const void* residual; /* float16 [M,N] (device, compact), or NULL; may be `y` itself */
  int32_t activation;   /* MI355X_WQ_ACT_* */
  int32_t reserved;     /* must be 0 */
} mi355x_wq_epilogue;

/* y[M,N] = epilogue( f16( x @ dequant(wq, scales)^T ) ); `ep` NULL or all-empty = plain matmul.
 * Same kernels as mi355x_wq_matmul; the epilogue runs on the accumulator registers, so the
 * matmul result makes no extra trip through HBM. */
MI355X_WQ_API int mi355x_wq_matmul_fused(const mi355x_wq_desc* desc, const void* x, const void* wq,
                           const void* scales, const mi355x_wq_epilogue* ep, void* y, int64_t m,
                           void* stream);

/* Same, with the kernel family forced (tests and benchmarks). */
MI355X_WQ_API int mi355x_wq_matmul_fused_ex(const mi355x_wq_desc* desc, const void* x, const void* wq,
                              const void* scales, const mi355x_wq_epilogue* ep, void* y, int64_t m,
                              void* stream, int kernel);

/* wd[N,K] = dequant(wq, scales), bit-exact with the float16 arithmetic of the
 * `decode` PrimFunc as the llvm target lowers it
 * (src/target/llvm/codegen_llvm.cc:820-852, 1271-1285). */
MI355X_WQ_API int mi355x_wq_dequantize(const mi355x_wq_desc* desc, const void* wq, const void* scales, void* wd,
                         void* stream);

/* Tile-major weight layout: a one-off permutation of the bytes of `wq` and `scales` into the order
 * in which the decode kernel consumes them -- for each tile of 16 rows and each 128 bytes of a row,
 * two blocks of 1 KB in which lane l of a wavefront owns bytes 16 l .. 16 l + 15 -- so that every
 * load instruction of the weight stream reads 1 KB contiguously.  The canonical row-major layout stays
 * the interchange format; this is what a parameter-preparation function run once at load time
 * produces (the reference's counterpart is a `relax.layout_transform` / packing PrimFunc applied to
 * the weights before they are bound: python/tvm/relax/op/manipulate.py:113-151,
 * python/tvm/relax/transform/transform.py:210-233).  Defined for the two benchmark quantizations:
 * int4 / group 32 with K % 256 == 0 and int8 / group 128 with K % 128 == 0.  Both tiled buffers
 * have the size of the canonical ones with N rounded up to a multiple of 16 (rows past N are zero).
 * Tiling followed by untiling returns the input bit for bit, and every kernel family computes the
 * same values in the same order from either layout (bit-identical outputs for the same family; the
 * automatic choice of family has crossovers of its own per layout, and two families differ in the
 * order of the float32 additions). */
MI355X_WQ_API int mi355x_wq_tiled_sizes(const mi355x_wq_desc* desc, int64_t* wq_bytes, int64_t* scales_bytes);

/* canonical (wq, scales) -> tile-major (wq_tiled, scales_tiled); all four 16-byte aligned, device. */
MI355X_WQ_API int mi355x_wq_tile_weights(const mi355x_wq_desc* desc, const void* wq, const void* scales,
                                        void* wq_tiled, void* scales_tiled, void* stream);

/* tile-major -> canonical (the inverse; used to hand the weights back in the interchange format). */
MI355X_WQ_API int mi355x_wq_untile_weights(const mi355x_wq_desc* desc, const void* wq_tiled, const void* scales_tiled,
                                          void* wq, void* scales, void* stream);

/* mi355x_wq_matmul_fused on tile-major weights (`ep` may be NULL).  The same three kernel families
 * (the decode kernel reads the contiguous stream, the skinny kernel and the direct-weight GEMM
 * address the layout) with crossovers measured on this layout; where the GEMM runs (more than 128 rows, more
 * than 64 on wider projections) K % 256 == 0 is required. */
MI355X_WQ_API int mi355x_wq_matmul_tiled(const mi355x_wq_desc* desc, const void* x, const void* wq_tiled,
                                        const void* scales_tiled, const mi355x_wq_epilogue* ep, void* y,
                                        int64_t m, void* stream);

/* Same, with the kernel family forced (tests and benchmarks). */
MI355X_WQ_API int mi355x_wq_matmul_tiled_ex(const mi355x_wq_desc* desc, const void* x, const void* wq_tiled,
                                           const void* scales_tiled, const mi355x_wq_epilogue* ep, void* y,
                                           int64_t m, void* stream, int kernel);

/* K split with a caller workspace.  Decode: for M <= 16 and projections whose 16-row tiles leave CUs idle for
 * whole rounds (5120 rows: 320 tiles on 256 CUs) or whose activations are large against one tile per CU,
 * the decode kernel splits K over two to four workgroups per tile; each writes a float32 partial tile
 * to the workspace, and the last to arrive adds them in the order of their K windows (the result does
 * not depend on the order of arrival), applies the epilogue and stores.  5120 x 13824 int8: 22 -> 20 us
 * at batch 1, 31 -> 23 us at 16 rows.  The reference's counterpart is CUTLASS split-K, whose workspace the generated host code
 * allocates per call (python/tvm/contrib/cutlass/build.py:335, conv2d_operation.py:417-418); here the
 * caller owns it, so that nothing is allocated under a stream capture or in a serving loop.
 *
 * mi355x_wq_workspace_bytes: the size mi355x_wq_matmul_ws needs to split K for (desc, m, layout) -- 16 KB of
 * arrival counters at the head, then 1 KB per 16-row tile and K window, so one workspace sized for the
 * largest projection serves projections of every shape; 0 if it
 * would not split (then the call equals mi355x_wq_matmul_fused / _tiled), -1 on an invalid descriptor.
 *
 * Above 64 rows the same call splits K for the direct-weight GEMM where 128 x 256 output tiles would leave
 * at least half of the CUs without one (e.g. 256 rows x 5120 columns: 40 tiles): two to eight workgroups
 * per tile, each on a window of at least 1024 (int8) or 2048 (int4) of K, 128 KB of float32 partials per
 * tile and window behind the same 16 KB of counters, summed in window order as above.  Measured, int8 at
 * 256 rows: 5120 x 13824 91 -> 63 us, 15360 x 5120 71 -> 60 us, 5120 x 5120 39 -> 37 us; int4 at 128-256
 * rows x 4096 x 11008: 50 -> 40-45 us; shapes the split would slow (short K, int4 with more tiles) report 0.
 * From 17 to 64 rows the split runs 64 x 128 tiles (32 KB of partials per tile and window) where the column tiles
 * fill at most half of the CUs and the other kernels have grown past its fixed cost: with K >= 8192 from 33 rows on
 * (int8 on canonical weights: from 25), with shorter K only for int4 on canonical weights above 48 rows with 96 or
 * more column tiles; 4096 x 11008 int4 at 64 rows 31 -> 22 us, 5120 x 13824 int8 at 64 rows 50 -> 34 us.
 * (Above 64 rows on narrow projections, where the plain call runs the register-activation kernel in row slices,
 * 0 is reported: that path is the faster one there.)
 * Workspace rules: device memory, 16-byte aligned, all zero before its first use (the kernel leaves it
 * ready for the next call); calls that share a workspace must not overlap in time (one stream, or
 * ordered by events); a workspace that is NULL or smaller than required disables the split for that call. */
MI355X_WQ_API int64_t mi355x_wq_workspace_bytes(const mi355x_wq_desc* desc, int64_t m, int tiled);
MI355X_WQ_API int mi355x_wq_matmul_ws(const mi355x_wq_desc* desc, const void* x, const void* wq, const void* scales,
                                     const mi355x_wq_epilogue* ep, void* y, int64_t m, void* stream, int tiled,
                                     void* workspace, int64_t workspace_bytes);

/* mi355x_wq_matmul_ws without a workspace argument and without any allocation: the partial tiles and
 * arrival counters of the K split live in a device array that is part of the library's code object
 * (mi355x_wq_static_ws_bytes() bytes: 16 KB of counters + 4 MB of partial tiles per GPU, held until the
 * process ends).  It has no counterpart in the reference: it exists for callers that cannot allocate
 * device memory or pass a buffer they own -- code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  The call itself calls no hipMalloc / hipFree or allocating library routine.
 * Same results as mi355x_wq_matmul_ws with a sufficient workspace, bit for bit.  Where the split does not
 * apply the call equals mi355x_wq_matmul_fused / _tiled; a problem whose split needs more than the array
 * holds (mi355x_wq_workspace_bytes(...) > mi355x_wq_static_ws_bytes()) is refused with -1 -- use the
 * caller-workspace form for it.  All calls on one GPU share that GPU's array: calls that overlap in time
 * on one GPU (two streams, two threads) race; the kernel returns the counters to zero, so consecutive
 * calls need no clearing. */
MI355X_WQ_API int mi355x_wq_matmul_static_ws(const mi355x_wq_desc* desc, const void* x, const void* wq,
                                            const void* scales, const mi355x_wq_epilogue* ep, void* y, int64_t m,
                                            void* stream, int tiled);
MI355X_WQ_API int64_t mi355x_wq_static_ws_bytes(void);

/* Validates a descriptor and a row count without touching the GPU: 0 if
 * mi355x_wq_matmul would accept them. */
MI355X_WQ_API int mi355x_wq_check(const mi355x_wq_desc* desc, int64_t m);

/* Which family AUTO dispatch uses for `m` rows (MI355X_WQ_KERNEL_*), or -1. */
MI355X_WQ_API int mi355x_wq_select_kernel(const mi355x_wq_desc* desc, int64_t m);

/* Thread-local description of the last failure on this thread ("" if none). */
MI355X_WQ_API const char* mi355x_wq_last_error(void);

/* Library version: major * 10000 + minor * 100 + patch. */
MI355X_WQ_API int mi355x_wq_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_WQ_H_ */
