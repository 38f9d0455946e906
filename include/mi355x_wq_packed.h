/*
 * mi355x_wq_packed.h -- the TVM-facing boundary: PackedFunc entries with the
 * exact C ABI Relax's VM calls for an external (BYOC) function, taking DLPack
 * tensors in destination-passing style and forwarding to mi355x_wq.h.
 *
 * The TVM / DLPack value types are restated here (layout-identical, own names) so
 * that this header needs neither a TVM nor a DLPack install:
 *   TVMValue, type codes  : include/tvm/runtime/c_runtime_api.h:167-207
 *   DLTensor              : the public DLPack specification (v0.x, as used by
 *                           include/tvm/runtime/c_runtime_api.h:72)
 *   kDLROCM = 10          : include/tvm/runtime/c_runtime_api.h:136 / DLPack
 */
#ifndef MI355X_WQ_PACKED_H_
#define MI355X_WQ_PACKED_H_

#include <stdint.h>

#ifndef MI355X_WQ_API
#define MI355X_WQ_API __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi355x_dl_device {
  int32_t device_type; /* 10 = ROCm */
  int32_t device_id;
} mi355x_dl_device;

typedef struct mi355x_dl_dtype {
  uint8_t code; /* 0 int, 1 uint, 2 float */
  uint8_t bits;
  uint16_t lanes;
} mi355x_dl_dtype;

typedef struct mi355x_dl_tensor {
  void* data;
  mi355x_dl_device device;
  int32_t ndim;
  mi355x_dl_dtype dtype;
  int64_t* shape;
  int64_t* strides; /* NULL = compact row-major */
  uint64_t byte_offset;
} mi355x_dl_tensor;

typedef union mi355x_tvm_value {
  int64_t v_int64;
  double v_float64;
  void* v_handle;
  const char* v_str;
  mi355x_dl_dtype v_type;
  mi355x_dl_device v_device;
} mi355x_tvm_value;

enum {
  MI355X_TVM_NULLPTR = 4,          /* kTVMNullptr */
  MI355X_TVM_DLTENSOR_HANDLE = 7,  /* kTVMDLTensorHandle */
  MI355X_TVM_NDARRAY_HANDLE = 13,  /* kTVMNDArrayHandle: v_handle is also a DLTensor* */
  MI355X_DL_ROCM = 10
};

/*
 * Fixed-name entries, signature TVMBackendPackedCFunc
 * (include/tvm/runtime/c_backend_api.h:49-51).  They are what a library module
 * resolves with dlsym (src/runtime/library_module.cc:45-58, 74-88) and what the
 * generated cutlass entry `<sym>(TVMValue*, int*, int, TVMValue*, int*)` is for
 * the reference backend (src/relay/backend/contrib/codegen_c/codegen_c.h:101-121,
 * 163-235).  Arguments, all tensors (type code 7 or 13):
 *   matmul     : x[M,K] f16, wq[N,K*bits/32] u32, scales[N,K/group] f16, y[M,N] f16 (output, last)
 *   matmul_bias / matmul_bias_relu : x, wq, scales, bias[N] f16, y
 *   matmul_residual                : x, wq, scales, residual[M,N] f16, y
 *   matmul_silu_mul                : x, wq, scales, y[M,N/2] f16 (gate rows then up rows in wq: MI355X_WQ_ACT_SILU_MUL)
 *   dequantize : wq, scales, wd[N,K] f16 (output, last)
 * group is K / scales.shape[1]; the zero point is 7 (q4f16) or 0 (q8f16).
 * Return 0, or -1 after recording the message with TVMAPISetLastError (when the
 * host process exports it) and in mi355x_wq_last_error().  *out_ret_tcode is left
 * untouched (the loader pre-sets kTVMNullptr: "no return value").
 */
MI355X_WQ_API int mi355x_q4f16_matmul(mi355x_tvm_value* args, int* type_codes, int num_args,
                        mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul(mi355x_tvm_value* args, int* type_codes, int num_args,
                        mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q4f16_matmul_bias(mi355x_tvm_value* args, int* type_codes, int num_args,
                             mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q4f16_matmul_bias_relu(mi355x_tvm_value* args, int* type_codes, int num_args,
                                  mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                  void* resource_handle);
MI355X_WQ_API int mi355x_q4f16_matmul_residual(mi355x_tvm_value* args, int* type_codes, int num_args,
                                 mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                 void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul_bias(mi355x_tvm_value* args, int* type_codes, int num_args,
                             mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul_bias_relu(mi355x_tvm_value* args, int* type_codes, int num_args,
                                  mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                  void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul_residual(mi355x_tvm_value* args, int* type_codes, int num_args,
                                 mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                 void* resource_handle);
/* matmul + bias + nn.gelu (MI355X_WQ_ACT_GELU), the reference's *_bias_gelu composite members
 * (python/tvm/contrib/cutlass/gen_tensor_op.py:375-380): args x, wq, scales, bias, out */
MI355X_WQ_API int mi355x_q4f16_matmul_bias_gelu(mi355x_tvm_value* args, int* type_codes, int num_args,
                                  mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                  void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul_bias_gelu(mi355x_tvm_value* args, int* type_codes, int num_args,
                                  mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                  void* resource_handle);
MI355X_WQ_API int mi355x_q4f16_matmul_silu_mul(mi355x_tvm_value* args, int* type_codes, int num_args,
                                 mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                 void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul_silu_mul(mi355x_tvm_value* args, int* type_codes, int num_args,
                                 mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                                 void* resource_handle);
MI355X_WQ_API int mi355x_q4f16_dequantize(mi355x_tvm_value* args, int* type_codes, int num_args,
                            mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                            void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_dequantize(mi355x_tvm_value* args, int* type_codes, int num_args,
                            mi355x_tvm_value* out_ret_value, int* out_ret_tcode,
                            void* resource_handle);

/* Tile-major weight layout (mi355x_wq_tile_weights / mi355x_wq_matmul_tiled in mi355x_wq.h) as
 * destination-passing externs, the way a parameter-preparation function and the model's main
 * function would call them (R.call_tir with one or two outputs: src/relax/transform/call_tir_rewrite.cc:94-110):
 *   tile_weights(wq[N, K*bits/32] u32, scales[N, K/group] f16, wq_tiled[Np, K*bits/32] u32, scales_tiled[Np, K/group] f16)
 *   matmul_tiled(x[M, K] f16, wq_tiled[Np, ...], scales_tiled[Np, ...], y[M, N] f16)
 * with Np = N rounded up to a multiple of 16: the tile-major buffers are declared as tensors of the
 * canonical shape with whole tiles of rows (N itself comes from y). */
MI355X_WQ_API int mi355x_q4f16_tile_weights(mi355x_tvm_value* args, int* type_codes, int num_args,
                              mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_tile_weights(mi355x_tvm_value* args, int* type_codes, int num_args,
                              mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q4f16_matmul_tiled(mi355x_tvm_value* args, int* type_codes, int num_args,
                              mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul_tiled(mi355x_tvm_value* args, int* type_codes, int num_args,
                              mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);

/* Decode with a workspace (mi355x_wq_matmul_ws in mi355x_wq.h) as a destination-passing extern:
 *   matmul_ws(x[M, K] f16, wq[N, K*bits/32] u32, scales[N, K/group] f16, workspace[bytes] u8, y[M, N] f16)
 * The workspace is a 1-d uint8 tensor the module allocates once (R.builtin.alloc_tensor, zero filled),
 * sized with mi355x_wq_workspace_bytes for its largest projection, and passes to every call on the
 * stream; an empty or too small one makes the call equal to matmul. */
MI355X_WQ_API int mi355x_q4f16_matmul_ws(mi355x_tvm_value* args, int* type_codes, int num_args,
                              mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);
MI355X_WQ_API int mi355x_q8f16_matmul_ws(mi355x_tvm_value* args, int* type_codes, int num_args,
                              mi355x_tvm_value* out_ret_value, int* out_ret_tcode, void* resource_handle);

/*
 * Per-symbol call description for generated entries.  FuseOpsByPattern orders the
 * parameters of a composite function by first use
 * (src/relax/transform/fuse_ops.cc:495-517), so the extern usually receives
 * (wq, scales, x, y) rather than (x, wq, scales, y); the codegen hook records the
 * role of each argument here, the way CodegenCutlass records arg0/arg1/arg2
 * (src/relax/backend/contrib/cutlass/codegen.cc:175-184).
 */
typedef struct mi355x_wq_callspec {
  int32_t op;         /* 0 = matmul, 1 = dequantize */
  int32_t bits;       /* 4 or 8 */
  int32_t group;      /* 0 = infer from the scales shape */
  int32_t zero_point; /* 7 for q4f16, 0 for q8f16 */
  int32_t arg_x;      /* argument index of each role; arg_x ignored for dequantize */
  int32_t arg_wq;
  int32_t arg_scales;
  int32_t arg_out;
  int32_t num_args;   /* expected argument count: 4 (matmul) / 3 (dequantize) + fused operands */
  /* fused epilogue of a matmul composite (mi355x_wq_epilogue in mi355x_wq.h) */
  int32_t arg_bias;     /* argument index of bias [N] or [1,N] float16, or -1 */
  int32_t arg_residual; /* argument index of residual [M,N] float16, or -1 */
  int32_t activation;   /* MI355X_WQ_ACT_* */
} mi355x_wq_callspec;

/* The body every entry (fixed-name or generated trampoline) forwards to. */
MI355X_WQ_API int mi355x_wq_packed_call(const mi355x_wq_callspec* spec, mi355x_tvm_value* args, int* type_codes,
                          int num_args);
/* The same body for entries generated with the hook's option {"workspace": true}: decode matmuls (M <= 16) may
 * split K across workgroups on the library's own scratch array (mi355x_wq_matmul_static_ws in mi355x_wq.h:
 * nothing is allocated; calls that overlap in time on one GPU must not both take this path).  The
 * reference's counterpart is the per-backend options map RunCodegen hands to the hook
 * (src/relax/transform/run_codegen.cc:155-162), which its cutlass backend reads for its split-K /
 * tuning switches (python/tvm/contrib/cutlass/build.py:695-696). */
MI355X_WQ_API int mi355x_wq_packed_call_scratch(const mi355x_wq_callspec* spec, mi355x_tvm_value* args, int* type_codes,
                                               int num_args);

/* Stream used by the packed entries on the calling thread (hipStream_t as void*;
 * NULL = null stream, TVM's default: src/runtime/rocm/rocm_common.h:53-63). */
MI355X_WQ_API void mi355x_wq_packed_set_stream(void* stream);
MI355X_WQ_API void* mi355x_wq_packed_get_stream(void);

/*
 * Registers every fixed-name entry above as "mi355x.<name without the mi355x_ prefix>"
 * ("mi355x.q4f16_matmul", "mi355x.q4f16_matmul_bias", ..., "mi355x.q8f16_dequantize") in TVM's
 * global function table through the C API
 * (TVMFuncCreateFromCFunc + TVMFuncRegisterGlobal,
 * include/tvm/runtime/c_runtime_api.h:362-405), resolved from the already loaded
 * TVM runtime with dlsym -- the same effect as TVM_REGISTER_GLOBAL
 * (include/tvm/runtime/registry.h:339-340; idiom of
 * src/runtime/contrib/rocblas/rocblas.cc:68-102), so `R.call_tir("mi355x.q4f16_matmul", ...)`
 * resolves through the VM's registry fallback (src/runtime/relax_vm/vm.cc:705-716).
 * Returns the number of functions registered, or -1 (no TVM runtime in the process).
 */
MI355X_WQ_API int mi355x_wq_register_tvm_globals(int allow_override);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_WQ_PACKED_H_ */
