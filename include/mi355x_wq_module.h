/*
 * mi355x_wq_module.h -- the runtime module of one offloaded subgraph: the part of a BYOC backend
 * that survives export_library / load_module and receives its constants at load time.
 *
 * What it replaces in the reference: a backend whose codegen returns a runtime module with
 * SaveToBinary, a `runtime.module.loadbinary_<type_key>` loader and an `__init_<symbol>` function
 * (src/runtime/contrib/json/json_runtime.h:57-135), initialised by the const-loader module that
 * wraps it (src/runtime/const_loader_module.cc:68-79, 126-148) with the constants that
 * relax.transform.RunCodegen collected for the symbol (src/relax/transform/run_codegen.cc:57-65).
 * The object here is that module behind a C ABI: a TVM-side ModuleNode is a thin shim over it
 * (GetFunction -> mi355x_wq_module_get_function, SaveToBinary -> ..._save_to_binary, the registered
 * loader -> ..._load_from_binary).
 *
 * Calling convention.  The module is created with the call description of the whole composite
 * (mi355x_wq_callspec: every role has a slot in the full argument list) and the list of slots that
 * are constants.  `__init_<symbol>` binds one tensor per constant, in the order of the constant
 * names; `<symbol>` then takes the remaining arguments in the order of their slots, outputs last
 * (destination-passing style, src/relax/transform/call_tir_rewrite.cc:94-110), e.g. for
 * slots (wq, scales, x, y) with wq and scales constant: `<symbol>(x, y)`.
 *
 * Constants may live in host memory (device type 1: what the const loader holds after
 * load_module -- NDArrays are always saved as CPU arrays, include/tvm/runtime/ndarray.h:453-465)
 * or on the ROCm device.  Host constants are copied to the current HIP device at init and owned by
 * the module; device constants are borrowed (the caller keeps them alive, as the const loader
 * does).  With MI355X_WQ_MODULE_TILE_WEIGHTS the weights are converted once, at init, to the
 * tile-major layout of mi355x_wq_tile_weights and every call runs mi355x_wq_matmul_tiled on the
 * module's own copy (bit-identical results, 4-18 % faster decode); a composite with the gated tail
 * (silu_mul), which is computed on canonical weights only, keeps its canonical constants.  Init allocates
 * device memory; calls allocate nothing.
 */
#ifndef MI355X_WQ_MODULE_H_
#define MI355X_WQ_MODULE_H_

#include <stdint.h>

#include "mi355x_wq_packed.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mi355x_wq_module mi355x_wq_module;

/* TVMPackedCFunc (include/tvm/runtime/c_runtime_api.h:351-363): what TVMFuncCreateFromCFunc wraps
 * into a PackedFunc together with `resource_handle`. */
typedef int (*mi355x_wq_packed_cfunc)(mi355x_tvm_value* args, int* type_codes, int num_args, void* ret,
                                      void* resource_handle);

enum {
  MI355X_WQ_MODULE_TILE_WEIGHTS = 1, /* convert bound weights to the tile-major layout at init (where it is defined) */
  MI355X_WQ_MODULE_LIBRARY_SCRATCH = 2, /* decode calls may split K on the library's scratch array (mi355x_wq_matmul_static_ws);
                                           a split that needs more than the array holds runs unsplit */
  MI355X_WQ_MODULE_OWN_WORKSPACE = 4,   /* init allocates the K split's workspace for calls of up to
                                           mi355x_wq_module_set_workspace_rows rows; calls run mi355x_wq_matmul_ws on it */
  MI355X_DL_CPU = 1                  /* kDLCPU */
};

/* The module's type key, "mi355x_wq": the loader is registered as
 * "runtime.module.loadbinary_mi355x_wq" (src/runtime/library_module.cc:107-123 looks that name up). */
MI355X_WQ_API const char* mi355x_wq_module_type_key(void);

/* Creates the module of one composite function.  `spec` describes the full argument list;
 * `const_args[i]` is the slot bound by the constant named `const_names[i]` (slots of wq, scales or
 * bias; never x, the residual or the output).  A module without constants needs no init call.
 * MI355X_WQ_MODULE_TILE_WEIGHTS needs both wq and scales among the constants of a matmul; for a
 * (bits, group, K) the tile-major layout is not defined for, init keeps the canonical constants.
 * Returns 0 and the module in *out, or -1 (mi355x_wq_last_error). */
MI355X_WQ_API int mi355x_wq_module_create(const char* symbol, const mi355x_wq_callspec* spec,
                                         const char* const* const_names, const int32_t* const_args,
                                         int32_t num_consts, int32_t flags, mi355x_wq_module** out);

/* With MI355X_WQ_MODULE_OWN_WORKSPACE: the row count up to which calls may split K across workgroups.  Init
 * (which knows N and K from the bound weights) allocates mi355x_wq_workspace_bytes maximised over 1 .. rows and
 * zeroes it; calls of up to `rows` rows then go through mi355x_wq_matmul_ws on that buffer and still allocate
 * nothing, calls of more rows run as without a workspace.  The reference's counterpart is the split-K workspace
 * its generated host code allocates inside every call (python/tvm/contrib/cutlass/gemm_operation.py:294-295,
 * sized at python/tvm/contrib/cutlass/build.py:335), which an unchanged Relax module gets without asking; here it
 * is the module that owns it, so that a call can be captured in a HIP graph.  To be set before
 * __init_<symbol> runs; the count is part of the saved module.  Calls on one module must not overlap in time
 * (they share the buffer).  Returns 0 or -1. */
MI355X_WQ_API int mi355x_wq_module_set_workspace_rows(mi355x_wq_module* mod, int32_t rows);

/* Frees the module and the device memory it owns (copies of host constants, tile-major weights, workspace). */
MI355X_WQ_API void mi355x_wq_module_destroy(mi355x_wq_module* mod);

/* "get_symbol" / "get_const_vars" / "get_json" of the reference module
 * (json_runtime.h:74-79, 143) as plain accessors; the strings live as long as the module. */
MI355X_WQ_API const char* mi355x_wq_module_symbol(const mi355x_wq_module* mod);
MI355X_WQ_API int32_t mi355x_wq_module_num_consts(const mi355x_wq_module* mod);
MI355X_WQ_API const char* mi355x_wq_module_const_name(const mi355x_wq_module* mod, int32_t i);
MI355X_WQ_API const char* mi355x_wq_module_json(const mi355x_wq_module* mod);
MI355X_WQ_API int32_t mi355x_wq_module_initialized(const mi355x_wq_module* mod);

/* GetFunction: "<symbol>" and "__init_<symbol>" give a TVMPackedCFunc and the resource handle to
 * wrap with it; any other name gives *func = NULL (the reference returns PackedFunc(nullptr),
 * json_runtime.h:100-102).  Returns 0, or -1 for NULL arguments.
 *   __init_<symbol>(c0, c1, ...) : one tensor handle (type code 7 or 13) per constant, in the order of
 *                                  the constant names; the TVM shim unpacks the Array<NDArray> that
 *                                  the const loader passes (const_loader_module.cc:140-146).  The
 *                                  first call binds, later calls return 0 and change nothing
 *                                  (json_runtime.h:91-98).
 *   <symbol>(non-constant args)  : fails with "The module has not been initialized" before init
 *                                  (json_runtime.h:82). */
MI355X_WQ_API int mi355x_wq_module_get_function(mi355x_wq_module* mod, const char* name,
                                               mi355x_wq_packed_cfunc* func, void** resource_handle);

/* What the two functions forward to, for callers without PackedFunc plumbing. */
MI355X_WQ_API int mi355x_wq_module_init(mi355x_wq_module* mod, const mi355x_dl_tensor* const* consts,
                                       int32_t num_consts);
MI355X_WQ_API int mi355x_wq_module_call(mi355x_wq_module* mod, mi355x_tvm_value* args, int* type_codes,
                                       int num_args);

/* SaveToBinary (json_runtime.h:105-116), in dmlc::Stream's little-endian encoding: the symbol
 * (uint64 length + bytes), the call description as JSON text (same encoding), the constant names
 * (uint64 count, then strings).  Returns the number of bytes of the encoding and writes it when
 * `capacity` suffices; -1 on error.  The type key in front of it is the container's business
 * (src/runtime/library_module.cc:155-173). */
MI355X_WQ_API int64_t mi355x_wq_module_save_to_binary(const mi355x_wq_module* mod, void* buffer, int64_t capacity);

/* LoadFromBinary (json_runtime.h:118-134): reads one module from `buffer`, reports the bytes
 * consumed, returns 0 or -1 (truncated or malformed input never reads past `size`).  The module
 * comes back uninitialised: its constants arrive through __init_<symbol>. */
MI355X_WQ_API int mi355x_wq_module_load_from_binary(const void* buffer, int64_t size, int64_t* consumed,
                                                   mi355x_wq_module** out);

/* The same from the three fields already read from a stream (what a registered
 * `runtime.module.loadbinary_mi355x_wq` has in hand after stream->Read of symbol, JSON and names). */
MI355X_WQ_API int mi355x_wq_module_create_from_json(const char* symbol, const char* json, const char* const* const_names,
                                                   int32_t num_consts, mi355x_wq_module** out);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_WQ_MODULE_H_ */
