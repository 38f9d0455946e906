"""ctypes binding of libmi355x_wq.so (the C ABI declared in include/*.h)."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
SO_PATH = os.path.join(CSRC, "libmi355x_wq.so")

KERNEL_AUTO, KERNEL_GEMV, KERNEL_GEMM, KERNEL_SKINNY = 0, 1, 2, 3
ACT_NONE, ACT_RELU, ACT_SILU_MUL, ACT_GELU = 0, 1, 2, 3
ACTIVATIONS = {None: ACT_NONE, "none": ACT_NONE, "relu": ACT_RELU, "relax.nn.relu": ACT_RELU, "silu_mul": ACT_SILU_MUL,
               "gelu": ACT_GELU, "relax.nn.gelu": ACT_GELU}

# every symbol include/mi355x_wq.h, include/mi355x_wq_packed.h and include/mi355x_wq_module.h declare
EXPORTED_SYMBOLS = (
    "mi355x_wq_matmul", "mi355x_wq_matmul_ex", "mi355x_wq_matmul_fused", "mi355x_wq_matmul_fused_ex",
    "mi355x_wq_dequantize", "mi355x_wq_check",
    "mi355x_wq_tiled_sizes", "mi355x_wq_tile_weights", "mi355x_wq_untile_weights", "mi355x_wq_matmul_tiled", "mi355x_wq_matmul_tiled_ex",
    "mi355x_wq_workspace_bytes", "mi355x_wq_matmul_ws", "mi355x_wq_matmul_static_ws", "mi355x_wq_static_ws_bytes",
    "mi355x_wq_select_kernel", "mi355x_wq_last_error", "mi355x_wq_version",
    "mi355x_q4f16_matmul", "mi355x_q8f16_matmul", "mi355x_q4f16_matmul_bias", "mi355x_q8f16_matmul_bias",
    "mi355x_q4f16_matmul_bias_relu", "mi355x_q8f16_matmul_bias_relu", "mi355x_q4f16_matmul_residual",
    "mi355x_q8f16_matmul_residual", "mi355x_q4f16_matmul_bias_gelu", "mi355x_q8f16_matmul_bias_gelu",
    "mi355x_q4f16_matmul_silu_mul", "mi355x_q8f16_matmul_silu_mul", "mi355x_q4f16_dequantize",
    "mi355x_q8f16_dequantize", "mi355x_q4f16_tile_weights", "mi355x_q8f16_tile_weights",
    "mi355x_q4f16_matmul_tiled", "mi355x_q8f16_matmul_tiled", "mi355x_q4f16_matmul_ws", "mi355x_q8f16_matmul_ws",
    "mi355x_wq_packed_call", "mi355x_wq_packed_call_scratch", "mi355x_wq_packed_set_stream",
    "mi355x_wq_packed_get_stream", "mi355x_wq_register_tvm_globals",
    "mi355x_wq_module_type_key", "mi355x_wq_module_create", "mi355x_wq_module_destroy", "mi355x_wq_module_symbol",
    "mi355x_wq_module_num_consts", "mi355x_wq_module_const_name", "mi355x_wq_module_json",
    "mi355x_wq_module_initialized", "mi355x_wq_module_get_function", "mi355x_wq_module_init",
    "mi355x_wq_module_call", "mi355x_wq_module_save_to_binary", "mi355x_wq_module_load_from_binary",
    "mi355x_wq_module_create_from_json", "mi355x_wq_module_set_workspace_rows",
)
PACKED_ENTRIES = tuple(s for s in EXPORTED_SYMBOLS if s.startswith(("mi355x_q4f16_", "mi355x_q8f16_")))


class WqDesc(C.Structure):
    """mi355x_wq_desc"""
    _fields_ = [("bits", C.c_int32), ("group", C.c_int32), ("zero_point", C.c_int32),
                ("reserved", C.c_int32), ("n", C.c_int64), ("k", C.c_int64)]


class WqEpilogue(C.Structure):
    """mi355x_wq_epilogue"""
    _fields_ = [("bias", C.c_void_p), ("residual", C.c_void_p), ("activation", C.c_int32),
                ("reserved", C.c_int32)]


class WqError(RuntimeError):
    """A call into the library returned -1; the message is the library's own."""


_lib = None


def build(verbose: bool = False) -> str:
    """Compile the library for gfx950 in-tree (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-B", "-j8", "-C", CSRC, "all"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
    if res.returncode != 0:
        raise RuntimeError("building libmi355x_wq.so failed")
    return SO_PATH


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise ImportError(
            f"{SO_PATH} is missing: build it with `make -C {CSRC}` "
            "(or __graft_entry__.build()); there is no fallback path")
    L = C.CDLL(SO_PATH)
    vp, i64, ci = C.c_void_p, C.c_int64, C.c_int
    dp = C.POINTER(WqDesc)
    ep = C.POINTER(WqEpilogue)
    L.mi355x_wq_matmul.argtypes = [dp, vp, vp, vp, vp, i64, vp]
    L.mi355x_wq_matmul_ex.argtypes = [dp, vp, vp, vp, vp, i64, vp, ci]
    L.mi355x_wq_matmul_fused.argtypes = [dp, vp, vp, vp, ep, vp, i64, vp]
    L.mi355x_wq_matmul_fused_ex.argtypes = [dp, vp, vp, vp, ep, vp, i64, vp, ci]
    L.mi355x_wq_dequantize.argtypes = [dp, vp, vp, vp, vp]
    L.mi355x_wq_tiled_sizes.argtypes = [dp, C.POINTER(i64), C.POINTER(i64)]
    L.mi355x_wq_tile_weights.argtypes = [dp, vp, vp, vp, vp, vp]
    L.mi355x_wq_untile_weights.argtypes = [dp, vp, vp, vp, vp, vp]
    L.mi355x_wq_matmul_tiled.argtypes = [dp, vp, vp, vp, ep, vp, i64, vp]
    L.mi355x_wq_matmul_tiled_ex.argtypes = [dp, vp, vp, vp, ep, vp, i64, vp, ci]
    L.mi355x_wq_workspace_bytes.argtypes = [dp, i64, ci]
    L.mi355x_wq_workspace_bytes.restype = i64
    L.mi355x_wq_matmul_ws.argtypes = [dp, vp, vp, vp, ep, vp, i64, vp, ci, vp, i64]
    L.mi355x_wq_matmul_static_ws.argtypes = [dp, vp, vp, vp, ep, vp, i64, vp, ci]
    L.mi355x_wq_static_ws_bytes.restype = i64
    L.mi355x_wq_check.argtypes = [dp, i64]
    L.mi355x_wq_select_kernel.argtypes = [dp, i64]
    L.mi355x_wq_last_error.restype = C.c_char_p
    L.mi355x_wq_packed_set_stream.argtypes = [vp]
    L.mi355x_wq_packed_get_stream.restype = vp
    L.mi355x_wq_register_tvm_globals.argtypes = [ci]
    for name in PACKED_ENTRIES:
        getattr(L, name).argtypes = [vp, C.POINTER(ci), ci, vp, C.POINTER(ci), vp]
    L.mi355x_wq_packed_call.argtypes = [vp, vp, C.POINTER(ci), ci]
    L.mi355x_wq_packed_call_scratch.argtypes = [vp, vp, C.POINTER(ci), ci]
    i32 = C.c_int32
    L.mi355x_wq_module_type_key.restype = C.c_char_p
    L.mi355x_wq_module_create.argtypes = [C.c_char_p, vp, C.POINTER(C.c_char_p), C.POINTER(i32), i32, i32, C.POINTER(vp)]
    L.mi355x_wq_module_destroy.argtypes = [vp]
    L.mi355x_wq_module_destroy.restype = None
    for name in ("symbol", "json"):
        getattr(L, "mi355x_wq_module_" + name).argtypes = [vp]
        getattr(L, "mi355x_wq_module_" + name).restype = C.c_char_p
    L.mi355x_wq_module_const_name.argtypes = [vp, i32]
    L.mi355x_wq_module_const_name.restype = C.c_char_p
    L.mi355x_wq_module_num_consts.argtypes = [vp]
    L.mi355x_wq_module_initialized.argtypes = [vp]
    L.mi355x_wq_module_get_function.argtypes = [vp, C.c_char_p, C.POINTER(vp), C.POINTER(vp)]
    L.mi355x_wq_module_init.argtypes = [vp, C.POINTER(vp), i32]
    L.mi355x_wq_module_call.argtypes = [vp, vp, C.POINTER(ci), ci]
    L.mi355x_wq_module_save_to_binary.argtypes = [vp, vp, i64]
    L.mi355x_wq_module_save_to_binary.restype = i64
    L.mi355x_wq_module_load_from_binary.argtypes = [vp, i64, C.POINTER(i64), C.POINTER(vp)]
    L.mi355x_wq_module_create_from_json.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(C.c_char_p), i32, C.POINTER(vp)]
    L.mi355x_wq_module_set_workspace_rows.argtypes = [vp, i32]
    _lib = L
    return L


def last_error() -> str:
    # a message may quote bytes of a damaged module file, which need not be UTF-8
    return load().mi355x_wq_last_error().decode(errors="backslashreplace")


def make_desc(bits: int, group: int, n: int, k: int, zero_point: int | None = None) -> WqDesc:
    if zero_point is None:
        zero_point = 7 if bits == 4 else 0
    return WqDesc(bits, group, zero_point, 0, n, k)


def check(rc: int) -> None:
    if rc != 0:
        raise WqError(last_error())
