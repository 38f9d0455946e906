"""ctypes front end of oracle/wq_oracle.c (test infrastructure only)."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libwq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "wq_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libwq_oracle.so"])
    return _SO


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        p = C.c_void_p
        i64 = C.c_int64
        L.wq_oracle_f16_to_f32.restype = C.c_float
        L.wq_oracle_f16_to_f32.argtypes = [C.c_uint16]
        L.wq_oracle_f32_to_f16.restype = C.c_uint16
        L.wq_oracle_f32_to_f16.argtypes = [C.c_float]
        L.wq_oracle_unpack_q4.argtypes = [p, i64, i64, p]
        L.wq_oracle_unpack_q8.argtypes = [p, i64, i64, p]
        L.wq_oracle_dequant.argtypes = [C.c_int, i64, p, p, i64, i64, p, C.c_int]
        L.wq_oracle_matmul_f32acc.argtypes = [p, p, i64, i64, i64, p, C.c_int]
        L.wq_oracle_cast_f16.argtypes = [p, i64, p]
        L.wq_oracle_wq_matmul.argtypes = [C.c_int, i64, p, p, p, i64, i64, i64, p, p, p, C.c_int]
        L.wq_oracle_epilogue.argtypes = [p, i64, i64, p, C.c_int, p]
        L.wq_oracle_epilogue.restype = None
        L.wq_oracle_silu_mul.argtypes = [p, i64, i64, p]
        L.wq_oracle_silu_mul.restype = None
        _lib = L
    return _lib


def _ptr(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def f16_to_f32_all() -> np.ndarray:
    L = lib()
    return np.array([L.wq_oracle_f16_to_f32(h) for h in range(65536)], dtype=np.float32)


def f32_to_f16(values: np.ndarray) -> np.ndarray:
    L = lib()
    v = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(v.shape, dtype=np.uint16)
    L.wq_oracle_cast_f16(_ptr(v), v.size, _ptr(out))
    return out.view(np.float16)


def unpack(wq: np.ndarray, bits: int) -> np.ndarray:
    L = lib()
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    n, kw = wq.shape
    k = kw * (32 // bits)
    if bits == 4:
        out = np.empty((n, k), dtype=np.uint8)
        L.wq_oracle_unpack_q4(_ptr(wq), n, k, _ptr(out))
    else:
        out = np.empty((n, k), dtype=np.int8)
        L.wq_oracle_unpack_q8(_ptr(wq), n, k, _ptr(out))
    return out


def dequant(wq, s, bits: int, group: int, nthreads: int = 1) -> np.ndarray:
    L = lib()
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    s = np.ascontiguousarray(s, dtype=np.float16)
    n, kw = wq.shape
    k = kw * (32 // bits)
    wd = np.empty((n, k), dtype=np.float16)
    rc = L.wq_oracle_dequant(bits, group, _ptr(wq), _ptr(s), n, k, _ptr(wd), nthreads)
    if rc != 0:
        raise ValueError("wq_oracle_dequant rejected the arguments")
    return wd


def matmul_f32acc(x, wd, nthreads: int = 1) -> np.ndarray:
    L = lib()
    x = np.ascontiguousarray(x, dtype=np.float16)
    wd = np.ascontiguousarray(wd, dtype=np.float16)
    m, k = x.shape
    n = wd.shape[0]
    y32 = np.empty((m, n), dtype=np.float32)
    L.wq_oracle_matmul_f32acc(_ptr(x), _ptr(wd), m, n, k, _ptr(y32), nthreads)
    return y32


def wq_matmul(x, wq, s, bits: int, group: int, nthreads: int = 1) -> np.ndarray:
    L = lib()
    x = np.ascontiguousarray(x, dtype=np.float16)
    wq = np.ascontiguousarray(wq, dtype=np.uint32)
    s = np.ascontiguousarray(s, dtype=np.float16)
    m, k = x.shape
    n = wq.shape[0]
    wd = np.empty((n, k), dtype=np.float16)
    y32 = np.empty((m, n), dtype=np.float32)
    y = np.empty((m, n), dtype=np.float16)
    rc = L.wq_oracle_wq_matmul(bits, group, _ptr(x), _ptr(wq), _ptr(s), m, n, k,
                               _ptr(wd), _ptr(y32), _ptr(y), nthreads)
    if rc != 0:
        raise ValueError("wq_oracle_wq_matmul rejected the arguments")
    return y


def epilogue(y, bias=None, activation=None, residual=None) -> np.ndarray:
    """Fused tail on a copy of y [M,N] float16: + bias[N], relu or gelu, + residual[M,N]."""
    L = lib()
    if activation == "silu_mul":
        if bias is not None or residual is not None:
            raise ValueError("the gated tail takes no bias or residual")
        src = np.ascontiguousarray(y, dtype=np.float16)
        m, n = src.shape
        if n % 2 != 0:
            raise ValueError("the gated tail needs an even number of output columns")
        gated = np.empty((m, n // 2), dtype=np.float16)
        L.wq_oracle_silu_mul(_ptr(src), m, n, _ptr(gated))
        return gated
    out = np.array(y, dtype=np.float16, order="C", copy=True)
    m, n = out.shape
    if activation not in (None, "none", "relu", "relax.nn.relu", "gelu", "relax.nn.gelu"):
        raise ValueError(f"unsupported activation {activation!r}")
    b = None if bias is None else np.ascontiguousarray(np.asarray(bias, dtype=np.float16).reshape(-1))
    r = None if residual is None else np.ascontiguousarray(residual, dtype=np.float16)
    if b is not None and b.shape != (n,):
        raise ValueError("bias must have N elements")
    if r is not None and r.shape != (m, n):
        raise ValueError("residual must be [M, N]")
    L.wq_oracle_epilogue(_ptr(out), m, n, None if b is None else _ptr(b),
                         {"relu": 1, "relax.nn.relu": 1, "gelu": 3, "relax.nn.gelu": 3}.get(activation, 0),
                         None if r is None else _ptr(r))
    return out


def wq_matmul_fused(x, wq, s, bits: int, group: int, bias=None, activation=None, residual=None,
                    nthreads: int = 1) -> np.ndarray:
    return epilogue(wq_matmul(x, wq, s, bits, group, nthreads=nthreads), bias, activation, residual)


def max_threads() -> int:
    return int(lib().wq_oracle_max_threads())
