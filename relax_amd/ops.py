"""Torch-tensor front end of the C ABI.  Torch is used for device memory and streams only."""
from __future__ import annotations

import torch

from . import lib as _lib


def _stream_ptr(stream=None) -> int:
    s = stream if stream is not None else torch.cuda.current_stream()
    return int(s.cuda_stream)


def _as_u32_storage(wq: torch.Tensor) -> torch.Tensor:
    # torch has no arithmetic on uint32; int32 storage with the same bits is accepted
    if wq.dtype not in (torch.int32, torch.uint32):
        raise TypeError(f"wq must be int32/uint32 storage of packed words, got {wq.dtype}")
    return wq


def wq_matmul(x: torch.Tensor, wq: torch.Tensor, scales: torch.Tensor, bits: int, group: int,
              zero_point: int | None = None, out: torch.Tensor | None = None, kernel: int = 0,
              variant: int = 0, stream=None, bias: torch.Tensor | None = None,
              activation: str | None = None, residual: torch.Tensor | None = None,
              tiled_n: int | None = None, workspace: torch.Tensor | None = None) -> torch.Tensor:
    """y[M,N] = f16(x[M,K] @ dequant(wq, scales)^T) on the current HIP device (asynchronous).

    Optional fused epilogue, each step one float16 operation: ``+ bias[N]``, then ``activation``
    ("relu" or "gelu"), then ``+ residual[M,N]`` (``residual`` may be ``out`` itself); or ``activation="silu_mul"``
    alone: the output is ``[M, N/2] = multiply(nn.silu(y[:, :N/2]), y[:, N/2:])``.

    ``tiled_n=N``: ``wq`` and ``scales`` are the tile-major buffers `wq_tile_weights` returns
    for an N-row matrix (their row count is N rounded up to 16).

    ``workspace``: a device buffer from `wq_workspace` (zeroed once, then reusable by calls that do
    not overlap in time); lets the decode kernel split K across workgroups where that pays."""
    if workspace is not None:
        if kernel != 0 or variant != 0:
            raise ValueError("a workspace goes with the library's own kernel choice")
        return _wq_matmul_ws(x, wq, scales, bits, group, tiled_n, zero_point, out, stream, bias, activation,
                             residual, workspace)
    if tiled_n is not None:
        return _wq_matmul_tiled(x, wq, scales, bits, group, tiled_n, zero_point, out, stream, bias,
                                activation, residual, kernel | (variant << 8))
    L = _lib.load()
    wq = _as_u32_storage(wq)
    if not (x.is_cuda and wq.is_cuda and scales.is_cuda):
        raise ValueError("x, wq and scales must be device tensors")
    if x.dtype != torch.float16 or scales.dtype != torch.float16:
        raise TypeError("x and scales must be float16")
    if not (x.is_contiguous() and wq.is_contiguous() and scales.is_contiguous()):
        raise ValueError("x, wq and scales must be compact row-major")
    m, k = x.shape
    n = wq.shape[0]
    if wq.shape[1] * (32 // bits) != k:
        raise ValueError(f"wq has {wq.shape[1]} words per row, expected {k * bits // 32} for K={k}")
    if tuple(scales.shape) != (n, k // group):
        raise ValueError(f"scales has shape {tuple(scales.shape)}, expected {(n, k // group)}")
    # the gated tail ("silu_mul": multiply(nn.silu(gate), up) on the two halves of a gate+up projection) halves the output
    out_cols = n // 2 if activation == "silu_mul" else n
    if out is None:
        out = torch.empty((m, out_cols), dtype=torch.float16, device=x.device)
    elif tuple(out.shape) != (m, out_cols) or out.dtype != torch.float16 or not out.is_contiguous():
        raise ValueError(f"out must be a compact float16 [{m}, {out_cols}] tensor")
    desc = _lib.make_desc(bits, group, n, k, zero_point)
    if bias is None and residual is None and activation is None:
        rc = L.mi355x_wq_matmul_ex(desc, x.data_ptr(), wq.data_ptr(), scales.data_ptr(), out.data_ptr(),
                                   m, _stream_ptr(stream), kernel | (variant << 8))
        _lib.check(rc)
        return out
    if activation not in _lib.ACTIVATIONS:
        raise ValueError(f"unsupported activation {activation!r}")
    if bias is not None:
        if not bias.is_cuda or bias.dtype != torch.float16 or not bias.is_contiguous() or \
                tuple(bias.shape) not in ((n,), (1, n)):
            raise ValueError(f"bias must be a compact float16 device tensor of shape ({n},) or (1, {n})")
    if residual is not None:
        if not residual.is_cuda or residual.dtype != torch.float16 or not residual.is_contiguous() or \
                tuple(residual.shape) != (m, n):
            raise ValueError(f"residual must be a compact float16 device tensor of shape ({m}, {n})")
    ep = _lib.WqEpilogue(bias.data_ptr() if bias is not None else None,
                         residual.data_ptr() if residual is not None else None,
                         _lib.ACTIVATIONS[activation], 0)
    rc = L.mi355x_wq_matmul_fused_ex(desc, x.data_ptr(), wq.data_ptr(), scales.data_ptr(), ep,
                                     out.data_ptr(), m, _stream_ptr(stream), kernel | (variant << 8))
    _lib.check(rc)
    return out


def _tiled_sizes(L, desc):
    import ctypes as C

    wb, sb = C.c_int64(0), C.c_int64(0)
    _lib.check(L.mi355x_wq_tiled_sizes(desc, C.byref(wb), C.byref(sb)))
    return wb.value, sb.value


def wq_tile_weights(wq: torch.Tensor, scales: torch.Tensor, bits: int, group: int,
                    stream=None) -> tuple[torch.Tensor, torch.Tensor]:
    """Canonical (wq[N, K*bits/32], scales[N, K/group]) -> the tile-major buffers of
    `mi355x_wq_tile_weights`, as tensors of the canonical shapes with N rounded up to 16 rows (their
    bytes are in tile-major order, not row-major).  A one-off, done when weights are loaded."""
    L = _lib.load()
    wq = _as_u32_storage(wq)
    if not (wq.is_cuda and scales.is_cuda and wq.is_contiguous() and scales.is_contiguous()):
        raise ValueError("wq and scales must be compact device tensors")
    n, k = wq.shape[0], wq.shape[1] * (32 // bits)
    if scales.dtype != torch.float16 or tuple(scales.shape) != (n, k // group):
        raise ValueError(f"scales must be float16 of shape {(n, k // group)}")
    desc = _lib.make_desc(bits, group, n, k)
    wb, sb = _tiled_sizes(L, desc)
    rows = (n + 15) // 16 * 16  # whole tiles; same row length as the canonical tensors
    wq_t = torch.empty((rows, wq.shape[1]), dtype=torch.int32, device=wq.device)
    s_t = torch.empty((rows, scales.shape[1]), dtype=torch.float16, device=wq.device)
    assert wq_t.numel() * 4 == wb and s_t.numel() * 2 == sb
    _lib.check(L.mi355x_wq_tile_weights(desc, wq.data_ptr(), scales.data_ptr(), wq_t.data_ptr(), s_t.data_ptr(),
                                        _stream_ptr(stream)))
    return wq_t, s_t


def wq_untile_weights(wq_tiled: torch.Tensor, scales_tiled: torch.Tensor, bits: int, group: int, n: int, k: int,
                      stream=None) -> tuple[torch.Tensor, torch.Tensor]:
    """The inverse of `wq_tile_weights`: back to the canonical interchange layout."""
    L = _lib.load()
    desc = _lib.make_desc(bits, group, n, k)
    wb, sb = _tiled_sizes(L, desc)
    if wq_tiled.numel() * wq_tiled.element_size() != wb or scales_tiled.numel() * scales_tiled.element_size() != sb:
        raise ValueError(f"tile-major buffers must hold {wb} and {sb} bytes")
    wq = torch.empty((n, k * bits // 32), dtype=torch.int32, device=wq_tiled.device)
    s = torch.empty((n, k // group), dtype=torch.float16, device=wq_tiled.device)
    _lib.check(L.mi355x_wq_untile_weights(desc, wq_tiled.data_ptr(), scales_tiled.data_ptr(), wq.data_ptr(),
                                          s.data_ptr(), _stream_ptr(stream)))
    return wq, s


def _wq_matmul_tiled(x, wq_t, s_t, bits, group, n, zero_point, out, stream, bias, activation, residual,
                     kernel=0):
    L = _lib.load()
    if not (x.is_cuda and wq_t.is_cuda and s_t.is_cuda):
        raise ValueError("x, wq and scales must be device tensors")
    if x.dtype != torch.float16 or s_t.dtype != torch.float16 or not x.is_contiguous():
        raise TypeError("x and scales must be float16, x compact")
    m, k = x.shape
    desc = _lib.make_desc(bits, group, n, k, zero_point)
    wb, sb = _tiled_sizes(L, desc)
    if wq_t.numel() * wq_t.element_size() != wb or s_t.numel() * s_t.element_size() != sb:
        raise ValueError(f"tile-major buffers must hold {wb} and {sb} bytes for N={n}, K={k}")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    elif tuple(out.shape) != (m, n) or out.dtype != torch.float16 or not out.is_contiguous():
        raise ValueError("out must be a compact float16 [M, N] tensor")
    if activation not in _lib.ACTIVATIONS:
        raise ValueError(f"unsupported activation {activation!r}")
    ep = _lib.WqEpilogue(bias.data_ptr() if bias is not None else None,
                         residual.data_ptr() if residual is not None else None,
                         _lib.ACTIVATIONS[activation], 0)
    _lib.check(L.mi355x_wq_matmul_tiled_ex(desc, x.data_ptr(), wq_t.data_ptr(), s_t.data_ptr(), ep, out.data_ptr(),
                                           m, _stream_ptr(stream), kernel))
    return out


def wq_workspace_bytes(bits: int, group: int, n: int, k: int, m: int, tiled: bool = False,
                       zero_point: int | None = None) -> int:
    """Bytes of workspace `wq_matmul(..., workspace=)` needs to split K for this problem; 0 = it would not."""
    L = _lib.load()
    nbytes = L.mi355x_wq_workspace_bytes(_lib.make_desc(bits, group, n, k, zero_point), m, 1 if tiled else 0)
    if nbytes < 0:
        raise _lib.WqError(_lib.last_error())
    return int(nbytes)


def wq_workspace(nbytes: int, device="cuda") -> torch.Tensor | None:
    """A zeroed workspace of `nbytes` (None for 0).  Size it for the largest problem that will use it."""
    return torch.zeros(nbytes, dtype=torch.uint8, device=device) if nbytes > 0 else None


def _wq_matmul_ws(x, wq, scales, bits, group, tiled_n, zero_point, out, stream, bias, activation, residual, workspace):
    L = _lib.load()
    if not (x.is_cuda and wq.is_cuda and scales.is_cuda and workspace.is_cuda):
        raise ValueError("x, wq, scales and workspace must be device tensors")
    if x.dtype != torch.float16 or scales.dtype != torch.float16 or not x.is_contiguous():
        raise TypeError("x and scales must be float16, x compact")
    if not (wq.is_contiguous() and scales.is_contiguous() and workspace.is_contiguous()):
        raise ValueError("wq, scales and workspace must be compact")
    m, k = x.shape
    n = tiled_n if tiled_n is not None else wq.shape[0]
    desc = _lib.make_desc(bits, group, n, k, zero_point)
    if tiled_n is not None:
        wb, sb = _tiled_sizes(L, desc)
        if wq.numel() * wq.element_size() != wb or scales.numel() * scales.element_size() != sb:
            raise ValueError(f"tile-major buffers must hold {wb} and {sb} bytes for N={n}, K={k}")
    elif wq.shape[1] * (32 // bits) != k or tuple(scales.shape) != (n, k // group):
        raise ValueError("wq / scales do not match x's K")
    out_cols = n // 2 if activation == "silu_mul" else n  # the gated tail halves the output
    if out is None:
        out = torch.empty((m, out_cols), dtype=torch.float16, device=x.device)
    elif tuple(out.shape) != (m, out_cols) or out.dtype != torch.float16 or not out.is_contiguous():
        raise ValueError(f"out must be a compact float16 [{m}, {out_cols}] tensor")
    if activation not in _lib.ACTIVATIONS:
        raise ValueError(f"unsupported activation {activation!r}")
    ep = _lib.WqEpilogue(bias.data_ptr() if bias is not None else None,
                         residual.data_ptr() if residual is not None else None,
                         _lib.ACTIVATIONS[activation], 0)
    _lib.check(L.mi355x_wq_matmul_ws(desc, x.data_ptr(), wq.data_ptr(), scales.data_ptr(), ep, out.data_ptr(), m,
                                     _stream_ptr(stream), 1 if tiled_n is not None else 0, workspace.data_ptr(),
                                     workspace.numel() * workspace.element_size()))
    return out


def wq_dequantize(wq: torch.Tensor, scales: torch.Tensor, bits: int, group: int,
                  zero_point: int | None = None, out: torch.Tensor | None = None,
                  stream=None) -> torch.Tensor:
    """wd[N,K] float16, bit-exact with the CPU path's `decode`."""
    L = _lib.load()
    wq = _as_u32_storage(wq)
    if not (wq.is_cuda and scales.is_cuda):
        raise ValueError("wq and scales must be device tensors")
    if not (wq.is_contiguous() and scales.is_contiguous()):
        raise ValueError("wq and scales must be compact row-major")
    n = wq.shape[0]
    k = wq.shape[1] * (32 // bits)
    if scales.dtype != torch.float16 or tuple(scales.shape) != (n, k // group):
        raise ValueError(f"scales must be float16 of shape {(n, k // group)}")
    if out is None:
        out = torch.empty((n, k), dtype=torch.float16, device=wq.device)
    desc = _lib.make_desc(bits, group, n, k, zero_point)
    rc = L.mi355x_wq_dequantize(desc, wq.data_ptr(), scales.data_ptr(), out.data_ptr(),
                                _stream_ptr(stream))
    _lib.check(rc)
    return out
