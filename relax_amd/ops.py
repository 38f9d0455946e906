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
              activation: str | None = None, residual: torch.Tensor | None = None) -> torch.Tensor:
    """y[M,N] = f16(x[M,K] @ dequant(wq, scales)^T) on the current HIP device (asynchronous).

    Optional fused epilogue, each step one float16 operation: ``+ bias[N]``, then ``activation``
    ("relu"), then ``+ residual[M,N]`` (``residual`` may be ``out`` itself)."""
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
    if out is None:
        out = torch.empty((m, n), dtype=torch.float16, device=x.device)
    elif tuple(out.shape) != (m, n) or out.dtype != torch.float16 or not out.is_contiguous():
        raise ValueError("out must be a compact float16 [M, N] tensor")
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
