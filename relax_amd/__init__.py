"""MI355X-native weight-only-quantized dequantize + matmul behind Relax's BYOC boundary.

The compute path is the in-tree HIP library `relax_amd/csrc/libmi355x_wq.so`
(C ABI in `include/mi355x_wq.h`, TVM PackedFunc entries in
`include/mi355x_wq_packed.h`).  There is no CPU fallback: loading fails loudly
when the library has not been built.
"""
from . import lib  # noqa: F401
from .ops import (wq_dequantize, wq_matmul, wq_tile_weights, wq_untile_weights, wq_workspace,  # noqa: F401
                  wq_workspace_bytes)
from .quant import pack_q4, pack_q8, quantize_q4f16, quantize_q8f16  # noqa: F401

__all__ = ["lib", "wq_matmul", "wq_dequantize", "wq_tile_weights", "wq_untile_weights", "wq_workspace", "wq_workspace_bytes", "pack_q4", "pack_q8", "quantize_q4f16",
           "quantize_q8f16"]
