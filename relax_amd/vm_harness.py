"""A minimal stand-in for the caller side of the boundary: what Relax's VM does
around one external call, so the PackedFunc entries can be exercised without TVM.

It reproduces, for tensors only,
  * `VirtualMachineImpl::RunInstrCall` packing registers into `TVMValue[]` +
    type-code arrays (src/runtime/relax_vm/vm.cc:727-778): every tensor goes in as
    kTVMNDArrayHandle (13) whose handle is a `DLTensor*`
    (include/tvm/runtime/ndarray.h:430-436);
  * `WrapPackedFunc` calling the C symbol with six arguments and turning a
    non-zero return into an error carrying the callee's message
    (src/runtime/library_module.cc:74-88);
  * `CallTIRMutator`'s destination-passing convention: the caller allocates the
    output and appends it after the inputs (src/relax/transform/call_tir_rewrite.cc:43-120).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import lib as _lib

K_TVM_NULLPTR = 4
K_TVM_DLTENSOR_HANDLE = 7
K_TVM_NDARRAY_HANDLE = 13
K_DL_ROCM = 10


class DLDevice(C.Structure):
    _fields_ = [("device_type", C.c_int32), ("device_id", C.c_int32)]


class DLDataType(C.Structure):
    _fields_ = [("code", C.c_uint8), ("bits", C.c_uint8), ("lanes", C.c_uint16)]


class DLTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("device", DLDevice), ("ndim", C.c_int32),
                ("dtype", DLDataType), ("shape", C.POINTER(C.c_int64)),
                ("strides", C.POINTER(C.c_int64)), ("byte_offset", C.c_uint64)]


class TVMValue(C.Union):
    _fields_ = [("v_int64", C.c_int64), ("v_float64", C.c_double), ("v_handle", C.c_void_p),
                ("v_str", C.c_char_p), ("v_type", DLDataType), ("v_device", DLDevice)]


class CallSpec(C.Structure):
    """mi355x_wq_callspec; the fused-operand roles default to "absent" (-1)."""
    _fields_ = [(n, C.c_int32) for n in ("op", "bits", "group", "zero_point", "arg_x", "arg_wq",
                                         "arg_scales", "arg_out", "num_args", "arg_bias",
                                         "arg_residual", "activation")]

    def __init__(self, *args, **kw):
        if len(args) < 10:
            kw.setdefault("arg_bias", -1)
        if len(args) < 11:
            kw.setdefault("arg_residual", -1)
        super().__init__(*args, **kw)


_DTYPES = {
    torch.float16: (2, 16), torch.float32: (2, 32), torch.int32: (0, 32), torch.int8: (0, 8),
    torch.uint8: (1, 8), torch.int64: (0, 64),
}
if hasattr(torch, "uint32"):
    _DTYPES[torch.uint32] = (1, 32)


class TensorArg:
    """Owns the DLTensor struct (and its shape/strides arrays) describing a torch tensor."""

    def __init__(self, t: torch.Tensor, *, as_uint32: bool = False, with_strides: bool = False,
                 byte_offset: int = 0, device_type: int | None = None):
        self.tensor = t  # keep the memory alive
        code, bits = _DTYPES[t.dtype]
        if as_uint32:
            if t.dtype not in (torch.int32, getattr(torch, "uint32", torch.int32)):
                raise TypeError("as_uint32 needs 32-bit integer storage")
            code, bits = 1, 32
        self._shape = (C.c_int64 * t.dim())(*t.shape)
        self._strides = (C.c_int64 * t.dim())(*t.stride()) if with_strides else None
        dev_type = device_type if device_type is not None else (K_DL_ROCM if t.is_cuda else 1)
        dev_id = t.device.index if t.is_cuda and t.device.index is not None else 0
        self.dl = DLTensor(
            C.c_void_p(t.data_ptr() - byte_offset), DLDevice(dev_type, dev_id), t.dim(),
            DLDataType(code, bits, 1), self._shape,
            self._strides if with_strides else C.POINTER(C.c_int64)(), byte_offset)

    @property
    def handle(self) -> int:
        return C.addressof(self.dl)


class PackedError(RuntimeError):
    """The callee returned non-zero; the text is what TVM would put into its TVMError."""


def call_packed(symbol, args, *, type_code: int = K_TVM_NDARRAY_HANDLE, spec: CallSpec | None = None):
    """Invoke an exported entry (by name) or the generic entry with `spec`, VM style."""
    L = _lib.load()
    n = len(args)
    values = (TVMValue * max(n, 1))()
    codes = (C.c_int * max(n, 1))()
    for i, a in enumerate(args):
        if isinstance(a, TensorArg):
            values[i].v_handle = a.handle
            codes[i] = type_code
        elif a is None:
            values[i].v_handle = None
            codes[i] = K_TVM_NULLPTR
        else:  # plain integers travel as kDLInt (0)
            values[i].v_int64 = int(a)
            codes[i] = 0
    if spec is not None:
        # the body generated entries forward to: mi355x_wq_packed_call, or its _scratch twin by name
        forward = L.mi355x_wq_packed_call_scratch if symbol == "mi355x_wq_packed_call_scratch" else L.mi355x_wq_packed_call
        rc = forward(C.addressof(spec), C.addressof(values), codes, n)
    else:
        fn = getattr(L, symbol)
        ret_value = TVMValue()
        ret_code = C.c_int(K_TVM_NULLPTR)
        rc = fn(C.addressof(values), codes, n, C.addressof(ret_value), C.byref(ret_code), None)
        if rc == 0 and ret_code.value != K_TVM_NULLPTR:
            raise PackedError(f"{symbol} set a return value (type code {ret_code.value}); "
                              "DPS externs return nothing")
    if rc != 0:
        raise PackedError(_lib.last_error())


def set_stream(stream=None) -> None:
    """Make the packed entries launch on `stream` (default: torch's current stream)."""
    s = stream if stream is not None else torch.cuda.current_stream()
    _lib.load().mi355x_wq_packed_set_stream(int(s.cuda_stream))


def call_dps(symbol: str, inputs, out_shape, out_dtype=torch.float16, **tensor_kw):
    """`call_tir(ExternFunc(symbol), inputs, out_sinfo)` after CallTIRRewrite: allocate, append, call."""
    dev = inputs[0].device
    out = torch.empty(out_shape, dtype=out_dtype, device=dev)
    targs = [TensorArg(t, as_uint32=(t.dtype == torch.int32), **tensor_kw) for t in inputs]
    targs.append(TensorArg(out))
    call_packed(symbol, targs)
    return out
