"""The runtime module of an offloaded subgraph and the machinery around it that makes a compiled
model survive `export_library` / `load_module`, without TVM in the process.

  * `SubgraphModule` wraps the library's module object (include/mi355x_wq_module.h), the
    counterpart of a JSON-runtime backend module (src/runtime/contrib/json/json_runtime.h:57-135):
    `get_function("<symbol>")`, `get_function("__init_<symbol>")`, `save_to_binary`, `load_from_binary`.
  * `ConstLoader` restates the const-loader module that wraps such modules
    (src/runtime/const_loader_module.cc:48-253): it holds the constants by name and the names each
    symbol needs, runs `__init_<symbol>` on the first lookup of a symbol and serialises its
    constants in `NDArray::Save`'s encoding (include/tvm/runtime/ndarray.h:447-496), always as host
    arrays.
  * `export_library` / `load_module` write and read the module blob of an exported library in the
    encoding `ProcessModuleBlob` parses (src/runtime/library_module.cc:136-199): a uint64 byte
    count, then a dmlc stream of (type key, payload) records and the `_import_tree` in CSR form.
    The blob is what the reference embeds in the shared object as `__tvm_dev_mblob`; here it is
    the whole file, because the kernels live in the prebuilt library rather than in generated code.

The round trip this enables is the one of tests/python/relax/test_transform_codegen_pass.py:57-65.
"""
from __future__ import annotations

import ctypes as C
import struct

import numpy as np
import torch

from . import lib as _lib
from .vm_harness import (K_TVM_NDARRAY_HANDLE, K_TVM_NULLPTR, CallSpec, PackedError, TensorArg, TVMValue)

TILE_WEIGHTS = 1
LIBRARY_SCRATCH = 2
OWN_WORKSPACE = 4
ND_ARRAY_MAGIC = 0xDD5E40F096B4A13F  # kTVMNDArrayMagic, include/tvm/runtime/ndarray.h:447
_PACKED_CFUNC = C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_void_p, C.c_void_p)


# ---- dmlc::Stream encoding (little endian; strings and vectors carry a uint64 count) -------------
class _Writer:
    def __init__(self):
        self.parts = []

    def u64(self, v):
        self.parts.append(struct.pack("<Q", v))

    def string(self, s):
        b = s.encode() if isinstance(s, str) else bytes(s)
        self.u64(len(b))
        self.parts.append(b)

    def strings(self, items):
        self.u64(len(items))
        for s in items:
            self.string(s)

    def u64s(self, items):
        self.u64(len(items))
        self.parts.append(struct.pack(f"<{len(items)}Q", *items))

    def raw(self, b):
        self.parts.append(bytes(b))

    def bytes(self):
        return b"".join(self.parts)


class _Reader:
    def __init__(self, data, pos=0):
        self.data, self.pos = data, pos

    def take(self, n):
        if n < 0 or self.pos + n > len(self.data):
            raise ValueError("module blob is truncated")
        out = self.data[self.pos:self.pos + n]
        self.pos += n
        return out

    def u64(self):
        return struct.unpack("<Q", self.take(8))[0]

    def string(self):
        return self.take(self.u64()).decode()

    def strings(self):
        return [self.string() for _ in range(self.u64())]

    def u64s(self):
        n = self.u64()
        return list(struct.unpack(f"<{n}Q", self.take(8 * n)))


_NP_CODES = {"i": 0, "u": 1, "f": 2}


def save_ndarray(w: _Writer, a: np.ndarray) -> None:
    """NDArray::Save: magic, reserved, a CPU device, ndim, dtype, shape, byte count, data."""
    a = np.ascontiguousarray(a)
    w.u64(ND_ARRAY_MAGIC)
    w.u64(0)
    w.raw(struct.pack("<iii", 1, 0, a.ndim))
    w.raw(struct.pack("<BBH", _NP_CODES[a.dtype.kind], a.dtype.itemsize * 8, 1))
    w.raw(struct.pack(f"<{a.ndim}q", *a.shape))
    w.u64(a.nbytes)
    w.raw(a.tobytes())


def load_ndarray(r: _Reader) -> np.ndarray:
    if r.u64() != ND_ARRAY_MAGIC:
        raise ValueError("Invalid DLTensor file format")
    r.u64()
    _dev_type, _dev_id, ndim = struct.unpack("<iii", r.take(12))
    code, bits, lanes = struct.unpack("<BBH", r.take(4))
    if not 0 <= ndim <= 8 or lanes != 1 or code not in (0, 1, 2) or bits not in (8, 16, 32, 64):
        raise ValueError("unsupported tensor header in module blob")
    shape = struct.unpack(f"<{ndim}q", r.take(8 * ndim))
    nbytes = r.u64()
    dtype = np.dtype({0: "i", 1: "u", 2: "f"}[code] + str(bits // 8))
    if nbytes != int(np.prod(shape, dtype=np.int64)) * dtype.itemsize:
        raise ValueError("Invalid DLTensor file format")
    return np.frombuffer(r.take(nbytes), dtype=dtype).reshape(shape).copy()


# ---- the backend module -----------------------------------------------------------------------
def _as_tensor_arg(t):
    if isinstance(t, TensorArg):
        return t
    if isinstance(t, np.ndarray):  # host constant, as the const loader holds it after a load
        if t.dtype in (np.uint32, np.int32):  # torch has no uint32 arithmetic: packed words travel as int32 storage
            return TensorArg(torch.from_numpy(t.view(np.int32)), as_uint32=True)
        return TensorArg(torch.from_numpy(t))
    return TensorArg(t, as_uint32=(t.dtype == torch.int32))


class SubgraphModule:
    """One composite function's runtime module (type key "mi355x_wq")."""

    def __init__(self, handle: int):
        self._h = C.c_void_p(handle)
        self._keep = []  # device constants borrowed by the module must outlive it

    @classmethod
    def create(cls, symbol: str, spec: CallSpec, const_names=(), const_args=(), flags: int = 0,
               workspace_rows: int = 0) -> "SubgraphModule":
        """`workspace_rows` (with OWN_WORKSPACE among the flags): init allocates the K split's workspace for calls
        of up to that many rows."""
        L = _lib.load()
        n = len(const_names)
        names = (C.c_char_p * max(n, 1))(*[s.encode() for s in const_names])
        slots = (C.c_int32 * max(n, 1))(*const_args)
        out = C.c_void_p()
        _lib.check(L.mi355x_wq_module_create(symbol.encode(), C.addressof(spec), names, slots, n, flags, C.byref(out)))
        mod = cls(out.value)
        if workspace_rows:
            _lib.check(L.mi355x_wq_module_set_workspace_rows(mod._h, workspace_rows))
        return mod

    @classmethod
    def load_from_binary(cls, data: bytes, pos: int = 0):
        """Returns (module, bytes consumed)."""
        L = _lib.load()
        buf = (C.c_char * max(len(data) - pos, 1)).from_buffer_copy(data[pos:] or b"\0")
        used, out = C.c_int64(), C.c_void_p()
        _lib.check(L.mi355x_wq_module_load_from_binary(C.addressof(buf), len(data) - pos, C.byref(used), C.byref(out)))
        return cls(out.value), used.value

    type_key = "mi355x_wq"

    def save_to_binary(self) -> bytes:
        L = _lib.load()
        n = L.mi355x_wq_module_save_to_binary(self._h, None, 0)
        if n < 0:
            raise _lib.WqError(_lib.last_error())
        buf = (C.c_char * n)()
        L.mi355x_wq_module_save_to_binary(self._h, C.addressof(buf), n)
        return bytes(buf)

    @property
    def symbol(self) -> str:
        return _lib.load().mi355x_wq_module_symbol(self._h).decode()

    @property
    def const_names(self):
        L = _lib.load()
        return [L.mi355x_wq_module_const_name(self._h, i).decode() for i in range(L.mi355x_wq_module_num_consts(self._h))]

    @property
    def json(self) -> str:
        return _lib.load().mi355x_wq_module_json(self._h).decode()

    @property
    def initialized(self) -> bool:
        return bool(_lib.load().mi355x_wq_module_initialized(self._h))

    def get_function(self, name: str):
        """`ModuleNode::GetFunction`: a callable taking tensors, or None for a name the module lacks."""
        L = _lib.load()
        fn, res = C.c_void_p(), C.c_void_p()
        _lib.check(L.mi355x_wq_module_get_function(self._h, name.encode(), C.byref(fn), C.byref(res)))
        if not fn.value:
            return None
        cfunc = _PACKED_CFUNC(fn.value)

        def packed(*tensors):
            targs = [_as_tensor_arg(t) for t in tensors]
            n = len(targs)
            values = (TVMValue * max(n, 1))()
            codes = (C.c_int * max(n, 1))()
            for i, a in enumerate(targs):
                values[i].v_handle = a.handle
                codes[i] = K_TVM_NDARRAY_HANDLE
            if cfunc(C.addressof(values), codes, n, None, res) != 0:
                raise PackedError(_lib.last_error())
            if name.startswith("__init_"):
                self._keep.extend(targs)
            return None
        return packed

    def close(self) -> None:
        if self._h:
            _lib.load().mi355x_wq_module_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class ConstLoader:
    """const_loader_module.cc: constants by name, required names by symbol, init on first lookup."""

    type_key = "const_loader"

    def __init__(self, const_var_ndarray: dict, const_vars_by_symbol: dict, imports=()):
        for sym, names in const_vars_by_symbol.items():
            for v in names:
                if v not in const_var_ndarray:
                    raise KeyError(f"ConstLoaderModuleNode is missing entry for constant '{v}' for function '{sym}'")
        self.const_var_ndarray = dict(const_var_ndarray)
        self.const_vars_by_symbol = {k: list(v) for k, v in const_vars_by_symbol.items()}
        self.initialized = {k: False for k in const_vars_by_symbol}
        self.imports = list(imports)

    def get_function(self, name: str):
        if name in self.initialized and not self.initialized[name]:
            self._init_submodule(name)
            self.initialized[name] = True
        for m in self.imports:
            f = m.get_function(name)
            if f is not None:
                return f
        return None

    def _init_submodule(self, symbol: str) -> None:
        for m in self.imports:
            init = m.get_function("__init_" + symbol)
            if init is not None:
                init(*[self.const_var_ndarray[v] for v in self.const_vars_by_symbol[symbol]])
                return

    def save_to_binary(self) -> bytes:
        w = _Writer()
        names = list(self.const_var_ndarray)
        w.strings(names)
        w.u64(len(names))
        for v in names:
            a = self.const_var_ndarray[v]
            if isinstance(a, torch.Tensor):  # saved as a host array whatever device it lives on
                a = a.cpu().numpy()
                if a.dtype == np.int32:  # packed words held in int32 storage are uint32 tensors
                    a = a.view(np.uint32)
            save_ndarray(w, a)
        symbols = list(self.const_vars_by_symbol)
        w.strings(symbols)
        w.u64(len(symbols))
        for s in symbols:
            w.strings(self.const_vars_by_symbol[s])
        return w.bytes()

    @classmethod
    def load_from_binary(cls, r: _Reader) -> "ConstLoader":
        names = r.strings()
        if r.u64() != len(names):
            raise ValueError("The number of variables and ndarray counts must match")
        arrays = [load_ndarray(r) for _ in names]
        symbols = r.strings()
        if r.u64() != len(symbols):
            raise ValueError("Loading number of symbols failed")
        by_symbol = {s: r.strings() for s in symbols}
        return cls(dict(zip(names, arrays)), by_symbol)


def export_library(root: ConstLoader) -> bytes:
    """The module blob of `root` and its imports (`_import_tree`: row pointers, child indices)."""
    mods = [root] + list(root.imports)
    w = _Writer()
    w.u64(len(mods) + 1)
    for m in mods:
        w.string(m.type_key)
        w.raw(m.save_to_binary())
    w.string("_import_tree")
    w.u64s([0, len(root.imports)] + [len(root.imports)] * len(root.imports))
    w.u64s(list(range(1, len(mods))))
    body = w.bytes()
    return struct.pack("<Q", len(body)) + body


def load_module(blob: bytes) -> ConstLoader:
    """`ProcessModuleBlob`: rebuild the modules, then the import relations; the first is the root."""
    r = _Reader(blob)
    nbytes = r.u64()
    if nbytes != len(blob) - 8:
        raise ValueError("module blob is truncated")
    mods, row_ptr, children = [], [], []
    for _ in range(r.u64()):
        tkey = r.string()
        if tkey == "_import_tree":
            row_ptr, children = r.u64s(), r.u64s()
        elif tkey == ConstLoader.type_key:
            mods.append(ConstLoader.load_from_binary(r))
        elif tkey == SubgraphModule.type_key:
            m, used = SubgraphModule.load_from_binary(blob, r.pos)
            r.take(used)
            mods.append(m)
        else:
            raise ValueError(f"Binary was created using {{{tkey}}} but a loader of that name is not registered")
    if not mods or len(row_ptr) != len(mods) + 1:
        raise ValueError("modules cannot be empty when import tree is present")
    for i, m in enumerate(mods):
        for j in range(row_ptr[i], row_ptr[i + 1]):
            if children[j] >= len(mods) or not isinstance(m, ConstLoader):
                raise ValueError("malformed import tree")
            m.imports.append(mods[children[j]])
    return mods[0]
