"""CPU tests of the subgraph runtime module and of what carries it through export / load: creation
and its argument checks, the binary encodings (against bytes assembled by hand from the formats the
reference documents in code), rejection of damaged input, and the const loader's bookkeeping.
Nothing here computes: no GPU is touched."""
import struct

import numpy as np
import pytest

from relax_amd import lib, module as M
from relax_amd.vm_harness import CallSpec, PackedError


def spec_matmul(bits=4, order=("wq", "scales", "x", "out"), **kw):
    slots = {r: i for i, r in enumerate(order)}
    return CallSpec(op=0, bits=bits, group=0, zero_point=7 if bits == 4 else 0, arg_x=slots["x"], arg_wq=slots["wq"],
                    arg_scales=slots["scales"], arg_out=slots["out"], num_args=len(order),
                    arg_bias=slots.get("bias", -1), arg_residual=slots.get("residual", -1), **kw)


def dmlc_string(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def test_create_and_accessors():
    m = M.SubgraphModule.create("fused_decode_matmul_mi355x0", spec_matmul(), ["param_0", "param_1"], [0, 1])
    assert m.symbol == "fused_decode_matmul_mi355x0" and m.const_names == ["param_0", "param_1"]
    assert not m.initialized
    assert m.get_function("get_symbol") is None and m.get_function("__init_other") is None
    assert m.get_function(m.symbol) is not None and m.get_function("__init_" + m.symbol) is not None
    assert lib.load().mi355x_wq_module_type_key() == b"mi355x_wq"
    # a module without constants has nothing to wait for
    assert M.SubgraphModule.create("s", spec_matmul()).initialized


def test_call_before_init_reports_the_reference_message():
    """json_runtime.h:82: ICHECK(initialized_) << "The module has not been initialized"."""
    m = M.SubgraphModule.create("sym", spec_matmul(), ["a", "b"], [0, 1])
    with pytest.raises(PackedError, match="sym: The module has not been initialized"):
        m.get_function("sym")()


@pytest.mark.parametrize("kwargs, message", [
    (dict(const_names=["a"], const_args=[2]), "not the slot of wq, scales or bias"),          # x
    (dict(const_names=["a"], const_args=[3]), "not the slot of wq, scales or bias"),          # the output
    (dict(const_names=["a", "b"], const_args=[0, 0]), "bound by two constants"),
    (dict(const_names=["a"], const_args=[7]), "not the slot"),
    (dict(const_names=["a"], const_args=[0], flags=M.TILE_WEIGHTS), "wq and scales are both constants"),
    (dict(const_names=["a", "b"], const_args=[0, 1], flags=8), "unknown flags"),
    (dict(const_names=["a"], const_args=[0], flags=M.OWN_WORKSPACE), "needs a matmul whose wq and scales are both constants"),
    (dict(const_names=["a", "b"], const_args=[0, 1], flags=M.TILE_WEIGHTS, workspace_rows=8), "go with MI355X_WQ_MODULE_OWN_WORKSPACE"),
    (dict(const_names=["a", "b"], const_args=[0, 1], flags=M.OWN_WORKSPACE, workspace_rows=-1), "workspace rows must be between"),
    (dict(const_names=["a", "b"], const_args=[0, 1], flags=M.OWN_WORKSPACE, workspace_rows=(1 << 20) + 1), "workspace rows must be between"),
    (dict(const_names=["a", ""], const_args=[0, 1]), "has no name"),
])
def test_create_rejects(kwargs, message):
    with pytest.raises(lib.WqError, match=message):
        M.SubgraphModule.create("sym", spec_matmul(), **kwargs)


def test_create_rejects_bad_specs():
    bad = spec_matmul()
    bad.bits = 5
    with pytest.raises(lib.WqError, match="bits must be 4 or 8"):
        M.SubgraphModule.create("sym", bad)
    bad = spec_matmul()
    bad.num_args = 5
    with pytest.raises(lib.WqError, match="has 4 arguments, the spec says 5"):
        M.SubgraphModule.create("sym", bad)
    with pytest.raises(lib.WqError, match="empty symbol"):
        M.SubgraphModule.create("", spec_matmul())
    res = spec_matmul(order=("wq", "scales", "x", "residual", "out"))
    with pytest.raises(lib.WqError, match="not the slot of wq, scales or bias"):
        M.SubgraphModule.create("sym", res, ["r"], [3])  # the residual is an activation, never a constant


def test_binary_form_is_the_documented_stream_encoding():
    """SaveToBinary writes symbol, graph JSON, constant names (json_runtime.h:105-116) with dmlc's
    uint64-length strings; the expected bytes are put together here without the library."""
    spec = spec_matmul(bits=8, order=("x", "wq", "scales", "bias", "out"), activation=1)
    m = M.SubgraphModule.create("f0", spec, ["w", "s", "b"], [1, 2, 3], M.TILE_WEIGHTS)
    json = ('{"version": 1, "op": "matmul", "bits": 8, "group": 0, "zero_point": 0, "num_args": 5, "arg_x": 0, '
            '"arg_wq": 1, "arg_scales": 2, "arg_out": 4, "arg_bias": 3, "arg_residual": -1, "activation": 1, '
            '"flags": 1, "workspace_rows": 0, "const_args": [1, 2, 3]}')
    assert m.json == json
    expect = dmlc_string("f0") + dmlc_string(json) + struct.pack("<Q", 3) + dmlc_string("w") + dmlc_string("s") + dmlc_string("b")
    assert m.save_to_binary() == expect
    back, used = M.SubgraphModule.load_from_binary(expect + b"trailing bytes of the next module")
    assert used == len(expect)
    assert (back.symbol, back.const_names, back.json, back.initialized) == ("f0", ["w", "s", "b"], json, False)
    assert back.save_to_binary() == expect
    # the rows a module's own workspace is sized for travel with it (a description without the key: none)
    ws = M.SubgraphModule.create("f1", spec_matmul(), ["w", "s"], [0, 1], M.TILE_WEIGHTS | M.OWN_WORKSPACE, workspace_rows=256)
    assert '"flags": 5, "workspace_rows": 256,' in ws.json
    ws_back, _ = M.SubgraphModule.load_from_binary(ws.save_to_binary())
    assert ws_back.json == ws.json and ws_back.save_to_binary() == ws.save_to_binary()
    # JSON written by another producer: other key order and white space
    other = '{ "const_args":[1,2,3],"flags":1,"activation":1,"arg_residual":-1,"arg_bias":3,"arg_out":4,\n"arg_scales":2,' \
            '"arg_wq":1,"arg_x":0,"num_args":5,"zero_point":0,"group":0,"bits":8,"op":"matmul","version":1 }'
    again, _ = M.SubgraphModule.load_from_binary(dmlc_string("f0") + dmlc_string(other) + expect[len(dmlc_string("f0") + dmlc_string(json)):])
    assert again.json == json


def test_damaged_binaries_are_refused():
    m = M.SubgraphModule.create("f0", spec_matmul(), ["w", "s"], [0, 1])
    good = m.save_to_binary()
    for cut in range(len(good)):
        with pytest.raises(lib.WqError, match="Loading|call description"):
            M.SubgraphModule.load_from_binary(good[:cut])
    head = dmlc_string("f0")
    tail = struct.pack("<Q", 2) + dmlc_string("w") + dmlc_string("s")
    for bad_json in ['{"version": 2, "op": "matmul", "const_args": []}', '{"version": 1, "op": "conv2d", "const_args": []}',
                     '{"version": 1, "op": "matmul", "bits": 4, "surprise": 1, "const_args": []}', '[1, 2]', '',
                     m.json[:-1], m.json + "x", m.json.replace("[0, 1]", "[0, 1, 2, 3, 4]"),
                     m.json.replace('"bits": 4', '"bits": 44444444444')]:
        with pytest.raises(lib.WqError, match="call description is not one this library wrote"):
            M.SubgraphModule.load_from_binary(head + dmlc_string(bad_json) + tail)
    # valid JSON that describes an invalid module goes through the same checks as create
    with pytest.raises(lib.WqError, match="bound by two constants"):
        M.SubgraphModule.load_from_binary(head + dmlc_string(m.json.replace("[0, 1]", "[1, 1]")) + tail)
    with pytest.raises(lib.WqError, match="1 constant names for 2 constant slots"):
        M.SubgraphModule.load_from_binary(head + dmlc_string(m.json) + struct.pack("<Q", 1) + dmlc_string("w"))
    # a length field that points far beyond the buffer
    with pytest.raises(lib.WqError, match="Loading symbol name failed"):
        M.SubgraphModule.load_from_binary(struct.pack("<Q", 1 << 62) + b"abc")


def test_ndarray_encoding_matches_the_reference_layout():
    """NDArray::Save (include/tvm/runtime/ndarray.h:447-496): magic, reserved, {kDLCPU, 0}, ndim, dtype,
    shape, byte count, data."""
    a = np.array([[1, 2, 3], [4, 5, 0xFFFFFFFF]], dtype=np.uint32)
    w = M._Writer()
    M.save_ndarray(w, a)
    expect = (struct.pack("<QQ", 0xDD5E40F096B4A13F, 0) + struct.pack("<ii", 1, 0) + struct.pack("<i", 2) +
              struct.pack("<BBH", 1, 32, 1) + struct.pack("<qq", 2, 3) + struct.pack("<Q", 24) + a.tobytes())
    assert w.bytes() == expect
    back = M.load_ndarray(M._Reader(expect))
    assert back.dtype == np.uint32 and np.array_equal(back, a)
    h = np.array([1.5, -2.0], dtype=np.float16)
    w = M._Writer()
    M.save_ndarray(w, h)
    assert w.bytes()[28:32] == struct.pack("<BBH", 2, 16, 1)
    assert np.array_equal(M.load_ndarray(M._Reader(w.bytes())), h)
    with pytest.raises(ValueError, match="Invalid DLTensor file format"):
        M.load_ndarray(M._Reader(b"\0" * 64))


def test_const_loader_and_module_blob_round_trip():
    """const_loader_module.cc:151-184 (save) / 186-233 (load) and the blob of library_module.cc:136-199."""
    m0 = M.SubgraphModule.create("f0", spec_matmul(), ["p0", "p1"], [0, 1], M.TILE_WEIGHTS)
    m1 = M.SubgraphModule.create("f1", spec_matmul(bits=8, order=("x", "wq", "scales", "out")), ["p2", "p3"], [1, 2])
    consts = {"p0": np.arange(32, dtype=np.uint32).reshape(2, 16), "p1": np.ones((2, 4), np.float16),
              "p2": np.arange(64, dtype=np.uint32).reshape(2, 32), "p3": np.full((2, 1), 0.5, np.float16)}
    root = M.ConstLoader(consts, {"f0": ["p0", "p1"], "f1": ["p2", "p3"]}, [m0, m1])
    blob = M.export_library(root)
    assert struct.unpack("<Q", blob[:8])[0] == len(blob) - 8
    assert struct.unpack("<Q", blob[8:16])[0] == 4  # const_loader, two backend modules, the import tree
    assert blob[16:16 + 20] == dmlc_string("const_loader")
    back = M.load_module(blob)
    assert back.const_vars_by_symbol == root.const_vars_by_symbol
    assert all(np.array_equal(back.const_var_ndarray[k], v) and back.const_var_ndarray[k].dtype == v.dtype for k, v in consts.items())
    assert [m.symbol for m in back.imports] == ["f0", "f1"] and [m.json for m in back.imports] == [m0.json, m1.json]
    assert M.export_library(back) == blob
    assert back.get_function("not_there") is None
    with pytest.raises(KeyError, match="missing entry for constant 'p9' for function 'f0'"):
        M.ConstLoader(consts, {"f0": ["p9"]})
    for cut in (7, 30, len(blob) // 2, len(blob) - 1):
        with pytest.raises((ValueError, lib.WqError)):
            M.load_module(blob[:cut])
    unknown = bytearray(blob)
    unknown[24:36] = b"const_loadex"
    with pytest.raises(ValueError, match="a loader of that name is not registered"):
        M.load_module(bytes(unknown))


def test_randomly_damaged_binaries_never_crash_the_loader():
    """4000 single- and multi-byte corruptions of a good module: each either loads as a module that
    passes the creation checks or is refused with a message; none reads outside the buffer."""
    m = M.SubgraphModule.create("fused_q4_0", spec_matmul(order=("wq", "scales", "bias", "x", "out")), ["w", "s", "b"], [0, 1, 2],
                                M.TILE_WEIGHTS)
    good = bytearray(m.save_to_binary())
    rng = np.random.default_rng(7)
    loaded = refused = 0
    for _ in range(4000):
        bad = bytearray(good)
        for _ in range(int(rng.integers(1, 4))):
            bad[int(rng.integers(0, len(bad)))] = int(rng.integers(0, 256))
        if rng.integers(0, 4) == 0:
            bad = bad[:int(rng.integers(0, len(bad)))]
        try:
            back, used = M.SubgraphModule.load_from_binary(bytes(bad))
            assert 0 < used <= len(bad) and back.json.startswith('{"version": 1')
            loaded += 1
        except lib.WqError as e:
            assert str(e)
            refused += 1
    assert loaded + refused == 4000 and refused > 1000
