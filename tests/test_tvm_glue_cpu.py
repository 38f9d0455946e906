"""The text side of the Relax glue: generated entries compile against the restated C ABI,
export the requested symbols and forward to the library with the recorded argument roles."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from relax_amd import lib, vm_harness  # noqa: E402
from relax_amd.tvm_glue import CallSpec, trampoline_source  # noqa: E402
from relax_amd.tvm_glue.patterns import BACKEND, DECODE_FUNCS  # noqa: E402

SYM = "fused_decode_q4f16_relax_permute_dims_relax_matmul_relax_astype_mi355x"


def build_entries(tmp_path, entries):
    src = tmp_path / "entries.c"
    src.write_text(trampoline_source(entries))
    so = str(tmp_path / "libentries.so")
    libdir = os.path.dirname(lib.SO_PATH)
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-DMI355X_WQ_STANDALONE", "-shared", "-fPIC",
                           "-o", so, str(src), "-L" + libdir, "-lmi355x_wq", "-Wl,-rpath," + libdir])
    lib.load()
    return C.CDLL(so)


def call_entry(entry_lib, symbol, tensors):
    n = len(tensors)
    vals = (vm_harness.TVMValue * n)()
    codes = (C.c_int * n)()
    for i, t in enumerate(tensors):
        vals[i].v_handle = t.handle
        codes[i] = vm_harness.K_TVM_NDARRAY_HANDLE
    ret = vm_harness.TVMValue()
    rc_code = C.c_int(vm_harness.K_TVM_NULLPTR)
    fn = getattr(entry_lib, symbol)
    fn.argtypes = [C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_void_p, C.POINTER(C.c_int), C.c_void_p]
    rc = fn(C.addressof(vals), codes, n, C.addressof(ret), C.byref(rc_code), None)
    return rc, rc_code.value


def test_generated_entries_compile_and_forward(tmp_path):
    # FuseOpsByPattern hands the extern (wq, scales, x, y): roles x=2, wq=0, scales=1, out=3
    entries = [(SYM, CallSpec(0, 4, 0, 7, 2, 0, 1, 3)),
               ("fused_q8_mi355x", CallSpec(0, 8, 128, 0, 2, 0, 1, 3)),
               ("decode_only_mi355x", CallSpec(1, 4, 0, 7, 0, 0, 1, 2))]
    L = build_entries(tmp_path, entries)
    x = torch.zeros((2, 64), dtype=torch.float16)
    wq = torch.zeros((16, 8), dtype=torch.int32)
    s = torch.zeros((16, 2), dtype=torch.float16)
    y = torch.zeros((2, 16), dtype=torch.float16)
    dev = dict(device_type=10)
    t = [vm_harness.TensorArg(wq, as_uint32=True, **dev), vm_harness.TensorArg(s, **dev),
         vm_harness.TensorArg(x, **dev), vm_harness.TensorArg(y, **dev)]
    # the roles are honoured: with the arguments in (x, wq, scales, y) order the entry sees a float16 "wq"
    wrong = [t[2], t[0], t[1], t[3]]
    rc, code = call_entry(L, SYM, wrong)
    assert rc == -1 and code == vm_harness.K_TVM_NULLPTR
    assert "argument 0 (wq): expected dtype uint32" in lib.last_error()
    if not torch.cuda.is_available():
        rc, _ = call_entry(L, SYM, t)  # every check passes; there is just no device here
        assert rc == -1 and "no usable HIP device" in lib.last_error()
    # explicit group 128 contradicts the 2 scale columns of K = 32 (q8 reading of the same words)
    rc, _ = call_entry(L, "fused_q8_mi355x", t)
    assert rc == -1 and "does not match K=32 / group=128" in lib.last_error()
    rc, _ = call_entry(L, "decode_only_mi355x", t)
    assert rc == -1 and "expects 3 arguments, got 4" in lib.last_error()


def test_trampoline_generator_rejects_bad_input():
    with pytest.raises(ValueError, match="not a C identifier"):
        trampoline_source([("bad-name", CallSpec(0, 4, 0, 7, 0, 1, 2, 3))])
    with pytest.raises(ValueError, match="not a permutation"):
        trampoline_source([("f", CallSpec(0, 4, 0, 7, 0, 0, 2, 3))])
    with pytest.raises(ValueError, match="duplicate"):
        trampoline_source([("f", CallSpec(0, 4, 0, 7, 0, 1, 2, 3)), ("f", CallSpec(0, 4, 0, 7, 0, 1, 2, 3))])
    with pytest.raises(ValueError, match="bits"):
        trampoline_source([("f", CallSpec(0, 3, 0, 7, 0, 1, 2, 3))])


def test_pattern_table_metadata():
    assert BACKEND == "mi355x"
    assert DECODE_FUNCS["decode_q4f16"] == {"bits": 4, "zero_point": 7}
    assert DECODE_FUNCS["decode_q8f16"] == {"bits": 8, "zero_point": 0}


def test_quantize_helpers_round_trip():
    from oracle import wq_oracle as O
    from relax_amd import pack_q4, pack_q8, quantize_q4f16, quantize_q8f16

    rng = np.random.default_rng(0)
    w4 = rng.integers(0, 16, size=(5, 64))
    w8 = rng.integers(-128, 128, size=(5, 64))
    assert np.array_equal(pack_q4(w4), O.pack_q4(w4)) and np.array_equal(O.unpack_q4(pack_q4(w4)), w4)
    assert np.array_equal(pack_q8(w8), O.pack_q8(w8)) and np.array_equal(O.unpack_q8(pack_q8(w8)), w8)
    w = rng.standard_normal((8, 256)).astype(np.float32)
    wq, s = quantize_q4f16(w)
    assert np.abs(O.dequant_q4f16(wq, s).astype(np.float32) - w).max() <= 0.51 * float(s.max()) + 1e-3
    wq, s = quantize_q8f16(w)
    assert np.abs(O.dequant_q8f16(wq, s).astype(np.float32) - w).max() <= 0.51 * float(s.max()) + 1e-3
    with pytest.raises(ValueError):
        pack_q4(np.full((1, 8), 16))


# ---------------------------------------------------------------- role derivation on a stand-in IR
@pytest.fixture
def fake_tvm(monkeypatch):
    import sys

    from tests.support import fake_relax

    tvm, relax = fake_relax.as_module()
    monkeypatch.setitem(sys.modules, "tvm", tvm)
    monkeypatch.setitem(sys.modules, "tvm.relax", relax)
    return fake_relax


def test_roles_of_plain_and_fused_composites(fake_tvm):
    from relax_amd.tvm_glue.codegen import ACT_NONE, ACT_RELU, spec_from_function

    m, n = 4, 48
    s = spec_from_function(fake_tvm.quantized_linear())
    assert (s.arg_wq, s.arg_scales, s.arg_x, s.arg_out, s.num_args) == (0, 1, 2, 3, 4)
    assert (s.arg_bias, s.arg_residual, s.activation, s.bits, s.zero_point) == (-1, -1, ACT_NONE, 4, 7)
    s = spec_from_function(fake_tvm.quantized_linear("decode_q8f16", tail=[("add", [n])]))
    assert (s.bits, s.zero_point, s.arg_bias, s.arg_residual, s.arg_out, s.num_args) == (8, 0, 3, -1, 4, 5)
    s = spec_from_function(fake_tvm.quantized_linear(tail=[("add", [1, n]), ("relu",)]))
    assert (s.arg_bias, s.arg_residual, s.activation) == (3, -1, ACT_RELU)
    s = spec_from_function(fake_tvm.quantized_linear(tail=[("add", [m, n])]))
    assert (s.arg_bias, s.arg_residual, s.activation, s.arg_out) == (-1, 3, ACT_NONE, 4)
    # add(residual, y): the operand order of the add does not matter
    s = spec_from_function(fake_tvm.quantized_linear(tail=[("add", [m, n], True)]))
    assert (s.arg_bias, s.arg_residual) == (-1, 3)
    s = spec_from_function(fake_tvm.quantized_linear(tail=[("add", [n]), ("relu",), ("add", [m, n])]))
    assert (s.arg_bias, s.arg_residual, s.activation, s.arg_out, s.num_args) == (3, 4, ACT_RELU, 5, 6)
    s.validate()
    # outer parameters in another order: roles follow the call arguments, not the positions
    s = spec_from_function(fake_tvm.quantized_linear(tail=[("add", [n])], outer_order=[2, 3, 0, 1]))
    assert (s.arg_x, s.arg_bias, s.arg_wq, s.arg_scales, s.arg_out) == (0, 1, 2, 3, 4)


def test_role_derivation_rejects_tails_the_epilogue_cannot_express(fake_tvm):
    from relax_amd.tvm_glue.codegen import spec_from_function

    m, n = 4, 48
    with pytest.raises(ValueError, match="in this order"):  # relu after a [M,N] add
        spec_from_function(fake_tvm.quantized_linear(tail=[("add", [m, n]), ("add", [m, n])]))
    with pytest.raises(ValueError, match="only fused between"):
        spec_from_function(fake_tvm.quantized_linear(tail=[("add", [m, n]), ("relu",)]))
    with pytest.raises(ValueError, match="only fused between"):
        spec_from_function(fake_tvm.quantized_linear(tail=[("relu",), ("relu",)]))
    f = fake_tvm.quantized_linear()
    f.body.blocks[0].bindings[0].value.attrs["Composite"] = "cutlass.matmul"
    with pytest.raises(ValueError, match="does not belong to backend"):
        spec_from_function(f)


def test_generated_fused_entry_forwards_all_roles(tmp_path):
    # (wq, scales, x, bias, residual, y) with relu between the adds
    spec = CallSpec(0, 4, 0, 7, 2, 0, 1, 5, 3, 4, 1)
    L = build_entries(tmp_path, [("fused_tail_mi355x", spec)])
    dev = dict(device_type=10)
    x = torch.zeros((2, 64), dtype=torch.float16)
    wq = torch.zeros((16, 8), dtype=torch.int32)
    s = torch.zeros((16, 2), dtype=torch.float16)
    y = torch.zeros((2, 16), dtype=torch.float16)
    bias = torch.zeros(16, dtype=torch.float16)
    res = torch.zeros((2, 16), dtype=torch.float16)
    t = [vm_harness.TensorArg(wq, as_uint32=True, **dev), vm_harness.TensorArg(s, **dev),
         vm_harness.TensorArg(x, **dev), vm_harness.TensorArg(bias, **dev),
         vm_harness.TensorArg(res, **dev), vm_harness.TensorArg(y, **dev)]
    rc, _ = call_entry(L, "fused_tail_mi355x", [t[0], t[1], t[2], t[4], t[3], t[5]])  # bias and residual swapped
    assert rc == -1 and "bias has shape (2, 16)" in lib.last_error()
    rc, _ = call_entry(L, "fused_tail_mi355x", t[:5])
    assert rc == -1 and "expects 6 arguments, got 5" in lib.last_error()
    if not torch.cuda.is_available():
        rc, _ = call_entry(L, "fused_tail_mi355x", t)
        assert rc == -1 and "no usable HIP device" in lib.last_error()
    with pytest.raises(ValueError, match="activation"):
        trampoline_source([("f", CallSpec(0, 4, 0, 7, 0, 1, 2, 3, -1, -1, 9))])
    with pytest.raises(ValueError, match="no fused operands"):
        trampoline_source([("f", CallSpec(1, 4, 0, 7, 0, 0, 1, 3, 2, -1, 0))])


def constants_of(func):
    """What RunCodegen's PostOrderVisit collects: every Constant of the function body, named
    <symbol>_<codegen>_const_<i> in visiting order (src/relax/transform/run_codegen.cc:120-129)."""
    from tests.support import fake_relax

    found = []

    def walk(e):
        if isinstance(e, fake_relax.Constant) and e not in found:
            found.append(e)
        for child in getattr(e, "args", []) + getattr(e, "fields", []):
            walk(child)
        if isinstance(e, fake_relax.Function):
            walk(e.body)
        if isinstance(e, fake_relax.SeqExpr):
            for block in e.blocks:
                for b in block.bindings:
                    walk(b.value)
            walk(e.body)

    walk(func)
    return {c: f"fused_mi355x_mi355x_const_{i}" for i, c in enumerate(found)}


def test_bound_weights_give_a_module_plan(fake_tvm):
    from relax_amd import module as M
    from relax_amd.tvm_glue.codegen import ACT_RELU, MODULE_TILE_WEIGHTS, module_plan, spec_from_function
    from relax_amd.vm_harness import CallSpec as CSpec

    n = 48
    f = fake_tvm.quantized_linear(bound=("wq", "scales"))
    assert [p.name_hint for p in f.params] == ["x_outer"]
    with pytest.raises(ValueError, match="use module_plan"):
        spec_from_function(f)
    names = constants_of(f)
    plan = module_plan(f, names)
    s = plan.spec
    assert plan.symbol == "fused_mi355x" and plan.flags == MODULE_TILE_WEIGHTS
    assert plan.const_names == ("fused_mi355x_mi355x_const_0", "fused_mi355x_mi355x_const_1") and plan.const_args == (0, 1)
    assert (s.arg_wq, s.arg_scales, s.arg_x, s.arg_out, s.num_args) == (0, 1, 2, 3, 4)  # the VM calls <symbol>(x, out)
    # bias bound as well, residual a parameter, relu in between
    f = fake_tvm.quantized_linear("decode_q8f16", tail=[("add", [n]), ("relu",), ("add", [4, n])],
                                  bound=("wq", "scales", "operand0"))
    plan = module_plan(f, constants_of(f))
    s = plan.spec
    assert plan.const_args == (0, 1, 2) and len(plan.const_names) == 3
    assert (s.bits, s.arg_wq, s.arg_scales, s.arg_bias, s.arg_x, s.arg_residual, s.arg_out, s.activation) == \
        (8, 0, 1, 2, 3, 4, 5, ACT_RELU)
    # only the weights bound, scales a parameter: no tile-major conversion (it needs both)
    f = fake_tvm.quantized_linear(bound=("wq",))
    plan = module_plan(f, constants_of(f))
    assert plan.flags == 0 and plan.const_args == (0,) and (plan.spec.arg_wq, plan.spec.arg_scales, plan.spec.arg_x) == (0, 1, 2)
    # the plan is what the library's module accepts, and the module reports the same constants
    f = fake_tvm.quantized_linear(tail=[("add", [n])], bound=("wq", "scales", "operand0"))
    plan = module_plan(f, constants_of(f))
    s = plan.spec
    mod = M.SubgraphModule.create(plan.symbol, CSpec(op=s.op, bits=s.bits, group=s.group, zero_point=s.zero_point, arg_x=s.arg_x,
                                                     arg_wq=s.arg_wq, arg_scales=s.arg_scales, arg_out=s.arg_out,
                                                     num_args=s.num_args, arg_bias=s.arg_bias, arg_residual=s.arg_residual,
                                                     activation=s.activation),
                                  list(plan.const_names), list(plan.const_args), plan.flags)
    assert mod.const_names == list(plan.const_names) and not mod.initialized
    # a constant RunCodegen did not name
    with pytest.raises(ValueError, match="has no name in constant_names"):
        module_plan(f, {})
    # an activation operand can not be a constant
    f = fake_tvm.quantized_linear(tail=[("add", [4, n])], bound=("wq", "scales", "operand0"))
    with pytest.raises(ValueError, match="residual of the composite is a constant"):
        module_plan(f, constants_of(f))
