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
    # gelu behind the bias (the *_bias_gelu members of the reference's table), with and without a residual
    from relax_amd.tvm_glue.codegen import ACT_GELU
    s = spec_from_function(fake_tvm.quantized_linear("decode_q8f16", tail=[("add", [n]), ("gelu",)]))
    assert (s.arg_bias, s.arg_residual, s.activation, s.arg_out) == (3, -1, ACT_GELU, 4)
    s = spec_from_function(fake_tvm.quantized_linear(tail=[("add", [n]), ("gelu",), ("add", [m, n])]))
    assert (s.arg_bias, s.arg_residual, s.activation, s.arg_out, s.num_args) == (3, 4, ACT_GELU, 5, 6)
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
    with pytest.raises(ValueError, match="gelu is only fused between"):
        spec_from_function(fake_tvm.quantized_linear(tail=[("relu",), ("gelu",)]))
    with pytest.raises(ValueError, match="gelu is only fused between"):
        spec_from_function(fake_tvm.quantized_linear(tail=[("add", [m, n]), ("gelu",)]))
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
    f = fake_tvm.quantized_linear(bound=("wq", "scales"), k=256)
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
    # K for which the tile-major layout is not defined (int4 needs K % 256 == 0): the canonical constants
    # stay, the module still loads (the flag is only set where the conversion exists)
    for k in (128, 352):
        f = fake_tvm.quantized_linear(bound=("wq", "scales"), k=k)
        assert module_plan(f, constants_of(f)).flags == 0
    f = fake_tvm.quantized_linear("decode_q8f16", bound=("wq", "scales"), k=384)  # int8: K % 128 == 0 suffices
    assert module_plan(f, constants_of(f)).flags == MODULE_TILE_WEIGHTS
    f = fake_tvm.quantized_linear(bound=("wq", "scales"), k=256)
    assert module_plan(f, constants_of(f), tile_weights=False).flags == 0
    # the gated tail is computed on canonical weights only: a gate+up composite keeps its canonical constants (a
    # module that converted them would refuse every call)
    f = fake_tvm.quantized_linear(bound=("wq", "scales"), k=256, tail=[("silu_mul",)])
    plan = module_plan(f, constants_of(f))
    assert plan.flags == 0 and plan.spec.activation == 2 and (plan.spec.arg_x, plan.spec.arg_out, plan.spec.num_args) == (2, 3, 4)
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


# ---------------------------------------------------------------- fixtures in the shape of the reference's goldens
def test_annotated_function_in_the_shape_of_the_reference_golden(fake_tvm):
    """tests/python/relax/test_transform_fuse_ops_by_pattern.py:41-81 (Conv2dReLU_composite_annotated) with the
    operators swapped for decode / permute_dims / matmul / astype: outer function with Codegen and
    global_symbol, a local Primitive + Composite function whose body is one dataflow block, parameters in
    first-use order, the symbol built from the callee names."""
    from relax_amd.tvm_glue.codegen import ACT_NONE, _derive_roles, spec_from_function

    symbol = fake_tvm.fused_name("decode_q4f16") + "_mi355x"
    assert symbol == SYM  # fused + callee names (fuse_ops.cc:370-395), dots -> underscores, + "_" + backend (:1009)
    f = fake_tvm.quantized_linear(symbol=symbol, golden_names=True)
    # the golden's structure
    assert f.attrs == {"Codegen": "mi355x", "global_symbol": symbol}
    local_binding, call_binding = f.body.blocks[0].bindings
    composite = local_binding.value
    assert composite.attrs == {"Primitive": 1, "Composite": "mi355x.q4f16_matmul"}
    assert isinstance(composite.body.blocks[0], fake_tvm.DataflowBlock) and len(composite.body.blocks) == 1
    assert call_binding.value.op is local_binding.var and f.body.body is call_binding.var
    # first-use order of the grouped bindings: decode's tuple (wq, scales), then matmul's x
    assert [p.name_hint for p in composite.params] == ["wq", "s", "x"]
    assert [p.name_hint for p in f.params] == ["wq1", "s1", "x1"]
    decode, act, roles, outer = _derive_roles(f)
    assert decode == "decode_q4f16" and act == ACT_NONE and len(outer) == 3
    assert roles == {"wq": ("param", 0), "scales": ("param", 1), "x": ("param", 2)}
    s = spec_from_function(f)
    assert (s.arg_wq, s.arg_scales, s.arg_x, s.arg_out, s.num_args) == (0, 1, 2, 3, 4)
    # the q8 flavour and a fused tail get their own names
    assert fake_tvm.fused_name("decode_q8f16", [("add", [48]), ("relu",)]) == \
        "fused_decode_q8f16_relax_permute_dims_relax_matmul_relax_astype_relax_add_relax_nn_relu"
    assert fake_tvm.fused_name("decode_q4f16", [("add", [48]), ("gelu",)]) == \
        "fused_decode_q4f16_relax_permute_dims_relax_matmul_relax_astype_relax_add_relax_nn_gelu"


def test_call_form_after_run_codegen_matches_the_call_description(fake_tvm):
    """tests/python/relax/test_transform_codegen_pass.py:184-251: RunCodegen turns every call of the annotated
    function into call_tir(ExternFunc(symbol), (the call's own arguments), out_sinfo), one extern for repeated
    calls; the lowered call appends the output (call_tir_rewrite.cc:94-110).  The call description must
    address exactly that argument list."""
    from relax_amd.tvm_glue.codegen import spec_from_function, trampoline_source

    symbol = fake_tvm.fused_name("decode_q4f16") + "_mi355x"
    f = fake_tvm.quantized_linear(symbol=symbol, golden_names=True, m=16, n=32, k=64)
    spec = spec_from_function(f)
    wq1, s1, data = fake_tvm.Var("weight1"), fake_tvm.Var("scale1"), fake_tvm.Var("data")
    wq2, s2 = fake_tvm.Var("weight2"), fake_tvm.Var("scale2")
    lv = fake_tvm.partitioned_main(symbol, (wq1, s1, data), [16, 32])
    gv = fake_tvm.partitioned_main(symbol, (wq2, s2, fake_tvm.Var("lv")), [16, 32])
    for call in (lv, gv):
        assert call.args[0].global_symbol == symbol                 # the same extern for both calls
        args = call.args[1].fields
        assert len(args) + 1 == spec.num_args and spec.arg_out == len(args)
        assert args[spec.arg_wq].name_hint.startswith("weight") and args[spec.arg_scales].name_hint.startswith("scale")
        assert args[spec.arg_x].name_hint in ("data", "lv")
        assert call.sinfo_args[0].shape == [16, 32] and call.sinfo_args[0].dtype == "float16"
    # one generated entry serves both calls
    assert trampoline_source([(symbol, spec)]).count("int " + symbol + "(") == 1


def test_bound_constants_stay_inside_the_composite(fake_tvm):
    """tests/python/relax/test_transform_fuse_ops_by_pattern.py:432-446: after BindParams the weight is a
    relax.Constant argument of the operator inside the fused function, not a parameter."""
    f = fake_tvm.quantized_linear(bound=("wq", "scales"), golden_names=True, k=256)
    composite = f.body.blocks[0].bindings[0].value
    decode_call = composite.body.blocks[0].bindings[0].value
    wq, scales = decode_call.args[1].fields
    assert isinstance(wq, fake_tvm.Constant) and isinstance(scales, fake_tvm.Constant)
    assert [p.name_hint for p in composite.params] == ["x"] and [p.name_hint for p in f.params] == ["x1"]


@pytest.mark.parametrize("kwargs,message", [
    (dict(out_dtype=""), "out_dtype float32"),             # float16 accumulation on the CPU path
    (dict(out_dtype="float16"), "out_dtype float32"),
    (dict(astype_dtype="float32"), "must produce float16"),
    (dict(axes=[0, 1]), "2-d transpose"),
    (dict(x_dtype="float32"), "x must be float16"),
])
def test_role_derivation_rejects_composites_the_kernels_do_not_compute(fake_tvm, kwargs, message):
    from relax_amd.tvm_glue.codegen import spec_from_function

    with pytest.raises(ValueError, match=message):
        spec_from_function(fake_tvm.quantized_linear(**kwargs))


def test_role_derivation_accepts_the_explicit_transpose_and_checks_operand_types(fake_tvm):
    from relax_amd.tvm_glue.codegen import spec_from_function

    assert spec_from_function(fake_tvm.quantized_linear(axes=[1, 0])).arg_x == 2
    f = fake_tvm.quantized_linear()
    decode_call = f.body.blocks[0].bindings[0].value.body.blocks[0].bindings[0].value
    decode_call.args[1].fields[0].struct_info.dtype = "int32"
    with pytest.raises(ValueError, match="packed weights must be uint32"):
        spec_from_function(f)


def test_hook_honours_its_options(fake_tvm, monkeypatch):
    """RunCodegen hands the hook a per-backend options map (src/relax/transform/run_codegen.cc:155-162)."""
    import sys

    from relax_amd.tvm_glue import codegen

    created = []
    registry = {
        "relax.ext.mi355x.create_module": lambda *a: created.append(("module",) + a) or ("module", a[0]),
        "runtime.CSourceModuleCreate": lambda *a: created.append(("csource",) + a) or ("csource", a[2]),
    }
    monkeypatch.setattr(sys.modules["tvm"], "get_global_func", lambda name: registry[name], raising=False)
    bound = fake_tvm.quantized_linear(bound=("wq", "scales"), k=256, symbol="bound_mi355x")
    free = fake_tvm.quantized_linear(symbol="free_mi355x")
    names = constants_of(bound)
    # defaults: tile-major conversion on, no scratch
    mods = codegen.relax_ext_mi355x([bound, free], None, names)
    assert [m[0] for m in mods] == ["module", "csource"]
    # (the creator's last two arguments: the module's flags and the rows its workspace is sized for)
    assert created[0][-2:] == (codegen.MODULE_TILE_WEIGHTS, 0) and "mi355x_wq_packed_call(&spec" in created[1][1]
    created.clear()
    # workspace: a function with bound weights gets a workspace of its own, sized at load for 2048 rows unless the
    # options say otherwise; a function whose weights are parameters goes through the library's scratch array
    codegen.relax_ext_mi355x([bound, free], {"tile_weights": False, "workspace": True}, names)
    assert created[0][-2:] == (codegen.MODULE_OWN_WORKSPACE, 2048)
    assert "mi355x_wq_packed_call_scratch(&spec" in created[1][1] and created[1][3] == ["free_mi355x"]
    created.clear()
    codegen.relax_ext_mi355x([bound], {"workspace": 1, "workspace_rows": 64}, names)  # integers as TVM passes them
    assert created[0][-2:] == (codegen.MODULE_TILE_WEIGHTS | codegen.MODULE_OWN_WORKSPACE, 64)
    created.clear()
    codegen.relax_ext_mi355x([bound], {"workspace_rows": 64}, names)  # rows without the switch: no workspace
    assert created[0][-2:] == (codegen.MODULE_TILE_WEIGHTS, 0)
    created.clear()
    # only the packed weights bound: N and K are known at load, the group is not -- the library's scratch array
    half_bound = fake_tvm.quantized_linear(bound=("wq",), k=256, symbol="half_mi355x")
    codegen.relax_ext_mi355x([half_bound], {"workspace": True}, constants_of(half_bound))
    assert created[0][-2:] == (codegen.MODULE_LIBRARY_SCRATCH, 0)
    with pytest.raises(ValueError, match="unknown option 'tile_weight'"):
        codegen.relax_ext_mi355x([free], {"tile_weight": True}, {})
    with pytest.raises(ValueError, match="workspace_rows must be between"):
        codegen.relax_ext_mi355x([bound], {"workspace": True, "workspace_rows": 0}, names)


def test_gated_tail_of_a_gate_up_projection(fake_tvm):
    """multiply(nn.silu(split(y, 2)[0]), split(y, 2)[1]) behind the cast: the call description carries
    ACT_SILU_MUL and no fused operands; anything else around the split is refused."""
    from relax_amd.tvm_glue.codegen import ACT_SILU_MUL, CallSpec as Spec, spec_from_function, trampoline_source

    s = spec_from_function(fake_tvm.quantized_linear(n=64, tail=[("silu_mul",)]))
    assert (s.activation, s.arg_bias, s.arg_residual, s.arg_wq, s.arg_scales, s.arg_x, s.arg_out, s.num_args) == \
        (ACT_SILU_MUL, -1, -1, 0, 1, 2, 3, 4)
    import re
    assert re.search(r"-1,\s*-1, 2\};", trampoline_source([("gated_mi355x", s)]))  # ... arg_bias, arg_residual, activation
    assert spec_from_function(fake_tvm.quantized_linear(n=64, tail=[("silu_mul", 2, 1)])).activation == ACT_SILU_MUL
    for tail, message in [([("silu_mul", 4)], "splits the output in two"),
                          ([("silu_mul", 2, 0)], "along its last axis"),
                          ([("silu_mul", 2, -1, True)], "first half"),
                          ([("add", [64]), ("silu_mul",)], "must halve the matmul result itself"),
                          ([("silu_mul",), ("relu",)], "no further operations"),
                          ([("silu_mul",), ("add", [4, 32])], "no bias and no residual")]:
        with pytest.raises(ValueError, match=message):
            spec_from_function(fake_tvm.quantized_linear(n=64, tail=tail))
    with pytest.raises(ValueError, match="no bias and no residual"):
        Spec(0, 4, 0, 7, 2, 0, 1, 4, 3, -1, ACT_SILU_MUL).validate()


def test_finalize_compiles_and_links_what_the_hook_emitted(fake_tvm, monkeypatch, tmp_path):
    """finalize() (counterpart of finalize_modules_relax, python/tvm/contrib/cutlass/build.py:856-879) run against a
    stand-in for the two TVM calls it makes.  `export_library` is what it is in TVM for a module tree with C-source
    modules (python/tvm/runtime/module.py:450-560): write each module's source, compile with `cc` and the caller's
    `options`, link one shared object; `load_module` opens it.  The stand-in really compiles -- so the link options
    finalize passes (library directory, -lmi355x_wq, rpath) and the generated source are exercised together -- and the
    entry of the hook's C-source module is then called through the loaded object."""
    import sys
    import types

    from relax_amd.tvm_glue import codegen

    class CSourceModule:
        def __init__(self, source, fmt, symbols, consts):
            self.source, self.format, self.symbols = source, fmt, list(symbols)

    class Executable:
        class Mod:
            def __init__(self, imports):
                self.imports = imports

            def export_library(self, path, cc="g++", options=()):
                files = []
                for i, m in enumerate(self.imports):
                    src = tmp_path / f"lib{i}.{m.format}"  # "cc": compiled as C++, as export_library does
                    src.write_text(m.source)
                    files.append(str(src))
                subprocess.check_call([cc, "-shared", "-fPIC", "-Wall", "-Werror", "-DMI355X_WQ_STANDALONE", "-o", path]
                                      + files + list(options))

        def __init__(self, imports):
            self.mod = Executable.Mod(imports)

    registry = {"runtime.CSourceModuleCreate": CSourceModule}
    tvm = sys.modules["tvm"]
    monkeypatch.setattr(tvm, "get_global_func", lambda name: registry[name], raising=False)
    monkeypatch.setattr(tvm, "runtime", types.SimpleNamespace(load_module=lambda path: C.CDLL(path)), raising=False)

    free = fake_tvm.quantized_linear(symbol="free_mi355x")
    mods = codegen.relax_ext_mi355x([free], None, {})
    assert len(mods) == 1 and mods[0].symbols == ["free_mi355x"] and mods[0].format == "cc"
    out = str(tmp_path / "model.so")
    loaded = codegen.finalize(Executable(mods), lib.SO_PATH, out)
    assert os.path.exists(out)
    lib.load()
    # the loaded object exports the hook's symbol with the backend calling convention, bound to the library's entry:
    # FuseOpsByPattern order (wq, scales, x, y); a float16 tensor in the wq slot is refused by the library's own check
    x = torch.zeros((2, 64), dtype=torch.float16)
    wq = torch.zeros((16, 8), dtype=torch.int32)
    s = torch.zeros((16, 2), dtype=torch.float16)
    y = torch.zeros((2, 16), dtype=torch.float16)
    dev = dict(device_type=10)
    t = [vm_harness.TensorArg(wq, as_uint32=True, **dev), vm_harness.TensorArg(s, **dev),
         vm_harness.TensorArg(x, **dev), vm_harness.TensorArg(y, **dev)]
    rc, _ = call_entry(loaded, "free_mi355x", [t[2], t[0], t[1], t[3]])
    assert rc == -1 and "argument 0 (wq): expected dtype uint32" in lib.last_error()
    if not torch.cuda.is_available():
        rc, _ = call_entry(loaded, "free_mi355x", t)
        assert rc == -1 and "no usable HIP device" in lib.last_error()
