"""GPU tests of the subgraph runtime module: constants bound through `__init_<symbol>` (device
tensors borrowed, host arrays copied), the call with the remaining arguments, the one-off tile-major
conversion, and the export -> load -> run round trip
(the shape of tests/python/relax/test_transform_codegen_pass.py:57-65)."""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from relax_amd import lib, module as M, vm_harness  # noqa: E402
from relax_amd.vm_harness import CallSpec, PackedError  # noqa: E402
from tests.test_gpu_parity import _dev, assert_close  # noqa: E402


def spec_for(bits, order, op=0, **kw):
    slots = {r: i for i, r in enumerate(order)}
    return CallSpec(op=op, bits=bits, group=0, zero_point=7 if bits == 4 else 0, arg_x=slots.get("x", 0),
                    arg_wq=slots["wq"], arg_scales=slots["scales"], arg_out=slots["out"], num_args=len(order),
                    arg_bias=slots.get("bias", -1), arg_residual=slots.get("residual", -1), **kw)


def plain(bits, x, wq, s):
    return vm_harness.call_dps("mi355x_q%df16_matmul" % bits, [x, wq, s], (x.shape[0], wq.shape[0]))


@pytest.mark.parametrize("bits, m, n, k", [(4, 1, 4096, 4096), (4, 8, 200, 352), (4, 200, 136, 256), (8, 16, 5120, 5120),
                                           (8, 3, 72, 384), (4, 64, 1024, 2048)])
def test_bound_device_constants_give_the_plain_call_bit_for_bit(bits, m, n, k):
    vm_harness.set_stream()
    x, wq, s, g = O.make_case(31, m, n, k, bits)
    dx, dw, ds = _dev(x), _dev(wq), _dev(s)
    mod = M.SubgraphModule.create("f", spec_for(bits, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1])
    init, run = mod.get_function("__init_f"), mod.get_function("f")
    init(dw, ds)
    assert mod.initialized
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    run(dx, y)
    torch.cuda.synchronize()
    assert torch.equal(y, plain(bits, dx, dw, ds))
    assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (bits, m, n, k))
    # init is once only: a second call with other tensors returns and changes nothing (json_runtime.h:91-98)
    init(torch.zeros_like(dw), torch.zeros_like(ds))
    y2 = torch.empty_like(y)
    run(dx, y2)
    assert torch.equal(y2, y)


def test_host_constants_are_copied_to_the_device_at_init():
    """After load_module the const loader holds host arrays (NDArrays are saved as CPU arrays)."""
    vm_harness.set_stream()
    for bits, m, n, k in [(4, 4, 512, 1024), (8, 1, 320, 640)]:
        x, wq, s, g = O.make_case(32, m, n, k, bits)
        mod = M.SubgraphModule.create("f", spec_for(bits, ("x", "wq", "scales", "out")), ["w", "s"], [1, 2])
        mod.get_function("__init_f")(wq, s)  # numpy arrays
        y = torch.empty((m, n), dtype=torch.float16, device="cuda")
        mod.get_function("f")(_dev(x), y)
        torch.cuda.synchronize()
        assert torch.equal(y, plain(bits, _dev(x), _dev(wq), _dev(s)))
        mod.close()  # frees the module's device copies


@pytest.mark.parametrize("bits, n, k", [(4, 4096, 4096), (8, 5120, 5120), (4, 200, 512)])
def test_tile_major_conversion_at_init(bits, n, k):
    """With the flag the module keeps its own tile-major copy and runs every call on it; results
    equal mi355x_wq_matmul_tiled on weights tiled by hand, and the canonical path within tolerance."""
    from relax_amd import wq_matmul, wq_tile_weights

    vm_harness.set_stream()
    group = 32 if bits == 4 else 128
    for m in (1, 8, 48, 256):
        x, wq, s, g = O.make_case(33, m, n, k, bits)
        dx, dw, ds = _dev(x), _dev(wq), _dev(s)
        mod = M.SubgraphModule.create("f", spec_for(bits, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.TILE_WEIGHTS)
        mod.get_function("__init_f")(wq if m == 8 else dw, s if m == 8 else ds)
        y = torch.empty((m, n), dtype=torch.float16, device="cuda")
        mod.get_function("f")(dx, y)
        torch.cuda.synchronize()
        wt, st = wq_tile_weights(dw, ds, bits=bits, group=group)
        assert torch.equal(y, wq_matmul(dx, wt, st, bits=bits, group=group, tiled_n=n))
        assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (bits, m, n, k))


def test_fused_operands_bias_constant_residual_argument():
    vm_harness.set_stream()
    bits, m, n, k = 4, 8, 1024, 1024
    x, wq, s, g = O.make_case(34, m, n, k, bits)
    rng = np.random.default_rng(5)
    bias = rng.standard_normal(n).astype(np.float16)
    res = rng.standard_normal((m, n)).astype(np.float16)
    order = ("wq", "scales", "bias", "x", "residual", "out")
    mod = M.SubgraphModule.create("g", spec_for(bits, order, activation=1), ["w", "s", "b"], [0, 1, 2], M.TILE_WEIGHTS)
    mod.get_function("__init_g")(_dev(wq), _dev(s), bias)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    mod.get_function("g")(_dev(x), _dev(res), y)
    torch.cuda.synchronize()
    want = c_oracle.wq_matmul_fused(x, wq, s, bits, g, bias=bias, activation="relu", residual=res)
    assert_close(y.cpu().numpy(), want, "bias + relu + residual through the module")


def test_dequantize_module():
    vm_harness.set_stream()
    x, wq, s, g = O.make_case(35, 1, 96, 256, 4)
    mod = M.SubgraphModule.create("d", spec_for(4, ("wq", "scales", "out"), op=1), ["w", "s"], [0, 1])
    mod.get_function("__init_d")(wq, s)
    wd = torch.empty((96, 256), dtype=torch.float16, device="cuda")
    mod.get_function("d")(wd)
    torch.cuda.synchronize()
    assert np.array_equal(wd.cpu().numpy().view(np.uint16), c_oracle.dequant(wq, s, 4, g, 8).view(np.uint16))


def test_argument_errors():
    vm_harness.set_stream()
    x, wq, s, g = O.make_case(36, 2, 64, 128, 4)
    mod = M.SubgraphModule.create("f", spec_for(4, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1])
    with pytest.raises(PackedError, match="__init_f expects 2 constants, got 1"):
        mod.get_function("__init_f")(_dev(wq))
    assert not mod.initialized
    y = torch.empty((2, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(PackedError, match="has not been initialized"):
        mod.get_function("f")(_dev(x), y)
    mod.get_function("__init_f")(_dev(wq), _dev(s))
    with pytest.raises(PackedError, match="f expects 2 arguments .2 of the composite's 4 are bound constants., got 3"):
        mod.get_function("f")(_dev(x), y, y)
    with pytest.raises(PackedError, match="x has 64 columns but the weights have K=128"):
        mod.get_function("f")(_dev(x[:, :64].copy()), y)
    # constants of the wrong type are named when the call validates them
    bad = M.SubgraphModule.create("f", spec_for(4, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1])
    bad.get_function("__init_f")(_dev(s), _dev(s))
    with pytest.raises(PackedError, match="wq.*expected dtype uint32"):
        bad.get_function("f")(_dev(x), y)
    tiled = M.SubgraphModule.create("f", spec_for(4, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.TILE_WEIGHTS)
    with pytest.raises(PackedError, match="wq must be uint32"):
        tiled.get_function("__init_f")(_dev(s), _dev(s))
    assert not tiled.initialized


def test_export_load_run_round_trip(tmp_path):
    """Two projections of a layer with bound weights: run, export, load the file in place of the
    original, run again -- same bits (check_roundtrip, test_transform_codegen_pass.py:57-65)."""
    vm_harness.set_stream()
    cases = {"fused_q4_0": (4, 4096, 4096, ("wq", "scales", "x", "out"), M.TILE_WEIGHTS),
             "fused_q8_1": (8, 1280, 5120, ("x", "wq", "scales", "out"), 0)}
    consts, by_symbol, mods, inputs = {}, {}, [], {}
    for i, (sym, (bits, n, k, order, flags)) in enumerate(cases.items()):
        x, wq, s, g = O.make_case(40 + i, 8, n, k, bits)
        names = [f"{sym}_const_0", f"{sym}_const_1"]
        consts[names[0]], consts[names[1]] = _dev(wq), _dev(s)
        by_symbol[sym] = names
        slots = [order.index("wq"), order.index("scales")]
        mods.append(M.SubgraphModule.create(sym, spec_for(bits, order), names, slots, flags))
        inputs[sym] = (x, wq, s, g, bits)
    exec0 = M.ConstLoader(consts, by_symbol, mods)
    path = tmp_path / "exec.bin"
    path.write_bytes(M.export_library(exec0))
    exec1 = M.load_module(path.read_bytes())
    assert all(isinstance(v, np.ndarray) for v in exec1.const_var_ndarray.values())  # host arrays after a load
    for sym, (x, wq, s, g, bits) in inputs.items():
        outs = []
        for ex in (exec0, exec1):
            y = torch.empty((8, wq.shape[0]), dtype=torch.float16, device="cuda")
            ex.get_function(sym)(_dev(x), y)  # the first lookup runs __init_<symbol>
            torch.cuda.synchronize()
            outs.append(y)
        assert torch.equal(outs[0], outs[1])
        assert_close(outs[1].cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), sym)
    assert all(exec1.initialized.values()) and all(m.initialized for m in exec1.imports)


def test_module_call_captured_in_a_hip_graph():
    """Calls allocate nothing, so a module call can sit in a captured decode step."""
    vm_harness.set_stream()
    x, wq, s, g = O.make_case(44, 1, 4096, 4096, 4)
    mod = M.SubgraphModule.create("f", spec_for(4, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.TILE_WEIGHTS)
    mod.get_function("__init_f")(wq, s)
    dx = _dev(x)
    y = torch.empty((1, 4096), dtype=torch.float16, device="cuda")
    run = mod.get_function("f")
    run(dx, y)
    torch.cuda.synchronize()
    eager = y.clone()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        vm_harness.set_stream(stream)
        with torch.cuda.graph(graph, stream=stream):
            run(dx, y)
    vm_harness.set_stream()
    for _ in range(3):
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager)


def test_empty_batch_and_empty_projection():
    """M = 0 and N = 0 are legal shapes: nothing is launched, nothing fails (host constants, tile flag)."""
    vm_harness.set_stream()
    x, wq, s, g = O.make_case(45, 2, 64, 256, 4)
    mod = M.SubgraphModule.create("f", spec_for(4, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.TILE_WEIGHTS)
    mod.get_function("__init_f")(wq, s)
    mod.get_function("f")(torch.empty((0, 256), dtype=torch.float16, device="cuda"),
                          torch.empty((0, 64), dtype=torch.float16, device="cuda"))
    y = torch.empty((2, 64), dtype=torch.float16, device="cuda")
    mod.get_function("f")(_dev(x), y)  # and the module still computes afterwards
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, 4, g), "after an empty call")
    none = M.SubgraphModule.create("e", spec_for(4, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.TILE_WEIGHTS)
    none.get_function("__init_e")(torch.empty((0, 32), dtype=torch.int32, device="cuda"),
                                  torch.empty((0, 8), dtype=torch.float16, device="cuda"))
    none.get_function("e")(_dev(x), torch.empty((2, 0), dtype=torch.float16, device="cuda"))
    torch.cuda.synchronize()


@pytest.mark.parametrize("bits, n, k, group", [(4, 200, 352, None), (4, 96, 96, None), (8, 136, 320, 64)])
def test_tile_weights_flag_where_the_layout_is_not_defined(bits, n, k, group):
    """The flag is a request: for a (bits, group, K) without a tile-major layout (int4 with K % 256 != 0,
    group sizes other than 32 / 128) init keeps the canonical constants and calls run on them."""
    vm_harness.set_stream()
    for m in (1, 8, 70):
        x, wq, s, g = O.make_case(41, m, n, k, bits, group)
        assert lib.load().mi355x_wq_tiled_sizes(lib.make_desc(bits, g, n, k), None, None) == -1
        mod = M.SubgraphModule.create("f", spec_for(bits, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.TILE_WEIGHTS)
        mod.get_function("__init_f")(wq, s)  # host constants, as after load_module
        assert mod.initialized
        y = torch.empty((m, n), dtype=torch.float16, device="cuda")
        mod.get_function("f")(_dev(x), y)
        torch.cuda.synchronize()
        assert torch.equal(y, plain(bits, _dev(x), _dev(wq), _dev(s)))
        assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=8), (bits, m, n, k))
        mod.close()


def test_library_scratch_flag_and_packed_call_scratch():
    """MI355X_WQ_MODULE_LIBRARY_SCRATCH / mi355x_wq_packed_call_scratch: decode calls may split K on the
    library's scratch array; results equal the caller-workspace entry bit for bit, also on tile-major weights,
    and the module survives export -> load with the flag."""
    import relax_amd

    vm_harness.set_stream()
    bits, m, n, k = 8, 16, 5120, 13824
    x, wq, s, g = O.make_case(42, m, n, k, bits)
    dx, dw, ds = _dev(x), _dev(wq), _dev(s)
    need = relax_amd.wq_workspace_bytes(bits, g, n, k, m)
    assert need > 0
    want = relax_amd.wq_matmul(dx, dw, ds, bits, g, workspace=relax_amd.wq_workspace(need))
    for flags in (M.LIBRARY_SCRATCH, M.LIBRARY_SCRATCH | M.TILE_WEIGHTS):
        mod = M.SubgraphModule.create("f", spec_for(bits, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], flags)
        mod, _ = M.SubgraphModule.load_from_binary(mod.save_to_binary())
        mod.get_function("__init_f")(dw, ds)
        y = torch.empty((m, n), dtype=torch.float16, device="cuda")
        mod.get_function("f")(dx, y)
        torch.cuda.synchronize()
        if flags & M.TILE_WEIGHTS:
            wt, st = relax_amd.wq_tile_weights(dw, ds, bits, g)
            need_t = relax_amd.wq_workspace_bytes(bits, g, n, k, m, tiled=True)
            ref = relax_amd.wq_matmul(dx, wt, st, bits, g, tiled_n=n, workspace=relax_amd.wq_workspace(max(need_t, 16)))
            torch.cuda.synchronize()
            assert torch.equal(y.view(torch.int16), ref.view(torch.int16))
        else:
            assert torch.equal(y.view(torch.int16), want.view(torch.int16))
        assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), ("scratch", flags))
        mod.close()
    # the generated entries' forwarding function, called directly
    spec = spec_for(bits, ("x", "wq", "scales", "out"))
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    targs = [vm_harness.TensorArg(t, as_uint32=(t.dtype == torch.int32)) for t in (dx, dw, ds, y)]
    vm_harness.call_packed("mi355x_wq_packed_call_scratch", targs, spec=spec)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))


def test_gated_composite_with_bound_weights():
    """A gate+up projection whose weights are bound constants -- the normal case of an LLM -- with the tile-major
    request on: the gated tail runs on canonical weights only, so init keeps the canonical constants and the calls
    compute; decode and prefill row counts, host and device constants, through export -> load."""
    import relax_amd

    vm_harness.set_stream()
    for bits, n, k, rows in ((4, 512, 1024, (1, 8, 160)), (8, 256, 1280, (3, 16))):
        x_all, wq, s, g = O.make_case(46 + bits, max(rows), n, k, bits)
        dw, ds = _dev(wq), _dev(s)
        mod = M.SubgraphModule.create("gu", spec_for(bits, ("wq", "scales", "x", "out"), activation=lib.ACT_SILU_MUL),
                                      ["w", "s"], [0, 1], M.TILE_WEIGHTS)
        mod, _ = M.SubgraphModule.load_from_binary(mod.save_to_binary())
        mod.get_function("__init_gu")(wq, s)  # host arrays, as after load_module
        for m in rows:
            dx = _dev(np.ascontiguousarray(x_all[:m]))
            y = torch.empty((m, n // 2), dtype=torch.float16, device="cuda")
            mod.get_function("gu")(dx, y)
            direct = relax_amd.wq_matmul(dx, dw, ds, bits, g, activation="silu_mul")
            torch.cuda.synchronize()
            assert torch.equal(y.view(torch.int16), direct.view(torch.int16)), (bits, m)
            ref = c_oracle.wq_matmul_fused(x_all[:m], wq, s, bits, g, activation="silu_mul", nthreads=8).astype(np.float64)
            h = np.abs(c_oracle.wq_matmul(x_all[:m], wq, s, bits, g, nthreads=8).astype(np.float64))
            err = np.abs(y.cpu().numpy().astype(np.float64) - ref)
            assert np.all(err <= (1e-2 + 1e-2 * np.abs(ref)) * 2 * (1.0 + h[:, :n // 2] + h[:, n // 2:])), (bits, m, float(err.max()))
        mod.close()


@pytest.mark.parametrize("bits, n, k, rows", [(8, 15360, 5120, (256,)), (8, 5120, 5120, (256, 1)), (8, 27648, 5120, (256,)),
                                              (8, 5120, 13824, (256, 16, 1)), (4, 4096, 11008, (8, 16, 200))])
@pytest.mark.parametrize("flags", [M.OWN_WORKSPACE, M.OWN_WORKSPACE | M.TILE_WEIGHTS])
def test_module_owned_workspace(bits, n, k, rows, flags):
    """MI355X_WQ_MODULE_OWN_WORKSPACE: init allocates and zeroes the K split's workspace for calls of up to
    `workspace_rows` rows; calls equal the caller-workspace entry bit for bit and match the oracle; the buffer's
    counters are back at zero after every call; a call of more rows than it was sized for runs as the plain call;
    the setting survives export -> load."""
    import relax_amd

    vm_harness.set_stream()
    tiled = bool(flags & M.TILE_WEIGHTS)
    x_all, wq, s, g = O.make_case(60 + bits + n % 7, max(rows), n, k, bits)
    dw, ds = _dev(wq), _dev(s)
    wt, st = relax_amd.wq_tile_weights(dw, ds, bits, g) if tiled else (dw, ds)
    mod = M.SubgraphModule.create("f", spec_for(bits, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], flags, workspace_rows=256)
    mod, _ = M.SubgraphModule.load_from_binary(mod.save_to_binary())
    mod.get_function("__init_f")(dw, ds)
    split_somewhere = False
    for m in rows:
        x = np.ascontiguousarray(x_all[:m])
        dx = _dev(x)
        y = torch.empty((m, n), dtype=torch.float16, device="cuda")
        mod.get_function("f")(dx, y)
        mod.get_function("f")(dx, y)  # (a second call finds the counters at zero again)
        need = relax_amd.wq_workspace_bytes(bits, g, n, k, m, tiled=tiled)
        split_somewhere |= need > 0
        ws = relax_amd.wq_workspace(max(need, 16))
        ref = relax_amd.wq_matmul(dx, wt, st, bits, g, workspace=ws, **({"tiled_n": n} if tiled else {}))
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), ref.view(torch.int16)), (bits, n, k, m, flags)
        want = c_oracle.wq_matmul(x[:4], wq, s, bits, g, nthreads=16)
        assert_close(y[:4].cpu().numpy(), want, (bits, n, k, m, flags), ulp_fraction=0.01)
    if m >= 64:  # every tile against float32 torch on the bit-exact dequantized weights
        wd = relax_amd.wq_dequantize(dw, ds, bits, g).float()
        full = (dx.float() @ wd.t())
        err = (y.float() - full).abs()
        assert bool((err <= 2e-2 + 1e-2 * full.abs()).all()), float(err.max())
    # (int8 with K = 5120: 27648 rows never split; the others only on tile-major weights, since the plain call loads
    # the canonical layout by whole cache lines)
    assert split_somewhere or (bits == 8 and k == 5120 and (n == 27648 or not tiled)), "these shapes are meant to split K at some row count"
    # more rows than the workspace was sized for: the plain call
    m = 300
    x, _, _, _ = O.make_case(61, m, 16, k, bits)
    dx = _dev(x)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    mod.get_function("f")(dx, y)
    plain_y = relax_amd.wq_matmul(dx, wt, st, bits, g, **({"tiled_n": n} if tiled else {}))
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), plain_y.view(torch.int16))
    mod.close()


def test_module_owned_workspace_in_a_hip_graph():
    """Calls on the module's workspace allocate nothing: captured, replayed, equal to eager."""
    vm_harness.set_stream()
    bits, m, n, k = 8, 256, 5120, 13824
    x, wq, s, g = O.make_case(63, m, n, k, bits)
    mod = M.SubgraphModule.create("f", spec_for(bits, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.OWN_WORKSPACE,
                                  workspace_rows=m)
    mod.get_function("__init_f")(_dev(wq), _dev(s))
    dx = _dev(x)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    run = mod.get_function("f")
    run(dx, y)
    torch.cuda.synchronize()
    eager = y.clone()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        vm_harness.set_stream(stream)
        with torch.cuda.graph(graph, stream=stream):
            run(dx, y)
    vm_harness.set_stream()
    for _ in range(3):
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager)


def test_scratch_option_falls_back_where_the_array_is_too_small():
    """A decode split that would need more than the library's 4 MB array runs unsplit through the packed and module
    paths (the option is a speed-up, not a reason to fail); the direct entry point still refuses."""
    import relax_amd

    vm_harness.set_stream()
    bits, m, n, k = 8, 1, 17408, 8192
    x, wq, s, g = O.make_case(64, m, n, k, bits)
    dx, dw, ds = _dev(x), _dev(wq), _dev(s)
    L = lib.load()
    need = relax_amd.wq_workspace_bytes(bits, g, n, k, m)
    assert need > L.mi355x_wq_static_ws_bytes(), "the case is meant to exceed the scratch array"
    want = relax_amd.wq_matmul(dx, dw, ds, bits, g)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    targs = [vm_harness.TensorArg(t, as_uint32=(t.dtype == torch.int32)) for t in (dx, dw, ds, y)]
    vm_harness.call_packed("mi355x_wq_packed_call_scratch", targs, spec=spec_for(bits, ("x", "wq", "scales", "out")))
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))
    mod = M.SubgraphModule.create("f", spec_for(bits, ("wq", "scales", "x", "out")), ["w", "s"], [0, 1], M.LIBRARY_SCRATCH)
    mod.get_function("__init_f")(dw, ds)
    y.zero_()
    mod.get_function("f")(dx, y)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), want.view(torch.int16))
    desc = lib.make_desc(bits, g, n, k)
    assert L.mi355x_wq_matmul_static_ws(desc, dx.data_ptr(), dw.data_ptr(), ds.data_ptr(), None, y.data_ptr(), m, None, 0) == -1
    assert "use mi355x_wq_matmul_ws" in lib.last_error()


def test_activations_with_leading_extents():
    """x[B, S, K] against the 2-d weight (src/relax/op/tensor/linear_algebra.cc:46-114): B * S rows; the output, the
    residual and (with unit extents) the bias carry the same leading extents."""
    vm_harness.set_stream()
    bits, n, k = 4, 96, 512
    x, wq, s, g = O.make_case(65, 10, n, k, bits)
    rng = np.random.default_rng(6)
    bias = rng.standard_normal(n).astype(np.float16)
    res = rng.standard_normal((10, n)).astype(np.float16)
    dw, ds = _dev(wq), _dev(s)
    x3 = _dev(x).reshape(2, 5, k)
    y3 = vm_harness.call_dps("mi355x_q4f16_matmul", [x3, dw, ds], (2, 5, n))
    torch.cuda.synchronize()
    assert_close(y3.reshape(10, n).cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g), "x[2, 5, K]")
    spec = spec_for(bits, ("x", "wq", "scales", "bias", "residual", "out"), activation=lib.ACT_RELU)
    y = torch.empty((2, 5, n), dtype=torch.float16, device="cuda")
    targs = [vm_harness.TensorArg(t, as_uint32=(t.dtype == torch.int32))
             for t in (x3, dw, ds, _dev(bias).reshape(1, 1, n), _dev(res).reshape(2, 5, n), y)]
    vm_harness.call_packed("mi355x_wq_packed_call", targs, spec=spec)
    torch.cuda.synchronize()
    want = c_oracle.wq_matmul_fused(x, wq, s, bits, g, bias=bias, activation="relu", residual=res)
    assert_close(y.reshape(10, n).cpu().numpy(), want, "fused tail on x[2, 5, K]")
    # a 1-d x is one row; the gated tail halves the last extent
    y1 = vm_harness.call_dps("mi355x_q4f16_matmul", [x3[0, 0], dw, ds], (n,))
    yg = vm_harness.call_dps("mi355x_q4f16_matmul_silu_mul", [x3, dw, ds], (2, 5, n // 2))
    torch.cuda.synchronize()
    assert torch.equal(y1, y3[0, 0])
    assert yg.shape == (2, 5, n // 2)
    for bad_shape, message in (((10, n), "leading extents of x"), ((5, 2, n), "leading extents of x"), ((2, 5, n + 1), "expected")):
        with pytest.raises(PackedError, match=message):
            vm_harness.call_dps("mi355x_q4f16_matmul", [x3, dw, ds], bad_shape)
    with pytest.raises(PackedError, match="leading extents of x"):
        targs[4] = vm_harness.TensorArg(_dev(res))  # a 2-d residual beside a 3-d x
        vm_harness.call_packed("mi355x_wq_packed_call", targs, spec=spec)
    with pytest.raises(PackedError, match="compact"):
        wide = torch.zeros((2, 5, 2 * k), dtype=torch.float16, device="cuda")
        vm_harness.call_packed("mi355x_wq_packed_call",
                               [vm_harness.TensorArg(wide[:, :, :k], with_strides=True)] + targs[1:3] + [vm_harness.TensorArg(y)],
                               spec=spec_for(bits, ("x", "wq", "scales", "out")))
