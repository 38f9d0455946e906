"""Seeded random problems through every optional feature at once: caller workspace (K split of the decode
kernel and of the GEMM, wherever the library splits), tile-major weights, and each tail (bias / relu / residual,
gelu, the gated silu-mul), against the oracle.  Shapes are drawn so that a good share of them split: few column
tiles, long K.

Bar: the matmul tolerance (max-abs 1e-2 + relative 1e-2 against the oracle, taken before the tail); a call with
a workspace is deterministic; the arrival counters are back at zero after every call."""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tests.test_gpu_parity import ATOL, RTOL, _dev, _fused_operands, assert_close  # noqa: E402


def _problems(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        bits = int(rng.choice([4, 8]))
        group = 32 if bits == 4 else 128
        k = 256 * int(rng.choice([4, 8, 16, 20, 32, 43, 54]))
        m = int(rng.choice([1, 4, 8, 12, 16, 17, 24, 33, 48, 64, 65, 128, 200, 256]))
        n = int(rng.choice([500, 1000, 2040, 4096, 5120])) if m > 16 else int(rng.choice([1000, 4090, 5120]))
        out.append((bits, group, m, n, k, str(rng.choice(["none", "relu", "gelu", "silu_mul"])), bool(rng.random() < 0.4)))
    return out


@pytest.mark.parametrize("chunk", range(4))
def test_random_problems_with_workspace_layouts_and_tails(chunk):
    import relax_amd

    big = relax_amd.wq_workspace(48 << 20)
    for bits, group, m, n, k, tail, tiled in _problems(7000 + chunk, 10):
        if tail == "silu_mul":
            n -= n % 2
            tiled = False  # the gated tail reads canonical weights
        what = (bits, m, n, k, tail, tiled)
        x, wq, s, g = O.make_case(chunk * 1000 + m + n + k, m, n, k, bits, group)
        rows = np.arange(m) if m <= 32 else np.sort(np.random.default_rng(m).choice(m, 24, replace=False))
        want_plain = c_oracle.wq_matmul(x[rows], wq, s, bits, g, nthreads=16)
        bias, res = _fused_operands(m + n, m, n)
        kw = {}
        if tail == "relu":
            kw = dict(bias=_dev(bias), activation="relu", residual=_dev(res))
            want = O.epilogue(want_plain, bias, "relu", res[rows])
        elif tail == "gelu":
            kw = dict(bias=_dev(bias), activation="gelu")
            want = O.epilogue(want_plain, bias, "gelu", None)
        elif tail == "silu_mul":
            kw = dict(activation="silu_mul")
            want = O.epilogue(want_plain, None, "silu_mul", None)
        else:
            want = want_plain
        dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
        if tiled:
            dwq, ds = relax_amd.wq_tile_weights(dwq, ds, bits, g)
            kw["tiled_n"] = n
        need = relax_amd.wq_workspace_bytes(bits, g, n, k, m, tiled=tiled)
        assert need <= big.numel(), what
        try:
            y0 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, **kw)
            y1 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=big, **kw)
            y2 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=big, **kw)
        except relax_amd.lib.WqError as e:
            # the gated tail above 16 rows needs the direct-weight kernel's K and group; nothing else may refuse
            assert tail == "silu_mul" and "direct-weight" in str(e), (what, str(e))
            continue
        torch.cuda.synchronize()
        assert int(big[:16384].view(torch.int32).abs().sum()) == 0, what
        assert torch.equal(y1.view(torch.int16), y2.view(torch.int16)), what
        for y in (y0, y1):
            got = y.cpu().numpy()[rows].astype(np.float64)
            ref = want.astype(np.float64)
            mag = np.abs(want_plain.astype(np.float64))
            if tail == "silu_mul":
                half = n // 2
                mag = 2.0 * (1.0 + mag[:, :half] + mag[:, half:]) * (1.0 + np.abs(ref))
            elif tail in ("relu", "gelu"):
                mag = mag + np.abs(bias.astype(np.float64))[None, :]
            bound = 1.2 * (ATOL + RTOL * mag) + 2.0 ** -9 * (np.abs(ref) + (mag if tail != "silu_mul" else 0))
            assert np.all(np.isfinite(got)) and np.all(np.abs(got - ref) <= bound), (what, float(np.abs(got - ref).max()))


@pytest.mark.parametrize("chunk", range(3))
def test_random_call_descriptions_through_the_packed_boundary(chunk):
    """The generic PackedFunc entry with random argument orders, every activation and both scratch modes,
    against the C ABI's result for the same problem (bit for bit: it is the same kernel on the same stream)."""
    import relax_amd
    from relax_amd import vm_harness
    from relax_amd.vm_harness import CallSpec, TensorArg

    vm_harness.set_stream()
    rng = np.random.default_rng(8100 + chunk)
    for _ in range(10):
        bits = int(rng.choice([4, 8]))
        g = 32 if bits == 4 else 128
        m = int(rng.choice([1, 8, 16, 40, 130]))
        n = 2 * int(rng.integers(20, 300))
        k = 256 * int(rng.integers(1, 9))
        act = int(rng.choice([0, 1, 2, 3]))
        with_bias = act != 2 and bool(rng.random() < 0.6)
        with_res = act != 2 and bool(rng.random() < 0.5)
        x, wq, s, _ = O.make_case(int(rng.integers(1 << 20)), m, n, k, bits)
        bias, res = _fused_operands(m + n, m, n)
        out_cols = n // 2 if act == 2 else n
        out = torch.empty((m, out_cols), dtype=torch.float16, device="cuda")
        tensors = {"x": _dev(x), "wq": _dev(wq), "scales": _dev(s), "out": out}
        if with_bias:
            tensors["bias"] = _dev(bias)
        if with_res:
            tensors["residual"] = _dev(res)
        order = list(tensors)
        rng.shuffle(order)
        pos = {name: i for i, name in enumerate(order)}
        spec = CallSpec(op=0, bits=bits, group=0, zero_point=7 if bits == 4 else 0, arg_x=pos["x"], arg_wq=pos["wq"],
                        arg_scales=pos["scales"], arg_out=pos["out"], num_args=len(order),
                        arg_bias=pos.get("bias", -1), arg_residual=pos.get("residual", -1), activation=act)
        args = [TensorArg(tensors[name], as_uint32=(name == "wq")) for name in order]
        scratch = bool(rng.random() < 0.5)
        vm_harness.call_packed("mi355x_wq_packed_call_scratch" if scratch else "mi355x_wq_packed_call", args, spec=spec)
        torch.cuda.synchronize()
        name = {0: None, 1: "relu", 2: "silu_mul", 3: "gelu"}[act]
        want = relax_amd.wq_matmul(tensors["x"], tensors["wq"], tensors["scales"], bits, g,
                                   bias=tensors.get("bias"), activation=name, residual=tensors.get("residual"))
        torch.cuda.synchronize()
        what = (bits, m, n, k, name, with_bias, with_res, order, scratch)
        if scratch and m <= 16 and relax_amd.wq_workspace_bytes(bits, g, n, k, m) > 0:
            # the scratch entry splits K where the plain call does not: same tolerance, other summation order
            assert_close(out.cpu().numpy(), want.cpu().numpy(), what, ulp_fraction=0.01)
        else:
            assert torch.equal(out.view(torch.int16), want.view(torch.int16)), what
