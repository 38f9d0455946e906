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
