"""GPU parity of the gelu tail: y = [f16(x W^T) + bias] -> nn.gelu -> [+ residual].

Bar.  gelu is the float16 operation sequence x * (0.5 + erf(x * sqrt(0.5)) * 0.5) whose only
implementation-defined part is the last bit of the float32 erf.  Hence: (1) at least 99.9 % of the outputs
equal the oracle's tail applied to the same kernel's plain output bit for bit, the rest within |x| * 2^-10
plus one float16 ulp (one ulp of e moves c by at most 2^-11 after its own rounding); (2) the whole result is
within the matmul tolerance (max-abs 1e-2 + relative 1e-2, taken before the tail) of the oracle's fused result
-- gelu's slope is at most 1.13, so the tolerance carries over.
"""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tests.test_gpu_parity import ATOL, RTOL, FUSED_SHAPES, _fused_operands, run_fused, run_matmul  # noqa: E402


def check(got, got_plain, want_plain, bias, res, what):
    pre = got_plain if bias is None else O.add_f16(got_plain, bias.reshape(1, -1))
    want = O.epilogue(got_plain, bias, "gelu", res)
    off = got.view(np.uint16) != want.view(np.uint16)
    assert off.sum() <= max(1, got.size // 1000), (what, int(off.sum()), got.size)
    if off.any():
        ulp = np.spacing(np.abs(want[off]).astype(np.float16)).astype(np.float64)
        slack = np.abs(pre[off].astype(np.float64)) * 2.0 ** -10 + ulp
        assert np.all(np.abs(got[off].astype(np.float64) - want[off].astype(np.float64)) <= slack), what
    ref = O.epilogue(want_plain, bias, "gelu", res).astype(np.float64)
    mag = np.abs(want_plain.astype(np.float64)) + (0 if bias is None else np.abs(bias.astype(np.float64))[None, :])
    bound = 1.13 * (ATOL + RTOL * mag) + 2.0 ** -9 * (np.abs(ref) + mag)
    err = np.abs(got.astype(np.float64) - ref)
    assert np.all(np.isfinite(got)) and np.all(err <= bound), (what, float(err.max()))


@pytest.mark.parametrize("tail", ["bias_gelu", "gelu", "bias_gelu_residual"])
@pytest.mark.parametrize("bits,m,n,k", FUSED_SHAPES)
def test_gelu_tail_every_kernel_family(bits, m, n, k, tail):
    x, wq, s, g = O.make_case(1700 + m + n, m, n, k, bits)
    b, r = _fused_operands(m * 5 + n, m, n)
    bias = b if "bias" in tail else None
    res = r if "residual" in tail else None
    got_plain = run_matmul(x, wq, s, bits, g)
    got = run_fused(x, wq, s, bits, g, bias, "gelu", res)
    want_plain = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    check(got, got_plain, want_plain, bias, res, (tail, bits, m, n, k))


@pytest.mark.parametrize("kernel,variant,bits,m,n,k", [
    ("GEMV", 14, 4, 3, 40, 352), ("GEMV", 25, 4, 1, 64, 1024), ("SKINNY", 1, 4, 20, 40, 256),
    ("GEMM", 1, 4, 70, 136, 448), ("GEMM", 11, 4, 300, 200, 128), ("GEMM", 21, 4, 129, 520, 1280),
    ("GEMM", 22, 8, 65, 300, 1792), ("GEMM", 24, 4, 256, 512, 768), ("GEMM", 25, 4, 128, 256, 1280),
])
def test_gelu_tail_explicit_kernel_variants(kernel, variant, bits, m, n, k):
    from relax_amd import lib

    fam = getattr(lib, "KERNEL_" + kernel)
    x, wq, s, g = O.make_case(1800 + m + n, m, n, k, bits)
    bias, res = _fused_operands(m + 3 * n, m, n)
    got_plain = run_matmul(x, wq, s, bits, g, kernel=fam, variant=variant)
    got = run_fused(x, wq, s, bits, g, bias, "gelu", res, kernel=fam, variant=variant)
    want_plain = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    check(got, got_plain, want_plain, bias, res, (kernel, variant, bits, m, n, k))


def test_gelu_on_every_float16_value_through_the_kernel():
    """One-hot activations read the dequantized weights back; with unit scales and a bias sweeping all
    float16 values the tail sees every input: the device's erf against the oracle's on all of them."""
    import relax_amd

    h = np.arange(65536, dtype=np.uint16).view(np.float16)
    vals = h[np.isfinite(h)]
    n = vals.size
    k = 128
    x = np.zeros((1, k), dtype=np.float16)
    # all-zero int8 weights: the accumulator is 0, the tail's input is the bias itself
    wq = np.zeros((n, k // 4), dtype=np.uint32)
    s = np.ones((n, 1), dtype=np.float16)
    got = run_fused(x, wq, s, 8, 128, vals, "gelu", None)
    want = O.gelu_f16(vals.reshape(1, -1))
    off = got.view(np.uint16) != want.view(np.uint16)
    assert off.sum() <= n // 1000, int(off.sum())
    ulp = np.spacing(np.abs(want[off]).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(got[off].astype(np.float64) - want[off].astype(np.float64)) <=
                  np.abs(vals.reshape(1, -1)[off].astype(np.float64)) * 2.0 ** -10 + ulp)


def test_packed_bias_gelu_entry():
    """mi355x_q4f16_matmul_bias_gelu called the way the VM calls a PackedFunc."""
    from relax_amd import vm_harness
    from tests.test_gpu_parity import _dev

    bits, m, n, k = 4, 8, 96, 512
    x, wq, s, g = O.make_case(1901, m, n, k, bits)
    bias, _ = _fused_operands(5, m, n)
    vm_harness.set_stream()
    out = vm_harness.call_dps("mi355x_q4f16_matmul_bias_gelu", [_dev(x), _dev(wq), _dev(s), _dev(bias)], (m, n))
    torch.cuda.synchronize()
    plain = run_matmul(x, wq, s, bits, g)
    check(out.cpu().numpy(), plain, c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), bias, None, "packed")


@pytest.mark.parametrize("bits,m,n,k", [(4, 8, 200, 1024), (4, 40, 72, 256), (4, 300, 520, 512), (8, 129, 260, 1024)])
def test_gelu_with_the_residual_in_the_output_buffer(bits, m, n, k):
    """y = gelu(x W^T + b) + y in place.  Above 64 rows the direct-weight kernel applies gelu in a pass of its
    own, which an in-place residual rules out: the library then runs the kernels that fuse the whole tail."""
    import relax_amd
    from relax_amd import lib
    from tests.test_gpu_parity import _dev

    x, wq, s, g = O.make_case(2000 + m, m, n, k, bits)
    bias, res = _fused_operands(m + n, m, n)
    h = _dev(res).clone()
    relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, g, bias=_dev(bias), activation="gelu", residual=h, out=h)
    torch.cuda.synchronize()
    # the plain output of the kernel that ran: the LDS-staged pipeline above 64 rows, the default one otherwise
    fam, var = (lib.KERNEL_GEMM, 12) if m > 64 else (0, 0)
    got_plain = run_matmul(x, wq, s, bits, g, kernel=fam, variant=var)
    check(h.cpu().numpy(), got_plain, c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), bias, res, ("in place", bits, m))
    if m > 64:
        with pytest.raises(lib.WqError, match="buffer of its own"):
            relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, g, bias=_dev(bias), activation="gelu", residual=h,
                                out=h, kernel=lib.KERNEL_GEMM, variant=21)


@pytest.mark.parametrize("bits,m,n,k", [(4, 300, 520, 512), (8, 129, 260, 1024), (4, 600, 136, 768)])
def test_gelu_in_place_on_tile_major_weights(bits, m, n, k):
    """The same on tile-major weights, which only the direct-weight and the register-activation kernel read: the
    rows run through the latter, which fuses gelu, in blocks of as many rows as it takes.  (A module with bound
    weights converts them to this layout when it loads.)"""
    import relax_amd
    from tests.test_gpu_parity import _dev

    x, wq, s, g = O.make_case(2100 + m, m, n, k, bits)
    bias, res = _fused_operands(m + n + 1, m, n)
    wt, st = relax_amd.wq_tile_weights(_dev(wq), _dev(s), bits, g)
    h = _dev(res).clone()
    relax_amd.wq_matmul(_dev(x), wt, st, bits, g, bias=_dev(bias), activation="gelu", residual=h, out=h, tiled_n=n)
    torch.cuda.synchronize()
    want = c_oracle.wq_matmul_fused(x, wq, s, bits, g, bias=bias, activation="gelu", residual=res, nthreads=16).astype(np.float64)
    err = np.abs(h.cpu().numpy().astype(np.float64) - want)
    assert np.all(err <= 1.5 * (ATOL + RTOL * np.abs(want)) + 2.0 ** -9 * np.abs(want)), (bits, m, float(err.max()))
    # and with the residual in a buffer of its own the same values come out (two passes on the direct-weight kernel)
    sep = relax_amd.wq_matmul(_dev(x), wt, st, bits, g, bias=_dev(bias), activation="gelu", residual=_dev(res), tiled_n=n)
    torch.cuda.synchronize()
    err2 = np.abs(sep.cpu().numpy().astype(np.float64) - want)
    assert np.all(err2 <= 1.5 * (ATOL + RTOL * np.abs(want)) + 2.0 ** -9 * np.abs(want)), (bits, m, float(err2.max()))


def test_tail_golden_fixtures():
    """The committed fixtures of the gelu and gated tails: at least 99.9 % of the outputs equal the fixture's tail
    applied to this kernel's own matmul output bit for bit, and everything within the matmul tolerance of the fixture."""
    import glob
    import os

    import relax_amd
    from relax_amd import lib
    from tests.test_gpu_parity import _dev

    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "tail_*.npz")))
    assert len(files) >= 2
    for f in files:
        z = np.load(f)
        bits, g, act = int(z["bits"]), int(z["group"]), str(z["activation"])
        bias = z["bias"] if "bias" in z.files else None
        m = z["x"].shape[0]
        fam = lib.KERNEL_GEMV if m <= 16 else lib.KERNEL_GEMM
        dx, dwq, ds = _dev(z["x"]), _dev(z["wq"]), _dev(z["scales"])
        h = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=fam).cpu().numpy()
        got = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=fam, bias=None if bias is None else _dev(bias),
                                  activation=act).cpu().numpy()
        own = O.epilogue(h, bias, act, None)
        assert (got.view(np.uint16) != own.view(np.uint16)).sum() <= max(1, got.size // 1000), f
        err = np.abs(got.astype(np.float64) - z["y"].astype(np.float64))
        mag = np.abs(z["y_plain"].astype(np.float64))
        if act == "silu_mul":
            half = mag.shape[1] // 2
            mag = 2.0 * (1.0 + mag[:, :half] + mag[:, half:]) * (1.0 + np.abs(z["y"].astype(np.float64)))
        assert np.all(err <= 1.2 * (ATOL + RTOL * mag) + 2.0 ** -9 * np.abs(z["y"].astype(np.float64))), (f, float(err.max()))
