"""GPU parity of the gated tail: y[M, N/2] = multiply(nn.silu(h[:, :N/2]), h[:, N/2:]), h = f16(x W^T).

Bar.  The kernels that fuse the tail walk the weight rows in an interleaved gate / up order but add up
every row exactly as the plain call does, so h is the plain call's output bit for bit; the tail is five
float16 operations whose only implementation-defined part is the last bit of the float32 exponential.
Hence: (1) at least 99.9 % of the outputs equal the oracle's tail applied to the plain call's output bit
for bit, the rest within 4 float16 ulp; (2) the whole result is within the matmul tolerance (max-abs
1e-2 + relative 1e-2) of the oracle's matmul followed by its tail.
"""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tests.test_gpu_parity import ATOL, RTOL, _dev  # noqa: E402


def gated_and_plain(x, wq, s, bits, g, kernel=0, variant=0):
    import relax_amd

    from relax_amd import lib

    xd, wqd, sd = _dev(x), _dev(wq), _dev(s)
    y = relax_amd.wq_matmul(xd, wqd, sd, bits, g, activation="silu_mul", kernel=kernel, variant=variant)
    # the plain output of the same kernel family (left to itself the library may pick the skinny kernel
    # for the plain call, whose float32 sums are added in another order)
    family = kernel if kernel else (lib.KERNEL_GEMV if x.shape[0] <= 16 else lib.KERNEL_GEMM)
    h = relax_amd.wq_matmul(xd, wqd, sd, bits, g, kernel=family, variant=variant)
    torch.cuda.synchronize()
    return y.cpu().numpy(), h.cpu().numpy()


def check(y, h, x, wq, s, bits, g, what, full_oracle=True):
    m, n = h.shape
    assert y.shape == (m, n // 2), what
    want = c_oracle.epilogue(h, activation="silu_mul")          # the oracle's tail on this kernel's own h
    same = y.view(np.uint16) == want.view(np.uint16)
    both_nan = np.isnan(y) & np.isnan(want)
    off = ~(same | both_nan)
    assert off.sum() <= max(1, y.size // 1000), (what, int(off.sum()), y.size)
    if off.any():
        ulp = np.maximum(np.spacing(np.abs(want[off]).astype(np.float16)).astype(np.float64), 2.0 ** -24)
        assert np.all(np.abs(y[off].astype(np.float64) - want[off].astype(np.float64)) <= 4 * ulp), what
    if full_oracle:
        ref = c_oracle.wq_matmul_fused(x, wq, s, bits, g, activation="silu_mul", nthreads=16).astype(np.float64)
        err = np.abs(y.astype(np.float64) - ref)
        # the tail multiplies two outputs: their errors add, relative to |gate * up| and to each factor
        h64 = np.abs(c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16).astype(np.float64))
        scale = 1.0 + h64[:, :n // 2] + h64[:, n // 2:]
        assert np.all(err <= (ATOL + RTOL * np.abs(ref)) * 2 * scale), (what, float(err.max()))


@pytest.mark.parametrize("variant", [0, 14, 15, 24, 25, 12, 18])
@pytest.mark.parametrize("bits,m,n,k", [(4, 1, 64, 256), (4, 8, 200, 1024), (4, 16, 48, 2048), (4, 3, 22, 352),
                                         (8, 1, 64, 256), (8, 16, 40, 640), (8, 5, 130, 384)])
def test_decode_kernel_gated_tail(variant, bits, m, n, k):
    from relax_amd import lib

    x, wq, s, g = O.make_case(900 + m + n, m, n, k, bits)
    try:
        y, h = gated_and_plain(x, wq, s, bits, g, kernel=lib.KERNEL_GEMV if variant else 0, variant=variant)
    except lib.WqError as e:
        assert variant != 0 and "does not apply" in str(e)  # two-chunk variants on K they cannot split
        return
    check(y, h, x, wq, s, bits, g, (variant, bits, m, n, k))


@pytest.mark.parametrize("variant", [0, 21, 22, 23, 24, 25])
@pytest.mark.parametrize("bits,m,n,k", [(4, 70, 136, 768), (4, 300, 200, 1024), (4, 129, 520, 1280), (4, 17, 64, 512),
                                         (8, 65, 300, 1792), (8, 513, 260, 1024)])
def test_direct_weight_gemm_gated_tail(variant, bits, m, n, k):
    from relax_amd import lib

    x, wq, s, g = O.make_case(950 + m + n, m, n, k, bits)
    try:
        y, h = gated_and_plain(x, wq, s, bits, g, kernel=lib.KERNEL_GEMM if variant else 0, variant=variant)
    except lib.WqError as e:
        assert variant != 0 and "does not apply" in str(e)
        return
    check(y, h, x, wq, s, bits, g, (variant, bits, m, n, k))


@pytest.mark.parametrize("m", [1, 8, 512])
def test_gate_up_projection_of_llama7b_at_full_size(m):
    """22016 x 4096 (11008 gate rows, 11008 up rows): the projection the tail exists for."""
    n, k = 22016, 4096
    x, wq, s, g = O.make_case(77, m, n, k, 4)
    y, h = gated_and_plain(x, wq, s, 4, g)
    if m <= 8:
        check(y, h, x, wq, s, 4, g, ("gate+up", m))
    else:
        check(y, h, x, wq, s, 4, g, ("gate+up", m), full_oracle=False)
        rows = [0, 255, 511]
        ref = c_oracle.wq_matmul_fused(x[rows], wq, s, 4, g, activation="silu_mul", nthreads=16).astype(np.float64)
        assert np.all(np.abs(y[rows].astype(np.float64) - ref) <= 4 * (ATOL + RTOL * np.abs(ref)))


def test_gated_tail_through_the_packed_entry_and_what_it_refuses():
    import relax_amd
    from relax_amd import lib, vm_harness

    vm_harness.set_stream()
    x, wq, s, g = O.make_case(5, 4, 96, 512, 4)
    xd, wqd, sd = _dev(x), _dev(wq), _dev(s)
    y = vm_harness.call_dps("mi355x_q4f16_matmul_silu_mul", [xd, wqd, sd], (4, 48))
    direct = relax_amd.wq_matmul(xd, wqd, sd, 4, g, activation="silu_mul")
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), direct.view(torch.int16))
    with pytest.raises(vm_harness.PackedError, match="expected \\(4, 48\\)"):
        vm_harness.call_dps("mi355x_q4f16_matmul_silu_mul", [xd, wqd, sd], (4, 96))
    bias = torch.zeros(96, dtype=torch.float16, device="cuda")
    with pytest.raises(lib.WqError, match="no bias and no residual"):
        relax_amd.wq_matmul(xd, wqd, sd, 4, g, activation="silu_mul", bias=bias)
    with pytest.raises(lib.WqError, match="not implemented by the skinny kernel"):
        relax_amd.wq_matmul(xd, wqd, sd, 4, g, activation="silu_mul", kernel=lib.KERNEL_SKINNY)
    x2, wq2, s2, g2 = O.make_case(6, 2, 33, 256, 4)
    with pytest.raises(lib.WqError, match="even N"):
        relax_amd.wq_matmul(_dev(x2), _dev(wq2), _dev(s2), 4, g2, activation="silu_mul")
    x3, wq3, s3, g3 = O.make_case(7, 100, 64, 352, 4)  # M > 64 needs the direct-weight kernel: K % 256 == 0
    with pytest.raises(lib.WqError, match="needs the direct-weight kernel"):
        relax_amd.wq_matmul(_dev(x3), _dev(wq3), _dev(s3), 4, g3, activation="silu_mul")
    wt, st = relax_amd.wq_tile_weights(wqd, sd, 4, g)
    with pytest.raises(lib.WqError, match="canonical weights only"):
        relax_amd.wq_matmul(xd, wt, st, 4, g, activation="silu_mul", tiled_n=96)
