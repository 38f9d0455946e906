"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle.

Bar: integer unpack + dequantized weights bit-exact; float16 outputs within
max-abs 1e-2 and relative 1e-2 of the oracle (float32 accumulation in a
different order is the only permitted difference).
"""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

ATOL = 1e-2
RTOL = 1e-2


def _dev(a: np.ndarray):
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    return torch.from_numpy(a).cuda()


def assert_close(got: np.ndarray, want: np.ndarray, what="", ulp_fraction=0.001):
    got64, want64 = got.astype(np.float64), want.astype(np.float64)
    assert got.shape == want.shape, what
    assert np.all(np.isfinite(got64)), what
    err = np.abs(got64 - want64)
    bound = ATOL + RTOL * np.abs(want64)
    worst = int(np.argmax(err - bound))
    assert np.all(err <= bound), (what, float(err.flat[worst]), float(want64.flat[worst]))
    # the tolerance above is the contract; the kernels are expected to sit within ~1 float16 ulp
    ulp = np.maximum(np.abs(want64), 2.0**-14) * 2.0**-10
    # (an output much smaller than the terms it sums can be off by more: the float32 accumulation
    # error is absolute; allow 0.1 % of the outputs, and two of them in small cases)
    off = int(np.sum(err > 1.01 * ulp + 1e-6))
    assert off <= max(2, int(got.size * ulp_fraction)), (what, "%d outputs off by > 1 ulp" % off)


def run_matmul(x, wq, s, bits, group, kernel=0, variant=0):
    import relax_amd

    y = relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, group, kernel=kernel, variant=variant)
    torch.cuda.synchronize()
    return y.cpu().numpy()


# ------------------------------------------------------------------ dequantize: bit exact
@pytest.mark.parametrize("bits,n,k", [(4, 64, 256), (4, 37, 352), (4, 4096, 4096), (8, 64, 256),
                                       (8, 21, 384), (8, 5120, 5120)])
def test_dequantize_bit_exact(bits, n, k):
    import relax_amd

    _, wq, s, g = O.make_case(10 + bits, 1, n, k, bits)
    wd = relax_amd.wq_dequantize(_dev(wq), _dev(s), bits, g)
    torch.cuda.synchronize()
    want = c_oracle.dequant(wq, s, bits, g, nthreads=8)
    assert np.array_equal(wd.cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("bits,group,n,k", [
    (4, 32, 1, 32), (4, 32, 3, 8224), (4, 32, 257, 2080),      # the quad kernel: one quad, ragged last wavefronts
    (8, 128, 1, 128), (8, 128, 9, 8320), (8, 128, 130, 1152),
    (4, 64, 33, 4096), (4, 128, 7, 256), (4, 256, 5, 2304),     # other groups: one lane per 8 weights, rows of
    (8, 32, 5, 96), (8, 64, 19, 2112), (8, 16, 3, 48),          # more and of fewer than 256 units
])
def test_dequantize_groups_and_ragged_ends(bits, group, n, k):
    """Both dequantize kernels: the quad-per-lane one of the two standard quantizations at sizes that end inside a
    wavefront, and the general one at other group sizes, on rows longer and shorter than a workgroup's span."""
    import relax_amd

    _, wq, s, g = O.make_case(300 + n + k, 1, n, k, bits, group)
    wd = relax_amd.wq_dequantize(_dev(wq), _dev(s), bits, g)
    torch.cuda.synchronize()
    want = c_oracle.dequant(wq, s, bits, g, nthreads=8)
    assert np.array_equal(wd.cpu().numpy().view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("bits", [4, 8])
def test_dequantize_every_field_value_and_special_scales(bits):
    """All field values against scales that give zeros, subnormals, the largest finite value and inf."""
    import relax_amd

    g = 32 if bits == 4 else 128
    special = np.array([0.0, -0.0, 1.0, -1.0, 6e-8, 1e-5, 6.1e-5, 0.0123, 511.75, 8188.0, 65504.0, np.inf],
                       dtype=np.float16)
    n, groups = 16 if bits == 4 else 256, special.size
    if bits == 4:
        w = np.repeat(np.arange(16)[:, None], groups * g, axis=1)
        wq = O.pack_q4(w)
    else:
        w = np.repeat((np.arange(256) - 128)[:, None], groups * g, axis=1)
        wq = O.pack_q8(w)
    s = np.repeat(special[None, :], n, axis=0)
    got = relax_amd.wq_dequantize(_dev(wq), _dev(s), bits, g).cpu().numpy()
    want = O.dequant(wq, s, bits, g)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])


# ------------------------------------------------------------------ GEMV kernel (activations staged in LDS)
GEMV_SHAPES = [
    (4, 1, 64, 256), (4, 1, 40, 352), (4, 3, 16, 32), (4, 8, 200, 1024), (4, 16, 48, 2048),
    (4, 5, 33, 1152), (4, 2, 24, 11008),
    (8, 1, 64, 256), (8, 2, 40, 384), (8, 16, 24, 128), (8, 7, 72, 640), (8, 4, 16, 1280),
]


GEMV_VARIANTS = [wpc * 10 + shape for wpc in (1, 2, 4) for shape in range(1, 9)]  # workgroups per CU x kernel shape


@pytest.mark.parametrize("variant", GEMV_VARIANTS)
def test_gemv_kernel_variants_match_oracle(variant):
    """Every tuning variant on every shape it accepts (a variant that needs K to be a multiple of
    its super step, or more LDS than a CU has, refuses with an error, which is checked to be that)."""
    from relax_amd import lib

    ran = 0
    for bits, m, n, k in GEMV_SHAPES:
        x, wq, s, g = O.make_case(300 + m + n, m, n, k, bits)
        try:
            got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_GEMV, variant=variant)
        except lib.WqError as e:
            assert "does not apply" in str(e)
            continue
        ran += 1
        want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=8)
        assert_close(got, want, (variant, bits, m, n, k))
    assert ran >= 2


@pytest.mark.parametrize("bits,m,n,k", [(4, 16, 4112, 4096), (4, 12, 1000, 11008), (8, 16, 520, 13824)])
def test_gemv_k_phases_when_activations_exceed_lds(bits, m, n, k):
    """M*K too large for one LDS staging pass: K is walked in phases with per-wavefront partial tiles."""
    from relax_amd import lib

    x, wq, s, g = O.make_case(17, m, n, k, bits)
    got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_GEMV)
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    assert_close(got, want, (bits, m, n, k))


@pytest.mark.parametrize("m", [1, 8])
def test_vocabulary_sized_projection(m):
    """N = 152064 (an lm_head): more row tiles per workgroup than the GEMV kernel's LDS slots hold, so the
    default dispatch uses the register-activation kernel; forcing the GEMV family is refused."""
    from relax_amd import lib

    n, k = 152064, 1024
    x, wq, s, g = O.make_case(19, m, n, k, 4)
    got = run_matmul(x, wq, s, 4, g)
    want = c_oracle.wq_matmul(x, wq, s, 4, g, nthreads=16)
    assert_close(got, want, ("lm_head", m))
    with pytest.raises(lib.WqError, match="does not apply"):
        run_matmul(x, wq, s, 4, g, kernel=lib.KERNEL_GEMV)


def test_gemv_refuses_more_than_16_rows():
    from relax_amd import lib

    x, wq, s, g = O.make_case(1, 17, 16, 256, 4)
    with pytest.raises(lib.WqError, match="outside 1..16"):
        run_matmul(x, wq, s, 4, g, kernel=lib.KERNEL_GEMV)
    assert_close(run_matmul(x, wq, s, 4, g), c_oracle.wq_matmul(x, wq, s, 4, g), "auto uses another family")


# ------------------------------------------------------------------ skinny kernel (activations in registers)
SKINNY_VARIANTS = [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11]


@pytest.mark.parametrize("variant", SKINNY_VARIANTS)
@pytest.mark.parametrize("bits,m,n,k", [
    (4, 1, 64, 256), (4, 1, 40, 352), (4, 3, 16, 32), (4, 8, 200, 1024), (4, 16, 48, 2048),
    (4, 17, 33, 352), (4, 33, 64, 512), (4, 64, 80, 1152),
    (8, 1, 64, 256), (8, 2, 40, 384), (8, 16, 24, 128), (8, 20, 72, 640), (8, 64, 16, 1280),
])
def test_skinny_kernel_matches_oracle(variant, bits, m, n, k):
    from relax_amd import lib

    x, wq, s, g = O.make_case(100 + m + n, m, n, k, bits)
    got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_SKINNY, variant=variant)
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=8)
    assert_close(got, want, (variant, bits, m, n, k))


@pytest.mark.parametrize("variant", [21, 22, 25, 26, 27, 28, 31])
@pytest.mark.parametrize("bits,m,n,k", [
    (4, 17, 33, 352), (4, 33, 64, 512), (4, 64, 80, 1152), (4, 48, 4096, 4096), (4, 31, 1000, 11008),
    (8, 20, 72, 640), (8, 64, 16, 1280), (8, 33, 5120, 5120), (8, 50, 300, 13824),
])
def test_skinny_kernel_with_staged_activations(variant, bits, m, n, k):
    """Variants 21 ...: the activations of a k-step loaded line by line and handed to the operand lanes through
    LDS.  The MFMAs see the same operands in the same order as in the direct variants: bit-equal to them, on both
    weight layouts, and within tolerance of the oracle.  One row block (M <= 16) has no staged build."""
    import relax_amd
    from relax_amd import lib

    x, wq, s, g = O.make_case(150 + m + n, m, n, k, bits)
    got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_SKINNY, variant=variant)
    direct = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_SKINNY, variant=variant - 20)
    assert np.array_equal(got.view(np.uint16), direct.view(np.uint16))
    assert_close(got, c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (variant, bits, m, n, k), ulp_fraction=0.005)
    if k % 256 == 0:
        wt, st = relax_amd.wq_tile_weights(_dev(wq), _dev(s), bits, g)
        tiled = relax_amd.wq_matmul(_dev(x), wt, st, bits, g, tiled_n=n, kernel=lib.KERNEL_SKINNY, variant=variant)
        torch.cuda.synchronize()
        assert np.array_equal(tiled.cpu().numpy().view(np.uint16), got.view(np.uint16))
    # one row block: the same builds, bit-equal to the direct form as well
    few = run_matmul(x[:8], wq, s, bits, g, kernel=lib.KERNEL_SKINNY, variant=variant)
    few_direct = run_matmul(x[:8], wq, s, bits, g, kernel=lib.KERNEL_SKINNY, variant=variant - 20)
    assert np.array_equal(few.view(np.uint16), few_direct.view(np.uint16))


@pytest.mark.parametrize("bits,m,n,k", [
    (4, 65, 4096, 4096), (4, 96, 200, 1280), (4, 128, 2048, 8192), (4, 81, 33, 352), (4, 112, 1000, 11008),
    (8, 80, 5120, 5120), (8, 128, 300, 2304), (8, 97, 72, 640), (8, 66, 5120, 13824),
    (8, 192, 5120, 5120), (8, 161, 200, 1280), (4, 256, 2048, 8192), (4, 200, 136, 768), (8, 250, 40, 384),
])
def test_skinny_kernel_in_row_slices(bits, m, n, k):
    """65 .. 256 rows: the register-activation kernel runs the rows as two to four grid slices of whole 16-row
    blocks (81 rows: 48 + 33).  Forced and, where the selection picks it, by default; against the oracle, bit-equal on
    tile-major weights, and with a fused tail whose residual and output rows belong to the second slice too."""
    import relax_amd
    from relax_amd import lib

    x, wq, s, g = O.make_case(170 + m + n, m, n, k, bits)
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_SKINNY)
    assert_close(got, want, ("sliced", bits, m, n, k), ulp_fraction=0.005)
    if lib.load().mi355x_wq_select_kernel(lib.make_desc(bits, g, n, k), m) == lib.KERNEL_SKINNY:
        assert np.array_equal(run_matmul(x, wq, s, bits, g).view(np.uint16), got.view(np.uint16))
    if k % 256 == 0:
        wt, st = relax_amd.wq_tile_weights(_dev(wq), _dev(s), bits, g)
        tiled = relax_amd.wq_matmul(_dev(x), wt, st, bits, g, tiled_n=n, kernel=lib.KERNEL_SKINNY)
        torch.cuda.synchronize()
        assert np.array_equal(tiled.cpu().numpy().view(np.uint16), got.view(np.uint16))
    rng = np.random.default_rng(m + n)
    bias = rng.standard_normal(n).astype(np.float16)
    res = rng.standard_normal((m, n)).astype(np.float16)
    fused = relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, g, kernel=lib.KERNEL_SKINNY, bias=_dev(bias),
                                activation="relu", residual=_dev(res))
    torch.cuda.synchronize()
    want_f = c_oracle.wq_matmul_fused(x, wq, s, bits, g, bias=bias, activation="relu", residual=res, nthreads=16)
    assert_close(fused.cpu().numpy(), want_f, ("sliced fused", bits, m, n, k), ulp_fraction=0.005)


def test_config1_single_gemv_4096():
    """The reference's CPU-runnable case: x[1,4096] ~ N(0,1), W int4 4096x4096, group 32, zero point 7."""
    x, wq, s, g = O.make_case(0, 1, 4096, 4096, 4)
    got = run_matmul(x, wq, s, 4, g)
    want = c_oracle.wq_matmul(x, wq, s, 4, g, nthreads=8)
    assert_close(got, want, "config 1")


@pytest.mark.parametrize("m", [1, 8])
@pytest.mark.parametrize("n,k", [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)])
def test_config2_llama7b_decode_projections(m, n, k):
    x, wq, s, g = O.make_case(2, m, n, k, 4)
    got = run_matmul(x, wq, s, 4, g)
    want = c_oracle.wq_matmul(x, wq, s, 4, g, nthreads=16)
    assert_close(got, want, ("config 2", m, n, k))


@pytest.mark.parametrize("m", [1, 16])
@pytest.mark.parametrize("n,k", [(15360, 5120), (5120, 5120), (27648, 5120), (5120, 13824)])
def test_config4_q8_llama13b_skinny(m, n, k):
    x, wq, s, g = O.make_case(4, m, n, k, 8)
    got = run_matmul(x, wq, s, 8, g)
    want = c_oracle.wq_matmul(x, wq, s, 8, g, nthreads=16)
    assert_close(got, want, ("config 4", m, n, k))


# ------------------------------------------------------------------ GEMM kernel
@pytest.mark.parametrize("bits,m,n,k", [
    (4, 65, 128, 64), (4, 128, 128, 512), (4, 200, 200, 352), (4, 300, 72, 96), (4, 1, 16, 32),
    (8, 65, 128, 64), (8, 129, 136, 384), (8, 256, 256, 1152), (8, 7, 40, 16 * 9),
])
def test_gemm_kernel_matches_oracle(bits, m, n, k):
    from relax_amd import lib

    group = (32 if bits == 4 else 16) if k % 128 else None
    x, wq, s, g = O.make_case(200 + m + n, m, n, k, bits, group)
    got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_GEMM)
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=8)
    assert_close(got, want, (bits, m, n, k))


@pytest.mark.parametrize("variant,bits,m,n,k", [
    (21, 4, 300, 200, 256), (21, 4, 129, 520, 1280), (21, 8, 129, 72, 256), (21, 8, 513, 260, 1024),
    (22, 4, 300, 200, 512), (22, 4, 129, 520, 1280), (22, 4, 70, 136, 768), (22, 8, 513, 260, 1024),
    (22, 8, 65, 300, 1792),
    (23, 4, 300, 200, 256), (23, 4, 65, 520, 1280), (23, 8, 129, 72, 256), (23, 8, 513, 260, 1024),
    (24, 4, 300, 200, 512), (24, 4, 65, 520, 1280), (24, 4, 70, 136, 768), (24, 8, 513, 260, 1024),
    (24, 8, 100, 64, 1792),
    (25, 4, 300, 200, 1024), (25, 4, 65, 520, 1280), (25, 4, 70, 136, 2304), (25, 8, 513, 260, 1024),
    (25, 8, 100, 64, 1792),
    (27, 8, 129, 72, 256), (27, 8, 513, 260, 1024), (28, 8, 513, 260, 1024), (28, 8, 100, 64, 1792),
    (29, 8, 513, 260, 1024), (29, 8, 100, 64, 1792), (27, 4, 300, 200, 256)])
def test_gemm_direct_weight_variants_match_oracle(variant, bits, m, n, k):
    """Direct-weight kernel, 128-row tiles with one (21) and two (22) K groups, 64-row tiles (23, 24) and
    64 x 128 tiles with four K groups (25); 27 - 29: the 64-row builds with every lane loading its own row's pieces
    (23 - 25 load int8 weights in the canonical layout by whole cache lines through LDS):
    ragged M and N, K of one macro step, an even and an odd number of 256-wide macro steps (the second
    K group is then the shorter one)."""
    from relax_amd import lib

    x, wq, s, g = O.make_case(500 + m + n, m, n, k, bits)
    got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_GEMM, variant=variant)
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    assert_close(got, want, (variant, bits, m, n, k))


@pytest.mark.parametrize("m,n,k", [(256, 5120, 5120), (200, 5000, 1024), (64, 130, 512), (256, 15360, 5120),
                                   (100, 5120, 13824), (256, 264, 2048), (33, 64, 1024), (65, 1, 256), (70, 4097, 768)])
def test_gemm_line_wise_weight_loads_equal_the_direct_ones(m, n, k):
    """int8 weights in the canonical layout, 64-row tiles: the builds that load whole cache lines of the weight rows
    and hand the pieces to the lanes through wavefront-private LDS (variants 23 - 25) against the builds in which
    every lane loads its own pieces (27 - 29).  Same lanes, same registers, same order of additions: bit for bit,
    with the fused tails and on a ragged N (the last rows clamped), a single row and K of one and two macro steps."""
    import relax_amd
    from relax_amd import lib

    x, wq, s, g = O.make_case(8800 + m + n + k, m, n, k, 8)
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    bias = _dev(np.linspace(-1, 1, n).astype(np.float16))
    res = _dev(np.full((m, n), 0.25, dtype=np.float16))
    ran = 0
    for hop, direct in ((23, 27), (24, 28), (25, 29)):
        for kw in ({}, {"bias": bias, "activation": "relu", "residual": res}):
            try:
                ya = relax_amd.wq_matmul(dx, dwq, ds, 8, g, kernel=lib.KERNEL_GEMM, variant=direct, **kw)
            except lib.WqError:
                continue  # (K too short for the K groups of this variant)
            yb = relax_amd.wq_matmul(dx, dwq, ds, 8, g, kernel=lib.KERNEL_GEMM, variant=hop, **kw)
            torch.cuda.synchronize()
            assert torch.equal(ya.view(torch.int16), yb.view(torch.int16)), (m, n, k, hop, sorted(kw))
            ran += 1
    assert ran >= 2
    if n % 2 == 0:
        # the gated tail walks the weight rows in the interleaved gate / up order
        ya = relax_amd.wq_matmul(dx, dwq, ds, 8, g, kernel=lib.KERNEL_GEMM, variant=27, activation="silu_mul")
        yb = relax_amd.wq_matmul(dx, dwq, ds, 8, g, kernel=lib.KERNEL_GEMM, variant=23, activation="silu_mul")
        torch.cuda.synchronize()
        assert torch.equal(ya.view(torch.int16), yb.view(torch.int16)), (m, n, k, "gated")


@pytest.mark.parametrize("bits,m,n,k", [(4, 600, 15323, 512), (8, 1000, 8200, 768)])
def test_gemm_whole_rounds_plus_half_height_rest(bits, m, n, k):
    """Variant 26, the default when it applies: the column tiles that fill whole rounds of the CUs as
    128 x 256 tiles, the rest as 64 x 256 tiles in a second launch.  Same arithmetic per output as
    variant 22 (bit-equal), ragged M and N, canonical and tile-major weights."""
    import relax_amd
    from relax_amd import lib

    x, wq, s, g = O.make_case(600 + m, m, n, k, bits)
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    y26 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=lib.KERNEL_GEMM, variant=26)
    y22 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=lib.KERNEL_GEMM, variant=22)
    auto = relax_amd.wq_matmul(dx, dwq, ds, bits, g)
    wq_t, s_t = relax_amd.wq_tile_weights(dwq, ds, bits, g)
    t26 = relax_amd.wq_matmul(dx, wq_t, s_t, bits, g, kernel=lib.KERNEL_GEMM, variant=26, tiled_n=n)
    torch.cuda.synchronize()
    for other in (y22, auto, t26):
        assert torch.equal(y26.view(torch.int16), other.view(torch.int16))
    assert_close(y26.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (26, bits, m, n, k))
    # where the rest would be more than half a round the variant declines
    x2, wq2, s2, _ = O.make_case(601, 256, 256, 512, bits)
    with pytest.raises(lib.WqError, match="does not apply"):
        run_matmul(x2, wq2, s2, bits, g, kernel=lib.KERNEL_GEMM, variant=26)


def test_gemm_direct_weight_variant_refuses_other_layouts():
    """K not a multiple of 256 or a non-default group size: the variant refuses, the default dispatch
    falls back to another GEMM kernel with the same result."""
    from relax_amd import lib

    for bits, m, n, k, group in [(4, 200, 96, 320, 32), (4, 200, 96, 512, 64), (8, 200, 96, 512, 64)]:
        x, wq, s, g = O.make_case(9, m, n, k, bits, group)
        for variant in (21, 22, 23, 24, 25):
            with pytest.raises(lib.WqError, match="does not apply"):
                run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_GEMM, variant=variant)
        assert_close(run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_GEMM),
                     c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=8), (bits, m, n, k, group))


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 11, 12, 13])
@pytest.mark.parametrize("bits,m,n,k", [(4, 300, 200, 128), (4, 70, 136, 448), (4, 513, 72, 320),
                                         (8, 129, 72, 256), (8, 513, 260, 1024)])
def test_gemm_tile_variants_match_oracle(variant, bits, m, n, k):
    """Generic (1-6) and software-pipelined (11-13) tile shapes, ragged M and N, odd and even k-step counts."""
    from relax_amd import lib

    x, wq, s, g = O.make_case(400 + m + n, m, n, k, bits)
    got = run_matmul(x, wq, s, bits, g, kernel=lib.KERNEL_GEMM, variant=variant)
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    assert_close(got, want, (variant, bits, m, n, k))


def test_gemm_pipelined_variant_refuses_k_not_multiple_of_64():
    from relax_amd import lib

    x, wq, s, g = O.make_case(1, 70, 32, 96, 4)
    with pytest.raises(lib.WqError, match="does not apply"):
        run_matmul(x, wq, s, 4, g, kernel=lib.KERNEL_GEMM, variant=11)
    assert_close(run_matmul(x, wq, s, 4, g, kernel=lib.KERNEL_GEMM), c_oracle.wq_matmul(x, wq, s, 4, g), "generic")


@pytest.mark.parametrize("bits,m,n,k",
                         [(4, m, n, k) for m in (512, 2048)
                          for n, k in ((12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008))] +
                         [(8, 256, n, k) for n, k in ((15360, 5120), (5120, 5120), (27648, 5120), (5120, 13824))])
def test_gemm_full_size_rows_against_oracle_and_all_tiles_against_torch(bits, m, n, k):
    """Every prefill shape of the q4f16 configuration (M = 512 and 2048 on the four Llama-2-7B
    projections) and of the q8f16 configuration at M = 256 (the four Llama-2-13B projections), at full
    size: a sample of rows against the oracle (seconds on the host), and every output tile against a
    float32 torch matmul of the bit-exact dequantized weights."""
    import relax_amd

    x, wq, s, g = O.make_case(3, m, n, k, bits)
    xd, wqd, sd = _dev(x), _dev(wq), _dev(s)
    y = relax_amd.wq_matmul(xd, wqd, sd, bits, g)
    wd = relax_amd.wq_dequantize(wqd, sd, bits, g)
    ref = (xd.float() @ wd.float().T)
    torch.cuda.synchronize()
    err = (y.float() - ref).abs()
    bound = ATOL + RTOL * ref.abs()
    assert bool((err <= bound).all()), float((err - bound).max())
    rows = np.random.default_rng(5).choice(m, size=4, replace=False)
    want = c_oracle.wq_matmul(x[rows], wq, s, bits, g, nthreads=16)
    assert_close(y.cpu().numpy()[rows], want, ("rows", bits, m, n, k))


# ------------------------------------------------------------------ properties at full size
def test_one_hot_rows_read_back_dequantized_weights_full_size():
    """x = e_j: y[r, :] must equal column j of the dequantized weights exactly (no accumulation)."""
    import relax_amd

    n, k = 22016, 4096
    _, wq, s, g = O.make_case(6, 1, n, k, 4)
    picks = [0, 31, 32, 2047, 4095]
    x = np.zeros((len(picks), k), dtype=np.float16)
    for r, j in enumerate(picks):
        x[r, j] = 1
    got = run_matmul(x, wq, s, 4, g)
    wd = relax_amd.wq_dequantize(_dev(wq), _dev(s), 4, g).cpu().numpy()
    assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(wd[:, picks].T).view(np.uint16))


def test_identical_rows_give_identical_outputs_and_kernel_families_agree():
    from relax_amd import lib

    x1, wq, s, g = O.make_case(7, 1, 4096, 4096, 4)
    x = np.repeat(x1, 48, axis=0)
    a = run_matmul(x, wq, s, 4, g, kernel=lib.KERNEL_SKINNY)
    assert np.all(a.view(np.uint16) == a.view(np.uint16)[0:1])
    b = run_matmul(x, wq, s, 4, g, kernel=lib.KERNEL_GEMM)
    assert np.all(b.view(np.uint16) == b.view(np.uint16)[0:1])
    assert_close(a, b.astype(np.float16), "families")


# ------------------------------------------------------------------ golden fixtures
def test_golden_fixtures():
    import glob
    import os

    files = sorted(f for f in glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz"))
                   if not os.path.basename(f).startswith(("fused_", "tiled_", "tail_")))
    assert files, "no golden fixtures found"
    import relax_amd

    for f in files:
        z = np.load(f)
        bits, g = int(z["bits"]), int(z["group"])
        got = run_matmul(z["x"], z["wq"], z["scales"], bits, g)
        assert_close(got, z["y"], f)
        wd = relax_amd.wq_dequantize(_dev(z["wq"]), _dev(z["scales"]), bits, g).cpu().numpy()
        assert np.array_equal(wd.view(np.uint16), z["wd"].view(np.uint16)), f


# ------------------------------------------------------------------ fused tail: bias, relu, residual
def _fused_operands(seed, m, n):
    rng = np.random.default_rng(seed)
    return ((0.5 * rng.standard_normal(n)).astype(np.float16), rng.standard_normal((m, n)).astype(np.float16))


def run_fused(x, wq, s, bits, group, bias=None, activation=None, residual=None, kernel=0, variant=0, out=None):
    import relax_amd

    y = relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, group, kernel=kernel, variant=variant,
                            bias=None if bias is None else _dev(bias), activation=activation,
                            residual=None if residual is None else _dev(residual), out=out)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def assert_fused(got, got_plain, want_plain, bias, act, res, what):
    """The fused output must be (a) bit for bit the float16 tail applied to the same kernel's plain
    output, and (b) within the matmul tolerance -- taken on the value before the tail, where
    cancellation has not yet shrunk the reference -- of the oracle's fused result."""
    tail_of_plain = O.epilogue(got_plain, bias, act, res)
    assert np.array_equal(got.view(np.uint16), tail_of_plain.view(np.uint16)), what
    want = O.epilogue(want_plain, bias, act, res).astype(np.float64)
    err = np.abs(got.astype(np.float64) - want)
    pre = np.abs(want_plain.astype(np.float64)) + (0 if bias is None else np.abs(bias.astype(np.float64))[None, :])
    bound = ATOL + RTOL * pre + 2.0**-10 * np.abs(want)
    assert np.all(np.isfinite(got)) and np.all(err <= bound), (what, float(err.max()))


FUSED_SHAPES = [  # bits, M, N, K -> kernel family under AUTO dispatch
    (4, 1, 200, 1024), (4, 8, 96, 352), (8, 16, 40, 256),       # GEMV
    (4, 33, 72, 256), (8, 64, 48, 384),                          # skinny
    (4, 300, 520, 512), (8, 129, 260, 1024), (4, 2048, 256, 768),  # GEMM, direct-weight kernel
    (4, 200, 96, 320), (4, 70, 32, 96),                          # GEMM, pipelined / generic fallbacks
]


@pytest.mark.parametrize("tail", ["bias", "bias_relu", "residual", "bias_relu_residual", "bias_residual"])
@pytest.mark.parametrize("bits,m,n,k", FUSED_SHAPES)
def test_fused_tail_every_kernel_family(bits, m, n, k, tail):
    x, wq, s, g = O.make_case(700 + m + n, m, n, k, bits)
    b, r = _fused_operands(m * 7 + n, m, n)
    bias = b if "bias" in tail else None
    res = r if "residual" in tail else None
    act = "relu" if "relu" in tail else None
    got_plain = run_matmul(x, wq, s, bits, g)
    got = run_fused(x, wq, s, bits, g, bias, act, res)
    want_plain = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    assert_fused(got, got_plain, want_plain, bias, act, res, (tail, bits, m, n, k))
    if act:
        assert got.min() >= 0 if res is None else True


@pytest.mark.parametrize("kernel,variant,bits,m,n,k", [
    ("GEMV", 14, 4, 3, 40, 352), ("GEMV", 25, 4, 1, 64, 1024), ("GEMV", 11, 8, 16, 24, 128),
    ("SKINNY", 1, 4, 20, 40, 256), ("SKINNY", 6, 8, 48, 24, 256),
    ("GEMM", 1, 4, 70, 136, 448), ("GEMM", 4, 8, 129, 72, 256), ("GEMM", 11, 4, 300, 200, 128),
    ("GEMM", 13, 8, 513, 260, 1024), ("GEMM", 21, 4, 129, 520, 1280), ("GEMM", 22, 8, 65, 300, 1792),
    ("GEMM", 23, 8, 129, 72, 256), ("GEMM", 24, 4, 70, 136, 768), ("GEMM", 25, 4, 129, 200, 1280),
])
def test_fused_tail_explicit_kernel_variants(kernel, variant, bits, m, n, k):
    from relax_amd import lib

    fam = getattr(lib, "KERNEL_" + kernel)
    x, wq, s, g = O.make_case(800 + m + n, m, n, k, bits)
    bias, res = _fused_operands(m + 3 * n, m, n)
    got_plain = run_matmul(x, wq, s, bits, g, kernel=fam, variant=variant)
    got = run_fused(x, wq, s, bits, g, bias, "relu", res, kernel=fam, variant=variant)
    want_plain = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    assert_fused(got, got_plain, want_plain, bias, "relu", res, (kernel, variant, bits, m, n, k))


@pytest.mark.parametrize("bits,m,n,k", [(4, 1, 4096, 4096), (4, 8, 200, 1024), (4, 40, 72, 256), (4, 256, 512, 512)])
def test_fused_residual_in_place(bits, m, n, k):
    """h += x W^T: the residual is the output buffer itself (each element is read, then written,
    by the one thread that owns it)."""
    import relax_amd

    x, wq, s, g = O.make_case(900 + m, m, n, k, bits)
    _, res = _fused_operands(m + n, m, n)
    separate = run_fused(x, wq, s, bits, g, residual=res)
    h = _dev(res.copy())
    out = relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, g, residual=h, out=h)
    torch.cuda.synchronize()
    assert out.data_ptr() == h.data_ptr()
    assert np.array_equal(h.cpu().numpy().view(np.uint16), separate.view(np.uint16))


@pytest.mark.parametrize("variant", [21, 22, 23, 24, 25])
@pytest.mark.parametrize("n,shift", [(521, 0), (520, 1), (64, 1), (129, 1)])
def test_gemm_output_pairs_fall_back_when_rows_or_bases_are_not_4_byte_aligned(variant, n, shift):
    """The direct-weight GEMM writes two adjacent columns per lane with one 4-byte access; with an
    odd row length, or y / bias / residual that start on an odd float16, it must write (and read
    the epilogue operands) element by element -- same bits either way."""
    import relax_amd
    from relax_amd import lib

    bits, m, k = 4, 130, 1280
    x, wq, s, g = O.make_case(950 + n + shift, m, n, k, bits)
    bias, res = _fused_operands(n + shift, m, n)
    want_plain = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)

    def shifted(a):  # a device copy of `a` that starts `shift` float16 into its allocation
        flat = torch.empty(a.size + shift, dtype=torch.float16, device="cuda")
        view = flat[shift:].view(a.shape)
        view.copy_(torch.from_numpy(a))
        return view

    xd, wd, sd = _dev(x), _dev(wq), _dev(s)
    y_plain = shifted(np.zeros((m, n), np.float16))
    relax_amd.wq_matmul(xd, wd, sd, bits, g, kernel=lib.KERNEL_GEMM, variant=variant, out=y_plain)
    y_fused = shifted(np.zeros((m, n), np.float16))
    relax_amd.wq_matmul(xd, wd, sd, bits, g, kernel=lib.KERNEL_GEMM, variant=variant, out=y_fused,
                        bias=shifted(bias), activation="relu", residual=shifted(res))
    torch.cuda.synchronize()
    assert y_plain.data_ptr() % 4 == (2 * shift) % 4
    got_plain, got = y_plain.cpu().numpy(), y_fused.cpu().numpy()
    assert_close(got_plain, want_plain, (variant, n, shift))
    assert_fused(got, got_plain, want_plain, bias, "relu", res, (variant, n, shift))


def test_fused_special_values_follow_the_cpu_rules():
    """relu(-0) = +0, an overflowing bias add gives inf, inf + (-inf) residual gives NaN."""
    m, n, k = 2, 32, 64
    w = np.full((n, k), 7, dtype=np.int64)          # dequantizes to 0: the matmul result is +0 everywhere
    w[:, 0] = 8                                     # ... except x[:, 0] * scale
    wq = O.pack_q4(w)
    s = np.full((n, k // 32), 1.0, dtype=np.float16)
    x = np.zeros((m, k), dtype=np.float16)
    x[0, 0], x[1, 0] = -0.0, 60000.0                # row 0: -0 * 1 = -0 accumulates to +0 (sum starts at +0)
    bias = np.zeros(n, dtype=np.float16)
    bias[0], bias[1], bias[2] = -0.0, 60000.0, -1.0
    res = np.zeros((m, n), dtype=np.float16)
    res[1, 3] = -np.inf
    got = run_fused(x, wq, s, 4, 32, bias, "relu", res)
    want = c_oracle.wq_matmul_fused(x, wq, s, 4, 32, bias, "relu", res)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint16)[~nan], want.view(np.uint16)[~nan])
    assert got[0, 0].view(np.uint16) == 0 and np.isinf(got[1, 1]) and got[0, 2] == 0 and got[1, 3] == -np.inf


def test_fused_golden_fixtures():
    import glob
    import os

    from tests.test_golden_cpu import fused_operands

    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "fused_*.npz")))
    assert len(files) >= 3
    for f in files:
        z = np.load(f)
        bits, g = int(z["bits"]), int(z["group"])
        bias, act, res = fused_operands(z)
        got_plain = run_matmul(z["x"], z["wq"], z["scales"], bits, g)
        got = run_fused(z["x"], z["wq"], z["scales"], bits, g, bias, act, res)
        assert_fused(got, got_plain, z["y_plain"], bias, act, res, f)


def test_fused_argument_checks():
    import relax_amd

    x, wq, s, g = O.make_case(1, 2, 32, 64, 4)
    xd, wd, sd = _dev(x), _dev(wq), _dev(s)
    with pytest.raises(ValueError, match="unsupported activation"):
        relax_amd.wq_matmul(xd, wd, sd, 4, g, activation="tanh")
    with pytest.raises(ValueError, match="bias must be"):
        relax_amd.wq_matmul(xd, wd, sd, 4, g, bias=torch.zeros(31, dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError, match="residual must be"):
        relax_amd.wq_matmul(xd, wd, sd, 4, g, residual=torch.zeros((1, 32), dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError, match="bias must be"):
        relax_amd.wq_matmul(xd, wd, sd, 4, g, bias=torch.zeros(32, dtype=torch.float32, device="cuda"))


# ------------------------------------------------------------------ int4 zero points other than 7
@pytest.mark.parametrize("zero_point", [0, 8, 15])
def test_int4_zero_points(zero_point):
    """The descriptor carries the zero point (0..15 for int4); every kernel family must honour it:
    dequantize bit for bit, the matmuls within tolerance of the NumPy oracle with that zero point."""
    import relax_amd
    from relax_amd import lib

    for m, n, k, kernel, variant in [(1, 64, 256, lib.KERNEL_GEMV, 0), (8, 40, 352, lib.KERNEL_GEMV, 14),
                                     (33, 48, 256, lib.KERNEL_SKINNY, 0), (129, 300, 512, lib.KERNEL_GEMM, 22),
                                     (70, 136, 768, lib.KERNEL_GEMM, 24), (200, 96, 320, lib.KERNEL_GEMM, 12),
                                     (70, 32, 96, lib.KERNEL_GEMM, 1)]:
        x, wq, s, g = O.make_case(40 + zero_point + m, m, n, k, 4)
        wd = O.dequant_q4f16(wq, s, g, zero_point)
        want = O.cast_f16(O.matmul_f32acc(x, wd))
        xd, wqd, sd = _dev(x), _dev(wq), _dev(s)
        got_wd = relax_amd.wq_dequantize(wqd, sd, 4, g, zero_point=zero_point).cpu().numpy()
        assert np.array_equal(got_wd.view(np.uint16), wd.view(np.uint16)), (zero_point, n, k)
        got = relax_amd.wq_matmul(xd, wqd, sd, 4, g, zero_point=zero_point, kernel=kernel, variant=variant)
        torch.cuda.synchronize()
        assert_close(got.cpu().numpy(), want, (zero_point, m, n, k, kernel, variant))


# ------------------------------------------------------------------ group sizes other than 32 / 128
@pytest.mark.parametrize("bits,group", [(4, 64), (4, 128), (4, 256), (8, 16), (8, 32), (8, 64), (8, 256)])
def test_other_group_sizes_every_family(bits, group):
    """group = 32 * 2^n (int4) or 16 * 2^n (int8): the default dispatch of every family, dequantize bit-exact."""
    import relax_amd

    for m, n, k in [(1, 64, 1024), (8, 40, 768), (16, 24, 2048), (33, 48, 512), (64, 80, 1024),
                    (200, 136, 512), (129, 300, 1280)]:
        x, wq, s, g = O.make_case(60 + m + group, m, n, k, bits, group)
        assert g == group
        got = run_matmul(x, wq, s, bits, g)
        want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=8)
        assert_close(got, want, (bits, group, m, n, k))
    _, wq, s, g = O.make_case(61, 1, 72, 2048, bits, group)
    wd = relax_amd.wq_dequantize(_dev(wq), _dev(s), bits, g).cpu().numpy()
    assert np.array_equal(wd.view(np.uint16), c_oracle.dequant(wq, s, bits, g).view(np.uint16))


# ------------------------------------------------------------------ seeded random shapes, default dispatch
def _random_shapes(seed, count):
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        bits = int(rng.choice([4, 8]))
        base = 32 if bits == 4 else 16
        group = base * int(rng.choice([1, 1, 1, 2, 4] if bits == 4 else [8, 8, 8, 1, 2]))
        k = group * int(rng.integers(1, 2048 // group + 1))
        if rng.random() < 0.4:
            k = 256 * int(rng.integers(1, 9))          # the direct-weight GEMM's K
            group = 32 if bits == 4 else 128
        m = int(rng.choice([1, 2, 3, 5, 8, 13, 16, 17, 31, 64, 65, 100, 129, 257, 300]))
        n = int(rng.integers(1, 700))
        shapes.append((bits, group, m, n, k))
    return shapes


@pytest.mark.parametrize("chunk", range(6))
def test_seeded_random_shapes_default_dispatch(chunk):
    """Ragged N (any value from 1), every M class, K any multiple of the group: the default dispatch against
    the oracle, plain and with the full fused tail."""
    for bits, group, m, n, k in _random_shapes(1000 + chunk, 12):
        x, wq, s, g = O.make_case(chunk * 100 + m + n, m, n, k, bits, group)
        want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
        got = run_matmul(x, wq, s, bits, g)
        assert_close(got, want, (bits, group, m, n, k))
        bias, res = _fused_operands(m + n + k, m, n)
        fused = run_fused(x, wq, s, bits, g, bias, "relu", res)
        assert_fused(fused, got, want, bias, "relu", res, ("fused", bits, group, m, n, k))


@pytest.mark.parametrize("bits,n,k", [(8, 98309, 16384), (4, 131077, 24576)])
def test_weights_between_one_and_two_gib(bits, n, k):
    """The largest operands the library accepts: 1.5 GiB of packed weights, i.e. byte offsets past 2^30 in
    every kernel family (the direct-weight GEMM declines them and the general GEMM runs).  The weights
    are drawn on the GPU; the oracle checks the first rows, the rows around the 1 GiB offset and the
    ragged last rows, for 1, 32 and 128 activation rows."""
    import relax_amd
    from relax_amd import lib

    group = 32 if bits == 4 else 128
    row_bytes = k * bits // 8
    assert 2**30 < n * row_bytes < 2**31
    gen = torch.Generator(device="cuda").manual_seed(23)
    wq = torch.randint(-2**31, 2**31 - 1, (n, k * bits // 32), dtype=torch.int32, device="cuda", generator=gen)
    if bits == 8:  # no byte 0x80: the quantizer's range is -127..127
        wq = torch.where((wq & 0x80) != 0, wq | 0x01, wq)
        wq = torch.where((wq & 0x8000) != 0, wq | 0x0100, wq)
        wq = torch.where((wq & 0x800000) != 0, wq | 0x010000, wq)
        wq = torch.where(wq < 0, wq | 0x01000000, wq)
    s = (torch.rand((n, k // group), device="cuda", generator=gen) * 0.008 + 0.002).to(torch.float16)
    mid = 2**30 // row_bytes
    rows = np.r_[0:24, mid - 20:mid + 20, n - 37:n]
    wq_rows = wq[torch.from_numpy(rows).cuda()].cpu().numpy().view(np.uint32)
    s_rows = s[torch.from_numpy(rows).cuda()].cpu().numpy()
    for m, kernel in ((1, lib.KERNEL_AUTO), (32, lib.KERNEL_AUTO), (128, lib.KERNEL_AUTO), (4, lib.KERNEL_SKINNY)):
        x = (torch.randn((m, k), device="cuda", generator=gen) * 0.25).to(torch.float16)
        y = relax_amd.wq_matmul(x, wq, s, bits, group, kernel=kernel)
        torch.cuda.synchronize()
        got = y[:, torch.from_numpy(rows).cuda()].cpu().numpy()
        want = c_oracle.wq_matmul(x.cpu().numpy(), wq_rows, s_rows, bits, group, nthreads=16)
        # (sums of 16384 - 24576 terms: the absolute float32 accumulation error is a few times that of
        # the other cases, so a few more outputs land 2 ulp away; the tolerance itself is unchanged)
        assert_close(got, want, ("1.5 GiB", bits, m), ulp_fraction=0.01)
    # dequantize: the same sampled rows, bit exact
    wd = relax_amd.wq_dequantize(wq, s, bits, group)
    torch.cuda.synchronize()
    got = wd[torch.from_numpy(rows).cuda()].cpu().numpy()
    want = c_oracle.dequant(wq_rows, s_rows, bits, group, nthreads=16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
