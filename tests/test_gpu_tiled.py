"""GPU tests of the tile-major weight layout: the device transform against the oracle's loop
restatement, the round trip back to the interchange layout, and the matmul on tile-major weights
against the matmul on canonical weights (same kernel, same arithmetic order: bit-identical) and
against the CPU oracle."""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tests.test_gpu_parity import _dev, assert_close, assert_fused, _fused_operands  # noqa: E402


def _tiled(wq, s, bits, group):
    import relax_amd

    return relax_amd.wq_tile_weights(_dev(wq), _dev(s), bits, group)


@pytest.mark.parametrize("bits,n,k", [(4, 16, 256), (4, 37, 512), (4, 1000, 1024), (8, 16, 128), (8, 50, 384),
                                      (8, 333, 1280), (4, 4096, 4096), (8, 5120, 5120)])
def test_tile_weights_matches_the_loop_restatement_and_round_trips(bits, n, k):
    import relax_amd

    rng = np.random.default_rng(n + k)
    group = 32 if bits == 4 else 128
    wq = rng.integers(0, 2**32, size=(n, k * bits // 32), dtype=np.uint64).astype(np.uint32)
    s = rng.standard_normal((n, k // group)).astype(np.float16)
    wt, st = _tiled(wq, s, bits, group)
    torch.cuda.synchronize()
    if n * k <= 2_000_000:   # the loop restatement is slow: small cases only
        want_w, want_s = O.tile_weights(wq, s, bits)
        assert np.array_equal(wt.cpu().numpy().view(np.uint32), want_w)
        assert np.array_equal(st.cpu().numpy().view(np.uint16), want_s.view(np.uint16))
    else:                    # large cases: the oracle's independent inverse must return the input
        w_back, s_back = O.untile_weights(wt.cpu().numpy().view(np.uint32), st.cpu().numpy(), bits, n)
        assert np.array_equal(w_back, wq) and np.array_equal(s_back.view(np.uint16), s.view(np.uint16))
    w2, s2 = relax_amd.wq_untile_weights(wt, st, bits, group, n, k)
    torch.cuda.synchronize()
    assert np.array_equal(w2.cpu().numpy().view(np.uint32), wq)
    assert np.array_equal(s2.cpu().numpy().view(np.uint16), s.view(np.uint16))


def test_tile_weights_reproduces_the_committed_fixtures():
    import glob
    import os

    import relax_amd

    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "tiled_*.npz")))
    assert len(files) >= 2
    for f in files:
        z = np.load(f)
        bits, g = int(z["bits"]), int(z["group"])
        wt, st = _tiled(z["wq"], z["scales"], bits, g)
        w2, s2 = relax_amd.wq_untile_weights(_dev(z["wq_tiled"]), _dev(z["scales_tiled"]), bits, g, *(
            z["wq"].shape[0], z["wq"].shape[1] * (32 // bits)))
        torch.cuda.synchronize()
        assert np.array_equal(wt.cpu().numpy().view(np.uint32), z["wq_tiled"]), f
        assert np.array_equal(st.cpu().numpy().view(np.uint16), z["scales_tiled"].view(np.uint16)), f
        assert np.array_equal(w2.cpu().numpy().view(np.uint32), z["wq"]), f
        assert np.array_equal(s2.cpu().numpy().view(np.uint16), z["scales"].view(np.uint16)), f


GEMV_CASES = [(4, 1, 48, 256), (4, 3, 100, 512), (4, 16, 72, 1024), (4, 8, 4096, 4096), (4, 1, 22016, 4096),
              (4, 16, 4096, 11008), (4, 5, 1000, 8192), (8, 2, 40, 128), (8, 16, 72, 384), (8, 1, 5120, 5120),
              (8, 16, 5120, 13824), (8, 7, 333, 1280)]
SKINNY_CASES = [(4, 17, 136, 768), (4, 64, 200, 1280), (4, 40, 4096, 4096), (4, 16, 4096, 4096), (4, 24, 12288, 4096),
                (8, 33, 300, 2304), (8, 48, 5120, 5120), (4, 20, 6200, 512), (4, 30, 16400, 256),
                (4, 20, 5120, 512), (4, 1, 152064, 256), (4, 40, 16400, 256), (8, 30, 16400, 256)]  # every tile-major skinny variant
GEMM_CASES = [(4, 70, 136, 768), (4, 300, 521, 1024), (4, 2048, 4096, 4096), (4, 48, 12288, 4096), (4, 24, 22016, 4096),
              (8, 129, 72, 256), (8, 513, 260, 1024), (8, 256, 5120, 5120)]


@pytest.mark.parametrize("bits,m,n,k", GEMV_CASES + SKINNY_CASES + GEMM_CASES)
def test_matmul_on_tile_major_weights_is_bit_identical_to_canonical(bits, m, n, k):
    import relax_amd

    x, wq, s, g = O.make_case(40 + m + n, m, n, k, bits)
    wt, st = _tiled(wq, s, bits, g)
    xd = _dev(x)
    # compare within one kernel family: the layouts share the kernels, not every crossover
    from relax_amd import lib
    fam = lib.KERNEL_GEMV if m <= 16 and (bits, m, n, k) in GEMV_CASES else \
        (lib.KERNEL_SKINNY if (bits, m, n, k) in SKINNY_CASES else lib.KERNEL_GEMM)
    y_canon = relax_amd.wq_matmul(xd, _dev(wq), _dev(s), bits, g, kernel=fam)
    y_forced = relax_amd.wq_matmul(xd, wt, st, bits, g, tiled_n=n, kernel=fam)
    assert np.array_equal(y_forced.cpu().numpy().view(np.uint16), y_canon.cpu().numpy().view(np.uint16))
    y_tiled = relax_amd.wq_matmul(xd, wt, st, bits, g, tiled_n=n)   # the entry's own choice of kernel
    torch.cuda.synchronize()
    if m * n * k <= 3e9:
        assert_close(y_tiled.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (bits, m, n, k))


@pytest.mark.parametrize("bits,m,n,k", [(4, 4, 200, 1024), (8, 16, 72, 384), (4, 130, 520, 1280), (8, 70, 300, 1024)])
def test_fused_tail_on_tile_major_weights(bits, m, n, k):
    import relax_amd

    x, wq, s, g = O.make_case(60 + m + n, m, n, k, bits)
    bias, res = _fused_operands(m + n, m, n)
    wt, st = _tiled(wq, s, bits, g)
    plain = relax_amd.wq_matmul(_dev(x), wt, st, bits, g, tiled_n=n)
    fused = relax_amd.wq_matmul(_dev(x), wt, st, bits, g, tiled_n=n, bias=_dev(bias), activation="relu",
                                residual=_dev(res))
    torch.cuda.synchronize()
    want_plain = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    assert_fused(fused.cpu().numpy(), plain.cpu().numpy(), want_plain, bias, "relu", res, (bits, m, n, k))


def test_tile_major_entries_called_vm_style():
    """tile_weights in a parameter-preparation step, matmul_tiled in the model: both as DPS externs."""
    from relax_amd import vm_harness

    vm_harness.set_stream()
    for bits, m, n, k in [(4, 1, 4096, 4096), (4, 8, 50, 512), (8, 16, 333, 1280), (4, 200, 136, 256)]:
        x, wq, s, g = O.make_case(70 + m, m, n, k, bits)
        rows = (n + 15) // 16 * 16
        wd, sd = _dev(wq), _dev(s)
        wt = torch.empty((rows, wq.shape[1]), dtype=torch.int32, device="cuda")
        st = torch.empty((rows, s.shape[1]), dtype=torch.float16, device="cuda")
        vm_harness.call_packed("mi355x_q%df16_tile_weights" % bits,
                               [vm_harness.TensorArg(wd, as_uint32=True), vm_harness.TensorArg(sd),
                                vm_harness.TensorArg(wt, as_uint32=True), vm_harness.TensorArg(st)])
        y = vm_harness.call_dps("mi355x_q%df16_matmul_tiled" % bits, [_dev(x), wt, st], (m, n))
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (bits, m, n, k))
    # shapes that do not fit are refused with the reason
    with pytest.raises(vm_harness.PackedError, match="rounded up to 16"):
        vm_harness.call_dps("mi355x_q4f16_matmul_tiled", [_dev(x), wt[:128], st[:128]], (m, n))


def test_tile_major_layout_is_refused_where_it_is_not_defined():
    import relax_amd
    from relax_amd import lib

    wq = torch.zeros((32, 24), dtype=torch.int32, device="cuda")     # int4, K = 192: not a multiple of 256
    s = torch.zeros((32, 6), dtype=torch.float16, device="cuda")
    with pytest.raises(lib.WqError, match="K % 256 == 0"):
        relax_amd.wq_tile_weights(wq, s, 4, 32)
    wq = torch.zeros((32, 64), dtype=torch.int32, device="cuda")     # int4, K = 512 but group 64
    s = torch.zeros((32, 8), dtype=torch.float16, device="cuda")
    with pytest.raises(lib.WqError, match="group 32"):
        relax_amd.wq_tile_weights(wq, s, 4, 64)
    # int8 with K % 128 == 0 but K % 256 != 0: decode and the register-activation kernel (up to 128 rows on a
    # narrow projection) run, a GEMM-sized batch is refused
    x, wq8, s8, g = O.make_case(80, 200, 64, 384, 8)
    wt, st = relax_amd.wq_tile_weights(_dev(wq8), _dev(s8), 8, g)
    relax_amd.wq_matmul(_dev(x[:8]), wt, st, 8, g, tiled_n=64)
    y100 = relax_amd.wq_matmul(_dev(x[:100]), wt, st, 8, g, tiled_n=64)
    ref100 = relax_amd.wq_matmul(_dev(x[:100]), _dev(wq8), _dev(s8), 8, g)
    torch.cuda.synchronize()
    assert torch.equal(y100.view(torch.int16), ref100.view(torch.int16))
    with pytest.raises(lib.WqError, match="direct-weight kernel"):
        relax_amd.wq_matmul(_dev(x), wt, st, 8, g, tiled_n=64)


@pytest.mark.parametrize("chunk", range(4))
def test_seeded_random_shapes_on_tile_major_weights(chunk):
    """Ragged N from 1, every M class, every K the layout is defined for: the tiled entry's own kernel
    choice against the oracle, plain and with the full fused tail, and the transform's round trip."""
    import relax_amd

    rng = np.random.default_rng(2000 + chunk)
    for _ in range(12):
        bits = int(rng.choice([4, 8]))
        g = 32 if bits == 4 else 128
        k = 256 * int(rng.integers(1, 9))
        m = int(rng.choice([1, 2, 3, 5, 8, 13, 16, 17, 31, 40, 64, 65, 100, 129, 257, 300]))
        n = int(rng.integers(1, 700))
        x, wq, s, _ = O.make_case(chunk * 100 + m + n, m, n, k, bits, g)
        wt, st = _tiled(wq, s, bits, g)
        w2, s2 = relax_amd.wq_untile_weights(wt, st, bits, g, n, k)
        got = relax_amd.wq_matmul(_dev(x), wt, st, bits, g, tiled_n=n)
        bias, res = _fused_operands(m + n + k, m, n)
        fused = relax_amd.wq_matmul(_dev(x), wt, st, bits, g, tiled_n=n, bias=_dev(bias), activation="relu",
                                    residual=_dev(res))
        torch.cuda.synchronize()
        assert np.array_equal(w2.cpu().numpy().view(np.uint32), wq), (bits, m, n, k)
        assert np.array_equal(s2.cpu().numpy().view(np.uint16), s.view(np.uint16)), (bits, m, n, k)
        want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
        assert_close(got.cpu().numpy(), want, (bits, m, n, k))
        assert_fused(fused.cpu().numpy(), got.cpu().numpy(), want, bias, "relu", res, ("fused", bits, m, n, k))


def test_tile_major_weights_of_one_and_a_half_gib():
    """The largest weight operand: 98309 x 16384 int8 (1.5 GiB, ragged last tile).  Tiling round-trips bit
    for bit, the register-activation kernel gives the canonical layout's bits (whose parity
    with the oracle test_weights_between_one_and_two_gib checks), and more than 64 rows are refused:
    only the direct-weight GEMM reads this layout, and it addresses operands below 1 GiB."""
    import relax_amd
    from relax_amd import lib

    bits, group, n, k = 8, 128, 98309, 16384
    gen = torch.Generator(device="cuda").manual_seed(29)
    wq = torch.randint(-2**31, 2**31 - 1, (n, k * bits // 32), dtype=torch.int32, device="cuda", generator=gen)
    s = (torch.rand((n, k // group), device="cuda", generator=gen) * 0.008 + 0.002).to(torch.float16)
    wq_t, s_t = relax_amd.wq_tile_weights(wq, s, bits, group)
    wq_back, s_back = relax_amd.wq_untile_weights(wq_t, s_t, bits, group, n, k)
    assert torch.equal(wq_back, wq) and torch.equal(s_back.view(torch.int16), s.view(torch.int16))
    del wq_back, s_back
    # (6145 row tiles are more than the decode kernel's LDS slots hold: every batch runs the
    # register-activation kernel, as on the canonical layout)
    for m, kernel in ((1, lib.KERNEL_SKINNY), (8, lib.KERNEL_SKINNY), (32, lib.KERNEL_SKINNY), (4, lib.KERNEL_AUTO)):
        x = (torch.randn((m, k), device="cuda", generator=gen) * 0.25).to(torch.float16)
        y_c = relax_amd.wq_matmul(x, wq, s, bits, group, kernel=kernel)
        y_t = relax_amd.wq_matmul(x, wq_t, s_t, bits, group, kernel=kernel, tiled_n=n)
        torch.cuda.synchronize()
        assert torch.equal(y_c.view(torch.int16), y_t.view(torch.int16)), (m, kernel)
    x = torch.zeros((128, k), dtype=torch.float16, device="cuda")
    with pytest.raises(lib.WqError, match="direct-weight kernel"):
        relax_amd.wq_matmul(x, wq_t, s_t, bits, group, tiled_n=n)
