"""The decode kernel where the work does not divide evenly: row counts that are no multiple of the grid's tiles, K that
is no multiple of the wavefronts' super steps (the super steps are dealt out evenly, the first wavefronts take one
more), activations with more than one or two 16-byte vectors per thread, and activations walked in several K
phases -- the weight stream runs across the phase boundaries and, up to eight rows, a phase's activations are
requested while the phase before it streams."""
import numpy as np
import pytest
import torch

from oracle import c_oracle, wq_oracle as O

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 1e-2


def _dev(a):
    return torch.from_numpy(a.view(np.int32) if a.dtype == np.uint32 else a).cuda()


def _close(got, want, what):
    got, want = got.astype(np.float64), want.astype(np.float64)
    assert np.all(np.isfinite(got)), what
    err = np.abs(got - want)
    assert np.all(err <= ATOL + RTOL * np.abs(want)), (what, float(err.max()))
    ulp = np.maximum(np.abs(want), 2.0**-14) * 2.0**-10
    assert int(np.sum(err > 1.01 * ulp + 1e-6)) <= max(2, got.size // 200), (what, "more than 0.5 % off by over an ulp")


# N with a rest of tiles on grids of 256, 512 and 1024 workgroups; K whose super steps do not divide by 4, 8 or 16
# wavefronts (11008 = 43 super steps of 256, 2304 int8 = 18 of 128, 1152 int4 = 9 of 128 at one chunk per lane)
@pytest.mark.parametrize("bits,n,k", [(4, 4100, 1024), (4, 5000, 2048), (8, 6144, 512), (4, 9000, 768), (8, 5000, 1152),
                                       (4, 22016, 4096), (4, 520, 11008), (8, 264, 2304), (4, 72, 1152)])
def test_uneven_tiles_and_super_steps(bits, n, k):
    import relax_amd
    from relax_amd import lib

    rows = (1, 2, 3, 5, 8, 16)
    x_all, wq, s, g = O.make_case(900 + n + bits, max(rows), n, k, bits)
    want_all = c_oracle.wq_matmul(x_all, wq, s, bits, g, nthreads=16)
    dwq, ds = _dev(wq), _dev(s)
    tiled = relax_amd.wq_tile_weights(dwq, ds, bits, g) if k % 256 == 0 else None
    for m in rows:
        dx = _dev(np.ascontiguousarray(x_all[:m]))
        ran = 0
        for variant in (0, 15, 25, 14, 24, 18, 11, 12, 17):
            try:
                y = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=lib.KERNEL_GEMV, variant=variant)
            except lib.WqError:
                continue  # (a shape of the kernel that does not apply to this K says so)
            torch.cuda.synchronize()
            ran += 1
            _close(y.cpu().numpy(), want_all[:m], (bits, n, k, m, variant))
            if tiled is not None and variant in (0, 15, 25, 18, 12):
                yt = relax_amd.wq_matmul(dx, tiled[0], tiled[1], bits, g, tiled_n=n, kernel=lib.KERNEL_GEMV, variant=variant)
                torch.cuda.synchronize()
                # same lanes, same chunks, same order on both layouts
                assert torch.equal(yt.view(torch.int16), y.view(torch.int16)), ("tile-major", bits, n, k, m, variant)
        assert ran >= 3, (m, ran)


@pytest.mark.parametrize("bits,m,n,k", [(4, 8, 4096, 11008), (4, 5, 4100, 11008), (4, 16, 1024, 11008), (8, 16, 1040, 13824),
                                         (8, 8, 5000, 13824), (4, 3, 520, 45056), (4, 2, 300, 90112), (4, 8, 4096, 22016)])
def test_k_phases(bits, m, n, k):
    """Activations beyond the LDS: K is walked in phases, the weight stream runs across the phase boundaries and (up
    to eight rows) a phase's activations are requested while the phase before it streams."""
    import relax_amd
    from relax_amd import lib

    x, wq, s, g = O.make_case(970 + m + bits, m, n, k, bits)
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    ran = 0
    for variant in (0, 15, 14, 18, 25):
        try:
            y = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=lib.KERNEL_GEMV, variant=variant)
        except lib.WqError:
            continue
        torch.cuda.synchronize()
        got = y.cpu().numpy().astype(np.float64)
        err = np.abs(got - want.astype(np.float64))
        assert np.all(err <= ATOL + RTOL * np.abs(want.astype(np.float64))), (bits, m, n, k, variant, float(err.max()))
        ran += 1
    assert ran >= 2, ran


# (bits, group, K, rows): the staging builds of the eight-wavefront kernel -- exactly one, two or three 16-byte
# activation vectors per thread (rows of at least 512 vectors: K >= 4096), a column of up to four, eight or sixteen rows
# per thread, the general flat index (rows of fewer than 512 vectors at batch 1 - 2; more than three vectors per thread)
# -- for both scale layouts of each width (one scale per chunk / per super step).
@pytest.mark.parametrize("bits,group,k,rows", [
    (4, 32, 4096, (1, 2, 3, 4, 5, 8, 9, 16)),    # 1 and 2 vectors; columns of 4 / 8 / 16 rows
    (4, 32, 6144, (1, 2)),                       # 768 vectors per row: 2 and 3 vectors
    (4, 32, 11008, (1, 2)),                      # 1376 per row: 3 vectors; 2752 in all: flat index
    (4, 128, 4096, (1, 2, 4, 8, 16)),            # one scale per super step
    (4, 128, 6144, (1, 2)),
    (4, 32, 2048, (1, 2, 7)),                    # rows of 256 vectors: flat index with the division
    (8, 128, 4096, (1, 2, 3, 8, 16)),
    (8, 128, 5120, (1, 2)),                      # 640 per row: 2 and 3 vectors
    (8, 128, 11008, (1, 2)),
    (8, 16, 4096, (1, 2, 6)),                    # int8 with one scale per chunk
    (8, 128, 2048, (1, 2, 12)),
])
def test_activation_staging_builds(bits, group, k, rows):
    import relax_amd
    from relax_amd import lib

    n = 530  # 34 tiles, the last one ragged
    x_all, wq, s, g = O.make_case(7000 + bits * 131 + group + k, max(rows), n, k, bits, group=group)
    want_all = c_oracle.wq_matmul(x_all, wq, s, bits, g, nthreads=16)
    dwq, ds = _dev(wq), _dev(s)
    standard = (bits, group) in ((4, 32), (8, 128)) and k % 256 == 0
    tiled = relax_amd.wq_tile_weights(dwq, ds, bits, g) if standard else None
    for m in rows:
        dx = _dev(np.ascontiguousarray(x_all[:m]))
        for variant in (15, 25):
            y = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=lib.KERNEL_GEMV, variant=variant)
            torch.cuda.synchronize()
            _close(y.cpu().numpy(), want_all[:m], (bits, group, k, m, variant))
            if tiled is not None:
                yt = relax_amd.wq_matmul(dx, tiled[0], tiled[1], bits, g, tiled_n=n, kernel=lib.KERNEL_GEMV, variant=variant)
                torch.cuda.synchronize()
                assert torch.equal(yt.view(torch.int16), y.view(torch.int16)), ("tile-major", bits, group, k, m, variant)
        # the fused tail behind the exact builds' plain-store fast path: bias + residual
        bias = _dev(np.linspace(-1, 1, n).astype(np.float16))
        res = _dev(np.full((m, n), 0.5, dtype=np.float16))
        yf = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=lib.KERNEL_GEMV, variant=15, bias=bias, residual=res)
        y0 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=lib.KERNEL_GEMV, variant=15)
        torch.cuda.synchronize()
        want_f = ((y0.cpu().numpy() + bias.cpu().numpy()[None, :]).astype(np.float16) + np.float16(0.5)).astype(np.float16)
        assert np.array_equal(yf.cpu().numpy().view(np.int16), want_f.view(np.int16)), ("fused", bits, group, k, m)
