"""Every kernel build the library can be asked for by (family, variant), on both weight layouts and both bit
widths, against the oracle at small shapes: the default selection reaches only part of the template
instantiations, a caller that forces a variant reaches the rest."""
import numpy as np
import pytest
import torch

from oracle import c_oracle, wq_oracle as O

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 1e-2


def _dev(a):
    return torch.from_numpy(a.view(np.int32) if a.dtype == np.uint32 else a).cuda()


def _families():
    from relax_amd import lib

    gemv = [10 * wpc + shape for wpc in (1, 2, 4) for shape in range(1, 9)]
    skinny = list(range(1, 12)) + list(range(21, 32))
    gemm = list(range(1, 7)) + [11, 12, 13] + list(range(21, 30))
    return [("gemv", lib.KERNEL_GEMV, gemv, (1, 3, 8, 16)),
            ("skinny", lib.KERNEL_SKINNY, skinny, (2, 16, 20, 40, 64, 100)),
            ("gemm", lib.KERNEL_GEMM, gemm, (70, 150, 300))]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("family", ["gemv", "skinny", "gemm"])
def test_every_variant_on_both_layouts(bits, family):
    import relax_amd
    from relax_amd import lib

    name, kernel, variants, rows = next(f for f in _families() if f[0] == family)
    ran, refused = 0, 0
    # (the second group size of each bit width reaches the builds with fewer / more scales per load;
    # the tile-major layout is defined for the standard group sizes only)
    for n, k, group in ((200, 1024, None), (72, 2304, None), (136, 1024, 128 if bits == 4 else 32),
                        (40, 1536, 64 if bits == 4 else 16)):
        x_all, wq, s, g = O.make_case(400 + bits + n, max(rows), n, k, bits, group)
        want_all = c_oracle.wq_matmul(x_all, wq, s, bits, g, nthreads=16).astype(np.float64)
        dwq, ds = _dev(wq), _dev(s)
        wt, st = relax_amd.wq_tile_weights(dwq, ds, bits, g) if group is None else (None, None)
        for m in rows:
            dx = _dev(np.ascontiguousarray(x_all[:m]))
            want = want_all[:m]
            for variant in variants:
                for tiled in ((False, True) if wt is not None else (False,)):
                    try:
                        if tiled:
                            y = relax_amd.wq_matmul(dx, wt, st, bits, g, tiled_n=n, kernel=kernel, variant=variant)
                        else:
                            y = relax_amd.wq_matmul(dx, dwq, ds, bits, g, kernel=kernel, variant=variant)
                    except lib.WqError:
                        refused += 1  # (a variant that does not exist or does not fit this problem says so)
                        continue
                    torch.cuda.synchronize()
                    got = y.cpu().numpy().astype(np.float64)
                    err = np.abs(got - want)
                    assert np.all(err <= ATOL + RTOL * np.abs(want)), (name, bits, variant, tiled, m, n, k, float(err.max()))
                    ran += 1
    assert ran > 4 * len(variants), (name, ran, refused)  # most combinations exist


@pytest.mark.parametrize("bits,group,tiled,m", [(8, 16, False, 6), (8, 16, False, 8), (8, 64, False, 16),
                                                (8, 128, True, 12), (8, 128, True, 16)])
def test_k_split_builds_of_other_groups(bits, group, tiled, m):
    """The decode kernel's K split on int8 group sizes other than 128 (more scales per load), and on tile-major
    int8 weights from the row count on where the library splits them: builds the other workspace tests do not
    launch."""
    import relax_amd

    n, k = 5120, 13824
    x, wq, s, g = O.make_case(500 + bits + group + m, m, n, k, bits, group)
    need = relax_amd.wq_workspace_bytes(bits, g, n, k, m, tiled=tiled)
    if need == 0:
        pytest.skip("the library does not split this problem")
    ws = relax_amd.wq_workspace(need)
    dwq, ds = _dev(wq), _dev(s)
    if tiled:
        dwq, ds = relax_amd.wq_tile_weights(dwq, ds, bits, g)
    y = relax_amd.wq_matmul(_dev(x), dwq, ds, bits, g, workspace=ws, **({"tiled_n": n} if tiled else {}))
    torch.cuda.synchronize()
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16).astype(np.float64)
    err = np.abs(y.cpu().numpy().astype(np.float64) - want)
    assert np.all(err <= ATOL + RTOL * np.abs(want)), float(err.max())
    assert int(ws[:16384].view(torch.int32).abs().sum()) == 0
