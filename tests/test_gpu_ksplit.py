"""GPU parity of the decode kernel's cross-workgroup K split (mi355x_wq_matmul_ws, caller workspace).

Bar as for the other matmul tests: float16 outputs within max-abs 1e-2 and relative 1e-2 of the oracle;
beyond that the split is deterministic (the partial tiles are added in the order of their K windows,
whichever workgroup arrives last), leaves its workspace ready for the next call, and a call whose
workspace is missing or too small is the plain call bit for bit."""
import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tests.test_gpu_parity import _dev, assert_close, assert_fused, _fused_operands  # noqa: E402

# (bits, M, N, K): shapes the library splits -- long K with one tile per CU, or 320 tiles on 256 CUs
CASES = [(4, 10, 4096, 11008), (4, 16, 4096, 11008), (8, 8, 5120, 13824), (8, 6, 5120, 13824),
         (8, 16, 5120, 13824), (4, 9, 4090, 11008), (8, 7, 5115, 13824), (4, 12, 2048, 22016)]


@pytest.mark.parametrize("bits,m,n,k", CASES)
def test_k_split_matches_the_oracle_and_is_deterministic(bits, m, n, k):
    import relax_amd

    x, wq, s, g = O.make_case(41, m, n, k, bits)
    need = relax_amd.wq_workspace_bytes(bits, g, n, k, m)
    assert need > 0, "the case is meant to split"
    ws = relax_amd.wq_workspace(need)
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    y1 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws)
    torch.cuda.synchronize()
    assert int(ws[:16384].view(torch.int32).abs().sum()) == 0, "arrival counters are back at zero"
    want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    # (K of 11008 - 22016: the float32 accumulation error is absolute and grows with the length of the
    # sum, so a few more outputs than elsewhere land two float16 ulp away; the tolerance is unchanged)
    assert_close(y1.cpu().numpy(), want, ("k split", bits, m, n, k), ulp_fraction=0.005)
    for _ in range(3):  # same workspace, back to back: same bits
        y2 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    # tile-major weights: the same windows in the same order where the library splits there too
    wq_t, s_t = relax_amd.wq_tile_weights(dwq, ds, bits, g)
    y3 = relax_amd.wq_matmul(dx, wq_t, s_t, bits, g, tiled_n=n, workspace=ws)
    torch.cuda.synchronize()
    if relax_amd.wq_workspace_bytes(bits, g, n, k, m, tiled=True) > 0:
        assert torch.equal(y1.view(torch.int16), y3.view(torch.int16))
    else:
        assert_close(y3.cpu().numpy(), want, ("tile-major, no split", bits, m, n, k), ulp_fraction=0.005)


@pytest.mark.parametrize("bits,m,n,k", [(4, 12, 4096, 11008), (8, 16, 5120, 13824)])
def test_k_split_applies_the_fused_tail_once(bits, m, n, k):
    """bias + relu + residual behind the sum of the partial tiles: applied by the workgroup that adds them."""
    import relax_amd

    x, wq, s, g = O.make_case(43, m, n, k, bits)
    bias, res = _fused_operands(43, m, n)
    ws = relax_amd.wq_workspace(relax_amd.wq_workspace_bytes(bits, g, n, k, m))
    assert ws is not None
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    plain = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws)
    fused = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws, bias=_dev(bias), activation="relu",
                                residual=_dev(res))
    torch.cuda.synchronize()
    want_plain = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
    assert_fused(fused.cpu().numpy(), plain.cpu().numpy(), want_plain, bias, "relu", res, (bits, m, n, k))
    # in place on the residual: y = h + W x written over h
    h = _dev(res).clone()
    relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws, residual=h, out=h)
    torch.cuda.synchronize()
    assert_fused(h.cpu().numpy(), plain.cpu().numpy(), want_plain, None, None, res, ("in place", bits, m))


def test_missing_or_small_workspace_is_the_plain_call():
    import relax_amd
    from relax_amd import lib

    bits, m, n, k = 8, 8, 5120, 13824
    x, wq, s, g = O.make_case(47, m, n, k, bits)
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    plain = relax_amd.wq_matmul(dx, dwq, ds, bits, g)
    need = relax_amd.wq_workspace_bytes(bits, g, n, k, m)
    small = torch.zeros(need - 16, dtype=torch.uint8, device="cuda")
    y = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=small)
    torch.cuda.synchronize()
    assert torch.equal(plain.view(torch.int16), y.view(torch.int16))
    assert int(small.sum()) == 0, "a workspace that is too small is not touched"
    # problems the library does not split ignore the workspace: 33 rows on a wide projection (172 tiles of
    # 64 x 128 already fill the CUs), and a wide projection at 8 rows
    for m2, n2, k2 in ((33, 22016, 4096), (8, 12288, 4096)):
        x2, wq2, s2, _ = O.make_case(48, m2, n2, k2, 4)
        assert relax_amd.wq_workspace_bytes(4, 32, n2, k2, m2) == 0
        a = relax_amd.wq_matmul(_dev(x2), _dev(wq2), _dev(s2), 4, 32)
        b = relax_amd.wq_matmul(_dev(x2), _dev(wq2), _dev(s2), 4, 32, workspace=small)
        torch.cuda.synchronize()
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)) and int(small.sum()) == 0
    # a forced kernel family and a workspace do not go together
    with pytest.raises(ValueError, match="own kernel choice"):
        relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=small, kernel=lib.KERNEL_GEMV)


def test_one_workspace_serves_projections_of_different_shapes():
    """A module passes the same workspace to all its projections: the counters sit at a fixed place, so
    the partial tiles one shape leaves behind are never read as another shape's counters."""
    import relax_amd

    shapes = [(8, 16, 5120, 13824), (4, 12, 4096, 11008), (8, 8, 5120, 13824), (4, 16, 4096, 11008)]
    cases = [(bits, O.make_case(57 + i, m, n, k, bits)) for i, (bits, m, n, k) in enumerate(shapes)]
    need = max(relax_amd.wq_workspace_bytes(bits, g, wq.shape[0], x.shape[1], x.shape[0]) for bits, (x, wq, s, g) in cases)
    ws = relax_amd.wq_workspace(need)
    first = {}
    for rnd in range(3):
        for i, (bits, (x, wq, s, g)) in enumerate(cases):
            y = relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, g, workspace=ws)
            torch.cuda.synchronize()
            if rnd == 0:
                first[i] = y
                assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), shapes[i],
                             ulp_fraction=0.005)
            else:
                assert torch.equal(y.view(torch.int16), first[i].view(torch.int16)), (rnd, shapes[i])


def test_k_split_in_a_hip_graph_replays_like_eager():
    """The down projection of a decoder layer at 12 rows with its residual, captured once with the
    workspace and replayed with eager work in between: every replay gives the eager bits, and a second
    projection sharing the workspace in the same graph does not disturb the first."""
    import relax_amd

    m, n, k = 12, 4096, 11008
    x, wq, s, g = O.make_case(53, m, n, k, 4)
    x2, wq2, s2, _ = O.make_case(54, m, n, k, 4)
    dx, dwq, ds, dx2, dwq2, ds2 = _dev(x), _dev(wq), _dev(s), _dev(x2), _dev(wq2), _dev(s2)
    ws = relax_amd.wq_workspace(relax_amd.wq_workspace_bytes(4, g, n, k, m))
    eager1 = relax_amd.wq_matmul(dx, dwq, ds, 4, g, workspace=ws)
    eager2 = relax_amd.wq_matmul(dx2, dwq2, ds2, 4, g, workspace=ws)
    torch.cuda.synchronize()
    y1 = torch.empty_like(eager1)
    y2 = torch.empty_like(eager2)
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=st):
            relax_amd.wq_matmul(dx, dwq, ds, 4, g, workspace=ws, out=y1)
            relax_amd.wq_matmul(dx2, dwq2, ds2, 4, g, workspace=ws, out=y2)
    torch.cuda.synchronize()
    for rep in range(4):
        y1.zero_()
        y2.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y1.view(torch.int16), eager1.view(torch.int16)), rep
        assert torch.equal(y2.view(torch.int16), eager2.view(torch.int16)), rep
        # the program's own eager work between replays, on the same workspace
        again = relax_amd.wq_matmul(dx, dwq, ds, 4, g, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(again.view(torch.int16), eager1.view(torch.int16))


def test_workspace_entry_called_vm_style():
    """matmul_ws as a destination-passing extern with a 1-d uint8 workspace tensor."""
    from relax_amd import vm_harness
    import relax_amd

    vm_harness.set_stream()
    for bits, m, n, k in [(8, 8, 5120, 13824), (4, 16, 4096, 11008), (4, 8, 50, 512), (8, 256, 5120, 8192),
                          (4, 64, 4096, 11008)]:  # decode split, no split, the GEMM's split above and below 64 rows
        x, wq, s, g = O.make_case(60 + m, m, n, k, bits)
        need = relax_amd.wq_workspace_bytes(bits, g, n, k, m)
        ws = torch.zeros(max(need, 64), dtype=torch.uint8, device="cuda")
        y = vm_harness.call_dps("mi355x_q%df16_matmul_ws" % bits, [_dev(x), _dev(wq), _dev(s), ws], (m, n))
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (bits, m, n, k),
                     ulp_fraction=0.005)
        if need:
            direct = relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, g, workspace=ws)
            torch.cuda.synchronize()
            assert torch.equal(direct.view(torch.int16), y.view(torch.int16))
    with pytest.raises(vm_harness.PackedError, match="5 tensor arguments"):
        vm_harness.call_dps("mi355x_q4f16_matmul_ws", [_dev(x), _dev(wq), _dev(s)], (m, n))
    with pytest.raises(vm_harness.PackedError, match="workspace"):
        vm_harness.call_dps("mi355x_q4f16_matmul_ws", [_dev(x), _dev(wq), _dev(s), ws.view(torch.int8)], (m, n))


def test_k_split_is_stable_while_another_stream_keeps_the_gpu_busy():
    """Two hundred split launches on one stream, each into its own output, while a second stream runs
    prefill-sized GEMMs that change which workgroup of a tile arrives last: every output has the bits of
    the first.  (The sum is taken in the order of the K windows, not in the order of arrival.)"""
    import relax_amd

    bits, m, n, k = 8, 8, 5120, 13824
    x, wq, s, g = O.make_case(61, m, n, k, bits)
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    ws = relax_amd.wq_workspace(relax_amd.wq_workspace_bytes(bits, g, n, k, m))
    ref = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws)
    xb, wqb, sb, gb = O.make_case(62, 512, 4096, 4096, 4)
    dxb, dwqb, dsb = _dev(xb), _dev(wqb), _dev(sb)
    torch.cuda.synchronize()
    outs = [torch.empty_like(ref) for _ in range(200)]
    side, main = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(60):
            relax_amd.wq_matmul(dxb, dwqb, dsb, 4, gb)
    with torch.cuda.stream(main):
        for y in outs:
            relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws, out=y)
    torch.cuda.synchronize()
    bad = [i for i, y in enumerate(outs) if not torch.equal(y.view(torch.int16), ref.view(torch.int16))]
    assert not bad, bad[:10]
    assert int(ws[:16384].view(torch.int32).abs().sum()) == 0


# (bits, M, N, K): prefill-side shapes whose 128 x 256 tiles fill at most half of the CUs (int8 in the canonical
# layout splits from K = 8192 on: below that the plain call's line-wise weight loads do as well)
GEMM_CASES = [(8, 256, 5120, 8192), (8, 256, 5120, 13824), (8, 256, 15360, 8192), (4, 256, 4096, 11008),
              (4, 160, 4096, 11008), (4, 200, 4090, 8192), (8, 200, 5120, 8192), (8, 384, 1000, 8192),
              # 17 .. 64 rows: 64 x 128 tiles, four K groups per workgroup
              (4, 64, 12288, 4096), (4, 56, 12288, 4096), (8, 25, 5120, 13824), (4, 41, 4090, 11008),
              (8, 60, 1000, 8192), (4, 64, 4096, 11008), (8, 64, 5120, 8192), (4, 33, 2000, 8448)]


@pytest.mark.parametrize("bits,m,n,k", GEMM_CASES)
def test_gemm_k_split_matches_the_oracle_and_is_deterministic(bits, m, n, k):
    import relax_amd

    x, wq, s, g = O.make_case(71, m, n, k, bits)
    need = relax_amd.wq_workspace_bytes(bits, g, n, k, m)
    assert need > 16384, "the case is meant to split"
    ws = relax_amd.wq_workspace(need)
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    y1 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws)
    torch.cuda.synchronize()
    assert int(ws[:16384].view(torch.int32).abs().sum()) == 0, "arrival counters are back at zero"
    rows = sorted({0, 1, m // 2, m - 2, m - 1} | set(np.random.default_rng(5).integers(0, m, 11).tolist()))  # (all rows when m is small)
    want = c_oracle.wq_matmul(x[rows], wq, s, bits, g, nthreads=16)
    assert_close(y1.cpu().numpy()[rows], want, ("gemm k split", bits, m, n, k), ulp_fraction=0.005)
    # every tile, against float32 torch on the dequantized weights (the oracle's rows pin the arithmetic)
    ref = dx.float() @ relax_amd.wq_dequantize(dwq, ds, bits, g).float().T
    err = (y1.float() - ref).abs()
    assert bool((err <= 1e-2 + 1e-2 * ref.abs()).all()), float(err.max())
    for _ in range(3):
        y2 = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(y1.view(torch.int16), y2.view(torch.int16))
    # without a workspace: the plain kernels, same tolerance against the oracle
    y0 = relax_amd.wq_matmul(dx, dwq, ds, bits, g)
    torch.cuda.synchronize()
    assert_close(y0.cpu().numpy()[rows], want, ("plain", bits, m, n, k), ulp_fraction=0.005)
    # tile-major weights: the same windows in the same order where the library splits there the same way
    wq_t, s_t = relax_amd.wq_tile_weights(dwq, ds, bits, g)
    y3 = relax_amd.wq_matmul(dx, wq_t, s_t, bits, g, tiled_n=n, workspace=ws)
    torch.cuda.synchronize()
    assert int(ws[:16384].view(torch.int32).abs().sum()) == 0
    if relax_amd.wq_workspace_bytes(bits, g, n, k, m, tiled=True) == need:
        assert torch.equal(y1.view(torch.int16), y3.view(torch.int16))
    else:
        assert_close(y3.cpu().numpy()[rows], want, ("tile-major", bits, m, n, k), ulp_fraction=0.005)


def test_gemm_k_split_applies_the_fused_tail_once():
    import relax_amd

    bits, m, n, k = 8, 256, 4096, 11008
    x, wq, s, g = O.make_case(73, m, n, k, bits)
    bias, res = _fused_operands(73, m, n)
    ws = relax_amd.wq_workspace(relax_amd.wq_workspace_bytes(bits, g, n, k, m))
    dx, dwq, ds = _dev(x), _dev(wq), _dev(s)
    plain = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws)
    fused = relax_amd.wq_matmul(dx, dwq, ds, bits, g, workspace=ws, bias=_dev(bias), activation="relu",
                                residual=_dev(res))
    torch.cuda.synchronize()
    rows = [0, 7, 128, 255]
    want_plain = c_oracle.wq_matmul(x[rows], wq, s, bits, g, nthreads=16)
    assert_fused(fused.cpu().numpy()[rows], plain.cpu().numpy()[rows], want_plain, bias, "relu", res[rows],
                 (bits, m, n, k))


def test_one_workspace_serves_decode_and_prefill_shapes():
    """The decode kernel's split and the GEMM's share the counters at the head of the workspace."""
    import relax_amd

    shapes = [(8, 256, 4096, 4096), (4, 12, 4096, 11008), (4, 256, 4096, 11008), (8, 16, 5120, 13824)]
    cases = [(bits, O.make_case(81 + i, m, n, k, bits)) for i, (bits, m, n, k) in enumerate(shapes)]
    need = max(relax_amd.wq_workspace_bytes(bits, g, wq.shape[0], x.shape[1], x.shape[0]) for bits, (x, wq, s, g) in cases)
    ws = relax_amd.wq_workspace(need)
    first = {}
    for rnd in range(3):
        for i, (bits, (x, wq, s, g)) in enumerate(cases):
            y = relax_amd.wq_matmul(_dev(x), _dev(wq), _dev(s), bits, g, workspace=ws)
            torch.cuda.synchronize()
            if rnd == 0:
                first[i] = y
                rows = [0, x.shape[0] - 1]
                assert_close(y.cpu().numpy()[rows], c_oracle.wq_matmul(x[rows], wq, s, bits, g, nthreads=16),
                             shapes[i], ulp_fraction=0.005)
            else:
                assert torch.equal(y.view(torch.int16), first[i].view(torch.int16)), (rnd, shapes[i])
