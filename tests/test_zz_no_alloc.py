"""mi355x_wq_matmul_static_ws: the decode kernel's K split on the library's own device array.

Called through the C ABI and held against mi355x_wq_matmul_ws (caller workspace) bit for bit, on
two calls in a row, the second with a smaller input; a problem whose split needs more than the
array holds is refused, and problems without a split equal the plain call.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle, wq_oracle as O

pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(a.view(np.int32) if a.dtype == np.uint32 else a).cuda()


def _call(L, lib, name, desc, x, wq, s, y, m, ep=None, extra=()):
    rc = getattr(L, name)(desc, x.data_ptr(), wq.data_ptr(), s.data_ptr(), ep, y.data_ptr(), m,
                          int(torch.cuda.current_stream().cuda_stream), 0, *extra)
    if rc != 0:
        raise lib.WqError(lib.last_error())


def test_static_scratch_entry_matches_the_caller_workspace_entry_on_consecutive_calls():
    from relax_amd import lib

    L = lib.load()
    limit = L.mi355x_wq_static_ws_bytes()
    assert limit == 16384 + (4 << 20)
    # first call: int8 5120 x 13824 at 16 rows (four K windows, 1.3 MB of partial tiles) with a fused tail;
    # second call: the smaller int4 4096 x 11008 at 12 rows (two windows), plain
    cases = [(8, 16, 5120, 13824, True), (4, 12, 4096, 11008, False), (8, 6, 5120, 13824, False)]
    for bits, m, n, k, fused in cases:
        x, wq, s, g = O.make_case(70 + m, m, n, k, bits)
        desc = lib.make_desc(bits, g, n, k)
        need = L.mi355x_wq_workspace_bytes(desc, m, 0)
        assert 0 < need <= limit, (bits, m, n, k, need)
        xd, wqd, sd = _dev(x), _dev(wq), _dev(s)
        ep = None
        if fused:
            rng = np.random.default_rng(1)
            bias = _dev(rng.standard_normal(n).astype(np.float16))
            res = _dev(rng.standard_normal((m, n)).astype(np.float16))
            ep = lib.WqEpilogue(bias.data_ptr(), res.data_ptr(), lib.ACT_RELU, 0)
        ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        y_ws = torch.empty((m, n), dtype=torch.float16, device="cuda")
        y_st = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        y_st2 = torch.full((m, n), float("nan"), dtype=torch.float16, device="cuda")
        _call(L, lib, "mi355x_wq_matmul_ws", desc, xd, wqd, sd, y_ws, m, ep, (ws.data_ptr(), need))
        _call(L, lib, "mi355x_wq_matmul_static_ws", desc, xd, wqd, sd, y_st, m, ep)
        _call(L, lib, "mi355x_wq_matmul_static_ws", desc, xd, wqd, sd, y_st2, m, ep)  # again: the counters are back at zero
        torch.cuda.synchronize()
        assert torch.equal(y_st.view(torch.int16), y_ws.view(torch.int16)), (bits, m, n, k)
        assert torch.equal(y_st2.view(torch.int16), y_ws.view(torch.int16)), (bits, m, n, k)
        if not fused:
            want = c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16)
            got = y_st.cpu().numpy().astype(np.float64)
            assert np.all(np.abs(got - want.astype(np.float64)) <= 1e-2 + 1e-2 * np.abs(want.astype(np.float64)))


def test_static_scratch_entry_without_a_split_and_beyond_its_size():
    from relax_amd import lib

    L = lib.load()
    # no split for this problem: the call equals the plain one
    x, wq, s, g = O.make_case(3, 4, 640, 1024, 4)
    desc = lib.make_desc(4, g, 640, 1024)
    assert L.mi355x_wq_workspace_bytes(desc, 4, 0) == 0
    xd, wqd, sd = _dev(x), _dev(wq), _dev(s)
    y0 = torch.empty((4, 640), dtype=torch.float16, device="cuda")
    y1 = torch.empty_like(y0)
    lib.check(L.mi355x_wq_matmul(desc, xd.data_ptr(), wqd.data_ptr(), sd.data_ptr(), y0.data_ptr(), 4,
                                 int(torch.cuda.current_stream().cuda_stream)))
    _call(L, lib, "mi355x_wq_matmul_static_ws", desc, xd, wqd, sd, y1, 4)
    torch.cuda.synchronize()
    assert torch.equal(y0.view(torch.int16), y1.view(torch.int16))
    # a split that needs more than the array holds: refused before any launch, the output untouched
    n, k, m = 17408, 8192, 1
    desc = lib.make_desc(8, 128, n, k)
    need = L.mi355x_wq_workspace_bytes(desc, m, 0)
    assert need > L.mi355x_wq_static_ws_bytes()
    wq_big = torch.zeros((n, k // 4), dtype=torch.int32, device="cuda")
    s_big = torch.ones((n, k // 128), dtype=torch.float16, device="cuda")
    x_big = torch.ones((m, k), dtype=torch.float16, device="cuda")
    y_big = torch.full((m, n), 5.0, dtype=torch.float16, device="cuda")
    with pytest.raises(lib.WqError, match="scratch"):
        _call(L, lib, "mi355x_wq_matmul_static_ws", desc, x_big, wq_big, s_big, y_big, m)
    torch.cuda.synchronize()
    assert bool((y_big == 5.0).all())
