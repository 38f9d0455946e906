"""GPU tests of the PackedFunc boundary: the VM-style call path (DLPack tensors, DPS output,
generated entries with permuted roles) and the decoder-layer chain of configuration 5."""
import ctypes as C
import os

import numpy as np
import pytest

from oracle import c_oracle, wq_oracle as O

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

from tests.test_gpu_parity import ATOL, RTOL, _dev, assert_close  # noqa: E402


def test_fixed_name_entries_called_vm_style():
    from relax_amd import vm_harness

    vm_harness.set_stream()
    for bits, m, n, k in [(4, 1, 4096, 4096), (4, 8, 64, 352), (4, 200, 136, 256), (8, 16, 5120, 5120)]:
        x, wq, s, g = O.make_case(21, m, n, k, bits)
        y = vm_harness.call_dps("mi355x_q%df16_matmul" % bits, [_dev(x), _dev(wq), _dev(s)], (m, n))
        wd = vm_harness.call_dps("mi355x_q%df16_dequantize" % bits, [_dev(wq), _dev(s)], (n, k))
        torch.cuda.synchronize()
        assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, bits, g, nthreads=16), (bits, m, n, k))
        assert np.array_equal(wd.cpu().numpy().view(np.uint16), c_oracle.dequant(wq, s, bits, g, 8).view(np.uint16))


def test_dltensor_handle_type_code_strides_and_byte_offset():
    """Type code 7 as well as 13; explicit compact strides; a view whose data pointer is the base of
    the allocation and whose start is carried in byte_offset (the cutlass glue ignores that field,
    python/tvm/contrib/cutlass/gemm_operation.py:280-283; this boundary honours it)."""
    from relax_amd import vm_harness

    vm_harness.set_stream()
    x, wq, s, g = O.make_case(22, 4, 48, 128, 4)
    big = torch.zeros((8, 128), dtype=torch.float16, device="cuda")
    big[4:] = _dev(x)
    y = torch.empty((4, 48), dtype=torch.float16, device="cuda")
    args = [vm_harness.TensorArg(big[4:], with_strides=True, byte_offset=4 * 128 * 2),
            vm_harness.TensorArg(_dev(wq), as_uint32=True), vm_harness.TensorArg(_dev(s)),
            vm_harness.TensorArg(y)]
    vm_harness.call_packed("mi355x_q4f16_matmul", args, type_code=vm_harness.K_TVM_DLTENSOR_HANDLE)
    torch.cuda.synchronize()
    assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, 4, g), "byte_offset view")
    # a misaligned view is refused, not silently mis-read
    odd = vm_harness.TensorArg(big.view(-1)[4:4 + 4 * 128].view(4, 128))
    with pytest.raises(vm_harness.PackedError, match="16-byte aligned"):
        vm_harness.call_packed("mi355x_q4f16_matmul", [odd] + args[1:])
    # tensors on another device id than the current one
    other = vm_harness.TensorArg(_dev(x))
    other.dl.device.device_id = 3
    with pytest.raises(vm_harness.PackedError, match="on device 3 but the first tensor is on device 0"):
        vm_harness.call_packed("mi355x_q4f16_matmul", [other] + args[1:])


def test_generated_entry_with_permuted_roles(tmp_path):
    from relax_amd import vm_harness
    from relax_amd.tvm_glue import CallSpec
    from tests.test_tvm_glue_cpu import SYM, build_entries, call_entry

    L = build_entries(tmp_path, [(SYM, CallSpec(0, 4, 0, 7, 2, 0, 1, 3))])
    vm_harness.set_stream()
    x, wq, s, g = O.make_case(23, 8, 4096, 4096, 4)
    y = torch.empty((8, 4096), dtype=torch.float16, device="cuda")
    t = [vm_harness.TensorArg(_dev(wq), as_uint32=True), vm_harness.TensorArg(_dev(s)),
         vm_harness.TensorArg(_dev(x)), vm_harness.TensorArg(y)]
    rc, code = call_entry(L, SYM, t)
    torch.cuda.synchronize()
    assert rc == 0 and code == vm_harness.K_TVM_NULLPTR
    assert_close(y.cpu().numpy(), c_oracle.wq_matmul(x, wq, s, 4, g, nthreads=16), "generated entry")


@pytest.mark.parametrize("m", [4, 1024])
def test_config5_decoder_layer_chain(m):
    """One Llama-2-7B-shaped decoder layer's four quantized matmuls back to back, as the VM would call
    them (DPS externs), the float16 residual flowing through.  Attention and the MLP activation are
    replaced by fixed elementwise stand-ins that are identical on both sides:
        qkv = x Wqkv^T;  a = (qkv[:, :4096] / 2 + qkv[:, 4096:8192] / 4 + qkv[:, 8192:] / 4) / 32
        h   = x + (a Wo^T) / 32
        gu  = h Wgu^T;   z = (gu[:, :11008] / 32) * (gu[:, 11008:] / 32)      (float16 products)
        out = h + (z Wd^T) / 32
    (powers of two keep the stand-ins exact and the activations of random-weight layers bounded.)
    The CPU side runs the oracle on a sample of rows (each row is independent)."""
    from relax_amd import vm_harness

    vm_harness.set_stream()
    shapes = {"qkv": (12288, 4096), "o": (4096, 4096), "gu": (22016, 4096), "down": (4096, 11008)}
    rng = np.random.default_rng(55)
    x = (rng.standard_normal((m, 4096)) * 0.5).astype(np.float16)
    W = {}
    for i, (name, (n, k)) in enumerate(shapes.items()):
        _, wq, s, g = O.make_case(60 + i, 1, n, k, 4)
        W[name] = (wq, s)

    def layer(xh, matmul, f16):
        qkv = matmul(xh, "qkv")
        a = f16(f16(f16(qkv[:, :4096] * f16(0.5)) + f16(qkv[:, 4096:8192] * f16(0.25))) + f16(qkv[:, 8192:] * f16(0.25)))
        a = f16(a * f16(1 / 32))
        h = f16(xh + f16(matmul(a, "o") * f16(1 / 32)))
        gu = matmul(h, "gu")
        z = f16(f16(gu[:, :11008] * f16(1 / 32)) * f16(gu[:, 11008:] * f16(1 / 32)))
        return f16(h + f16(matmul(z, "down") * f16(1 / 32)))

    dW = {k: (_dev(v[0]), _dev(v[1])) for k, v in W.items()}

    def gpu_matmul(t, name):
        return vm_harness.call_dps("mi355x_q4f16_matmul", [t.contiguous(), dW[name][0], dW[name][1]],
                                   (t.shape[0], shapes[name][0]))

    out = layer(_dev(x), gpu_matmul, lambda v: v if torch.is_tensor(v) else torch.tensor(v, dtype=torch.float16, device="cuda"))
    torch.cuda.synchronize()
    rows = np.arange(m) if m <= 4 else np.random.default_rng(5).choice(m, size=4, replace=False)

    def cpu_matmul(t, name):
        return c_oracle.wq_matmul(np.ascontiguousarray(t), W[name][0], W[name][1], 4, 32, nthreads=16)

    want = layer(x[rows], cpu_matmul, lambda v: np.asarray(v, dtype=np.float16))
    got = out.cpu().numpy()[rows]
    # four chained matmuls: each adds at most the single-matmul tolerance on top of the propagated error
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert np.all(np.isfinite(got)) and np.all(err <= 4 * (ATOL + RTOL * np.abs(want.astype(np.float64)))), float(err.max())
    assert float(np.mean(err)) < 2e-3


def test_fused_fixed_name_entries_called_vm_style():
    """matmul_bias / matmul_bias_relu / matmul_residual as DPS externs: same bits as the tensor front end."""
    import relax_amd
    from relax_amd import vm_harness

    vm_harness.set_stream()
    for bits, m, n, k in [(4, 1, 4096, 4096), (4, 40, 136, 256), (8, 300, 520, 1024)]:
        x, wq, s, g = O.make_case(31, m, n, k, bits)
        rng = np.random.default_rng(m)
        bias = rng.standard_normal(n).astype(np.float16)
        res = rng.standard_normal((m, n)).astype(np.float16)
        xd, wd, sd, bd, rd = _dev(x), _dev(wq), _dev(s), _dev(bias), _dev(res)
        for sym, extra, kw in (("matmul_bias", bd, dict(bias=bd)),
                               ("matmul_bias", bd.reshape(1, n), dict(bias=bd)),
                               ("matmul_bias_relu", bd, dict(bias=bd, activation="relu")),
                               ("matmul_residual", rd, dict(residual=rd))):
            y = vm_harness.call_dps("mi355x_q%df16_%s" % (bits, sym), [xd, wd, sd, extra], (m, n))
            ref = relax_amd.wq_matmul(xd, wd, sd, bits, g, **kw)
            torch.cuda.synchronize()
            assert np.array_equal(y.cpu().numpy().view(np.uint16), ref.cpu().numpy().view(np.uint16)), (sym, bits, m)
        want = c_oracle.wq_matmul_fused(x, wq, s, bits, g, bias, "relu", None, nthreads=16)
        got = relax_amd.wq_matmul(xd, wd, sd, bits, g, bias=bd, activation="relu").cpu().numpy()
        err = np.abs(got.astype(np.float64) - want.astype(np.float64))
        assert np.all(err <= 2 * ATOL + RTOL * np.abs(want.astype(np.float64)))


def test_generated_entry_with_bias_relu_and_residual(tmp_path):
    import relax_amd
    from relax_amd import vm_harness
    from relax_amd.tvm_glue import CallSpec
    from tests.test_tvm_glue_cpu import build_entries, call_entry

    L = build_entries(tmp_path, [("fused_tail_mi355x", CallSpec(0, 4, 0, 7, 2, 0, 1, 5, 3, 4, 1))])
    vm_harness.set_stream()
    m, n, k = 8, 4096, 4096
    x, wq, s, g = O.make_case(33, m, n, k, 4)
    rng = np.random.default_rng(3)
    bias, res = rng.standard_normal(n).astype(np.float16), rng.standard_normal((m, n)).astype(np.float16)
    y = torch.empty((m, n), dtype=torch.float16, device="cuda")
    xd, wd, sd, bd, rd = _dev(x), _dev(wq), _dev(s), _dev(bias), _dev(res)
    t = [vm_harness.TensorArg(wd, as_uint32=True), vm_harness.TensorArg(sd), vm_harness.TensorArg(xd),
         vm_harness.TensorArg(bd), vm_harness.TensorArg(rd), vm_harness.TensorArg(y)]
    rc, code = call_entry(L, "fused_tail_mi355x", t)
    torch.cuda.synchronize()
    assert rc == 0 and code == vm_harness.K_TVM_NULLPTR
    ref = relax_amd.wq_matmul(xd, wd, sd, 4, g, bias=bd, activation="relu", residual=rd)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy().view(np.uint16), ref.cpu().numpy().view(np.uint16))


@pytest.mark.parametrize("m", [4, 1024])
def test_decoder_layer_chain_with_fused_residuals(m):
    """The layer chain with the two residual adds fused into the O and down projections:
        a   = stand-in(qkv) / 1024;   h   = x + a Wo^T        (residual fused)
        z   = stand-in(gu)  / 32;     out = h + z Wd^T        (residual fused)
    Bit-equal to the same chain with separate float16 adds on the GPU, and within tolerance of the
    oracle on a sample of rows."""
    import relax_amd

    shapes = {"qkv": (12288, 4096), "o": (4096, 4096), "gu": (22016, 4096), "down": (4096, 11008)}
    rng = np.random.default_rng(56)
    x = (rng.standard_normal((m, 4096)) * 0.5).astype(np.float16)
    W = {}
    for i, (name, (n, k)) in enumerate(shapes.items()):
        _, wq, s, g = O.make_case(70 + i, 1, n, k, 4)
        W[name] = (wq, s)

    def layer(xh, matmul, f16):
        qkv = matmul(xh, "qkv", None)
        a = f16(f16(f16(qkv[:, :4096] * f16(0.5)) + f16(qkv[:, 4096:8192] * f16(0.25))) + f16(qkv[:, 8192:] * f16(0.25)))
        a = f16(a * f16(1 / 1024))
        h = matmul(a, "o", xh)
        gu = matmul(h, "gu", None)
        z = f16(f16(gu[:, :11008] * f16(1 / 32)) * f16(gu[:, 11008:] * f16(1 / 32)))
        z = f16(z * f16(1 / 32))
        return matmul(z, "down", h)

    dW = {k: (_dev(v[0]), _dev(v[1])) for k, v in W.items()}
    tf16 = lambda v: v if torch.is_tensor(v) else torch.tensor(v, dtype=torch.float16, device="cuda")  # noqa: E731

    def gpu_fused(t, name, res):
        return relax_amd.wq_matmul(t.contiguous(), dW[name][0], dW[name][1], 4, 32, residual=res)

    def gpu_separate(t, name, res):
        y = relax_amd.wq_matmul(t.contiguous(), dW[name][0], dW[name][1], 4, 32)
        return y if res is None else y + res

    fused = layer(_dev(x), gpu_fused, tf16)
    separate = layer(_dev(x), gpu_separate, tf16)
    torch.cuda.synchronize()
    assert np.array_equal(fused.cpu().numpy().view(np.uint16), separate.cpu().numpy().view(np.uint16))
    rows = np.arange(m) if m <= 4 else np.random.default_rng(5).choice(m, size=4, replace=False)

    def cpu_matmul(t, name, res):
        return c_oracle.wq_matmul_fused(np.ascontiguousarray(t), W[name][0], W[name][1], 4, 32,
                                        residual=None if res is None else np.ascontiguousarray(res), nthreads=16)

    want = layer(x[rows], cpu_matmul, lambda v: np.asarray(v, dtype=np.float16))
    got = fused.cpu().numpy()[rows]
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert np.all(np.isfinite(got)) and np.all(err <= 4 * (ATOL + RTOL * np.abs(want.astype(np.float64)))), float(err.max())


def test_layer_chain_captured_in_a_hip_graph_replays_like_eager():
    """A serving loop captures the VM-style call chain once and replays it: the packed entries launch
    on the stream set for the thread, nothing in them allocates, synchronizes or records a memset.
    Three replays with new inputs in the static buffers, eager work and synchronizations in between,
    each compared bit for bit with the eager chain."""
    import relax_amd
    from relax_amd import vm_harness

    shapes = {"qkv": (768, 512), "o": (512, 256), "gu": (1024, 512), "down": (512, 512)}
    W = {}
    for i, (name, (n, k)) in enumerate(shapes.items()):
        _, wq, s, g = O.make_case(80 + i, 1, n, k, 4)
        W[name] = (_dev(wq), _dev(s))
    m = 8
    x_static = torch.zeros((m, 512), dtype=torch.float16, device="cuda")
    bufs = {name: torch.empty((m, n), dtype=torch.float16, device="cuda") for name, (n, _) in shapes.items()}
    h = torch.empty((m, 512), dtype=torch.float16, device="cuda")

    def targ(t):
        return vm_harness.TensorArg(t, as_uint32=(t.dtype == torch.int32))

    def chain():
        # qkv -> slice stand-in -> o (+ residual x) -> gate/up -> product stand-in -> down (+ residual h)
        vm_harness.call_packed("mi355x_q4f16_matmul", [targ(x_static), targ(W["qkv"][0]), targ(W["qkv"][1]), targ(bufs["qkv"])])
        a = (bufs["qkv"][:, :256] * 0.0625).contiguous()
        vm_harness.call_packed("mi355x_q4f16_matmul_residual",
                               [targ(a), targ(W["o"][0]), targ(W["o"][1]), targ(x_static), targ(bufs["o"])])
        h.copy_(bufs["o"])
        vm_harness.call_packed("mi355x_q4f16_matmul", [targ(h), targ(W["gu"][0]), targ(W["gu"][1]), targ(bufs["gu"])])
        z = (bufs["gu"][:, :512] * bufs["gu"][:, 512:] * 0.0625).contiguous()
        vm_harness.call_packed("mi355x_q4f16_matmul_residual",
                               [targ(z), targ(W["down"][0]), targ(W["down"][1]), targ(h), targ(bufs["down"])])
        return bufs["down"]

    rng = np.random.default_rng(9)
    inputs = [torch.from_numpy((rng.standard_normal((m, 512)) * 0.5).astype(np.float16)).cuda() for _ in range(3)]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        vm_harness.set_stream(side)
        x_static.copy_(inputs[0])
        chain()  # warm-up outside the capture: code objects, per-kernel attributes
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            chain()
        for x_in in inputs:
            x_static.copy_(x_in)
            graph.replay()
            side.synchronize()
            got = bufs["down"].clone()
            # eager reference on the same stream, with unrelated eager work in between
            _ = relax_amd.wq_matmul(x_in, W["qkv"][0], W["qkv"][1], 4, 32)
            want = chain().clone()
            side.synchronize()
            assert torch.isfinite(got).all()
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    vm_harness.set_stream(torch.cuda.current_stream())


def test_concurrent_callers_on_their_own_streams():
    """Several VM threads call the packed entries at once, each on its own stream and its own problem
    (src/runtime/relax_vm/vm.cc:780-790: a VM runs on its caller's thread).  The stream and the error
    text are per thread; results must equal the single-threaded ones bit for bit."""
    import threading

    import relax_amd
    from relax_amd import lib, vm_harness

    cases = [(4, 1, 4096, 4096), (4, 8, 200, 1024), (8, 40, 136, 512), (4, 200, 520, 1024), (8, 300, 260, 1024)]
    jobs = []
    for i, (bits, m, n, k) in enumerate(cases):
        x, wq, s, g = O.make_case(300 + i, m, n, k, bits)
        xd, wd, sd = _dev(x), _dev(wq), _dev(s)
        want = relax_amd.wq_matmul(xd, wd, sd, bits, g)
        jobs.append((bits, m, n, xd, wd, sd, want))
    torch.cuda.synchronize()
    errors = []

    def worker(idx):
        try:
            bits, m, n, xd, wd, sd, want = jobs[idx]
            stream = torch.cuda.Stream()
            vm_harness.set_stream(stream)
            assert lib.load().mi355x_wq_packed_get_stream() == stream.cuda_stream
            for it in range(40):
                y = torch.empty((m, n), dtype=torch.float16, device="cuda")
                args = [vm_harness.TensorArg(xd), vm_harness.TensorArg(wd, as_uint32=True), vm_harness.TensorArg(sd),
                        vm_harness.TensorArg(y)]
                vm_harness.call_packed("mi355x_q%df16_matmul" % bits, args)
                if it % 8 == idx % 8:   # a failing call in between: the message belongs to this thread
                    with pytest.raises(vm_harness.PackedError, match="expects 4 arguments, got 3"):
                        vm_harness.call_packed("mi355x_q%df16_matmul" % bits, args[:3])
                stream.synchronize()
                if not torch.equal(y.view(torch.int16), want.view(torch.int16)):
                    errors.append((idx, it, "result differs"))
        except BaseException as e:  # noqa: BLE001 - reported by the main thread
            errors.append((idx, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(jobs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not any(t.is_alive() for t in threads), "a caller thread did not finish"
    assert not errors, errors[:3]
    vm_harness.set_stream()
