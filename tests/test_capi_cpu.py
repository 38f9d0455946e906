"""Host-side tests of the C ABI and the PackedFunc boundary that need no GPU: the library
loads, exports every declared symbol, and rejects bad arguments before touching the device."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from relax_amd import lib, vm_harness  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = []
    for h in ("mi355x_wq.h", "mi355x_wq_packed.h", "mi355x_wq_module.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        names += re.findall(r"MI355X_WQ_API\s+[\w\s\*]+?\b(mi355x_\w+)\s*\(", text)
    return names


def test_library_exports_every_declared_symbol():
    L = lib.load()
    names = declared_symbols()
    assert len(names) == 58 and set(names) == set(lib.EXPORTED_SYMBOLS)
    for n in names:
        assert hasattr(L, n), n
    assert L.mi355x_wq_version() >= 100
    # only the C ABI is exported: no C++ symbols leak out of the shared object
    out = subprocess.run(["nm", "-D", "--defined-only", lib.SO_PATH], capture_output=True, text=True).stdout
    exported = [l.split()[-1] for l in out.splitlines() if " T " in l]
    assert sorted(exported) == sorted(names)


def test_tile_major_layout_entry_checks_without_a_gpu():
    L = lib.load()
    wb, sb = C.c_int64(0), C.c_int64(0)
    assert L.mi355x_wq_tiled_sizes(lib.make_desc(4, 32, 100, 512), C.byref(wb), C.byref(sb)) == 0
    assert (wb.value, sb.value) == (112 * 256, 112 * 16 * 2)       # 100 rows -> 112: whole 16-row tiles
    assert L.mi355x_wq_tiled_sizes(lib.make_desc(8, 128, 16, 384), C.byref(wb), C.byref(sb)) == 0
    assert (wb.value, sb.value) == (16 * 384, 16 * 3 * 2)
    assert L.mi355x_wq_tiled_sizes(lib.make_desc(4, 32, 100, 320), C.byref(wb), C.byref(sb)) == -1
    assert "K % 256 == 0" in lib.last_error()
    assert L.mi355x_wq_tiled_sizes(lib.make_desc(4, 64, 100, 512), None, None) == -1 and "group 32" in lib.last_error()
    d, ok = lib.make_desc(4, 32, 64, 256), 0x10000
    assert L.mi355x_wq_tile_weights(d, ok, ok + 0x1000, ok, ok + 0x2000, None) == -1 and "in-place" in lib.last_error()
    assert L.mi355x_wq_tile_weights(d, ok, ok + 8, ok + 0x1000, ok + 0x2000, None) == -1 \
        and "scales" in lib.last_error() and "16-byte aligned" in lib.last_error()
    assert L.mi355x_wq_untile_weights(d, None, ok, ok, ok, None) == -1 and "wq_tiled is NULL" in lib.last_error()
    assert L.mi355x_wq_matmul_tiled(lib.make_desc(4, 32, 64, 320), ok, ok, ok, None, ok, 4, None) == -1 \
        and "tile-major layout" in lib.last_error()


def test_workspace_size_query_without_a_gpu():
    """mi355x_wq_workspace_bytes: 16 KB of arrival counters plus the partial tiles (1 KB per 16-row tile
    and K window) where the decode kernel would split K, 0 where it would not, -1 on an invalid descriptor.
    (The rule reads the CU count; without a GPU the library assumes the 256 CUs of an MI355X.)"""
    L = lib.load()
    q = L.mi355x_wq_workspace_bytes
    assert q(lib.make_desc(8, 128, 5120, 13824), 8, 0) == 16384 + 320 * 3 * 1024         # three windows
    assert q(lib.make_desc(8, 128, 5120, 13824), 1, 0) == 0      # (activations that fit the LDS: 10-row tiles even the CUs out)
    assert q(lib.make_desc(8, 128, 5120, 13824), 16, 0) == 16384 + 320 * 4 * 1024        # 16 rows: four fit the LDS
    assert q(lib.make_desc(4, 32, 4096, 11008), 9, 0) == 16384 + 256 * 2 * 1024          # activations beyond the LDS
    assert q(lib.make_desc(4, 32, 4096, 11008), 8, 0) == 0                                # (int4 up to 8 rows: K phases)
    assert q(lib.make_desc(8, 128, 4096, 11008), 8, 0) == 16384 + 256 * 2 * 1024
    assert q(lib.make_desc(4, 32, 4096, 11008), 1, 0) == 0
    assert q(lib.make_desc(4, 32, 12288, 4096), 8, 0) == 0 and q(lib.make_desc(4, 32, 4096, 4096), 16, 0) == 0
    assert q(lib.make_desc(8, 128, 5120, 13824), 4, 1) == 0                              # tile-major: from 12 rows on
    assert q(lib.make_desc(8, 128, 5120, 13824), 16, 1) == 16384 + 320 * 4 * 1024
    # 17 .. 64 rows: the GEMM's split on 64 x 128 tiles (32 KB per tile and window) from the measured row counts on
    assert q(lib.make_desc(4, 32, 4096, 11008), 48, 0) == 16384 + 32 * 8 * 32768
    assert q(lib.make_desc(4, 32, 4096, 11008), 33, 0) == 16384 + 32 * 8 * 32768          # three row blocks on
    assert q(lib.make_desc(4, 32, 4096, 11008), 33, 1) == 16384 + 32 * 8 * 32768
    assert q(lib.make_desc(4, 32, 4096, 11008), 32, 0) == 0 and q(lib.make_desc(4, 32, 4096, 4096), 48, 0) == 0
    assert q(lib.make_desc(8, 128, 5120, 13824), 25, 0) == 16384 + 40 * 6 * 32768
    assert q(lib.make_desc(8, 128, 5120, 13824), 24, 0) == 0
    assert q(lib.make_desc(8, 128, 5120, 13824), 32, 1) == 0                              # tile-major int8: from 33
    assert q(lib.make_desc(4, 32, 4096, 4096), 64, 1) == 0                                # tile-major, short K: never
    # short K: int4 on canonical weights only, from 49 rows and 96 column tiles on
    assert q(lib.make_desc(4, 32, 4096, 4096), 64, 0) == 0 and q(lib.make_desc(8, 128, 5120, 5120), 64, 0) == 0
    assert q(lib.make_desc(4, 32, 12288, 4096), 64, 0) == 16384 + 96 * 2 * 32768
    assert q(lib.make_desc(4, 32, 12288, 4096), 48, 0) == 0
    assert q(lib.make_desc(4, 32, 22016, 4096), 64, 0) == 0                              # 172 tiles fill the CUs
    # above 64 rows: 128 x 256 tiles (128 KB per tile and window)
    assert q(lib.make_desc(8, 128, 5120, 13824), 256, 0) == 16384 + 40 * 6 * 131072
    assert q(lib.make_desc(4, 32, 4096, 4096), 512, 0) == 0
    assert q(lib.make_desc(4, 32, 4096, 320), 8, 1) == 0                                 # layout not defined: no split
    assert q(lib.make_desc(5, 32, 4096, 4096), 8, 0) == -1 and "bits" in lib.last_error()
    ok = 0x10000
    assert L.mi355x_wq_matmul_ws(lib.make_desc(4, 32, 64, 256), ok, ok, ok, None, ok, 4, None, 0, ok + 4, 1 << 20) == -1 \
        and "workspace" in lib.last_error() and "16-byte aligned" in lib.last_error()


@pytest.mark.parametrize("kw,msg", [
    (dict(bits=5), "bits must be 4 or 8"),
    (dict(group=48), "group must be 32 times a power of two"),
    (dict(bits=8, group=24, zero_point=0), "group must be 16 times a power of two"),
    (dict(zero_point=16), "zero_point must be in 0..15"),
    (dict(bits=8, group=128, zero_point=3), "zero_point must be 0 for 8-bit"),
    (dict(k=4096 + 32, group=64), "not a multiple of the group size"),
    (dict(n=-1), "negative extent"),
    (dict(n=1 << 30, k=1 << 14), "operand too large"),
])
def test_descriptor_validation(kw, msg):
    L = lib.load()
    args = dict(bits=4, group=32, n=4096, k=4096, zero_point=7)
    args.update(kw)
    d = lib.make_desc(args["bits"], args["group"], args["n"], args["k"], args["zero_point"])
    assert L.mi355x_wq_check(d, 1) == -1
    assert msg in lib.last_error()


def test_reserved_field_and_null_descriptor():
    L = lib.load()
    d = lib.make_desc(4, 32, 64, 64)
    d.reserved = 1
    assert L.mi355x_wq_check(d, 1) == -1 and "reserved" in lib.last_error()
    assert L.mi355x_wq_check(None, 1) == -1 and "NULL" in lib.last_error()


def test_kernel_selection_by_rows():
    L = lib.load()
    d = lib.make_desc(4, 32, 4096, 4096)
    assert L.mi355x_wq_select_kernel(d, 1) == lib.KERNEL_GEMV
    assert L.mi355x_wq_select_kernel(d, 8) == lib.KERNEL_GEMV
    # 16 rows x 4096 = 128 KB of activations still fit the LDS in one piece
    assert L.mi355x_wq_select_kernel(d, 16) == lib.KERNEL_GEMV
    # 16 rows x 8192 = 256 KB would be staged in K phases: int4 from 9 rows on goes to the register-activation kernel
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 4096, 8192), 16) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 4096, 8192), 9) == lib.KERNEL_GEMV   # 144 KB: one piece
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 4096, 11008), 9) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 5120, 13824), 16) == lib.KERNEL_GEMV
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 22016, 4096), 16) == lib.KERNEL_GEMV
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 4096, 11008), 2) == lib.KERNEL_GEMV
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 4096, 11008), 8) == lib.KERNEL_GEMV
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 4096, 2048), 8) == lib.KERNEL_SKINNY  # a 4 MB matrix
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 22016, 11008), 8) == lib.KERNEL_GEMV
    # a vocabulary-sized projection: too many row tiles per workgroup for the GEMV kernel's LDS slots
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 152064, 4096), 1) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 32000, 4096), 1) == lib.KERNEL_GEMV
    assert L.mi355x_wq_select_kernel(d, 17) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(d, 64) == lib.KERNEL_SKINNY
    # 65..128 rows on narrow projections: two grid slices of the register-activation kernel
    assert L.mi355x_wq_select_kernel(d, 65) == lib.KERNEL_SKINNY and L.mi355x_wq_select_kernel(d, 128) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(d, 129) == lib.KERNEL_GEMM
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 5120, 5120), 192) == lib.KERNEL_SKINNY  # three slices
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 5120, 5120), 193) == lib.KERNEL_GEMM
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 2048, 8192), 256) == lib.KERNEL_SKINNY   # four
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 2048, 8192), 257) == lib.KERNEL_GEMM
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 8192, 8192), 128) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 5120, 13824), 128) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 10240, 5120), 112) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 15360, 5120), 65) == lib.KERNEL_GEMM
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 12288, 4096), 65) == lib.KERNEL_GEMM
    # 17..64 rows on wide projections: the GEMM's 64x128 tile costs the same for any row count, the
    # skinny kernel grows with it
    wide, mid = lib.make_desc(4, 32, 22016, 4096), lib.make_desc(4, 32, 12288, 4096)
    assert L.mi355x_wq_select_kernel(wide, 16) == lib.KERNEL_GEMV
    assert L.mi355x_wq_select_kernel(wide, 32) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(wide, 33) == lib.KERNEL_GEMM
    assert L.mi355x_wq_select_kernel(mid, 64) == lib.KERNEL_SKINNY  # 96 column tiles: never
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 8192, 4096), 64) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 27648, 5120), 24) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 27648, 5120), 40) == lib.KERNEL_GEMM
    assert L.mi355x_wq_select_kernel(lib.make_desc(8, 128, 15360, 5120), 48) == lib.KERNEL_SKINNY
    assert L.mi355x_wq_select_kernel(lib.make_desc(4, 32, 22016, 4000), 48) == lib.KERNEL_SKINNY  # K % 256 != 0
    assert L.mi355x_wq_select_kernel(d, -1) == -1


def test_pointer_checks_happen_before_any_launch():
    L = lib.load()
    d = lib.make_desc(4, 32, 64, 64)
    ok = 0x10000
    assert L.mi355x_wq_matmul(d, None, ok, ok, ok, 1, None) == -1 and "x is NULL" in lib.last_error()
    assert L.mi355x_wq_matmul(d, ok, ok + 8, ok, ok, 1, None) == -1 and "wq" in lib.last_error() \
        and "16-byte aligned" in lib.last_error()
    assert L.mi355x_wq_matmul(d, ok, ok, ok + 1, ok, 1, None) == -1 and "scales" in lib.last_error()
    assert L.mi355x_wq_dequantize(d, ok, ok, ok + 4, None) == -1 and "wd" in lib.last_error()
    # empty problems succeed without touching the device
    assert L.mi355x_wq_matmul(d, None, None, None, None, 0, None) == 0
    d0 = lib.make_desc(4, 32, 0, 64)
    assert L.mi355x_wq_matmul(d0, None, None, None, None, 3, None) == 0
    assert L.mi355x_wq_dequantize(d0, None, None, None, None) == 0
    assert L.mi355x_wq_matmul_ex(d, ok, ok, ok, ok, 300, None, lib.KERNEL_SKINNY) == -1 \
        and "exceeds 256" in lib.last_error()
    assert L.mi355x_wq_matmul_ex(d, ok, ok, ok, ok, 1, None, 77) == -1 and "unknown kernel family" in lib.last_error()


# ---------------------------------------------------------------- PackedFunc boundary, error paths
def _cpu_case(m=2, n=16, k=64, bits=4):
    per = 32 // bits
    g = 32 if bits == 4 else 16
    x = torch.zeros((m, k), dtype=torch.float16)
    wq = torch.zeros((n, k // per), dtype=torch.int32)
    s = torch.zeros((n, k // g), dtype=torch.float16)
    y = torch.zeros((m, n), dtype=torch.float16)
    return x, wq, s, y


def _args(x, wq, s, y, **kw):
    return [vm_harness.TensorArg(x, **kw), vm_harness.TensorArg(wq, as_uint32=True, **kw),
            vm_harness.TensorArg(s, **kw), vm_harness.TensorArg(y, **kw)]


def test_packed_rejects_host_tensors():
    with pytest.raises(vm_harness.PackedError, match="expected a ROCm tensor"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(*_cpu_case()))


def test_packed_argument_count_and_type_codes():
    x, wq, s, y = _cpu_case()
    a = _args(x, wq, s, y, device_type=10)
    with pytest.raises(vm_harness.PackedError, match="expects 4 arguments, got 3"):
        vm_harness.call_packed("mi355x_q4f16_matmul", a[:3])
    with pytest.raises(vm_harness.PackedError, match="expects 3 arguments, got 4"):
        vm_harness.call_packed("mi355x_q4f16_dequantize", a)
    with pytest.raises(vm_harness.PackedError, match="expected a tensor"):
        vm_harness.call_packed("mi355x_q4f16_matmul", [a[0], 5, a[2], a[3]])
    with pytest.raises(vm_harness.PackedError, match="expected a tensor"):
        vm_harness.call_packed("mi355x_q4f16_matmul", [a[0], None, a[2], a[3]])


def test_packed_dtype_shape_and_stride_checks():
    x, wq, s, y = _cpu_case()
    dev = dict(device_type=10)
    with pytest.raises(vm_harness.PackedError, match=r"argument 1 \(wq\): expected dtype uint32"):
        vm_harness.call_packed("mi355x_q4f16_matmul", [
            vm_harness.TensorArg(x, **dev), vm_harness.TensorArg(wq, **dev),  # int32, not uint32
            vm_harness.TensorArg(s, **dev), vm_harness.TensorArg(y, **dev)])
    with pytest.raises(vm_harness.PackedError, match=r"argument 0 \(x\): expected dtype float16"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(x.float(), wq, s, y, **dev))
    with pytest.raises(vm_harness.PackedError, match="x has 32 columns but the weights have K=64"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(x[:, :32].contiguous(), wq, s, y, **dev))
    with pytest.raises(vm_harness.PackedError, match=r"y has shape \(2, 8\), expected \(2, 16\)"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(x, wq, s, y[:, :8].contiguous(), **dev))
    with pytest.raises(vm_harness.PackedError, match="scales has 8 rows but wq has 16"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(x, wq, s[:8].contiguous(), y, **dev))
    # a 1-d x is one row of its length (leading extents fold into the rows): 128 columns against K = 64
    with pytest.raises(vm_harness.PackedError, match="x has 128 columns but the weights have K=64"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(x.reshape(-1), wq, s, y, **dev)[:1] +
                               _args(x, wq, s, y, **dev)[1:])
    # the weights stay 2-d
    with pytest.raises(vm_harness.PackedError, match=r"argument 1 \(wq\): expected a 2-d tensor"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(x, wq, s, y, **dev)[:1] +
                               [vm_harness.TensorArg(wq.reshape(2, 8, -1), as_uint32=True, **dev)] + _args(x, wq, s, y, **dev)[2:])
    # x[1, 2, K] with a 2-d output: the leading extents must repeat
    with pytest.raises(vm_harness.PackedError, match="with the leading extents of x"):
        vm_harness.call_packed("mi355x_q4f16_matmul", _args(x.reshape(1, 2, -1), wq, s, y, **dev))
    xt = torch.zeros((64, 2), dtype=torch.float16).t()  # shape (2, 64), strides (1, 2)
    with pytest.raises(vm_harness.PackedError, match="not compact row-major"):
        vm_harness.call_packed("mi355x_q4f16_matmul", [
            vm_harness.TensorArg(xt, with_strides=True, **dev)] + _args(x, wq, s, y, **dev)[1:])
    # K / scales columns must give a legal group: 64 / 3 is not an integer
    with pytest.raises(vm_harness.PackedError, match="cannot infer the group size"):
        vm_harness.call_packed("mi355x_q4f16_matmul",
                               _args(x, wq, torch.zeros((16, 3), dtype=torch.float16), y, **dev))
    # q8 entry on q4-shaped data: K = 8 words * 4 = 32, x has 64 columns
    with pytest.raises(vm_harness.PackedError, match="x has 64 columns but the weights have K=32"):
        vm_harness.call_packed("mi355x_q8f16_matmul", _args(x, wq, s, y, **dev))


def test_packed_empty_output_is_a_no_op():
    x, wq, s, y = _cpu_case(m=0)
    vm_harness.call_packed("mi355x_q4f16_matmul", _args(x, wq, s, y, device_type=10))


def test_generic_entry_checks_the_call_spec():
    x, wq, s, y = _cpu_case()
    a = _args(x, wq, s, y, device_type=10)
    bad = vm_harness.CallSpec(0, 4, 0, 7, 0, 1, 1, 3, 4)  # two roles on argument 1
    with pytest.raises(vm_harness.PackedError, match="not a permutation"):
        vm_harness.call_packed(None, a, spec=bad)
    with pytest.raises(vm_harness.PackedError, match="unknown op"):
        vm_harness.call_packed(None, a, spec=vm_harness.CallSpec(7, 4, 0, 7, 0, 1, 2, 3, 4))
    # explicit group that contradicts the scales shape
    with pytest.raises(vm_harness.PackedError, match="does not match K=64 / group=64"):
        vm_harness.call_packed(None, a, spec=vm_harness.CallSpec(0, 4, 64, 7, 0, 1, 2, 3, 4))
    # roles permuted the way FuseOpsByPattern orders them: (wq, scales, x, y)
    permuted = [a[1], a[2], a[0], a[3]]
    spec = vm_harness.CallSpec(0, 4, 0, 7, 2, 0, 1, 3, 4)
    if not torch.cuda.is_available():  # all checks pass; only the missing device stops the call
        with pytest.raises(vm_harness.PackedError, match="no usable HIP device"):
            vm_harness.call_packed(None, permuted, spec=spec)


def test_fused_entries_check_their_extra_operand():
    x, wq, s, y = _cpu_case()
    dev = dict(device_type=10)
    a = _args(x, wq, s, y, **dev)
    bias = vm_harness.TensorArg(torch.zeros(16, dtype=torch.float16), **dev)
    bias2d = vm_harness.TensorArg(torch.zeros((1, 16), dtype=torch.float16), **dev)
    res = vm_harness.TensorArg(torch.zeros((2, 16), dtype=torch.float16), **dev)
    for sym in ("mi355x_q4f16_matmul_bias", "mi355x_q4f16_matmul_bias_relu", "mi355x_q4f16_matmul_residual"):
        with pytest.raises(vm_harness.PackedError, match="expects 5 arguments, got 4"):
            vm_harness.call_packed(sym, a)
    with pytest.raises(vm_harness.PackedError, match=r"bias has shape \(1, 8\), expected \(16\) or \(1, 16\)"):
        vm_harness.call_packed("mi355x_q4f16_matmul_bias", a[:3] + [
            vm_harness.TensorArg(torch.zeros(8, dtype=torch.float16), **dev), a[3]])
    with pytest.raises(vm_harness.PackedError, match=r"bias has shape \(2, 16\)"):
        vm_harness.call_packed("mi355x_q4f16_matmul_bias", a[:3] + [res, a[3]])
    with pytest.raises(vm_harness.PackedError, match=r"argument 3 \(bias\): expected dtype float16"):
        vm_harness.call_packed("mi355x_q4f16_matmul_bias_relu", a[:3] + [
            vm_harness.TensorArg(torch.zeros(16, dtype=torch.float32), **dev), a[3]])
    with pytest.raises(vm_harness.PackedError, match=r"residual has shape \(1, 16\), expected \(2, 16\)"):
        vm_harness.call_packed("mi355x_q4f16_matmul_residual", a[:3] + [bias2d, a[3]])
    with pytest.raises(vm_harness.PackedError, match=r"residual has shape \(1, 16\), expected \(2, 16\)"):
        vm_harness.call_packed("mi355x_q4f16_matmul_residual", a[:3] + [bias, a[3]])
    if not torch.cuda.is_available():  # every check passes; only the missing device stops the calls
        for sym, extra in (("mi355x_q4f16_matmul_bias", bias), ("mi355x_q4f16_matmul_bias", bias2d),
                           ("mi355x_q4f16_matmul_bias_relu", bias), ("mi355x_q4f16_matmul_residual", res)):
            with pytest.raises(vm_harness.PackedError, match="no usable HIP device"):
                vm_harness.call_packed(sym, a[:3] + [extra, a[3]])
    # generic entry: bias and residual together, roles permuted; bad activation / roles rejected
    spec = vm_harness.CallSpec(0, 4, 0, 7, 2, 0, 1, 5, 6, 3, 4, 1)
    order = [a[1], a[2], a[0], bias, res, a[3]]
    if not torch.cuda.is_available():
        with pytest.raises(vm_harness.PackedError, match="no usable HIP device"):
            vm_harness.call_packed(None, order, spec=spec)
    with pytest.raises(vm_harness.PackedError, match="not a permutation"):
        vm_harness.call_packed(None, order, spec=vm_harness.CallSpec(0, 4, 0, 7, 2, 0, 1, 5, 6, 3, 3, 0))
    with pytest.raises(vm_harness.PackedError, match="dequantize takes no fused operands"):
        vm_harness.call_packed(None, a[1:], spec=vm_harness.CallSpec(1, 4, 0, 7, 0, 0, 1, 2, 3, 1, -1, 0))


def test_fused_c_entry_validates_the_epilogue():
    L = lib.load()
    d = lib.make_desc(4, 32, 16, 64)
    ep = lib.WqEpilogue(None, None, 7, 0)
    assert L.mi355x_wq_matmul_fused(d, 16, 16, 16, ep, 16, 2, None) == -1
    assert "unknown epilogue activation 7" in lib.last_error()
    ep = lib.WqEpilogue(None, None, 0, 1)
    assert L.mi355x_wq_matmul_fused(d, 16, 16, 16, ep, 16, 2, None) == -1
    assert "epilogue.reserved must be 0" in lib.last_error()
    ep = lib.WqEpilogue(3, None, 1, 0)  # odd bias pointer
    assert L.mi355x_wq_matmul_fused(d, 16, 16, 16, ep, 16, 2, None) == -1
    assert "bias" in lib.last_error() and "aligned" in lib.last_error()
    ep = lib.WqEpilogue(None, 5, 0, 0)
    assert L.mi355x_wq_matmul_fused(d, 16, 16, 16, ep, 16, 2, None) == -1
    assert "residual" in lib.last_error() and "aligned" in lib.last_error()
    # an empty output is a no-op whatever the epilogue
    assert L.mi355x_wq_matmul_fused(d, None, None, None, lib.WqEpilogue(None, None, 1, 0), None, 0, None) == 0


def test_stream_setter_round_trip():
    L = lib.load()
    L.mi355x_wq_packed_set_stream(0x1230)
    assert L.mi355x_wq_packed_get_stream() == 0x1230
    L.mi355x_wq_packed_set_stream(None)
    assert not L.mi355x_wq_packed_get_stream()


# ---------------------------------------------------------------- registration in a TVM-like registry
REGISTRY_SCRIPT = r"""
import ctypes as C, os, sys
sys.path.insert(0, {root!r})
from relax_amd import lib, vm_harness
import torch
L = lib.load()
assert L.mi355x_wq_register_tvm_globals(0) == -1 and "no TVM runtime" in lib.last_error()
fake = C.CDLL({fake!r}, mode=C.RTLD_GLOBAL)
fake.fake_tvm_name.restype = C.c_char_p
fake.fake_tvm_last_error.restype = C.c_char_p
assert L.mi355x_wq_register_tvm_globals(0) == 20
names = sorted(fake.fake_tvm_name(i).decode() for i in range(fake.fake_tvm_count()))
assert names == sorted("mi355x." + s[len("mi355x_"):] for s in lib.PACKED_ENTRIES), names
# call a registered function the way the registry would, with host tensors: it must fail and the
# message must arrive in the host's last-error slot (what LOG(FATAL) << TVMGetLastError() prints)
idx = [fake.fake_tvm_name(i).decode() for i in range(10)].index("mi355x.q4f16_matmul")
x = torch.zeros((1, 64), dtype=torch.float16); wq = torch.zeros((16, 8), dtype=torch.int32)
s = torch.zeros((16, 2), dtype=torch.float16); y = torch.zeros((1, 16), dtype=torch.float16)
ta = [vm_harness.TensorArg(x), vm_harness.TensorArg(wq, as_uint32=True), vm_harness.TensorArg(s),
      vm_harness.TensorArg(y)]
vals = (vm_harness.TVMValue * 4)(); codes = (C.c_int * 4)()
for i, t in enumerate(ta):
    vals[i].v_handle = t.handle; codes[i] = 13
fake.fake_tvm_call.argtypes = [C.c_int, C.c_void_p, C.POINTER(C.c_int), C.c_int]
assert fake.fake_tvm_call(idx, C.addressof(vals), codes, 4) == -1
assert b"expected a ROCm tensor" in fake.fake_tvm_last_error()
print("registry ok")
"""


def test_registration_through_the_tvm_c_api(tmp_path):
    fake = str(tmp_path / "libfake_tvm.so")
    subprocess.check_call(["gcc", "-shared", "-fPIC", "-o", fake,
                           os.path.join(ROOT, "tests", "support", "fake_tvm_registry.c")])
    # own process: the fake registry must not stay loaded for the other tests
    out = subprocess.run([sys.executable, "-c", REGISTRY_SCRIPT.format(root=ROOT, fake=fake)],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "registry ok" in out.stdout, out.stdout + out.stderr


# ---------------------------------------------------------------- the headers are plain C, usable without Python
C_CLIENT = r"""
#include <stdio.h>
#include <string.h>
#include "mi355x_wq.h"
#include "mi355x_wq_packed.h"
#include "mi355x_wq_module.h"

int main(void) {
  mi355x_wq_desc d = {4, 32, 7, 0, 4096, 4096};
  mi355x_wq_epilogue ep = {NULL, NULL, MI355X_WQ_ACT_RELU, 0};
  mi355x_wq_callspec spec = {0, 4, 0, 7, 0, 1, 2, 3, 4, -1, -1, MI355X_WQ_ACT_NONE};
  if (mi355x_wq_version() < 100) return 1;
  if (mi355x_wq_check(&d, 8) != 0) return 2;
  if (mi355x_wq_select_kernel(&d, 8) != MI355X_WQ_KERNEL_GEMV) return 3;
  d.group = 48;
  if (mi355x_wq_check(&d, 8) != -1 || strstr(mi355x_wq_last_error(), "group") == NULL) return 4;
  d.group = 32;
  /* a NULL operand is refused before anything touches the GPU */
  if (mi355x_wq_matmul_fused(&d, NULL, NULL, NULL, &ep, NULL, 8, NULL) != -1) return 5;
  if (strstr(mi355x_wq_last_error(), "x is NULL") == NULL) return 6;
  if (mi355x_wq_packed_call(&spec, NULL, NULL, 4) != -1) return 7;
  if (sizeof(mi355x_dl_tensor) != 48 || sizeof(mi355x_tvm_value) != 8) return 8;  /* DLPack / TVMValue ABI sizes */
  {
    /* the subgraph module from plain C: create, look a function up, save, load, destroy */
    const char* names[2] = {"w", "s"};
    int32_t slots[2] = {1, 2};
    mi355x_wq_module *mod = NULL, *back = NULL;
    mi355x_wq_packed_cfunc fn = NULL;
    void* res = NULL;
    char buf[512];
    int64_t used = 0, n;
    if (mi355x_wq_module_create("sym0", &spec, names, slots, 2, 0, &mod) != 0) return 9;
    if (mi355x_wq_module_get_function(mod, "__init_sym0", &fn, &res) != 0 || fn == NULL || res != (void*)mod) return 10;
    if (mi355x_wq_module_get_function(mod, "other", &fn, &res) != 0 || fn != NULL) return 11;
    n = mi355x_wq_module_save_to_binary(mod, buf, (int64_t)sizeof(buf));
    if (n <= 0 || n > (int64_t)sizeof(buf)) return 12;
    if (mi355x_wq_module_load_from_binary(buf, n, &used, &back) != 0 || used != n) return 13;
    if (strcmp(mi355x_wq_module_symbol(back), "sym0") != 0 || mi355x_wq_module_num_consts(back) != 2) return 14;
    if (strcmp(mi355x_wq_module_json(back), mi355x_wq_module_json(mod)) != 0) return 15;
    mi355x_wq_module_destroy(back);
    if (mi355x_wq_module_create_from_json("sym1", mi355x_wq_module_json(mod), names, 2, &back) != 0) return 16;
    if (strcmp(mi355x_wq_module_symbol(back), "sym1") != 0 || mi355x_wq_module_initialized(back) != 0) return 17;
    mi355x_wq_module_destroy(back);
    if (mi355x_wq_module_create_from_json("sym1", "{}", names, 2, &back) != -1 || back != NULL) return 18;
    mi355x_wq_module_destroy(mod);
  }
  puts("c client ok");
  return 0;
}
"""


def test_headers_compile_as_c99_and_link(tmp_path):
    src = tmp_path / "client.c"
    src.write_text(C_CLIENT)
    exe = str(tmp_path / "client")
    libdir = os.path.dirname(lib.SO_PATH)
    subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                           "-o", exe, str(src), "-L" + libdir, "-lmi355x_wq", "-Wl,-rpath," + libdir])
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0 and "c client ok" in out.stdout, (out.returncode, out.stdout, out.stderr)
