"""bench.py's host-side logic, without a GPU: the one-GPU rule, the traffic figure's digest check and the workload's
byte count."""
import hashlib
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and "--gpus must be 1" in r.stderr
    assert r.stdout.strip() == ""  # no JSON line that could be taken for a measurement


def test_traffic_is_reported_only_for_the_sources_it_was_measured_on(tmp_path):
    src = tmp_path / "kernel.hip"
    src.write_text("__global__ void k() {}\n")
    digest = bench.kernel_sources_digest([str(src)])
    assert digest == hashlib.sha256(src.read_bytes()).hexdigest()
    prof = tmp_path / "profile.md"
    prof.write_text(f"# a summary\n\ntraffic_bytes_per_launch: 123456\nkernel_sources_sha256: {digest}\n")
    assert bench.measured_traffic(str(prof), [str(src)]) == 123456
    src.write_text("__global__ void k() { }\n")  # the kernel changed: the figure is stale
    assert bench.measured_traffic(str(prof), [str(src)]) is None
    assert bench.measured_traffic(str(tmp_path / "missing.md"), [str(src)]) is None
    prof.write_text("traffic_bytes_per_launch: 123456\n")  # no digest: not trusted
    assert bench.measured_traffic(str(prof), [str(src)]) is None


def test_tracked_profiles_carry_both_lines():
    for name in ("gemv_decode_llama7b.md", "gemm_prefill_llama7b.md"):
        text = open(os.path.join(ROOT, "profiles", name)).read()
        assert "\ntraffic_bytes_per_launch: " in text and "\nkernel_sources_sha256: " in text, name


def test_decode_workload_bytes():
    # packed int4 weights + float16 group scales + x + y, the four projections at batch 1 and batch 8
    total = 0
    for _, n, k in bench.LLAMA7B:
        for m in bench.DECODE_BATCHES:
            total += n * k // 2 + n * (k // 32) * 2 + m * k * 2 + m * n * 2
    assert total == 8 * 28_607_040
    assert [(n, k) for _, n, k in bench.LLAMA7B] == [(12288, 4096), (4096, 4096), (22016, 4096), (4096, 11008)]
    assert tuple(bench.DECODE_BATCHES) == (1, 8)
