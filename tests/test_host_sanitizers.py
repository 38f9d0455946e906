"""The host side of the library under AddressSanitizer and UndefinedBehaviorSanitizer.

`make -C relax_amd/csrc sanitize` compiles wq_capi.cpp, wq_packed.cpp and wq_module.cpp with
-fsanitize=address,undefined (host pass only), links them with the ordinary kernel objects into
tests/host_sanitize/san_driver and runs it: argument validation, the PackedFunc boundary and the
module's binary loader / JSON reader on every truncation and thousands of corruptions of a good
module.  No GPU is needed; a sanitizer report or a failed expectation fails the make target.
"""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_code_is_clean_under_asan_and_ubsan():
    res = subprocess.run(["make", "-C", os.path.join(ROOT, "relax_amd", "csrc"), "sanitize"],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1500)
    out = res.stdout
    assert res.returncode == 0, out[-4000:]
    assert "host sanitizer run: ok" in out, out[-4000:]
    assert "ERROR: AddressSanitizer" not in out and "runtime error:" not in out, out[-4000:]
