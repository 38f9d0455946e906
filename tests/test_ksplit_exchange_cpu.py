"""The cross-workgroup K split exchanges partial tiles and arrival counters without cache-wide fences; that is
sound only while every access to those words is an agent-scope access performed at the memory side (`sc1`).  A
plain load could be served from a stale line of the reader's L2 (the workspace is rewritten by every launch), a
plain store could stay dirty in the writer's L2.  This test reads the two kernels' sources and refuses any access
to the exchanged words that is not one of the agent-scope forms."""
import os
import re

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "relax_amd", "csrc")


def _kernel_body(text, marker):
    """From `marker` to the end of the enclosing kernel (the next line that starts a namespace block)."""
    start = text.index(marker)
    end = text.index("\nnamespace {", start)
    return text[start:end]


def _statements(body):
    # comments out, then split on ';' (good enough for the straight-line exchange code)
    body = re.sub(r"//[^\n]*", "", body)
    return [s.strip() for s in body.split(";") if s.strip()]


def test_decode_split_touches_partials_and_counters_only_through_agent_scope_atomics():
    text = open(os.path.join(CSRC, "wq_gemv.hip")).read()
    body = _kernel_body(text, "// K split over R workgroups: every workgroup writes its float32 partial tile")
    touched = 0
    for st in _statements(body):
        if not re.search(r"\b(partials_|counters_|part)\b", st):
            continue
        touched += 1
        if re.match(r"(float\* const part = partials_ \+|const .* = )", st) and "*part" not in st and "part[" not in st \
                and "__hip_atomic" not in st:
            continue  # pointer arithmetic, no access
        assert "__hip_atomic_" in st and "__HIP_MEMORY_SCOPE_AGENT" in st, st
        assert re.search(r"__hip_atomic_(store|load|fetch_add)\(", st), st
        assert "partials_[" not in re.sub(r"__hip_atomic_\w+\(&partials_\[", "", st), st
    assert touched >= 5, touched
    # and nothing dereferences them outside that block
    outside = text.replace(body, "")
    kernel = outside[outside.index("__global__"):outside.index("\nnamespace {", outside.index("__global__"))]
    assert not re.search(r"(partials_|counters_)\s*\[", kernel), "an access to the workspace outside the exchange block"


def test_gemm_split_touches_partials_and_counters_only_through_sc1_accesses():
    text = open(os.path.join(CSRC, "wq_gemm_direct.hip")).read()
    kernel = text[text.index("__global__"):]
    kernel = kernel[:kernel.index("\nnamespace {")]
    code = re.sub(r"//[^\n]*", "", kernel)
    # the partial tiles are reached through one buffer resource, and every load / store on it carries the sc1 bit
    # (auxiliary operand 0x10 of the raw buffer intrinsics)
    assert len(re.findall(r"make_rsrc\(partials", code)) == 1
    uses = re.findall(r"__builtin_amdgcn_raw_buffer_(?:load|store)_b128\((?:[^;]*?)\brp\b[^;]*?\)\s*;", code, re.S)
    assert len(uses) >= 2, len(uses)
    for u in uses:
        assert re.search(r",\s*0,\s*0x10\)\s*;$", u), u
    assert not re.search(r"\bpartials\s*\[", code), "a plain access to the partial tiles"
    # the counters: atomic add and atomic store at agent scope, nothing else
    for st in _statements(code):
        if re.search(r"\bcounters\b", st) and "unsigned int* counters" not in st:
            assert re.search(r"__hip_atomic_(fetch_add|store)\(&counters\[", st) and "__HIP_MEMORY_SCOPE_AGENT" in st, st
