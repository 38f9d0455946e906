"""Pattern entries for `relax.transform.FuseOpsByPattern` (the table the reference passes
ad hoc, python/tvm/relax/transform/transform.py:324-356; priority = list order).

The composite the backend takes over is the idiomatic weight-only-quantized linear layer

    Wd  = R.call_tir(decode_q{4,8}f16, (Wq, S), R.Tensor((N, K), "float16"))
    y32 = R.matmul(x, R.permute_dims(Wd), out_dtype="float32")
    y   = R.astype(y32, "float16")

`matmul(x, permute_dims(W))` is what `relax.op.linear` expands to
(python/tvm/relax/op/linear_algebra.py:54-90).  The pattern name's prefix before the
first "." becomes the `Codegen` attribute, i.e. the backend name
(src/relax/transform/fuse_ops.cc:1039-1044).

Verified by reading, not by running: TVM cannot be built or imported in this build's
environment.
"""
from __future__ import annotations

BACKEND = "mi355x"

# decode PrimFunc global symbols the patterns look for, with the quantization they imply
DECODE_FUNCS = {
    "decode_q4f16": {"bits": 4, "zero_point": 7},
    "decode_q8f16": {"bits": 8, "zero_point": 0},
}


def patterns():
    """[(name, DFPattern)] for FuseOpsByPattern(patterns, annotate_codegen=True)."""
    from tvm.relax.dpl import is_call_tir, is_op, wildcard  # python/tvm/relax/dpl/pattern.py:678-837

    table = []
    for fn_name, q in DECODE_FUNCS.items():
        decoded = is_call_tir(fn_name, [wildcard(), wildcard()])
        weight_t = is_op("relax.permute_dims")(decoded)
        mm = is_op("relax.matmul")(wildcard(), weight_t)
        table.append((f"{BACKEND}.q{q['bits']}f16_matmul", is_op("relax.astype")(mm)))
    return table


def partition(mod):
    """FuseOpsByPattern + RunCodegen with this backend, the two calls of
    tests/python/relax/test_codegen_cutlass.py:223-240 for the cutlass backend."""
    from tvm import relax

    from .codegen import register

    register()
    mod = relax.transform.FuseOpsByPattern(patterns(), annotate_codegen=True)(mod)
    return relax.transform.RunCodegen()(mod)
