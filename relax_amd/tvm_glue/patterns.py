"""Pattern entries for `relax.transform.FuseOpsByPattern` (the table the reference passes
ad hoc, python/tvm/relax/transform/transform.py:324-356; priority = list order).

The composite the backend takes over is the idiomatic weight-only-quantized linear layer

    Wd  = R.call_tir(decode_q{4,8}f16, (Wq, S), R.Tensor((N, K), "float16"))
    y32 = R.matmul(x, R.permute_dims(Wd), out_dtype="float32")
    y   = R.astype(y32, "float16")

optionally followed by the element-wise tail the reference's `make_matmul_pattern(with_bias,
activation)` describes for its CUTLASS backend (python/tvm/relax/dpl/pattern.py:1049-1095:
`add`, then `relax.nn.relu` or `relax.nn.gelu`), and by the residual add of a decoder layer:

    y = R.add(y, bias)            # bias [N] or [1, N]
    y = R.nn.relu(y)
    y = R.add(y, residual)        # residual [M, N]

or by the gated tail of a Llama MLP, whose gate and up projections share one weight matrix (gate rows,
then as many up rows):

    sp  = R.split(y, 2, axis=-1)                   # the last axis, by either of its two indices
    out = R.multiply(R.nn.silu(sp[0]), sp[1])      # [M, N/2]; multiply is matched in both operand orders

x may carry leading extents, `x[B, S, K]` against the 2-d weight (src/relax/op/tensor/linear_algebra.cc:46-114):
the kernels see M = B * S rows.

`matmul(x, permute_dims(W))` is what `relax.op.linear` expands to
(python/tvm/relax/op/linear_algebra.py:54-90).  The pattern name's prefix before the
first "." becomes the `Codegen` attribute, i.e. the backend name
(src/relax/transform/fuse_ops.cc:1039-1044).

TVM cannot be built or imported in this build's environment; the table is executed against a stand-in
`tvm.relax.dpl` whose matcher follows src/relax/ir/dataflow_matcher.cc (tests/support/fake_dpl.py).
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
    from tvm.relax.dpl import is_call_tir, is_op, is_tuple_get_item, wildcard  # python/tvm/relax/dpl/pattern.py:678-837
    from tvm.tir import IntImm

    def core(fn_name):
        # Only the float32-accumulating form is taken: with out_dtype "" or "float16" the CPU path
        # accumulates in float16 (python/tvm/relax/transform/legalize_ops.py:250-258), which the kernels
        # do not reproduce.  A string matches a DataType attribute (src/relax/ir/dataflow_matcher.cc:128-133).
        decoded = is_call_tir(fn_name, [wildcard(), wildcard()])
        weight_t = is_op("relax.permute_dims")(decoded)
        mm = is_op("relax.matmul")(wildcard().has_dtype("float16"), weight_t).has_attr({"out_dtype": "float32"})
        return is_op("relax.astype")(mm).has_attr({"dtype": "float16"})

    # Longest tail first: earlier entries have priority (transform.py:337-339).  A pattern cannot
    # tell a [N] bias from a [M, N] residual (no shape predicate without concrete extents); the
    # codegen hook decides from the operand's shape and rejects what the epilogue cannot express.
    table = []
    for fn_name, q in DECODE_FUNCS.items():
        base = f"{BACKEND}.q{q['bits']}f16_matmul"
        add1 = lambda: is_op("relax.add")(core(fn_name), wildcard())  # noqa: E731
        relu = lambda: is_op("relax.nn.relu")(add1())                 # noqa: E731
        gelu = lambda: is_op("relax.nn.gelu")(add1())                 # noqa: E731
        # The section count of relax.op.split is an int64 IntImm (python/tvm/relax/op/manipulate.py:238-240) and an
        # object-valued attribute is compared structurally, dtype included (src/relax/ir/dataflow_matcher.cc:139-147):
        # a Python 2 would arrive as an int32 IntImm and never match.  The axis is an `int` field, compared by value
        # (:110-114) and stored as written: the last axis of a 2-d or 3-d output is -1, 1 or 2 -- an attribute
        # pattern holds one value per key, hence the alternatives.  (A 3-d output split along axis 1 would match
        # too; the hook refuses it.)  One pattern object for the split: both halves must come from the same one.
        split = is_op("relax.split")(core(fn_name))
        two = IntImm("int64", 2)
        halves = (split.has_attr({"indices_or_sections": two, "axis": -1})
                  | split.has_attr({"indices_or_sections": two, "axis": 1})
                  | split.has_attr({"indices_or_sections": two, "axis": 2}))
        gated = is_op("relax.multiply")(is_op("relax.nn.silu")(is_tuple_get_item(halves, 0)),
                                        is_tuple_get_item(halves, 1))
        table.append((base + "_silu_mul", gated))
        table.append((base + "_add_relu_add", is_op("relax.add")(relu(), wildcard())))
        table.append((base + "_add_add", is_op("relax.add")(add1(), wildcard())))
        table.append((base + "_add_gelu_add", is_op("relax.add")(gelu(), wildcard())))
        table.append((base + "_add_relu", relu()))
        table.append((base + "_add_gelu", gelu()))
        table.append((base + "_add", add1()))
        table.append((base, core(fn_name)))
    return table


def partition(mod):
    """FuseOpsByPattern + RunCodegen with this backend, the two calls of
    tests/python/relax/test_codegen_cutlass.py:223-240 for the cutlass backend."""
    from tvm import relax

    from .codegen import register

    register()
    mod = relax.transform.FuseOpsByPattern(patterns(), annotate_codegen=True)(mod)
    return relax.transform.RunCodegen()(mod)
