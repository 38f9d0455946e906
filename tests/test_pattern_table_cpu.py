"""The pattern table executed: every entry of `patterns()` against stand-in IR of the composites, with a matcher
that follows the reference's rules (tests/support/fake_dpl.py <-> src/relax/ir/dataflow_matcher.cc), applied the
way FuseOpsByPattern applies a table (src/relax/transform/fuse_ops.cc:1050-1066).  The reference keeps patterns and
matcher tests side by side the same way (tests/python/relax/test_transform_fuse_ops_by_pattern.py:341-385)."""
import sys

import pytest

from tests.support import fake_dpl, fake_relax
from tests.support.fake_dpl import IntImm


@pytest.fixture
def table(monkeypatch):
    fake_dpl.install(monkeypatch, sys.modules)
    from relax_amd.tvm_glue.patterns import patterns

    return patterns()


def _body(func):
    """The bindings of the composite inside an annotated function: what `main` held before FuseOpsByPattern."""
    composite = func.body.blocks[0].bindings[0].value
    return composite.body.blocks[0].bindings


TAILS = {
    "": (),
    "_add": (("add", [48]),),
    "_add_relu": (("add", [48]), ("relu",)),
    "_add_gelu": (("add", [1, 48]), ("gelu",)),
    "_add_add": (("add", [48]), ("add", [4, 48])),
    "_add_relu_add": (("add", [48]), ("relu",), ("add", [4, 48])),
    "_add_gelu_add": (("add", [48]), ("gelu",), ("add", [4, 48])),
    "_silu_mul": (("silu_mul",),),
}


@pytest.mark.parametrize("decode,prefix", [("decode_q4f16", "mi355x.q4f16_matmul"), ("decode_q8f16", "mi355x.q8f16_matmul")])
@pytest.mark.parametrize("suffix", sorted(TAILS))
def test_every_entry_claims_its_composite_and_the_longest_wins(table, decode, prefix, suffix):
    names = [n for n, _ in table]
    assert len(names) == len(set(names)) == 16
    func = fake_relax.quantized_linear(decode=decode, tail=TAILS[suffix])
    bindings = _body(func)
    groups = fake_dpl.partition(bindings, table)
    # one group, under the entry named for exactly this tail, holding every binding of the chain
    assert [g[0] for g in groups] == [prefix + suffix], groups
    assert len(groups[0][1]) == len(bindings), (groups, [b.var.name_hint for b in bindings])
    # and the entry itself matches rooted at the last call, the entries for other tails of equal or greater
    # length do not
    own = dict(table)[prefix + suffix]
    var2val = {b.var: b.value for b in bindings}
    assert fake_dpl.match(own, bindings[-1].value, var2val) is not None
    other = "decode_q8f16" if decode == "decode_q4f16" else "decode_q4f16"
    assert fake_dpl.partition(_body(fake_relax.quantized_linear(decode=other, tail=TAILS[suffix])), [(prefix + suffix, own)]) == []


def test_operands_in_the_other_order_still_match(table):
    """relax.add and relax.multiply are matched in both argument orders (dataflow_matcher.cc:252-258)."""
    func = fake_relax.quantized_linear(tail=(("add", [48], True), ("relu",), ("add", [4, 48], True)))
    assert [g[0] for g in fake_dpl.partition(_body(func), table)] == ["mi355x.q4f16_matmul_add_relu_add"]
    func = fake_relax.quantized_linear(tail=(("silu_mul", 2, -1, False, True),))
    assert [g[0] for g in fake_dpl.partition(_body(func), table)] == ["mi355x.q4f16_matmul_silu_mul"]


@pytest.mark.parametrize("kwargs", [dict(out_dtype=""), dict(out_dtype="float16"), dict(astype_dtype="float32"),
                                    dict(x_dtype="float32"), dict(decode="decode_q3f16")])
def test_what_the_kernels_do_not_compute_stays_on_the_default_path(table, kwargs):
    """float16 accumulation (out_dtype "" or float16), a float32 result, float32 activations or another decode
    function: no entry matches, nothing is grouped."""
    func = fake_relax.quantized_linear(tail=(("add", [48]),), **kwargs)
    assert fake_dpl.partition(_body(func), table) == []


@pytest.mark.parametrize("step", [("silu_mul", 4, -1), ("silu_mul", 2, 0), ("silu_mul", 2, -1, True)])
def test_a_split_that_is_not_the_gated_tail_leaves_the_plain_matmul(table, step):
    """Four sections, a split along the rows, or silu on the second half: the gated entry does not match and the
    projection partitions as the plain matmul (the split, silu and multiply stay outside)."""
    func = fake_relax.quantized_linear(tail=(step,))
    groups = fake_dpl.partition(_body(func), table)
    assert [g[0] for g in groups] == ["mi355x.q4f16_matmul"], groups
    assert groups[0][1] == ["wd", "wt", "y32", "y"]


def test_the_split_attribute_is_compared_with_its_dtype(table):
    """The section count is an object-valued attribute: an int32 IntImm (what a Python int becomes on the pattern
    side) is not structurally equal to the int64 one relax.op.split stores, so a pattern written with a bare 2
    never matches; the axis is an int field and compares by value."""
    from tests.support.fake_dpl import is_op, wildcard

    func = fake_relax.quantized_linear(tail=(("silu_mul",),))
    bindings = _body(func)
    split = next(b.value for b in bindings if getattr(b.value, "op", None) is not None and getattr(b.value.op, "name", "") == "relax.split")
    var2val = {b.var: b.value for b in bindings}
    assert fake_dpl.match(is_op("relax.split")(wildcard()).has_attr({"indices_or_sections": 2}), split, var2val) is None
    assert fake_dpl.match(is_op("relax.split")(wildcard()).has_attr({"indices_or_sections": IntImm("int64", 2)}), split, var2val)
    assert fake_dpl.match(is_op("relax.split")(wildcard()).has_attr({"axis": -1}), split, var2val)
    assert fake_dpl.match(is_op("relax.split")(wildcard()).has_attr({"axis": 1}), split, var2val) is None
    assert fake_dpl.match(is_op("relax.split")(wildcard()).has_attr({"no_such_attribute": 1}), split, var2val) is None


def test_three_dimensional_activations_partition_and_give_the_same_roles(table, monkeypatch):
    """x[B, S, K] against the 2-d weight (src/relax/op/tensor/linear_algebra.cc:46-114): the entries match, the hook
    folds the leading extents into the rows."""
    from relax_amd.tvm_glue import codegen

    for tail, name in (((), "mi355x.q4f16_matmul"), ((("add", [48]), ("add", [2, 5, 48])), "mi355x.q4f16_matmul_add_add"),
                       ((("silu_mul", 2, 2),), "mi355x.q4f16_matmul_silu_mul"), ((("silu_mul", 2, -1),), "mi355x.q4f16_matmul_silu_mul")):
        func = fake_relax.quantized_linear(tail=tail, x_shape=[2, 5, 128])
        assert [g[0] for g in fake_dpl.partition(_body(func), table)] == [name]
        spec = codegen.spec_from_function(func)
        assert (spec.arg_wq, spec.arg_scales, spec.arg_x) == (0, 1, 2)
        assert (spec.arg_bias, spec.arg_residual) == ((3, 4) if len(tail) == 2 else (-1, -1))
    # a 3-d output split along its middle axis matches the entry (an attribute pattern cannot see the rank) and is
    # refused by the hook
    func = fake_relax.quantized_linear(tail=(("silu_mul", 2, 1),), x_shape=[2, 5, 128])
    assert [g[0] for g in fake_dpl.partition(_body(func), table)] == ["mi355x.q4f16_matmul_silu_mul"]
    with pytest.raises(ValueError, match="last axis"):
        codegen.spec_from_function(func)
