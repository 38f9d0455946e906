"""A few dozen lines standing in for the `tvm.relax` classes that `spec_from_function` touches,
so that the role derivation can run without TVM.  Only structure is modelled: expressions,
bindings, functions with attributes, variables with a shape."""
import types


class Expr:
    def same_as(self, other):
        return self is other


class StructInfo:
    def __init__(self, shape, dtype=None):
        self.shape = list(shape)
        self.dtype = dtype


class Attrs:
    """Call attributes with attribute access, like an Attrs node (MatmulAttrs.out_dtype, ...).  The Python type
    of a field stands for the C++ type of the reference's field, which decides how a pattern's attribute test
    compares it (src/relax/ir/dataflow_matcher.cc:108-150): `int` for an int field (SplitAttrs.axis), `DataType`
    for a DataType field (MatmulAttrs.out_dtype, AstypeAttrs.dtype), `IntImm` / list for an object-valued field
    (SplitAttrs.indices_or_sections, PermuteDimsAttrs.axes)."""

    def __init__(self, **fields):
        self.__dict__.update(fields)


class IntImm:
    """tvm.tir.IntImm: a value with a dtype; structural equality tells int32 from int64."""

    def __init__(self, dtype, value):
        self.dtype, self.value = str(dtype), int(value)

    def __int__(self):
        return self.value

    def __index__(self):
        return self.value

    def __repr__(self):
        return f"IntImm({self.dtype!r}, {self.value})"


class DataType(str):
    """A DataType attribute field: reads back as its string in Python."""


class Var(Expr):
    def __init__(self, name, shape=None, dtype=None):
        self.name_hint = name
        self.struct_info = StructInfo(shape or [], dtype)

    def __hash__(self):
        return id(self)

    def __eq__(self, other):
        return self is other


class Constant(Expr):
    """A bound parameter: data plus shape; hashable by identity like the real node."""

    def __init__(self, shape, data=None, dtype=None):
        self.struct_info = StructInfo(shape, dtype)
        self.data = data

    def __hash__(self):
        return id(self)

    def __eq__(self, other):
        return self is other


class GlobalVar(Expr):
    def __init__(self, name):
        self.name_hint = name


class Op(Expr):
    def __init__(self, name):
        self.name = name


class Tuple(Expr):
    def __init__(self, fields):
        self.fields = list(fields)


class ExternFunc(Expr):
    """The callee of a call_tir after RunCodegen: a symbol resolved at run time."""

    def __init__(self, global_symbol):
        self.global_symbol = global_symbol


class TupleGetItem(Expr):
    def __init__(self, tuple_value, index):
        self.tuple_value, self.index = tuple_value, index


class Call(Expr):
    def __init__(self, op, args, attrs=None, sinfo_args=None):
        self.op = op
        self.args = list(args)
        self.attrs = attrs
        self.sinfo_args = list(sinfo_args or [])


class VarBinding:
    def __init__(self, var, value):
        self.var, self.value = var, value


class BindingBlock:
    def __init__(self, bindings):
        self.bindings = list(bindings)


class DataflowBlock(BindingBlock):
    """`with R.dataflow():` -- the body of a composite is one of these in the reference's goldens."""


class SeqExpr(Expr):
    def __init__(self, blocks, body):
        self.blocks, self.body = list(blocks), body


class Function(Expr):
    def __init__(self, params, body, attrs=None):
        self.params, self.body, self.attrs = list(params), body, dict(attrs or {})


def as_module():
    """A module object usable as `tvm` with a `relax` attribute."""
    relax = types.ModuleType("tvm.relax")
    for cls in (Var, Call, Function, Tuple, GlobalVar, SeqExpr, BindingBlock, DataflowBlock, VarBinding, Constant, ExternFunc, TupleGetItem, Op):
        setattr(relax, cls.__name__, cls)
    tvm = types.ModuleType("tvm")
    tvm.relax = relax
    return tvm, relax


def quantized_linear(decode="decode_q4f16", m=4, n=48, k=128, tail=(), outer_order=None, bound=(),
                     out_dtype="float32", astype_dtype="float16", axes=None, x_shape=None, x_dtype="float16",
                     symbol="fused_mi355x", golden_names=False):
    """The annotated function FuseOpsByPattern(annotate_codegen=True) produces for
    decode -> permute_dims -> matmul -> astype followed by `tail`, a sequence of
    ("add", shape) / ("relu",) / ("gelu",) steps.  Composite parameters are ordered by first use:
    (wq, scales, x, <tail operands in order>).  `outer_order` permutes the outer parameters.
    `bound` names operands ("wq", "scales", "operand<i>") that BindParams turned into constants: they sit
    inside the composite as Constant nodes and are no parameters."""
    per = 8 if "q4" in decode else 4
    group = 32 if "q4" in decode else 128
    wq = Constant([n, k // per], dtype="uint32") if "wq" in bound else Var("wq", [n, k // per], "uint32")
    s = Constant([n, k // group], dtype="float16") if "scales" in bound else Var("s", [n, k // group], "float16")
    x = Var("x", x_shape or [m, k], x_dtype)
    lead = list(x_shape[:-1]) if x_shape else [m]  # matmul broadcasts the leading extents of x over the 2-d weight
    params = [p for p in (wq, s, x) if isinstance(p, Var)]
    binds = []
    wd = Var("wd", [n, k], "float16")
    binds.append(VarBinding(wd, Call(Op("relax.call_tir"), [GlobalVar(decode), Tuple([wq, s])])))
    wt = Var("wt", [k, n], "float16")
    binds.append(VarBinding(wt, Call(Op("relax.permute_dims"), [wd], Attrs(axes=axes))))
    y32 = Var("y32", lead + [n], out_dtype or x_dtype)
    binds.append(VarBinding(y32, Call(Op("relax.matmul"), [x, wt], Attrs(out_dtype=DataType(out_dtype)))))
    cur = Var("y", lead + [n], astype_dtype)
    binds.append(VarBinding(cur, Call(Op("relax.astype"), [y32], Attrs(dtype=DataType(astype_dtype)))))
    for i, step in enumerate(tail):
        nxt = Var(f"t{i}", lead + [n], "float16")
        if step[0] == "silu_mul":
            # sp = split(y, 2, axis); out = multiply(nn.silu(sp[0]), sp[1]); step = ("silu_mul", sections, axis, swapped)
            sections = step[1] if len(step) > 1 else 2
            axis = step[2] if len(step) > 2 else -1
            swapped = len(step) > 3 and step[3]
            sp = Var("sp")
            # (relax.op.split stores a section count as an int64 IntImm and the axis as given,
            # python/tvm/relax/op/manipulate.py:238-240, src/relax/op/tensor/manipulate.cc:635-660)
            binds.append(VarBinding(sp, Call(Op("relax.split"), [cur],
                                             Attrs(indices_or_sections=IntImm("int64", sections), axis=int(axis)))))
            h0, h1 = Var("gate", lead + [n // 2], "float16"), Var("up", lead + [n // 2], "float16")
            binds.append(VarBinding(h0, TupleGetItem(sp, 1 if swapped else 0)))
            binds.append(VarBinding(h1, TupleGetItem(sp, 0 if swapped else 1)))
            act = Var("act", lead + [n // 2], "float16")
            binds.append(VarBinding(act, Call(Op("relax.nn.silu"), [h0])))
            nxt = Var(f"t{i}", lead + [n // 2], "float16")
            flipped = len(step) > 4 and step[4]  # multiply(up, silu(gate)): the same product
            binds.append(VarBinding(nxt, Call(Op("relax.multiply"), [h1, act] if flipped else [act, h1])))
            cur = nxt
            continue
        if step[0] == "add":
            operand = Constant(step[1], dtype="float16") if f"operand{i}" in bound else Var(f"operand{i}", step[1], "float16")
            if isinstance(operand, Var):
                params.append(operand)
            args = [cur, operand] if len(step) < 3 or not step[2] else [operand, cur]
            binds.append(VarBinding(nxt, Call(Op("relax.add"), args)))
        else:
            binds.append(VarBinding(nxt, Call(Op("relax.nn." + step[0]), [cur])))
        cur = nxt
    name = "mi355x.q4f16_matmul" if "q4" in decode else "mi355x.q8f16_matmul"
    # The shape of the reference's golden for FuseOpsByPattern(annotate_codegen=True)
    # (tests/python/relax/test_transform_fuse_ops_by_pattern.py:41-81): an outer function with the attributes
    # Codegen and global_symbol whose body binds a local function -- attributes Primitive = 1 and Composite,
    # its body one dataflow block -- to a variable, calls it with the outer parameters in the same order,
    # and returns the result of that call.
    composite = Function(params, SeqExpr([DataflowBlock(binds)], cur), {"Primitive": 1, "Composite": name})
    suffix = "1" if golden_names else "_outer"
    outer = [Var(p.name_hint + suffix, p.struct_info.shape, p.struct_info.dtype) for p in params]
    order = outer_order or list(range(len(outer)))
    outer_params = [outer[i] for i in order]
    local = Var("gv1" if golden_names else "local_func")
    gv = Var("gv11" if golden_names else "gv", list(cur.struct_info.shape), "float16")
    body = SeqExpr([BindingBlock([VarBinding(local, composite), VarBinding(gv, Call(local, outer))])], gv)
    return Function(outer_params, body, {"Codegen": "mi355x", "global_symbol": symbol})


def fused_name(decode, tail=()):
    """The name FuseOpsByPattern gives the grouped bindings: "fused", then "_" + the callee of every binding
    in order -- the PrimFunc's name for a call_tir, the operator's name otherwise
    (src/relax/transform/fuse_ops.cc:370-395, 477) -- with dots turned into underscores when the function is
    added to the module (include/tvm/relax/utils.h:49-50).  With annotate_codegen the outer function's symbol
    is that name + "_" + backend (src/relax/transform/fuse_ops.cc:1007-1010)."""
    parts = ["fused", decode, "relax.permute_dims", "relax.matmul", "relax.astype"]
    parts += ["relax.add" if step[0] == "add" else "relax.nn." + step[0] for step in tail]
    return "_".join(parts).replace(".", "_")


def partitioned_main(symbol, args, out_shape):
    """What RunCodegen leaves in `main` for one offloaded call: call_tir(ExternFunc(symbol), (args...),
    out_sinfo) with the call's own arguments in their order
    (tests/python/relax/test_transform_codegen_pass.py:230-251; src/relax/transform/run_codegen.cc:76-104)."""
    out = StructInfo(out_shape, "float16")
    return Call(Op("relax.call_tir"), [ExternFunc(symbol), Tuple(list(args))], sinfo_args=[out])
