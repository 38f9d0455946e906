"""A few dozen lines standing in for the `tvm.relax` classes that `spec_from_function` touches,
so that the role derivation can run without TVM.  Only structure is modelled: expressions,
bindings, functions with attributes, variables with a shape."""
import types


class Expr:
    def same_as(self, other):
        return self is other


class StructInfo:
    def __init__(self, shape):
        self.shape = list(shape)


class Var(Expr):
    def __init__(self, name, shape=None):
        self.name_hint = name
        self.struct_info = StructInfo(shape or [])

    def __hash__(self):
        return id(self)

    def __eq__(self, other):
        return self is other


class Constant(Expr):
    """A bound parameter: data plus shape; hashable by identity like the real node."""

    def __init__(self, shape, data=None):
        self.struct_info = StructInfo(shape)
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


class Call(Expr):
    def __init__(self, op, args):
        self.op = op
        self.args = list(args)


class VarBinding:
    def __init__(self, var, value):
        self.var, self.value = var, value


class BindingBlock:
    def __init__(self, bindings):
        self.bindings = list(bindings)


class SeqExpr(Expr):
    def __init__(self, blocks, body):
        self.blocks, self.body = list(blocks), body


class Function(Expr):
    def __init__(self, params, body, attrs=None):
        self.params, self.body, self.attrs = list(params), body, dict(attrs or {})


def as_module():
    """A module object usable as `tvm` with a `relax` attribute."""
    relax = types.ModuleType("tvm.relax")
    for cls in (Var, Call, Function, Tuple, GlobalVar, SeqExpr, BindingBlock, VarBinding, Constant):
        setattr(relax, cls.__name__, cls)
    tvm = types.ModuleType("tvm")
    tvm.relax = relax
    return tvm, relax


def quantized_linear(decode="decode_q4f16", m=4, n=48, k=128, tail=(), outer_order=None, bound=()):
    """The annotated function FuseOpsByPattern(annotate_codegen=True) produces for
    decode -> permute_dims -> matmul -> astype followed by `tail`, a sequence of
    ("add", shape) / ("relu",) steps.  Composite parameters are ordered by first use:
    (wq, scales, x, <tail operands in order>).  `outer_order` permutes the outer parameters.
    `bound` names operands ("wq", "scales", "operand<i>") that BindParams turned into constants: they sit
    inside the composite as Constant nodes and are no parameters."""
    per = 8 if "q4" in decode else 4
    group = 32 if "q4" in decode else 128
    wq = Constant([n, k // per]) if "wq" in bound else Var("wq", [n, k // per])
    s = Constant([n, k // group]) if "scales" in bound else Var("s", [n, k // group])
    x = Var("x", [m, k])
    params = [p for p in (wq, s, x) if isinstance(p, Var)]
    binds = []
    wd = Var("wd", [n, k])
    binds.append(VarBinding(wd, Call(Op("relax.call_tir"), [GlobalVar(decode), Tuple([wq, s])])))
    wt = Var("wt", [k, n])
    binds.append(VarBinding(wt, Call(Op("relax.permute_dims"), [wd])))
    y32 = Var("y32", [m, n])
    binds.append(VarBinding(y32, Call(Op("relax.matmul"), [x, wt])))
    cur = Var("y", [m, n])
    binds.append(VarBinding(cur, Call(Op("relax.astype"), [y32])))
    for i, step in enumerate(tail):
        nxt = Var(f"t{i}", [m, n])
        if step[0] == "add":
            operand = Constant(step[1]) if f"operand{i}" in bound else Var(f"operand{i}", step[1])
            if isinstance(operand, Var):
                params.append(operand)
            args = [cur, operand] if len(step) < 3 or not step[2] else [operand, cur]
            binds.append(VarBinding(nxt, Call(Op("relax.add"), args)))
        else:
            binds.append(VarBinding(nxt, Call(Op("relax.nn.relu"), [cur])))
        cur = nxt
    name = "mi355x.q4f16_matmul" if "q4" in decode else "mi355x.q8f16_matmul"
    composite = Function(params, SeqExpr([BindingBlock(binds)], cur), {"Composite": name})
    outer = [Var(p.name_hint + "_outer", p.struct_info.shape) for p in params]
    order = outer_order or list(range(len(outer)))
    outer_params = [outer[i] for i in order]
    local = Var("local_func")
    gv = Var("gv", [m, n])
    body = SeqExpr([BindingBlock([VarBinding(local, composite), VarBinding(gv, Call(local, outer))])], gv)
    return Function(outer_params, body, {"Codegen": "mi355x", "global_symbol": "fused_mi355x"})
