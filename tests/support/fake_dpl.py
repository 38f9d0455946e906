"""A stand-in for `tvm.relax.dpl` and the pieces of `tvm.tir` / `tvm.ir` the pattern table touches, with a
matcher that follows the reference's rules (src/relax/ir/dataflow_matcher.cc), so that the table can be
executed against the stand-in IR of `fake_relax` without TVM:

  * a variable stands for the value bound to it (TryGetValOfVar, :51-67);
  * a call pattern matches the callee, then the arguments in order, and for `relax.add` / `relax.multiply`
    also in reverse (:216-262);
  * an attribute pattern on a call compares every listed attribute the way MatchRetValue does (:108-150):
    what the attribute's C++ field is decides the rule -- an `int` field compares by value with an IntImm of
    any dtype, a `DataType` field with a string, an object-valued field (an IntImm, an Array) by
    StructuralEqual, *dtype included*;
  * the pattern side's dictionary goes through `make_node("DictAttrs", ...)`
    (python/tvm/relax/dpl/pattern.py:109-123): a Python int becomes an int32 IntImm, a str a String;
  * a data-type pattern compares the tensor's dtype (:457-464); a tuple-get-item pattern the index (unless it
    is -1) and the tuple (:355-362); a tuple pattern field by field (:364-381); a global-variable pattern the
    name (:487-492).

`partition()` restates how FuseOpsByPattern applies a table (src/relax/transform/fuse_ops.cc:1050-1066,
904-955): one pattern after the other over the whole function, every call a candidate root; what a pattern
has grouped is a composite function afterwards, which no later pattern looks into.
"""
import types

from . import fake_relax as R


# ---- the value types of attributes (defined beside the stand-in IR that carries them) ------------------
IntImm, DataType = R.IntImm, R.DataType


def structural_equal(a, b):
    if isinstance(a, IntImm) or isinstance(b, IntImm):
        return isinstance(a, IntImm) and isinstance(b, IntImm) and a.dtype == b.dtype and a.value == b.value
    if isinstance(a, (list, tuple)) or isinstance(b, (list, tuple)):
        return isinstance(a, (list, tuple)) and isinstance(b, (list, tuple)) and len(a) == len(b) and \
            all(structural_equal(x, y) for x, y in zip(a, b))
    return type(a) is type(b) and a == b


def _to_dict_attr(v):
    """make_node("DictAttrs", key=v): how a Python value arrives on the pattern side."""
    if isinstance(v, bool):
        return IntImm("bool", int(v))
    if isinstance(v, int):
        return IntImm("int32", v)
    return v


def match_ret_value(lhs, rhs):
    """MatchRetValue(lhs = the pattern's value, rhs = the attribute as reflection returns it)."""
    if isinstance(rhs, bool) or (isinstance(rhs, int) and not isinstance(rhs, IntImm)):  # kDLInt: an `int` / `bool` field
        return isinstance(lhs, IntImm) and lhs.value == int(rhs)
    if isinstance(rhs, DataType):                                                        # kTVMDataType
        assert isinstance(lhs, str), "PatternMatcher: Unsupported TVMDataType"
        return str(lhs) == str(rhs)
    if isinstance(rhs, str):                                                             # kTVMStr / String object
        return isinstance(lhs, str) and lhs == rhs
    return structural_equal(lhs, rhs)                                                    # kTVMObjectHandle


# ---- patterns --------------------------------------------------------------------------------------------
class DFPattern:
    def __call__(self, *args, varg_default_wildcard=False):
        return CallPattern(self, list(args), varg_default_wildcard)

    def __or__(self, other):
        return OrPattern(self, other)

    def has_attr(self, attrs):
        return AttrPattern(self, {k: _to_dict_attr(v) for k, v in attrs.items()})

    def has_dtype(self, dtype):
        return DataTypePattern(self, dtype)


class WildcardPattern(DFPattern):
    pass


class ExprPattern(DFPattern):
    def __init__(self, expr):
        self.expr = expr


class GlobalVarPattern(DFPattern):
    def __init__(self, name_hint=""):
        self.name_hint = name_hint


class CallPattern(DFPattern):
    def __init__(self, op, args, varg_default_wildcard=False):
        self.op, self.args, self.varg_default_wildcard = op, args, varg_default_wildcard


class TuplePattern(DFPattern):
    def __init__(self, fields):
        self.fields = list(fields)


class TupleGetItemPattern(DFPattern):
    def __init__(self, tuple_value, index=None):
        self.tuple, self.index = tuple_value, (-1 if index is None else index)


class AttrPattern(DFPattern):
    def __init__(self, pattern, attrs):
        self.pattern, self.attrs = pattern, attrs


class DataTypePattern(DFPattern):
    def __init__(self, pattern, dtype):
        self.pattern, self.dtype = pattern, dtype


class OrPattern(DFPattern):
    def __init__(self, left, right):
        self.left, self.right = left, right


def wildcard():
    return WildcardPattern()


def is_op(op_name):
    return ExprPattern(R.Op(op_name))


def is_tuple_get_item(tuple_value, index=None):
    return TupleGetItemPattern(tuple_value, index)


def is_call_tir(func_name, args=None):
    args = wildcard() if args is None else TuplePattern(args) if isinstance(args, (list, tuple)) else args
    return is_op("relax.call_tir")(GlobalVarPattern(func_name), args)


# ---- the matcher -----------------------------------------------------------------------------------------
class Matcher:
    def __init__(self, var2val):
        self.var2val, self.memo = var2val, {}

    def value_of(self, expr):
        if isinstance(expr, R.Var) and expr in self.var2val:
            return self.var2val[expr]
        return expr

    def visit(self, pat, expr0):
        expr = self.value_of(expr0)
        if id(pat) in self.memo:  # a pattern object matches one expression only
            return expr is self.memo[id(pat)]
        saved = dict(self.memo)
        ok = getattr(self, "visit_" + type(pat).__name__)(pat, expr)
        if ok:
            self.memo[id(pat)] = expr
        else:
            self.memo = saved
        return ok

    def visit_WildcardPattern(self, pat, expr):
        return True

    def visit_ExprPattern(self, pat, expr):
        return isinstance(expr, R.Op) and isinstance(pat.expr, R.Op) and expr.name == pat.expr.name

    def visit_GlobalVarPattern(self, pat, expr):
        return isinstance(expr, R.GlobalVar) and pat.name_hint in ("", expr.name_hint)

    def visit_OrPattern(self, pat, expr):
        return self.visit(pat.left, expr) or self.visit(pat.right, expr)

    def visit_TuplePattern(self, pat, expr):
        return isinstance(expr, R.Tuple) and len(pat.fields) == len(expr.fields) and \
            all(self.visit(p, f) for p, f in zip(pat.fields, expr.fields))

    def visit_TupleGetItemPattern(self, pat, expr):
        return isinstance(expr, R.TupleGetItem) and pat.index in (-1, expr.index) and self.visit(pat.tuple, expr.tuple_value)

    def visit_DataTypePattern(self, pat, expr):
        # (no jump to the bound value is needed: a variable has the dtype of its value)
        dtype = getattr(getattr(expr, "struct_info", None), "dtype", None)
        return dtype is not None and str(dtype) == str(pat.dtype) and self.visit(pat.pattern, expr)

    def visit_AttrPattern(self, pat, expr):
        if not self.visit(pat.pattern, expr) or not isinstance(expr, R.Call):
            return False
        fields = {} if expr.attrs is None else vars(expr.attrs)
        return all(name in fields and match_ret_value(want, fields[name]) for name, want in pat.attrs.items())

    def visit_CallPattern(self, pat, expr):
        if not isinstance(expr, R.Call) or not self.visit(pat.op, expr.op):
            return False
        if (pat.varg_default_wildcard and len(expr.args) < len(pat.args)) or \
                (not pat.varg_default_wildcard and len(expr.args) != len(pat.args)):
            return False
        saved = dict(self.memo)
        if all(self.visit(p, a) for p, a in zip(pat.args, expr.args)):
            return True
        self.memo = dict(saved)
        commutative = isinstance(pat.op, ExprPattern) and pat.op.expr.name in ("relax.add", "relax.multiply")
        if commutative and all(self.visit(p, a) for p, a in zip(pat.args, reversed(expr.args))):
            return True
        self.memo = saved
        return False


def match(pattern, expr, var2val):
    """The matched expressions by pattern object, or None (ExtractMatchedExpr)."""
    m = Matcher(var2val)
    return dict(m.memo) if m.visit(pattern, expr) else None


def partition(func_body_bindings, table):
    """Applies `table` ([(name, pattern)], in order) to a list of VarBindings the way FuseOpsByPattern does.
    Returns [(name, [names of the variables whose bindings the entry grouped, in program order])]."""
    live = list(func_body_bindings)
    groups = []
    for name, pattern in table:
        var2val = {b.var: b.value for b in live}
        value_to_var = {id(b.value): b.var for b in live}
        for b in list(live):
            if b not in live or not isinstance(b.value, R.Call):
                continue
            found = match(pattern, b.value, var2val)
            if found is None:
                continue
            grouped = {id(b.value)} | {id(e) for e in found.values() if isinstance(e, R.Call)}
            members = [q for q in live if id(q.value) in grouped]
            # a tuple-get-item between two grouped calls travels with them (its value is no call, so no
            # pattern lists it: MakeGroupedFunctions keeps bindings whose variable is grouped with its users)
            member_vars = {q.var for q in members}
            for q in live:
                if isinstance(q.value, R.TupleGetItem) and q.value.tuple_value in member_vars:
                    members.append(q)
            members = [q for q in live if q in members]
            groups.append((name, [q.var.name_hint for q in members]))
            live = [q for q in live if q not in members]
            var2val = {q.var: q.value for q in live}
    return groups


def install(monkeypatch, sys_modules):
    """Puts `tvm`, `tvm.relax`, `tvm.relax.dpl` and `tvm.tir` stand-ins into sys.modules."""
    tvm, relax = R.as_module()
    dpl = types.ModuleType("tvm.relax.dpl")
    for f in (wildcard, is_op, is_tuple_get_item, is_call_tir):
        setattr(dpl, f.__name__, f)
    tir = types.ModuleType("tvm.tir")
    tir.IntImm = IntImm
    relax.dpl, tvm.tir = dpl, tir
    for name, mod in (("tvm", tvm), ("tvm.relax", relax), ("tvm.relax.dpl", dpl), ("tvm.tir", tir)):
        monkeypatch.setitem(sys_modules, name, mod)
    return tvm
