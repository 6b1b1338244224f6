"""Mirror of custos' expression DSL (`Combiner` / `Resolve` / `ToCLSource`).

Reference: src/two_way_ops/combiner.rs:8-116 (builder methods),
src/two_way_ops/resolve.rs:25-141 (leaf), src/two_way_ops/ops.rs,
ops/unary.rs, ops/cmps.rs (the text every node prints) and
src/two_way_ops/to_cl_source.rs:7-11 (scalars print with `{:?}`).

A closure `lambda x: x.sin().mul(2.0).add(1.0)` called with a `Resolve`
builds a tree whose `to_cl_source()` is the string the reference would hand to
its GPU backends; that string is what the C ABI compiles.
"""
from __future__ import annotations

import numpy as np

_BINARY_INFIX = {"add": "+", "sub": "-", "mul": "*", "div": "/", "geq": ">=", "leq": "<=", "eq": "=="}
_BINARY_CALL = {"pow": "pow", "min": "min", "max": "max"}
_UNARY_CALL = {
    "sin": "sin", "cos": "cos", "tan": "tan", "tanh": "tanh", "exp": "exp",
    "ln": "log", "abs": "abs", "sqrt": "sqrt",
}


def _wrap(v):
    return v if isinstance(v, Expr) else Const(v)


class Expr:
    """One node of an expression tree (`Combiner`)."""

    op = ""
    args: tuple = ()

    # -- binary --
    def add(self, rhs): return Node("add", self, _wrap(rhs))
    def sub(self, rhs): return Node("sub", self, _wrap(rhs))
    def mul(self, rhs): return Node("mul", self, _wrap(rhs))
    def div(self, rhs): return Node("div", self, _wrap(rhs))
    def pow(self, rhs): return Node("pow", self, _wrap(rhs))
    def min(self, rhs): return Node("min", self, _wrap(rhs))
    def max(self, rhs): return Node("max", self, _wrap(rhs))
    def geq(self, rhs): return Node("geq", self, _wrap(rhs))
    def leq(self, rhs): return Node("leq", self, _wrap(rhs))
    def eq(self, rhs): return Node("eq", self, _wrap(rhs))

    def val(self, value):
        """The literal `value` as a node (`value.to_val()`, src/two_way_ops/resolve.rs:61-79), for a closure
        that needs one on the left: `v.val(1.0).sub(v.tanh())`."""
        return Const(value)

    # -- unary --
    def sin(self): return Node("sin", self)
    def cos(self): return Node("cos", self)
    def tan(self): return Node("tan", self)
    def tanh(self): return Node("tanh", self)
    def exp(self): return Node("exp", self)
    def ln(self): return Node("ln", self)
    def abs(self): return Node("abs", self)
    def neg(self): return Node("neg", self)
    def identity(self): return Node("identity", self)
    # not a reference Combiner method; `Float::sqrt` exists (src/number.rs:320-322)
    def sqrt(self): return Node("sqrt", self)

    def to_cl_source(self, dtype: str = "f32") -> str:
        raise NotImplementedError


class Node(Expr):
    def __init__(self, op, *args):
        self.op = op
        self.args = args

    def to_cl_source(self, dtype: str = "f32") -> str:
        a = [x.to_cl_source(dtype) for x in self.args]
        if self.op in _BINARY_INFIX:
            return f"({a[0]} {_BINARY_INFIX[self.op]} {a[1]})"
        if self.op in _BINARY_CALL:
            return f"{_BINARY_CALL[self.op]}({a[0]}, {a[1]})"
        if self.op in _UNARY_CALL:
            return f"{_UNARY_CALL[self.op]}({a[0]})"
        if self.op == "neg":
            return f"-({a[0]})"
        if self.op == "identity":
            return a[0]
        raise ValueError(self.op)


class Const(Expr):
    """A scalar operand.  Printed like Rust's `{:?}` for the element type."""

    op = "const"

    def __init__(self, value):
        self.value = value

    def to_cl_source(self, dtype: str = "f32") -> str:
        v = self.value
        if isinstance(v, str):
            return v
        if isinstance(v, (bool, np.bool_)):
            return "true" if v else "false"
        if isinstance(v, (int, np.integer)):
            return str(int(v))
        return format_float(float(v), dtype)


def format_float(v: float, dtype: str = "f32") -> str:
    """Shortest text that round-trips in the element type, with Rust's spelling
    of whole numbers ("2.0"), infinities ("inf") and NaN ("NaN")."""
    if np.isnan(v):
        return "NaN"
    if np.isinf(v):
        return "inf" if v > 0 else "-inf"
    if dtype == "f64":
        s = repr(float(v))
    else:
        # f16 / bf16 expressions are computed in f32
        s = np.format_float_positional(np.float32(v), unique=True, trim="0")
        if len(s) > 24:
            s = np.format_float_scientific(np.float32(v), unique=True, trim="0")
    if s.endswith("."):
        s += "0"
    if "." not in s and "e" not in s and "n" not in s:
        s += ".0"
    return s


class Resolve(Expr):
    """Leaf: a marker name for source generation (src/two_way_ops/resolve.rs:25-30)."""

    op = "var"

    def __init__(self, marker: str = "x", index: int = 0):
        self.marker = marker
        self.index = index

    @staticmethod
    def with_marker(marker: str, index: int = 0) -> "Resolve":
        return Resolve(marker, index)

    def to_cl_source(self, dtype: str = "f32") -> str:
        return self.marker


def to_marker(*names: str):
    """`"x".to_marker()` / `("x", "y").to_marker()` (src/two_way_ops/resolve.rs:33-61)."""
    rs = tuple(Resolve(n, i) for i, n in enumerate(names))
    return rs[0] if len(rs) == 1 else rs


def to_val(v) -> Const:
    """`2f64.to_val()`: a scalar used as a whole expression."""
    return Const(v)


def fused_source(ops, dtype: str = "f32", marker: str = "x") -> str:
    """`operations_to_fused_src` (src/devices/fusing.rs:4-19): one
    "x = <expr>;\\n" line per unary op."""
    return "".join(f"{marker} = {_wrap(op(Resolve(marker))).to_cl_source(dtype)};\n" for op in ops)
