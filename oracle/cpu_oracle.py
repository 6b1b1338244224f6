"""ctypes wrapper of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Only tests, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py`
may import this module; the shipped package never does.  It loads
`oracle/libcustos_cpu_oracle.so` (built from custos_cpu_oracle.c by
`make -C oracle`) and turns the closure a test passes (`lambda v: v.mul(2.0).add(1.0)`) into the
oracle's postfix program with a tracer of its own (`Traced`): nothing of the package under test is
imported here, so a mistake in the package's expression classes (a swapped operand, a wrong node) is
not shared by the oracle.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libcustos_cpu_oracle.so")

OPS = {
    "var0": 0, "var1": 1, "const": 2, "add": 3, "sub": 4, "mul": 5, "div": 6, "pow": 7,
    "min": 8, "max": 9, "geq": 10, "leq": 11, "eq_cpuref": 12, "eq": 13, "sin": 14, "cos": 15,
    "tan": 16, "tanh": 17, "exp": 18, "ln": 19, "abs": 20, "neg": 21, "identity": 22, "sqrt": 23,
    "var2": 24, "var3": 25,
}

# oracle_dtype values and numpy storage types
DTYPES = {
    "f32": (0, np.float32), "f64": (1, np.float64), "i32": (2, np.int32), "i64": (3, np.int64),
    "f16": (4, np.uint16), "f16_pernode": (5, np.uint16), "u8": (6, np.uint8), "i8": (7, np.int8),
    "i16": (8, np.int16), "u16": (9, np.uint16), "u32": (10, np.uint32), "u64": (11, np.uint64),
    "bf16": (12, np.uint16), "bf16_pernode": (13, np.uint16),
}


class Ins(C.Structure):
    _fields_ = [("op", C.c_int32), ("reserved", C.c_int32), ("cst", C.c_double)]


_lib = None


def build() -> None:
    subprocess.run(["make", "-C", HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        _lib = C.CDLL(LIB)
        _lib.oracle_f16_to_f32.restype = C.c_float
        _lib.oracle_f16_to_f32.argtypes = [C.c_uint16]
        _lib.oracle_f32_to_f16.restype = C.c_uint16
        _lib.oracle_f32_to_f16.argtypes = [C.c_float]
        _lib.oracle_bf16_to_f32.restype = C.c_float
        _lib.oracle_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.oracle_f32_to_bf16.restype = C.c_uint16
        _lib.oracle_f32_to_bf16.argtypes = [C.c_float]
    return _lib


class Traced:
    """A value inside a closure that is being traced: the postfix program that computes it, as a
    tuple of (node name, literal or None).  The methods are the reference's `Combiner` methods
    (src/two_way_ops/combiner.rs:8-116; `sqrt` is the added node): `lhs.op(rhs)` evaluates lhs, then
    rhs, then the node (src/two_way_ops/ops.rs:15-314), so its program is lhs's, rhs's, the node.
    `val` makes a literal (`2.0.to_val()`, src/two_way_ops/resolve.rs:61-79) where a closure needs one
    on the left: `v.val(1.0).sub(v.tanh())`."""

    __slots__ = ("prog",)

    def __init__(self, prog):
        self.prog = tuple(prog)

    @staticmethod
    def _operand(v):
        if isinstance(v, Traced):
            return v.prog
        if isinstance(v, (bool, int, float, str, np.integer, np.floating, np.bool_)):
            return (("const", v),)
        raise TypeError(f"the oracle cannot trace an operand of type {type(v).__name__}: closures take their literals as "
                        "numbers or through `v.val(number)`")

    def _two(self, name, rhs):
        return Traced(self.prog + Traced._operand(rhs) + ((name, None),))

    def _one(self, name):
        return Traced(self.prog + ((name, None),))

    def val(self, value):
        return Traced(Traced._operand(value))

    def add(self, rhs): return self._two("add", rhs)
    def sub(self, rhs): return self._two("sub", rhs)
    def mul(self, rhs): return self._two("mul", rhs)
    def div(self, rhs): return self._two("div", rhs)
    def pow(self, rhs): return self._two("pow", rhs)
    def min(self, rhs): return self._two("min", rhs)
    def max(self, rhs): return self._two("max", rhs)
    def geq(self, rhs): return self._two("geq", rhs)
    def leq(self, rhs): return self._two("leq", rhs)
    def eq(self, rhs): return self._two("eq", rhs)
    def sin(self): return self._one("sin")
    def cos(self): return self._one("cos")
    def tan(self): return self._one("tan")
    def tanh(self): return self._one("tanh")
    def exp(self): return self._one("exp")
    def ln(self): return self._one("ln")
    def abs(self): return self._one("abs")
    def neg(self): return self._one("neg")
    def identity(self): return self._one("identity")
    def sqrt(self): return self._one("sqrt")


def trace(f, n_vars=1):
    """The closure `f` applied to `n_vars` traced operands."""
    result = f(*[Traced((("var%d" % i, None),)) for i in range(n_vars)])
    if not isinstance(result, Traced):
        result = Traced(Traced._operand(result))
    return result


def compile_rpn(traced, dtype: str = "f32", eq_mode: str = "eq"):
    """Traced closure -> postfix program of the C oracle.

    `eq_mode="eq"` evaluates `eq` as a == b (what the reference's GPU sources
    compute and what the HIP kernels do); `"eq_cpuref"` as a <= b, the
    reference CPU `Eval` (src/two_way_ops/ops/cmps.rs:135).
    Scalars are converted to the element type here, exactly once.
    """
    def const_value(v):
        if isinstance(v, str):
            v = float(v) if dtype in ("f32", "f64", "f16", "bf16", "f16_pernode", "bf16_pernode") else int(float(v))
        if dtype in ("f32", "f16", "bf16", "f16_pernode", "bf16_pernode"):
            return float(np.float32(v))
        if dtype == "f64":
            return float(v)
        return float(int(v))

    arr = (Ins * len(traced.prog))()
    for i, (name, literal) in enumerate(traced.prog):
        if name == "eq":
            name = eq_mode
        arr[i].op = OPS[name]
        arr[i].cst = const_value(literal) if name == "const" else 0.0
    return arr


def _as_storage(a, dtype):
    return np.ascontiguousarray(a, dtype=DTYPES[dtype][1])


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


def _rc(rc, what):
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed with {rc}")


def apply_fn(f, *ins, dtype="f32", eq_mode="eq"):
    """out[i] = f(in0[i], ...) -- src/devices/cpu_stack_ops.rs:7-15."""
    arrs = [_as_storage(a, dtype) for a in ins]
    n = arrs[0].size
    prog = compile_rpn(trace(f, len(arrs)), dtype, eq_mode)
    out = np.zeros(n, dtype=DTYPES[dtype][1])
    ptrs = (C.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    _rc(lib().oracle_apply_fn(DTYPES[dtype][0], prog, len(prog), ptrs, len(arrs), _ptr(out), C.c_size_t(n)), "apply_fn")
    return out


def fused_apply_fn(ops, x, dtype="f32"):
    """Sequential per-element application -- src/devices/cpu/cpu_device.rs:204-232."""
    x = _as_storage(x, dtype)
    progs = [compile_rpn(trace(op), dtype) for op in ops]
    lens = (C.c_int * len(progs))(*[len(p) for p in progs])
    total = sum(len(p) for p in progs)
    flat = (Ins * max(total, 1))()
    k = 0
    for p in progs:
        for ins in p:
            flat[k].op, flat[k].cst = ins.op, ins.cst
            k += 1
    out = np.zeros(x.size, dtype=DTYPES[dtype][1])
    _rc(lib().oracle_fused_apply_fn(DTYPES[dtype][0], flat, lens, len(progs), _ptr(x), _ptr(out), C.c_size_t(x.size)), "fused_apply_fn")
    return out


def add_unary_grad(f, lhs, lhs_grad, out_grad, dtype="f32"):
    """Returns the updated lhs_grad -- src/devices/cpu_stack_ops.rs:18-30."""
    lhs = _as_storage(lhs, dtype)
    g = _as_storage(lhs_grad, dtype).copy()
    o = _as_storage(out_grad, dtype)
    prog = compile_rpn(trace(f), dtype)
    _rc(lib().oracle_add_unary_grad(DTYPES[dtype][0], prog, len(prog), _ptr(lhs), _ptr(g), _ptr(o), C.c_size_t(lhs.size)), "add_unary_grad")
    return g


def eval_scalar(f, *vals, dtype="f32", eq_mode="eq"):
    """`f(v.to_val()).eval()` for one set of scalar operands."""
    ctype, fn = {
        "f32": (C.c_float, "oracle_eval_f32"),
        "f64": (C.c_double, "oracle_eval_f64"),
        "i32": (C.c_int32, "oracle_eval_i32"),
    }[dtype]
    prog = compile_rpn(trace(f, max(len(vals), 1)), dtype, eq_mode)
    vars_ = (ctype * max(len(vals), 1))(*vals)
    res = ctype()
    _rc(getattr(lib(), fn)(prog, len(prog), vars_, len(vals), C.byref(res)), "eval")
    return res.value


def f32_to_f16_bits(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    l = lib()
    return np.array([l.oracle_f32_to_f16(float(v)) for v in a], dtype=np.uint16)


def f16_bits_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    l = lib()
    return np.array([l.oracle_f16_to_f32(int(v)) for v in a], dtype=np.float32)


# ---- monomorphic benchmark loops ----

def _call(name, *arrs_and_n):
    fn = getattr(lib(), name)
    fn.restype = None
    args = [(_ptr(a) if isinstance(a, np.ndarray) else C.c_size_t(a)) for a in arrs_and_n]
    fn(*args)


def c1_exp(x):
    out = np.empty_like(x)
    _call("oracle_c1_exp_f32", x, out, x.size)
    return out


def c2_chain_fused(x, out=None):
    out = np.empty_like(x) if out is None else out
    _call("oracle_c2_chain_fused_f32", x, out, x.size)
    return out


def c2_chain_unfused(x):
    ta, tb, out = np.empty_like(x), np.empty_like(x), np.empty_like(x)
    _call("oracle_c2_chain_unfused_f32", x, ta, tb, out, x.size)
    return out


def c3_tanh_fwd(x):
    y = np.empty_like(x)
    _call("oracle_c3_tanh_fwd_f32", x, y, x.size)
    return y


def c3_tanh_bwd(x, x_grad, y_grad):
    g = x_grad.copy()
    _call("oracle_c3_tanh_bwd_f32", x, g, y_grad, x.size)
    return g


def c4_chain_f16(x_bits):
    out = np.empty_like(x_bits)
    _call("oracle_c4_chain_f16", x_bits, out, x_bits.size)
    return out


def c5_graph(a, b, c):
    t, u, y = np.empty_like(a), np.empty_like(a), np.empty_like(a)
    _call("oracle_c5_graph_f32", a, b, c, t, u, y, a.size)
    return t, u, y
