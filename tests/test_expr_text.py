"""Expression text: the Python `Combiner` mirror must print the strings the
reference asserts for `to_cl_source`, and the library's parser must accept
them, re-print them unchanged and emit typed HIP C for them.  CPU only."""
import re

import numpy as np

import pytest

from custos_amd import Resolve, capi, to_marker, to_val
from custos_amd.expr import format_float, fused_source


def test_reference_strings():
    x = Resolve("x")
    assert x.exp().to_cl_source() == "exp(x)"                                              # mod.rs:73
    assert Resolve("val").tan().neg().to_cl_source() == "-(tan(val))"                      # mod.rs:90
    xx, yy = to_marker("x", "y")
    assert xx.mul(3.).pow(yy.add(1.)).to_cl_source() == "pow((x * 3.0), (y + 1.0))"        # mod.rs:103
    vx, other = to_marker("var_x", "other")
    assert vx.eq(other).to_cl_source("i32") == "(var_x == other)"                          # mod.rs:116
    assert vx.geq(0).mul(vx).to_cl_source("i32") == "((var_x >= 0) * var_x)"               # mod.rs:130
    assert vx.add(3).to_cl_source("i32") == "(var_x + 3)"                                  # mod.rs:144
    assert vx.geq(4).to_cl_source("i32") == "(var_x >= 4)"                                 # mod.rs:158
    assert xx.add(yy).to_cl_source() == "(x + y)"                                          # mod.rs:176
    assert xx.add(yy).mul(3.6).sub(yy).to_cl_source() == "(((x + y) * 3.6) - y)"           # mod.rs:192
    assert x.add(2.).mul(x).add(x.mul(8.)).mul(5.).to_cl_source() == "((((x + 2.0) * x) + (x * 8.0)) * 5.0)"  # mod.rs:201
    assert x.mul(x).add(2.).to_cl_source() == "((x * x) + 2.0)"                            # resolve.rs:22
    assert x.add(x).mul(2.).to_cl_source() == "((x + x) * 2.0)"                            # resolve.rs:117
    assert to_marker("x").to_cl_source() == "x"                                            # resolve.rs:40
    assert x.sin().to_cl_source() == "sin(x)" and x.cos().to_cl_source() == "cos(x)"       # op_hint.rs:63,71
    assert x.ln().to_cl_source() == "log(x)"                                               # op_hint.rs:79
    assert x.identity().to_cl_source() == "x"                                              # ops/unary.rs:19-24
    assert x.max(3.).min(5.).to_cl_source() == "min(max(x, 3.0), 5.0)"
    assert x.add("1.0").to_cl_source() == "(x + 1.0)"                                      # cuda/ops.rs:254
    assert to_val(2.0).to_cl_source("f64") == "2.0"


def test_operand_order_of_every_binary_node(oracle):
    """`lhs.op(rhs)` prints the receiver first, as every `ToCLSource` of the reference does
    (src/two_way_ops/ops.rs:28-310: "({} * {})", "({} + {})", "({} - {})", "({} / {})", "pow({}, {})",
    "min({}, {})", "max({}, {})"; ops/cmps.rs:17-130: "({} >= {})", "({} <= {})", "({} == {})"), and the
    oracle's postfix program takes its operands in that order too: the receiver is the left operand
    of the scalar evaluation (asymmetric inputs tell the two orders apart)."""
    a, b = to_marker("a", "b")
    formats = {"mul": "(a * b)", "add": "(a + b)", "sub": "(a - b)", "div": "(a / b)", "pow": "pow(a, b)", "min": "min(a, b)",
               "max": "max(a, b)", "geq": "(a >= b)", "leq": "(a <= b)", "eq": "(a == b)"}
    for op, text in formats.items():
        assert getattr(a, op)(b).to_cl_source() == text, op
        assert capi.expr_canonical(text, ["a", "b"]) == text
    scalar = {"sub": 7.0 - 2.0, "div": 7.0 / 2.0, "pow": 49.0, "geq": 1.0, "leq": 0.0, "min": 2.0, "max": 7.0}
    for op, want in scalar.items():
        assert oracle.eval_scalar(lambda x, y, op=op: getattr(x, op)(y), 7.0, 2.0) == want, op


def test_fused_source():
    # src/devices/fusing.rs:104-120
    ops = [lambda x: x.sin(), lambda x: x.neg(), lambda x: x.cos()]
    assert fused_source(ops) == "x = sin(x);\nx = -(x);\nx = cos(x);\n"


def test_float_formatting():
    assert format_float(2.0) == "2.0" and format_float(3.6) == "3.6" and format_float(-0.5) == "-0.5"
    assert format_float(float("inf")) == "inf" and format_float(float("-inf")) == "-inf"
    assert format_float(float("nan")) == "NaN"
    assert format_float(0.1, "f64") == "0.1"
    assert float(format_float(1e-7)) == pytest.approx(1e-7)


REFERENCE_TEXTS = [
    ("exp(x)", ["x"]),
    ("-(tan(val))", ["val"]),
    ("pow((x * 3.0), (y + 1.0))", ["x", "y"]),
    ("(var_x == other)", ["var_x", "other"]),
    ("((var_x >= 0) * var_x)", ["var_x"]),
    ("(var_x + 3)", ["var_x"]),
    ("(x + y)", ["x", "y"]),
    ("(((x + y) * 3.6) - y)", ["x", "y"]),
    ("((((x + 2.0) * x) + (x * 8.0)) * 5.0)", ["x"]),
    ("min(max(x, 3.0), 5.0)", ["x"]),
    ("(x[idx] + 1.0)", ["x[idx]"]),                   # marker used by cuda/ops.rs:165
    ("(lhs[idx] * -2.5e-3)", ["lhs[idx]"]),
    ("sqrt(abs(x))", ["x"]),
    ("((x <= inf) * -inf)", ["x"]),
    ("2.0", ["x"]),
    ("x", ["x"]),
]


@pytest.mark.parametrize("text,markers", REFERENCE_TEXTS)
def test_parser_round_trip(text, markers):
    assert capi.expr_canonical(text, markers) == text


def test_fused_statement_list_nests():
    got = capi.expr_canonical("x = sin(x);\nx = -(x);\nx = cos(x);\n", ["x"])
    assert got == "cos(-(sin(x)))"


@pytest.mark.parametrize("bad,code", [
    ("(x +)", capi.ERR_EXPR_SYNTAX),
    ("sin(x", capi.ERR_EXPR_SYNTAX),
    ("foo(x)", capi.ERR_EXPR_SYNTAX),
    ("(x + y)", capi.ERR_EXPR_UNKNOWN_MARKER),
    ("", capi.ERR_EXPR_SYNTAX),
    ("x x", capi.ERR_EXPR_SYNTAX),
    ("y = sin(x);", capi.ERR_EXPR_UNKNOWN_MARKER),
])
def test_parser_errors(bad, code):
    with pytest.raises(capi.CustosHipError) as e:
        capi.expr_canonical(bad, ["x"])
    assert e.value.code == code
    assert e.value.message  # a message is always set


def test_emit_types_literals_and_no_contraction():
    src, _ = capi.expr_emit(capi.KIND_APPLY, "f32", "((x * 2.0) + 1.0)", ["x"])
    assert "0x1p+1f" in src and "0x1p+0f" in src          # f32-typed literals, never a double 2.0
    assert not re.search(r"[^x0-9a-f.p+]2\.0[^f]", src.split("\n", 1)[1])
    assert "fma" not in src.lower()
    assert "const float t2 = (float)(t0 * t1);" in src     # one statement per node
    assert "CustosConsts" not in src
    src64, _ = capi.expr_emit(capi.KIND_APPLY, "f64", "((x * 2.0) + 1.0)", ["x"])
    assert "typedef double S;" in src64 and "0x1p+1;" in src64
    srci, _ = capi.expr_emit(capi.KIND_APPLY, "i32", "((x >= 0) * x)", ["x"])
    assert "typedef int S;" in srci and "(unsigned int)" in srci
    srch, _ = capi.expr_emit(capi.KIND_APPLY, "f16", "(exp((x * 0.5)) * x)", ["x"])
    assert "typedef _Float16 S;" in srch and "typedef float C;" in srch
    assert "ext_vector_type(8)" in srch                     # 16-byte vectors of halves


def test_shared_form_takes_literals_as_launch_parameters():
    """The form compiled once an expression has been seen with a second set of literal values."""
    src, _ = capi.expr_emit(capi.KIND_APPLY, "f32", "((x * 2.0) + 1.0)", ["x"], shared=True)
    assert "struct CustosConsts { C c[2]; };" in src and "const float t1 = kc.c[0];" in src
    assert "0x1p+1f" not in src
    assert src.startswith("// generated by custos-hip: ((x * c0) + c1)\n")
    assert "CUSTOS_KC_ENTRY const u64 mode)" in src         # the block is an argument by value of every entry point
    consts = capi.expr_constants("f32", "((x * 2.0) + 1.0)", ["x"])
    assert consts.dtype == np.float32 and consts.tolist() == [2.0, 1.0]
    src64, _ = capi.expr_emit(capi.KIND_APPLY, "f64", "((x * 2.0) + 1.0)", ["x"], shared=True)
    assert "const double t1 = kc.c[0];" in src64
    assert capi.expr_constants("f64", "((x * 0.1) + 1.0)", ["x"]).tolist() == [0.1, 1.0]
    assert capi.expr_constants("f16", "(exp((x * 0.5)) * x)", ["x"]).dtype == np.float32   # the compute type
    assert capi.expr_constants("i8", "(x + -3)", ["x"]).tolist() == [-3]
    nan_inf = capi.expr_constants("f32", "min(max(x, -inf), NaN)", ["x"])
    assert nan_inf[0] == -np.inf and np.isnan(nan_inf[1])
    # no literal: no parameter block, and the shared form is the only form
    plain, h = capi.expr_emit(capi.KIND_APPLY, "f32", "sin(x)", ["x"], shared=True)
    assert "CustosConsts" not in plain and len(capi.expr_constants("f32", "sin(x)", ["x"])) == 0
    assert (plain, h) == capi.expr_emit(capi.KIND_APPLY, "f32", "sin(x)", ["x"])
    # the divisor of an integer division stays in the code: the compiler turns it into a multiplication
    src, h3 = capi.expr_emit(capi.KIND_APPLY, "i32", "((x / 3) + 2)", ["x"], shared=True)
    assert "((int)3LL)" in src and "struct CustosConsts { C c[1]; };" in src
    assert capi.expr_constants("i32", "((x / 3) + 2)", ["x"]).tolist() == [2]
    assert capi.expr_emit(capi.KIND_APPLY, "i32", "((x / 4) + 2)", ["x"], shared=True)[1] != h3
    assert capi.expr_emit(capi.KIND_APPLY, "i32", "((x / 3) + 7)", ["x"], shared=True)[1] == h3
    # a float division by a literal is a parameter like any other
    assert "kc.c[0]" in capi.expr_emit(capi.KIND_APPLY, "f32", "(x / 3.0)", ["x"], shared=True)[0]
    # more than 32 literals: all of them stay
    many = "x"
    for i in range(33):
        many = f"({many} + {i + 1}.0)"
    src, _ = capi.expr_emit(capi.KIND_APPLY, "f32", many, ["x"], shared=True)
    assert "CustosConsts" not in src and "0x1p+1f" in src
    assert len(capi.expr_constants("f32", many, ["x"])) == 0
    # every element type compiles in the shared form
    for dtype in capi.DTYPES:
        text = "((x * 3) + 1)" if dtype[0] in "iu" else "(exp((x * 0.5)) + 1.5)"
        for kind in (capi.KIND_APPLY, capi.KIND_UNARY_GRAD):
            assert "kc.c[1]" in capi.expr_emit(kind, dtype, text, ["x"], shared=True)[0]


def test_expressions_that_ended_the_compiler_do_compile():
    """With the packed f32 instructions off, the backend could not select a two-element f32
    negation that the SLP vectorizer formed in front of a packed f32 -> f16 conversion; the
    compiler's fatal error ends the process, so these would not even fail."""
    for dtype, text, markers in (("f16_pernode", "-(((min(a, c) <= -1.0535643) / a))", ["a", "b", "c"]),
                                 ("f16_pernode", "(a + ((min(b, a) * (a <= a)) + -3.632779))", ["a", "b"]),
                                 ("f16", "-((a / b))", ["a", "b"]),
                                 ("f16_pernode", "-((a - max(b, 1.9355469)))", ["a", "b"])):
        for kind in (capi.KIND_APPLY,) + ((capi.KIND_UNARY_GRAD,) if len(markers) == 1 else ()):
            assert capi.expr_build_code_object(kind, dtype, text, markers) > 0


def test_min_max_emitted_as_selects():
    src, _ = capi.expr_emit(capi.KIND_APPLY, "f32", "min(max(x, 0.0), 6.0)", ["x"])
    assert "fmax" not in src and "fmin" not in src
    assert "(t0 > t1) ? t0 : t1" in src


def test_hash_ignores_literal_spelling_but_not_value_or_type():
    h = lambda text, dt="f32", kind=capi.KIND_APPLY: capi.expr_emit(kind, dt, text, ["x"])[1]
    assert h("(x * 2.0)") == h("(x * 2)") == h("(x * 2.00)") == h("(x*2.0)")
    assert h("(x * 2.0)") != h("(x * 2.5)")
    assert h("(x * 2.0)") != h("(x * 2.0)", "f64")
    assert h("(x * 2.0)") != h("(x * 2.0)", "f32", capi.KIND_UNARY_GRAD)
    assert h("(x * 2.0)") != h("(2.0 * x)")
    # f32 rounding of the literal decides, not the text
    assert h("(x * 0.1)") == h("(x * 0.100000001)")
    assert h("(x * 0.1)", "f64") != h("(x * 0.100000001)", "f64")


def test_shared_hash_ignores_literal_values_but_not_structure_or_type():
    h = lambda text, dt="f32", kind=capi.KIND_APPLY: capi.expr_emit(kind, dt, text, ["x"], shared=True)[1]
    c = lambda text, dt="f32": capi.expr_constants(dt, text, ["x"]).tolist()
    assert h("(x * 2.0)") == h("(x * 2)") == h("(x * 2.5)") == h("(x * -1e9)")
    assert c("(x * 2.0)") == c("(x * 2)") == c("(x * 2.00)") == [2.0] and c("(x * 2.5)") == [2.5]
    assert h("(x * 2.0)") != capi.expr_emit(capi.KIND_APPLY, "f32", "(x * 2.0)", ["x"])[1]
    assert h("(x * 2.0)") != h("(x * 2.0)", "f64")
    assert h("(x * 2.0)") != h("(x * 2.0)", "f32", capi.KIND_UNARY_GRAD)
    assert h("(x * 2.0)") != h("(2.0 * x)")
    assert h("(x * 2.0)") != h("(x + 2.0)")
    assert c("(x * 0.1)") == c("(x * 0.100000001)")
    assert c("(x * 0.1)", "f64") != c("(x * 0.100000001)", "f64")


def test_tuning_is_part_of_the_key_and_source():
    t = capi.Tuning(256, 4, 0, -1)
    src, h1 = capi.expr_emit(capi.KIND_APPLY, "f32", "x", ["x"], t)
    assert "#define CUSTOS_BLOCK 256" in src and "custos_tile4(" in src and "custos_tile2(" not in src
    # launch shape left open: the kernel holds the tile functions for two vectors per thread and for one,
    # and every launch names its vectors per thread and its workgroup size in its mode word
    src2, h2 = capi.expr_emit(capi.KIND_APPLY, "f32", "x", ["x"])
    assert "#define CUSTOS_BLOCK 128" in src2 and "custos_tile2(" in src2 and "custos_tile1(" in src2
    assert "const u64 U = (mode >> 8) & 15;" in src2 and "#define CUSTOS_BT (64u << ((mode >> 13) & 3))" in src2
    assert "#define CUSTOS_BT CUSTOS_BLOCK" in src
    # the cache policy is never compiled in: it is an operand of the launch, so one kernel per
    # expression serves every launch size
    src4, h4 = capi.expr_emit(capi.KIND_APPLY, "f32", "x", ["x"], capi.Tuning(0, 0, 0, 3))
    assert src4 == src2 and h4 == h2
    assert "__builtin_amdgcn_raw_buffer_load_b128(rs, offset, 0, 2)" in src2
    src5, h5 = capi.expr_emit(capi.KIND_APPLY, "f32", "x", ["x"], capi.Tuning(0, 2, 0, -1))
    assert len({h1, h2, h5}) == 3                # "open" and "fixed to the same value" are different keys
    assert "custos_tile1(" not in src5
    assert "const u64 mode" in src2


def test_one_entry_point_per_translation_unit():
    """What `custos_hip_expr_compile` compiles is ONE function, as the reference's cache does per text
    (src/devices/cuda/kernel_cache.rs:39-61): the entry points for merged launches are translation
    units of their own, compiled when a graph build or `custos_hip_kernel_prepare_merged` asks for
    them.  An expression is expanded once per element of a tile (2 vectors x 4 elements, and 1 x 4 for
    the one-wavefront shape) and once for the scalar elements at the edges of a view -- thirteen times
    in the unit of the single launch, where the one unit of all three entry points held 41."""
    chain = fused_source([lambda v: v.sin(), lambda v: v.mul(2.0), lambda v: v.add(1.0), lambda v: v.max(0.0),
                          lambda v: v.sub(0.5)], "f32")
    text, _ = capi.expr_emit(capi.KIND_APPLY, "f32", chain, ["x"])
    units = re.split(r"\n// ---- translation unit of the entry point \w+ ----\n", text)
    assert len(units) == 3
    name = re.search(r"custos_apply_f32_\w{16}", units[0]).group(0)
    for unit, suffix in zip(units, ("", "_batched", "_ragged")):
        entries = re.findall(r'extern "C" __global__ void __launch_bounds__\(CUSTOS_BLOCK\)\n(\w+)\(', unit)
        assert entries == [name + suffix]
        # the per-element function is called from the tile's element loop and from ONE loop over
        # the scalar elements (head and tail of a view together)
        assert len(re.findall(r"custos_elem\(", unit)) == 4        # definition + two tile functions + edges
        assert len(re.findall(r"custos_sin\(", unit)) == 2         # wrapper definition + the one use in the expression
    assert "for (u64 e = gid; e < n_edge; e += n_threads)" in units[0]


def test_integer_rejects_transcendentals_and_fractions():
    for bad in ("sin(x)", "pow(x, 2)", "(x + 1.5)"):
        with pytest.raises(capi.CustosHipError) as e:
            capi.expr_emit(capi.KIND_APPLY, "i32", bad, ["x"])
        assert e.value.code == capi.ERR_EXPR_UNSUPPORTED
    capi.expr_emit(capi.KIND_APPLY, "i32", "(x + 1.0)", ["x"])  # integral value is fine


def test_unary_grad_takes_one_marker():
    with pytest.raises(capi.CustosHipError) as e:
        capi.expr_emit(capi.KIND_UNARY_GRAD, "f32", "(x + y)", ["x", "y"])
    assert e.value.code == capi.ERR_ARITY_MISMATCH
    src, _ = capi.expr_emit(capi.KIND_UNARY_GRAD, "f32", "cos(x)", ["x"])
    assert "const C prod = o * d;" in src and "const C sum = g + prod;" in src


def test_marker_arguments_validated():
    for markers in ([], ["x", "x"], ["a", "b", "c", "d", "e"]):
        with pytest.raises(capi.CustosHipError) as e:
            capi.expr_emit(capi.KIND_APPLY, "f32", "x", markers)
        assert e.value.code == capi.ERR_INVALID_ARGUMENT


def test_parser_survives_malformed_input():
    """Random token soup and mutated valid expressions: every input is either compiled to text
    or rejected with a message; nothing crashes, nesting is bounded."""
    import random
    rng = random.Random(7)
    atoms = ["x", "y", "(", ")", " ", "+", "-", "*", "/", ",", "sin", "cos", "tan", "tanh", "exp", "log", "abs",
             "sqrt", "pow", "min", "max", ">=", "<=", "==", "1.0", "2", "0.5e3", "inf", "NaN", "1e400", "=", ";",
             "\n", "x = ", "z", "1.", ".5", "0x10", "-(", "((", "))", "\x00", "\xff"]
    good = ["(x + y)", "pow((x * 3.0), (y + 1.0))", "x = sin(x);\nx = -(x);\nx = cos(x);\n", "((x >= 0) * x)",
            "-(tan(x))", "max(x, 0.0)"]
    accepted = rejected = 0
    for it in range(6000):
        if it % 3 == 0:
            s = list(rng.choice(good))
            for _ in range(rng.randint(1, 3)):
                pos = rng.randrange(len(s)) if s else 0
                kind = rng.randrange(3)
                if kind == 0 and s:
                    del s[pos:pos + rng.randint(1, 3)]
                elif kind == 1:
                    s.insert(pos, rng.choice(atoms))
                elif s:
                    s[pos] = chr(rng.randrange(1, 128))
            s = "".join(s)
        else:
            s = "".join(rng.choice(atoms) for _ in range(rng.randint(1, 24)))
        s = s.replace("\x00", "")          # C strings end at NUL
        for dtype in rng.sample(list(capi.DTYPES), 2):
            try:
                src, _ = capi.expr_emit(rng.choice([capi.KIND_APPLY, capi.KIND_UNARY_GRAD]), dtype, s, ["x", "y"])
                assert "custos_expr" in src
                accepted += 1
            except capi.CustosHipError as e:
                assert str(e)
                rejected += 1
    assert accepted > 20 and rejected > 1000
    for depth in (300, 100000):
        with pytest.raises(capi.CustosHipError) as e:
            capi.expr_emit(capi.KIND_APPLY, "f32", "(" * depth + "x" + ")" * depth, ["x"])
        assert "nested too deeply" in str(e.value)
        with pytest.raises(capi.CustosHipError):
            capi.expr_emit(capi.KIND_APPLY, "f32", "sin(" * depth + "x" + ")" * depth, ["x"])
