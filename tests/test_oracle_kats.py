"""Pins the CPU oracle against every known answer the reference holds for this
path, plus closed forms that catch a wrong sign, operand order or rounding."""
import math

import numpy as np
import pytest

from tests.helpers import assert_bits_equal


def f32(v):
    return float(np.float32(v))


def test_exp_is_e(oracle):
    # src/two_way_ops/mod.rs:63-68: f(1f32).eval() == core::f32::consts::E exactly
    assert np.float32(oracle.eval_scalar(lambda x: x.exp(), 1.0)) == np.float32(math.e)


def test_neg_tan(oracle):
    # src/two_way_ops/mod.rs:79-85
    assert abs(oracle.eval_scalar(lambda x: x.tan().neg(), 2.0) - 2.1850398) < 1e-6


def test_pow(oracle):
    # src/two_way_ops/mod.rs:96-100: (3*3)^(2+1) == 729 exactly
    assert oracle.eval_scalar(lambda x, y: x.mul(3.).pow(y.add(1.)), 3.0, 2.0) == 729.0


def test_int_kats(oracle):
    ev = lambda f, *v: oracle.eval_scalar(f, *v, dtype="i32")
    assert ev(lambda x, y: x.eq(y), 3, 3) == 1                 # mod.rs:108-111
    assert ev(lambda x: x.geq(0).mul(x), 3) == 3               # mod.rs:122-125
    assert ev(lambda x: x.add(3), 3) == 6                      # mod.rs:136-139
    assert ev(lambda x: x.geq(4), 3) == 0                      # mod.rs:150-153
    assert ev(lambda x: x.add(2).add(x.mul(8)), 4) == 38       # mod.rs:165-167


def test_eq_variants(oracle):
    # the reference CPU Eval of eq is `<=` (ops/cmps.rs:135); its GPU text is `==`
    f = lambda x, y: x.eq(y)
    assert oracle.eval_scalar(f, 2, 3, dtype="i32", eq_mode="eq") == 0
    assert oracle.eval_scalar(f, 2, 3, dtype="i32", eq_mode="eq_cpuref") == 1
    assert oracle.eval_scalar(f, 3, 2, dtype="i32", eq_mode="eq_cpuref") == 0


def test_two_args(oracle):
    # src/two_way_ops/mod.rs:180-188: ((4+3)*3.6)-3 ~ 22.2
    assert abs(oracle.eval_scalar(lambda x, y: x.add(y).mul(3.6).sub(y), 4.0, 3.0) - 22.2) < 1e-5


def test_eval_doc_examples(oracle):
    # src/two_way_ops/eval.rs:10-12 and resolve.rs:14-17
    assert oracle.eval_scalar(lambda x: x.add(2.5).mul(3.5), 1.5) == 14.0
    assert oracle.eval_scalar(lambda x: x.mul(x).add(2.), 1.5) == 4.25


def test_clip(oracle):
    # src/two_way_ops/mod.rs:206-217
    out = oracle.apply_fn(lambda x: x.max(3.).min(5.), [1., 3., 4., 6., 3., 2.], dtype="f64")
    assert out.tolist() == [3., 3., 4., 5., 3., 3.]


def test_apply_int_add(oracle):
    # src/two_way_ops/mod.rs:236-245
    out = oracle.apply_fn(lambda x: x.add(3), [3, 3, 4, 5, 3, 2], dtype="i32")
    assert out.tolist() == [6, 6, 7, 8, 6, 5]


def test_more_complex_f64(oracle):
    # src/two_way_ops/mod.rs:262-283: literals asserted by the reference
    out = oracle.apply_fn(lambda x: x.mul(2.).add(4.).sin().mul(x).add(1.), [3., 3., 4., 5., 3., 2.], dtype="f64")
    want = [-0.6320633326681093, -0.6320633326681093, -1.1462916720017398, 5.953036778474352,
            -0.6320633326681093, 2.978716493246764]
    assert np.allclose(out, want, rtol=0, atol=1e-15)


def test_stored_ops_chain(oracle):
    # src/two_way_ops/mod.rs:360-388: ln -> cos -> sin applied in sequence equals the nested call
    ops = [lambda x: x.ln(), lambda x: x.cos(), lambda x: x.sin()]
    got = oracle.fused_apply_fn(ops, np.array([3.4], dtype=np.float32))[0]
    want = np.sin(np.cos(np.log(np.float32(3.4), dtype=np.float32), dtype=np.float32), dtype=np.float32)
    assert abs(float(got) - float(want)) <= float(np.spacing(np.float32(1.0)))
    nested = oracle.apply_fn(lambda x: x.ln().cos().sin(), np.array([3.4], dtype=np.float32))[0]
    assert got == nested


def test_apply_mul2(oracle):
    # src/unary.rs:15-18
    assert oracle.apply_fn(lambda x: x.mul(2.), [1., 2., 3., 3., 2., 1.], dtype="f64").tolist() == [2., 4., 6., 6., 4., 2.]


def test_unary_grad_const(oracle):
    # src/unary.rs:40-47: lhs_grad += 1 * 2
    out = oracle.add_unary_grad(lambda x: x.val(2.0), [1., 2., 3., 3., 2., 1.], [0.] * 6, [1.] * 6, dtype="f64")
    assert out.tolist() == [2.] * 6


def test_unary_grad_int(oracle):
    # src/devices/cuda/ops.rs:259-272: lhs=[1..6], grad=[1..6], out=1, f = 2x+1 -> [4,7,10,13,16,19]
    out = oracle.add_unary_grad(lambda x: x.mul(2).add(1), [1, 2, 3, 4, 5, 6], [1, 2, 3, 4, 5, 6], [1] * 6, dtype="i32")
    assert out.tolist() == [4, 7, 10, 13, 16, 19]
    # src/devices/cuda/ops.rs:279-294: f = x+2 -> [4,6,8,10,12,14]
    out = oracle.add_unary_grad(lambda x: x.add(2), [1, 2, 3, 4, 5, 6], [1, 2, 3, 4, 5, 6], [1] * 6, dtype="i32")
    assert out.tolist() == [4, 6, 8, 10, 12, 14]


def test_apply_string_literal(oracle):
    # src/devices/cuda/ops.rs:250-257: x.add("1.0") -> [2..7]
    out = oracle.apply_fn(lambda x: x.add("1.0"), [1., 2., 3., 4., 5., 6.])
    assert out.tolist() == [2., 3., 4., 5., 6., 7.]


def test_sin_cos_reference_vectors(oracle):
    # src/unary.rs:150-155,195-200: forward sin and gradient cos at 1..4
    x = np.array([1., 2., 3., 4.])
    sin_want = [0.8414709848078965, 0.9092974268256817, 0.1411200080598672, -0.7568024953079282]
    cos_want = [0.5403023058681398, -0.4161468365471424, -0.9899924966004454, -0.6536436208636119]
    assert oracle.apply_fn(lambda v: v.sin(), x, dtype="f64").tolist() == sin_want
    # src/unary.rs:268-275 asserts the gradient with assert_eq! (exact, f64)
    assert oracle.add_unary_grad(lambda v: v.cos(), x, np.zeros(4), np.ones(4), dtype="f64").tolist() == cos_want
    # f32 versions agree to f32 precision
    assert np.allclose(oracle.apply_fn(lambda v: v.sin(), x), sin_want, atol=1e-7)


def test_min_max_are_selects(oracle):
    # src/number.rs:201-209: max = if a > b {a} else {b}; min = if a < b {a} else {b}
    nan, inf = float("nan"), float("inf")
    mx = lambda a, b: oracle.eval_scalar(lambda x, y: x.max(y), a, b)
    mn = lambda a, b: oracle.eval_scalar(lambda x, y: x.min(y), a, b)
    assert mx(nan, 1.0) == 1.0 and math.isnan(mx(1.0, nan))      # NaN on the left returns rhs
    assert mn(nan, 1.0) == 1.0 and math.isnan(mn(1.0, nan))
    assert math.copysign(1.0, mx(-0.0, 0.0)) == 1.0               # -0 > 0 is false -> rhs (+0)
    assert math.copysign(1.0, mx(0.0, -0.0)) == -1.0              # 0 > -0 is false -> rhs (-0)
    assert mx(-inf, inf) == inf and mn(-inf, inf) == -inf


def test_operand_order_and_signs(oracle):
    ev = oracle.eval_scalar
    assert ev(lambda x, y: x.sub(y), 5.0, 3.0) == 2.0
    assert ev(lambda x, y: x.div(y), 1.0, 4.0) == 0.25
    assert ev(lambda x, y: x.pow(y), 2.0, 10.0) == 1024.0
    assert ev(lambda x, y: x.geq(y), 1.0, 2.0) == 0.0 and ev(lambda x, y: x.leq(y), 1.0, 2.0) == 1.0
    assert ev(lambda x: x.neg(), 2.5) == -2.5 and ev(lambda x: x.abs(), -2.5) == 2.5
    assert ev(lambda x: x.identity(), -7.25) == -7.25
    assert ev(lambda x: x.sqrt(), 6.25) == 2.5
    assert ev(lambda x: x.ln(), 1.0) == 0.0
    assert ev(lambda x: x.tanh(), 0.0) == 0.0


def test_one_rounding_per_node_no_fma(oracle):
    # a*b+c with a*b inexact: fused and unfused results differ; the oracle must be the unfused one
    a, b, c = np.float32(1 + 3 * 2.0 ** -23), np.float32(1 + 3 * 2.0 ** -23), np.float32(-1.0)
    got = np.float32(oracle.eval_scalar(lambda x, y: x.mul(y).add(float(c)), float(a), float(b)))
    unfused = np.float32(np.float32(a * b) + c)
    fused = np.float32(np.float64(a) * np.float64(b) + np.float64(c))
    assert unfused != fused
    assert got == unfused
    g = oracle.add_unary_grad(lambda x: x.identity(), np.array([a]), np.array([c]), np.array([b]))[0]
    assert g == unfused


def test_denormals_are_kept(oracle):
    tiny = np.float32(1e-40)
    out = oracle.apply_fn(lambda x: x.mul(0.5), np.array([tiny], dtype=np.float32))[0]
    assert out == np.float32(tiny * np.float32(0.5)) and out != 0


def test_monomorphic_loops_equal_interpreter(oracle):
    from custos_amd import synth
    n = 4099
    x = synth.uniform_f32(0, n, -np.pi, np.pi)
    ops = [lambda v: v.sin(), lambda v: v.mul(2.0), lambda v: v.add(1.0), lambda v: v.max(0.0), lambda v: v.sub(0.5)]
    want = oracle.fused_apply_fn(ops, x)
    assert_bits_equal(oracle.c2_chain_fused(x), want)
    assert_bits_equal(oracle.c2_chain_unfused(x), want)
    assert_bits_equal(oracle.c1_exp(x), oracle.apply_fn(lambda v: v.exp(), x))
    assert_bits_equal(oracle.c3_tanh_fwd(x), oracle.apply_fn(lambda v: v.tanh(), x))
    g = synth.uniform_f32(1, n, -1, 1)
    o = synth.uniform_f32(2, n, -1, 1)
    tanh_grad = lambda v: v.val(1.0).sub(v.tanh().mul(v.tanh()))
    assert_bits_equal(oracle.c3_tanh_bwd(x, g, o), oracle.add_unary_grad(tanh_grad, x, g, o))
    xb = synth.uniform_f16_bits(0, n, -2, 2)
    c4 = lambda v: v.mul(0.5).exp().mul(v).add(v.mul(v))
    assert_bits_equal(oracle.c4_chain_f16(xb), oracle.apply_fn(c4, xb, dtype="f16"))
    a, b, c = (synth.uniform_f32(s, n, 0, 1) for s in (1, 2, 3))
    t, u, y = oracle.c5_graph(a, b, c)
    assert_bits_equal(y, oracle.apply_fn(lambda p, q, r: p.mul(q).add(r).abs().sqrt().mul(0.3), a, b, c))


def test_f16_conversion_brute_force(oracle):
    # every half value round-trips, and widening matches numpy's float16 exactly
    bits = np.arange(65536, dtype=np.uint16)
    wide = oracle.f16_bits_to_f32(bits)
    np_wide = bits.view(np.float16).astype(np.float32)
    assert_bits_equal(wide, np_wide, "f16->f32")
    finite = np.isfinite(np_wide)
    back = oracle.f32_to_f16_bits(wide)
    assert np.array_equal(back[finite], bits[finite])
    # all rounding boundaries: midpoints between adjacent halves and their f32 neighbours
    pos = np_wide[(bits < 0x7c00)]
    mids = ((pos[:-1].astype(np.float64) + pos[1:].astype(np.float64)) / 2).astype(np.float32)
    cand = np.concatenate([mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                           np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e-8, 2.98e-8, 2.9802322e-8, 5.96e-8, 6e-8,
                                     np.inf, 0.0], dtype=np.float32)])
    cand = np.concatenate([cand, -cand])
    with np.errstate(over="ignore"):
        want = cand.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16_bits(cand), want)
    assert oracle.f32_to_f16_bits(np.array([np.nan], dtype=np.float32))[0] & 0x7c00 == 0x7c00


def test_bf16_conversion(oracle):
    l = oracle.lib()
    rng = np.random.default_rng(0)
    vals = rng.standard_normal(20000).astype(np.float32) * np.float32(100)
    for v in vals[:4000]:
        b = l.oracle_f32_to_bf16(float(v))
        u = np.float32(v).view(np.uint32)
        want = (int(u) + 0x7FFF + ((int(u) >> 16) & 1)) >> 16
        assert b == want & 0xFFFF
        assert np.float32(l.oracle_bf16_to_f32(b)).view(np.uint32) == np.uint32(b << 16)
    # ties go to even
    assert l.oracle_f32_to_bf16(float(np.uint32(0x3F808000).view(np.float32))) == 0x3F80
    assert l.oracle_f32_to_bf16(float(np.uint32(0x3F818000).view(np.float32))) == 0x3F82


def test_per_node_rounding_against_independent_half_arithmetic(oracle):
    """The per-node modes (every node rounded to the storage type, src/number.rs:487-676) against
    arithmetic that does not go through the restatement: numpy's float16 operators are IEEE
    binary16 operations, and for + - * / sqrt "f32 operation, then one rounding" IS the correctly
    rounded 16-bit operation (24 >= 2*11 + 2 significand bits), so both must agree bit for bit.
    bf16 has no numpy type: each step is done in f32 and rounded with the integer formula."""
    from custos_amd import synth
    n = 20011
    xb = synth.uniform_f16_bits(31, n, -3, 3)
    yb = synth.uniform_f16_bits(32, n, 0.5, 2)
    f = lambda a, b: a.mul(0.3).add(b).mul(a).div(b.add(1.7)).sub(0.1).abs().sqrt().max(0.25).neg()
    x, y = xb.view(np.float16), yb.view(np.float16)
    h = np.float16
    with np.errstate(all="ignore"):
        r = np.sqrt(np.abs(((x * h(0.3) + y) * x) / (y + h(1.7)) - h(0.1)))
        r = -np.where(r > h(0.25), r, h(0.25))
    assert r.dtype == np.float16
    assert_bits_equal(oracle.apply_fn(f, xb, yb, dtype="f16_pernode"), r.view(np.uint16))
    # the f32-compute mode rounds once and gives other bits for a good part of the inputs
    assert (oracle.apply_fn(f, xb, yb, dtype="f16") != r.view(np.uint16)).mean() > 0.01

    def bf(v):  # f32 -> nearest-even bf16 -> f32 (finite values)
        u = np.asarray(v, dtype=np.float32).view(np.uint32).astype(np.uint64)
        u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
        return u.astype(np.uint32).view(np.float32)

    xs = bf(synth.uniform_f32(33, n, -3, 3))
    ys = bf(synth.uniform_f32(34, n, 0.5, 2))
    f32 = np.float32
    with np.errstate(all="ignore"):
        t = bf(xs * bf(f32(0.3)))
        t = bf(t + ys)
        t = bf(t * xs)
        t = bf(t / bf(ys + bf(f32(1.7))))
        t = bf(t - bf(f32(0.1)))
        t = bf(np.sqrt(np.abs(t)))
        t = -np.where(t > f32(0.25), t, f32(0.25))
    to_bits = lambda v: (v.view(np.uint32) >> 16).astype(np.uint16)
    assert_bits_equal(oracle.apply_fn(f, to_bits(xs), to_bits(ys), dtype="bf16_pernode"), to_bits(t))

    # gradient: g + round(o * d), both per-node (src/devices/cpu_stack_ops.rs:27-29 in 16-bit arithmetic)
    d = lambda v: v.mul(v).mul(3.0).add(0.7)
    g0 = synth.uniform_f16_bits(35, n, -1, 1)
    with np.errstate(all="ignore"):
        want = g0.view(np.float16) + y * ((x * x) * h(3.0) + h(0.7))
    assert_bits_equal(oracle.add_unary_grad(d, xb, g0, yb, dtype="f16_pernode"), want.view(np.uint16))


def test_integer_wrap(oracle):
    out = oracle.apply_fn(lambda x: x.mul(2), [2 ** 30, -(2 ** 30) - 1], dtype="i32")
    assert out.tolist() == [-(2 ** 31), 2 ** 31 - 2]
    out = oracle.apply_fn(lambda x: x.add(200), [100], dtype="u8")
    assert out.tolist() == [44]


def test_malformed_program_is_rejected(oracle):
    import ctypes as C
    prog = (oracle.Ins * 1)()
    prog[0].op = oracle.OPS["add"]
    res = C.c_float()
    assert oracle.lib().oracle_eval_f32(prog, 1, (C.c_float * 1)(1.0), 1, C.byref(res)) != 0
    with pytest.raises(RuntimeError):
        oracle.apply_fn(lambda x: x.sin(), [1, 2], dtype="i32")


def test_per_node_f16_routines_against_numpy_float16(oracle):
    """The routine nodes of the per-node f16 mode (`Float for f16`: f32 routine, one rounding,
    src/number.rs:543-608) against numpy's float16 ufuncs, which are another implementation of
    "widen, f32 routine, round": all 65 536 inputs per node, NaN where numpy has NaN, the same
    infinities, never more than one unit of f16 apart, and over 99 % of the results bit-identical
    (the two f32 routines, glibc's and numpy's, may differ in the last place before the rounding)."""
    bits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    x = bits.view(np.float16)
    nodes = {"exp": (lambda v: v.exp(), np.exp), "sin": (lambda v: v.sin(), np.sin), "cos": (lambda v: v.cos(), np.cos),
             "tan": (lambda v: v.tan(), np.tan), "tanh": (lambda v: v.tanh(), np.tanh), "ln": (lambda v: v.ln(), np.log),
             "sqrt": (lambda v: v.sqrt(), np.sqrt)}
    ordered = lambda b: np.where(b.astype(np.int32) & 0x8000, -(b.astype(np.int32) & 0x7fff), b.astype(np.int32) & 0x7fff)
    for name, (f, ufunc) in nodes.items():
        with np.errstate(all="ignore"):
            ref = ufunc(x)
        assert ref.dtype == np.float16
        want = ref.view(np.uint16)
        got = oracle.apply_fn(f, bits, dtype="f16_pernode")
        nan = np.isnan(ref)
        assert np.array_equal(np.isnan(got.view(np.float16)), nan), name
        inf = np.isinf(ref)
        assert np.array_equal(got[inf], want[inf]), name
        rest = ~nan & ~inf
        dist = np.abs(ordered(got[rest]) - ordered(want[rest]))
        assert dist.max() <= 1, f"{name}: {dist.max()} units of f16 apart at bits {bits[rest][dist.argmax()]:#06x}"
        assert (dist == 0).mean() > 0.99, f"{name}: {(dist == 0).mean():.4f} bit-identical"
        if name == "sqrt":
            assert dist.max() == 0


def test_per_node_bf16_routines_against_torch_bfloat16(oracle):
    """The routine nodes of the per-node bf16 mode (`Float for bf16`: f32 routine, one rounding,
    src/number.rs:610-676) against torch's CPU bfloat16 operators, another implementation of "widen,
    f32 routine, round to nearest even": all 65 536 inputs per node, NaN where torch has NaN, the same
    infinities, never more than one unit of bf16 apart and over 99 % bit-identical (the two f32
    routines may differ in the last place before the rounding); sqrt and the arithmetic on random
    pairs bit for bit."""
    torch = pytest.importorskip("torch")
    bits = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
    x = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)
    as_bits = lambda t: t.view(torch.int16).numpy().view(np.uint16)
    nodes = {"exp": (lambda v: v.exp(), torch.exp), "sin": (lambda v: v.sin(), torch.sin), "cos": (lambda v: v.cos(), torch.cos),
             "tan": (lambda v: v.tan(), torch.tan), "tanh": (lambda v: v.tanh(), torch.tanh), "ln": (lambda v: v.ln(), torch.log),
             "sqrt": (lambda v: v.sqrt(), torch.sqrt)}
    ordered = lambda b: np.where(b.astype(np.int32) & 0x8000, -(b.astype(np.int32) & 0x7fff), b.astype(np.int32) & 0x7fff)
    for name, (f, op) in nodes.items():
        ref = op(x)
        assert ref.dtype == torch.bfloat16
        want = as_bits(ref)
        got = oracle.apply_fn(f, bits, dtype="bf16_pernode")
        nan = torch.isnan(ref).numpy()
        got_nan = ((got & 0x7f80) == 0x7f80) & ((got & 0x007f) != 0)
        assert np.array_equal(got_nan, nan), name
        inf = torch.isinf(ref).numpy()
        assert np.array_equal(got[inf], want[inf]), name
        rest = ~nan & ~inf
        dist = np.abs(ordered(got[rest]) - ordered(want[rest]))
        assert dist.max() <= 1, f"{name}: {dist.max()} units of bf16 apart at bits {bits[rest][dist.argmax()]:#06x}"
        assert (dist == 0).mean() > 0.99, f"{name}: {(dist == 0).mean():.4f} bit-identical"
        if name == "sqrt":
            assert dist.max() == 0
    rng = np.random.default_rng(11)
    a_bits = rng.integers(0, 1 << 16, size=1 << 18, dtype=np.uint32).astype(np.uint16)
    b_bits = rng.integers(0, 1 << 16, size=1 << 18, dtype=np.uint32).astype(np.uint16)
    ta = torch.from_numpy(a_bits.view(np.int16).copy()).view(torch.bfloat16)
    tb = torch.from_numpy(b_bits.view(np.int16).copy()).view(torch.bfloat16)
    for name, f, op in (("add", lambda p, q: p.add(q), torch.add), ("sub", lambda p, q: p.sub(q), torch.sub),
                        ("mul", lambda p, q: p.mul(q), torch.mul), ("div", lambda p, q: p.div(q), torch.div)):
        ref = op(ta, tb)
        want = as_bits(ref)
        got = oracle.apply_fn(f, a_bits, b_bits, dtype="bf16_pernode")
        nan = torch.isnan(ref).numpy()
        assert np.array_equal(((got & 0x7f80) == 0x7f80) & ((got & 0x007f) != 0), nan), name
        assert np.array_equal(got[~nan], want[~nan]), name


def test_the_oracle_stands_on_its_own():
    """The oracle traces closures with a tracer of its own: a process that evaluates an expression through it
    has imported nothing of the package under test (a mistake in the package's expression classes cannot be
    shared), and the non-commutative nodes keep the order lhs, rhs on known answers."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys\n"
        "from oracle import cpu_oracle as o\n"
        "assert o.apply_fn(lambda v: v.val(10.0).sub(v), [1.0, 4.0]).tolist() == [9.0, 6.0]\n"
        "assert o.apply_fn(lambda a, b: a.div(b), [8.0], [2.0]).tolist() == [4.0]\n"
        "assert o.apply_fn(lambda a, b: a.pow(b), [2.0], [3.0]).tolist() == [8.0]\n"
        "assert o.apply_fn(lambda a, b: a.geq(b).sub(a.leq(b)), [3.0, 1.0], [2.0, 2.0]).tolist() == [1.0, -1.0]\n"
        "assert o.apply_fn(lambda v: v.sub(1.0).mul(2.0), [4.0]).tolist() == [6.0]\n"
        "assert not [m for m in sys.modules if m.split('.')[0] == 'custos_amd'], 'the oracle imported the package'\n"
    )
    proc = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-800:]
