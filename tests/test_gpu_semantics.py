"""GPU parity for node semantics, element types, addressing and error paths."""
import ctypes as C

import numpy as np
import pytest

from custos_amd import Const, capi, synth
from tests.helpers import assert_bits_equal, ulp_distance_f16, ulp_distance_f32

pytestmark = pytest.mark.gpu

SPECIALS = np.array([0.0, -0.0, 1.0, -1.0, 0.5, 3.0, -3.0, np.inf, -np.inf, np.nan, 1e-40, -1e-40, 1.17549435e-38,
                     3.4028235e38, -3.4028235e38, 1e-45, 2.5, -2.5, 65504.0, 1e20], dtype=np.float32)


def pairs():
    a = np.repeat(SPECIALS, SPECIALS.size)
    b = np.tile(SPECIALS, SPECIALS.size)
    return a, b


BINARY_EXACT = {
    "add": lambda p, q: p.add(q), "sub": lambda p, q: p.sub(q), "mul": lambda p, q: p.mul(q),
    "div": lambda p, q: p.div(q), "min": lambda p, q: p.min(q), "max": lambda p, q: p.max(q),
    "geq": lambda p, q: p.geq(q), "leq": lambda p, q: p.leq(q), "eq": lambda p, q: p.eq(q),
}


@pytest.mark.parametrize("name", sorted(BINARY_EXACT))
def test_binary_nodes_on_special_values(hip, oracle, name):
    """+ - * / min max and the comparisons are bit-exact, including signed zeros,
    NaN, infinities and denormals (nothing is flushed, min/max are selects)."""
    a, b = pairs()
    f = BINARY_EXACT[name]
    got = hip.apply_fn2(hip.buffer(a), hip.buffer(b), f).read()
    assert_bits_equal(got, oracle.apply_fn(f, a, b), name)


def test_eq_as_the_cpu_device_evaluates_it(oracle):
    """The reference's CPU `Eval` of `eq` is `<=` (src/two_way_ops/ops/cmps.rs:135) while its GPU kernels are
    the text `(a == b)`.  Kernels compute `==` by default; with CUSTOS_HIP_EQ_AS_CPU_EVAL they compute what
    CPU<Base> computes, bit for bit against the oracle's restatement of that `Eval`, NaNs and zeros included;
    the two forms are different kernels, and switching back brings `==` back."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        a, b = pairs()
        ints_a = np.array([1, 2, 3, 4, 5, -7, 0], dtype=np.int32)
        ints_b = np.array([1, 3, 2, 4, -5, -7, 1], dtype=np.int32)
        eq = lambda p, q: p.eq(q)
        clip_eq = lambda p, q: p.eq(q).mul(p).add(q)          # an eq node inside a larger expression
        exact = dev.apply_fn2(dev.buffer(a), dev.buffer(b), eq).read()
        assert_bits_equal(exact, oracle.apply_fn(eq, a, b), "== by default")
        dev.set_eq_policy(capi.EQ_AS_CPU_EVAL)
        for f in (eq, clip_eq):
            got = dev.apply_fn2(dev.buffer(a), dev.buffer(b), f).read()
            assert_bits_equal(got, oracle.apply_fn(f, a, b, eq_mode="eq_cpuref"), "eq as CPU<Base> evaluates it")
        got = dev.apply_fn2(dev.buffer(ints_a, "i32"), dev.buffer(ints_b, "i32"), eq).read()
        assert got.tolist() == [1, 1, 0, 1, 0, 1, 1]           # a <= b; eq(3, 3) = 1 is the value src/two_way_ops/mod.rs:108-111 holds
        assert not np.array_equal(exact, dev.apply_fn2(dev.buffer(a), dev.buffer(b), eq).read())
        dev.set_eq_policy(capi.EQ_EXACT)
        assert_bits_equal(dev.apply_fn2(dev.buffer(a), dev.buffer(b), eq).read(), exact, "== again")
        with pytest.raises(capi.CustosHipError):
            dev.set_eq_policy(7)
    finally:
        dev.close()


@pytest.mark.parametrize("name,f", [("neg", lambda v: v.neg()), ("abs", lambda v: v.abs()), ("identity", lambda v: v.identity()),
                                    ("sqrt", lambda v: v.sqrt()), ("relu_geq", lambda v: v.geq(0.).mul(v)),
                                    ("relu_max", lambda v: v.max(0.)), ("clip", lambda v: v.max(3.).min(5.))])
def test_unary_exact_nodes(hip, oracle, name, f):
    x = np.concatenate([SPECIALS, synth.uniform_f32(11, 5000, -10, 10), synth.uniform_f32(12, 5000, 0, 1e-38)])
    got = hip.apply_fn(hip.buffer(x), f).read()
    assert_bits_equal(got, oracle.apply_fn(f, x), name)


def test_division_and_sqrt_are_correctly_rounded(hip, oracle):
    n = 1 << 18
    a = synth.uniform_f32(21, n, -100, 100)
    b = synth.uniform_f32(22, n, -7, 7)
    assert_bits_equal(hip.apply_fn2(hip.buffer(a), hip.buffer(b), lambda p, q: p.div(q)).read(),
                      oracle.apply_fn(lambda p, q: p.div(q), a, b))
    c = np.abs(a) * np.float32(1e-3)
    assert_bits_equal(hip.apply_fn(hip.buffer(c), lambda v: v.sqrt()).read(), oracle.apply_fn(lambda v: v.sqrt(), c))


def test_mul_add_is_not_contracted(hip, oracle):
    n = 1 << 16
    a = synth.uniform_f32(31, n, 1, 2)
    b = synth.uniform_f32(32, n, 1, 2)
    f = lambda p, q: p.mul(q).sub(2.25)
    want = oracle.apply_fn(f, a, b)
    fused = (a.astype(np.float64) * b.astype(np.float64) - 2.25).astype(np.float32)
    assert (want != fused).any()  # the inputs do distinguish fma from mul+add
    assert_bits_equal(hip.apply_fn2(hip.buffer(a), hip.buffer(b), f).read(), want)


TRANSCENDENTAL = {
    "exp": (lambda v: v.exp(), -87.0, 88.0), "sin": (lambda v: v.sin(), -100.0, 100.0),
    "cos": (lambda v: v.cos(), -100.0, 100.0), "tan": (lambda v: v.tan(), -1.5, 1.5),
    "tanh": (lambda v: v.tanh(), -10.0, 10.0), "ln": (lambda v: v.ln(), 1e-30, 1e30),
}


@pytest.mark.parametrize("name", sorted(TRANSCENDENTAL))
def test_transcendental_ulp(hip, oracle, name):
    """f32 transcendentals: within 4 ulp of the CPU path (libm)."""
    f, lo, hi = TRANSCENDENTAL[name]
    n = 1 << 19
    x = synth.uniform_f32(41, n, lo, hi)
    if name == "ln":
        x = np.exp(synth.uniform_f32(41, n, np.log(lo), np.log(hi))).astype(np.float32)
    got = hip.apply_fn(hip.buffer(x), f).read()
    want = oracle.apply_fn(f, x)
    d = ulp_distance_f32(got, want)
    assert d.max() <= 4, (name, int(d.max()), x[np.argmax(d)])


WIDE = {
    "exp": lambda v: v.exp(), "sin": lambda v: v.sin(), "cos": lambda v: v.cos(), "tan": lambda v: v.tan(),
    "tanh": lambda v: v.tanh(), "ln": lambda v: v.ln(), "sqrt": lambda v: v.sqrt(),
}


@pytest.mark.parametrize("name", sorted(WIDE))
def test_transcendentals_over_all_float_bit_patterns(hip, oracle, name):
    """2^22 random f32 bit patterns (every exponent, both signs, denormals, inf, NaN):
    within 4 ulp of the CPU path everywhere, NaN where it is NaN, same infinities.
    Overflow, underflow into denormals and huge arguments of sin/cos/tan are all in here."""
    n = 1 << 22
    bits = (synth.splitmix64(77, n) >> np.uint64(32)).astype(np.uint32)
    x = bits.view(np.float32)
    got = hip.apply_fn(hip.buffer(x), WIDE[name]).read()
    want = oracle.apply_fn(WIDE[name], x)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan), name
    d = ulp_distance_f32(got[~nan], want[~nan])
    worst = int(np.argmax(d))
    assert d.max() <= (0 if name == "sqrt" else 4), (name, int(d.max()), x[~nan][worst], got[~nan][worst], want[~nan][worst])


def test_pow_ulp(hip, oracle):
    n = 1 << 18
    a = synth.uniform_f32(51, n, 0.01, 20)
    b = synth.uniform_f32(52, n, -5, 5)
    f = lambda p, q: p.pow(q)
    d = ulp_distance_f32(hip.apply_fn2(hip.buffer(a), hip.buffer(b), f).read(), oracle.apply_fn(f, a, b))
    assert d.max() <= 4
    # src/two_way_ops/mod.rs:96-100: an exact case
    got = hip.apply_fn2(hip.buffer([3.0]), hip.buffer([2.0]), lambda x, y: x.mul(3.).pow(y.add(1.))).read()
    assert got[0] == 729.0


def test_sin_large_arguments(hip, oracle):
    x = np.concatenate([synth.uniform_f32(61, 1 << 16, -1e6, 1e6), synth.uniform_f32(62, 1 << 16, -1e30, 1e30)])
    got = hip.apply_fn(hip.buffer(x), lambda v: v.sin()).read()
    assert ulp_distance_f32(got, oracle.apply_fn(lambda v: v.sin(), x)).max() <= 4


def test_reference_int_vectors(hip):
    # src/two_way_ops/mod.rs:236-245, src/devices/cuda/ops.rs:259-272,279-294 (eager here)
    out = hip.apply_fn(hip.buffer([3, 3, 4, 5, 3, 2], "i32"), lambda x: x.add(3))
    assert out.read().tolist() == [6, 6, 7, 8, 6, 5]
    lhs = hip.buffer([1, 2, 3, 4, 5, 6], "i32")
    g = hip.buffer([1, 2, 3, 4, 5, 6], "i32")
    o = hip.buffer([1, 1, 1, 1, 1, 1], "i32")
    hip.add_unary_grad(lhs, g, o, lambda x: x.mul(2).add(1))
    assert g.read().tolist() == [4, 7, 10, 13, 16, 19]
    out = hip.apply_fn(hip.buffer([1., 2., 3., 4., 5., 6.]), lambda x: x.add("1.0"))  # cuda/ops.rs:250-257
    assert out.read().tolist() == [2., 3., 4., 5., 6., 7.]
    out = hip.apply_fn(hip.buffer([1., 3., 4., 6., 3., 2.]), lambda x: x.max(3.).min(5.))  # mod.rs:206-217
    assert out.read().tolist() == [3., 3., 4., 5., 3., 3.]


def test_unary_grad_doc_example(hip):
    # src/unary.rs:40-47
    from custos_amd import to_val
    a = hip.buffer([1., 2., 3., 3., 2., 1.], "f64")
    og = hip.buffer([1.] * 6, "f64")
    g = hip.buffer([0.] * 6, "f64")
    hip.add_unary_grad(a, g, og, lambda x: to_val(2.0))
    assert g.read().tolist() == [2.] * 6


INT_TYPES = ["i8", "u8", "i16", "u16", "i32", "u32", "i64", "u64"]


@pytest.mark.parametrize("dtype", INT_TYPES)
def test_integer_types_wrap_like_the_cpu(hip, oracle, dtype):
    npdt = np.dtype(capi.DTYPES[dtype][1])
    info = np.iinfo(npdt)
    rng = np.random.default_rng(7)
    x = rng.integers(info.min, info.max, size=10007, dtype=npdt, endpoint=True)
    y = rng.integers(info.min, info.max, size=10007, dtype=npdt, endpoint=True)
    f = lambda p, q: p.mul(q).add(p).sub(3).max(q).geq(p).add(p.min(q)).mul(5)
    got = hip.apply_fn2(hip.buffer(x, dtype), hip.buffer(y, dtype), f).read()
    assert_bits_equal(got, oracle.apply_fn(f, x, y, dtype=dtype), dtype)
    g = rng.integers(info.min, info.max, size=10007, dtype=npdt, endpoint=True)
    gb = hip.buffer(g, dtype)
    hip.add_unary_grad(hip.buffer(x, dtype), gb, hip.buffer(y, dtype), lambda v: v.mul(2).add(1))
    assert_bits_equal(gb.read(), oracle.add_unary_grad(lambda v: v.mul(2).add(1), x, g, y, dtype=dtype), dtype + " grad")


@pytest.mark.parametrize("dtype", ["i8", "u8"])
def test_every_pair_of_8bit_integers(hip, oracle, dtype):
    """All 65 536 operand pairs of the 8-bit types through every two-operand node, bit for bit (wrapping
    arithmetic, truncating division, comparisons to 1/0).  Division leaves out what panics in the
    reference: a zero divisor, and -128 / -1."""
    npdt = np.dtype(capi.DTYPES[dtype][1])
    info = np.iinfo(npdt)
    values = np.arange(info.min, info.max + 1, dtype=np.int64).astype(npdt)
    a, b = np.repeat(values, 256), np.tile(values, 256)
    ab, bb = hip.buffer(a, dtype), hip.buffer(b, dtype)
    for name, f in BINARY_EXACT.items():
        if name == "div":
            continue
        assert_bits_equal(hip.apply_fn2(ab, bb, f).read(), oracle.apply_fn(f, a, b, dtype=dtype), f"{dtype} {name}")
    ok = (b != 0) & ~((a == info.min) & (b.astype(np.int64) == -1))
    ad, bd = a[ok], b[ok]
    div = BINARY_EXACT["div"]
    got = hip.apply_fn2(hip.buffer(ad, dtype), hip.buffer(bd, dtype), div).read()
    assert_bits_equal(got, oracle.apply_fn(div, ad, bd, dtype=dtype), f"{dtype} div")
    # the oracle's division is C's, which truncates like Rust's: checked against numpy here
    q = np.trunc(ad.astype(np.float64) / bd.astype(np.float64)).astype(npdt)
    assert_bits_equal(got, q, f"{dtype} div against truncation")


def test_integer_division(hip, oracle):
    x = np.array([7, -7, 100, -100, 0, 5], dtype=np.int32)
    y = np.array([2, 2, -3, -3, 5, 5], dtype=np.int32)
    f = lambda p, q: p.div(q)
    assert_bits_equal(hip.apply_fn2(hip.buffer(x, "i32"), hip.buffer(y, "i32"), f).read(), oracle.apply_fn(f, x, y, dtype="i32"))


def test_f64(hip, oracle):
    n = 50001
    rng = np.random.default_rng(3)
    x = rng.uniform(-3, 3, n)
    exact = lambda v: v.mul(1.7).add(0.3).max(0.25).sub(v).div(3.0).abs().neg()
    assert_bits_equal(hip.apply_fn(hip.buffer(x, "f64"), exact).read(), oracle.apply_fn(exact, x, dtype="f64"))
    got = hip.apply_fn(hip.buffer(x, "f64"), lambda v: v.mul(2.).add(4.).sin().mul(v).add(1.)).read()
    want = oracle.apply_fn(lambda v: v.mul(2.).add(4.).sin().mul(v).add(1.), x, dtype="f64")
    assert np.max(np.abs(got - want)) <= 8 * np.finfo(np.float64).eps
    # src/two_way_ops/mod.rs:262-283
    ref = hip.apply_fn(hip.buffer([3., 3., 4., 5., 3., 2.], "f64"), lambda v: v.mul(2.).add(4.).sin().mul(v).add(1.)).read()
    assert np.allclose(ref, [-0.6320633326681093, -0.6320633326681093, -1.1462916720017398, 5.953036778474352,
                             -0.6320633326681093, 2.978716493246764], rtol=0, atol=1e-14)


def test_f64_transcendentals(hip, oracle):
    """f64 routine nodes against the oracle (glibc, under 1 ulp) on random inputs.  BASELINE states no
    f64 tolerance; the bound here is 4 units in the last place of the f64 result, measured on the bit
    patterns (the device's routines are documented to 1-2 ulp)."""
    n = 20001
    rng = np.random.default_rng(11)
    x = rng.uniform(-3, 3, n)
    pos = rng.uniform(1e-3, 50, n)
    y = rng.uniform(-3, 3, n)

    def ulps(got, want):
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        return np.abs(got[ok].view(np.int64) - want[ok].view(np.int64)).max()

    for name, f, arg in (("exp", lambda v: v.exp(), x), ("cos", lambda v: v.cos(), x), ("sin", lambda v: v.sin(), x),
                         ("tan", lambda v: v.tan(), x), ("tanh", lambda v: v.tanh(), x), ("ln", lambda v: v.ln(), pos)):
        got = hip.apply_fn(hip.buffer(arg, "f64"), f).read()
        want = oracle.apply_fn(f, arg, dtype="f64")
        assert ulps(got, want) <= 4, f"f64 {name}: {ulps(got, want)} ulp"
    power = lambda a, b: a.pow(b)
    got = hip.apply_fn2(hip.buffer(pos, "f64"), hip.buffer(y, "f64"), power).read()
    assert ulps(got, oracle.apply_fn(power, pos, y, dtype="f64")) <= 4
    # special values: the same infinities, zeros and NaNs
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 709.9, -745.2, 5e-324, 1e308])
    for name, f in (("exp", lambda v: v.exp()), ("tanh", lambda v: v.tanh()), ("ln", lambda v: v.ln()), ("cos", lambda v: v.cos())):
        got = hip.apply_fn(hip.buffer(special, "f64"), f).read()
        want = oracle.apply_fn(f, special, dtype="f64")
        assert np.array_equal(np.isnan(got), np.isnan(want)), name
        assert np.array_equal(np.isinf(got), np.isinf(want)) and np.array_equal(np.signbit(got[~np.isnan(want)]), np.signbit(want[~np.isnan(want)])), name
        fin = np.isfinite(want)
        assert np.abs(got[fin].view(np.int64) - want[fin].view(np.int64)).max() <= 4, name


def test_bf16(hip, oracle):
    n = 40003
    x32 = synth.uniform_f32(71, n, -4, 4)
    xb = (x32.view(np.uint32) >> 16).astype(np.uint16)
    f = lambda v: v.mul(1.5).add(v.mul(v)).sub(0.125)
    got = hip.apply_fn(hip.buffer(xb, "bf16"), f).read()
    assert_bits_equal(got, oracle.apply_fn(f, xb, dtype="bf16"))


def test_f16_specials_and_rounding(hip, oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = lambda v: v.mul(1.0009765625).add(0.00006103515625)   # forces re-rounding of every half
    got = hip.apply_fn(hip.buffer(bits.view(np.float16), "f16"), f).read().view(np.uint16)
    want = oracle.apply_fn(f, bits, dtype="f16")
    nan = np.isnan(want.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    assert np.isnan(got.view(np.float16)[nan]).all()


@pytest.mark.parametrize("off_in,off_out", [(0, 0), (1, 1), (3, 3), (1, 2), (0, 3), (2, 0)])
@pytest.mark.parametrize("n", [1, 2, 7, 1000, 8191, 70000])
def test_unaligned_views(hip, oracle, off_in, off_out, n):
    """Sub-ranges that are not 16-byte aligned: equal phase takes the vector path with a
    scalar head and tail, different phases take the scalar path; neighbours stay untouched."""
    total = n + 8
    x = synth.uniform_f32(81, total, -2, 2)
    xb = hip.buffer(x)
    outb = hip.buffer(np.full(total, 7.0, dtype=np.float32))
    f = lambda v: v.mul(3.0).sub(1.0)
    hip.apply_fn(xb.slice(off_in, off_in + n), f, out=outb.slice(off_out, off_out + n))
    got = outb.read()
    want = np.full(total, 7.0, dtype=np.float32)
    want[off_out:off_out + n] = oracle.apply_fn(f, x[off_in:off_in + n])
    assert_bits_equal(got, want)


def test_every_launch_shape_the_library_picks_gives_the_same_bits(oracle):
    """Large launches over views with a scalar head and tail, in every shape the library picks by itself:
    one-wavefront workgroups with one vector per thread (nothing of the launch before is revisited), 128
    threads x 2 vectors (the same launch again), alternating directions, directly and as a replayed
    recording; and a recorded chain that mostly writes (temporal loads, stores past the cache)."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        n = (12 << 20) + 7                           # 48 MiB per array and a ragged end
        x = synth.uniform_f32(83, n + 16, -2, 2)
        f = lambda v: v.mul(3.0).sub(1.0)
        xb, ob = dev.buffer(x), dev.alloc(n + 16)
        seen = set()
        for off in (0, 1, 3):                        # aligned; equal phase with a head; (same phase in and out)
            want = oracle.apply_fn(f, x[off:off + n])
            for repeat in range(3):
                ob.clear()
                dev.apply_fn(xb.slice(off, off + n), f, out=ob.slice(off, off + n))
                seen.add(dev.last_launch_shape()[0])
                assert_bits_equal(ob.slice(off, off + n).read(), want, f"offset {off}, launch {repeat}")
            dev.capture_begin()
            dev.apply_fn(xb.slice(off, off + n), f, out=ob.slice(off, off + n))
            g = dev.capture_end()
            for replay in range(3):
                ob.clear()                            # (a fill in between: the replay revisits nothing it wrote)
                g.launch()
                assert_bits_equal(ob.slice(off, off + n).read(), want, f"offset {off}, replay {replay}")
            g.destroy()
        assert seen == {1, 2}
        # 1 read + 3 writes, 192 MiB: the joined kernel of three recorded launches
        a, b, c = dev.alloc(n), dev.alloc(n), dev.alloc(n)
        g1, g2 = (lambda v: v.abs().sqrt()), (lambda v: v.neg().max(-1.0))
        dev.capture_begin()
        dev.apply_fn(xb.slice(0, n), f, out=a)
        dev.apply_fn(a, g1, out=b)
        dev.apply_fn(b, g2, out=c)
        g = dev.capture_end()
        assert (g.kernel_nodes, g.fused_launches) == (1, 2)
        assert dev.last_launch_shape()[1] == (2 | 64)           # stores non-temporal and written through, loads temporal
        for replay in range(2):
            g.launch()
            wa = oracle.apply_fn(f, x[:n])
            wb = oracle.apply_fn(g1, wa)
            assert_bits_equal(a.read(), wa)
            assert_bits_equal(b.read(), wb)
            assert_bits_equal(c.read(), oracle.apply_fn(g2, wb))
        g.destroy()
    finally:
        dev.close()


def test_f16_unaligned_views(hip, oracle):
    total = 5000
    xb = synth.uniform_f16_bits(5, total, -2, 2)
    buf = hip.buffer(xb.view(np.float16), "f16")
    out = hip.buffer(np.zeros(total, dtype=np.float16), "f16")
    f = lambda v: v.mul(2.0).add(0.5)
    for off, n in [(1, 4000), (3, 17), (8, 4992), (5, 1)]:
        out.clear()
        hip.apply_fn(buf.slice(off, off + n), f, out=out.slice(off, off + n))
        got = out.read().view(np.uint16)
        want = np.zeros(total, dtype=np.uint16)
        want[off:off + n] = oracle.apply_fn(f, xb[off:off + n], dtype="f16")
        assert_bits_equal(got, want)


def test_in_place_and_overlap(hip, oracle):
    n = 100000
    x = synth.uniform_f32(91, n, -2, 2)
    xb = hip.buffer(x)
    f = lambda v: v.mul(v).add(1.0)
    hip.apply_fn(xb, f, out=xb)  # exact alias is allowed
    assert_bits_equal(xb.read(), oracle.apply_fn(f, x))
    with pytest.raises(capi.CustosHipError) as e:
        hip.apply_fn(xb.slice(0, 1000), f, out=xb.slice(4, 1004))
    assert e.value.code == capi.ERR_BAD_OVERLAP


def test_four_operands(hip, oracle):
    n = 30011
    arrs = [synth.uniform_f32(100 + i, n, -2, 2) for i in range(4)]
    f = lambda a, b, c, d: a.mul(b).add(c).max(d).sub(a.min(d))
    got = hip.apply_fn_n([hip.buffer(v) for v in arrs], f).read()
    assert_bits_equal(got, oracle.apply_fn(f, *arrs))


def test_tuning_variants_agree(hip, oracle):
    n = 300007
    x = synth.uniform_f32(111, n, -2, 2)
    f = lambda v: v.mul(1.25).add(0.5).max(0.0)
    want = oracle.apply_fn(f, x)
    xb = hip.buffer(x)
    try:
        for block, unroll, bpc, nt in [(64, 1, 0, -1), (256, 4, 0, 1), (1024, 8, 0, 2), (256, 3, 2, 3), (512, 2, 1, 0)]:
            hip.set_tuning(block, unroll, bpc, nt)
            assert_bits_equal(hip.apply_fn(xb, f).read(), want, f"{block}x{unroll} bpc={bpc} nt={nt}")
    finally:
        hip.set_tuning()


def test_both_traversal_directions_and_all_shapes(hip, oracle):
    """Every launch shape the library can pick (vectors per thread x cache policy x direction)
    computes the same bits: views with heads and tails, a unary gradient, a persistent grid."""
    n = 100003
    x = synth.uniform_f32(7, n + 5, -2, 2)
    y = synth.uniform_f32(8, n + 5, 0.5, 2)
    f = lambda a, b: a.mul(b).add(0.25).max(0.0)
    d = lambda v: v.mul(2.0).add(1.0)
    xb, yb = hip.buffer(x), hip.buffer(y)
    try:
        for unroll in (1, 2, 3):
            for nt in (-1, 3):
                for bpc in (0, 1):
                    hip.set_tuning(0, unroll, bpc, nt, 2)          # every launch the other way round
                    for launch in range(2):                        # so: both directions
                        for off in (0, 1, 3):                      # aligned, and views with a scalar head
                            xs, ys = xb.slice(off, off + n), yb.slice(off, off + n)
                            got = hip.apply_fn2(xs, ys, f).read()
                            assert_bits_equal(got, oracle.apply_fn(f, x[off:off + n], y[off:off + n]),
                                              f"unroll={unroll} nt={nt} bpc={bpc} launch={launch} off={off}")
                        g0 = np.full(n, 0.5, dtype=np.float32)
                        gb = hip.buffer(g0)
                        hip.add_unary_grad(xb.slice(0, n), gb, yb.slice(0, n), d)
                        assert_bits_equal(gb.read(), oracle.add_unary_grad(d, x[:n], g0, y[:n]))
    finally:
        hip.set_tuning()


def test_launch_shape_follows_the_bytes_touched(hip):
    """One kernel per expression: the launch shape (vectors per thread, cache policy, direction) is
    an operand of every launch, so no launch of any size compiles anything after `expr_compile`
    has returned (the reference compiles once per text too: src/devices/cuda/kernel_cache.rs:39-61)."""
    src = "((x * 3.0) - 1.0)"
    k = hip.compile(capi.KIND_APPLY, "f32", src, ("x",))
    kg = hip.compile(capi.KIND_UNARY_GRAD, "f32", "(x * 2.0)", ("x",))
    identity = hip.alloc(16)
    hip.copy(identity, hip.alloc(16))             # the library's own copy kernel is compiled on first use
    c0, _ = hip.cache_stats()
    big = hip.alloc(1 << 29, zeroed=False)        # 2 GiB
    xs = synth.uniform_f32(21, 1 << 12, -1, 1)
    hip.write(big.slice(0, 1 << 12), xs)
    for log2n in range(10, 29, 3):                # 4 KiB ... 1 GiB per operand
        n = 1 << log2n
        src_buf, dst_buf = big.slice(0, n), big.slice(1 << 28, (1 << 28) + n)
        capi.check(hip.lib.custos_hip_apply_fn(hip.handle, k, src_buf.ptr, dst_buf.ptr, n), hip.handle)
        capi.check(hip.lib.custos_hip_add_unary_grad(hip.handle, kg, src_buf.ptr, dst_buf.ptr, src_buf.ptr, n), hip.handle)
        assert hip.kernel_name(k, n) == hip.kernel_name(k)
        hip.capture_begin()
        capi.check(hip.lib.custos_hip_apply_fn(hip.handle, k, src_buf.ptr, dst_buf.ptr, n), hip.handle)
        graph = hip.capture_end()
        graph.launch()
        hip.sync()
        graph.destroy()
        assert hip.cache_stats()[0] == c0, f"a launch over 2^{log2n} elements compiled something"
    want = xs * np.float32(3.0) - np.float32(1.0)
    assert_bits_equal(big.slice(1 << 28, (1 << 28) + (1 << 12)).read(), want)
    del big
    try:
        hip.set_tuning(0, 2, 0, 3, 1)
        pinned = hip.compile(capi.KIND_APPLY, "f32", src, ("x",))
        assert hip.kernel_name(pinned) != hip.kernel_name(k)     # vectors per thread pinned: another kernel
        assert "custos_tile1(" not in hip.kernel_source(pinned)
    finally:
        hip.set_tuning()
    # results do not depend on the variant: a 2^25-element launch (256 MiB touched) and its head
    n = 1 << 25
    xb = hip.alloc(n, zeroed=False)
    base = synth.uniform_f32(3, 1 << 16, -1, 1)
    hip.copy(xb.slice(0, 1 << 16), hip.buffer(base))
    filled = 1 << 16
    while filled < n:
        hip.copy(xb.slice(filled, 2 * filled), xb.slice(0, filled))
        filled *= 2
    want = (base * np.float32(3.0) - np.float32(1.0)).astype(np.float32)
    for launch in range(2):
        out = hip.apply_fn(xb, lambda v: v.mul(3.0).sub(1.0))
        for start in (0, n // 2, n - (1 << 16)):
            assert_bits_equal(out.slice(start, start + (1 << 16)).read(), want, f"launch {launch} window {start}")
    big_launch = hip.apply_fn(hip.alloc(1 << 27), lambda v: v.mul(3.0).sub(1.0))   # 1 GiB touched, zeros in
    assert np.all(big_launch.slice((1 << 27) - 4096, 1 << 27).read() == np.float32(-1.0))


def test_kernel_cache(hip):
    c0, h0 = hip.cache_stats()
    k1 = hip.compile(capi.KIND_APPLY, "f32", "tan(cos(((x * 41.0) + 0.125)))", ("x",))
    k2 = hip.compile(capi.KIND_APPLY, "f32", "tan(cos(((x*41) + 0.1250)))", ("x",))
    k3 = hip.compile(capi.KIND_APPLY, "f32", "tan(cos(((y * 41.0) + 0.125)))", ("y",))
    c1, h1 = hip.cache_stats()
    assert k1.value == k2.value == k3.value
    assert c1 - c0 == 1 and h1 - h0 == 2
    k4 = hip.compile(capi.KIND_UNARY_GRAD, "f32", "tan(cos(((x * 41.0) + 0.125)))", ("x",))
    assert k4.value != k1.value
    assert hip.kernel_name(k1).startswith("custos_apply_f32_") and hip.kernel_name(k1) in hip.kernel_source(k1)
    assert hip.kernel_name(k4).startswith("custos_unary_grad_f32_")


def test_literals_are_launch_parameters(hip, oracle):
    """The first set of literal values of an expression is compiled into the code; the second
    compiles the form that takes them as launch parameters, and every later set of values is a
    handle on that code (the reference compiles each distinct text,
    src/devices/cuda/kernel_cache.rs:45-61)."""
    rng = np.random.default_rng(77)
    x = rng.uniform(-3, 3, 100003).astype(np.float32)
    xb = hip.buffer(x)
    first = hip.compile(capi.KIND_APPLY, "f32", "max(cos(((x * 1.5) - 0.25)), -0.75)", ("x",))
    assert "CustosConsts" not in hip.kernel_source(first) and "0x1.8p+0f" in hip.kernel_source(first)
    c0, _ = hip.cache_stats()
    for step in range(40):
        a, b, c = np.float32(1.0 + step * 0.37), np.float32(step * 0.11 - 2.0), np.float32(-0.05 * step)
        f = lambda v: v.mul(float(a)).sub(float(b)).cos().max(float(c))
        out = hip.apply_fn(xb, f)
        assert ulp_distance_f32(out.read(), oracle.apply_fn(f, x)).max() <= 4, f"step {step}"
        exact = hip.apply_fn(xb, lambda v: v.mul(float(a)).sub(float(b)).max(float(c)))
        assert_bits_equal(exact.read(), np.maximum(x * a - b, c), f"exact step {step}")
    c1, _ = hip.cache_stats()
    # the shared form of the first expression; the second expression once for its first values, once shared
    assert c1 - c0 == 3
    k_a = hip.compile(capi.KIND_APPLY, "f32", "max(cos(((x * 2.5) - 0.25)), -0.75)", ("x",))
    k_b = hip.compile(capi.KIND_APPLY, "f32", "max(cos(((x*2.50) - 0.250)), -0.75)", ("x",))
    k_c = hip.compile(capi.KIND_APPLY, "f32", "max(cos(((x * 3.5) - 0.25)), -0.75)", ("x",))
    assert k_a.value == k_b.value and k_a.value != k_c.value            # same values: same handle
    assert hip.kernel_name(k_a) == hip.kernel_name(k_c) != hip.kernel_name(first)   # same code, other values
    assert hip.kernel_source(k_a) == hip.kernel_source(k_c) and "struct CustosConsts { C c[3]; };" in hip.kernel_source(k_a)
    again = hip.compile(capi.KIND_APPLY, "f32", "max(cos(((x * 1.5) - 0.25)), -0.75)", ("x",))
    assert again.value == first.value                                   # the first values keep their kernel
    assert hip.cache_stats()[0] == c1
    # the shared code and the one with the values compiled in give the same bits
    f15 = lambda v: v.mul(1.5).sub(0.25).cos().max(-0.75)
    in_code = hip.apply_fn(xb, f15).read()
    try:
        hip.set_literal_policy(capi.LITERALS_AS_PARAMETERS)
        as_parameters = hip.apply_fn(xb, f15).read()
        fresh = hip.compile(capi.KIND_APPLY, "f32", "tanh(((x * 1.25) + 7.0))", ("x",))
        assert "kc.c[1]" in hip.kernel_source(fresh)                    # shared form at once
        hip.set_literal_policy(capi.LITERALS_IN_CODE)
        before = hip.cache_stats()[0]
        for k in (1.0, 2.0, 3.0):
            got = hip.apply_fn(xb, lambda v: v.mul(k).add(k).abs().mul(k)).read()
            assert_bits_equal(got, np.abs(x * np.float32(k) + np.float32(k)) * np.float32(k), f"in code {k}")
        assert hip.cache_stats()[0] - before == 3                       # the reference's behaviour: one per text
    finally:
        hip.set_literal_policy(capi.LITERALS_ADAPTIVE)
    assert_bits_equal(as_parameters, in_code, "policy")
    # integer types, a two-operand expression, the gradient kind, special values
    xi = rng.integers(-1000, 1000, 5001).astype(np.int32)
    for k in (3, -7, 2**31 - 1, -2**31):
        got = hip.apply_fn(hip.buffer(xi, "i32"), lambda v: v.mul(k).add(k)).read()
        assert_bits_equal(got, (xi.astype(np.int64) * k + k).astype(np.int32), f"i32 {k}")
    xd = rng.uniform(-2, 2, 4099)
    for k in (0.1, 1e300, -0.0, float("inf")):
        got = hip.apply_fn(hip.buffer(xd, "f64"), lambda v: v.mul(k).min(k)).read()
        prod = xd * k
        assert_bits_equal(got, np.where(prod < k, prod, k), f"f64 {k}")
    y = rng.uniform(-1, 1, x.size).astype(np.float32)
    g = rng.uniform(-1, 1, x.size).astype(np.float32)
    for k in (0.5, 4.0):
        got = hip.apply_fn2(xb, hip.buffer(y), lambda l, r: l.mul(k).add(r.mul(k + 1))).read()
        assert_bits_equal(got, x * np.float32(k) + y * np.float32(k + 1), f"two operands {k}")
        lhs_grad = hip.buffer(g)
        hip.add_unary_grad(xb, lhs_grad, hip.buffer(y), lambda v: v.mul(k))
        assert_bits_equal(lhs_grad.read(), g + y * (x * np.float32(k)), f"gradient {k}")


def test_launch_shapes_of_shared_code(hip):
    """A launch large enough for another launch shape runs the same code: one compilation per form
    (values in the code, values as parameters), not one per shape or per set of literal values --
    launched directly and from a recorded graph."""
    n = 1 << 23                                   # 32 MiB per array: the 64 MiB launch takes non-temporal accesses
    rng = np.random.default_rng(5)
    x = rng.uniform(-8, 8, n).astype(np.float32)
    xb, out = hip.buffer(x), hip.alloc(n)
    c0, _ = hip.cache_stats()
    names = set()
    for step, (a, b) in enumerate([(1.25, 0.5), (2.5, 0.75), (3.75, 1.0), (5.0, 1.25), (6.25, 1.5)]):
        src = f"min(((x * {a}) - {b}), (x * {b}))"
        k = hip.compile(capi.KIND_APPLY, "f32", src, ("x",))
        names.add(hip.kernel_name(k, n))
        want = np.minimum(x * np.float32(a) - np.float32(b), x * np.float32(b))
        capi.check(hip.lib.custos_hip_apply_fn(hip.handle, k, xb.ptr, out.ptr, n), hip.handle)
        assert_bits_equal(out.read(), want, f"direct {step}")
        out.clear()
        hip.capture_begin()
        capi.check(hip.lib.custos_hip_apply_fn(hip.handle, k, xb.ptr, out.ptr, n), hip.handle)
        graph = hip.capture_end()
        for _ in range(3):
            graph.launch()
        assert_bits_equal(out.read(), want, f"graph {step}")
        graph.destroy()
    c1, _ = hip.cache_stats()
    assert c1 - c0 == 2 and len(names) == 2


def test_error_paths(hip):
    with pytest.raises(capi.CustosHipError) as e:
        hip.alloc(0)
    assert e.value.code == capi.ERR_ZERO_LENGTH_BUFFER          # src/devices/cuda/api/cuda.rs:69-71
    import custos_amd
    with pytest.raises(capi.CustosHipError) as e:
        custos_amd.HIP(1000)
    assert e.value.code == capi.ERR_INVALID_DEVICE_INDEX        # src/devices/cuda/api/cuda.rs:36-39
    k_apply = hip.compile(capi.KIND_APPLY, "f32", "(x + 1.0)", ("x",))
    k_grad = hip.compile(capi.KIND_UNARY_GRAD, "f32", "(x + 1.0)", ("x",))
    b = hip.alloc(16)
    rc = hip.lib.custos_hip_add_unary_grad(hip.handle, k_apply, b.ptr, b.ptr, b.ptr, 16)
    assert rc == capi.ERR_KIND_MISMATCH
    rc = hip.lib.custos_hip_apply_fn(hip.handle, k_grad, b.ptr, b.ptr, 16)
    assert rc == capi.ERR_KIND_MISMATCH
    k2 = hip.compile(capi.KIND_APPLY, "f32", "(x + y)", ("x", "y"))
    rc = hip.lib.custos_hip_apply_fn(hip.handle, k2, b.ptr, b.ptr, 16)
    assert rc == capi.ERR_ARITY_MISMATCH
    rc = hip.lib.custos_hip_apply_fn(hip.handle, k_apply, 0, b.ptr, 16)
    assert rc == capi.ERR_INVALID_ARGUMENT
    rc = hip.lib.custos_hip_apply_fn(hip.handle, k_apply, b.ptr + 2, b.ptr, 4)
    assert rc == capi.ERR_INVALID_ARGUMENT                       # not aligned to the element size
    assert hip.lib.custos_hip_apply_fn(hip.handle, k_apply, b.ptr, b.ptr, 0) == 0   # empty input is a no-op
    with pytest.raises(capi.CustosHipError):
        hip.compile(capi.KIND_APPLY, "f32", "(x +", ("x",))
    # the device is still usable after errors
    assert hip.apply_fn(hip.buffer([1.0, 2.0]), lambda v: v.add(1.0)).read().tolist() == [2.0, 3.0]


def test_alloc_is_zeroed_and_clear_write_copy(hip):
    for n in (1, 5, 1000, 100003):
        assert not hip.alloc(n).read().any()
        assert not hip.alloc(n, "u8").read().any()
    x = synth.uniform_f32(5, 1001, 1, 2)
    b = hip.buffer(x)
    c = hip.alloc(1001)
    hip.copy(c, b)
    assert_bits_equal(c.read(), x)
    v = b.slice(3, 990)
    v.clear()
    want = x.copy()
    want[3:990] = 0
    assert_bits_equal(b.read(), want)                            # neighbours of a cleared view stay
    b.write(np.arange(1001, dtype=np.float32))
    assert b.read()[1000] == 1000.0
    u = hip.buffer([1, 2, 3, 4, 5, 6], "u32")                    # src/devices/cuda/ops.rs:242-247
    u.clear()
    assert u.read().tolist() == [0] * 6


@pytest.mark.parametrize("dtype,value", [("f32", 1.0), ("f32", -0.0), ("f64", 0.1), ("i32", -7), ("u8", 200), ("i16", -300),
                                         ("u64", 2**63 + 5), ("f16", 1.0), ("f32", 0.0)])
def test_fill_sets_every_element_and_nothing_else(hip, dtype, value):
    """custos_hip_fill over views of every offset phase and length class: the bytes at the unaligned
    edges, the 16-byte body and the neighbours of the view."""
    np_type = np.dtype(capi.DTYPES[dtype][1])
    item = np_type.itemsize
    n = 5000
    rng = np.random.default_rng(3)
    background = rng.integers(0, 256, n * item, dtype=np.uint8).view(np_type)
    for lo, length in ((0, n), (1, n - 2), (3, 1), (5, 16 // item + 1), (7, 1000), (2, 0), (16 // item, 333)):
        buf = hip.buffer(background, dtype)
        hip.fill(buf.slice(lo, lo + length), value)
        want = background.copy()
        want[lo:lo + length] = np.asarray(value, dtype=np_type)
        assert_bits_equal(buf.read().view(np.uint8), want.view(np.uint8), f"{dtype} fill of [{lo}, {lo + length})")


def test_short_reads_at_every_phase_and_length(hip):
    """Reads of up to 64 KiB are staged through pinned memory by the identity kernel; longer ones and
    reads while recording go through the runtime's copy.  Same bytes at every offset phase, for
    byte-granular and word-granular lengths, on both sides of the limit."""
    n = (64 << 10) + 4096
    data = np.random.default_rng(9).integers(0, 256, n, dtype=np.uint8)
    buf = hip.buffer(data, "u8")
    for lo in (0, 1, 3, 4, 13, 16, 4095):
        for length in (1, 2, 3, 4, 15, 16, 17, 1000, 4096, (64 << 10) - 1, 64 << 10, (64 << 10) + 1):
            got = buf.slice(lo, lo + length).read()
            assert_bits_equal(got, data[lo:lo + length], f"read of [{lo}, {lo + length})")
    words = hip.buffer(np.arange(5000, dtype=np.uint32), "u32")
    hip.apply_fn(words, lambda v: v.add(1), out=words)                 # a read waits for the work before it
    assert words.slice(7, 4000).read().tolist() == list(range(8, 4001))
    hip.capture_begin()
    try:
        assert_bits_equal(buf.slice(5, 300).read(), data[5:300], "read while recording")
    finally:
        hip.capture_end().destroy()


def test_short_writes_in_a_row_keep_their_own_data(hip):
    """Writes of up to 64 KiB go through a ring of 16 pinned staging slots without a wait; the host
    array may change right after the call, and more writes in a row than there are slots must not
    overwrite data a launch has still to read."""
    rng = np.random.default_rng(10)
    n = (64 << 10) + 64
    target = hip.alloc(n * 40, "u8")
    want = np.zeros(n * 40, np.uint8)
    scratch = np.empty(n, np.uint8)
    lengths = [1, 3, 4, 16, 17, 1000, 4096, (64 << 10) - 1, 64 << 10, (64 << 10) + 1]
    for i in range(40):                                    # no read, no sync in between
        length = lengths[i % len(lengths)]
        lo = i * n + int(rng.integers(0, 32))
        scratch[:length] = rng.integers(0, 256, length, dtype=np.uint8)
        want[lo:lo + length] = scratch[:length]
        target.slice(lo, lo + length).write(scratch[:length])
        scratch[:length] = 0xEE                            # the caller reuses its array at once
    assert_bits_equal(target.read(), want)
    # stream order: a write, a kernel on what was written, a write over the kernel's input
    a, b = hip.alloc(1000), hip.alloc(1000)
    for step in range(20):
        a.write(np.full(1000, float(step), np.float32))
        hip.apply_fn(a, lambda v: v.add(0.5), out=b)
        a.write(np.full(1000, -1.0, np.float32))
        assert b.read()[::333].tolist() == [step + 0.5] * 4
        assert a.read()[0] == -1.0


def test_fill_is_recorded_like_a_clear(hip):
    n = 3001
    a, b = hip.alloc(n), hip.alloc(n)
    hip.capture_begin()
    hip.fill(a, 2.5)
    hip.apply_fn(a, lambda v: v.mul(2.0), out=b)
    hip.fill(a, -1.0)
    g = hip.capture_end()
    assert not a.read().any(), "nothing may run while recording"
    for _ in range(2):
        g.launch()
        hip.sync()
        assert_bits_equal(b.read(), np.full(n, 5.0, np.float32))
        assert_bits_equal(a.read(), np.full(n, -1.0, np.float32))
        b.clear()
    g.destroy()


def test_fill_rejects_what_it_cannot_do(hip):
    buf = hip.alloc(64, "u8")
    value = (C.c_ubyte * 16)(*range(16))
    for ptr, nbytes, size in ((buf.ptr + 1, 8, 4), (buf.ptr, 6, 4), (buf.ptr, 12, 3), (buf.ptr, 32, 32), (buf.ptr, 8, 0)):
        rc = hip.lib.custos_hip_fill(hip.handle, ptr, nbytes, value, size)
        assert rc == capi.ERR_INVALID_ARGUMENT, (ptr - buf.ptr, nbytes, size)
    assert hip.lib.custos_hip_fill(hip.handle, buf.ptr, 32, value, 16) == 0          # a 16-byte value
    assert buf.read()[:32].tolist() == list(range(16)) * 2


RELU_SRC = """extern "C" __global__ void relu(float* lhs, float* out, int numElements) {
    int idx = blockDim.x * blockIdx.x + threadIdx.x;
    if (idx < numElements) out[idx] = max(lhs[idx], 0.0f);
}
"""
ADD_SRC = """extern "C" __global__ void add(float* lhs, float* rhs, float* out, int numElements) {
    int idx = blockDim.x * blockIdx.x + threadIdx.x;
    if (idx < numElements) out[idx] = lhs[idx] + rhs[idx];
}
"""


def test_caller_written_kernels(hip):
    """`launch_kernel1d` with user source: the add / relu ops of tests/graph/mod.rs:90-127."""
    n = 100003
    a = synth.uniform_f32(1, n, -2, 2)
    b = synth.uniform_f32(2, n, -2, 2)
    ab, bb, cb, db = hip.buffer(a), hip.buffer(b), hip.alloc(n), hip.alloc(n)
    c0, h0 = hip.cache_stats()
    hip.launch_kernel1d(n, ADD_SRC, "add", [ab, bb, cb, n])
    hip.launch_kernel1d(n, RELU_SRC, "relu", [cb, db, n])
    hip.launch_kernel1d(n, ADD_SRC, "add", [db, ab, cb, n])       # cached: same source and name
    c1, h1 = hip.cache_stats()
    assert (c1 - c0, h1 - h0) == (2, 1)
    want = np.maximum(a + b, np.float32(0)) + a
    assert_bits_equal(cb.read(), want.astype(np.float32))
    hip.launch_kernel(ADD_SRC, "add", (4, 1, 1), (256, 1, 1), 0, [ab, bb, db, 1000])
    got = db.read()
    assert_bits_equal(got[:1000], (a + b)[:1000])
    assert_bits_equal(got[1000:], np.maximum(a + b, np.float32(0))[1000:])
    # errors: bad source, wrong entry point for the kernel kind
    with pytest.raises(capi.CustosHipError) as e:
        hip.compile_source("this is not HIP", "nope")
    assert e.value.code == capi.ERR_COMPILE
    k = hip.compile_source(ADD_SRC, "add")
    assert hip.lib.custos_hip_apply_fn(hip.handle, k, ab.ptr, cb.ptr, 10) == capi.ERR_KIND_MISMATCH


def test_caller_written_kernels_in_a_graph_are_fences(hip, oracle):
    """A recorded user kernel has unknown memory use: everything before it runs first,
    everything after it runs later, while the expression kernels around it still merge."""
    n = 4096
    xs = [synth.uniform_f32(10 + i, n, -2, 2) for i in range(8)]
    bufs = [hip.buffer(x) for x in xs]
    mids = [hip.alloc(n) for _ in xs]
    outs = [hip.alloc(n) for _ in xs]
    f = lambda v: v.mul(2.0)
    hip.capture_begin()
    for b, m in zip(bufs, mids):
        hip.apply_fn(b, f, out=m)
    hip.launch_kernel1d(n, RELU_SRC, "relu", [mids[0], outs[0], n])      # fence
    for m, o in zip(mids[1:], outs[1:]):
        hip.apply_fn(m, f, out=o)
    g = hip.capture_end()
    assert g.stats() == (8 + 1 + 7, 3, 3)
    g.launch()
    hip.sync()
    assert_bits_equal(outs[0].read(), np.maximum(xs[0] * np.float32(2), np.float32(0)))
    for x, o in zip(xs[1:], outs[1:]):
        assert_bits_equal(o.read(), (x * np.float32(4)).astype(np.float32))


def test_disk_cache_of_code_objects(tmp_path, monkeypatch, oracle):
    """CUSTOS_HIP_KERNEL_CACHE_DIR: a second device loads the code object instead of compiling, and
    what the loaded code computes is what the CPU oracle computes."""
    import custos_amd
    monkeypatch.setenv("CUSTOS_HIP_KERNEL_CACHE_DIR", str(tmp_path / "kcache"))
    x = synth.uniform_f32(5, 1000, -1, 1)
    f = lambda v: v.mul(0.37).add(11.5)
    want = oracle.apply_fn(f, x)
    first = custos_amd.HIP(0)
    assert_bits_equal(first.apply_fn(first.buffer(x), f).read(), want)
    assert first.cache_stats()[0] == 1 and first.disk_cache_hits() == 0
    files = list((tmp_path / "kcache").iterdir())
    assert len(files) == 1 and files[0].suffix == ".co" and "gfx950" in files[0].name
    first.close()
    second = custos_amd.HIP(0)
    got = second.apply_fn(second.buffer(x), f).read()
    assert second.cache_stats()[0] == 0 and second.disk_cache_hits() == 1
    assert_bits_equal(got, want)
    # a damaged file is ignored and replaced
    files[0].write_bytes(b"garbage")
    third = custos_amd.HIP(0)
    assert_bits_equal(third.apply_fn(third.buffer(x), f).read(), want)
    assert third.cache_stats()[0] == 1 and third.disk_cache_hits() == 0
    second.close()
    third.close()


def test_more_than_2p32_bytes_and_elements(hip):
    """64-bit indexing: a u8 buffer of 2^32 + 77 elements (more than 4 GiB in, 4 GiB out)."""
    n = (1 << 32) + 77
    src = hip.alloc(n, "u8", zeroed=False)
    pattern = (np.arange(1 << 20, dtype=np.uint32) * 7 + 3).astype(np.uint8)
    hip.write(src.slice(0, 1 << 20), pattern)
    filled = 1 << 20
    while filled < n:                                   # replicate on the device by doubling copies
        step = min(filled, n - filled)
        hip.copy(src.slice(filled, filled + step), src.slice(0, step))
        filled += step
    out = hip.apply_fn(src, lambda v: v.mul(3).add(1))
    want = (pattern.astype(np.uint32) * 3 + 1).astype(np.uint8)
    for start in (0, (1 << 31) - (1 << 19), (1 << 32) - (1 << 20), n - (1 << 20)):
        off = start % (1 << 20)
        got = out.slice(start, start + (1 << 20)).read()
        assert_bits_equal(got, np.roll(want, -off), f"window at {start}")
    tail = out.slice(n - 77, n).read()
    assert_bits_equal(tail, np.roll(want, -((n - 77) % (1 << 20)))[:77])


@pytest.mark.parametrize("dtype", ["f32", "f64", "f16", "f16_pernode", "bf16"])
def test_min_max_of_zeros_return_the_second_operand(hip, oracle, dtype):
    """`Number::min` / `max` are selects (src/number.rs:201-209): for two zeros of different sign
    they return the second operand, where the hardware's min / max return -0 / +0.  The compiler
    swaps the select for the instruction when it can rule NaNs out: a literal operand, operands
    that are comparison results."""
    n = 4099
    base = dtype.split("_")[0]
    if base == "f16":
        xb = synth.uniform_f16_bits(41, n, -3, 3)
        xb[3::5], xb[4::5] = 0x8000, 0x0000
        view = lambda a: a.view(np.float16)
    elif base == "bf16":
        xb = (synth.uniform_f32(41, n, -3, 3).view(np.uint32) >> 16).astype(np.uint16)
        xb[3::5], xb[4::5] = 0x8000, 0x0000
        view = lambda a: a
    else:
        xb = synth.uniform_f32(41, n, -3, 3).astype(np.float32 if dtype == "f32" else np.float64)
        xb[3::5], xb[4::5] = -0.0, 0.0
        view = lambda a: a
    x = hip.buffer(view(xb), dtype)
    cases = (("min(x, 0)", lambda v: v.min(0.0)), ("max(x, 0)", lambda v: v.max(0.0)),
             ("min(x, -0)", lambda v: v.min(-0.0)), ("max(x, -0)", lambda v: v.max(-0.0)),
             ("min(0, x)", lambda v: v.val(0.0).min(v)), ("max(0, x)", lambda v: v.val(0.0).max(v)),
             ("min(-0, x)", lambda v: v.val(-0.0).min(v)), ("max(-0, x)", lambda v: v.val(-0.0).max(v)),
             ("min(x, x >= 9)", lambda v: v.min(v.geq(9.0))), ("max(x >= 9, -(x >= 9))", lambda v: v.geq(9.0).max(v.geq(9.0).neg())),
             ("min(-(x >= 9), x >= 9)", lambda v: v.geq(9.0).neg().min(v.geq(9.0))), ("max(x, x * 0)", lambda v: v.max(v.mul(0.0))),
             ("min(|x|, -(|x| * 0))", lambda v: v.abs().min(v.abs().mul(0.0).neg())))
    for name, f in cases:
        got = hip.apply_fn(x, f).read()
        want = oracle.apply_fn(f, xb, dtype=dtype)
        assert_bits_equal(got.view(np.uint16) if base in ("f16", "bf16") else got, want, f"{dtype}: {name}")


@pytest.mark.parametrize("dtype", ["f16", "f16_pernode", "bf16", "bf16_pernode", "f32"])
def test_products_keep_the_sign_of_zero(hip, oracle, dtype):
    """0 * negative = -0, also where the product is rounded to a 16-bit type next: a compiler
    that folds product and rounding into one fused multiply-add with a +0 addend loses the
    sign.  Vector body, partial tile and scalar tail (n is not a multiple of the vector)."""
    n = 4099
    base = dtype.split("_")[0]
    if base == "f16":
        xb = synth.uniform_f16_bits(31, n, -3, 3)
        xb[5::7] = 0x8000
        view = lambda a: a.view(np.float16)
    elif base == "bf16":
        xb = (synth.uniform_f32(31, n, -3, 3).view(np.uint32) >> 16).astype(np.uint16)
        xb[5::7] = 0x8000
        view = lambda a: a
    else:
        xb = synth.uniform_f32(31, n, -3, 3)
        xb[5::7] = -0.0
        view = lambda a: a
    x = hip.buffer(view(xb), dtype)
    for name, f in (("x * 0", lambda v: v.mul(0.0)), ("(x >= 9) * (x + x)", lambda v: v.geq(9.0).mul(v.add(v))),
                    ("-(x * 0)", lambda v: v.mul(0.0).neg()), ("(x * 0) * 5", lambda v: v.mul(0.0).mul(5.0)),
                    ("x * (x - x)", lambda v: v.mul(v.sub(v)))):
        got = hip.apply_fn(x, f).read()
        want = oracle.apply_fn(f, xb, dtype=dtype)
        if base != "f32":
            got = got.view(np.uint16)
        assert_bits_equal(got, want, f"{dtype}: {name}")
        bits = got.view(np.uint32) if base == "f32" else got
        assert ((bits << 1) == 0).all() and (bits != 0).any() and (bits == 0).any(), name   # zeros of both signs
    g0 = xb.copy()
    gb = hip.buffer(view(g0), dtype)
    hip.add_unary_grad(x, gb, x, lambda v: v.mul(0.0))          # g + x * (x * 0)
    got = gb.read()
    assert_bits_equal(got.view(np.uint16) if base != "f32" else got,
                      oracle.add_unary_grad(lambda v: v.mul(0.0), xb, g0, xb, dtype=dtype), f"{dtype}: gradient")


@pytest.mark.parametrize("dtype", ["f16_pernode", "bf16_pernode"])
def test_per_node_rounding_of_16bit_floats(hip, oracle, dtype):
    """Every node rounded to the storage type, what the reference's `half` arithmetic does
    (src/number.rs:487-676).  + - * / sqrt of 16-bit operands computed in f32 and rounded once
    are the correctly rounded 16-bit results, so these chains are bit-exact against the CPU
    restatement; they differ from the f32-compute mode, which rounds only at the store."""
    n = 50003
    base = dtype.split("_")[0]
    if base == "f16":
        xb = synth.uniform_f16_bits(21, n, -3, 3)
        yb = synth.uniform_f16_bits(22, n, 0.5, 2)
    else:
        xb = (synth.uniform_f32(21, n, -3, 3).view(np.uint32) >> 16).astype(np.uint16)
        yb = (synth.uniform_f32(22, n, 0.5, 2).view(np.uint32) >> 16).astype(np.uint16)
    view = (lambda a: a.view(np.float16)) if base == "f16" else (lambda a: a)
    f = lambda a, b: a.mul(0.3).add(b).mul(a).div(b.add(1.7)).sub(0.1).abs().sqrt().max(0.25).neg()
    x, y = hip.buffer(view(xb), dtype), hip.buffer(view(yb), dtype)
    got = hip.apply_fn2(x, y, f).read().view(np.uint16)
    assert_bits_equal(got, oracle.apply_fn(f, xb, yb, dtype=dtype))
    once = hip.apply_fn2(hip.buffer(view(xb), base), hip.buffer(view(yb), base), f).read().view(np.uint16)
    assert (once != got).mean() > 0.01          # the two modes really differ
    assert_bits_equal(once, oracle.apply_fn(f, xb, yb, dtype=base))

    # gradient: the product is rounded too, then the sum
    d = lambda v: v.mul(v).mul(3.0).add(0.7)
    g0 = (yb ^ 0x8000).astype(np.uint16)
    gb = hip.buffer(view(g0), dtype)
    hip.add_unary_grad(x, gb, y, d)
    assert_bits_equal(gb.read().view(np.uint16), oracle.add_unary_grad(d, xb, g0, yb, dtype=dtype))

    # transcendentals: f32 routine then one rounding; within one unit of the 16-bit type
    t = lambda v: v.sin().mul(v.mul(0.25).exp()).add(v.tanh())
    got = hip.apply_fn(x, t).read().view(np.uint16)
    want = oracle.apply_fn(t, xb, dtype=dtype)
    if base == "f16":
        dist = ulp_distance_f16(got, want)
    else:
        key = lambda b: np.where(b & 0x8000, 0x8000 - (b & 0x7fff).astype(np.int32), 0x8000 + (b & 0x7fff).astype(np.int32))
        dist = np.abs(key(got) - key(want))
    # a chain of three rounded nodes: one unit of disagreement in a node can move the result
    assert dist.max() <= 2 and (dist == 0).mean() > 0.98


def _random_tree(rng, leaves, depth, integer, unsigned=False):
    """A random expression over `leaves` built from the nodes whose results are exact."""
    if depth == 0 or rng.random() < 0.15:
        if rng.random() < 0.25:
            if integer:
                return leaves[0].val(int(rng.integers(0 if unsigned else -5, 6)))
            return leaves[0].val(float(np.float32(rng.uniform(-4, 4))))
        return leaves[int(rng.integers(len(leaves)))]
    a = _random_tree(rng, leaves, depth - 1, integer, unsigned)
    # (`abs` needs `Float` in the reference's CPU evaluation, src/two_way_ops/ops/unary.rs:246)
    ops1 = ["neg", "identity"] + ([] if integer else ["abs", "sqrtabs"])
    ops2 = ["add", "sub", "mul", "min", "max", "geq", "leq", "eq"] + ([] if integer else ["div"])
    if rng.random() < 0.25:
        op = ops1[int(rng.integers(len(ops1)))]
        return a.abs().sqrt() if op == "sqrtabs" else getattr(a, op)()
    b = _random_tree(rng, leaves, depth - 1, integer, unsigned)
    return getattr(a, ops2[int(rng.integers(len(ops2)))])(b)


_INT_RANGES = {"i8": (-128, 128), "u8": (0, 256), "i16": (-32768, 32768), "u16": (0, 60000), "i32": (-70000, 70000),
               "u32": (0, 1 << 32), "i64": (-(1 << 40), 1 << 40), "u64": (0, 1 << 63)}


def _random_tree_cases(dtype, trials):
    """(trial, build, tree, input arrays) of the random-tree test for one element type."""
    from custos_amd.expr import Resolve
    rng = np.random.default_rng(sum(map(ord, dtype)))
    integer = dtype[0] in "iu"
    n = 4099
    for trial in range(trials):
        k = int(rng.integers(1, 5))
        seed = int(rng.integers(1 << 30))
        build = lambda *leaves, seed=seed: _random_tree(np.random.default_rng(seed), list(leaves), 4, integer, dtype[0] == "u")
        tree = build(*[Resolve(nm, i) for i, nm in enumerate(("a", "b", "c", "d")[:k])])
        if isinstance(tree, (Const, Resolve)):
            continue
        if dtype.startswith("f16"):
            arrs = [synth.uniform_f16_bits(200 + trial * 4 + i, n, -3, 3) for i in range(k)]
            arrs[0][:8] = [0x0000, 0x8000, 0x7c00, 0xfc00, 0x7e00, 0x0001, 0x8001, 0x7bff]
        elif dtype.startswith("bf16"):
            arrs = [(synth.uniform_f32(200 + trial * 4 + i, n, -3, 3).view(np.uint32) >> 16).astype(np.uint16) for i in range(k)]
            arrs[0][:8] = [0x0000, 0x8000, 0x7f80, 0xff80, 0x7fc0, 0x0001, 0x8001, 0x7f7f]
        elif integer:
            lo, hi = _INT_RANGES[dtype]
            npdt = np.dtype(capi.DTYPES[dtype][1])
            arrs = [rng.integers(lo, hi, size=n, dtype=np.uint64 if dtype == "u64" else np.int64).astype(npdt) for _ in range(k)]
        else:
            npdt = np.dtype(capi.DTYPES[dtype][1])
            arrs = [synth.uniform_f32(200 + trial * 4 + i, n, -3, 3).astype(npdt) for i in range(k)]
            arrs[0][:SPECIALS.size] = SPECIALS.astype(npdt)
        yield trial, build, tree, arrs


@pytest.mark.parametrize("dtype", ["f32", "f64", "i32", "u16", "f16_pernode", "f16", "bf16", "bf16_pernode",
                                   "i8", "u8", "i16", "i64", "u32", "u64"])
def test_random_expression_trees_are_bit_exact(hip, oracle, dtype):
    """Random trees of up to 31 nodes over one to four operands, built from the nodes whose
    results are exact: parser, operand order, literal typing and emitted code against the CPU
    restatement evaluating the same tree, bit for bit (NaNs compare as NaN); and with the
    literals compiled in against the literals as launch parameters."""
    import os
    half = dtype.split("_")[0] in ("f16", "bf16")
    for trial, build, tree, arrs in _random_tree_cases(dtype, int(os.environ.get("CUSTOS_RANDOM_TREES", "10"))):
        bufs = [hip.buffer(a.view(np.float16) if dtype.startswith("f16") else a, dtype) for a in arrs]
        got = hip.apply_fn_n(bufs, build).read()
        want = oracle.apply_fn(build, *arrs, dtype=dtype)
        what = f"trial {trial}: {tree.to_cl_source(dtype)}"
        # the form that takes the literals as launch parameters gives the same bits
        hip.set_literal_policy(capi.LITERALS_AS_PARAMETERS)
        try:
            shared = hip.apply_fn_n(bufs, build).read()
        finally:
            hip.set_literal_policy(capi.LITERALS_ADAPTIVE)
        assert shared.view(np.uint8).tobytes() == got.view(np.uint8).tobytes(), f"literal parameters, {what}"
        if half:
            got = got.view(np.uint16)
            if dtype.startswith("f16"):
                nan = lambda b: (b & 0x7fff) > 0x7c00
            else:
                nan = lambda b: (b & 0x7fff) > 0x7f80
            same = (got == want) | (nan(got) & nan(want))
            assert same.all(), f"{what} differs at {np.flatnonzero(~same)[:5]}"
        else:
            nan = None
            assert_bits_equal(got, want, what)
        if len(arrs) == 1:
            # the same tree as the derivative of a unary gradient: g + o * f(x), the buffer's own
            # values rotated serve as g and o
            g0, o = np.roll(arrs[0], 1), np.roll(arrs[0], 2)
            as_buf = lambda a: hip.buffer(a.view(np.float16) if dtype.startswith("f16") else a, dtype)
            gb = as_buf(g0)
            hip.add_unary_grad(bufs[0], gb, as_buf(o), build)
            got_g = gb.read()
            want_g = oracle.add_unary_grad(build, arrs[0], g0, o, dtype=dtype)
            if half:
                got_g = got_g.view(np.uint16)
                same = (got_g == want_g) | (nan(got_g) & nan(want_g))
                assert same.all(), f"gradient, {what} differs at {np.flatnonzero(~same)[:5]}"
            else:
                assert_bits_equal(got_g, want_g, f"gradient, {what}")


def test_launch_shape_follows_the_launches_around_it(oracle):
    """A launch of 64 MiB and more that reads what one of the last launches wrote is part of a
    chain: temporal accesses while the chain's working set stays in the 256 MiB memory-side cache,
    loads past the caches and stores written through beyond that.  Results are the same either way."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        n = 1 << 23                                   # 32 MiB per array
        x = synth.uniform_f32(3, n, -2, 2)
        f = lambda v: v.mul(1.5).sub(0.25)
        g = lambda v: v.abs().add(1.0)
        a, b, c = dev.buffer(x), dev.alloc(n), dev.alloc(n)
        base = dev.launch_hint_stats()
        dev.apply_fn(a, f, out=b)                     # reads what no launch wrote
        dev.apply_fn(b, g, out=c)                     # consumer after producer, 96 MiB in all
        dev.apply_fn(c, f, out=b)
        s1 = dev.launch_hint_stats()
        assert (s1[0] - base[0], s1[1] - base[1], s1[2] - base[2]) == (1, 2, 0)
        want = (np.abs(x * np.float32(1.5) - np.float32(0.25)) + np.float32(1.0)) * np.float32(1.5) - np.float32(0.25)
        assert_bits_equal(b.read(), want)
        # the same chain over arrays that do not fit: 3 x 128 MiB
        big = 1 << 25
        xb = synth.uniform_f32(4, big, -2, 2)
        p, q, r = dev.buffer(xb), dev.alloc(big), dev.alloc(big)
        dev.apply_fn(p, f, out=q)
        dev.apply_fn(q, g, out=r)
        dev.apply_fn(r, f, out=q)
        s2 = dev.launch_hint_stats()
        assert (s2[0] - s1[0], s2[1] - s1[1], s2[2] - s1[2]) == (1, 0, 2)
        wantb = (np.abs(xb * np.float32(1.5) - np.float32(0.25)) + np.float32(1.0)) * np.float32(1.5) - np.float32(0.25)
        assert_bits_equal(q.read(), wantb)
        # a streaming chain whose kernels all read one more array
        w = dev.buffer(synth.uniform_f32(5, big, 0.5, 1.5))
        mul = lambda u, v: u.mul(v)
        for _ in range(2):
            dev.apply_fn2(q, w, mul, out=r)
            dev.apply_fn2(r, w, mul, out=q)
        s2b = dev.launch_hint_stats()
        assert s2b[2] - s2[2] == 4
        wb = synth.uniform_f32(5, big, 0.5, 1.5)
        assert_bits_equal(q.read(), ((((wantb * wb) * wb) * wb) * wb))
        s2 = s2b
        # in a recorded graph the first kernel counts as part of the chain too: a later level reads its output
        dev.set_graph_fusing(False)          # (joined, the two launches would be one node)
        dev.capture_begin()
        dev.apply_fn(a, f, out=b)
        dev.apply_fn(b, g, out=c)
        graph = dev.capture_end()
        s3 = dev.launch_hint_stats()
        assert (s3[0] - s2[0], s3[1] - s2[1], s3[2] - s2[2]) == (0, 2, 0)
        for _ in range(3):
            graph.launch()
        assert_bits_equal(c.read(), np.abs(x * np.float32(1.5) - np.float32(0.25)) + np.float32(1.0))
        graph.destroy()
    finally:
        dev.close()


def test_temporal_accesses_while_the_working_set_fits_the_l2s(oracle):
    """A launch of up to 32 MiB keeps temporal accesses only while it and the launches before it touch no
    more than 32 MiB together (the eight L2s); after launches that do not leave the L2s to it, it streams
    like a larger one.  Directly issued launches and the nodes of a graph."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        loads = 1 | 64
        n = 3 << 20                                   # 12 MiB per array
        x = synth.uniform_f32(11, n, -2, 2)
        f = lambda v: v.mul(1.5).sub(0.25)
        a, b, c, d = dev.buffer(x), dev.alloc(n), dev.alloc(n), dev.alloc(n)
        dev.apply_fn(a, f, out=b)                     # 24 MiB, nothing before it
        assert dev.last_launch_shape() == (2, 0, False)
        dev.apply_fn(a, f, out=b)                     # the same 24 MiB again
        assert dev.last_launch_shape() == (2, 0, False)
        dev.apply_fn(b, f, out=c)                     # 36 MiB with the launches before
        assert dev.last_launch_shape() == (2, loads, False)
        dev.apply_fn(c, f, out=d)
        assert dev.last_launch_shape() == (2, loads, False)
        want = x
        for _ in range(3):
            want = want * np.float32(1.5) - np.float32(0.25)
        assert_bits_equal(d.read(), want)
        small = dev.buffer(x[: 1 << 20])              # 8 MiB and less: not tracked, temporal
        dev.apply_fn(small, f)
        assert dev.last_launch_shape() == (2, 0, False)
        # the window is eight launches: after eight over the same 24 MiB the ninth has the L2s to itself
        for _ in range(9):
            dev.apply_fn(a, f, out=b)
        assert dev.last_launch_shape() == (2, 0, False)
        # in a graph: the levels before a node count, the last ones before the first (a graph is replayed)
        dev.capture_begin()
        dev.apply_fn(a, f, out=b)
        dev.apply_fn(b, f, out=c)
        dev.apply_fn(c, f, out=d)
        graph = dev.capture_end()
        assert dev.last_launch_shape() == (2, loads, False)
        for _ in range(3):
            graph.launch()
        assert_bits_equal(d.read(), want)
        graph.destroy()
        dev.capture_begin()
        dev.apply_fn(a, f, out=b)
        graph = dev.capture_end()                     # one 24 MiB node alone
        assert dev.last_launch_shape() == (2, 0, False)
        graph.launch()
        graph.destroy()
    finally:
        dev.close()


def test_mid_sized_launches_leave_the_cache_to_their_neighbours(oracle):
    """A two-pointer launch of 256 to 768 MiB keeps its stores in the memory-side cache while it has the
    cache to itself (the same launch again and again), and streams them past it once the launches before it
    touched other memory as well (tanh forward between gradient launches over other arrays).  And a launch of
    more than 32 MiB that touches nothing the launch before it wrote runs as one-wavefront workgroups with one
    vector per thread; one that comes back to what was just written keeps two vectors per thread."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        loads, both = 1 | 64, 3
        n = 1 << 26                                   # 256 MiB per array
        x, y = dev.alloc(n), dev.alloc(n)
        fwd = lambda v: v.tanh()
        dev.apply_fn(x, fwd, out=y)                   # nothing before it
        assert dev.last_launch_shape() == (1, loads, True)
        dev.apply_fn(x, fwd, out=y)                   # nothing else in between: it overwrites what was just written
        assert dev.last_launch_shape() == (2, loads, True)
        g, o, x2 = dev.alloc(n), dev.alloc(n), dev.alloc(n)
        dev.add_unary_grad(x2, g, o, lambda v: v.mul(2.0))      # (another input: nothing the launch before it read)
        assert dev.last_launch_shape() == (1, loads, True)      # three pointers: always loads only; y is not among them
        dev.apply_fn(x, fwd, out=y)                   # g and o were touched since, and g is what was written last
        assert dev.last_launch_shape() == (1, both, True)
        dev.apply_fn(y, fwd, out=x)                   # reads what the launch before it wrote
        assert dev.last_launch_shape()[0] == 2
        assert np.all(y.slice(n - 4096, n).read() == 0)
    finally:
        dev.close()


def test_a_launch_that_reads_what_the_one_before_read_keeps_the_input_cached(oracle):
    """`out = device.apply_fn(&x, f)` in a loop alternates between two output blocks: each launch touches
    nothing the launch before it wrote and reads what it read, and loads that input with temporal accesses
    while everything else streams past the cache (its direction alternates from 256 MiB touched on, as for other launches).  The same for the gradient
    launch behind the forward launch of the same x (x is kept, the other operands stream) and the forward
    launch behind it.  Same bits as the oracle in every shape."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        loads = 1 | 64
        keep_first = 3 | 64 | 1 << 8
        n = (1 << 24) + 3                             # 64 MiB per array
        xs = synth.uniform_f32(77, n, -2, 2)
        x = dev.buffer(xs)
        outs = [dev.alloc(n), dev.alloc(n)]
        f = lambda v: v.mul(1.5).add(0.25)
        want = oracle.apply_fn(f, xs)
        dev.apply_fn(x, f, out=outs[0])
        assert dev.last_launch_shape() == (1, loads, False)      # nothing before it
        for step in range(1, 5):
            dev.apply_fn(x, f, out=outs[step & 1])
            assert dev.last_launch_shape() == (1, keep_first, False), step
        for out in outs:
            assert_bits_equal(out.read(), want)
        gs, os_ = synth.uniform_f32(79, n, -1, 1), synth.uniform_f32(78, n, -1, 1)
        g, o = dev.buffer(gs), dev.buffer(os_)
        grad = lambda v: v.mul(2.0)
        for step in range(3):
            dev.add_unary_grad(x, g, o, grad)                    # reads x as the launch before it did, and two arrays more
            assert dev.last_launch_shape() == (1, keep_first, False)
            gs = oracle.add_unary_grad(grad, xs, gs, os_)
            dev.apply_fn(x, f, out=outs[0])                      # x again; nothing the gradient launch wrote
            assert dev.last_launch_shape() == (1, keep_first, False)
        assert_bits_equal(g.read(), gs)
        assert_bits_equal(outs[0].read(), want)
        dev.apply_fn(x, f, out=outs[0])                          # overwrites what was just written: the usual shape
        assert dev.last_launch_shape()[0] == 2
        y = dev.alloc(n)
        dev.apply_fn2(o, x, lambda p, q: p.add(q), out=y)        # x is its second input
        assert dev.last_launch_shape() == (1, 3 | 64 | 2 << 8, False)
        assert_bits_equal(y.read(), oracle.apply_fn(lambda p, q: p.add(q), os_, xs))
        big = 1 << 26                                             # 512 MiB touched per launch: the direction alternates as well
        bx, bouts = dev.alloc(big), [dev.alloc(big), dev.alloc(big)]
        for step in range(3):
            dev.apply_fn(bx, f, out=bouts[step & 1])
        assert dev.last_launch_shape() == (1, keep_first, True)
        assert (bouts[0].slice(big - 4096, big).read() == np.float32(0.25)).all()
    finally:
        dev.close()


def test_more_than_two_to_the_32_elements(hip):
    """Indices are 64-bit throughout: 2^32 + 5 one-byte elements (4 GiB in, 4 GiB out), launched
    directly and from a replayed graph; windows around 2^31, 2^32 and the scalar tail."""
    n = (1 << 32) + 5
    x = hip.alloc(n, "u8")
    pat = (np.arange(1 << 20, dtype=np.uint32) * 7 % 251).astype(np.uint8)
    starts = (0, (1 << 31) - 4096, (1 << 32) - (3 << 20), n - (1 << 20))
    for start in starts:
        x.slice(start, start + (1 << 20)).write(pat)
    want = (pat.astype(np.uint32) * 3 + 1).astype(np.uint8)
    f = lambda v: v.mul(3).add(1)
    out = hip.apply_fn(x, f)
    for start in starts:
        assert_bits_equal(out.slice(start, start + (1 << 20)).read(), want, f"window at {start}")
    assert np.all(out.slice(3 << 30, (3 << 30) + 4096).read() == 1)
    out.slice(n - 4096, n).clear()
    hip.capture_begin()
    hip.apply_fn(x, f, out=out)
    graph = hip.capture_end()
    graph.launch()
    graph.launch()                       # the second replay walks the tiles the other way round
    assert_bits_equal(out.slice(n - (1 << 20), n).read(), want, "tail after replays")
    graph.destroy()


def test_allocation_pool():
    """Freed blocks are handed out again: same address, zero-filled again, ordered behind the
    work that still used them; limit 0 switches the pool off; trim gives everything back."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        n = 300000
        x = synth.uniform_f32(1, n, -1, 1)
        a = dev.buffer(x)
        held0, reused0, allocated0 = dev.pool_stats()
        out = dev.apply_fn(a, lambda v: v.mul(2.0))
        addr = out.ptr
        want = (x * np.float32(2.0)).astype(np.float32)
        out.free()                                   # the kernel may still be running: no wait here
        held1, _, _ = dev.pool_stats()
        assert held1 >= n * 4
        again = dev.alloc(n)                         # same size class: the same block, zero-filled behind the kernel
        assert again.ptr == addr
        assert dev.pool_stats()[1] == reused0 + 1
        assert not again.read().any()
        again.free()
        smaller = dev.alloc(n - 100)                 # rounds to the same class
        assert smaller.ptr == addr
        dev.apply_fn(a.slice(0, n - 100), lambda v: v.mul(2.0), out=smaller)
        assert_bits_equal(smaller.read(), want[: n - 100])
        smaller.free()
        dev.pool_trim()
        assert dev.pool_stats()[0] == 0
        dev.set_pool_limit(0)
        b = dev.alloc(n)
        b.free()
        assert dev.pool_stats()[0] == 0              # went back to the driver
        dev.set_pool_limit(1 << 30)
        # many eager operations reuse two blocks instead of allocating each time
        _, reused, allocated = dev.pool_stats()
        for _ in range(50):
            dev.apply_fn(a, lambda v: v.add(1.0)).free()
        _, reused2, allocated2 = dev.pool_stats()
        assert allocated2 - allocated <= 1 and reused2 - reused >= 49
    finally:
        dev.close()


def test_small_blocks_are_cut_from_zeroed_slabs():
    """Blocks of up to 256 KiB are cut from 4 MiB allocations that are zero-filled once: new blocks are
    zero, neighbours in a slab do not touch each other (a launch over one leaves the blocks around it
    alone, up to the last byte of its rounded size), a freed block is reused and zero-filled again, and
    with the pool switched off a slab goes back to the driver with its last block, after which new
    blocks are zero again although the memory may be the same."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        n = 4000                                     # 16 000 bytes: rounds to 16 384, 256 blocks per slab
        blocks = [dev.alloc(n) for _ in range(600)]  # three slabs
        addrs = sorted(b.ptr for b in blocks)
        gaps = np.diff(np.array(addrs, dtype=np.uint64))
        assert (gaps >= 16384).all() and (gaps == 16384).sum() >= 590        # cut one after the other
        for b in blocks[::37]:
            assert not b.read().any()
        x = synth.uniform_f32(3, n, 1, 2)
        src = dev.buffer(x)
        for b in blocks[1::2]:
            dev.apply_fn(src, lambda v: v.mul(3.0), out=b)
        want = (x * np.float32(3.0)).astype(np.float32)
        for i in (0, 2, 254, 256, 300, 598):
            assert not blocks[i].read().any(), i     # even blocks stay zero next to written neighbours
        for i in (1, 255, 257, 599):
            assert_bits_equal(blocks[i].read(), want)
        # a freed block comes back from the pool, zero-filled again
        addr = blocks[1].ptr
        blocks[1].free()
        again = dev.alloc(n)
        assert again.ptr == addr and not again.read().any()
        blocks[1] = again
        # no pool: blocks go back one by one, a slab with its last block; what is allocated afterwards is zero
        dev.sync()
        dev.set_pool_limit(0)
        for b in blocks:
            b.free()
        src.free()
        assert dev.pool_stats()[0] == 0
        fresh = [dev.alloc(n) for _ in range(300)]
        for b in fresh[::29]:
            assert not b.read().any()
        # larger blocks are allocations of their own
        big = dev.alloc(100000)
        assert not big.read().any()
        for b in fresh:
            dev.apply_fn(big.slice(0, n), lambda v: v.add(1.5), out=b)
        assert (fresh[123].read() == np.float32(1.5)).all()
    finally:
        dev.close()


@pytest.mark.parametrize("dtype", ["f32", "f16", "i8", "f64"])
def test_no_launch_writes_outside_its_range(dtype):
    """Blocks that sit back to back in one slab: every kind of launch over the middle one and over
    views inside it (odd lengths, offsets that start off a 16-byte boundary: scalar head and tail,
    partial last tile), eagerly, recorded and joined, merged with equal and with different lengths,
    filled and copied -- and the guard blocks before and behind it keep their pattern to the byte."""
    import custos_amd
    dev = custos_amd.HIP(0)
    try:
        item = np.dtype(capi.DTYPES[dtype][1]).itemsize
        per512 = 512 // item
        guard_n = 8 * per512                      # whole size classes: no slack between the blocks
        mid_n = 20 * per512
        pattern = (np.arange(guard_n * item, dtype=np.uint32) * 37 + 11).astype(np.uint8)
        as_elems = lambda raw: raw.view(capi.DTYPES[dtype][1])
        before = dev.buffer(as_elems(pattern), dtype)
        mid = dev.alloc(mid_n, dtype)
        behind = dev.buffer(as_elems(pattern), dtype)
        second = dev.alloc(mid_n, dtype)
        last = dev.buffer(as_elems(pattern), dtype)
        assert mid.ptr == before.ptr + guard_n * item and behind.ptr == mid.ptr + mid_n * item
        assert second.ptr == behind.ptr + guard_n * item and last.ptr == second.ptr + mid_n * item
        src = dev.buffer(np.ones(mid_n, dtype=capi.DTYPES[dtype][1]), dtype)
        f = lambda v: v.add(1) if dtype == "i8" else v.mul(1.5).add(0.25)
        g = lambda v: v.add(v)
        views = [(0, mid_n), (1, mid_n), (0, mid_n - 1), (3, mid_n - 5), (7, 7 + 33), (mid_n - 9, mid_n), (5, 5 + 16 * per512 + 3)]
        for lo, hi in views:
            dev.apply_fn(src.slice(lo, hi), f, out=mid.slice(lo, hi))                 # eager
            dev.apply_fn2(src.slice(lo, hi), mid.slice(lo, hi), lambda p, q: p.add(q), out=second.slice(lo, hi))
            if dtype in ("f32", "f64"):
                dev.add_unary_grad(src.slice(lo, hi), mid.slice(lo, hi), second.slice(lo, hi), lambda v: v.mul(2.0))
            dev.fill(mid.slice(lo, hi), 3)
            dev.clear(second.slice(lo, hi))
            dev.copy(mid.slice(lo, hi), src.slice(lo, hi))
        for merged in (True, False):
            dev.set_graph_batching(merged)
            dev.capture_begin()
            for lo, hi in views:                                                          # recorded: joined, merged (ragged)
                dev.apply_fn(src.slice(lo, hi), f, out=mid.slice(lo, hi))
                dev.apply_fn(mid.slice(lo, hi), g, out=second.slice(lo, hi))
            graph = dev.capture_end()
            graph.launch()
            graph.launch()
            dev.sync()
            graph.destroy()
        dev.set_graph_batching(True)
        dev.capture_begin()
        for k in range(6):                                                                # equal lengths, aligned: one merged grid
            lo = k * 3 * per512
            dev.apply_fn(src.slice(lo, lo + 3 * per512), f, out=mid.slice(lo, lo + 3 * per512))
        dev.apply_fn(src.slice(18 * per512, mid_n), f, out=mid.slice(18 * per512, mid_n))
        graph = dev.capture_end()
        graph.launch()
        dev.sync()
        graph.destroy()
        for name, guard in (("before", before), ("behind", behind), ("last", last)):
            assert np.array_equal(guard.read().view(np.uint8), pattern), f"{dtype}: the block {name} was written"
    finally:
        dev.close()


def test_device_to_device_copies(hip):
    """Aligned ranges go through the library's copy kernel, unaligned ones through the runtime:
    the same bytes either way, small and larger than the memory-side cache."""
    for n in (1, 3, 4, 1000, 4096, 100003, (1 << 26) + 4):
        src = hip.alloc(n + 8, "u8" if n < 10 else "f32", zeroed=False)
        dt = np.uint8 if n < 10 else np.float32
        period = min(n + 8, 1 << 20)
        pattern = (np.arange(period, dtype=np.uint32) * 2654435761 >> 7).astype(dt)
        hip.write(src.slice(0, period), pattern)
        filled = period
        while filled < n + 8:
            step = min(filled, n + 8 - filled)
            hip.copy(src.slice(filled, filled + step), src.slice(0, step))
            filled += step
        for so, do in ((0, 0), (4, 4), (1, 0), (0, 3)):
            dst = hip.alloc(n + 8, src.dtype)
            hip.copy(dst.slice(do, do + n), src.slice(so, so + n))
            tail = min(n, 5000)
            got = dst.slice(do + n - tail, do + n + 1).read()
            idx = (np.arange(so + n - tail, so + n) % period)
            assert_bits_equal(got[:tail], pattern[idx], f"n={n} src+{so} dst+{do}")
            assert got[tail] == 0                       # nothing written past the range
            head = dst.slice(0, do + min(n, 64)).read()
            assert not head[:do].any()
            assert_bits_equal(head[do:], pattern[(np.arange(so, so + min(n, 64))) % period])


def test_a_block_is_freed_once(hip):
    """A second free of the same address is an error, as is the free of an address the device handle
    never handed out; neither puts a block into the pool twice."""
    ptr = C.c_uint64(0)
    lib, h = hip.lib, hip.handle
    capi.check(lib.custos_hip_alloc(h, 4096, capi.ALLOC_ZEROED, C.byref(ptr)), h)
    assert lib.custos_hip_free(h, ptr.value) == 0
    assert lib.custos_hip_free(h, ptr.value) == capi.ERR_INVALID_ARGUMENT
    assert "freed already" in capi.last_error(h)
    assert lib.custos_hip_free(h, ptr.value + 16) == capi.ERR_INVALID_ARGUMENT
    assert lib.custos_hip_free(h, 0) == 0
    # the pool holds the block once: two allocations of that size get two different addresses
    a, b = hip.alloc(1024), hip.alloc(1024)
    assert a.ptr != b.ptr
    # blocks still held when the handle is destroyed go back to the driver with it
    import custos_amd
    other = custos_amd.HIP(0)
    held = [other.alloc(1 << 20) for _ in range(4)]
    other.close()
    for buf in held:
        buf.ptr = 0
