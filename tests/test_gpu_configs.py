"""GPU parity for the five benchmark configurations, at sizes the CPU oracle
finishes in seconds, and size-independent properties at the full sizes."""
import numpy as np
import pytest

from custos_amd import capi, synth
from tests.helpers import assert_bits_equal, ulp_distance_f16, ulp_distance_f32

pytestmark = pytest.mark.gpu

C2_OPS = [lambda v: v.sin(), lambda v: v.mul(2.0), lambda v: v.add(1.0), lambda v: v.max(0.0), lambda v: v.sub(0.5)]
TANH_GRAD = lambda v: v.val(1.0).sub(v.tanh().mul(v.tanh()))
C4 = lambda v: v.mul(0.5).exp().mul(v).add(v.mul(v))


def test_c1_exp_full_size(hip, oracle):
    """configs[0]: apply_fn(exp), f32 N = 2^20, U[-4,4) seed 0.  Tolerance: 4 ulp."""
    n = 1 << 20
    x = synth.uniform_f32(0, n, -4, 4)
    got = hip.apply_fn(hip.buffer(x), lambda v: v.exp()).read()
    assert ulp_distance_f32(got, oracle.c1_exp(x)).max() <= 4


def test_c2_fused_equals_unfused_on_gpu_and_oracle(hip, oracle):
    """configs[1] at N = 2^22: the fused kernel must give exactly what five separate
    launches give (same device functions, same roundings), and both must sit
    within sin's 4 ulp of the CPU chain."""
    n = (1 << 22) + 17
    x = synth.uniform_f32(0, n, -np.pi, np.pi)
    xb = hip.buffer(x)
    fused = hip.fused_apply_fn(xb, C2_OPS).read()
    cur = xb
    for op in C2_OPS:
        cur = hip.apply_fn(cur, op)
    assert_bits_equal(fused, cur.read(), "fused vs unfused on the GPU")
    want = oracle.c2_chain_fused(x)
    # sin(x) within 4 ulp (|sin| <= 1: ulp <= 2^-24 * 2 below 1), then *2 doubles the absolute error
    assert np.max(np.abs(fused.astype(np.float64) - want.astype(np.float64))) <= 4 * 2 * 2.0 ** -24 * 2
    # where the CPU result is exactly -0.5 (relu clipped) the GPU must agree except within rounding of the clip edge
    s = oracle.apply_fn(lambda v: v.sin(), x)
    safe = np.abs(s.astype(np.float64) * 2 + 1) > 1e-5
    assert np.array_equal((fused == np.float32(-0.5))[safe], (want == np.float32(-0.5))[safe])


def test_c2_sin_ulp(hip, oracle):
    n = 1 << 20
    x = synth.uniform_f32(0, n, -np.pi, np.pi)
    got = hip.apply_fn(hip.buffer(x), lambda v: v.sin()).read()
    assert ulp_distance_f32(got, oracle.apply_fn(lambda v: v.sin(), x)).max() <= 4


def test_c3_tanh_forward_backward(hip, oracle):
    """configs[2] at N = 2^20: y = tanh(x); x_grad += y_grad * (1 - tanh(x)^2), x_grad starts at 0.1."""
    n = (1 << 20) + 3
    x = synth.normal_f32(0, n)
    yg = synth.uniform_f32(1, n, -1, 1)
    g0 = np.full(n, 0.1, dtype=np.float32)
    xb = hip.buffer(x)
    y = hip.apply_fn(xb, lambda v: v.tanh()).read()
    assert ulp_distance_f32(y, oracle.c3_tanh_fwd(x)).max() <= 4
    gb = hip.buffer(g0)
    hip.add_unary_grad(xb, gb, hip.buffer(yg), TANH_GRAD)
    got = gb.read()
    want = oracle.c3_tanh_bwd(x, g0, yg)
    # d = 1 - t*t: 4 ulp on t (|t| <= 1) gives at most 2*4*2^-24 absolute on d, plus roundings of the products
    assert np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) <= 12 * 2.0 ** -24
    # the update itself is exact arithmetic: with d computed by the GPU's own tanh it is bit-identical
    t = hip.apply_fn(xb, lambda v: v.tanh()).read()
    d = (np.float32(1.0) - t * t).astype(np.float32)
    assert_bits_equal(got, (g0 + (yg * d).astype(np.float32)).astype(np.float32), "g + (o * d)")


def test_c4_half_chain(hip, oracle):
    """configs[3] at N = 2^20: f16 storage, f32 compute, one rounding.
    Tolerance: 1 f16 ulp of the f32 reference rounded to f16."""
    n = (1 << 20) + 5
    xb = synth.uniform_f16_bits(0, n, -2, 2)
    got = hip.apply_fn(hip.buffer(xb.view(np.float16), "f16"), C4).read().view(np.uint16)
    want = oracle.c4_chain_f16(xb)
    d = ulp_distance_f16(got, want)
    assert d.max() <= 1
    assert (d == 0).mean() > 0.99


def test_c4_exact_part_is_bit_exact(hip, oracle):
    n = 70001
    xb = synth.uniform_f16_bits(3, n, -2, 2)
    f = lambda v: v.mul(0.5).mul(v).add(v.mul(v)).sub(0.25)
    got = hip.apply_fn(hip.buffer(xb.view(np.float16), "f16"), f).read().view(np.uint16)
    assert_bits_equal(got, oracle.apply_fn(f, xb, dtype="f16"))


def test_c5_graph_replay(hip, oracle):
    """configs[4] scaled to 64 buffers: per buffer t = a*b; u = t+c; y = sqrt(abs(u))*0.3,
    captured once and replayed; every replay must reproduce the eager result bit for bit
    (all five node kinds are correctly rounded)."""
    nbuf, n = 64, 4096
    a = [synth.uniform_f32(1, n, 0, 1, offset=i * n) for i in range(nbuf)]
    b = [synth.uniform_f32(2, n, 0, 1, offset=i * n) for i in range(nbuf)]
    c = [synth.uniform_f32(3, n, 0, 1, offset=i * n) for i in range(nbuf)]
    ab, bb, cb = ([hip.buffer(v) for v in arrs] for arrs in (a, b, c))
    t = [hip.alloc(n) for _ in range(nbuf)]
    u = [hip.alloc(n) for _ in range(nbuf)]
    y = [hip.alloc(n) for _ in range(nbuf)]
    unary = [lambda v: v.abs().sqrt(), lambda v: v.mul(0.3)]

    def record():
        hip.capture_begin()
        for i in range(nbuf):
            hip.apply_fn2(ab[i], bb[i], lambda p, q: p.mul(q), out=t[i])
            hip.apply_fn2(t[i], cb[i], lambda p, q: p.add(q), out=u[i])
            hip.fused_apply_fn(u[i], unary, out=y[i])
        return hip.capture_end()

    for batching, fusing in ((True, True), (True, False), (False, True), (False, False)):
        hip.set_graph_batching(batching)
        hip.set_graph_fusing(fusing)
        try:
            graph = record()
        finally:
            hip.set_graph_batching(True)
            hip.set_graph_fusing(True)
        recorded, kernel_nodes, levels = graph.stats()
        # the three launches of a buffer become one kernel that reads a, b, c and writes t, u, y
        assert (recorded, levels, graph.fused_launches) == ((3 * nbuf, 1, 2 * nbuf) if fusing else (3 * nbuf, 3, 0))
        # the 64 independent chains run side by side; with batching every level is ONE launch
        per_buffer = 1 if fusing else 3
        assert kernel_nodes == (per_buffer if batching else per_buffer * nbuf)
        # nothing ran while recording: outputs are still the zeros of alloc / of the last clear
        assert not y[0].read().any()
        for replay in range(3):
            graph.launch()
            hip.sync()
            for i in (0, 1, nbuf // 2, nbuf - 1):
                tt, uu, yy = oracle.c5_graph(a[i], b[i], c[i])
                what = f"batching={batching} fusing={fusing} replay {replay} buffer {i}"
                assert_bits_equal(t[i].read(), tt, what)
                assert_bits_equal(u[i].read(), uu, what)
                assert_bits_equal(y[i].read(), yy, what)
            for i in range(nbuf):
                t[i].clear()
                u[i].clear()
                y[i].clear()
            hip.sync()
        graph.destroy()


@pytest.mark.parametrize("log2n", [28])
def test_c2_full_size_properties(hip, oracle, log2n):
    """configs[1] at the full N = 2^28: checks that need no full CPU pass.
    (a) a window at the start, the middle and the end against the oracle,
    (b) the output of a periodic input is periodic (every tile computes the same function),
    (c) range: relu(.)-0.5 lies in [-0.5, 2.5]."""
    n = 1 << log2n
    period = 1 << 20
    base = synth.uniform_f32(0, period, -np.pi, np.pi)
    xb = hip.alloc(n, zeroed=False)
    for k in range(n // period):
        hip.copy(xb.slice(k * period, (k + 1) * period), hip.buffer(base)) if k == 0 else None
    # replicate on the device by doubling copies
    filled = period
    while filled < n:
        hip.copy(xb.slice(filled, 2 * filled), xb.slice(0, filled))
        filled *= 2
    out = hip.fused_apply_fn(xb, C2_OPS)
    want = oracle.c2_chain_fused(base)
    first = out.slice(0, period).read()
    assert np.max(np.abs(first - want)) <= 16 * 2.0 ** -24
    for start in (n // 2, n - period, 5 * period):
        assert_bits_equal(out.slice(start, start + period).read(), first, f"window at {start}")
    assert first.min() >= -0.5 and first.max() <= 2.5
    # a checksum over everything: all 2^28/2^20 windows XOR to zero when the count is even
    acc = hip.alloc(period)
    hip.copy(acc, out.slice(0, period))
    bits = np.zeros(period, dtype=np.uint32)
    for k in range(0, n // period, 37):
        bits ^= out.slice(k * period, (k + 1) * period).read().view(np.uint32) ^ first.view(np.uint32)
    assert not bits.any()


def _replicate(hip, base, n, dtype="f32"):
    """A device buffer of n elements holding `base` repeated (device-side doubling copies)."""
    period = base.size
    buf = hip.alloc(n, dtype, zeroed=False)
    hip.copy(buf.slice(0, period), hip.buffer(base, dtype))
    filled = period
    while filled < n:
        hip.copy(buf.slice(filled, 2 * filled), buf.slice(0, filled))
        filled *= 2
    return buf


def _all_windows_equal(buf, period, first, stride=29):
    """Every window of `period` elements holds the bits of `first` (sampled every `stride` windows
    plus the last one)."""
    bits = first.view(f"u{first.itemsize}")
    windows = list(range(0, buf.len // period, stride)) + [buf.len // period - 1]
    for k in windows:
        got = buf.slice(k * period, (k + 1) * period).read().view(bits.dtype)
        if not np.array_equal(got, bits):
            return False
    return True


def test_c3_full_size_properties(hip, oracle):
    """configs[2] at the full N = 2^26: forward and backward over a periodic input give a periodic
    output whose first window matches the oracle; the gradient accumulates (a second backward
    adds the same amount again)."""
    n, period = 1 << 26, 1 << 18
    x = synth.normal_f32(0, period)
    yg = synth.uniform_f32(1, period, -1, 1)
    xb, ygb = _replicate(hip, x, n), _replicate(hip, yg, n)
    gb = _replicate(hip, np.full(period, 0.1, dtype=np.float32), n)
    y = hip.apply_fn(xb, lambda v: v.tanh())
    first = y.slice(0, period).read()
    assert ulp_distance_f32(first, oracle.c3_tanh_fwd(x)).max() <= 4
    assert _all_windows_equal(y, period, first)
    hip.add_unary_grad(xb, gb, ygb, TANH_GRAD)
    g1 = gb.slice(0, period).read()
    want = oracle.c3_tanh_bwd(x, np.full(period, 0.1, dtype=np.float32), yg)
    assert np.max(np.abs(g1.astype(np.float64) - want.astype(np.float64))) <= 12 * 2.0 ** -24
    assert _all_windows_equal(gb, period, g1)
    hip.add_unary_grad(xb, gb, ygb, TANH_GRAD)
    g2 = gb.slice(0, period).read()
    step = (g1 - np.float32(0.1)).astype(np.float32)
    assert np.max(np.abs(g2.astype(np.float64) - (g1.astype(np.float64) + step))) <= 4 * 2.0 ** -24
    assert _all_windows_equal(gb, period, g2)


def test_c4_full_size_properties(hip, oracle):
    """configs[3] at the full N = 2^28 (f16 storage): periodic input, periodic output, first
    window within one f16 unit of the oracle."""
    n, period = 1 << 28, 1 << 20
    xbits = synth.uniform_f16_bits(0, period, -2, 2)
    xb = _replicate(hip, xbits.view(np.float16), n, "f16")
    out = hip.apply_fn(xb, C4)
    first = out.slice(0, period).read()
    d = ulp_distance_f16(first.view(np.uint16), oracle.c4_chain_f16(xbits))
    assert d.max() <= 1 and (d == 0).mean() > 0.99
    assert _all_windows_equal(out, period, first)


def test_c5_full_size_graph(hip, oracle):
    """configs[4] at its full shape, 1024 buffers of 4096 f32: ONE kernel node for 3072 recorded
    launches (the three launches of a buffer joined, the 1024 joined launches merged), 100 replays,
    every buffer bit-exact against the oracle after the first and the last."""
    nbuf, m = 1024, 4096
    a = synth.uniform_f32(1, nbuf * m, 0, 1)
    b = synth.uniform_f32(2, nbuf * m, 0, 1)
    c = synth.uniform_f32(3, nbuf * m, 0, 1)
    A, B, Cc = hip.buffer(a), hip.buffer(b), hip.buffer(c)
    T, U, Y = hip.alloc(nbuf * m), hip.alloc(nbuf * m), hip.alloc(nbuf * m)
    hip.capture_begin()
    for i in range(nbuf):
        s = slice(i * m, (i + 1) * m)
        hip.apply_fn2(A.slice(s.start, s.stop), B.slice(s.start, s.stop), lambda p, q: p.mul(q), out=T.slice(s.start, s.stop))
        hip.apply_fn2(T.slice(s.start, s.stop), Cc.slice(s.start, s.stop), lambda p, q: p.add(q), out=U.slice(s.start, s.stop))
        hip.fused_apply_fn(U.slice(s.start, s.stop), [lambda v: v.abs().sqrt(), lambda v: v.mul(0.3)], out=Y.slice(s.start, s.stop))
    g = hip.capture_end()
    assert g.stats() == (3 * nbuf, 1, 1) and g.fused_launches == 2 * nbuf
    want_t, want_u, want = oracle.c5_graph(a, b, c)
    for replay in range(100):
        if replay in (0, 99):
            for buf in (T, U, Y):
                buf.clear()
        g.launch()
        if replay in (0, 99):
            hip.sync()
            assert_bits_equal(T.read(), want_t, f"t, replay {replay}")
            assert_bits_equal(U.read(), want_u, f"u, replay {replay}")
            assert_bits_equal(Y.read(), want, f"replay {replay}")
    g.destroy()
