"""First GPU parity checks through the C ABI: apply_fn, two-operand apply,
fused chain and unary gradient against the CPU oracle."""
import numpy as np
import pytest

from custos_amd import synth
from tests.helpers import assert_bits_equal, ulp_distance_f32

pytestmark = pytest.mark.gpu


def test_apply_fn_reference_vector(hip):
    # src/unary.rs:15-18
    a = hip.buffer([1., 2., 3., 3., 2., 1.])
    out = hip.apply_fn(a, lambda x: x.mul(2.))
    assert out.read().tolist() == [2., 4., 6., 6., 4., 2.]


def test_c1_exp_f32(hip, oracle):
    n = 1 << 20
    x = synth.uniform_f32(0, n, -4, 4)
    got = hip.apply_fn(hip.buffer(x), lambda v: v.exp()).read()
    want = oracle.c1_exp(x)
    assert ulp_distance_f32(got, want).max() <= 4  # tolerance: 4 ulp for f32 transcendentals


@pytest.mark.parametrize("n", [1, 3, 4, 5, 63, 64, 65, 1023, 4096, 4097, 100003])
def test_exact_arithmetic_ragged_sizes(hip, oracle, n):
    x = synth.uniform_f32(7, n, -3, 3)
    f = lambda v: v.mul(1.7).add(0.3).max(0.25).sub(v).div(3.0).abs().neg()
    got = hip.apply_fn(hip.buffer(x), f).read()
    assert_bits_equal(got, oracle.apply_fn(f, x), f"n={n}")


def test_two_operand(hip, oracle):
    n = 10007
    x = synth.uniform_f32(1, n, -2, 2)
    y = synth.uniform_f32(2, n, -2, 2)
    f = lambda a, b: a.add(b).mul(3.6).sub(b)
    got = hip.apply_fn2(hip.buffer(x), hip.buffer(y), f).read()
    assert_bits_equal(got, oracle.apply_fn(f, x, y))


def test_fused_chain_c2_small(hip, oracle):
    n = (1 << 18) + 5
    x = synth.uniform_f32(0, n, -np.pi, np.pi)
    ops = [lambda v: v.sin(), lambda v: v.mul(2.0), lambda v: v.add(1.0), lambda v: v.max(0.0), lambda v: v.sub(0.5)]
    got = hip.fused_apply_fn(hip.buffer(x), ops).read()
    want = oracle.fused_apply_fn(ops, x)
    # sin within 4 ulp; the following exact ops scale that error by at most 2 in absolute terms
    sin_ulp = np.spacing(np.float32(1.0))
    assert np.max(np.abs(got - want)) <= 4 * 2 * sin_ulp
    # the oracle's compiled loop for this chain and its expression interpreter are two pieces of
    # code: on these inputs they agree bit for bit, and the kernel is as close to either
    loop = oracle.c2_chain_fused(x)
    assert_bits_equal(loop, want)
    assert got.dtype == loop.dtype and got.shape == loop.shape
    assert np.max(np.abs(got - loop)) <= 4 * 2 * sin_ulp


def test_add_unary_grad_exact(hip, oracle):
    n = 5003
    x = synth.uniform_f32(3, n, -2, 2)
    g = synth.uniform_f32(4, n, -1, 1)
    o = synth.uniform_f32(5, n, -1, 1)
    f = lambda v: v.mul(2.0).add(1.0)
    gb = hip.buffer(g)
    hip.add_unary_grad(hip.buffer(x), gb, hip.buffer(o), f)
    assert_bits_equal(gb.read(), oracle.add_unary_grad(f, x, g, o))
