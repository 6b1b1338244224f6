"""The committed fixtures of tests/golden: seeded inputs and oracle outputs of the five
configurations, checked against the generator + oracle (CPU) and against the HIP kernels."""
import json
import os

import numpy as np
import pytest

from custos_amd import synth
from tests.helpers import ulp_distance_f16, ulp_distance_f32

HERE = os.path.dirname(os.path.abspath(__file__))
G = json.load(open(os.path.join(HERE, "golden", "config_vectors.json")))
N = 24


def arr(name, key, dtype):
    return np.array(G[name][key], dtype=f"u{np.dtype(dtype).itemsize}").view(dtype)


def test_splitmix64_known_answers():
    # the published first outputs of SplitMix64 for seed 0
    want = [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F, 0xF88BB8A8724C81EC]
    assert [int(v) for v in synth.splitmix64(0, 4)] == want == G["splitmix64_seed0"]
    # any slice can be generated alone
    whole = synth.uniform_f32(3, 1000, -1, 1)
    assert np.array_equal(synth.uniform_f32(3, 100, -1, 1, offset=700), whole[700:800])
    u = synth.unit_f32(5, 100000)
    assert u.min() >= 0 and u.max() < 1 and abs(u.mean() - 0.5) < 0.01
    z = synth.normal_f32(0, 200000)
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1) < 0.01


def test_generator_and_oracle_reproduce_the_fixture(oracle):
    assert np.array_equal(synth.uniform_f32(0, N, -4, 4), arr("c1_exp", "x", np.float32))
    assert np.array_equal(oracle.c1_exp(arr("c1_exp", "x", np.float32)), arr("c1_exp", "y", np.float32))
    assert np.array_equal(synth.uniform_f32(0, N, -np.pi, np.pi), arr("c2_chain", "x", np.float32))
    assert np.array_equal(oracle.c2_chain_fused(arr("c2_chain", "x", np.float32)), arr("c2_chain", "y", np.float32))
    x = arr("c3_tanh", "x", np.float32)
    assert np.array_equal(synth.normal_f32(0, N), x)
    assert np.array_equal(oracle.c3_tanh_fwd(x), arr("c3_tanh", "y", np.float32))
    g = oracle.c3_tanh_bwd(x, np.full(N, 0.1, dtype=np.float32), arr("c3_tanh", "y_grad", np.float32))
    assert np.array_equal(g, arr("c3_tanh", "x_grad", np.float32))
    assert np.array_equal(synth.uniform_f16_bits(0, N, -2, 2), arr("c4_half", "x", np.uint16))
    assert np.array_equal(oracle.c4_chain_f16(arr("c4_half", "x", np.uint16)), arr("c4_half", "y", np.uint16))
    t, u, y = oracle.c5_graph(*(arr("c5_graph", k, np.float32) for k in "abc"))
    assert np.array_equal(y, arr("c5_graph", "y", np.float32))


@pytest.mark.gpu
def test_hip_matches_the_fixture(hip):
    got = hip.apply_fn(hip.buffer(arr("c1_exp", "x", np.float32)), lambda v: v.exp()).read()
    assert ulp_distance_f32(got, arr("c1_exp", "y", np.float32)).max() <= 4
    ops = [lambda v: v.sin(), lambda v: v.mul(2.0), lambda v: v.add(1.0), lambda v: v.max(0.0), lambda v: v.sub(0.5)]
    got = hip.fused_apply_fn(hip.buffer(arr("c2_chain", "x", np.float32)), ops).read()
    assert np.max(np.abs(got - arr("c2_chain", "y", np.float32))) <= 16 * 2.0 ** -24
    xb = hip.buffer(arr("c3_tanh", "x", np.float32))
    got = hip.apply_fn(xb, lambda v: v.tanh()).read()
    assert ulp_distance_f32(got, arr("c3_tanh", "y", np.float32)).max() <= 4
    gb = hip.buffer(np.full(N, 0.1, dtype=np.float32))
    hip.add_unary_grad(xb, gb, hip.buffer(arr("c3_tanh", "y_grad", np.float32)),
                       lambda v: v.val(1.0).sub(v.tanh().mul(v.tanh())))
    assert np.max(np.abs(gb.read() - arr("c3_tanh", "x_grad", np.float32))) <= 12 * 2.0 ** -24
    xh = arr("c4_half", "x", np.uint16)
    got = hip.apply_fn(hip.buffer(xh.view(np.float16), "f16"), lambda v: v.mul(0.5).exp().mul(v).add(v.mul(v))).read()
    assert ulp_distance_f16(got.view(np.uint16), arr("c4_half", "y", np.uint16)).max() <= 1
    a, b, c = (hip.buffer(arr("c5_graph", k, np.float32)) for k in "abc")
    y = hip.apply_fn_n([a, b, c], lambda p, q, r: p.mul(q).add(r).abs().sqrt().mul(0.3)).read()
    assert np.array_equal(y.view(np.uint32), arr("c5_graph", "y", np.uint32))
