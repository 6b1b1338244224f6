"""Writes tests/golden/config_vectors.json: for each BASELINE configuration the first
elements of the seeded synthetic input and what the CPU oracle computes for them,
as raw bit patterns.  Run from the repository root:  python tests/golden/make_config_vectors.py

The file is a regression fixture for the oracle + input generator pair (it does not
pin the oracle against the reference; the reference's own vectors do that in
tests/test_oracle_kats.py)."""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from custos_amd import synth  # noqa: E402
from oracle import cpu_oracle  # noqa: E402

N = 24


def bits(a):
    a = np.ascontiguousarray(a)
    return [int(v) for v in a.view(f"u{a.itemsize}")]


def main():
    out = {}
    x = synth.uniform_f32(0, N, -4, 4)
    out["c1_exp"] = {"x": bits(x), "y": bits(cpu_oracle.c1_exp(x))}
    x = synth.uniform_f32(0, N, -np.pi, np.pi)
    out["c2_chain"] = {"x": bits(x), "y": bits(cpu_oracle.c2_chain_fused(x))}
    x = synth.normal_f32(0, N)
    yg = synth.uniform_f32(1, N, -1, 1)
    g0 = np.full(N, 0.1, dtype=np.float32)
    out["c3_tanh"] = {"x": bits(x), "y_grad": bits(yg), "y": bits(cpu_oracle.c3_tanh_fwd(x)),
                      "x_grad": bits(cpu_oracle.c3_tanh_bwd(x, g0, yg))}
    xh = synth.uniform_f16_bits(0, N, -2, 2)
    out["c4_half"] = {"x": bits(xh), "y": bits(cpu_oracle.c4_chain_f16(xh))}
    a, b, c = (synth.uniform_f32(s, N, 0, 1) for s in (1, 2, 3))
    t, u, y = cpu_oracle.c5_graph(a, b, c)
    out["c5_graph"] = {"a": bits(a), "b": bits(b), "c": bits(c), "y": bits(y)}
    out["splitmix64_seed0"] = [int(v) for v in synth.splitmix64(0, 4)]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
