"""Every one of the 2^32 f32 bit patterns through the one-operand routine nodes, against the CPU oracle.

About two minutes per node on 16 host threads, so the sweep is opt-in: CUSTOS_EXHAUSTIVE=1.  The
everyday suite covers the same nodes on 2^22 random bit patterns (test_gpu_semantics.py).  The
bound is the one stated for f32 transcendentals: at most 4 ulp from the CPU path (libm), NaN exactly
where the CPU path gives NaN, the same infinities; sqrt, abs and neg are bit-exact."""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from helpers import ulp_distance_f32

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("CUSTOS_EXHAUSTIVE") != "1", reason="minutes per node: set CUSTOS_EXHAUSTIVE=1")]

NODES = {
    "exp": (lambda v: v.exp(), 4), "sin": (lambda v: v.sin(), 4), "cos": (lambda v: v.cos(), 4), "tan": (lambda v: v.tan(), 4),
    "tanh": (lambda v: v.tanh(), 4), "ln": (lambda v: v.ln(), 4), "sqrt": (lambda v: v.sqrt(), 0),
    "abs": (lambda v: v.abs(), 0), "neg": (lambda v: v.neg(), 0),
}
CHUNK = 1 << 26
THREADS = 16


def _compare(oracle, f, x, got):
    """(worst distance, its input bits, inputs per distance 0..8+) over one slice; NaNs must coincide."""
    want = oracle.apply_fn(f, x)
    nan = np.isnan(want)
    if not np.array_equal(np.isnan(got), nan):
        bad = np.flatnonzero(np.isnan(got) != nan)[0]
        return -1, int(x.view(np.uint32)[bad]), None
    d = ulp_distance_f32(np.where(nan, np.float32(0), got), np.where(nan, np.float32(0), want))
    worst = int(np.argmax(d))
    return int(d[worst]), int(x.view(np.uint32)[worst]), np.bincount(np.minimum(d, 8), minlength=9)


@pytest.mark.parametrize("name", list(NODES))
def test_every_f32_bit_pattern(hip, oracle, name):
    f, bound = NODES[name]
    xb, ob = hip.alloc(CHUNK, zeroed=False), hip.alloc(CHUNK, zeroed=False)
    histogram = np.zeros(9, dtype=np.int64)
    worst, worst_bits = 0, 0
    piece = CHUNK // THREADS
    with ThreadPoolExecutor(THREADS) as pool:
        for start in range(0, 1 << 32, CHUNK):
            x = np.arange(start, start + CHUNK, dtype=np.uint32).view(np.float32)
            hip.write(xb, x)
            hip.apply_fn(xb, f, out=ob)
            got = ob.read()
            jobs = [pool.submit(_compare, oracle, f, x[i:i + piece], got[i:i + piece]) for i in range(0, CHUNK, piece)]
            for job in jobs:
                dist, bits, counts = job.result()
                assert dist >= 0, f"{name}: NaN on one side only for input bits {bits:#010x}"
                histogram += counts
                if dist > worst:
                    worst, worst_bits = dist, bits
    print(f"\n{name}: worst {worst} ulp at input bits {worst_bits:#010x}; inputs by distance 0..7, 8+: {histogram.tolist()}", flush=True)
    assert histogram.sum() == 1 << 32
    assert worst <= bound, (name, worst, hex(worst_bits))
