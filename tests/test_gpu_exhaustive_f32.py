"""Every one of the 2^32 f32 bit patterns through the one-operand nodes, and 2^30 random pairs of bit
patterns through the two-operand nodes, against the CPU oracle.

The whole sweep takes three and a half minutes with the oracle on 16 host threads: CUSTOS_EXHAUSTIVE=1.
Without it every test runs a slice of its sweep: every 64th f32 bit pattern (2^26 inputs per node, one
from every run of 64 consecutive patterns, so every exponent, both signs, denormals, infinities and
NaNs are there), 2^24 random pairs per two-operand node, 2^25 random f64 patterns per node.  The
bound is the one stated for f32 transcendentals: at most 4 ulp from the CPU path (libm), NaN exactly
where the CPU path gives NaN, the same infinities; sqrt, abs and neg are bit-exact."""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from helpers import ulp_distance_f32

pytestmark = pytest.mark.gpu
FULL = os.environ.get("CUSTOS_EXHAUSTIVE") == "1"

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
    """All 2^32 patterns with CUSTOS_EXHAUSTIVE=1, else one from every run of 64 consecutive patterns."""
    f, bound = NODES[name]
    xb, ob = hip.alloc(CHUNK, zeroed=False), hip.alloc(CHUNK, zeroed=False)
    histogram = np.zeros(9, dtype=np.int64)
    worst, worst_bits = 0, 0
    piece = CHUNK // THREADS
    with ThreadPoolExecutor(THREADS) as pool:
        for start in range(0, 1 << 32, CHUNK) if FULL else (0,):
            if FULL:
                x = np.arange(start, start + CHUNK, dtype=np.uint32).view(np.float32)
            else:
                # one pattern from every run of 64: run r contributes its pattern number 37 r mod 64
                run = np.arange(CHUNK, dtype=np.uint32)
                x = ((run << np.uint32(6)) | ((run * np.uint32(37)) & np.uint32(63))).view(np.float32)
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
    assert histogram.sum() == (1 << 32 if FULL else CHUNK)
    assert worst <= bound, (name, worst, hex(worst_bits))


BINARY = {
    "add": (lambda p, q: p.add(q), 0), "sub": (lambda p, q: p.sub(q), 0), "mul": (lambda p, q: p.mul(q), 0),
    "div": (lambda p, q: p.div(q), 0), "min": (lambda p, q: p.min(q), 0), "max": (lambda p, q: p.max(q), 0),
    "geq": (lambda p, q: p.geq(q), 0), "leq": (lambda p, q: p.leq(q), 0), "eq": (lambda p, q: p.eq(q), 0),
    "pow": (lambda p, q: p.pow(q), 4),
}
PAIR_CHUNKS = 16          # x 2^26 pairs = 2^30 pairs per node


def _compare2(oracle, f, a, b, got, exact):
    want = oracle.apply_fn(f, a, b)
    nan = np.isnan(want)
    if not np.array_equal(np.isnan(got), nan):
        bad = np.flatnonzero(np.isnan(got) != nan)[0]
        return -1, (int(a.view(np.uint32)[bad]), int(b.view(np.uint32)[bad]))
    if exact:
        same = (got.view(np.uint32) == want.view(np.uint32)) | nan
        if not same.all():
            bad = np.flatnonzero(~same)[0]
            return 1 << 40, (int(a.view(np.uint32)[bad]), int(b.view(np.uint32)[bad]))
        return 0, (0, 0)
    d = ulp_distance_f32(np.where(nan, np.float32(0), got), np.where(nan, np.float32(0), want))
    worst = int(np.argmax(d))
    return int(d[worst]), (int(a.view(np.uint32)[worst]), int(b.view(np.uint32)[worst]))


@pytest.mark.parametrize("name", list(BINARY))
def test_two_operand_nodes_on_2p30_random_pairs_of_bit_patterns(hip, oracle, name):
    """Pairs of arbitrary bit patterns (every exponent, both signs, denormals, infinities, NaNs on either
    side): + - * / min max and the comparisons bit for bit outside NaN payloads, pow within 4 ulp."""
    from custos_amd import synth
    f, bound = BINARY[name]
    CHUNK = globals()["CHUNK"] if FULL else 1 << 24
    ab, bb, ob = (hip.alloc(CHUNK, zeroed=False) for _ in range(3))
    piece = CHUNK // THREADS
    worst, worst_pair = 0, (0, 0)
    with ThreadPoolExecutor(THREADS) as pool:
        for chunk in range(PAIR_CHUNKS if FULL else 1):
            words = synth.splitmix64(1000 + chunk, CHUNK)
            a = (words >> np.uint64(32)).astype(np.uint32).view(np.float32)
            b = (words & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.float32)
            hip.write(ab, a)
            hip.write(bb, b)
            hip.apply_fn2(ab, bb, f, out=ob)
            got = ob.read()
            jobs = [pool.submit(_compare2, oracle, f, a[i:i + piece], b[i:i + piece], got[i:i + piece], bound == 0)
                    for i in range(0, CHUNK, piece)]
            for job in jobs:
                dist, pair = job.result()
                assert dist >= 0, f"{name}: NaN on one side only for input bits {pair[0]:#010x}, {pair[1]:#010x}"
                if dist > worst:
                    worst, worst_pair = dist, pair
    print(f"\n{name}: worst {worst} ulp at input bits {worst_pair[0]:#010x}, {worst_pair[1]:#010x}", flush=True)
    assert worst <= bound, (name, worst, [hex(v) for v in worst_pair])


F64_CHUNK = 1 << 25
F64_CHUNKS = 8            # x 2^25 = 2^28 bit patterns per node


def _ulp_distance_f64(a, b):
    """Units in the last place between f64 arrays, through the order-preserving map to unsigned."""
    def ordered(v):
        u = np.ascontiguousarray(v, dtype=np.float64).view(np.uint64)
        return np.where(u >> np.uint64(63) != 0, ~u, u | np.uint64(1 << 63))
    ua, ub = ordered(a), ordered(b)
    return np.maximum(ua, ub) - np.minimum(ua, ub)


def _compare64(oracle, f, x, got):
    want = oracle.apply_fn(f, x, dtype="f64")
    nan = np.isnan(want)
    if not np.array_equal(np.isnan(got), nan):
        bad = np.flatnonzero(np.isnan(got) != nan)[0]
        return -1, int(x.view(np.uint64)[bad]), None
    d = _ulp_distance_f64(np.where(nan, 0.0, got), np.where(nan, 0.0, want))
    worst = int(np.argmax(d))
    return int(d[worst]), int(x.view(np.uint64)[worst]), np.bincount(np.minimum(d, np.uint64(8)).astype(np.int64), minlength=9)


@pytest.mark.parametrize("name", list(NODES))
def test_f64_nodes_on_2p28_random_bit_patterns(hip, oracle, name):
    """f64: no tolerance is stated for it; 4 units in the last place is this repository's bound."""
    from custos_amd import synth
    f, bound = NODES[name]
    xb, ob = hip.alloc(F64_CHUNK, "f64", zeroed=False), hip.alloc(F64_CHUNK, "f64", zeroed=False)
    histogram = np.zeros(9, dtype=np.int64)
    worst, worst_bits = 0, 0
    piece = F64_CHUNK // THREADS
    with ThreadPoolExecutor(THREADS) as pool:
        for chunk in range(F64_CHUNKS if FULL else 1):
            x = synth.splitmix64(2000 + chunk, F64_CHUNK).view(np.float64)
            hip.write(xb, x)
            hip.apply_fn(xb, f, out=ob)
            got = ob.read()
            jobs = [pool.submit(_compare64, oracle, f, x[i:i + piece], got[i:i + piece]) for i in range(0, F64_CHUNK, piece)]
            for job in jobs:
                dist, bits, counts = job.result()
                assert dist >= 0, f"f64 {name}: NaN on one side only for input bits {bits:#018x}"
                histogram += counts
                if dist > worst:
                    worst, worst_bits = dist, bits
    print(f"\nf64 {name}: worst {worst} ulp at input bits {worst_bits:#018x}; inputs by distance 0..7, 8+: {histogram.tolist()}", flush=True)
    assert worst <= bound, (name, worst, hex(worst_bits))
