"""Every 16-bit input, every unary node, every 16-bit element type, against the CPU oracle.

The reference computes a unary node of a 16-bit float as the f32 routine followed by one rounding
to nearest even (src/number.rs:543-608); the kernels may take another route to the f32 value
(the hardware exp2 behind `exp`), so all 65 536 input bit patterns are swept per node and type:
`sqrt`, `abs`, `neg` bit for bit; `exp sin cos tan tanh ln` within one unit of the storage type,
NaN where the oracle has NaN, the same infinities and the same zeros in sign."""
import numpy as np
import pytest

from custos_amd import Resolve, capi

pytestmark = pytest.mark.gpu

ALL_BITS = np.arange(1 << 16, dtype=np.uint32).astype(np.uint16)
EXACT = {"sqrt": lambda v: v.sqrt(), "abs": lambda v: v.abs(), "neg": lambda v: v.neg()}
ROUTINES = {"exp": lambda v: v.exp(), "sin": lambda v: v.sin(), "cos": lambda v: v.cos(), "tan": lambda v: v.tan(),
            "tanh": lambda v: v.tanh(), "ln": lambda v: v.ln()}


def _layout(dtype):
    """(exponent mask, mantissa mask) of the 16-bit storage type."""
    return (0x7c00, 0x03ff) if dtype.startswith("f16") else (0x7f80, 0x007f)


def _is_nan(bits, dtype):
    e, m = _layout(dtype)
    return ((bits & e) == e) & ((bits & m) != 0)


def _ordered(bits):
    """Bit patterns mapped to integers that count units of the type along the real line."""
    b = bits.astype(np.int32)
    return np.where(b & 0x8000, -(b & 0x7fff), b & 0x7fff)


def _run(hip, dtype, f):
    view = ALL_BITS.view(np.float16) if dtype.startswith("f16") else ALL_BITS
    return hip.apply_fn(hip.buffer(view, dtype), f).read().view(np.uint16)


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f16_pernode", "bf16_pernode"])
@pytest.mark.parametrize("node", sorted(EXACT))
def test_exact_nodes_over_all_inputs(hip, oracle, dtype, node):
    got = _run(hip, dtype, EXACT[node])
    want = oracle.apply_fn(EXACT[node], ALL_BITS, dtype=dtype)
    nan = _is_nan(want, dtype)
    assert np.array_equal(_is_nan(got, dtype), nan), f"{node} over {dtype}: NaN where the oracle has none, or the reverse"
    # The payload of a NaN is outside the contract.  The reference itself is of two minds: `abs` of
    # an f16 goes through f32 and back, which sets the quiet bit of a signalling NaN, `neg` flips
    # the sign bit and leaves it (half crate: from_f32 / Neg; src/number.rs:597-600).
    assert np.array_equal(got[~nan], want[~nan]), f"{node} over {dtype}"


@pytest.mark.parametrize("dtype", ["f16", "bf16", "f16_pernode", "bf16_pernode"])
@pytest.mark.parametrize("node", sorted(ROUTINES))
def test_transcendental_nodes_over_all_inputs(hip, oracle, dtype, node):
    got = _run(hip, dtype, ROUTINES[node])
    want = oracle.apply_fn(ROUTINES[node], ALL_BITS, dtype=dtype)
    e, _ = _layout(dtype)
    nan = _is_nan(want, dtype)
    assert np.array_equal(_is_nan(got, dtype), nan), f"{node} over {dtype}: NaN where the oracle has none, or the reverse"
    inf = ((want & 0x7fff) == e) & ~nan
    assert np.array_equal(got[inf], want[inf]), f"{node} over {dtype}: infinities differ"
    finite = ~nan & ~inf
    assert not (((got & 0x7fff) == e) & finite).any(), f"{node} over {dtype}: infinity where the oracle is finite"
    dist = np.abs(_ordered(got[finite]) - _ordered(want[finite]))
    worst = int(dist.max())
    where = ALL_BITS[finite][int(dist.argmax())]
    assert worst <= 1, f"{node} over {dtype}: {worst} units apart at input bits {where:#06x}"
    # a zero keeps its sign (sin(-0) = -0, tanh(-0) = -0)
    zero = finite & ((want & 0x7fff) == 0)
    exact_zero_inputs = zero & ((ALL_BITS & 0x7fff) == 0)
    assert np.array_equal(got[exact_zero_inputs], want[exact_zero_inputs]), f"{node} over {dtype}: sign of zero"
    assert (dist == 0).mean() > 0.99, f"{node} over {dtype}: only {(dist == 0).mean():.4f} of the results are bit-identical"
