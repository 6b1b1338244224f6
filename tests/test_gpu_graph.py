"""Capture once / replay many through the C ABI (the `Lazy` run of a GPU device)."""
import numpy as np
import pytest

from custos_amd import capi, synth
from tests.helpers import assert_bits_equal

pytestmark = pytest.mark.gpu


def _add_add_mul(hip, lhs, rhs, out):
    """The op sequence of src/devices/cuda/lazy.rs:96-145: out = lhs+rhs; rhs = out+lhs; lhs = out*rhs."""
    add = lambda p, q: p.add(q)
    mul = lambda p, q: p.mul(q)
    hip.apply_fn2(lhs, rhs, add, out=out)
    hip.apply_fn2(out, lhs, add, out=rhs)
    hip.apply_fn2(out, rhs, mul, out=lhs)


def test_lazy_run_reference_vectors(hip):
    # src/devices/cuda/lazy.rs:96-145
    lhs = hip.buffer([1, 2, 3, 4, 5, 6], "i32")
    rhs = hip.buffer([1, 2, 3, 4, 5, 6], "i32")
    out = hip.alloc(6, "i32")
    hip.capture_begin()
    assert hip.is_capturing()
    _add_add_mul(hip, lhs, rhs, out)
    # recorded, not run: reads while recording see the old contents
    assert out.read().tolist() == [0] * 6
    assert lhs.read().tolist() == [1, 2, 3, 4, 5, 6]
    assert rhs.read().tolist() == [1, 2, 3, 4, 5, 6]
    graph = hip.capture_end()
    assert not hip.is_capturing()
    assert graph.kernel_nodes == 3
    graph.launch()
    hip.sync()
    assert out.read().tolist() == [2, 4, 6, 8, 10, 12]
    assert rhs.read().tolist() == [3, 6, 9, 12, 15, 18]
    assert lhs.read().tolist() == [6, 24, 54, 96, 150, 216]
    graph.destroy()


def test_lazy_run_multiple_times(hip):
    # src/devices/cuda/lazy.rs:148-196: ten runs with the inputs rewritten before each
    lhs = hip.buffer([1, 2, 3, 4, 5, 6], "i32")
    rhs = hip.buffer([1, 2, 3, 4, 5, 6], "i32")
    out = hip.alloc(6, "i32")
    hip.capture_begin()
    out.clear()              # a clear is recorded as a kernel node, too
    _add_add_mul(hip, lhs, rhs, out)
    graph = hip.capture_end()
    assert graph.kernel_nodes == 4
    for _ in range(10):
        lhs.write([1, 2, 3, 4, 5, 6])
        rhs.write([1, 2, 3, 4, 5, 6])
        graph.launch()
        hip.sync()
        assert out.read().tolist() == [2, 4, 6, 8, 10, 12]
        assert rhs.read().tolist() == [3, 6, 9, 12, 15, 18]
        assert lhs.read().tolist() == [6, 24, 54, 96, 150, 216]


def test_replays_match_eager_with_eager_work_between(hip, oracle):
    n = 100003
    x = synth.uniform_f32(1, n, -2, 2)
    xb = hip.buffer(x)
    mid = hip.alloc(n)
    out = hip.alloc(n)
    f1 = lambda v: v.mul(1.5).add(0.25)
    f2 = lambda v: v.max(0.0).sub(0.125)
    eager = hip.apply_fn(hip.apply_fn(xb, f1), f2).read()
    assert_bits_equal(eager, oracle.apply_fn(f2, oracle.apply_fn(f1, x)))
    hip.capture_begin()
    hip.apply_fn(xb, f1, out=mid)
    hip.apply_fn(mid, f2, out=out)
    graph = hip.capture_end()
    scratch = hip.alloc(n)
    for i in range(5):
        out.clear()
        hip.apply_fn(xb, lambda v: v.add(float(i)), out=scratch)   # unrelated eager work between replays
        hip.sync()
        graph.launch()
        hip.sync()
        assert_bits_equal(out.read(), eager, f"replay {i}")
        assert_bits_equal(scratch.read(), (x + np.float32(i)).astype(np.float32))


def test_alloc_write_read_while_recording(hip):
    hip.capture_begin()
    b = hip.alloc(1000)                      # allowed while recording, zero-filled right away
    assert not b.read().any()
    b.write(np.arange(1000, dtype=np.float32))
    assert b.read()[999] == 999.0
    out = hip.alloc(1000)
    hip.apply_fn(b, lambda v: v.mul(2.0), out=out)
    assert not out.read().any()
    g = hip.capture_end()
    g.launch()
    hip.sync()
    assert out.read()[999] == 1998.0


def test_capture_state_errors(hip):
    with pytest.raises(capi.CustosHipError) as e:
        hip.capture_end()
    assert e.value.code == capi.ERR_CAPTURE_STATE
    hip.capture_begin()
    with pytest.raises(capi.CustosHipError) as e:
        hip.capture_begin()
    assert e.value.code == capi.ERR_CAPTURE_STATE
    with pytest.raises(capi.CustosHipError) as e:
        hip.sync()
    assert e.value.code == capi.ERR_CAPTURE_STATE
    g = hip.capture_end()
    assert g.kernel_nodes == 0
    g.launch()                               # an empty graph replays fine
    hip.sync()
