"""The calibration sweep of launch shapes (`python -m custos_amd.calibrate`)."""
import pytest

from custos_amd import calibrate, capi


def test_pinned_shapes_are_valid_tunings():
    shapes = calibrate.pinned_shapes()
    assert len(shapes) == 12 and len({name for name, _ in shapes}) == 12
    for name, (block, unroll, per_cu, policy, direction) in shapes:
        assert block == 0 and per_cu == 0 and unroll in (1, 2) and direction in (1, 2)
        assert policy in (-1, 3, 1 | 64), name


@pytest.mark.gpu
def test_sweep_of_small_launches(hip):
    shapes = [s for s in calibrate.pinned_shapes() if s[0] in ("u2Tf", "u1Wa")]
    cells = list(calibrate.sweep(hip, ("rep1", "grad", "chain", "c3"), sizes_mib=(2,), shapes=shapes, settle_s=0.002))
    assert [(name, mib) for name, mib, _ in cells] == [("rep1", 2), ("grad", 2), ("chain", 2), ("c3", 2)]
    for _, _, rates in cells:
        assert list(rates) == ["auto", "u1Wa", "u2Tf"] and all(50 < v < 100000 for v in rates.values()), rates
    # the sweep leaves every knob open again
    import ctypes as C
    t = capi.Tuning()
    capi.check(hip.lib.custos_hip_get_tuning(hip.handle, C.byref(t)), hip.handle)
    assert (t.unroll, t.nontemporal, t.direction) == (0, 0, 0)
