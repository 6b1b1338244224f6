"""Shared comparison helpers for the parity tests."""
import numpy as np


def ulp_distance_f32(a, b):
    """Distance in units in the last place between two f32 arrays (monotone integer map)."""
    a = np.ascontiguousarray(a, dtype=np.float32).view(np.int32).astype(np.int64)
    b = np.ascontiguousarray(b, dtype=np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, np.int64(-(2 ** 31)) - a, a)
    b = np.where(b < 0, np.int64(-(2 ** 31)) - b, b)
    return np.abs(a - b)


def ulp_distance_f16(a_bits, b_bits):
    a = np.ascontiguousarray(a_bits, dtype=np.uint16).view(np.int16).astype(np.int64)
    b = np.ascontiguousarray(b_bits, dtype=np.uint16).view(np.int16).astype(np.int64)
    a = np.where(a < 0, np.int64(-(2 ** 15)) - a, a)
    b = np.where(b < 0, np.int64(-(2 ** 15)) - b, b)
    return np.abs(a - b)


def assert_bits_equal(got, want, what=""):
    got = np.ascontiguousarray(got)
    want = np.ascontiguousarray(want)
    assert got.dtype == want.dtype and got.shape == want.shape, (got.dtype, want.dtype, got.shape, want.shape)
    gb = got.view(np.uint8)
    wb = want.view(np.uint8)
    if not np.array_equal(gb, wb):
        # NaNs may differ in payload: compare as "both NaN"
        if got.dtype.kind == "f":
            both_nan = np.isnan(got) & np.isnan(want)
            same = (got.view(f"u{got.itemsize}") == want.view(f"u{want.itemsize}")) | both_nan
            if same.all():
                return
            idx = np.flatnonzero(~same)[:8]
        else:
            idx = np.flatnonzero(got != want)[:8]
        raise AssertionError(f"{what}: {idx.size}+ mismatches, first at {idx.tolist()}: got {got[idx]}, want {want[idx]}")
