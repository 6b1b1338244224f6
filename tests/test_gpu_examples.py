"""The C++ usage examples run on the device and report what they checked themselves."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("name, expect", [
    ("lazy_and_fusing", "1 kernel node(s) in the replayed graph"),
    ("unary_autograd", "d/dx"),
    ("modules_usage", "ok"),
])
def test_example_runs(name, expect):
    exe = os.path.join(ROOT, "examples", name)
    if not os.path.exists(exe):
        pytest.fail(f"{exe} is not built (make -C examples)")
    proc = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout[-500:] + proc.stderr[-500:]
    assert expect in proc.stdout
    assert "FAIL" not in proc.stdout and "mismatch" not in proc.stdout.lower()
