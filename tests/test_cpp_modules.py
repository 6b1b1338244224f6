"""Runs the C++ tests of the host-side module stack (tests/cpp).

`host_tests` needs no GPU: expression DSL known answers, the reference's cache
trace vectors, and Base / Lazy / Graph / Autograd on the host test device.
`hip_tests` runs the same module tests on the `HIP` device over the C ABI."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp")
EXAMPLES = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "examples")


def _binary(name, where=HERE):
    path = os.path.join(where, name)
    if not os.path.exists(path):
        subprocess.run(["make", "-C", where, name], check=True, capture_output=True)
    return path


def _run(name, timeout):
    proc = subprocess.run([_binary(name)], capture_output=True, text=True, timeout=timeout)
    tail = "\n".join(proc.stdout.splitlines()[-60:])
    assert proc.returncode == 0, f"{name} failed:\n{tail}\n{proc.stderr[-2000:]}"
    assert "0 failure(s)" in proc.stdout
    return proc.stdout


def test_host_module_stack():
    out = _run("host_tests", 120)
    # the suite really ran: spot-check a few case names
    for case in ("cache_trace_neural_net", "graph_fuse_after_binary_ops", "autograd_lazy_accumulates", "combiner_pow"):
        assert f"[  OK  ] {case}" in out


@pytest.mark.gpu
def test_hip_module_stack():
    out = _run("hip_tests", 300)
    for case in ("hip_lazy_run_replays_one_graph", "hip_fused_chain_is_one_kernel", "graph_fuse_chain_optimized",
                 "autograd_tanh_config"):
        assert f"[  OK  ] {case}" in out


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["lazy_and_fusing", "unary_autograd", "modules_usage"])
def test_examples_run(name):
    proc = subprocess.run([_binary(name, EXAMPLES)], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    if name == "lazy_and_fusing":
        assert "1 kernel node(s)" in proc.stdout and "1 graph build(s)" in proc.stdout
    if name == "modules_usage":
        assert proc.stdout.count(" ok\n") == 6 and "FAILED" not in proc.stdout
