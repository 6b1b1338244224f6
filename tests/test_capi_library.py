"""The C-ABI library loads, exports every symbol the header declares, and its
run-time compilation pipeline produces gfx950 code objects.  No GPU needed."""
import os
import re
import subprocess

import pytest

import custos_amd
from custos_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "custos_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(custos_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = custos_amd.load_library()
    names = declared_functions()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/custos_hip.h but not exported"


def test_binding_covers_the_header():
    assert sorted(capi.PROTOTYPES) == declared_functions()


def test_exported_symbols_are_only_the_c_abi():
    out = subprocess.run(["nm", "-D", "--defined-only", custos_amd.lib_path()], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    assert set(declared_functions()) <= exported


def test_header_is_plain_c():
    src = '#include "custos_hip.h"\nint main(void){ custos_hip_tuning t = {0}; (void)t; return CUSTOS_HIP_OK; }\n'
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only", "-I", os.path.dirname(HEADER), "-x", "c", "-"],
                       input=src, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_no_device_means_error_not_fallback():
    """Without a GPU, creating a device fails with a HIP error or an index error: nothing computes on the CPU."""
    import ctypes as C
    lib = custos_amd.load_library()
    count = C.c_int32(-1)
    rc = lib.custos_hip_device_count(C.byref(count))
    if rc == 0 and count.value > 0:
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    rc = lib.custos_hip_device_create(0, C.byref(h))
    assert rc != 0 and not h.value
    assert capi.last_error(None)
    with pytest.raises(capi.CustosHipError):
        custos_amd.HIP(0)


def test_entry_points_reject_a_null_device():
    """Every entry point that takes a device handle answers a null one with an error code, not a crash."""
    import ctypes as C
    lib = custos_amd.load_library()
    out = C.c_void_p()
    value = C.c_float(1.0)
    calls = [
        lambda: lib.custos_hip_sync(None),
        lambda: lib.custos_hip_capture_begin(None),
        lambda: lib.custos_hip_capture_end(None, C.byref(out)),
        lambda: lib.custos_hip_capture_end_reuse(None, None, C.byref(out)),
        lambda: lib.custos_hip_set_graph_edges(None, capi.GRAPH_EDGES_CHAIN),
        lambda: lib.custos_hip_set_graph_verify(None, 1),
        lambda: lib.custos_hip_fill(None, 256, 4, C.byref(value), 4),
        lambda: lib.custos_hip_clear(None, 256, 4),
        lambda: lib.custos_hip_read(None, C.byref(value), 256, 4),
        lambda: lib.custos_hip_write(None, 256, C.byref(value), 4),
        lambda: lib.custos_hip_graph_edge_count(None, None),
    ]
    for number, call in enumerate(calls):
        assert call() == capi.ERR_INVALID_ARGUMENT, number


@pytest.mark.parametrize("dtype", ["f32", "f64", "f16", "bf16", "i32", "i64", "u8", "i8", "i16", "u16", "u32", "u64",
                                   "f16_pernode", "bf16_pernode"])
def test_offline_compile_every_dtype(dtype):
    text = "((x * 2) + 1)" if dtype[0] in "iu" else "sqrt(abs(((x * 2.0) + 1.0)))"
    assert capi.expr_build_code_object(capi.KIND_APPLY, dtype, text, ["x"]) > 1000
    assert capi.expr_build_code_object(capi.KIND_UNARY_GRAD, dtype, text, ["x"]) > 1000


def test_offline_compile_all_nodes_and_arities():
    text = "pow(min(max((sin(a) + cos(b)), (tan(c) - tanh(d))), exp(a)), (log(abs(b)) / (-(c) * (a >= b))))"
    assert capi.expr_build_code_object(capi.KIND_APPLY, "f32", text, ["a", "b", "c", "d"]) > 1000
    assert capi.expr_build_code_object(capi.KIND_APPLY, "f64", "((a <= b) == c)", ["a", "b", "c"]) > 1000
    fused = "x = sin(x);\nx = (x * 2.0);\nx = (x + 1.0);\nx = max(x, 0.0);\nx = (x - 0.5);\n"
    assert capi.expr_build_code_object(capi.KIND_APPLY, "f32", fused, ["x"]) > 1000


def test_chosen_device_idx_env(monkeypatch):
    lib = custos_amd.load_library()
    monkeypatch.delenv("CUSTOS_HIP_DEVICE_IDX", raising=False)
    assert lib.custos_hip_chosen_device_idx() == 0
    monkeypatch.setenv("CUSTOS_HIP_DEVICE_IDX", "3")
    assert lib.custos_hip_chosen_device_idx() == 3
    monkeypatch.setenv("CUSTOS_HIP_DEVICE_IDX", "junk")
    assert lib.custos_hip_chosen_device_idx() == 0


def test_product_never_imports_the_oracle():
    """The shipped package and library must not reference the CPU oracle."""
    pkg = os.path.join(ROOT, "custos_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "cpu_oracle" not in text and "custos_cpu_oracle" not in text, os.path.join(dirpath, f)


def test_launch_shape_by_bytes_touched():
    """The shape for the knobs a caller leaves open, for a launch that comes after nothing: temporal
    accesses up to the L2 capacity; above, loads past the caches and temporal stores written through at
    once (what a launch wrote last is what the next launch over the same buffers starts on: the largest
    launches alternate their direction).  What the launches before a launch change is tested on the GPU."""
    MiB = 1 << 20
    shape = capi.preferred_shape
    loads = 1 | 64                                         # non-temporal loads, stores written through at once
    assert shape(8 * MiB, 2) == (2, 0, False)              # config 1: 2^20 f32 in, out
    assert shape(32 * MiB, 2) == (2, 0, False)             # what the eight L2s hold together
    assert shape(32 * MiB + 1, 2) == (2, loads, False)
    assert shape(48 * MiB, 3) == (2, loads, False)         # config 5, one recorded level merged
    assert shape(64 * MiB, 4) == (2, loads, False)         # config 5 after element-wise fusing
    assert shape(128 * MiB, 2) == (2, loads, False) and shape(256 * MiB, 2) == (2, loads, False)
    assert shape(257 * MiB, 2) == (2, loads, True)
    assert shape(512 * MiB, 2) == (2, loads, True)         # config 3 forward, the first time
    assert shape(768 * MiB, 3) == (2, loads, True)         # config 3 backward
    assert shape(1024 * MiB, 2) == (2, loads, True)        # config 4
    assert shape(2048 * MiB, 2) == (2, loads, True)        # config 2
    with pytest.raises(capi.CustosHipError):
        shape(1, 0)


def test_launch_shape_by_what_a_launch_revisits_and_writes():
    """The two refinements of the choice: a launch of more than 32 MiB that touches nothing the launch before
    it wrote streams as one-wavefront workgroups with one vector per thread; a kernel that writes through at
    least two pointers more than it reads through keeps its input in the cache instead of its outputs, from
    128 MiB touched on.  The rest of the choice does not move with either."""
    MiB = 1 << 20
    shape = capi.preferred_shape_of
    loads, both, stores = 1 | 64, 3, 2 | 64
    for footprint, n_ops in ((8 * MiB, 2), (32 * MiB, 2), (64 * MiB, 4), (512 * MiB, 2), (2048 * MiB, 2)):
        assert shape(footprint, n_ops)[:3] == capi.preferred_shape(footprint, n_ops)        # revisiting, one output: as before
        assert shape(footprint, n_ops)[3] == 0
    # revisits nothing
    assert shape(32 * MiB, 2, revisits=False) == (2, 0, False, 0)                            # the L2s still hold it
    assert shape(32 * MiB + 1, 2, revisits=False) == (1, loads, False, 64)
    assert shape(48 * MiB, 3, revisits=False) == (1, loads, False, 64)
    assert shape(512 * MiB, 2, revisits=False) == (1, loads, True, 64)                       # config 3 forward after backward
    assert shape(512 * MiB, 2, working_set_bytes=1280 * MiB, revisits=False) == (1, both, True, 64)
    assert shape(768 * MiB, 3, revisits=False) == (1, loads, True, 64)                       # config 3 backward after forward
    assert shape(2048 * MiB, 2, revisits=False) == (1, loads, True, 64)                      # the first launch of an unfused chain
    assert shape(20 * MiB, 2, working_set_bytes=60 * MiB, revisits=False) == (2, loads, False, 0)   # small launches keep 128 x 2
    # its first input is what the launch before it read as well, and it touches nothing that launch wrote
    keep_first = 3 | 64 | 1 << 8                  # everything streams past the cache but input 0
    assert shape(32 * MiB, 2, revisits=2) == (2, 0, False, 0)
    assert shape(512 * MiB, 2, revisits=2) == (1, keep_first, True, 64)                      # y = f(x) into another buffer every time
    assert shape(768 * MiB, 3, revisits=2) == (1, keep_first, True, 64)                      # config 3 backward after forward of the same x
    assert shape(48 * MiB, 2, revisits=2) == (1, keep_first, False, 64)                      # (alternating from 256 MiB on, as ever)
    assert shape(256 * MiB + 1, 2, revisits=2) == (1, keep_first, True, 64)
    assert shape(2048 * MiB, 2, revisits=2) == (1, keep_first, True, 64)
    assert shape(20 * MiB, 2, working_set_bytes=60 * MiB, revisits=2) == (2, loads, False, 0)
    # three or more pointers over more than 768 MiB: one-wavefront workgroups whatever came before
    assert shape(1024 * MiB, 3) == (1, loads, True, 64)
    assert shape(2048 * MiB, 4) == (1, loads, True, 64)
    assert shape(768 * MiB + 1, 3) == (1, loads, True, 64)
    assert shape(768 * MiB, 3) == (2, loads, True, 0)                                        # config 3 backward, repeated by itself
    assert shape(2048 * MiB, 2) == (2, loads, True, 0)                                       # two pointers keep 128 x 2
    # mostly writes
    assert shape(4096 * MiB, 4, n_written=3) == (1, stores, True, 64)                        # config 2 recorded unfused: 1R + 3W
    assert shape(256 * MiB, 4, n_written=3) == (2, stores, False, 0)
    assert shape(128 * MiB, 4, n_written=3) == (2, stores, False, 0)
    assert shape(127 * MiB, 4, n_written=3) == (2, loads, False, 0)                          # below: the usual policy is ahead
    assert shape(96 * MiB, 6, n_written=3) == (2, loads, False, 0)                           # config 5 as recorded: 3R + 3W
    assert shape(1024 * MiB, 4, n_written=2) == (1, loads, True, 64)                         # 2R + 2W
    assert shape(768 * MiB, 4, n_written=2) == (2, loads, True, 0)
    assert shape(1024 * MiB, 3, n_written=2) == (1, loads, True, 64)                         # 1R + 2W: one more, not two
    assert shape(1280 * MiB, 5, n_written=2) == (1, loads, True, 64)                         # config 3 joined: 3R + 2W
    assert shape(1536 * MiB, 6, n_written=5) == (1, stores, True, 64)                        # 1R + 5W
    assert shape(512 * MiB, 6, n_written=5) == (2, stores, True, 0)
    assert shape(1536 * MiB, 6, n_written=5, revisits=False) == (1, stores, True, 64)
    with pytest.raises(capi.CustosHipError):
        shape(1 * MiB, 2, n_written=3)


def test_operands_of_different_lengths_are_rejected_on_the_host():
    """A shorter operand would be read or written beyond its end on the device: the binding checks
    lengths and element types before anything reaches the library (no device needed to see it)."""
    from custos_amd.device import HIP, Buffer
    dev = object.__new__(HIP)          # no library call is made before the checks
    dev.lib, dev.handle = None, None
    a, b = Buffer(dev, 256, 8, "f32", owned=False), Buffer(dev, 512, 7, "f32", owned=False)
    h = Buffer(dev, 1024, 8, "f16", owned=False)
    ident = lambda *v: v[0]
    for call in (lambda: dev.apply_fn(a, ident, out=b), lambda: dev.apply_fn2(a, b, ident), lambda: dev.apply_fn2(a, a, ident, out=b),
                 lambda: dev.apply_fn_n([a, a, b], ident), lambda: dev.apply_fn_n([a, a], ident, out=b),
                 lambda: dev.fused_apply_fn(a, [ident], out=b), lambda: dev.add_unary_grad(a, b, a, ident),
                 lambda: dev.add_unary_grad(a, a, b, ident), lambda: dev.apply_fn2(a, h, ident)):
        with pytest.raises(ValueError):
            call()


@pytest.mark.parametrize("dtype", ["f32", "f64", "f16", "bf16", "i32", "i64", "u8", "i8", "i16", "u16", "u32", "u64",
                                   "f16_pernode", "bf16_pernode"])
def test_chain_kernels_compile_for_every_dtype(dtype):
    """The kernel a graph build makes of a producer and its consumers: several expressions, several outputs."""
    last = "max(v0, v1)" if dtype[0] in "iu" else "(sqrt(abs(v0)) * 0.3)"
    stages = [("(v0 * v1)", [0, 1], 0), ("(v0 + v1)", [-1, 2], 1), (last, [-2, -1] if dtype[0] in "iu" else [-2], 2)]
    text, size = capi.chain_emit(dtype, stages, 3, 3, compile_it=True)
    assert size > 1000
    entry = re.search(r"custos_chain_\w+", text).group(0)
    for suffix in ("(", "_batched(", "_ragged("):
        assert entry + suffix in text
    # three inputs, three outputs; a stage takes an earlier stage's value as it was stored
    assert "const S* in2, S* out0, S* out1, S* out2" in text
    assert "const S t1 = custos_store(custos_expr_s1(r0, e2 CUSTOS_KC_ARG));" in text


def test_chain_kernels_take_literals_as_parameters():
    """Stages whose own kernels take their literals as launch parameters keep doing so in the joined
    kernel: one block of scalars, every stage's slots behind those of the stages before it."""
    stages = [("((v0 * 0.5) + 0.75)", [0], 0), ("(v0 / 3.0)", [-1], 1), ("max(v0, 0.25)", [-2], 2)]
    for dtype in ("f32", "f64", "f16", "bf16_pernode", "i32", "u8"):
        st = stages if dtype[0] not in "iu" else [("((v0 * 5) + 7)", [0], 0), ("(v0 / 3)", [-1], 1), ("max(v0, 2)", [-2], 2)]
        text, size = capi.chain_emit(dtype, st, 1, 3, compile_it=True, literals_as_parameters=True)
        assert size > 1000
        # integer divisors stay in the code (a division by a known value is a multiplication)
        n_params = 3 if dtype[0] in "iu" else 4
        assert f"struct CustosConsts {{ C c[{n_params}]; }};" in text
        assert "kc.c[2]" in text and f"kc.c[{n_params - 1}]" in text and f"kc.c[{n_params}]" not in text
    in_code, _ = capi.chain_emit("f32", stages, 1, 3)
    assert "CustosConsts {" not in in_code and "kc.c[" not in in_code


def test_chain_kernel_stores_what_is_overwritten_only_once():
    """x = f(x); x = g(x) in place: the first store is dropped, the second stage reads the first value from a register."""
    text, _ = capi.chain_emit("f32", [("(v0 * 2.0)", [0], -1), ("(v0 + 1.0)", [-1], 0)], 1, 1)
    assert "o[0] = t1;" in text and "o[0] = t0;" not in text and "S* out1" not in text


def test_chain_emit_rejects_malformed_stages():
    ok = [("(v0 * v1)", [0, 1], 0)]
    bad = [
        ([("(v0 * v1)", [0, 2], 0)], 2, 1),            # reads an input that does not exist
        ([("(v0 * v1)", [0, -1], 0)], 2, 1),           # reads itself
        ([("(v0 * v1)", [0, 1], 1)], 2, 1),            # writes an output that does not exist
        ([("(v0 * ", [0], 0)], 1, 1),                  # not an expression
        (ok * 9, 2, 1),                                # too many stages
        (ok, 0, 1), (ok, 2, 0), (ok, 9, 1), (ok, 2, 7),
    ]
    for stages, n_in, n_out in bad:
        with pytest.raises(capi.CustosHipError):
            capi.chain_emit("f32", stages, n_in, n_out)
    with pytest.raises(capi.CustosHipError):
        capi.chain_emit("i32", [("sin(v0)", [0], 0)], 1, 1)    # no such node over integers


def _operand_sets_answer(rows, written, length):
    """What the checks of a merged launch must say, pair by pair."""
    for row in rows:
        if any(a == 0 or a % 16 for a in row):
            return capi.ERR_INVALID_ARGUMENT
    for row in rows:
        out = row[written]
        if any(i != written and a != out and a < out + length and out < a + length for i, a in enumerate(row)):
            return capi.ERR_BAD_OVERLAP
    for s, row in enumerate(rows):
        out = row[written]
        for t, other in enumerate(rows):
            if t != s and any(a < out + length and out < a + length for a in other):
                return capi.ERR_BAD_OVERLAP
    return 0


def test_operand_checks_of_merged_launches_against_all_pairs():
    """The linear-time operand checks (host only) against the comparison of every pair of operands, on
    random tables dense enough that about half of them hold a conflict, and on the edge cases: operands
    exactly one length apart, an output equal to an input, inputs shared between rows, rows that meet
    at the boundary of the pieces the check cuts memory into."""
    import ctypes as C
    import random
    lib = capi.load_library()

    def answer(rows, written, length):
        flat = (C.c_uint64 * (len(rows) * len(rows[0])))(*[a for row in rows for a in row])
        return lib.custos_hip_check_operand_sets(flat, len(rows[0]), len(rows), written, length)

    base = 0x7F0000000000
    assert answer([[base, base + 4096], [base + 64, base + 4096 + 64]], 1, 64) == 0                       # exactly one length apart
    assert answer([[base, base + 4096], [base + 48, base + 4096 + 64]], 1, 64) == 0                       # inputs may overlap
    assert answer([[base, base + 4096], [base + 64, base + 4096 + 48]], 1, 64) == capi.ERR_BAD_OVERLAP    # outputs may not
    assert answer([[base, base], [base + 64, base + 64]], 1, 64) == 0                                     # out == in
    assert answer([[base, base + 16]], 1, 64) == capi.ERR_BAD_OVERLAP                                     # partial, inside a row
    assert answer([[base, base + 4096], [base + 4096 + 16, base + 8192]], 1, 64) == capi.ERR_BAD_OVERLAP  # reads another row's output
    assert answer([[base, base + 4096], [base + 4096 - 48, base + 8192]], 1, 64) == capi.ERR_BAD_OVERLAP  # ... from the piece before
    assert answer([[base, base + 4096 + 16], [base + 4096 + 64, base + 8192]], 1, 64) == capi.ERR_BAD_OVERLAP  # ... from the piece after
    assert answer([[base + 8, base + 4096]], 1, 64) == capi.ERR_INVALID_ARGUMENT
    assert answer([[0, base + 4096]], 1, 64) == capi.ERR_INVALID_ARGUMENT
    assert answer([[16, 4096]], 1, 48) == 0                                                               # the first piece of memory
    rng = random.Random(5)
    seen = {0: 0, capi.ERR_BAD_OVERLAP: 0}
    for case in range(600):
        n_ptrs = rng.choice([2, 3, 4])
        written = rng.choice([n_ptrs - 1, 1]) if n_ptrs == 3 else n_ptrs - 1
        n_sets = rng.randint(1, 40)
        length = 16 * rng.randint(1, 12)
        room = length * n_sets * n_ptrs * rng.choice([1, 2, 4, 40]) // 16
        rows = []
        for s in range(n_sets):
            row = [base + 16 * rng.randrange(room) for _ in range(n_ptrs)]
            if rng.random() < 0.2:
                row[0] = row[written]                          # in place
            rows.append(row)
        if rng.random() < 0.5:
            # tables made valid on purpose: outputs spaced out behind the room of the inputs
            at = base + 16 * room + 4096
            for s, row in enumerate(rows):
                row[written] = at
                at += length + 16 * rng.randrange(3)
                if rng.random() < 0.2:
                    row[0] = row[written]
        want = _operand_sets_answer(rows, written, length)
        assert answer(rows, written, length) == want, (case, rows, written, length)
        seen[want] += 1
    assert seen[0] > 100 and seen[capi.ERR_BAD_OVERLAP] > 100, seen
