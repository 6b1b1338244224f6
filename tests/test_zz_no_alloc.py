"""The allocation-free merged launch (`custos_hip_apply_fn_many_noalloc`) against the entry points
it is a variant of: a recording of the same independent launches, built into a graph (whose merged
node reads its operand table from an allocation of the graph) and replayed.  Two calls in a row on
the shared static table, the second one smaller; results bit for bit equal to the graph's and to
the CPU oracle's."""
import ctypes as C

import numpy as np
import pytest

from custos_amd import Resolve, capi, synth

pytestmark = pytest.mark.gpu


def _graph_result(hip, kernel, arity, rows, n):
    """The same launches recorded, built and replayed (custos_hip_capture_end + custos_hip_graph_launch)."""
    lib, h = hip.lib, hip.handle
    hip.capture_begin()
    for row in rows:
        if arity == "grad":
            capi.check(lib.custos_hip_add_unary_grad(h, kernel, row[0].ptr, row[1].ptr, row[2].ptr, n), h)
        else:
            ins = (C.c_uint64 * (len(row) - 1))(*[b.ptr for b in row[:-1]])
            capi.check(lib.custos_hip_apply_fn_n(h, kernel, ins, len(row) - 1, row[-1].ptr, n), h)
    graph = hip.capture_end()
    assert graph.kernel_nodes == 1  # merged: its kernel reads the table the graph allocated
    graph.launch()
    hip.sync()
    graph.destroy()


def _case(hip, oracle, n_sets, n, seed):
    """a*b+c*0.5 over `n_sets` operand sets of `n` f32 elements: allocation-free call, graph, oracle."""
    expr = lambda a, b, c: a.mul(b).add(c.mul(0.5))
    src = expr(Resolve("a", 0), Resolve("b", 1), Resolve("c", 2)).to_cl_source("f32")
    kernel = hip.compile(capi.KIND_APPLY, "f32", src, ("a", "b", "c"))
    hip.prepare_merged(kernel)                    # compiles and loads: where allocation is allowed
    host = [[synth.uniform_f32(seed + 3 * s + k, n, -2, 2) for k in range(3)] for s in range(n_sets)]
    rows = [[hip.buffer(v) for v in hs] + [hip.alloc(n)] for hs in host]
    rows_graph = [[r[0], r[1], r[2], hip.alloc(n)] for r in rows]
    hip.sync()
    pool_before, compiled_before = hip.pool_stats(), hip.compile_stats()[0]
    hip.apply_fn_many_noalloc(kernel, rows, n)
    # nothing was allocated, taken from the pool or compiled on the way
    assert hip.pool_stats() == pool_before and hip.compile_stats()[0] == compiled_before
    got = [r[3].read() for r in rows]
    _graph_result(hip, kernel, 3, rows_graph, n)
    for s in range(n_sets):
        want = oracle.apply_fn(expr, *host[s])
        assert np.array_equal(got[s].view(np.uint32), want.view(np.uint32)), f"set {s} differs from the CPU oracle"
        assert np.array_equal(got[s].view(np.uint32), rows_graph[s][3].read().view(np.uint32)), f"set {s} differs from the graph"


def test_two_calls_in_a_row_second_smaller(hip, oracle):
    _case(hip, oracle, n_sets=37, n=4096 + 5, seed=100)
    _case(hip, oracle, n_sets=5, n=1000, seed=900)


def test_unary_grad_and_literal_parameters(hip, oracle):
    """Unary-gradient kernels, and kernels that take their literals as launch parameters (the table
    rows then carry the values), through the same static table."""
    n, n_sets = 2048 + 3, 9
    grad = lambda v: v.mul(2.0).add(1.0)
    kernel = hip.compile(capi.KIND_UNARY_GRAD, "f32", grad(Resolve("x")).to_cl_source("f32"), ("x",))
    hip.prepare_merged(kernel)
    xs = [synth.uniform_f32(10 + s, n, -1, 1) for s in range(n_sets)]
    gs = [synth.uniform_f32(40 + s, n, -1, 1) for s in range(n_sets)]
    os_ = [synth.uniform_f32(70 + s, n, -1, 1) for s in range(n_sets)]
    rows = [[hip.buffer(xs[s]), hip.buffer(gs[s]), hip.buffer(os_[s])] for s in range(n_sets)]
    hip.apply_fn_many_noalloc(kernel, rows, n)
    for s in range(n_sets):
        want = oracle.add_unary_grad(grad, xs[s], gs[s], os_[s])
        assert np.array_equal(rows[s][1].read().view(np.uint32), want.view(np.uint32))
    # same structure, other literal values: the second text shares code and carries its values
    hip.set_literal_policy(capi.LITERALS_AS_PARAMETERS)
    try:
        f = lambda v: v.mul(1.25).sub(0.75)
        k2 = hip.compile(capi.KIND_APPLY, "f32", f(Resolve("x")).to_cl_source("f32"), ("x",))
        hip.prepare_merged(k2)
        outs = [hip.alloc(n) for _ in range(n_sets)]
        hip.apply_fn_many_noalloc(k2, [[rows[s][0], outs[s]] for s in range(n_sets)], n)
        for s in range(n_sets):
            want = oracle.apply_fn(f, xs[s])
            assert np.array_equal(outs[s].read().view(np.uint32), want.view(np.uint32))
    finally:
        hip.set_literal_policy(capi.LITERALS_ADAPTIVE)


def test_calls_through_two_handles_take_turns_on_the_table(hip, oracle):
    """Two device handles on one GPU share the GPU's table but launch on streams of their own: a call
    makes its stream wait for the launch of the table's last user before it rewrites the rows.  Long
    grids, so that the other handle's launch is still running when the next call comes."""
    import custos_amd
    other = custos_amd.HIP(0)
    try:
        n, n_sets = (1 << 18) + 7, 24
        f = lambda v: v.mul(3.0).sub(1.0)
        g = lambda v: v.abs().sqrt()
        handles = [(hip, f), (other, g)]
        kernels, rows, hosts = [], [], []
        for i, (dev, fn) in enumerate(handles):
            k = dev.compile(capi.KIND_APPLY, "f32", fn(Resolve("x")).to_cl_source("f32"), ("x",))
            dev.prepare_merged(k)
            xs = [synth.uniform_f32(300 + 50 * i + s, n, -2, 2) for s in range(n_sets)]
            kernels.append(k)
            hosts.append(xs)
            rows.append([[dev.buffer(x), dev.alloc(n)] for x in xs])
        for round_ in range(6):                       # A, B, A, B ... without a wait in between
            for i, (dev, _) in enumerate(handles):
                dev.apply_fn_many_noalloc(kernels[i], rows[i], n)
        for i, (dev, fn) in enumerate(handles):
            for s in range(n_sets):
                want = oracle.apply_fn(fn, hosts[i][s])
                assert np.array_equal(rows[i][s][1].read().view(np.uint32), want.view(np.uint32)), f"handle {i}, set {s}"
    finally:
        other.close()


def test_an_identical_call_finds_its_rows_in_the_table(hip, oracle):
    """A serving loop calls with the same kernel, length and addresses again and again: the rows stay
    in the table and only the launch is issued.  New data in the same buffers is picked up; a call
    with other rows in between, through this handle or another, makes the next one send its rows again."""
    import custos_amd
    n, n_sets = 3000, 17
    f = lambda a, b: a.mul(b).add(0.25)
    kernel = hip.compile(capi.KIND_APPLY, "f32", f(Resolve("a", 0), Resolve("b", 1)).to_cl_source("f32"), ("a", "b"))
    hip.prepare_merged(kernel)
    ins = [[hip.alloc(n), hip.alloc(n)] for _ in range(n_sets)]
    rows = [[a, b, hip.alloc(n)] for a, b in ins]
    other = custos_amd.HIP(0)
    try:
        k_other = other.compile(capi.KIND_APPLY, "f32", "(x * 2.0)", ("x",))
        other.prepare_merged(k_other)
        rows_other = [[other.alloc(64), other.alloc(64)] for _ in range(40)]       # more rows than `rows`: all of them overwritten
        for step in range(6):
            host = [[synth.uniform_f32(7000 + 100 * step + 2 * s + k, n, -2, 2) for k in range(2)] for s in range(n_sets)]
            for s in range(n_sets):
                hip.write(ins[s][0], host[s][0])
                hip.write(ins[s][1], host[s][1])
            if step == 2:
                hip.apply_fn_many_noalloc(kernel, rows[:5], n)                      # other rows through this handle
            if step == 4:
                other.apply_fn_many_noalloc(k_other, rows_other, 64)                # other rows through another handle
                other.sync()
            hip.apply_fn_many_noalloc(kernel, rows, n)
            for s in range(n_sets):
                want = oracle.apply_fn(f, *host[s])
                assert np.array_equal(rows[s][2].read().view(np.uint32), want.view(np.uint32)), f"step {step}, set {s}"
    finally:
        other.close()


def test_limits_and_operand_checks(hip):
    kernel = hip.compile(capi.KIND_APPLY, "f32", "(x * 2.0)", ("x",))
    a, b = hip.alloc(4096), hip.alloc(4096)
    lib, h = hip.lib, hip.handle
    def call(rows, per_set, n):
        flat = (C.c_uint64 * len(rows))(*rows)
        return lib.custos_hip_apply_fn_many_noalloc(h, kernel, flat, per_set, len(rows) // per_set, n)
    # loading code allocates: the entry point for merged launches has to be there before the call
    fresh = hip.compile(capi.KIND_APPLY, "f32", "(tan(x) - 0.4321)", ("x",))    # (an expression no other test uses)
    flat = (C.c_uint64 * 2)(a.ptr, b.ptr)
    assert lib.custos_hip_apply_fn_many_noalloc(h, fresh, flat, 2, 1, 16) == capi.ERR_NOT_PREPARED
    assert "custos_hip_kernel_prepare_merged" in capi.last_error(h)
    hip.prepare_merged(kernel)
    # beyond the static table: 8192 words / 2 addresses per set = 4096 sets
    assert call([a.ptr, b.ptr] * 4097, 2, 16) == capi.ERR_TOO_LARGE
    assert "static operand table" in capi.last_error(h)
    assert call([a.ptr, b.ptr], 3, 16) == capi.ERR_ARITY_MISMATCH
    assert call([a.ptr + 4, b.ptr + 4], 2, 16) == capi.ERR_INVALID_ARGUMENT           # not 16-byte aligned
    assert call([a.ptr, a.ptr + 64], 2, 64) == capi.ERR_BAD_OVERLAP                   # partial overlap in a set
    assert call([a.ptr, b.ptr, a.ptr + 1024, b.ptr + 64], 2, 64) == capi.ERR_BAD_OVERLAP  # two sets write one range
    assert call([a.ptr, b.ptr, b.ptr, a.ptr + 8192], 2, 64) == capi.ERR_BAD_OVERLAP   # a set reads what another writes
    assert call([a.ptr, a.ptr], 2, 64) == 0                                           # exact alias is fine
    hip.capture_begin()
    try:
        assert call([a.ptr, b.ptr], 2, 16) == capi.ERR_CAPTURE_STATE
    finally:
        hip.capture_end().destroy()
    hip.sync()
