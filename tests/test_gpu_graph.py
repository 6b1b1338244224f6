"""Capture once / replay many through the C ABI (the `Lazy` run of a GPU device)."""
import numpy as np
import pytest

import custos_amd
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
    # every launch reads what the one before wrote, and writes an operand of an earlier one in
    # place: the three are joined into one kernel (each lane loads before it stores)
    assert graph.kernel_nodes == 1 and graph.fused_launches == 2
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
    assert graph.kernel_nodes == 2      # the clear, and the three launches joined
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
    hip.sync()                               # legal: waits for what was in flight when the recording began
    g = hip.capture_end()
    assert g.kernel_nodes == 0
    g.launch()                               # an empty graph replays fine
    hip.sync()


def test_batched_launch_with_tails_and_mixed_lengths(hip, oracle):
    """Independent launches of one kernel merge into one grid, whatever their lengths
    (a scalar tail per buffer included); unaligned views stay separate nodes."""
    f = lambda v: v.mul(1.5).add(0.25)
    lens = [1003] * 40 + [7] * 5 + [4096] * 3 + [1]
    xs = [synth.uniform_f32(100 + i, n, -2, 2) for i, n in enumerate(lens)]
    bufs = [hip.buffer(x) for x in xs]
    outs = [hip.alloc(n) for n in lens]
    big = hip.buffer(synth.uniform_f32(7, 1003 + 3, -2, 2))
    big_out = hip.alloc(1003 + 3)
    hip.capture_begin()
    for b, o in zip(bufs, outs):
        hip.apply_fn(b, f, out=o)
    hip.apply_fn(big.slice(3, 1006), f, out=big_out.slice(3, 1006))   # same length, not 16-byte aligned
    g = hip.capture_end()
    recorded, kernel_nodes, levels = g.stats()
    assert recorded == len(lens) + 1 and levels == 1
    assert kernel_nodes == 1 + 1          # one grid for all lengths; the unaligned view
    for _ in range(2):
        g.launch()
        hip.sync()
        for x, o in zip(xs, outs):
            assert_bits_equal(o.read(), oracle.apply_fn(f, x))
        assert_bits_equal(big_out.read()[3:], oracle.apply_fn(f, big.read()[3:]))
        assert not big_out.read()[:3].any()


def test_merged_launches_of_different_lengths(hip, oracle):
    """Launches of one kernel over many lengths (multi-tensor apply): one grid with a block
    map; equal lengths alone keep the division-based grid; a launch that fills the chip on its
    own is left out of the merge.  Unary-gradient kernels and 16-bit types merge the same way."""
    f = lambda v: v.mul(0.75).sub(0.5)
    rng = np.random.default_rng(5)
    lens = [int(n) for n in rng.integers(1, 3000, size=200)] + [256, 257, 255, 1024, 1 << 16]
    xs = [synth.uniform_f32(300 + i, n, -4, 4) for i, n in enumerate(lens)]
    bufs = [hip.buffer(x) for x in xs]
    outs = [hip.alloc(n) for n in lens]
    huge_n = 16384 * 1024 + 4096          # more tiles than a merged launch takes
    huge = hip.buffer(synth.uniform_f32(9, huge_n, -1, 1))
    huge_out = hip.alloc(huge_n)
    hip.capture_begin()
    for b, o in zip(bufs, outs):
        hip.apply_fn(b, f, out=o)
    hip.apply_fn(huge, f, out=huge_out)
    g = hip.capture_end()
    assert g.stats() == (len(lens) + 1, 2, 1)
    for _ in range(2):
        for o in outs:
            o.clear()
        g.launch()
        hip.sync()
        for x, o in zip(xs, outs):
            assert_bits_equal(o.read(), oracle.apply_fn(f, x))
        assert_bits_equal(huge_out.read(), oracle.apply_fn(f, huge.read()))
    g.destroy()

    # equal lengths only: the uniform grid, still one node.  (As recorded: eight launches that read
    # the same input are otherwise joined into kernels that load it once, six outputs at most each.)
    for fusing, want_stats in ((False, (8, 1, 1)), (True, (8, 2, 1))):
        hip.set_graph_fusing(fusing)
        hip.capture_begin()
        same = [hip.alloc(lens[0]) for _ in range(8)]
        for o in same:
            hip.apply_fn(bufs[0], f, out=o)
        g = hip.capture_end()
        hip.set_graph_fusing(True)
        assert g.stats() == want_stats
        g.launch()
        hip.sync()
        for o in same:
            assert_bits_equal(o.read(), oracle.apply_fn(f, xs[0]))
        g.destroy()

    # unary gradient, f16 storage, lengths with tails
    d = lambda v: v.mul(2.0)
    glens = [5, 64, 1000, 1001, 4099]
    lhs = [synth.uniform_f32(40 + i, n, -2, 2).astype(np.float16) for i, n in enumerate(glens)]
    og = [synth.uniform_f32(60 + i, n, -1, 1).astype(np.float16) for i, n in enumerate(glens)]
    g0 = [np.full(n, 0.5, np.float16) for n in glens]
    lb = [hip.buffer(a, "f16") for a in lhs]
    ob = [hip.buffer(a, "f16") for a in og]
    gb = [hip.buffer(a, "f16") for a in g0]
    hip.capture_begin()
    for l, gr, o in zip(lb, gb, ob):
        hip.add_unary_grad(l, gr, o, d)
    g = hip.capture_end()
    assert g.stats() == (len(glens), 1, 1)
    g.launch()
    hip.sync()
    for l, gr0, o, gr in zip(lhs, g0, og, gb):
        want = oracle.add_unary_grad(d, l.view(np.uint16), gr0.view(np.uint16), o.view(np.uint16), dtype="f16")
        assert_bits_equal(gr.read().view(np.uint16), want)
    g.destroy()


@pytest.fixture
def checked_graphs(hip):
    """Every graph built inside the test is checked by brute force against the recorded conflicts."""
    hip.set_graph_verify(True)
    yield hip
    hip.set_graph_verify(False)
    hip.set_graph_edges(capi.GRAPH_EDGES_CHAIN)
    hip.set_graph_fusing(True)


EDGE_MODES = {"level joins": capi.GRAPH_EDGES_LEVEL_JOINS, "per node": capi.GRAPH_EDGES_PER_NODE, "chain": capi.GRAPH_EDGES_CHAIN,
              "chain by level": capi.GRAPH_EDGES_CHAIN_BY_LEVEL}


@pytest.mark.parametrize("edges", list(EDGE_MODES))
def test_recorded_dependencies_random(checked_graphs, oracle, edges):
    """Random programs over a small pool of buffers, with in-place updates, views and clears:
    replaying the built graph (ordered by level joins, per-node edges or as one chain; merged launches)
    must equal running the same calls eagerly, bit for bit.  One trial in three uses aligned half-buffer
    views, one views of any offset and length (partial overlaps between operations, scalar launches),
    one whole buffers (chains of launches that join).  The library also checks each graph's ordering by
    brute force."""
    import os
    hip = checked_graphs
    hip.set_graph_edges(EDGE_MODES[edges])
    rng = np.random.default_rng(1234)
    n = 2048
    fns1 = [lambda v: v.mul(1.25).add(0.5), lambda v: v.neg().max(-3.0), lambda v: v.abs().sqrt(), lambda v: v.mul(v).min(9.0)]
    fns2 = [lambda p, q: p.add(q), lambda p, q: p.mul(q).sub(0.125), lambda p, q: p.max(q)]
    fused_launches = 0
    for trial in range(int(os.environ.get("CUSTOS_RANDOM_PROGRAMS", "6"))):   # more for a longer run
        nbuf = 6
        init = [synth.uniform_f32(trial * 10 + i, n, -2, 2) for i in range(nbuf)]
        program = []
        for _ in range(40):
            kind = rng.integers(0, 5)
            if trial % 3 == 1:
                lo = int(rng.integers(0, 1500))
                ln = int(rng.integers(1, n - lo + 1))
            elif trial % 3 == 0:
                lo, ln = int(rng.integers(0, 3)) * 512, 1024     # [lo, lo + 1024) keeps 16-byte phases equal
            else:
                lo, ln = 0, n                                     # whole buffers: most launches join their producers
            if kind == 0:
                program.append(("u", int(rng.integers(len(fns1))), int(rng.integers(nbuf)), int(rng.integers(nbuf)), lo, ln))
            elif kind in (1, 2):
                a, b, o = (int(v) for v in rng.integers(nbuf, size=3))
                program.append(("b", int(rng.integers(len(fns2))), a, b, o, lo, ln))
            elif kind == 3:
                program.append(("g", int(rng.integers(len(fns1))), *(int(v) for v in rng.choice(nbuf, size=3, replace=False)), lo, ln))
            else:
                program.append(("c", int(rng.integers(nbuf)), lo, ln))

        def run(bufs):
            for op in program:
                lo, ln = op[-2], op[-1]
                view = lambda i: bufs[i].slice(lo, lo + ln)
                if op[0] == "u":
                    _, fi, src, dst = op[:4]
                    hip.apply_fn(view(src), fns1[fi], out=view(dst))
                elif op[0] == "b":
                    _, fi, a, b, o = op[:5]
                    if a == b:
                        continue
                    hip.apply_fn2(view(a), view(b), fns2[fi], out=view(o))
                elif op[0] == "g":
                    _, fi, x, g, o = op[:5]
                    hip.add_unary_grad(view(x), view(g), view(o), fns1[fi])
                else:
                    view(op[1]).clear()

        eager = [hip.buffer(x) for x in init]
        run(eager)
        hip.sync()
        want = [b.read() for b in eager]
        run(eager)          # a second replay continues from the first one's results, like a second eager run
        hip.sync()
        want_twice = [b.read() for b in eager]
        # once with producers joined into their consumers (the default), once as recorded
        for fusing in (True, False):
            lazy = [hip.buffer(x) for x in init]
            hip.set_graph_fusing(fusing)
            try:
                hip.capture_begin()
                run(lazy)
                g = hip.capture_end()
            finally:
                hip.set_graph_fusing(True)
            fused_launches += g.fused_launches
            assert fusing or g.fused_launches == 0
            for b, x in zip(lazy, init):
                assert_bits_equal(b.read(), x, "nothing may run while recording")
            g.launch()
            hip.sync()
            for i, b in enumerate(lazy):
                assert_bits_equal(b.read(), want[i], f"trial {trial} fusing {fusing} buffer {i} (levels {g.stats()})")
            g.launch()
            hip.sync()
            for i, b in enumerate(lazy):
                assert_bits_equal(b.read(), want_twice[i], f"trial {trial} fusing {fusing} second replay, buffer {i}")
            g.destroy()
    assert fused_launches > 0, "no trial joined a producer with its consumer"


def test_per_node_edges_let_independent_chains_run_apart(checked_graphs, oracle):
    """Two chains over different buffers with different kernels, one twice as long as the other,
    then a caller-written kernel (unknown memory use: ordered against everything) and one more
    launch per chain.  With an edge per dependency no node waits for the other chain (fewer edges
    than level joins need); as one chain the nodes follow each other in level order.  The same
    bits in every mode, replay after replay."""
    hip = checked_graphs
    hip.set_graph_fusing(False)         # this test is about the nodes as recorded (joined, each chain would be one kernel)
    n = 30011
    x, y = synth.uniform_f32(31, n, -2, 2), synth.uniform_f32(32, n, -2, 2)
    f = lambda v: v.mul(1.5).sub(0.25)
    h = lambda v: v.abs().add(0.5)
    scale = """extern "C" __global__ void halve(float* p, unsigned long long n) {
        unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x;
        if (i < n) p[i] = p[i] * 0.5f;
    }"""

    def program(a, b):
        for _ in range(4):
            hip.apply_fn(a, f, out=a)
        for _ in range(2):
            hip.apply_fn(b, h, out=b)
        hip.launch_kernel(scale, "halve", ((n + 255) // 256, 1, 1), (256, 1, 1), 0, [a, np.uint64(n)])
        hip.apply_fn(a, h, out=a)
        hip.apply_fn(b, f, out=b)

    ea, eb = hip.buffer(x), hip.buffer(y)
    edges = {}
    hip.set_graph_direct_replay(0)
    try:
        for per_node, mode in EDGE_MODES.items():
            hip.set_graph_edges(mode)
            a, b = hip.buffer(x), hip.buffer(y)
            hip.capture_begin()
            program(a, b)
            g = hip.capture_end()
            assert g.stats() == (9, 9, 6)
            edges[per_node] = g.edge_count()
            ca, cb = hip.buffer(x), hip.buffer(y)
            for replay in range(3):
                g.launch()
                program(ca, cb)
                hip.sync()
                assert_bits_equal(a.read(), ca.read(), f"per_node={per_node} replay {replay}, first chain")
                assert_bits_equal(b.read(), cb.read(), f"per_node={per_node} replay {replay}, second chain")
            g.destroy()
    finally:
        hip.set_graph_direct_replay(4)
    # per-node: 3 edges inside the first chain, 1 inside the second, 2 into the caller-written kernel, 2 out of it
    assert edges["per node"] == 8
    assert edges["chain"] == 8          # nine nodes one after the other
    assert edges["chain by level"] == 8
    assert edges["level joins"] == 11
    want = x
    for _ in range(4):
        want = oracle.apply_fn(f, want)
    want = oracle.apply_fn(h, want * np.float32(0.5))
    program(ea, eb)
    hip.sync()
    assert_bits_equal(ea.read(), want)


@pytest.mark.parametrize("edges", ["chain", "chain by level", "per node"])
def test_large_launches_in_recording_order(checked_graphs, oracle, edges):
    """Recordings with launches of 8 MiB and more: one chain follows the recording where the
    dependencies allow.  Random programs over four buffers of 2^20 elements (in-place updates, two-operand
    launches between buffers, clears, a caller-written kernel), every graph checked by the library's ordering
    check, replays compared with eager execution bit for bit."""
    hip = checked_graphs
    hip.set_graph_edges(EDGE_MODES[edges])
    hip.set_graph_direct_replay(0)
    n = 1 << 20
    rng = np.random.default_rng(77)
    fns1 = [lambda v: v.mul(1.25).add(0.5), lambda v: v.neg().max(-3.0), lambda v: v.abs().sqrt()]
    fns2 = [lambda p, q: p.add(q), lambda p, q: p.mul(q).sub(0.125)]
    halve = """extern "C" __global__ void halve(float* p, unsigned long long n) {
        unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x;
        if (i < n) p[i] = p[i] * 0.5f;
    }"""
    try:
        import os
        for trial in range(int(os.environ.get("CUSTOS_LARGE_RANDOM_PROGRAMS", "4"))):   # more for a longer run
            init = [synth.uniform_f32(200 + trial * 4 + i, n, -2, 2) for i in range(4)]
            program = []
            for chain in rng.permutation(4):                      # chain by chain, as user code records
                for _ in range(int(rng.integers(1, 4))):
                    program.append(("u", int(rng.integers(len(fns1))), int(chain)))
            for _ in range(3):                                     # then work across the chains
                a, b, o = (int(v) for v in rng.choice(4, size=3, replace=False))
                program.append(("b", int(rng.integers(len(fns2))), a, b, o))
            program.insert(int(rng.integers(len(program))), ("k", int(rng.integers(4))))
            program.append(("c", int(rng.integers(4))))
            program.append(("u", 0, int(rng.integers(4))))

            def run(bufs):
                for op in program:
                    if op[0] == "u":
                        hip.apply_fn(bufs[op[2]], fns1[op[1]], out=bufs[op[2]])
                    elif op[0] == "b":
                        hip.apply_fn2(bufs[op[2]], bufs[op[3]], fns2[op[1]], out=bufs[op[4]])
                    elif op[0] == "k":
                        hip.launch_kernel(halve, "halve", ((n + 255) // 256, 1, 1), (256, 1, 1), 0, [bufs[op[1]], np.uint64(n)])
                    else:
                        bufs[op[1]].clear()

            eager = [hip.buffer(x) for x in init]
            lazy = [hip.buffer(x) for x in init]
            hip.capture_begin()
            run(lazy)
            g = hip.capture_end()
            for replay in range(2):
                run(eager)
                g.launch()
                hip.sync()
                for i in range(4):
                    assert_bits_equal(lazy[i].read(), eager[i].read(), f"{edges}, trial {trial}, replay {replay}, buffer {i}")
            g.destroy()
    finally:
        hip.set_graph_direct_replay(4)


def test_ordering_check_accepts_merged_and_fenced_graphs(checked_graphs):
    """The brute-force check runs on a graph of merged launches in every edge mode."""
    hip = checked_graphs
    n, count = 4096, 64
    xs = [hip.buffer(synth.uniform_f32(100 + i, n, 0, 1)) for i in range(count)]
    ts = [hip.alloc(n) for _ in range(count)]
    for fusing in (False, True):
        hip.set_graph_fusing(fusing)
        for mode in EDGE_MODES.values():
            hip.set_graph_edges(mode)
            hip.capture_begin()
            for x, t in zip(xs, ts):
                hip.apply_fn(x, lambda v: v.mul(2.0), out=t)
                hip.apply_fn(t, lambda v: v.add(1.0), out=x)
            g = hip.capture_end()
            assert g.stats() == ((2 * count, 1, 1) if fusing else (2 * count, 2, 2))
            g.launch()
            hip.sync()
            g.destroy()


def test_a_repeated_recording_reuses_its_graph(hip, oracle):
    """A caller that records its program again before every run (the reference's Lazy::run does)
    gets the graph it already has as long as the recording is the same; another length, another
    buffer, another literal or another graph setting builds a new one."""
    n = 9000
    x = synth.uniform_f32(41, n, -2, 2)
    a, b, c = hip.buffer(x), hip.alloc(n), hip.alloc(n)
    f = lambda v: v.mul(1.5).sub(0.25)

    def record(src=a, dst=c, length=n, fn=f):
        hip.capture_begin()
        hip.apply_fn(src.slice(0, length), lambda v: v.abs(), out=b.slice(0, length))
        hip.apply_fn(b.slice(0, length), fn, out=dst.slice(0, length))

    record()
    g = hip.capture_end_reuse(None)
    want = oracle.apply_fn(f, np.abs(x))
    for run in range(3):
        c.clear()
        record()
        again = hip.capture_end_reuse(g)
        assert again is g, f"run {run}: the same recording built a new graph"
        assert not hip.is_capturing()
        again.launch()
        hip.sync()
        assert_bits_equal(c.read(), want)
    d = hip.alloc(n)
    changes = {"shorter": dict(length=n - 1), "other output": dict(dst=d), "other literal": dict(fn=lambda v: v.mul(1.5).sub(0.5))}
    for what, change in changes.items():
        record(**change)
        other = hip.capture_end_reuse(g)
        assert other is not g, what
        other.launch()
        hip.sync()
        other.destroy()
    try:
        hip.set_graph_direct_replay(0)
        record()
        other = hip.capture_end_reuse(g)
        assert other is not g, "graph settings changed"
        other.destroy()
    finally:
        hip.set_graph_direct_replay(4)
    c.clear()
    record()
    assert hip.capture_end_reuse(g) is g
    g.launch()
    hip.sync()
    assert_bits_equal(c.read(), want)
    g.destroy()


def test_graph_settings_and_reuse_reject_bad_calls(hip):
    import ctypes as C
    out = C.c_void_p()
    assert hip.lib.custos_hip_capture_end_reuse(hip.handle, None, C.byref(out)) == capi.ERR_CAPTURE_STATE   # not recording
    assert hip.lib.custos_hip_set_graph_edges(hip.handle, 4) == capi.ERR_INVALID_ARGUMENT
    assert hip.lib.custos_hip_set_graph_edges(hip.handle, -1) == capi.ERR_INVALID_ARGUMENT
    other = custos_amd.HIP(0)
    try:
        other.capture_begin()
        theirs = other.capture_end()
        hip.capture_begin()
        try:
            rc = hip.lib.custos_hip_capture_end_reuse(hip.handle, theirs.handle, C.byref(out))
            assert rc == capi.ERR_INVALID_ARGUMENT          # a graph of another device
            assert hip.is_capturing()                        # and the recording is still open
        finally:
            hip.capture_end().destroy()
        theirs.destroy()
    finally:
        other.close()


def test_lazy_run_sequence_of_an_unmodified_lazy_module(hip, oracle):
    """The call sequence of a device under the reference's own Lazy module (src/modules/lazy.rs:190-197,
    src/devices/cuda/lazy.rs:31-72): recording starts when the device is set up, buffers are allocated and
    written while it records, every run calls all operations again and then the device's run, results are
    read while the next recording is already open.  Every operation must run exactly once per run."""
    n = 5000
    x = synth.uniform_f32(51, n, 0.5, 2)
    hip.capture_begin()                                  # lazy_setup
    try:
        a, acc = hip.buffer(x), hip.alloc(n)             # allocation and writes execute at once
        graph = None
        for run in range(1, 5):
            hip.apply_fn2(acc, a, lambda p, q: p.add(q), out=acc)      # call_lazily: recorded, not run
            new = hip.capture_end_reuse(graph)                          # LazyRun::run
            assert graph is None or new is graph
            graph = new
            graph.launch()
            hip.sync()
            hip.capture_begin()
            assert_bits_equal(acc.read(), (x * np.float32(run)).astype(np.float32), f"run {run}")   # read while recording
    finally:
        hip.capture_end().destroy()
    graph.destroy()


def test_a_recording_that_repeats_the_one_before_and_then_does_not(hip, oracle):
    """A recording that repeats the previous one launch for launch is compared while it is made and
    stores nothing; where it stops repeating -- another operand in the middle, fewer launches, more
    launches, a clear or a copy between them, the graph of the previous run destroyed -- it becomes an
    ordinary recording with the part that matched in front.  Every variation against the CPU oracle."""
    n, k = 3000, 12
    f = lambda p, q: p.mul(q).add(0.5)
    g = lambda v: v.abs().sqrt()
    xs = [synth.uniform_f32(600 + i, n, -2, 2) for i in range(k + 1)]
    a = [hip.buffer(x) for x in xs]
    t = [hip.alloc(n) for _ in range(k)]
    y = [hip.alloc(n) for _ in range(k)]

    def record(pairs, extra=None):
        """t[i] = f(a[i], a[j]); y[i] = g(t[i]) for (i, j) in pairs; `extra(i)` may record something in between."""
        for i, j in pairs:
            hip.apply_fn2(a[i], a[j], f, out=t[i])
            if extra:
                extra(i)
            hip.apply_fn(t[i], g, out=y[i])

    def check(pairs, cleared=(), filled={}):
        hip.sync()
        for i, j in pairs:
            want_t = oracle.apply_fn(f, xs[i], xs[j])
            assert_bits_equal(t[i].read(), want_t, f"t[{i}]")
            want_y = np.zeros(n, dtype=np.float32) if i in cleared else oracle.apply_fn(g, want_t)
            if i in filled:
                want_y = np.broadcast_to(np.asarray(filled[i], dtype=np.float32), (n,))
            assert_bits_equal(y[i].read(), want_y, f"y[{i}]")

    zeros = np.zeros(n, dtype=np.float32)

    def reset():
        for b in t + y:
            b.write(zeros)                              # (a write executes at once; a clear would be recorded)

    same = [(i, i + 1) for i in range(k)]
    hip.capture_begin()
    try:
        record(same)
        graph = hip.capture_end_reuse(None)
        graph.launch()
        hip.capture_begin()
        check(same)
        builds = 1
        def run(pairs, expect_same, extra=None, cleared=(), filled={}):
            nonlocal graph, builds
            reset()
            before = hip.capture_stats()
            record(pairs, extra)
            new = hip.capture_end_reuse(graph)
            assert (new is graph) == expect_same, (pairs, expect_same)
            after = hip.capture_stats()
            # a repeated recording is recognised while it is made, a new one builds a graph
            assert (after[0] - before[0], after[1] - before[1], after[2] - before[2]) == ((1, 0, 0) if expect_same else (0, 0, 1))
            if new is not graph:
                graph.destroy()
                graph = new
                builds += 1
            graph.launch()
            hip.capture_begin()
            check(pairs, cleared, filled)
        run(same, True)
        run(same, True)
        middle = [(i, (i + 2) % (k + 1)) if i == 5 else (i, i + 1) for i in range(k)]
        run(middle, False)                              # another operand in launch 10 of 24
        run(middle, True)
        run(same, False)
        run(same[:7], False)                            # stops early
        run(same[:7], True)
        run(same, False)                                # goes on after the previous one ended
        run(same, True)
        # a recorded clear of y[2] between the two launches of buffer 3: it follows the launch that wrote y[2]
        run(same, False, extra=lambda i: y[2].clear() if i == 3 else None, cleared=(2,))
        run(same, True, extra=lambda i: y[2].clear() if i == 3 else None, cleared=(2,))
        run(same, False, extra=lambda i: y[1].clear() if i == 3 else None, cleared=(1,))     # another buffer cleared
        run(same, False, extra=lambda i: hip.fill(y[1], 2.5) if i == 3 else None, filled={1: 2.5})   # another value
        run(same, True, extra=lambda i: hip.fill(y[1], 2.5) if i == 3 else None, filled={1: 2.5})
        # a recorded copy is compared like a launch (it is one, of the identity kernel)
        run(same, False, extra=lambda i: hip.copy(y[0], a[4]) if i == 3 else None, filled={0: xs[4]})
        run(same, True, extra=lambda i: hip.copy(y[0], a[4]) if i == 3 else None, filled={0: xs[4]})
        # a launch of caller-written source is compared by its kernel, its shape and its argument values
        scale = '''extern "C" __global__ void scale(float* p, float by, int n) {
            int i = blockIdx.x * blockDim.x + threadIdx.x;
            if (i < n) p[i] *= by;
        }'''
        def scaled(i, by):
            if i == 3:
                hip.launch_kernel1d(n, scale, "scale", [y[0], by, n])
        y0 = oracle.apply_fn(g, oracle.apply_fn(f, xs[0], xs[1]))
        run(same, False, extra=lambda i: scaled(i, 2.0), filled={0: y0 * np.float32(2.0)})
        run(same, True, extra=lambda i: scaled(i, 2.0), filled={0: y0 * np.float32(2.0)})
        run(same, False, extra=lambda i: scaled(i, 4.0), filled={0: y0 * np.float32(4.0)})    # another argument value
        run(same, False)
        # the first launch already differs
        other = [(0, 2)] + same[1:]
        run(other, False)
        # the graph of the run before is gone: the next recording is compared with nothing
        graph.destroy()
        graph = None
        reset()
        record(same)
        graph = hip.capture_end_reuse(None)
        graph.launch()
        hip.capture_begin()
        check(same)
        run(same, True)
    finally:
        hip.capture_end().destroy()
    if graph is not None:
        graph.destroy()


def test_recording_begins_without_a_wait_and_immediate_work_takes_it(hip):
    """The same sequence with the run's wait deferred: the graph is launched, the next recording begins
    while it is still running, and what executes at once during a recording (a read, a write, an
    allocation with its zero fill, a wait) is ordered behind it."""
    n = (1 << 24) + 5
    ones = np.ones(n, dtype=np.int32)
    hip.capture_begin()
    try:
        step, acc = hip.buffer(ones, "i32"), hip.buffer(np.zeros(n, dtype=np.int32), "i32")
        graph, runs = None, 0
        def run(times):
            nonlocal graph, runs
            for _ in range(times):
                hip.apply_fn2(acc, step, lambda p, q: p.add(q), out=acc)
                new = hip.capture_end_reuse(graph)
                assert graph is None or new is graph
                graph = new
                graph.launch()                       # no wait
                hip.capture_begin()
                runs += 1
        run(6)
        got = acc.read()                             # a read while recording waits for the six launches
        assert (got == runs).all(), (got.min(), got.max(), runs)
        run(6)
        step.write(ones * 10)                        # so does a write: the launches before it added 1 each
        run(2)
        hip.sync()                                   # and a wait
        got = acc.read()
        assert (got == 12 + 20).all(), (got.min(), got.max())
        # an allocation while recording: the block of a buffer freed with launches still reading it
        # comes back from the pool and is zero-filled outside the compute stream's order
        step.write(ones)
        run(6)
        freed = acc.ptr
        acc.free()
        again = hip.alloc(n, dtype="i32")
        assert again.ptr == freed
        got = again.read()
        assert not got.any(), "the zero fill ran while a launch was still writing the block"
    finally:
        hip.capture_end().destroy()
    if graph is not None:
        graph.destroy()


@pytest.mark.parametrize("n", [5000, 5001])
def test_recorded_copy_nodes(hip, n):
    """Recorded device-to-device copies are launches of the identity kernel (kernel nodes that
    merge and alternate like any other launch); only byte-granular ranges at different 16-byte
    phases stay memcpy nodes of the runtime."""
    x = synth.uniform_f32(3, n, -1, 1)
    a, b, c = hip.buffer(x), hip.alloc(n), hip.alloc(n)
    hip.capture_begin()
    hip.copy(b, a)
    hip.apply_fn(b, lambda v: v.mul(2.0), out=c)
    hip.copy(a, c)
    g = hip.capture_end()
    assert g.stats() == (3, 3, 3)
    g.launch()
    hip.sync()
    assert_bits_equal(a.read(), (x * np.float32(2.0)).astype(np.float32))
    g.launch()
    hip.sync()
    assert_bits_equal(a.read(), (x * np.float32(4.0)).astype(np.float32))
    g.destroy()

    raw = (np.arange(4099, dtype=np.uint32) * 37 % 251).astype(np.uint8)
    p, q = hip.buffer(raw, "u8"), hip.alloc(4099 + 16, "u8")
    hip.capture_begin()
    hip.copy(q.slice(3, 3 + 4096), p.slice(1, 1 + 4096))      # phases 3 and 1: the runtime's copy
    hip.copy(q.slice(4100, 4100 + 9), p.slice(4, 4 + 9))      # both at phase 4: the identity kernel over bytes
    g = hip.capture_end()
    assert g.stats()[:2] == (2, 1)
    g.launch()
    hip.sync()
    got = q.read()
    assert_bits_equal(got[3:3 + 4096], raw[1:1 + 4096])
    assert_bits_equal(got[4100:4109], raw[4:13])
    assert not got[:3].any() and not got[4099:4100].any() and not got[4109:].any()
    g.destroy()


@pytest.mark.parametrize("direct_max", [0, 1, 4])
def test_short_chain_replays_the_same_as_a_graph_or_as_plain_launches(hip, oracle, direct_max):
    # A chain of at most `direct_max` nodes is replayed as plain launches on the compute
    # stream, anything else as an instantiated graph: same results either way, replay after replay.
    n = 70001
    x = synth.uniform_f32(11, n, -2, 2)
    a, b, c = hip.buffer(x), hip.alloc(n), hip.alloc(n)
    scale = """extern "C" __global__ void scale3(float* p, unsigned long long n) {
        unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x;
        if (i < n) p[i] = p[i] * 3.0f;
    }"""
    hip.set_graph_direct_replay(direct_max)
    try:
        hip.capture_begin()
        b.clear()
        hip.apply_fn(a, lambda v: v.mul(2.0).add(1.0), out=b)
        hip.copy(c, b)
        hip.launch_kernel(scale, "scale3", ((n + 255) // 256, 1, 1), (256, 1, 1), 0, [c, np.uint64(n)])
        g = hip.capture_end()
    finally:
        hip.set_graph_direct_replay(4)
    assert g.stats() == (4, 4, 4)          # clear, kernel, copy (the identity kernel), caller-written kernel
    want = oracle.apply_fn(lambda v: v.mul(2.0).add(1.0), x) * np.float32(3.0)
    for replay in range(3):
        c.clear()
        g.launch()
        hip.sync()
        assert_bits_equal(c.read(), want, f"direct_max={direct_max} replay {replay}")
    g.destroy()


def test_alternating_direction_in_replayed_graphs(hip, oracle):
    """Nodes that alternate their direction (here forced for every size): a directly replayed
    chain with an odd number of them flips on every replay, an instantiated graph keeps the
    directions it was built with; results are the same bits on every replay."""
    n = 40001
    x = synth.uniform_f32(13, n, -2, 2)
    f = lambda v: v.mul(1.5).sub(0.25)
    want1 = oracle.apply_fn(f, x)
    want3 = oracle.apply_fn(f, oracle.apply_fn(f, want1))
    try:
        hip.set_tuning(0, 0, 0, 0, 2)
        for direct_max, steps in ((4, 1), (4, 3), (0, 3)):
            hip.set_graph_direct_replay(direct_max)
            a, b, c, d = hip.buffer(x), hip.alloc(n), hip.alloc(n), hip.alloc(n)
            hip.capture_begin()
            hip.apply_fn(a, f, out=b)
            if steps == 3:
                hip.apply_fn(b, f, out=c)
                hip.apply_fn(c, f, out=d)
            g = hip.capture_end()
            last = b if steps == 1 else d
            for replay in range(4):
                last.clear()
                g.launch()
                hip.sync()
                assert_bits_equal(last.read(), want1 if steps == 1 else want3, f"direct_max={direct_max} steps={steps} replay={replay}")
            g.destroy()
    finally:
        hip.set_tuning()
        hip.set_graph_direct_replay(4)


def test_merged_launches_carry_their_own_literals(hip):
    """Launches of one expression with different literal values are merged into one grid; every
    segment reads its own values from its table row (equal and different lengths, several dtypes)."""
    rng = np.random.default_rng(21)
    for dtype, np_t, lengths in (("f32", np.float32, [4096] * 48), ("f32", np.float32, [1000 + 37 * i for i in range(48)]),
                                 ("f64", np.float64, [515 + 8 * i for i in range(20)]), ("i16", np.int16, [4096 + 8 * i for i in range(20)]),
                                 ("f16", np.float16, [2048] * 24)):
        hip.set_literal_policy(capi.LITERALS_AS_PARAMETERS)
        try:
            ins, outs, wants = [], [], []
            for i, length in enumerate(lengths):
                if dtype[0] == "i":
                    data = rng.integers(-100, 100, length).astype(np_t)
                    a, b = int(i - 7), int(3 * i + 1)
                    wants.append((data.astype(np.int64) * a + b).astype(np_t))
                else:
                    data = rng.uniform(-2, 2, length).astype(np_t)
                    a, b = float(i) * 0.25 - 3.0, 1.0 / (i + 1)
                    if dtype == "f16":
                        wide = data.astype(np.float32)
                        wants.append(np.maximum(wide * np.float32(a), np.float32(b)).astype(np.float16))
                    else:
                        wants.append(np.maximum(data * np_t(a), np_t(b)))
                ins.append((hip.buffer(data, dtype), a, b))
            hip.capture_begin()
            for buf, a, b in ins:
                if dtype[0] == "i":
                    outs.append(hip.apply_fn(buf, lambda v: v.mul(a).add(b)))
                else:
                    outs.append(hip.apply_fn(buf, lambda v: v.mul(a).max(b)))
            graph = hip.capture_end()
            assert graph.kernel_nodes == 1, (dtype, graph.kernel_nodes)
            for _ in range(2):
                graph.launch()
            for out, want in zip(outs, wants):
                got = out.read()
                assert got.view(np.uint8).tobytes() == np.ascontiguousarray(want).view(np.uint8).tobytes(), dtype
            graph.destroy()
        finally:
            hip.set_literal_policy(capi.LITERALS_ADAPTIVE)


def test_merged_gradient_launches_carry_their_own_literals(hip):
    """The same for the unary-gradient kind: g += o * (x * k_i), one grid for all k_i."""
    rng = np.random.default_rng(22)
    hip.set_literal_policy(capi.LITERALS_AS_PARAMETERS)
    try:
        sets = []
        for i in range(40):
            length = 700 + 64 * i
            x, g, o = (rng.uniform(-1, 1, length).astype(np.float32) for _ in range(3))
            k = 0.5 + i
            sets.append((hip.buffer(x), hip.buffer(g), hip.buffer(o), k, g + o * (x * np.float32(k))))
        hip.capture_begin()
        for xb, gb, ob, k, _ in sets:
            hip.add_unary_grad(xb, gb, ob, lambda v: v.mul(k))
        graph = hip.capture_end()
        assert graph.kernel_nodes == 1
        graph.launch()
        for _, gb, _, _, want in sets:
            assert_bits_equal(gb.read(), want, "gradient")
        graph.destroy()
    finally:
        hip.set_literal_policy(capi.LITERALS_ADAPTIVE)


def test_unmerged_graph_nodes_take_literals_by_value(hip):
    """With merging off every launch is a kernel node of its own in an instantiated hipGraph and
    takes its literal values as an argument by value."""
    rng = np.random.default_rng(23)
    hip.set_literal_policy(capi.LITERALS_AS_PARAMETERS)
    hip.set_graph_batching(False)
    try:
        data = [rng.uniform(-2, 2, 3000 + 16 * i).astype(np.float32) for i in range(12)]
        bufs = [hip.buffer(d) for d in data]
        hip.capture_begin()
        outs = [hip.apply_fn(b, lambda v: v.mul(float(i) + 0.5).sub(1.0 / (i + 2))) for i, b in enumerate(bufs)]
        graph = hip.capture_end()
        assert graph.kernel_nodes == len(bufs)
        for _ in range(3):
            graph.launch()
        for i, (d, out) in enumerate(zip(data, outs)):
            assert_bits_equal(out.read(), d * np.float32(i + 0.5) - np.float32(1.0 / (i + 2)), f"node {i}")
        graph.destroy()
    finally:
        hip.set_graph_batching(True)
        hip.set_literal_policy(capi.LITERALS_ADAPTIVE)


def test_waits_follow_the_work(hip):
    """`custos_hip_sync` after a graph launch polls, and for work it has seen take milliseconds
    sleeps up to shortly before the predicted end: a launch + wait of a 5 ms graph must not cost
    more wall time than the graph takes on the device (plus slack), run after run, and a short
    graph right after it must not inherit the long graph's prediction."""
    import time
    n = 1 << 26
    x = hip.alloc(n)
    hip.write(x.slice(0, 1 << 12), synth.uniform_f32(3, 1 << 12, -1, 1))
    bufs = [hip.alloc(n) for _ in range(2)]
    k = hip.compile(capi.KIND_APPLY, "f32", "((x * 1.0001) + 0.25)", ("x",))
    hip.set_graph_direct_replay(0)
    hip.set_graph_fusing(False)                   # 48 launches that take their time (joined they would be six)
    try:
        hip.capture_begin()
        src = x
        for i in range(48):                       # a chain: each launch reads what the one before wrote
            dst = bufs[i % 2]
            capi.check(hip.lib.custos_hip_apply_fn(hip.handle, k, src.ptr, dst.ptr, n), hip.handle)
            src = dst
        long_graph = hip.capture_end()
        hip.capture_begin()
        capi.check(hip.lib.custos_hip_apply_fn(hip.handle, k, x.ptr, bufs[0].ptr, 1 << 12), hip.handle)
        short_graph = hip.capture_end()
    finally:
        hip.set_graph_direct_replay(4)
        hip.set_graph_fusing(True)
    long_graph.launch()
    hip.sync()
    hip.timer_begin()
    long_graph.launch()
    device_ms = hip.timer_end()
    assert device_ms > 2.0                    # long enough for the wait to sleep through most of it
    walls = []
    for _ in range(6):
        t0 = time.perf_counter()
        long_graph.launch()
        hip.sync()
        walls.append((time.perf_counter() - t0) * 1e3)
    assert max(walls[1:]) < 1.5 * device_ms + 0.3, (walls, device_ms)
    t0 = time.perf_counter()
    short_graph.launch()
    hip.sync()
    assert (time.perf_counter() - t0) * 1e3 < 0.5 * device_ms + 0.3    # not slept on the long graph's account
    want = x.slice(0, 1 << 12).read()
    for _ in range(1):
        want = want * np.float32(1.0001) + np.float32(0.25)
    assert_bits_equal(bufs[0].slice(0, 1 << 12).read(), want)
    long_graph.destroy()
    short_graph.destroy()


def _both_ways(hip, inputs, program, dtype="f32"):
    """Runs `program(bufs)` eagerly and as a replayed graph (twice) over copies of `inputs`; the graph's
    buffers must equal the eager ones bit for bit after every replay.  Returns the graph's
    (kernel nodes, launches joined into later ones)."""
    eager = [hip.buffer(x, dtype) for x in inputs]
    lazy = [hip.buffer(x, dtype) for x in inputs]
    hip.capture_begin()
    program(lazy)
    g = hip.capture_end()
    shape = (g.kernel_nodes, g.fused_launches)
    for replay in range(2):
        program(eager)
        g.launch()
        hip.sync()
        for i, (a, b) in enumerate(zip(lazy, eager)):
            assert_bits_equal(a.read(), b.read(), f"replay {replay}, buffer {i}")
    g.destroy()
    return shape


def test_producers_join_their_consumers(hip):
    """Recorded apply launches that read, element for element, what an earlier one wrote become one
    kernel with it; every buffer still gets what the separate launches gave it."""
    n = 5003
    xs = [synth.uniform_f32(200 + i, n, -2, 2) for i in range(6)]
    f = lambda v: v.mul(1.5).sub(0.25)
    g = lambda v: v.abs().sqrt()
    h = lambda v: v.neg().max(-1.0)
    add = lambda p, q: p.add(q)
    mul = lambda p, q: p.mul(q)

    def fan_out(b):                 # two consumers of one result
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn(b[1], g, out=b[2])
        hip.apply_fn(b[1], h, out=b[3])
    assert _both_ways(hip, xs, fan_out) == (1, 2)

    def diamond(b):                 # two producers of one consumer
        hip.apply_fn(b[0], f, out=b[2])
        hip.apply_fn(b[1], g, out=b[3])
        hip.apply_fn2(b[2], b[3], add, out=b[4])
        hip.apply_fn2(b[4], b[2], mul, out=b[5])
    assert _both_ways(hip, xs, diamond) == (1, 3)

    def in_place(b):                # the same buffer read and written by every launch: one output
        for fn in (f, g, h):
            hip.apply_fn(b[0], fn, out=b[0])
    assert _both_ways(hip, xs, in_place) == (1, 2)

    def writes_an_input_of_its_producer(b):
        hip.apply_fn2(b[0], b[1], add, out=b[2])
        hip.apply_fn2(b[2], b[1], mul, out=b[0])      # b[0] was read by the first launch
        hip.apply_fn(b[0], f, out=b[1])               # and b[1] by both
    assert _both_ways(hip, xs, writes_an_input_of_its_producer) == (1, 2)

    def same_operand_twice(b):
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn2(b[1], b[1], mul, out=b[2])
    assert _both_ways(hip, xs, same_operand_twice) == (1, 1)

    def another_length(b):          # the consumer reads a part only: another launch geometry
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn(b[1].slice(0, 4000), g, out=b[2].slice(0, 4000))
    assert _both_ways(hip, xs, another_length) == (2, 0)

    def shifted(b):                 # the same length, but element i of the consumer is element i + 16 of the producer
        hip.apply_fn(b[0].slice(0, 4000), f, out=b[1].slice(0, 4000))
        hip.apply_fn(b[1].slice(16, 4016), g, out=b[2].slice(0, 4000))
    assert _both_ways(hip, xs, shifted) == (2, 0)

    def shifted_output(b):          # the consumer writes over a shifted part of what the producer read
        hip.apply_fn(b[0].slice(0, 4000), f, out=b[1].slice(0, 4000))
        hip.apply_fn(b[1].slice(0, 4000), g, out=b[0].slice(8, 4008))
    assert _both_ways(hip, xs, shifted_output) == (2, 0)

    def input_rewritten_in_between(b):
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn(b[0], h, out=b[0])               # writes what the first launch read
        hip.apply_fn(b[1], g, out=b[2])               # may not take the first launch along past that
    assert _both_ways(hip, xs, input_rewritten_in_between) == (3, 0)

    def result_copied_in_between(b):
        hip.apply_fn(b[0], f, out=b[1])
        hip.copy(b[3], b[1])                          # a copy reads the result: it has to be in memory by then
        hip.apply_fn(b[1], g, out=b[2])
    assert _both_ways(hip, xs, result_copied_in_between) == (3, 0)

    def gradient_launches_join_too(b):                # x_grad += out_grad * f'(x) is the expression g + (o * f'(x)) stored to g
        hip.apply_fn(b[0], f, out=b[1])               # y1 = f(x)
        hip.apply_fn(b[1], g, out=b[2])               # y2 = g(y1)
        hip.add_unary_grad(b[1], b[4], b[3], lambda v: v.mul(0.5).abs())   # g1 += g2 * g'(y1)
        hip.add_unary_grad(b[0], b[5], b[4], lambda v: v.mul(2.0))         # gx += g1 * f'(x)
        hip.add_unary_grad(b[0], b[5], b[3], lambda v: v.neg())            # and once more into the same gradient
    assert _both_ways(hip, xs, gradient_launches_join_too) == (1, 4)

    def cleared_in_between(b):
        hip.apply_fn(b[0], f, out=b[1])
        b[0].clear()
        hip.apply_fn(b[1], g, out=b[2])
    assert _both_ways(hip, xs, cleared_in_between) == (3, 0)

    def untouched_in_between(b):    # launches on other buffers in between do not matter
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn(b[3], h, out=b[4])
        b[5].clear()
        hip.apply_fn(b[1], g, out=b[2])
    assert _both_ways(hip, xs, untouched_in_between) == (3, 1)

    def forward_and_gradient_share_their_input(b):    # y = f(x); g += o * f'(x): x is loaded once
        hip.apply_fn(b[0], f, out=b[1])
        hip.add_unary_grad(b[0], b[2], b[3], lambda v: v.mul(0.5).abs())
    assert _both_ways(hip, xs, forward_and_gradient_share_their_input) == (1, 1)

    def readers_of_one_input(b):    # five launches that read b[0] and nothing of each other
        for i, fn in enumerate((f, g, h, f, g)):
            hip.apply_fn(b[0], fn, out=b[1 + i])
    assert _both_ways(hip, xs, readers_of_one_input) == (1, 4)

    def common_operand_of_separate_chains(b):         # b[5] is read by three chains that have nothing else in common
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn2(b[1], b[5], add, out=b[1])
        hip.apply_fn(b[2], g, out=b[3])
        hip.apply_fn2(b[3], b[5], add, out=b[3])      # the one open reader of b[5] so far comes along
        hip.apply_fn(b[4], h, out=b[4])
        hip.apply_fn2(b[4], b[5], mul, out=b[4])      # and so does the joined launch
    assert _both_ways(hip, xs, common_operand_of_separate_chains) == (1, 5)

    def common_operand_of_many_chains(b):             # a kernel holds eight expressions: the fourth chain starts anew,
        for _ in range(5):                            # and with two open readers of b[5] the fifth joins neither
            hip.apply_fn(b[0], f, out=b[1])
            hip.apply_fn2(b[1], b[5], add, out=b[2])
            b = b[2:4] + b[0:2] + b[4:]               # the next chain over the other buffers (b[5] stays)
    five = _both_ways(hip, xs, common_operand_of_many_chains)
    assert five[0] >= 2 and five[0] + five[1] >= 8

    def reader_after_a_writer(b):   # the second reader comes after the input was rewritten: not the same value
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn(b[2], h, out=b[0])
        hip.apply_fn(b[0], g, out=b[3])
    assert _both_ways(hip, xs, reader_after_a_writer) == (2, 1)

    def long_chain(b):              # at most eight expressions per kernel
        for i in range(20):
            hip.apply_fn(b[i % 2], f if i % 3 else h, out=b[(i + 1) % 2])
    assert _both_ways(hip, xs, long_chain) == (3, 17)

    def unaligned(b):               # views that start 3 elements into their buffers: scalar head and tail
        v = [q.slice(3, 3 + 1001) for q in b]
        hip.apply_fn2(v[0], v[1], mul, out=v[2])
        hip.apply_fn2(v[2], v[3], add, out=v[4])
        hip.apply_fn(v[4], g, out=v[5])
    assert _both_ways(hip, xs, unaligned) == (1, 2)

    def other_phase(b):             # producer and consumer views start at different offsets within 16 bytes
        hip.apply_fn(b[0].slice(1, 1001), f, out=b[1].slice(1, 1001))
        hip.apply_fn(b[1].slice(1, 1001), g, out=b[2].slice(2, 1002))
    assert _both_ways(hip, xs, other_phase)[1] in (0, 1)


@pytest.mark.parametrize("dtype", ["f32", "f64", "f16", "bf16", "f16_pernode", "bf16_pernode", "i32", "u8", "i64"])
def test_joined_launches_in_every_element_type(hip, dtype):
    """t = a * b; u = t + c; y = max(u, t) as one kernel: what a later stage takes from an earlier one is
    the STORED value (rounded to the storage type), so every buffer equals the launch-by-launch result."""
    n = 4099
    npdt = np.dtype(capi.DTYPES[dtype][1])
    rng = np.random.default_rng(5)
    if dtype[0] in "iu":
        info = np.iinfo(npdt)
        xs = [rng.integers(info.min, info.max, size=n, dtype=npdt, endpoint=True) for _ in range(3)]
    elif npdt == np.uint16:           # 16-bit floats travel as bits
        from oracle import cpu_oracle
        conv = cpu_oracle.f32_to_f16_bits if dtype.startswith("f16") else (lambda a: (a.view(np.uint32) >> 16).astype(np.uint16))
        xs = [conv(synth.uniform_f32(300 + i, n, -3, 3)) for i in range(3)]
    else:
        xs = [synth.uniform_f32(300 + i, n, -3, 3).astype(npdt) for i in range(3)]
    xs += [np.zeros(n, dtype=npdt) for _ in range(3)]

    def program(b):
        hip.apply_fn2(b[0], b[1], lambda p, q: p.mul(q), out=b[3])
        hip.apply_fn2(b[3], b[2], lambda p, q: p.add(q), out=b[4])
        hip.apply_fn2(b[4], b[3], lambda p, q: p.max(q), out=b[5])
        hip.add_unary_grad(b[3], b[5], b[4], lambda v: v.mul(3).add(1))    # b5 += b4 * (3 * b3 + 1)
    assert _both_ways(hip, xs, program, dtype) == (1, 3)


def test_joined_launches_of_many_buffers_merge(hip):
    """Chains over many buffers of different lengths: each chain one kernel, all of them one grid."""
    lengths = [256 * (1 + i % 7) + 4 * (i % 3) for i in range(40)]
    xs = [synth.uniform_f32(400 + i, ln, -2, 2) for i, ln in enumerate(lengths)]
    zeros = [np.zeros(ln, dtype=np.float32) for ln in lengths]

    def program(b):
        k = len(lengths)
        for i in range(k):
            hip.apply_fn(b[i], lambda v: v.mul(0.5).add(1.0), out=b[k + i])
            hip.apply_fn2(b[k + i], b[i], lambda p, q: p.mul(q), out=b[2 * k + i])
    assert _both_ways(hip, xs + zeros + zeros, program) == (1, 40)


@pytest.fixture
def fresh_device():
    """A device handle of its own: which literal values a kernel has seen decides whether they are in
    its code, so a test of that starts from nothing."""
    dev = custos_amd.HIP(0)
    yield dev
    dev.close()


def test_changing_literals_do_not_compile_chain_after_chain(fresh_device):
    """A literal is part of a joined kernel's code, or one of its launch parameters, as it is for the
    launch's own kernel: an expression that keeps arriving with new values (its literals have become
    launch parameters by then) still joins, and a graph per value compiles nothing."""
    hip = fresh_device
    n = 4096
    x = synth.uniform_f32(7, n, -2, 2)
    a, b, c = hip.buffer(x), hip.alloc(n), hip.alloc(n)

    def record(rate):
        hip.capture_begin()
        hip.apply_fn(a, lambda v: v.mul(rate).add(0.75), out=b)
        hip.apply_fn(b, lambda v: v.abs().sqrt().mul(rate), out=c)
        return hip.capture_end()

    def check(rate, g):
        assert (g.kernel_nodes, g.fused_launches) == (1, 1)
        b.clear()
        c.clear()
        g.launch()
        hip.sync()
        want_b = x * np.float32(rate) + np.float32(0.75)
        assert_bits_equal(b.read(), want_b)
        assert_bits_equal(c.read(), np.sqrt(np.abs(want_b)) * np.float32(rate))
        g.destroy()

    check(0.5, record(0.5))                           # the first values: compiled into the code
    check(0.25, record(0.25))                         # the second: the forms that take them as parameters are compiled
    before = hip.cache_stats()[0]
    for step in range(3, 9):
        check(1.0 / step, record(1.0 / step))
    assert hip.cache_stats()[0] == before             # six more values, nothing compiled
    # many buffers with a value of their own each: one merged launch, every row its own parameters
    bufs = [(hip.buffer(x), hip.alloc(n), hip.alloc(n)) for _ in range(12)]
    hip.capture_begin()
    for i, (p, q, r) in enumerate(bufs):
        rate = 0.3 + 0.01 * i
        hip.apply_fn(p, lambda v: v.mul(rate).add(0.75), out=q)
        hip.apply_fn(q, lambda v: v.abs().sqrt().mul(rate), out=r)
    g = hip.capture_end()
    assert (g.kernel_nodes, g.fused_launches) == (1, 12)
    g.launch()
    hip.sync()
    for i, (p, q, r) in enumerate(bufs):
        rate = np.float32(0.3 + 0.01 * i)
        want_q = x * rate + np.float32(0.75)
        assert_bits_equal(q.read(), want_q, f"buffer {i}")
        assert_bits_equal(r.read(), np.sqrt(np.abs(want_q)) * rate, f"buffer {i}")
    g.destroy()
    # one unit: the joined kernel's entry point for merged launches, which nothing had asked for before
    assert hip.cache_stats()[0] == before + 1


def test_graph_names_its_kernels(hip):
    """The entry points a built graph launches, as a profiler lists them."""
    n = 2048
    a, b, c = hip.buffer(synth.uniform_f32(1, n, -1, 1)), hip.alloc(n), hip.alloc(n)
    hip.capture_begin()
    hip.apply_fn(a, lambda v: v.mul(2.0), out=b)
    hip.apply_fn(b, lambda v: v.add(1.0), out=c)
    c.slice(0, 16).clear()
    g = hip.capture_end()
    names = g.kernel_names()
    assert len(names) == g.kernel_nodes == 2
    assert names[0].startswith("custos_chain_f32_") and names[1] == "custos_fill_zero"
    import ctypes as C
    name = C.c_char_p()
    assert hip.lib.custos_hip_graph_node_kernel(g.handle, 2, C.byref(name)) == capi.ERR_INVALID_ARGUMENT
    g.destroy()


def test_a_graph_build_compiles_joined_kernels_within_a_time_budget(fresh_device):
    """Four chains of four different shapes.  With no time for new kernels nothing is joined and the graph
    says so; with a budget that the first compilation uses up, one chain is joined and the others replay as
    the launches they were recorded as; with time enough, the next build finds that kernel cached and
    compiles the other three.  Results are the eager ones every time."""
    hip = fresh_device
    n = 3000
    xs = [synth.uniform_f32(500 + i, n, -2, 2) for i in range(4)]
    fns = [lambda v: v.mul(1.5), lambda v: v.abs().sqrt(), lambda v: v.neg().max(-1.0), lambda v: v.add(0.25).min(1.0)]

    def program(b):
        for i in range(4):                            # chain i: fns[i] twice, then fns[(i + 1) % 4]
            hip.apply_fn(b[i], fns[i], out=b[4 + i])
            hip.apply_fn(b[4 + i], fns[i], out=b[8 + i])
            hip.apply_fn(b[8 + i], fns[(i + 1) % 4], out=b[4 + i])

    def build(bufs):
        hip.capture_begin()
        program(bufs)
        return hip.capture_end()

    zeros = [np.zeros(n, dtype=np.float32) for _ in range(8)]
    for f in fns:                                     # the launches' own kernels exist before anything is counted
        hip.apply_fn(hip.buffer(xs[0]), f)
    before = hip.compile_stats()[0]
    try:
        hip.set_graph_fusing_budget(0)
        assert _both_ways(hip, xs + zeros, program) == (12, 0)
        g = build([hip.buffer(x) for x in xs + zeros])
        launches, reason = g.unjoined()
        assert launches == 12 and "budget" in reason and "0 ms" in reason
        g.destroy()
        assert hip.compile_stats()[0] == before
        hip.set_graph_fusing_budget(1)                # the first compilation starts, and spends more than that
        assert _both_ways(hip, xs + zeros, program) == (1 + 9, 2)
        assert hip.compile_stats()[0] - before == 1
        hip.set_graph_fusing_budget(0)                # a cached kernel needs no budget
        g = build([hip.buffer(x) for x in xs + zeros])
        assert g.unjoined()[0] == 9 and (g.kernel_nodes, g.fused_launches) == (1 + 9, 2)
        g.destroy()
        assert hip.compile_stats()[0] - before == 1
        hip.set_graph_fusing_budget(60000)
        assert _both_ways(hip, xs + zeros, program) == (4, 8)
        assert hip.compile_stats()[0] - before == 4
        g = build([hip.buffer(x) for x in xs + zeros])
        assert g.unjoined() == (0, "")
        g.destroy()
    finally:
        hip.set_graph_fusing_budget(1000)


def test_a_joined_kernel_that_does_not_compile_is_reported(fresh_device, monkeypatch):
    """A chain whose kernel the compiler rejects replays as the launches it was recorded as, and the graph
    carries the compiler's message instead of losing it."""
    hip = fresh_device
    n = 2000
    x = synth.uniform_f32(77, n, -2, 2)
    f, g_ = (lambda v: v.mul(1.25)), (lambda v: v.add(0.5))
    for fn in (f, g_):
        hip.apply_fn(hip.buffer(x), fn)

    def program(b):
        hip.apply_fn(b[0], f, out=b[1])
        hip.apply_fn(b[1], g_, out=b[2])

    monkeypatch.setenv("CUSTOS_HIP_FAIL_COMPILE_OF", "custos_chain_")   # compilations of such kernels fail
    try:
        assert _both_ways(hip, [x, np.zeros(n, np.float32), np.zeros(n, np.float32)], program) == (2, 0)
        hip.capture_begin()
        program([hip.buffer(x), hip.alloc(n), hip.alloc(n)])
        graph = hip.capture_end()
        launches, reason = graph.unjoined()
        assert launches == 2 and "hiprtc" in reason
        graph.destroy()
    finally:
        monkeypatch.delenv("CUSTOS_HIP_FAIL_COMPILE_OF")
    assert _both_ways(hip, [x, np.zeros(n, np.float32), np.zeros(n, np.float32)], program) == (1, 1)
