#!/usr/bin/env python3
"""Benchmark of the element-wise hot path on one MI355X.

Default workload (BASELINE.json configs[1]): the fused unary chain
y = relu(sin(x)*2.0 + 1.0) - 0.5 (five unary ops fused into one kernel) over
f32 N = 2^28, x uniform in [-pi, pi) from seed 0.  One "step" is one launch of
the fused kernel over the whole buffer (replayed as the one-node graph a `Lazy`
run holds), inputs resident in HBM.

Prints ONE JSON line: metric/value (GB/s on the algorithmic 8 B per element),
the roofline of the fused kernel (HIP-event timed on the compute stream) and a
CPU baseline (the oracle's compiled loop, one thread, on a stated sample).

The same line carries `other_configs`: the other four BASELINE configurations
(c1 exp, c3 tanh forward+backward, c4 f16 chain, c5 graph replay), each with
elements/s, GB/s and the CPU port timed beside it (skip with --no-others).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--log2n L] [--no-others]
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch of the fused chain at N = 2^28 with the default launch shape, from two
# `rocprofv3 --pmc` runs (FETCH_SIZE, then WRITE_SIZE) scaled by the identity-copy kernel of
# known size; commands and raw counter values: profiles/fused_chain_f32_n2p28_hbm_traffic.md
MEASURED_TRAFFIC_C2_N2P28 = 2147557720

C2_OPS = [
    lambda v: v.sin(),
    lambda v: v.mul(2.0),
    lambda v: v.add(1.0),
    lambda v: v.max(0.0),
    lambda v: v.sub(0.5),
]


def gen_chunked(fn, n, chunk=1 << 24):
    """Generates a large synthetic array chunk by chunk (bounded host memory)."""
    out = None
    for off in range(0, n, chunk):
        part = fn(min(chunk, n - off), off)
        if out is None:
            out = np.empty(n, dtype=part.dtype)
        out[off:off + part.size] = part
    return out


def time_steps(dev, step, steps, warmup, settle_ms=0.0):
    """`warmup` untimed steps, then `steps` timed ones.  `settle_ms` > 0 first repeats the step
    untimed until that much time has passed: after an idle period (host-side data generation,
    the CPU baseline) the device needs about 30 ms of work to return to its steady clocks."""
    if settle_ms > 0:
        t_end = time.perf_counter() + settle_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(8):
                step()
            dev.sync()
    for _ in range(warmup):
        step()
    dev.sync()
    t_wall = time.perf_counter()
    dev.timer_begin()
    for _ in range(steps):
        step()
    ms_events = dev.timer_end()
    dev.sync()
    wall_ms = (time.perf_counter() - t_wall) * 1e3
    return ms_events, wall_ms


def cpu_baseline_c2(x, sample_elems):
    from oracle import cpu_oracle

    xs = np.ascontiguousarray(x[:sample_elems])
    out = np.empty_like(xs)
    cpu_oracle.c2_chain_fused(xs[: 1 << 16])  # touch code and libm once
    t0 = time.perf_counter()
    cpu_oracle.c2_chain_fused(xs, out)
    dt = time.perf_counter() - t0
    return {
        "value": round(8.0 * xs.size / dt / 1e9, 4),
        "unit": "GB/s",
        "elements_per_s": round(xs.size / dt, 1),
        "cores": 1,
        "host_cores": os.cpu_count(),
        "kind": "port",
        "sample": f"fused chain, compiled C loop (oracle_c2_chain_fused_f32), first {xs.size} of the same elements, "
                  f"1 thread, {dt:.2f} s",
    }, out


def bench_c2(dev, args):
    import custos_amd
    from custos_amd import capi, synth
    from custos_amd.expr import fused_source

    n = 1 << args.log2n
    tuned = bool(args.block or args.unroll or args.blocks_per_cu or args.nontemporal or args.direction)
    x = gen_chunked(lambda m, off: synth.uniform_f32(0, m, -np.pi, np.pi, off), n)
    xb = dev.buffer(x)
    out = dev.alloc(n, "f32")

    src = fused_source(C2_OPS, "f32")
    kernel = dev.compile(capi.KIND_APPLY, "f32", src, ("x",))
    lib, h = dev.lib, dev.handle

    def fused_step():
        capi.check(lib.custos_hip_apply_fn(h, kernel, xb.ptr, out.ptr, n), h)

    algo_bytes = 8.0 * n

    # The comparisons run first (they also bring the device to its steady clocks: the first
    # ~30 ms of back-to-back launches after start-up run up to 15 % slower), the headline last.

    # unfused comparison: five apply_fn launches through intermediates (40 B/elt moved)
    kernels = [dev.compile(capi.KIND_APPLY, "f32", custos_amd.expr._wrap(op(custos_amd.Resolve("x"))).to_cl_source("f32"), ("x",))
               for op in C2_OPS]
    tmp_a, tmp_b = dev.alloc(n, "f32"), dev.alloc(n, "f32")
    chain = [(xb, tmp_a), (tmp_a, tmp_b), (tmp_b, tmp_a), (tmp_a, tmp_b), (tmp_b, out)]

    def unfused_step():
        for k, (src_b, dst_b) in zip(kernels, chain):
            capi.check(lib.custos_hip_apply_fn(h, k, src_b.ptr, dst_b.ptr, n), h)

    ums, _ = time_steps(dev, unfused_step, max(1, args.steps // 4), max(1, args.warmup // 2), settle_ms=50)
    unfused_ms = ums / max(1, args.steps // 4)

    # plain copy (identity expression) over the same buffers: the achievable 1R+1W rate on
    # this box, and the known-size dispatch the profiler counters are scaled by
    copy_kernel = dev.compile(capi.KIND_APPLY, "f32", "x", ("x",))

    def copy_step():
        capi.check(lib.custos_hip_apply_fn(h, copy_kernel, xb.ptr, tmp_a.ptr, n), h)

    cms, _ = time_steps(dev, copy_step, max(1, args.steps // 2), max(1, args.warmup // 2))
    copy_ms = cms / max(1, args.steps // 2)

    # The fused step with the launch shape pinned to plain HBM streaming: every launch walks the
    # array from the first tile to the last, non-temporal accesses, two vectors per thread.  (By
    # default every launch of this size walks the array against the direction of the launch
    # before it and so starts on the last 256 MiB the memory-side cache still holds.)
    streaming = None
    if not tuned:
        dev.set_tuning(0, 2, 0, 3, 1)
        skernel = dev.compile(capi.KIND_APPLY, "f32", src, ("x",))
        dev.capture_begin()
        capi.check(lib.custos_hip_apply_fn(h, skernel, xb.ptr, out.ptr, n), h)
        sgraph = dev.capture_end()
        sms, _ = time_steps(dev, sgraph.launch, args.steps, args.warmup, settle_ms=100)
        sgraph.destroy()
        dev.set_tuning(0, 0, 0, 0, 0)
        streaming = {"ms_per_step": round(sms / args.steps, 5),
                     "GBps": round(algo_bytes / (sms / args.steps * 1e-3) / 1e9, 2),
                     "kernel": dev.kernel_name(skernel),
                     "shape": "tiles first to last, non-temporal loads and stores, 2 vectors per thread"}

    dms, _ = time_steps(dev, fused_step, args.steps, args.warmup, settle_ms=100)   # the fused kernel launched directly
    direct_ms = dms / args.steps

    # Headline.  One step = what `Lazy::run` does from the second run on: replay the graph that
    # holds the fused kernel.  (The first run records and builds it; that is outside the timed region.)
    dev.capture_begin()
    fused_step()
    graph = dev.capture_end()
    assert graph.kernel_nodes == 1
    ms, wall_ms = time_steps(dev, graph.launch, args.steps, args.warmup, settle_ms=100)
    per_launch_ms = ms / args.steps
    graph.destroy()
    gbs = algo_bytes / (per_launch_ms * 1e-3) / 1e9

    # parity of the very buffer that was timed, on the CPU sample
    fused_step()
    got = out.read()
    base, want = cpu_baseline_c2(x, min(n, 1 << args.cpu_log2n))
    diff = float(np.max(np.abs(got[: want.size] - want)))
    tol = 8 * float(np.spacing(np.float32(1.0)))
    if not diff <= tol:
        raise SystemExit(f"bench: fused chain differs from the CPU oracle: max abs diff {diff} > {tol}")

    return {
        "metric": "fused unary-chain GB/s and % of HBM peak, f32 N=2^28, 1xMI355X",
        "value": round(gbs, 2),
        "unit": "GB/s",
        "ms_per_step": round(per_launch_ms, 5),
        "config": {
            "workload": f"c2: fused relu(sin(x)*2+1)-0.5, f32, N=2^{args.log2n}, x~U[-pi,pi) seed 0, "
                        "Lazy+Graph unary fusion -> 1 kernel",
            "elements": n,
            "algorithmic_bytes_per_element": 8,
        },
        "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "elements_per_s": round(n / (per_launch_ms * 1e-3), 1),
        "wall_ms_per_step": round(wall_ms / args.steps, 5),
        "direct_launch": {"ms_per_step": round(direct_ms, 5), "GBps": round(algo_bytes / (direct_ms * 1e-3) / 1e9, 2)},
        "hbm_streaming_only": streaming,
        "unfused": {
            "ms_per_step": round(unfused_ms, 5),
            "effective_GBps_on_8B_basis": round(algo_bytes / (unfused_ms * 1e-3) / 1e9, 2),
            "moved_GBps_on_40B_basis": round(5 * algo_bytes / (unfused_ms * 1e-3) / 1e9, 2),
            "speedup_fused": round(unfused_ms / per_launch_ms, 3),
        },
        "copy_kernel": {
            "name": dev.kernel_name(copy_kernel, n),
            "ms_per_launch": round(copy_ms, 5),
            "GBps": round(algo_bytes / (copy_ms * 1e-3) / 1e9, 2),
            "bytes_per_launch": algo_bytes,
        },
        "max_abs_diff_vs_cpu_oracle": diff,
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_C2_N2P28 if (args.log2n == 28 and not tuned) else None,
            "kernel": dev.kernel_name(kernel, n),
            "algorithmic_bytes_per_launch": algo_bytes,
            "avg_launch_ms": round(per_launch_ms, 5),
        },
        "cpu_baseline": base,
    }


def _cpu_time(fn, *a):
    t0 = time.perf_counter()
    r = fn(*a)
    return time.perf_counter() - t0, r


def _entry(name, n, bytes_per_elt, ms, cpu_s, cpu_n, note=""):
    gbs = bytes_per_elt * n / (ms * 1e-3) / 1e9
    return {
        "workload": name,
        "elements": n,
        "algorithmic_bytes_per_element": bytes_per_elt,
        "ms": round(ms, 5),
        "GBps": round(gbs, 2),
        "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
        "elements_per_s": round(n / (ms * 1e-3), 1),
        "cpu_port_1thread": {
            "elements_per_s": round(cpu_n / cpu_s, 1),
            "GBps": round(bytes_per_elt * cpu_n / cpu_s / 1e9, 4),
            "sample_elements": cpu_n,
        },
        **({"note": note} if note else {}),
    }


def bench_others(dev, args):
    """The other BASELINE configurations (c1, c3, c4, c5), each with its CPU port beside it."""
    import custos_amd
    from custos_amd import Const, capi, synth
    from custos_amd.expr import fused_source
    from oracle import cpu_oracle

    lib, h = dev.lib, dev.handle
    steps, warm = max(5, args.steps // 2), max(2, args.warmup // 2)
    out = {}

    # c1: apply_fn(exp), f32 N = 2^20 (latency-bound: 8 MiB of traffic)
    n = 1 << 20
    x = synth.uniform_f32(0, n, -4, 4)
    xb, ob = dev.buffer(x), dev.alloc(n)
    k = dev.compile(capi.KIND_APPLY, "f32", "exp(x)", ("x",))
    ms, _ = time_steps(dev, lambda: capi.check(lib.custos_hip_apply_fn(h, k, xb.ptr, ob.ptr, n), h), steps * 4, warm, settle_ms=50)
    cpu_s, want = _cpu_time(cpu_oracle.c1_exp, x)
    got = ob.read()
    assert np.max(np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))) <= 4
    out["c1"] = _entry("c1: apply_fn(exp), f32 N=2^20, U[-4,4) seed 0", n, 8, ms / (steps * 4), cpu_s, n)
    out["c1"]["kernel"] = dev.kernel_name(k, n)

    # c3: unary_ew tanh forward + backward, f32 N = 2^26
    n = 1 << 26
    x = gen_chunked(lambda m, off: synth.normal_f32(0, m, off), n)
    yg = gen_chunked(lambda m, off: synth.uniform_f32(1, m, -1, 1, off), n)
    xb, ygb, yb = dev.buffer(x), dev.buffer(yg), dev.alloc(n)
    gb = dev.buffer(np.full(n, 0.1, dtype=np.float32))
    kf = dev.compile(capi.KIND_APPLY, "f32", "tanh(x)", ("x",))
    grad_src = Const(1.0).sub(custos_amd.Resolve("x").tanh().mul(custos_amd.Resolve("x").tanh())).to_cl_source("f32")
    kb = dev.compile(capi.KIND_UNARY_GRAD, "f32", grad_src, ("x",))

    def c3_step():
        capi.check(lib.custos_hip_apply_fn(h, kf, xb.ptr, yb.ptr, n), h)
        capi.check(lib.custos_hip_add_unary_grad(h, kb, xb.ptr, gb.ptr, ygb.ptr, n), h)

    ms, _ = time_steps(dev, c3_step, steps, warm, settle_ms=50)
    ms_f, _ = time_steps(dev, lambda: capi.check(lib.custos_hip_apply_fn(h, kf, xb.ptr, yb.ptr, n), h), steps, warm, settle_ms=50)
    ms_b, _ = time_steps(dev, lambda: capi.check(lib.custos_hip_add_unary_grad(h, kb, xb.ptr, gb.ptr, ygb.ptr, n), h), steps, warm, settle_ms=50)
    cn = min(n, 1 << 24)
    g0 = np.full(cn, 0.1, dtype=np.float32)
    cpu_s, _ = _cpu_time(lambda: (cpu_oracle.c3_tanh_fwd(x[:cn]), cpu_oracle.c3_tanh_bwd(x[:cn], g0, yg[:cn])))
    e = _entry("c3: unary_ew tanh fwd + bwd (x_grad += y_grad*(1-tanh(x)^2)), f32 N=2^26", n, 24, ms / steps, cpu_s, cn)
    e["forward"] = {"ms": round(ms_f / steps, 5), "GBps": round(8 * n / (ms_f / steps * 1e-3) / 1e9, 2),
                    "kernel": dev.kernel_name(kf, n)}
    e["backward"] = {"ms": round(ms_b / steps, 5), "GBps": round(16 * n / (ms_b / steps * 1e-3) / 1e9, 2),
                     "kernel": dev.kernel_name(kb, n)}
    out["c3"] = e
    del xb, ygb, yb, gb

    # c4: f16 storage / f32 compute chain exp(x*0.5)*x + x^2, N = 2^28
    n = 1 << args.log2n
    xh = gen_chunked(lambda m, off: synth.uniform_f16_bits(0, m, -2, 2, off), n)
    xb, ob = dev.buffer(xh.view(np.float16), "f16"), dev.alloc(n, "f16")
    c4 = lambda v: v.mul(0.5).exp().mul(v).add(v.mul(v))
    k = dev.compile(capi.KIND_APPLY, "f16", c4(custos_amd.Resolve("x")).to_cl_source("f16"), ("x",))
    ms, _ = time_steps(dev, lambda: capi.check(lib.custos_hip_apply_fn(h, k, xb.ptr, ob.ptr, n), h), steps, warm, settle_ms=50)
    cn = min(n, 1 << 24)
    cpu_s, want = _cpu_time(cpu_oracle.c4_chain_f16, np.ascontiguousarray(xh[:cn]))
    got = ob.slice(0, cn).read().view(np.uint16)
    d = np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
    assert d.max() <= 1, "c4 differs from the CPU port by more than 1 f16 ulp"
    out["c4"] = _entry(f"c4: f16 chain exp(x*0.5)*x + x^2, f32 compute, N=2^{args.log2n}", n, 4, ms / steps, cpu_s, cn)
    out["c4"]["kernel"] = dev.kernel_name(k, n)
    del xb, ob

    # c5: 1024 buffers x 4096 f32: t=a*b; u=t+c; y=sqrt(abs(u))*0.3, one graph, 100 replays
    nbuf, m = 1024, 4096
    mk = lambda seed: dev.buffer(gen_chunked(lambda q, off: synth.uniform_f32(seed, q, 0, 1, off), nbuf * m))
    A, B, Cc = mk(1), mk(2), mk(3)
    T, U, Y = dev.alloc(nbuf * m), dev.alloc(nbuf * m), dev.alloc(nbuf * m)
    kmul = dev.compile(capi.KIND_APPLY, "f32", "(x * y)", ("x", "y"))
    kadd = dev.compile(capi.KIND_APPLY, "f32", "(x + y)", ("x", "y"))
    kun = dev.compile(capi.KIND_APPLY, "f32", fused_source([lambda v: v.abs().sqrt(), lambda v: v.mul(0.3)]), ("x",))
    dev.capture_begin()
    for i in range(nbuf):
        o = i * m * 4
        capi.check(lib.custos_hip_apply_fn2(h, kmul, A.ptr + o, B.ptr + o, T.ptr + o, m), h)
        capi.check(lib.custos_hip_apply_fn2(h, kadd, T.ptr + o, Cc.ptr + o, U.ptr + o, m), h)
        capi.check(lib.custos_hip_apply_fn(h, kun, U.ptr + o, Y.ptr + o, m), h)
    t0 = time.perf_counter()
    graph = dev.capture_end()
    build_s = time.perf_counter() - t0
    replays = 100
    ms, wall = time_steps(dev, graph.launch, replays, 3, settle_ms=50)
    a, b, c = A.read(), B.read(), Cc.read()
    cpu_s, (_, _, want) = _cpu_time(cpu_oracle.c5_graph, a, b, c)
    assert np.array_equal(Y.read().view(np.uint32), want.view(np.uint32)), "c5 replay differs from the CPU port"
    e = _entry("c5: 1024 x f32[4096], t=a*b; u=t+c; y=sqrt(abs(u))*0.3, one hipGraph, 100 replays", nbuf * m, 16,
               ms / replays, cpu_s, nbuf * m, note="GB/s on the minimal 16 B/element; the recorded 3-kernel form moves 32 B/element")
    e["us_per_replay"] = round(ms / replays * 1e3, 2)
    e["wall_us_per_replay"] = round(wall / replays * 1e3, 2)
    e["graph_kernel_nodes"] = graph.kernel_nodes
    e["recorded_launches"] = 3 * nbuf
    e["graph_build_ms"] = round(build_s * 1e3, 2)
    e["kernels"] = [dev.kernel_name(q, nbuf * m) + "_batched" for q in (kmul, kadd, kun)]
    graph.destroy()

    # the same work after element-wise fusing (what `Lazy::elementwise_fusing` of the host stack
    # records): one three-operand kernel per buffer, 16 B/element, merged into one kernel node
    kf = dev.compile(capi.KIND_APPLY, "f32", "(sqrt(abs(((a * b) + c))) * 0.3)", ("a", "b", "c"))
    Y.clear()
    dev.capture_begin()
    for i in range(nbuf):
        o = i * m * 4
        ptrs = (C.c_uint64 * 3)(A.ptr + o, B.ptr + o, Cc.ptr + o)
        capi.check(lib.custos_hip_apply_fn_n(h, kf, ptrs, 3, Y.ptr + o, m), h)
    fgraph = dev.capture_end()
    fms, fwall = time_steps(dev, fgraph.launch, replays, 3, settle_ms=50)
    assert np.array_equal(Y.read().view(np.uint32), want.view(np.uint32)), "c5 fused replay differs from the CPU port"
    e["fused"] = {
        "us_per_replay": round(fms / replays * 1e3, 2),
        "wall_us_per_replay": round(fwall / replays * 1e3, 2),
        "GBps": round(16 * nbuf * m / (fms / replays * 1e-3) / 1e9, 2),
        "graph_kernel_nodes": fgraph.kernel_nodes,
        "expression": "(sqrt(abs(((a * b) + c))) * 0.3)",
        "kernel": dev.kernel_name(kf, nbuf * m) + "_batched",
    }
    out["c5"] = e
    fgraph.destroy()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--direct-replay", type=int, default=None,
                    help="longest recorded chain replayed as plain launches (library default 4; 0 = always a hipGraph)")
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=["c2"])
    ap.add_argument("--log2n", type=int, default=28)
    ap.add_argument("--cpu-log2n", dest="cpu_log2n", type=int, default=28,
                    help="log2 of the element count of the CPU baseline sample")
    ap.add_argument("--block", type=int, default=0)
    ap.add_argument("--unroll", type=int, default=0)
    ap.add_argument("--blocks-per-cu", dest="blocks_per_cu", type=int, default=0)
    ap.add_argument("--nontemporal", type=int, default=0)
    ap.add_argument("--direction", type=int, default=0,
                    help="1: tiles first to last; 2: every launch the other way round; 0: library default")
    ap.add_argument("--no-others", dest="others", action="store_false",
                    help="skip the other BASELINE configurations (c1, c3, c4, c5)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU; the element-wise path needs no second one "
                         "(--gpus must be 1)")

    import custos_amd

    dev = custos_amd.HIP(0)
    if args.direct_replay is not None:
        dev.set_graph_direct_replay(args.direct_replay)
    if args.block or args.unroll or args.blocks_per_cu or args.nontemporal or args.direction:
        dev.set_tuning(args.block, args.unroll, args.blocks_per_cu, args.nontemporal, args.direction)
    info = dev.info()
    res = {"c2": bench_c2}[args.workload](dev, args)
    if args.others:
        res["other_configs"] = bench_others(dev, args)
    res.update({
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "device": {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units},
    })
    print(json.dumps(res))


if __name__ == "__main__":
    main()
