#!/usr/bin/env python3
"""Benchmark of the element-wise hot path on one MI355X.

Default workload (BASELINE.json configs[1]): the fused unary chain
y = relu(sin(x)*2.0 + 1.0) - 0.5 (five unary ops fused into one kernel) over
f32 N = 2^28, x uniform in [-pi, pi) from seed 0.  One "step" is one launch of
the fused kernel over the whole buffer, inputs resident in HBM.

Prints ONE JSON line: metric/value (GB/s on the algorithmic 8 B per element),
the roofline of the fused kernel (HIP-event timed on the compute stream) and a
CPU baseline (the oracle's compiled loop, one thread, on a stated sample).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c2|c3|c4|c5] [--log2n L]
"""
from __future__ import annotations

import argparse
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
MEASURED_TRAFFIC_C2_N2P28 = 2147505869

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


def time_steps(dev, step, steps, warmup):
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
    tuned = bool(args.block or args.unroll or args.blocks_per_cu or args.nontemporal)
    x = gen_chunked(lambda m, off: synth.uniform_f32(0, m, -np.pi, np.pi, off), n)
    xb = dev.buffer(x)
    out = dev.alloc(n, "f32")

    src = fused_source(C2_OPS, "f32")
    kernel = dev.compile(capi.KIND_APPLY, "f32", src, ("x",))
    lib, h = dev.lib, dev.handle

    def fused_step():
        capi.check(lib.custos_hip_apply_fn(h, kernel, xb.ptr, out.ptr, n), h)

    ms, wall_ms = time_steps(dev, fused_step, args.steps, args.warmup)
    per_launch_ms = ms / args.steps
    algo_bytes = 8.0 * n
    gbs = algo_bytes / (per_launch_ms * 1e-3) / 1e9

    # unfused comparison: five apply_fn launches through intermediates (40 B/elt moved)
    kernels = [dev.compile(capi.KIND_APPLY, "f32", custos_amd.expr._wrap(op(custos_amd.Resolve("x"))).to_cl_source("f32"), ("x",))
               for op in C2_OPS]
    tmp_a, tmp_b = dev.alloc(n, "f32"), dev.alloc(n, "f32")
    chain = [(xb, tmp_a), (tmp_a, tmp_b), (tmp_b, tmp_a), (tmp_a, tmp_b), (tmp_b, out)]

    def unfused_step():
        for k, (src_b, dst_b) in zip(kernels, chain):
            capi.check(lib.custos_hip_apply_fn(h, k, src_b.ptr, dst_b.ptr, n), h)

    ums, _ = time_steps(dev, unfused_step, max(1, args.steps // 4), max(1, args.warmup // 2))
    unfused_ms = ums / max(1, args.steps // 4)

    # plain copy (identity expression) over the same buffers: the achievable 1R+1W rate on
    # this box, and the known-size dispatch the profiler counters are scaled by
    copy_kernel = dev.compile(capi.KIND_APPLY, "f32", "x", ("x",))

    def copy_step():
        capi.check(lib.custos_hip_apply_fn(h, copy_kernel, xb.ptr, tmp_a.ptr, n), h)

    cms, _ = time_steps(dev, copy_step, max(1, args.steps // 2), max(1, args.warmup // 2))
    copy_ms = cms / max(1, args.steps // 2)

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
        "unfused": {
            "ms_per_step": round(unfused_ms, 5),
            "effective_GBps_on_8B_basis": round(algo_bytes / (unfused_ms * 1e-3) / 1e9, 2),
            "moved_GBps_on_40B_basis": round(5 * algo_bytes / (unfused_ms * 1e-3) / 1e9, 2),
            "speedup_fused": round(unfused_ms / per_launch_ms, 3),
        },
        "copy_kernel": {
            "name": dev.kernel_name(copy_kernel),
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
            "kernel": dev.kernel_name(kernel),
            "algorithmic_bytes_per_launch": algo_bytes,
            "avg_launch_ms": round(per_launch_ms, 5),
        },
        "cpu_baseline": base,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--log2n", type=int, default=28)
    ap.add_argument("--cpu-log2n", dest="cpu_log2n", type=int, default=28,
                    help="log2 of the element count of the CPU baseline sample")
    ap.add_argument("--block", type=int, default=0)
    ap.add_argument("--unroll", type=int, default=0)
    ap.add_argument("--blocks-per-cu", dest="blocks_per_cu", type=int, default=0)
    ap.add_argument("--nontemporal", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU; the element-wise path needs no second one "
                         "(--gpus must be 1)")

    import custos_amd

    dev = custos_amd.HIP(0)
    if args.block or args.unroll or args.blocks_per_cu or args.nontemporal:
        dev.set_tuning(args.block, args.unroll, args.blocks_per_cu, args.nontemporal)
    info = dev.info()
    res = {"c2": bench_c2}[args.workload](dev, args)
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
