#!/usr/bin/env python3
"""Benchmark of the element-wise hot path on one MI355X.

Default workload (BASELINE.json configs[1]): y = relu(sin(x)*2.0 + 1.0) - 0.5, five unary
operations fused into ONE kernel, over f32 N = 2^28, x uniform in [-pi, pi) from seed 0, inputs
resident in HBM.  What is timed, and where:

  value / ms_per_step   this process, through the C ABI: one step = one replay of the one-node
                        recording that holds the fused kernel, pinned to plain HBM streaming (every
                        launch walks the array from the first tile to the last with non-temporal
                        accesses, so nothing of the previous launch is found in the memory-side
                        cache); exactly --steps replays between two events on the library's compute
                        stream, no wait between steps.
  sustained / roofline  the same replay back to back for at least two seconds with an event between
                        every two launches: mean (what `roofline.achieved` is quoted on), median, the
                        rate 99 % of the launches reach, and the slowest launch.
  default_replay        the same recording with the library's own launch shape: launches alternate
                        their direction and so start on the 256 MiB the memory-side cache still holds.
  module_stack          child processes started before this one touches the GPU: the C++ module
                        stacks on the HIP device (c2: HIP<Graph<Lazy<Base>>>, five apply_fn calls,
                        optimize_mem_graph, unary_fusing, run(); the other configurations likewise).
  first_use             child processes with an empty compiler cache, then a warm one: what the first
                        call of a new expression costs (compilation included).
  cpu_baseline          the oracle's compiled loop for the same chain, one thread.

`other_configs` carries the other four BASELINE configurations (c1 exp, c3 tanh forward +
backward, c4 f16 chain, c5 graph replay), each with elements/s, GB/s and the CPU port beside it
(skip with --no-others).  Phases other than the headline run at least 50 launches and 50 ms of
device time whatever --steps says.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--log2n L] [--no-others]
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import re
import subprocess
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch of the streaming-pinned fused chain at N = 2^28, from two `rocprofv3 --pmc`
# runs (FETCH_SIZE, then WRITE_SIZE) scaled by the identity-copy kernel of known size: the number
# is read from the summary of those runs, which also holds the commands and the raw counters.
TRAFFIC_PROFILE = "profiles/fused_chain_f32_n2p28_hbm_traffic.md"

MIN_LAUNCHES = 50      # floor of every timed phase except the headline's --steps
MIN_DEVICE_MS = 50.0

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


def launcher(dev, fn, *args):
    """A step that calls one entry point of the library with fixed arguments."""
    h = dev.handle

    def step():
        rc = fn(h, *args)
        if rc:
            from custos_amd import capi
            capi.check(rc, h)
    return step


def settle(dev, step, settle_ms):
    """Runs `step` untimed: once with a wait (whatever a first call costs stays outside), then
    for `settle_ms` of back-to-back work.  After an idle period (host-side data generation, the
    CPU baseline) the device needs some tens of milliseconds of work to return to its steady clocks."""
    step()
    dev.sync()
    t_end = time.perf_counter() + settle_ms * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(8):
            step()
        dev.sync()


def time_exactly(dev, step, steps, warmup, settle_ms=100.0):
    """`warmup` untimed steps, then EXACTLY `steps` timed ones between two events on the compute
    stream, bracketed by waits.  Returns (event ms, wall ms)."""
    settle(dev, step, settle_ms)
    for _ in range(warmup):
        step()
    dev.sync()
    t_wall = time.perf_counter()
    dev.timer_begin()
    for _ in range(steps):
        step()
    ms_events = dev.timer_end()
    dev.sync()
    return ms_events, (time.perf_counter() - t_wall) * 1e3


def time_floor(dev, step, launches_per_step=1, settle_ms=60.0):
    """Mean ms per step over at least MIN_LAUNCHES launches and MIN_DEVICE_MS of device time."""
    settle(dev, step, settle_ms)
    dev.timer_begin()
    for _ in range(8):
        step()
    guess = max(dev.timer_end() / 8, 1e-4)
    steps = int(max(-(-MIN_LAUNCHES // launches_per_step), -(-MIN_DEVICE_MS // guess)))
    dev.sync()
    dev.timer_begin()
    for _ in range(steps):
        step()
    return dev.timer_end() / steps, steps


def per_step_stats(dev, step, steps):
    """Every step's own duration: a mark on the compute stream between every two steps."""
    steps = min(max(steps, MIN_LAUNCHES), 4000)
    dev.sync()
    dev.timer_mark(0)
    for i in range(steps):
        step()
        dev.timer_mark(i + 1)
    ms = np.array([dev.timer_between(i, i + 1) for i in range(steps)])
    return {"steps": steps, "mean_ms": round(float(ms.mean()), 5), "median_ms": round(float(np.median(ms)), 5),
            "min_ms": round(float(ms.min()), 5), "max_ms": round(float(ms.max()), 5)}


def sustained_stats(dev, step, bytes_per_step, seconds=2.0, chunk=None):
    """`step` back to back for at least `seconds` of device time, twice.  First between two events only:
    the mean launch duration with nothing else on the stream (an event between two launches costs about
    1 % of a 0.3 ms launch).  Then with an event between every two steps, for the distribution: median,
    the rate 99 % of the launches reach, the slowest launch.  The events of a chunk are read while the
    device is idle for a moment; every chunk starts behind a few untimed steps."""
    chunk = chunk or (2048 if seconds >= 1.0 else 64)   # (short regions are for runs under a profiler)
    dev.sync()
    dev.timer_begin()
    for _ in range(16):
        step()
    guess_ms = max(dev.timer_end() / 16, 1e-4)
    launches = max(chunk, int(seconds * 1e3 / guess_ms))
    dev.timer_begin()
    for _ in range(launches):
        step()
    plain_ms = dev.timer_end()
    durations = []
    total_ms = 0.0
    while total_ms < seconds * 1e3 and len(durations) * chunk < 200000:
        for _ in range(4):
            step()
        dev.timer_mark(0)
        for i in range(chunk):
            step()
            dev.timer_mark(i + 1)
        ms = np.array([dev.timer_between(i, i + 1) for i in range(chunk)])
        durations.append(ms)
        total_ms += float(ms.sum())
    ms = np.concatenate(durations)
    gbs = bytes_per_step / (ms * 1e-3) / 1e9
    return {
        "launches": launches, "device_seconds": round(plain_ms * 1e-3, 3),
        "mean_ms": round(plain_ms / launches, 5),
        "mean_GBps": round(bytes_per_step / (plain_ms / launches * 1e-3) / 1e9, 2),
        "with_an_event_between_launches": {
            "launches": int(ms.size), "device_seconds": round(total_ms * 1e-3, 3),
            "mean_ms": round(float(ms.mean()), 5), "median_ms": round(float(np.median(ms)), 5),
            "p99_ms": round(float(np.percentile(ms, 99)), 5), "max_ms": round(float(ms.max()), 5),
            "mean_GBps": round(bytes_per_step / (float(ms.mean()) * 1e-3) / 1e9, 2),
        },
        "median_GBps": round(float(np.median(gbs)), 2),
        "p99_GBps": round(float(np.percentile(gbs, 1)), 2),
        "min_GBps": round(float(gbs.min()), 2),
        "what": "mean: back to back between two events; median, p99 (99 % of the launches are at least this fast) and min (the "
                "slowest launch) from a second pass with an event between every two launches, which costs each launch about 1 %",
    }


def module_stack(config, steps, warmup, log2n=None, fuse=False, dump=None, stack=None, inputs=(), settle_ms=None, env=None,
                 rerecord=False):
    """Runs examples/bench_module_stack as a child process and returns its JSON line."""
    exe = os.path.join(ROOT, "examples", "bench_module_stack")
    if not os.path.exists(exe):
        return {"error": f"{exe} is not built (make -C examples)"}
    cmd = [exe, "--config", config, "--steps", str(steps), "--warmup", str(warmup)]
    if log2n is not None:
        cmd += ["--log2n", str(log2n)]
    if fuse:
        cmd += ["--fuse"]
    if rerecord:
        cmd += ["--rerecord"]
    if stack:
        cmd += ["--stack", stack]
    if settle_ms is not None:
        cmd += ["--settle-ms", str(settle_ms)]
    for flag, path in zip(("--input", "--input2"), inputs):
        cmd += [flag, path]
    if dump:
        cmd += ["--dump", str(dump[0]), dump[1]]
    try:
        proc = subprocess.run(cmd, capture_output=True, text=True, timeout=240, env=env)
    except subprocess.TimeoutExpired:
        return {"error": "timed out"}
    if proc.returncode != 0:
        return {"error": (proc.stderr or proc.stdout)[-400:]}
    return json.loads(proc.stdout.strip().splitlines()[-1])


def cold_cache_env(tmp):
    """An environment in which the ROCm compiler library finds none of its cached results: its cache
    sits under the home directory (or where AMD_COMGR_CACHE_DIR / XDG_CACHE_HOME point)."""
    env = dict(os.environ)
    env.update({"HOME": tmp, "XDG_CACHE_HOME": os.path.join(tmp, ".cache"), "AMD_COMGR_CACHE_DIR": os.path.join(tmp, "comgr")})
    env.pop("CUSTOS_HIP_KERNEL_CACHE_DIR", None)
    return env


FIRST_CALL_EXPRESSIONS = {
    "c1": (lambda: "exp(x)", 1 << 20),
    "c2": (lambda: __import__("custos_amd.expr", fromlist=["fused_source"]).fused_source(C2_OPS, "f32"), 1 << 20),
}


def first_call_child(which):
    """(child process) One first call of an expression: compile, launch over a small buffer, wait."""
    import custos_amd
    from custos_amd import capi

    make_src, n = FIRST_CALL_EXPRESSIONS[which]
    dev = custos_amd.HIP(0)
    x, out = dev.alloc(n), dev.alloc(n)
    dev.sync()
    t0 = time.perf_counter()
    kernel = dev.compile(capi.KIND_APPLY, "f32", make_src(), ("x",))
    t1 = time.perf_counter()
    capi.check(dev.lib.custos_hip_apply_fn(dev.handle, kernel, x.ptr, out.ptr, n), dev.handle)
    dev.sync()
    t2 = time.perf_counter()
    units, hiprtc_ms = dev.compile_stats()
    print(json.dumps({"first_call_ms": round((t2 - t0) * 1e3, 2), "compile_ms": round((t1 - t0) * 1e3, 2),
                      "translation_units": units, "hiprtc_ms": round(hiprtc_ms, 2)}))


def first_use(tmp, with_c5):
    """First-call cost of c1 and c2 (this process's interpreter, C ABI) and first run() of c5 through the
    module stack, each in a fresh process with an empty compiler cache and again with the cache the
    first process left."""
    env = cold_cache_env(tmp)
    own = dict(env, CUSTOS_HIP_KERNEL_CACHE_DIR=os.path.join(tmp, "custos_code_objects"))
    out = {"what": "a fresh process each; cold = the ROCm compiler library's cache is empty (temporary HOME), warm = the "
                   "same again on the cache the cold process left, code_objects_on_disk = the same again with the library's "
                   "own cache of code objects (CUSTOS_HIP_KERNEL_CACHE_DIR, off by default) filled by a process before; "
                   "first_call_ms = custos_hip_expr_compile + the first launch + a wait"}
    for which in ("c1", "c2"):
        entry = {}
        for state in ("cold", "warm", "fill", "code_objects_on_disk"):
            try:
                proc = subprocess.run([sys.executable, os.path.abspath(__file__), "--first-call", which], capture_output=True,
                                      text=True, timeout=120, env=own if state in ("fill", "code_objects_on_disk") else env)
                if state == "fill":
                    continue
                entry[state] = json.loads(proc.stdout.strip().splitlines()[-1]) if proc.returncode == 0 else {"error": proc.stderr[-300:]}
            except (subprocess.TimeoutExpired, ValueError, IndexError) as e:
                entry[state] = {"error": str(e)[-300:]}
        out[which] = entry
    if with_c5:
        for fuse in (False, True):
            entry = {}
            for state in ("cold", "warm", "fill", "code_objects_on_disk"):
                r = module_stack("c5", 1, 0, fuse=fuse, settle_ms=0, env=own if state in ("fill", "code_objects_on_disk") else env)
                if state == "fill":
                    continue
                entry[state] = {"first_run_ms": r.get("first_run_ms"), "kernel_nodes": r.get("kernel_nodes")} if "error" not in r else r
            out["c5_module_stack" + ("_after_elementwise_fusing" if fuse else "")] = entry
    return out


def measured_traffic(kernel_label):
    """(bytes per launch, source) for the kernel the roofline is quoted on, from the committed
    summary of the rocprofv3 counter runs; (None, None) when the summary does not hold it."""
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
    except OSError:
        return None, None
    m = re.search(rf"^traffic_bytes_per_launch\[{re.escape(kernel_label)}\]\s*=\s*(\d+)", text, flags=re.M)
    return (int(m.group(1)), TRAFFIC_PROFILE) if m else (None, None)


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


def check_chain(got, want, what):
    m = min(got.size, want.size)
    diff = float(np.max(np.abs(got[:m] - want[:m])))
    tol = 8 * float(np.spacing(np.float32(1.0)))
    if not diff <= tol:
        raise SystemExit(f"bench: {what} differs from the CPU oracle: max abs diff {diff} > {tol}")
    return diff


def bench_c2(dev, args, stack):
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
    lib = dev.lib
    fused_step = launcher(dev, lib.custos_hip_apply_fn, kernel, xb.ptr, out.ptr, n)
    algo_bytes = 8.0 * n
    gbs_of = lambda ms: algo_bytes / (ms * 1e-3) / 1e9

    # The comparisons run first, the headline last.

    # unfused comparison: five apply_fn launches through intermediates (40 B/elt moved)
    kernels = [dev.compile(capi.KIND_APPLY, "f32", custos_amd.expr._wrap(op(custos_amd.Resolve("x"))).to_cl_source("f32"), ("x",))
               for op in C2_OPS]
    tmp_a, tmp_b = dev.alloc(n, "f32"), dev.alloc(n, "f32")
    chain = [(xb, tmp_a), (tmp_a, tmp_b), (tmp_b, tmp_a), (tmp_a, tmp_b), (tmp_b, out)]
    unfused_steps = [launcher(dev, lib.custos_hip_apply_fn, k, s.ptr, d.ptr, n) for k, (s, d) in zip(kernels, chain)]

    def unfused_step():
        for one in unfused_steps:
            one()

    unfused_ms, unfused_n = time_floor(dev, unfused_step, launches_per_step=5)
    # the same five launches recorded and replayed: the graph build joins them into one kernel that
    # still writes both intermediates (1 read + 3 writes per element instead of 5 + 5)
    dev.capture_begin()
    unfused_step()
    recorded_unfused = dev.capture_end()
    recorded_ms, recorded_n = time_floor(dev, recorded_unfused.launch)
    recorded_nodes, recorded_joined = recorded_unfused.kernel_nodes, recorded_unfused.fused_launches
    recorded_kernels = recorded_unfused.kernel_names()
    recorded_unfused.destroy()

    # plain copy (identity expression) over the same buffers: the achievable 1R+1W rate on
    # this box, and the known-size dispatch the profiler counters are scaled by
    copy_kernel = dev.compile(capi.KIND_APPLY, "f32", "x", ("x",))
    copy_ms, copy_n = time_floor(dev, launcher(dev, lib.custos_hip_apply_fn, copy_kernel, xb.ptr, tmp_a.ptr, n))

    direct_ms, direct_n = time_floor(dev, fused_step)   # the fused kernel launched directly, not replayed

    # The library's own launch shape: launches alternate their direction and start on the 256 MiB the
    # memory-side cache still holds.  One step = what a lazy run does from its second run on: replay the
    # recording that holds the fused kernel.
    dev.capture_begin()
    fused_step()
    graph = dev.capture_end()
    assert graph.kernel_nodes == 1
    dms, _ = time_exactly(dev, graph.launch, max(args.steps, MIN_LAUNCHES), args.warmup)
    dms /= max(args.steps, MIN_LAUNCHES)
    default_replay = {"ms_per_step": round(dms, 5), "GBps": round(gbs_of(dms), 2), "frac_of_peak": round(gbs_of(dms) / HBM_PEAK_GBS, 4),
                      "per_step": per_step_stats(dev, graph.launch, args.steps), "kernel": dev.kernel_name(kernel),
                      "what": "the library's own launch shape: launches alternate their direction and start on the 256 MiB "
                              "the memory-side cache still holds, so part of this rate is not HBM bandwidth"}
    graph.destroy()

    # Headline.  The same step pinned to plain HBM streaming: every launch walks the array from the first
    # tile to the last, non-temporal loads and stores, so nothing of the previous launch is found in the
    # memory-side cache (one-wavefront workgroups with one vector per thread stream best that way).
    # (With a launch shape given on the command line, that shape is what is timed.)
    if not tuned:
        dev.set_tuning(64, 1, 0, 3 | 64, 1)
    skernel = dev.compile(capi.KIND_APPLY, "f32", src, ("x",))
    dev.capture_begin()
    capi.check(lib.custos_hip_apply_fn(dev.handle, skernel, xb.ptr, out.ptr, n), dev.handle)
    graph = dev.capture_end()
    if not tuned:
        dev.set_tuning(0, 0, 0, 0, 0)
    assert graph.kernel_nodes == 1
    ms, wall_ms = time_exactly(dev, graph.launch, args.steps, args.warmup)
    per_launch_ms = ms / args.steps
    gbs = gbs_of(per_launch_ms)
    per_step = per_step_stats(dev, graph.launch, args.steps)
    sustained = sustained_stats(dev, graph.launch, algo_bytes, seconds=args.sustain_seconds)
    shape = ("the launch shape given on the command line" if tuned else
             "tiles first to last, non-temporal loads, non-temporal stores written through at once, one-wavefront "
             "workgroups, 1 vector per thread")

    # parity of the very buffer that was timed, on the CPU sample
    graph.launch()
    got = out.read()
    graph.destroy()
    base, want = cpu_baseline_c2(x, min(n, 1 << args.cpu_log2n))
    diff = check_chain(got, want, "the fused chain")
    if stack.get("dump") is not None:
        stack["max_abs_diff_vs_cpu_oracle"] = check_chain(stack.pop("dump"), want, "the module stack's fused chain")

    roof_ms = sustained["mean_ms"]
    roof_kernel = dev.kernel_name(skernel)
    traffic, traffic_source = measured_traffic("c2 streaming") if (not tuned and args.log2n == 28) else (None, None)
    return {
        "metric": "fused unary-chain GB/s and % of HBM peak, f32 N=2^28, 1xMI355X",
        "value": round(gbs, 2),
        "unit": "GB/s",
        "ms_per_step": round(per_launch_ms, 5),
        "config": {
            "workload": f"c2: y = relu(sin(x)*2+1)-0.5 as ONE fused kernel (the text that unary fusing of the five recorded "
                        f"apply_fn operations emits), f32, N=2^{args.log2n}, x~U[-pi,pi) seed 0; one step = one replay of the "
                        "one-node recording through custos_hip_graph_launch (C ABI) in the HBM-only launch shape (" + shape +
                        "), no wait between steps; the library's own launch shape: default_replay; the same workload through "
                        "the C++ module stack: module_stack",
            "elements": n,
            "algorithmic_bytes_per_element": 8,
        },
        "kernel": roof_kernel,
        "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "elements_per_s": round(n / (per_launch_ms * 1e-3), 1),
        "wall_ms_per_step": round(wall_ms / args.steps, 5),
        "per_step": per_step,
        "sustained": sustained,
        "default_replay": default_replay,
        "module_stack": stack,
        "direct_launch": {"ms_per_step": round(direct_ms, 5), "GBps": round(gbs_of(direct_ms), 2), "launches": direct_n,
                          "what": "the fused kernel launched directly (custos_hip_apply_fn), the library's own launch shape"},
        "unfused": {
            "ms_per_step": round(unfused_ms, 5),
            "steps": unfused_n,
            "effective_GBps_on_8B_basis": round(gbs_of(unfused_ms), 2),
            "moved_GBps_on_40B_basis": round(5 * gbs_of(unfused_ms), 2),
            "speedup_fused": round(unfused_ms / per_launch_ms, 3),
            "recorded_and_replayed": {
                "ms_per_replay": round(recorded_ms, 5), "replays": recorded_n, "kernel_nodes": recorded_nodes,
                "launches_joined_into_later_ones": recorded_joined, "kernels": recorded_kernels,
                "effective_GBps_on_8B_basis": round(gbs_of(recorded_ms), 2),
                "moved_GBps_on_16B_basis": round(2 * gbs_of(recorded_ms), 2),
                "what": "the five launches recorded without unary fusing; the graph build joins them into one kernel "
                        "that still writes the two intermediate buffers (1 read + 3 writes: 16 B/element)",
            },
        },
        "copy_kernel": {
            "name": dev.kernel_name(copy_kernel),
            "ms_per_launch": round(copy_ms, 5),
            "launches": copy_n,
            "GBps": round(gbs_of(copy_ms), 2),
            "bytes_per_launch": algo_bytes,
        },
        "max_abs_diff_vs_cpu_oracle": diff,
        "roofline": {
            "bound": "hbm",
            "achieved": round(gbs_of(roof_ms), 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(gbs_of(roof_ms) / HBM_PEAK_GBS, 4),
            "frac_median": round(sustained["median_GBps"] / HBM_PEAK_GBS, 4),
            "frac_p99": round(sustained["p99_GBps"] / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel": roof_kernel,
            "algorithmic_bytes_per_launch": algo_bytes,
            "avg_launch_ms": round(roof_ms, 5),
            "launches": sustained["launches"],
            "what": "the headline's kernel and launch shape (HBM only) over the `sustained` region: algorithmic bytes / mean launch "
                    "duration between two events on the library's compute stream (launches back to back); frac_median and "
                    "frac_p99 from the pass with an event between every two launches",
        },
        "cpu_baseline": base,
    }


def cpu_oracle_chain(x):
    from oracle import cpu_oracle
    return cpu_oracle.c2_chain_fused(np.ascontiguousarray(x))


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


def bench_others(dev, args, stack_c5):
    """The other BASELINE configurations (c1, c3, c4, c5), each with its CPU port beside it."""
    import custos_amd
    from custos_amd import Const, capi, synth
    from custos_amd.expr import fused_source
    from oracle import cpu_oracle

    lib, h = dev.lib, dev.handle
    out = {}

    # c1: apply_fn(exp), f32 N = 2^20 (latency-bound: 8 MiB of traffic)
    n = 1 << 20
    x = synth.uniform_f32(0, n, -4, 4)
    xb, ob = dev.buffer(x), dev.alloc(n)
    k = dev.compile(capi.KIND_APPLY, "f32", "exp(x)", ("x",))
    step = launcher(dev, lib.custos_hip_apply_fn, k, xb.ptr, ob.ptr, n)
    ms, launches = time_floor(dev, step)
    cpu_s, want = _cpu_time(cpu_oracle.c1_exp, x)
    got = ob.read()
    assert np.max(np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))) <= 4
    out["c1"] = _entry("c1: apply_fn(exp), f32 N=2^20, U[-4,4) seed 0", n, 8, ms, cpu_s, n,
                       note="back-to-back launches through the C ABI from Python: the larger of the kernel's time "
                            "and the host's time per launch")
    out["c1"]["launches"] = launches
    out["c1"]["kernel"] = dev.kernel_name(k)
    # the same through the C++ device, eager: `HIP<Base>::apply_fn` call after call, child process
    stack_c1 = dict(stack_c5.pop("c1", {"skipped": True}))
    if "dump" in stack_c1:
        first = stack_c1.pop("dump")
        assert np.max(np.abs(first.view(np.int32).astype(np.int64) - want[: first.size].view(np.int32).astype(np.int64))) <= 4
        stack_c1["max_ulp_vs_cpu_oracle"] = int(np.max(np.abs(first.view(np.int32).astype(np.int64) - want[: first.size].view(np.int32).astype(np.int64))))
    out["c1"]["module_stack"] = stack_c1
    # the same launch recorded 64 times into one graph (every launch writes the same output, so
    # the graph is a chain of 64 nodes): the device's time per launch, without the host's
    if args.hipgraph:
        dev.capture_begin()
        for i in range(64):
            capi.check(lib.custos_hip_apply_fn(h, k, xb.ptr, ob.ptr, n), h)
        g = dev.capture_end()
        gms, _ = time_floor(dev, g.launch, launches_per_step=g.kernel_nodes)
        out["c1"]["in_a_graph"] = {"us_per_launch": round(gms / g.kernel_nodes * 1e3, 3), "kernel_nodes": g.kernel_nodes,
                                   "what": "64 such launches into the same output recorded as one hipGraph (a chain of 64 nodes)"}
        g.destroy()

    # c3: unary_ew tanh forward + backward, f32 N = 2^26
    n = 1 << 26
    x = gen_chunked(lambda m, off: synth.normal_f32(0, m, off), n)
    yg = gen_chunked(lambda m, off: synth.uniform_f32(1, m, -1, 1, off), n)
    xb, ygb, yb = dev.buffer(x), dev.buffer(yg), dev.alloc(n)
    gb = dev.buffer(np.full(n, 0.1, dtype=np.float32))
    kf = dev.compile(capi.KIND_APPLY, "f32", "tanh(x)", ("x",))
    grad_src = Const(1.0).sub(custos_amd.Resolve("x").tanh().mul(custos_amd.Resolve("x").tanh())).to_cl_source("f32")
    kb = dev.compile(capi.KIND_UNARY_GRAD, "f32", grad_src, ("x",))
    fwd = launcher(dev, lib.custos_hip_apply_fn, kf, xb.ptr, yb.ptr, n)
    bwd = launcher(dev, lib.custos_hip_add_unary_grad, kb, xb.ptr, gb.ptr, ygb.ptr, n)

    def c3_step():
        fwd()
        bwd()

    ms, c3_steps = time_floor(dev, c3_step, launches_per_step=2)
    ms_f, _ = time_floor(dev, fwd)
    ms_b, _ = time_floor(dev, bwd)
    cn = min(n, 1 << 24)
    g0 = np.full(cn, 0.1, dtype=np.float32)
    cpu_s, _ = _cpu_time(lambda: (cpu_oracle.c3_tanh_fwd(x[:cn]), cpu_oracle.c3_tanh_bwd(x[:cn], g0, yg[:cn])))
    e = _entry("c3: unary_ew tanh fwd + bwd (x_grad += y_grad*(1-tanh(x)^2)), f32 N=2^26", n, 24, ms, cpu_s, cn)
    e["steps"] = c3_steps
    alone = "the same launch repeated by itself (in the sequence above each kernel finds what the other left in the caches)"
    e["forward"] = {"ms": round(ms_f, 5), "GBps": round(8 * n / (ms_f * 1e-3) / 1e9, 2), "kernel": dev.kernel_name(kf), "what": alone}
    e["backward"] = {"ms": round(ms_b, 5), "GBps": round(16 * n / (ms_b * 1e-3) / 1e9, 2), "kernel": dev.kernel_name(kb), "what": alone}
    # forward + backward recorded once and replayed (a lazy run of the two): the graph build joins them
    # into one kernel that loads x once (20 instead of 24 B/element) and writes y and x_grad
    dev.capture_begin()
    c3_step()
    g3 = dev.capture_end()
    # (one replay over a fresh gradient, checked against the CPU port on the first 2^20 elements)
    m3 = 1 << 20
    gb.slice(0, m3).write(np.full(m3, 0.1, dtype=np.float32))
    yb.slice(0, m3).clear()
    g3.launch()
    dev.sync()
    want_y = cpu_oracle.c3_tanh_fwd(x[:m3])
    want_g = cpu_oracle.c3_tanh_bwd(x[:m3], np.full(m3, 0.1, dtype=np.float32), yg[:m3])
    got_y, got_g = yb.slice(0, m3).read(), gb.slice(0, m3).read()
    assert np.max(np.abs(got_y.view(np.int32).astype(np.int64) - want_y.view(np.int32).astype(np.int64))) <= 4, "c3 replay: y"
    assert np.max(np.abs(got_g - want_g)) <= 2e-6, "c3 replay: x_grad"
    ms_g, replays_g = time_floor(dev, g3.launch)
    e["recorded_and_replayed"] = {"ms": round(ms_g, 5), "replays": replays_g, "kernel_nodes": g3.kernel_nodes,
                                  "launches_joined_into_later_ones": g3.fused_launches, "kernels": g3.kernel_names(),
                                  "GBps_on_24B": round(24 * n / (ms_g * 1e-3) / 1e9, 2),
                                  "moved_GBps_on_20B": round(20 * n / (ms_g * 1e-3) / 1e9, 2)}
    g3.destroy()
    # the same through the C++ module stacks (child processes that ran before this one touched the GPU)
    stacks3 = stack_c5.pop("c3", {"skipped": True})
    for name, r in (stacks3.items() if "skipped" not in stacks3 else ()):
        if "dump" not in r:
            continue
        both = r.pop("dump")
        k3 = both.size // 2
        dy = np.abs(both[:k3].view(np.int32).astype(np.int64) - cpu_oracle.c3_tanh_fwd(x[:k3]).view(np.int32).astype(np.int64))
        dg = np.abs(both[k3:] - cpu_oracle.c3_tanh_bwd(x[:k3], np.full(k3, 0.1, dtype=np.float32), yg[:k3]))
        if dy.max() > 4 or dg.max() > 2e-6:
            raise SystemExit(f"bench: c3 through the module stack ({name}) differs from the CPU oracle: {dy.max()} ulp, {dg.max()}")
        r["max_ulp_y_vs_cpu_oracle"], r["max_abs_diff_x_grad_vs_cpu_oracle"] = int(dy.max()), float(dg.max())
    e["module_stack"] = stacks3
    out["c3"] = e
    del xb, ygb, yb, gb

    # c4: f16 storage / f32 compute chain exp(x*0.5)*x + x^2, N = 2^28
    n = 1 << args.log2n
    xh = gen_chunked(lambda m, off: synth.uniform_f16_bits(0, m, -2, 2, off), n)
    xb, ob = dev.buffer(xh.view(np.float16), "f16"), dev.alloc(n, "f16")
    c4 = lambda v: v.mul(0.5).exp().mul(v).add(v.mul(v))
    k = dev.compile(capi.KIND_APPLY, "f16", c4(custos_amd.Resolve("x")).to_cl_source("f16"), ("x",))
    ms, c4_steps = time_floor(dev, launcher(dev, lib.custos_hip_apply_fn, k, xb.ptr, ob.ptr, n))
    cn = min(n, 1 << 24)
    cpu_s, want = _cpu_time(cpu_oracle.c4_chain_f16, np.ascontiguousarray(xh[:cn]))
    got = ob.slice(0, cn).read().view(np.uint16)
    d = np.abs(got.view(np.int16).astype(np.int32) - want.view(np.int16).astype(np.int32))
    assert d.max() <= 1, "c4 differs from the CPU port by more than 1 f16 ulp"
    out["c4"] = _entry(f"c4: f16 chain exp(x*0.5)*x + x^2, f32 compute, N=2^{args.log2n}", n, 4, ms, cpu_s, cn)
    out["c4"]["launches"] = c4_steps
    out["c4"]["kernel"] = dev.kernel_name(k)
    stack4 = stack_c5.pop("c4", {"skipped": True})
    if "dump" in stack4:
        first = stack4.pop("dump")
        d4 = np.abs(first.view(np.int16).astype(np.int32) - want[: first.size].view(np.int16).astype(np.int32))
        if d4.max() > 1:
            raise SystemExit("bench: c4 through the module stack differs from the CPU port by more than 1 f16 ulp")
        stack4["max_f16_ulp_vs_cpu_oracle"] = int(d4.max())
    out["c4"]["module_stack"] = stack4
    del xb, ob

    # c5: 1024 buffers x 4096 f32: t=a*b; u=t+c; y=sqrt(abs(u))*0.3, recorded once, replayed
    nbuf, m = 1024, 4096
    mk = lambda seed: dev.buffer(gen_chunked(lambda q, off: synth.uniform_f32(seed, q, 0, 1, off), nbuf * m))
    A, B, Cc = mk(1), mk(2), mk(3)
    T, U, Y = dev.alloc(nbuf * m), dev.alloc(nbuf * m), dev.alloc(nbuf * m)
    kmul = dev.compile(capi.KIND_APPLY, "f32", "(x * y)", ("x", "y"))
    kadd = dev.compile(capi.KIND_APPLY, "f32", "(x + y)", ("x", "y"))
    kun = dev.compile(capi.KIND_APPLY, "f32", fused_source([lambda v: v.abs().sqrt(), lambda v: v.mul(0.3)]), ("x",))
    a, b, c = A.read(), B.read(), Cc.read()
    cpu_s, (_, _, want) = _cpu_time(cpu_oracle.c5_graph, a, b, c)

    def record_c5(fused_kernel=None):
        dev.capture_begin()
        for i in range(nbuf):
            o = i * m * 4
            if fused_kernel is None:
                capi.check(lib.custos_hip_apply_fn2(h, kmul, A.ptr + o, B.ptr + o, T.ptr + o, m), h)
                capi.check(lib.custos_hip_apply_fn2(h, kadd, T.ptr + o, Cc.ptr + o, U.ptr + o, m), h)
                capi.check(lib.custos_hip_apply_fn(h, kun, U.ptr + o, Y.ptr + o, m), h)
            else:
                ptrs = (C.c_uint64 * 3)(A.ptr + o, B.ptr + o, Cc.ptr + o)
                capi.check(lib.custos_hip_apply_fn_n(h, fused_kernel, ptrs, 3, Y.ptr + o, m), h)
        t0 = time.perf_counter()
        graph = dev.capture_end()
        return graph, time.perf_counter() - t0

    def timed_c5(graph, what):
        Y.clear()
        ms_, replays = time_floor(dev, graph.launch, launches_per_step=max(1, graph.kernel_nodes))
        assert np.array_equal(Y.read().view(np.uint32), want.view(np.uint32)), f"c5 {what} differs from the CPU port"
        return {"us_per_replay": round(ms_ * 1e3, 2), "replays": replays, "GBps_on_16B": round(16 * nbuf * m / (ms_ * 1e-3) / 1e9, 2),
                "kernel_nodes": graph.kernel_nodes, "replayed_as": what}

    default_direct = args.direct_replay if args.direct_replay is not None else 4
    graph, build_s = record_c5()
    plain = timed_c5(graph, f"{graph.kernel_nodes} plain launches on the compute stream (a recording of at most "
                            f"{default_direct} nodes is not instantiated as a hipGraph)" if default_direct >= graph.kernel_nodes
                     else "one hipGraphLaunch")
    e = _entry("c5: 1024 x f32[4096], t=a*b; u=t+c; y=sqrt(abs(u))*0.3, 3072 launches recorded once, then replayed",
               nbuf * m, 16, plain["us_per_replay"] * 1e-3, cpu_s, nbuf * m,
               note="GB/s on the minimal 16 B/element; the graph build joins the three launches of a buffer into one "
                    "kernel that still writes t, u and y (24 B/element) and merges the 1024 joined launches into one "
                    "grid; launch by launch the recording moves 32 B/element")
    e["us_per_replay"] = plain["us_per_replay"]
    e["replayed_as"] = plain["replayed_as"]
    e["replays"] = plain["replays"]
    e["graph_kernel_nodes"] = graph.kernel_nodes
    e["recorded_launches"] = 3 * nbuf
    e["graph_build_ms"] = round(build_s * 1e3, 2)
    e["launches_joined_into_later_ones"] = graph.fused_launches
    e["kernel"] = graph.kernel_names()[0]
    graph.destroy()
    # the same recording instantiated as a hipGraph and replayed with one hipGraphLaunch
    if args.hipgraph:
        dev.set_graph_direct_replay(0)
        graph, _ = record_c5()
        e["as_hipgraph"] = timed_c5(graph, f"one hipGraphLaunch of the instantiated {graph.kernel_nodes}-node graph")
        graph.destroy()
        dev.set_graph_direct_replay(default_direct)
    # without joining producers and consumers: one merged launch per recorded level
    dev.set_graph_fusing(False)
    graph, _ = record_c5()
    e["launch_by_launch"] = timed_c5(graph, f"{graph.kernel_nodes} plain launches, one per recorded level (custos_hip_set_graph_fusing off)")
    e["launch_by_launch"]["kernels"] = [dev.kernel_name(q) + "_batched" for q in (kmul, kadd, kun)]
    graph.destroy()
    dev.set_graph_fusing(True)

    # the same work after element-wise fusing (the text `Lazy::elementwise_fusing` of the host stack
    # emits for these operations): one three-operand kernel per buffer, 16 B/element, one node
    kfused = dev.compile(capi.KIND_APPLY, "f32", "(sqrt(abs(((a * b) + c))) * 0.3)", ("a", "b", "c"))
    graph, _ = record_c5(kfused)
    e["fused"] = timed_c5(graph, "1 plain launch on the compute stream")
    e["fused"]["expression"] = "(sqrt(abs(((a * b) + c))) * 0.3)"
    e["fused"]["kernel"] = dev.kernel_name(kfused) + "_batched"
    e["fused"]["GBps"] = e["fused"]["GBps_on_16B"]
    graph.destroy()
    # the same fused expression over the same 1024 operand sets through the entry point that allocates
    # nothing (its table sits in a static device array).  A call identical to the last one finds its
    # rows in the table; a call with other rows is checked on the host and sends its rows through a
    # pinned staging slot: timed here with the sets in two orders, alternating.
    dev.prepare_merged(kfused)
    sets = [(A.ptr + i * m * 4, B.ptr + i * m * 4, Cc.ptr + i * m * 4, Y.ptr + i * m * 4) for i in range(nbuf)]
    rows = (C.c_uint64 * (4 * nbuf))(*[p for row in sets for p in row])
    rows_backwards = (C.c_uint64 * (4 * nbuf))(*[p for row in reversed(sets) for p in row])
    Y.clear()
    na_step = launcher(dev, lib.custos_hip_apply_fn_many_noalloc, kfused, rows, 4, nbuf, m)
    na_ms, na_calls = time_floor(dev, na_step)
    assert np.array_equal(Y.read().view(np.uint32), want.view(np.uint32)), "c5 through the allocation-free entry point differs"
    Y.clear()
    na_other = launcher(dev, lib.custos_hip_apply_fn_many_noalloc, kfused, rows_backwards, 4, nbuf, m)
    def na_alternating():
        na_step()
        na_other()
    alt_ms, alt_calls = time_floor(dev, na_alternating)
    assert np.array_equal(Y.read().view(np.uint32), want.view(np.uint32)), "c5 through the allocation-free entry point differs"
    # sixteen orders in turn: more than the entry point remembers, so every call is checked in full
    Y.clear()
    rotated = [launcher(dev, lib.custos_hip_apply_fn_many_noalloc, kfused,
                        (C.c_uint64 * (4 * nbuf))(*[p for row in sets[k * 61:] + sets[:k * 61] for p in row]), 4, nbuf, m) for k in range(16)]
    def na_new_every_time():
        for call in rotated:
            call()
    new_ms, new_calls = time_floor(dev, na_new_every_time)
    assert np.array_equal(Y.read().view(np.uint32), want.view(np.uint32)), "c5 through the allocation-free entry point differs"
    e["fused"]["allocation_free_entry_point"] = {
        "us_per_call": round(na_ms * 1e3, 2), "calls": na_calls, "GBps_on_16B": round(16 * nbuf * m / (na_ms * 1e-3) / 1e9, 2),
        "us_per_call_alternating_two_tables": round(alt_ms * 1e3 / 2, 2), "calls_alternating": 2 * alt_calls,
        "us_per_call_with_rows_never_seen": round(new_ms * 1e3 / 16, 2), "calls_never_seen": 16 * new_calls,
        "what": "custos_hip_apply_fn_many_noalloc over the same 1024 operand sets, back to back from Python; us_per_call: the same "
                "call again and again (its rows are still in the table: one launch); alternating two tables: both have passed the "
                "operand checks before, 32 KiB of table rows go through a staging slot and the copy kernel before each launch; "
                "rows never seen: sixteen orders of the sets in turn, each call checked in full on the host (4096 address ranges, "
                "in time linear in their number) before its rows are sent"}
    again = stack_c5.get("recorded_again_before_every_run")
    if isinstance(again, dict) and "dump" in again:
        got = again.pop("dump")
        if not np.array_equal(got.view(np.uint32), np.ascontiguousarray(want).reshape(-1)[:got.size].view(np.uint32)):
            raise SystemExit("bench: c5 recorded again before every run differs from the CPU oracle")
        again["first_outputs_equal_the_cpu_oracle_bit_for_bit"] = int(got.size)
    e["module_stack"] = stack_c5
    out["c5"] = e
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
    ap.add_argument("--no-hipgraph", dest="hipgraph", action="store_false",
                    help="skip the two comparisons that launch an instantiated hipGraph (c1 in a 64-node graph, c5 as a "
                         "3-node graph): for runs under rocprofv3, whose kernel tracing ended the process in hipGraphLaunch")
    ap.add_argument("--no-module-stack", dest="module_stack", action="store_false",
                    help="skip the child processes that time the C++ module stack")
    ap.add_argument("--no-first-use", dest="first_use", action="store_false",
                    help="skip the child processes that measure first calls with an empty compiler cache")
    ap.add_argument("--sustain-seconds", dest="sustain_seconds", type=float, default=2.0,
                    help="device time of the back-to-back region behind `sustained` and `roofline`")
    ap.add_argument("--first-call", dest="first_call", choices=sorted(FIRST_CALL_EXPRESSIONS), default=None, help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.first_call:
        first_call_child(args.first_call)
        return
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU; the element-wise path needs no second one "
                         "(--gpus must be 1)")
    if args.steps < 1 or args.warmup < 0:
        raise SystemExit("bench.py: --steps must be positive, --warmup not negative")

    # The module stack and the first-use measurements run in child processes, one after the other,
    # before this process touches the GPU.
    stack, stack_c5, first = {"skipped": True}, {"skipped": True}, {"skipped": True}
    with tempfile.TemporaryDirectory() as tmp:
        if args.first_use:
            first = first_use(os.path.join(tmp, "home"), with_c5=args.others and args.module_stack)
        if args.module_stack:
            dump = os.path.join(tmp, "c2_first.f32")
            stack = module_stack("c2", max(args.steps, MIN_LAUNCHES), args.warmup, log2n=args.log2n, dump=(1 << 20, dump))
            if "error" not in stack and os.path.exists(dump):
                stack["dump"] = np.fromfile(dump, dtype=np.float32)
        if args.module_stack and args.others:
            from custos_amd import synth
            stack_c5 = {"as_recorded": module_stack("c5", 500, 20), "after_elementwise_fusing": module_stack("c5", 500, 20, fuse=True)}
            # the reference's own Lazy module records every operation again before each run
            dump5 = os.path.join(tmp, "c5_rerecorded.f32")
            again = module_stack("c5", 200, 20, rerecord=True, dump=(4096, dump5))
            if "error" not in again and os.path.exists(dump5):
                again["dump"] = np.fromfile(dump5, dtype=np.float32)
            stack_c5["recorded_again_before_every_run"] = again
            dump1 = os.path.join(tmp, "c1_first.f32")
            stack_c5["c1"] = module_stack("c1", 200, 20, dump=(1 << 20, dump1))
            if "error" not in stack_c5["c1"] and os.path.exists(dump1):
                stack_c5["c1"]["dump"] = np.fromfile(dump1, dtype=np.float32)
            # c3 and c4 read their inputs from files (the same synthetic arrays this process generates later)
            n3, n4 = 1 << 26, 1 << args.log2n
            x3, yg3, x4 = (os.path.join(tmp, f) for f in ("c3_x.f32", "c3_yg.f32", "c4_x.f16"))
            gen_chunked(lambda q, off: synth.normal_f32(0, q, off), n3).tofile(x3)
            gen_chunked(lambda q, off: synth.uniform_f32(1, q, -1, 1, off), n3).tofile(yg3)
            gen_chunked(lambda q, off: synth.uniform_f16_bits(0, q, -2, 2, off), n4).tofile(x4)
            stack_c5["c3"] = {}
            for which in ("eager", "lazy", "joined"):
                dump3 = os.path.join(tmp, f"c3_{which}.f32")
                r = module_stack("c3", MIN_LAUNCHES, 10, stack=which, inputs=(x3, yg3), dump=(1 << 20, dump3))
                if "error" not in r and os.path.exists(dump3):
                    r["dump"] = np.fromfile(dump3, dtype=np.float32)
                stack_c5["c3"][which] = r
            dump4 = os.path.join(tmp, "c4_first.f16")
            stack_c5["c4"] = module_stack("c4", MIN_LAUNCHES, 10, log2n=args.log2n, inputs=(x4,), dump=(1 << 20, dump4))
            if "error" not in stack_c5["c4"] and os.path.exists(dump4):
                stack_c5["c4"]["dump"] = np.fromfile(dump4, dtype=np.uint16)

    import custos_amd

    dev = custos_amd.HIP(0)
    if args.direct_replay is not None:
        dev.set_graph_direct_replay(args.direct_replay)
    if args.block or args.unroll or args.blocks_per_cu or args.nontemporal or args.direction:
        dev.set_tuning(args.block, args.unroll, args.blocks_per_cu, args.nontemporal, args.direction)
    info = dev.info()
    res = {"c2": bench_c2}[args.workload](dev, args, stack)
    res["first_use"] = first
    if args.others:
        res["other_configs"] = bench_others(dev, args, stack_c5)
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
