"""Checks the automatic launch shape against pinned shapes on the box at hand.

    python -m custos_amd.calibrate [scenario ...] [--sizes 64,128,...] [--markdown]

The library picks vectors per thread, cache policy and tile direction of every launch from the
bytes the launch touches (`custos_hip_preferred_shape`).  The rules were fitted on one machine;
this sweep shows whether they hold on another: for every scenario and size it times the automatic
choice and every pinned shape (`custos_hip_set_tuning`) and prints GB/s on the algorithmic bytes,
the best pinned shape and how far the automatic choice is from it.

Scenarios (all f32):
    rep1   out = x*1.0001 + 0.5, the same launch again and again          (1 read + 1 write)
    rep3   out = x*1.0001 + y                                              (2 reads + 1 write)
    grad   g = g + o * (x*0.001), the in-place gradient kernel             (3 reads + 1 write)
    chain  three unary launches in a cycle over three arrays, eager
    c3     tanh forward, then its gradient kernel                          (24 B per element)
Sizes are MiB touched by one launch.  Pinned shapes: `u<vectors per thread><policy><direction>`,
policy T = temporal, N = non-temporal loads and stores, W = non-temporal loads and stores written
through at once; direction f = first tile to last, a = alternating from launch to launch.
"""
import argparse
import time

import numpy as np

from . import capi
from .device import HIP

MiB = 1 << 20
POLICY = {"T": -1, "N": 3, "W": 1 | 64}
SCENARIOS = ("rep1", "rep3", "grad", "chain", "c3")
ARRAYS = {"rep1": 2, "rep3": 3, "grad": 3, "chain": 2, "c3": 4}     # operands of ONE launch (c3: of the pair)


def pinned_shapes():
    return [(f"u{u}{p}{'a' if d == 2 else 'f'}", (0, u, 0, POLICY[p], d)) for u in (1, 2) for p in "TNW" for d in (1, 2)]


def _filled(dev, n, base):
    buf = dev.alloc(n, zeroed=False)
    have = min(n, base.size)
    dev.write(buf.slice(0, have), base[:have])
    while have < n:
        chunk = min(have, n - have)
        dev.copy(buf.slice(have, have + chunk), buf.slice(0, chunk))
        have += chunk
    return buf


def _time(dev, step, ms_guess, settle_s=0.03):
    end = time.perf_counter() + settle_s
    while time.perf_counter() < end:
        for _ in range(4):
            step()
        dev.sync()
    reps = int(max(10, min(20000, 25.0 / max(ms_guess, 0.001))))     # about 25 ms of device time
    dev.sync()
    dev.timer_begin()
    for _ in range(reps):
        step()
    return dev.timer_end() / reps


def _scenario(dev, name, n, bufs):
    """(step function, algorithmic bytes per step)."""
    lib, h = dev.lib, dev.handle
    ck = lambda rc: capi.check(rc, h)
    if name == "rep1":
        k = dev.compile(capi.KIND_APPLY, "f32", "((x * 1.0001) + 0.5)", ("x",))
        return (lambda: ck(lib.custos_hip_apply_fn(h, k, bufs[0].ptr, bufs[1].ptr, n))), 8 * n
    if name == "rep3":
        k = dev.compile(capi.KIND_APPLY, "f32", "((x * 1.0001) + y)", ("x", "y"))
        return (lambda: ck(lib.custos_hip_apply_fn2(h, k, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, n))), 12 * n
    if name == "grad":
        k = dev.compile(capi.KIND_UNARY_GRAD, "f32", "(x * 0.001)", ("x",))
        return (lambda: ck(lib.custos_hip_add_unary_grad(h, k, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, n))), 16 * n
    if name == "chain":
        ks = [dev.compile(capi.KIND_APPLY, "f32", s, ("x",)) for s in ("((x * 1.0001) + 0.5)", "(x - 0.5)", "max(x, -3.0)")]

        def step():
            for i in range(3):
                ck(lib.custos_hip_apply_fn(h, ks[i], bufs[i].ptr, bufs[(i + 1) % 3].ptr, n))
        return step, 3 * 8 * n
    if name == "c3":
        kf = dev.compile(capi.KIND_APPLY, "f32", "tanh(x)", ("x",))
        kb = dev.compile(capi.KIND_UNARY_GRAD, "f32", "(1.0 - (tanh(x) * tanh(x)))", ("x",))

        def step():
            ck(lib.custos_hip_apply_fn(h, kf, bufs[0].ptr, bufs[1].ptr, n))
            ck(lib.custos_hip_add_unary_grad(h, kb, bufs[0].ptr, bufs[2].ptr, bufs[3].ptr, n))
        return step, 24 * n
    raise ValueError(f"unknown scenario {name}")


def sweep(dev, scenarios=SCENARIOS, sizes_mib=(64, 128, 256, 512, 768, 1024, 2048), shapes=None, settle_s=0.03):
    """Yields (scenario, MiB, {shape name: GB/s}) with "auto" first; leaves the device's tuning open."""
    shapes = pinned_shapes() if shapes is None else shapes
    base = np.random.default_rng(0).uniform(-1, 1, 1 << 22).astype(np.float32)
    for name in scenarios:
        for mib in sizes_mib:
            if name == "chain" and mib > 768:
                continue
            n = mib * MiB // (4 * ARRAYS[name])
            bufs = [_filled(dev, n, base) for _ in range(3 if name == "chain" else ARRAYS[name])]
            rates = {}
            try:
                for shape, tuning in [("auto", (0, 0, 0, 0, 0))] + list(shapes):
                    dev.set_tuning(*tuning)
                    step, nbytes = _scenario(dev, name, n, bufs)
                    # (the first timing of a cell follows allocations and fills: a longer run-in)
                    ms = _time(dev, step, nbytes / 6.5e9, settle_s * (4 if shape == "auto" else 1))
                    rates[shape] = nbytes / (ms * 1e-3) / 1e9
            finally:
                dev.set_tuning(0, 0, 0, 0, 0)
                dev.sync()
                for b in bufs:
                    b.free()
                dev.pool_trim()
            yield name, mib, rates


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("scenarios", nargs="*", default=list(SCENARIOS))
    ap.add_argument("--sizes", default="64,128,256,512,768,1024,2048", help="MiB touched per launch, comma separated")
    ap.add_argument("--markdown", action="store_true", help="print a table instead of one line per cell")
    args = ap.parse_args(argv)
    sizes = [int(v) for v in args.sizes.split(",")]
    dev = HIP(0)
    names = ["auto"] + [s for s, _ in pinned_shapes()]
    if args.markdown:
        print("| scenario | MiB | " + " | ".join(names) + " | best pinned | auto vs best |")
        print("|---|---|" + "---|" * (len(names) + 2))
    cells = within1 = within4 = 0
    for name, mib, rates in sweep(dev, args.scenarios, sizes):
        pinned = {k: v for k, v in rates.items() if k != "auto"}
        best = max(pinned, key=pinned.get)
        gap = rates["auto"] / pinned[best] - 1.0
        cells += 1
        within1 += gap >= -0.01
        within4 += gap >= -0.04
        if args.markdown:
            print(f"| {name} | {mib} | " + " | ".join(f"{rates[k]:.0f}" for k in names) + f" | {best} | {gap * 100:+.1f} % |", flush=True)
        else:
            print(f"{name:5s} {mib:5d} MiB: " + " ".join(f"{k}:{v:.0f}" for k, v in rates.items()) + f"  best {best}  auto {gap * 100:+.1f} %", flush=True)
    print(f"automatic choice within 1 % of the best pinned shape in {within1} of {cells} cells, within 4 % in {within4}")
    dev.close()
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
