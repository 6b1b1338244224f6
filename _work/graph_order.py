"""How a recorded program replays under the node orders of a built graph (`custos_hip_set_graph_edges`):
joins between dependency levels, an edge per dependency, one chain level by level, and one chain that
follows the recording where launches are large (the default).

    python3 examples/graph_order.py            # needs an AMD GPU; prints microseconds per replay

Each program is recorded once per order and replayed; the results of the three orders are compared
bit for bit before the timing."""
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import numpy as np

from custos_amd import capi
from custos_amd.device import HIP

ORDERS = (("level joins", capi.GRAPH_EDGES_LEVEL_JOINS), ("per node", capi.GRAPH_EDGES_PER_NODE),
          ("chain by level", capi.GRAPH_EDGES_CHAIN_BY_LEVEL), ("chain", capi.GRAPH_EDGES_CHAIN))
SOURCES = ("((x * 1.0001) + 0.5)", "max(x, -3.0)", "(x - 0.25)", "abs(x)", "(x * 0.999)", "(x + 0.125)", "min(x, 7.0)", "-(x)")


def main():
    dev = HIP(0)
    kernels = [dev.compile(capi.KIND_APPLY, "f32", s, ("x",)) for s in SOURCES]
    dev.set_graph_direct_replay(0)       # always an instantiated graph, so that only the order differs

    def launch(k, buf):
        capi.check(dev.lib.custos_hip_apply_fn(dev.handle, kernels[k], buf.ptr, buf.ptr, buf.len), dev.handle)

    def chains(lengths, elements, kernel_of=lambda chain, depth: chain, chain_by_chain=False):
        """One in-place chain of launches per buffer; recorded level by level like interleaved user code,
        or chain by chain."""
        bufs = [dev.alloc(n) for n in elements]

        def record():
            if chain_by_chain:
                for chain, buf in enumerate(bufs):
                    for depth in range(lengths[chain]):
                        launch(kernel_of(chain, depth) % len(kernels), buf)
                return
            for depth in range(max(lengths)):
                for chain, buf in enumerate(bufs):
                    if depth < lengths[chain]:
                        launch(kernel_of(chain, depth) % len(kernels), buf)
        return bufs, record

    programs = [
        ("two chains of 8 launches, 16 MiB and 16 KiB buffers", chains([8, 8], [1 << 22, 1 << 12], lambda c, d: 4 * c + d % 4)),
        ("4 chains of 16 launches, 16 KiB buffers, one kernel per chain", chains([16] * 4, [1 << 12] * 4)),
        ("8 chains of 2..16 launches, 256 KiB buffers", chains([2 * (c + 1) for c in range(8)], [1 << 16] * 8)),
        ("8 chains of 4 launches, another kernel at every level, 1 MiB buffers", chains([4] * 8, [1 << 18] * 8, lambda c, d: c + d)),
        ("4 chains of 4 launches, 64 MiB buffers", chains([4] * 4, [1 << 24] * 4, lambda c, d: c + d)),
        ("16 chains of 4 launches, 16 MiB buffers, recorded chain by chain",
         chains([4] * 16, [1 << 22] * 16, lambda c, d: c + d, chain_by_chain=True)),
    ]
    print(f"{'program':70s} {'nodes':>5s} " + " ".join(f"{name:>14s}" for name, _ in ORDERS))
    for title, (bufs, record) in programs:
        rng = np.random.default_rng(0)
        inputs = [rng.uniform(-1, 1, b.len).astype(np.float32) for b in bufs]
        times, results, nodes = [], [], 0
        for _, mode in ORDERS:
            dev.set_graph_edges(mode)
            for b, x in zip(bufs, inputs):
                b.write(x)
            dev.capture_begin()
            record()
            graph = dev.capture_end()
            nodes = graph.stats()[1]
            graph.launch()
            dev.sync()
            results.append([b.read() for b in bufs])
            reps = 30 if bufs[0].len >= 1 << 22 else 200
            for _ in range(10):
                graph.launch()
            dev.sync()
            dev.timer_begin()
            for _ in range(reps):
                graph.launch()
            times.append(dev.timer_end() / reps * 1e3)
            graph.destroy()
        for other in results[1:]:
            for got, want in zip(other, results[0]):
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "the orders disagree"
        print(f"{title:70s} {nodes:5d} " + " ".join(f"{t:11.1f} us" for t in times), flush=True)
    dev.set_graph_edges(capi.GRAPH_EDGES_CHAIN)
    dev.close()


if __name__ == "__main__":
    main()
