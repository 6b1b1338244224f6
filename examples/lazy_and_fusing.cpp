// Record five unary operations lazily, let the graph module fuse them into one
// kernel, run them as one replayed graph.
// Counterpart of examples/lazy_and_fusing.rs in the reference, with the fused
// chain of the bench: relu(sin(x) * 2 + 1) - 0.5.
#include <cmath>
#include <cstdio>
#include <vector>

#include "custos/custos.hpp"

using namespace custos;

int main() {
    HIP<Graph<Lazy<Base>>> device(0);
    std::vector<float> host(1 << 20);
    for (size_t i = 0; i < host.size(); i++) host[i] = -3.0f + 6.0f * static_cast<float>(i) / host.size();
    auto buf = device.buffer(host);

    auto s = device.apply_fn(buf, [](auto x) { return x.sin(); });
    auto m = device.apply_fn(s, [](auto x) { return x.mul(2.f); });
    auto a = device.apply_fn(m, [](auto x) { return x.add(1.f); });
    auto r = device.apply_fn(a, [](auto x) { return x.max(0.f); });
    auto out = device.apply_fn(r, [](auto x) { return x.sub(0.5f); });

    // intermediate buffers that nothing else reads share one allocation ...
    device.optimize_mem_graph();
    // ... and the five operations become one kernel: one load, five operations, one store
    device.unary_fusing();
    // records the (single) launch, builds the graph, launches it
    device.run();
    // later runs only replay
    for (int i = 0; i < 3; i++) device.run();

    const std::vector<float> got = out.replace().read();
    double worst = 0;
    for (size_t i = 0; i < host.size(); i++) {
        const float want = std::fmax(std::sin(host[i]) * 2.f + 1.f, 0.f) - 0.5f;
        worst = std::fmax(worst, std::fabs(got[i] - want));
    }
    std::printf("%zu elements, %zu kernel node(s) in the replayed graph, %llu graph build(s), max abs error %.3g\n",
                host.size(), device.graph_kernel_nodes(), static_cast<unsigned long long>(device.graph_builds()), worst);
    return (worst < 1e-6 && device.graph_kernel_nodes() == 1 && device.graph_builds() == 1) ? 0 : 1;
}
