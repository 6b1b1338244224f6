// Times the benchmark configurations the way user code runs them: through the module
// stack `HIP<Graph<Lazy<Base>>>`, with the reference's run semantics (every `run()` launches
// the recorded graph and waits for it: src/devices/cuda/lazy.rs:31-49).
//
//   c1  eager `apply_fn(|x| x.exp())` on `HIP<Base>` over 2^20 f32, again and again: every call prints
//       the expression, looks the kernel up, retrieves a new output buffer and launches; nothing
//       waits between the calls (the reference's eager launches do not wait either), one wait at
//       the end of each timed batch of 64 calls
//   c2  five `apply_fn` calls (sin, *2, +1, max 0, -0.5) on a lazily recorded f32 buffer,
//       `optimize_mem_graph`, `unary_fusing`, then `run()` again and again
//       (the shape of src/op_hint.rs:121-140 and examples/lazy_and_fusing.rs)
//   c5  1024 buffers of 4096 f32: t = a*b; u = t+c; y = sqrt(abs(u))*0.3, recorded once, run
//       again and again; `--fuse` also calls `elementwise_fusing` first
//
// Every run is timed on the host clock around `device.run()`, wait included, and the program
// prints one JSON line (mean, median and minimum per run).  `bench.py` starts it as a child
// process; with `--dump K FILE` the first K outputs are written to FILE so that the caller can
// compare them with its own reference.
//
// Inputs are the synthetic ones of the benchmark: SplitMix64 over a counter, 24 bits mapped to
// lo + u * (hi - lo) in f32 arithmetic.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "custos/custos.hpp"

using namespace custos;
using Dev = HIP<Graph<Lazy<Base>>>;

static uint64_t splitmix64(uint64_t seed, uint64_t index) {
    uint64_t z = seed + (index + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static std::vector<float> uniform_f32(uint64_t seed, size_t n, float lo, float span, size_t offset = 0) {
    std::vector<float> v(n);
    for (size_t i = 0; i < n; i++) {
        const float u = static_cast<float>(splitmix64(seed, offset + i) >> 40) * 0x1p-24f;
        const float scaled = u * span;
        v[i] = lo + scaled;
    }
    return v;
}

struct Timing {
    double mean_us, median_us, min_us;
};

// `settle_ms`: after the first run (which records, compiles and builds the graph) runs are
// repeated untimed until that much time has passed; after an idle period the device needs some
// tens of milliseconds of work to return to its steady clocks.
template <class F>
static Timing time_runs(F run, int warmup, int steps, int settle_ms) {
    run();
    const auto settled = std::chrono::steady_clock::now() + std::chrono::milliseconds(settle_ms);
    while (std::chrono::steady_clock::now() < settled) run();
    for (int i = 0; i < warmup; i++) run();
    std::vector<double> us(static_cast<size_t>(steps));
    for (int i = 0; i < steps; i++) {
        const auto t0 = std::chrono::steady_clock::now();
        run();
        us[static_cast<size_t>(i)] = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    }
    double sum = 0;
    for (double v : us) sum += v;
    std::sort(us.begin(), us.end());
    return {sum / steps, us[us.size() / 2], us.front()};
}

static void dump(Dev& device, uint64_t ptr, size_t count, const char* path) {
    std::vector<float> first(count);
    device.read_raw(first.data(), ptr, count * sizeof(float));
    FILE* f = std::fopen(path, "wb");
    if (!f || std::fwrite(first.data(), sizeof(float), count, f) != count) {
        std::fprintf(stderr, "cannot write %s\n", path);
        std::exit(2);
    }
    std::fclose(f);
}

int main(int argc, char** argv) {
    std::string config = "c2", dump_path;
    int log2n = 0, steps = 100, warmup = 20, settle_ms = 150;
    size_t dump_count = 0;
    bool fuse = false;
    for (int i = 1; i < argc; i++) {
        const std::string a = argv[i];
        auto value = [&]() -> const char* {
            if (i + 1 >= argc) {
                std::fprintf(stderr, "%s needs a value\n", a.c_str());
                std::exit(2);
            }
            return argv[++i];
        };
        if (a == "--config") config = value();
        else if (a == "--log2n") log2n = std::atoi(value());
        else if (a == "--steps") steps = std::atoi(value());
        else if (a == "--warmup") warmup = std::atoi(value());
        else if (a == "--settle-ms") settle_ms = std::atoi(value());
        else if (a == "--fuse") fuse = true;
        else if (a == "--dump") {
            dump_count = static_cast<size_t>(std::atoll(value()));
            dump_path = value();
        } else {
            std::fprintf(stderr, "unknown argument %s\n", a.c_str());
            return 2;
        }
    }
    if (steps < 1 || warmup < 0 || settle_ms < 0 || (log2n != 0 && (log2n < 4 || log2n > 32))) return 2;

    try {
        if (config == "c1") {
            const size_t n = size_t(1) << (log2n ? log2n : 20);
            HIP<Base> device(0);
            auto buf = device.buffer(uniform_f32(0, n, -4.f, 8.f));
            const int batch = 64;
            auto out = device.apply_fn(buf, [](auto x) { return x.exp(); });
            const Timing t = time_runs(
                [&] {
                    for (int i = 0; i < batch; i++) out = device.apply_fn(buf, [](auto x) { return x.exp(); });
                    device.sync();
                },
                warmup, steps, settle_ms);
            if (dump_count) {
                std::vector<float> first(std::min(dump_count, n));
                device.read_raw(first.data(), out.ptr(), first.size() * sizeof(float));
                FILE* f = std::fopen(dump_path.c_str(), "wb");
                if (!f || std::fwrite(first.data(), sizeof(float), first.size(), f) != first.size()) return 2;
                std::fclose(f);
            }
            std::printf("{\"config\": \"c1\", \"stack\": \"HIP<Base>\", \"calls\": \"apply_fn(exp) x %d, sync()\", \"waits\": false, "
                        "\"elements\": %zu, \"steps\": %d, \"warmup\": %d, \"us_per_call\": %.3f, \"median_us\": %.3f, "
                        "\"min_us\": %.3f, \"GBps\": %.2f}\n",
                        batch, n, steps, warmup, t.mean_us / batch, t.median_us / batch, t.min_us / batch,
                        8.0 * static_cast<double>(n) / (t.mean_us / batch * 1e-6) / 1e9);
        } else if (config == "c2") {
            const size_t n = size_t(1) << (log2n ? log2n : 28);
            Dev device(0);
            const float pi = 3.14159265358979323846f;
            auto buf = device.buffer(uniform_f32(0, n, -pi, static_cast<float>(3.14159265358979323846 - -3.14159265358979323846)));
            auto s = device.apply_fn(buf, [](auto x) { return x.sin(); });
            auto m = device.apply_fn(s, [](auto x) { return x.mul(2.f); });
            auto a = device.apply_fn(m, [](auto x) { return x.add(1.f); });
            auto r = device.apply_fn(a, [](auto x) { return x.max(0.f); });
            auto out = device.apply_fn(r, [](auto x) { return x.sub(0.5f); });
            device.optimize_mem_graph();
            device.unary_fusing();
            const Timing t = time_runs([&] { device.run(); }, warmup, steps, settle_ms);
            if (dump_count) dump(device, out.replace().ptr(), std::min(dump_count, n), dump_path.c_str());
            const double gbs = 8.0 * static_cast<double>(n) / (t.mean_us * 1e-6) / 1e9;
            std::printf("{\"config\": \"c2\", \"stack\": \"HIP<Graph<Lazy<Base>>>\", \"calls\": \"5 x apply_fn, optimize_mem_graph, "
                        "unary_fusing, run()\", \"waits\": true, \"elements\": %zu, \"steps\": %d, \"warmup\": %d, "
                        "\"us_per_run\": %.3f, \"median_us\": %.3f, \"min_us\": %.3f, \"GBps\": %.2f, \"GBps_median\": %.2f, "
                        "\"kernel_nodes\": %zu, \"graph_builds\": %llu}\n",
                        n, steps, warmup, t.mean_us, t.median_us, t.min_us, gbs,
                        8.0 * static_cast<double>(n) / (t.median_us * 1e-6) / 1e9, device.graph_kernel_nodes(),
                        static_cast<unsigned long long>(device.graph_builds()));
        } else if (config == "c5") {
            const size_t nbuf = 1024, m = 4096;
            Dev device(0);
            std::vector<Buffer<float, Dev>> as, bs, cs, ys;
            for (size_t i = 0; i < nbuf; i++) {
                as.push_back(device.buffer(uniform_f32(1, m, 0.f, 1.f, i * m)));
                bs.push_back(device.buffer(uniform_f32(2, m, 0.f, 1.f, i * m)));
                cs.push_back(device.buffer(uniform_f32(3, m, 0.f, 1.f, i * m)));
            }
            for (size_t i = 0; i < nbuf; i++) {
                auto t = device.apply_fn2(as[i], bs[i], [](auto x, auto y) { return x.mul(y); });
                auto u = device.apply_fn2(t, cs[i], [](auto x, auto y) { return x.add(y); });
                ys.push_back(device.apply_fn(u, [](auto x) { return x.abs().sqrt().mul(0.3f); }));
            }
            if (fuse) device.elementwise_fusing();
            const Timing t = time_runs([&] { device.run(); }, warmup, steps, settle_ms);
            if (dump_count) dump(device, ys[0].replace().ptr(), std::min(dump_count, m), dump_path.c_str());
            const double gbs = 16.0 * static_cast<double>(nbuf * m) / (t.mean_us * 1e-6) / 1e9;
            std::printf("{\"config\": \"c5\", \"stack\": \"HIP<Graph<Lazy<Base>>>\", \"calls\": \"1024 x (apply_fn2, apply_fn2, apply_fn)%s, "
                        "run()\", \"waits\": true, \"elements\": %zu, \"steps\": %d, \"warmup\": %d, \"us_per_run\": %.3f, "
                        "\"median_us\": %.3f, \"min_us\": %.3f, \"GBps_on_16B\": %.2f, \"kernel_nodes\": %zu, \"graph_builds\": %llu}\n",
                        fuse ? ", elementwise_fusing" : "", nbuf * m, steps, warmup, t.mean_us, t.median_us, t.min_us, gbs,
                        device.graph_kernel_nodes(), static_cast<unsigned long long>(device.graph_builds()));
        } else {
            std::fprintf(stderr, "unknown config %s\n", config.c_str());
            return 2;
        }
    } catch (const std::exception& e) {
        std::fprintf(stderr, "bench_module_stack: %s\n", e.what());
        return 1;
    }
    return 0;
}
