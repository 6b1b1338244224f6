// Times the benchmark configurations the way user code runs them: through the module
// stacks of the C++ mirror on the `HIP` device.
//
//   c1  eager `apply_fn(|x| x.exp())` on `HIP<Base>` over 2^20 f32, again and again: every call prints
//       the expression, looks the kernel up, retrieves a new output buffer and launches; nothing
//       waits between the calls (the reference's eager launches do not wait either), one wait at
//       the end of each timed batch of 64 calls
//   c2  five `apply_fn` calls (sin, *2, +1, max 0, -0.5) on a lazily recorded f32 buffer of
//       `HIP<Graph<Lazy<Base>>>`, `optimize_mem_graph`, `unary_fusing`, then `run()` again and again
//       (the shape of src/op_hint.rs:121-140 and examples/lazy_and_fusing.rs)
//   c3  `unary_ew` tanh with its gradient function (src/unary.rs:97-132) over 2^26 f32, three ways:
//       `--stack eager`  `HIP<Autograd<Base>>`: every step calls `unary_ew` (a new output buffer, the
//                        forward launch, a gradient function on the tape) and `backward` (the tape
//                        runs the gradient launch);
//       `--stack lazy`   `HIP<Autograd<Lazy<Base>>>`: `unary_ew` recorded once, every step is `run()`
//                        (the forward graph) and `backward` (the gradient launch, eagerly), the loop
//                        of src/unary.rs:284-341;
//       `--stack joined` `HIP<Lazy<Base>>`: `apply_fn` and `add_unary_grad` both recorded, every step is
//                        `run()`: the graph build joins the two launches into one kernel that loads x once.
//       The seed of the backward pass is y_grad itself: it is written into y's gradient buffer once,
//       on the device, before the timed steps (what src/unary.rs:383 does with `grad_mut_unbound`), and
//       `backward_from` starts the tape from it.
//   c4  eager `apply_fn(|x| exp(x*0.5)*x + x*x)` on `HIP<Base>` over 2^28 f16
//   c5  1024 buffers of 4096 f32: t = a*b; u = t+c; y = sqrt(abs(u))*0.3, recorded once, run
//       again and again; `--fuse` also calls `elementwise_fusing` first
//       `--rerecord`: the call sequence of the reference's unmodified `Lazy` module on this device
//       (src/modules/lazy.rs:190-197 calls every recorded operation again before each run, and the
//       device's `LazyRun::run` follows: custos_hip_capture_end_reuse, custos_hip_graph_launch,
//       custos_hip_capture_begin), straight through the C ABI: 3072 recorded launches per run, the
//       graph of the run before handed back because the recording is the same
//
// Two figures per configuration, both on the host clock.  `us_per_run`: `steps` steps in a row and one
// wait for the device at the end, divided by `steps`: what a loop of runs costs when nothing looks at
// the results in between (a run returns once its work is queued; `read`, `sync` and the like take the
// wait).  `run_and_wait`: every step followed by `sync()`, timed one by one: what a run costs when
// its result is looked at straight away (the reference's run always waits: src/devices/cuda/lazy.rs:31-49).
// The program prints one JSON line; `bench.py` starts it as a child process.  With `--dump K FILE` the
// first K outputs of a last, separate step are written to FILE so that the caller can compare them with
// its own reference; c3 and c4 read their inputs from files the caller wrote (`--input`, `--input2`).
//
// Inputs of c1, c2, c5 are the synthetic ones of the benchmark: SplitMix64 over a counter, 24 bits
// mapped to lo + u * (hi - lo) in f32 arithmetic.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "custos/custos.hpp"

using namespace custos;
using Dev = HIP<Graph<Lazy<Base>>>;
using Clock = std::chrono::steady_clock;

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

template <class T>
static std::vector<T> read_file(const std::string& path, size_t count) {
    static_assert(std::is_trivially_copyable_v<T>, "raw element type");
    std::vector<T> v(count);
    FILE* f = std::fopen(path.c_str(), "rb");
    if (!f || std::fread(static_cast<void*>(v.data()), sizeof(T), count, f) != count) {
        std::fprintf(stderr, "cannot read %zu elements from %s\n", count, path.c_str());
        std::exit(2);
    }
    std::fclose(f);
    return v;
}

static void write_file(const std::string& path, const void* data, size_t bytes, bool append = false) {
    FILE* f = std::fopen(path.c_str(), append ? "ab" : "wb");
    if (!f || std::fwrite(data, 1, bytes, f) != bytes) {
        std::fprintf(stderr, "cannot write %s\n", path.c_str());
        std::exit(2);
    }
    std::fclose(f);
}

static double us_since(Clock::time_point t0) { return std::chrono::duration<double, std::micro>(Clock::now() - t0).count(); }

struct Timing {
    double queued_us;                      // per step: `steps` steps and one wait
    double wait_mean_us, wait_median_us, wait_min_us;  // per step: every step followed by a wait
    int steps;
};

// `settle_ms`: after the first step (which records, compiles and builds the graph) steps are
// repeated untimed until that much time has passed; after an idle period the device needs some
// tens of milliseconds of work to return to its steady clocks.
template <class F, class W>
static Timing time_runs(F step, W wait, int warmup, int steps, int settle_ms) {
    step();
    wait();
    const auto settled = Clock::now() + std::chrono::milliseconds(settle_ms);
    while (Clock::now() < settled) {
        for (int i = 0; i < 8; i++) step();
        wait();
    }
    for (int i = 0; i < warmup; i++) step();
    wait();
    Timing t{};
    t.steps = steps;
    const auto t0 = Clock::now();
    for (int i = 0; i < steps; i++) step();
    wait();
    t.queued_us = us_since(t0) / steps;
    std::vector<double> us(static_cast<size_t>(steps));
    for (int i = 0; i < steps; i++) {
        const auto t1 = Clock::now();
        step();
        wait();
        us[static_cast<size_t>(i)] = us_since(t1);
    }
    double sum = 0;
    for (double v : us) sum += v;
    std::sort(us.begin(), us.end());
    t.wait_mean_us = sum / steps;
    t.wait_median_us = us[us.size() / 2];
    t.wait_min_us = us.front();
    return t;
}

static std::string timing_json(const Timing& t, double bytes_per_step) {
    char buf[512];
    std::snprintf(buf, sizeof buf,
                  "\"steps\": %d, \"us_per_run\": %.3f, \"GBps\": %.2f, \"run_and_wait\": {\"mean_us\": %.3f, \"median_us\": %.3f, "
                  "\"min_us\": %.3f, \"GBps_median\": %.2f}",
                  t.steps, t.queued_us, bytes_per_step / (t.queued_us * 1e-6) / 1e9, t.wait_mean_us, t.wait_median_us, t.wait_min_us,
                  bytes_per_step / (t.wait_median_us * 1e-6) / 1e9);
    return buf;
}

template <class D>
static void dump_f32(D& device, uint64_t ptr, size_t count, const std::string& path, bool append = false) {
    std::vector<float> first(count);
    device.read_raw(first.data(), ptr, count * sizeof(float));
    write_file(path, first.data(), count * sizeof(float), append);
}

static auto tanh_forward = [](auto x) { return x.tanh(); };
static auto tanh_gradient = [](auto x) { return Scalar<float>(1.f).sub(x.tanh().mul(x.tanh())); };

int main(int argc, char** argv) {
    std::string config = "c2", dump_path, input, input2, stack = "eager";
    int log2n = 0, steps = 100, warmup = 20, settle_ms = 150;
    size_t dump_count = 0;
    bool fuse = false, rerecord = false;
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
        else if (a == "--stack") stack = value();
        else if (a == "--log2n") log2n = std::atoi(value());
        else if (a == "--steps") steps = std::atoi(value());
        else if (a == "--warmup") warmup = std::atoi(value());
        else if (a == "--settle-ms") settle_ms = std::atoi(value());
        else if (a == "--input") input = value();
        else if (a == "--input2") input2 = value();
        else if (a == "--fuse") fuse = true;
        else if (a == "--rerecord") rerecord = true;
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
                },
                [&] { device.sync(); }, warmup, steps, settle_ms);
            if (dump_count) dump_f32(device, out.ptr(), std::min(dump_count, n), dump_path);
            std::printf("{\"config\": \"c1\", \"stack\": \"HIP<Base>\", \"calls\": \"apply_fn(exp) x %d, sync()\", "
                        "\"elements\": %zu, \"steps\": %d, \"warmup\": %d, \"us_per_call\": %.3f, \"median_us\": %.3f, "
                        "\"min_us\": %.3f, \"GBps\": %.2f}\n",
                        batch, n, steps, warmup, t.wait_mean_us / batch, t.wait_median_us / batch, t.wait_min_us / batch,
                        8.0 * static_cast<double>(n) / (t.wait_mean_us / batch * 1e-6) / 1e9);
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
            const auto first = Clock::now();
            device.run();
            device.sync();
            const double first_run_ms = us_since(first) * 1e-3;
            const Timing t = time_runs([&] { device.run(); }, [&] { device.sync(); }, warmup, steps, settle_ms);
            if (dump_count) dump_f32(device, out.replace().ptr(), std::min(dump_count, n), dump_path);
            std::printf("{\"config\": \"c2\", \"stack\": \"HIP<Graph<Lazy<Base>>>\", \"calls\": \"5 x apply_fn, optimize_mem_graph, "
                        "unary_fusing, run()\", \"elements\": %zu, \"warmup\": %d, %s, \"first_run_ms\": %.2f, "
                        "\"kernel_nodes\": %zu, \"graph_builds\": %llu}\n",
                        n, warmup, timing_json(t, 8.0 * static_cast<double>(n)).c_str(), first_run_ms, device.graph_kernel_nodes(),
                        static_cast<unsigned long long>(device.graph_builds()));
        } else if (config == "c3") {
            const size_t n = size_t(1) << (log2n ? log2n : 26);
            if (input.empty() || input2.empty()) {
                std::fprintf(stderr, "c3 needs --input (x) and --input2 (y_grad)\n");
                return 2;
            }
            const std::vector<float> xs = read_file<float>(input, n), ygs = read_file<float>(input2, n);
            const std::vector<float> tenth(n, 0.1f);
            const double bytes = 24.0 * static_cast<double>(n);
            const size_t k = std::min(dump_count, n);
            if (stack == "eager") {
                using D = HIP<Autograd<Base>>;
                D device(0);
                auto x = device.buffer(xs).require_grad();
                auto x_grad = x.grad(device);
                uint64_t y_ptr = 0;
                bool moved = false;
                auto step = [&] {
                    auto y = device.unary_ew(x, tanh_forward, tanh_gradient);
                    if (y_ptr == 0) {
                        // the first output: its gradient buffer is made and takes y_grad, once
                        y_ptr = y.ptr();
                        auto y_grad = y.grad(device);
                        y_grad.write(ygs);
                    }
                    moved = moved || y.ptr() != y_ptr;  // (the pool hands every step's output the same block)
                    device.backward_from(y, [](auto&) {});
                };
                const Timing t = time_runs(step, [&] { device.sync(); }, warmup, steps, settle_ms);
                if (moved) {
                    std::fprintf(stderr, "c3: the output buffer moved between steps, so its gradient was not y_grad\n");
                    return 1;
                }
                if (k) {
                    x_grad.write(tenth);
                    auto y = device.unary_ew(x, tanh_forward, tanh_gradient);
                    device.backward_from(y, [](auto&) {});
                    dump_f32(device, y.ptr(), k, dump_path);
                    dump_f32(device, x_grad.ptr(), k, dump_path, true);
                }
                std::printf("{\"config\": \"c3\", \"stack\": \"HIP<Autograd<Base>>\", \"calls\": \"per step: unary_ew(tanh, 1 - tanh^2), "
                            "backward from y_grad in y's gradient buffer\", \"elements\": %zu, \"warmup\": %d, %s}\n",
                            n, warmup, timing_json(t, bytes).c_str());
            } else if (stack == "lazy") {
                using D = HIP<Autograd<Lazy<Base>>>;
                D device(0);
                auto x = device.buffer(xs).require_grad();
                auto x_grad = x.grad(device);
                auto y = device.unary_ew(x, tanh_forward, tanh_gradient);
                device.run();
                {
                    auto y_grad = y.replace().grad(device);
                    y_grad.write(ygs);
                }
                auto step = [&] {
                    device.run();
                    device.backward_from(y.replace(), [](auto&) {});
                };
                const Timing t = time_runs(step, [&] { device.sync(); }, warmup, steps, settle_ms);
                if (k) {
                    x_grad.write(tenth);
                    step();
                    dump_f32(device, y.replace().ptr(), k, dump_path);
                    dump_f32(device, x_grad.ptr(), k, dump_path, true);
                }
                std::printf("{\"config\": \"c3\", \"stack\": \"HIP<Autograd<Lazy<Base>>>\", \"calls\": \"unary_ew recorded once; per step: "
                            "run(), backward from y_grad in y's gradient buffer\", \"elements\": %zu, \"warmup\": %d, %s, "
                            "\"kernel_nodes\": %zu, \"graph_builds\": %llu}\n",
                            n, warmup, timing_json(t, bytes).c_str(), device.graph_kernel_nodes(),
                            static_cast<unsigned long long>(device.graph_builds()));
            } else if (stack == "joined") {
                using D = HIP<Lazy<Base>>;
                D device(0);
                auto x = device.buffer(xs);
                auto x_grad = device.buffer(tenth);
                auto y_grad = device.buffer(ygs);
                auto y = device.apply_fn(x, tanh_forward);
                device.add_unary_grad(x, x_grad, y_grad, tanh_gradient);
                const Timing t = time_runs([&] { device.run(); }, [&] { device.sync(); }, warmup, steps, settle_ms);
                if (k) {
                    x_grad.write(tenth);
                    device.run();
                    dump_f32(device, y.replace().ptr(), k, dump_path);
                    dump_f32(device, x_grad.ptr(), k, dump_path, true);
                }
                std::printf("{\"config\": \"c3\", \"stack\": \"HIP<Lazy<Base>>\", \"calls\": \"apply_fn(tanh) and add_unary_grad recorded once; "
                            "per step: run() (one kernel: x is loaded once, 20 B/element moved)\", \"elements\": %zu, \"warmup\": %d, %s, "
                            "\"kernel_nodes\": %zu, \"graph_builds\": %llu}\n",
                            n, warmup, timing_json(t, bytes).c_str(), device.graph_kernel_nodes(),
                            static_cast<unsigned long long>(device.graph_builds()));
            } else {
                std::fprintf(stderr, "unknown stack %s\n", stack.c_str());
                return 2;
            }
        } else if (config == "c4") {
            const size_t n = size_t(1) << (log2n ? log2n : 28);
            if (input.empty()) {
                std::fprintf(stderr, "c4 needs --input (x as f16 bits)\n");
                return 2;
            }
            HIP<Base> device(0);
            auto x = device.buffer(read_file<f16>(input, n));
            auto chain = [](auto v) { return v.mul(0.5f).exp().mul(v).add(v.mul(v)); };
            auto out = device.apply_fn(x, chain);
            const Timing t = time_runs([&] { out = device.apply_fn(x, chain); }, [&] { device.sync(); }, warmup, steps, settle_ms);
            if (dump_count) {
                std::vector<f16> first(std::min(dump_count, n));
                device.read_raw(first.data(), out.ptr(), first.size() * sizeof(f16));
                write_file(dump_path, first.data(), first.size() * sizeof(f16));
            }
            std::printf("{\"config\": \"c4\", \"stack\": \"HIP<Base>\", \"calls\": \"per step: apply_fn(exp(x*0.5)*x + x*x), f16\", "
                        "\"elements\": %zu, \"warmup\": %d, %s}\n",
                        n, warmup, timing_json(t, 4.0 * static_cast<double>(n)).c_str());
        } else if (config == "c5" && rerecord) {
            const size_t nbuf = 1024, m = 4096;
            custos_hip_device* dev = nullptr;
            auto check = [&](int32_t rc) {
                if (rc != 0) throw std::runtime_error(custos_hip_last_error(dev));
            };
            check(custos_hip_device_create(0, &dev));
            static const char* const kXY[] = {"x", "y"};
            auto compile = [&](const char* src, int32_t n_markers) {
                custos_hip_kernel* k = nullptr;
                check(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, src, kXY, n_markers, &k));
                return k;
            };
            std::vector<uint64_t> a(nbuf), b(nbuf), c(nbuf), t(nbuf), u(nbuf), y(nbuf);
            for (size_t i = 0; i < nbuf; i++) {
                for (auto* v : {&a, &b, &c, &t, &u, &y}) check(custos_hip_alloc(dev, m * sizeof(float), CUSTOS_HIP_ALLOC_ZEROED, &(*v)[i]));
                const auto ha = uniform_f32(1, m, 0.f, 1.f, i * m), hb = uniform_f32(2, m, 0.f, 1.f, i * m), hc = uniform_f32(3, m, 0.f, 1.f, i * m);
                check(custos_hip_write(dev, a[i], ha.data(), m * sizeof(float)));
                check(custos_hip_write(dev, b[i], hb.data(), m * sizeof(float)));
                check(custos_hip_write(dev, c[i], hc.data(), m * sizeof(float)));
            }
            custos_hip_graph* graph = nullptr;
            uint64_t builds = 0;
            check(custos_hip_capture_begin(dev));  // LazySetup::lazy_setup
            auto run = [&] {
                // Lazy::run calls every recorded operation; each asks for its kernel by the text of its
                // expression and launches it (src/devices/cuda/ops.rs:144-177 formats and looks up per call too)
                for (size_t i = 0; i < nbuf; i++) {
                    check(custos_hip_apply_fn2(dev, compile("(x * y)", 2), a[i], b[i], t[i], m));
                    check(custos_hip_apply_fn2(dev, compile("(x + y)", 2), t[i], c[i], u[i], m));
                    check(custos_hip_apply_fn(dev, compile("(sqrt(abs(x)) * 0.3)", 1), u[i], y[i], m));
                }
                custos_hip_graph* now = nullptr;  // LazyRun::run of the device
                check(custos_hip_capture_end_reuse(dev, graph, &now));
                if (now != graph) {
                    if (graph) check(custos_hip_graph_destroy(dev, graph));
                    graph = now;
                    builds++;
                }
                check(custos_hip_graph_launch(dev, graph));
                check(custos_hip_capture_begin(dev));
            };
            const auto first = Clock::now();
            run();
            check(custos_hip_sync(dev));
            const double first_run_ms = us_since(first) * 1e-3;
            const Timing tm = time_runs(run, [&] { check(custos_hip_sync(dev)); }, warmup, steps, settle_ms);
            if (dump_count) {
                std::vector<float> firsts(std::min(dump_count, m));
                check(custos_hip_read(dev, firsts.data(), y[0], firsts.size() * sizeof(float)));
                write_file(dump_path, firsts.data(), firsts.size() * sizeof(float));
            }
            size_t kernel_nodes = 0;
            check(custos_hip_graph_node_count(graph, &kernel_nodes));
            std::printf("{\"config\": \"c5\", \"stack\": \"C ABI in the order of the reference's Lazy module\", \"calls\": \"per run: 1024 x "
                        "(expr_compile + apply_fn2, expr_compile + apply_fn2, expr_compile + apply_fn) again, capture_end_reuse, graph_launch, capture_begin\", \"elements\": %zu, "
                        "\"warmup\": %d, %s, \"first_run_ms\": %.2f, \"kernel_nodes\": %zu, \"graph_builds\": %llu}\n",
                        nbuf * m, warmup, timing_json(tm, 16.0 * static_cast<double>(nbuf * m)).c_str(), first_run_ms, kernel_nodes,
                        static_cast<unsigned long long>(builds));
            check(custos_hip_device_destroy(dev));
        } else if (config == "c5") {
            const size_t nbuf = 1024, m = 4096;
            Dev device(0);
            std::vector<Buffer<float, Dev>> as, bs, cs, ys;
            for (size_t i = 0; i < nbuf; i++) {
                as.push_back(device.buffer(uniform_f32(1, m, 0.f, 1.f, i * m)));
                bs.push_back(device.buffer(uniform_f32(2, m, 0.f, 1.f, i * m)));
                cs.push_back(device.buffer(uniform_f32(3, m, 0.f, 1.f, i * m)));
            }
            device.sync();
            const auto recording = Clock::now();
            for (size_t i = 0; i < nbuf; i++) {
                auto t = device.apply_fn2(as[i], bs[i], [](auto x, auto y) { return x.mul(y); });
                auto u = device.apply_fn2(t, cs[i], [](auto x, auto y) { return x.add(y); });
                ys.push_back(device.apply_fn(u, [](auto x) { return x.abs().sqrt().mul(0.3f); }));
            }
            if (fuse) device.elementwise_fusing();
            const double record_ms = us_since(recording) * 1e-3;
            const auto first = Clock::now();
            device.run();
            device.sync();
            const double first_run_ms = us_since(first) * 1e-3;
            const Timing t = time_runs([&] { device.run(); }, [&] { device.sync(); }, warmup, steps, settle_ms);
            if (dump_count) dump_f32(device, ys[0].replace().ptr(), std::min(dump_count, m), dump_path);
            std::printf("{\"config\": \"c5\", \"stack\": \"HIP<Graph<Lazy<Base>>>\", \"calls\": \"1024 x (apply_fn2, apply_fn2, apply_fn)%s, "
                        "run()\", \"elements\": %zu, \"warmup\": %d, %s, \"record_ms\": %.2f, \"first_run_ms\": %.2f, \"kernel_nodes\": %zu, "
                        "\"graph_builds\": %llu}\n",
                        fuse ? ", elementwise_fusing" : "", nbuf * m, warmup, timing_json(t, 16.0 * static_cast<double>(nbuf * m)).c_str(),
                        record_ms, first_run_ms, device.graph_kernel_nodes(), static_cast<unsigned long long>(device.graph_builds()));
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
