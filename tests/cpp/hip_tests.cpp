// The module-stack tests on the HIP device (needs an MI355X), plus what only a
// GPU device has: graph capture/replay behind `run()`.
#include <atomic>
#include <thread>

#include "check.hpp"
#include "custos/custos.hpp"
#include "module_tests.hpp"

using namespace custos;

// f32 transcendentals are within 4 ulp of libm, f64 ones within a few ulp
REGISTER_MODULE_TESTS(HIP, 1e-6)

// src/devices/cuda/lazy.rs:96-196: add, add, mul recorded, nothing runs before run();
// ten runs with rewritten inputs replay one instantiated graph
TEST_CASE(hip_lazy_run_replays_one_graph) {
    using D = HIP<Lazy<Base, int32_t>>;
    D device;
    auto lhs = device.buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto rhs = device.buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto out = lhs.empty_like();
    auto add = [](auto a, auto b) { return a.add(b); };
    auto mul = [](auto a, auto b) { return a.mul(b); };
    device.add_op(std::tie(lhs, rhs, out), [add](Buffer<int32_t, D>& l, Buffer<int32_t, D>& r, Buffer<int32_t, D>& o, D& d) { d.apply_fn2_impl(l, r, o, add); });
    device.add_op(std::tie(out, lhs, rhs), [add](Buffer<int32_t, D>& l, Buffer<int32_t, D>& r, Buffer<int32_t, D>& o, D& d) { d.apply_fn2_impl(l, r, o, add); });
    device.add_op(std::tie(out, rhs, lhs), [mul](Buffer<int32_t, D>& l, Buffer<int32_t, D>& r, Buffer<int32_t, D>& o, D& d) { d.apply_fn2_impl(l, r, o, mul); });
    CHECK_VEC_EQ(out.read(), (std::vector<int32_t>(6, 0)));
    CHECK_VEC_EQ(lhs.read(), (std::vector<int32_t>{1, 2, 3, 4, 5, 6}));
    for (int i = 0; i < 10; i++) {
        lhs.write({1, 2, 3, 4, 5, 6});
        rhs.write({1, 2, 3, 4, 5, 6});
        device.run();
        CHECK_VEC_EQ(out.read(), (std::vector<int32_t>{2, 4, 6, 8, 10, 12}));
        CHECK_VEC_EQ(rhs.read(), (std::vector<int32_t>{3, 6, 9, 12, 15, 18}));
        CHECK_VEC_EQ(lhs.read(), (std::vector<int32_t>{6, 24, 54, 96, 150, 216}));
    }
    CHECK_EQ(device.graph_builds(), uint64_t(1));      // recorded once, replayed ten times
    // every op ran once per run, not twice; the three launches, each reading what the one before
    // wrote, are joined into one kernel
    CHECK_EQ(device.graph_kernel_nodes(), size_t(1));
    // a new operation invalidates the graph: the next run records again
    auto extra = device.apply_fn(out, [](auto x) { return x.add(1); });
    lhs.write({1, 2, 3, 4, 5, 6});
    rhs.write({1, 2, 3, 4, 5, 6});
    device.run();
    CHECK_EQ(device.graph_builds(), uint64_t(2));
    CHECK_EQ(device.graph_kernel_nodes(), size_t(1));
    // as recorded: one node per operation
    device.set_graph_fusing(false);
    auto more = device.apply_fn(out, [](auto x) { return x.add(2); });
    lhs.write({1, 2, 3, 4, 5, 6});
    rhs.write({1, 2, 3, 4, 5, 6});
    device.run();
    CHECK_EQ(device.graph_builds(), uint64_t(3));
    CHECK_EQ(device.graph_kernel_nodes(), size_t(5));
    CHECK_VEC_EQ(more.replace().read(), (std::vector<int32_t>{4, 6, 8, 10, 12, 14}));
    CHECK_VEC_EQ(lhs.read(), (std::vector<int32_t>{6, 24, 54, 96, 150, 216}));
    CHECK_VEC_EQ(extra.replace().read(), (std::vector<int32_t>{3, 5, 7, 9, 11, 13}));
}

// ---- a run returns once its graph is queued; whatever looks at the results next waits ----
//
// The reference's run waits for the stream (src/devices/cuda/lazy.rs:42-43).  The cases below
// go through every way a program can look at device memory, or take it away, after a run, with
// launches long enough (2^22 and more elements, several runs queued) that they are still in
// flight when the next call is made; each is run with the deferred wait (the default) and with
// the wait inside every run, and must see the same values.

namespace {
using LazyI32 = HIP<Lazy<Base, int32_t>>;
constexpr size_t kInFlightLen = (size_t(1) << 22) + 3;

// acc += step, recorded once
void record_accumulate(LazyI32& device, Buffer<int32_t, LazyI32>& acc, Buffer<int32_t, LazyI32>& step) {
    auto add = [](auto a, auto b) { return a.add(b); };
    device.add_op(std::tie(acc, step),
                  [add](Buffer<int32_t, LazyI32>& a, Buffer<int32_t, LazyI32>& o, LazyI32& d) { d.apply_fn2_impl(a, o, a, add); });
}
}  // namespace

TEST_CASE(hip_run_defers_its_wait_and_read_takes_it) {
    for (bool waits : {false, true}) {
        LazyI32 device;
        CHECK(!device.run_waits());  // deferred by default
        device.set_run_waits(waits);
        auto acc = device.buffer(std::vector<int32_t>(kInFlightLen, 0));
        auto one = device.buffer(std::vector<int32_t>(kInFlightLen, 1));
        record_accumulate(device, acc, one);
        for (int i = 0; i < 25; i++) device.run();
        CHECK_VEC_EQ(acc.read(), (std::vector<int32_t>(kInFlightLen, 25)));
        device.run();
        device.sync();
        CHECK_VEC_EQ(acc.read(), (std::vector<int32_t>(kInFlightLen, 26)));
        CHECK_EQ(device.graph_builds(), uint64_t(1));
    }
}

// A write into an operand lands behind the run that is still reading it: short writes go
// through a staging slot and a copy kernel, long ones through the runtime's copy; both on the
// compute stream.
TEST_CASE(hip_write_after_a_run_lands_behind_it) {
    for (bool waits : {false, true})
        for (size_t n : {size_t(1000), kInFlightLen}) {
            LazyI32 device;
            device.set_run_waits(waits);
            // a long launch in front, so that the short program is still queued when the write comes
            auto big = device.buffer(std::vector<int32_t>(kInFlightLen, 0));
            auto big_step = device.buffer(std::vector<int32_t>(kInFlightLen, 1));
            auto acc = device.buffer(std::vector<int32_t>(n, 0));
            auto step = device.buffer(std::vector<int32_t>(n, 3));
            record_accumulate(device, big, big_step);
            record_accumulate(device, acc, step);
            for (int i = 0; i < 4; i++) device.run();
            step.write(std::vector<int32_t>(n, 100));  // the four runs before must have added 3 each
            for (int i = 0; i < 2; i++) device.run();
            CHECK_VEC_EQ(acc.read(), (std::vector<int32_t>(n, 4 * 3 + 2 * 100)));
            CHECK_VEC_EQ(big.read(), (std::vector<int32_t>(kInFlightLen, 6)));
        }
}

// A buffer dropped while runs that use it are queued: its block goes to the pool, the next
// buffer of that size gets the block, and everything that touches it is ordered behind the runs.
TEST_CASE(hip_buffer_dropped_while_runs_are_queued) {
    for (bool waits : {false, true}) {
        LazyI32 device;
        device.set_run_waits(waits);
        auto acc = device.buffer(std::vector<int32_t>(kInFlightLen, 0));
        uint64_t dropped_ptr = 0;
        {
            auto step = device.buffer(std::vector<int32_t>(kInFlightLen, 7));
            dropped_ptr = step.ptr();
            record_accumulate(device, acc, step);
            for (int i = 0; i < 6; i++) device.run();
        }
        // the recorded operation names a buffer that is gone: the error is the run's own, thrown at
        // once, and the runs queued before it are not disturbed
        CHECK_THROWS_KIND(device.run(), DeviceError::InvalidLazyBuf);
        auto fresh = device.buffer(std::vector<int32_t>(kInFlightLen, -1));  // takes the dropped block
        CHECK_EQ(fresh.ptr(), dropped_ptr);
        CHECK_VEC_EQ(acc.read(), (std::vector<int32_t>(kInFlightLen, 42)));
        CHECK_VEC_EQ(fresh.read(), (std::vector<int32_t>(kInFlightLen, -1)));
    }
}

// With a pool that keeps nothing, a dropped buffer goes back to the driver, which waits first.
TEST_CASE(hip_buffer_freed_to_the_driver_while_runs_are_queued) {
    LazyI32 device;
    CHECK_EQ(custos_hip_set_pool_limit(device.handle(), 0), CUSTOS_HIP_OK);
    auto acc = device.buffer(std::vector<int32_t>(kInFlightLen, 0));
    {
        auto step = device.buffer(std::vector<int32_t>(kInFlightLen, 5));
        record_accumulate(device, acc, step);
        for (int i = 0; i < 6; i++) device.run();
    }
    CHECK_VEC_EQ(acc.read(), (std::vector<int32_t>(kInFlightLen, 30)));
}

// The device dropped with runs in flight: its destructor waits before memory, graph and
// streams go.
TEST_CASE(hip_device_dropped_while_runs_are_queued) {
    for (int round = 0; round < 3; round++) {
        LazyI32 device;
        auto acc = device.buffer(std::vector<int32_t>(kInFlightLen, 0));
        auto one = device.buffer(std::vector<int32_t>(kInFlightLen, 1));
        record_accumulate(device, acc, one);
        for (int i = 0; i < 8; i++) device.run();
    }
    CHECK(true);
}

// A changed program is recorded again while the runs of the old one are queued: the new
// recording allocates and the old graph is destroyed, both behind those runs; `exec_now`
// launches directly on the same stream.
TEST_CASE(hip_program_changed_while_runs_are_queued) {
    for (bool waits : {false, true}) {
        LazyI32 device;
        device.set_run_waits(waits);
        auto acc = device.buffer(std::vector<int32_t>(kInFlightLen, 0));
        auto one = device.buffer(std::vector<int32_t>(kInFlightLen, 1));
        record_accumulate(device, acc, one);
        for (int i = 0; i < 5; i++) device.run();
        auto twice = device.apply_fn(acc, [](auto x) { return x.mul(2); });  // lazily allocated output
        device.run();  // records acc += 1; twice = acc * 2
        CHECK_EQ(device.graph_builds(), uint64_t(2));
        CHECK_VEC_EQ(twice.replace().read(), (std::vector<int32_t>(kInFlightLen, 12)));
        for (int i = 0; i < 3; i++) device.run();
        device.exec_now(0);  // drains the two operations: one more pass, eagerly
        CHECK_EQ(device.ops_count(), size_t(0));
        CHECK_VEC_EQ(acc.read(), (std::vector<int32_t>(kInFlightLen, 10)));
        CHECK_VEC_EQ(twice.replace().read(), (std::vector<int32_t>(kInFlightLen, 20)));
    }
}

// One device per thread (tests/threading/threads.rs:5-25; the reference's devices are not
// shared between threads either): three threads, each with a device handle of its own on the
// same GPU, compile, launch, record and read at the same time.
TEST_CASE(hip_one_device_per_thread) {
    std::atomic<int> wrong{0};
    auto eager = [&wrong](int seed) {
        HIP<Base> device(0);
        std::vector<float> xs(50000 + 17 * seed);
        for (size_t i = 0; i < xs.size(); i++) xs[i] = static_cast<float>(i % 1000) * 0.25f + static_cast<float>(seed);
        auto buf = device.buffer(xs);
        for (int round = 0; round < 50; round++) {
            const float k = static_cast<float>(seed * 100 + round);  // a new constant: a new kernel every round
            auto out = device.apply_fn(buf, [k](auto x) { return x.mul(2.f).add(k); });
            const std::vector<float> got = out.read();
            for (size_t i = 0; i < xs.size(); i++) wrong += got[i] != xs[i] * 2.f + k;
        }
    };
    auto lazy = [&wrong]() {
        HIP<Graph<Lazy<Base>>> device(0);
        std::vector<float> xs(30011, 1.5f);
        auto buf = device.buffer(xs);
        auto a = device.apply_fn(buf, [](auto x) { return x.add(1.f); });
        auto b = device.apply_fn(a, [](auto x) { return x.mul(3.f); });
        device.unary_fusing();
        for (int round = 0; round < 50; round++) {
            buf.write(std::vector<float>(xs.size(), static_cast<float>(round)));
            device.run();
            const std::vector<float> got = b.replace().read();
            for (float v : got) wrong += v != (static_cast<float>(round) + 1.f) * 3.f;
        }
    };
    std::thread t1(eager, 1), t2(eager, 2), t3(lazy);
    t1.join();
    t2.join();
    t3.join();
    CHECK_EQ(wrong.load(), 0);
}

// A closure that captures a scalar prints a new text for every value
// (src/two_way_ops/resolve.rs:131-141); the reference compiles each text
// (src/devices/cuda/kernel_cache.rs:45-61).  Here: one compilation for the first value,
// one for the form that takes the value as a launch parameter, none after that --
// eager, recorded into graphs, and merged into one grid.
TEST_CASE(hip_captured_scalars_share_one_kernel) {
    HIP<Base> device;
    std::vector<float> xs(4099);
    for (size_t i = 0; i < xs.size(); i++) xs[i] = static_cast<float>(i) * 0.125f - 200.f;
    auto x = device.buffer(xs);
    const uint64_t before = device.cache_stats().first;
    for (int step = 0; step < 30; step++) {
        const float lr = 0.01f * static_cast<float>(step + 1), eps = 1.f / static_cast<float>(step + 3);
        auto out = device.apply_fn(x, [lr, eps](auto v) { return v.mul(lr).add(eps).abs().min(lr); });
        const std::vector<float> got = out.read();
        for (size_t i = 0; i < xs.size(); i++) {
            const float t = std::fabs(xs[i] * lr + eps);
            CHECK_EQ(got[i], t < lr ? t : lr);
        }
    }
    CHECK_EQ(device.cache_stats().first - before, uint64_t(2));

    // recorded: 64 buffers, each scaled by its own factor, replayed as a graph
    using D = HIP<Lazy<Base>>;
    D lazy;
    std::vector<Buffer<float, D>> ins, outs;
    for (int b = 0; b < 64; b++) ins.push_back(lazy.buffer(std::vector<float>(1000 + 8 * b, static_cast<float>(b))));
    for (int b = 0; b < 64; b++) {
        const float k = 0.5f + static_cast<float>(b % 4);   // four distinct factors
        outs.push_back(lazy.apply_fn(ins[static_cast<size_t>(b)], [k](auto v) { return v.mul(k).sub(1.f); }));
    }
    const uint64_t compiled_before = lazy.cache_stats().first;
    lazy.run();
    CHECK(lazy.cache_stats().first - compiled_before <= uint64_t(2));
    // two grids: the launches whose factor was compiled into the code, and all the others,
    // whose table rows carry each launch's own factor
    CHECK_EQ(lazy.graph_kernel_nodes(), size_t(2));
    for (int b = 0; b < 64; b++) {
        const float k = 0.5f + static_cast<float>(b % 4);
        CHECK_VEC_EQ(outs[static_cast<size_t>(b)].replace().read(), (std::vector<float>(1000 + 8 * b, static_cast<float>(b) * k - 1.f)));
    }
}

// BASELINE configs[1] in miniature, through the whole stack: five apply_fn calls on
// Graph<Lazy<Base>>, fused into one kernel node, bit-identical to the unfused device result
TEST_CASE(hip_fused_chain_is_one_kernel) {
    std::vector<float> xs(10007);
    for (size_t i = 0; i < xs.size(); i++) xs[i] = -3.14159f + 6.28318f * static_cast<float>(i) / xs.size();
    std::vector<float> unfused;
    {
        HIP<Base> eager;
        auto b = eager.buffer<float>(xs);
        auto o = eager.apply_fn(b, [](auto x) { return x.sin(); });
        o = eager.apply_fn(o, [](auto x) { return x.mul(2.f); });
        o = eager.apply_fn(o, [](auto x) { return x.add(1.f); });
        o = eager.apply_fn(o, [](auto x) { return x.max(0.f); });
        o = eager.apply_fn(o, [](auto x) { return x.sub(0.5f); });
        unfused = o.read();
    }
    HIP<Graph<Lazy<Base>>> dev;
    auto buf = dev.buffer<float>(xs);
    auto o1 = dev.apply_fn(buf, [](auto x) { return x.sin(); });
    auto o2 = dev.apply_fn(o1, [](auto x) { return x.mul(2.f); });
    auto o3 = dev.apply_fn(o2, [](auto x) { return x.add(1.f); });
    auto o4 = dev.apply_fn(o3, [](auto x) { return x.max(0.f); });
    auto o5 = dev.apply_fn(o4, [](auto x) { return x.sub(0.5f); });
    dev.optimize_mem_graph();
    dev.unary_fusing();
    dev.run();
    CHECK_EQ(dev.graph_kernel_nodes(), size_t(1));
    CHECK_VEC_EQ(o5.replace().read(), unfused);
    for (int i = 0; i < 3; i++) dev.run();
    CHECK_EQ(dev.graph_builds(), uint64_t(1));
    CHECK_VEC_EQ(o5.replace().read(), unfused);
}

// BASELINE configs[4] through the whole stack, scaled to 64 buffers: per buffer two
// two-operand ops and a unary chain are recorded (256 operations); element-wise fusing
// turns each buffer's four operations into one three-operand kernel, and the graph
// builder merges the 64 independent launches into ONE kernel node.
TEST_CASE(hip_config5_fuses_and_batches_to_one_node) {
    using D = HIP<Graph<Lazy<Base>>>;
    const size_t nbuf = 64, n = 4096;
    auto fill = [](size_t seed, size_t n) {
        std::vector<float> v(n);
        uint64_t s = 0x9E3779B97F4A7C15ull * (seed + 1);
        for (auto& x : v) {
            s ^= s << 13; s ^= s >> 7; s ^= s << 17;
            x = float(s >> 40) * (1.0f / 16777216.0f);
        }
        return v;
    };
    D dev;
    std::vector<Buffer<float, D>> a, b, c, y;
    std::vector<Buffer<float, D>> keep;
    for (size_t i = 0; i < nbuf; i++) {
        a.push_back(dev.buffer<float>(fill(3 * i, n)));
        b.push_back(dev.buffer<float>(fill(3 * i + 1, n)));
        c.push_back(dev.buffer<float>(fill(3 * i + 2, n)));
    }
    for (size_t i = 0; i < nbuf; i++) {
        auto t = dev.apply_fn2(a[i], b[i], [](auto p, auto q) { return p.mul(q); });
        auto u = dev.apply_fn2(t, c[i], [](auto p, auto q) { return p.add(q); });
        auto v = dev.apply_fn(u, [](auto x) { return x.abs().sqrt(); });
        y.push_back(dev.apply_fn(v, [](auto x) { return x.mul(0.3f); }));
        keep.push_back(std::move(t));
        keep.push_back(std::move(u));
        keep.push_back(std::move(v));
    }
    CHECK_EQ(dev.ops_count(), 4 * nbuf);
    dev.optimize_mem_graph();
    dev.elementwise_fusing();
    for (int r = 0; r < 3; r++) dev.run();
    CHECK_EQ(dev.graph_builds(), uint64_t(1));
    CHECK_EQ(dev.graph_kernel_nodes(), size_t(1));
    for (size_t i : {size_t(0), size_t(17), nbuf - 1}) {
        auto av = a[i].read(), bv = b[i].read(), cv = c[i].read();
        std::vector<float> want(n);
        for (size_t k = 0; k < n; k++) {
            float t = av[k] * bv[k];
            float u = t + cv[k];
            float s = std::sqrt(std::fabs(u));
            want[k] = s * 0.3f;
        }
        CHECK_VEC_EQ(y[i].replace().read(), want);
    }
}

static std::string ew_src(const char* fn_name, char op) {
    // src/devices/cuda/lazy.rs:81-93
    return std::string("extern \"C\" __global__ void ") + fn_name +
           "(int* lhs, int* rhs, int* out, int len) {\n"
           "    int idx = blockIdx.x * blockDim.x + threadIdx.x;\n"
           "    if (idx >= len) return;\n"
           "    out[idx] = lhs[idx] " + op + " rhs[idx];\n}\n";
}

// src/devices/cuda/lazy.rs:198-240 (test_cuda_eager_without_lazy): caller-written kernels, launched directly
TEST_CASE(hip_launch_kernel1d_eager) {
    HIP<Base> device;
    auto lhs = device.buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto rhs = device.buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto out = lhs.empty_like();
    const int len = 6;
    device.launch_kernel1d(6, ew_src("add", '+'), "add", lhs, rhs, out, len);
    device.launch_kernel1d(6, ew_src("add", '+'), "add", out, lhs, rhs, len);
    device.launch_kernel1d(6, ew_src("mul", '*'), "mul", out, rhs, lhs, len);
    CHECK_VEC_EQ(out.read(), (std::vector<int32_t>{2, 4, 6, 8, 10, 12}));
    CHECK_VEC_EQ(rhs.read(), (std::vector<int32_t>{3, 6, 9, 12, 15, 18}));
    CHECK_VEC_EQ(lhs.read(), (std::vector<int32_t>{6, 24, 54, 96, 150, 216}));
    // explicit launch shape (cuda_device.rs:99-112)
    const uint32_t grid[3] = {1, 1, 1}, block[3] = {64, 1, 1};
    device.launch_kernel(ew_src("add", '+'), "add", grid, block, 0, lhs, rhs, out, len);
    CHECK_VEC_EQ(out.read(), (std::vector<int32_t>{9, 30, 63, 108, 165, 234}));
}

// src/devices/cuda/lazy.rs:96-196: the same kernels recorded as operations of Lazy and replayed
TEST_CASE(hip_launch_kernel1d_lazy) {
    using D = HIP<Lazy<Base, int32_t>>;
    D device;
    auto lhs = device.buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto rhs = device.buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto out = lhs.empty_like();
    auto op = [](const char* name, char c) {
        return [name, c](Buffer<int32_t, D>& l, Buffer<int32_t, D>& r, Buffer<int32_t, D>& o, D& d) {
            d.launch_kernel1d(l.len(), ew_src(name, c), name, l, r, o, static_cast<int>(l.len()));
        };
    };
    device.add_op(std::tie(lhs, rhs, out), op("add", '+'));
    device.add_op(std::tie(out, lhs, rhs), op("add", '+'));
    device.add_op(std::tie(out, rhs, lhs), op("mul", '*'));
    CHECK_VEC_EQ(out.read(), (std::vector<int32_t>(6, 0)));
    for (int i = 0; i < 10; i++) {
        lhs.write({1, 2, 3, 4, 5, 6});
        rhs.write({1, 2, 3, 4, 5, 6});
        device.run();
    }
    CHECK_EQ(device.graph_builds(), uint64_t(1));
    CHECK_EQ(device.graph_kernel_nodes(), size_t(3));
    CHECK_VEC_EQ(out.read(), (std::vector<int32_t>{2, 4, 6, 8, 10, 12}));
    CHECK_VEC_EQ(rhs.read(), (std::vector<int32_t>{3, 6, 9, 12, 15, 18}));
    CHECK_VEC_EQ(lhs.read(), (std::vector<int32_t>{6, 24, 54, 96, 150, 216}));
}

TEST_CASE(hip_backend_errors_surface) {
    bool threw = false;
    try {
        HIP<Base> nope(1000);
    } catch (const Error& e) {
        threw = e.kind == DeviceError::Backend && e.code == CUSTOS_HIP_ERR_INVALID_DEVICE_INDEX;
    }
    CHECK(threw);
}

// BASELINE configuration 4 through the C++ device: f16 storage, the expression computed in f32
// and rounded once at the store -- within one unit of the last place of the host's value
TEST_CASE(hip_f16_chain_f32_compute) {
    HIP<Base> device;
    const size_t n = 100003;
    std::vector<f16> xs(n);
    for (size_t i = 0; i < n; i++) xs[i] = f16(-2.f + 4.f * static_cast<float>((i * 7919) % n) / n);
    auto out = device.apply_fn(device.buffer(xs), [](auto x) { return x.mul(0.5f).exp().mul(x).add(x.mul(x)); });
    const std::vector<f16> got = out.read();
    size_t exact = 0, off_by_more = 0;
    for (size_t i = 0; i < n; i++) {
        const float x = xs[i];
        const uint16_t want = f16(std::exp(x * 0.5f) * x + x * x).bits;
        const int dist = std::abs(static_cast<int>(got[i].bits) - static_cast<int>(want));
        exact += dist == 0;
        off_by_more += dist > 1;
    }
    CHECK_EQ(off_by_more, size_t(0));
    CHECK(exact > n * 99 / 100);
}

// The three node orders of a built graph over the C ABI: two chains of different lengths and
// kernels, a caller-written kernel in between, a fill; every order checked by the library's
// brute-force ordering check and giving the same values; a repeated recording reuses its graph.
TEST_CASE(hip_graph_orders_reuse_and_fill) {
    HIP<Base> device;
    custos_hip_device* dev = device.handle();
    const size_t n = 20011;
    std::vector<float> xs(n), ys(n);
    for (size_t i = 0; i < n; i++) {
        xs[i] = 0.25f + static_cast<float>(i % 97) * 0.125f;
        ys[i] = -3.f + static_cast<float>(i % 31) * 0.5f;
    }
    const char* halve = "extern \"C\" __global__ void halve(float* p, unsigned long long n) {\n"
                        "  unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x;\n"
                        "  if (i < n) p[i] = p[i] * 0.5f;\n}\n";
    custos_hip_kernel *f = nullptr, *h = nullptr, *scale = nullptr;
    const char* marker = "x";
    CHECK_EQ(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, "((x * 1.5) - 0.25)", &marker, 1, &f), 0);
    CHECK_EQ(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, "(abs(x) + 0.5)", &marker, 1, &h), 0);
    CHECK_EQ(custos_hip_source_compile(dev, halve, "halve", &scale), 0);
    CHECK_EQ(custos_hip_set_graph_verify(dev, 1), 0);
    CHECK_EQ(custos_hip_set_graph_direct_replay(dev, 0), 0);
    CHECK_EQ(custos_hip_set_graph_fusing(dev, 0), 0);  // the nodes as recorded (joined, a's and b's launches would be three kernels)
    std::vector<std::vector<float>> results;
    const size_t want_edges[3] = {11, 8, 8};
    for (int32_t mode : {CUSTOS_HIP_GRAPH_EDGES_LEVEL_JOINS, CUSTOS_HIP_GRAPH_EDGES_PER_NODE, CUSTOS_HIP_GRAPH_EDGES_CHAIN}) {
        CHECK_EQ(custos_hip_set_graph_edges(dev, mode), 0);
        auto a = device.buffer(xs), b = device.buffer(ys);
        auto c = device.buffer(std::vector<float>(n, 7.f));
        custos_hip_graph* graph = nullptr;
        for (int recording = 0; recording < 3; recording++) {
            CHECK_EQ(custos_hip_capture_begin(dev), 0);
            for (int i = 0; i < 4; i++) CHECK_EQ(custos_hip_apply_fn(dev, f, a.ptr(), a.ptr(), n), 0);
            for (int i = 0; i < 2; i++) CHECK_EQ(custos_hip_apply_fn(dev, h, b.ptr(), b.ptr(), n), 0);
            unsigned long long count = n;
            uint64_t a_ptr = a.ptr();
            void* params[2] = {&a_ptr, &count};
            size_t sizes[2] = {8, 8};
            CHECK_EQ(custos_hip_source_launch1d(dev, scale, n, params, sizes, 2), 0);
            CHECK_EQ(custos_hip_apply_fn(dev, h, a.ptr(), a.ptr(), n), 0);
            CHECK_EQ(custos_hip_apply_fn(dev, f, b.ptr(), b.ptr(), n), 0);
            custos_hip_graph* now = nullptr;
            CHECK_EQ(custos_hip_capture_end_reuse(dev, graph, &now), 0);
            CHECK(recording == 0 || now == graph);         // the same program: the same graph, nothing built
            graph = now;
        }
        size_t edges = 0, recorded = 0, kernels = 0, levels = 0;
        CHECK_EQ(custos_hip_graph_edge_count(graph, &edges), 0);
        CHECK_EQ(custos_hip_graph_stats(graph, &recorded, &kernels, &levels), 0);
        CHECK_EQ(edges, want_edges[mode]);
        CHECK_EQ(recorded, size_t(9));
        CHECK_EQ(levels, size_t(6));
        // another recording (one more fill) is another graph
        const float two = 2.f;
        CHECK_EQ(custos_hip_capture_begin(dev), 0);
        CHECK_EQ(custos_hip_fill(dev, c.ptr(), n * sizeof(float), &two, sizeof(float)), 0);
        CHECK_EQ(custos_hip_apply_fn(dev, f, c.ptr(), c.ptr(), n), 0);
        custos_hip_graph* other = nullptr;
        CHECK_EQ(custos_hip_capture_end_reuse(dev, graph, &other), 0);
        CHECK(other != graph);
        CHECK_VEC_EQ(c.read(), std::vector<float>(n, 7.f));   // nothing ran while recording
        for (int replay = 0; replay < 2; replay++) {
            CHECK_EQ(custos_hip_graph_launch(dev, graph), 0);
            CHECK_EQ(custos_hip_graph_launch(dev, other), 0);
        }
        CHECK_EQ(custos_hip_sync(dev), 0);
        CHECK_VEC_EQ(c.read(), std::vector<float>(n, 2.f * 1.5f - 0.25f));
        std::vector<float> got = a.read(), got_b = b.read();
        got.insert(got.end(), got_b.begin(), got_b.end());
        results.push_back(std::move(got));
        CHECK_EQ(custos_hip_graph_destroy(dev, other), 0);
        CHECK_EQ(custos_hip_graph_destroy(dev, graph), 0);
    }
    CHECK_VEC_EQ(results[1], results[0]);
    CHECK_VEC_EQ(results[2], results[0]);
    // against the host, for the first chain's first replay: not needed bit for bit here (the
    // Python suite does that); the values must be finite and the chains must have run twice
    CHECK(results[0][0] != xs[0]);
    CHECK_EQ(custos_hip_set_graph_verify(dev, 0), 0);
}

// The merged launch whose operand table sits in a static device array (no allocation on the
// way): the same values as one launch per operand set, on two calls in a row, the second smaller;
// sizes beyond the table and operand sets that overlap are refused.
TEST_CASE(hip_apply_fn_many_noalloc) {
    HIP<Base> device;
    custos_hip_device* dev = device.handle();
    custos_hip_kernel* k = device.compile(CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, "((a * b) + 0.5)", {"a", "b"});
    {
        // the entry point for merged launches is loaded where allocation is allowed, not by the call
        auto a = device.new_buffer<float>(16), b = device.new_buffer<float>(16), o = device.new_buffer<float>(16);
        const uint64_t row[3] = {a.ptr(), b.ptr(), o.ptr()};
        CHECK_EQ(custos_hip_apply_fn_many_noalloc(dev, k, row, 3, 1, 16), static_cast<int32_t>(CUSTOS_HIP_ERR_NOT_PREPARED));
        CHECK_EQ(custos_hip_kernel_prepare_merged(dev, k), 0);
    }
    for (const auto& shape : {std::pair<size_t, size_t>{19, 3001}, std::pair<size_t, size_t>{4, 130}}) {
        const size_t sets = shape.first, n = shape.second;
        std::vector<Buffer<float, HIP<Base>>> as, bs, outs, singles;
        std::vector<uint64_t> rows;
        for (size_t s = 0; s < sets; s++) {
            std::vector<float> av(n), bv(n);
            for (size_t i = 0; i < n; i++) av[i] = 0.5f + static_cast<float>((i * 7 + s) % 13), bv[i] = 1.25f - static_cast<float>((i + 3 * s) % 5);
            as.push_back(device.buffer(av));
            bs.push_back(device.buffer(bv));
            outs.push_back(device.new_buffer<float>(n));
            singles.push_back(device.new_buffer<float>(n));
            rows.insert(rows.end(), {as[s].ptr(), bs[s].ptr(), outs[s].ptr()});
            CHECK_EQ(custos_hip_apply_fn2(dev, k, as[s].ptr(), bs[s].ptr(), singles[s].ptr(), n), 0);
        }
        CHECK_EQ(custos_hip_apply_fn_many_noalloc(dev, k, rows.data(), 3, sets, n), 0);
        for (size_t s = 0; s < sets; s++) CHECK_VEC_EQ(outs[s].read(), singles[s].read());
        // a set that writes what another set reads
        std::vector<uint64_t> clash = rows;
        clash[5] = as[0].ptr();
        CHECK_EQ(custos_hip_apply_fn_many_noalloc(dev, k, clash.data(), 3, sets, n), static_cast<int32_t>(CUSTOS_HIP_ERR_BAD_OVERLAP));
    }
    std::vector<uint64_t> too_many(3 * 3000, 256);
    CHECK_EQ(custos_hip_apply_fn_many_noalloc(dev, k, too_many.data(), 3, 3000, 16), static_cast<int32_t>(CUSTOS_HIP_ERR_TOO_LARGE));
    CHECK_EQ(custos_hip_apply_fn_many_noalloc(dev, k, too_many.data(), 2, 10, 16), static_cast<int32_t>(CUSTOS_HIP_ERR_ARITY_MISMATCH));
}

// The call sequence of a device under the reference's own Lazy module (src/modules/lazy.rs:190-197:
// every recorded operation is called again before each run; each asks for its kernel by text and
// launches it), through the C ABI: a recording that repeats the one before is recognised as it is
// made, one that stops repeating (another operand, fewer or more operations, a clear in between)
// becomes an ordinary recording, and every run leaves what the same calls issued eagerly leave.
TEST_CASE(hip_program_recorded_again_before_every_run) {
    HIP<Base> device;
    custos_hip_device* dev = device.handle();
    const size_t n = 2000, nbuf = 9;
    const char* xy[] = {"x", "y"};
    std::vector<Buffer<float, HIP<Base>>> a, t, y, te, ye;
    for (size_t i = 0; i <= nbuf; i++) {
        std::vector<float> v(n);
        for (size_t e = 0; e < n; e++) v[e] = 0.25f * static_cast<float>((e * 5 + i * 11) % 23) - 2.f;
        a.push_back(device.buffer(v));
    }
    for (size_t i = 0; i < nbuf; i++) {
        t.push_back(device.new_buffer<float>(n)), y.push_back(device.new_buffer<float>(n));
        te.push_back(device.new_buffer<float>(n)), ye.push_back(device.new_buffer<float>(n));
    }
    struct Step {
        size_t i, j;
        int clear_y = -1;  // index of a y buffer cleared between the two launches of the step, or -1
    };
    auto issue = [&](const std::vector<Step>& program, std::vector<Buffer<float, HIP<Base>>>& ts, std::vector<Buffer<float, HIP<Base>>>& ys) {
        for (const Step& s : program) {
            custos_hip_kernel* k = nullptr;
            CHECK_EQ(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, "((x * y) + 0.5)", xy, 2, &k), 0);
            CHECK_EQ(custos_hip_apply_fn2(dev, k, a[s.i].ptr(), a[s.j].ptr(), ts[s.i].ptr(), n), 0);
            if (s.clear_y >= 0) CHECK_EQ(custos_hip_clear(dev, ys[static_cast<size_t>(s.clear_y)].ptr(), n * sizeof(float)), 0);
            CHECK_EQ(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, "sqrt(abs(x))", xy, 1, &k), 0);
            CHECK_EQ(custos_hip_apply_fn(dev, k, ts[s.i].ptr(), ys[s.i].ptr(), n), 0);
        }
    };
    std::vector<Step> same, middle, shorter, cleared;
    for (size_t i = 0; i < nbuf; i++) same.push_back({i, i + 1});
    middle = same, middle[4].j = 0;
    shorter.assign(same.begin(), same.begin() + 5);
    cleared = same, cleared[6].clear_y = 2;
    custos_hip_graph* graph = nullptr;
    const std::vector<float> zeros(n, 0.f);
    auto run = [&](const std::vector<Step>& program, bool expect_same) {
        for (size_t i = 0; i < nbuf; i++) {
            // (writes execute at once while the device records; a clear would be recorded)
            for (auto* buffers : {&t, &y, &te, &ye}) CHECK_EQ(custos_hip_write(dev, (*buffers)[i].ptr(), zeros.data(), n * sizeof(float)), 0);
        }
        uint64_t before[3], after[3];
        CHECK_EQ(custos_hip_capture_stats(dev, &before[0], &before[1], &before[2]), 0);
        issue(program, t, y);
        custos_hip_graph* now = nullptr;
        CHECK_EQ(custos_hip_capture_end_reuse(dev, graph, &now), 0);
        CHECK_EQ(now == graph, expect_same);
        CHECK_EQ(custos_hip_capture_stats(dev, &after[0], &after[1], &after[2]), 0);
        CHECK_EQ(after[0] - before[0], expect_same ? 1u : 0u);
        CHECK_EQ(after[2] - before[2], expect_same ? 0u : 1u);
        if (now != graph) {
            if (graph) CHECK_EQ(custos_hip_graph_destroy(dev, graph), 0);
            graph = now;
        }
        CHECK_EQ(custos_hip_graph_launch(dev, graph), 0);
        issue(program, te, ye);  // the same calls, eagerly
        CHECK_EQ(custos_hip_capture_begin(dev), 0);
        for (size_t i = 0; i < nbuf; i++) {
            CHECK_VEC_EQ(t[i].read(), te[i].read());
            CHECK_VEC_EQ(y[i].read(), ye[i].read());
        }
    };
    CHECK_EQ(custos_hip_capture_begin(dev), 0);
    run(same, false);
    run(same, true);
    run(same, true);
    run(middle, false);
    run(middle, true);
    run(shorter, false);
    run(shorter, true);
    run(same, false);
    run(cleared, false);
    run(cleared, true);
    run(same, false);
    // random walks: each program is the one before with one change at a random place (another
    // operand, a clear put in or taken out, the end cut off, a step appended), or no change
    uint64_t state = 12345;
    auto next = [&](uint64_t below) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        return (state >> 33) % below;
    };
    std::vector<Step> program = same;
    for (int round = 0; round < 40; round++) {
        std::vector<Step> changed = program;
        switch (next(6)) {
            case 0: break;
            case 1: changed[next(changed.size())].j = next(nbuf + 1); break;
            case 2: changed[next(changed.size())].clear_y = static_cast<int>(next(nbuf)); break;
            case 3: changed[next(changed.size())].clear_y = -1; break;
            case 4: if (changed.size() > 1) changed.resize(1 + next(changed.size() - 1)); break;
            default: if (changed.size() < 2 * nbuf) changed.push_back({next(nbuf), next(nbuf + 1)}); break;
        }
        bool equal = changed.size() == program.size();
        for (size_t k = 0; equal && k < changed.size(); k++)
            equal = changed[k].i == program[k].i && changed[k].j == program[k].j && changed[k].clear_y == program[k].clear_y;
        run(changed, equal);
        program = changed;
    }
    custos_hip_graph* last = nullptr;
    CHECK_EQ(custos_hip_capture_end(dev, &last), 0);
    CHECK_EQ(custos_hip_graph_destroy(dev, last), 0);
    CHECK_EQ(custos_hip_graph_destroy(dev, graph), 0);
}

// Random programs of apply and gradient launches over whole buffers and half views, through the C
// ABI: the replayed graph (producers joined into their consumers, equal launches merged) leaves every
// buffer exactly as the same calls issued one by one do, replay after replay; with joining switched
// off as well.
TEST_CASE(hip_joined_launches_random_programs) {
    HIP<Base> device;
    custos_hip_device* dev = device.handle();
    const size_t n = 3000, nbuf = 6;
    const char* m1[] = {"x"};
    const char* m2[] = {"x", "y"};
    std::vector<custos_hip_kernel*> unary, binary, grads;
    for (const char* src : {"((x * 1.25) + 0.5)", "max(-(x), -3.0)", "sqrt(abs(x))", "min((x * x), 9.0)"}) {
        custos_hip_kernel* k = nullptr;
        CHECK_EQ(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, src, m1, 1, &k), 0);
        unary.push_back(k);
        CHECK_EQ(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_UNARY_GRAD, CUSTOS_HIP_F32, src, m1, 1, &k), 0);
        grads.push_back(k);
    }
    for (const char* src : {"(x + y)", "((x * y) - 0.125)", "max(x, y)"}) {
        custos_hip_kernel* k = nullptr;
        CHECK_EQ(custos_hip_expr_compile(dev, CUSTOS_HIP_KIND_APPLY, CUSTOS_HIP_F32, src, m2, 2, &k), 0);
        binary.push_back(k);
    }
    struct Op {
        int kind, fn, a, b, c;
        size_t lo, len;
    };
    uint64_t state = 12345;
    auto next = [&](uint64_t below) {
        state = state * 6364136223846793005ull + 1442695040888963407ull;
        return (state >> 33) % below;
    };
    size_t joined = 0;
    for (int trial = 0; trial < 6; trial++) {
        std::vector<Op> program;
        for (int i = 0; i < 30; i++) {
            Op op{static_cast<int>(next(4)), 0, static_cast<int>(next(nbuf)), static_cast<int>(next(nbuf)), static_cast<int>(next(nbuf)), 0, n};
            if (next(4) == 0) op.lo = next(2) * 1500, op.len = 1500;   // a half view now and then
            op.fn = static_cast<int>(next(op.kind == 0 ? unary.size() : op.kind == 3 ? grads.size() : binary.size()));
            if (op.kind == 3 && (op.a == op.b || op.b == op.c || op.a == op.c)) op.kind = 0;   // gradient operands are distinct buffers
            program.push_back(op);
        }
        std::vector<std::vector<float>> init(nbuf, std::vector<float>(n));
        for (size_t b = 0; b < nbuf; b++)
            for (size_t i = 0; i < n; i++) init[b][i] = static_cast<float>(static_cast<int>(next(4001)) - 2000) * 0.001f;
        auto run = [&](std::vector<Buffer<float, HIP<Base>>>& bufs) {
            for (const Op& op : program) {
                const uint64_t a = bufs[op.a].ptr() + op.lo * 4, b = bufs[op.b].ptr() + op.lo * 4, c = bufs[op.c].ptr() + op.lo * 4;
                if (op.kind == 0) CHECK_EQ(custos_hip_apply_fn(dev, unary[op.fn], a, b, op.len), 0);
                else if (op.kind == 3) CHECK_EQ(custos_hip_add_unary_grad(dev, grads[op.fn], a, b, c, op.len), 0);
                else CHECK_EQ(custos_hip_apply_fn2(dev, binary[op.fn], a, b, c, op.len), 0);
            }
        };
        for (int fusing = 1; fusing >= 0; fusing--) {
            std::vector<Buffer<float, HIP<Base>>> eager, lazy;
            for (size_t b = 0; b < nbuf; b++) eager.push_back(device.buffer(init[b])), lazy.push_back(device.buffer(init[b]));
            CHECK_EQ(custos_hip_set_graph_fusing(dev, fusing), 0);
            CHECK_EQ(custos_hip_capture_begin(dev), 0);
            run(lazy);
            custos_hip_graph* graph = nullptr;
            CHECK_EQ(custos_hip_capture_end(dev, &graph), 0);
            size_t fused = 0;
            CHECK_EQ(custos_hip_graph_fused_launches(graph, &fused), 0);
            CHECK(fusing || fused == 0);
            joined += fused;
            for (int replay = 0; replay < 2; replay++) {
                run(eager);
                CHECK_EQ(custos_hip_graph_launch(dev, graph), 0);
                for (size_t b = 0; b < nbuf; b++) {
                    const std::vector<float> got = lazy[b].read(), want = eager[b].read();
                    CHECK(std::memcmp(got.data(), want.data(), n * sizeof(float)) == 0);
                }
            }
            CHECK_EQ(custos_hip_graph_destroy(dev, graph), 0);
        }
    }
    CHECK_EQ(custos_hip_set_graph_fusing(dev, 1), 0);
    CHECK(joined > 20);
}

int main(int argc, char** argv) { return check::run(argc, argv); }
