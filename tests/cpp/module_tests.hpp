// Tests of the module stack, generic over the device so that the same bodies
// run on the host test device and on the HIP device -- the way the reference
// instantiates one generic test per device (src/unary.rs:160-241).
// Each case names the reference test it restates.
#pragma once

#include <cmath>
#include <cstdlib>
#include <vector>

#include "check.hpp"
#include "custos/device.hpp"
#include "custos/serde.hpp"

namespace module_tests {

using namespace custos;

static const std::vector<double> SIN_1_4 = {0.8414709848078965, 0.9092974268256817, 0.1411200080598672, -0.7568024953079282};
static const std::vector<double> COS_1_4 = {0.5403023058681398, -0.4161468365471424, -0.9899924966004454, -0.6536436208636119};

template <class V>
std::vector<double> scaled(const V& v, double k) {
    std::vector<double> out;
    for (auto x : v) out.push_back(x * k);
    return out;
}

// ---- Base ----

// src/unary.rs:12-19 (doc test), src/two_way_ops/mod.rs:204-217, 236-245
template <template <class> class DEV>
void base_apply_fn() {
    DEV<Base> device;
    auto a = device.template buffer<double>({1., 2., 3., 3., 2., 1.});
    auto out = device.apply_fn(a, [](auto x) { return x.mul(2.); });
    CHECK_VEC_EQ(out.read(), (std::vector<double>{2., 4., 6., 6., 4., 2.}));

    auto c = device.template buffer<float>({1.f, 3.f, 4.f, 6.f, 3.f, 2.f});
    auto clipped = device.apply_fn(c, [](auto x) { return x.max(3.f).min(5.f); });
    CHECK_VEC_EQ(clipped.read(), (std::vector<float>{3.f, 3.f, 4.f, 5.f, 3.f, 3.f}));

    auto i = device.template buffer<int32_t>({3, 3, 4, 5, 3, 2});
    auto i3 = device.apply_fn(i, [](auto x) { return x.add(3); });
    CHECK_VEC_EQ(i3.read(), (std::vector<int32_t>{6, 6, 7, 8, 6, 5}));
}

// src/unary.rs:36-49 (doc test), src/devices/cuda/ops.rs:259-272
template <template <class> class DEV>
void base_add_unary_grad() {
    DEV<Base> device;
    auto a = device.template buffer<double>({1., 2., 3., 3., 2., 1.});
    auto out_grad = device.template buffer<double>({1., 1., 1., 1., 1., 1.});
    auto lhs_grad = device.template buffer<double>({0., 0., 0., 0., 0., 0.});
    device.add_unary_grad(a, lhs_grad, out_grad, [](auto) { return to_val(2.0); });
    CHECK_VEC_EQ(lhs_grad.read(), (std::vector<double>(6, 2.)));

    auto lhs = device.template buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto g = device.template buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto o = device.template buffer<int32_t>({1, 1, 1, 1, 1, 1});
    device.add_unary_grad(lhs, g, o, [](auto x) { return x.mul(2).add(1); });
    CHECK_VEC_EQ(g.read(), (std::vector<int32_t>{4, 7, 10, 13, 16, 19}));
}

// src/unary.rs:139-158: without Autograd, unary_ew is just the forward pass
template <template <class> class DEV>
void base_unary_ew_forward_only() {
    DEV<Base> device;
    auto buf = device.template buffer<double>({1., 2., 3., 4.});
    auto out = device.unary_ew(buf, [](auto x) { return x.sin(); }, [](auto x) { return x.cos(); });
    CHECK_ROUGHLY(out.read(), SIN_1_4, 1e-12);
}

// src/devices/cpu/cpu_device.rs:135-157: zero length is an error
template <template <class> class DEV>
void base_zero_length_is_an_error() {
    DEV<Base> device;
    CHECK_THROWS_KIND(device.template new_buffer<float>(0), DeviceError::ZeroLengthBuffer);
    CHECK_THROWS_KIND(device.template buffer<float>(std::vector<float>{}), DeviceError::ZeroLengthBuffer);
    auto b = device.template new_buffer<float>(4);
    CHECK_VEC_EQ(b.read(), (std::vector<float>(4, 0.f)));  // Buffer::new is zeroed
    CHECK_THROWS_KIND(b.write(std::vector<float>(3, 1.f)), DeviceError::ShapeLengthMismatch);
}

// ---- Lazy ----

// src/modules/lazy.rs:553-566
template <template <class> class DEV>
void lazy_retrieve_ids() {
    DEV<Lazy<Base, int32_t>> device;
    Buffer<int32_t, DEV<Lazy<Base, int32_t>>> buf(device, 10);
    CHECK(buf.has_data());
    CHECK_EQ(buf.id().id, buf.ptr());
    auto x = device.template retrieve<int32_t>(10);
    CHECK(!x.has_data());
    CHECK(x.id() == (Id{0, 10}));
    auto y = device.template retrieve<int32_t>(10);
    CHECK(y.id() == (Id{1, 10}));
}

// src/modules/lazy.rs:568-585, 634-646, 649-662
template <template <class> class DEV>
void lazy_apply_fn_runs_at_run() {
    DEV<Lazy<Base, int32_t>> device;
    Buffer<int32_t, DEV<Lazy<Base, int32_t>>> buf(device, 10);
    auto out = device.apply_fn(buf, [](auto x) { return x.add(3); });
    CHECK_EQ(device.ops_count(), size_t(1));
    CHECK_THROWS_KIND(out.read(), DeviceError::InvalidLazyBuf);  // no memory behind the handle yet
    device.modules.alloc_later(device);
    CHECK_VEC_EQ(out.replace().read(), (std::vector<int32_t>(10, 0)));  // allocated zeroed, not computed
    device.run();
    CHECK_VEC_EQ(out.replace().read(), (std::vector<int32_t>(10, 3)));
    device.run();  // operations stay recorded: a second run recomputes the same
    CHECK_VEC_EQ(out.replace().read(), (std::vector<int32_t>(10, 3)));
}

// src/modules/lazy.rs:618-632
template <template <class> class DEV>
void lazy_dropped_buffer_is_invalid() {
    DEV<Lazy<Base, int32_t>> device;
    {
        Buffer<int32_t, DEV<Lazy<Base, int32_t>>> buf(device, 10);
        auto out = device.apply_fn(buf, [](auto x) { return x.add(3); });
    }
    CHECK_THROWS_KIND(device.run(), DeviceError::InvalidLazyBuf);
}

// src/modules/lazy.rs:674-698: a user-defined two-operand op next to apply_fn
template <template <class> class DEV>
void lazy_add_and_apply_fn() {
    DEV<Lazy<Base, int32_t>> device;
    Buffer<int32_t, DEV<Lazy<Base, int32_t>>> buf(device, 10);
    auto lhs = device.apply_fn(buf, [](auto x) { return x.add(3); });
    auto rhs = device.template buffer<int32_t>({1, 2, 3, 4, 5, 6, 7, 8, 9, 10});
    CHECK_VEC_EQ(rhs.read(), (std::vector<int32_t>{1, 2, 3, 4, 5, 6, 7, 8, 9, 10}));
    auto out = device.apply_fn2(lhs, rhs, [](auto a, auto b) { return a.add(b); });
    device.run();
    CHECK_VEC_EQ(lhs.replace().read(), (std::vector<int32_t>(10, 3)));
    CHECK_VEC_EQ(out.replace().read(), (std::vector<int32_t>{4, 5, 6, 7, 8, 9, 10, 11, 12, 13}));
}

// src/devices/cuda/ops.rs:274-295
template <template <class> class DEV>
void lazy_add_unary_grad() {
    DEV<Lazy<Base, int32_t>> device;
    auto lhs = device.template buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto lhs_grad = device.template buffer<int32_t>({1, 2, 3, 4, 5, 6});
    auto out = device.template buffer<int32_t>({1, 1, 1, 1, 1, 1});
    device.add_unary_grad(lhs, lhs_grad, out, [](auto x) { return x.add(2); });
    CHECK_VEC_EQ(lhs_grad.read(), (std::vector<int32_t>{1, 2, 3, 4, 5, 6}));
    device.run();
    CHECK_VEC_EQ(lhs_grad.read(), (std::vector<int32_t>{4, 6, 8, 10, 12, 14}));
}

// src/modules/lazy.rs:725-757 and 759-790
template <template <class> class DEV>
void lazy_exec_now_and_last_n() {
    using D = DEV<Lazy<Base, int32_t>>;
    for (int variant = 0; variant < 2; variant++) {
        D device;
        auto out = device.template retrieve<int32_t>(4);
        device.add_op(std::tie(out), [](Buffer<int32_t, D>& o, D&) { o.clear(); });
        {
            auto a = device.template buffer<int32_t>({1, 2, 3, 4});
            auto b = device.template buffer<int32_t>({1, 2, 3, 4});
            device.add_op(std::tie(a, b, out), [](Buffer<int32_t, D>& x, Buffer<int32_t, D>& y, Buffer<int32_t, D>& o, D& dev) {
                dev.apply_fn2_impl(x, y, o, [](auto p, auto q) { return p.add(q); });
            });
            if (variant == 0) device.exec_now(1);
            else device.exec_last_n(1);
            CHECK_VEC_EQ(out.replace().read(), (std::vector<int32_t>{2, 4, 6, 8}));
            CHECK_EQ(device.ops_count(), size_t(1));  // the executed operation was consumed
        }
        device.run();  // only the clear is left; a and b are gone but no longer needed
        CHECK_VEC_EQ(out.replace().read(), (std::vector<int32_t>(4, 0)));
    }
}

// src/modules/lazy/lazy_graph.rs:117-125
template <template <class> class DEV>
void lazy_duplicate_parent_is_rejected() {
    using D = DEV<Lazy<Base, int32_t>>;
    D device;
    auto a = device.template buffer<int32_t>({1, 2, 3, 4});
    CHECK_THROWS_KIND(device.add_op(std::tie(a, a), [](Buffer<int32_t, D>&, Buffer<int32_t, D>&, D&) {}),
                      DeviceError::DuplicateParent);
}

// src/op_hint.rs:41-84
template <template <class> class DEV>
void lazy_op_hints() {
    DEV<Lazy<Base>> dev;
    auto buf = dev.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
    auto o1 = dev.apply_fn(buf, [](auto x) { return x.sin(); });
    auto o2 = dev.apply_fn(o1, [](auto x) { return x.cos(); });
    auto o3 = dev.apply_fn(o2, [](auto x) { return x.ln(); });
    const auto& ops = dev.modules.graph;
    CHECK_EQ(ops.size(), size_t(3));
    const char* want[] = {"sin(x)", "cos(x)", "log(x)"};
    for (int i = 0; i < 3; i++) {
        CHECK(ops[i].hint_kind == OpHintKind::Unary);
        auto h = std::static_pointer_cast<UnaryHint<float>>(ops[i].unary_hint);
        CHECK_EQ(h->to_cl_source("x"), std::string(want[i]));
    }
    // src/op_hint.rs:86-114: evaluating the hints in sequence is the fused chain
    float v = 3.f;
    for (auto& op : ops) v = std::static_pointer_cast<UnaryHint<float>>(op.unary_hint)->eval(v);
    CHECK(std::fabs(v - std::log(std::cos(std::sin(3.f)))) < 1e-6);
    // optimizing without a Graph module has no cache traces (src/modules/lazy.rs:494-511)
    CHECK_THROWS_KIND(dev.unary_fusing(), DeviceError::MissingCacheTraces);
    CHECK_THROWS_KIND(dev.optimize_mem_graph(), DeviceError::MissingCacheTraces);
}

// ---- Graph + Lazy: fusion ----

// src/op_hint.rs:116-141 (CPU), 198-219 (CUDA): optimize_mem_graph, unary_fusing, run
template <template <class> class DEV>
void graph_fuse_chain(bool optimize_mem) {
    DEV<Graph<Lazy<Base>>> dev;
    auto buf = dev.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
    auto o1 = dev.apply_fn(buf, [](auto x) { return x.sin(); });
    auto o2 = dev.apply_fn(o1, [](auto x) { return x.cos(); });
    auto o3 = dev.apply_fn(o2, [](auto x) { return x.ln(); });
    if (optimize_mem) dev.optimize_mem_graph();
    else dev.modules.modules.alloc_later(dev);  // src/op_hint.rs:157
    dev.unary_fusing();
    const auto& ops = dev.modules.modules.graph;
    CHECK(ops[0].hint_kind == OpHintKind::UnaryFused);
    CHECK(ops[1].arg_ids.empty() && ops[2].arg_ids.empty());  // no-ops
    dev.run();
    auto got = o3.replace().read();
    std::vector<double> want;
    for (float x : {1.f, 2.f, 3.f, 4.f, 5.f}) want.push_back(std::log(std::cos(std::sin(x))));
    CHECK_ROUGHLY(got, want, 1e-3);
    if (optimize_mem) {
        // the whole trace shares one allocation
        CHECK_EQ(o1.replace().ptr(), o3.replace().ptr());
        CHECK_EQ(o2.replace().ptr(), o3.replace().ptr());
    } else {
        // intermediates of a fused chain are never computed
        CHECK_VEC_EQ(o1.replace().read(), (std::vector<float>(5, 0.f)));
        CHECK_VEC_EQ(o2.replace().read(), (std::vector<float>(5, 0.f)));
    }
}

// src/op_hint.rs:167-196
template <template <class> class DEV>
void graph_fuse_chain_with_checkpoint() {
    DEV<Graph<Lazy<Base>>> dev;
    auto buf = dev.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
    auto out1 = dev.apply_fn(buf, [](auto x) { return x.sin(); }).checkpoint();
    auto out = dev.apply_fn(out1, [](auto x) { return x.cos(); });
    auto out2 = dev.apply_fn(out, [](auto x) { return x.ln(); });
    dev.modules.modules.alloc_later(dev);
    dev.unary_fusing();
    dev.run();
    CHECK_VEC_EQ(out.replace().read(), (std::vector<float>(5, 0.f)));
    std::vector<double> s, full;
    for (float x : {1.f, 2.f, 3.f, 4.f, 5.f}) {
        s.push_back(std::sin(x));
        full.push_back(std::log(std::cos(std::sin(x))));
    }
    CHECK_ROUGHLY(out1.replace().read(), s, 1e-3);
    CHECK_ROUGHLY(out2.replace().read(), full, 1e-3);
}

// src/op_hint.rs:221-251: two independent chains, recorded interleaved
template <template <class> class DEV>
void graph_fuse_two_chains(double tol) {
    DEV<Graph<Lazy<Base>>> dev;
    auto buf = dev.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
    auto rhs = dev.template buffer<float>({8.f, 2.f, 3.f, 4.f, 5.f});
    auto out1 = dev.apply_fn(buf, [](auto x) { return x.sin(); });
    auto out = dev.apply_fn(rhs, [](auto x) { return x.sin(); });
    auto out2 = dev.apply_fn(out, [](auto x) { return x.cos(); });
    auto out1b = dev.apply_fn(out1, [](auto x) { return x.abs(); });
    auto out3 = dev.apply_fn(out1b, [](auto x) { return x.ln(); });
    dev.optimize_mem_graph();
    dev.unary_fusing();
    dev.run();
    std::vector<double> w3, w2;
    for (float x : {1.f, 2.f, 3.f, 4.f, 5.f}) w3.push_back(std::log(std::fabs(std::sin(x))));
    for (float x : {8.f, 2.f, 3.f, 4.f, 5.f}) w2.push_back(std::cos(std::sin(x)));
    CHECK_ROUGHLY(out3.replace().read(), w3, tol);
    CHECK_ROUGHLY(out2.replace().read(), w2, tol);
}

// A trace that starts with a two-operand op and continues with a unary chain:
// the reference drops the whole trace here; the unary run must be fused and the
// other operations must stay.
template <template <class> class DEV>
void graph_fuse_after_binary_ops() {
    DEV<Graph<Lazy<Base>>> dev;
    auto a = dev.template buffer<float>({0.5f, 0.25f, 0.75f, 1.f});
    auto b = dev.template buffer<float>({2.f, 4.f, 0.5f, 3.f});
    auto c = dev.template buffer<float>({-3.f, 0.f, 0.125f, 1.f});
    auto t = dev.apply_fn2(a, b, [](auto x, auto y) { return x.mul(y); });
    auto u = dev.apply_fn2(t, c, [](auto x, auto y) { return x.add(y); });
    auto v = dev.apply_fn(u, [](auto x) { return x.abs().sqrt(); });
    auto y = dev.apply_fn(v, [](auto x) { return x.mul(0.3f); });
    const size_t before = dev.ops_count();
    dev.modules.modules.alloc_later(dev);
    dev.unary_fusing();
    CHECK_EQ(dev.ops_count(), before);
    const auto& ops = dev.modules.modules.graph;
    CHECK(ops[0].hint_kind == OpHintKind::None && !ops[0].arg_ids.empty());   // the mul stays
    CHECK(ops[1].hint_kind == OpHintKind::None && !ops[1].arg_ids.empty());   // the add stays
    CHECK(ops[2].hint_kind == OpHintKind::UnaryFused);
    CHECK(ops[3].arg_ids.empty());
    dev.run();
    std::vector<float> want;
    const float av[] = {0.5f, 0.25f, 0.75f, 1.f}, bv[] = {2.f, 4.f, 0.5f, 3.f}, cv[] = {-3.f, 0.f, 0.125f, 1.f};
    for (int i = 0; i < 4; i++) {
        float tt = av[i] * bv[i];
        float uu = tt + cv[i];
        float s = std::sqrt(std::fabs(uu));
        want.push_back(s * 0.3f);
    }
    CHECK_VEC_EQ(y.replace().read(), want);  // every node is correctly rounded: exact on every device
}

// src/modules/graph/opt_graph/optimize.rs:560-590 (test_lazy_from_retrieve): aliasing
template <template <class> class DEV>
void graph_optimize_mem_aliases() {
    DEV<Graph<Lazy<Base>>> device;
    auto x = device.template buffer<float>(std::vector<float>(1000, 1.f));
    auto b = device.template buffer<float>(std::vector<float>(1000, 1.1f));
    auto squared = device.template retrieve<float>(1000, x, x);
    auto add = device.template retrieve<float>(1000, b, x);
    auto mul_b = device.template retrieve<float>(1000, add, b);
    auto mul = device.template retrieve<float>(1000, squared, x);
    auto out = device.template retrieve<float>(1000, mul, mul_b);
    auto traces = device.modules.graph_trans.opt_graph.cache_traces();
    CHECK_EQ(traces.size(), size_t(2));
    CHECK(traces[0] == (CacheTrace{2, {5, 6}}));
    CHECK(traces[1] == (CacheTrace{3, {4}}));
    device.optimize_mem_graph();
    device.run();
    CHECK_EQ(squared.replace().ptr(), mul.replace().ptr());
    CHECK_EQ(squared.replace().ptr(), out.replace().ptr());
    CHECK_EQ(add.replace().ptr(), mul_b.replace().ptr());
    CHECK(squared.replace().ptr() != add.replace().ptr());
}

// examples/lazy_and_fusing.rs:4-24
template <template <class> class DEV>
void example_lazy_and_fusing() {
    DEV<Graph<Lazy<Base>>> device;
    auto buf = device.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
    auto out1 = device.apply_fn(buf, [](auto x) { return x.add(1.f); });
    auto out2 = device.apply_fn(out1, [](auto x) { return x.sin(); });
    device.optimize_mem_graph();
    device.unary_fusing();
    device.run();
    auto in = buf.read();
    auto got = out2.replace().read();
    for (size_t i = 0; i < in.size(); i++) CHECK(std::fabs(got[i] - std::sin(in[i] + 1.f)) < 0.01);
}

// ---- Autograd ----

// src/unary.rs:160-204
template <template <class> class DEV>
void autograd_unary_ew() {
    DEV<Autograd<Base>> device;
    auto buf = device.template buffer<float>({1.f, 2.f, 3.f, 4.f}).require_grad();
    auto out = device.unary_ew(buf, [](auto x) { return x.sin(); }, [](auto x) { return x.cos(); });
    CHECK_ROUGHLY(out.read(), SIN_1_4, 1e-6);
    out.backward();
    CHECK_ROUGHLY(buf.grad(device).read(), COS_1_4, 1e-6);
}

// src/unary.rs:74-85 (doc test)
template <template <class> class DEV>
void autograd_doc_example() {
    DEV<Autograd<Base>> device;
    auto buf = device.template buffer<double>({1., 2., 3., 3., 2., 1.}).require_grad();
    auto out = device.unary_ew(buf, [](auto x) { return x.mul(2.); }, [](auto) { return to_val(2.0); });
    CHECK_VEC_EQ(out.read(), (std::vector<double>{2., 4., 6., 6., 4., 2.}));
    out.backward();
    CHECK_VEC_EQ(buf.grad(device).read(), (std::vector<double>(6, 2.)));
}

// src/unary.rs:243-282: ten rounds, gradient cleared in between
template <template <class> class DEV>
void autograd_multiple_times(double tol) {
    DEV<Autograd<Base>> device;
    auto buf = device.template buffer<double>({1., 2., 3., 4.}).require_grad();
    for (int i = 0; i < 10; i++) {
        auto out = device.unary_ew(buf, [](auto x) { return x.sin(); }, [](auto x) { return x.cos(); });
        CHECK_ROUGHLY(out.read(), SIN_1_4, tol);
        out.backward();
        CHECK_ROUGHLY(buf.grad(device).read(), COS_1_4, tol);
        auto g = buf.grad(device);
        g.clear();
    }
}

// src/unary.rs:284-326: lazy + autograd, gradients accumulate over repeated run/backward
template <template <class> class DEV>
void autograd_lazy_accumulates(double tol) {
    DEV<Autograd<Lazy<Base, double>>> device;
    auto buf = device.template buffer<double>({1., 2., 3., 4.}).require_grad();
    auto out = device.unary_ew(buf, [](auto x) { return x.sin(); }, [](auto x) { return x.cos(); });
    for (int i = 1; i < 10; i++) {
        device.run();
        CHECK_ROUGHLY(out.replace().read(), SIN_1_4, tol);
        out.backward();
        CHECK_ROUGHLY(buf.grad(device).read(), scaled(COS_1_4, i), tol * 10);
    }
}

// src/unary.rs:328-368: the input of unary_ew is itself lazily computed; second variant
// consumes the first operation with exec_last_n
template <template <class> class DEV>
void autograd_lazy_input(bool exec_last, double tol) {
    DEV<Autograd<Lazy<Base, double>>> device;
    auto buf = device.template buffer<double>({0., 1., 2., 3.}).require_grad();
    auto buf1 = device.apply_fn(buf, [](auto x) { return x.add(1.); });
    if (exec_last) device.exec_last_n(1);
    auto out = device.unary_ew(buf1, [](auto x) { return x.sin(); }, [](auto x) { return x.cos(); });
    for (int i = 1; i < 10; i++) {
        device.run();
        CHECK_ROUGHLY(out.replace().read(), SIN_1_4, tol);
        out.backward();
        CHECK_ROUGHLY(buf1.grad(device).read(), scaled(COS_1_4, i), tol * 10);
    }
}

// src/modules/autograd.rs:494-512
template <template <class> class DEV>
void autograd_grad_new_api() {
    using D = DEV<Autograd<Base>>;
    D device;
    auto lhs = device.template buffer<int32_t>({1, 2, 3, 4}).require_grad();
    auto out = lhs.empty_like();
    device.add_grad_fn(std::tie(lhs, out), [](Buffer<int32_t, D>& l, Buffer<int32_t, D>& o, D& dev) {
        auto lg = l.grad(dev);
        dev.add_unary_grad(l, lg, o.grad(dev), [](auto x) { return x.add(3); });
    });
    out.backward();
    CHECK(lhs.try_grad(device).has_value());
    CHECK_VEC_EQ(lhs.try_grad(device)->read(), (std::vector<int32_t>{4, 5, 6, 7}));
}

// src/modules/autograd.rs:514-542
template <template <class> class DEV>
void autograd_disabling() {
    using D = DEV<Autograd<Base>>;
    D device;
    auto lhs = device.template buffer<int32_t>({1, 2, 3, 4}).require_grad();
    auto out = lhs.empty_like();
    bool called = false;
    device.disable_grad();
    device.add_grad_fn(std::tie(lhs, out), [&called](Buffer<int32_t, D>&, Buffer<int32_t, D>&, D&) { called = true; });
    out.backward();
    CHECK(!called);
    CHECK(!lhs.try_grad(device).has_value());
    device.enable_grad();
    device.add_grad_fn(std::tie(lhs, out), [](Buffer<int32_t, D>& l, Buffer<int32_t, D>& o, D& dev) {
        auto lg = l.grad(dev);
        dev.add_unary_grad(l, lg, o.grad(dev), [](auto x) { return x.add(3); });
    });
    out.backward();
    CHECK_VEC_EQ(lhs.try_grad(device)->read(), (std::vector<int32_t>{4, 5, 6, 7}));
}

// src/modules/autograd.rs:544-590
template <template <class> class DEV>
void autograd_requires_grad_chaining() {
    DEV<Autograd<Base>> device;
    auto lhs = device.template buffer<int32_t>({1, 2, 3, 4}).require_grad();
    CHECK(device.modules.requires_grad_of(lhs.id()) && lhs.requires_grad());
    auto no_grad = device.template buffer<int32_t>({1, 2, 3, 4}).no_grad();
    CHECK(!device.modules.requires_grad_of(no_grad.id()));
    auto rhs = device.template buffer<int32_t>({1, 2, 3, 4}).no_grad();
    CHECK(!rhs.requires_grad());
    CHECK(device.template retrieve<int32_t>(rhs.len(), lhs, rhs).requires_grad());
    CHECK(device.template retrieve<int32_t>(rhs.len(), lhs).requires_grad());
    CHECK(!device.template retrieve<int32_t>(rhs.len(), rhs).requires_grad());
    CHECK(!device.template retrieve<int32_t>(rhs.len(), no_grad, rhs).requires_grad());
    auto out = device.template retrieve<int32_t>(rhs.len(), lhs, rhs);
    CHECK(device.modules.requires_grad_of(out.id()));
}

// src/modules/autograd.rs:434-456: gradient function over buffers kept by Lazy
template <template <class> class DEV>
void autograd_grad_fn_with_lazy_source() {
    using D = DEV<Autograd<Lazy<Base>>>;
    D device;
    auto buf = Buffer<float, D>(device, 10).require_grad();
    Buffer<float, D> out(device, 10);
    device.add_grad_fn(std::tie(buf, out), [](Buffer<float, D>& b, Buffer<float, D>& o, D& dev) {
        auto bg = b.grad(dev);
        // buf.grad = 5 * out.grad, through the unary-gradient kernel on a zeroed gradient
        dev.add_unary_grad(b, bg, o.grad(dev), [](auto) { return to_val(5.f); });
    });
    out.backward();
    CHECK_VEC_EQ(buf.grad(device).read(), (std::vector<float>(10, 5.f)));
}

// src/modules/autograd.rs:458-478: the gradient function's buffer went out of scope
template <template <class> class DEV>
void autograd_grad_fn_out_of_scope() {
    using D = DEV<Autograd<Lazy<Base>>>;
    D device;
    Buffer<float, D> out(device, 10);
    {
        auto buf = Buffer<float, D>(device, 10).require_grad();
        device.add_grad_fn(std::tie(buf, out), [](Buffer<float, D>&, Buffer<float, D>&, D&) {});
    }
    CHECK_THROWS_KIND(out.backward(), DeviceError::InvalidLazyBuf);
}

// BASELINE configs[2] in miniature: tanh forward, backward with a given out gradient,
// x_grad pre-filled with 0.1
template <template <class> class DEV>
void autograd_tanh_config(double tol) {
    using D = DEV<Autograd<Base>>;
    D device;
    std::vector<float> xs = {-1.5f, -0.25f, 0.f, 0.5f, 2.f}, yg = {1.f, -0.5f, 0.25f, 0.75f, -1.f};
    auto x = device.template buffer<float>(xs).require_grad();
    {
        auto g = x.grad(device);
        g.write(std::vector<float>(5, 0.1f));
    }
    auto y = device.unary_ew(x, [](auto v) { return v.tanh(); },
                             [](auto v) { return Scalar<float>(1.f).sub(v.tanh().mul(v.tanh())); });
    y.backward_with(yg);
    std::vector<double> want_y, want_g;
    for (int i = 0; i < 5; i++) {
        double t = std::tanh(static_cast<double>(xs[i]));
        want_y.push_back(t);
        want_g.push_back(0.1 + yg[i] * (1 - t * t));
    }
    CHECK_ROUGHLY(y.read(), want_y, tol);
    CHECK_ROUGHLY(x.grad(device).read(), want_g, tol);
}

// ---- element-wise fusion of any arity (beyond the reference's unary-only fusing) ----

// BASELINE configs[4] per buffer: t = a*b; u = t+c; y = sqrt(abs(u))*0.3 -> one three-operand kernel
template <template <class> class DEV>
void elementwise_fuse_binary_then_unary() {
    DEV<Graph<Lazy<Base>>> dev;
    const std::vector<float> av = {0.5f, 0.25f, 0.75f, 1.f, 0.1f}, bv = {2.f, 4.f, 0.5f, 3.f, 0.7f}, cv = {-3.f, 0.f, 0.125f, 1.f, 0.3f};
    auto a = dev.template buffer<float>(av);
    auto b = dev.template buffer<float>(bv);
    auto c = dev.template buffer<float>(cv);
    auto t = dev.apply_fn2(a, b, [](auto x, auto y) { return x.mul(y); });
    auto u = dev.apply_fn2(t, c, [](auto x, auto y) { return x.add(y); });
    auto v = dev.apply_fn(u, [](auto x) { return x.abs().sqrt(); });
    auto y = dev.apply_fn(v, [](auto x) { return x.mul(0.3f); });
    dev.optimize_mem_graph();
    dev.elementwise_fusing();
    const auto& ops = dev.modules.modules.graph;
    CHECK_EQ(ops.size(), size_t(4));
    CHECK(ops[0].arg_ids.empty() && ops[1].arg_ids.empty() && ops[2].arg_ids.empty());  // inlined
    CHECK(ops[3].hint_kind == OpHintKind::UnaryFused);
    CHECK_EQ(ops[3].fused_source, std::string("(sqrt(abs(((a * b) + c))) * 0.3)"));
    CHECK_EQ(ops[3].arg_ids.size(), size_t(4));  // out + three operand buffers
    dev.run();
    std::vector<float> want;
    for (size_t i = 0; i < av.size(); i++) {
        float tt = av[i] * bv[i];
        float uu = tt + cv[i];
        float s = std::sqrt(std::fabs(uu));
        want.push_back(s * 0.3f);
    }
    CHECK_VEC_EQ(y.replace().read(), want);  // one rounding per node: identical to the unfused result
    dev.run();
    CHECK_VEC_EQ(y.replace().read(), want);
}

// what must NOT be inlined: two readers, checkpoints, user-filled outputs, more than four
// operand buffers, operands overwritten in between, buffers a gradient function needs
template <template <class> class DEV>
void elementwise_fuse_respects_limits() {
    using D = DEV<Graph<Lazy<Base>>>;
    auto count_live = [](const D& dev) {
        size_t n = 0;
        for (const auto& op : dev.modules.modules.graph) n += !op.arg_ids.empty();
        return n;
    };
    {   // two readers of t: t stays, and both readers stay
        D dev;
        auto a = dev.template buffer<float>({1.f, 2.f, 3.f});
        auto t = dev.apply_fn(a, [](auto x) { return x.mul(2.f); });
        auto u = dev.apply_fn(t, [](auto x) { return x.add(1.f); });
        auto w = dev.apply_fn(t, [](auto x) { return x.sub(1.f); });
        dev.elementwise_fusing();
        CHECK_EQ(count_live(dev), size_t(3));
        dev.run();
        CHECK_VEC_EQ(u.replace().read(), (std::vector<float>{3.f, 5.f, 7.f}));
        CHECK_VEC_EQ(w.replace().read(), (std::vector<float>{1.f, 3.f, 5.f}));
        CHECK_VEC_EQ(t.replace().read(), (std::vector<float>{2.f, 4.f, 6.f}));
    }
    {   // a checkpoint is kept (src/buffer.rs:131-137)
        D dev;
        auto a = dev.template buffer<float>({1.f, 2.f, 3.f});
        auto t = dev.apply_fn(a, [](auto x) { return x.mul(2.f); }).checkpoint();
        auto u = dev.apply_fn(t, [](auto x) { return x.add(1.f); });
        auto w = dev.apply_fn(u, [](auto x) { return x.neg(); });
        dev.elementwise_fusing();
        CHECK_EQ(count_live(dev), size_t(2));  // t alone, u+w fused
        dev.run();
        CHECK_VEC_EQ(t.replace().read(), (std::vector<float>{2.f, 4.f, 6.f}));
        CHECK_VEC_EQ(w.replace().read(), (std::vector<float>{-3.f, -5.f, -7.f}));
    }
    {   // five distinct operand buffers do not fit one kernel: the chain is cut
        D dev;
        std::vector<Buffer<float, D>> in;
        for (int i = 0; i < 6; i++) in.push_back(dev.template buffer<float>({float(i + 1), 1.f, 2.f}));
        auto add = [](auto x, auto y) { return x.add(y); };
        auto s1 = dev.apply_fn2(in[0], in[1], add);
        auto s2 = dev.apply_fn2(s1, in[2], add);
        auto s3 = dev.apply_fn2(s2, in[3], add);
        auto s4 = dev.apply_fn2(s3, in[4], add);
        auto s5 = dev.apply_fn2(s4, in[5], add);
        dev.elementwise_fusing();
        for (const auto& op : dev.modules.modules.graph) CHECK(op.arg_ids.size() <= 5);  // out + at most 4 operands
        CHECK(count_live(dev) < 5 && count_live(dev) >= 2);
        dev.run();
        CHECK_VEC_EQ(s5.replace().read(), (std::vector<float>{21.f, 6.f, 12.f}));
    }
    {   // an operand is overwritten between producer and reader: no inlining across the write
        D dev;
        auto a = dev.template buffer<float>({1.f, 2.f, 3.f});
        auto g = dev.template buffer<float>({10.f, 10.f, 10.f});
        auto o = dev.template buffer<float>({1.f, 1.f, 1.f});
        auto t = dev.apply_fn(g, [](auto x) { return x.mul(2.f); });                  // reads g = 10
        dev.add_unary_grad(a, g, o, [](auto x) { return x.identity(); });           // g += a  (unhinted: writes g)
        auto u = dev.apply_fn(t, [](auto x) { return x.add(1.f); });
        dev.elementwise_fusing();
        dev.run();
        CHECK_VEC_EQ(u.replace().read(), (std::vector<float>{21.f, 21.f, 21.f}));   // from g before the update
        CHECK_VEC_EQ(g.read(), (std::vector<float>{11.f, 12.f, 13.f}));
    }
}

// a buffer a gradient function needs is computed even though it has a single reader
template <template <class> class DEV>
void elementwise_fuse_keeps_tape_buffers(double tol) {
    DEV<Autograd<Graph<Lazy<Base, double>, double>>> dev;
    auto buf = dev.template buffer<double>({0., 1., 2., 3.}).require_grad();
    auto buf1 = dev.apply_fn(buf, [](auto x) { return x.add(1.); });
    auto out = dev.unary_ew(buf1, [](auto x) { return x.sin(); }, [](auto x) { return x.cos(); });
    dev.elementwise_fusing();
    dev.run();
    CHECK_ROUGHLY(out.replace().read(), SIN_1_4, tol);
    CHECK_VEC_EQ(buf1.replace().read(), (std::vector<double>{1., 2., 3., 4.}));  // not inlined away
    out.backward();
    CHECK_ROUGHLY(buf1.grad(dev).read(), COS_1_4, tol);
}

// random element-wise programs: fused and unfused runs agree bit for bit
template <template <class> class DEV>
void elementwise_fuse_random_programs() {
    using D = DEV<Graph<Lazy<Base>>>;
    uint64_t rng = 0x9E3779B97F4A7C15ull;
    auto next = [&rng](uint64_t m) {
        rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
        return rng % m;
    };
    const char* more = std::getenv("CUSTOS_RANDOM_PROGRAMS");   // more trials for a longer run
    const int trials = more ? std::atoi(more) : 12;
    for (int trial = 0; trial < trials; trial++) {
        std::vector<std::vector<int>> prog;  // {kind, fn, in0, in1}
        const int n_leaf = 3, n_ops = 10;
        for (int i = 0; i < n_ops; i++) {
            int avail = n_leaf + i;
            prog.push_back({int(next(2)), int(next(3)), int(next(avail)), int(next(avail))});
        }
        std::vector<std::vector<float>> results[2];
        for (int fused = 0; fused < 2; fused++) {
            D dev;
            std::vector<Buffer<float, D>> vals;
            for (int l = 0; l < n_leaf; l++) {
                std::vector<float> v(37);
                for (size_t k = 0; k < v.size(); k++) v[k] = 0.1f * float((l + 1) * (k % 11)) - 1.5f;
                vals.push_back(dev.template buffer<float>(v));
            }
            for (const auto& op : prog) {
                if (op[0] == 0) {
                    if (op[1] == 0) vals.push_back(dev.apply_fn(vals[op[2]], [](auto x) { return x.mul(1.5f).add(0.25f); }));
                    else if (op[1] == 1) vals.push_back(dev.apply_fn(vals[op[2]], [](auto x) { return x.abs().sqrt(); }));
                    else vals.push_back(dev.apply_fn(vals[op[2]], [](auto x) { return x.neg().max(-2.f); }));
                } else {
                    int l = op[2], r = op[3];
                    if (l == r) r = (r + 1) % (int)vals.size();  // operands of one operation are distinct buffers
                    if (op[1] == 0) vals.push_back(dev.apply_fn2(vals[l], vals[r], [](auto x, auto y) { return x.add(y); }));
                    else if (op[1] == 1) vals.push_back(dev.apply_fn2(vals[l], vals[r], [](auto x, auto y) { return x.mul(y).sub(0.5f); }));
                    else vals.push_back(dev.apply_fn2(vals[l], vals[r], [](auto x, auto y) { return x.min(y); }));
                }
            }
            if (fused) dev.elementwise_fusing();
            else dev.modules.modules.alloc_later(dev);
            dev.run();
            // only buffers nobody else reads are guaranteed to be computed after fusing: compare the sinks
            std::vector<int> reads(vals.size(), 0);
            for (size_t i = 0; i < prog.size(); i++) {
                reads[prog[i][2]]++;
                if (prog[i][0] == 1) reads[prog[i][3] == prog[i][2] ? (prog[i][3] + 1) % int(n_leaf + i) : prog[i][3]]++;
            }
            for (size_t i = n_leaf; i < vals.size(); i++)
                if (reads[i] != 1) results[fused].push_back(vals[i].replace().read());
        }
        CHECK_EQ(results[0].size(), results[1].size());
        for (size_t i = 0; i < results[0].size() && i < results[1].size(); i++) CHECK_VEC_EQ(results[1][i], results[0][i]);
    }
}

// src/modules/lazy/lazy_graph.rs:253-370 (test_lazy_op_args, .._no_out_but_use, .._no_out_but_use_loop,
// .._with_ew_fn): recorded operations get their arguments by id when the graph runs
template <template <class> class DEV>
void lazy_custom_operations() {
    DEV<Lazy<Base>> device;
    auto lhs = device.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
    auto rhs = device.template buffer<float>({1.f, 2.f, 6.f, 4.f, 5.f});
    auto out = device.template retrieve<float>(lhs.len(), lhs, rhs);
    int calls = 0;
    using Buf = Buffer<float, DEV<Lazy<Base>>>;
    for (int i = 0; i < 10; i++)
        device.add_op(std::tie(lhs, rhs, out), [&calls](const Buf& l, const Buf& r, Buf& o, DEV<Lazy<Base>>&) {
            CHECK_VEC_EQ(l.read(), (std::vector<float>{1.f, 2.f, 3.f, 4.f, 5.f}));
            CHECK_VEC_EQ(r.read(), (std::vector<float>{1.f, 2.f, 6.f, 4.f, 5.f}));
            CHECK(o.has_data());
            calls++;
        });
    device.add_op(std::tie(lhs, rhs), [&calls](const Buf& l, const Buf& r, DEV<Lazy<Base>>&) {
        CHECK_EQ(l.len(), r.len());
        calls++;
    });
    // an operation that writes its output from the host (the reference's `ew_fn`)
    device.add_op(std::tie(out, lhs), [](Buf& o, const Buf& l, DEV<Lazy<Base>>&) {
        std::vector<float> v = l.read();
        for (float& x : v) x += 10.f;
        o.write(v);
    });
    CHECK_EQ(calls, 0);
    CHECK_EQ(device.ops_count(), size_t(12));
    device.run();
    CHECK_EQ(calls, 11);
    CHECK_VEC_EQ(out.replace().read(), (std::vector<float>{11.f, 12.f, 13.f, 14.f, 15.f}));
}

// src/modules/lazy.rs:842-856 (test_lazy_cached_two_producers): Lazy answers the retrieve itself
template <template <class> class DEV>
void lazy_over_cached() {
    DEV<Lazy<Cached<Base>>> device;
    auto lhs = device.template buffer<int>({1, 2, 3, 4});
    auto rhs = device.template buffer<int>({1, 2, 3, 4});
    auto out = device.template retrieve<int>(10, lhs, rhs);
    CHECK(out.flag() == AllocFlag::Lazy);
    CHECK_EQ(device.modules.modules.cached_allocations(), size_t(0));
    auto sum = device.apply_fn2(lhs, rhs, [](auto x, auto y) { return x.add(y); });
    device.run();
    CHECK_VEC_EQ(sum.replace().read(), (std::vector<int>{2, 4, 6, 8}));
}

// src/modules/graph/opt_graph/optimize.rs:395-449 (test_from_retrieve_sine_neural_net)
template <template <class> class DEV>
void graph_cached_neural_net_traces() {
    DEV<Graph<Cached<Base>>> device;
    auto ones = [&](size_t n, int v = 1) { return device.template buffer<int>(std::vector<int>(n, v)); };
    auto w1 = ones(10 * 64), b1 = ones(64), w2 = ones(64 * 64), b2 = ones(64), w3 = ones(64 * 64), b3 = ones(64);
    auto w4 = ones(64), b4 = ones(1), inputs = ones(10 * 100), targets = ones(100, 2);
    auto a1 = device.template retrieve<int>(100 * 64, inputs, w1);
    auto a2 = device.template retrieve<int>(100 * 64, a1, b1);
    auto a2b = device.template retrieve<int>(100 * 64, a2, a2);
    auto a3 = device.template retrieve<int>(100 * 64, a2b, w2);
    auto a4 = device.template retrieve<int>(100 * 64, a3, b2);
    auto a4b = device.template retrieve<int>(100 * 64, a4, a4);
    auto a5 = device.template retrieve<int>(100 * 64, a4b, w3);
    auto a6 = device.template retrieve<int>(100 * 64, a5, b3);
    auto a6b = device.template retrieve<int>(100 * 64, a6, a6);
    auto a7 = device.template retrieve<int>(100, a6b, w4);
    auto a8 = device.template retrieve<int>(100, a7, b4);
    auto loss = device.template retrieve<int>(100, a8, targets);
    auto traces = device.modules.graph_trans.opt_graph.cache_traces();
    CHECK_EQ(traces.size(), size_t(2));
    CHECK(traces[0] == (CacheTrace{10, {11, 12, 13, 14, 15, 16, 17, 18}}));
    CHECK(traces[1] == (CacheTrace{19, {20, 21}}));
}

// src/modules/graph/opt_graph/optimize.rs:566-612 (.._optimize_cache) and :614-657
// (test_mismatched_optimized_types_cached): ids after optimising the cached allocations
template <template <class> class DEV>
void cached_sliced_chained_optimize(bool mismatched) {
    DEV<Graph<Cached<Base>>> device;
    auto x = device.template buffer<float>(std::vector<float>(1000, 1.f));
    auto b = device.template buffer<float>(std::vector<float>(1000, 1.1f));
    for (size_t i : device.range(0, 2)) {
        {
            auto squared = device.template retrieve<float>(1000, x, x);
            auto add = device.template retrieve<float>(1000, b, x);
            Id mul_b_id;
            // the reference retrieves `mul_b` as u8 in the mismatched case
            auto mul_b_f = mismatched ? Buffer<float, DEV<Graph<Cached<Base>>>>() : device.template retrieve<float>(1000, add, b);
            auto mul_b_u = mismatched ? device.template retrieve<unsigned char>(1000, add, b)
                                      : Buffer<unsigned char, DEV<Graph<Cached<Base>>>>();
            mul_b_id = mismatched ? mul_b_u.id() : mul_b_f.id();
            auto mul = device.template retrieve<float>(1000, squared, x);
            auto out = mismatched ? device.template retrieve<float>(1000, mul, mul_b_u)
                                  : device.template retrieve<float>(1000, mul, mul_b_f);
            if (i == 0) CHECK(squared.id() != mul.id());
            if (i == 1) {
                CHECK(squared.id() == mul.id());
                CHECK(squared.id() == out.id());
                if (mismatched) CHECK(add.id().id != mul_b_id.id);
                else CHECK(add.id() == mul_b_id);
            }
        }
        if (i == 0) device.optimize_mem_graph();
    }
}

// src/modules/graph/opt_graph/optimize.rs:659-690 (test_mismatched_optimized_types_lazy, which
// expects a panic): here the buffer of the other type keeps its own allocation and the run works
template <template <class> class DEV>
void lazy_mismatched_types_keep_their_allocation() {
    DEV<Graph<Lazy<Base>>> device;
    auto x = device.template buffer<float>(std::vector<float>(1000, 1.f));
    auto b = device.template buffer<float>(std::vector<float>(1000, 1.1f));
    auto squared = device.template retrieve<float>(1000, x, x);
    auto add = device.template retrieve<float>(1000, b, x);
    auto mul_b = device.template retrieve<unsigned char>(1000, add, b);
    auto mul = device.template retrieve<float>(1000, squared, x);
    auto out = device.template retrieve<float>(1000, mul, mul_b);
    device.optimize_mem_graph();
    device.run();
    CHECK_EQ(squared.replace().ptr(), mul.replace().ptr());
    CHECK_EQ(squared.replace().ptr(), out.replace().ptr());
    CHECK(add.replace().ptr() != mul_b.replace().ptr());
    CHECK_EQ(mul_b.replace().len(), size_t(1000));
}

// src/modules/autograd.rs:335-431: the pool of buffers by id that gradient functions look
// their arguments up in when no Lazy module keeps one
template <template <class> class DEV>
void autograd_no_grads_pool() {
    {
        // test_buffer_creation_autograd_register_manual / _get_buf / _unregister
        DEV<Autograd<Cached<Base>>> device;
        Id id;
        {
            auto buf = device.template new_buffer<float>(10);
            id = buf.id();
            auto it = device.modules.state.no_grads_pool.find(id.id);
            CHECK(it != device.modules.state.no_grads_pool.end());
            if (it != device.modules.state.no_grads_pool.end()) {
                CHECK_EQ(it->second.ptr, buf.ptr());
                CHECK_EQ(it->second.len, size_t(10));
                CHECK(it->second.type == std::type_index(typeid(float)));
            }
        }
        CHECK(device.modules.state.no_grads_pool.find(id.id) == device.modules.state.no_grads_pool.end());
    }
    {
        // test_buffer_new_and_retrieve
        DEV<Autograd<Cached<Base>>> device;
        auto lhs = device.template new_buffer<float>(10);
        for (size_t epoch : device.range(0, 100)) {
            (void)epoch;
            auto x = device.template retrieve<float>(100);
            CHECK_EQ(x.len(), size_t(100));
        }
        CHECK_EQ(device.modules.state.no_grads_pool.size(), size_t(2));
    }
    {
        // test_cached_before_autograd
        DEV<Cached<Autograd<Base>>> device;
        auto lhs = device.template new_buffer<float>(10);
        for (size_t epoch : device.range(0, 100)) {
            (void)epoch;
            auto x = device.template retrieve<float>(100);
            CHECK_EQ(x.len(), size_t(100));
        }
        CHECK_EQ(device.modules.modules.state.no_grads_pool.size(), size_t(2));
    }
    {
        // test_tape_return_without_autograd (panics in the reference), .._with_grad_allocation
        DEV<Base> plain;
        auto buf = plain.template new_buffer<float>(10);
        bool threw = false;
        try {
            buf.grad();
        } catch (const std::logic_error&) {
            threw = true;
        }
        CHECK(threw);
        DEV<Autograd<Base>> device;
        auto buf2 = device.template new_buffer<float>(10);
        auto g = buf2.grad();
        CHECK_VEC_EQ(g.read(), std::vector<float>(10, 0.f));
    }
}

// ---- 16-bit floats ----

// `half::f16` / `half::bf16` as element types (src/number.rs:487-676, src/devices/cdatatype.rs:53-62):
// the per-node types give the same bits on the device as the host evaluation of the expression
template <template <class> class DEV, class H>
void half_per_node_type() {
    DEV<Base> device;
    const size_t n = 2003;
    std::vector<H> xs(n), ys(n);
    for (size_t i = 0; i < n; i++) {
        xs[i] = H(-3.f + 6.f * static_cast<float>((i * 7919) % n) / n);
        ys[i] = H(0.5f + 1.5f * static_cast<float>((i * 104729) % n) / n);
    }
    auto f = [](auto a, auto b) { return a.mul(0.3f).add(b).mul(a).div(b.add(1.7f)).sub(0.1f).abs().sqrt().max(0.25f).neg(); };
    auto bx = device.buffer(xs), by = device.buffer(ys);
    const std::vector<H> got = device.apply_fn2(bx, by, f).read();
    size_t wrong = 0;
    for (size_t i = 0; i < n; i++)
        wrong += got[i].bits != eval<H>(f(Resolve<H>::with_val(xs[i]), Resolve<H>::with_val(ys[i]))).bits;
    CHECK_EQ(wrong, size_t(0));
    // gradient: g + round(o * d), both rounded
    auto d = [](auto v) { return v.mul(v).mul(3.f).add(0.7f); };
    std::vector<H> g0(n, H(0.5f));
    auto bg = device.buffer(g0);
    device.add_unary_grad(bx, bg, by, d);
    const std::vector<H> g1 = bg.read();
    wrong = 0;
    for (size_t i = 0; i < n; i++) wrong += g1[i].bits != (g0[i] + ys[i] * eval<H>(d(Resolve<H>::with_val(xs[i])))).bits;
    CHECK_EQ(wrong, size_t(0));
}

// ---- Read / WriteBuf / ClearBuf ----

// tests/write.rs:6-87, tests/read.rs:4-13, tests/clear.rs:7-43
template <template <class> class DEV>
void write_read_clear() {
    DEV<Base> device;
    auto buf = device.template new_buffer<double>(5);
    buf.write({1., 2., 3., 4., 5.});
    CHECK_VEC_EQ(buf.read(), (std::vector<double>{1., 2., 3., 4., 5.}));
    auto dst = device.template new_buffer<int32_t>(4);
    auto src = device.template buffer<int32_t>({1, 2, -5, 4});
    device.write_buf(dst, src);
    CHECK_VEC_EQ(dst.read(), (std::vector<int32_t>{1, 2, -5, 4}));
    CHECK_VEC_EQ(src.read(), (std::vector<int32_t>{1, 2, -5, 4}));
    auto shorter = device.template new_buffer<int32_t>(3);
    CHECK_THROWS_KIND(device.write_buf(shorter, src), DeviceError::ShapeLengthMismatch);
    auto a = device.template buffer<double>({3., 1., 3., 4.});
    CHECK_VEC_EQ(a.read(), (std::vector<double>{3., 1., 3., 4.}));
    auto c = device.template buffer<double>({1., 2., 3., 4., 5., 6.});
    CHECK_VEC_EQ(c.read(), (std::vector<double>{1., 2., 3., 4., 5., 6.}));
    c.clear();
    CHECK_VEC_EQ(c.read(), (std::vector<double>(6, 0.)));
    // an odd number of narrow elements: the clear stops at the buffer's last byte
    auto bytes = device.template buffer<uint8_t>(std::vector<uint8_t>(37, 9));
    auto next = device.template buffer<uint8_t>(std::vector<uint8_t>(37, 7));
    bytes.clear();
    CHECK_VEC_EQ(bytes.read(), (std::vector<uint8_t>(37, 0)));
    CHECK_VEC_EQ(next.read(), (std::vector<uint8_t>(37, 7)));
}

// ---- CopySlice / CloneBuf ----

// tests/slice_buf.rs:5-84, tests/clone_buf.rs:5-49
template <template <class> class DEV>
void copy_slice_and_clone_buf() {
    DEV<Base> device;
    auto source = device.template buffer<float>({1.f, 2.f, 6.f, 2.f, 4.f});
    auto actual = device.copy_slice(source, 1, 3);
    CHECK_VEC_EQ(actual.read(), (std::vector<float>{2.f, 6.f}));
    auto dest = device.template new_buffer<float>(10);
    device.copy_slice_all(source, dest, {{2, 5, 7, 10}, {1, 3, 3, 5}});
    CHECK_VEC_EQ(dest.read(), (std::vector<float>{0.f, 0.f, 0.f, 2.f, 6.f, 0.f, 0.f, 6.f, 2.f, 4.f}));
    // out of bounds: the reference panics
    CHECK_THROWS_KIND(device.copy_slice_all(source, dest, {{2, 5, 8, 11}, {1, 3, 3, 5}}), DeviceError::ShapeLengthMismatch);
    CHECK_THROWS_KIND(device.copy_slice(source, 3, 6), DeviceError::ShapeLengthMismatch);
    CHECK_THROWS_KIND(device.copy_slice_to(source, 0, 2, dest, 0, 3), DeviceError::ShapeLengthMismatch);
    // src/op_traits.rs:60-66
    auto dest2 = device.template buffer<float>({5.f, 4.f, 3.f, 2.f, 1.f});
    device.copy_slice_to(source, 1, 3, dest2, 3, 5);
    CHECK_VEC_EQ(dest2.read(), (std::vector<float>{5.f, 4.f, 3.f, 2.f, 6.f}));
    auto self_cloned = source.clone();   // tests/clone_buf.rs:17-23 (test_self_buf_clone)
    CHECK_VEC_EQ(self_cloned.read(), source.read());
    auto cloned = device.clone_buf(source);
    CHECK_VEC_EQ(cloned.read(), source.read());
    CHECK(cloned.ptr() != source.ptr());
    auto ints = device.template buffer<int>({7, 8, 9});
    CHECK_VEC_EQ(device.clone_buf(ints).read(), (std::vector<int>{7, 8, 9}));
}

// ---- Cached ----

// tests/cache.rs:24-45 (test_caching_cpu)
template <template <class> class DEV>
void cached_same_allocation_every_epoch() {
    DEV<Cached<Base>> device;
    uint64_t old_ptr = 0;
    for (size_t epoch : device.range(0, 100)) {
        (void)epoch;
        auto out = device.template retrieve<float>(10);
        CHECK(old_ptr == 0 || out.ptr() == old_ptr);
        CHECK(out.flag() == AllocFlag::Cached);
        old_ptr = out.ptr();
    }
    CHECK_EQ(device.modules.cached_allocations(), size_t(1));
    // outside a range the cursor keeps counting: a new position, a new allocation
    auto next = device.template retrieve<float>(10);
    CHECK(next.ptr() != old_ptr);
    CHECK_EQ(device.modules.cached_allocations(), size_t(2));
}

// src/modules/cached.rs:544-569 (test_multi_level_retrieve): five retrieves, five positions
template <template <class> class DEV>
void cached_multi_level_retrieve() {
    DEV<Cached<Base>> device;
    std::vector<uint64_t> first;
    for (size_t epoch : device.range(0, 3)) {
        std::vector<uint64_t> ptrs;
        auto a = device.template retrieve<float>(10);
        ptrs.push_back(a.ptr());
        for (int i = 0; i < 3; i++) {
            auto b = device.template retrieve<float>(20);
            CHECK_EQ(b.len(), size_t(20));
            ptrs.push_back(b.ptr());
        }
        if (epoch == 0) {
            first = ptrs;
            for (size_t i = 0; i < ptrs.size(); i++)
                for (size_t j = i + 1; j < ptrs.size(); j++) CHECK(ptrs[i] != ptrs[j]);
        } else {
            CHECK(ptrs == first);
        }
    }
    CHECK_EQ(device.modules.cached_allocations(), size_t(4));
}

// src/modules/cached.rs:572-602 (test_add_cached_layer): operations on a cached device
template <template <class> class DEV>
void cached_apply_fn_and_unary_ew() {
    DEV<Cached<Base>> device;
    auto base = device.template buffer<float>({1.f, 2.f, 3.f, 4.f});
    uint64_t first = 0;
    for (size_t epoch : device.range(0, 10)) {
        auto y = device.apply_fn(base, [](auto x) { return x.mul(2.f).add(1.f); });
        CHECK_VEC_EQ(y.read(), (std::vector<float>{3.f, 5.f, 7.f, 9.f}));
        if (epoch == 0) first = y.ptr();
        CHECK_EQ(y.ptr(), first);
        auto z = device.unary_ew(base, [](auto x) { return x.neg(); }, [](auto x) { return x.mul(0.f).sub(1.f); });
        CHECK_VEC_EQ(z.read(), (std::vector<float>{-1.f, -2.f, -3.f, -4.f}));
        CHECK(z.ptr() != y.ptr());
    }
    CHECK_EQ(device.modules.cached_allocations(), size_t(2));
    // `device.cached(|| ..)` (src/features.rs:101-109): the closure's retrieves are replayed
    uint64_t in_closure = 0;
    for (int i = 0; i < 3; i++)
        device.cached([&] {
            auto w = device.apply_fn(base, [](auto x) { return x.add(1.f); });
            CHECK(in_closure == 0 || w.ptr() == in_closure);
            in_closure = w.ptr();
            CHECK_VEC_EQ(w.read(), (std::vector<float>{2.f, 3.f, 4.f, 5.f}));
        });
    CHECK_EQ(device.modules.cached_allocations(), size_t(3));
}

// tests/graph/graph.rs:10-41 (test_graph) and :78-108 (test_graph_cu): after
// `optimize_mem_graph` the three results of the chain share one allocation
template <template <class> class DEV>
void cached_graph_optimize_aliases() {
    DEV<Graph<Cached<Base>>> device;
    auto a = device.template buffer<int>({1, 2, 3, 4, 5, 6});
    auto b = device.template buffer<int>({2, 3, 1, 4, 0, 5});
    const size_t live_before = device.modules.modules.cached_allocations();
    CHECK_EQ(live_before, size_t(0));
    for (size_t epoch : device.range(0, 3)) {
        {
            auto c = device.apply_fn2(a, b, [](auto x, auto y) { return x.add(y); });
            CHECK_VEC_EQ(c.read(), (std::vector<int>{3, 5, 4, 8, 5, 11}));
            auto d = device.apply_fn(c, [](auto x) { return x.max(0); });
            CHECK_VEC_EQ(d.read(), (std::vector<int>{3, 5, 4, 8, 5, 11}));
            auto e = device.apply_fn2(d, b, [](auto x, auto y) { return x.add(y); });
            CHECK_VEC_EQ(e.read(), (std::vector<int>{5, 8, 5, 12, 5, 16}));
            if (epoch >= 1) {
                CHECK_EQ(c.ptr(), d.ptr());
                CHECK_EQ(c.ptr(), e.ptr());
            } else {
                CHECK(c.ptr() != d.ptr());
                // replacing allocations that handles still use is refused
                CHECK_THROWS_KIND(device.optimize_mem_graph(), DeviceError::CachedInUse);
            }
        }
        device.optimize_mem_graph();
        CHECK_EQ(device.modules.modules.cached_allocations(), size_t(1));
    }
    CHECK_VEC_EQ(a.read(), (std::vector<int>{1, 2, 3, 4, 5, 6}));
    CHECK_VEC_EQ(b.read(), (std::vector<int>{2, 3, 1, 4, 0, 5}));
}

template <template <class> class DEV>
void cached_errors() {
    {
        DEV<Cached<Base>> device;
        for (size_t epoch : device.range(0, 2)) {
            if (epoch == 0) {
                auto x = device.template retrieve<float>(8);
            } else {
                // the same cursor position asked for another element type or length
                CHECK_THROWS_KIND(device.template retrieve<int>(8), DeviceError::TypeMismatch);
                CHECK_THROWS_KIND(device.template retrieve<float>(9), DeviceError::ShapeLengthMismatch);
                auto x = device.template retrieve<float>(8);
                CHECK_EQ(x.len(), size_t(8));
            }
        }
        // src/modules/cached.rs:448-455; no Graph module, no cache traces
        CHECK_THROWS_KIND(device.unary_fusing(), DeviceError::UnaryFusingUnsupported);
        CHECK_THROWS_KIND(device.optimize_mem_graph(), DeviceError::MissingCacheTraces);
    }
    {
        // buffers of another type in a trace keep their allocation (cached.rs:430-441)
        DEV<Graph<Cached<Base>>> device;
        auto a = device.template buffer<float>({1.f, 2.f});
        {
            auto c = device.template retrieve<float>(2, a);
            auto d = device.template retrieve<int>(2, c);
            auto e = device.template retrieve<float>(2, d);
            (void)e;
        }
        device.optimize_mem_graph();
        CHECK_EQ(device.modules.modules.cached_allocations(), size_t(2));
    }
}

// operands of one operation have one length: a shorter one would be read or written beyond its
// end on the device (`DeviceError::ShapeLengthMismatch`, src/error.rs)
template <template <class> class DEV>
void operand_lengths_must_match() {
    DEV<Base> dev;
    auto six = dev.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f, 6.f});
    auto five = dev.template buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
    auto grad = dev.template buffer<float>({0.f, 0.f, 0.f, 0.f, 0.f, 0.f});
    CHECK_THROWS_KIND(dev.apply_fn2(six, five, [](auto x, auto y) { return x.add(y); }), DeviceError::ShapeLengthMismatch);
    CHECK_THROWS_KIND(dev.add_unary_grad(six, five, six, [](auto x) { return x.mul(2.f); }), DeviceError::ShapeLengthMismatch);
    CHECK_THROWS_KIND(dev.add_unary_grad(six, grad, five, [](auto x) { return x.mul(2.f); }), DeviceError::ShapeLengthMismatch);
    dev.add_unary_grad(six, grad, six, [](auto x) { return x.mul(2.f); });
    CHECK_VEC_EQ(grad.read(), (std::vector<float>{2.f, 8.f, 18.f, 32.f, 50.f, 72.f}));  // 0 + x * 2x
}

// Buffers as sequences of elements: the token stream the reference pins for a pointer of ten
// i32 (src/devices/cuda/cuda_ptr.rs:163-189, src/devices/cpu/cpu_ptr.rs:402-424), and the round
// trip device -> sequence -> new device buffer for every element type, as tokens and as JSON.
template <class T, class D>
void serde_round_trip(D& dev, const std::vector<T>& values) {
    auto buf = dev.template buffer<T>(values);
    const std::vector<serde::Token> tokens = serde::to_tokens(buf);
    CHECK_EQ(tokens.size(), values.size() + 2);
    CHECK(tokens.front() == serde::Token::seq(values.size()) && tokens.back() == serde::Token::seq_end());
    auto back = serde::from_tokens<T>(dev, tokens);
    CHECK(back.ptr() != buf.ptr());
    const std::vector<T> a = buf.read(), b = back.read(), c = serde::from_json<T>(dev, serde::to_json(buf)).read();
    CHECK_EQ(b.size(), values.size());
    CHECK(std::memcmp(a.data(), b.data(), a.size() * sizeof(T)) == 0);
    CHECK_EQ(c.size(), values.size());
    CHECK(std::memcmp(a.data(), c.data(), a.size() * sizeof(T)) == 0);
}

template <template <class> class DEV>
void serde_of_buffers() {
    using D = DEV<Base>;
    D dev;
    auto ten = dev.template buffer<int32_t>({1, 2, 3, 4, 5, 6, 7, 8, 9, 10});
    std::vector<serde::Token> want = {serde::Token::seq(10)};
    for (int32_t v = 1; v <= 10; v++) want.push_back({serde::TokenKind::I32, static_cast<uint64_t>(v)});
    want.push_back(serde::Token::seq_end());
    CHECK(serde::to_tokens(ten) == want);
    CHECK_EQ(serde::to_json(ten), std::string("[1,2,3,4,5,6,7,8,9,10]"));
    CHECK_VEC_EQ(serde::from_tokens<int32_t>(dev, want).read(), (std::vector<int32_t>{1, 2, 3, 4, 5, 6, 7, 8, 9, 10}));
    CHECK_EQ(serde::to_json(dev.template buffer<float>({1.5f, -0.25f, 3.f, 0.1f})), std::string("[1.5,-0.25,3.0,0.1]"));
    CHECK_VEC_EQ(serde::from_json<float>(dev, " [ 1.5 , -0.25,3.0 ,1e-3 ] ").read(), (std::vector<float>{1.5f, -0.25f, 3.f, 1e-3f}));

    serde_round_trip<int8_t>(dev, {-128, -1, 0, 1, 127});
    serde_round_trip<uint8_t>(dev, {0, 1, 200, 255});
    serde_round_trip<int16_t>(dev, {-32768, -2, 0, 32767});
    serde_round_trip<uint16_t>(dev, {0, 1, 65535});
    serde_round_trip<int32_t>(dev, {INT32_MIN, -7, 0, 9, INT32_MAX});
    serde_round_trip<uint32_t>(dev, {0u, 3u, 4000000000u, UINT32_MAX});
    serde_round_trip<int64_t>(dev, {INT64_MIN, -5, 0, 5, INT64_MAX});
    serde_round_trip<uint64_t>(dev, {0ull, 1ull, 1ull << 63, UINT64_MAX});
    serde_round_trip<float>(dev, {0.f, -0.f, 1.f, 0.1f, -3.4028235e38f, 1.17549435e-38f, 1e-45f, 16777217.f});
    serde_round_trip<double>(dev, {0., -0., 0.1, 1. / 3., -1.7976931348623157e308, 4.9e-324, 2.2250738585072014e-308});
    serde_round_trip<f16>(dev, {f16(1.f), f16(-0.333f), f16::from_bits(0x0001), f16::from_bits(0x7bff), f16::from_bits(0xfc00)});
    serde_round_trip<bf16>(dev, {bf16(1.f), bf16(-3.14f), bf16::from_bits(0x0001), bf16::from_bits(0x7f7f)});
    serde_round_trip<f16_pernode>(dev, {f16_pernode(0.5f), f16_pernode(-65504.f)});
    serde_round_trip<bf16_pernode>(dev, {bf16_pernode(0.5f), bf16_pernode(1e30f)});

    // what is not a sequence of this element type is an error, not a buffer
    std::vector<serde::Token> wrong_kind = want;
    wrong_kind[3].kind = serde::TokenKind::F32;
    CHECK_THROWS_KIND(serde::from_tokens<int32_t>(dev, wrong_kind), DeviceError::TypeMismatch);
    CHECK_THROWS_KIND(serde::from_tokens<float>(dev, want), DeviceError::TypeMismatch);
    std::vector<serde::Token> short_one = want;
    short_one.erase(short_one.begin() + 4);
    CHECK_THROWS_KIND(serde::from_tokens<int32_t>(dev, short_one), DeviceError::ShapeLengthMismatch);
    CHECK_THROWS_KIND(serde::from_tokens<int32_t>(dev, {serde::Token::seq(0), serde::Token::seq_end()}), DeviceError::ZeroLengthBuffer);
    CHECK_THROWS_KIND(serde::from_json<int32_t>(dev, "[1,2.5]"), DeviceError::TypeMismatch);
    CHECK_THROWS_KIND(serde::from_json<uint8_t>(dev, "[1,256]"), DeviceError::TypeMismatch);
    CHECK_THROWS_KIND(serde::from_json<int32_t>(dev, "[1,2"), DeviceError::ShapeLengthMismatch);
    CHECK_THROWS_KIND(serde::from_json<int32_t>(dev, "[]"), DeviceError::ZeroLengthBuffer);
}

}  // namespace module_tests

// Registers every generic case for one device template.
#define REGISTER_MODULE_TESTS(DEV, TOL)                                                           \
    TEST_CASE(base_apply_fn) { module_tests::base_apply_fn<DEV>(); }                              \
    TEST_CASE(base_add_unary_grad) { module_tests::base_add_unary_grad<DEV>(); }                  \
    TEST_CASE(base_unary_ew_forward_only) { module_tests::base_unary_ew_forward_only<DEV>(); }    \
    TEST_CASE(base_zero_length_is_an_error) { module_tests::base_zero_length_is_an_error<DEV>(); } \
    TEST_CASE(lazy_retrieve_ids) { module_tests::lazy_retrieve_ids<DEV>(); }                      \
    TEST_CASE(lazy_apply_fn_runs_at_run) { module_tests::lazy_apply_fn_runs_at_run<DEV>(); }      \
    TEST_CASE(lazy_dropped_buffer_is_invalid) { module_tests::lazy_dropped_buffer_is_invalid<DEV>(); } \
    TEST_CASE(lazy_add_and_apply_fn) { module_tests::lazy_add_and_apply_fn<DEV>(); }              \
    TEST_CASE(lazy_add_unary_grad) { module_tests::lazy_add_unary_grad<DEV>(); }                  \
    TEST_CASE(lazy_exec_now_and_last_n) { module_tests::lazy_exec_now_and_last_n<DEV>(); }        \
    TEST_CASE(lazy_duplicate_parent_is_rejected) { module_tests::lazy_duplicate_parent_is_rejected<DEV>(); } \
    TEST_CASE(lazy_op_hints) { module_tests::lazy_op_hints<DEV>(); }                              \
    TEST_CASE(graph_fuse_chain_optimized) { module_tests::graph_fuse_chain<DEV>(true); }          \
    TEST_CASE(graph_fuse_chain_alloc_later) { module_tests::graph_fuse_chain<DEV>(false); }       \
    TEST_CASE(graph_fuse_chain_with_checkpoint) { module_tests::graph_fuse_chain_with_checkpoint<DEV>(); } \
    TEST_CASE(graph_fuse_two_chains) { module_tests::graph_fuse_two_chains<DEV>(TOL); }           \
    TEST_CASE(graph_fuse_after_binary_ops) { module_tests::graph_fuse_after_binary_ops<DEV>(); }  \
    TEST_CASE(graph_optimize_mem_aliases) { module_tests::graph_optimize_mem_aliases<DEV>(); }    \
    TEST_CASE(example_lazy_and_fusing) { module_tests::example_lazy_and_fusing<DEV>(); }          \
    TEST_CASE(autograd_unary_ew) { module_tests::autograd_unary_ew<DEV>(); }                      \
    TEST_CASE(autograd_doc_example) { module_tests::autograd_doc_example<DEV>(); }                \
    TEST_CASE(autograd_multiple_times) { module_tests::autograd_multiple_times<DEV>(TOL); }       \
    TEST_CASE(autograd_lazy_accumulates) { module_tests::autograd_lazy_accumulates<DEV>(TOL); }   \
    TEST_CASE(autograd_lazy_input) { module_tests::autograd_lazy_input<DEV>(false, TOL); }        \
    TEST_CASE(autograd_lazy_input_exec_last) { module_tests::autograd_lazy_input<DEV>(true, TOL); } \
    TEST_CASE(autograd_grad_new_api) { module_tests::autograd_grad_new_api<DEV>(); }              \
    TEST_CASE(autograd_disabling) { module_tests::autograd_disabling<DEV>(); }                    \
    TEST_CASE(autograd_requires_grad_chaining) { module_tests::autograd_requires_grad_chaining<DEV>(); } \
    TEST_CASE(autograd_grad_fn_with_lazy_source) { module_tests::autograd_grad_fn_with_lazy_source<DEV>(); } \
    TEST_CASE(autograd_grad_fn_out_of_scope) { module_tests::autograd_grad_fn_out_of_scope<DEV>(); } \
    TEST_CASE(autograd_tanh_config) { module_tests::autograd_tanh_config<DEV>(1e-6); }                \
    TEST_CASE(elementwise_fuse_binary_then_unary) { module_tests::elementwise_fuse_binary_then_unary<DEV>(); } \
    TEST_CASE(elementwise_fuse_respects_limits) { module_tests::elementwise_fuse_respects_limits<DEV>(); } \
    TEST_CASE(elementwise_fuse_keeps_tape_buffers) { module_tests::elementwise_fuse_keeps_tape_buffers<DEV>(TOL); } \
    TEST_CASE(elementwise_fuse_random_programs) { module_tests::elementwise_fuse_random_programs<DEV>(); } \
    TEST_CASE(lazy_custom_operations) { module_tests::lazy_custom_operations<DEV>(); }            \
    TEST_CASE(lazy_over_cached) { module_tests::lazy_over_cached<DEV>(); }                        \
    TEST_CASE(graph_cached_neural_net_traces) { module_tests::graph_cached_neural_net_traces<DEV>(); } \
    TEST_CASE(cached_sliced_chained_optimize) { module_tests::cached_sliced_chained_optimize<DEV>(false); } \
    TEST_CASE(cached_mismatched_types_optimize) { module_tests::cached_sliced_chained_optimize<DEV>(true); } \
    TEST_CASE(lazy_mismatched_types_keep_their_allocation) { module_tests::lazy_mismatched_types_keep_their_allocation<DEV>(); } \
    TEST_CASE(autograd_no_grads_pool) { module_tests::autograd_no_grads_pool<DEV>(); }            \
    TEST_CASE(half_f16_per_node) { module_tests::half_per_node_type<DEV, f16_pernode>(); }        \
    TEST_CASE(half_bf16_per_node) { module_tests::half_per_node_type<DEV, bf16_pernode>(); }      \
    TEST_CASE(write_read_clear) { module_tests::write_read_clear<DEV>(); }                        \
    TEST_CASE(copy_slice_and_clone_buf) { module_tests::copy_slice_and_clone_buf<DEV>(); }        \
    TEST_CASE(cached_same_allocation_every_epoch) { module_tests::cached_same_allocation_every_epoch<DEV>(); } \
    TEST_CASE(cached_multi_level_retrieve) { module_tests::cached_multi_level_retrieve<DEV>(); }  \
    TEST_CASE(cached_apply_fn_and_unary_ew) { module_tests::cached_apply_fn_and_unary_ew<DEV>(); } \
    TEST_CASE(cached_graph_optimize_aliases) { module_tests::cached_graph_optimize_aliases<DEV>(); } \
    TEST_CASE(cached_errors) { module_tests::cached_errors<DEV>(); }                              \
    TEST_CASE(serde_of_buffers) { module_tests::serde_of_buffers<DEV>(); }                        \
    TEST_CASE(operand_lengths_must_match) { module_tests::operand_lengths_must_match<DEV>(); }
