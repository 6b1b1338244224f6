// A user-defined operation on the HIP device, run under different module stacks.
// Counterpart of examples/modules_usage.rs in the reference: there `ElementWise::add` is
// written once per device (retrieve the output, register the gradient function, add the
// operation) and the module stack decides whether it runs at once, at `run()`, or fused.
// Here the operation is written once against the device interface, first with the
// expression vocabulary and then with a kernel of its own.
#include <cmath>
#include <cstdio>
#include <vector>

#include "custos/custos.hpp"

using namespace custos;

// out = lhs + rhs, with d out / d lhs = d out / d rhs = 1 (modules_usage.rs:36-64).
template <class T, class D>
Buffer<T, D> add(D& device, Buffer<T, D>& lhs, Buffer<T, D>& rhs) {
    Buffer<T, D> out = device.apply_fn2(lhs, rhs, [](auto l, auto r) { return l.add(r); });
    device.add_grad_fn(std::tie(lhs, rhs, out), [](Buffer<T, D>& l, Buffer<T, D>& r, Buffer<T, D>& o, D& dev) {
        // x_grad += out_grad * 1 for both operands
        Buffer<T, D> o_grad = o.grad(dev);
        for (Buffer<T, D>* operand : {&l, &r}) {
            if (!operand->requires_grad()) continue;
            Buffer<T, D> grad = operand->grad(dev);
            dev.add_unary_grad(*operand, grad, o_grad, [](auto) { return to_val(T(1)); });
        }
    });
    return out;
}

// The same operation as a kernel the caller wrote (modules_usage.rs:69-94 does this for
// OpenCL): compiled once per (source, name), launched over `len` elements.
template <class D>
Buffer<float, D> add_with_own_kernel(D& device, Buffer<float, D>& lhs, Buffer<float, D>& rhs) {
    static const char* src = R"(
        extern "C" __global__ void add_ew(const float* lhs, const float* rhs, float* out, unsigned long long len) {
            unsigned long long i = blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x;
            if (i < len) out[i] = lhs[i] + rhs[i];
        })";
    Buffer<float, D> out = device.template retrieve<float>(lhs.len(), lhs, rhs);
    device.add_op(std::tie(lhs, rhs, out), [](Buffer<float, D>& l, Buffer<float, D>& r, Buffer<float, D>& o, D& dev) {
        dev.launch_kernel1d(o.len(), src, "add_ew", l, r, o, static_cast<unsigned long long>(o.len()));
    });
    return out;
}

template <class V>
static bool same(const V& got, const V& expected) {
    return got == expected;
}

int main() {
    int failures = 0;
    auto expect = [&failures](bool ok, const char* what) {
        std::printf("%-58s %s\n", what, ok ? "ok" : "FAILED");
        failures += !ok;
    };

    {  // only the Base module: the operation runs at once
        HIP<Base> device(0);
        auto lhs = device.buffer<int32_t>({1, 2, 3, 4, 5});
        auto rhs = device.buffer<int32_t>({1, 2, 3, 4, 5});
        auto out = add(device, lhs, rhs);
        expect(same(out.read(), std::vector<int32_t>{2, 4, 6, 8, 10}), "Base: add runs at once");
        auto fl = device.buffer<float>({1.f, 2.f, 3.f});
        auto fr = device.buffer<float>({0.5f, 0.25f, 0.125f});
        expect(same(add_with_own_kernel(device, fl, fr).read(), std::vector<float>{1.5f, 2.25f, 3.125f}),
               "Base: the caller's own kernel");
    }
    {  // Lazy: nothing runs, and nothing is allocated, before run()
        HIP<Lazy<Base>> device(0);
        auto lhs = device.buffer<int32_t>({1, 2, 3, 4, 5});
        auto rhs = device.buffer<int32_t>({1, 2, 3, 4, 5});
        auto out = add(device, lhs, rhs);
        device.run();
        expect(same(out.replace().read(), std::vector<int32_t>{2, 4, 6, 8, 10}), "Lazy: add runs at run()");
        lhs.write({10, 20, 30, 40, 50});
        device.run();  // replays the recorded graph
        expect(same(out.replace().read(), std::vector<int32_t>{11, 22, 33, 44, 55}) && device.graph_builds() == 1,
               "Lazy: a second run replays the same graph");
    }
    {  // Graph<Lazy>: the user operation and two unary ones end up in one kernel
        HIP<Graph<Lazy<Base>>> device(0);
        auto lhs = device.buffer<float>({1.f, 2.f, 3.f, 4.f, 5.f});
        auto rhs = device.buffer<float>({0.f, 1.f, 2.f, 3.f, 4.f});
        auto sum = add(device, lhs, rhs);
        auto out1 = device.apply_fn(sum, [](auto x) { return x.add(1.f); });
        auto out2 = device.apply_fn(out1, [](auto x) { return x.sin(); });
        device.optimize_mem_graph();
        device.elementwise_fusing();
        device.run();
        bool ok = device.graph_kernel_nodes() == 1;
        const std::vector<float> l = lhs.read(), r = rhs.read(), got = out2.replace().read();
        for (size_t i = 0; i < got.size(); i++) ok = ok && std::fabs(got[i] - std::sin(l[i] + r[i] + 1.f)) < 1e-6f;
        expect(ok, "Graph<Lazy>: add, +1 and sin fused into one kernel");
    }
    {  // Autograd: the gradient function registered by `add` runs in the backward pass
        HIP<Autograd<Base>> device(0);
        auto lhs = device.buffer<float>({1.f, 2.f, 3.f}).require_grad();
        auto rhs = device.buffer<float>({4.f, 5.f, 6.f}).require_grad();
        auto sum = add(device, lhs, rhs);
        auto out = add(device, sum, rhs);
        out.backward();
        expect(same(out.read(), std::vector<float>{9.f, 12.f, 15.f}) && same(lhs.grad().read(), std::vector<float>(3, 1.f)) &&
                   same(rhs.grad().read(), std::vector<float>(3, 2.f)),
               "Autograd: d(lhs + 2*rhs) = (1, 2)");
    }
    return failures;
}
