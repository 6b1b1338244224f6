// Forward and backward of an element-wise operation with the Autograd module:
// y = tanh(x), x_grad += y_grad * (1 - tanh(x)^2).
// Counterpart of the `unary_ew` documentation example (src/unary.rs:70-96) and of
// examples/cuda_usage.rs in the reference.
#include <cmath>
#include <cstdio>
#include <vector>

#include "custos/custos.hpp"

using namespace custos;

int main() {
    HIP<Autograd<Base>> device(0);

    auto cleared = device.buffer<int>({5, 3, 2, 4, 6, 2});
    cleared.clear();
    for (int v : cleared.read())
        if (v != 0) return 1;

    auto x = device.buffer<float>({-2.f, -0.5f, 0.f, 0.5f, 1.f, 3.f}).require_grad();
    auto y = device.unary_ew(
        x, [](auto v) { return v.tanh(); },
        [](auto v) { return Scalar<float>(1.f).sub(v.tanh().mul(v.tanh())); });
    y.backward();  // seeds y's gradient with ones

    const std::vector<float> xs = x.read(), ys = y.read(), gs = x.grad().read();
    double worst = 0;
    for (size_t i = 0; i < xs.size(); i++) {
        const double t = std::tanh(static_cast<double>(xs[i]));
        worst = std::fmax(worst, std::fabs(ys[i] - t));
        worst = std::fmax(worst, std::fabs(gs[i] - (1 - t * t)));
        std::printf("x = %5.2f   tanh = %9.6f   d/dx = %9.6f\n", xs[i], ys[i], gs[i]);
    }
    return worst < 1e-6 ? 0 : 1;
}
