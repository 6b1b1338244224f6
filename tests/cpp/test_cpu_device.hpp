// `TestCPU<Mods>`: a host device for the tests of the module stack.
//
// TEST INFRASTRUCTURE ONLY.  It plays the role the reference's `CPU<Mods>`
// plays in its own test suite (the CPU device is "the fake" every module
// combination is tested on): malloc'ed memory and the scalar loops of
// src/devices/cpu_stack_ops.rs:7-30 / src/devices/cpu/cpu_device.rs:204-232,
// evaluating the expression trees with `eval()`.  The shipped library never
// includes this header; the HIP device has no host evaluation path.
#pragma once

#include <cstdlib>
#include <cstring>

#include "custos/device.hpp"

namespace custos {

template <class Mods>
class TestCPU : public Device<TestCPU<Mods>, Mods> {
   public:
    using Self = TestCPU<Mods>;
    TestCPU() { this->modules.setup(*this); }
    TestCPU(const TestCPU&) = delete;
    ~TestCPU() { this->modules.teardown(*this); }

    size_t live_allocations = 0;
    size_t lazy_runs = 0;

    size_t unzeroed_allocations = 0;

    uint64_t alloc_raw(size_t bytes, bool zeroed, size_t) {
        void* p = std::calloc(bytes, 1);  // CPU alloc is zero-initialised (cpu_ptr.rs:74-85)
        // an allocation the caller promised to overwrite: poison it, so that a test sees
        // any element the operation leaves out
        if (!zeroed) {
            std::memset(p, 0xCD, bytes);
            unzeroed_allocations++;
        }
        live_allocations++;
        return reinterpret_cast<uint64_t>(p);
    }
    void free_raw(uint64_t ptr) {
        std::free(reinterpret_cast<void*>(ptr));
        live_allocations--;
    }
    void read_raw(void* dst, uint64_t src, size_t bytes) { std::memcpy(dst, reinterpret_cast<void*>(src), bytes); }
    void write_raw(uint64_t dst, const void* src, size_t bytes) { std::memcpy(reinterpret_cast<void*>(dst), src, bytes); }
    void clear_raw(uint64_t ptr, size_t bytes) { std::memset(reinterpret_cast<void*>(ptr), 0, bytes); }
    void fill_raw(uint64_t ptr, size_t bytes, const void* value, size_t value_bytes) {
        for (size_t at = 0; at < bytes; at += value_bytes) std::memcpy(reinterpret_cast<char*>(ptr) + at, value, value_bytes);
    }
    void copy_raw(uint64_t dst, uint64_t src, size_t bytes) {
        std::memmove(reinterpret_cast<void*>(dst), reinterpret_cast<void*>(src), bytes);
    }

    // apply_fn_slice (cpu_stack_ops.rs:7-15)
    template <class T, class F>
    void apply_fn_impl(const Buffer<T, Self>& x, Buffer<T, Self>& out, F f) {
        const T* xs = reinterpret_cast<const T*>(x.ptr());
        T* os = reinterpret_cast<T*>(out.ptr());
        for (size_t i = 0; i < x.len() && i < out.len(); i++) os[i] = eval<T>(f(Resolve<T>::with_val(xs[i])));
    }
    template <class T, class F>
    void apply_fn2_impl(const Buffer<T, Self>& l, const Buffer<T, Self>& r, Buffer<T, Self>& out, F f) {
        const T* ls = reinterpret_cast<const T*>(l.ptr());
        const T* rs = reinterpret_cast<const T*>(r.ptr());
        T* os = reinterpret_cast<T*>(out.ptr());
        for (size_t i = 0; i < l.len(); i++) os[i] = eval<T>(f(Resolve<T>::with_val(ls[i]), Resolve<T>::with_val(rs[i])));
    }
    // add_unary_grad (cpu_stack_ops.rs:18-30)
    template <class T, class F>
    void add_unary_grad_impl(const Buffer<T, Self>& lhs, Buffer<T, Self>& lhs_grad, const Buffer<T, Self>& out, F f) {
        const T* ls = reinterpret_cast<const T*>(lhs.ptr());
        const T* os = reinterpret_cast<const T*>(out.ptr());
        T* gs = reinterpret_cast<T*>(lhs_grad.ptr());
        for (size_t i = 0; i < lhs.len(); i++) {
            const T prod = os[i] * eval<T>(f(Resolve<T>::with_val(ls[i])));
            gs[i] = gs[i] + prod;
        }
    }
    // CPU unary_fuse_op (cpu_device.rs:204-232)
    template <class T>
    std::function<void(Buffer<T, Self>&, const Buffer<T, Self>&, Self&)> unary_fuse_op(
        std::vector<std::shared_ptr<UnaryHint<T>>> ops) {
        return [ops = std::move(ops)](Buffer<T, Self>& out, const Buffer<T, Self>& buf, Self&) {
            const T* xs = reinterpret_cast<const T*>(buf.ptr());
            T* os = reinterpret_cast<T*>(out.ptr());
            for (size_t i = 0; i < buf.len(); i++) {
                T cur = xs[i];
                for (const auto& op : ops) cur = op->eval(cur);
                os[i] = cur;
            }
        };
    }
    template <class T>
    std::function<void(Buffer<T, Self>&, const std::vector<Buffer<T, Self>>&, Self&)> elementwise_fuse_op(
        std::shared_ptr<FusedExpr<T>> expr) {
        return [expr](Buffer<T, Self>& out, const std::vector<Buffer<T, Self>>& ins, Self&) {
            T* os = reinterpret_cast<T*>(out.ptr());
            for (size_t i = 0; i < out.len(); i++) {
                T vals[4];
                for (size_t k = 0; k < ins.size(); k++) vals[k] = reinterpret_cast<const T*>(ins[k].ptr())[i];
                os[i] = expr->eval(vals);
            }
        };
    }

    void lazy_setup() {}
    template <class Replay>
    void lazy_run(uint64_t, Replay replay) {
        lazy_runs++;
        replay();
    }
};

}  // namespace custos
