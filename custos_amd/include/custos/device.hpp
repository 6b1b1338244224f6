// The device-side trait surface, as one CRTP base.
//
// A concrete device (`HIP<Mods>`) derives from `Device<HIP<Mods>, Mods>` and
// supplies the primitives (raw memory, the three element-wise launches, the
// lazy-run hook).  This base supplies what the reference gets from
// `impl_device_traits!` and its blanket impls:
//   Retriever::retrieve            src/devices.rs:158-193
//   AddOperation::{add_op,eagerly} src/features.rs:409-488
//   AddGradFn::add_grad_fn         src/features.rs:186-261
//   ApplyFunction::apply_fn        src/unary.rs:7-28,   src/devices/cuda/ops.rs:119-141
//   UnaryGrad::add_unary_grad      src/unary.rs:31-58,  src/devices/cuda/ops.rs:179-199
//   UnaryElementWiseMayGrad        src/unary.rs:62-132
//   Run / ExecNow / Optimize       src/features.rs:142-154,505-532,660-672
//   Read / WriteBuf / ClearBuf     src/op_traits.rs:6-197
//   backward / grad                src/buffer/impl_autograd.rs:20-197, autograd/tape.rs:39-117
#pragma once

#include <initializer_list>
#include <optional>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>

#include "buffer.hpp"
#include "modules.hpp"

namespace custos {

template <class Derived, class Mods>
class Device {
   public:
    Mods modules;

    Derived& self() { return static_cast<Derived&>(*this); }

    // ---- buffers ----

    // `device.buffer([..])`: allocate, upload, announce to the modules (src/buffer.rs:80-93)
    template <class T>
    Buffer<T, Derived> buffer(const std::vector<T>& data) {
        if (data.empty()) throw Error(DeviceError::ZeroLengthBuffer);
        uint64_t ptr = self().alloc_raw(data.size() * sizeof(T), /*zeroed=*/false, data.size());
        self().write_raw(ptr, data.data(), data.size() * sizeof(T));
        auto b = Buffer<T, Derived>::from_parts(&self(), ptr, data.size(), Id{ptr, data.size()}, AllocFlag::None);
        modules.on_new_buffer(self(), b);
        return b;
    }
    template <class T>
    Buffer<T, Derived> buffer(std::initializer_list<T> data) {
        return buffer(std::vector<T>(data));
    }

    // `Buffer::new(&device, len)`: zero-initialised (src/devices/cpu/cpu_device.rs:133-145)
    template <class T>
    Buffer<T, Derived> new_buffer(size_t len) {
        if (len == 0) throw Error(DeviceError::ZeroLengthBuffer);
        uint64_t ptr = self().alloc_raw(len * sizeof(T), /*zeroed=*/true, len);
        auto b = Buffer<T, Derived>::from_parts(&self(), ptr, len, Id{ptr, len}, AllocFlag::None);
        modules.on_new_buffer(self(), b);
        return b;
    }

    // `device.retrieve(len, parents)`
    template <class T, class... P>
    Buffer<T, Derived> retrieve(size_t len, const P&... parents) {
        if (len == 0) throw Error(DeviceError::ZeroLengthBuffer);
        std::vector<Id> ids{parents.id()...};
        std::vector<bool> rg{parents.requires_grad()...};
        return modules.template retrieve<T>(self(), len, ids, rg);
    }

    // `retrieve` for the output of an operation that writes every element: when the
    // operation runs at once (no Lazy module) the allocation need not be zero-filled
    // first -- one memory pass less per eager operation.  Lazily retrieved buffers are
    // zero-filled as always (a fused-away intermediate keeps its zeros).
    template <class T, class... P>
    Buffer<T, Derived> retrieve_output(size_t len, const P&... parents) {
        struct Scope {
            bool& flag;
            explicit Scope(bool& f) : flag(f) { flag = true; }
            ~Scope() { flag = false; }
        } scope(output_hint_);
        return retrieve<T>(len, parents...);
    }
    bool output_hint() const { return output_hint_; }

    template <class T>
    std::vector<T> read(const Buffer<T, Derived>& buf) {
        if (!buf.has_data()) throw Error(DeviceError::InvalidLazyBuf);
        std::vector<T> out(buf.len());
        self().read_raw(out.data(), buf.ptr(), buf.len() * sizeof(T));
        return out;
    }
    template <class T>
    void write(Buffer<T, Derived>& buf, const std::vector<T>& data) {
        if (!buf.has_data()) throw Error(DeviceError::InvalidLazyBuf);
        if (data.size() != buf.len()) throw Error(DeviceError::ShapeLengthMismatch);
        self().write_raw(buf.ptr(), data.data(), data.size() * sizeof(T));
    }
    template <class T>
    void clear(Buffer<T, Derived>& buf) {
        if (!buf.has_data()) throw Error(DeviceError::InvalidLazyBuf);
        self().clear_raw(buf.ptr(), buf.len() * sizeof(T));
    }
    // Every element set to `value`, on the device (no host array, no transfer).
    template <class T>
    void fill(Buffer<T, Derived>& buf, T value) {
        if (!buf.has_data()) throw Error(DeviceError::InvalidLazyBuf);
        self().fill_raw(buf.ptr(), buf.len() * sizeof(T), &value, sizeof(T));
    }
    // `WriteBuf::write_buf`
    template <class T>
    void write_buf(Buffer<T, Derived>& dst, const Buffer<T, Derived>& src) {
        if (dst.len() != src.len()) throw Error(DeviceError::ShapeLengthMismatch);
        self().copy_raw(dst.ptr(), src.ptr(), src.len() * sizeof(T));
    }

    // `CopySlice::copy_slice_to` (src/op_traits.rs:68-75, src/devices/cuda/ops.rs:66-87):
    // elements [src_begin, src_end) of `source` into `dest` from `dst_begin` on,
    // device to device.  Ranges that leave either buffer are an error (the reference panics).
    template <class T>
    void copy_slice_to(const Buffer<T, Derived>& source, size_t src_begin, size_t src_end, Buffer<T, Derived>& dest,
                       size_t dst_begin, size_t dst_end) {
        if (!source.has_data() || !dest.has_data()) throw Error(DeviceError::InvalidLazyBuf);
        if (src_begin > src_end || src_end > source.len() || dst_begin > dst_end || dst_end > dest.len() ||
            src_end - src_begin != dst_end - dst_begin)
            throw Error(DeviceError::ShapeLengthMismatch);
        if (src_end == src_begin) return;
        self().copy_raw(dest.ptr() + dst_begin * sizeof(T), source.ptr() + src_begin * sizeof(T),
                        (src_end - src_begin) * sizeof(T));
    }
    // `CopySlice::copy_slice` (src/op_traits.rs:41-53): a new buffer holding the slice
    template <class T>
    Buffer<T, Derived> copy_slice(const Buffer<T, Derived>& buf, size_t begin, size_t end) {
        if (begin > end || end > buf.len()) throw Error(DeviceError::ShapeLengthMismatch);
        Buffer<T, Derived> copied = new_buffer<T>(end - begin);
        copy_slice_to(buf, begin, end, copied, 0, end - begin);
        return copied;
    }
    // `CopySlice::copy_slice_all` (src/devices/cuda/ops.rs:89-98): (source range, dest range) pairs
    struct SlicePair {
        size_t src_begin, src_end, dst_begin, dst_end;
    };
    template <class T>
    void copy_slice_all(const Buffer<T, Derived>& source, Buffer<T, Derived>& dest, const std::vector<SlicePair>& ranges) {
        for (const SlicePair& r : ranges) copy_slice_to(source, r.src_begin, r.src_end, dest, r.dst_begin, r.dst_end);
    }
    // `CloneBuf::clone_buf` (src/op_traits.rs:176-197)
    template <class T>
    Buffer<T, Derived> clone_buf(const Buffer<T, Derived>& buf) {
        return copy_slice(buf, 0, buf.len());
    }

    // ---- operations ----

    // `device.add_op((&mut out, buf), |(out, buf), dev| ...)`.
    // Eager modules call `fn` now with the very arguments; with `Lazy` enabled it
    // is recorded together with the argument ids and called at `run()` with the
    // buffers those ids name then.
    template <class F, class... B>
    void add_op(std::tuple<B&...> args, F fn) {
        if (!modules.is_lazy_enabled()) {
            std::apply([&](B&... b) { fn(b..., self()); }, args);
            return;
        }
        modules.add_op(self(), make_operation(args, std::move(fn)));
    }

    // `device.add_grad_fn((buf, &out), |(buf, out), dev| ...)`: pushed onto the
    // tape when an Autograd module is present, else dropped.
    template <class F, class... B>
    void add_grad_fn(std::tuple<B&...> args, F fn) {
        if (modules.autograd() == nullptr || !modules.is_grad_enabled()) return;
        modules.add_grad_fn(make_operation(args, std::move(fn)));
    }

    // Runs `f` with lazy recording switched off (src/features.rs:438-444).
    template <class F>
    void eagerly(F f) {
        const bool before = modules.is_lazy_enabled();
        modules.set_lazy_enabled(false);
        try {
            f();
        } catch (...) {
            modules.set_lazy_enabled(before);
            throw;
        }
        modules.set_lazy_enabled(before);
    }
    size_t ops_count() const { return modules.ops_count(); }

    // `device.apply_fn(&buf, |x| ...)`: retrieve out, add the op, tag it with the unary hint.
    template <class T, class F>
    Buffer<T, Derived> apply_fn(const Buffer<T, Derived>& buf, F f) {
        Buffer<T, Derived> out = retrieve_output<T>(buf.len(), buf);
        add_op(std::tie(out, buf), [f](Buffer<T, Derived>& o, const Buffer<T, Derived>& x, Derived& dev) {
            dev.apply_fn_impl(x, o, f);
        });
        modules.set_op_hint(erase_hint(unary<T>(f)));
        modules.set_expr_hint(AnyExprHint{expr_hint1<T>(f), std::type_index(typeid(T)), {1}, 0});
        return out;
    }

    // A two-operand element-wise operation in the reference's style for user ops
    // (retrieve + add_op, like the `add` of tests/graph/mod.rs:90-127), with the
    // expression written in the `Combiner` vocabulary: out[i] = f(lhs[i], rhs[i]).
    template <class T, class F>
    Buffer<T, Derived> apply_fn2(const Buffer<T, Derived>& lhs, const Buffer<T, Derived>& rhs, F f) {
        // (a shorter operand would be read beyond its end on the device)
        if (rhs.len() != lhs.len()) throw Error(DeviceError::ShapeLengthMismatch);
        Buffer<T, Derived> out = retrieve_output<T>(lhs.len(), lhs, rhs);
        add_op(std::tie(lhs, rhs, out),
               [f](const Buffer<T, Derived>& l, const Buffer<T, Derived>& r, Buffer<T, Derived>& o, Derived& dev) {
                   dev.apply_fn2_impl(l, r, o, f);
               });
        modules.set_expr_hint(AnyExprHint{expr_hint2<T>(f), std::type_index(typeid(T)), {0, 1}, 2});
        return out;
    }

    // `device.add_unary_grad(&lhs, &mut lhs_grad, &out_grad, |x| ...)`
    template <class T, class F>
    void add_unary_grad(const Buffer<T, Derived>& lhs, Buffer<T, Derived>& lhs_grad,
                        const Buffer<T, Derived>& out_grad, F lhs_grad_fn) {
        if (lhs_grad.len() != lhs.len() || out_grad.len() != lhs.len()) throw Error(DeviceError::ShapeLengthMismatch);
        add_op(std::tie(lhs, lhs_grad, out_grad),
               [lhs_grad_fn](const Buffer<T, Derived>& l, Buffer<T, Derived>& g, const Buffer<T, Derived>& o, Derived& dev) {
                   dev.add_unary_grad_impl(l, g, o, lhs_grad_fn);
               });
    }

    // `device.unary_ew(&mut buf, forward, grad)` (src/unary.rs:97-132)
    template <class T, class FO, class GO>
    Buffer<T, Derived> unary_ew(Buffer<T, Derived>& buf, FO forward_fn, GO grad_fn) {
        Buffer<T, Derived> out = apply_fn(buf, forward_fn);
        add_grad_fn(std::tie(buf, out), [grad_fn](Buffer<T, Derived>& b, Buffer<T, Derived>& o, Derived& dev) {
            if (!b.requires_grad()) return;
            // lazy execution is already disabled during the backward pass
            dev.eagerly([&] {
                Buffer<T, Derived> b_grad = b.grad(dev);
                Buffer<T, Derived> o_grad = o.grad(dev);
                dev.add_unary_grad(b, b_grad, o_grad, grad_fn);
            });
        });
        return out;
    }

    // ---- run / exec_now / optimize ----

    void run() { modules.run(self()); }
    // `exec_now(&device, range)`: run and consume the recorded operations [begin, end)
    void exec_now(size_t begin, size_t end = static_cast<size_t>(-1)) { modules.exec_now(self(), begin, end); }
    // `exec_last_n` (src/features.rs:520-531)
    void exec_last_n(size_t last_n) {
        const size_t n = modules.ops_count();
        modules.exec_now(self(), n - std::min(n, last_n), n);
    }
    void optimize_mem_graph() { modules.optimize_mem_graph(self(), nullptr); }
    void unary_fusing() { modules.unary_fusing(self(), nullptr); }
    // Fuses element-wise operations of any arity (unary chains included); needs `Graph`.
    void elementwise_fusing() { modules.elementwise_fusing(self(), nullptr, {}); }

    // ---- cursor (src/features.rs:68-109, src/range.rs:9-62) ----

    // `for epoch in device.range(begin..end)`: every epoch starts with the cursor
    // where it was when the loop began, so the n-th retrieve of an epoch finds what
    // the n-th retrieve of the epoch before allocated (with a `Cached` module).
    class CursorRange {
       public:
        class Iter {
           public:
            Iter(Derived* dev, size_t at, size_t previous) : dev_(dev), at_(at), previous_(previous) {}
            size_t operator*() const {
                dev_->modules.set_cursor(previous_);
                return at_;
            }
            Iter& operator++() {
                at_++;
                return *this;
            }
            bool operator!=(const Iter& o) const { return at_ < o.at_; }

           private:
            Derived* dev_;
            size_t at_, previous_;
        };
        CursorRange(Derived* dev, size_t begin, size_t end) : dev_(dev), begin_(begin), end_(end), previous_(dev->modules.cursor()) {}
        Iter begin() const { return Iter(dev_, begin_, previous_); }
        Iter end() const { return Iter(dev_, end_, previous_); }

       private:
        Derived* dev_;
        size_t begin_, end_, previous_;
    };
    CursorRange range(size_t begin, size_t end) { return CursorRange(&self(), begin, end); }
    CursorRange range(size_t end) { return CursorRange(&self(), 0, end); }
    size_t cursor() const { return modules.cursor(); }
    void set_cursor(size_t c) { modules.set_cursor(c); }
    // `device.cached(|| ...)`: runs `cb` and rewinds the cursor, so that the next call
    // retrieves the same allocations again (src/features.rs:101-109).
    template <class F>
    void cached(F cb) {
        const size_t previous = modules.cursor();
        cb();
        modules.set_cursor(previous);
    }

    // ---- autograd ----

    // Gradient buffer of `id`, allocated zeroed on first use (autograd/gradients.rs:90-126).
    template <class T>
    Buffer<T, Derived> grad_of(Id id) {
        AutogradState* ag = modules.autograd();
        if (!ag) throw std::logic_error("Autograd<> is not available.");
        auto it = ag->grads.find(id.id);
        if (it == ag->grads.end()) {
            uint64_t ptr = self().alloc_raw(id.len * sizeof(T), /*zeroed=*/true, id.len);
            it = ag->grads.emplace(id.id, AnyBuf{ptr, id.len, std::type_index(typeid(T)), true, sizeof(T)}).first;
        }
        if (it->second.type != std::type_index(typeid(T))) throw Error(DeviceError::TypeMismatch);
        return Buffer<T, Derived>::from_parts(&self(), it->second.ptr, it->second.len, Id{it->second.ptr, it->second.len},
                                              AllocFlag::Wrapper);
    }

    template <class T>
    std::optional<Buffer<T, Derived>> try_grad_of(Id id) {
        AutogradState* ag = modules.autograd();
        if (!ag || ag->grads.find(id.id) == ag->grads.end()) return std::nullopt;
        return grad_of<T>(id);
    }

    // `Gradients::zero_grad` (autograd/gradients.rs:30-42)
    void zero_grad() {
        AutogradState* ag = modules.autograd();
        if (!ag) return;
        for (auto& kv : ag->grads) {
            auto rg = ag->buf_requires_grad.find(kv.first);
            if (rg == ag->buf_requires_grad.end() || rg->second)
                self().clear_raw(kv.second.ptr, kv.second.len * kv.second.elem_size);
        }
    }

    // Seeds `buf`'s gradient and replays the tape in reverse, eagerly; the tape is
    // kept when lazy recording is on (tape.rs:39-83, impl_autograd.rs:37-56).
    template <class T>
    void backward_seeded(const Buffer<T, Derived>& buf, const std::vector<T>& seed) {
        backward_from(buf, [&](Buffer<T, Derived>& g) { write(g, seed); });
    }
    // `Buffer::backward`: a seed of ones.  The reference builds `vec![T::one(); len]` on the host
    // and writes it to the device (impl_autograd.rs:20-34, tape.rs:53-64); here the gradient is
    // filled on the device.
    template <class T>
    void backward_ones(const Buffer<T, Derived>& buf) {
        backward_from(buf, [&](Buffer<T, Derived>& g) { fill(g, T(1)); });
    }
    template <class T, class Seed>
    void backward_from(const Buffer<T, Derived>& buf, Seed seed) {
        AutogradState* ag = modules.autograd();
        if (!ag) return;
        Buffer<T, Derived> g = grad_of<T>(buf.id());
        seed(g);
        const bool lazy_enabled = modules.is_lazy_enabled();
        Buffers* buffers = modules.buffers();
        eagerly([&] {
            for (size_t i = ag->tape.size(); i-- > 0;) ag->tape[i].op(*buffers, &self());
        });
        if (!lazy_enabled) ag->tape.clear();
    }

    void set_grad_enabled(bool e) { modules.set_grad_enabled(e); }
    void enable_grad() { modules.set_grad_enabled(true); }
    void disable_grad() { modules.set_grad_enabled(false); }

   private:
    bool output_hint_ = false;

    template <class BufT>
    static BufT view_of(Derived& dev, Buffers& bufs, Id id) {
        using B = std::remove_const_t<BufT>;
        using T = typename B::value_type;
        auto it = bufs.find(id.id);
        if (it == bufs.end() || it->second.ptr == 0) throw Error(DeviceError::InvalidLazyBuf);
        if (it->second.type != std::type_index(typeid(T))) throw Error(DeviceError::TypeMismatch);
        return B::from_parts(&dev, it->second.ptr, it->second.len, id, AllocFlag::Wrapper,
                             dev.modules.requires_grad_of(id));
    }

    template <class F, class... B, size_t... I>
    static void call_with_views(F& fn, Derived& dev, Buffers& bufs, const std::vector<Id>& ids,
                                std::index_sequence<I...>) {
        std::tuple<std::remove_const_t<B>...> views{view_of<std::remove_const_t<B>>(dev, bufs, ids[I])...};
        fn(std::get<I>(views)..., dev);
    }

    template <class F, class... B>
    Operation make_operation(std::tuple<B&...> args, F fn) {
        Operation op;
        std::apply([&](B&... b) { (op.arg_ids.push_back(b.id()), ...); }, args);
        // every parent must be unique (src/modules/lazy/lazy_graph.rs:117-125)
        for (size_t i = 0; i < op.arg_ids.size(); i++)
            for (size_t j = i + 1; j < op.arg_ids.size(); j++)
                if (op.arg_ids[i].id == op.arg_ids[j].id) throw Error(DeviceError::DuplicateParent);
        std::vector<Id> ids = op.arg_ids;
        op.op = [fn, ids](Buffers& bufs, void* devp) mutable {
            Derived& dev = *static_cast<Derived*>(devp);
            call_with_views<F, B...>(fn, dev, bufs, ids, std::index_sequence_for<B...>{});
        };
        return op;
    }
};

}  // namespace custos
