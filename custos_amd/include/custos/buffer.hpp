// `Buffer<T, D>`: a typed array on device `D`.
// Reference: src/buffer.rs:43-137 (struct, new, require_grad, checkpoint),
// src/buffer/impl_autograd.rs:20-197 (backward, grad), src/id.rs (HasId),
// src/devices/cuda/cuda_ptr.rs:7-89 (base pointer: address, len, flag).
#pragma once

#include <optional>
#include <utility>
#include <vector>

#include "core.hpp"

namespace custos {

template <class T, class D>
class Buffer {
   public:
    using value_type = T;

    Buffer() = default;

    // `Buffer::new(&device, len)`: zero-initialised, owning.
    Buffer(D& device, size_t len) { *this = device.template new_buffer<T>(len); }

    // `Buffer::from((&device, slice))`
    Buffer(D& device, const std::vector<T>& data) { *this = device.template buffer<T>(data); }

    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
    Buffer(Buffer&& o) noexcept { steal(o); }
    Buffer& operator=(Buffer&& o) noexcept {
        if (this != &o) {
            release();
            steal(o);
        }
        return *this;
    }
    ~Buffer() { release(); }

    // Built by devices and modules.
    static Buffer from_parts(D* device, uint64_t ptr, size_t len, Id id, AllocFlag flag, bool requires_grad = false) {
        Buffer b;
        b.device_ = device;
        b.ptr_ = ptr;
        b.len_ = len;
        b.id_ = id;
        b.flag_ = flag;
        b.requires_grad_ = requires_grad;
        return b;
    }

    size_t len() const { return len_; }
    bool is_empty() const { return len_ == 0; }
    Id id() const { return id_; }
    uint64_t ptr() const { return ptr_; }
    AllocFlag flag() const { return flag_; }
    D& device() const { return *device_; }
    bool has_data() const { return ptr_ != 0; }

    // A non-owning copy of the handle (`ShallowCopy`).
    Buffer shallow() const { return from_parts(device_, ptr_, len_, id_, flag_ == AllocFlag::Lazy ? AllocFlag::Lazy : AllocFlag::Wrapper, requires_grad_); }
    // `PtrType::set_flag` (src/devices/cuda/cuda_ptr.rs:51-61): who frees the memory.
    void set_flag(AllocFlag flag) { flag_ = flag; }

    // `Read::read`: device -> host.
    std::vector<T> read() const { return device_->read(*this); }
    // `WriteBuf::write`
    void write(const std::vector<T>& data) { device_->write(*this, data); }
    // `ClearBuf::clear`
    void clear() { device_->clear(*this); }

    // The real buffer behind a lazily retrieved handle (`ReplaceBuf::replace_buf`,
    // src/modules/lazy.rs:430-455); the handle itself when there is nothing to replace.
    Buffer replace() const { return device_->modules.template replace_buf<T>(*device_, *this); }

    // src/buffer.rs:104-128
    Buffer require_grad() && {
        requires_grad_ = true;
        device_->modules.set_requires_grad(id_, true);
        return std::move(*this);
    }
    Buffer no_grad() && {
        requires_grad_ = false;
        device_->modules.set_requires_grad(id_, false);
        return std::move(*this);
    }
    bool requires_grad() const { return requires_grad_; }
    void set_requires_grad_flag(bool v) { requires_grad_ = v; }

    // Excludes the buffer from cache traces and unary fusing (src/buffer.rs:131-137).
    Buffer checkpoint() && {
        device_->modules.set_checkpoint_buffer(id_);
        return std::move(*this);
    }

    // src/buffer/impl_autograd.rs:20-56
    void backward() const { device_->backward_ones(*this); }
    void backward_with(const std::vector<T>& seed) const { device_->backward_seeded(*this, seed); }

    // Gradient of this buffer, allocated (zeroed) on first use
    // (src/buffer/impl_autograd.rs:95-100,188-197).
    Buffer grad(D& device) const { return device.template grad_of<T>(id_); }
    Buffer grad() const { return device_->template grad_of<T>(id_); }
    // The gradient if this buffer requires one and it has been allocated
    // (src/buffer/impl_autograd.rs:102-125).
    std::optional<Buffer> try_grad(D& device) const {
        if (!requires_grad_) return std::nullopt;
        return device.template try_grad_of<T>(id_);
    }

    // `impl Clone for Buffer` (src/buffer.rs:598-606): a new buffer with the same contents.
    Buffer clone() const { return device_->clone_buf(*this); }
    // `buf.empty_like()`: a new zeroed buffer of the same length.
    Buffer empty_like() const { return device_->template new_buffer<T>(len_); }

   private:
    void steal(Buffer& o) {
        device_ = o.device_;
        ptr_ = o.ptr_;
        len_ = o.len_;
        id_ = o.id_;
        flag_ = o.flag_;
        requires_grad_ = o.requires_grad_;
        o.device_ = nullptr;
        o.ptr_ = 0;
        o.flag_ = AllocFlag::Wrapper;
    }
    void release() {
        if (device_ && flag_ == AllocFlag::None && ptr_ != 0) {
            device_->modules.on_drop_buffer(id_);
            device_->free_raw(ptr_);
        } else if (device_ && flag_ == AllocFlag::Cached && ptr_ != 0) {
            device_->modules.on_release_cached(ptr_);
        }
        device_ = nullptr;
        ptr_ = 0;
    }

    D* device_ = nullptr;
    uint64_t ptr_ = 0;
    size_t len_ = 0;
    Id id_{};
    AllocFlag flag_ = AllocFlag::Wrapper;
    bool requires_grad_ = false;
};

}  // namespace custos
