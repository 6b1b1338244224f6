// Plumbing shared by the modules: errors, ids, type-erased buffer records,
// recorded operations and unary op hints.
// Reference: src/error.rs:25-57 (DeviceError), src/id.rs:5-37 (Id),
// src/flag.rs:6-27 (AllocFlag), src/op_hint.rs:5-35 (OpHint, unary()).
#pragma once

#include <cstddef>
#include <cstdint>
#include <functional>
#include <memory>
#include <stdexcept>
#include <string>
#include <typeindex>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "combiner.hpp"

namespace custos {

enum class DeviceError {
    MissingCacheTraces,      // optimize / fuse without a Graph module
    GraphOptimization,
    InvalidLazyBuf,          // an operation's buffer went out of scope before run()
    UnaryFusingUnsupported,
    ZeroLengthBuffer,
    ShapeLengthMismatch,
    DuplicateParent,         // "each parent (id) must be unique" (lazy_graph.rs:121-123)
    IdCollision,             // "IDs collided!" (src/modules/lazy.rs:354-357)
    TypeMismatch,            // a recorded buffer is used with another element type
    CachedInUse,             // a cached allocation is replaced while a buffer handle still uses it
    Backend,                 // the device library reported an error (code in Error::code)
};

inline const char* device_error_str(DeviceError e) {
    switch (e) {
        case DeviceError::MissingCacheTraces: return "No cache traces were given";
        case DeviceError::GraphOptimization: return "This graph can't be optimized.";
        case DeviceError::InvalidLazyBuf:
            return "Invalid lazy buffer was provided in operation. Did the buffer go out of scope?";
        case DeviceError::UnaryFusingUnsupported: return "Unary fusing not supported.";
        case DeviceError::ZeroLengthBuffer: return "Zero length buffers are not supported";
        case DeviceError::ShapeLengthMismatch: return "Given length does not match the data length";
        case DeviceError::DuplicateParent: return "each parent (id) must be unique";
        case DeviceError::IdCollision: return "IDs collided! Maybe a device address already occupies this id.";
        case DeviceError::TypeMismatch: return "Type data does not match";
        case DeviceError::CachedInUse: return "A cached allocation is still in use by a buffer";
        case DeviceError::Backend: return "device library error";
    }
    return "";
}

// `crate::Error`: what a failing `Result` carries in the reference.
class Error : public std::runtime_error {
   public:
    DeviceError kind;
    int code;  // status of the device library for DeviceError::Backend, else 0
    explicit Error(DeviceError k) : std::runtime_error(device_error_str(k)), kind(k), code(0) {}
    Error(DeviceError k, int c, const std::string& msg) : std::runtime_error(msg), kind(k), code(c) {}
};

using UniqueId = uint64_t;

struct Id {
    UniqueId id = 0;
    size_t len = 0;
    bool operator==(const Id& o) const { return id == o.id && len == o.len; }
    bool operator!=(const Id& o) const { return !(*this == o); }
};

enum class AllocFlag {
    None,     // the holder owns the allocation
    Wrapper,  // a shallow copy: never frees (src/flag.rs:24-26)
    Lazy,     // an id without memory yet
    Cached,   // memory kept by a Cached module; the handle only reports its drop (src/flag.rs:14-16)
};

// Type-erased shallow copy of a buffer, what modules keep per id
// (`Box<dyn BoxedShallowCopy>` in the reference).
struct AnyBuf {
    uint64_t ptr = 0;
    size_t len = 0;
    std::type_index type = std::type_index(typeid(void));
    bool module_owned = false;  // allocated by a module (Lazy::alloc_later, gradients), freed by it
    size_t elem_size = 0;
};

using Buffers = std::unordered_map<UniqueId, AnyBuf>;

// ---- unary op hints (src/op_hint.rs:5-35) ----

template <class T>
struct UnaryHint {
    // `op(resolve).to_cl_source()` with the given marker
    std::function<std::string(const char*)> to_cl_source;
    // `op(resolve).eval()`
    std::function<T(T)> eval;
};

enum class OpHintKind { None, Unary, UnaryFused };

template <class T>
struct OpHint {
    OpHintKind kind = OpHintKind::None;
    std::shared_ptr<UnaryHint<T>> unary;  // set for Unary
};

// `unary(f)`: wraps an expression factory so it can be re-evaluated or re-printed later.
template <class T, class F>
OpHint<T> unary(F f) {
    auto h = std::make_shared<UnaryHint<T>>();
    h->to_cl_source = [f](const char* marker) { return custos::to_cl_source(f(Resolve<T>::with_marker(marker))); };
    h->eval = [f](T v) { return custos::eval<T>(f(Resolve<T>::with_val(v))); };
    return OpHint<T>{OpHintKind::Unary, std::move(h)};
}

// ---- expression hints of any arity ----
//
// The reference tags only unary operations (`OpHint::Unary`), so only unary
// chains can be fused.  Every element-wise operation recorded through
// `apply_fn` / `apply_fn2` additionally carries an `ExprHint`: the expression
// over k operands, re-printable with any operand texts and evaluable on the
// host.  `Lazy::elementwise_fusing` composes them across operations.
template <class T>
struct ExprHint {
    int arity = 1;
    // the expression's text with `operands[i]` in place of the i-th marker
    std::function<std::string(const std::vector<std::string>& operands)> to_cl_source;
    // the expression's value for the operand values `vals[0..arity)`
    std::function<T(const T* vals)> eval;
};

template <class T, class F>
std::shared_ptr<ExprHint<T>> expr_hint1(F f) {
    auto h = std::make_shared<ExprHint<T>>();
    h->arity = 1;
    h->to_cl_source = [f](const std::vector<std::string>& m) {
        return custos::to_cl_source(f(Resolve<T>::with_marker(m[0].c_str())));
    };
    h->eval = [f](const T* v) { return custos::eval<T>(f(Resolve<T>::with_val(v[0]))); };
    return h;
}

template <class T, class F>
std::shared_ptr<ExprHint<T>> expr_hint2(F f) {
    auto h = std::make_shared<ExprHint<T>>();
    h->arity = 2;
    h->to_cl_source = [f](const std::vector<std::string>& m) {
        return custos::to_cl_source(f(Resolve<T>::with_marker(m[0].c_str()), Resolve<T>::with_marker(m[1].c_str())));
    };
    h->eval = [f](const T* v) { return custos::eval<T>(f(Resolve<T>::with_val(v[0]), Resolve<T>::with_val(v[1]))); };
    return h;
}

// Several hinted operations composed into one expression over `leaves.size()`
// distinct operand buffers.  Item inputs >= 0 name a leaf, inputs < 0 name
// another item (~input).
template <class T>
struct FusedExpr {
    struct Item {
        std::shared_ptr<ExprHint<T>> hint;
        std::vector<int> inputs;
    };
    std::vector<Item> items;
    int root = 0;
    std::vector<Id> leaves;

    std::string to_cl_source(const std::vector<std::string>& leaf_markers) const { return print(root, leaf_markers); }
    T eval(const T* leaf_vals) const { return eval_item(root, leaf_vals); }
    size_t op_count() const { return items.size(); }

   private:
    std::string print(int item, const std::vector<std::string>& leaf_markers) const {
        std::vector<std::string> operands;
        for (int in : items[item].inputs) operands.push_back(in >= 0 ? leaf_markers[in] : print(~in, leaf_markers));
        return items[item].hint->to_cl_source(operands);
    }
    T eval_item(int item, const T* leaf_vals) const {
        T vals[8];
        const auto& ins = items[item].inputs;
        for (size_t i = 0; i < ins.size(); i++) vals[i] = ins[i] >= 0 ? leaf_vals[ins[i]] : eval_item(~ins[i], leaf_vals);
        return items[item].hint->eval(vals);
    }
};

// `operations_to_fused_src` (src/devices/fusing.rs:4-19)
template <class T>
std::string operations_to_fused_src(const std::vector<std::shared_ptr<UnaryHint<T>>>& ops) {
    std::string acc;
    for (const auto& op : ops) acc += std::string("x = ") + op->to_cl_source("x") + ";\n";
    return acc;
}

}  // namespace custos
