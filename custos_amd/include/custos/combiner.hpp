// Expression DSL: `Combiner` builder methods, `Eval` and `ToCLSource`.
//
// C++ mirror of the reference's src/two_way_ops/{combiner,eval,resolve,ops,
// ops/unary,ops/cmps,to_cl_source}.rs.  A generic lambda
//     [](auto x) { return x.sin().mul(2.0f).add(1.0f); }
// called with `Resolve<T>` builds a type tree; every node has
//     eval()          the value, one operation in T per node (Eval),
//     to_cl_source()  the text the reference prints (ToCLSource).
// The HIP device only uses the text; eval() is the host-side meaning of a node.
#pragma once

#include <charconv>
#include <cmath>
#include <cstdint>
#include <string>
#include <type_traits>

#include "half.hpp"

namespace custos {

template <class Derived>
struct Combiner;

template <class N> struct Scalar;
struct Text;
template <class C, class R> struct Mul;
template <class C, class R> struct Add;
template <class C, class R> struct Sub;
template <class C, class R> struct Div;
template <class C, class R> struct Pow;
template <class C, class R> struct Min;
template <class C, class R> struct Max;
template <class C, class R> struct GEq;
template <class C, class R> struct LEq;
template <class C, class R> struct Eq;
template <class C> struct Exp;
template <class C> struct Sin;
template <class C> struct Cos;
template <class C> struct Tan;
template <class C> struct Tanh;
template <class C> struct Ln;
template <class C> struct Abs;
template <class C> struct Neg;
template <class C> struct Sqrt;
template <class C> struct Identity;

namespace detail {
// what an operand becomes inside a node: scalars and text are wrapped, trees stay
template <class R, class = void>
struct Wrapped {
    using type = R;
};
template <class R>
struct Wrapped<R, std::enable_if_t<std::is_arithmetic_v<R> || is_half16<R>::value>> {
    using type = Scalar<R>;
};
template <class R>
struct Wrapped<R, std::enable_if_t<std::is_convertible_v<R, const char*>>> {
    using type = Text;
};
template <class R>
using wrapped_t = typename Wrapped<R>::type;
template <class R>
wrapped_t<R> wrap_operand(R r);
}  // namespace detail

// Builder methods: src/two_way_ops/combiner.rs:8-116
template <class Derived>
struct Combiner {
    const Derived& self() const { return static_cast<const Derived&>(*this); }

    template <class R> auto add(R rhs) const { return Add<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto mul(R rhs) const { return Mul<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto sub(R rhs) const { return Sub<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto div(R rhs) const { return Div<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto pow(R rhs) const { return Pow<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto min(R rhs) const { return Min<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto max(R rhs) const { return Max<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto geq(R rhs) const { return GEq<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto leq(R rhs) const { return LEq<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }
    template <class R> auto eq(R rhs) const { return Eq<Derived, detail::wrapped_t<R>>(self(), detail::wrap_operand(rhs)); }

    auto sin() const { return Sin<Derived>(self()); }
    auto cos() const { return Cos<Derived>(self()); }
    auto tan() const { return Tan<Derived>(self()); }
    auto tanh() const { return Tanh<Derived>(self()); }
    auto exp() const { return Exp<Derived>(self()); }
    auto ln() const { return Ln<Derived>(self()); }
    auto abs() const { return Abs<Derived>(self()); }
    auto neg() const { return Neg<Derived>(self()); }
    auto sqrt() const { return Sqrt<Derived>(self()); }
    auto identity() const { return Identity<Derived>(self()); }
};

namespace detail {

// Scalars print like Rust's `{:?}` (src/two_way_ops/to_cl_source.rs:7-11):
// shortest text that round-trips, whole floats keep a ".0".
template <class N>
std::string scalar_source(N v) {
    if constexpr (std::is_floating_point_v<N>) {
        if (std::isnan(v)) return "NaN";
        if (std::isinf(v)) return v > 0 ? "inf" : "-inf";
        char buf[64];
        auto res = std::to_chars(buf, buf + sizeof buf, v);
        std::string s(buf, res.ptr);
        if (s.find_first_of(".en") == std::string::npos) s += ".0";
        return s;
    } else if constexpr (is_half16<N>::value) {
        return scalar_source(static_cast<float>(v));
    } else if constexpr (std::is_same_v<N, bool>) {
        return v ? "true" : "false";
    } else {
        return std::to_string(v);
    }
}

}  // namespace detail

// A scalar operand (`impl<T: Numeric> Combiner for T`, src/two_way_ops/eval.rs:17-24).
template <class N>
struct Scalar : Combiner<Scalar<N>> {
    N value;
    explicit constexpr Scalar(N v) : value(v) {}
    template <class T>
    T eval() const {
        return static_cast<T>(value);
    }
    std::string to_cl_source() const { return detail::scalar_source(value); }
};

// A piece of source text used as an operand (`impl ToCLSource for &'static str`).
struct Text : Combiner<Text> {
    std::string text;
    explicit Text(std::string t) : text(std::move(t)) {}
    template <class T>
    T eval() const {
        return static_cast<T>(std::stod(text));
    }
    std::string to_cl_source() const { return text; }
};

namespace detail {
template <class R>
wrapped_t<R> wrap_operand(R r) {
    if constexpr (std::is_arithmetic_v<R> || is_half16<R>::value) return Scalar<R>(r);
    else if constexpr (std::is_convertible_v<R, const char*>) return Text(std::string(r));
    else return r;
}
}  // namespace detail

#define CUSTOS_BINARY_NODE(Name, EVAL_EXPR, FMT_PRE, FMT_MID, FMT_POST)                           \
    template <class C, class R>                                                                   \
    struct Name : Combiner<Name<C, R>> {                                                          \
        C comb;                                                                                   \
        R rhs;                                                                                    \
        Name(C c, R r) : comb(std::move(c)), rhs(std::move(r)) {}                                 \
        template <class T>                                                                        \
        T eval() const {                                                                          \
            const T a = comb.template eval<T>();                                                  \
            const T b = rhs.template eval<T>();                                                   \
            return EVAL_EXPR;                                                                     \
        }                                                                                         \
        std::string to_cl_source() const {                                                        \
            return std::string(FMT_PRE) + comb.to_cl_source() + FMT_MID + rhs.to_cl_source() + FMT_POST; \
        }                                                                                         \
    };

// src/two_way_ops/ops.rs:15-314
CUSTOS_BINARY_NODE(Mul, static_cast<T>(a * b), "(", " * ", ")")
CUSTOS_BINARY_NODE(Add, static_cast<T>(a + b), "(", " + ", ")")
CUSTOS_BINARY_NODE(Sub, static_cast<T>(a - b), "(", " - ", ")")
CUSTOS_BINARY_NODE(Div, static_cast<T>(a / b), "(", " / ", ")")
CUSTOS_BINARY_NODE(Pow, static_cast<T>(std::pow(a, b)), "pow(", ", ", ")")
// Number::min / Number::max are selects on < and > (src/number.rs:201-209)
CUSTOS_BINARY_NODE(Min, (a < b ? a : b), "min(", ", ", ")")
CUSTOS_BINARY_NODE(Max, (a > b ? a : b), "max(", ", ", ")")
// src/two_way_ops/ops/cmps.rs:6-139.  The reference's CPU `Eq::eval` compares
// with `<=` (cmps.rs:135) while its source text is "=="; eval() here follows
// the text, like every GPU backend of the reference does.
CUSTOS_BINARY_NODE(GEq, static_cast<T>(a >= b), "(", " >= ", ")")
CUSTOS_BINARY_NODE(LEq, static_cast<T>(a <= b), "(", " <= ", ")")
CUSTOS_BINARY_NODE(Eq, static_cast<T>(a == b), "(", " == ", ")")
#undef CUSTOS_BINARY_NODE

#define CUSTOS_UNARY_NODE(Name, EVAL_EXPR, FMT_PRE)                                               \
    template <class C>                                                                            \
    struct Name : Combiner<Name<C>> {                                                             \
        C comb;                                                                                   \
        explicit Name(C c) : comb(std::move(c)) {}                                                \
        template <class T>                                                                        \
        T eval() const {                                                                          \
            const T a = comb.template eval<T>();                                                  \
            return EVAL_EXPR;                                                                     \
        }                                                                                         \
        std::string to_cl_source() const { return std::string(FMT_PRE) + "(" + comb.to_cl_source() + ")"; } \
    };

// src/two_way_ops/ops/unary.rs:27-267
CUSTOS_UNARY_NODE(Exp, static_cast<T>(std::exp(a)), "exp")
CUSTOS_UNARY_NODE(Sin, static_cast<T>(std::sin(a)), "sin")
CUSTOS_UNARY_NODE(Cos, static_cast<T>(std::cos(a)), "cos")
CUSTOS_UNARY_NODE(Tan, static_cast<T>(std::tan(a)), "tan")
CUSTOS_UNARY_NODE(Tanh, static_cast<T>(std::tanh(a)), "tanh")
CUSTOS_UNARY_NODE(Ln, static_cast<T>(std::log(a)), "log")
CUSTOS_UNARY_NODE(Abs, static_cast<T>(a < 0 ? -a : (a == 0 ? T(0) : a)), "abs")
CUSTOS_UNARY_NODE(Neg, static_cast<T>(-a), "-")
// not a reference node; `Float::sqrt` (src/number.rs:320-322)
CUSTOS_UNARY_NODE(Sqrt, static_cast<T>(std::sqrt(a)), "sqrt")
#undef CUSTOS_UNARY_NODE

// src/two_way_ops/ops/unary.rs:6-33: prints and evaluates as its operand
template <class C>
struct Identity : Combiner<Identity<C>> {
    C comb;
    explicit Identity(C c) : comb(std::move(c)) {}
    template <class T>
    T eval() const {
        return comb.template eval<T>();
    }
    std::string to_cl_source() const { return comb.to_cl_source(); }
};

// Leaf: a value for eval, a marker name for source (src/two_way_ops/resolve.rs:25-141).
// A leaf made from a value (`to_val`) prints that value: the reference prints
// the default marker "x" for it, so `|x| 2.0.to_val()` means 2 on its CPU
// device and x on its GPU devices; here it means 2 everywhere.
template <class T>
struct Resolve : Combiner<Resolve<T>> {
    T val{};
    const char* marker = "x";
    bool is_value = false;

    static Resolve with_val(T v) {
        Resolve r;
        r.val = v;
        r.is_value = true;
        return r;
    }
    static Resolve with_marker(const char* m) {
        Resolve r;
        r.marker = m;
        return r;
    }

    template <class U = T>
    U eval() const {
        return static_cast<U>(val);
    }
    std::string to_cl_source() const { return is_value ? detail::scalar_source(val) : std::string(marker); }
};

// `v.to_val()` and `"x".to_marker()` (src/two_way_ops/resolve.rs:33-80)
template <class T>
Resolve<T> to_val(T v) {
    return Resolve<T>::with_val(v);
}
template <class T>
Resolve<T> to_marker(const char* m) {
    return Resolve<T>::with_marker(m);
}

// Evaluates a tree in its leaf type: `f(x.to_val()).eval()`.
template <class T, class E>
T eval(const E& e) {
    return detail::wrap_operand(e).template eval<T>();
}
template <class E>
std::string to_cl_source(const E& e) {
    return detail::wrap_operand(e).to_cl_source();
}

}  // namespace custos
