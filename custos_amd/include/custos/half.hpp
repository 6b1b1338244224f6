// 16-bit floating-point element types for the host side.
//
// The reference takes `f16` / `bf16` from the `half` crate and implements its
// `Number` / `Float` traits for them by widening to f32, operating there and
// rounding back (src/number.rs:487-676).  These types do the same: every
// arithmetic operator and math function below goes through `float` and rounds
// to nearest even, so evaluating an expression on the host rounds at every node.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstring>
#include <type_traits>

namespace custos {

namespace detail {

inline uint32_t f32_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
inline float f32_from_bits(uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// IEEE binary32 -> binary16, round to nearest even; NaN stays NaN (quiet).
inline uint16_t f32_to_f16_bits(float f) {
    const uint32_t u = f32_bits(f);
    const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
    const uint32_t mag = u & 0x7fffffffu;
    if (mag >= 0x7f800000u) return static_cast<uint16_t>(sign | (mag > 0x7f800000u ? 0x7e00u : 0x7c00u));
    if (mag >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);  // rounds to at least 65520: infinity
    if (mag < 0x38800000u) {
        // below the smallest normal half (2^-14): the result is a subnormal, a multiple of 2^-24
        if (mag < 0x33000000u) return sign;  // below 2^-25: zero (2^-25 itself ties to even = zero)
        const int shift = 126 - static_cast<int>(mag >> 23);  // 14..24 bits dropped from the 24-bit significand
        const uint32_t sig = (mag & 0x7fffffu) | 0x800000u;
        const uint32_t kept = sig >> shift, rest = sig & ((1u << shift) - 1), half = 1u << (shift - 1);
        return static_cast<uint16_t>(sign | (kept + ((rest > half || (rest == half && (kept & 1u))) ? 1u : 0u)));
    }
    // normal: rebias the exponent (127 -> 15), keep 10 significand bits, round on the 13 dropped ones
    const uint32_t rebased = mag - 0x38000000u;
    const uint32_t kept = rebased >> 13, rest = rebased & 0x1fffu;
    return static_cast<uint16_t>(sign | (kept + ((rest > 0x1000u || (rest == 0x1000u && (kept & 1u))) ? 1u : 0u)));
}

inline float f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu, sig = h & 0x3ffu;
    if (exp == 0x1fu) return f32_from_bits(sign | 0x7f800000u | (sig << 13));
    if (exp != 0) return f32_from_bits(sign | ((exp + 112u) << 23) | (sig << 13));
    if (sig == 0) return f32_from_bits(sign);
    const float magnitude = static_cast<float>(sig) * 5.9604644775390625e-8f;  // sig * 2^-24, exact
    return sign ? -magnitude : magnitude;
}

inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

}  // namespace detail

// CRTP base: storage, conversions and the arithmetic of a 16-bit float.
template <class Derived>
struct Half16 {
    uint16_t bits = 0;

    Half16() = default;
    Half16(float v) : bits(Derived::encode(v)) {}
    operator float() const { return Derived::decode(bits); }

    static Derived from_bits(uint16_t b) {
        Derived d;
        d.bits = b;
        return d;
    }

    friend Derived operator+(Derived a, Derived b) { return Derived(float(a) + float(b)); }
    friend Derived operator-(Derived a, Derived b) { return Derived(float(a) - float(b)); }
    friend Derived operator*(Derived a, Derived b) { return Derived(float(a) * float(b)); }
    friend Derived operator/(Derived a, Derived b) { return Derived(float(a) / float(b)); }
    friend Derived operator-(Derived a) { return from_bits(static_cast<uint16_t>(a.bits ^ 0x8000u)); }
};

// f16 / bf16: f32 compute and one rounding at the store in the device kernels.
struct f16 : Half16<f16> {
    using Half16<f16>::Half16;
    static uint16_t encode(float v) { return detail::f32_to_f16_bits(v); }
    static float decode(uint16_t b) { return detail::f16_bits_to_f32(b); }
};
struct bf16 : Half16<bf16> {
    using Half16<bf16>::Half16;
    static uint16_t encode(float v) { return detail::f32_to_bf16_bits(v); }
    static float decode(uint16_t b) { return detail::f32_from_bits(static_cast<uint32_t>(b) << 16); }
};
// The same storage with every node of an expression rounded to 16 bits on the
// device too: bit-identical to evaluating the expression with these host types
// for + - * / sqrt and the exact nodes.
struct f16_pernode : Half16<f16_pernode> {
    using Half16<f16_pernode>::Half16;
    static uint16_t encode(float v) { return detail::f32_to_f16_bits(v); }
    static float decode(uint16_t b) { return detail::f16_bits_to_f32(b); }
};
struct bf16_pernode : Half16<bf16_pernode> {
    using Half16<bf16_pernode>::Half16;
    static uint16_t encode(float v) { return detail::f32_to_bf16_bits(v); }
    static float decode(uint16_t b) { return detail::f32_from_bits(static_cast<uint32_t>(b) << 16); }
};

template <class T>
struct is_half16 : std::false_type {};
template <> struct is_half16<f16> : std::true_type {};
template <> struct is_half16<bf16> : std::true_type {};
template <> struct is_half16<f16_pernode> : std::true_type {};
template <> struct is_half16<bf16_pernode> : std::true_type {};

}  // namespace custos
