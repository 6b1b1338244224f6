// Serialisation of buffers as a sequence of their elements.
//
// The reference derives `Serialize` / `Deserialize` for `Buffer` and skips the device
// (src/buffer.rs:42-49); what is written is the base pointer's data: a device pointer reads its
// memory into a host pointer and serialises that as a sequence of `len` elements, and
// deserialising collects the sequence on the host, allocates on the device and writes
// (src/devices/cuda/cuda_ptr.rs:121-157, src/devices/cpu/cpu_ptr.rs:320-393).  serde is
// format-agnostic; the reference pins the format-independent token stream
// (`Seq{len}`, one token per element, `SeqEnd`: cuda_ptr.rs:163-189).  The same two views here:
// the token stream, and a JSON array, which is what serde_json makes of such a sequence.
// 16-bit floats travel as their 16 bits (the `half` crate's types are newtypes over `u16`).
#pragma once

#include <cinttypes>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

#include "buffer.hpp"
#include "half.hpp"

namespace custos {
namespace serde {

enum class TokenKind { Seq, SeqEnd, I8, I16, I32, I64, U8, U16, U32, U64, F32, F64 };

struct Token {
    TokenKind kind = TokenKind::SeqEnd;
    uint64_t bits = 0;  // Seq: the length; integers: the value (two's complement); F32 / F64: the IEEE bits

    static Token seq(uint64_t len) { return {TokenKind::Seq, len}; }
    static Token seq_end() { return {TokenKind::SeqEnd, 0}; }
    bool operator==(const Token& o) const { return kind == o.kind && bits == o.bits; }
    bool operator!=(const Token& o) const { return !(*this == o); }
};

template <class T>
struct ElementKind;
#define CUSTOS_SERDE_KIND(T, K)                           \
    template <>                                           \
    struct ElementKind<T> {                               \
        static constexpr TokenKind value = TokenKind::K;  \
    };
CUSTOS_SERDE_KIND(int8_t, I8)
CUSTOS_SERDE_KIND(int16_t, I16)
CUSTOS_SERDE_KIND(int32_t, I32)
CUSTOS_SERDE_KIND(int64_t, I64)
CUSTOS_SERDE_KIND(uint8_t, U8)
CUSTOS_SERDE_KIND(uint16_t, U16)
CUSTOS_SERDE_KIND(uint32_t, U32)
CUSTOS_SERDE_KIND(uint64_t, U64)
CUSTOS_SERDE_KIND(float, F32)
CUSTOS_SERDE_KIND(double, F64)
CUSTOS_SERDE_KIND(f16, U16)
CUSTOS_SERDE_KIND(bf16, U16)
CUSTOS_SERDE_KIND(f16_pernode, U16)
CUSTOS_SERDE_KIND(bf16_pernode, U16)
#undef CUSTOS_SERDE_KIND

template <class T>
Token element_token(const T& v) {
    Token t;
    t.kind = ElementKind<T>::value;
    if constexpr (is_half16<T>::value) {
        t.bits = v.bits;
    } else if constexpr (std::is_floating_point_v<T>) {
        std::memcpy(&t.bits, &v, sizeof(T));
    } else {
        t.bits = static_cast<uint64_t>(static_cast<int64_t>(v));
    }
    return t;
}

template <class T>
T element_from_token(const Token& t) {
    if (t.kind != ElementKind<T>::value) throw Error(DeviceError::TypeMismatch);
    if constexpr (is_half16<T>::value) {
        return T::from_bits(static_cast<uint16_t>(t.bits));
    } else if constexpr (std::is_floating_point_v<T>) {
        T v;
        std::memcpy(&v, &t.bits, sizeof(T));
        return v;
    } else {
        return static_cast<T>(static_cast<int64_t>(t.bits));
    }
}

// `Serialize for Buffer`: the elements, read from the device, as `Seq{len} e0 .. SeqEnd`.
template <class T, class D>
std::vector<Token> to_tokens(const Buffer<T, D>& buf) {
    const std::vector<T> host = buf.read();
    std::vector<Token> out;
    out.reserve(host.size() + 2);
    out.push_back(Token::seq(host.size()));
    for (const T& v : host) out.push_back(element_token(v));
    out.push_back(Token::seq_end());
    return out;
}

// `Deserialize for Buffer`: collects the sequence on the host, allocates on `device`, writes.
// A sequence that is not one (`Seq{len}`, exactly len elements of T's kind, `SeqEnd`) is a
// `ShapeLengthMismatch` / `TypeMismatch`; an empty one a `ZeroLengthBuffer`, like any allocation.
template <class T, class D>
Buffer<T, D> from_tokens(D& device, const std::vector<Token>& tokens) {
    if (tokens.size() < 2 || tokens.front().kind != TokenKind::Seq || tokens.back().kind != TokenKind::SeqEnd ||
        tokens.front().bits != tokens.size() - 2)
        throw Error(DeviceError::ShapeLengthMismatch);
    std::vector<T> host;
    host.reserve(tokens.size() - 2);
    for (size_t i = 1; i + 1 < tokens.size(); i++) host.push_back(element_from_token<T>(tokens[i]));
    return device.template buffer<T>(host);
}

// ---- the same sequence as text: a JSON array ----

namespace detail {

template <class T>
void print_element(std::string* out, const T& v) {
    char text[40];
    if constexpr (is_half16<T>::value) {
        std::snprintf(text, sizeof text, "%u", static_cast<unsigned>(v.bits));
    } else if constexpr (std::is_floating_point_v<T>) {
        // (JSON has no spelling for them; serde_json writes `null`, which it then cannot read back)
        if (!std::isfinite(v)) throw Error(DeviceError::Backend, 0, "a JSON array cannot hold a NaN or an infinity");
        // shortest text that reads back to the same bits
        const int digits = sizeof(T) == 4 ? 9 : 17;
        for (int p = 1; p <= digits; p++) {
            std::snprintf(text, sizeof text, "%.*g", p, static_cast<double>(v));
            if (static_cast<T>(std::strtod(text, nullptr)) == v) break;
        }
        if (!std::strpbrk(text, ".eE")) std::strcat(text, ".0");
    } else if constexpr (std::is_signed_v<T>) {
        std::snprintf(text, sizeof text, "%" PRId64, static_cast<int64_t>(v));
    } else {
        std::snprintf(text, sizeof text, "%" PRIu64, static_cast<uint64_t>(v));
    }
    *out += text;
}

template <class T>
T parse_element(const char* begin, const char** end) {
    char* stop = nullptr;
    if constexpr (is_half16<T>::value) {
        const unsigned long long bits = std::strtoull(begin, &stop, 10);
        if (stop == begin || bits > 0xffffu) throw Error(DeviceError::TypeMismatch);
        *end = stop;
        return T::from_bits(static_cast<uint16_t>(bits));
    } else if constexpr (std::is_floating_point_v<T>) {
        const double v = std::strtod(begin, &stop);
        if (stop == begin) throw Error(DeviceError::TypeMismatch);
        *end = stop;
        return static_cast<T>(v);
    } else if constexpr (std::is_signed_v<T>) {
        const long long v = std::strtoll(begin, &stop, 10);
        if (stop == begin || static_cast<long long>(static_cast<T>(v)) != v || *stop == '.' || *stop == 'e' || *stop == 'E')
            throw Error(DeviceError::TypeMismatch);
        *end = stop;
        return static_cast<T>(v);
    } else {
        if (*begin == '-') throw Error(DeviceError::TypeMismatch);
        const unsigned long long v = std::strtoull(begin, &stop, 10);
        if (stop == begin || static_cast<unsigned long long>(static_cast<T>(v)) != v || *stop == '.' || *stop == 'e' || *stop == 'E')
            throw Error(DeviceError::TypeMismatch);
        *end = stop;
        return static_cast<T>(v);
    }
}

inline const char* skip_space(const char* p) {
    while (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r') p++;
    return p;
}

}  // namespace detail

template <class T, class D>
std::string to_json(const Buffer<T, D>& buf) {
    const std::vector<T> host = buf.read();
    std::string out = "[";
    for (size_t i = 0; i < host.size(); i++) {
        if (i) out += ",";
        detail::print_element(&out, host[i]);
    }
    return out + "]";
}

template <class T, class D>
Buffer<T, D> from_json(D& device, const std::string& text) {
    const char* p = detail::skip_space(text.c_str());
    if (*p != '[') throw Error(DeviceError::ShapeLengthMismatch);
    p = detail::skip_space(p + 1);
    std::vector<T> host;
    while (*p != ']') {
        if (!host.empty()) {
            if (*p != ',') throw Error(DeviceError::ShapeLengthMismatch);
            p = detail::skip_space(p + 1);
        }
        host.push_back(detail::parse_element<T>(p, &p));
        p = detail::skip_space(p);
        if (*p == '\0') throw Error(DeviceError::ShapeLengthMismatch);
    }
    if (*detail::skip_space(p + 1) != '\0') throw Error(DeviceError::ShapeLengthMismatch);
    return device.template buffer<T>(host);
}

}  // namespace serde
}  // namespace custos
