// Minimal test harness: named cases, CHECK macros, exit code = failures.
#pragma once

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

namespace check {

struct Case {
    std::string name;
    std::function<void()> fn;
};
inline std::vector<Case>& cases() {
    static std::vector<Case> c;
    return c;
}
inline int& failures() {
    static int f = 0;
    return f;
}
struct Registrar {
    Registrar(const char* name, std::function<void()> fn) { cases().push_back({name, std::move(fn)}); }
};

template <class T>
std::string show(const std::vector<T>& v) {
    std::ostringstream o;
    o.precision(17);
    o << "[";
    for (size_t i = 0; i < v.size() && i < 16; i++) o << (i ? ", " : "") << +v[i];
    if (v.size() > 16) o << ", ...";
    o << "]";
    return o.str();
}

inline void fail(const char* file, int line, const std::string& msg) {
    std::printf("    FAIL %s:%d: %s\n", file, line, msg.c_str());
    failures()++;
}

template <class A, class B>
bool roughly_eq(const std::vector<A>& a, const std::vector<B>& b, double tol) {
    if (a.size() != b.size()) return false;
    for (size_t i = 0; i < a.size(); i++)
        if (!(std::fabs(static_cast<double>(a[i]) - static_cast<double>(b[i])) < tol)) return false;
    return true;
}

// Runs every registered case whose name contains `filter` (all when empty).
inline int run(int argc, char** argv) {
    std::string filter = argc > 1 ? argv[1] : "";
    int ran = 0;
    for (auto& c : cases()) {
        if (!filter.empty() && c.name.find(filter) == std::string::npos) continue;
        std::printf("[ RUN  ] %s\n", c.name.c_str());
        std::fflush(stdout);
        int before = failures();
        try {
            c.fn();
        } catch (const std::exception& e) {
            fail("<exception>", 0, std::string("uncaught: ") + e.what());
        }
        std::printf("[ %s ] %s\n", failures() == before ? " OK " : "FAIL", c.name.c_str());
        std::fflush(stdout);
        ran++;
    }
    std::printf("%d case(s), %d failure(s)\n", ran, failures());
    return failures() ? 1 : 0;
}

}  // namespace check

#define TEST_CASE(name)                                            \
    static void name();                                            \
    static check::Registrar reg_##name(#name, name);               \
    static void name()

#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) check::fail(__FILE__, __LINE__, "CHECK(" #cond ")");        \
    } while (0)

#define CHECK_EQ(a, b)                                                                           \
    do {                                                                                         \
        auto va__ = (a);                                                                         \
        auto vb__ = (b);                                                                         \
        if (!(va__ == vb__)) {                                                                   \
            std::ostringstream o__;                                                              \
            o__.precision(17);                                                                   \
            o__ << "CHECK_EQ(" #a ", " #b "): " << va__ << " vs " << vb__;                      \
            check::fail(__FILE__, __LINE__, o__.str());                                          \
        }                                                                                        \
    } while (0)

#define CHECK_VEC_EQ(a, b)                                                                       \
    do {                                                                                         \
        auto va__ = (a);                                                                         \
        decltype(va__) vb__ = b;                                                                 \
        if (!(va__ == vb__))                                                                     \
            check::fail(__FILE__, __LINE__, "CHECK_VEC_EQ(" #a "): " + check::show(va__) + " vs " + check::show(vb__)); \
    } while (0)

#define CHECK_ROUGHLY(a, b, tol)                                                                 \
    do {                                                                                         \
        auto va__ = (a);                                                                         \
        std::vector<double> vb__ = b;                                                            \
        if (!check::roughly_eq(va__, vb__, tol))                                                 \
            check::fail(__FILE__, __LINE__, "CHECK_ROUGHLY(" #a "): " + check::show(va__) + " vs " + check::show(vb__)); \
    } while (0)

#define CHECK_THROWS_KIND(expr, KIND)                                                            \
    do {                                                                                         \
        bool threw__ = false;                                                                    \
        try {                                                                                    \
            expr;                                                                                \
        } catch (const custos::Error& e__) {                                                     \
            threw__ = e__.kind == (KIND);                                                        \
            if (!threw__) check::fail(__FILE__, __LINE__, std::string("wrong error kind: ") + e__.what()); \
            threw__ = true;                                                                      \
        }                                                                                        \
        if (!threw__) check::fail(__FILE__, __LINE__, "expected " #KIND " from " #expr);         \
    } while (0)
