#include "expr.hpp"

#include <cctype>
#include <cerrno>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "../../include/custos_hip.h"

namespace custos_hip {

bool op_is_binary(Op op) { return op >= Op::Add && op <= Op::Eq; }
bool op_is_unary(Op op) { return op >= Op::Sin && op <= Op::Sqrt; }

bool dtype_valid(int32_t v) { return v >= 0 && v <= static_cast<int32_t>(DType::BF16_PERNODE); }

bool dtype_rounds_per_node(DType t) { return t == DType::F16_PERNODE || t == DType::BF16_PERNODE; }

size_t dtype_size(DType t) {
    switch (t) {
        case DType::F64:
        case DType::I64:
        case DType::U64: return 8;
        case DType::F32:
        case DType::I32:
        case DType::U32: return 4;
        case DType::F16:
        case DType::BF16:
        case DType::F16_PERNODE:
        case DType::BF16_PERNODE:
        case DType::I16:
        case DType::U16: return 2;
        default: return 1;
    }
}

bool dtype_is_float(DType t) {
    return t == DType::F32 || t == DType::F64 || t == DType::F16 || t == DType::BF16 || dtype_rounds_per_node(t);
}

bool dtype_is_signed(DType t) {
    return t == DType::I8 || t == DType::I16 || t == DType::I32 || t == DType::I64 ||
           dtype_is_float(t);
}

const char* dtype_storage_c(DType t) {
    switch (t) {
        case DType::F32: return "float";
        case DType::F64: return "double";
        case DType::I32: return "int";
        case DType::I64: return "long long";
        case DType::F16:
        case DType::F16_PERNODE: return "_Float16";
        case DType::BF16:
        case DType::BF16_PERNODE: return "unsigned short";
        case DType::U8: return "unsigned char";
        case DType::I8: return "signed char";
        case DType::I16: return "short";
        case DType::U16: return "unsigned short";
        case DType::U32: return "unsigned int";
        case DType::U64: return "unsigned long long";
    }
    return "float";
}

const char* dtype_compute_c(DType t) {
    if (t == DType::F16 || t == DType::BF16 || dtype_rounds_per_node(t)) return "float";
    return dtype_storage_c(t);
}

uint64_t fnv1a64(const void* data, size_t n, uint64_t h) {
    const unsigned char* p = static_cast<const unsigned char*>(data);
    for (size_t i = 0; i < n; i++) {
        h ^= p[i];
        h *= 0x100000001b3ull;
    }
    return h;
}

// ---------------------------------------------------------------------------
// parser
// ---------------------------------------------------------------------------

namespace {

struct Parser {
    const std::string& s;
    const std::vector<std::string>& markers;
    size_t pos = 0;
    Expr* e;
    ParseError* err;
    // Node that the first marker resolves to (the previous statement's value
    // inside a fused statement list), or -1 for a plain Var leaf.
    int bound0 = -1;
    std::vector<int> var_node;  // cache: one Var node per operand

    Parser(const std::string& src, const std::vector<std::string>& m, Expr* out, ParseError* er)
        : s(src), markers(m), e(out), err(er), var_node(m.size(), -1) {}

    bool fail(int code, const std::string& msg) {
        if (err && err->code == 0) {
            err->code = code;
            err->message = msg + " (at offset " + std::to_string(pos) + " of \"" + s + "\")";
        }
        return false;
    }

    void skip_ws() {
        while (pos < s.size() && std::isspace(static_cast<unsigned char>(s[pos]))) pos++;
    }

    bool at_end() {
        skip_ws();
        return pos >= s.size();
    }

    int add_node(const Node& n) {
        e->nodes.push_back(n);
        return static_cast<int>(e->nodes.size()) - 1;
    }

    int var(int k) {
        if (k == 0 && bound0 >= 0) return bound0;
        if (var_node[k] < 0) {
            Node n;
            n.op = Op::Var;
            n.var = k;
            var_node[k] = add_node(n);
        }
        return var_node[k];
    }

    static bool ident_start(char c) { return std::isalpha(static_cast<unsigned char>(c)) || c == '_'; }
    static bool ident_char(char c) { return std::isalnum(static_cast<unsigned char>(c)) || c == '_'; }

    // identifier, optionally followed by one bracket group: x, var_x, lhs[idx]
    std::string read_name() {
        size_t start = pos;
        while (pos < s.size() && ident_char(s[pos])) pos++;
        if (pos < s.size() && s[pos] == '[') {
            size_t close = s.find(']', pos);
            if (close != std::string::npos) pos = close + 1;
        }
        return s.substr(start, pos - start);
    }

    bool read_number(std::string* lit) {
        size_t start = pos;
        if (pos < s.size() && (s[pos] == '-' || s[pos] == '+')) pos++;
        if (s.compare(pos, 3, "inf") == 0 || s.compare(pos, 3, "NaN") == 0 ||
            s.compare(pos, 3, "nan") == 0) {
            pos += 3;
            *lit = s.substr(start, pos - start);
            return true;
        }
        size_t digits = 0;
        while (pos < s.size() && std::isdigit(static_cast<unsigned char>(s[pos]))) pos++, digits++;
        if (pos < s.size() && s[pos] == '.') {
            pos++;
            while (pos < s.size() && std::isdigit(static_cast<unsigned char>(s[pos]))) pos++, digits++;
        }
        if (digits == 0) {
            pos = start;
            return false;
        }
        if (pos < s.size() && (s[pos] == 'e' || s[pos] == 'E')) {
            size_t save = pos;
            pos++;
            if (pos < s.size() && (s[pos] == '-' || s[pos] == '+')) pos++;
            size_t ed = 0;
            while (pos < s.size() && std::isdigit(static_cast<unsigned char>(s[pos]))) pos++, ed++;
            if (ed == 0) pos = save;
        }
        // C suffixes a caller may have typed by hand ("1.0f")
        if (pos < s.size() && (s[pos] == 'f' || s[pos] == 'F')) pos++;
        *lit = s.substr(start, pos - start);
        if (!lit->empty() && (lit->back() == 'f' || lit->back() == 'F')) lit->pop_back();
        return true;
    }

    bool expect(char c) {
        skip_ws();
        if (pos < s.size() && s[pos] == c) {
            pos++;
            return true;
        }
        return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, std::string("expected '") + c + "'");
    }

    bool parse(int* out, int depth) {
        if (depth > 256) return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "expression nested too deeply");
        skip_ws();
        if (pos >= s.size()) return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "unexpected end of expression");
        char c = s[pos];

        if (c == '(') {
            pos++;
            int lhs = -1;
            if (!parse(&lhs, depth + 1)) return false;
            skip_ws();
            if (pos < s.size() && s[pos] == ')') {  // plain parentheses
                pos++;
                *out = lhs;
                return true;
            }
            Op op;
            if (s.compare(pos, 2, ">=") == 0) op = Op::GEq, pos += 2;
            else if (s.compare(pos, 2, "<=") == 0) op = Op::LEq, pos += 2;
            else if (s.compare(pos, 2, "==") == 0) op = Op::Eq, pos += 2;
            else if (s[pos] == '+') op = Op::Add, pos++;
            else if (s[pos] == '-') op = Op::Sub, pos++;
            else if (s[pos] == '*') op = Op::Mul, pos++;
            else if (s[pos] == '/') op = Op::Div, pos++;
            else return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "expected a binary operator");
            int rhs = -1;
            if (!parse(&rhs, depth + 1)) return false;
            if (!expect(')')) return false;
            Node n;
            n.op = op;
            n.a = lhs;
            n.b = rhs;
            *out = add_node(n);
            return true;
        }

        if (c == '-') {
            size_t look = pos + 1;
            while (look < s.size() && s[look] == ' ') look++;
            if (look < s.size() && s[look] == '(') {  // "-(e)": Neg
                pos = look + 1;
                int inner = -1;
                if (!parse(&inner, depth + 1)) return false;
                if (!expect(')')) return false;
                Node n;
                n.op = Op::Neg;
                n.a = inner;
                *out = add_node(n);
                return true;
            }
        }

        if (c == '-' || c == '+' || c == '.' || std::isdigit(static_cast<unsigned char>(c))) {
            Node n;
            n.op = Op::Const;
            if (!read_number(&n.lit)) return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "malformed number");
            *out = add_node(n);
            return true;
        }

        if (ident_start(c)) {
            size_t save = pos;
            std::string name = read_name();
            // markers win over function names and over inf/NaN
            for (size_t k = 0; k < markers.size(); k++) {
                if (markers[k] == name) {
                    *out = var(static_cast<int>(k));
                    return true;
                }
            }
            if (name == "inf" || name == "NaN" || name == "nan") {
                Node n;
                n.op = Op::Const;
                n.lit = name;
                *out = add_node(n);
                return true;
            }
            skip_ws();
            if (pos < s.size() && s[pos] == '(') {
                struct Fn {
                    const char* name;
                    Op op;
                    int arity;
                };
                static const Fn fns[] = {
                    {"exp", Op::Exp, 1},   {"sin", Op::Sin, 1},   {"cos", Op::Cos, 1},
                    {"tan", Op::Tan, 1},   {"tanh", Op::Tanh, 1}, {"log", Op::Ln, 1},
                    {"abs", Op::Abs, 1},   {"sqrt", Op::Sqrt, 1}, {"pow", Op::Pow, 2},
                    {"min", Op::Min, 2},   {"max", Op::Max, 2},
                };
                for (const Fn& f : fns) {
                    if (name != f.name) continue;
                    pos++;  // '('
                    Node n;
                    n.op = f.op;
                    if (!parse(&n.a, depth + 1)) return false;
                    if (f.arity == 2) {
                        if (!expect(',')) return false;
                        if (!parse(&n.b, depth + 1)) return false;
                    }
                    if (!expect(')')) return false;
                    *out = add_node(n);
                    return true;
                }
                pos = save;
                return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "unknown function '" + name + "'");
            }
            pos = save;
            return fail(CUSTOS_HIP_ERR_EXPR_UNKNOWN_MARKER, "unknown marker '" + name + "'");
        }

        return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, std::string("unexpected character '") + c + "'");
    }

    // "name = expr ;" ?  (a single '=', not "==")
    bool looks_like_statement() {
        size_t p = pos;
        while (p < s.size() && std::isspace(static_cast<unsigned char>(s[p]))) p++;
        if (p >= s.size() || !ident_start(s[p])) return false;
        while (p < s.size() && ident_char(s[p])) p++;
        if (p < s.size() && s[p] == '[') {
            size_t close = s.find(']', p);
            if (close == std::string::npos) return false;
            p = close + 1;
        }
        while (p < s.size() && std::isspace(static_cast<unsigned char>(s[p]))) p++;
        return p + 1 < s.size() && s[p] == '=' && s[p + 1] != '=';
    }

    bool run() {
        if (markers.empty() || markers.size() > 4)
            return fail(CUSTOS_HIP_ERR_INVALID_ARGUMENT, "1 to 4 markers are required");
        for (size_t i = 0; i < markers.size(); i++)
            for (size_t j = i + 1; j < markers.size(); j++)
                if (markers[i] == markers[j])
                    return fail(CUSTOS_HIP_ERR_INVALID_ARGUMENT, "markers must be distinct");
        e->nodes.clear();
        e->n_vars = static_cast<int>(markers.size());
        if (at_end()) return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "empty expression");

        if (looks_like_statement()) {
            int cur = -1;
            while (!at_end()) {
                skip_ws();
                std::string target = read_name();
                if (target != markers[0])
                    return fail(CUSTOS_HIP_ERR_EXPR_UNKNOWN_MARKER,
                                "fused statements must assign the first marker, got '" + target + "'");
                if (!expect('=')) return false;
                bound0 = cur;
                int value;
                if (!parse(&value, 0)) return false;
                if (!expect(';')) return false;
                cur = value;
            }
            e->root = cur;
        } else {
            int value;
            if (!parse(&value, 0)) return false;
            if (!at_end()) return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "trailing characters");
            e->root = value;
        }
        // an expression may be just the marker: make sure the node exists
        if (e->root < 0) return fail(CUSTOS_HIP_ERR_EXPR_SYNTAX, "empty expression");
        return true;
    }
};

// ---------------------------------------------------------------------------
// literals
// ---------------------------------------------------------------------------

struct Literal {
    bool is_nan = false;
    double f = 0.0;        // float dtypes (already rounded to f32 where the compute type is float)
    long long i = 0;       // signed integer dtypes
    unsigned long long u = 0;
};

bool literal_special(const std::string& lit, double* v) {
    std::string t = lit;
    bool neg = false;
    if (!t.empty() && (t[0] == '-' || t[0] == '+')) {
        neg = t[0] == '-';
        t = t.substr(1);
    }
    if (t == "inf") {
        *v = neg ? -INFINITY : INFINITY;
        return true;
    }
    if (t == "NaN" || t == "nan") {
        *v = NAN;
        return true;
    }
    return false;
}

bool convert_literal(const std::string& lit, DType dtype, Literal* out, ParseError* err) {
    auto fail = [&](const std::string& m) {
        if (err && err->code == 0) {
            err->code = CUSTOS_HIP_ERR_EXPR_UNSUPPORTED;
            err->message = m;
        }
        return false;
    };
    double special;
    if (literal_special(lit, &special)) {
        if (!dtype_is_float(dtype)) return fail("literal '" + lit + "' has no integer value");
        out->is_nan = std::isnan(special);
        out->f = special;
        return true;
    }
    const char* begin = lit.c_str();
    char* end = nullptr;
    errno = 0;
    if (dtype == DType::F64) {
        out->f = std::strtod(begin, &end);
        return *end == '\0' || fail("malformed literal '" + lit + "'");
    }
    if (dtype_is_float(dtype)) {
        // one correctly rounded conversion to f32: the value rustc gives the literal
        out->f = static_cast<double>(std::strtof(begin, &end));
        return *end == '\0' || fail("malformed literal '" + lit + "'");
    }
    bool integral_text = lit.find_first_of(".eE") == std::string::npos;
    if (integral_text) {
        if (dtype_is_signed(dtype)) {
            out->i = std::strtoll(begin, &end, 10);
            out->u = static_cast<unsigned long long>(out->i);
        } else {
            if (lit[0] == '-') {
                out->i = std::strtoll(begin, &end, 10);
                out->u = static_cast<unsigned long long>(out->i);
            } else {
                out->u = std::strtoull(begin, &end, 10);
                out->i = static_cast<long long>(out->u);
            }
        }
        if (*end != '\0' || errno == ERANGE) return fail("malformed integer literal '" + lit + "'");
        return true;
    }
    double d = std::strtod(begin, &end);
    if (*end != '\0' || std::floor(d) != d || std::fabs(d) > 9.0e15)
        return fail("literal '" + lit + "' is not an integer but the element type is");
    out->i = static_cast<long long>(d);
    out->u = static_cast<unsigned long long>(out->i);
    return true;
}

std::string literal_c(const Literal& l, DType dtype) {
    char buf[96];
    if (dtype_is_float(dtype)) {
        bool dbl = dtype == DType::F64;
        if (l.is_nan) return dbl ? "__builtin_nan(\"\")" : "__builtin_nanf(\"\")";
        if (std::isinf(l.f)) {
            std::string v = dbl ? "__builtin_huge_val()" : "__builtin_huge_valf()";
            return l.f < 0 ? "(-" + v + ")" : v;
        }
        std::snprintf(buf, sizeof buf, dbl ? "%a" : "%af", l.f);
        return buf;
    }
    if (dtype_is_signed(dtype)) {
        if (l.i == INT64_MIN) return std::string("((") + dtype_compute_c(dtype) + ")(-9223372036854775807LL - 1))";
        std::snprintf(buf, sizeof buf, "((%s)%lldLL)", dtype_compute_c(dtype), l.i);
    } else {
        std::snprintf(buf, sizeof buf, "((%s)%lluULL)", dtype_compute_c(dtype), l.u);
    }
    return buf;
}

}  // namespace

bool parse_expr(const std::string& src, const std::vector<std::string>& markers, Expr* out,
                ParseError* err) {
    if (err) *err = ParseError{};
    Parser p(src, markers, out, err);
    return p.run();
}

// ---------------------------------------------------------------------------
// printing in the reference's format
// ---------------------------------------------------------------------------

static void print_node(const Expr& e, int idx, const std::vector<std::string>& markers, const ConstPlan* plan,
                       std::string* out) {
    const Node& n = e.nodes[idx];
    auto rec = [&](int k) { print_node(e, k, markers, plan, out); };
    auto infix = [&](const char* op) {
        *out += "(";
        rec(n.a);
        *out += op;
        rec(n.b);
        *out += ")";
    };
    auto call1 = [&](const char* name) {
        *out += name;
        *out += "(";
        rec(n.a);
        *out += ")";
    };
    auto call2 = [&](const char* name) {
        *out += name;
        *out += "(";
        rec(n.a);
        *out += ", ";
        rec(n.b);
        *out += ")";
    };
    switch (n.op) {
        case Op::Var: *out += markers[n.var]; break;
        case Op::Const:
            if (plan && plan->slot[static_cast<size_t>(idx)] >= 0) *out += "c" + std::to_string(plan->slot[static_cast<size_t>(idx)]);
            else *out += n.lit;
            break;
        case Op::Add: infix(" + "); break;
        case Op::Sub: infix(" - "); break;
        case Op::Mul: infix(" * "); break;
        case Op::Div: infix(" / "); break;
        case Op::GEq: infix(" >= "); break;
        case Op::LEq: infix(" <= "); break;
        case Op::Eq: infix(" == "); break;
        case Op::Pow: call2("pow"); break;
        case Op::Min: call2("min"); break;
        case Op::Max: call2("max"); break;
        case Op::Sin: call1("sin"); break;
        case Op::Cos: call1("cos"); break;
        case Op::Tan: call1("tan"); break;
        case Op::Tanh: call1("tanh"); break;
        case Op::Exp: call1("exp"); break;
        case Op::Ln: call1("log"); break;
        case Op::Abs: call1("abs"); break;
        case Op::Sqrt: call1("sqrt"); break;
        case Op::Neg: call1("-"); break;
    }
}

std::string to_cl_source(const Expr& e, const std::vector<std::string>& markers, const ConstPlan* plan) {
    std::string out;
    if (e.root >= 0) print_node(e, e.root, markers, plan, &out);
    return out;
}

// ---------------------------------------------------------------------------
// literals as launch parameters
// ---------------------------------------------------------------------------

namespace {

// The bytes of a literal in the compute type, as the compiler would materialise `literal_c`.
void append_literal_bytes(const Literal& l, DType dtype, std::vector<unsigned char>* out) {
    unsigned char raw[8];
    size_t n;
    if (dtype == DType::F64) {
        uint64_t bits;
        std::memcpy(&bits, &l.f, 8);
        if (l.is_nan) bits = 0x7ff8000000000000ull;
        std::memcpy(raw, &bits, n = 8);
    } else if (dtype_is_float(dtype)) {
        const float f = static_cast<float>(l.f);  // exact: already rounded to f32
        uint32_t bits;
        std::memcpy(&bits, &f, 4);
        if (l.is_nan) bits = 0x7fc00000u;
        std::memcpy(raw, &bits, n = 4);
    } else {
        const uint64_t v = dtype_is_signed(dtype) ? static_cast<uint64_t>(l.i) : l.u;
        std::memcpy(raw, &v, 8);  // little endian: the low bytes are the narrower value
        n = dtype_size(dtype);
    }
    out->insert(out->end(), raw, raw + n);
}

}  // namespace

bool plan_constants(const Expr& e, DType dtype, bool all_in_code, ConstPlan* plan, ParseError* err) {
    plan->slot.assign(e.nodes.size(), -1);
    plan->n_params = 0;
    plan->bytes.clear();
    if (all_in_code) return true;
    std::vector<bool> in_code(e.nodes.size(), false);
    if (!dtype_is_float(dtype))
        for (const Node& n : e.nodes)
            if (n.op == Op::Div && n.b >= 0 && e.nodes[static_cast<size_t>(n.b)].op == Op::Const) in_code[static_cast<size_t>(n.b)] = true;
    int wanted = 0;
    for (size_t i = 0; i < e.nodes.size(); i++) wanted += e.nodes[i].op == Op::Const && !in_code[i];
    if (wanted > kMaxConstParams) return true;
    for (size_t i = 0; i < e.nodes.size(); i++) {
        if (e.nodes[i].op != Op::Const || in_code[i]) continue;
        Literal l;
        if (!convert_literal(e.nodes[i].lit, dtype, &l, err)) return false;
        plan->slot[i] = plan->n_params++;
        append_literal_bytes(l, dtype, &plan->bytes);
    }
    return true;
}

// ---------------------------------------------------------------------------
// hashing
// ---------------------------------------------------------------------------

bool hash_expr(const Expr& e, DType dtype, const ConstPlan& plan, uint64_t* hash, ParseError* err,
               std::vector<uint64_t>* code_literals) {
    uint64_t h = fnv1a64("custos-expr-v2", 14);
    int32_t head[3] = {static_cast<int32_t>(dtype), e.n_vars, e.root};
    h = fnv1a64(head, sizeof head, h);
    for (size_t i = 0; i < e.nodes.size(); i++) {
        const Node& n = e.nodes[i];
        int32_t rec[5] = {static_cast<int32_t>(n.op), n.a, n.b, n.var, plan.slot[i]};
        h = fnv1a64(rec, sizeof rec, h);
        if (n.op == Op::Const && plan.slot[i] < 0) {
            Literal l;
            if (!convert_literal(n.lit, dtype, &l, err)) return false;
            if (dtype_is_float(dtype)) {
                uint64_t bits;
                double v = l.is_nan ? NAN : l.f;
                std::memcpy(&bits, &v, 8);
                if (l.is_nan) bits = 0x7ff8000000000000ull;
                h = fnv1a64(&bits, 8, h);
                if (code_literals) code_literals->push_back(bits);
            } else {
                h = fnv1a64(&l.u, 8, h);
                if (code_literals) code_literals->push_back(l.u);
            }
        }
    }
    *hash = h;
    return true;
}

// ---------------------------------------------------------------------------
// HIP C emission
// ---------------------------------------------------------------------------

bool emit_expr_body(const Expr& e, DType dtype, const ConstPlan& plan, std::string* out, ParseError* err) {
    auto fail = [&](const std::string& m) {
        if (err && err->code == 0) {
            err->code = CUSTOS_HIP_ERR_EXPR_UNSUPPORTED;
            err->message = m;
        }
        return false;
    };
    const bool flt = dtype_is_float(dtype);
    const bool dbl = dtype == DType::F64;
    const std::string C = dtype_compute_c(dtype);
    auto t = [](int k) { return "t" + std::to_string(k); };
    auto mathfn = [&](const char* base) { return std::string(base) + (dbl ? "" : "f"); };
    // + - * : floats as written (one IEEE operation); integers wrap like Rust's
    // release arithmetic, so they are computed in an unsigned type that is at
    // least as wide as int (no promotion to a signed type, no signed overflow)
    // and cast back to the element type.
    const std::string U = dtype_size(dtype) == 8 ? "unsigned long long" : "unsigned int";
    auto arith = [&](const Node& n, const char* op) {
        if (flt) return "(" + C + ")(" + t(n.a) + op + t(n.b) + ")";
        return "(" + C + ")((" + U + ")" + t(n.a) + op + "(" + U + ")" + t(n.b) + ")";
    };

    std::string body;
    for (size_t i = 0; i < e.nodes.size(); i++) {
        const Node& n = e.nodes[i];
        std::string rhs;
        switch (n.op) {
            case Op::Var: rhs = "v" + std::to_string(n.var); break;
            case Op::Const: {
                if (plan.slot[i] >= 0) {
                    rhs = "kc.c[" + std::to_string(plan.slot[i]) + "]";
                    break;
                }
                Literal l;
                if (!convert_literal(n.lit, dtype, &l, err)) return false;
                rhs = literal_c(l, dtype);
                break;
            }
            case Op::Add: rhs = arith(n, " + "); break;
            case Op::Sub: rhs = arith(n, " - "); break;
            case Op::Mul: rhs = arith(n, " * "); break;
            case Op::Div: rhs = "(" + C + ")(" + t(n.a) + " / " + t(n.b) + ")"; break;
            case Op::Pow:
                if (!flt) return fail("pow is not defined for integer element types");
                rhs = mathfn("pow") + "(" + t(n.a) + ", " + t(n.b) + ")";
                break;
            // Number::min / Number::max: a select on < and > (src/number.rs:201-209),
            // not fmin/fmax: NaN and signed-zero behaviour differ.
            case Op::Min:
            case Op::Max: {
                const char* cmp = n.op == Op::Min ? " < " : " > ";
                // hipcc turns the select into v_min / v_max where it can prove that a NaN
                // cannot change the outcome (a constant second operand, operands that are
                // comparison results, ...).  For two zeros of different sign those return -0
                // (min) and +0 (max), the select returns the second operand.  So unless the
                // second operand is a literal for which both agree, it reaches the select
                // through custos_pick, and the compiler sees no min / max pattern.
                bool plain = !flt;
                const Node& second = e.nodes[static_cast<size_t>(n.b)];
                if (flt && second.op == Op::Const) {
                    Literal l;
                    if (!convert_literal(second.lit, dtype, &l, err)) return false;
                    const bool zero = !l.is_nan && l.f == 0.0;
                    const bool negative_zero = zero && std::signbit(l.f);
                    plain = plan.slot[static_cast<size_t>(n.b)] >= 0 || !zero ||
                            (n.op == Op::Min ? negative_zero : !negative_zero);
                }
                if (plain) rhs = "(" + t(n.a) + cmp + t(n.b) + ") ? " + t(n.a) + " : " + t(n.b);
                else rhs = "custos_pick(" + t(n.a) + cmp + t(n.b) + ", " + t(n.a) + ", " + t(n.b) + ")";
                break;
            }
            case Op::GEq: rhs = "(" + C + ")(" + t(n.a) + " >= " + t(n.b) + ")"; break;
            case Op::LEq: rhs = "(" + C + ")(" + t(n.a) + " <= " + t(n.b) + ")"; break;
            case Op::Eq: rhs = "(" + C + ")(" + t(n.a) + " == " + t(n.b) + ")"; break;
            case Op::Sin:
            case Op::Cos:
            case Op::Tan:
            case Op::Tanh:
            case Op::Exp:
            case Op::Ln:
            case Op::Sqrt: {
                if (!flt) return fail("transcendental nodes are not defined for integer element types");
                const char* name = n.op == Op::Sin    ? "custos_sin"
                                   : n.op == Op::Cos  ? "custos_cos"
                                   : n.op == Op::Tan  ? "custos_tan"
                                   : n.op == Op::Tanh ? "custos_tanh"
                                   : n.op == Op::Exp  ? "custos_exp"
                                   : n.op == Op::Ln   ? "custos_log"
                                                      : "custos_sqrt";
                rhs = std::string(name) + "(" + t(n.a) + ")";
                break;
            }
            case Op::Abs:
                if (flt) rhs = mathfn("fabs") + "(" + t(n.a) + ")";
                else if (dtype_is_signed(dtype))
                    rhs = "(" + t(n.a) + " < 0) ? (" + C + ")((" + U + ")0 - (" + U + ")" + t(n.a) + ") : " + t(n.a);
                else rhs = t(n.a);
                break;
            case Op::Neg:
                if (flt) rhs = "-" + t(n.a);
                else rhs = "(" + C + ")((" + U + ")0 - (" + U + ")" + t(n.a) + ")";
                break;
        }
        // Per-node rounding (what `half`'s f16 / bf16 arithmetic does, src/number.rs:487-676):
        // every node that computes is rounded to the storage type.  Selects, comparisons,
        // abs and neg are exact in the storage type already.
        const bool computes = n.op == Op::Const || n.op == Op::Add || n.op == Op::Sub || n.op == Op::Mul ||
                              n.op == Op::Div || n.op == Op::Pow || (op_is_unary(n.op) && n.op != Op::Abs && n.op != Op::Neg);
        if (dtype_rounds_per_node(dtype) && computes) rhs = "custos_round(" + rhs + ")";
        body += "    const " + C + " " + t(static_cast<int>(i)) + " = " + rhs + ";\n";
    }
    body += "    return " + t(e.root) + ";\n";
    *out = body;
    return true;
}

}  // namespace custos_hip
