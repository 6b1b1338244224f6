// Expression IR for element-wise kernels.
//
// The text form is what custos' `ToCLSource` impls print for a `Combiner`
// tree (reference: src/two_way_ops/ops.rs, ops/unary.rs, ops/cmps.rs,
// resolve.rs:131-141, to_cl_source.rs:7-11) and what
// `operations_to_fused_src` prints for a fused chain (src/devices/fusing.rs:4-19).
// It is parsed into a small DAG, hashed structurally, and emitted as typed
// HIP C in SSA form with one statement (= one rounding) per node.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace custos_hip {

enum class Op : uint8_t {
    Var,
    Const,
    // binary
    Add,
    Sub,
    Mul,
    Div,
    Pow,
    Min,
    Max,
    GEq,
    LEq,
    Eq,
    // unary
    Sin,
    Cos,
    Tan,
    Tanh,
    Exp,
    Ln,
    Abs,
    Neg,
    Sqrt,
};

bool op_is_binary(Op op);
bool op_is_unary(Op op);

struct Node {
    Op op = Op::Const;
    int a = -1;       // operand node index
    int b = -1;       // second operand node index (binary ops)
    int var = 0;      // Op::Var: operand index
    std::string lit;  // Op::Const: literal text as given
};

// Nodes are stored in evaluation order; operands always precede their user.
struct Expr {
    std::vector<Node> nodes;
    int root = -1;
    int n_vars = 0;
};

// Element types; numeric values equal `custos_hip_dtype`.
enum class DType : int32_t {
    F32 = 0,
    F64 = 1,
    I32 = 2,
    I64 = 3,
    F16 = 4,
    BF16 = 5,
    U8 = 6,
    I8 = 7,
    I16 = 8,
    U16 = 9,
    U32 = 10,
    U64 = 11,
    F16_PERNODE = 12,   // f16 storage, every node rounded to f16
    BF16_PERNODE = 13,  // bf16 storage, every node rounded to bf16
};

bool dtype_valid(int32_t v);
size_t dtype_size(DType t);
bool dtype_is_float(DType t);
bool dtype_is_signed(DType t);
bool dtype_rounds_per_node(DType t);  // 16-bit float whose every node is rounded to the storage type
const char* dtype_storage_c(DType t);  // C type of an element in memory
const char* dtype_compute_c(DType t);  // C type the nodes are evaluated in

struct ParseError {
    int code = 0;  // a custos_hip_status value, 0 = ok
    std::string message;
};

// Parses either one expression or a statement list "m = e;\n m = e;\n" in which
// `m` must be markers[0] and every statement reads the previous one's value.
bool parse_expr(const std::string& src, const std::vector<std::string>& markers, Expr* out,
                ParseError* err);

// Which literals of an expression are launch parameters.  A closure like `|x| x.mul(lr)`
// prints a new text for every value of `lr` (src/two_way_ops/resolve.rs:131-141); compiled
// in, every value would be a kernel of its own.  In the shared form of a kernel a literal
// is slot `slot[node]` of a block of scalars the kernel takes by value, and kernels that
// differ only in such values share their code.  Kept in the code even then: divisors of
// integer divisions (the compiler turns a division by a known value into a multiplication),
// and every literal of an expression with more than kMaxConstParams of them.  With
// `all_in_code` no literal is a parameter (the form compiled for one set of values).
constexpr int kMaxConstParams = 32;
struct ConstPlan {
    std::vector<int> slot;             // per node: parameter slot, or -1
    int n_params = 0;
    std::vector<unsigned char> bytes;  // the values, n_params elements of the compute type
};
bool plan_constants(const Expr& e, DType dtype, bool all_in_code, ConstPlan* plan, ParseError* err);

// Re-prints a tree in the reference's ToCLSource format (literals as given; with a plan,
// parameters print as c0, c1, ...).
std::string to_cl_source(const Expr& e, const std::vector<std::string>& markers, const ConstPlan* plan = nullptr);

// Structural 64-bit hash: node kinds, operand wiring, which literals are parameters, and
// the *values* of the literals that stay in the code after conversion to the element type
// ("2", "2.0" and "2.00" hash alike).
// `code_literals` (optional) receives those values' bits in node order.
bool hash_expr(const Expr& e, DType dtype, const ConstPlan& plan, uint64_t* hash, ParseError* err,
               std::vector<uint64_t>* code_literals = nullptr);

// Emits the body of `custos_expr`: SSA statements over v0..v{n-1} of the
// compute type (parameters read `kc.c[slot]`) and a final `return`.
bool emit_expr_body(const Expr& e, DType dtype, const ConstPlan& plan, std::string* out, ParseError* err);

uint64_t fnv1a64(const void* data, size_t n, uint64_t seed = 0xcbf29ce484222325ull);

}  // namespace custos_hip
