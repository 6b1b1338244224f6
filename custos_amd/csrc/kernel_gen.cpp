#include "kernel_gen.hpp"

#include <algorithm>
#include <cstdio>

#include "../../include/custos_hip.h"

namespace custos_hip {

Tuning normalize_tuning(int block_threads, int unroll, int blocks_per_cu, int nontemporal, int direction) {
    Tuning t;
    if (block_threads > 0) {
        block_threads = std::max(64, std::min(1024, block_threads));
        t.block_threads = (block_threads / 64) * 64;
    }
    if (unroll > 0) t.unroll = std::min(16, unroll);
    t.blocks_per_cu = blocks_per_cu > 0 ? std::min(64, blocks_per_cu) : 0;
    if (nontemporal != 0) t.nontemporal = nontemporal < 0 ? 0 : (nontemporal & (3 | kStoresWriteThrough));
    if (direction == 1 || direction == 2) t.direction = direction;
    return t;
}

// Launch shape by the bytes a launch touches, measured on MI355X (8 x 4 MiB L2,
// 256 MiB memory-side cache, HBM3E) over buffers of random data (buffers of
// zeros run 5-10 % faster and hide differences).  Abbreviations: cache policy T
// (all temporal), N (loads and stores non-temporal), W (non-temporal loads,
// temporal stores written through to device scope at once); tiles always first
// to last (f) or every launch the other way round (a).  Two vectors per thread
// throughout (one was never more than 1 % ahead with W).  GB/s on the
// algorithmic bytes.
//
// While the launch and the launches just before it touch no more than 32 MiB
// together (what the eight L2s hold): T.  The in-place gradient kernel repeated
// over 28 MiB: T 9144, W 7569.  A launch that would fit the L2s after launches
// that do not leave them to it streams like a large one (tanh forward, 20 MiB,
// + backward, 30 MiB, over 40 MiB of arrays: W 6073, T 5227; three merged
// launches of 48, 48 and 32 MiB in a replayed graph: 23.6 us with W or T
// throughout, 25.1 us with W, W, T).
//
// Above: W.  Already just above the L2s, where the working set still fits the
// memory-side cache, T loses to it (1R+1W repeated over 48 MiB: T 6012, W 8951;
// 2R+1W 7146 / 6307; gradient kernel 7201 / 6406; tanh forward + backward over
// 40 MiB 6073 / 5227): temporal accesses thrash the L2s and leave dirty lines to
// be evicted later, W is served by the memory-side cache.  Loads pass the caches by; the stores stay in the memory-side cache,
// so the 256 MiB written last are still there when the next launch over the same
// buffers starts at that end (direction a, above 256 MiB) and a consumer finds
// them; writing them through at once instead of leaving them dirty in an L2
// smooths the write traffic (worth 2-5 % by itself).  The same launch repeated,
// W / N / T:
//   1R+1W   128 MiB 7382 / 6589 / 6803   512 MiB 7395 / 6510 / 6009   1 GiB 7513 / 6536 / 6124
//           2 GiB   6987 / 6418 / 6169
//   2R+1W   512 MiB 7345 / 6583 / 5840   1 GiB 7085 / 6521 / 5917
//   3R+1W (gradient kernel, in place)    768 MiB 7616 / 6257 / 5492   2 GiB 6756 / 6355 / 5725
// Chains (a launch reads what the launch before it wrote; eager cycle over three
// arrays, by the bytes one launch touches): 128 MiB W 6948, T 6779; 256 MiB 7241 /
// 5653; 512 MiB 7279 / 5993.  A rule that kept T for chains whose working set fits
// the memory-side cache lost 1-3 % to W wherever it applied and is gone, as is one
// that kept single operands temporal.
//
// Exception: a launch through two pointers of 256-768 MiB that is not part of a
// chain takes N when the launches before it touched other memory as well (its
// working set is larger than the launch).  Repeated alone it is slower that way
// (512 MiB: 6510 against 7395) and keeps W; but as the forward kernel of tanh
// forward + backward over 2^26 elements its temporal stores push out what the
// backward kernel keeps: 7090 on 24 bytes per element with N for the forward
// kernel, 6200 with W.
//
// Two refinements, both about launches whose traffic the memory-side cache cannot help:
//
// A launch that touches nothing the launch before it wrote (an eager chain's first launch over
// a fresh input, a loop whose every call gets another output block, anything that streams through
// more memory than the caches hold) runs as one-wavefront workgroups with one vector per thread
// once it touches more than 32 MiB.  Distinct (x, out) pairs over 2 GiB in turn, 1R+1W, GB/s with
// 128 x 2 / 64 x 1: 32 MiB launches 4629 / 4795, 64 MiB 5407 / 5720, 128 MiB 5977 / 6283, 256 MiB
// 6350 / 6625, 1 GiB 6449 / 6759; every kernel tried (copy, sin, tanh, exp, the f16 chain) goes
// from 6350-6420 to 6740-6800 that way.  The same launch repeated over the same buffers, which
// starts on what the cache still holds, loses 2-13 % with that shape and keeps 128 x 2.
//
// A launch that writes through at least two pointers more than it reads through (a joined chain
// that still stores its intermediates) takes temporal loads and non-temporal stores written
// through at once: what the cache keeps for the launch that comes back is then the input, which
// that launch reads, instead of outputs, which it only overwrites.  1R+3W over 2^28 f32: 5634 ->
// 6161-6310; 1R+5W 5436 -> 5885; over 2^26: 6749 -> 7230, 6141 -> 7196.  (With two inputs it is
// the other way round: 2R+2W over 2^26 7150 / 6362; and below 128 MiB touched the usual policy is
// ahead: 1R+3W over 64 MiB 8204 / 7779, 1R+5W over 96 MiB 7868 / 6714.)
LaunchShape preferred_shape(unsigned long long footprint_bytes, int n_operands, CacheHint hint,
                            unsigned long long working_set_bytes, bool revisits, int n_written, int keep_inputs) {
    constexpr unsigned long long MiB = 1ull << 20;
    // non-temporal loads with temporal stores that are written through at once / both non-temporal /
    // temporal loads with non-temporal stores that are written through at once
    constexpr int kLoads = 1 | kStoresWriteThrough, kBoth = 3, kStores = 2 | kStoresWriteThrough;
    const unsigned long long working_set = std::max(footprint_bytes, working_set_bytes);
    if (working_set <= kL2WorkingSet) return {2, 0, false, 0};
    LaunchShape shape{2, kLoads, footprint_bytes > 256 * MiB, 0};
    if (n_written >= n_operands - n_written + 2 && footprint_bytes >= 128 * MiB)
        shape.nontemporal = kStores;
    else if (footprint_bytes > 256 * MiB && n_operands < 3 && footprint_bytes < 768 * MiB && hint != CacheHint::Streams &&
             working_set > footprint_bytes)
        shape.nontemporal = kBoth;
    if (!revisits && footprint_bytes > kL2WorkingSet) shape.unroll = 1, shape.block = 64;
    // The same shape for a launch through three or more pointers over more than 768 MiB, whatever
    // came before it (x*a + y over 2^26..2^27 elements per operand: 7096 -> 7335 and 6921 -> 7322 GB/s;
    // the in-place gradient kernel 7214 -> 7477 and 6724 -> 6958; joined kernels over 2^28 elements:
    // 1R+2W 6170 -> 6680, 2R+2W 6260 -> 6750, 1R+3W 6180 -> 6360; tanh forward + gradient joined,
    // 3R+2W over 2^26: 7783 -> 8516 on 24 bytes per element).  A launch through two pointers keeps
    // 128 x 2 there (7500 against 6771), and up to 768 MiB the shapes are equal for all of them.
    if (n_operands >= 3 && footprint_bytes > 768 * MiB) shape.unroll = 1, shape.block = 64;
    // It touches nothing the launch before it wrote but reads, through the inputs `keep_inputs` names,
    // what that launch read as well (`y = f(x)` into another buffer every time, what
    // `out = device.apply_fn(&x, f)` in a loop does; the gradient launch behind the forward launch of
    // the same x, and the next forward launch behind it): the memory-side cache is worth more to
    // those inputs than to anything else the launch moves.  They are loaded with temporal accesses,
    // everything else streams past the cache, and the launch starts where the one before it ended.
    if (!revisits && keep_inputs != 0 && footprint_bytes > kL2WorkingSet) {
        shape.nontemporal = 3 | kStoresWriteThrough | (keep_inputs & kKeepInputMask) << kKeepInputShift;
        shape.alternate = footprint_bytes > 256 * MiB;
    }
    return shape;
}

std::vector<std::string> hiprtc_options(const std::string& arch) {
    return {
        "--offload-arch=" + arch,
        "-O3",
        "-std=c++17",
        // a*b+c must stay two roundings: the CPU device never fuses
        "-ffp-contract=off",
        // IEEE division and square root (bit-exact with the CPU device)
        "-fhip-fp32-correctly-rounded-divide-sqrt",
        // keep f32 arithmetic on the scalar-per-lane instructions
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        // No v_fma_mix*: hipcc folds `(_Float16)(a * b)` into v_fma_mixlo_f16 a, b, +0, and
        // adding +0 turns a product of -0 into +0 (the CPU device keeps the sign).  Costs
        // nothing measurable on the f16 chain; keeping the product apart from the rounding
        // with an empty asm instead cost 5 %.
        "-Xclang", "-target-feature", "-Xclang", "-fma-mix-insts",
        // No SLP vectorizer: without the packed f32 instructions the backend cannot select the
        // two-element f32 negation the vectorizer forms in front of a packed f32 -> f16
        // conversion ("Cannot select: v2f32 = bitcast", which ends the process); the kernels
        // are written in 16-byte vectors already and gain nothing from it.
        "-fno-slp-vectorize",
    };
}

namespace {

// Conversions between the storage and the compute type, and the math wrappers
// the emitted expression calls.
std::string prelude(DType dtype, int vec, int n_consts) {
    std::string s;
    s += "typedef unsigned long long u64;\n";
    s += std::string("typedef ") + dtype_storage_c(dtype) + " S;\n";
    s += std::string("typedef ") + dtype_compute_c(dtype) + " C;\n";
    s += "typedef S vec_t __attribute__((ext_vector_type(" + std::to_string(vec) + ")));\n";
    // The literals of the expression that are launch parameters: one block of scalars, an
    // argument by value of every entry point (it sits in the kernel argument segment, every
    // read of it is a scalar load).  KC_PARAM / KC_ARG thread it through the helper functions.
    if (n_consts > 0) {
        s += "struct CustosConsts { C c[" + std::to_string(n_consts) + "]; };\n";
        s += "#define CUSTOS_KC_ENTRY const CustosConsts kc,\n";
        s += "#define CUSTOS_KC_PARAM , const CustosConsts& kc\n";
        s += "#define CUSTOS_KC_ARG , kc\n";
    } else {
        s += "#define CUSTOS_KC_ENTRY\n#define CUSTOS_KC_PARAM\n#define CUSTOS_KC_ARG\n";
    }
    if (dtype == DType::BF16 || dtype == DType::BF16_PERNODE) {
        s += R"(static __device__ __forceinline__ C custos_load(S s) {
    return __builtin_bit_cast(float, (unsigned int)s << 16);
}
static __device__ __forceinline__ S custos_store(C c) {
    unsigned int x = __builtin_bit_cast(unsigned int, c);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (S)((x >> 16) | 0x0040u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (S)(x >> 16);
}
)";
    } else {
        s += "static __device__ __forceinline__ C custos_load(S s) { return (C)s; }\n";
        s += "static __device__ __forceinline__ S custos_store(C c) { return (S)c; }\n";
    }
    if (dtype_rounds_per_node(dtype))
        s += "static __device__ __forceinline__ C custos_round(C c) { return custos_load(custos_store(c)); }\n";
    // `first ? a : b` with b passed through an empty asm (no instruction) on its way into the
    // select, so that the compiler cannot turn it into v_min / v_max; see the min / max nodes
    // in emit_expr_body.  (The asm sits outside the conditional, else it becomes a branch.)
    if (dtype_is_float(dtype))
        s += "static __device__ __forceinline__ C custos_pick(bool first, C a, C b) {\n"
             "    __asm__(\"\" : \"+v\"(b));\n    return first ? a : b;\n}\n";
    if (dtype == DType::F64) {
        s += R"(static __device__ __forceinline__ double custos_sin(double a) { return sin(a); }
static __device__ __forceinline__ double custos_cos(double a) { return cos(a); }
static __device__ __forceinline__ double custos_tan(double a) { return tan(a); }
static __device__ __forceinline__ double custos_tanh(double a) { return tanh(a); }
static __device__ __forceinline__ double custos_exp(double a) { return exp(a); }
static __device__ __forceinline__ double custos_log(double a) { return log(a); }
static __device__ __forceinline__ double custos_sqrt(double a) { return sqrt(a); }
)";
    } else if (dtype_is_float(dtype)) {
        // 16-bit storage types: the result is rounded to 11 (f16) or 8 (bf16)
        // significant bits at the store, so exp may take the hardware exp2
        // directly: relative error <= |a| * 2^-24 (argument rounding) + 1 ulp,
        // below 5e-6 over the whole finite range, against a half-ulp of 2.4e-4
        // for f16.  The correctly-rounded-to-f32 path costs about 3x the ALU work
        // and makes the f16 chain ALU-bound instead of HBM-bound.  sin / cos /
        // tanh / log keep the full-precision routines: their results pass through
        // zero, where only a relative bound in f32 keeps the 16-bit result within
        // one ulp.
        // bf16 has f32's exponent range, and the hardware exp2 gives 0 where the result is an
        // f32 denormal (inputs below -87.3, which the reference's expf turns into bf16
        // denormals): there the exponent is raised by 64 and the result scaled back, a
        // multiplication that rounds into the denormal range correctly.
        if (dtype == DType::BF16 || dtype == DType::BF16_PERNODE)
            s += "static __device__ __forceinline__ float custos_exp(float a) {\n"
                 "    const float t = a * 0x1.715476p+0f;\n"
                 "    const bool tiny = t < -126.0f;\n"
                 "    return __builtin_amdgcn_exp2f(tiny ? t + 64.0f : t) * (tiny ? 0x1p-64f : 1.0f);\n}\n";
        else if (dtype == DType::F16 || dtype == DType::F16_PERNODE)
            s += "static __device__ __forceinline__ float custos_exp(float a) {\n"
                 "    return __builtin_amdgcn_exp2f(a * 0x1.715476p+0f);\n}\n";
        else
            s += "static __device__ __forceinline__ float custos_exp(float a) { return expf(a); }\n";
        s += R"(static __device__ __forceinline__ float custos_sin(float a) { return sinf(a); }
static __device__ __forceinline__ float custos_cos(float a) { return cosf(a); }
static __device__ __forceinline__ float custos_tan(float a) { return tanf(a); }
static __device__ __forceinline__ float custos_tanh(float a) { return tanhf(a); }
static __device__ __forceinline__ float custos_log(float a) { return logf(a); }
static __device__ __forceinline__ float custos_sqrt(float a) { return sqrtf(a); }
)";
    }
    return s;
}

std::string expr_fn(const KernelSpec& k, const std::string& body) {
    std::string s = "static __device__ __forceinline__ C custos_expr(";
    for (int i = 0; i < k.expr.n_vars; i++) {
        if (i) s += ", ";
        s += "const C v" + std::to_string(i);
    }
    s += " CUSTOS_KC_PARAM) {\n" + body + "}\n";
    return s;
}

// lhs_grad + (out_grad * d): product rounded, then the sum rounded
// (src/devices/cpu_stack_ops.rs:27-29); integers wrap.
std::string grad_fn(DType dtype) {
    if (dtype_rounds_per_node(dtype))
        return "static __device__ __forceinline__ C custos_grad(const C g, const C o, const C d) {\n"
               "    const C prod = custos_round(o * d);\n    const C sum = g + prod;\n    return sum;\n}\n";
    if (dtype_is_float(dtype))
        return "static __device__ __forceinline__ C custos_grad(const C g, const C o, const C d) {\n"
               "    const C prod = o * d;\n    const C sum = g + prod;\n    return sum;\n}\n";
    const char* U = dtype_size(dtype) == 8 ? "unsigned long long" : "unsigned int";
    return std::string("static __device__ __forceinline__ C custos_grad(const C g, const C o, const C d) {\n") +
           "    const C prod = (C)((" + U + ")o * (" + U + ")d);\n" +
           "    return (C)((" + U + ")g + (" + U + ")prod);\n}\n";
}

// The constant plan of one stage of a chain: its own slots, moved behind the parameters of the
// stages before it (`base`).
bool stage_plan(const ChainStage& stage, DType dtype, int base, ConstPlan* plan, ParseError* err) {
    if (stage.slot.empty()) return plan_constants(stage.expr, dtype, /*all_in_code=*/true, plan, err);
    if (stage.slot.size() != stage.expr.nodes.size()) {
        err->code = CUSTOS_HIP_ERR_INVALID_ARGUMENT;
        err->message = "malformed chain stage";
        return false;
    }
    plan->slot = stage.slot;
    for (int& s : plan->slot)
        if (s >= 0) s += base;
    plan->n_params = stage.n_params;
    plan->bytes.clear();
    return true;
}

// Text of the per-element function, the tile function and the entry points of one kernel
// (every translation unit holds the functions and ONE entry point: emit_kernel_source).  Operand naming inside a kernel: in0.. are the inputs, `out` the output; for a unary
// gradient 0 = lhs, 1 = lhs_grad (also the output), 2 = out_grad.
struct KernelText {
    const KernelSpec& k;
    const int n_in;    // inputs of the expression
    const int n_ops;   // values custos_elem takes
    const int n_ptrs;  // pointers per operand set (table row of a merged launch)
    const int const_words;  // 8-byte words of a table row that hold the literal parameters
    std::string params;     // pointer parameters of the single-launch entry point
    std::string vec_ptrs;   // declarations of the vector views of the operands
    std::string tile_args;  // the input views custos_tile takes
    std::string out_views;  // the output views custos_tile takes

    explicit KernelText(const KernelSpec& spec)
        : k(spec),
          n_in(spec.kind == Kind::Chain ? spec.n_ext : spec.expr.n_vars),
          n_ops(spec.kind == Kind::Apply ? spec.expr.n_vars : spec.kind == Kind::Chain ? spec.n_ext : 3),
          n_ptrs(kernel_pointers(spec)),
          const_words(static_cast<int>((spec.consts.bytes.size() + 7) / 8)),
          out_views("vout, ") {
        if (k.kind == Kind::Chain) {
            out_views.clear();
            for (int i = 0; i < n_in; i++) {
                const std::string id = std::to_string(i);
                params += "const S* in" + id + ", ";
                vec_ptrs += "    const vec_t* vin" + id + " = (const vec_t*)(in" + id + " + head);\n";
            }
            for (int j = 0; j < k.n_outs; j++) {
                const std::string id = std::to_string(j);
                params += std::string(j ? ", " : "") + "S* out" + id;
                vec_ptrs += "    vec_t* vout" + id + " = (vec_t*)(out" + id + " + head);\n";
                out_views += "vout" + id + ", ";
            }
        } else if (k.kind == Kind::Apply) {
            for (int i = 0; i < n_in; i++) {
                const std::string id = std::to_string(i);
                params += "const S* in" + id + ", ";
                vec_ptrs += "    const vec_t* vin" + id + " = (const vec_t*)(in" + id + " + head);\n";
            }
            params += "S* out";
            vec_ptrs += "    vec_t* vout = (vec_t*)(out + head);\n";
        } else {
            params = "const S* in0, S* out, const S* in2";
            vec_ptrs = "    const vec_t* vin0 = (const vec_t*)(in0 + head);\n"
                       "    const vec_t* vin2 = (const vec_t*)(in2 + head);\n"
                       "    vec_t* vout = (vec_t*)(out + head);\n"
                       "    const vec_t* vin1 = vout;\n"
                       "    const S* in1 = out;\n";
        }
        for (int i = 0; i < n_ops; i++) {
            if (k.kind == Kind::UnaryGrad && i == 1) continue;  // vin1 is vout
            tile_args += "vin" + std::to_string(i) + ", ";
        }
    }

    // "pre0post, pre1post, ..." over the values custos_elem takes
    std::string list(const std::string& pre, const std::string& post) const {
        std::string r;
        for (int i = 0; i < n_ops; i++) r += std::string(i ? ", " : "") + pre + std::to_string(i) + post;
        return r;
    }

    // Per-element function on storage values: `custos_elem(in0.., [g])`.
    std::string elem_fn() const {
        std::string s;
        if (k.kind == Kind::Chain) return chain_fn();
        if (k.kind == Kind::Apply) {
            s += "static __device__ __forceinline__ S custos_elem(";
            for (int i = 0; i < n_in; i++) s += std::string(i ? ", " : "") + "const S s" + std::to_string(i);
            s += " CUSTOS_KC_PARAM) {\n    return custos_store(custos_expr(";
            for (int i = 0; i < n_in; i++) s += std::string(i ? ", " : "") + "custos_load(s" + std::to_string(i) + ")";
            s += " CUSTOS_KC_ARG));\n}\n";
        } else {
            s += grad_fn(k.dtype);
            s += "static __device__ __forceinline__ S custos_elem(const S s0, const S s1, const S s2 CUSTOS_KC_PARAM) {\n"
                 "    return custos_store(custos_grad(custos_load(s1), custos_load(s2), custos_expr(custos_load(s0) CUSTOS_KC_ARG)));\n}\n";
        }
        return s;
    }

    // One element outside the vector body: `out[idx] = custos_elem(in0[idx], ..)`; a chain
    // stores every output.
    std::string scalar_stmt(const std::string& idx) const {
        if (k.kind != Kind::Chain) return "out[" + idx + "] = custos_elem(" + list("in", "[" + idx + "]") + " CUSTOS_KC_ARG);";
        std::string s = "{ S o[" + std::to_string(k.n_outs) + "]; custos_chain(" + list("in", "[" + idx + "]") + ", o CUSTOS_KC_ARG);";
        for (int j = 0; j < k.n_outs; j++) s += " out" + std::to_string(j) + "[" + idx + "] = o[" + std::to_string(j) + "];";
        return s + " }";
    }

    // Chain: one function per stage, and `custos_chain(s0.., o)`, which evaluates the stages in
    // order on storage values and leaves the value of every output pointer in `o`.  A stage that
    // reads an earlier one takes its result as it was stored (rounded to the storage type).
    std::string chain_fn() const {
        std::string s;
        int base = 0;
        for (size_t st = 0; st < k.stages.size(); st++) {
            const ChainStage& stage = k.stages[st];
            ConstPlan plan;
            ParseError err;
            std::string body;
            // (checked when the spec was built)
            (void)stage_plan(stage, k.dtype, base, &plan, &err);
            (void)emit_expr_body(stage.expr, k.dtype, plan, &body, &err);
            base += stage.n_params;
            s += "static __device__ __forceinline__ C custos_expr_s" + std::to_string(st) + "(";
            for (int v = 0; v < stage.expr.n_vars; v++) s += std::string(v ? ", " : "") + "const C v" + std::to_string(v);
            s += " CUSTOS_KC_PARAM) {\n" + body + "}\n";
        }
        s += "static __device__ __forceinline__ void custos_chain(";
        for (int i = 0; i < n_in; i++) s += "const S s" + std::to_string(i) + ", ";
        s += "S* o CUSTOS_KC_PARAM) {\n";
        for (int i = 0; i < n_in; i++) s += "    const C e" + std::to_string(i) + " = custos_load(s" + std::to_string(i) + ");\n";
        for (size_t st = 0; st < k.stages.size(); st++) {
            const ChainStage& stage = k.stages[st];
            const std::string id = std::to_string(st);
            s += "    const S t" + id + " = custos_store(custos_expr_s" + id + "(";
            for (size_t v = 0; v < stage.source.size(); v++) {
                const int from = stage.source[v];
                s += std::string(v ? ", " : "") + (from >= 0 ? "e" + std::to_string(from) : "r" + std::to_string(-from - 1));
            }
            s += " CUSTOS_KC_ARG));\n    const C r" + id + " = custos_load(t" + id + ");\n    (void)r" + id + ";\n";
            if (stage.out >= 0) s += "    o[" + std::to_string(stage.out) + "] = t" + id + ";\n";
        }
        s += "}\n";
        return s;
    }

    // Chain: one tile, all loads before the first store, one store per output.
    // Whether input `i` is loaded with non-temporal accesses: bit 1 of the mode word, unless the
    // launch wants this input kept in the cache (bits 3..6, inputs 0..3).
    static std::string load_policy(int i) {
        if (i >= 4) return "mode & 2";
        return "(mode & 2) && !(mode & " + std::to_string(8 << i) + ")";
    }

    std::string chain_tile_fn(int unroll) const {
        const std::string U = std::to_string(unroll);
        std::string s = "static __device__ __forceinline__ void custos_tile" + U + "(";
        for (int i = 0; i < n_in; i++) s += "const vec_t* vin" + std::to_string(i) + ", ";
        for (int j = 0; j < k.n_outs; j++) s += "vec_t* vout" + std::to_string(j) + ", ";
        s += "const u64 first, const u64 n_vec, const u64 mode CUSTOS_KC_PARAM) {\n";
        s += "    const u64 left = (n_vec - first) * 16;\n";
        s += "    const int bound = left > 0x7ffffff0ull ? 0x7ffffff0 : (int)left;\n";
        for (int i = 0; i < n_in; i++)
            s += "    const custos_rsrc rs" + std::to_string(i) + " = custos_make_rsrc(vin" + std::to_string(i) + " + first, bound);\n";
        for (int j = 0; j < k.n_outs; j++)
            s += "    const custos_rsrc rso" + std::to_string(j) + " = custos_make_rsrc(vout" + std::to_string(j) + " + first, bound);\n";
        s += "    const unsigned int lane = threadIdx.x * 16u;\n";
        for (int i = 0; i < n_in; i++) s += "    vec_t a" + std::to_string(i) + "[" + U + "];\n";
        s += "#pragma unroll\n    for (int u = 0; u < " + U + "; u++) {\n";
        for (int i = 0; i < n_in; i++) {
            const std::string id = std::to_string(i);
            s += "        a" + id + "[u] = custos_ld(rs" + id + ", lane + (unsigned int)u * (CUSTOS_BT * 16u), " + load_policy(i) + ");\n";
        }
        s += "    }\n";
        s += "#pragma unroll\n    for (int u = 0; u < " + U + "; u++) {\n";
        for (int j = 0; j < k.n_outs; j++) s += "        vec_t r" + std::to_string(j) + ";\n";
        s += "#pragma unroll\n        for (int k = 0; k < CUSTOS_VEC; k++) {\n";
        s += "            S o[" + std::to_string(k.n_outs) + "];\n";
        s += "            custos_chain(" + list("a", "[u][k]") + ", o CUSTOS_KC_ARG);\n";
        for (int j = 0; j < k.n_outs; j++) s += "            r" + std::to_string(j) + "[k] = o[" + std::to_string(j) + "];\n";
        s += "        }\n";
        for (int j = 0; j < k.n_outs; j++)
            s += "        custos_st(rso" + std::to_string(j) + ", lane + (unsigned int)u * (CUSTOS_BT * 16u), r" + std::to_string(j) + ", mode);\n";
        s += "    }\n}\n";
        return s;
    }

    // The numbers of vectors per thread this kernel has a tile function for: the caller's
    // choice, or the two shapes the library picks from per launch (2 with workgroups of
    // CUSTOS_BLOCK threads; 1 with one-wavefront workgroups, for launches that stream from and
    // to memory without finding anything in the caches).
    std::vector<int> unrolls() const {
        if (k.auto_unroll) return {2, 1};
        return {k.tuning.unroll};
    }

    // `custos_tile<U>(args)` for the launch's number of vectors per thread `U`.
    std::string tile_call(const std::string& indent, const std::string& args) const {
        const std::vector<int> us = unrolls();
        if (us.size() == 1) return indent + "custos_tile" + std::to_string(us[0]) + "(" + args + ");\n";
        return indent + "if (U == 2) custos_tile2(" + args + ");\n" + indent + "else custos_tile1(" + args + ");\n";
    }

    // Tiles of a range of `n_vec` vectors, without a division by a run-time value (which would
    // cost every wavefront a 64-bit division routine): a constant divisor, or, where the launch
    // names its shape, a shift (64 << b threads times 1 or 2 vectors).
    std::string n_tiles_expr() const {
        if (k.auto_unroll) return "((n_vec + tile_vecs - 1) >> (6 + ((mode >> 13) & 3) + (U >> 1)))";
        const std::string tv = "((u64)CUSTOS_BLOCK * " + std::to_string(k.tuning.unroll) + ")";
        return "(n_vec + " + tv + " - 1) / " + tv;
    }

    // `const u64 U = ...;`: vectors per thread of this launch, from the mode word
    std::string unroll_of_mode() const {
        if (!k.auto_unroll) return "    const u64 U = " + std::to_string(k.tuning.unroll) + ";\n";
        return "    const u64 U = (mode >> 8) & 15;\n";
    }

    // One tile of `unroll` vectors per thread, starting at vector `first` of the operands (the
    // same for the whole workgroup): every lane loads all its vectors, then computes and stores.
    // The operands are addressed through buffer descriptors whose base is the tile's first
    // vector and whose size is what is left of the vector range from there on: the hardware
    // returns zeros for a load beyond it and drops a store, so a partial last tile runs the
    // same instructions as a full one, and the cache policy of the launch (uniform: a scalar
    // branch around the instruction) is an immediate operand of each load and store.  An output
    // may be exactly one of the inputs: every lane has loaded all its vectors before its first
    // store.
    std::string tile_fn(int unroll) const {
        if (k.kind == Kind::Chain) return chain_tile_fn(unroll);
        const std::string U = std::to_string(unroll);
        std::string ptr_params;
        for (int i = 0; i < n_ops; i++) {
            if (k.kind == Kind::UnaryGrad && i == 1) continue;
            ptr_params += "const vec_t* vin" + std::to_string(i) + ", ";
        }
        std::string s;
        s += "static __device__ __forceinline__ void custos_tile" + U + "(" + ptr_params +
             "vec_t* vout, const u64 first, const u64 n_vec, const u64 mode CUSTOS_KC_PARAM) {\n";
        s += "    const u64 left = (n_vec - first) * 16;\n";
        s += "    const int bound = left > 0x7ffffff0ull ? 0x7ffffff0 : (int)left;\n";
        for (int i = 0; i < n_ops; i++) {
            const std::string id = std::to_string(i);
            if (k.kind == Kind::UnaryGrad && i == 1) {
                s += "    const custos_rsrc rs1 = custos_make_rsrc(vout + first, bound);\n";
                continue;
            }
            s += "    const custos_rsrc rs" + id + " = custos_make_rsrc(vin" + id + " + first, bound);\n";
        }
        s += k.kind == Kind::UnaryGrad ? "    const custos_rsrc rso = rs1;\n" : "    const custos_rsrc rso = custos_make_rsrc(vout + first, bound);\n";
        s += "    const unsigned int lane = threadIdx.x * 16u;\n";
        for (int i = 0; i < n_ops; i++) s += "    vec_t a" + std::to_string(i) + "[" + U + "];\n";
        s += "#pragma unroll\n    for (int u = 0; u < " + U + "; u++) {\n";
        for (int i = 0; i < n_ops; i++) {
            const std::string id = std::to_string(i);
            s += "        a" + id + "[u] = custos_ld(rs" + id + ", lane + (unsigned int)u * (CUSTOS_BT * 16u), " + load_policy(i) + ");\n";
        }
        s += "    }\n";
        s += "#pragma unroll\n    for (int u = 0; u < " + U + "; u++) {\n";
        s += "        vec_t r;\n#pragma unroll\n        for (int k = 0; k < CUSTOS_VEC; k++) r[k] = custos_elem(" +
             list("a", "[u][k]") + " CUSTOS_KC_ARG);\n";
        s += "        custos_st(rso, lane + (unsigned int)u * (CUSTOS_BT * 16u), r, mode);\n    }\n";
        s += "}\n";
        return s;
    }

    // Entry point for one launch over one set of operands.  `mode`: bit 0 walks the tiles from
    // the last to the first (see Tuning::direction), bits 1..6 the cache policy, bits 8..11 the
    // vectors per thread (kernel_gen.hpp, launch_mode).
    std::string single_entry() const {
        std::string s;
        s += "extern \"C\" __global__ void __launch_bounds__(CUSTOS_BLOCK)\n";
        s += k.name + "(" + params + ", const u64 n, const u64 head, const u64 n_vec, CUSTOS_KC_ENTRY const u64 mode) {\n";
        s += vec_ptrs;
        s += "    const u64 rev = mode & 1;\n";
        s += unroll_of_mode();
        s += "    const u64 tile_vecs = (u64)CUSTOS_BT * U;\n";
        s += "    const u64 n_tiles = mode >> 16;\n";
        s += "    for (u64 tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {\n";
        s += tile_call("        ", tile_args + out_views + "(rev ? n_tiles - 1 - tile : tile) * tile_vecs, n_vec, mode CUSTOS_KC_ARG");
        s += "    }\n";
        // Elements outside the 16-byte aligned body: `head` leading ones and the
        // tail. Lanes beyond the count are masked off by the wavefront's EXEC.  Most launches
        // have none (bit 12 of the mode word): one scalar test instead of per-lane arithmetic.
        // (One loop over both, so that the expression is expanded once for them.)
        s += "    if (!(mode & 4096)) return;\n";
        s += "    const u64 gid = (u64)blockIdx.x * CUSTOS_BT + threadIdx.x;\n";
        s += "    const u64 n_threads = (u64)gridDim.x * CUSTOS_BT;\n";
        s += "    const u64 body_end = head + n_vec * CUSTOS_VEC;\n";
        s += "    const u64 n_edge = head + (n - body_end);\n";
        s += "    for (u64 e = gid; e < n_edge; e += n_threads) {\n";
        s += "        const u64 i = e < head ? e : e - head + body_end;\n";
        s += "        " + scalar_stmt("i") + "\n    }\n";
        s += "}\n";
        return s;
    }

    // In a merged launch every segment brings its own literal parameters: they follow the
    // operand addresses (and the length) in its table row, so launches of one kernel merge
    // whatever their values.  The row is the same for the whole workgroup: scalar loads.
    std::string row_consts(int first_word) const {
        if (const_words == 0) return "";
        return "    CustosConsts kc;\n    __builtin_memcpy(&kc, ptrs + " + std::to_string(first_word) + ", sizeof(kc));\n";
    }

    // operand pointers of a merged launch, read from the table row `ptrs`
    std::string table_operands() const {
        std::string s;
        if (k.kind == Kind::Chain) {
            for (int i = 0; i < n_in; i++)
                s += "    const S* in" + std::to_string(i) + " = (const S*)ptrs[" + std::to_string(i) + "];\n";
            for (int j = 0; j < k.n_outs; j++)
                s += "    S* out" + std::to_string(j) + " = (S*)ptrs[" + std::to_string(n_in + j) + "];\n";
        } else if (k.kind == Kind::Apply) {
            for (int i = 0; i < n_in; i++)
                s += "    const S* in" + std::to_string(i) + " = (const S*)ptrs[" + std::to_string(i) + "];\n";
            s += "    S* out = (S*)ptrs[" + std::to_string(n_in) + "];\n";
        } else {
            s += "    const S* in0 = (const S*)ptrs[0];\n    S* out = (S*)ptrs[1];\n    const S* in2 = (const S*)ptrs[2];\n";
        }
        return s;
    }

    // Entry point for many independent launches of equal length in one grid (graph replay of
    // many small buffers).  `table` holds, per segment, the operand addresses in the order of
    // the single-launch parameters; every address is 16-byte aligned.  Workgroup b works on
    // tile b % tiles_per_seg of segment b / tiles_per_seg; the last tile of a segment also
    // does the tail.
    std::string batched_entry() const {
        std::string s;
        s += "extern \"C\" __global__ void __launch_bounds__(CUSTOS_BLOCK)\n";
        s += k.name + "_batched(const u64* __restrict__ table, const u64 n, const u64 n_vec, const u64 tiles_per_seg, const u64 mode) {\n";
        s += unroll_of_mode();
        // (a grid has fewer than 2^31 workgroups: a 32-bit division, a third of the 64-bit one)
        s += "    const unsigned int blk = (mode & 1) ? gridDim.x - 1 - blockIdx.x : blockIdx.x;\n";
        s += "    const unsigned int per_seg = (unsigned int)tiles_per_seg;\n";
        s += "    const u64 seg = blk / per_seg;\n";
        s += "    const u64 tile = blk - (unsigned int)seg * per_seg;\n";
        s += "    const u64* ptrs = table + seg * " + std::to_string(n_ptrs + const_words) + ";\n";
        s += row_consts(n_ptrs);
        s += "    const u64 head = 0;\n";
        s += table_operands();
        s += vec_ptrs;
        s += tile_call("    ", tile_args + out_views + "tile * (u64)CUSTOS_BT * U, n_vec, mode CUSTOS_KC_ARG");
        s += "    if (tile == tiles_per_seg - 1)\n";
        s += "        for (u64 i = n_vec * CUSTOS_VEC + threadIdx.x; i < n; i += CUSTOS_BT) " + scalar_stmt("i") + "\n";
        s += "    (void)head;\n}\n";
        return s;
    }

    // Entry point for launches of different lengths in one grid.  A table row holds the
    // operand addresses (16-byte aligned) and the element count of its segment;
    // `block_map[b]` = segment << 32 | tile tells workgroup b its work.
    std::string ragged_entry() const {
        std::string s;
        s += "extern \"C\" __global__ void __launch_bounds__(CUSTOS_BLOCK)\n";
        s += k.name + "_ragged(const u64* __restrict__ table, const u64* __restrict__ block_map, const u64 mode) {\n";
        s += unroll_of_mode();
        s += "    const u64 where = block_map[(mode & 1) ? gridDim.x - 1 - blockIdx.x : blockIdx.x];\n";
        s += "    const u64 seg = where >> 32;\n";
        s += "    const u64 tile = where & 0xffffffffull;\n";
        s += "    const u64* ptrs = table + seg * " + std::to_string(n_ptrs + 1 + const_words) + ";\n";
        s += "    const u64 n = ptrs[" + std::to_string(n_ptrs) + "];\n";
        s += row_consts(n_ptrs + 1);
        s += "    const u64 n_vec = n / CUSTOS_VEC;\n";
        s += "    const u64 tile_vecs = (u64)CUSTOS_BT * U;\n";
        s += "    const u64 n_tiles = n_vec == 0 ? 1 : " + n_tiles_expr() + ";\n";
        s += "    const u64 head = 0;\n";
        s += table_operands();
        s += vec_ptrs;
        s += tile_call("    ", tile_args + out_views + "tile * tile_vecs, n_vec, mode CUSTOS_KC_ARG");
        s += "    if (tile == n_tiles - 1)\n";
        s += "        for (u64 i = n_vec * CUSTOS_VEC + threadIdx.x; i < n; i += CUSTOS_BT) " + scalar_stmt("i") + "\n";
        s += "    (void)head;\n}\n";
        return s;
    }
};

}  // namespace

bool build_kernel_spec(Kind kind, DType dtype, const std::string& src,
                       const std::vector<std::string>& markers, const Tuning& tuning,
                       bool literals_in_code, KernelSpec* out, ParseError* err, bool with_source) {
    KernelSpec k;
    k.kind = kind;
    k.dtype = dtype;
    k.tuning = tuning;
    if (!parse_expr(src, markers, &k.expr, err)) return false;
    if (tuning.eq_as_leq)
        for (Node& n : k.expr.nodes)
            if (n.op == Op::Eq) n.op = Op::LEq;
    if (kind == Kind::UnaryGrad && k.expr.n_vars != 1) {
        err->code = CUSTOS_HIP_ERR_ARITY_MISMATCH;
        err->message = "a unary gradient expression takes exactly one marker";
        return false;
    }
    // Vectors per thread left open: the kernel holds a tile function for two and for one, and
    // every launch names the one it takes.  The cache policy is never part of the code: it is a
    // field of the mode word of every launch.
    k.auto_unroll = tuning.unroll <= 0;
    if (k.auto_unroll) k.tuning.unroll = 2;
    k.tuning.nontemporal = -1;
    k.tuning.direction = 0;
    if (!plan_constants(k.expr, dtype, literals_in_code, &k.consts, err)) return false;
    for (const Node& n : k.expr.nodes) k.n_literals += n.op == Op::Const;
    uint64_t h;
    if (!hash_expr(k.expr, dtype, k.consts, &h, err, &k.code_literals)) return false;
    k.markers = markers;
    // (the key holds the vectors per thread as requested: 0 = chosen per launch)
    int32_t tail[5] = {static_cast<int32_t>(kind), k.tuning.block_threads, k.auto_unroll ? 0 : k.tuning.unroll,
                       k.tuning.blocks_per_cu, 21 /* template version */};
    k.hash = fnv1a64(tail, sizeof tail, h);
    k.vec_elems = static_cast<int>(16 / dtype_size(dtype));
    {
        static const char* const dtype_names[] = {"f32", "f64", "i32", "i64", "f16", "bf16",
                                                  "u8",  "i8",  "i16", "u16", "u32", "u64",
                                                  "f16n", "bf16n"};
        char hex[17];
        std::snprintf(hex, sizeof hex, "%016llx", static_cast<unsigned long long>(k.hash));
        k.name = std::string(kind == Kind::Apply ? "custos_apply_" : "custos_unary_grad_") +
                 dtype_names[static_cast<int>(dtype)] + "_" + hex;
    }

    if (with_source && !emit_kernel_source(&k, err)) return false;
    *out = std::move(k);
    return true;
}

bool emit_kernel_source(KernelSpec* spec, ParseError* err, EntrySet which) {
    KernelSpec& k = *spec;
    std::string body;
    if (k.kind == Kind::Chain) {
        // (the stage functions are emitted by KernelText; here only what cannot be compiled is found)
        for (const ChainStage& stage : k.stages) {
            ConstPlan plan;
            std::string unused;
            if (!stage_plan(stage, k.dtype, 0, &plan, err)) return false;
            if (!emit_expr_body(stage.expr, k.dtype, plan, &unused, err)) return false;
        }
    } else if (!emit_expr_body(k.expr, k.dtype, k.consts, &body, err)) {
        return false;
    }

    std::string s;
    s += "// generated by custos-hip: " + (k.kind == Kind::Chain ? k.chain_text : to_cl_source(k.expr, k.markers, &k.consts)) + "\n";
    // CUSTOS_BLOCK: the most threads a workgroup of this kernel has.  CUSTOS_BT: the threads of the
    // launch at hand -- a kernel whose shape the caller left open reads them from bits 13-14 of its
    // mode word (64 << bits), like the vectors per thread from bits 8-11.
    s += "#define CUSTOS_BLOCK " + std::to_string(k.tuning.block_threads) + "\n";
    s += k.auto_unroll ? "#define CUSTOS_BT (64u << ((mode >> 13) & 3))\n" : "#define CUSTOS_BT CUSTOS_BLOCK\n";
    s += "#define CUSTOS_VEC " + std::to_string(k.vec_elems) + "\n";
    s += prelude(k.dtype, k.vec_elems, k.consts.n_params);
    // Loads and stores of one 16-byte vector through a buffer descriptor, with the cache policy
    // of the launch as the instruction's immediate operand: temporal, or non-temporal (2) for
    // what streams past the caches.
    s += R"(typedef unsigned int custos_u4 __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t custos_rsrc;
static __device__ __forceinline__ custos_rsrc custos_make_rsrc(const vec_t* p, const int bytes) {
    return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, bytes, 0x00020000);
}
static __device__ __forceinline__ vec_t custos_ld(const custos_rsrc rs, const unsigned int offset, const bool nt) {
    custos_u4 v;
    if (nt) v = __builtin_amdgcn_raw_buffer_load_b128(rs, offset, 0, 2);
    else v = __builtin_amdgcn_raw_buffer_load_b128(rs, offset, 0, 0);
    return __builtin_bit_cast(vec_t, v);
}
static __device__ __forceinline__ void custos_st(const custos_rsrc rs, const unsigned int offset, const vec_t v, const u64 mode) {
    const custos_u4 bits = __builtin_bit_cast(custos_u4, v);
    if (mode & 4) {
        if (mode & 128) __builtin_amdgcn_raw_buffer_store_b128(bits, rs, offset, 0, 18);
        else __builtin_amdgcn_raw_buffer_store_b128(bits, rs, offset, 0, 2);
    } else {
        if (mode & 128) __builtin_amdgcn_raw_buffer_store_b128(bits, rs, offset, 0, 16);
        else __builtin_amdgcn_raw_buffer_store_b128(bits, rs, offset, 0, 0);
    }
}
)";
    if (k.kind != Kind::Chain) s += expr_fn(k, body);

    const KernelText text(k);
    s += text.elem_fn();
    for (int unroll : text.unrolls()) s += text.tile_fn(unroll);
    s += which == EntrySet::Single ? text.single_entry() : which == EntrySet::Batched ? text.batched_entry() : text.ragged_entry();

    k.source[static_cast<int>(which)] = std::move(s);
    return true;
}

int kernel_pointers(const KernelSpec& k) {
    if (k.kind == Kind::Chain) return k.n_ext + k.n_outs;
    return k.kind == Kind::UnaryGrad ? 3 : k.expr.n_vars + 1;
}

bool build_chain_spec(DType dtype, std::vector<ChainStage> stages, int n_ext, int n_outs, const Tuning& tuning,
                      KernelSpec* out, ParseError* err, bool with_source) {
    KernelSpec k;
    k.kind = Kind::Chain;
    k.dtype = dtype;
    k.tuning = tuning;
    k.auto_unroll = tuning.unroll <= 0;
    if (k.auto_unroll) k.tuning.unroll = 2;
    k.tuning.nontemporal = -1;
    k.tuning.direction = 0;
    k.n_ext = n_ext;
    k.n_outs = n_outs;
    if (stages.empty() || stages.size() > static_cast<size_t>(kMaxChainStages) || n_ext < 1 || n_ext > kMaxChainInputs ||
        n_outs < 1 || n_outs > kMaxChainOutputs) {
        err->code = CUSTOS_HIP_ERR_INVALID_ARGUMENT;
        err->message = "a chain kernel takes 1 to 8 stages, 1 to 8 inputs and 1 to 6 outputs";
        return false;
    }
    // key and text: every stage's expression (literal values included), where its variables come
    // from and where its value goes
    uint64_t h = fnv1a64("custos-chain", 12);
    for (size_t st = 0; st < stages.size(); st++) {
        const ChainStage& stage = stages[st];
        if (static_cast<int>(stage.source.size()) != stage.expr.n_vars || stage.out >= n_outs) {
            err->code = CUSTOS_HIP_ERR_INVALID_ARGUMENT;
            err->message = "malformed chain stage";
            return false;
        }
        ConstPlan plan;
        if (!stage_plan(stage, dtype, k.consts.n_params, &plan, err)) return false;
        k.consts.n_params += stage.n_params;
        uint64_t hs;
        std::vector<uint64_t> literals;
        if (!hash_expr(stage.expr, dtype, plan, &hs, err, &literals)) return false;
        h = fnv1a64(&hs, sizeof hs, h);
        std::vector<std::string> names;
        for (int from : stage.source) {
            if (from >= n_ext || -from - 1 >= static_cast<int>(st)) {
                err->code = CUSTOS_HIP_ERR_INVALID_ARGUMENT;
                err->message = "a chain stage reads an input or a stage that does not exist";
                return false;
            }
            h = fnv1a64(&from, sizeof from, h);
            names.push_back(from >= 0 ? "x" + std::to_string(from) : "s" + std::to_string(-from - 1));
        }
        h = fnv1a64(&stage.out, sizeof stage.out, h);
        for (const Node& n : stage.expr.nodes) k.n_literals += n.op == Op::Const;
        k.code_literals.insert(k.code_literals.end(), literals.begin(), literals.end());
        k.chain_text += "s" + std::to_string(st) + " = " + to_cl_source(stage.expr, names, &plan) +
                        (stage.out >= 0 ? " -> out" + std::to_string(stage.out) : std::string()) + "; ";
    }
    int32_t tail[7] = {static_cast<int32_t>(Kind::Chain), k.tuning.block_threads, k.auto_unroll ? 0 : k.tuning.unroll,
                       k.tuning.blocks_per_cu, n_ext, n_outs, 21 /* template version */};
    k.hash = fnv1a64(tail, sizeof tail, h);
    k.vec_elems = static_cast<int>(16 / dtype_size(dtype));
    k.stages = std::move(stages);
    // (the values travel with every launch of the kernel; here only their size counts)
    size_t param_bytes = 0;
    for (const ChainStage& stage : k.stages) param_bytes += stage.param_bytes;
    k.consts.bytes.assign(param_bytes, 0);
    {
        static const char* const dtype_names[] = {"f32", "f64", "i32", "i64", "f16", "bf16", "u8", "i8", "i16", "u16", "u32", "u64",
                                                  "f16n", "bf16n"};
        char hex[17];
        std::snprintf(hex, sizeof hex, "%016llx", static_cast<unsigned long long>(k.hash));
        k.name = std::string("custos_chain_") + dtype_names[static_cast<int>(dtype)] + "_" + hex;
    }
    if (with_source && !emit_kernel_source(&k, err)) return false;
    *out = std::move(k);
    return true;
}

bool same_code(const KernelSpec& a, const KernelSpec& b) {
    if (a.kind != b.kind || a.dtype != b.dtype || a.hash != b.hash) return false;
    if (a.tuning.block_threads != b.tuning.block_threads || a.tuning.unroll != b.tuning.unroll ||
        a.tuning.blocks_per_cu != b.tuning.blocks_per_cu || a.auto_unroll != b.auto_unroll)
        return false;
    // (a chain's text spells its stages, their wiring and every literal)
    if (a.kind == Kind::Chain) return a.n_ext == b.n_ext && a.n_outs == b.n_outs && a.chain_text == b.chain_text;
    if (a.expr.n_vars != b.expr.n_vars || a.expr.root != b.expr.root || a.expr.nodes.size() != b.expr.nodes.size()) return false;
    for (size_t i = 0; i < a.expr.nodes.size(); i++) {
        const Node& x = a.expr.nodes[i];
        const Node& y = b.expr.nodes[i];
        if (x.op != y.op || x.a != y.a || x.b != y.b || x.var != y.var) return false;
    }
    return a.consts.slot == b.consts.slot && a.code_literals == b.code_literals;
}

}  // namespace custos_hip
