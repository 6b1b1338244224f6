/*
 * CPU oracle for the custos element-wise path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of what custos' `CPU<Base>` device computes
 * for `apply_fn`, `add_unary_grad` and fused unary chains.  It exists to check
 * the HIP kernels and to time a CPU baseline.  Nothing in the shipped library
 * may call it; only tests, the smoke check and the bench's cpu_baseline leg do.
 *
 * An expression is handed over as a postfix (RPN) program of `oracle_ins`.
 * Every node is evaluated in the element type with exactly one rounding, like
 * the reference's `Eval` impls (src/two_way_ops/ops.rs, ops/unary.rs,
 * ops/cmps.rs), transcendental functions go to the platform libm exactly as
 * Rust's `f32::sin` etc. do (src/number.rs:273-346).
 *
 * Pinning status (which independent check holds each function in place):
 *   - node arithmetic, min/max select, comparisons: reference known-answer
 *     values (src/two_way_ops/mod.rs tests, src/two_way_ops/eval.rs:10-12,
 *     src/two_way_ops/resolve.rs:14-17) + IEEE closed forms / brute force on
 *     special values (tests/test_oracle_kats.py).
 *   - transcendentals: the literal vectors the reference asserts
 *     (src/unary.rs:150-155,195-200; src/two_way_ops/mod.rs:68,275-282).
 *   - apply / unary-grad loops: reference vectors (src/unary.rs:15-18,40-47;
 *     src/devices/cuda/ops.rs:254-272).
 *   - f16 <-> f32 conversion: brute force against numpy's float16 (an
 *     independent implementation) over all 65536 halves, all rounding
 *     midpoints and their neighbours.
 *   - nodes evaluated per node in f16 / bf16 (ORC_F16_PERNODE, ORC_BF16_PERNODE):
 *     the third-party `half` crate (2.3) the reference depends on is not
 *     vendored and the reference's tests never exercise 16-bit values on this
 *     path.  Its published algorithm (widen to f32, f32 operation, round to
 *     nearest even) and the reference's own `Float for f16` (`from_f32(
 *     to_f32().sin())` ..., src/number.rs:543-676) are restated here; for
 *     + - * / sqrt that equals the correctly rounded 16-bit operation, which
 *     tests/test_oracle_kats.py checks bit for bit against numpy's float16
 *     operators and, for bf16, against f32 steps rounded with the integer
 *     formula.  No reference vector exists for the transcendental nodes of
 *     these two modes; they are pinned against two other implementations of
 *     "widen, f32 routine, round": numpy's float16 ufuncs (f16) and torch's CPU
 *     bfloat16 operators (bf16), all 65536 inputs per node, never more than one
 *     unit of the 16-bit type apart and over 99 % bit-identical (the f32
 *     routines may differ in the last place before the rounding).  The
 *     reference's f16 `tan` calls `cos` (src/number.rs:575-577); that defect is
 *     not reproduced.
 */
#ifndef CUSTOS_CPU_ORACLE_H
#define CUSTOS_CPU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum oracle_op {
    ORC_VAR0 = 0,   /* first marker  (x / lhs) */
    ORC_VAR1 = 1,   /* second marker (y / rhs) */
    ORC_CONST = 2,
    ORC_ADD = 3,
    ORC_SUB = 4,
    ORC_MUL = 5,
    ORC_DIV = 6,
    ORC_POW = 7,
    ORC_MIN = 8,    /* if a < b { a } else { b }   src/number.rs:206-209 */
    ORC_MAX = 9,    /* if a > b { a } else { b }   src/number.rs:201-204 */
    ORC_GEQ = 10,
    ORC_LEQ = 11,
    ORC_EQ_CPUREF = 12, /* the reference CPU Eval of `eq`: a <= b (src/two_way_ops/ops/cmps.rs:135) */
    ORC_EQ = 13,        /* a == b: what the reference's GPU source "(a == b)" computes */
    ORC_SIN = 14,
    ORC_COS = 15,
    ORC_TAN = 16,
    ORC_TANH = 17,
    ORC_EXP = 18,
    ORC_LN = 19,
    ORC_ABS = 20,
    ORC_NEG = 21,
    ORC_IDENTITY = 22,
    ORC_SQRT = 23,  /* not a reference Combiner node; Float::sqrt (src/number.rs:320-322) */
    ORC_VAR2 = 24,  /* third marker, for fused multi-operand expressions */
    ORC_VAR3 = 25
};

typedef struct oracle_ins {
    int32_t op;
    int32_t reserved;
    double cst;     /* ORC_CONST payload; converted to the element type once */
} oracle_ins;

/* Element type selectors for the generic entry points. */
enum oracle_dtype {
    ORC_F32 = 0,
    ORC_F64 = 1,
    ORC_I32 = 2,
    ORC_I64 = 3,
    ORC_F16_F32 = 4,     /* f16 storage, f32 compute, one RNE rounding at the store */
    ORC_F16_PERNODE = 5, /* f16 storage, every node rounded to f16 (half crate) */
    ORC_U8 = 6,
    ORC_I8 = 7,
    ORC_I16 = 8,
    ORC_U16 = 9,
    ORC_U32 = 10,
    ORC_U64 = 11,
    ORC_BF16_F32 = 12,   /* bf16 storage, f32 compute, one RNE rounding at the store */
    ORC_BF16_PERNODE = 13 /* bf16 storage, every node rounded to bf16 (half crate) */
};

/* out[i] = f(in0[i], in1[i], ...)   -- src/devices/cpu_stack_ops.rs:7-15.
 * `ins` has `n_in` operand arrays (1..4).  Returns 0, or -1 on a malformed program. */
int oracle_apply_fn(int dtype, const oracle_ins *prog, int n_prog,
                    const void *const *ins, int n_in, void *out, size_t n);

/* Fused unary chain: per element, cur = x[i]; for each program cur = prog_k(cur);
 * out[i] = cur    -- src/devices/cpu/cpu_device.rs:204-232.
 * `progs` is the concatenation of the programs, `prog_lens[k]` their lengths. */
int oracle_fused_apply_fn(int dtype, const oracle_ins *progs, const int *prog_lens,
                          int n_progs, const void *x, void *out, size_t n);

/* lhs_grad[i] += out_grad[i] * f(lhs[i])   -- src/devices/cpu_stack_ops.rs:18-30 */
int oracle_add_unary_grad(int dtype, const oracle_ins *prog, int n_prog, const void *lhs,
                          void *lhs_grad, const void *out_grad, size_t n);

/* Scalar evaluation of one program (for known-answer tests). */
int oracle_eval_f32(const oracle_ins *prog, int n_prog, const float *vars, int n_vars, float *res);
int oracle_eval_f64(const oracle_ins *prog, int n_prog, const double *vars, int n_vars, double *res);
int oracle_eval_i32(const oracle_ins *prog, int n_prog, const int32_t *vars, int n_vars, int32_t *res);

/* IEEE binary16 <-> binary32, round-to-nearest-even, integer arithmetic only. */
uint16_t oracle_f32_to_f16(float f);
float oracle_f16_to_f32(uint16_t h);
uint16_t oracle_f32_to_bf16(float f);
float oracle_bf16_to_f32(uint16_t h);

/* clear_slice  -- src/devices/cpu_stack_ops.rs:33-37 */
void oracle_clear(void *buf, size_t bytes);

/*
 * Monomorphic loops for the benchmark configurations: what rustc produces for
 * the reference closures after inlining (a compiled loop, not an interpreter).
 * They are used for the timed CPU baseline and are tested equal to the
 * interpreter above.
 */
/* C1: out = exp(x) */
void oracle_c1_exp_f32(const float *x, float *out, size_t n);
/* C2 unfused: five apply_fn passes sin, *2, +1, max(.,0), -0.5 through `tmp` buffers */
void oracle_c2_chain_unfused_f32(const float *x, float *tmp_a, float *tmp_b, float *out, size_t n);
/* C2 fused: one pass, ops applied in sequence per element */
void oracle_c2_chain_fused_f32(const float *x, float *out, size_t n);
/* C3: forward y = tanh(x) */
void oracle_c3_tanh_fwd_f32(const float *x, float *y, size_t n);
/* C3: backward x_grad += y_grad * (1 - tanh(x)*tanh(x)) */
void oracle_c3_tanh_bwd_f32(const float *x, float *x_grad, const float *y_grad, size_t n);
/* C4: f16 storage, f32 compute: y = exp(x*0.5)*x + x*x, rounded once */
void oracle_c4_chain_f16(const uint16_t *x, uint16_t *out, size_t n);
/* C5: t = a*b; u = t+c; y = sqrt(abs(u))*0.3 (three passes, as recorded) */
void oracle_c5_graph_f32(const float *a, const float *b, const float *c, float *t, float *u,
                         float *y, size_t n);

#ifdef __cplusplus
}
#endif
#endif
