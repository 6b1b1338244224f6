/*
 * CPU oracle for the custos element-wise path.  TEST INFRASTRUCTURE ONLY:
 * see custos_cpu_oracle.h for what it restates and how each part is pinned.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math -fPIC -shared ... -lm
 * (-ffp-contract=off because Rust never contracts a*b+c into an fma).
 */
#include "custos_cpu_oracle.h"

#include <math.h>
#include <string.h>

#define ORC_STACK 64

/* ------------------------------------------------------------------ */
/* half / bfloat16 conversion, integer arithmetic only                 */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

static inline float bits_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t oracle_f32_to_f16(float f)
{
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;

    if (mag >= 0x7f800000u) { /* inf / nan */
        if (mag == 0x7f800000u)
            return (uint16_t)(sign | 0x7c00u);
        /* keep it a NaN: quiet bit + top payload bits */
        return (uint16_t)(sign | 0x7e00u | ((mag >> 13) & 0x01ffu));
    }
    if (mag >= 0x477ff000u) /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    if (mag < 0x33000001u) /* <= 2^-25: rounds to zero (2^-25 is a tie to even = 0) */
        return (uint16_t)sign;

    int32_t e = (int32_t)(mag >> 23) - 127; /* unbiased exponent */
    uint32_t m = (mag & 0x007fffffu) | 0x00800000u; /* 24-bit significand */
    uint32_t shift, half_bits;
    if (e >= -14) {
        /* normal half: keep 10 fraction bits */
        shift = 13;
        half_bits = ((uint32_t)(e + 15) << 10) + ((m >> shift) & 0x3ffu);
    } else {
        /* subnormal half: value = m * 2^(e-23), unit = 2^-24 */
        shift = (uint32_t)(13 + (-14 - e));
        half_bits = m >> shift;
    }
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (half_bits & 1u)))
        half_bits += 1; /* may carry into the exponent, which is the right result */
    return (uint16_t)(sign | half_bits);
}

float oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    if (e == 0x1f)
        return bits_f32(sign | 0x7f800000u | (m << 13));
    if (e == 0) {
        if (m == 0)
            return bits_f32(sign);
        /* subnormal: normalise */
        int shift = 0;
        while (!(m & 0x400u)) {
            m <<= 1;
            shift++;
        }
        m &= 0x3ffu;
        return bits_f32(sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (m << 13));
    }
    return bits_f32(sign | ((e + 127 - 15) << 23) | (m << 13));
}

uint16_t oracle_f32_to_bf16(float f)
{
    uint32_t x = f32_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u)
        return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}

float oracle_bf16_to_f32(uint16_t h)
{
    return bits_f32((uint32_t)h << 16);
}

/* ------------------------------------------------------------------ */
/* RPN interpreters                                                    */
/* ------------------------------------------------------------------ */

#define VAR_INDEX(op) ((op) == ORC_VAR0 ? 0 : (op) == ORC_VAR1 ? 1 : (op) == ORC_VAR2 ? 2 : 3)

/* Floating point interpreter.  ROUND(v) is applied after every node: the
 * identity for f32/f64 (the C expression is already in type T), a round trip
 * through f16 for the per-node half mode. */
#define DEFINE_FLOAT_EVAL(NAME, T, SIN, COS, TAN, TANH, EXP, LN, POW, FABS, SQRT, ROUND)          \
    static int NAME(const oracle_ins *prog, int n_prog, const T *vars, int n_vars, T *res)        \
    {                                                                                             \
        T st[ORC_STACK];                                                                          \
        int sp = 0;                                                                               \
        for (int pc = 0; pc < n_prog; pc++) {                                                     \
            int op = prog[pc].op;                                                                 \
            if (op == ORC_VAR0 || op == ORC_VAR1 || op == ORC_VAR2 || op == ORC_VAR3) {           \
                int vi = VAR_INDEX(op);                                                           \
                if (vi >= n_vars || sp >= ORC_STACK)                                              \
                    return -1;                                                                    \
                st[sp++] = vars[vi];                                                              \
                continue;                                                                         \
            }                                                                                     \
            if (op == ORC_CONST) {                                                                \
                if (sp >= ORC_STACK)                                                              \
                    return -1;                                                                    \
                st[sp++] = ROUND((T)prog[pc].cst);                                                \
                continue;                                                                         \
            }                                                                                     \
            if (op >= ORC_ADD && op <= ORC_EQ) { /* binary */                                     \
                if (sp < 2)                                                                       \
                    return -1;                                                                    \
                T b = st[--sp];                                                                   \
                T a = st[--sp];                                                                   \
                T r;                                                                              \
                switch (op) {                                                                     \
                case ORC_ADD: r = a + b; break;                                                   \
                case ORC_SUB: r = a - b; break;                                                   \
                case ORC_MUL: r = a * b; break;                                                   \
                case ORC_DIV: r = a / b; break;                                                   \
                case ORC_POW: r = POW(a, b); break;                                               \
                case ORC_MIN: r = (a < b) ? a : b; break;                                         \
                case ORC_MAX: r = (a > b) ? a : b; break;                                         \
                case ORC_GEQ: r = (T)(a >= b); break;                                             \
                case ORC_LEQ: r = (T)(a <= b); break;                                             \
                case ORC_EQ_CPUREF: r = (T)(a <= b); break;                                       \
                default: r = (T)(a == b); break;                                                  \
                }                                                                                 \
                st[sp++] = ROUND(r);                                                              \
                continue;                                                                         \
            }                                                                                     \
            if (sp < 1)                                                                           \
                return -1;                                                                        \
            T a = st[sp - 1];                                                                     \
            T r;                                                                                  \
            switch (op) {                                                                         \
            case ORC_SIN: r = SIN(a); break;                                                      \
            case ORC_COS: r = COS(a); break;                                                      \
            case ORC_TAN: r = TAN(a); break;                                                      \
            case ORC_TANH: r = TANH(a); break;                                                    \
            case ORC_EXP: r = EXP(a); break;                                                      \
            case ORC_LN: r = LN(a); break;                                                        \
            case ORC_ABS: r = FABS(a); break;                                                     \
            case ORC_NEG: r = -a; break;                                                          \
            case ORC_IDENTITY: r = a; break;                                                      \
            case ORC_SQRT: r = SQRT(a); break;                                                    \
            default: return -1;                                                                   \
            }                                                                                     \
            st[sp - 1] = ROUND(r);                                                                \
        }                                                                                         \
        if (sp != 1)                                                                              \
            return -1;                                                                            \
        *res = st[0];                                                                             \
        return 0;                                                                                 \
    }

#define NO_ROUND(v) (v)
#define F16_ROUND(v) (oracle_f16_to_f32(oracle_f32_to_f16(v)))
#define BF16_ROUND(v) (oracle_bf16_to_f32(oracle_f32_to_bf16(v)))

DEFINE_FLOAT_EVAL(eval_f32, float, sinf, cosf, tanf, tanhf, expf, logf, powf, fabsf, sqrtf, NO_ROUND)
DEFINE_FLOAT_EVAL(eval_f64, double, sin, cos, tan, tanh, exp, log, pow, fabs, sqrt, NO_ROUND)
/* half crate semantics: convert to f32, f32 libm / f32 arithmetic, round to f16 (src/number.rs:543-608).
 * The reference's f16 `tan` calls `cos` (src/number.rs:575-577); not reproduced here. */
DEFINE_FLOAT_EVAL(eval_f16_pernode, float, sinf, cosf, tanf, tanhf, expf, logf, powf, fabsf, sqrtf, F16_ROUND)
/* the same for half::bf16 (src/number.rs:610-676) */
DEFINE_FLOAT_EVAL(eval_bf16_pernode, float, sinf, cosf, tanf, tanhf, expf, logf, powf, fabsf, sqrtf, BF16_ROUND)

static int eval_16(int dtype, const oracle_ins *prog, int n_prog, const float *vars, int n_vars, float *res)
{
    if (dtype == ORC_F16_PERNODE)
        return eval_f16_pernode(prog, n_prog, vars, n_vars, res);
    if (dtype == ORC_BF16_PERNODE)
        return eval_bf16_pernode(prog, n_prog, vars, n_vars, res);
    return eval_f32(prog, n_prog, vars, n_vars, res);
}

/* Integer interpreter: arithmetic wraps (Rust release mode), computed in the
 * unsigned counterpart U then cast back to T; transcendental nodes do not
 * exist for integers in the reference (they need `Float`) and are rejected. */
#define DEFINE_INT_EVAL(NAME, T, U)                                                               \
    static int NAME(const oracle_ins *prog, int n_prog, const T *vars, int n_vars, T *res)        \
    {                                                                                             \
        T st[ORC_STACK];                                                                          \
        int sp = 0;                                                                               \
        for (int pc = 0; pc < n_prog; pc++) {                                                     \
            int op = prog[pc].op;                                                                 \
            if (op == ORC_VAR0 || op == ORC_VAR1 || op == ORC_VAR2 || op == ORC_VAR3) {           \
                int vi = VAR_INDEX(op);                                                           \
                if (vi >= n_vars || sp >= ORC_STACK)                                              \
                    return -1;                                                                    \
                st[sp++] = vars[vi];                                                              \
                continue;                                                                         \
            }                                                                                     \
            if (op == ORC_CONST) {                                                                \
                if (sp >= ORC_STACK)                                                              \
                    return -1;                                                                    \
                st[sp++] = (T)(long long)prog[pc].cst;                                            \
                continue;                                                                         \
            }                                                                                     \
            if (op >= ORC_ADD && op <= ORC_EQ) {                                                  \
                if (sp < 2)                                                                       \
                    return -1;                                                                    \
                T b = st[--sp];                                                                   \
                T a = st[--sp];                                                                   \
                T r;                                                                              \
                switch (op) {                                                                     \
                case ORC_ADD: r = (T)((U)a + (U)b); break;                                        \
                case ORC_SUB: r = (T)((U)a - (U)b); break;                                        \
                case ORC_MUL: r = (T)((U)a * (U)b); break;                                        \
                case ORC_DIV:                                                                     \
                    if (b == 0)                                                                   \
                        return -2;                                                                \
                    if ((T)-1 < 0 && b == (T)-1)                                                  \
                        r = (T)((U)0 - (U)a);                                                     \
                    else                                                                          \
                        r = (T)(a / b);                                                           \
                    break;                                                                        \
                case ORC_POW: return -2;                                                          \
                case ORC_MIN: r = (a < b) ? a : b; break;                                         \
                case ORC_MAX: r = (a > b) ? a : b; break;                                         \
                case ORC_GEQ: r = (T)(a >= b); break;                                             \
                case ORC_LEQ: r = (T)(a <= b); break;                                             \
                case ORC_EQ_CPUREF: r = (T)(a <= b); break;                                       \
                default: r = (T)(a == b); break;                                                  \
                }                                                                                 \
                st[sp++] = r;                                                                     \
                continue;                                                                         \
            }                                                                                     \
            if (sp < 1)                                                                           \
                return -1;                                                                        \
            T a = st[sp - 1];                                                                     \
            switch (op) {                                                                         \
            case ORC_NEG: st[sp - 1] = (T)((U)0 - (U)a); break;                                   \
            case ORC_IDENTITY: break;                                                             \
            default: return -2;                                                                   \
            }                                                                                     \
        }                                                                                         \
        if (sp != 1)                                                                              \
            return -1;                                                                            \
        *res = st[0];                                                                             \
        return 0;                                                                                 \
    }

DEFINE_INT_EVAL(eval_i8, int8_t, uint8_t)
DEFINE_INT_EVAL(eval_u8, uint8_t, uint8_t)
DEFINE_INT_EVAL(eval_i16, int16_t, uint16_t)
DEFINE_INT_EVAL(eval_u16, uint16_t, uint16_t)
DEFINE_INT_EVAL(eval_i32, int32_t, uint32_t)
DEFINE_INT_EVAL(eval_u32, uint32_t, uint32_t)
DEFINE_INT_EVAL(eval_i64, int64_t, uint64_t)
DEFINE_INT_EVAL(eval_u64, uint64_t, uint64_t)

int oracle_eval_f32(const oracle_ins *prog, int n_prog, const float *vars, int n_vars, float *res)
{
    return eval_f32(prog, n_prog, vars, n_vars, res);
}

int oracle_eval_f64(const oracle_ins *prog, int n_prog, const double *vars, int n_vars, double *res)
{
    return eval_f64(prog, n_prog, vars, n_vars, res);
}

int oracle_eval_i32(const oracle_ins *prog, int n_prog, const int32_t *vars, int n_vars, int32_t *res)
{
    return eval_i32(prog, n_prog, vars, n_vars, res);
}

/* ------------------------------------------------------------------ */
/* element access by dtype                                             */
/* ------------------------------------------------------------------ */

/* Storage <-> compute conversion for the 16-bit float modes. */
static inline float load16(int dtype, const void *p, size_t i)
{
    uint16_t h = ((const uint16_t *)p)[i];
    return (dtype == ORC_BF16_F32 || dtype == ORC_BF16_PERNODE) ? oracle_bf16_to_f32(h) : oracle_f16_to_f32(h);
}

static inline void store16(int dtype, void *p, size_t i, float v)
{
    ((uint16_t *)p)[i] = (dtype == ORC_BF16_F32 || dtype == ORC_BF16_PERNODE) ? oracle_f32_to_bf16(v) : oracle_f32_to_f16(v);
}

static inline int is_16bit_float(int dtype)
{
    return dtype == ORC_F16_F32 || dtype == ORC_F16_PERNODE || dtype == ORC_BF16_F32 || dtype == ORC_BF16_PERNODE;
}

#define MAX_IN 4

/* Loops over typed arrays: src/devices/cpu_stack_ops.rs:7-15 (zip over x and out). */
#define TYPED_APPLY(T, EVAL)                                                                      \
    do {                                                                                          \
        T vars[MAX_IN];                                                                           \
        for (size_t i = 0; i < n; i++) {                                                          \
            for (int k = 0; k < n_in; k++)                                                        \
                vars[k] = ((const T *)ins[k])[i];                                                 \
            T r;                                                                                  \
            int rc = EVAL(prog, n_prog, vars, n_in, &r);                                          \
            if (rc)                                                                               \
                return rc;                                                                        \
            ((T *)out)[i] = r;                                                                    \
        }                                                                                         \
        return 0;                                                                                 \
    } while (0)

int oracle_apply_fn(int dtype, const oracle_ins *prog, int n_prog, const void *const *ins,
                    int n_in, void *out, size_t n)
{
    if (n_in < 1 || n_in > MAX_IN)
        return -1;
    switch (dtype) {
    case ORC_F32: TYPED_APPLY(float, eval_f32);
    case ORC_F64: TYPED_APPLY(double, eval_f64);
    case ORC_I8: TYPED_APPLY(int8_t, eval_i8);
    case ORC_U8: TYPED_APPLY(uint8_t, eval_u8);
    case ORC_I16: TYPED_APPLY(int16_t, eval_i16);
    case ORC_U16: TYPED_APPLY(uint16_t, eval_u16);
    case ORC_I32: TYPED_APPLY(int32_t, eval_i32);
    case ORC_U32: TYPED_APPLY(uint32_t, eval_u32);
    case ORC_I64: TYPED_APPLY(int64_t, eval_i64);
    case ORC_U64: TYPED_APPLY(uint64_t, eval_u64);
    case ORC_F16_F32:
    case ORC_BF16_F32:
    case ORC_BF16_PERNODE:
    case ORC_F16_PERNODE: {
        float vars[MAX_IN];
        for (size_t i = 0; i < n; i++) {
            for (int k = 0; k < n_in; k++)
                vars[k] = load16(dtype, ins[k], i);
            float r;
            int rc = eval_16(dtype, prog, n_prog, vars, n_in, &r);
            if (rc)
                return rc;
            store16(dtype, out, i, r);
        }
        return 0;
    }
    default: return -1;
    }
}

/* Sequential application of the fused programs per element:
 * src/devices/cpu/cpu_device.rs:218-228.  For the 16-bit "f32 compute" modes
 * the running value stays in f32 between the programs and is rounded once. */
#define TYPED_FUSED(T, EVAL)                                                                      \
    do {                                                                                          \
        for (size_t i = 0; i < n; i++) {                                                          \
            T cur = ((const T *)x)[i];                                                            \
            const oracle_ins *p = progs;                                                          \
            for (int k = 0; k < n_progs; k++) {                                                   \
                T r;                                                                              \
                int rc = EVAL(p, prog_lens[k], &cur, 1, &r);                                      \
                if (rc)                                                                           \
                    return rc;                                                                    \
                cur = r;                                                                          \
                p += prog_lens[k];                                                                \
            }                                                                                     \
            ((T *)out)[i] = cur;                                                                  \
        }                                                                                         \
        return 0;                                                                                 \
    } while (0)

int oracle_fused_apply_fn(int dtype, const oracle_ins *progs, const int *prog_lens, int n_progs,
                          const void *x, void *out, size_t n)
{
    switch (dtype) {
    case ORC_F32: TYPED_FUSED(float, eval_f32);
    case ORC_F64: TYPED_FUSED(double, eval_f64);
    case ORC_I8: TYPED_FUSED(int8_t, eval_i8);
    case ORC_U8: TYPED_FUSED(uint8_t, eval_u8);
    case ORC_I16: TYPED_FUSED(int16_t, eval_i16);
    case ORC_U16: TYPED_FUSED(uint16_t, eval_u16);
    case ORC_I32: TYPED_FUSED(int32_t, eval_i32);
    case ORC_U32: TYPED_FUSED(uint32_t, eval_u32);
    case ORC_I64: TYPED_FUSED(int64_t, eval_i64);
    case ORC_U64: TYPED_FUSED(uint64_t, eval_u64);
    case ORC_F16_F32:
    case ORC_BF16_F32:
    case ORC_BF16_PERNODE:
    case ORC_F16_PERNODE: {
        for (size_t i = 0; i < n; i++) {
            float cur = load16(dtype, x, i);
            const oracle_ins *p = progs;
            for (int k = 0; k < n_progs; k++) {
                float r;
                int rc = eval_16(dtype, p, prog_lens[k], &cur, 1, &r);
                if (rc)
                    return rc;
                cur = r;
                p += prog_lens[k];
            }
            store16(dtype, out, i, cur);
        }
        return 0;
    }
    default: return -1;
    }
}

/* *lhs_grad += *out * f(lhs): the product is rounded, then the sum is rounded
 * (src/devices/cpu_stack_ops.rs:27-29). */
#define TYPED_GRAD(T, EVAL, MULADD)                                                               \
    do {                                                                                          \
        for (size_t i = 0; i < n; i++) {                                                          \
            T v = ((const T *)lhs)[i];                                                            \
            T d;                                                                                  \
            int rc = EVAL(prog, n_prog, &v, 1, &d);                                               \
            if (rc)                                                                               \
                return rc;                                                                        \
            T g = ((T *)lhs_grad)[i];                                                             \
            T o = ((const T *)out_grad)[i];                                                       \
            ((T *)lhs_grad)[i] = MULADD(T, g, o, d);                                              \
        }                                                                                         \
        return 0;                                                                                 \
    } while (0)

#define FLOAT_MULADD(T, g, o, d) ((g) + ((o) * (d)))
#define WRAP_MULADD_I8(T, g, o, d) ((T)((uint8_t)(g) + (uint8_t)((uint8_t)(o) * (uint8_t)(d))))
#define WRAP_MULADD_I16(T, g, o, d) ((T)((uint16_t)(g) + (uint16_t)((uint16_t)(o) * (uint16_t)(d))))
#define WRAP_MULADD_I32(T, g, o, d) ((T)((uint32_t)(g) + (uint32_t)(o) * (uint32_t)(d)))
#define WRAP_MULADD_I64(T, g, o, d) ((T)((uint64_t)(g) + (uint64_t)(o) * (uint64_t)(d)))

int oracle_add_unary_grad(int dtype, const oracle_ins *prog, int n_prog, const void *lhs,
                          void *lhs_grad, const void *out_grad, size_t n)
{
    switch (dtype) {
    case ORC_F32: TYPED_GRAD(float, eval_f32, FLOAT_MULADD);
    case ORC_F64: TYPED_GRAD(double, eval_f64, FLOAT_MULADD);
    case ORC_I8: TYPED_GRAD(int8_t, eval_i8, WRAP_MULADD_I8);
    case ORC_U8: TYPED_GRAD(uint8_t, eval_u8, WRAP_MULADD_I8);
    case ORC_I16: TYPED_GRAD(int16_t, eval_i16, WRAP_MULADD_I16);
    case ORC_U16: TYPED_GRAD(uint16_t, eval_u16, WRAP_MULADD_I16);
    case ORC_I32: TYPED_GRAD(int32_t, eval_i32, WRAP_MULADD_I32);
    case ORC_U32: TYPED_GRAD(uint32_t, eval_u32, WRAP_MULADD_I32);
    case ORC_I64: TYPED_GRAD(int64_t, eval_i64, WRAP_MULADD_I64);
    case ORC_U64: TYPED_GRAD(uint64_t, eval_u64, WRAP_MULADD_I64);
    case ORC_F16_F32:
    case ORC_BF16_F32: {
        /* f32 compute: g + (o * d) in f32, one rounding at the store */
        for (size_t i = 0; i < n; i++) {
            float v = load16(dtype, lhs, i), d;
            int rc = eval_f32(prog, n_prog, &v, 1, &d);
            if (rc)
                return rc;
            float g = load16(dtype, lhs_grad, i), o = load16(dtype, out_grad, i);
            float prod = o * d;
            store16(dtype, lhs_grad, i, g + prod);
        }
        return 0;
    }
    case ORC_BF16_PERNODE:
    case ORC_F16_PERNODE: {
        for (size_t i = 0; i < n; i++) {
            float v = load16(dtype, lhs, i), d;
            int rc = eval_16(dtype, prog, n_prog, &v, 1, &d);
            if (rc)
                return rc;
            float g = load16(dtype, lhs_grad, i), o = load16(dtype, out_grad, i);
            float prod = dtype == ORC_BF16_PERNODE ? BF16_ROUND(o * d) : F16_ROUND(o * d);
            store16(dtype, lhs_grad, i, g + prod);
        }
        return 0;
    }
    default: return -1;
    }
}

void oracle_clear(void *buf, size_t bytes)
{
    memset(buf, 0, bytes);
}

/* ------------------------------------------------------------------ */
/* monomorphic benchmark loops                                         */
/* ------------------------------------------------------------------ */

void oracle_c1_exp_f32(const float *x, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++)
        out[i] = expf(x[i]);
}

static inline float max_sel(float a, float b)
{
    return a > b ? a : b;
}

void oracle_c2_chain_unfused_f32(const float *x, float *tmp_a, float *tmp_b, float *out, size_t n)
{
    /* five apply_fn calls on CPU<Base>: every call is its own pass over memory */
    for (size_t i = 0; i < n; i++)
        tmp_a[i] = sinf(x[i]);
    for (size_t i = 0; i < n; i++)
        tmp_b[i] = tmp_a[i] * 2.0f;
    for (size_t i = 0; i < n; i++)
        tmp_a[i] = tmp_b[i] + 1.0f;
    for (size_t i = 0; i < n; i++)
        tmp_b[i] = max_sel(tmp_a[i], 0.0f);
    for (size_t i = 0; i < n; i++)
        out[i] = tmp_b[i] - 0.5f;
}

void oracle_c2_chain_fused_f32(const float *x, float *out, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        float v = sinf(x[i]);
        v = v * 2.0f;
        v = v + 1.0f;
        v = max_sel(v, 0.0f);
        v = v - 0.5f;
        out[i] = v;
    }
}

void oracle_c3_tanh_fwd_f32(const float *x, float *y, size_t n)
{
    for (size_t i = 0; i < n; i++)
        y[i] = tanhf(x[i]);
}

void oracle_c3_tanh_bwd_f32(const float *x, float *x_grad, const float *y_grad, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        float t = tanhf(x[i]);
        float tt = tanhf(x[i]); /* the grad closure evaluates tanh(x) for both factors */
        float sq = t * tt;
        float d = 1.0f - sq;
        float prod = y_grad[i] * d;
        x_grad[i] = x_grad[i] + prod;
    }
}

void oracle_c4_chain_f16(const uint16_t *x, uint16_t *out, size_t n)
{
    for (size_t i = 0; i < n; i++) {
        float v = oracle_f16_to_f32(x[i]);
        float h = v * 0.5f;
        float e = expf(h);
        float p = e * v;
        float sq = v * v;
        out[i] = oracle_f32_to_f16(p + sq);
    }
}

void oracle_c5_graph_f32(const float *a, const float *b, const float *c, float *t, float *u,
                         float *y, size_t n)
{
    for (size_t i = 0; i < n; i++)
        t[i] = a[i] * b[i];
    for (size_t i = 0; i < n; i++)
        u[i] = t[i] + c[i];
    for (size_t i = 0; i < n; i++) {
        float s = sqrtf(fabsf(u[i]));
        y[i] = s * 0.3f;
    }
}
