/*
 * zyx_oracle.c -- CPU restatement of the arithmetic zyx's C/CPU backend performs
 * for the ops that the MI355X HIP backend accelerates.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker the HIP kernels are compared
 * with, and the CPU baseline timed beside them. Nothing in the product library
 * (zyx_amd/, include/) links, imports or calls it.
 *
 * The reference is Rust and generates its C kernels at run time, so no reference
 * source can be compiled here; every function restates the cited reference code
 * (paths relative to the reference checkout) and is pinned by the reference's own
 * golden vectors in tests/test_oracle_*.py. Functions that no golden vector or
 * closed form pins say "parity unpinned" in their comment.
 *
 * Conventions followed (zyx/src/codegen/c.rs):
 *   - all float math runs in `float` registers, bf16/f16 are widened on load and
 *     truncated on store (c.rs:135-140, 199-201, 456-497, 615-629);
 *   - reductions keep one register accumulator, initialised to 0 / dtype.min,
 *     and fold `acc = x (+) acc` serially over the reduce axis
 *     (zyx/src/kernel/linearize.rs:920-952, zyx/src/dtype.rs:207-224);
 *   - Max is fmax (c.rs:602), Mod is (int)x % (int)y (c.rs:598);
 *   - the outermost output loop is `#pragma omp parallel for` (c.rs:89-91);
 *   - built with -O3 -ffast-math -fno-associative-math (zyx/src/backend/c.rs:221-227).
 */
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ZO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* RNG: zyx/src/rng.rs                                                        */
/* ------------------------------------------------------------------------- */

typedef struct {
    uint64_t s[4];
} zo_rng;

static inline uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

/* splitmix64 x4 seeding, rng.rs:15-57 */
ZO_API void zo_rng_seed(zo_rng *r, uint64_t state) {
    for (int i = 0; i < 4; i++) {
        state += 0x9e3779b97f4a7c15ull;
        uint64_t z = state;
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        r->s[i] = z ^ (z >> 31);
    }
}

/* xoshiro256++, rng.rs:65-80 */
ZO_API uint64_t zo_rng_next_u64(zo_rng *r) {
    uint64_t *s = r->s;
    uint64_t res = rotl64(s[0] + s[3], 23) + s[0];
    uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return res;
}

/* next_f32, rng.rs:98-110: LCG step on the low 32 bits, modulo 2^32-1, divided by
 * (float)(2^32-1) == 2^32. The value can be exactly 1.0f (v >= 2^32-128). */
static inline float zo_next_f32(zo_rng *r) {
    uint32_t seed = (uint32_t)zo_rng_next_u64(r);
    uint32_t v = (uint32_t)(1664525u * seed + 1013904223u) % 0xffffffffu;
    return (float)v / (float)0xffffffffu;
}

/* Tensor::rand for u8: one full 64-bit draw per element, low byte (rng.rs:92-95,131). */
ZO_API void zo_rand_u8(zo_rng *r, uint8_t *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = (uint8_t)zo_rng_next_u64(r);
}
ZO_API void zo_rand_u32(zo_rng *r, uint32_t *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = (uint32_t)zo_rng_next_u64(r);
}
/* Tensor::rand for floats, row-major sequential draws (zyx/src/tensor/mod.rs:516-597). */
ZO_API void zo_rand_f32(zo_rng *r, float *out, int64_t n) {
    for (int64_t i = 0; i < n; i++) out[i] = zo_next_f32(r);
}
/* Tensor::uniform: rand * (hi - lo) + lo in f32 (tensor/mod.rs:637-648). */
ZO_API void zo_uniform_f32(zo_rng *r, float *out, int64_t n, float lo, float hi) {
    float span = hi - lo;
    for (int64_t i = 0; i < n; i++) out[i] = zo_next_f32(r) * span + lo;
}
/* Tensor::randint for signed ints: next_u64 % range + lo (rng.rs:186-208). */
ZO_API void zo_randint_i32(zo_rng *r, int32_t *out, int64_t n, int64_t lo, int64_t hi) {
    uint64_t range = (uint64_t)(hi - lo);
    for (int64_t i = 0; i < n; i++) out[i] = (int32_t)((int64_t)(zo_rng_next_u64(r) % range) + lo);
}
/* Tensor::randn (tensor/mod.rs:603-613): one rand([2, n]) draw, then
 * cos(2*pi*u0[i]) * sqrt(-2*ln(1 - u1[i])). The reference evaluates cos/ln/sqrt as
 * device kernels, so its bits depend on the backend; here host libm is used and the
 * same buffer feeds both sides of every parity test. A draw u1 == 1.0f (possible,
 * see zo_next_f32) would give ln(0) = -inf: it is clamped to the largest float
 * below one, which changes that one sample and nothing after it. */
ZO_API void zo_randn_f32(zo_rng *r, float *out, int64_t n, float scale) {
    float *u0 = (float *)malloc(sizeof(float) * (size_t)n);
    for (int64_t i = 0; i < n; i++) u0[i] = zo_next_f32(r);
    const float two_pi = 2.0f * 3.14159265358979323846f;
    for (int64_t i = 0; i < n; i++) {
        float u1 = zo_next_f32(r);
        if (u1 >= 1.0f) u1 = 0.99999994f;
        float x1 = cosf(u0[i] * two_pi);
        float x2 = sqrtf(logf(1.0f - u1) * -2.0f);
        out[i] = x1 * x2 * scale;
    }
    free(u0);
}

/* ------------------------------------------------------------------------- */
/* 16-bit float storage: zyx/src/codegen/c.rs:456-497, zyx/src/scalar.rs:33-45 */
/* ------------------------------------------------------------------------- */

static inline float bf16_load(uint16_t h) {
    uint32_t b = (uint32_t)h << 16;
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static inline uint16_t bf16_store(float v) { /* truncation, not round-to-nearest */
    uint32_t b;
    memcpy(&b, &v, 4);
    return (uint16_t)(b >> 16);
}
static inline float f16_load(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, man = h & 0x3ffu, ex = (h >> 10) & 0x1fu, f;
    if (ex == 0) { /* subnormal: man * 2^-24 exactly, as zyx/src/scalar.rs:155-165 */
        float sub = ldexpf((float)man, -24);
        return sign ? -sub : sub;
    } else if (ex == 31) f = sign | 0x7f800000u | (man << 13);
    else f = sign | ((ex + 112u) << 23) | (man << 13);
    float r;
    memcpy(&r, &f, 4);
    return r;
}
static inline uint16_t f16_store(float v) { /* mantissa truncated, subnormals flushed */
    uint32_t f;
    memcpy(&f, &v, 4);
    uint32_t sign = (f >> 16) & 0x8000u, ex = (f >> 23) & 0xffu, man = f & 0x7fffffu;
    if (ex == 0) return (uint16_t)sign;
    if (ex == 255) return (uint16_t)(sign | 0x7c00u | (man >> 13));
    int ne = (int)ex - 127 + 15;
    if (ne >= 31) return (uint16_t)(sign | 0x7c00u);
    if (ne <= 0) return (uint16_t)sign;
    return (uint16_t)(sign | ((uint32_t)ne << 10) | (man >> 13));
}
ZO_API void zo_f32_to_bf16(const float *x, uint16_t *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = bf16_store(x[i]);
}
ZO_API void zo_bf16_to_f32(const uint16_t *x, float *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = bf16_load(x[i]);
}
ZO_API void zo_f32_to_f16(const float *x, uint16_t *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = f16_store(x[i]);
}
ZO_API void zo_f16_to_f32(const uint16_t *x, float *y, int64_t n) {
    for (int64_t i = 0; i < n; i++) y[i] = f16_load(x[i]);
}

/* dtype codes follow zyx/src/dtype.rs:20-47 */
enum { ZO_BF16 = 0, ZO_F16, ZO_F32, ZO_F64, ZO_U8, ZO_U16, ZO_U32, ZO_U64, ZO_I8, ZO_I16, ZO_I32, ZO_I64, ZO_BOOL };

static inline float load_as_f32(const void *p, int dtype, int64_t i) {
    switch (dtype) {
    case ZO_BF16: return bf16_load(((const uint16_t *)p)[i]);
    case ZO_F16: return f16_load(((const uint16_t *)p)[i]);
    default: return ((const float *)p)[i];
    }
}
static inline void store_from_f32(void *p, int dtype, int64_t i, float v) {
    switch (dtype) {
    case ZO_BF16: ((uint16_t *)p)[i] = bf16_store(v); break;
    case ZO_F16: ((uint16_t *)p)[i] = f16_store(v); break;
    default: ((float *)p)[i] = v; break;
    }
}

/* ------------------------------------------------------------------------- */
/* Primitive unary / binary ops on float registers: zyx/src/kernel/ops.rs:187-261,
 * zyx/src/codegen/c.rs:290-304, 593-611                                        */
/* ------------------------------------------------------------------------- */

enum { /* unary */
    ZO_U_NEG = 0, ZO_U_EXP, ZO_U_EXP2, ZO_U_LN, ZO_U_LOG2, ZO_U_RECIPROCAL, ZO_U_SQRT, ZO_U_SIN, ZO_U_COS,
    ZO_U_FLOOR, ZO_U_TRUNC, ZO_U_ABS,
    /* composites from zyx/src/tensor/elementwise.rs */
    ZO_U_RELU = 32, ZO_U_TANH, ZO_U_GELU, ZO_U_SIGMOID, ZO_U_RSQRT
};
enum { /* binary */
    ZO_B_ADD = 0, ZO_B_SUB, ZO_B_MUL, ZO_B_DIV, ZO_B_POW, ZO_B_MOD, ZO_B_CMPLT, ZO_B_CMPGT, ZO_B_MAX,
    ZO_B_NOTEQ, ZO_B_EQ, ZO_B_CMPGE
};

/* tanh = (exp(x+x) - 1) / (exp(x+x) + 1) (zyx/src/tensor/elementwise.rs:585-588);
 * inf/inf = NaN once exp(2x) overflows (x > ~44.36). */
static inline float zo_tanh(float z) {
    float e = expf(z + z);
    return (e - 1.0f) / (e + 1.0f);
}
/* gelu (elementwise.rs:168-170), in the reference's operation order:
 * (x * 0.5) * (tanh((x + ((x*x)*x) * 0.044715) * sqrt(2/pi)) + 1) */
static inline float zo_gelu(float x) {
    float inner = (x + ((x * x) * x) * 0.044715f) * sqrtf(2.0f / 3.14159265358979323846f);
    return (x * 0.5f) * (zo_tanh(inner) + 1.0f);
}

/* d gelu / dx, the product/chain rules (zyx/src/graph/autograd.rs:87-134) applied to the expression above;
 * tanh saturates to 1 where exp(2z) overflows. */
static inline float zo_gelu_grad(float x) {
    const float k = sqrtf(2.0f / 3.14159265358979323846f), x2 = x * x;
    const float z = (x + x2 * x * 0.044715f) * k;
    const float t = (z + z) > 88.0f ? 1.0f : zo_tanh(z);
    return 0.5f * (1.0f + t) + (0.5f * x) * ((1.0f - t * t) * (k * (1.0f + 0.134145f * x2)));
}

static inline float zo_unary(int op, float x) {
    switch (op) {
    case ZO_U_NEG: return -x;
    case ZO_U_EXP: return expf(x);
    case ZO_U_EXP2: return exp2f(x);
    case ZO_U_LN: return logf(x);
    case ZO_U_LOG2: return log2f(x);
    case ZO_U_RECIPROCAL: return 1.0f / x;
    case ZO_U_SQRT: return sqrtf(x);
    case ZO_U_SIN: return sinf(x);
    case ZO_U_COS: return cosf(x);
    case ZO_U_FLOOR: return floorf(x);
    case ZO_U_TRUNC: return truncf(x);
    case ZO_U_ABS: return fabsf(x);
    case ZO_U_RELU: return (float)(x > 0.0f) * x; /* (x>0).cast * x, elementwise.rs:289-293 */
    case ZO_U_TANH: return zo_tanh(x);
    case ZO_U_GELU: return zo_gelu(x);
    case ZO_U_SIGMOID: { float e = expf(x); return e / (e + 1.0f); } /* elementwise.rs:457-460 */
    case ZO_U_RSQRT: return sqrtf(1.0f / x);            /* elementwise.rs:305-307 */
    default: return NAN;
    }
}
static inline float zo_binary(int op, float x, float y) {
    switch (op) {
    case ZO_B_ADD: return x + y;
    case ZO_B_SUB: return x - y;
    case ZO_B_MUL: return x * y;
    case ZO_B_DIV: return x / y;
    case ZO_B_POW: return exp2f(log2f(x) * y); /* unfold_pows, kernel/fold_constants.rs:639-653 */
    case ZO_B_MOD: return (float)((int)x % (int)y);
    case ZO_B_CMPLT: return (float)(x < y);
    case ZO_B_CMPGT: return (float)(x > y);
    case ZO_B_CMPGE: return (float)(x >= y);
    case ZO_B_MAX: return fmaxf(x, y);
    case ZO_B_NOTEQ: return (float)(x != y);
    case ZO_B_EQ: return (float)(x == y);
    default: return NAN;
    }
}

/* y[i] = op(x[i]) for a float dtype (f32/bf16/f16 storage). */
ZO_API void zo_unary_map(int op, int dtype, const void *x, void *y, int64_t n) {
#pragma omp parallel for
    for (int64_t i = 0; i < n; i++) store_from_f32(y, dtype, i, zo_unary(op, load_as_f32(x, dtype, i)));
}
/* z[r,c] = op(x[r,c], y[...]) where y is same-shape (ybc=0), a row vector of
 * length cols broadcast over rows (ybc=1) or one scalar (ybc=2). */
ZO_API void zo_binary_map(int op, int dtype, const void *x, const void *y, void *z, int64_t rows, int64_t cols,
                          int ybc) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            int64_t i = r * cols + c;
            int64_t j = ybc == 0 ? i : (ybc == 1 ? c : 0);
            store_from_f32(z, dtype, i, zo_binary(op, load_as_f32(x, dtype, i), load_as_f32(y, dtype, j)));
        }
}

/* ------------------------------------------------------------------------- */
/* Reductions: zyx/src/tensor/reduce_ops.rs:45-147, kernel/linearize.rs:920-952 */
/* ------------------------------------------------------------------------- */

/* Sum / max over the last axis of a [rows, cols] float tensor. Accumulates in f32
 * (reduce_acc_dtype) and stores in `dtype`. op: 0 = sum, 1 = max. */
ZO_API void zo_reduce_rows(int op, int dtype, const void *x, void *y, int64_t rows, int64_t cols) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        float acc = op == 0 ? 0.0f : -FLT_MAX;
        for (int64_t c = 0; c < cols; c++) {
            float v = load_as_f32(x, dtype, r * cols + c);
            acc = op == 0 ? v + acc : fmaxf(v, acc);
        }
        store_from_f32(y, dtype, r, acc);
    }
}
/* Sum / max over axis 0 of [rows, cols]: one serial loop per output column. */
ZO_API void zo_reduce_cols(int op, int dtype, const void *x, void *y, int64_t rows, int64_t cols) {
#pragma omp parallel for
    for (int64_t c = 0; c < cols; c++) {
        float acc = op == 0 ? 0.0f : -FLT_MAX;
        for (int64_t r = 0; r < rows; r++) {
            float v = load_as_f32(x, dtype, r * cols + c);
            acc = op == 0 ? v + acc : fmaxf(v, acc);
        }
        store_from_f32(y, dtype, c, acc);
    }
}
/* Integer sums accumulate in i32 for narrower ints, i64 stays i64 (reduce_ops.rs:52-60). */
ZO_API void zo_reduce_rows_i32(int op, const int32_t *x, int32_t *y, int64_t rows, int64_t cols) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        int32_t acc = op == 0 ? 0 : INT32_MIN;
        for (int64_t c = 0; c < cols; c++) {
            int32_t v = x[r * cols + c];
            acc = op == 0 ? (int32_t)((uint32_t)v + (uint32_t)acc) : (v > acc ? v : acc);
        }
        y[r] = acc;
    }
}

/* ------------------------------------------------------------------------- */
/* softmax (+ row sum, + row argmax): zyx/src/tensor/mod.rs:1457-1461, 2245-2269 */
/* ------------------------------------------------------------------------- */

/* For every row of x[rows, cols] (f32):
 *   m = max_c x;  e = exp(x - m);  s = sum_c e;  y = e / s          (softmax)
 *   rowsum = sum_c y                                                 (Tensor::sum)
 *   arg = max_c( (y == max_c y) * c )  -> the LARGEST index among ties, i32
 * Every reduce is the serial register accumulator of the C backend. y, rowsum and
 * arg may each be NULL. */
ZO_API void zo_softmax_rows_f32(const float *x, float *y, float *rowsum, int32_t *arg, int64_t rows, int64_t cols) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        const float *xr = x + r * cols;
        float *tmp = y ? y + r * cols : (float *)malloc(sizeof(float) * (size_t)cols);
        float m = -FLT_MAX;
        for (int64_t c = 0; c < cols; c++) m = fmaxf(xr[c], m);
        float s = 0.0f;
        for (int64_t c = 0; c < cols; c++) {
            tmp[c] = expf(xr[c] - m);
            s = tmp[c] + s;
        }
        float ys = 0.0f, ymax = -FLT_MAX;
        for (int64_t c = 0; c < cols; c++) {
            tmp[c] = tmp[c] / s;
            ys = tmp[c] + ys;
            ymax = fmaxf(tmp[c], ymax);
        }
        if (rowsum) rowsum[r] = ys;
        if (arg) {
            int32_t a = INT32_MIN;
            for (int64_t c = 0; c < cols; c++) {
                int32_t idx = (int32_t)(tmp[c] == ymax) * (int32_t)c;
                a = idx > a ? idx : a;
            }
            arg[r] = a;
        }
        if (!y) free(tmp);
    }
}

/* The same chain on 16-bit storage (bf16 / f16; dtype codes as everywhere in this file): elements widen to f32
 * registers, softmax's max / sub / exp / sum / div stay in f32 inside its kernel (zyx/src/codegen/c.rs:615-629) and y is
 * narrowed by truncation on store (:491-496); the sum and the argmax that follow are kernels of their own and read the
 * stored y; the sum is stored truncated. Built from the f32 row function above and the load / store conversions that
 * the narrow-store goldens pin. y, rowsum and arg may each be NULL. */
ZO_API void zo_softmax_rows(int dtype, const void *x, void *y, void *rowsum, int32_t *arg, int64_t rows, int64_t cols) {
    if (dtype == ZO_F32) {
        zo_softmax_rows_f32((const float *)x, (float *)y, (float *)rowsum, arg, rows, cols);
        return;
    }
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        float *tmp = (float *)malloc(sizeof(float) * (size_t)(cols > 0 ? cols : 1));
        float m = -FLT_MAX;
        for (int64_t c = 0; c < cols; c++) m = fmaxf(load_as_f32(x, dtype, r * cols + c), m);
        float s = 0.0f;
        for (int64_t c = 0; c < cols; c++) {
            tmp[c] = expf(load_as_f32(x, dtype, r * cols + c) - m);
            s = tmp[c] + s;
        }
        uint16_t *stored = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)(cols > 0 ? cols : 1));
        for (int64_t c = 0; c < cols; c++) store_from_f32(stored, dtype, c, tmp[c] / s);
        float ys = 0.0f, ymax = -FLT_MAX;
        for (int64_t c = 0; c < cols; c++) {
            tmp[c] = load_as_f32(stored, dtype, c);
            ys = tmp[c] + ys;
            ymax = fmaxf(tmp[c], ymax);
        }
        if (y)
            for (int64_t c = 0; c < cols; c++) ((uint16_t *)y)[r * cols + c] = stored[c];
        if (rowsum) store_from_f32(rowsum, dtype, r, ys);
        if (arg) {
            int32_t a = INT32_MIN;
            for (int64_t c = 0; c < cols; c++) {
                int32_t idx = (int32_t)(tmp[c] == ymax) * (int32_t)c;
                a = idx > a ? idx : a;
            }
            arg[r] = a;
        }
        free(stored);
        free(tmp);
    }
}

/* Same rows, but every accumulation in double: the "what the mathematics fixes"
 * companion used to bound how far serial f32 summation itself is from the truth. */
ZO_API void zo_softmax_rows_f64acc(const float *x, float *y, float *rowsum, int64_t rows, int64_t cols) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        const float *xr = x + r * cols;
        double m = -DBL_MAX, s = 0.0, ys = 0.0;
        for (int64_t c = 0; c < cols; c++) m = xr[c] > m ? xr[c] : m;
        for (int64_t c = 0; c < cols; c++) s += exp((double)xr[c] - m);
        for (int64_t c = 0; c < cols; c++) {
            double v = exp((double)xr[c] - m) / s;
            if (y) y[r * cols + c] = (float)v;
            ys += v;
        }
        if (rowsum) rowsum[r] = (float)ys;
    }
}

/* argmax over the last axis for any f32 tensor (tensor/mod.rs:2245-2269). */
ZO_API void zo_argmax_rows_f32(const float *x, int32_t *arg, int64_t rows, int64_t cols) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        const float *xr = x + r * cols;
        float m = -FLT_MAX;
        for (int64_t c = 0; c < cols; c++) m = fmaxf(xr[c], m);
        int32_t a = INT32_MIN;
        for (int64_t c = 0; c < cols; c++) {
            int32_t idx = (int32_t)(xr[c] == m) * (int32_t)c;
            a = idx > a ? idx : a;
        }
        arg[r] = a;
    }
}

/* ------------------------------------------------------------------------- */
/* dot: zyx/src/tensor/mod.rs:1469-1518                                       */
/* ------------------------------------------------------------------------- */

/* C[m,n] = sum_k A[m,k] * B[k,n], the broadcast-multiply + serial k reduce the
 * reference lowers to. in_dtype is the storage dtype of A and B; products and the
 * accumulator live in float registers; the result is stored as out_dtype
 * (`dot` on bf16 stores bf16, truncating; `dot_dtype(F32)` stores f32).
 *  transb != 0 reads B as [n,k] (Linear's W stored [out,in], linear.rs:38-44), transa != 0
 * reads A as [k,m] (the x.t() of a weight gradient). */
ZO_API void zo_matmul_float(int in_dtype, int out_dtype, const void *a, const void *b, void *c, int64_t m, int64_t n,
                            int64_t k, int transb, int transa) {
#pragma omp parallel for
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
            float acc = 0.0f;
            for (int64_t p = 0; p < k; p++) {
                float x = load_as_f32(a, in_dtype, transa ? p * m + i : i * k + p);
                float y = load_as_f32(b, in_dtype, transb ? j * k + p : p * n + j);
                acc = x * y + acc;
            }
            store_from_f32(c, out_dtype, i * n + j, acc);
        }
}
/* The same product with a double accumulator: tolerance anchor for bf16/f32 GEMM. */
ZO_API void zo_matmul_f64acc(int in_dtype, const void *a, const void *b, double *c, int64_t m, int64_t n, int64_t k,
                             int transb) {
#pragma omp parallel for
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
            double acc = 0.0;
            for (int64_t p = 0; p < k; p++)
                acc += (double)load_as_f32(a, in_dtype, i * k + p) *
                       (double)load_as_f32(b, in_dtype, transb ? j * k + p : p * n + j);
            c[i * n + j] = acc;
        }
}
/* Integer dot is exact (wrapping) in the operand dtype. */
ZO_API void zo_matmul_i64(const int64_t *a, const int64_t *b, int64_t *c, int64_t m, int64_t n, int64_t k) {
#pragma omp parallel for
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
            uint64_t acc = 0;
            for (int64_t p = 0; p < k; p++) acc += (uint64_t)a[i * k + p] * (uint64_t)b[p * n + j];
            c[i * n + j] = (int64_t)acc;
        }
}
ZO_API void zo_matmul_i32(const int32_t *a, const int32_t *b, int32_t *c, int64_t m, int64_t n, int64_t k) {
#pragma omp parallel for
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
            uint32_t acc = 0;
            for (int64_t p = 0; p < k; p++) acc += (uint32_t)a[i * k + p] * (uint32_t)b[p * n + j];
            c[i * n + j] = (int32_t)acc;
        }
}

/* Linear epilogue on an f32 [m,n] tensor: + bias[n] (bias stored as bias_dtype),
 * then act: 0 none, 1 relu, 2 gelu (linear.rs:38-44, elementwise.rs:168-170,289-293). */
ZO_API void zo_bias_act_f32(float *c, const void *bias, int bias_dtype, int64_t m, int64_t n, int act) {
#pragma omp parallel for
    for (int64_t i = 0; i < m; i++)
        for (int64_t j = 0; j < n; j++) {
            float v = c[i * n + j];
            if (bias) v = v + load_as_f32(bias, bias_dtype, j);
            if (act == 1) v = zo_unary(ZO_U_RELU, v);
            else if (act == 2) v = zo_gelu(v);
            c[i * n + j] = v;
        }
}

/* ------------------------------------------------------------------------- */
/* Fused elementwise chains                                                   */
/* ------------------------------------------------------------------------- */

/* Evaluates an accumulator program (the encoding of ZHIP_K_ELEMENTWISE in
 * include/zyx_hip.h; the encoding is this build's, each op's meaning is the reference's:
 * UOp/BOp zyx/src/kernel/ops.rs:187-261 as emitted by zyx/src/codegen/c.rs:290-304,
 * 593-611, composites zyx/src/tensor/elementwise.rs) element by element, the way the C
 * backend's fused kernel would: float registers, narrowing only on the final store.
 * in_desc[k] = dtype | bcast << 8 (bcast 0 full, 1 row vector, 2 column vector, 3 scalar). */
static inline float ew_load(const void *p, int dtype, int64_t i) {
    switch (dtype) {
    case ZO_BF16: return bf16_load(((const uint16_t *)p)[i]);
    case ZO_F16: return f16_load(((const uint16_t *)p)[i]);
    case ZO_F32: return ((const float *)p)[i];
    case ZO_I32: return (float)((const int32_t *)p)[i];
    default: return (float)((const uint8_t *)p)[i];
    }
}
static inline int32_t ew_load_i(const void *p, int dtype, int64_t i) {
    return dtype == ZO_I32 ? ((const int32_t *)p)[i] : (int32_t)((const uint8_t *)p)[i];
}
enum { EW_LOAD = 0, EW_SAVE, EW_NEG, EW_BITNOT, EW_EXP, EW_EXP2, EW_LN, EW_LOG2, EW_RECIPROCAL, EW_SQRT, EW_SIN, EW_COS,
       EW_FLOOR, EW_TRUNC, EW_ABS, EW_ADD, EW_SUB, EW_MUL, EW_DIV, EW_POW, EW_MOD, EW_CMPLT, EW_CMPGT, EW_CMPGE, EW_MAX,
       EW_OR, EW_AND, EW_BITXOR, EW_BITOR, EW_BITAND, EW_SHL, EW_SHR, EW_NOTEQ, EW_EQ, EW_RSUB, EW_RDIV, EW_WHERE,
       EW_MAD, EW_RELU, EW_TANH, EW_GELU, EW_SIGMOID, EW_RSQRT, EW_CAST_INT, EW_GELU_GRAD };

static inline float ew_op_f(int op, float x, float a, float b) {
    switch (op) {
    case EW_LOAD: return a;
    case EW_NEG: return zo_unary(ZO_U_NEG, x);
    case EW_EXP: return zo_unary(ZO_U_EXP, x);
    case EW_EXP2: return zo_unary(ZO_U_EXP2, x);
    case EW_LN: return zo_unary(ZO_U_LN, x);
    case EW_LOG2: return zo_unary(ZO_U_LOG2, x);
    case EW_RECIPROCAL: return zo_unary(ZO_U_RECIPROCAL, x);
    case EW_SQRT: return zo_unary(ZO_U_SQRT, x);
    case EW_SIN: return zo_unary(ZO_U_SIN, x);
    case EW_COS: return zo_unary(ZO_U_COS, x);
    case EW_FLOOR: return zo_unary(ZO_U_FLOOR, x);
    case EW_TRUNC: return zo_unary(ZO_U_TRUNC, x);
    case EW_ABS: return zo_unary(ZO_U_ABS, x);
    case EW_ADD: return zo_binary(ZO_B_ADD, x, a);
    case EW_SUB: return zo_binary(ZO_B_SUB, x, a);
    case EW_MUL: return zo_binary(ZO_B_MUL, x, a);
    case EW_DIV: return zo_binary(ZO_B_DIV, x, a);
    case EW_POW: return zo_binary(ZO_B_POW, x, a);
    case EW_MOD: return zo_binary(ZO_B_MOD, x, a);
    case EW_CMPLT: return zo_binary(ZO_B_CMPLT, x, a);
    case EW_CMPGT: return zo_binary(ZO_B_CMPGT, x, a);
    case EW_CMPGE: return zo_binary(ZO_B_CMPGE, x, a);
    case EW_MAX: return zo_binary(ZO_B_MAX, x, a);
    case EW_OR: return (float)(x != 0.0f || a != 0.0f);
    case EW_AND: return (float)(x != 0.0f && a != 0.0f);
    case EW_NOTEQ: return zo_binary(ZO_B_NOTEQ, x, a);
    case EW_EQ: return zo_binary(ZO_B_EQ, x, a);
    case EW_RSUB: return zo_binary(ZO_B_SUB, a, x);
    case EW_RDIV: return zo_binary(ZO_B_DIV, a, x);
    case EW_WHERE: return x != 0.0f ? a : b;
    case EW_MAD: return x * a + b;
    case EW_RELU: return zo_unary(ZO_U_RELU, x);
    case EW_TANH: return zo_unary(ZO_U_TANH, x);
    case EW_GELU: return zo_unary(ZO_U_GELU, x);
    case EW_SIGMOID: return zo_unary(ZO_U_SIGMOID, x);
    case EW_RSQRT: return zo_unary(ZO_U_RSQRT, x);
    case EW_CAST_INT: return truncf(x);
    case EW_GELU_GRAD: return zo_gelu_grad(x);
    default: return x;
    }
}
static inline int32_t ew_op_i(int op, int32_t x, int32_t a, int32_t b) {
    uint32_t ux = (uint32_t)x, ua = (uint32_t)a;
    switch (op) {
    case EW_LOAD: return a;
    case EW_NEG: return (int32_t)(0u - ux);
    case EW_BITNOT: return ~x;
    case EW_ABS: return x < 0 ? (int32_t)(0u - ux) : x;
    case EW_ADD: return (int32_t)(ux + ua);
    case EW_SUB: return (int32_t)(ux - ua);
    case EW_MUL: return (int32_t)(ux * ua);
    case EW_DIV: return a == 0 ? 0 : (a == -1 ? (int32_t)(0u - ux) : x / a);
    case EW_MOD: return (a == 0 || a == -1) ? 0 : x % a;
    case EW_CMPLT: return x < a;
    case EW_CMPGT: return x > a;
    case EW_CMPGE: return x >= a;
    case EW_MAX: return x > a ? x : a;
    case EW_OR: return x || a;
    case EW_AND: return x && a;
    case EW_BITXOR: return x ^ a;
    case EW_BITOR: return x | a;
    case EW_BITAND: return x & a;
    case EW_SHL: return (int32_t)(ux << (a & 31));
    case EW_SHR: return x >> (a & 31);
    case EW_NOTEQ: return x != a;
    case EW_EQ: return x == a;
    case EW_RSUB: return (int32_t)(ua - ux);
    case EW_RDIV: return x == 0 ? 0 : (x == -1 ? (int32_t)(0u - ua) : a / x);
    case EW_WHERE: return x != 0 ? a : b;
    case EW_MAD: return (int32_t)(ux * ua + (uint32_t)b);
    case EW_RELU: return x > 0 ? x : 0;
    default: return x;
    }
}

ZO_API void zo_ew_chain(int reg_class, int out_dtype, int n_in, const int32_t *in_desc, const void *const *in,
                        int n_instr, const uint32_t *code, const float *consts, void *out, int64_t rows, int64_t cols) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            int64_t i = r * cols + c;
            float fa = 0, ft = 0;
            int32_t ia = 0, it = 0;
            for (int j = 0; j < n_instr; j++) {
                int op = code[j] & 0xff, s[2] = {(int)((code[j] >> 8) & 0xff), (int)((code[j] >> 16) & 0xff)};
                if (op == EW_SAVE) { ft = fa; it = ia; continue; }
                float fv[2] = {0, 0};
                int32_t iv[2] = {0, 0};
                for (int q = 0; q < 2; q++) {
                    int src = s[q];
                    if (src < 4) {
                        if (src >= n_in) continue;
                        int dt = in_desc[src] & 0xff, bc = (in_desc[src] >> 8) & 0xff;
                        int64_t idx = bc == 0 ? i : bc == 1 ? c : bc == 2 ? r : 0;
                        if (reg_class == ZO_I32) iv[q] = ew_load_i(in[src], dt, idx);
                        else fv[q] = ew_load(in[src], dt, idx);
                    } else if (src == 0x10) { fv[q] = ft; iv[q] = it; }
                    else if (src >= 0x20 && src < 0x28) { fv[q] = consts[src - 0x20]; iv[q] = (int32_t)consts[src - 0x20]; }
                }
                if (reg_class == ZO_I32) ia = ew_op_i(op, ia, iv[0], iv[1]);
                else fa = ew_op_f(op, fa, fv[0], fv[1]);
            }
            if (reg_class == ZO_I32) {
                if (out_dtype == ZO_I32) ((int32_t *)out)[i] = ia;
                else ((uint8_t *)out)[i] = (uint8_t)ia;
            } else {
                switch (out_dtype) {
                case ZO_BF16: ((uint16_t *)out)[i] = bf16_store(fa); break;
                case ZO_F16: ((uint16_t *)out)[i] = f16_store(fa); break;
                case ZO_F32: ((float *)out)[i] = fa; break;
                case ZO_I32: ((int32_t *)out)[i] = (int32_t)fa; break; /* C cast: toward zero */
                default: ((uint8_t *)out)[i] = (uint8_t)(int32_t)fa; break;
                }
            }
        }
}


/* ------------------------------------------------------------------------- */
/* Normalisation layers and the classification loss                           */
/* ------------------------------------------------------------------------- */

/* LayerNorm over the last axis (zyx-nn/src/layer_norm.rs:98-135):
 *   mean = sum(x) / n;  var = sum((x - mean)^2) / (n - 1)   (Tensor::var: correction 1,
 *   zyx/src/tensor/reduce_ops.rs:795-805, 111-123)
 *   y = (x - mean) / sqrt(var + eps) (* w) (+ b)
 * evaluated as one fused float-register kernel; storage dtype f32 or bf16. */
ZO_API void zo_layer_norm(int dtype, const void *x, const void *w, const void *b, void *y, int64_t rows, int64_t cols,
                          float eps) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        float s = 0.0f;
        for (int64_t c = 0; c < cols; c++) s = load_as_f32(x, dtype, r * cols + c) + s;
        float mean = s / (float)cols;
        float v = 0.0f;
        for (int64_t c = 0; c < cols; c++) {
            float d = load_as_f32(x, dtype, r * cols + c) - mean;
            v = d * d + v;
        }
        float den = sqrtf(v / (float)(cols - 1) + eps);
        for (int64_t c = 0; c < cols; c++) {
            float o = (load_as_f32(x, dtype, r * cols + c) - mean) / den;
            if (w) o = o * load_as_f32(w, dtype, c);
            if (b) o = o + load_as_f32(b, dtype, c);
            store_from_f32(y, dtype, r * cols + c, o);
        }
    }
}
/* RMSNorm (zyx-nn/src/rms_norm.rs:26-32): x * sqrt(1 / (mean(x*x) + eps)) * scale */
ZO_API void zo_rms_norm(int dtype, const void *x, const void *w, void *y, int64_t rows, int64_t cols, float eps) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        float s = 0.0f;
        for (int64_t c = 0; c < cols; c++) {
            float v = load_as_f32(x, dtype, r * cols + c);
            s = v * v + s;
        }
        float sc = sqrtf(1.0f / (s / (float)cols + eps));
        for (int64_t c = 0; c < cols; c++) {
            float o = load_as_f32(x, dtype, r * cols + c) * sc;
            if (w) o = o * load_as_f32(w, dtype, c);
            store_from_f32(y, dtype, r * cols + c, o);
        }
    }
}
/* Tensor::cross_entropy with class-index targets, reduction None (zyx/src/tensor/mod.rs:
 * 1639-1655): m = x - max_c x; ls = m - ln(sum_c exp(m)); loss = sum_c (-ls[c]) * onehot[c]
 * with onehot = (label == arange) (:1920-1946). grad (optional) is d(gscale * sum_r loss)/dx
 * = (softmax - onehot) * gscale: what the reference's reverse rules for Sub/Exp/Ln/Sum/Max/Mul
 * (zyx/src/graph/autograd.rs:87-134, 155-162) add up to; pinned by finite differences. */
ZO_API void zo_cross_entropy(const float *x, const int32_t *labels, float *loss, float *grad, int64_t rows,
                             int64_t cols, float gscale) {
#pragma omp parallel for
    for (int64_t r = 0; r < rows; r++) {
        const float *xr = x + r * cols;
        float mx = -FLT_MAX, s = 0.0f, l = 0.0f;
        for (int64_t c = 0; c < cols; c++) mx = fmaxf(xr[c], mx);
        for (int64_t c = 0; c < cols; c++) s = expf(xr[c] - mx) + s;
        float lns = logf(s);
        for (int64_t c = 0; c < cols; c++) {
            float ls = (xr[c] - mx) - lns;
            l = (-ls) * (float)(labels[r] == (int32_t)c) + l;
            if (grad) grad[r * cols + c] = (expf(xr[c] - mx) / s - (float)(labels[r] == (int32_t)c)) * gscale;
        }
        if (loss) loss[r] = l;
    }
}

/* ------------------------------------------------------------------------- */
/* conv2d and max-pool                                                        */
/* ------------------------------------------------------------------------- */

/* Tensor::conv (zyx/src/tensor/mod.rs:2583-2680), 4-D NCHW, groups = 1. The reference pads,
 * takes the pool view [bs, 1, cin, 1, oy, ox, ky, kx], multiplies by the weight and sums over
 * (cin, ky, kx) with one serial f32 register accumulator in that order, then adds the bias.
 * Padding is a 0/1 mask multiplied onto a clamped load (zyx/src/kernel/linearize.rs:349-382):
 * for finite inputs that is a zero tap. Restated here as the direct cross-correlation that
 * view reduces to -- the config-4 shape itself is pinned only by this textbook form. */
ZO_API void zo_conv2d(int dtype, int out_dtype, const void *x, const void *w, const void *bias, void *y, int64_t N,
                      int64_t C, int64_t H, int64_t W, int64_t Co, int64_t KH, int64_t KW, int sy, int sx, int py, int px,
                      int dy, int dx, int relu) {
    int64_t OH = (H + 2 * py - dy * (KH - 1) - 1) / sy + 1, OW = (W + 2 * px - dx * (KW - 1) - 1) / sx + 1;
#pragma omp parallel for collapse(2)
    for (int64_t n = 0; n < N; n++)
        for (int64_t co = 0; co < Co; co++)
            for (int64_t oy = 0; oy < OH; oy++)
                for (int64_t ox = 0; ox < OW; ox++) {
                    float acc = 0.0f;
                    for (int64_t c = 0; c < C; c++)
                        for (int64_t ky = 0; ky < KH; ky++)
                            for (int64_t kx = 0; kx < KW; kx++) {
                                int64_t iy = oy * sy - py + ky * dy, ix = ox * sx - px + kx * dx;
                                int ok = iy >= 0 && iy < H && ix >= 0 && ix < W;
                                float xv = ok ? load_as_f32(x, dtype, ((n * C + c) * H + iy) * W + ix) : 0.0f;
                                acc = xv * load_as_f32(w, dtype, ((co * C + c) * KH + ky) * KW + kx) + acc;
                            }
                    /* a 16-bit sum is stored (truncated) before the bias is added to it in a second kernel */
                    if (bias) {
                        if (dtype != ZO_F32 && out_dtype != ZO_F32) {
                            uint16_t t = dtype == ZO_BF16 ? bf16_store(acc) : f16_store(acc);
                            acc = dtype == ZO_BF16 ? bf16_load(t) : f16_load(t);
                        }
                        acc = acc + load_as_f32(bias, dtype, co);
                    }
                    if (relu) acc = (float)(acc > 0.0f) * acc;
                    store_from_f32(y, out_dtype, ((n * Co + co) * OH + oy) * OW + ox, acc);
                }
}

/* Tensor::max_pool (zyx/src/tensor/mod.rs:2706-2741): pad with dtype.min, window view, max. */
ZO_API void zo_max_pool2d(int dtype, const void *x, void *y, int64_t planes, int64_t H, int64_t W, int64_t KH, int64_t KW,
                          int sy, int sx, int py, int px, int dy, int dx) {
    int64_t OH = (H + 2 * py - dy * (KH - 1) - 1) / sy + 1, OW = (W + 2 * px - dx * (KW - 1) - 1) / sx + 1;
    float lowest = dtype == ZO_F32 ? -FLT_MAX : bf16_load(0xff7f);
#pragma omp parallel for
    for (int64_t pl = 0; pl < planes; pl++)
        for (int64_t oy = 0; oy < OH; oy++)
            for (int64_t ox = 0; ox < OW; ox++) {
                float m = lowest;
                for (int64_t ky = 0; ky < KH; ky++)
                    for (int64_t kx = 0; kx < KW; kx++) {
                        int64_t iy = oy * sy - py + ky * dy, ix = ox * sx - px + kx * dx;
                        float v = (iy >= 0 && iy < H && ix >= 0 && ix < W) ? load_as_f32(x, dtype, (pl * H + iy) * W + ix) : lowest;
                        m = fmaxf(v, m);
                    }
                store_from_f32(y, dtype, (pl * OH + oy) * OW + ox, m);
            }
}

/* ---- attention core of CausalSelfAttention::forward (zyx-nn/src/causal_self_attention.rs:36-74) ----------
 * qkv[B,T,3C] is the c_attn output; split([c,c,c],2), reshape [b,t,h,c/h], transpose(1,2) address
 * q/k/v of head h at column h*dh of the first/second/third C columns. att = q.dot(k.t()) * scale,
 * softmax(-1) (max, sub, exp, sum, div: zyx/src/tensor/mod.rs:1457-1461), eval-mode dropout
 * (att / (1-p), zyx/src/tensor/mod.rs:822-828), att.dot(v), transpose(1,2).reshape([b,t,c]).
 * f32 registers, serial sums, one narrowing store for y. lse (optional) = max + ln(sum). */
ZO_API void zo_attention(int dtype, const void *qkv, void *y, float *lse, int64_t B, int64_t T, int64_t H, int64_t dh,
                         float scale, float keep, int causal) {
    const int64_t Cc = H * dh, ld = 3 * Cc;
#pragma omp parallel
    {
        float *s = (float *)malloc(sizeof(float) * (size_t)(T > 0 ? T : 1));
#pragma omp for collapse(2)
        for (int64_t bh = 0; bh < B * H; bh++)
            for (int64_t t = 0; t < T; t++) {
                const int64_t b = bh / H, h = bh % H;
                const int64_t qo = (b * T + t) * ld + h * dh;
                const int64_t n = causal ? t + 1 : T; /* a query sees keys 0..t: the rest are filled with -inf, exp gives 0 */
                for (int64_t j = 0; j < n; j++) {
                    const int64_t ko = (b * T + j) * ld + Cc + h * dh;
                    float a = 0.0f;
                    for (int64_t d = 0; d < dh; d++) a = load_as_f32(qkv, dtype, qo + d) * load_as_f32(qkv, dtype, ko + d) + a;
                    s[j] = a * scale;
                }
                float m = s[0];
                for (int64_t j = 1; j < n; j++) m = fmaxf(m, s[j]);
                float sum = 0.0f;
                for (int64_t j = 0; j < n; j++) {
                    s[j] = expf(s[j] - m);
                    sum = s[j] + sum;
                }
                for (int64_t j = 0; j < n; j++) s[j] = (s[j] / sum) / keep;
                for (int64_t d = 0; d < dh; d++) {
                    float a = 0.0f;
                    for (int64_t j = 0; j < n; j++) a = s[j] * load_as_f32(qkv, dtype, (b * T + j) * ld + 2 * Cc + h * dh + d) + a;
                    store_from_f32(y, dtype, (b * T + t) * Cc + h * dh + d, a);
                }
                if (lse) lse[bh * T + t] = m + logf(sum);
            }
        free(s);
    }
}

/* Gradient of the above w.r.t. qkv given dy[B,T,C] (the chain of autograd rules Mul/Div/Exp/Sub/Sum,
 * zyx/src/graph/autograd.rs:87-134, collapses to the softmax Jacobian; the max term cancels):
 * P = softmax(scale q k^T) / keep; dV = P^T dO; dP = dO V^T / keep; dS = Ps o (dP - rowsum(Ps o dP)),
 * Ps = softmax; dQ = scale dS K; dK = scale dS^T Q. Accumulated in f64, stored in `dtype`. */
ZO_API void zo_attention_bwd(int dtype, const void *qkv, const void *dy, void *dqkv, int64_t B, int64_t T, int64_t H,
                             int64_t dh, float scale, float keep, int causal) {
    const int64_t Cc = H * dh, ld = 3 * Cc;
#pragma omp parallel for
    for (int64_t bh = 0; bh < B * H; bh++) {
        const int64_t b = bh / H, h = bh % H;
        double *P = (double *)malloc(sizeof(double) * (size_t)(T * T + 1));
        double *dS = (double *)malloc(sizeof(double) * (size_t)(T * T + 1));
        for (int64_t t = 0; t < T; t++) {
            const int64_t qo = (b * T + t) * ld + h * dh;
            double m = -INFINITY, sum = 0.0;
            const int64_t n = causal ? t + 1 : T;
            for (int64_t j = n; j < T; j++) P[t * T + j] = dS[t * T + j] = 0.0; /* masked: probability and its gradient are 0 */
            for (int64_t j = 0; j < n; j++) {
                const int64_t ko = (b * T + j) * ld + Cc + h * dh;
                double a = 0.0;
                for (int64_t d = 0; d < dh; d++) a += (double)load_as_f32(qkv, dtype, qo + d) * (double)load_as_f32(qkv, dtype, ko + d);
                P[t * T + j] = a * (double)scale;
                if (P[t * T + j] > m) m = P[t * T + j];
            }
            for (int64_t j = 0; j < n; j++) {
                P[t * T + j] = exp(P[t * T + j] - m);
                sum += P[t * T + j];
            }
            double dot = 0.0;
            for (int64_t j = 0; j < n; j++) {
                P[t * T + j] /= sum;
                double dp = 0.0;
                for (int64_t d = 0; d < dh; d++)
                    dp += (double)load_as_f32(dy, dtype, (b * T + t) * Cc + h * dh + d) *
                          (double)load_as_f32(qkv, dtype, (b * T + j) * ld + 2 * Cc + h * dh + d);
                dS[t * T + j] = dp / (double)keep;
                dot += P[t * T + j] * dS[t * T + j];
            }
            for (int64_t j = 0; j < n; j++) dS[t * T + j] = P[t * T + j] * (dS[t * T + j] - dot);
        }
        for (int64_t t = 0; t < T; t++)
            for (int64_t d = 0; d < dh; d++) {
                double dq = 0.0, dk = 0.0, dv = 0.0;
                for (int64_t j = 0; j < T; j++) {
                    dq += dS[t * T + j] * (double)load_as_f32(qkv, dtype, (b * T + j) * ld + Cc + h * dh + d);
                    dk += dS[j * T + t] * (double)load_as_f32(qkv, dtype, (b * T + j) * ld + h * dh + d);
                    dv += P[j * T + t] / (double)keep * (double)load_as_f32(dy, dtype, (b * T + j) * Cc + h * dh + d);
                }
                store_from_f32(dqkv, dtype, (b * T + t) * ld + h * dh + d, (float)(dq * (double)scale));
                store_from_f32(dqkv, dtype, (b * T + t) * ld + Cc + h * dh + d, (float)(dk * (double)scale));
                store_from_f32(dqkv, dtype, (b * T + t) * ld + 2 * Cc + h * dh + d, (float)dv);
            }
        free(P);
        free(dS);
    }
}

/* ---- gradients of LayerNorm / RMSNorm (zyx-nn/src/layer_norm.rs:98-135, rms_norm.rs:26-32) -----------------
 * The reverse rules of zyx/src/graph/autograd.rs:87-134, 299-379 applied to the forward expressions; f64
 * arithmetic, one store in `dtype`. LayerNorm's variance divides by n-1. w, add, dw, db may be null. */
ZO_API void zo_norm_bwd(int dtype, int rms, const void *x, const void *w, const void *dy, const void *add, void *dx,
                        void *dw, void *db, int64_t rows, int64_t cols, float eps) {
    double *aw = (double *)calloc((size_t)cols + 1, sizeof(double)), *ab = (double *)calloc((size_t)cols + 1, sizeof(double));
    for (int64_t r = 0; r < rows; r++) {
        double mean = 0.0, ss = 0.0;
        for (int64_t c = 0; c < cols; c++) mean += (double)load_as_f32(x, dtype, r * cols + c);
        mean = rms ? 0.0 : mean / (double)cols;
        for (int64_t c = 0; c < cols; c++) {
            double d = (double)load_as_f32(x, dtype, r * cols + c) - mean;
            ss += d * d;
        }
        const double rstd = rms ? sqrt(1.0 / (ss / (double)cols + (double)eps)) : 1.0 / sqrt(ss / (double)(cols - 1) + (double)eps);
        double s1 = 0.0, s2 = 0.0;
        for (int64_t c = 0; c < cols; c++) {
            const double g = (double)load_as_f32(dy, dtype, r * cols + c) * (w ? (double)load_as_f32(w, dtype, c) : 1.0);
            const double xh = ((double)load_as_f32(x, dtype, r * cols + c) - mean) * rstd;
            s1 += g;
            s2 += g * xh;
            aw[c] += (double)load_as_f32(dy, dtype, r * cols + c) * xh;
            ab[c] += (double)load_as_f32(dy, dtype, r * cols + c);
        }
        for (int64_t c = 0; c < cols; c++) {
            const double g = (double)load_as_f32(dy, dtype, r * cols + c) * (w ? (double)load_as_f32(w, dtype, c) : 1.0);
            const double xh = ((double)load_as_f32(x, dtype, r * cols + c) - mean) * rstd;
            double o = rms ? rstd * (g - xh * s2 / (double)cols) : rstd * (g - s1 / (double)cols - xh * s2 / (double)(cols - 1));
            if (add) o += (double)load_as_f32(add, dtype, r * cols + c);
            store_from_f32(dx, dtype, r * cols + c, (float)o);
        }
    }
    for (int64_t c = 0; c < cols; c++) {
        if (dw) store_from_f32(dw, dtype, c, (float)aw[c]);
        if (db) store_from_f32(db, dtype, c, (float)ab[c]);
    }
    free(aw);
    free(ab);
}
