// Fused elementwise chain: one pass over HBM for a whole chain of zyx primitive ops.
//
// zyx fuses chains of UOp/BOp/Cast nodes over same-shape (or broadcast) operands into
// one generated kernel (zyx/src/kernel/ops.rs:187-261, zyx/src/codegen/c.rs:262-306,
// 586-613). Here the chain is a tiny accumulator program interpreted per 4-element
// vector: every branch depends only on kernel arguments, so a wave never diverges and
// the cost per instruction is a few scalar ops on top of the VALU work. Operands are
// fetched straight from memory where the chain names them (128-bit loads for full
// tensors and row vectors), nothing is indexed dynamically in registers.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

template <typename R> __device__ __forceinline__ R from_f32(float v) { return (R)v; }

// ---- operand fetch -------------------------------------------------------------------
template <typename R, int V>
__device__ __forceinline__ void load_elems(const void *__restrict__ base, int dtype, int64_t idx, R (&dst)[V]) {
    switch (dtype) {
    case DT_F32: {
        const float *p = (const float *)base + idx;
        if (V == 4) {
            f32x4 v = *(const f32x4 *)p;
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)v[k];
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)p[k];
        }
        break;
    }
    case DT_I32: {
        const int32_t *p = (const int32_t *)base + idx;
        if (V == 4) {
            i32x4 v = *(const i32x4 *)p;
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)v[k];
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)p[k];
        }
        break;
    }
    case DT_BF16: case DT_F16: {
        const uint16_t *p = (const uint16_t *)base + idx;
        uint16_t h[V];
        if (V == 4) {
            uint2 v = *(const uint2 *)p;
            h[0] = (uint16_t)v.x; h[1] = (uint16_t)(v.x >> 16); h[2 % V] = (uint16_t)v.y; h[3 % V] = (uint16_t)(v.y >> 16);
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) h[k] = p[k];
        }
#pragma unroll
        for (int k = 0; k < V; k++) dst[k] = (R)(dtype == DT_BF16 ? bf16_to_f32(h[k]) : f16_to_f32(h[k]));
        break;
    }
    default: { // U8 / Bool
        const uint8_t *p = (const uint8_t *)base + idx;
#pragma unroll
        for (int k = 0; k < V; k++) dst[k] = (R)p[k];
        break;
    }
    }
}

template <typename R> __device__ __forceinline__ R load_one(const void *__restrict__ base, int dtype, int64_t idx) {
    R d[1];
    load_elems<R, 1>(base, dtype, idx, d);
    return d[0];
}

template <typename R, int V>
__device__ __forceinline__ void fetch(const Elementwise &P, int src, int64_t i0, int64_t row, int64_t col,
                                      const R (&t)[V], R (&dst)[V]) {
    if (src < 4) {
        const void *base = P.in[src];
        int dt = P.in_dtype[src];
        switch (P.in_bcast[src]) {
        case 0: load_elems<R, V>(base, dt, i0, dst); break;
        case 1: load_elems<R, V>(base, dt, col, dst); break;
        case 2: {
            R v = load_one<R>(base, dt, row);
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = v;
            break;
        }
        default: {
            R v = load_one<R>(base, dt, 0);
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = v;
            break;
        }
        }
    } else if (src == 0x10) {
#pragma unroll
        for (int k = 0; k < V; k++) dst[k] = t[k];
    } else {
        R v = from_f32<R>(P.consts[(src - 0x20) & 7]);
#pragma unroll
        for (int k = 0; k < V; k++) dst[k] = v;
    }
}

// ---- scalar op semantics ----------------------------------------------------------------
// tanh as the reference writes it, (e^{2z}-1)/(e^{2z}+1) (elementwise.rs:585-588), made
// saturating where e^{2z} overflows and the reference's own value is inf/inf.
__device__ __forceinline__ float ref_tanh(float z) {
    float e = expf(z + z);
    float r = (e - 1.0f) / (e + 1.0f);
    return (z + z) > 88.0f ? 1.0f : r;
}
__device__ __forceinline__ float ref_gelu(float x) {
    float inner = (x + ((x * x) * x) * 0.044715f) * 0.79788456080286535588f;
    return (x * 0.5f) * (ref_tanh(inner) + 1.0f);
}

__device__ __forceinline__ float ref_gelu_grad(float x) {
    const float k = 0.79788456080286535588f, x2 = x * x;
    const float t = ref_tanh((x + x2 * x * 0.044715f) * k);
    return 0.5f * (1.0f + t) + (0.5f * x) * ((1.0f - t * t) * (k * (1.0f + 0.134145f * x2)));
}

__device__ __forceinline__ float op_f(int op, float x, float a, float b) {
    switch (op) {
    case 0: return a;                                  // LOAD
    case 2: return -x;                                 // NEG
    case 4: return expf(x);
    case 5: return exp2f(x);
    case 6: return logf(x);
    case 7: return log2f(x);
    case 8: return 1.0f / x;
    case 9: return sqrtf(x);
    case 10: return sinf(x);
    case 11: return cosf(x);
    case 12: return floorf(x);
    case 13: return truncf(x);
    case 14: return fabsf(x);
    case 15: return x + a;
    case 16: return x - a;
    case 17: return x * a;
    case 18: return x / a;
    case 19: return exp2f(log2f(x) * a);               // Pow is unfolded to exp2(log2(x)*y)
    case 20: return (float)((int)x % ((int)a == 0 ? 1 : (int)a)); // (int)x % (int)y
    case 21: return x < a ? 1.0f : 0.0f;
    case 22: return x > a ? 1.0f : 0.0f;
    case 23: return x >= a ? 1.0f : 0.0f;
    case 24: return fmaxf(x, a);
    case 25: return (x != 0.0f || a != 0.0f) ? 1.0f : 0.0f;
    case 26: return (x != 0.0f && a != 0.0f) ? 1.0f : 0.0f;
    case 32: return x != a ? 1.0f : 0.0f;
    case 33: return x == a ? 1.0f : 0.0f;
    case 34: return a - x;                             // RSUB
    case 35: return a / x;                             // RDIV
    case 36: return x != 0.0f ? a : b;                 // WHERE
    case 37: return x * a + b;                         // MAD
    case 38: return (x > 0.0f ? 1.0f : 0.0f) * x;      // RELU = (x > 0) * x
    case 39: return ref_tanh(x);
    case 40: return ref_gelu(x);
    case 41: { float e = expf(x); return e / (e + 1.0f); }
    case 42: return sqrtf(1.0f / x);                   // rsqrt = reciprocal().sqrt()
    case 43: return truncf(x);                         // CAST_INT inside a float chain
    case 44: return ref_gelu_grad(x);
    default: return x;
    }
}
__device__ __forceinline__ int32_t op_i(int op, int32_t x, int32_t a, int32_t b) {
    switch (op) {
    case 0: return a;
    case 2: return (int32_t)(0u - (uint32_t)x);
    case 3: return ~x;
    case 14: return x < 0 ? (int32_t)(0u - (uint32_t)x) : x;
    case 15: return (int32_t)((uint32_t)x + (uint32_t)a);
    case 16: return (int32_t)((uint32_t)x - (uint32_t)a);
    case 17: return (int32_t)((uint32_t)x * (uint32_t)a);
    case 18: return a == 0 ? 0 : (a == -1 ? (int32_t)(0u - (uint32_t)x) : x / a);
    case 20: return (a == 0 || a == -1) ? 0 : x % a;
    case 21: return x < a;
    case 22: return x > a;
    case 23: return x >= a;
    case 24: return x > a ? x : a;
    case 25: return (x != 0) || (a != 0);
    case 26: return (x != 0) && (a != 0);
    case 27: return x ^ a;
    case 28: return x | a;
    case 29: return x & a;
    case 30: return (int32_t)((uint32_t)x << (a & 31));
    case 31: return x >> (a & 31);
    case 32: return x != a;
    case 33: return x == a;
    case 34: return (int32_t)((uint32_t)a - (uint32_t)x);
    case 35: return x == 0 ? 0 : (x == -1 ? (int32_t)(0u - (uint32_t)a) : a / x);
    case 36: return x != 0 ? a : b;
    case 37: return (int32_t)((uint32_t)x * (uint32_t)a + (uint32_t)b);
    case 38: return x > 0 ? x : 0;
    default: return x;
    }
}
template <typename R> __device__ __forceinline__ R apply(int op, R x, R a, R b);
template <> __device__ __forceinline__ float apply<float>(int op, float x, float a, float b) { return op_f(op, x, a, b); }
template <> __device__ __forceinline__ int32_t apply<int32_t>(int op, int32_t x, int32_t a, int32_t b) {
    return op_i(op, x, a, b);
}

// ---- result store ---------------------------------------------------------------------
template <typename R, int V>
__device__ __forceinline__ void store_elems(void *__restrict__ base, int dtype, int64_t idx, const R (&v)[V]) {
    switch (dtype) {
    case DT_F32: {
        float *p = (float *)base + idx;
        if (V == 4) *(f32x4 *)p = f32x4{(float)v[0], (float)v[1 % V], (float)v[2 % V], (float)v[3 % V]};
        else {
#pragma unroll
            for (int k = 0; k < V; k++) p[k] = (float)v[k];
        }
        break;
    }
    case DT_I32: {
        int32_t *p = (int32_t *)base + idx;
        if (V == 4) *(i32x4 *)p = i32x4{(int32_t)v[0], (int32_t)v[1 % V], (int32_t)v[2 % V], (int32_t)v[3 % V]};
        else {
#pragma unroll
            for (int k = 0; k < V; k++) p[k] = (int32_t)v[k];
        }
        break;
    }
    case DT_BF16: case DT_F16: {
        uint16_t h[V];
#pragma unroll
        for (int k = 0; k < V; k++) h[k] = dtype == DT_BF16 ? f32_to_bf16_trunc((float)v[k]) : f32_to_f16_trunc((float)v[k]);
        uint16_t *p = (uint16_t *)base + idx;
        if (V == 4) *(uint2 *)p = make_uint2((uint32_t)h[0] | ((uint32_t)h[1 % V] << 16), (uint32_t)h[2 % V] | ((uint32_t)h[3 % V] << 16));
        else {
#pragma unroll
            for (int k = 0; k < V; k++) p[k] = h[k];
        }
        break;
    }
    default: { // U8 / Bool: (uint8_t)x
        uint8_t *p = (uint8_t *)base + idx;
#pragma unroll
        for (int k = 0; k < V; k++) p[k] = (uint8_t)(int32_t)v[k];
        break;
    }
    }
}

template <typename R, int V> __global__ __launch_bounds__(256) void elementwise_k(const Elementwise P) {
    const int64_t n = P.rows * P.cols;
    const int64_t nvec = n / V;
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += stride) {
        const int64_t i0 = v * V;
        int64_t row = 0, col = 0;
        if (P.need_rowcol) {
            if (n < (1ll << 31)) {
                uint32_t r = (uint32_t)i0 / (uint32_t)P.cols;
                row = r;
                col = (uint32_t)i0 - r * (uint32_t)P.cols;
            } else {
                row = i0 / P.cols;
                col = i0 - row * P.cols;
            }
        }
        R acc[V], t[V], a[V], b[V];
#pragma unroll
        for (int k = 0; k < V; k++) acc[k] = t[k] = a[k] = b[k] = (R)0;
        for (int j = 0; j < P.n_instr; j++) {
            const uint32_t ins = P.code[j];
            const int op = ins & 0xff, sa = (ins >> 8) & 0xff, sb = (ins >> 16) & 0xff;
            if (op == 1) { // SAVE
#pragma unroll
                for (int k = 0; k < V; k++) t[k] = acc[k];
                continue;
            }
            const bool unary = (op >= 2 && op <= 14) || (op >= 38);
            if (!unary) fetch<R, V>(P, sa, i0, row, col, t, a);
            if (op == 36 || op == 37) fetch<R, V>(P, sb, i0, row, col, t, b);
#pragma unroll
            for (int k = 0; k < V; k++) acc[k] = apply<R>(op, acc[k], a[k], b[k]);
        }
        store_elems<R, V>(P.out, P.out_dtype, i0, acc);
    }
}

} // namespace

hipError_t elementwise(const Elementwise &p, hipStream_t st) {
    const int64_t n = p.rows * p.cols;
    if (n <= 0) return hipSuccess;
    bool vec = n % 4 == 0 && reinterpret_cast<uintptr_t>(p.out) % 16 == 0;
    for (int k = 0; k < p.n_in; k++) {
        if (p.in_bcast[k] == 0 || p.in_bcast[k] == 1) vec = vec && reinterpret_cast<uintptr_t>(p.in[k]) % 16 == 0;
        if (p.in_bcast[k] == 1 || p.in_bcast[k] == 2) vec = vec && p.cols % 4 == 0;
    }
    const int64_t nvec = vec ? n / 4 : n;
    int64_t blocks = (nvec + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32; // grid-stride beyond 32 workgroups per CU
    dim3 grid((unsigned)blocks), block(256);
    if (p.reg_class == DT_I32) {
        if (vec) hipLaunchKernelGGL((elementwise_k<int32_t, 4>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((elementwise_k<int32_t, 1>), grid, block, 0, st, p);
    } else {
        if (vec) hipLaunchKernelGGL((elementwise_k<float, 4>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((elementwise_k<float, 1>), grid, block, 0, st, p);
    }
    return hipGetLastError();
}

} // namespace zk
