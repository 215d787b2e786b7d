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
#include "ew_ops.hpp"
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
        if (V % 4 == 0) {
#pragma unroll
            for (int q = 0; q < V / 4; q++) {
                f32x4 v = *(const f32x4 *)(p + 4 * q);
#pragma unroll
                for (int k = 0; k < 4; k++) dst[(4 * q + k) % V] = (R)v[k];
            }
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)p[k];
        }
        break;
    }
    case DT_I32: {
        const int32_t *p = (const int32_t *)base + idx;
        if (V % 4 == 0) {
#pragma unroll
            for (int q = 0; q < V / 4; q++) {
                i32x4 v = *(const i32x4 *)(p + 4 * q);
#pragma unroll
                for (int k = 0; k < 4; k++) dst[(4 * q + k) % V] = (R)v[k];
            }
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)p[k];
        }
        break;
    }
    case DT_BF16: case DT_F16: {
        const uint16_t *p = (const uint16_t *)base + idx;
        uint16_t h[V];
        if (V == 8) {
            i32x4 v = *(const i32x4 *)p;
#pragma unroll
            for (int q = 0; q < 4; q++) {
                h[(2 * q) % V] = (uint16_t)v[q];
                h[(2 * q + 1) % V] = (uint16_t)((uint32_t)v[q] >> 16);
            }
        } else if (V == 4) {
            uint2 v = *(const uint2 *)p;
            h[0] = (uint16_t)v.x; h[1 % V] = (uint16_t)(v.x >> 16); h[2 % V] = (uint16_t)v.y; h[3 % V] = (uint16_t)(v.y >> 16);
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) h[k] = p[k];
        }
        if (dtype == DT_BF16) { // uniform branch: only one of the two conversions is executed
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)bf16_to_f32(h[k]);
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) dst[k] = (R)f16_to_f32(h[k]);
        }
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

template <typename R> __device__ __forceinline__ R apply(int op, R x, R a, R b);
template <> __device__ __forceinline__ float apply<float>(int op, float x, float a, float b) { return zkew::op_f(op, x, a, b); }
template <> __device__ __forceinline__ int32_t apply<int32_t>(int op, int32_t x, int32_t a, int32_t b) {
    return zkew::op_i(op, x, a, b);
}

// ---- result store ---------------------------------------------------------------------
template <typename R, int V>
__device__ __forceinline__ void store_elems(void *__restrict__ base, int dtype, int64_t idx, const R (&v)[V]) {
    switch (dtype) {
    case DT_F32: {
        float *p = (float *)base + idx;
        if (V % 4 == 0) {
#pragma unroll
            for (int q = 0; q < V / 4; q++)
                *(f32x4 *)(p + 4 * q) = f32x4{(float)v[(4 * q) % V], (float)v[(4 * q + 1) % V], (float)v[(4 * q + 2) % V], (float)v[(4 * q + 3) % V]};
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) p[k] = (float)v[k];
        }
        break;
    }
    case DT_I32: {
        int32_t *p = (int32_t *)base + idx;
        if (V % 4 == 0) {
#pragma unroll
            for (int q = 0; q < V / 4; q++)
                *(i32x4 *)(p + 4 * q) = i32x4{(int32_t)v[(4 * q) % V], (int32_t)v[(4 * q + 1) % V], (int32_t)v[(4 * q + 2) % V], (int32_t)v[(4 * q + 3) % V]};
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) p[k] = (int32_t)v[k];
        }
        break;
    }
    case DT_BF16: case DT_F16: {
        uint16_t h[V];
        if (dtype == DT_BF16) {
#pragma unroll
            for (int k = 0; k < V; k++) h[k] = f32_to_bf16_trunc((float)v[k]);
        } else {
#pragma unroll
            for (int k = 0; k < V; k++) h[k] = f32_to_f16_trunc((float)v[k]);
        }
        uint16_t *p = (uint16_t *)base + idx;
        if (V == 8) {
            i32x4 w;
#pragma unroll
            for (int q = 0; q < 4; q++) w[q] = (int32_t)((uint32_t)h[(2 * q) % V] | ((uint32_t)h[(2 * q + 1) % V] << 16));
            *(i32x4 *)p = w;
        } else if (V == 4) *(uint2 *)p = make_uint2((uint32_t)h[0] | ((uint32_t)h[1 % V] << 16), (uint32_t)h[2 % V] | ((uint32_t)h[3 % V] << 16));
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
    // 16-bit results take 8 elements per thread and step, so that their stores (and 16-bit loads) are 128-bit too
    bool vec8 = vec && n % 8 == 0 && dtype_size(p.out_dtype) == 2;
    for (int k = 0; k < p.n_in; k++)
        if (p.in_bcast[k] == 1 || p.in_bcast[k] == 2) vec8 = vec8 && p.cols % 8 == 0;
    const int64_t nvec = vec8 ? n / 8 : (vec ? n / 4 : n);
    int64_t blocks = (nvec + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32; // grid-stride beyond 32 workgroups per CU
    dim3 grid((unsigned)blocks), block(256);
    if (p.reg_class == DT_I32) {
        if (vec8) hipLaunchKernelGGL((elementwise_k<int32_t, 8>), grid, block, 0, st, p);
        else if (vec) hipLaunchKernelGGL((elementwise_k<int32_t, 4>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((elementwise_k<int32_t, 1>), grid, block, 0, st, p);
    } else {
        if (vec8) hipLaunchKernelGGL((elementwise_k<float, 8>), grid, block, 0, st, p);
        else if (vec) hipLaunchKernelGGL((elementwise_k<float, 4>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((elementwise_k<float, 1>), grid, block, 0, st, p);
    }
    return hipGetLastError();
}

} // namespace zk
