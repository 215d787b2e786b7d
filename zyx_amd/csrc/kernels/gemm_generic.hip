// General GEMM for every shape, layout and float dtype the fast bf16 kernel does not take:
// f32 (v_mfma_f32_32x32x2_f32), and bf16 / f16 with ragged or small M, N, K
// (v_mfma_f32_32x32x16_{bf16,f16}). C = op(A) . op(B) (+ bias) (ReLU | GELU), f32
// accumulation, result stored as f32 or narrowed to the operand dtype with the C backend's
// truncating stores (zyx/src/codegen/c.rs:456-497).
//
// This is the Linear / dot of the small configs (zyx-nn/src/linear.rs:38-44,
// zyx/src/tensor/mod.rs:1469-1518), e.g. the 784 -> 128 -> 10 MLP, and of the backward
// products dW = X^T . dY, dX = dY . W that autograd's Mul/Expand/Reduce rules collapse to
// (zyx/src/graph/autograd.rs:120-125 and the rules kept in comments at :195-242, 269-295).
//
// 64 x 64 tile per 256-thread workgroup, 2 x 2 waves of one 32 x 32 MFMA tile each, K step
// 32. Operands are read with bounds checks (zero fill) straight from their natural layout,
// coalesced along whichever index is contiguous, and laid down K-contiguous in LDS with a
// row pad (8 elements for 16-bit types, 1 for f32), so fragment reads are the same for all four layouts.
// Small f32 problems (at most 256 tiles of 32 x 32) take gemm_small_f32_k instead: one launch, no staging.
#include <algorithm>

#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int GM = 64, GN = 64, GK = 32;
// LDS row padding: 16-bit rows of 80 bytes keep 128-bit fragment reads of 16 consecutive rows on distinct banks;
// f32 rows of 33 words do the same for the one-word reads of 32 consecutive rows.
template <typename S> constexpr int gpad() { return sizeof(S) == 4 ? 1 : 8; }

template <int DT> struct GT;
template <> struct GT<DT_F32> {
    typedef float S;
    static __device__ __forceinline__ float zero() { return 0.0f; }
};
template <> struct GT<DT_BF16> {
    typedef uint16_t S;
    static __device__ __forceinline__ uint16_t zero() { return 0; }
};
template <> struct GT<DT_F16> {
    typedef uint16_t S;
    static __device__ __forceinline__ uint16_t zero() { return 0; }
};

__device__ __forceinline__ float gelu_ref(float x) { // zyx/src/tensor/elementwise.rs:168-170, saturating tanh
    float inner = (x + ((x * x) * x) * 0.044715f) * 0.79788456080286535588f;
    float e = expf(inner + inner);
    float t = (inner + inner) > 88.0f ? 1.0f : (e - 1.0f) / (e + 1.0f);
    return (x * 0.5f) * (t + 1.0f);
}

// Copies a [rows x GK] operand tile into LDS as dst[row][k]. `rs`/`ks` are the element
// strides of the row index (m or n) and of k in global memory; one of them is 1.
template <typename S>
__device__ __forceinline__ void fill_tile(S *__restrict__ dst, const S *__restrict__ src, int64_t rs, int64_t ks,
                                          int64_t row0, int64_t k0, int64_t rows, int64_t K, S zero) {
    constexpr int GPAD = gpad<S>();
    const int t = threadIdx.x;
    if (ks == 1) { // K contiguous: consecutive threads walk along k
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int idx = e * 256 + t, r = idx >> 5, k = idx & 31;
            const int64_t gr = row0 + r, gk = k0 + k;
            dst[r * (GK + GPAD) + k] = (gr < rows && gk < K) ? src[gr * rs + gk] : zero;
        }
    } else { // row index contiguous: consecutive threads walk along the rows
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int idx = e * 256 + t, k = idx >> 6, r = idx & 63;
            const int64_t gr = row0 + r, gk = k0 + k;
            dst[r * (GK + GPAD) + k] = (gr < rows && gk < K) ? src[gr * rs + gk * ks] : zero;
        }
    }
}

template <int DT, int ODT>
__global__ __launch_bounds__(256) void gemm_generic_k(const GemmGeneric p) {
    typedef typename GT<DT>::S S;
    constexpr int GPAD = gpad<S>();
    __shared__ __attribute__((aligned(16))) S As[GM * (GK + GPAD)];
    __shared__ __attribute__((aligned(16))) S Bs[GN * (GK + GPAD)];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t m0 = (int64_t)blockIdx.y * GM, n0 = (int64_t)blockIdx.x * GN;
    // split-K: blockIdx.z = batch * splits + split; a split multiplies K range [k_lo, k_hi) and stores its raw
    // f32 partial tile into slice (batch, split) of the workspace, which gemm_generic_fold_k sums
    const int split = p.splits > 1 ? blockIdx.z % p.splits : 0, bz = p.splits > 1 ? blockIdx.z / p.splits : blockIdx.z;
    const int64_t k_lo = (int64_t)split * p.k_len, k_hi = p.splits > 1 ? (k_lo + p.k_len < p.K ? k_lo + p.k_len : p.K) : p.K;
    const S *A = (const S *)p.A + (int64_t)bz * p.batch_a, *B = (const S *)p.B + (int64_t)bz * p.batch_b;
    const int64_t a_rs = p.trans_a ? 1 : p.K, a_ks = p.trans_a ? p.M : 1;
    const int64_t b_rs = p.trans_b ? p.K : 1, b_ks = p.trans_b ? 1 : p.N;

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;

    for (int64_t k0 = k_lo; k0 < k_hi; k0 += GK) {
        __syncthreads(); // previous step's fragment reads are done
        fill_tile<S>(As, A, a_rs, a_ks, m0, k0, p.M, k_hi, GT<DT>::zero());
        fill_tile<S>(Bs, B, b_rs, b_ks, n0, k0, p.N, k_hi, GT<DT>::zero());
        __syncthreads();
        const S *ar = As + (wm * 32 + (lane & 31)) * (GK + GPAD);
        const S *br = Bs + (wn * 32 + (lane & 31)) * (GK + GPAD);
        if (DT == DT_F32) {
#pragma unroll
            for (int ks = 0; ks < GK; ks += 2) {
                float a = ((const float *)ar)[ks + (lane >> 5)], b = ((const float *)br)[ks + (lane >> 5)];
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int ks = 0; ks < GK; ks += 16) {
                const int off = ks + (lane >> 5) * 8;
                if (DT == DT_BF16) {
                    bf16x8 a = *(const bf16x8 *)((const uint16_t *)ar + off), b = *(const bf16x8 *)((const uint16_t *)br + off);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
                } else {
                    f16x8 a = *(const f16x8 *)((const uint16_t *)ar + off), b = *(const f16x8 *)((const uint16_t *)br + off);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
                }
            }
        }
    }

    // register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the 32 x 32 tile
    const int64_t col = n0 + wn * 32 + (lane & 31);
    if (col >= p.N) return; // no barrier follows
    if (p.splits > 1) {
        float *W = (float *)p.workspace + ((int64_t)bz * p.splits + split) * p.M * p.N;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int64_t row = m0 + wm * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (row < p.M) W[row * p.N + col] = acc[r];
        }
        return;
    }
    float bv = 0.0f;
    if (p.epilogue >= 1) {
        if (p.bias_dtype == DT_BF16) bv = bf16_to_f32(((const uint16_t *)p.bias)[col]);
        else if (p.bias_dtype == DT_F16) bv = f16_to_f32(((const uint16_t *)p.bias)[col]);
        else bv = ((const float *)p.bias)[col];
    }
    char *C = (char *)p.C + (int64_t)blockIdx.z * p.batch_c * (ODT == DT_F32 ? 4 : 2);
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int64_t row = m0 + wm * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (row >= p.M) continue;
        float v = acc[r] * p.alpha;
        if (p.epilogue >= 1) v += bv;
        if (p.epilogue == 2) v = (v > 0.0f ? 1.0f : 0.0f) * v;
        if (p.epilogue == 3) v = gelu_ref(v);
        const int64_t o = row * p.N + col;
        if (p.residual) {
            const char *R = (const char *)p.residual + (int64_t)blockIdx.z * p.batch_c * (ODT == DT_F32 ? 4 : 2);
            const float r = ODT == DT_F32 ? ((const float *)R)[o] : ODT == DT_BF16 ? bf16_to_f32(((const uint16_t *)R)[o]) : f16_to_f32(((const uint16_t *)R)[o]);
            v = p.residual_is_mask ? (r > 0.0f ? 1.0f : 0.0f) * v : v + r;
        }
        if (ODT == DT_F32) ((float *)C)[o] = v;
        else if (ODT == DT_BF16) ((uint16_t *)C)[o] = f32_to_bf16_trunc(v);
        else ((uint16_t *)C)[o] = f32_to_f16_trunc(v);
    }
}

// Sums the split-K partials [batch, splits, M, N] and applies alpha, bias, activation, residual and the store dtype.
template <int ODT> __global__ __launch_bounds__(256) void gemm_generic_fold_k(const GemmGeneric p) {
    const int64_t MN = p.M * p.N, i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= MN * p.batch) return;
    const int64_t bz = i / MN, o = i - bz * MN, col = o % p.N;
    const float *W = (const float *)p.workspace + bz * p.splits * MN + o;
    float a = W[0];
    for (int z = 1; z < p.splits; z++) a += W[(int64_t)z * MN];
    float v = a * p.alpha;
    if (p.epilogue >= 1) {
        if (p.bias_dtype == DT_BF16) v += bf16_to_f32(((const uint16_t *)p.bias)[col]);
        else if (p.bias_dtype == DT_F16) v += f16_to_f32(((const uint16_t *)p.bias)[col]);
        else v += ((const float *)p.bias)[col];
    }
    if (p.epilogue == 2) v = (v > 0.0f ? 1.0f : 0.0f) * v;
    if (p.epilogue == 3) v = gelu_ref(v);
    const int64_t oo = bz * p.batch_c + o;
    if (p.residual) {
        const float r = ODT == DT_F32 ? ((const float *)p.residual)[oo] : ODT == DT_BF16 ? bf16_to_f32(((const uint16_t *)p.residual)[oo]) : f16_to_f32(((const uint16_t *)p.residual)[oo]);
        v = p.residual_is_mask ? (r > 0.0f ? 1.0f : 0.0f) * v : v + r;
    }
    if (ODT == DT_F32) ((float *)p.C)[oo] = v;
    else if (ODT == DT_BF16) ((uint16_t *)p.C)[oo] = f32_to_bf16_trunc(v);
    else ((uint16_t *)p.C)[oo] = f32_to_f16_trunc(v);
}

// Small f32 products (the layers and gradients of an MLP on a batch of 64): launch latency and round trips to memory
// decide, not arithmetic. One workgroup per 32 x 32 tile of C; its NW waves split K and each accumulates a partial
// tile with v_mfma_f32_32x32x2_f32 from operands read straight from memory into registers (no staging, no barrier in
// the K loop, 8 independent loads per operand in flight); the partials meet in LDS and are summed in wave order, then
// the epilogue runs once. One launch where split-K over the 64 x 64 kernel needs a second one to fold.
// The two halves of a wave take the two halves of the wave's K slice, so each lane walks consecutive k: an operand
// stored with k contiguous (AV / BV: 16-byte aligned rows) is read 4 elements per load, one stored with the row index
// contiguous is read one element per load, coalesced across the 32 lanes of a half.
template <bool VEC>
__device__ __forceinline__ void load8(const float *__restrict__ row, int64_t ks, int64_t k0, int64_t k_hi, int64_t K, bool ok,
                                      float (&v)[8]) {
    if (VEC) {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int64_t k = k0 + 4 * q;
            const f32x4 t = *(const f32x4 *)(row + min(k, K - 4));
            const bool live = ok && k < k_hi; // k and k_hi are multiples of 4: a load is live or dead as a whole
#pragma unroll
            for (int e = 0; e < 4; e++) v[4 * q + e] = live ? t[e] : 0.0f;
        }
    } else {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int64_t k = k0 + u;
            const float t = row[min(k, K - 1) * ks];
            v[u] = ok && k < k_hi ? t : 0.0f;
        }
    }
}

template <int NW, bool AV, bool BV> __global__ __launch_bounds__(64 * NW) void gemm_small_f32_k(const GemmGeneric p) {
    __shared__ float part[NW][32 * 33];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = lane >> 5, l32 = lane & 31;
    const int64_t m0 = (int64_t)blockIdx.y * 32, n0 = (int64_t)blockIdx.x * 32, bz = blockIdx.z;
    const float *A = (const float *)p.A + bz * p.batch_a, *B = (const float *)p.B + bz * p.batch_b;
    const int64_t a_rs = p.trans_a ? 1 : p.K, a_ks = p.trans_a ? p.M : 1;
    const int64_t b_rs = p.trans_b ? p.K : 1, b_ks = p.trans_b ? 1 : p.N;
    int64_t half = ((p.K + NW - 1) / NW + 1) / 2;                    // k per lane half
    if (AV || BV) half = (half + 3) / 4 * 4;
    const int64_t k_lo = min(p.K, (2 * wave + h) * half), k_hi = min(p.K, k_lo + half);
    const int64_t row = m0 + l32, col = n0 + l32;
    const bool row_ok = row < p.M, col_ok = col < p.N;
    const float *ap = A + min(row, p.M - 1) * a_rs, *bp = B + min(col, p.N - 1) * b_rs;

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;
    for (int64_t s0 = 0; s0 < half; s0 += 8) { // both halves run the same number of steps: the MFMA needs the whole wave
        float a[8], b[8];
        load8<AV>(ap, a_ks, k_lo + s0, k_hi, p.K, row_ok, a);
        load8<BV>(bp, b_ks, k_lo + s0, k_hi, p.K, col_ok, b);
#pragma unroll
        for (int u = 0; u < 8; u++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
    }
    // register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of the tile
#pragma unroll
    for (int r = 0; r < 16; r++) part[wave][((r >> 2) * 8 + h * 4 + (r & 3)) * 33 + l32] = acc[r];
    __syncthreads();
    for (int e = threadIdx.x; e < 1024; e += 64 * NW) {
        const int rr = e >> 5, cc = e & 31;
        const int64_t orow = m0 + rr, ocol = n0 + cc;
        if (orow >= p.M || ocol >= p.N) continue;
        float sum = part[0][rr * 33 + cc];
#pragma unroll
        for (int w = 1; w < NW; w++) sum += part[w][rr * 33 + cc];
        float v = sum * p.alpha;
        if (p.epilogue >= 1) {
            if (p.bias_dtype == DT_BF16) v += bf16_to_f32(((const uint16_t *)p.bias)[ocol]);
            else if (p.bias_dtype == DT_F16) v += f16_to_f32(((const uint16_t *)p.bias)[ocol]);
            else v += ((const float *)p.bias)[ocol];
        }
        if (p.epilogue == 2) v = (v > 0.0f ? 1.0f : 0.0f) * v;
        if (p.epilogue == 3) v = gelu_ref(v);
        const int64_t o = bz * p.batch_c + orow * p.N + ocol;
        if (p.residual) {
            const float r = ((const float *)p.residual)[o];
            v = p.residual_is_mask ? (r > 0.0f ? 1.0f : 0.0f) * v : v + r;
        }
        ((float *)p.C)[o] = v;
    }
}

// waves per tile of the small kernel: about 16 k per wave, at most 8 waves; 0: the shape goes to the 64 x 64 kernel
int gemm_small_waves(const GemmGeneric &p) {
    if (p.dtype != DT_F32 || p.out_dtype != DT_F32 || p.K < 1) return 0;
    const int64_t tiles = ((p.M + 31) / 32) * ((p.N + 31) / 32) * p.batch;
    if (tiles > 256 || (p.N + 31) / 32 > 65535 || (p.M + 31) / 32 > 65535) return 0;
    int nw = 1;
    while (nw < 8 && p.K > 16 * nw) nw *= 2;
    return nw;
}

} // namespace

// Few output tiles and a long K (the weight-gradient and first-layer products of a small MLP): split K over
// workgroups so the chip has work and every workgroup waits for few round trips to memory.
int gemm_generic_splits(int64_t M, int64_t N, int64_t K, int64_t batch, int64_t *k_len) {
    const int64_t tiles = ((M + GM - 1) / GM) * ((N + GN - 1) / GN) * batch, steps = (K + GK - 1) / GK;
    int64_t s = 1;
    if (tiles < 128 && steps >= 2) s = std::min<int64_t>(std::min<int64_t>(steps, 256 / tiles), 64);
    if (s < 1) s = 1;
    const int64_t len = (steps + s - 1) / s * GK;
    s = (K + len - 1) / len;
    if (k_len) *k_len = len;
    return (int)s;
}
uint64_t gemm_generic_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t batch) {
    const int s = gemm_generic_splits(M, N, K, batch, nullptr);
    return s > 1 ? (uint64_t)s * batch * M * N * 4 : 0;
}

hipError_t gemm_generic(const GemmGeneric &p0, hipStream_t st) {
    GemmGeneric p = p0;
    if (p.M <= 0 || p.N <= 0 || p.batch <= 0) return hipSuccess;
    if (p.K < 0 || (p.M + GM - 1) / GM > 65535 || p.batch > 65535) return hipErrorInvalidValue;
    if (const int nw = gemm_small_waves(p)) {
        dim3 grid((unsigned)((p.N + 31) / 32), (unsigned)((p.M + 31) / 32), (unsigned)p.batch);
        // k-contiguous operands whose rows start 16-byte aligned take 4 elements per load
        const bool k4 = p.K % 4 == 0 && p.K >= 4;
        const bool av = k4 && !p.trans_a && (uintptr_t)p.A % 16 == 0 && p.batch_a % 4 == 0;
        const bool bv = k4 && p.trans_b && (uintptr_t)p.B % 16 == 0 && p.batch_b % 4 == 0;
#define ZK_S(NW) \
    do { \
        if (av && bv) hipLaunchKernelGGL((gemm_small_f32_k<NW, true, true>), grid, dim3(64 * NW), 0, st, p); \
        else if (av) hipLaunchKernelGGL((gemm_small_f32_k<NW, true, false>), grid, dim3(64 * NW), 0, st, p); \
        else if (bv) hipLaunchKernelGGL((gemm_small_f32_k<NW, false, true>), grid, dim3(64 * NW), 0, st, p); \
        else hipLaunchKernelGGL((gemm_small_f32_k<NW, false, false>), grid, dim3(64 * NW), 0, st, p); \
    } while (0)
        switch (nw) {
        case 1: ZK_S(1); break;
        case 2: ZK_S(2); break;
        case 4: ZK_S(4); break;
        default: ZK_S(8); break;
        }
#undef ZK_S
        return hipGetLastError();
    }
    if (gemm_f32_tiled_ok(p)) return gemm_f32_tiled(p, st);
    p.splits = gemm_generic_splits(p.M, p.N, p.K, p.batch, &p.k_len);
    if (p.splits > 1 && (!p.workspace || (int64_t)p.batch * p.splits > 65535)) return hipErrorInvalidValue;
    dim3 grid((unsigned)((p.N + GN - 1) / GN), (unsigned)((p.M + GM - 1) / GM), (unsigned)(p.batch * p.splits)), block(256);
#define ZK_G(D, O) hipLaunchKernelGGL((gemm_generic_k<D, O>), grid, block, 0, st, p)
    if (p.dtype == DT_F32 && p.out_dtype == DT_F32) ZK_G(DT_F32, DT_F32);
    else if (p.dtype == DT_BF16 && p.out_dtype == DT_F32) ZK_G(DT_BF16, DT_F32);
    else if (p.dtype == DT_BF16 && p.out_dtype == DT_BF16) ZK_G(DT_BF16, DT_BF16);
    else if (p.dtype == DT_F16 && p.out_dtype == DT_F32) ZK_G(DT_F16, DT_F32);
    else if (p.dtype == DT_F16 && p.out_dtype == DT_F16) ZK_G(DT_F16, DT_F16);
    else return hipErrorInvalidValue;
#undef ZK_G
    if (p.splits > 1) {
        dim3 fg((unsigned)((p.M * p.N * p.batch + 255) / 256));
        if (p.out_dtype == DT_F32) hipLaunchKernelGGL((gemm_generic_fold_k<DT_F32>), fg, block, 0, st, p);
        else if (p.out_dtype == DT_BF16) hipLaunchKernelGGL((gemm_generic_fold_k<DT_BF16>), fg, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_generic_fold_k<DT_F16>), fg, block, 0, st, p);
    }
    return hipGetLastError();
}

} // namespace zk
