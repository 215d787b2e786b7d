// Fused row softmax (+ row sum of the result, + row argmax of the result), f32; bf16 / f16 storage further down.
//
// Computes what zyx evaluates as >= 5 kernels for
//   y = x.softmax([-1]); s = y.sum([-1]); a = y.argmax_axis(-1)
// (zyx/src/tensor/mod.rs:1457-1461, 2245-2269; zyx/src/tensor/reduce_ops.rs:45-147)
// in one pass over HBM: x is read once, y written once.
//
// Register-resident variants. Many full rows of 1024 / 2048 / 4096 columns: four waves share a row (softmax_rows_split_k
// below; the benchmark's shape). Otherwise: one 64-lane wave owns one row of up to 4096 columns,
// each lane holding NV float4 (lane + 64*j addressing, so every load/store
// instruction of a wave covers 1 KiB of consecutive bytes). The three row
// reductions (max, sum of exp, sum/argmax of y) are DPP + readlane wave reductions:
// no LDS, no barriers. Four waves per workgroup -> rows/4 workgroups.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

// FULL: cols == 256*NV exactly, so no lane is ever masked.
template <int NV, bool FULL, bool WY, bool WS, bool WA>
__global__ __launch_bounds__(256) void softmax_rows_wave_k(const float *__restrict__ x, float *__restrict__ y,
                                                           float *__restrict__ rowsum, int32_t *__restrict__ arg,
                                                           int rows, int cols) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return; // whole wave leaves together; nothing below synchronises across waves
    const int nvec = cols >> 2;
    const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + (size_t)row * cols);

    f32x4 v[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        int i = lane + 64 * j;
        if (FULL || i < nvec) v[j] = load_stream(xr + i);
        else v[j] = f32x4{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
    }
    float m = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < NV; j++) m = fmaxf(fmaxf(fmaxf(v[j].x, v[j].y), fmaxf(v[j].z, v[j].w)), m);
    m = wave_allreduce_f32(m, OpMaxF());

    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        bool live = FULL || lane + 64 * j < nvec;
        v[j].x = live ? exp_neg(v[j].x - m) : 0.0f;
        v[j].y = live ? exp_neg(v[j].y - m) : 0.0f;
        v[j].z = live ? exp_neg(v[j].z - m) : 0.0f;
        v[j].w = live ? exp_neg(v[j].w - m) : 0.0f;
        s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
    }
    s = wave_allreduce_f32(s, OpAdd());
    const float inv = 1.0f / s; // y of the row maximum (its exp is exactly 1), hence max(y)

    float ys = 0.0f;
    int best = 0;
    f32x4 *yr = reinterpret_cast<f32x4 *>(y + (size_t)row * cols);
#pragma unroll
    for (int j = 0; j < NV; j++) {
        int i = lane + 64 * j;
        f32x4 o = v[j] * inv;
        if (WS) ys += (o.x + o.y) + (o.z + o.w);
        if (WA) { // largest column whose y equals max(y): max_k((y == ymax) * k)
            int c = i * 4;
            best = o.x == inv ? max(best, c) : best;
            best = o.y == inv ? max(best, c + 1) : best;
            best = o.z == inv ? max(best, c + 2) : best;
            best = o.w == inv ? max(best, c + 3) : best;
        }
        if (WY && (FULL || i < nvec)) store_stream(o, yr + i);
    }
    if (WS) {
        ys = wave_allreduce_f32(ys, OpAdd());
        if (lane == 0) rowsum[row] = ys;
    }
    if (WA) {
        best = wave_allreduce_i32(best, OpMaxI());
        if (lane == 0) arg[row] = best;
    }
}

// The same row split over W waves of a workgroup (W = 2 or 4; 4 / W rows per workgroup), NVL float4 per lane: a wave's
// requests cover 1024 * NVL / 256 KiB of consecutive bytes instead of the whole row, and there are W times as many
// waves to issue them; the three row reductions go through LDS (one barrier each). cols == 256 * NVL * W exactly.
template <int NVL, int W, bool WY, bool WS, bool WA>
__global__ __launch_bounds__(W < 4 ? 256 : 64 * W) void softmax_rows_split_k(const float *__restrict__ x, float *__restrict__ y,
                                                            float *__restrict__ rowsum, int32_t *__restrict__ arg, int rows) {
    constexpr int RPB = W < 4 ? 4 / W : 1, cols = 256 * NVL * W; // rows per workgroup
    __shared__ float red[3][16];
    __shared__ int redi[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, part = wave % W, rw = wave / W;
    const int row = blockIdx.x * RPB + rw;
    const bool live = row < rows; // every wave reaches every barrier
    const size_t base = (size_t)(live ? row : 0) * cols + (size_t)part * (256 * NVL);
    const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + base);
    f32x4 v[NVL];
#pragma unroll
    for (int j = 0; j < NVL; j++) v[j] = load_stream(xr + lane + 64 * j);
    float m = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < NVL; j++) m = fmaxf(fmaxf(fmaxf(v[j].x, v[j].y), fmaxf(v[j].z, v[j].w)), m);
    m = wave_allreduce_f32(m, OpMaxF());
    if (lane == 0) red[0][wave] = m;
    __syncthreads();
    m = red[0][rw * W];
#pragma unroll
    for (int k = 1; k < W; k++) m = fmaxf(m, red[0][rw * W + k]);

    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        v[j].x = exp_neg(v[j].x - m);
        v[j].y = exp_neg(v[j].y - m);
        v[j].z = exp_neg(v[j].z - m);
        v[j].w = exp_neg(v[j].w - m);
        s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
    }
    s = wave_allreduce_f32(s, OpAdd());
    if (lane == 0) red[1][wave] = s;
    __syncthreads();
    s = red[1][rw * W];
#pragma unroll
    for (int k = 1; k < W; k++) s += red[1][rw * W + k]; // the parts in column order, in every wave of the row
    const float inv = 1.0f / s;

    float ys = 0.0f;
    int best = 0;
    f32x4 *yr = reinterpret_cast<f32x4 *>(y + base);
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        const int i = lane + 64 * j;
        f32x4 o = v[j] * inv;
        if (WS) ys += (o.x + o.y) + (o.z + o.w);
        if (WA) {
            const int c = part * (256 * NVL) + i * 4;
            best = o.x == inv ? max(best, c) : best;
            best = o.y == inv ? max(best, c + 1) : best;
            best = o.z == inv ? max(best, c + 2) : best;
            best = o.w == inv ? max(best, c + 3) : best;
        }
        if (WY && live) store_stream(o, yr + i);
    }
    if (WS || WA) {
        if (WS) ys = wave_allreduce_f32(ys, OpAdd());
        if (WA) best = wave_allreduce_i32(best, OpMaxI());
        if (lane == 0) {
            red[2][wave] = ys;
            redi[wave] = best;
        }
        __syncthreads();
        if (part == 0 && lane == 0 && live) {
            if (WS) {
                float t = red[2][rw * W];
#pragma unroll
                for (int k = 1; k < W; k++) t += red[2][rw * W + k];
                rowsum[row] = t;
            }
            if (WA) {
                int t = redi[rw * W];
#pragma unroll
                for (int k = 1; k < W; k++) t = max(t, redi[rw * W + k]);
                arg[row] = t;
            }
        }
    }
}

// Rows of 4096 .. 32768 columns (a multiple of 4): one workgroup per row, W waves holding 1024 * NVL columns each in
// registers (a ragged last part reads the fold's neutral value), so that a long row is still read from memory once;
// the three row reductions go through LDS as in the split kernel. The three-pass kernel below, which these rows took
// before, runs 8192 .. 32768 columns at 0.20-0.31 of 8 TB/s.
template <int NVL, int W>
__global__ __launch_bounds__(64 * W) void softmax_rows_wide_k(const float *__restrict__ x, float *__restrict__ y,
                                                             float *__restrict__ rowsum, int32_t *__restrict__ arg, int cols) {
    __shared__ float red[3][16];
    __shared__ int redi[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = blockIdx.x;
    const int nvec = cols >> 2, v0 = wave * (64 * NVL) + lane; // this lane's first float4 of the row
    const f32x4 *xr = reinterpret_cast<const f32x4 *>(x + row * cols);
    f32x4 v[NVL];
    float m = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        const int i = v0 + 64 * j;
        v[j] = i < nvec ? load_stream(xr + i) : f32x4{-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX};
        m = fmaxf(fmaxf(fmaxf(v[j].x, v[j].y), fmaxf(v[j].z, v[j].w)), m);
    }
    m = wave_allreduce_f32(m, OpMaxF());
    if (lane == 0) red[0][wave] = m;
    __syncthreads();
    m = red[0][0];
#pragma unroll
    for (int k = 1; k < W; k++) m = fmaxf(m, red[0][k]);

    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        const bool live = v0 + 64 * j < nvec;
        v[j].x = live ? exp_neg(v[j].x - m) : 0.0f;
        v[j].y = live ? exp_neg(v[j].y - m) : 0.0f;
        v[j].z = live ? exp_neg(v[j].z - m) : 0.0f;
        v[j].w = live ? exp_neg(v[j].w - m) : 0.0f;
        s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
    }
    s = wave_allreduce_f32(s, OpAdd());
    if (lane == 0) red[1][wave] = s;
    __syncthreads();
    s = red[1][0];
#pragma unroll
    for (int k = 1; k < W; k++) s += red[1][k]; // the parts in column order, in every wave
    const float inv = 1.0f / s;

    float ys = 0.0f;
    int best = 0;
    f32x4 *yr = reinterpret_cast<f32x4 *>(y + row * cols);
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        const int i = v0 + 64 * j;
        if (i >= nvec) continue;
        const f32x4 o = v[j] * inv;
        ys += (o.x + o.y) + (o.z + o.w);
        const int c = i * 4; // largest column whose y equals max(y) = inv
        best = o.x == inv ? max(best, c) : best;
        best = o.y == inv ? max(best, c + 1) : best;
        best = o.z == inv ? max(best, c + 2) : best;
        best = o.w == inv ? max(best, c + 3) : best;
        if (y) store_stream(o, yr + i);
    }
    if (rowsum || arg) {
        ys = wave_allreduce_f32(ys, OpAdd());
        best = wave_allreduce_i32(best, OpMaxI());
        if (lane == 0) {
            red[2][wave] = ys;
            redi[wave] = best;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = red[2][0];
            int b = redi[0];
#pragma unroll
            for (int k = 1; k < W; k++) {
                t += red[2][k];
                b = max(b, redi[k]);
            }
            if (rowsum) rowsum[row] = t;
            if (arg) arg[row] = b;
        }
    }
}

// Any cols / alignment: one 256-thread workgroup per row, three passes over the row
// (rows of this size stay in L2 between passes), LDS only for the cross-wave folds.
template <class Op> __device__ __forceinline__ float block_allreduce_f32(float v, Op op, float *lds) {
    v = wave_allreduce_f32(v, op);
    __syncthreads(); // lds may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    return op(op(lds[0], lds[1]), op(lds[2], lds[3]));
}

__global__ __launch_bounds__(256) void softmax_rows_generic_k(const float *__restrict__ x, float *__restrict__ y,
                                                              float *__restrict__ rowsum, int32_t *__restrict__ arg,
                                                              int rows, int64_t cols) {
    __shared__ float lds[4];
    __shared__ int ldsi[4];
    const int64_t row = blockIdx.x; // grid == rows, every thread of the block reaches every barrier
    const float *xr = x + row * cols;
    float m = -FLT_MAX;
    for (int64_t c = threadIdx.x; c < cols; c += 256) m = fmaxf(xr[c], m);
    m = block_allreduce_f32(m, OpMaxF(), lds);
    float s = 0.0f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) s += exp_neg(xr[c] - m);
    s = block_allreduce_f32(s, OpAdd(), lds);
    const float inv = 1.0f / s;
    float ys = 0.0f;
    int best = 0;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
        float o = exp_neg(xr[c] - m) * inv;
        ys += o;
        best = o == inv ? max(best, (int)c) : best;
        if (y) y[row * cols + c] = o;
    }
    if (rowsum) {
        ys = block_allreduce_f32(ys, OpAdd(), lds);
        if (threadIdx.x == 0) rowsum[row] = ys;
    }
    if (arg) {
        best = wave_allreduce_i32(best, OpMaxI());
        if ((threadIdx.x & 63) == 0) ldsi[threadIdx.x >> 6] = best;
        __syncthreads();
        if (threadIdx.x == 0) arg[row] = max(max(ldsi[0], ldsi[1]), max(ldsi[2], ldsi[3]));
    }
}

// 16-bit storage (bf16 / f16), as the C backend computes it: elements widen to f32 registers, the exponentials, their
// sum and the quotient are f32, y is narrowed by truncation on store (zyx/src/codegen/c.rs:456-497, 491-496), and the
// row sum and the argmax that follow read the stored y, i.e. the truncated values; the row sum is stored truncated too.
template <int DT> __device__ __forceinline__ float widen(uint16_t h) { return DT == DT_BF16 ? bf16_to_f32(h) : f16_to_f32(h); }
template <int DT> __device__ __forceinline__ uint16_t narrow(float v) { return DT == DT_BF16 ? f32_to_bf16_trunc(v) : f32_to_f16_trunc(v); }

// One wave per row of up to 4096 columns held in registers, 4 columns (8 bytes) per lane and access.
template <int DT, int NV>
__global__ __launch_bounds__(256) void softmax_rows_wave16_k(const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                                                             uint16_t *__restrict__ rowsum, int32_t *__restrict__ arg,
                                                             int rows, int cols) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int nvec = cols >> 2;
    const uint2 *xr = reinterpret_cast<const uint2 *>(x + (size_t)row * cols);
    float v[NV][4];
    float m = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + 64 * j;
        if (i < nvec) {
            const uint2 t = xr[i];
            v[j][0] = widen<DT>((uint16_t)t.x); v[j][1] = widen<DT>((uint16_t)(t.x >> 16));
            v[j][2] = widen<DT>((uint16_t)t.y); v[j][3] = widen<DT>((uint16_t)(t.y >> 16));
        } else v[j][0] = v[j][1] = v[j][2] = v[j][3] = -FLT_MAX;
        m = fmaxf(fmaxf(fmaxf(v[j][0], v[j][1]), fmaxf(v[j][2], v[j][3])), m);
    }
    m = wave_allreduce_f32(m, OpMaxF());
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const bool live = lane + 64 * j < nvec;
#pragma unroll
        for (int k = 0; k < 4; k++) v[j][k] = live ? exp_neg(v[j][k] - m) : 0.0f;
        s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
    }
    s = wave_allreduce_f32(s, OpAdd());
    const float inv = 1.0f / s;
    const float ymax = widen<DT>(narrow<DT>(inv)); // the stored y of the row maximum (its exponential is exactly 1)
    float ys = 0.0f;
    int best = 0;
    uint2 *yr = reinterpret_cast<uint2 *>(y + (size_t)row * cols);
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = lane + 64 * j;
        if (i >= nvec) continue;
        uint16_t t[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            t[k] = narrow<DT>(v[j][k] * inv);
            const float f = widen<DT>(t[k]);
            ys += f;
            best = f == ymax ? max(best, i * 4 + k) : best; // largest column among ties
        }
        if (y) yr[i] = make_uint2((uint32_t)t[0] | ((uint32_t)t[1] << 16), (uint32_t)t[2] | ((uint32_t)t[3] << 16));
    }
    if (rowsum) {
        ys = wave_allreduce_f32(ys, OpAdd());
        if (lane == 0) rowsum[row] = narrow<DT>(ys);
    }
    if (arg) {
        best = wave_allreduce_i32(best, OpMaxI());
        if (lane == 0) arg[row] = best;
    }
}

// Any cols / alignment: one workgroup per row, three passes over the row.
template <int DT>
__global__ __launch_bounds__(256) void softmax_rows_generic16_k(const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                                                                uint16_t *__restrict__ rowsum, int32_t *__restrict__ arg,
                                                                int rows, int64_t cols) {
    __shared__ float lds[4];
    __shared__ int ldsi[4];
    const int64_t row = blockIdx.x;
    const uint16_t *xr = x + row * cols;
    float m = -FLT_MAX;
    for (int64_t c = threadIdx.x; c < cols; c += 256) m = fmaxf(widen<DT>(xr[c]), m);
    m = block_allreduce_f32(m, OpMaxF(), lds);
    float s = 0.0f;
    for (int64_t c = threadIdx.x; c < cols; c += 256) s += exp_neg(widen<DT>(xr[c]) - m);
    s = block_allreduce_f32(s, OpAdd(), lds);
    const float inv = 1.0f / s, ymax = widen<DT>(narrow<DT>(inv));
    float ys = 0.0f;
    int best = 0;
    for (int64_t c = threadIdx.x; c < cols; c += 256) {
        const uint16_t t = narrow<DT>(exp_neg(widen<DT>(xr[c]) - m) * inv);
        const float f = widen<DT>(t);
        ys += f;
        best = f == ymax ? max(best, (int)c) : best;
        if (y) y[row * cols + c] = t;
    }
    if (rowsum) {
        ys = block_allreduce_f32(ys, OpAdd(), lds);
        if (threadIdx.x == 0) rowsum[row] = narrow<DT>(ys);
    }
    if (arg) {
        best = wave_allreduce_i32(best, OpMaxI());
        if ((threadIdx.x & 63) == 0) ldsi[threadIdx.x >> 6] = best;
        __syncthreads();
        if (threadIdx.x == 0) arg[row] = max(max(ldsi[0], ldsi[1]), max(ldsi[2], ldsi[3]));
    }
}

// 16-bit rows split over W waves of a workgroup, NVL 16-byte vectors (8 elements) per lane: cols == 512 * NVL * W
// exactly. A wave's requests cover NVL KiB of consecutive bytes (2 KiB at 4096 columns). For bf16 the exponential is
// one multiply and one v_exp_f32: its relative error (about |x - max| * 6e-8) is far below the step of an 8-bit
// mantissa, so the truncated y differs from the long form's in one element of several thousand, always by one step; the
// eight-instruction form makes a kernel that moves half the bytes of the f32 one as slow as it (42 us at 8192 x 4096).
// f16 keeps the long form: below 2^-14 its conversion gives 0, a cliff of a whole step at which a 1e-6 error shows.
template <int DT, int NVL, int W>
__global__ __launch_bounds__(W < 4 ? 256 : 64 * W) void softmax_rows_split16_k(const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                                                                              uint16_t *__restrict__ rowsum,
                                                                              int32_t *__restrict__ arg, int rows) {
    constexpr int RPB = W < 4 ? 4 / W : 1, cols = 512 * NVL * W; // rows per workgroup
    __shared__ float red[3][16];
    __shared__ int redi[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, part = wave % W, rw = wave / W;
    const int row = blockIdx.x * RPB + rw;
    const bool live = row < rows; // every wave reaches every barrier
    const size_t base = (size_t)(live ? row : 0) * cols + (size_t)part * (512 * NVL);
    const uint4 *xr = reinterpret_cast<const uint4 *>(x + base);
    float v[NVL][8];
    float m = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        typedef uint32_t u32x4s __attribute__((ext_vector_type(4)));
        const u32x4s t = __builtin_nontemporal_load((const u32x4s *)(xr + lane + 64 * j)); // read once
        const uint32_t w[4] = {t[0], t[1], t[2], t[3]};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[j][2 * k] = widen<DT>((uint16_t)w[k]);
            v[j][2 * k + 1] = widen<DT>((uint16_t)(w[k] >> 16));
        }
#pragma unroll
        for (int k = 0; k < 8; k++) m = fmaxf(v[j][k], m);
    }
    m = wave_allreduce_f32(m, OpMaxF());
    if (lane == 0) red[0][wave] = m;
    __syncthreads();
    m = red[0][rw * W];
#pragma unroll
    for (int k = 1; k < W; k++) m = fmaxf(m, red[0][rw * W + k]);

    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
#pragma unroll
        for (int k = 0; k < 8; k++)
            v[j][k] = DT == DT_BF16 ? __builtin_amdgcn_exp2f((v[j][k] - m) * 1.44269502162933349609375f) : exp_neg(v[j][k] - m);
        s += ((v[j][0] + v[j][1]) + (v[j][2] + v[j][3])) + ((v[j][4] + v[j][5]) + (v[j][6] + v[j][7]));
    }
    s = wave_allreduce_f32(s, OpAdd());
    if (lane == 0) red[1][wave] = s;
    __syncthreads();
    s = red[1][rw * W];
#pragma unroll
    for (int k = 1; k < W; k++) s += red[1][rw * W + k]; // the parts in column order, in every wave of the row
    const float inv = 1.0f / s;
    const float ymax = widen<DT>(narrow<DT>(inv)); // the stored y of the row maximum (its exponential is exactly 1)

    float ys = 0.0f;
    int best = 0;
    uint4 *yr = reinterpret_cast<uint4 *>(y + base);
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        const int c0 = part * (512 * NVL) + (lane + 64 * j) * 8;
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint16_t lo = narrow<DT>(v[j][2 * k] * inv), hi = narrow<DT>(v[j][2 * k + 1] * inv);
            const float flo = widen<DT>(lo), fhi = widen<DT>(hi);
            ys += flo + fhi;
            best = flo == ymax ? max(best, c0 + 2 * k) : best; // largest column among ties
            best = fhi == ymax ? max(best, c0 + 2 * k + 1) : best;
            w[k] = (uint32_t)lo | ((uint32_t)hi << 16);
        }
        typedef uint32_t u32x4s __attribute__((ext_vector_type(4)));
        if (y && live) __builtin_nontemporal_store(u32x4s{w[0], w[1], w[2], w[3]}, (u32x4s *)(yr + lane + 64 * j));
    }
    if (rowsum || arg) {
        ys = wave_allreduce_f32(ys, OpAdd());
        best = wave_allreduce_i32(best, OpMaxI());
        if (lane == 0) {
            red[2][wave] = ys;
            redi[wave] = best;
        }
        __syncthreads();
        if (part == 0 && lane == 0 && live) {
            float t = red[2][rw * W];
            int b = redi[rw * W];
#pragma unroll
            for (int k = 1; k < W; k++) {
                t += red[2][rw * W + k];
                b = max(b, redi[rw * W + k]);
            }
            if (rowsum) rowsum[row] = narrow<DT>(t);
            if (arg) arg[row] = b;
        }
    }
}

// 16-bit rows of up to 65536 columns (a multiple of 8): one workgroup per row, W waves holding 512 * NVL columns each
// in registers, the last part ragged; otherwise as softmax_rows_split16_k. (These rows took the three-pass kernel before.)
template <int DT, int NVL, int W>
__global__ __launch_bounds__(64 * W) void softmax_rows_wide16_k(const uint16_t *__restrict__ x, uint16_t *__restrict__ y,
                                                               uint16_t *__restrict__ rowsum, int32_t *__restrict__ arg, int cols) {
    typedef uint32_t u32x4s __attribute__((ext_vector_type(4)));
    __shared__ float red[3][16];
    __shared__ int redi[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = blockIdx.x;
    const int nvec = cols >> 3, v0 = wave * (64 * NVL) + lane; // this lane's first 8-element vector of the row
    const u32x4s *xr = reinterpret_cast<const u32x4s *>(x + row * cols);
    float v[NVL][8];
    float m = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        if (v0 + 64 * j < nvec) {
            const u32x4s t = __builtin_nontemporal_load(xr + v0 + 64 * j); // read once
#pragma unroll
            for (int k = 0; k < 4; k++) {
                v[j][2 * k] = widen<DT>((uint16_t)t[k]);
                v[j][2 * k + 1] = widen<DT>((uint16_t)(t[k] >> 16));
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) v[j][k] = -FLT_MAX;
        }
#pragma unroll
        for (int k = 0; k < 8; k++) m = fmaxf(v[j][k], m);
    }
    m = wave_allreduce_f32(m, OpMaxF());
    if (lane == 0) red[0][wave] = m;
    __syncthreads();
    m = red[0][0];
#pragma unroll
    for (int k = 1; k < W; k++) m = fmaxf(m, red[0][k]);

    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        const bool live = v0 + 64 * j < nvec;
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const float e = DT == DT_BF16 ? __builtin_amdgcn_exp2f((v[j][k] - m) * 1.44269502162933349609375f) : exp_neg(v[j][k] - m);
            v[j][k] = live ? e : 0.0f;
        }
        s += ((v[j][0] + v[j][1]) + (v[j][2] + v[j][3])) + ((v[j][4] + v[j][5]) + (v[j][6] + v[j][7]));
    }
    s = wave_allreduce_f32(s, OpAdd());
    if (lane == 0) red[1][wave] = s;
    __syncthreads();
    s = red[1][0];
#pragma unroll
    for (int k = 1; k < W; k++) s += red[1][k];
    const float inv = 1.0f / s;
    const float ymax = widen<DT>(narrow<DT>(inv)); // the stored y of the row maximum (its exponential is exactly 1)

    float ys = 0.0f;
    int best = 0;
    u32x4s *yr = reinterpret_cast<u32x4s *>(y + row * cols);
#pragma unroll
    for (int j = 0; j < NVL; j++) {
        const int i = v0 + 64 * j;
        if (i >= nvec) continue;
        const int c0 = i * 8;
        u32x4s w;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint16_t lo = narrow<DT>(v[j][2 * k] * inv), hi = narrow<DT>(v[j][2 * k + 1] * inv);
            const float flo = widen<DT>(lo), fhi = widen<DT>(hi);
            ys += flo + fhi;
            best = flo == ymax ? max(best, c0 + 2 * k) : best; // largest column among ties
            best = fhi == ymax ? max(best, c0 + 2 * k + 1) : best;
            w[k] = (uint32_t)lo | ((uint32_t)hi << 16);
        }
        if (y) __builtin_nontemporal_store(w, yr + i);
    }
    if (rowsum || arg) {
        ys = wave_allreduce_f32(ys, OpAdd());
        best = wave_allreduce_i32(best, OpMaxI());
        if (lane == 0) {
            red[2][wave] = ys;
            redi[wave] = best;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            float t = red[2][0];
            int b = redi[0];
#pragma unroll
            for (int k = 1; k < W; k++) {
                t += red[2][k];
                b = max(b, redi[k]);
            }
            if (rowsum) rowsum[row] = narrow<DT>(t);
            if (arg) arg[row] = b;
        }
    }
}

template <int DT> static hipError_t softmax_rows16(const SoftmaxRows &p, hipStream_t st) {
    const uint16_t *x = (const uint16_t *)p.x;
    uint16_t *y = (uint16_t *)p.y, *rs = (uint16_t *)p.rowsum;
    const bool vec_ok = (p.cols % 4 == 0) && p.cols <= 4096 && (reinterpret_cast<uintptr_t>(p.x) % 8 == 0) &&
                        (p.y == nullptr || reinterpret_cast<uintptr_t>(p.y) % 8 == 0) && p.rows < (1ll << 31) - 4;
    const bool al16 = reinterpret_cast<uintptr_t>(p.x) % 16 == 0 && (p.y == nullptr || reinterpret_cast<uintptr_t>(p.y) % 16 == 0);
    if (al16 && p.rows >= 1024 && p.rows < (1ll << 31) - 4) {
        // (rows per workgroup: 4 / W for W < 4)
        if (p.cols == 1024) {
            hipLaunchKernelGGL((softmax_rows_split16_k<DT, 1, 2>), dim3((unsigned)((p.rows + 1) / 2)), dim3(256), 0, st, x, y, rs, p.arg, (int)p.rows);
            return hipGetLastError();
        }
        if (p.cols == 2048) {
            hipLaunchKernelGGL((softmax_rows_split16_k<DT, 1, 4>), dim3((unsigned)p.rows), dim3(256), 0, st, x, y, rs, p.arg, (int)p.rows);
            return hipGetLastError();
        }
        if (p.cols == 4096) {
            // (holding a compute unit at fewer workgroups with an unused LDS request, which helps the f32 kernel, does not
            // help here: 24.6 us without, 24.6 .. 31.2 us with 20,000 .. 52,000 bytes)
            hipLaunchKernelGGL((softmax_rows_split16_k<DT, 2, 4>), dim3((unsigned)p.rows), dim3(256), 0, st, x, y, rs, p.arg, (int)p.rows);
            return hipGetLastError();
        }
        if (p.cols == 8192) {
            hipLaunchKernelGGL((softmax_rows_split16_k<DT, 4, 4>), dim3((unsigned)p.rows), dim3(256), 0, st, x, y, rs, p.arg, (int)p.rows);
            return hipGetLastError();
        }
    }
    if (vec_ok) {
        dim3 grid((unsigned)((p.rows + 3) / 4)), block(256);
        const int64_t nvec = p.cols / 4;
#define ZK_W16(NV) hipLaunchKernelGGL((softmax_rows_wave16_k<DT, NV>), grid, block, 0, st, x, y, rs, p.arg, (int)p.rows, (int)p.cols)
        if (nvec <= 64) ZK_W16(1);
        else if (nvec <= 128) ZK_W16(2);
        else if (nvec <= 256) ZK_W16(4);
        else if (nvec <= 512) ZK_W16(8);
        else ZK_W16(16);
#undef ZK_W16
        return hipGetLastError();
    }
    if (p.rows >= (1ll << 31) || p.cols >= (1ll << 31)) return hipErrorInvalidValue;
    if (al16 && p.cols % 8 == 0 && p.cols > 4096 && p.cols <= 65536) {
        const dim3 grid((unsigned)p.rows);
        if (p.cols <= 8192) hipLaunchKernelGGL((softmax_rows_wide16_k<DT, 2, 8>), grid, dim3(512), 0, st, x, y, rs, p.arg, (int)p.cols);
        else if (p.cols <= 16384) hipLaunchKernelGGL((softmax_rows_wide16_k<DT, 2, 16>), grid, dim3(1024), 0, st, x, y, rs, p.arg, (int)p.cols);
        else if (p.cols <= 32768) hipLaunchKernelGGL((softmax_rows_wide16_k<DT, 4, 16>), grid, dim3(1024), 0, st, x, y, rs, p.arg, (int)p.cols);
        else hipLaunchKernelGGL((softmax_rows_wide16_k<DT, 8, 16>), grid, dim3(1024), 0, st, x, y, rs, p.arg, (int)p.cols);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(softmax_rows_generic16_k<DT>, dim3((unsigned)p.rows), dim3(256), 0, st, x, y, rs, p.arg, (int)p.rows, p.cols);
    return hipGetLastError();
}

// Four waves per row. Measured at 8192 x 4096 (all three outputs): 44.2 us against 47.8 us for one wave per row (two waves
// per row 45.5, eight 44.4, sixteen 50.7), and 43.4 us when an unused LDS request holds a compute unit at 4 workgroups
// (16 waves) on a grid of several rounds, so that one round's stores run beside the next one's loads.
template <int NVL> static hipError_t launch_split(const SoftmaxRows &p, hipStream_t st) {
    dim3 grid((unsigned)p.rows), block(256);
    const unsigned lds_pad = p.rows >= 4096 ? 40000u : 0u;
    const int sel = (p.y ? 1 : 0) | (p.rowsum ? 2 : 0) | (p.arg ? 4 : 0);
#define ZK_CASE(S, A, B, C)                                                                                           \
    case S:                                                                                                           \
        hipLaunchKernelGGL((softmax_rows_split_k<NVL, 4, A, B, C>), grid, block, lds_pad, st, (const float *)p.x, (float *)p.y, \
                           (float *)p.rowsum, p.arg, (int)p.rows);                                                    \
        break;
    switch (sel) {
        ZK_CASE(1, true, false, false) ZK_CASE(2, false, true, false) ZK_CASE(3, true, true, false)
        ZK_CASE(4, false, false, true) ZK_CASE(5, true, false, true) ZK_CASE(6, false, true, true)
        ZK_CASE(7, true, true, true)
    default: return hipErrorInvalidValue;
    }
#undef ZK_CASE
    return hipGetLastError();
}

template <int NV> static hipError_t launch_wave(const SoftmaxRows &p, hipStream_t st) {
    dim3 grid((unsigned)((p.rows + 3) / 4)), block(256);
    // Rows of 16 vectors per lane on a grid of several rounds: an unused LDS request holds a compute unit at 3 workgroups
    // (12 waves) instead of 8, so that the rounds overlap and one round's stores run beside the next one's loads; with
    // every wave resident at once all of them load, then all of them store (measured 47.8 against 48.0 us at
    // 8192 x 4096; 2, 4, 5, 6 and 8 workgroups per unit were all slower than 3).
    const unsigned lds_pad = (NV == 16 && grid.x >= 1536) ? 54000u : 0u;
    int rows = (int)p.rows, cols = (int)p.cols;
    int sel = (p.y ? 1 : 0) | (p.rowsum ? 2 : 0) | (p.arg ? 4 : 0);
    bool full = p.cols == 256 * NV;
#define ZK_CASE(S, A, B, C)                                                                                           \
    case S:                                                                                                           \
        if (full)                                                                                                     \
            hipLaunchKernelGGL((softmax_rows_wave_k<NV, true, A, B, C>), grid, block, lds_pad, st, (const float *)p.x, (float *)p.y, (float *)p.rowsum, \
                               p.arg, rows, cols);                                                                    \
        else                                                                                                          \
            hipLaunchKernelGGL((softmax_rows_wave_k<NV, false, A, B, C>), grid, block, 0, st, (const float *)p.x, (float *)p.y, (float *)p.rowsum, \
                               p.arg, rows, cols);                                                                    \
        break;
    switch (sel) {
        ZK_CASE(1, true, false, false) ZK_CASE(2, false, true, false) ZK_CASE(3, true, true, false)
        ZK_CASE(4, false, false, true) ZK_CASE(5, true, false, true) ZK_CASE(6, false, true, true)
        ZK_CASE(7, true, true, true)
    default: return hipErrorInvalidValue;
    }
#undef ZK_CASE
    return hipGetLastError();
}

hipError_t softmax_rows(const SoftmaxRows &p, hipStream_t st) {
    if (p.rows <= 0 || p.cols <= 0) return hipSuccess; // empty tensor: nothing to write
    if (p.dtype == DT_BF16) return softmax_rows16<DT_BF16>(p, st);
    if (p.dtype == DT_F16) return softmax_rows16<DT_F16>(p, st);
    if (p.dtype != DT_F32) return hipErrorInvalidValue;
    bool vec_ok = (p.cols % 4 == 0) && p.cols <= 4096 && (reinterpret_cast<uintptr_t>(p.x) % 16 == 0) &&
                  (p.y == nullptr || reinterpret_cast<uintptr_t>(p.y) % 16 == 0) && p.rows < (1ll << 31) - 4;
    if (vec_ok) {
        int64_t nvec = p.cols / 4;
        // many full rows of 1024, 2048 or 4096 columns: four waves per row
        if (p.rows >= 1024 && p.cols == 1024) return launch_split<1>(p, st);
        if (p.rows >= 1024 && p.cols == 2048) return launch_split<2>(p, st);
        if (p.rows >= 1024 && p.cols == 4096) return launch_split<4>(p, st);
        if (p.rows >= 1024 && p.cols > 2048) { // other lengths up to 4096: four waves per row as well, the last part ragged
            hipLaunchKernelGGL((softmax_rows_wide_k<4, 4>), dim3((unsigned)p.rows), dim3(256), 0, st, (const float *)p.x, (float *)p.y,
                               (float *)p.rowsum, p.arg, (int)p.cols);
            return hipGetLastError();
        }
        if (nvec <= 64) return launch_wave<1>(p, st);
        if (nvec <= 128) return launch_wave<2>(p, st);
        if (nvec <= 256) return launch_wave<4>(p, st);
        if (nvec <= 512) return launch_wave<8>(p, st);
        return launch_wave<16>(p, st);
    }
    if (p.rows >= (1ll << 31) || p.cols >= (1ll << 31)) return hipErrorInvalidValue;
    if (p.cols % 4 == 0 && p.cols > 4096 && p.cols <= 32768 && reinterpret_cast<uintptr_t>(p.x) % 16 == 0 &&
        (p.y == nullptr || reinterpret_cast<uintptr_t>(p.y) % 16 == 0)) {
        const float *x = (const float *)p.x;
        float *y = (float *)p.y, *rs = (float *)p.rowsum;
        const dim3 grid((unsigned)p.rows);
        // 4 KiB of a row per wave up to 16384 columns, 8 KiB beyond
        if (p.cols <= 8192) hipLaunchKernelGGL((softmax_rows_wide_k<4, 8>), grid, dim3(512), 0, st, x, y, rs, p.arg, (int)p.cols);
        else if (p.cols <= 16384) hipLaunchKernelGGL((softmax_rows_wide_k<4, 16>), grid, dim3(1024), 0, st, x, y, rs, p.arg, (int)p.cols);
        else hipLaunchKernelGGL((softmax_rows_wide_k<8, 16>), grid, dim3(1024), 0, st, x, y, rs, p.arg, (int)p.cols);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(softmax_rows_generic_k, dim3((unsigned)p.rows), dim3(256), 0, st, (const float *)p.x, (float *)p.y, (float *)p.rowsum, p.arg,
                       (int)p.rows, p.cols);
    return hipGetLastError();
}

} // namespace zk
