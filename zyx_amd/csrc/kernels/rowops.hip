// Row-wise fused kernels over x[rows, cols]: LayerNorm, RMSNorm, cross-entropy (forward and
// the gradient of its mean). One 64-lane wave owns one row; lanes stride over the columns
// (128-bit accesses when the row is 4-element aligned) and combine with DPP wave
// reductions. Rows of these ops are short (model width, class count): the row is re-read
// from L1/L2 for the second pass instead of being kept in registers, HBM sees it once.
//
//   LayerNorm  zyx-nn/src/layer_norm.rs:98-135: (x - mean) / sqrt(var + eps) * w + b with
//              var = sum((x - mean)^2) / (n - 1)  (Tensor::var uses correction 1,
//              zyx/src/tensor/reduce_ops.rs:795-805, 111-123)
//   RMSNorm    zyx-nn/src/rms_norm.rs:26-32: x * sqrt(1 / (mean(x^2) + eps)) * scale
//   their gradients: the reverse rules of zyx/src/graph/autograd.rs:87-134 (Sub, Mul, Div, the reduce
//              rules :299-379) applied to the expressions above collapse, per row, to
//              LayerNorm dx = rstd * (g - mean(g) - xh * sum(g*xh) / (n-1)), g = dy*w, xh = (x-mean)*rstd
//              RMSNorm   dx = r * g - r^3 * x * sum(g*x) / n;  dw = sum_rows dy*xh, db = sum_rows dy
//   cross_entropy zyx/src/tensor/mod.rs:1639-1655 with ln_softmax :1427-1431 and the class
//              index target turned into a one-hot by equal(arange) :1920-1946.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

template <int DT> struct RowIO; // DT: 0 f32, 1 bf16 storage
template <> struct RowIO<0> {
    typedef float S;
    static __device__ __forceinline__ float ld(const float *p, int64_t i) { return p[i]; }
    static __device__ __forceinline__ void ld4(const float *p, int64_t i, float (&v)[4]) {
        f32x4 t = *(const f32x4 *)(p + i);
        v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
    }
    static __device__ __forceinline__ void st(float *p, int64_t i, float v) { p[i] = v; }
    static __device__ __forceinline__ void st4(float *p, int64_t i, const float (&v)[4]) {
        *(f32x4 *)(p + i) = f32x4{v[0], v[1], v[2], v[3]};
    }
};
template <> struct RowIO<1> {
    typedef uint16_t S;
    static __device__ __forceinline__ float ld(const uint16_t *p, int64_t i) { return bf16_to_f32(p[i]); }
    static __device__ __forceinline__ void ld4(const uint16_t *p, int64_t i, float (&v)[4]) {
        uint2 t = *(const uint2 *)(p + i);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void st(uint16_t *p, int64_t i, float v) { p[i] = f32_to_bf16_trunc(v); }
    static __device__ __forceinline__ void st4(uint16_t *p, int64_t i, const float (&v)[4]) {
        *(uint2 *)(p + i) = make_uint2((__float_as_uint(v[0]) >> 16) | (__float_as_uint(v[1]) & 0xffff0000u),
                                       (__float_as_uint(v[2]) >> 16) | (__float_as_uint(v[3]) & 0xffff0000u));
    }
    // 8 consecutive elements, one 16-byte access
    static __device__ __forceinline__ void ld8(const uint16_t *p, int64_t i, float (&a)[4], float (&b)[4]) {
        const uint4 t = *(const uint4 *)(p + i);
        a[0] = __uint_as_float(t.x << 16); a[1] = __uint_as_float(t.x & 0xffff0000u);
        a[2] = __uint_as_float(t.y << 16); a[3] = __uint_as_float(t.y & 0xffff0000u);
        b[0] = __uint_as_float(t.z << 16); b[1] = __uint_as_float(t.z & 0xffff0000u);
        b[2] = __uint_as_float(t.w << 16); b[3] = __uint_as_float(t.w & 0xffff0000u);
    }
    static __device__ __forceinline__ void st8(uint16_t *p, int64_t i, const float (&a)[4], const float (&b)[4]) {
        *(uint4 *)(p + i) = make_uint4((__float_as_uint(a[0]) >> 16) | (__float_as_uint(a[1]) & 0xffff0000u),
                                       (__float_as_uint(a[2]) >> 16) | (__float_as_uint(a[3]) & 0xffff0000u),
                                       (__float_as_uint(b[0]) >> 16) | (__float_as_uint(b[1]) & 0xffff0000u),
                                       (__float_as_uint(b[2]) >> 16) | (__float_as_uint(b[3]) & 0xffff0000u));
    }
};

// A row of 256*NV columns held by one wave as NV vectors of 4 values per lane. f32, or an odd NV: vector j of a lane is
// columns (lane + 64*j)*4 .. +3. bf16 with an even NV: vectors 2q and 2q+1 are the two halves of the 8 columns
// (lane + 64*q)*8 .. +7, moved as one 16-byte access (the memory pipeline takes a vector instruction in about the same
// time whatever its width). Every access of the wave covers consecutive bytes either way.
template <int DT, int NV> struct RegRow {
    typedef RowIO<DT> IO;
    typedef typename IO::S S;
    static constexpr bool WIDE = DT == 1 && NV % 2 == 0;
    static __device__ __forceinline__ int col(int lane, int j) { return WIDE ? (lane + 64 * (j >> 1)) * 8 + (j & 1) * 4 : (lane + 64 * j) * 4; }
    static __device__ __forceinline__ void load(const S *p, int lane, float (&v)[NV][4]) {
        if constexpr (WIDE) {
#pragma unroll
            for (int q = 0; q < NV / 2; q++) IO::ld8(p, (lane + 64 * q) * 8, v[2 * q], v[2 * q + 1]);
        } else {
#pragma unroll
            for (int j = 0; j < NV; j++) IO::ld4(p, (lane + 64 * j) * 4, v[j]);
        }
    }
    // vectors j0 (and j0 + 1 when WIDE; j0 even then)
    static __device__ __forceinline__ void load_at(const S *p, int lane, int j0, float (&a)[4], float (&b)[4]) {
        if constexpr (WIDE) IO::ld8(p, (lane + 64 * (j0 >> 1)) * 8, a, b);
        else IO::ld4(p, (lane + 64 * j0) * 4, a);
    }
    static __device__ __forceinline__ void store_at(S *p, int lane, int j0, const float (&a)[4], const float (&b)[4]) {
        if constexpr (WIDE) IO::st8(p, (lane + 64 * (j0 >> 1)) * 8, a, b);
        else IO::st4(p, (lane + 64 * j0) * 4, a);
    }
    static constexpr int STEP = WIDE ? 2 : 1; // vectors per access
    // The lane's part of a row as it lies in memory (32-bit words), for a row fetched ahead of its use: 16-bit rows
    // stay packed until unpack(), half the registers of their f32 form.
    static constexpr int NW = NV * (int)sizeof(S);
    static __device__ __forceinline__ void load_raw(const S *p, int lane, uint32_t (&r)[NW]) {
        if constexpr (DT == 0 || WIDE) {
#pragma unroll
            for (int q = 0; q < NW / 4; q++) {
                const uint4 t = *(const uint4 *)(p + (lane + 64 * q) * (16 / (int)sizeof(S)));
                r[4 * q] = t.x; r[4 * q + 1] = t.y; r[4 * q + 2] = t.z; r[4 * q + 3] = t.w;
            }
        } else {
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const uint2 t = *(const uint2 *)(p + (lane + 64 * j) * 4);
                r[2 * j] = t.x; r[2 * j + 1] = t.y;
            }
        }
    }
    static __device__ __forceinline__ void unpack(const uint32_t (&r)[NW], float (&v)[NV][4]) {
#pragma unroll
        for (int j = 0; j < NV; j++) {
            if constexpr (DT == 0) {
#pragma unroll
                for (int k = 0; k < 4; k++) v[j][k] = __uint_as_float(r[4 * j + k]);
            } else { // words 2j, 2j+1 hold vector j in both 16-bit layouts
                v[j][0] = __uint_as_float(r[2 * j] << 16); v[j][1] = __uint_as_float(r[2 * j] & 0xffff0000u);
                v[j][2] = __uint_as_float(r[2 * j + 1] << 16); v[j][3] = __uint_as_float(r[2 * j + 1] & 0xffff0000u);
            }
        }
    }
};

// sum over one row of f(x[c]) with lanes striding over columns
template <int DT, bool VEC, class F>
__device__ __forceinline__ float row_sum(const typename RowIO<DT>::S *xr, int cols, int lane, F f) {
    float acc = 0.0f;
    if (VEC) {
        for (int c = lane * 4; c < cols; c += 256) {
            float v[4];
            RowIO<DT>::ld4(xr, c, v);
            acc += (f(v[0]) + f(v[1])) + (f(v[2]) + f(v[3]));
        }
    } else {
        for (int c = lane; c < cols; c += 64) acc += f(RowIO<DT>::ld(xr, c));
    }
    return wave_allreduce_f32(acc, OpAdd());
}

// MODE 0: LayerNorm, 1: RMSNorm. w / b may be null (no affine part).
template <int DT, int MODE, bool VEC>
__global__ __launch_bounds__(256) void norm_rows_k(const typename RowIO<DT>::S *__restrict__ x,
                                                   const typename RowIO<DT>::S *__restrict__ w,
                                                   const typename RowIO<DT>::S *__restrict__ b,
                                                   typename RowIO<DT>::S *__restrict__ y, int64_t rows, int cols, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return; // whole wave; no workgroup synchronisation below
    const typename RowIO<DT>::S *xr = x + row * cols;
    typename RowIO<DT>::S *yr = y + row * cols;
    float mean = 0.0f, scale;
    if (MODE == 0) {
        // mean = sum / n; var = sum((x - mean)^2) / (n - 1); both divisions as the reference writes them
        mean = row_sum<DT, VEC>(xr, cols, lane, [](float v) { return v; }) / (float)cols;
        const float m = mean;
        float var = row_sum<DT, VEC>(xr, cols, lane, [m](float v) { return (v - m) * (v - m); }) / (float)(cols - 1);
        scale = 1.0f / sqrtf(var + eps);
    } else {
        float ms = row_sum<DT, VEC>(xr, cols, lane, [](float v) { return v * v; }) / (float)cols;
        scale = sqrtf(1.0f / (ms + eps)); // rsqrt = reciprocal().sqrt(), zyx/src/tensor/elementwise.rs:305-307
    }
    auto apply = [&](float v, int c) {
        float o = MODE == 0 ? (v - mean) * scale : v * scale;
        if (w) o *= RowIO<DT>::ld(w, c);
        if (b) o += RowIO<DT>::ld(b, c);
        return o;
    };
    if (VEC) {
        for (int c = lane * 4; c < cols; c += 256) {
            float v[4], o[4];
            RowIO<DT>::ld4(xr, c, v);
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = apply(v[k], c + k);
            RowIO<DT>::st4(yr, c, o);
        }
    } else {
        for (int c = lane; c < cols; c += 64) RowIO<DT>::st(yr, c, apply(RowIO<DT>::ld(xr, c), c));
    }
}

// Rows of 256*NV columns (NV = 1, 2, 4, 8, 16): the wave keeps its row in registers (4*NV values per lane,
// vector j of a lane = columns (lane + 64*j)*4 .. +3, so every access of the wave covers consecutive bytes):
// the row is read from memory once. Same arithmetic as norm_rows_k.
template <int DT, int MODE, int NV>
__global__ __launch_bounds__(256) void norm_rows_reg_k(const typename RowIO<DT>::S *__restrict__ x,
                                                       const typename RowIO<DT>::S *__restrict__ w,
                                                       const typename RowIO<DT>::S *__restrict__ b,
                                                       typename RowIO<DT>::S *__restrict__ y, int64_t rows, float eps) {
    typedef RowIO<DT> IO;
    constexpr int cols = 256 * NV;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const typename IO::S *xr = x + row * cols;
    typename IO::S *yr = y + row * cols;
    typedef RegRow<DT, NV> RR;
    float v[NV][4];
    RR::load(xr, lane, v);
    // short rows: the affine parameters are requested with the row, not after the two reductions that follow it
    constexpr bool EARLY = DT == 1 && NV <= 4; // (f32 rows lose by it: 13.9 us against 12.6 us at 8192 x 1024)
    uint32_t wr[RR::NW], br[RR::NW];
    if constexpr (EARLY) {
        if (w) RR::load_raw(w, lane, wr);
        if (b) RR::load_raw(b, lane, br);
    }
    float mean = 0.0f, scale;
    if (MODE == 0) {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++) s += (v[j][0] + v[j][1]) + (v[j][2] + v[j][3]);
        mean = wave_allreduce_f32(s, OpAdd()) / (float)cols;
        float q = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++)
#pragma unroll
            for (int k = 0; k < 4; k++) q += (v[j][k] - mean) * (v[j][k] - mean);
        scale = 1.0f / sqrtf(wave_allreduce_f32(q, OpAdd()) / (float)(cols - 1) + eps);
    } else {
        float q = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++)
#pragma unroll
            for (int k = 0; k < 4; k++) q += v[j][k] * v[j][k];
        scale = sqrtf(1.0f / (wave_allreduce_f32(q, OpAdd()) / (float)cols + eps));
    }
    float wa[NV][4], ba[NV][4];
    if constexpr (EARLY) {
        if (w) RR::unpack(wr, wa);
        if (b) RR::unpack(br, ba);
    }
#pragma unroll
    for (int j0 = 0; j0 < NV; j0 += RR::STEP) {
        float o[2][4];
#pragma unroll
        for (int h = 0; h < RR::STEP; h++) {
            const int j = j0 + h, c = RR::col(lane, j);
            float wv[4] = {1.0f, 1.0f, 1.0f, 1.0f}, bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if constexpr (EARLY) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    if (w) wv[k] = wa[j][k];
                    if (b) bv[k] = ba[j][k];
                }
            } else {
                if (w) IO::ld4(w, c, wv);
                if (b) IO::ld4(b, c, bv);
            }
#pragma unroll
            for (int k = 0; k < 4; k++) {
                o[h][k] = MODE == 0 ? (v[j][k] - mean) * scale : v[j][k] * scale;
                if (w) o[h][k] *= wv[k];
                if (b) o[h][k] += bv[k];
            }
        }
        RR::store_at(yr, lane, j0, o[0], o[1]);
    }
}

// Rows of any multiple of 4 columns up to 16384: the row is held in the registers of W waves (256 * NV columns per
// wave, the last part ragged; 4 / W rows per workgroup for W < 4), read from memory once; the two row sums of the W
// parts meet in LDS in column order. (These widths - 768, 1280, 3072, 5120, 8192 ... - took norm_rows_k before, which
// reads the row three times: 0.18-0.29 of 8 TB/s at 8192 rows.)
template <int DT, int MODE, int NV, int W, int VE>
__global__ __launch_bounds__(W < 4 ? 256 : 64 * W) void norm_rows_wide_k(const typename RowIO<DT>::S *__restrict__ x,
                                                                      const typename RowIO<DT>::S *__restrict__ w,
                                                                      const typename RowIO<DT>::S *__restrict__ b,
                                                                      typename RowIO<DT>::S *__restrict__ y, int64_t rows, int cols,
                                                                      float eps) {
    // VE elements per vector: 4, or 8 for 16-bit rows of a multiple of 8 columns (16-byte accesses)
    typedef RowIO<DT> IO;
    constexpr int RPB = W < 4 ? 4 / W : 1;
    __shared__ float red[2][16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, part = wave % W, rw = wave / W;
    const int64_t row = (int64_t)blockIdx.x * RPB + rw;
    const bool live_row = row < rows; // every wave reaches every barrier
    const typename IO::S *xr = x + (live_row ? row : 0) * cols;
    const int nvec = cols / VE, v0 = part * (64 * NV) + lane;
    auto load = [&](const typename IO::S *p, int i, float (&t)[VE]) {
        if constexpr (VE == 8) {
            float a4[4], b4[4];
            IO::ld8(p, i * 8, a4, b4);
#pragma unroll
            for (int k = 0; k < 4; k++) t[k] = a4[k], t[4 + k] = b4[k];
        } else {
            IO::ld4(p, i * 4, t);
        }
    };
    float v[NV][VE];
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        if (v0 + 64 * j < nvec) load(xr, v0 + 64 * j, v[j]);
        else
#pragma unroll
            for (int k = 0; k < VE; k++) v[j][k] = 0.0f;
#pragma unroll
        for (int k = 0; k < VE; k += 4) s += (v[j][k] + v[j][k + 1]) + (v[j][k + 2] + v[j][k + 3]);
    }
    auto row_total = [&](float t, int slot) { // sum over the row's W parts, in column order, in every wave of the row
        t = wave_allreduce_f32(t, OpAdd());
        if (W == 1) return t;
        if (lane == 0) red[slot][wave] = t;
        __syncthreads();
        float r = red[slot][rw * W];
#pragma unroll
        for (int k = 1; k < W; k++) r += red[slot][rw * W + k];
        return r;
    };
    float mean = 0.0f, scale;
    if (MODE == 0) {
        mean = row_total(s, 0) / (float)cols;
        float q = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const bool live = v0 + 64 * j < nvec;
#pragma unroll
            for (int k = 0; k < VE; k++) q += live ? (v[j][k] - mean) * (v[j][k] - mean) : 0.0f;
        }
        scale = 1.0f / sqrtf(row_total(q, 1) / (float)(cols - 1) + eps);
    } else {
        float q = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++)
#pragma unroll
            for (int k = 0; k < VE; k++) q += v[j][k] * v[j][k]; // dead lanes hold zeros
        scale = sqrtf(1.0f / (row_total(q, 0) / (float)cols + eps));
    }
    if (!live_row) return; // past the last barrier
    typename IO::S *yr = y + row * cols;
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int i = v0 + 64 * j;
        if (i >= nvec) continue;
        float wv[VE], bv[VE], o[VE];
#pragma unroll
        for (int k = 0; k < VE; k++) wv[k] = 1.0f, bv[k] = 0.0f;
        if (w) load(w, i, wv);
        if (b) load(b, i, bv);
#pragma unroll
        for (int k = 0; k < VE; k++) {
            o[k] = MODE == 0 ? (v[j][k] - mean) * scale : v[j][k] * scale;
            if (w) o[k] *= wv[k];
            if (b) o[k] += bv[k];
        }
        if constexpr (VE == 8) {
            const float a4[4] = {o[0], o[1], o[2], o[3]}, b4[4] = {o[4], o[5], o[6], o[7]};
            IO::st8(yr, i * 8, a4, b4);
        } else {
            IO::st4(yr, i * 4, o);
        }
    }
}

// dx for rows of 256*NV columns with x and dy held in registers (one read of each), and the parameter gradients in
// the same pass: a workgroup of WAVES waves walks rows blockIdx*WAVES + wave, + gridDim*WAVES, ..., every lane keeps
// running sums of dy*xh and dy for its 4*NV columns, the waves of a workgroup add theirs up through LDS in wave order
// and the workgroup leaves one partial row pair in part[(blockIdx*2 + {0,1})*cols + c] for norm_bwd_param_sum_k.
// The order of every sum is fixed by the launch shape: results are reproducible. part may be null (no dw / db).
template <int DT, int MODE, int NV, int WAVES, bool AHEAD>
__global__ __launch_bounds__(WAVES * 64) void norm_bwd_dx_reg_k(const typename RowIO<DT>::S *__restrict__ x,
                                                                const typename RowIO<DT>::S *__restrict__ w,
                                                                const typename RowIO<DT>::S *__restrict__ dy,
                                                                const typename RowIO<DT>::S *__restrict__ add,
                                                                typename RowIO<DT>::S *__restrict__ dx, float *__restrict__ part,
                                                                int64_t rows, float eps) {
    typedef RowIO<DT> IO;
    typedef RegRow<DT, NV> RR;
    constexpr int cols = 256 * NV;
    __shared__ float fold[WAVES][2][cols]; // 128 KiB at most (16 waves x 1024 columns, 8 waves x 2048)
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float pw[NV][4], pb[NV][4];
#pragma unroll
    for (int j = 0; j < NV; j++)
#pragma unroll
        for (int k = 0; k < 4; k++) pw[j][k] = pb[j][k] = 0.0f;
    // AHEAD: the wave's next row (x, dy, add) is requested before the current one is worked on, in its memory form
    // (f32 rows of 1024 in an 8-wave workgroup: 29.3 us against 32.5 us at 8192 rows; the registers this takes spill
    // in a 16-wave workgroup, and 16-bit rows gain nothing from it).
    const int64_t stride = (int64_t)gridDim.x * WAVES;
    int64_t row = (int64_t)blockIdx.x * WAVES + wave;
    uint32_t nx[RR::NW], ng[RR::NW], na[RR::NW];
#pragma unroll
    for (int i = 0; i < RR::NW; i++) na[i] = 0u;
    if (AHEAD && row < rows) {
        RR::load_raw(x + row * cols, lane, nx);
        RR::load_raw(dy + row * cols, lane, ng);
        if (add) RR::load_raw(add + row * cols, lane, na);
    }
    for (; row < rows; row += stride) {
        const int64_t base = row * cols;
        float xv[NV][4], g[NV][4];
        uint32_t ca[RR::NW];
        if constexpr (AHEAD) {
            RR::unpack(nx, xv);
            RR::unpack(ng, g);
#pragma unroll
            for (int i = 0; i < RR::NW; i++) ca[i] = na[i];
            if (row + stride < rows) {
                const int64_t nb = (row + stride) * cols;
                RR::load_raw(x + nb, lane, nx);
                RR::load_raw(dy + nb, lane, ng);
                if (add) RR::load_raw(add + nb, lane, na);
            }
        } else {
            RR::load(x + base, lane, xv);
            RR::load(dy + base, lane, g);
        }
        float mean = 0.0f, rstd;
        if (MODE == 0) {
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++) s += (xv[j][0] + xv[j][1]) + (xv[j][2] + xv[j][3]);
            mean = wave_allreduce_f32(s, OpAdd()) / (float)cols;
            float q = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++)
#pragma unroll
                for (int k = 0; k < 4; k++) q += (xv[j][k] - mean) * (xv[j][k] - mean);
            rstd = 1.0f / sqrtf(wave_allreduce_f32(q, OpAdd()) / (float)(cols - 1) + eps);
        } else {
            float q = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++)
#pragma unroll
                for (int k = 0; k < 4; k++) q += xv[j][k] * xv[j][k];
            rstd = sqrtf(1.0f / (wave_allreduce_f32(q, OpAdd()) / (float)cols + eps));
        }
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++) {
            float wv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            if (w) IO::ld4(w, RR::col(lane, j), wv); // L1 / L2 hit: every row reads the same 4*NV values
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const float xh = (xv[j][k] - mean) * rstd; // mean is 0 for RMSNorm
                pw[j][k] = __builtin_fmaf(g[j][k], xh, pw[j][k]);
                pb[j][k] += g[j][k];
                g[j][k] *= wv[k];
                s1 += g[j][k];
                s2 += g[j][k] * (MODE == 0 ? xh : xv[j][k]);
            }
        }
        s1 = wave_allreduce_f32(s1, OpAdd());
        s2 = wave_allreduce_f32(s2, OpAdd());
        const float k1 = s1 / (float)cols, k2 = MODE == 0 ? s2 / (float)(cols - 1) : rstd * rstd * rstd * s2 / (float)cols;
        float av[NV][4];
        if constexpr (AHEAD) RR::unpack(ca, av); // zeros without add
#pragma unroll
        for (int j0 = 0; j0 < NV; j0 += RR::STEP) {
            float o[2][4];
            if constexpr (!AHEAD) {
#pragma unroll
                for (int k = 0; k < 4; k++) av[j0][k] = av[j0 + RR::STEP - 1][k] = 0.0f;
                if (add) RR::load_at(add + base, lane, j0, av[j0], av[j0 + RR::STEP - 1]);
            }
#pragma unroll
            for (int h = 0; h < RR::STEP; h++)
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const int j = j0 + h;
                    o[h][k] = (MODE == 0 ? rstd * ((g[j][k] - k1) - ((xv[j][k] - mean) * rstd) * k2) : rstd * g[j][k] - xv[j][k] * k2) + av[j][k];
                }
            RR::store_at(dx + base, lane, j0, o[0], o[1]);
        }
    }
    if (!part) return; // uniform over the workgroup
    // every wave lays its sums down, then a thread adds a column's WAVES values in wave order
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int c = RR::col(lane, j);
        *(f32x4 *)&fold[wave][0][c] = f32x4{pw[j][0], pw[j][1], pw[j][2], pw[j][3]};
        *(f32x4 *)&fold[wave][1][c] = f32x4{pb[j][0], pb[j][1], pb[j][2], pb[j][3]};
    }
    __syncthreads();
    for (int c = threadIdx.x; c < cols; c += WAVES * 64) {
        float a = fold[0][0][c], b = fold[0][1][c];
#pragma unroll
        for (int v = 1; v < WAVES; v++) {
            a += fold[v][0][c];
            b += fold[v][1][c];
        }
        part[((int64_t)blockIdx.x * 2) * cols + c] = a;
        part[((int64_t)blockIdx.x * 2 + 1) * cols + c] = b;
    }
}

// The same pass for rows of any multiple of 4 columns up to 256*NV (768, 1280, 1536 ...): vector lane + 64*j of a
// row belongs to the lane while it lies inside the row; lanes past the end hold zeros, which every sum but the
// variance's takes as they are. part rows are cols long.
template <int DT, int MODE, int NV, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void norm_bwd_dx_ragged_k(const typename RowIO<DT>::S *__restrict__ x,
                                                                   const typename RowIO<DT>::S *__restrict__ w,
                                                                   const typename RowIO<DT>::S *__restrict__ dy,
                                                                   const typename RowIO<DT>::S *__restrict__ add,
                                                                   typename RowIO<DT>::S *__restrict__ dx, float *__restrict__ part,
                                                                   int64_t rows, int cols, float eps) {
    typedef RowIO<DT> IO;
    constexpr int CAP = 256 * NV;
    __shared__ float fold[WAVES][2][CAP]; // 128 KiB at most
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nvec = cols >> 2;
    float pw[NV][4], pb[NV][4];
#pragma unroll
    for (int j = 0; j < NV; j++)
#pragma unroll
        for (int k = 0; k < 4; k++) pw[j][k] = pb[j][k] = 0.0f;
    const int64_t stride = (int64_t)gridDim.x * WAVES;
    for (int64_t row = (int64_t)blockIdx.x * WAVES + wave; row < rows; row += stride) {
        const int64_t base = row * cols;
        float xv[NV][4], g[NV][4];
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + 64 * j;
            if (i < nvec) {
                IO::ld4(x + base, i * 4, xv[j]);
                IO::ld4(dy + base, i * 4, g[j]);
            } else {
#pragma unroll
                for (int k = 0; k < 4; k++) xv[j][k] = g[j][k] = 0.0f;
            }
        }
        float mean = 0.0f, rstd;
        if (MODE == 0) {
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++) s += (xv[j][0] + xv[j][1]) + (xv[j][2] + xv[j][3]);
            mean = wave_allreduce_f32(s, OpAdd()) / (float)cols;
            float q = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const bool live = lane + 64 * j < nvec;
#pragma unroll
                for (int k = 0; k < 4; k++) q += live ? (xv[j][k] - mean) * (xv[j][k] - mean) : 0.0f;
            }
            rstd = 1.0f / sqrtf(wave_allreduce_f32(q, OpAdd()) / (float)(cols - 1) + eps);
        } else {
            float q = 0.0f;
#pragma unroll
            for (int j = 0; j < NV; j++)
#pragma unroll
                for (int k = 0; k < 4; k++) q += xv[j][k] * xv[j][k];
            rstd = sqrtf(1.0f / (wave_allreduce_f32(q, OpAdd()) / (float)cols + eps));
        }
        float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + 64 * j;
            float wv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            if (w && i < nvec) IO::ld4(w, i * 4, wv);
#pragma unroll
            for (int k = 0; k < 4; k++) { // a lane past the end: g = 0 leaves every sum as it is
                const float xh = (xv[j][k] - mean) * rstd;
                pw[j][k] = __builtin_fmaf(g[j][k], xh, pw[j][k]);
                pb[j][k] += g[j][k];
                g[j][k] *= wv[k];
                s1 += g[j][k];
                s2 += g[j][k] * (MODE == 0 ? xh : xv[j][k]);
            }
        }
        s1 = wave_allreduce_f32(s1, OpAdd());
        s2 = wave_allreduce_f32(s2, OpAdd());
        const float k1 = s1 / (float)cols, k2 = MODE == 0 ? s2 / (float)(cols - 1) : rstd * rstd * rstd * s2 / (float)cols;
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = lane + 64 * j;
            if (i >= nvec) continue;
            float av[4] = {0.0f, 0.0f, 0.0f, 0.0f}, o[4];
            if (add) IO::ld4(add + base, i * 4, av);
#pragma unroll
            for (int k = 0; k < 4; k++)
                o[k] = (MODE == 0 ? rstd * ((g[j][k] - k1) - ((xv[j][k] - mean) * rstd) * k2) : rstd * g[j][k] - xv[j][k] * k2) + av[k];
            IO::st4(dx + base, i * 4, o);
        }
    }
    if (!part) return; // uniform over the workgroup
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int c = (lane + 64 * j) * 4;
        *(f32x4 *)&fold[wave][0][c] = f32x4{pw[j][0], pw[j][1], pw[j][2], pw[j][3]};
        *(f32x4 *)&fold[wave][1][c] = f32x4{pb[j][0], pb[j][1], pb[j][2], pb[j][3]};
    }
    __syncthreads();
    for (int c = threadIdx.x; c < cols; c += WAVES * 64) {
        float a = fold[0][0][c], b = fold[0][1][c];
#pragma unroll
        for (int v = 1; v < WAVES; v++) {
            a += fold[v][0][c];
            b += fold[v][1][c];
        }
        part[((int64_t)blockIdx.x * 2) * cols + c] = a;
        part[((int64_t)blockIdx.x * 2 + 1) * cols + c] = b;
    }
}

// Cross-entropy, one wave per sample. loss[r] = sum_c -(ln_softmax(x)[r,c]) * target[r,c], computed as the reference
// does: m = x - max; ls = m - ln(sum exp(m)). Targets are class indices (target[r,c] = (c == label[r]); a label outside
// [0, cols) matches no class: loss 0) or, DENSE, an f32 [rows, cols] tensor of their own (one-hot or soft labels).
// grad (optional) = (softmax(x) * sum_c target - target) * gscale, the gradient of gscale * sum_r loss[r].
// One row by one wave; returns the row's loss (in every lane).
template <bool DENSE>
__device__ __forceinline__ float cross_entropy_row(const float *__restrict__ x, const void *__restrict__ target,
                                                   float *__restrict__ loss, float *__restrict__ grad, int64_t row, int cols,
                                                   float gscale, int lane) {
    const float *xr = x + row * cols;
    float mx = -FLT_MAX;
    for (int c = lane; c < cols; c += 64) mx = fmaxf(xr[c], mx);
    mx = wave_allreduce_f32(mx, OpMaxF());
    float s = 0.0f;
    for (int c = lane; c < cols; c += 64) s += expf(xr[c] - mx);
    s = wave_allreduce_f32(s, OpAdd());
    const float lns = logf(s);
    float l = 0.0f, tsum = 1.0f;
    int label = -1;
    const float *tr = nullptr;
    if (DENSE) {
        tr = (const float *)target + row * cols;
        float ts = 0.0f;
        for (int c = lane; c < cols; c += 64) {
            const float t = tr[c];
            l += -((xr[c] - mx) - lns) * t;
            ts += t;
        }
        l = wave_allreduce_f32(l, OpAdd());
        tsum = wave_allreduce_f32(ts, OpAdd());
    } else {
        label = ((const int32_t *)target)[row];
        if (label >= 0 && label < cols) l = -((xr[label] - mx) - lns);
    }
    if (loss && lane == 0) loss[row] = l;
    if (grad) {
        const float inv = 1.0f / s;
        for (int c = lane; c < cols; c += 64) {
            float p = expf(xr[c] - mx) * inv;
            if (DENSE) grad[row * cols + c] = (p * tsum - tr[c]) * gscale;
            else grad[row * cols + c] = (p - (c == label ? 1.0f : 0.0f)) * gscale;
        }
    }
    return l;
}

template <bool DENSE>
__global__ __launch_bounds__(256) void cross_entropy_k(const float *__restrict__ x, const void *__restrict__ target,
                                                       float *__restrict__ loss, float *__restrict__ grad, int64_t rows,
                                                       int cols, float gscale) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    cross_entropy_row<DENSE>(x, target, loss, grad, row, cols, gscale, threadIdx.x & 63);
}

// Class-index targets, rows of 2049-65536 classes: one row per workgroup of W waves, read once and held in registers
// (NE values per thread; VEC: rows of a multiple of 4 classes in 16-byte vectors, vector t + 64*W*j of the row in
// thread t, else element t + 64*W*j). The formulas are cross_entropy_row's; exp(x - max) is kept for the gradient.
// The W waves' maxima and sums meet in LDS and are combined in wave order.
template <int NE, int W, bool VEC>
__global__ __launch_bounds__(64 * W) void cross_entropy_wide_k(const float *__restrict__ x, const int32_t *__restrict__ labels,
                                                               float *__restrict__ loss, float *__restrict__ grad, int cols,
                                                               float gscale) {
    constexpr int T = 64 * W, G = VEC ? 4 : 1, NJ = NE / G;
    __shared__ float red[2][W];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int64_t row = blockIdx.x;
    const float *xr = x + row * cols;
    float v[NE];
    float mx = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int c = (t + T * j) * G;
        if (c < cols) {
            if constexpr (VEC) {
                const f32x4 q = *(const f32x4 *)(xr + c);
                v[4 * j] = q.x, v[4 * j + 1] = q.y, v[4 * j + 2] = q.z, v[4 * j + 3] = q.w;
            } else {
                v[j] = xr[c];
            }
        } else {
#pragma unroll
            for (int k = 0; k < G; k++) v[G * j + k] = -INFINITY; // exp(-inf - max) = 0 below
        }
    }
#pragma unroll
    for (int i = 0; i < NE; i++) mx = fmaxf(v[i], mx);
    mx = wave_allreduce_f32(mx, OpMaxF());
    if (lane == 0) red[0][wave] = mx;
    __syncthreads();
    mx = red[0][0];
#pragma unroll
    for (int k = 1; k < W; k++) mx = fmaxf(red[0][k], mx);
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < NE; i++) {
        v[i] = expf(v[i] - mx);
        s += v[i];
    }
    s = wave_allreduce_f32(s, OpAdd());
    if (lane == 0) red[1][wave] = s;
    __syncthreads();
    s = red[1][0];
#pragma unroll
    for (int k = 1; k < W; k++) s += red[1][k];
    const int label = labels[row];
    if (loss && t == 0) loss[row] = label >= 0 && label < cols ? -((xr[label] - mx) - logf(s)) : 0.0f;
    if (!grad) return;
    const float inv = 1.0f / s;
    float *gr = grad + row * cols;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int c = (t + T * j) * G;
        if (c >= cols) continue;
        float o[G];
#pragma unroll
        for (int k = 0; k < G; k++) o[k] = (v[G * j + k] * inv - (c + k == label ? 1.0f : 0.0f)) * gscale;
        if constexpr (VEC) *(f32x4 *)(gr + c) = f32x4{o[0], o[1], o[2], o[3]};
        else gr[c] = o[0];
    }
}

// The whole batch in one workgroup of 16 waves, which also leaves mean[0] = sum(loss) / rows (ReduceOp::Mean): every
// wave adds its rows' losses in row order, the 16 partial sums are added in wave order.
template <bool DENSE>
__global__ __launch_bounds__(1024) void cross_entropy_mean_k(const float *__restrict__ x, const void *__restrict__ target,
                                                             float *__restrict__ loss, float *__restrict__ grad,
                                                             float *__restrict__ mean, int64_t rows, int cols, float gscale) {
    __shared__ float part[16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float sum = 0.0f;
    for (int64_t row = wave; row < rows; row += 16) sum += cross_entropy_row<DENSE>(x, target, loss, grad, row, cols, gscale, lane);
    if (lane == 0) part[wave] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = part[0];
        for (int w = 1; w < 16; w++) t += part[w];
        mean[0] = t / (float)rows;
    }
}

// dx of one row per wave; also leaves the row's mean and 1/sigma in stats[row*2 ..] for the parameter gradients.
template <int DT, int MODE, bool VEC>
__global__ __launch_bounds__(256) void norm_bwd_dx_k(const typename RowIO<DT>::S *__restrict__ x,
                                                     const typename RowIO<DT>::S *__restrict__ w,
                                                     const typename RowIO<DT>::S *__restrict__ dy,
                                                     const typename RowIO<DT>::S *__restrict__ add,
                                                     typename RowIO<DT>::S *__restrict__ dx, float *__restrict__ stats,
                                                     int64_t rows, int cols, float eps) {
    typedef RowIO<DT> IO;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const typename IO::S *xr = x + row * cols, *gr = dy + row * cols, *ar = add ? add + row * cols : nullptr;
    typename IO::S *dr = dx + row * cols;
    float mean = 0.0f, rstd;
    if (MODE == 0) {
        mean = row_sum<DT, VEC>(xr, cols, lane, [](float v) { return v; }) / (float)cols;
        const float m = mean;
        float var = row_sum<DT, VEC>(xr, cols, lane, [m](float v) { return (v - m) * (v - m); }) / (float)(cols - 1);
        rstd = 1.0f / sqrtf(var + eps);
    } else {
        rstd = sqrtf(1.0f / (row_sum<DT, VEC>(xr, cols, lane, [](float v) { return v * v; }) / (float)cols + eps));
    }
    float s1 = 0.0f, s2 = 0.0f; // sum g, sum g * (xh | x)
    auto accum = [&](float xv, float gv, int c) {
        const float g = w ? gv * IO::ld(w, c) : gv;
        s1 += g;
        s2 += g * (MODE == 0 ? (xv - mean) * rstd : xv);
    };
    if (VEC) {
        for (int c = lane * 4; c < cols; c += 256) {
            float xv[4], gv[4];
            IO::ld4(xr, c, xv);
            IO::ld4(gr, c, gv);
#pragma unroll
            for (int k = 0; k < 4; k++) accum(xv[k], gv[k], c + k);
        }
    } else {
        for (int c = lane; c < cols; c += 64) accum(IO::ld(xr, c), IO::ld(gr, c), c);
    }
    s1 = wave_allreduce_f32(s1, OpAdd());
    s2 = wave_allreduce_f32(s2, OpAdd());
    const float k1 = s1 / (float)cols, k2 = MODE == 0 ? s2 / (float)(cols - 1) : rstd * rstd * rstd * s2 / (float)cols;
    auto apply = [&](float xv, float gv, float av, int c) {
        const float g = w ? gv * IO::ld(w, c) : gv;
        const float o = MODE == 0 ? rstd * ((g - k1) - ((xv - mean) * rstd) * k2) : rstd * g - xv * k2;
        return o + av;
    };
    if (VEC) {
        for (int c = lane * 4; c < cols; c += 256) {
            float xv[4], gv[4], av[4] = {0.0f, 0.0f, 0.0f, 0.0f}, o[4];
            IO::ld4(xr, c, xv);
            IO::ld4(gr, c, gv);
            if (ar) IO::ld4(ar, c, av);
#pragma unroll
            for (int k = 0; k < 4; k++) o[k] = apply(xv[k], gv[k], av[k], c + k);
            IO::st4(dr, c, o);
        }
    } else {
        for (int c = lane; c < cols; c += 64) IO::st(dr, c, apply(IO::ld(xr, c), IO::ld(gr, c), ar ? IO::ld(ar, c) : 0.0f, c));
    }
    if (lane == 0) {
        stats[row * 2] = mean;
        stats[row * 2 + 1] = rstd;
    }
}

// Partial parameter gradients. A workgroup owns a strip of 256 columns (lane -> 4 adjacent columns, 64 when the
// row width is not a multiple of 4) and one chunk of rows, split over its 4 waves and joined through LDS.
// part[(chunk*2 + 0)*cols + c] = sum dy*xh, part[(chunk*2 + 1)*cols + c] = sum dy over the chunk.
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void norm_bwd_param_k(const typename RowIO<DT>::S *__restrict__ x,
                                                        const typename RowIO<DT>::S *__restrict__ dy,
                                                        const float *__restrict__ stats, float *__restrict__ part,
                                                        int64_t rows, int cols, int64_t rows_per_chunk) {
    constexpr int W = VEC ? 4 : 1;
    __shared__ float lds[4][2][64 * W];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = (blockIdx.x * 64 + lane) * W;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_chunk, r1 = r0 + rows_per_chunk < rows ? r0 + rows_per_chunk : rows;
    float pw[W], pb[W];
#pragma unroll
    for (int k = 0; k < W; k++) pw[k] = pb[k] = 0.0f;
    if (c < cols) {
#pragma unroll 4
        for (int64_t r = r0 + wave; r < r1; r += 4) {
            const float mean = stats[r * 2], rstd = stats[r * 2 + 1];
            float g[4], xv[4];
            if (VEC) {
                RowIO<DT>::ld4(dy, r * cols + c, g);
                RowIO<DT>::ld4(x, r * cols + c, xv);
            } else {
                g[0] = RowIO<DT>::ld(dy, r * cols + c);
                xv[0] = RowIO<DT>::ld(x, r * cols + c);
            }
#pragma unroll
            for (int k = 0; k < W; k++) {
                pw[k] = __builtin_fmaf(g[k], (xv[k] - mean) * rstd, pw[k]);
                pb[k] += g[k];
            }
        }
    }
#pragma unroll
    for (int k = 0; k < W; k++) {
        lds[wave][0][lane * W + k] = pw[k];
        lds[wave][1][lane * W + k] = pb[k];
    }
    __syncthreads();
    if (wave == 0 && c < cols) {
#pragma unroll
        for (int k = 0; k < W; k++) {
            const int i = lane * W + k;
            part[((int64_t)blockIdx.y * 2) * cols + c + k] = (lds[0][0][i] + lds[1][0][i]) + (lds[2][0][i] + lds[3][0][i]);
            part[((int64_t)blockIdx.y * 2 + 1) * cols + c + k] = (lds[0][1][i] + lds[1][1][i]) + (lds[2][1][i] + lds[3][1][i]);
        }
    }
}
// A workgroup folds one of the two partial rows (blockIdx.y: 0 dw, 1 db) over 32 columns: lane % 32 -> column, the 32
// half-waves split the chunks (a few independent loads each), LDS joins them in a fixed order.
template <int DT>
__global__ __launch_bounds__(1024) void norm_bwd_param_sum_k(const float *__restrict__ part, typename RowIO<DT>::S *__restrict__ dw,
                                                             typename RowIO<DT>::S *__restrict__ db, int cols, int chunks) {
    __shared__ float lds[32][32];
    const int which = blockIdx.y;
    typename RowIO<DT>::S *out = which ? db : dw;
    if (!out) return; // uniform over the workgroup
    const int lane = threadIdx.x & 63, l32 = lane & 31, grp = (threadIdx.x >> 6) * 2 + (lane >> 5);
    const int c = blockIdx.x * 32 + l32;
    float s = 0.0f;
    if (c < cols) {
#pragma unroll 8
        for (int k = grp; k < chunks; k += 32) s += part[((int64_t)k * 2 + which) * cols + c];
    }
    lds[grp][l32] = s;
    __syncthreads();
    if (threadIdx.x < 32 && c < cols) {
        float t = 0.0f;
#pragma unroll
        for (int v = 0; v < 32; v++) t += lds[v][threadIdx.x];
        RowIO<DT>::st(out, c, t);
    }
}

int norm_bwd_chunks(int64_t rows) { return (int)(rows < 256 * 32 ? (rows + 31) / 32 : 256); }
// the fused register kernel: one workgroup per CU's worth of waves, at most 256 partial row pairs
constexpr int kFusedBlocks = 256;
template <int DT, int NV> constexpr bool fused_ahead() { return DT == 0 && NV == 4; }
template <int DT, int NV> constexpr int fused_waves() { return NV <= 4 && !fused_ahead<DT, NV>() ? 16 : 8; }

template <int DT, int MODE, int NV> void launch_norm_bwd_reg(const NormRowsBwd &p, float *part, int &chunks, hipStream_t st) {
    typedef typename RowIO<DT>::S S;
    constexpr int WAVES = fused_waves<DT, NV>();
    chunks = (int)((p.rows + WAVES - 1) / WAVES < kFusedBlocks ? (p.rows + WAVES - 1) / WAVES : kFusedBlocks);
    hipLaunchKernelGGL((norm_bwd_dx_reg_k<DT, MODE, NV, WAVES, fused_ahead<DT, NV>()>), dim3((unsigned)chunks), dim3(WAVES * 64), 0, st, (const S *)p.x,
                       (const S *)p.w, (const S *)p.dy, (const S *)p.add, (S *)p.dx, (p.dw || p.db) ? part : nullptr, p.rows, p.eps);
}

template <int DT, int MODE, int NV> void launch_norm_bwd_ragged(const NormRowsBwd &p, float *part, int &chunks, hipStream_t st) {
    typedef typename RowIO<DT>::S S;
    constexpr int WAVES = NV <= 4 ? 16 : 8;
    chunks = (int)((p.rows + WAVES - 1) / WAVES < kFusedBlocks ? (p.rows + WAVES - 1) / WAVES : kFusedBlocks);
    hipLaunchKernelGGL((norm_bwd_dx_ragged_k<DT, MODE, NV, WAVES>), dim3((unsigned)chunks), dim3(WAVES * 64), 0, st, (const S *)p.x, (const S *)p.w,
                       (const S *)p.dy, (const S *)p.add, (S *)p.dx, (p.dw || p.db) ? part : nullptr, p.rows, (int)p.cols, p.eps);
}

template <int DT, int MODE> hipError_t launch_norm_bwd(const NormRowsBwd &p, hipStream_t st) {
    typedef typename RowIO<DT>::S S;
    const int esz = (int)sizeof(S);
    auto al = [&](const void *q) { return reinterpret_cast<uintptr_t>(q) % (4 * esz) == 0; };
    const bool vec = p.cols % 4 == 0 && al(p.x) && al(p.dy) && al(p.dx) && al(p.add);
    float *stats = (float *)p.workspace, *part = stats + p.rows * 2;
    dim3 grid((unsigned)((p.rows + 3) / 4)), block(256);
    const bool al16 = vec && (!p.w || reinterpret_cast<uintptr_t>(p.w) % (4 * esz) == 0);
    int chunks = 0; // > 0: the dx kernel has left this many partial row pairs in part
    if (al16 && p.cols == 256) launch_norm_bwd_reg<DT, MODE, 1>(p, part, chunks, st);
    else if (al16 && p.cols == 512) launch_norm_bwd_reg<DT, MODE, 2>(p, part, chunks, st);
    else if (al16 && p.cols == 1024) launch_norm_bwd_reg<DT, MODE, 4>(p, part, chunks, st);
    else if (al16 && p.cols == 2048) launch_norm_bwd_reg<DT, MODE, 8>(p, part, chunks, st);
    else if (al16 && p.cols <= 256) launch_norm_bwd_ragged<DT, MODE, 1>(p, part, chunks, st);
    else if (al16 && p.cols <= 512) launch_norm_bwd_ragged<DT, MODE, 2>(p, part, chunks, st);
    else if (al16 && p.cols <= 768) launch_norm_bwd_ragged<DT, MODE, 3>(p, part, chunks, st);
    else if (al16 && p.cols <= 1024) launch_norm_bwd_ragged<DT, MODE, 4>(p, part, chunks, st);
    else if (al16 && p.cols <= 1280) launch_norm_bwd_ragged<DT, MODE, 5>(p, part, chunks, st);
    else if (al16 && p.cols <= 1536) launch_norm_bwd_ragged<DT, MODE, 6>(p, part, chunks, st);
    else if (al16 && p.cols <= 2048) launch_norm_bwd_ragged<DT, MODE, 8>(p, part, chunks, st);
    else if (vec) hipLaunchKernelGGL((norm_bwd_dx_k<DT, MODE, true>), grid, block, 0, st, (const S *)p.x, (const S *)p.w, (const S *)p.dy, (const S *)p.add, (S *)p.dx, stats, p.rows, (int)p.cols, p.eps);
    else hipLaunchKernelGGL((norm_bwd_dx_k<DT, MODE, false>), grid, block, 0, st, (const S *)p.x, (const S *)p.w, (const S *)p.dy, (const S *)p.add, (S *)p.dx, stats, p.rows, (int)p.cols, p.eps);
    if (p.dw || p.db) {
        if (chunks == 0) {
            chunks = norm_bwd_chunks(p.rows);
            const int64_t rpc = (p.rows + chunks - 1) / chunks;
            if (vec) hipLaunchKernelGGL((norm_bwd_param_k<DT, true>), dim3((unsigned)((p.cols + 255) / 256), (unsigned)chunks), block, 0, st, (const S *)p.x, (const S *)p.dy, stats, part, p.rows, (int)p.cols, rpc);
            else hipLaunchKernelGGL((norm_bwd_param_k<DT, false>), dim3((unsigned)((p.cols + 63) / 64), (unsigned)chunks), block, 0, st, (const S *)p.x, (const S *)p.dy, stats, part, p.rows, (int)p.cols, rpc);
        }
        hipLaunchKernelGGL((norm_bwd_param_sum_k<DT>), dim3((unsigned)((p.cols + 31) / 32), 2), dim3(1024), 0, st, part, (S *)p.dw, (S *)p.db, (int)p.cols, chunks);
    }
    return hipGetLastError();
}

template <int DT, int MODE> hipError_t launch_norm(const NormRows &p, hipStream_t st) {
    typedef typename RowIO<DT>::S S;
    dim3 grid((unsigned)((p.rows + 3) / 4)), block(256);
    const int esz = (int)sizeof(S);
    bool vec = p.cols % 4 == 0 && reinterpret_cast<uintptr_t>(p.x) % (4 * esz) == 0 && reinterpret_cast<uintptr_t>(p.y) % (4 * esz) == 0;
#define ZK_FWD_REG(NV) hipLaunchKernelGGL((norm_rows_reg_k<DT, MODE, NV>), grid, block, 0, st, (const S *)p.x, (const S *)p.w, (const S *)p.b, (S *)p.y, p.rows, p.eps)
    auto al = [&](const void *q) { return reinterpret_cast<uintptr_t>(q) % (4 * esz) == 0; };
    const bool al16 = vec && al(p.w) && al(p.b);
    if (al16 && p.cols == 256) ZK_FWD_REG(1);
    else if (al16 && p.cols == 512) ZK_FWD_REG(2);
    else if (al16 && p.cols == 1024) ZK_FWD_REG(4);
    else if (al16 && p.cols == 2048) ZK_FWD_REG(8);
    else if (al16 && p.cols == 4096) ZK_FWD_REG(16);
#undef ZK_FWD_REG
    else if (al16 && p.cols <= 16384) {
        // VE elements per 16-byte (or, 16-bit rows of an odd multiple of 4 columns, 8-byte) vector; W = waves per row
        // (4 * 64 * VE columns each at most); NV = 3 or 4 vectors per lane
        constexpr int VMAX = DT == 1 ? 8 : 4;
        const bool wide_vec = DT == 1 && p.cols > 1024 /* below, 8-byte vectors fill the lanes better */ && p.cols % 8 == 0 && reinterpret_cast<uintptr_t>(p.x) % 16 == 0 && reinterpret_cast<uintptr_t>(p.y) % 16 == 0 &&
                              (!p.w || reinterpret_cast<uintptr_t>(p.w) % 16 == 0) && (!p.b || reinterpret_cast<uintptr_t>(p.b) % 16 == 0);
        const int ve = wide_vec ? 8 : 4, cap = 256 * ve; // columns of a wave at NV = 4
        const int W = p.cols <= cap ? 1 : p.cols <= 2 * cap ? 2 : p.cols <= 4 * cap ? 4 : p.cols <= 8 * cap ? 8 : 16;
        const bool three = p.cols <= 3 * 64 * ve * W;
        const int rpb = W < 4 ? 4 / W : 1;
        const dim3 wgrid((unsigned)((p.rows + rpb - 1) / rpb)), wblock(W < 4 ? 256 : 64 * W);
#define ZK_WIDE(NVV, WV, VEV) hipLaunchKernelGGL((norm_rows_wide_k<DT, MODE, NVV, WV, VEV>), wgrid, wblock, 0, st, (const S *)p.x, (const S *)p.w, (const S *)p.b, (S *)p.y, p.rows, (int)p.cols, p.eps)
#define ZK_WIDE2(WV)                                                                                                              \
    do {                                                                                                                          \
        if (wide_vec && three) ZK_WIDE(3, WV, VMAX);                                                                              \
        else if (wide_vec) ZK_WIDE(4, WV, VMAX);                                                                                  \
        else if (three) ZK_WIDE(3, WV, 4);                                                                                        \
        else ZK_WIDE(4, WV, 4);                                                                                                   \
    } while (0)
        if (W == 1) ZK_WIDE2(1);
        else if (W == 2) ZK_WIDE2(2);
        else if (W == 4) ZK_WIDE2(4);
        else if (W == 8) ZK_WIDE2(8);
        else ZK_WIDE2(16);
#undef ZK_WIDE2
#undef ZK_WIDE
    } else if (vec) hipLaunchKernelGGL((norm_rows_k<DT, MODE, true>), grid, block, 0, st, (const S *)p.x, (const S *)p.w, (const S *)p.b, (S *)p.y, p.rows, (int)p.cols, p.eps);
    else hipLaunchKernelGGL((norm_rows_k<DT, MODE, false>), grid, block, 0, st, (const S *)p.x, (const S *)p.w, (const S *)p.b, (S *)p.y, p.rows, (int)p.cols, p.eps);
    return hipGetLastError();
}

} // namespace

hipError_t norm_rows(const NormRows &p, hipStream_t st) {
    if (p.rows <= 0 || p.cols <= 0) return hipSuccess;
    if (p.cols >= (1ll << 31) || (p.rows + 3) / 4 >= (1ll << 31)) return hipErrorInvalidValue;
    if (p.dtype == DT_F32) return p.rms ? launch_norm<0, 1>(p, st) : launch_norm<0, 0>(p, st);
    if (p.dtype == DT_BF16) return p.rms ? launch_norm<1, 1>(p, st) : launch_norm<1, 0>(p, st);
    return hipErrorInvalidValue;
}

uint64_t norm_rows_bwd_workspace_bytes(int64_t rows, int64_t cols) { // row statistics, then up to 256 partial row pairs
    return (uint64_t)rows * 8 + 256ull * 2 * (uint64_t)cols * 4;
}

hipError_t norm_rows_bwd(const NormRowsBwd &p, hipStream_t st) {
    if (p.rows <= 0 || p.cols <= 0) return hipSuccess;
    if (p.cols >= (1ll << 31) || (p.rows + 3) / 4 >= (1ll << 31) || !p.workspace ||
        p.workspace_bytes < norm_rows_bwd_workspace_bytes(p.rows, p.cols))
        return hipErrorInvalidValue;
    if (p.dtype == DT_F32) return p.rms ? launch_norm_bwd<0, 1>(p, st) : launch_norm_bwd<0, 0>(p, st);
    if (p.dtype == DT_BF16) return p.rms ? launch_norm_bwd<1, 1>(p, st) : launch_norm_bwd<1, 0>(p, st);
    return hipErrorInvalidValue;
}

hipError_t cross_entropy(const CrossEntropy &p, hipStream_t st) {
    if (p.rows <= 0 || p.cols <= 0) return hipSuccess;
    if (p.cols >= (1ll << 31) || (p.rows + 3) / 4 >= (1ll << 31)) return hipErrorInvalidValue;
    const void *target = p.dense ? (const void *)p.dense : (const void *)p.labels;
    if (p.mean) {
        if (p.rows > kCrossEntropyMeanRows) return hipErrorInvalidValue;
        if (p.dense) hipLaunchKernelGGL(cross_entropy_mean_k<true>, dim3(1), dim3(1024), 0, st, p.x, target, p.loss, p.grad, p.mean, p.rows, (int)p.cols, p.gscale);
        else hipLaunchKernelGGL(cross_entropy_mean_k<false>, dim3(1), dim3(1024), 0, st, p.x, target, p.loss, p.grad, p.mean, p.rows, (int)p.cols, p.gscale);
        return hipGetLastError();
    }
    if (!p.dense && p.cols > 2048 && p.cols <= 65536 && p.rows < (1ll << 31)) {
        const bool vec = p.cols % 4 == 0 && reinterpret_cast<uintptr_t>(p.x) % 16 == 0 && (!p.grad || reinterpret_cast<uintptr_t>(p.grad) % 16 == 0);
#define ZK_CE(NE, W)                                                                                                              \
    do {                                                                                                                          \
        if (vec) hipLaunchKernelGGL((cross_entropy_wide_k<NE, W, true>), dim3((unsigned)p.rows), dim3(64 * W), 0, st, p.x, p.labels, p.loss, p.grad, (int)p.cols, p.gscale); \
        else hipLaunchKernelGGL((cross_entropy_wide_k<NE, W, false>), dim3((unsigned)p.rows), dim3(64 * W), 0, st, p.x, p.labels, p.loss, p.grad, (int)p.cols, p.gscale); \
    } while (0)
        if (p.cols <= 4096) ZK_CE(16, 4);
        else if (p.cols <= 8192) ZK_CE(16, 8);
        else if (p.cols <= 16384) ZK_CE(16, 16);
        else if (p.cols <= 32768) ZK_CE(32, 16);
        else ZK_CE(64, 16);
#undef ZK_CE
        return hipGetLastError();
    }
    const dim3 grid((unsigned)((p.rows + 3) / 4));
    if (p.dense) hipLaunchKernelGGL(cross_entropy_k<true>, grid, dim3(256), 0, st, p.x, target, p.loss, p.grad, p.rows, (int)p.cols, p.gscale);
    else hipLaunchKernelGGL(cross_entropy_k<false>, grid, dim3(256), 0, st, p.x, target, p.loss, p.grad, p.rows, (int)p.cols, p.gscale);
    return hipGetLastError();
}

} // namespace zk
