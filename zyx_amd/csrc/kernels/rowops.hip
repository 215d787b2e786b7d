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

// Cross-entropy with class-index targets, one wave per sample. loss[r] = -(ln_softmax(x)[label])
// computed as the reference does: m = x - max; ls = m - ln(sum exp(m)); loss = sum_c -ls[c] * onehot[c].
// grad (optional) = (softmax(x) - onehot) * gscale, the gradient of gscale * sum_r loss[r].
// A label outside [0, cols) matches no class (all-zero one-hot): loss 0, grad = softmax * gscale.
__global__ __launch_bounds__(256) void cross_entropy_k(const float *__restrict__ x, const int32_t *__restrict__ labels,
                                                       float *__restrict__ loss, float *__restrict__ grad, int64_t rows,
                                                       int cols, float gscale) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *xr = x + row * cols;
    float mx = -FLT_MAX;
    for (int c = lane; c < cols; c += 64) mx = fmaxf(xr[c], mx);
    mx = wave_allreduce_f32(mx, OpMaxF());
    float s = 0.0f;
    for (int c = lane; c < cols; c += 64) s += expf(xr[c] - mx);
    s = wave_allreduce_f32(s, OpAdd());
    const float lns = logf(s);
    const int label = labels[row];
    if (loss && lane == 0) {
        float l = 0.0f;
        if (label >= 0 && label < cols) l = -((xr[label] - mx) - lns);
        loss[row] = l;
    }
    if (grad) {
        const float inv = 1.0f / s;
        for (int c = lane; c < cols; c += 64) {
            float p = expf(xr[c] - mx) * inv;
            grad[row * cols + c] = (p - (c == label ? 1.0f : 0.0f)) * gscale;
        }
    }
}

template <int DT, int MODE> hipError_t launch_norm(const NormRows &p, hipStream_t st) {
    typedef typename RowIO<DT>::S S;
    dim3 grid((unsigned)((p.rows + 3) / 4)), block(256);
    const int esz = (int)sizeof(S);
    bool vec = p.cols % 4 == 0 && reinterpret_cast<uintptr_t>(p.x) % (4 * esz) == 0 && reinterpret_cast<uintptr_t>(p.y) % (4 * esz) == 0;
    if (vec) hipLaunchKernelGGL((norm_rows_k<DT, MODE, true>), grid, block, 0, st, (const S *)p.x, (const S *)p.w, (const S *)p.b, (S *)p.y, p.rows, (int)p.cols, p.eps);
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

hipError_t cross_entropy(const CrossEntropy &p, hipStream_t st) {
    if (p.rows <= 0 || p.cols <= 0) return hipSuccess;
    if (p.cols >= (1ll << 31) || (p.rows + 3) / 4 >= (1ll << 31)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(cross_entropy_k, dim3((unsigned)((p.rows + 3) / 4)), dim3(256), 0, st, p.x, p.labels, p.loss, p.grad,
                       p.rows, (int)p.cols, p.gscale);
    return hipGetLastError();
}

} // namespace zk
