// gather / index_select / scatter along one axis of a tensor of rank <= 4.
//
// zyx builds these from a dense one-hot (zyx/src/tensor/index_ops.rs:321-445):
//   gather:  out[i] = sum_k onehot(idx[i])[k] * x[.., k, ..]        -> x[.., idx[i], ..]
//   scatter: out = self + sum over index positions j along the axis of
//                         onehot(idx[.., j, ..]) * src[.., j, ..]    (duplicates add up)
// with one wrap of negative indices (idx + (idx < 0) * dim) and an all-zero one-hot for
// anything still out of range: gather reads 0 there, scatter drops the contribution.
// Here gather is one indexed load per output element (any 1/2/4/8-byte dtype, bit copy), and
// scatter is evaluated per OUTPUT element, folding the matching index positions j in
// ascending order and adding `self` last -- the reference's summation order, so float
// results are deterministic and integer results exact.
#include "dtypes.hpp"
#include "kernels.hpp"

#include <algorithm>

namespace zk {

namespace {

__device__ __forceinline__ int64_t load_index(const void *idx, int idx64, int64_t i) {
    return idx64 ? ((const int64_t *)idx)[i] : (int64_t)((const int32_t *)idx)[i];
}

template <typename T> __global__ __launch_bounds__(256) void gather_k(const IndexOp p) {
    const int64_t total = p.os[0] * p.os[1] * p.os[2] * p.os[3];
    const T *x = (const T *)p.x;
    T *out = (T *)p.out;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        int64_t c[4], rem = i;
#pragma unroll
        for (int d = 3; d >= 0; d--) {
            c[d] = rem % p.os[d];
            rem /= p.os[d];
        }
        // index_select: a 1-D index addressed by the coordinate along the axis
        int64_t v = load_index(p.idx, p.idx64, p.select ? c[p.axis] : i);
        const int64_t dim = p.xs[p.axis];
        if (v < 0) v += dim;
        T r = (T)0;
        if (v >= 0 && v < dim) {
            c[p.axis] = v;
            r = x[((c[0] * p.xs[1] + c[1]) * p.xs[2] + c[2]) * p.xs[3] + c[3]];
        }
        out[i] = r;
    }
}

template <typename T> __global__ __launch_bounds__(256) void scatter_k(const IndexOp p) {
    // output has the shape of `self` (xs); idx and src have shape os
    const int64_t total = p.xs[0] * p.xs[1] * p.xs[2] * p.xs[3];
    const T *self = (const T *)p.x, *src = (const T *)p.src;
    T *out = (T *)p.out;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        int64_t c[4], rem = i;
#pragma unroll
        for (int d = 3; d >= 0; d--) {
            c[d] = rem % p.xs[d];
            rem /= p.xs[d];
        }
        bool covered = true; // index positions exist only inside the index tensor's extent
#pragma unroll
        for (int d = 0; d < 4; d++)
            if (d != p.axis && c[d] >= p.os[d]) covered = false;
        T acc = (T)0;
        if (covered) {
            const int64_t target = c[p.axis], dim = p.xs[p.axis];
            int64_t q[4] = {c[0], c[1], c[2], c[3]};
            for (int64_t j = 0; j < p.os[p.axis]; j++) {
                q[p.axis] = j;
                const int64_t pos = ((q[0] * p.os[1] + q[1]) * p.os[2] + q[2]) * p.os[3] + q[3];
                int64_t v = load_index(p.idx, p.idx64, pos);
                if (v < 0) v += dim;
                if (v == target) acc = acc + src[pos];
            }
        }
        out[i] = acc + self[i];
    }
}


} // namespace

hipError_t index_op(const IndexOp &p, hipStream_t st) {
    const int64_t total = p.scatter ? p.xs[0] * p.xs[1] * p.xs[2] * p.xs[3] : p.os[0] * p.os[1] * p.os[2] * p.os[3];
    if (total <= 0) return hipSuccess;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    dim3 grid((unsigned)blocks), block(256);
    if (!p.scatter) {
        switch (dtype_size(p.dtype)) {
        case 1: hipLaunchKernelGGL(gather_k<uint8_t>, grid, block, 0, st, p); break;
        case 2: hipLaunchKernelGGL(gather_k<uint16_t>, grid, block, 0, st, p); break;
        case 4: hipLaunchKernelGGL(gather_k<uint32_t>, grid, block, 0, st, p); break;
        default: hipLaunchKernelGGL(gather_k<uint64_t>, grid, block, 0, st, p); break;
        }
    } else {
        switch (p.dtype) {
        case DT_F32: hipLaunchKernelGGL(scatter_k<float>, grid, block, 0, st, p); break;
        case DT_I32: hipLaunchKernelGGL(scatter_k<uint32_t>, grid, block, 0, st, p); break; // wrapping adds
        case DT_U32: hipLaunchKernelGGL(scatter_k<uint32_t>, grid, block, 0, st, p); break;
        case DT_I64: case DT_U64: hipLaunchKernelGGL(scatter_k<uint64_t>, grid, block, 0, st, p); break;
        case DT_F64: hipLaunchKernelGGL(scatter_k<double>, grid, block, 0, st, p); break;
        default: return hipErrorInvalidValue;
        }
    }
    return hipGetLastError();
}

namespace {
// Range copy for small device-to-device moves (a batch sliced out of a resident dataset): a kernel launch costs the
// host a fraction of what the runtime's asynchronous memcpy does. 16 bytes per thread when both ends allow.
template <typename T> __global__ __launch_bounds__(256) void copy_range_k(T *__restrict__ dst, const T *__restrict__ src, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256) dst[i] = src[i];
}
} // namespace

hipError_t copy_range(void *dst, const void *src, uint64_t bytes, hipStream_t st) {
    if (bytes == 0) return hipSuccess;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const bool wide = ((uintptr_t)dst | (uintptr_t)src | bytes) % 16 == 0;
    const uint64_t n = wide ? bytes / 16 : bytes;
    const unsigned grid = (unsigned)std::min<uint64_t>((n + 255) / 256, 4096);
    if (wide) hipLaunchKernelGGL(copy_range_k<u32x4>, dim3(grid), dim3(256), 0, st, (u32x4 *)dst, (const u32x4 *)src, n);
    else hipLaunchKernelGGL(copy_range_k<uint8_t>, dim3(grid), dim3(256), 0, st, (uint8_t *)dst, (const uint8_t *)src, n);
    return hipGetLastError();
}

} // namespace zk
