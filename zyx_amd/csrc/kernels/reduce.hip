// Row (last-axis) and column (axis-0) sum / max reductions.
//
// Semantics: zyx/src/tensor/reduce_ops.rs:45-147 -- floats accumulate in f32 and are cast
// back to the input dtype on store, ints accumulate in i32; the accumulator starts at 0
// for sum and at the dtype's lowest finite value for max (zyx/src/kernel/linearize.rs:
// 920-952, zyx/src/dtype.rs:207-224). The reference folds serially; here each lane folds
// a strided slice with 128-bit loads and lanes are combined by DPP wave reductions (rows)
// or an LDS transpose-free fold over the four waves of a workgroup (columns). Long
// single rows / tall thin matrices are split over several workgroups whose partials a
// second, tiny launch folds.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

template <int OP, typename A> struct Fold;
template <> struct Fold<0, float> {
    static __device__ __forceinline__ float init() { return 0.0f; }
    static __device__ __forceinline__ float f(float a, float b) { return a + b; }
};
template <> struct Fold<1, float> {
    static __device__ __forceinline__ float init() { return -FLT_MAX; }
    static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); }
};
template <> struct Fold<0, int> {
    static __device__ __forceinline__ int init() { return 0; }
    static __device__ __forceinline__ int f(int a, int b) { return (int)((unsigned)a + (unsigned)b); }
};
template <> struct Fold<1, int> {
    static __device__ __forceinline__ int init() { return INT32_MIN; }
    static __device__ __forceinline__ int f(int a, int b) { return a > b ? a : b; }
};

// element access by dtype class: DT 0 = f32, 1 = bf16, 2 = f16, 3 = i32
template <int DT> struct Elem;
template <> struct Elem<0> {
    typedef float S; typedef float A;
    static __device__ __forceinline__ float ld(const float *p, int64_t i) { return p[i]; }
    static __device__ __forceinline__ void ld4(const float *p, int64_t i, float (&v)[4]) {
        f32x4 t = __builtin_nontemporal_load((const f32x4 *)(p + i)); // read once
        v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
    }
    static __device__ __forceinline__ void st(float *p, int64_t i, float v) { p[i] = v; }
};
template <> struct Elem<1> {
    typedef uint16_t S; typedef float A;
    static __device__ __forceinline__ float ld(const uint16_t *p, int64_t i) { return bf16_to_f32(p[i]); }
    static __device__ __forceinline__ void ld4(const uint16_t *p, int64_t i, float (&v)[4]) {
        typedef uint32_t u32x2nt __attribute__((ext_vector_type(2)));
        const u32x2nt tt = __builtin_nontemporal_load((const u32x2nt *)(p + i)); // read once
        const uint2 t = make_uint2(tt[0], tt[1]);
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
    }
    static __device__ __forceinline__ void ld8(const uint16_t *p, int64_t i, float (&v)[8]) {
        typedef uint32_t u32x4nt __attribute__((ext_vector_type(4)));
        const u32x4nt tt = __builtin_nontemporal_load((const u32x4nt *)(p + i)); // read once
        const uint4 t = make_uint4(tt[0], tt[1], tt[2], tt[3]);
        const unsigned w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[2 * k] = __uint_as_float(w[k] << 16);
            v[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ void st(uint16_t *p, int64_t i, float v) { p[i] = f32_to_bf16_trunc(v); }
};
template <> struct Elem<2> {
    typedef uint16_t S; typedef float A;
    static __device__ __forceinline__ float ld(const uint16_t *p, int64_t i) { return f16_to_f32(p[i]); }
    static __device__ __forceinline__ void ld4(const uint16_t *p, int64_t i, float (&v)[4]) {
        typedef uint32_t u32x2nt __attribute__((ext_vector_type(2)));
        const u32x2nt tt = __builtin_nontemporal_load((const u32x2nt *)(p + i)); // read once
        const uint2 t = make_uint2(tt[0], tt[1]);
        v[0] = f16_to_f32((uint16_t)t.x); v[1] = f16_to_f32((uint16_t)(t.x >> 16));
        v[2] = f16_to_f32((uint16_t)t.y); v[3] = f16_to_f32((uint16_t)(t.y >> 16));
    }
    static __device__ __forceinline__ void ld8(const uint16_t *p, int64_t i, float (&v)[8]) {
        typedef uint32_t u32x4nt __attribute__((ext_vector_type(4)));
        const u32x4nt tt = __builtin_nontemporal_load((const u32x4nt *)(p + i)); // read once
        const uint4 t = make_uint4(tt[0], tt[1], tt[2], tt[3]);
        const unsigned w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            v[2 * k] = f16_to_f32((uint16_t)w[k]);
            v[2 * k + 1] = f16_to_f32((uint16_t)(w[k] >> 16));
        }
    }
    static __device__ __forceinline__ void st(uint16_t *p, int64_t i, float v) { p[i] = f32_to_f16_trunc(v); }
};
template <> struct Elem<3> {
    typedef int32_t S; typedef int A;
    static __device__ __forceinline__ int ld(const int32_t *p, int64_t i) { return p[i]; }
    static __device__ __forceinline__ void ld4(const int32_t *p, int64_t i, int (&v)[4]) {
        i32x4 t = __builtin_nontemporal_load((const i32x4 *)(p + i)); // read once
        v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
    }
    static __device__ __forceinline__ void st(int32_t *p, int64_t i, int v) { p[i] = v; }
};

template <int OP> __device__ __forceinline__ float wave_fold(float v) {
    if (OP == 0) return wave_allreduce_f32(v, OpAdd());
    return wave_allreduce_f32(v, OpMaxF());
}
template <int OP> __device__ __forceinline__ int wave_fold(int v) {
    if (OP == 0) return wave_allreduce_i32(v, OpAdd());
    return wave_allreduce_i32(v, OpMaxI());
}

// Final store of result i: for the float dtypes optionally (acc * mul) / div + base[i], each step a separate f32
// operation in that order (`p - g * lr` with mul = -lr and base = p; a mean with div = n); integers store acc as is.
struct Epilogue {
    float mul, div;     // 0 = step absent
    const void *base;   // nullptr = absent; same dtype and length as out
};
template <int DT> __device__ __forceinline__ void store_result(typename Elem<DT>::S *out, int64_t i, typename Elem<DT>::A acc,
                                                               const Epilogue &e) {
    if constexpr (std::is_same<typename Elem<DT>::A, float>::value) {
#pragma clang fp contract(off)
        float v = acc;
        if (e.mul != 0.0f) v = v * e.mul;
        if (e.div != 0.0f) v = v / e.div;
        if (e.base) v = v + Elem<DT>::ld((const typename Elem<DT>::S *)e.base, i);
        Elem<DT>::st(out, i, v);
    } else {
        Elem<DT>::st(out, i, acc);
    }
}

// One wave folds columns [c0, c1) of one row. VEC: row start and c0 are 4-element aligned.
template <int DT, int OP, bool VEC>
__device__ __forceinline__ typename Elem<DT>::A fold_row_span(const typename Elem<DT>::S *__restrict__ xr, int64_t c0,
                                                              int64_t c1, int lane, int nlanes) {
    typedef typename Elem<DT>::A A;
    typedef Fold<OP, A> F;
    A acc = F::init();
    if constexpr (sizeof(typename Elem<DT>::S) == 2) {
        // 16-bit rows whose span is whole 16-byte pieces: 8 elements per request, eight requests in flight per lane
        if (VEC && ((c1 - c0) & 7) == 0 && (c0 & 7) == 0 && (reinterpret_cast<uintptr_t>(xr) & 15) == 0) {
            const int64_t nv = (c1 - c0) >> 3;
            int64_t i = lane;
            for (; i + 7 * nlanes < nv; i += 8 * nlanes) {
                A v[8][8];
#pragma unroll
                for (int u = 0; u < 8; u++) Elem<DT>::ld8(xr, c0 + (i + u * nlanes) * 8, v[u]);
#pragma unroll
                for (int u = 0; u < 8; u++)
                    acc = F::f(acc, F::f(F::f(F::f(v[u][0], v[u][1]), F::f(v[u][2], v[u][3])), F::f(F::f(v[u][4], v[u][5]), F::f(v[u][6], v[u][7]))));
            }
            for (; i < nv; i += nlanes) {
                A v[8];
                Elem<DT>::ld8(xr, c0 + i * 8, v);
                acc = F::f(acc, F::f(F::f(F::f(v[0], v[1]), F::f(v[2], v[3])), F::f(F::f(v[4], v[5]), F::f(v[6], v[7]))));
            }
            return acc;
        }
    }
    if (VEC) {
        int64_t nv = (c1 - c0) >> 2;
        int64_t i = lane;
        for (; i + 7 * nlanes < nv; i += 8 * nlanes) { // eight requests in flight per lane
            A v[8][4];
#pragma unroll
            for (int u = 0; u < 8; u++) Elem<DT>::ld4(xr, c0 + (i + u * nlanes) * 4, v[u]);
#pragma unroll
            for (int u = 0; u < 8; u++) acc = F::f(acc, F::f(F::f(v[u][0], v[u][1]), F::f(v[u][2], v[u][3])));
        }
        for (; i < nv; i += nlanes) {
            A v[4];
            Elem<DT>::ld4(xr, c0 + i * 4, v);
            acc = F::f(acc, F::f(F::f(v[0], v[1]), F::f(v[2], v[3])));
        }
        for (int64_t c = c0 + nv * 4 + lane; c < c1; c += nlanes) acc = F::f(acc, Elem<DT>::ld(xr, c));
    } else {
        for (int64_t c = c0 + lane; c < c1; c += nlanes) acc = F::f(acc, Elem<DT>::ld(xr, c));
    }
    return acc;
}

// rows: one wave per (row, segment); 4 waves per workgroup. With segs == 1 the result is
// stored as DT, otherwise the raw accumulator goes to partial[row * segs + seg].
template <int DT, int OP, bool VEC>
__global__ __launch_bounds__(256) void reduce_rows_wave_k(const typename Elem<DT>::S *__restrict__ x,
                                                          typename Elem<DT>::S *__restrict__ out,
                                                          typename Elem<DT>::A *__restrict__ partial, int64_t rows,
                                                          int64_t cols, int segs, int64_t seg_len, const Epilogue epi) {
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= rows * segs) return; // whole wave; no cross-wave synchronisation below
    const int64_t row = item / segs;
    const int seg = (int)(item - row * segs);
    const int64_t c0 = seg * seg_len, c1 = min(cols, c0 + seg_len);
    typename Elem<DT>::A acc = fold_row_span<DT, OP, VEC>(x + row * cols, c0, c1, lane, 64);
    acc = wave_fold<OP>(acc);
    if (lane == 0) {
        if (segs == 1) store_result<DT>(out, row, acc, epi);
        else partial[item] = acc;
    }
}

// rows, many of middling length: a workgroup per row, its W waves take a W-th each (a wave's requests then cover a
// few KiB of consecutive memory, which the memory system serves faster than one wave walking the whole row) and the
// parts meet in LDS. part_len is a multiple of 8 elements.
template <int DT, int OP, bool VEC, int W>
__global__ __launch_bounds__(64 * W) void reduce_rows_group_k(const typename Elem<DT>::S *__restrict__ x,
                                                              typename Elem<DT>::S *__restrict__ out, int64_t cols,
                                                              int64_t part_len, const Epilogue epi) {
    typedef typename Elem<DT>::A A;
    typedef Fold<OP, A> F;
    __shared__ A part[W];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t row = blockIdx.x;
    const int64_t c0 = min(cols, wave * part_len), c1 = min(cols, c0 + part_len);
    A acc = fold_row_span<DT, OP, VEC>(x + row * cols, c0, c1, lane, 64);
    acc = wave_fold<OP>(acc);
    if (lane == 0) part[wave] = acc;
    __syncthreads(); // every thread arrives: no early exit above
    if (threadIdx.x == 0) {
        A v = part[0];
#pragma unroll
        for (int w = 1; w < W; w++) v = F::f(v, part[w]);
        store_result<DT>(out, row, v, epi);
    }
}

// second stage: fold `segs` raw partials per row (accumulator type), store as DT.
template <int DT, int OP>
__global__ __launch_bounds__(256) void reduce_partials_k(const typename Elem<DT>::A *__restrict__ partial,
                                                         typename Elem<DT>::S *__restrict__ out, int64_t rows, int segs,
                                                         const Epilogue epi) {
    typedef typename Elem<DT>::A A;
    typedef Fold<OP, A> F;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    A acc = F::init();
    for (int s = lane; s < segs; s += 64) acc = F::f(acc, partial[row * segs + s]);
    acc = wave_fold<OP>(acc);
    if (lane == 0) store_result<DT>(out, row, acc, epi);
}

// columns: a workgroup owns a strip of 64 * W columns (lane -> W adjacent columns: 16 bytes per lane and row where
// width and alignment allow, W = 4 for 32-bit and 8 for 16-bit elements; W = 1 otherwise) and a chunk of rows split
// over its 4 waves.
template <int DT, int OP, int W>
__global__ __launch_bounds__(256) void reduce_cols_k(const typename Elem<DT>::S *__restrict__ x,
                                                     typename Elem<DT>::S *__restrict__ out,
                                                     typename Elem<DT>::A *__restrict__ partial, int64_t rows,
                                                     int64_t cols, int chunks, int64_t chunk_len, const Epilogue epi) {
    typedef typename Elem<DT>::A A;
    typedef Fold<OP, A> F;
    __shared__ A lds[4][64 * W];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t c = ((int64_t)blockIdx.x * 64 + lane) * W;
    const int chunk = blockIdx.y;
    const int64_t r0 = chunk * chunk_len, r1 = min(rows, r0 + chunk_len);
    A acc[W];
#pragma unroll
    for (int k = 0; k < W; k++) acc[k] = F::init();
    if (c < cols) {
#pragma unroll 8
        for (int64_t r = r0 + wave; r < r1; r += 4) { // unrolled: 8 independent row loads in flight per thread
            if constexpr (W == 8) {
                A v[8];
                Elem<DT>::ld8(x, r * cols + c, v);
#pragma unroll
                for (int k = 0; k < W; k++) acc[k] = F::f(acc[k], v[k]);
            } else if constexpr (W == 4) {
                A v[4];
                Elem<DT>::ld4(x, r * cols + c, v);
#pragma unroll
                for (int k = 0; k < W; k++) acc[k] = F::f(acc[k], v[k]);
            } else {
                acc[0] = F::f(acc[0], Elem<DT>::ld(x, r * cols + c));
            }
        }
    }
#pragma unroll
    for (int k = 0; k < W; k++) lds[wave][lane * W + k] = acc[k];
    __syncthreads(); // every thread of the workgroup arrives: no early exit above
    if (wave == 0 && c < cols) {
#pragma unroll
        for (int k = 0; k < W; k++) {
            A v = F::f(F::f(lds[0][lane * W + k], lds[1][lane * W + k]), F::f(lds[2][lane * W + k], lds[3][lane * W + k]));
            if (chunks == 1) store_result<DT>(out, c + k, v, epi);
            else partial[(int64_t)chunk * cols + c + k] = v;
        }
    }
}
// second stage for columns: partial[chunks, cols] (accumulator type) -> out[cols]
template <int DT, int OP>
__global__ __launch_bounds__(256) void reduce_col_partials_k(const typename Elem<DT>::A *__restrict__ partial,
                                                             typename Elem<DT>::S *__restrict__ out, int64_t cols,
                                                             int chunks, const Epilogue epi) {
    typedef typename Elem<DT>::A A;
    typedef Fold<OP, A> F;
    // a workgroup folds 64 columns: lane -> column, the 4 waves split the chunks, LDS joins them
    __shared__ A lds[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t c = (int64_t)blockIdx.x * 64 + lane;
    A acc = F::init();
    if (c < cols) {
#pragma unroll 8
        for (int k = wave; k < chunks; k += 4) acc = F::f(acc, partial[(int64_t)k * cols + c]);
    }
    lds[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && c < cols) store_result<DT>(out, c, F::f(F::f(lds[0][lane], lds[1][lane]), F::f(lds[2][lane], lds[3][lane])), epi);
}

struct RowPlan { int segs; int64_t seg_len; };
RowPlan plan_rows(int64_t rows, int64_t cols) {
    // enough waves to fill 256 CUs (~8 per CU) when there are few long rows
    int segs = 1;
    if (rows < 2048 && cols >= 8192) {
        int64_t want = (2048 + rows - 1) / rows;
        int64_t max_by_len = cols / 4096; // a segment keeps >= 4096 elements
        segs = (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, max_by_len), 1024));
    }
    int64_t seg_len = (cols + segs - 1) / segs;
    seg_len = (seg_len + 3) / 4 * 4; // keep segment starts 4-aligned
    segs = (int)((cols + seg_len - 1) / seg_len);
    return {segs, seg_len};
}
struct ColPlan { int chunks; int64_t chunk_len; };
ColPlan plan_cols(int64_t rows, int64_t cols, int width) { // width of a strip: 64, 256 or 512 columns
    int64_t strips = (cols + width - 1) / width;
    int chunks = 1;
    // two workgroups per compute unit (one for the widest strips) measured best at 8192 x 4096: more, shorter chunks
    // pay their start-up and the second stage's longer fold, fewer leave units idle
    const int64_t target = width >= 512 ? 256 : 512;
    if (strips < target && rows >= 256) {
        int64_t want = (target + strips - 1) / strips;
        chunks = (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, rows / 64), 4096));
    }
    int64_t chunk_len = (rows + chunks - 1) / chunks;
    chunks = (int)((rows + chunk_len - 1) / chunk_len);
    return {chunks, chunk_len};
}

template <int DT, int OP> hipError_t launch(const Reduce &p, hipStream_t st) {
    typedef typename Elem<DT>::S S;
    typedef typename Elem<DT>::A A;
    const S *x = (const S *)p.x;
    S *out = (S *)p.out;
    A *ws = (A *)p.workspace;
    const int esz = (int)sizeof(S);
    const Epilogue epi{p.mul, p.div, p.base};
    if (!p.axis0) {
        bool vec = (p.cols * esz) % (4 * esz) == 0 && p.cols % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
        RowPlan pl = plan_rows(p.rows, p.cols);
        if (pl.segs > 1 && (uint64_t)p.rows * pl.segs * sizeof(A) > p.workspace_bytes) return hipErrorInvalidValue;
        const int64_t row_bytes = p.cols * esz;
        if (pl.segs == 1 && p.rows >= 2048 && p.rows <= 0x7fffffff && row_bytes >= 8192 && row_bytes <= 65536) {
            // waves per row, measured at 8192 x 2048 .. 2048 x 16384 f32: rows of 16 KiB gain from eight (23.9 -> 21.9 us at
            // 8192 x 4096, 2 KiB per wave), shorter and longer rows do not (8 KiB: 12.2 vs 13.4 us; 32 KiB: 23.0 vs 25.0)
            const int W = row_bytes >= 12288 && row_bytes < 24576 ? 8 : 4;
            dim3 grid((unsigned)p.rows);
            const int64_t part_len = ((p.cols + W - 1) / W + 7) / 8 * 8;
#define ZK_ROWS(WV)                                                                                                               \
    do {                                                                                                                          \
        if (vec) hipLaunchKernelGGL((reduce_rows_group_k<DT, OP, true, WV>), grid, dim3(64 * WV), 0, st, x, out, p.cols, part_len, epi); \
        else hipLaunchKernelGGL((reduce_rows_group_k<DT, OP, false, WV>), grid, dim3(64 * WV), 0, st, x, out, p.cols, part_len, epi);    \
    } while (0)
            if (W == 8) ZK_ROWS(8);
            else ZK_ROWS(4);
#undef ZK_ROWS
            return hipGetLastError();
        }
        int64_t items = p.rows * pl.segs;
        dim3 grid((unsigned)((items + 3) / 4)), block(256);
        if (vec) hipLaunchKernelGGL((reduce_rows_wave_k<DT, OP, true>), grid, block, 0, st, x, out, ws, p.rows, p.cols, pl.segs, pl.seg_len, epi);
        else hipLaunchKernelGGL((reduce_rows_wave_k<DT, OP, false>), grid, block, 0, st, x, out, ws, p.rows, p.cols, pl.segs, pl.seg_len, epi);
        if (pl.segs > 1)
            hipLaunchKernelGGL((reduce_partials_k<DT, OP>), dim3((unsigned)((p.rows + 3) / 4)), block, 0, st, ws, out, p.rows, pl.segs, epi);
    } else {
        const bool al16 = reinterpret_cast<uintptr_t>(x) % 16 == 0;
        const int W = (esz == 2 && al16 && p.cols % 8 == 0) ? 8 : (al16 && p.cols % 4 == 0) ? 4 : 1;
        ColPlan pl = plan_cols(p.rows, p.cols, 64 * W);
        if (pl.chunks > 1 && (uint64_t)pl.chunks * p.cols * sizeof(A) > p.workspace_bytes) return hipErrorInvalidValue;
        int64_t strips = (p.cols + 64 * W - 1) / (64 * W);
        dim3 grid((unsigned)strips, (unsigned)pl.chunks), block(256);
        if constexpr (sizeof(S) == 2) {
            if (W == 8) hipLaunchKernelGGL((reduce_cols_k<DT, OP, 8>), grid, block, 0, st, x, out, ws, p.rows, p.cols, pl.chunks, pl.chunk_len, epi);
        }
        if (W == 4) hipLaunchKernelGGL((reduce_cols_k<DT, OP, 4>), grid, block, 0, st, x, out, ws, p.rows, p.cols, pl.chunks, pl.chunk_len, epi);
        else if (W == 1) hipLaunchKernelGGL((reduce_cols_k<DT, OP, 1>), grid, block, 0, st, x, out, ws, p.rows, p.cols, pl.chunks, pl.chunk_len, epi);
        if (pl.chunks > 1)
            hipLaunchKernelGGL((reduce_col_partials_k<DT, OP>), dim3((unsigned)((p.cols + 63) / 64)), block, 0, st, ws, out, p.cols, pl.chunks, epi);
    }
    return hipGetLastError();
}


// ---- argmax along one axis of a contiguous [outer, n, inner] view -----------------------------------------------
// Tensor::argmax_axis (zyx/src/tensor/mod.rs:2238-2269) is max_k((x == max_keepdim(x)) * k) cast to i32: the LARGEST
// index among equal maxima; the maximum is a reduce from the dtype's lowest finite value in which a NaN never wins
// (fmax), and a NaN never equals it, so NaN entries are skipped and a row without any finite candidate gives 0.
// One pass keeps (best value, largest index holding it); pairs combine associatively, so lanes, waves and workgroups
// may fold slices in any order and the result is the reference's.
template <typename A> struct Best {
    A v;
    int i;
};
template <typename A> __device__ __forceinline__ A lowest();
template <> __device__ __forceinline__ float lowest<float>() { return -FLT_MAX; }
template <> __device__ __forceinline__ int lowest<int>() { return INT32_MIN; }
template <typename A> __device__ __forceinline__ void best_take(Best<A> &b, A v, int i) {
    if (v > b.v) {
        b.v = v;
        b.i = i;
    } else if (v == b.v) {
        b.i = max(b.i, i);
    }
}
__device__ __forceinline__ float shfl_xor_any(float v, int m) { return __shfl_xor(v, m, 64); }
__device__ __forceinline__ int shfl_xor_any(int v, int m) { return __shfl_xor(v, m, 64); }
template <typename A> __device__ __forceinline__ Best<A> wave_best(Best<A> b) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        A ov = shfl_xor_any(b.v, m);
        int oi = __shfl_xor(b.i, m, 64);
        best_take(b, ov, oi);
    }
    return b;
}

// inner == 1: one wave per (row, segment) of x[rows, n]; lanes stride the span with 4-element loads when VEC.
template <int DT, bool VEC>
__global__ __launch_bounds__(256) void argmax_rows_k(const typename Elem<DT>::S *__restrict__ x, int32_t *__restrict__ out,
                                                     typename Elem<DT>::A *__restrict__ pv, int32_t *__restrict__ pi,
                                                     int64_t rows, int64_t n, int segs, int64_t seg_len) {
    typedef typename Elem<DT>::A A;
    const int lane = threadIdx.x & 63;
    const int64_t item = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= rows * segs) return; // whole wave
    const int64_t row = item / segs;
    const int seg = (int)(item - row * segs);
    const int64_t c0 = seg * seg_len, c1 = min(n, c0 + seg_len);
    const typename Elem<DT>::S *xr = x + row * n;
    Best<A> b{lowest<A>(), 0};
    if (VEC) {
        const int64_t nv = (c1 - c0) >> 2;
        for (int64_t i = lane; i < nv; i += 64) {
            A v[4];
            Elem<DT>::ld4(xr, c0 + i * 4, v);
#pragma unroll
            for (int k = 0; k < 4; k++) best_take(b, v[k], (int)(c0 + i * 4 + k));
        }
        for (int64_t c = c0 + nv * 4 + lane; c < c1; c += 64) best_take(b, Elem<DT>::ld(xr, c), (int)c);
    } else {
        for (int64_t c = c0 + lane; c < c1; c += 64) best_take(b, Elem<DT>::ld(xr, c), (int)c);
    }
    b = wave_best(b);
    if (lane == 0) {
        if (segs == 1) out[row] = b.i;
        else {
            pv[item] = b.v;
            pi[item] = b.i;
        }
    }
}
// second stage of both layouts: result r folds partial pairs r * stride_r + s * stride_s, s < parts
template <typename A>
__global__ __launch_bounds__(256) void argmax_partials_k(const A *__restrict__ pv, const int32_t *__restrict__ pi,
                                                         int32_t *__restrict__ out, int64_t n_out, int parts,
                                                         int64_t stride_r, int64_t stride_s) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= n_out) return;
    Best<A> b{lowest<A>(), 0};
    for (int s = 0; s < parts; s++) best_take(b, pv[r * stride_r + s * stride_s], pi[r * stride_r + s * stride_s]);
    out[r] = b.i;
}
// inner > 1: a workgroup owns 64 neighbouring inner positions of one outer slice (lane -> position, coalesced rows)
// and a chunk of the axis split over its 4 waves; LDS joins the waves.
template <int DT>
__global__ __launch_bounds__(256) void argmax_mid_k(const typename Elem<DT>::S *__restrict__ x, int32_t *__restrict__ out,
                                                    typename Elem<DT>::A *__restrict__ pv, int32_t *__restrict__ pi,
                                                    int64_t n, int64_t inner, int strips, int chunks, int64_t chunk_len) {
    typedef typename Elem<DT>::A A;
    __shared__ A lv[4][64];
    __shared__ int li[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t o = blockIdx.x / strips;
    const int64_t c = (int64_t)(blockIdx.x % strips) * 64 + lane;
    const int chunk = blockIdx.y;
    const int64_t r0 = chunk * chunk_len, r1 = min(n, r0 + chunk_len);
    Best<A> b{lowest<A>(), 0};
    if (c < inner) {
        const typename Elem<DT>::S *xo = x + o * n * inner + c;
#pragma unroll 8
        for (int64_t r = r0 + wave; r < r1; r += 4) best_take(b, Elem<DT>::ld(xo, r * inner), (int)r);
    }
    lv[wave][lane] = b.v;
    li[wave][lane] = b.i;
    __syncthreads(); // every thread arrives: no early exit above
    if (wave == 0 && c < inner) {
#pragma unroll
        for (int w = 1; w < 4; w++) best_take(b, lv[w][lane], li[w][lane]);
        if (chunks == 1) out[o * inner + c] = b.i;
        else {
            pv[(o * chunks + chunk) * inner + c] = b.v;
            pi[(o * chunks + chunk) * inner + c] = b.i;
        }
    }
}

struct ArgPlan { int parts; int64_t len; int strips; };
ArgPlan plan_argmax(int64_t outer, int64_t n, int64_t inner) {
    if (inner == 1) {
        RowPlan r = plan_rows(outer, n);
        return {r.segs, r.seg_len, 0};
    }
    const int64_t strips = (inner + 63) / 64, blocks = strips * outer;
    int chunks = 1;
    if (blocks < 1024 && n >= 256) chunks = (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>((1024 + blocks - 1) / blocks, n / 64), 4096));
    int64_t len = (n + chunks - 1) / chunks;
    chunks = (int)((n + len - 1) / len);
    return {chunks, len, (int)strips};
}

template <int DT> hipError_t launch_argmax(const ArgMax &p, hipStream_t st) {
    typedef typename Elem<DT>::S S;
    typedef typename Elem<DT>::A A;
    const S *x = (const S *)p.x;
    const ArgPlan pl = plan_argmax(p.outer, p.n, p.inner);
    const int64_t n_out = p.outer * p.inner;
    A *pv = (A *)p.workspace;
    int32_t *pi = (int32_t *)((char *)p.workspace + (uint64_t)n_out * pl.parts * 4);
    if (pl.parts > 1 && (uint64_t)n_out * pl.parts * 8 > p.workspace_bytes) return hipErrorInvalidValue;
    if (p.inner == 1) {
        const bool vec = p.n % 4 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
        dim3 grid((unsigned)((p.outer * pl.parts + 3) / 4)), block(256);
        if (vec) hipLaunchKernelGGL((argmax_rows_k<DT, true>), grid, block, 0, st, x, p.out, pv, pi, p.outer, p.n, pl.parts, pl.len);
        else hipLaunchKernelGGL((argmax_rows_k<DT, false>), grid, block, 0, st, x, p.out, pv, pi, p.outer, p.n, pl.parts, pl.len);
        if (pl.parts > 1)
            hipLaunchKernelGGL((argmax_partials_k<A>), dim3((unsigned)((n_out + 255) / 256)), block, 0, st, pv, pi, p.out, n_out, pl.parts, (int64_t)pl.parts, (int64_t)1);
    } else {
        dim3 grid((unsigned)(pl.strips * p.outer), (unsigned)pl.parts), block(256);
        hipLaunchKernelGGL((argmax_mid_k<DT>), grid, block, 0, st, x, p.out, pv, pi, p.n, p.inner, pl.strips, pl.parts, pl.len);
        if (pl.parts > 1) { // result (o, c) folds partial[(o * parts + s) * inner + c]: walk the outer slices one launch each
            for (int64_t o = 0; o < p.outer; o++)
                hipLaunchKernelGGL((argmax_partials_k<A>), dim3((unsigned)((p.inner + 255) / 256)), block, 0, st,
                                   pv + o * pl.parts * p.inner, pi + o * pl.parts * p.inner, p.out + o * p.inner, p.inner,
                                   pl.parts, (int64_t)1, p.inner);
        }
    }
    return hipGetLastError();
}

} // namespace

bool reduce_shape_ok(int64_t rows, int64_t cols, int axis0) {
    if (rows < 0 || cols < 0 || (cols && rows > (1ll << 40) / cols)) return false;
    if (rows == 0 || cols == 0) return (axis0 ? cols : rows) < (1ll << 33); // the fill of an empty reduce: 4 results per workgroup
    if (!axis0) return rows * plan_rows(rows, cols).segs < (1ll << 33); // 4 (row, segment) items per workgroup, grid.x < 2^31
    return (cols + 63) / 64 < (1ll << 31); // column strips along grid.x; chunks <= 4096 along grid.y
}

uint64_t reduce_workspace_bytes(int64_t rows, int64_t cols, int axis0) {
    if (rows <= 0 || cols <= 0) return 0;
    if (!axis0) {
        RowPlan pl = plan_rows(rows, cols);
        return pl.segs > 1 ? (uint64_t)rows * pl.segs * 4 : 0;
    }
    // whichever strip width the launch picks (alignment and dtype decide), its partials fit
    const int chunks = std::max(plan_cols(rows, cols, 64).chunks, std::max(plan_cols(rows, cols, 256).chunks, plan_cols(rows, cols, 512).chunks));
    return chunks > 1 ? (uint64_t)chunks * cols * 4 : 0;
}

hipError_t reduce(const Reduce &p, hipStream_t st) {
    if (p.rows < 0 || p.cols < 0) return hipErrorInvalidValue;
    int64_t n_out = p.axis0 ? p.cols : p.rows;
    if (n_out == 0) return hipSuccess;
    if ((p.axis0 ? p.rows : p.cols) == 0) {
        // reducing an empty axis leaves the accumulator's initial value; one tiny fill via
        // the partials kernel with zero segments
        switch (p.dtype * 2 + p.op) {
#define ZK_EMPTY(DTC, DT, OP)                                                                                        \
    case DTC * 2 + OP:                                                                                                \
        hipLaunchKernelGGL((reduce_partials_k<DT, OP>), dim3((unsigned)((n_out + 3) / 4)), dim3(256), 0, st,          \
                           (const typename Elem<DT>::A *)nullptr, (typename Elem<DT>::S *)p.out, n_out, 0,            \
                           Epilogue{p.mul, p.div, p.base});                                                            \
        return hipGetLastError();
            ZK_EMPTY(DT_F32, 0, 0) ZK_EMPTY(DT_F32, 0, 1) ZK_EMPTY(DT_BF16, 1, 0) ZK_EMPTY(DT_BF16, 1, 1)
            ZK_EMPTY(DT_F16, 2, 0) ZK_EMPTY(DT_F16, 2, 1) ZK_EMPTY(DT_I32, 3, 0) ZK_EMPTY(DT_I32, 3, 1)
#undef ZK_EMPTY
        default: return hipErrorInvalidValue;
        }
    }
    switch (p.dtype * 2 + p.op) {
    case DT_F32 * 2 + 0: return launch<0, 0>(p, st);
    case DT_F32 * 2 + 1: return launch<0, 1>(p, st);
    case DT_BF16 * 2 + 0: return launch<1, 0>(p, st);
    case DT_BF16 * 2 + 1: return launch<1, 1>(p, st);
    case DT_F16 * 2 + 0: return launch<2, 0>(p, st);
    case DT_F16 * 2 + 1: return launch<2, 1>(p, st);
    case DT_I32 * 2 + 0: return launch<3, 0>(p, st);
    case DT_I32 * 2 + 1: return launch<3, 1>(p, st);
    default: return hipErrorInvalidValue;
    }
}

bool argmax_shape_ok(int64_t outer, int64_t n, int64_t inner) {
    if (outer < 0 || n < 1 || inner < 0 || n >= (1ll << 31)) return false; // indices are i32; an empty axis has no arg-max
    if (outer == 0 || inner == 0) return true;
    if (outer > (1ll << 40) / inner || outer * inner > (1ll << 40) / n) return false;
    if (inner == 1) return outer * plan_rows(outer, n).segs < (1ll << 33);
    return (inner + 63) / 64 * outer < (1ll << 31);
}

uint64_t argmax_workspace_bytes(int64_t outer, int64_t n, int64_t inner) {
    if (outer <= 0 || n <= 0 || inner <= 0) return 0;
    const ArgPlan pl = plan_argmax(outer, n, inner);
    return pl.parts > 1 ? (uint64_t)outer * inner * pl.parts * 8 : 0;
}

hipError_t argmax(const ArgMax &p, hipStream_t st) {
    if (!argmax_shape_ok(p.outer, p.n, p.inner)) return hipErrorInvalidValue;
    const int64_t n_out = p.outer * p.inner;
    if (n_out == 0) return hipSuccess;
    switch (p.dtype) {
    case DT_F32: return launch_argmax<0>(p, st);
    case DT_BF16: return launch_argmax<1>(p, st);
    case DT_F16: return launch_argmax<2>(p, st);
    case DT_I32: return launch_argmax<3>(p, st);
    default: return hipErrorInvalidValue;
    }
}

} // namespace zk
