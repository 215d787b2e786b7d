// conv2d forward as an implicit GEMM on the matrix cores, and max-pooling.
//
// zyx lowers Tensor::conv (zyx/src/tensor/mod.rs:2583-2680) to pad -> pool view -> broadcast
// multiply with the weight -> sum over (cin, ky, kx) (+ bias), i.e. for NCHW input x and weight
// w[cout, cin, kh, kw]:
//   y[n, co, oy, ox] = sum_{c,ky,kx} x[n, c, oy*sy - py + ky*dy, ox*sx - px + kx*dx] * w[co, c, ky, kx]
// with zero outside the image (the reference multiplies by a 0/1 mask, zyx/src/kernel/
// linearize.rs:349-382; here out-of-image taps are simply not read). Products and sums are
// f32; bf16 tensors store the result truncated (zyx/src/tensor/reduce_ops.rs:134-136).
//
// GEMM view: C'[co, p] = W[co, k] . X'[k, p], k = (c, ky, kx), p = (n, oy, ox). The weight is
// the K-contiguous operand as stored; X' is gathered on the fly (im2col never exists in HBM).
// Pixels are the MFMA column index, so a wave's stores run along ox: contiguous in NCHW.
// 64 or 128 (cout) x 64 (pixels) per workgroup, K step 32, 2 x 2 waves.
// The k -> (input offset, dy, dx) table is built on the host at registration and read with
// wave-uniform (scalar) loads.
//
// Tensor::max_pool (zyx/src/tensor/mod.rs:2706-2741): pad with the dtype's lowest value,
// window view, max over the window: one thread per output element.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int CM = 64, CN = 64, CK = 32;
// LDS row padding: bf16 rows of 80 bytes keep the 128-bit fragment reads of 16 consecutive rows on distinct
// banks; f32 rows of 33 words do the same for the one-word reads of 32 consecutive rows.
template <int DT> constexpr int cpad() { return DT == DT_F32 ? 1 : 8; }

template <int DT> struct CT;
template <> struct CT<DT_F32> { typedef float S; };
template <> struct CT<DT_BF16> { typedef uint16_t S; };

// MT = 1: 64 (cout) x 64 (pixels) per workgroup, 2 x 2 waves of one 32 x 32 tile. MT = 2: 128 x 64, 2 x 2 waves of
// two stacked 32 x 32 tiles, so the gathered pixel tile is formed once for 128 output channels. The loads of K
// step s+1 are issued into registers before the MFMAs of step s and written to LDS after them.
template <int DT, int ODT, int MT>
__global__ __launch_bounds__(256) void conv2d_k(const Conv2d p) {
    typedef typename CT<DT>::S S;
    constexpr int TM = CM * MT, CPAD = cpad<DT>();
    __shared__ __attribute__((aligned(16))) S Ws[TM * (CK + CPAD)];
    __shared__ __attribute__((aligned(16))) S Xs[CN * (CK + CPAD)];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t co0 = (int64_t)blockIdx.y * TM, p0 = (int64_t)blockIdx.x * CN;
    const int64_t K = (int64_t)p.C * p.KH * p.KW, OHW = (int64_t)p.OH * p.OW, P = (int64_t)p.N * OHW;
    const S *W = (const S *)p.w, *X = (const S *)p.x;

    // this thread gathers pixel p0 + (t & 63) for 8 values of k per K tile
    const int64_t pix = p0 + (t & 63);
    const bool pix_ok = pix < P;
    const int64_t n = pix_ok ? pix / OHW : 0, rem = pix_ok ? pix - n * OHW : 0;
    const int oy = (int)(rem / p.OW), ox = (int)(rem - (int64_t)oy * p.OW);
    const int iy0 = oy * p.sy - p.py, ix0 = ox * p.sx - p.px;
    const S *xn = X + n * (int64_t)p.C * p.H * p.W + (int64_t)iy0 * p.W + ix0;

    f32x16 acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[m][r] = 0.0f;

    S rw[8 * MT], rx[8];
    auto fetch = [&](int64_t k0) {
#pragma unroll
        for (int e = 0; e < 8 * MT; e++) { // weight tile: K contiguous, consecutive threads along k
            const int idx = e * 256 + t, r = idx >> 5, k = idx & 31;
            const int64_t gr = co0 + r, gk = k0 + k;
            rw[e] = (gr < p.Cout && gk < K) ? W[gr * K + gk] : (S)0;
        }
#pragma unroll
        for (int e = 0; e < 8; e++) { // gathered tile: k is uniform over a wave, lanes walk along the pixels
            const int kl = __builtin_amdgcn_readfirstlane((t >> 6) + 4 * e);
            const int64_t gk = k0 + kl;
            S v = (S)0;
            if (gk < K) {
                const int32_t off = p.koff[gk];
                const int32_t dyx = p.kdyx[gk];
                const int iy = iy0 + (dyx >> 16), ix = ix0 + (dyx & 0xffff);
                if (pix_ok && iy >= 0 && iy < p.H && ix >= 0 && ix < p.W) v = xn[off];
            }
            rx[e] = v;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int e = 0; e < 8 * MT; e++) {
            const int idx = e * 256 + t;
            Ws[(idx >> 5) * (CK + CPAD) + (idx & 31)] = rw[e];
        }
#pragma unroll
        for (int e = 0; e < 8; e++) Xs[(t & 63) * (CK + CPAD) + (t >> 6) + 4 * e] = rx[e];
    };

    fetch(0);
    for (int64_t k0 = 0; k0 < K; k0 += CK) {
        __syncthreads(); // the previous step's fragment reads are done
        stash();
        __syncthreads();
        if (k0 + CK < K) fetch(k0 + CK); // in flight while the matrix cores work on this step
        const S *br = Xs + (wn * 32 + (lane & 31)) * (CK + CPAD);
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const S *ar = Ws + ((wm * MT + m) * 32 + (lane & 31)) * (CK + CPAD);
            if (DT == DT_F32) {
#pragma unroll
                for (int ks = 0; ks < CK; ks += 2) {
                    float a = ((const float *)ar)[ks + (lane >> 5)], b = ((const float *)br)[ks + (lane >> 5)];
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[m], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int ks = 0; ks < CK; ks += 16) {
                    const int off = ks + (lane >> 5) * 8;
                    bf16x8 a = *(const bf16x8 *)((const uint16_t *)ar + off), b = *(const bf16x8 *)((const uint16_t *)br + off);
                    acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[m], 0, 0, 0);
                }
            }
        }
    }

    // register r of lane l: row (cout) 8*(r/4) + 4*(l/32) + r%4, column (pixel) l%32
    const int64_t opix = p0 + wn * 32 + (lane & 31);
    if (opix >= P) return; // no barrier follows
    const int64_t on = opix / OHW, orem = opix - on * OHW;
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int64_t co = co0 + (wm * MT + m) * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (co >= p.Cout) continue;
            float v = acc[m][r];
            if (p.bias) v += DT == DT_F32 ? ((const float *)p.bias)[co] : bf16_to_f32(((const uint16_t *)p.bias)[co]);
            if (p.relu) v = (v > 0.0f ? 1.0f : 0.0f) * v;
            const int64_t o = (on * p.Cout + co) * OHW + orem;
            if (ODT == DT_F32) ((float *)p.y)[o] = v;
            else ((uint16_t *)p.y)[o] = f32_to_bf16_trunc(v);
        }
}

template <int DT>
__global__ __launch_bounds__(256) void max_pool2d_k(const MaxPool2d p) {
    typedef typename CT<DT>::S S;
    const int64_t total = p.planes * p.OH * p.OW;
    const S *X = (const S *)p.x;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t plane = i / ((int64_t)p.OH * p.OW), rem = i - plane * p.OH * p.OW;
        const int oy = (int)(rem / p.OW), ox = (int)(rem - (int64_t)oy * p.OW);
        const S *xp = X + plane * (int64_t)p.H * p.W;
        float m = DT == DT_F32 ? -FLT_MAX : -3.3895313892515355e38f; // dtype.min: f32::MIN / bf16::MIN (0xff7f)
        for (int ky = 0; ky < p.KH; ky++) {
            const int iy = oy * p.sy - p.py + ky * p.dy;
            if (iy < 0 || iy >= p.H) continue;
            for (int kx = 0; kx < p.KW; kx++) {
                const int ix = ox * p.sx - p.px + kx * p.dx;
                if (ix < 0 || ix >= p.W) continue;
                const float v = DT == DT_F32 ? ((const float *)xp)[(int64_t)iy * p.W + ix] : bf16_to_f32(((const uint16_t *)xp)[(int64_t)iy * p.W + ix]);
                m = fmaxf(v, m);
            }
        }
        if (DT == DT_F32) ((float *)p.y)[i] = m;
        else ((uint16_t *)p.y)[i] = f32_to_bf16_trunc(m);
    }
}

// 2 x 2 windows, stride 2, no padding or dilation, rows of a multiple of 8 elements (the pool after a convolution
// block): a thread reads 16 bytes of each of its two input rows. The running maximum starts at the dtype's lowest
// finite value like the general kernel's, so NaN and -inf inputs come out alike.
// f32, two outputs per thread: one 16-byte load per input row, so that the lanes of a load instruction read consecutive
// memory (with four outputs per thread the two loads of a row interleave at 32-byte steps).
__global__ __launch_bounds__(256) void max_pool2x2_f32_pairs_k(const MaxPool2d p) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    const int ow2 = p.OW >> 1;
    const int64_t total = p.planes * p.OH * ow2;
    const float lowest = -FLT_MAX;
    const float *x = (const float *)p.x;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t prow = i / ow2; // plane * OH + oy
        const int q = (int)(i - prow * ow2);
        const int64_t plane = prow / p.OH;
        const int oy = (int)(prow - plane * p.OH);
        const int64_t in0 = (plane * p.H + 2 * oy) * (int64_t)p.W + 4 * q;
        const f32x4 a = __builtin_nontemporal_load((const f32x4 *)(x + in0));
        const f32x4 b = __builtin_nontemporal_load((const f32x4 *)(x + in0 + p.W));
        const f32x2 v = {fmaxf(b[1], fmaxf(b[0], fmaxf(a[1], fmaxf(a[0], lowest)))),
                         fmaxf(b[3], fmaxf(b[2], fmaxf(a[3], fmaxf(a[2], lowest))))}; // window order
        __builtin_nontemporal_store(v, (f32x2 *)((float *)p.y + prow * p.OW + 2 * q));
    }
}

// bf16, four outputs per thread: one 16-byte load (8 elements) per input row.
__global__ __launch_bounds__(256) void max_pool2x2_bf16_k(const MaxPool2d p) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const int ow4 = p.OW >> 2;
    const int64_t total = p.planes * p.OH * ow4;
    const float lowest = -3.3895313892515355e38f;
    const uint16_t *x = (const uint16_t *)p.x;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t prow = i / ow4; // plane * OH + oy
        const int q = (int)(i - prow * ow4);
        const int64_t plane = prow / p.OH;
        const int oy = (int)(prow - plane * p.OH);
        const int64_t in0 = (plane * p.H + 2 * oy) * (int64_t)p.W + 8 * q;
        float r[2][8];
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const u32x4 t = __builtin_nontemporal_load((const u32x4 *)(x + in0 + (int64_t)a * p.W));
#pragma unroll
            for (int e = 0; e < 4; e++) {
                r[a][2 * e] = __uint_as_float(t[e] << 16);
                r[a][2 * e + 1] = __uint_as_float(t[e] & 0xffff0000u);
            }
        }
        float m[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            m[j] = fmaxf(r[1][2 * j + 1], fmaxf(r[1][2 * j], fmaxf(r[0][2 * j + 1], fmaxf(r[0][2 * j], lowest)))); // window order
        const u32x2 v = {(uint32_t)f32_to_bf16_trunc(m[0]) | ((uint32_t)f32_to_bf16_trunc(m[1]) << 16),
                         (uint32_t)f32_to_bf16_trunc(m[2]) | ((uint32_t)f32_to_bf16_trunc(m[3]) << 16)};
        __builtin_nontemporal_store(v, (u32x2 *)((uint16_t *)p.y + prow * p.OW + 4 * q));
    }
}

// Patch matrix of the convolution, transposed: a[k][pixel] with k = (c*KH + ky)*KW + kx (the order of the
// flattened weight [Cout, C*KH*KW]) and pixel = (n*OH + oy)*OW + ox; padding reads as 0. Rows of `a` run
// along the image rows of x, so reads and the 16-byte writes are both coalesced. One thread = 8 pixels.
__global__ __launch_bounds__(256) void im2col_t_bf16_k(const uint16_t *__restrict__ x, uint16_t *__restrict__ a, const Conv2d p,
                                                      int64_t pixels) {
    const int k = blockIdx.y;
    const int kx = k % p.KW, ky = (k / p.KW) % p.KH, c = k / (p.KW * p.KH);
    const int64_t pix0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (pix0 >= pixels) return;
    const int plane = p.OH * p.OW;
    int n = (int)(pix0 / plane), rem = (int)(pix0 - (int64_t)n * plane);
    int oy = rem / p.OW, ox = rem - oy * p.OW;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    const int iy0 = oy * p.sy - p.py + ky * p.dy, ix0 = ox * p.sx - p.px + kx * p.dx;
    if (p.sx == 1 && ox + 8 <= p.OW) {
        // the 8 pixels lie in one output row: one input row, 8 consecutive columns
        if (iy0 >= 0 && iy0 < p.H) {
            const uint16_t *row = x + (((int64_t)n * p.C + c) * p.H + iy0) * p.W;
            if (ix0 >= 0 && ix0 + 8 <= p.W) {
                typedef uint32_t u32x4a2 __attribute__((ext_vector_type(4), aligned(2)));
                const u32x4a2 t = *(const u32x4a2 *)(row + ix0); // 2-byte aligned 128-bit load
                w[0] = t[0]; w[1] = t[1]; w[2] = t[2]; w[3] = t[3];
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int ix = ix0 + e;
                    const uint32_t v = (ix >= 0 && ix < p.W) ? row[ix] : 0u;
                    w[e >> 1] |= v << (16 * (e & 1));
                }
            }
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int iy = oy * p.sy - p.py + ky * p.dy, ix = ox * p.sx - p.px + kx * p.dx;
            uint32_t v = 0;
            if (iy >= 0 && iy < p.H && ix >= 0 && ix < p.W) v = x[(((int64_t)n * p.C + c) * p.H + iy) * p.W + ix];
            w[e >> 1] |= v << (16 * (e & 1));
            if (++ox == p.OW) {
                ox = 0;
                if (++oy == p.OH) {
                    oy = 0;
                    n++;
                }
            }
        }
    }
    *(uint4 *)(a + (int64_t)k * pixels + pix0) = make_uint4(w[0], w[1], w[2], w[3]);
}

// Zero-padded copy of the input, xp[n, c, H + 2*py, W + 2*px]: with it every tap of every output pixel is an
// in-bounds read, so the GEMM can gather its patch rows with plain 128-bit loads and no masks.
__global__ __launch_bounds__(256) void pad_input_bf16_k(const uint16_t *__restrict__ x, uint16_t *__restrict__ xp, int H, int W,
                                                        int py, int px, int total) {
    // 32-bit index arithmetic (total < 2^30). A thread fills 8 consecutive elements of the padded array (one 128-bit
    // store; xp is 16-byte aligned): the position is decoded once by division and then stepped across row and
    // plane ends, the 8 source elements are neighbouring 2-byte loads.
    const int Hp = H + 2 * py, Wp = W + 2 * px;
    for (int i = (blockIdx.x * 256 + threadIdx.x) * 8; i < total; i += gridDim.x * 256 * 8) {
        int plane = i / (Hp * Wp);
        const int rem = i - plane * (Hp * Wp);
        int yy = rem / Wp, xx = rem - yy * Wp;
        uint32_t v[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int sy = yy - py, sx = xx - px;
            v[e] = (i + e < total && sy >= 0 && sy < H && sx >= 0 && sx < W) ? x[((int64_t)plane * H + sy) * W + sx] : 0u;
            if (++xx == Wp) {
                xx = 0;
                if (++yy == Hp) {
                    yy = 0;
                    ++plane;
                }
            }
        }
        if (i + 8 <= total) {
            typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
            u32x4 w = {v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16)};
            *(u32x4 *)(xp + i) = w;
        } else {
            for (int e = 0; i + e < total; e++) xp[i + e] = (uint16_t)v[e];
        }
    }
}

// bf16 convolutions whose lowered product fits the tiled MFMA GEMM exactly: patches . W^T with
// M = pixels (multiple of 256), N = Cout (multiple of 128), K = C*KH*KW (multiple of 64), no K split.
bool conv_uses_gemm(const Conv2d &p) {
    const int64_t pixels = (int64_t)p.N * p.OH * p.OW, K = (int64_t)p.C * p.KH * p.KW;
    return p.dtype == DT_BF16 && pixels > 0 && pixels % 256 == 0 && (p.OH * p.OW) % 4 == 0 && p.Cout % 128 == 0 && K % 64 == 0 &&
           K <= 65535 && pixels < (1ll << 30) && gemm_bf16_supported(pixels, p.Cout, K) && gemm_bf16_splits(pixels, p.Cout, K) == 1;
}
constexpr uint64_t kZeroBiasBytes = 4096 * 4;
// ... and whose patch rows are runs of 8 consecutive input columns (unit column stride, rows of 8k outputs): the
// GEMM gathers them itself from a padded copy of the input and no patch matrix is written.
bool conv_gathers_in_gemm(const Conv2d &p) {
    return conv_uses_gemm(p) && p.sx == 1 && p.OW % 8 == 0 &&
           (int64_t)p.N * p.C * (p.H + 2 * p.py) * (p.W + 2 * p.px) < (1ll << 30);
}

} // namespace

// scratch = [zero bias (for ReLU without bias)] [patch matrix K x pixels bf16]
uint64_t conv2d_scratch_bytes(const Conv2d &p) {
    if (conv3x3_direct_ok(p)) return kZeroBiasBytes + conv3x3_scratch_bytes(p); // the direct kernel: re-laid weights only
    if (!conv_uses_gemm(p) || p.Cout > 4096) return 0;
    if (conv_gathers_in_gemm(p)) // padded input (+ 16 bytes: the last 128-bit load may start 7 elements before the end)
        return kZeroBiasBytes + (uint64_t)p.N * p.C * (p.H + 2 * p.py) * (p.W + 2 * p.px) * 2 + 16;
    return kZeroBiasBytes + (uint64_t)p.C * p.KH * p.KW * (uint64_t)p.N * p.OH * p.OW * 2;
}

hipError_t conv2d(const Conv2d &p, hipStream_t st) {
    const int64_t P = (int64_t)p.N * p.OH * p.OW;
    if (P <= 0 || p.Cout <= 0) return hipSuccess;
    if (p.scratch && conv3x3_direct_ok(p)) return conv3x3_direct(p, (char *)p.scratch + kZeroBiasBytes, st);
    if (p.scratch && conv2d_scratch_bytes(p)) {
        // im2col (transposed) + GEMM: C[pixel, co] = sum_k a[k, pixel] * w[co, k], stored as NCHW by the epilogue
        uint16_t *a = (uint16_t *)((char *)p.scratch + kZeroBiasBytes);
        const int K = p.C * p.KH * p.KW;
        GemmBf16 g{};
        if (conv_gathers_in_gemm(p)) {
            const int Hp = p.H + 2 * p.py, Wp = p.W + 2 * p.px;
            const int total = p.N * p.C * Hp * Wp; // < 2^30, checked by conv_gathers_in_gemm
            int blocks = ((total + 7) / 8 + 255) / 256;
            if (blocks > 256 * 64) blocks = 256 * 64;
            hipLaunchKernelGGL(pad_input_bf16_k, dim3((unsigned)blocks), dim3(256), 0, st, (const uint16_t *)p.x, a, p.H, p.W, p.py, p.px, total);
            ConvGather &c = g.gather;
            c.ohw = p.OH * p.OW;
            c.ow = p.OW;
            c.img = p.C * Hp * Wp;
            c.row = p.sy * Wp;
            c.cs = Hp * Wp;
            c.rs = p.dy * Wp;
            c.dx = p.dx;
            c.khw = (uint32_t)(p.KH * p.KW);
            c.kw = (uint32_t)p.KW;
            c.magic_khw = (uint32_t)(((1ull << 32) + c.khw - 1) / c.khw);
            c.magic_kw = (uint32_t)(((1ull << 32) + c.kw - 1) / c.kw);
        } else
            hipLaunchKernelGGL(im2col_t_bf16_k, dim3((unsigned)((P / 8 + 255) / 256), (unsigned)K), dim3(256), 0, st, (const uint16_t *)p.x, a, p, P);
        g.M = P;
        g.N = p.Cout;
        g.K = K;
        g.trans_a = 1;
        g.trans_b = 1;
        g.epilogue = p.relu ? 2 : (p.bias ? 1 : 0);
        g.bias_dtype = DT_BF16;
        g.out_bf16 = p.out_dtype == DT_BF16;
        g.plane = p.OH * p.OW;
        g.A = a;
        g.B = p.w;
        g.bias = p.bias ? p.bias : p.scratch; // the head of scratch is kept zero
        g.C = p.y;
        return gemm_bf16(g, st);
    }
    const int mt = p.Cout > CM ? 2 : 1;
    const int64_t tm = CM * mt;
    if ((p.Cout + tm - 1) / tm > 65535 || (P + CN - 1) / CN >= (1ll << 31)) return hipErrorInvalidValue;
    dim3 grid((unsigned)((P + CN - 1) / CN), (unsigned)((p.Cout + tm - 1) / tm)), block(256);
#define ZK_CONV(D, O)                                                                   \
    if (mt == 2) hipLaunchKernelGGL((conv2d_k<D, O, 2>), grid, block, 0, st, p);        \
    else hipLaunchKernelGGL((conv2d_k<D, O, 1>), grid, block, 0, st, p)
    if (p.dtype == DT_F32 && p.out_dtype == DT_F32) { ZK_CONV(DT_F32, DT_F32); }
    else if (p.dtype == DT_BF16 && p.out_dtype == DT_BF16) { ZK_CONV(DT_BF16, DT_BF16); }
    else if (p.dtype == DT_BF16 && p.out_dtype == DT_F32) { ZK_CONV(DT_BF16, DT_F32); }
    else return hipErrorInvalidValue;
#undef ZK_CONV
    return hipGetLastError();
}

hipError_t max_pool2d(const MaxPool2d &p, hipStream_t st) {
    const int64_t total = p.planes * p.OH * p.OW;
    if (total <= 0) return hipSuccess;
    if (p.KH == 2 && p.KW == 2 && p.sy == 2 && p.sx == 2 && p.py == 0 && p.px == 0 && p.dy == 1 && p.dx == 1 && p.W % 8 == 0 &&
        p.H >= 2 && (uintptr_t)p.x % 16 == 0 && (uintptr_t)p.y % 16 == 0 && (p.dtype == DT_F32 || p.dtype == DT_BF16)) {
        const int64_t quads = p.planes * p.OH * (p.OW / 4);
        const unsigned grid = (unsigned)std::min<int64_t>((quads + 255) / 256, 256 * 32);
        if (p.dtype == DT_F32) { // config 4: 14.0 us with four outputs per thread, 10.2 us with two
            const int64_t items = p.planes * p.OH * (p.OW / 2);
            hipLaunchKernelGGL(max_pool2x2_f32_pairs_k, dim3((unsigned)std::min<int64_t>((items + 255) / 256, 256 * 64)), dim3(256), 0, st, p);
        }
        else hipLaunchKernelGGL(max_pool2x2_bf16_k, dim3(grid), dim3(256), 0, st, p);
        return hipGetLastError();
    }
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (p.dtype == DT_F32) hipLaunchKernelGGL((max_pool2d_k<DT_F32>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    else if (p.dtype == DT_BF16) hipLaunchKernelGGL((max_pool2d_k<DT_BF16>), dim3((unsigned)blocks), dim3(256), 0, st, p);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

} // namespace zk
