// LDS-tiled f32 GEMM on v_mfma_f32_32x32x2_f32 for products whose M and N are multiples of 64 and K of 32: what
// `Tensor::dot` of two f32 matrices needs at size (zyx/src/tensor/mod.rs:1469-1518; zyx/tests/05_misc.rs:820-842
// multiplies 1024^3; the reference's own custom-kernel matchers claim exactly this dtype, zyx/src/backend/cblas.rs:
// 265-268). Everything else about the product (ragged shapes, split-K, small problems) stays with gemm_generic.hip,
// which calls in here.
//
// Workgroup tile TM x TN (128 x 128 or 64 x 64), K tile 32, 4 waves in a 2 x 2 grid, each wave (TM/2) x (TN/2) of C in
// 32 x 32 MFMA tiles. Operands go global -> registers -> LDS, one K tile ahead of the multiply; one LDS stage (35 KiB,
// several workgroups share a CU and hide each other's barriers). Two LDS layouts, by which index runs along memory:
//   * k contiguous (A[M,K], B stored [N,K]): [k/4][row][4], so the four k a lane needs for four consecutive matrix
//     instructions are one ds_read_b128. The instruction takes A[row][k = lane/32] per lane: instruction j of a group
//     of four multiplies k = j and k = 4 + j of an 8-wide k step, lane half h holding k = 4h .. 4h + 3.
//   * row index contiguous (A stored [K,M], B[K,N]): [k][row] with rows padded so that the two k a wave reads at once
//     fall into different bank halves; four one-word reads per group of four instructions.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
constexpr int FK = 32; // K tile

// byte size of one operand tile of R rows in either layout, and the larger of the two
constexpr int kc_group_bytes(int R) { return R * 16 + 32; }          // one k/4 group: R rows of 16 bytes + pad
constexpr int mn_row_words(int R) { return R + 8; }                   // one k row: R words + pad
constexpr int tile_bytes(int R) { return 32 * mn_row_words(R) * 4 > 8 * kc_group_bytes(R) ? 32 * mn_row_words(R) * 4 : 8 * kc_group_bytes(R); }

__device__ __forceinline__ float gelu_exact(float x) { // zyx/src/tensor/elementwise.rs:168-170, saturating tanh
    float inner = (x + ((x * x) * x) * 0.044715f) * 0.79788456080286535588f;
    float e = expf(inner + inner);
    float t = (inner + inner) > 88.0f ? 1.0f : (e - 1.0f) / (e + 1.0f);
    return (x * 0.5f) * (t + 1.0f);
}

// One operand: R rows of the workgroup tile, KC = its k index runs along memory.
template <int R, bool KC> struct Operand {
    static constexpr int CHUNKS = R * FK / 4 / 256; // 16-byte chunks per thread and K tile
    // global address of chunk e of this thread in K tile kt; ld = elements between consecutive rows (KC) or k (MN)
    static __device__ __forceinline__ const f32x4 *src(const float *g, int64_t ld, int64_t row0, int kt, int e, int t) {
        const int idx = e * 256 + t;
        if (KC) return (const f32x4 *)(g + (row0 + (idx >> 3)) * ld + kt * FK + (idx & 7) * 4);
        return (const f32x4 *)(g + (int64_t)(kt * FK + idx / (R / 4)) * ld + row0 + (idx % (R / 4)) * 4);
    }
    static __device__ __forceinline__ int dst(int e, int t) { // byte offset inside the operand's LDS tile
        const int idx = e * 256 + t;
        if (KC) return (idx & 7) * kc_group_bytes(R) + (idx >> 3) * 16;
        return ((idx / (R / 4)) * mn_row_words(R) + (idx % (R / 4)) * 4) * 4;
    }
    // the four values lane (row = lane % 32, h = lane / 32) feeds to the four instructions of 8-wide k step s for the
    // 32-row block starting at r0: k = 8s + j + 4h, j = 0..3
    static __device__ __forceinline__ f32x4 frag(const uint8_t *lds, int r0, int s, int lane) {
        const int row = r0 + (lane & 31), h = lane >> 5;
        if (KC) return *(const f32x4 *)(lds + (2 * s + h) * kc_group_bytes(R) + row * 16);
        const float *p = (const float *)lds + (8 * s + 4 * h) * mn_row_words(R) + row;
        return f32x4{p[0], p[mn_row_words(R)], p[2 * mn_row_words(R)], p[3 * mn_row_words(R)]};
    }
};

template <int TM, int TN, bool AT, bool BT>
__global__ __launch_bounds__(256) void gemm_f32_tiled_k(const GemmGeneric p) {
    typedef Operand<TM, !AT> OA; // A[M,K] has k contiguous; stored [K,M] it has not
    typedef Operand<TN, BT> OB;  // B[K,N] has n contiguous; stored [N,K] it has k contiguous
    constexpr int MI = TM / 64, NJ = TN / 64;
    __shared__ __attribute__((aligned(16))) uint8_t lds_a[tile_bytes(TM)];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[tile_bytes(TN)];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, wm = wave >> 1, wn = wave & 1;
    const int64_t m0 = (int64_t)blockIdx.y * TM, n0 = (int64_t)blockIdx.x * TN;
    const float *A = (const float *)p.A + (int64_t)blockIdx.z * p.batch_a, *B = (const float *)p.B + (int64_t)blockIdx.z * p.batch_b;
    const int64_t lda = AT ? p.M : p.K, ldb = BT ? p.K : p.N;
    const int KT = (int)(p.K / FK);

    f32x16 acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    f32x4 ra[OA::CHUNKS], rb[OB::CHUNKS];
    auto gload = [&](int kt) {
#pragma unroll
        for (int e = 0; e < OA::CHUNKS; e++) ra[e] = *OA::src(A, lda, m0, kt, e, t);
#pragma unroll
        for (int e = 0; e < OB::CHUNKS; e++) rb[e] = *OB::src(B, ldb, n0, kt, e, t);
    };
    auto lwrite = [&] {
#pragma unroll
        for (int e = 0; e < OA::CHUNKS; e++) *(f32x4 *)(lds_a + OA::dst(e, t)) = ra[e];
#pragma unroll
        for (int e = 0; e < OB::CHUNKS; e++) *(f32x4 *)(lds_b + OB::dst(e, t)) = rb[e];
    };
    gload(0);
    lwrite();
    __syncthreads();
    for (int kt = 0; kt < KT; kt++) {
        if (kt + 1 < KT) gload(kt + 1); // in flight during the multiply
#pragma unroll
        for (int s = 0; s < FK / 8; s++) {
            f32x4 fa[MI], fb[NJ];
#pragma unroll
            for (int i = 0; i < MI; i++) fa[i] = OA::frag(lds_a, wm * (TM / 2) + i * 32, s, lane);
#pragma unroll
            for (int j = 0; j < NJ; j++) fb[j] = OB::frag(lds_b, wn * (TN / 2) + j * 32, s, lane);
#pragma unroll
            for (int q = 0; q < 4; q++) // q outermost: consecutive instructions work on different accumulators
#pragma unroll
                for (int i = 0; i < MI; i++)
#pragma unroll
                    for (int j = 0; j < NJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q], acc[i][j], 0, 0, 0);
        }
        __syncthreads(); // everybody has read this tile
        if (kt + 1 < KT) lwrite();
        __syncthreads();
    }

    // register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32 of a 32 x 32 tile
    float *C = (float *)p.C + (int64_t)blockIdx.z * p.batch_c;
    const float *Rz = p.residual ? (const float *)p.residual + (int64_t)blockIdx.z * p.batch_c : nullptr;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int64_t col = n0 + wn * (TN / 2) + j * 32 + (lane & 31);
        float bv = 0.0f;
        if (p.epilogue >= 1) {
            if (p.bias_dtype == DT_BF16) bv = bf16_to_f32(((const uint16_t *)p.bias)[col]);
            else if (p.bias_dtype == DT_F16) bv = f16_to_f32(((const uint16_t *)p.bias)[col]);
            else bv = ((const float *)p.bias)[col];
        }
#pragma unroll
        for (int i = 0; i < MI; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
#pragma clang fp contract(off)
                const int64_t row = m0 + wm * (TM / 2) + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                float v = acc[i][j][r] * p.alpha;
                if (p.epilogue >= 1) v += bv;
                if (p.epilogue == 2) v = (v > 0.0f ? 1.0f : 0.0f) * v;
                if (p.epilogue == 3) v = gelu_exact(v);
                const int64_t o = row * p.N + col;
                if (Rz) v = p.residual_is_mask ? (Rz[o] > 0.0f ? 1.0f : 0.0f) * v : v + Rz[o];
                C[o] = v;
            }
    }
}

template <int TM, int TN> hipError_t launch_tiled(const GemmGeneric &p, hipStream_t st) {
    dim3 grid((unsigned)(p.N / TN), (unsigned)(p.M / TM), (unsigned)p.batch), block(256);
    if (p.trans_a) {
        if (p.trans_b) hipLaunchKernelGGL((gemm_f32_tiled_k<TM, TN, true, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_f32_tiled_k<TM, TN, true, false>), grid, block, 0, st, p);
    } else {
        if (p.trans_b) hipLaunchKernelGGL((gemm_f32_tiled_k<TM, TN, false, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((gemm_f32_tiled_k<TM, TN, false, false>), grid, block, 0, st, p);
    }
    return hipGetLastError();
}

} // namespace

// f32 products this file takes: whole 64 x 64 tiles, whole K tiles, 16-byte aligned operands and batch strides, and
// enough tiles that splitting K would not pay (fewer: gemm_generic's split-K path).
bool gemm_f32_tiled_ok(const GemmGeneric &p) {
    if (p.dtype != DT_F32 || p.out_dtype != DT_F32 || p.M % 64 || p.N % 64 || p.K % FK || p.K < FK) return false;
    if ((uintptr_t)p.A % 16 || (uintptr_t)p.B % 16 || p.batch_a % 4 || p.batch_b % 4) return false;
    if (p.M / 64 > 65535 || p.N / 64 >= (1ll << 31) || p.batch > 65535) return false;
    return (p.M / 64) * (p.N / 64) * p.batch >= 128;
}

hipError_t gemm_f32_tiled(const GemmGeneric &p, hipStream_t st) {
    if (!gemm_f32_tiled_ok(p)) return hipErrorInvalidValue;
    // 128 x 128 tiles when they still give every CU a few workgroups; else 64 x 64
    if (p.M % 128 == 0 && p.N % 128 == 0 && (p.M / 128) * (p.N / 128) * p.batch >= 512) return launch_tiled<128, 128>(p, st);
    return launch_tiled<64, 64>(p, st);
}

} // namespace zk
