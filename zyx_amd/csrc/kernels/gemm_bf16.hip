// bf16 x bf16 -> f32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16).
//
// Replaces what zyx lowers `Tensor::dot` to (broadcast multiply + serial k reduce,
// zyx/src/tensor/mod.rs:1469-1518) and the WMMA auto-tensorisation path
// (zyx/src/kernel/mma.rs). Operand rounding follows the C backend: bf16 widens
// exactly, products and sums are f32 (zyx/src/codegen/c.rs:491-496, 615-629).
//
// Shape of the kernel
//   * workgroup tile 256 x 256, K step 64, 4 waves in a 2 x 2 grid, each wave owns a
//     128 x 128 block of C = 4 x 4 MFMA tiles of 32 x 32 = 256 accumulator registers;
//   * operands go HBM/L2 -> LDS with 16-byte direct-to-LDS loads (no VGPR staging),
//     two LDS stages of 64 KiB, the loads of K step t+1 are in flight while step t is
//     multiplied;
//   * LDS rows are XOR-swizzled at 16-byte granularity. Direct-to-LDS writes lane l of
//     a wave at base + 16*l, so the swizzle is applied on the global side: each lane
//     fetches the chunk that belongs in its LDS slot;
//   * K-contiguous operands (A[M,K], B stored [N,K]) are read back with ds_read_b128;
//     an operand stored with its M/N index contiguous (B[K,N]) is read with the
//     transposing ds_read_b64_tr_b16, which hands each lane four consecutive k of one
//     column;
//   * workgroups are numbered so that the 32 that share an XCD (ids congruent mod 8)
//     cover a compact 4 x 8 patch of tiles and re-use each other's panels in that
//     XCD's L2.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define ZK_LDS __attribute__((address_space(3)))
#define ZK_GLOBAL __attribute__((address_space(1)))

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int A_STAGE = BM * BK * 2;           // 32 KiB
constexpr int B_STAGE = BN * BK * 2;           // 32 KiB
constexpr int STAGE = A_STAGE + B_STAGE;       // 64 KiB
constexpr int GEMM_LDS = 2 * STAGE;            // 128 KiB

__device__ __forceinline__ void g2lds16(const void *g, ZK_LDS void *l) {
    __builtin_amdgcn_global_load_lds((const ZK_GLOBAL void *)g, l, 16, 0, 0);
}

// K-contiguous operand tile: R = 256 rows x 64 k, LDS layout [row][chunk ^ (row & 7)],
// 128-byte rows. One wave-load fills 8 rows; 8 loads per thread.
__device__ __forceinline__ void load_tile_kc(const uint16_t *__restrict__ g, int64_t ld, int row0, int k0,
                                             ZK_LDS uint8_t *lds, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int rbase = i * 32 + wave * 8;
        const int row = rbase + (lane >> 3);
        const int c = (lane & 7) ^ (row & 7);
        g2lds16(g + (int64_t)(row0 + row) * ld + k0 + c * 8, lds + rbase * 128);
    }
}
// MN-contiguous operand tile: 64 k rows x 256 columns, LDS layout [k][chunk ^ swz(k)],
// 512-byte rows, swz(k) = (k & 3) << 1. One wave-load fills 2 k rows.
__device__ __forceinline__ int swz_mn(int k) { return (k & 3) << 1; }
__device__ __forceinline__ void load_tile_mn(const uint16_t *__restrict__ g, int64_t ld, int col0, int k0,
                                             ZK_LDS uint8_t *lds, int wave, int lane) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int kbase = i * 8 + wave * 2;
        const int k = kbase + (lane >> 5);
        const int c = (lane & 31) ^ swz_mn(k);
        g2lds16(g + (int64_t)(k0 + k) * ld + col0 + c * 8, lds + kbase * 512);
    }
}

// Fragment of a K-contiguous tile for MFMA 32x32x16: lane -> row (lane & 31),
// k = ks*16 + (lane >> 5)*8 .. +7.
__device__ __forceinline__ bf16x8 frag_kc(const ZK_LDS uint8_t *lds, int row, int ks, int lane) {
    const int c = (ks * 2 + (lane >> 5)) ^ (row & 7);
    return *(const ZK_LDS bf16x8 *)(lds + row * 128 + c * 16);
}
// Same fragment out of an MN-contiguous tile through two transposing reads. In every
// group of 16 lanes, lane r points at 4 consecutive columns of k row (r >> 2); the
// hardware returns to lane i the column i of those 4 k rows.
__device__ __forceinline__ bf16x8 frag_mn(const ZK_LDS uint8_t *lds, int col_base, int ks, int lane) {
    const int g16 = lane >> 4, r = lane & 15;
    const int col = col_base + (g16 & 1) * 16 + (r & 3) * 4;
    const int kk = ks * 16 + (g16 >> 1) * 8 + (r >> 2);
    const int k0 = kk, k1 = kk + 4;
    const ZK_LDS uint8_t *p0 = lds + k0 * 512 + (((col >> 3) ^ swz_mn(k0)) << 4) + (col & 4) * 2;
    const ZK_LDS uint8_t *p1 = lds + k1 * 512 + (((col >> 3) ^ swz_mn(k1)) << 4) + (col & 4) * 2;
    bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)p0);
    bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)p1);
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ float gelu_fast(float x) {
    // 0.5x(1+tanh(z)) == x * sigmoid(2z); one exp2 and one reciprocal. Used for bf16
    // GEMM epilogues whose parity bar is 1e-3.
    const float z2 = 2.0f * 0.79788456080286535588f * (x + 0.044715f * x * x * x);
    const float e = __builtin_amdgcn_exp2f(-z2 * 1.44269504088896340736f);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// AT: A stored [K, M] (M contiguous) instead of [M, K]; BT: B stored [N, K] (K contiguous)
// instead of [K, N]. EPI: 0 none, 1 + bias, 2 + bias then ReLU, 3 + bias then GELU.
template <bool AT, bool BT, int EPI>
__global__ __launch_bounds__(256, 1) void gemm_bf16_k(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                                                      float *__restrict__ C, const void *__restrict__ bias,
                                                      int bias_dtype, int M, int N, int K) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // XCD-aware tile order: ids congruent mod 8 land on one XCD; give each XCD a patch
    // of 4 x 8 tiles (or the whole grid when it is smaller).
    const int tiles_m = M / BM, tiles_n = N / BN;
    int tm, tn;
    {
        const int b = blockIdx.x, nb = tiles_m * tiles_n;
        if (nb % 8 == 0 && tiles_m % 4 == 0 && tiles_n % 8 == 0 && (tiles_m / 4) * (tiles_n / 8) % 8 == 0) {
            const int xcd = b & 7, local = b >> 3;            // local: index among this XCD's tiles
            const int patches_n = tiles_n / 8;
            const int per_patch = 32;
            const int patch = (local / per_patch) * 8 + xcd;   // patches are dealt round-robin to XCDs
            const int in_patch = local % per_patch;
            tm = (patch / patches_n) * 4 + in_patch / 8;
            tn = (patch % patches_n) * 8 + in_patch % 8;
        } else {
            tm = b / tiles_n;
            tn = b % tiles_n;
        }
    }
    const int m0 = tm * BM, n0 = tn * BN;

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    auto issue_loads = [&](int kt, int stage) {
        ZK_LDS uint8_t *sa = smem + stage * STAGE, *sb = sa + A_STAGE;
        if (AT) load_tile_mn(A, M, m0, kt * BK, sa, wave, lane);
        else load_tile_kc(A, K, m0, kt * BK, sa, wave, lane);
        if (BT) load_tile_kc(B, K, n0, kt * BK, sb, wave, lane);
        else load_tile_mn(B, N, n0, kt * BK, sb, wave, lane);
    };

    const int KT = K / BK;
    issue_loads(0, 0);
    __builtin_amdgcn_s_waitcnt(0x0070); // vmcnt(0): the direct-to-LDS loads have landed
    __syncthreads();

    for (int kt = 0; kt < KT; kt++) {
        const int stage = kt & 1;
        if (kt + 1 < KT) issue_loads(kt + 1, stage ^ 1);
        const ZK_LDS uint8_t *sa = smem + stage * STAGE, *sb = sa + A_STAGE;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            bf16x8 af[4], bfr[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (AT) af[i] = frag_mn(sa, wm * 128 + i * 32, ks, lane);
                else af[i] = frag_kc(sa, wm * 128 + i * 32 + (lane & 31), ks, lane);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (BT) bfr[j] = frag_kc(sb, wn * 128 + j * 32 + (lane & 31), ks, lane);
                else bfr[j] = frag_mn(sb, wn * 128 + j * 32, ks, lane);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads(); // next stage is complete and everyone is done reading this one
    }

    // C tile of a 32x32 MFMA: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32.
    const int col_in = lane & 31, row_in = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int col = n0 + wn * 128 + j * 32 + col_in;
        float bv = 0.0f;
        if (EPI >= 1) {
            if (bias_dtype == DT_BF16) bv = bf16_to_f32(((const uint16_t *)bias)[col]);
            else bv = ((const float *)bias)[col];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int rbase = m0 + wm * 128 + i * 32 + row_in;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = rbase + (r >> 2) * 8 + (r & 3);
                float v = acc[i][j][r];
                if (EPI >= 1) v += bv;
                if (EPI == 2) v = (v > 0.0f ? 1.0f : 0.0f) * v;
                if (EPI == 3) v = gelu_fast(v);
                C[(int64_t)row * N + col] = v;
            }
        }
    }
}

template <bool AT, bool BT> hipError_t launch_epi(const GemmBf16 &p, hipStream_t st) {
    dim3 grid((unsigned)((p.M / BM) * (p.N / BN))), block(256);
#define ZK_GEMM(E)                                                                                                    \
    {                                                                                                                 \
        auto k = gemm_bf16_k<AT, BT, E>;                                                                              \
        static bool attr_set = false;                                                                                 \
        if (!attr_set) {                                                                                              \
            hipError_t e = hipFuncSetAttribute((const void *)k, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS); \
            if (e != hipSuccess) return e;                                                                            \
            attr_set = true;                                                                                          \
        }                                                                                                             \
        hipLaunchKernelGGL(k, grid, block, GEMM_LDS, st, (const uint16_t *)p.A, (const uint16_t *)p.B, (float *)p.C,  \
                           p.bias, p.bias_dtype, (int)p.M, (int)p.N, (int)p.K);                                       \
    }
    switch (p.epilogue) {
    case 0: ZK_GEMM(0) break;
    case 1: ZK_GEMM(1) break;
    case 2: ZK_GEMM(2) break;
    case 3: ZK_GEMM(3) break;
    default: return hipErrorInvalidValue;
    }
#undef ZK_GEMM
    return hipGetLastError();
}

} // namespace

bool gemm_bf16_supported(int64_t M, int64_t N, int64_t K) {
    return M > 0 && N > 0 && K > 0 && M % BM == 0 && N % BN == 0 && K % BK == 0 && M < (1 << 30) && N < (1 << 30) &&
           K < (1 << 30) && (M / BM) * (N / BN) < (1ll << 31);
}

hipError_t gemm_bf16(const GemmBf16 &p, hipStream_t st) {
    if (!gemm_bf16_supported(p.M, p.N, p.K)) return hipErrorInvalidValue;
    if (p.trans_a) return p.trans_b ? launch_epi<true, true>(p, st) : launch_epi<true, false>(p, st);
    return p.trans_b ? launch_epi<false, true>(p, st) : launch_epi<false, false>(p, st);
}

} // namespace zk
