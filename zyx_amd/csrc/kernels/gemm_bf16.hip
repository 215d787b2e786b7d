// bf16 x bf16 -> f32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16).
//
// Replaces what zyx lowers `Tensor::dot` to (broadcast multiply + serial k reduce,
// zyx/src/tensor/mod.rs:1469-1518) and the WMMA auto-tensorisation path
// (zyx/src/kernel/mma.rs). Operand rounding follows the C backend: bf16 widens
// exactly, products and sums are f32 (zyx/src/codegen/c.rs:491-496, 615-629).
//
// Shape of the kernel
//   * workgroup tile 256 x 256, K step 64, 4 waves in a 2 x 2 grid (one per SIMD), each
//     wave owns a 128 x 128 block of C = 4 x 4 MFMA tiles of 32 x 32 = 256 accumulator
//     registers (the AGPR half of the register file);
//   * operands go L2 -> VGPR -> LDS: every thread keeps one K tile (16 x 16 bytes) in
//     flight in registers; a chunk is written to LDS one tile time after its load was
//     issued and its registers are immediately reused for the load of the tile after.
//     Measured beside an MFMA stream on this part, a 1 KiB direct-to-LDS load costs the
//     matrix pipe ~42 cycles, a register-staged load + ds_write_b128 pair ~16;
//   * two LDS stages of 64 KiB; rows are XOR-swizzled at 16-byte granularity so that both
//     the ds_write_b128 of the staging path and the fragment reads are conflict-free;
//   * K-contiguous operands (A[M,K], B stored [N,K]) are read back with ds_read_b128; an
//     operand stored with its M/N index contiguous (B[K,N]) is read with the transposing
//     ds_read_b64_tr_b16, which hands each lane four consecutive k of one column;
//   * per k step (16 MFMAs) a wave issues 8 fragment reads for the next step, 4 LDS
//     writes and 4 global loads, slotted between the MFMAs;
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

// Workgroup tile BM x BNV x BK with BNV = 256 (4 waves of 128 x 128) or 128 (4 waves of 128 x 64, for outputs
// whose N is only a multiple of 128 or that have too few 256 x 256 tiles to occupy the chip).
constexpr int BM = 256, BK = 64;
constexpr int A_STAGE = BM * BK * 2;           // 32 KiB
constexpr int stage_bytes(int bnv) { return A_STAGE + bnv * BK * 2; }   // 64 KiB / 48 KiB
constexpr int lds_bytes(int bnv) { return 2 * stage_bytes(bnv); }       // 128 KiB / 96 KiB

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// K-contiguous operand tile: 256 rows x 64 k, LDS layout [row][chunk ^ key(row)], 128-byte
// rows, key(row) = (row >> 1) & 7: a 128-bit LDS access is served 16 lanes at a time over
// 64 banks (256 bytes), and 16 consecutive rows at one logical chunk occupy 16 different
// 16-byte slots modulo 256 bytes. Thread (wave w, lane l) moves, for i = 0..7, the chunk
// that belongs at row i*32 + w*8 + l/8, physical slot l%8.
__device__ __forceinline__ int swz_kc(int row) { return (row >> 1) & 7; }
struct TileKC { // NCHUNK chunks per thread = rows / 32
    static __device__ __forceinline__ const uint16_t *src(const uint16_t *g, int64_t ld, int row0, int k0, int i, int wave,
                                                         int lane, int limit) {
        const int row = i * 32 + wave * 8 + (lane >> 3);
        const int c = (lane & 7) ^ swz_kc(row);
        // rows past the operand's end (edge tiles) re-read its last row: in bounds, and never stored
        return g + (int64_t)min(row0 + row, limit - 1) * ld + k0 + c * 8;
    }
    static constexpr __host__ __device__ __forceinline__ int dst(int i, int wave, int lane) { return (i * 32 + wave * 8) * 128 + lane * 16; }
    static __device__ __forceinline__ int64_t k_advance(int64_t) { return BK; }
};
// MN-contiguous operand tile: 64 k rows x 256 columns, LDS layout [k][chunk ^ swz(k)],
// 512-byte rows, swz(k) = (k & 3) << 1. Thread (w, l) moves, for i = 0..7, the chunk at
// k row i*8 + w*2 + l/32, physical slot l%32.
// COLS = 128: 256-byte rows, swz(k) = (k & 3) << 2 (the four k rows of a transposing read then fall into four
// different 64-byte bank windows); thread (w, l) moves, for i = 0..3, the chunk at k row i*16 + w*4 + l/16.
template <int COLS> __device__ __forceinline__ int swz_mn(int k) { return COLS == 256 ? (k & 3) << 1 : (k & 3) << 2; }
template <int COLS> struct TileMN {
    static constexpr int CH = COLS / 8;          // 16-byte chunks per k row
    static constexpr int KPW = 64 / CH;          // k rows one wave covers per pass
    static constexpr int NCHUNK = COLS / 32;     // passes (chunks per thread)
    static __device__ __forceinline__ const uint16_t *src(const uint16_t *g, int64_t ld, int col0, int k0, int i, int wave,
                                                         int lane, int limit) {
        const int k = i * 4 * KPW + wave * KPW + lane / CH;
        const int c = (lane % CH) ^ swz_mn<COLS>(k);
        // chunks past the operand's end (edge tiles; the extent is a multiple of 8) re-read its last chunk
        return g + (int64_t)(k0 + k) * ld + min(col0 + c * 8, limit - 8);
    }
    static constexpr __host__ __device__ __forceinline__ int dst(int i, int wave, int lane) { return (i * 4 * KPW + wave * KPW) * COLS * 2 + lane * 16; }
    static __device__ __forceinline__ int64_t k_advance(int64_t ld) { return BK * ld; }
};

// Fragment addressing. Everything that depends on the lane is folded into a few byte
// offsets computed once before the K loop; stage, 32-row block and k step then only add
// compile-time constants, which the LDS instructions take as immediate offsets.
//
// K-contiguous tile, MFMA 32x32x16 operand: lane -> row (lane & 31), k = ks*16 +
// (lane >> 5)*8 .. +7, i.e. logical chunk ks*2 + (lane >> 5) at physical slot chunk ^ key.
// key(row) is unchanged by adding multiples of 16 rows, so one offset per k step serves
// every 32-row block: kc_off[ks] + block * 32 * 128.
__device__ __forceinline__ int frag_kc_off(int row, int ks, int lane) {
    return row * 128 + (((ks * 2 + (lane >> 5)) ^ swz_kc(row)) << 4);
}
__device__ __forceinline__ bf16x8 frag_kc(const ZK_LDS uint8_t *lds, int off) {
    return *(const ZK_LDS bf16x8 *)(lds + off);
}
// MN-contiguous tile through two transposing reads. In every group of 16 lanes, lane r
// points at 4 consecutive columns of k row (r >> 2); the hardware returns to lane i the
// column i of those 4 k rows. swz(k) only depends on k & 3 = (lane & 15) >> 2, so one
// offset per 32-column block serves all k steps and both halves: mn_off[block] +
// ks*16*512 (+ 4*512).
template <int COLS> __device__ __forceinline__ int frag_mn_off(int col_base, int lane) {
    const int g16 = lane >> 4, r = lane & 15;
    const int col = col_base + (g16 & 1) * 16 + (r & 3) * 4;
    const int k = (g16 >> 1) * 8 + (r >> 2);
    return k * COLS * 2 + (((col >> 3) ^ swz_mn<COLS>(k)) << 4) + (col & 4) * 2;
}
template <int COLS> __device__ __forceinline__ bf16x8 frag_mn(const ZK_LDS uint8_t *lds, int off) {
    bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)(lds + off));
    bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)(lds + off + 4 * COLS * 2));
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
// PLANE: 0 plain row-major C; 1 C stored [M / plane, N, plane] (NCHW result of a convolution whose patch matrix is
// operand A); 2 the same store, and operand A is not a matrix in memory at all: its [K, M] tile rows are gathered
// from a zero-padded NCHW input (`A` points at it, `g` describes it), 8 consecutive pixels per 128-bit load.
// TAIL: M and / or N are not multiples of the tile; edge tiles clamp their loads and mask their stores.
template <bool AT, bool BT, int EPI, int BNV, int PLANE, bool TAIL>
__global__ __launch_bounds__(256, 1) void gemm_bf16_k(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B,
                                                      void *__restrict__ Cv, const void *__restrict__ bias,
                                                      const void *__restrict__ residual, int bias_dtype, int out_bf16,
                                                      int M, int N, int K, int ldn, int splits, int plane, const ConvGather g) {
    // ldn: elements between rows of C, of the residual and of a [K, N] operand B: N, or the full width when this
    // launch computes a block of columns of a wider product
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    constexpr int NJ = BNV / 64;                 // 32-column MFMA blocks per wave
    constexpr int NB = BNV / 32;                 // B staging chunks per thread
    constexpr int NU = 8 + NB;                   // staging units per K tile
    constexpr int WN = BNV / 2;                  // columns per wave
    constexpr int STAGE = stage_bytes(BNV);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // XCD-aware tile order: ids congruent mod 8 land on one XCD; give each XCD a patch
    // of 4 x 8 tiles (or the whole grid when it is smaller).
    const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BNV - 1) / BNV;
    // split-K: workgroup z of a tile multiplies K range [z, z+1) * K/splits and stores its raw f32 partial
    // tile into slice z of Cv (a [splits, M, N] workspace that a second kernel folds)
    const int split = blockIdx.x / (tiles_m * tiles_n);
    const int k_len = K / splits;
    A += (int64_t)split * k_len * (AT ? M : 1);
    B += (int64_t)split * k_len * (BT ? 1 : ldn);
    if (splits > 1) Cv = (float *)Cv + (int64_t)split * M * N;
    int tm, tn;
    {
        const int b = blockIdx.x % (tiles_m * tiles_n), nb = tiles_m * tiles_n;
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
    const int m0 = tm * BM, n0 = tn * BNV;

    f32x16 acc[4][NJ];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < NJ; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    // Staging registers: ra[i] / rb[i] hold chunk i of the tile that is written to LDS
    // during the current K tile and re-loaded (two tiles ahead) right after the write.
    // Global addresses are a wave-uniform byte pointer that advances with the K tile plus a
    // per-thread 32-bit offset fixed for the whole kernel; LDS addresses are one per-thread
    // offset plus constants.
    typedef typename std::conditional<AT, TileMN<256>, TileKC>::type TA;
    typedef typename std::conditional<BT, TileKC, TileMN<BNV>>::type TB;
    const int64_t lda = AT ? M : K, ldb = BT ? K : ldn;
    uint32_t oa[8], ob[NB];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if (PLANE == 2) {
            // chunk i of this thread: k row i*8 + wave*2 + lane/32 of a K tile, pixels m0 + c*8 .. +7 (one output row)
            const int kr = i * 8 + wave * 2 + (lane >> 5);
            const int pix = m0 + (((lane & 31) ^ swz_mn<256>(kr)) << 3);
            const int img = pix / g.ohw, rem = pix - img * g.ohw, oy = rem / g.ow, ox = rem - oy * g.ow;
            oa[i] = (uint32_t)(img * g.img + oy * g.row + ox) * 2;
        } else oa[i] = (uint32_t)((TA::src(A, lda, m0, 0, i, wave, lane, M) - A) * 2);
    }
#pragma unroll
    for (int i = 0; i < NB; i++) ob[i] = (uint32_t)((TB::src(B, ldb, n0, 0, i, wave, lane, N) - B) * 2);
    const int da0 = TA::dst(0, wave, lane), db0 = A_STAGE + TB::dst(0, wave, lane);
    constexpr int da_step = TA::dst(1, 0, 0) - TA::dst(0, 0, 0), db_step = TB::dst(1, 0, 0) - TB::dst(0, 0, 0);
    const int64_t adv_a = TA::k_advance(lda) * 2, adv_b = TB::k_advance(ldb) * 2;
    u32x4 ra[8], rb[NB];
    // staging unit u = 0..NU-1. BNV = 256: operand A (u even) or B (u odd), chunk u >> 1. BNV = 128: every
    // third unit is a B chunk (u % 3 == 2 -> B chunk u / 3), the others A chunks 2*(u/3) + u%3.
    auto unit_is_b = [](int u) { return NJ == 4 ? (u & 1) != 0 : u % 3 == 2; };
    auto unit_chunk = [](int u) { return NJ == 4 ? u >> 1 : (u % 3 == 2 ? u / 3 : 2 * (u / 3) + u % 3); };
    auto gload = [&](int u, int kt) {
        const int i = unit_chunk(u);
        if (unit_is_b(u)) rb[i] = *(const u32x4 *)((const uint8_t *)B + kt * adv_b + ob[i]);
        else if (PLANE == 2) {
            // k = (c, ky, kx) of this chunk's row in K tile kt -> offset of that tap in the padded input
            const uint32_t k = (uint32_t)(kt * BK + i * 8 + wave * 2 + (lane >> 5));
            const uint32_t c = g.khw == 1 ? k : __umulhi(k, g.magic_khw), r = k - c * g.khw; // ceil(2^32 / 1) does not fit
            const uint32_t ky = g.kw == 1 ? r : __umulhi(r, g.magic_kw), kx = r - ky * g.kw;
            typedef uint32_t u32x4a2 __attribute__((ext_vector_type(4), aligned(2)));
            ra[i] = *(const u32x4a2 *)((const uint8_t *)A + oa[i] + (c * g.cs + ky * g.rs + kx * g.dx) * 2);
        } else ra[i] = *(const u32x4 *)((const uint8_t *)A + kt * adv_a + oa[i]);
    };
    auto lwrite = [&](int u, int da_base, int db_base) {
        const int i = unit_chunk(u);
        if (unit_is_b(u)) *(ZK_LDS u32x4 *)(smem + db_base + i * db_step) = rb[i];
        else *(ZK_LDS u32x4 *)(smem + da_base + i * da_step) = ra[i];
    };
    int fa_off[4], fb_off[4]; // per k step (K-contiguous) or per 32-wide block (MN-contiguous)
#pragma unroll
    for (int q = 0; q < 4; q++) {
        fa_off[q] = AT ? frag_mn_off<256>(wm * 128 + q * 32, lane) : frag_kc_off(wm * 128 + (lane & 31), q, lane);
        fb_off[q] = A_STAGE + (BT ? frag_kc_off(wn * WN + (lane & 31), q, lane) : frag_mn_off<BNV>(wn * WN + (q % NJ) * 32, lane));
    }

    const int KT = k_len / BK;
#pragma unroll
    for (int u = 0; u < NU; u++) gload(u, 0);
#pragma unroll
    for (int u = 0; u < NU; u++) {
        lwrite(u, da0, db0);
        gload(u, min(1, KT - 1));
    }
    __syncthreads();

    // Fragments are double-buffered in registers: while the 16 MFMAs of k step s run, the
    // 8 LDS reads of step s+1 are in flight. The step after the last one of a tile lives
    // in the other stage, so the hand-over barrier sits before the last step's MFMAs.
    bf16x8 af[2][4], bfr[2][NJ];
    // fragment r = 0..3: A block r; r = 4..3+NJ: B block r - 4. fa/fb are the four per-lane
    // offsets of each operand with the stage folded in.
    constexpr int NFRAG = 4 + NJ;
    auto load_frag = [&](const int (&fa)[4], const int (&fb)[4], int ks, int buf, int r) {
        if (r < 4) {
            if (AT) af[buf][r] = frag_mn<256>(smem, fa[r] + ks * 16 * 512);
            else af[buf][r] = frag_kc(smem, fa[ks] + r * 32 * 128);
        } else {
            const int j = r - 4;
            if (BT) bfr[buf][j] = frag_kc(smem, fb[ks] + j * 32 * 128);
            else bfr[buf][j] = frag_mn<BNV>(smem, fb[j] + ks * 16 * BNV * 2);
        }
    };
#pragma unroll
    for (int r = 0; r < NFRAG; r++) load_frag(fa_off, fb_off, 0, 0, r);

    // One K tile = 4 k steps of 16 MFMAs. During tile c (stage c & 1) each step writes two
    // staged chunk pairs of tile c+1 into the other stage and re-issues their loads for
    // tile c+2. The body is branch-free so that it stays one basic block (the compiler's
    // wait-count bookkeeping is exact only inside a block): tiles 0..KT-2 all hand over
    // (loads past the end re-fetch the final tile and are never written), the final tile
    // is peeled off below.
    // Address registers of the tile being multiplied (c*) and of the other stage (n*) are
    // formed once per tile: 18 adds, everything else in the loop is an immediate offset.
    int cfa[4], cfb[4], nfa[4], nfb[4], nda, ndb;
    auto set_stage = [&](int cur_off, int nxt_off) {
#pragma unroll
        for (int q = 0; q < 4; q++) {
            cfa[q] = fa_off[q] + cur_off;
            cfb[q] = fb_off[q] + cur_off;
            nfa[q] = fa_off[q] + nxt_off;
            nfb[q] = fb_off[q] + nxt_off;
        }
        nda = da0 + nxt_off;
        ndb = db0 + nxt_off;
    };
    // The instruction order of a k step is pinned by hand (a scheduling fence after every
    // MFMA and every group of memory operations). Measured on an MFMA stream, a
    // ds_write_b128 holds up the next MFMA of its SIMD for about the time its 1 KiB takes
    // to leave the register file; writing a staged chunk and immediately re-issuing the
    // load into its registers in one gap, and giving the neighbouring gaps one cheap
    // fragment read each, costs the least. Steps 0 and 1 move 6 staging units, step 2 the
    // last 4, step 3 only holds the hand-over barrier (after 4 MFMAs, so that the matrix
    // pipe has work queued while the waves meet) and the first reads of the next tile.
    auto k_step = [&](const int ks, int kt, const bool handover) {
        const int cur = ks & 1, nxt = cur ^ 1;
        const bool last = ks == BK / 16 - 1;
        constexpr int MF = 4 * NJ; // MFMAs per k step
        // BNV = 256: 6, 6, 4 staging units in steps 0..2 (after even MFMAs), one fragment read after every odd one.
        // BNV = 128: 4, 4, 4 units; 6 fragment reads over the 4 odd slots (2, 1, 2, 1).
        const int u0 = NJ == 4 ? ks * 6 : ks * 4, nu = NJ == 4 ? (ks < 2 ? 6 : (ks == 2 ? 4 : 0)) : (ks < 3 ? 4 : 0);
#pragma unroll
        for (int m = 0; m < MF; m++) {
            __builtin_amdgcn_sched_barrier(0);
            acc[m / NJ][m % NJ] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[cur][m / NJ], bfr[cur][m % NJ], acc[m / NJ][m % NJ], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (!last) {
                if ((m & 1) == 0 && handover && (m >> 1) < nu) {
                    lwrite(u0 + (m >> 1), nda, ndb);
                    gload(u0 + (m >> 1), min(kt + 2, KT - 1));
                }
                if (m & 1) {
                    if (NJ == 4) load_frag(cfa, cfb, ks + 1, nxt, m >> 1);
                    else {
                        const int s_ = m >> 1, r0 = s_ + (s_ + 1) / 2; // slots hold fragments {0,1}, {2}, {3,4}, {5}
                        load_frag(cfa, cfb, ks + 1, nxt, r0);
                        if ((s_ & 1) == 0) load_frag(cfa, cfb, ks + 1, nxt, r0 + 1);
                    }
                }
            } else if (handover) {
                constexpr int SYNC_AT = NJ == 4 ? 3 : 1;
                if (m == SYNC_AT) __syncthreads(); // tile kt+1 is complete in LDS; nobody reads this stage any more
                if (m >= SYNC_AT && m < SYNC_AT + NFRAG) load_frag(nfa, nfb, 0, nxt, m - SYNC_AT);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    int cur_off = 0;
    for (int kt = 0; kt < KT - 1; kt++) {
        set_stage(cur_off, cur_off ^ STAGE);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) k_step(ks, kt, true);
        cur_off ^= STAGE;
    }
    set_stage(cur_off, cur_off ^ STAGE);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) k_step(ks, KT - 1, false);
    __builtin_amdgcn_sched_barrier(0);

    // C tile of a 32x32 MFMA: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32.
    const int col_in = lane & 31, row_in = (lane >> 5) * 4;
    auto finish = [&](float v, float bv) {
        if (EPI >= 1) v += bv;
        if (EPI == 2) v = (v > 0.0f ? 1.0f : 0.0f) * v;
        if (EPI == 3) v = gelu_fast(v);
        return v;
    };
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        // the residual is added to the finished value as written, never fused into the activation's last multiply:
        // f32 and bf16 results of one product then differ by the store's truncation only, whatever the code shape
#pragma clang fp contract(off)
        const int col = n0 + wn * WN + j * 32 + col_in;
        float bv = 0.0f;
        if (EPI >= 1) {
            const int bc = TAIL ? min(col, N - 1) : col;
            if (bias_dtype == DT_BF16) bv = bf16_to_f32(((const uint16_t *)bias)[bc]);
            else bv = ((const float *)bias)[bc];
        }
        if (PLANE != 0) {
            // C is stored as [M / plane, N, plane] (the NCHW result of a convolution lowered to this product:
            // row = image * plane + pixel, column = channel). The four consecutive rows a lane holds per
            // register group are consecutive pixels of one image (plane % 4 == 0): one 16- or 8-byte store.
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int row = m0 + wm * 128 + i * 32 + row_in + g * 8;
                    const int img = row / plane, pix = row - img * plane;
                    const int64_t o = ((int64_t)img * N + col) * plane + pix;
                    float v[4];
#pragma unroll
                    for (int k = 0; k < 4; k++) v[k] = finish(acc[i][j][4 * g + k], bv);
                    if (out_bf16) *(uint2 *)((uint16_t *)Cv + o) = make_uint2((__float_as_uint(v[0]) >> 16) | (__float_as_uint(v[1]) & 0xffff0000u),
                                                                                (__float_as_uint(v[2]) >> 16) | (__float_as_uint(v[3]) & 0xffff0000u));
                    else *(f32x4 *)((float *)Cv + o) = f32x4{v[0], v[1], v[2], v[3]};
                }
        } else if (!out_bf16) {
            float *C = (float *)Cv;
            const float *R = (const float *)residual;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int rbase = m0 + wm * 128 + i * 32 + row_in;
                // 128-wide tiles: the residual values of the block are requested together, one memory latency per 16
                // loads (the 256-wide tile has no registers to spare for that: it would spill)
                float rv[BNV == 128 ? 16 : 1];
                if (BNV == 128 && R) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int row = rbase + (r >> 2) * 8 + (r & 3);
                        rv[BNV == 128 ? r : 0] = (TAIL && (row >= M || col >= N)) ? 0.0f : R[(int64_t)row * ldn + col];
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = rbase + (r >> 2) * 8 + (r & 3);
                    if (TAIL && (row >= M || col >= N)) continue;
                    const int64_t o = (int64_t)row * ldn + col;
                    float v = finish(acc[i][j][r], bv);
                    if (R) v += BNV == 128 ? rv[BNV == 128 ? r : 0] : R[o];
                    C[o] = v;
                }
            }
        } else {
            // bf16 result: neighbouring lanes trade one value of each register pair, so that the even lane
            // holds columns (c, c+1) of row r and the odd lane columns (c-1, c) of row r+1: 4-byte stores.
            uint16_t *C = (uint16_t *)Cv;
            const uint16_t *R = (const uint16_t *)residual;
            const int odd = lane & 1;
            // 128-wide tiles: the residual words of the whole column block are requested before the first is used,
            // one memory latency per 32 loads instead of one per load (the accumulators leave the compiler too few
            // registers to do this by itself; the 256-wide tile has none to spare at all and keeps load-then-use)
            constexpr bool BATCH = BNV == 128;
            uint32_t rr[BATCH ? 4 : 1][BATCH ? 8 : 1];
            if (BATCH && R) {
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int r = 0; r < 16; r += 2) {
                        const int row = m0 + wm * 128 + i * 32 + row_in + (r >> 2) * 8 + (r & 3) + odd;
                        rr[BATCH ? i : 0][BATCH ? r >> 1 : 0] =
                            (TAIL && (row >= M || col - odd + 1 >= N)) ? 0u : *(const uint32_t *)(R + (int64_t)row * ldn + (col - odd));
                    }
            }
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int rbase = m0 + wm * 128 + i * 32 + row_in;
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const float v0 = finish(acc[i][j][r], bv), v1 = finish(acc[i][j][r + 1], bv);
                    const float got = dpp_f32<kDppQuadXor1>(odd ? v0 : v1);
                    float lo = odd ? got : v0, hi = odd ? v1 : got;
                    if (TAIL && (rbase + (r >> 2) * 8 + (r & 3) + odd >= M || col - odd + 1 >= N)) continue; // N is even
                    const int64_t o = (int64_t)(rbase + (r >> 2) * 8 + (r & 3) + odd) * ldn + (col - odd);
                    if (R) {
                        const uint32_t w = BATCH ? rr[BATCH ? i : 0][BATCH ? r >> 1 : 0] : *(const uint32_t *)(R + o);
                        lo += __uint_as_float(w << 16);
                        hi += __uint_as_float(w & 0xffff0000u);
                    }
                    *(uint32_t *)(C + o) = (uint32_t)f32_to_bf16_trunc(lo) | ((uint32_t)f32_to_bf16_trunc(hi) << 16);
                }
            }
        }
    }
}

// Folds the [splits, M, N] f32 partials and applies the epilogue; one thread per 4 consecutive columns.
__global__ __launch_bounds__(256) void gemm_splitk_fold_k(const float *__restrict__ ws, void *__restrict__ Cv,
                                                          const void *__restrict__ bias, const void *__restrict__ residual,
                                                          int epi, int bias_dtype, int out_bf16, int64_t MN, int N, int splits) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= MN) return;
    f32x4 a = *(const f32x4 *)(ws + i);
    for (int z = 1; z < splits; z++) a += *(const f32x4 *)(ws + (int64_t)z * MN + i);
    const int col = (int)(i % N);
    float v[4] = {a[0], a[1], a[2], a[3]};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        if (epi >= 1) v[k] += bias_dtype == DT_BF16 ? bf16_to_f32(((const uint16_t *)bias)[col + k]) : ((const float *)bias)[col + k];
        if (epi == 2) v[k] = (v[k] > 0.0f ? 1.0f : 0.0f) * v[k];
        if (epi == 3) v[k] = gelu_fast(v[k]);
    }
    if (!out_bf16) {
        if (residual) {
            const f32x4 r = *(const f32x4 *)((const float *)residual + i);
#pragma unroll
            for (int k = 0; k < 4; k++) v[k] += r[k];
        }
        *(f32x4 *)((float *)Cv + i) = f32x4{v[0], v[1], v[2], v[3]};
    } else {
        if (residual) {
            const uint2 r = *(const uint2 *)((const uint16_t *)residual + i);
            v[0] += __uint_as_float(r.x << 16); v[1] += __uint_as_float(r.x & 0xffff0000u);
            v[2] += __uint_as_float(r.y << 16); v[3] += __uint_as_float(r.y & 0xffff0000u);
        }
        *(uint2 *)((uint16_t *)Cv + i) = make_uint2((__float_as_uint(v[0]) >> 16) | (__float_as_uint(v[1]) & 0xffff0000u),
                                                    (__float_as_uint(v[2]) >> 16) | (__float_as_uint(v[3]) & 0xffff0000u));
    }
}

template <bool AT, bool BT, int BNV, bool TAIL> hipError_t launch_epi(const GemmBf16 &p, hipStream_t st) {
    const int splits = p.ldn ? 1 : gemm_bf16_splits(p.M, p.N, p.K); // a column block of a wider product is never K-split
    if (p.plane && (TAIL || splits > 1 || p.residual || p.plane % 4 || p.M % p.plane)) return hipErrorInvalidValue;
    dim3 grid((unsigned)(((p.M + BM - 1) / BM) * ((p.N + BNV - 1) / BNV) * splits)), block(256);
    if (splits > 1) {
        if (!p.workspace) return hipErrorInvalidValue;
        hipLaunchKernelGGL((gemm_bf16_k<AT, BT, 0, BNV, 0, TAIL>), grid, block, lds_bytes(BNV), st, (const uint16_t *)p.A, (const uint16_t *)p.B,
                           p.workspace, nullptr, nullptr, 0, 0, (int)p.M, (int)p.N, (int)p.K, (int)p.N, splits, 0, ConvGather{});
        const int64_t MN = p.M * p.N;
        hipLaunchKernelGGL(gemm_splitk_fold_k, dim3((unsigned)((MN / 4 + 255) / 256)), block, 0, st, (const float *)p.workspace, p.C,
                           p.bias, p.residual, p.epilogue, p.bias_dtype, p.out_bf16, MN, (int)p.N, splits);
        return hipGetLastError();
    }
    if (p.plane) {
        // only the product a convolution lowers to stores this way: A^T . B^T, epilogues none / bias / bias + ReLU
        if (!(AT && BT) || p.epilogue > 2) return hipErrorInvalidValue;
#define ZK_GEMM_PL(E, G)                                                                                              \
    hipLaunchKernelGGL((gemm_bf16_k<true, true, E, BNV, G, false>), grid, block, lds_bytes(BNV), st, (const uint16_t *)p.A, \
                       (const uint16_t *)p.B, p.C, p.bias, p.residual, p.bias_dtype, p.out_bf16, (int)p.M, (int)p.N, (int)p.K, (int)p.N, 1, p.plane, p.gather);
        if (p.gather.khw) {
            switch (p.epilogue) {
            case 0: ZK_GEMM_PL(0, 2) break;
            case 1: ZK_GEMM_PL(1, 2) break;
            default: ZK_GEMM_PL(2, 2) break;
            }
        } else {
            switch (p.epilogue) {
            case 0: ZK_GEMM_PL(0, 1) break;
            case 1: ZK_GEMM_PL(1, 1) break;
            default: ZK_GEMM_PL(2, 1) break;
            }
        }
#undef ZK_GEMM_PL
        return hipGetLastError();
    }
#define ZK_GEMM(E)                                                                                                    \
    hipLaunchKernelGGL((gemm_bf16_k<AT, BT, E, BNV, 0, TAIL>), grid, block, lds_bytes(BNV), st, (const uint16_t *)p.A, \
                       (const uint16_t *)p.B, p.C, p.bias, p.residual, p.bias_dtype, p.out_bf16, (int)p.M, (int)p.N, (int)p.K, (int)(p.ldn ? p.ldn : p.N), 1, 0, ConvGather{});
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
template <bool AT, bool BT> hipError_t launch_width(const GemmBf16 &p, hipStream_t st) {
    const int bn = gemm_bf16_tile_n(p.M, p.N);
    const bool tail = p.M % BM != 0 || p.N % bn != 0;
    if (bn == 128) return tail ? launch_epi<AT, BT, 128, true>(p, st) : launch_epi<AT, BT, 128, false>(p, st);
    return tail ? launch_epi<AT, BT, 256, true>(p, st) : launch_epi<AT, BT, 256, false>(p, st);
}

template <bool AT, bool BT, int E, int BNV> hipError_t allow_lds() {
    hipError_t e;
    if (AT && BT && E <= 2) {
        e = hipFuncSetAttribute((const void *)gemm_bf16_k<true, true, (E <= 2 ? E : 0), BNV, 1, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes(BNV));
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute((const void *)gemm_bf16_k<true, true, (E <= 2 ? E : 0), BNV, 2, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes(BNV));
        if (e != hipSuccess) return e;
    }
    e = hipFuncSetAttribute((const void *)gemm_bf16_k<AT, BT, E, BNV, 0, true>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes(BNV));
    if (e != hipSuccess) return e;
    return hipFuncSetAttribute((const void *)gemm_bf16_k<AT, BT, E, BNV, 0, false>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes(BNV));
}
template <bool AT, bool BT> hipError_t allow_lds_epi() {
    hipError_t e;
    if ((e = allow_lds<AT, BT, 0, 256>()) != hipSuccess) return e;
    if ((e = allow_lds<AT, BT, 1, 256>()) != hipSuccess) return e;
    if ((e = allow_lds<AT, BT, 2, 256>()) != hipSuccess) return e;
    if ((e = allow_lds<AT, BT, 3, 256>()) != hipSuccess) return e;
    if ((e = allow_lds<AT, BT, 0, 128>()) != hipSuccess) return e;
    if ((e = allow_lds<AT, BT, 1, 128>()) != hipSuccess) return e;
    if ((e = allow_lds<AT, BT, 2, 128>()) != hipSuccess) return e;
    return allow_lds<AT, BT, 3, 128>();
}

} // namespace

// The kernels use 128 KiB of dynamic LDS, above the default per-workgroup limit: raise it
// once per device (the attribute lives with the device's copy of the code object).
hipError_t gemm_bf16_init() {
    hipError_t e;
    if ((e = allow_lds_epi<false, false>()) != hipSuccess) return e;
    if ((e = allow_lds_epi<false, true>()) != hipSuccess) return e;
    if ((e = allow_lds_epi<true, false>()) != hipSuccess) return e;
    return allow_lds_epi<true, true>();
}

// Shapes whose every tile is whole (what the plane-store and gather variants need).
bool gemm_bf16_supported(int64_t M, int64_t N, int64_t K) {
    return M > 0 && N > 0 && K > 0 && M % BM == 0 && N % 128 == 0 && K % BK == 0 && M < (1 << 30) && N < (1 << 30) &&
           K < (1 << 30) && (M / BM) * (N / 128) < (1ll << 27) && M * K < (1ll << 31) && N * K < (1ll << 31); // 32-bit byte offsets
}

// The same kernel with edge tiles: any M and N of at least 64 whose 128-bit loads and paired stores stay
// aligned, that is an extent that runs along memory in an operand ([K,M] A, [K,N] B) is a multiple of 8 and
// N is even for a bf16 result. Loads of an edge tile clamp to the operand's last row / chunk, stores are masked.
bool gemm_bf16_supported(int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int out_bf16) {
    if (gemm_bf16_supported(M, N, K)) return true;
    return M >= 64 && N >= 64 && K > 0 && K % BK == 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30) &&
           ((M + BM - 1) / BM) * ((N + 127) / 128) < (1ll << 27) && (!trans_a || M % 8 == 0) && (trans_b || N % 8 == 0) &&
           (!out_bf16 || N % 2 == 0) && M * K < (1ll << 31) && N * K < (1ll << 31);
}

// Tile width: 128 columns when that wastes fewer columns past N, or when 256-wide tiles would leave CUs idle.
int gemm_bf16_tile_n(int64_t M, int64_t N) {
    const int64_t tm = (M + BM - 1) / BM;
    return ((N + 127) / 128 * 128 != (N + 255) / 256 * 256 || tm * ((N + 255) / 256) < 192) ? 128 : 256;
}

// Split K when the output still has too few tiles to occupy the 256 CUs: the smallest power of two that
// brings tiles * splits to 192 or more, while every split keeps at least 4 K tiles. The fold kernel works on
// groups of 4 columns, so a ragged N that is not a multiple of 4 stays unsplit.
int gemm_bf16_splits(int64_t M, int64_t N, int64_t K) {
    if (N % 4 != 0) return 1;
    const int64_t tiles = ((M + BM - 1) / BM) * ((N + gemm_bf16_tile_n(M, N) - 1) / gemm_bf16_tile_n(M, N));
    int s = 1;
    while (tiles * s < 192 && s < 16 && K % (2 * s * BK) == 0 && K / (2 * s) >= 4 * BK) s *= 2;
    return s;
}
uint64_t gemm_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    const int s = gemm_bf16_splits(M, N, K);
    return s > 1 ? (uint64_t)s * M * N * 4 : 0;
}

namespace {
hipError_t launch_layout(const GemmBf16 &p, hipStream_t st) {
    if (p.trans_a) return p.trans_b ? launch_width<true, true>(p, st) : launch_width<true, false>(p, st);
    return p.trans_b ? launch_width<false, true>(p, st) : launch_width<false, false>(p, st);
}
} // namespace

// Columns of a tile-aligned product whose 256-wide tiles fill whole rounds of the 256 CUs, when the rest would leave
// a second round mostly idle and fits one round of 128-wide tiles (e.g. 8192 x 3072: 384 tiles = 1.5 rounds become
// 2048 columns = 256 tiles and 1024 columns = 256 narrower, cheaper tiles). 0: compute the product in one launch.
int64_t gemm_bf16_column_split(int64_t M, int64_t N, int64_t K) {
    if (M % BM || N % 256 || gemm_bf16_tile_n(M, N) != 256 || gemm_bf16_splits(M, N, K) != 1) return 0;
    const int64_t tm = M / BM, tiles = tm * (N / 256);
    if (tiles <= 256 || tiles % 256 == 0 || ((tiles / 256) * 256) % tm) return 0;
    const int64_t n1 = (tiles / 256) * 256 / tm * 256, n2 = N - n1;
    if (n2 <= 0 || tm * (n2 / 128) > 256 || gemm_bf16_tile_n(M, n2) != 128 || gemm_bf16_splits(M, n2, K) != 1) return 0;
    return n1;
}

hipError_t gemm_bf16(const GemmBf16 &p, hipStream_t st) {
    if (!gemm_bf16_supported(p.M, p.N, p.K, p.trans_a, p.trans_b, p.out_bf16)) return hipErrorInvalidValue;
    const int64_t n1 = (p.plane || p.ldn) ? 0 : gemm_bf16_column_split(p.M, p.N, p.K);
    if (n1) {
        GemmBf16 a = p, b = p;
        a.N = n1;
        a.ldn = b.ldn = p.N;
        b.N = p.N - n1;
        const int64_t csz = p.out_bf16 ? 2 : 4, bsz = p.bias_dtype == DT_BF16 ? 2 : 4;
        b.B = (const uint16_t *)p.B + (p.trans_b ? n1 * p.K : n1);
        b.C = (char *)p.C + n1 * csz;
        if (p.bias) b.bias = (const char *)p.bias + n1 * bsz;
        if (p.residual) b.residual = (const char *)p.residual + n1 * csz;
        hipError_t e = launch_layout(a, st);
        return e != hipSuccess ? e : launch_layout(b, st);
    }
    return launch_layout(p, st);
}

} // namespace zk
