// Backward of the attention core (zyx-nn/src/causal_self_attention.rs:36-74) with respect to the packed
// qkv[B, T, 3, H, dh], given dy[B, T, H*dh]. The reverse rules of zyx/src/graph/autograd.rs for the ops the
// forward is made of (Mul :120-125, Div :126-134, Exp :87-95, Sub :111-119, reduce sum / max :299-379)
// compose to the softmax Jacobian; with Ps = softmax(scale q k^T), y = Ps/keep . v:
//   D  = rowsum(dy o y)                       (equals rowsum(Ps o dPs); the max term cancels)
//   dV = Ps^T . dy / keep
//   dS = Ps o (dy . v^T / keep - D)
//   dQ = scale dS . k,   dK = scale dS^T . q
// Ps is recomputed from the saved lse = ln sum exp(scale q k^T) instead of being stored.
//
// Matrix-core path (bf16, dh = 64, T % 128 == 0), two launches:
//   attn_bwd_dkv_k  (second) one workgroup per (batch, head, 128 keys), a wave owns 32 keys and streams query
//                   tiles; S = Q.K^T is formed queries x keys so that a lane owns a key column and the
//                   exponentiated / differentiated tiles, packed to bf16, are the B operands of
//                   dV^T += dy^T.P and dK^T += Q^T.dS (dy^T and Q^T come through the transposing LDS read);
//                   the three steps of a 32-query sub-tile run in three consecutive iterations (software pipeline);
//   attn_bwd_dq_k   (first) one workgroup per (batch, head, 128 queries), S^T = K.Q^T keys x queries (a lane owns
//                   a query, lse and D are per-lane scalars), dQ^T += K^T.dS^T; leaves -D keep and lse log2(e) of its
//                   queries in the program's workspace;
// No atomics: every output element has one owner, results are reproducible.
//
// attn_bwd_small_*: any dh <= 256 and T, f32 or bf16 storage, f32 arithmetic, one wave per query / key.
#include <type_traits>
#include "attn_common.hpp"
#include "kernels.hpp"

namespace zk {

using namespace attn;

namespace {

constexpr int STAGE_BWD = 2 * TILE + 512; // two tiles + lse*log2(e) [64] + D [64]

// 64 lanes x 16 (or 4) bytes from global memory straight into LDS at `lds` (wave-uniform byte address) + 16 (4) * lane.
// Written as instructions, not through the compiler's builtin: for the builtin the compiler waits for every such
// load in flight (vmcnt(0)) before the next LDS read that may touch the same array. Completion is tracked by hand:
// callers wait with s_waitcnt vmcnt and a workgroup barrier before anybody reads what was loaded. The compiler's own
// vmcnt bookkeeping stays safe: these loads only ever make the counter larger than it assumes.
__device__ __forceinline__ void load16_to_lds(const void *g, ZK_LDS void *lds) {
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(base), "v"(g) : "memory");
}
__device__ __forceinline__ void load4_to_lds(const void *g, ZK_LDS void *lds) {
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" : : "s"(base), "v"(g) : "memory");
}

// dK and dV as one software pipeline per workgroup (128 keys, a wave owns 32) over sub-tiles of 32 queries: iteration
// j issues S = Q.K^T and dP = dy.V^T of sub-tile j+1 and the products dV^T += dy^T.P, dK^T += Q^T.dS of sub-tile j-1
// (16 matrix instructions) between slices of sub-tile j's vector work (exp2, dS = P o (dP/keep - D), bf16 packing),
// in an order pinned by scheduling fences, so that inside one wave the matrix pipe and the vector unit always have
// independent work. Q / dy tiles of 64 queries with their lse*log2(e) and D rows live in a ring of 4 LDS stages
// filled by direct global->LDS loads three tiles ahead; one workgroup barrier per tile.
template <bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_bwd_dkv_k(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ dy,
                                                         const float *__restrict__ lse2, const float *__restrict__ Dn,
                                                         uint16_t *__restrict__ dqkv, int T, int H, float c, float scale,
                                                         float inv_keep) {
    constexpr int NS = 4;
    __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[NS * STAGE_BWD];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
    int bh, kblk;
    const int nblk = T / 128;
    // CAUSAL: pairs with key > query carry probability 0; tiles that hold only such pairs are not visited (the loop
    // bounds), and the tiles the diagonal crosses zero the masked probabilities, which zeroes dS too. The number of tiles
    // then depends on the block: the blocks with the most tiles (here: the first keys) come first in the grid, so that
    // short workgroups fill in behind long ones. Ids congruent mod 8 still share a head (and its XCD's L2) when the number
    // of heads is a multiple of 8.
    if (CAUSAL) {
        const int BH = (int)gridDim.x / nblk;
        bh = blockIdx.x % BH;
        kblk = blockIdx.x / BH;
    } else head_and_block(nblk, bh, kblk);
    {
    const int bb = bh / H, h = bh % H;
    const int64_t C = (int64_t)H * DH, ld = 3 * C;
    const uint16_t *qp = qkv + (int64_t)bb * T * ld + h * DH, *kp = qp + C, *vp = kp + C;
    const uint16_t *dop = dy + (int64_t)bb * T * C + h * DH;
    const float *lsep = lse2 + (int64_t)bh * T, *Dp = Dn + (int64_t)bh * T;
    const int tk = kblk * 128 + wave * 32 + (lane & 31);

    bf16x8 kfr[4], vfr[4]; // B operands: lane -> key, k-slots = dh
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        kfr[ks] = *(const bf16x8 *)(kp + (int64_t)tk * ld + ks * 16 + hh * 8);
        vfr[ks] = *(const bf16x8 *)(vp + (int64_t)tk * ld + ks * 16 + hh * 8);
    }

    // staging: lane l of a wave-load fetches the chunk that belongs at row l/8, physical slot l%8 of 8 tile rows;
    // wave w moves rows i*32 + w*8 .. +7 (i = 0, 1) of both tiles, waves 0 and 1 also the 64 lse and the 64 D values
    uint32_t gq[2], gdo[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int row = i * 32 + wave * 8 + (lane >> 3), cc = (lane & 7) ^ tile_f(row);
        gq[i] = (uint32_t)(row * ld + cc * 8) * 2;
        gdo[i] = (uint32_t)(row * C + cc * 8) * 2;
    }
    auto stage_tile = [&](int qt, int stage) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int rows = (i * 32 + wave * 8) * 128;
            load16_to_lds((const uint8_t *)qp + (int64_t)qt * TROWS * ld * 2 + gq[i], (ZK_LDS void *)(smem + stage + rows));
            load16_to_lds((const uint8_t *)dop + (int64_t)qt * TROWS * C * 2 + gdo[i], (ZK_LDS void *)(smem + stage + TILE + rows));
        }
        if (wave == 0) load4_to_lds(lsep + qt * TROWS + lane, (ZK_LDS void *)(smem + stage + 2 * TILE));
        else if (wave == 1) load4_to_lds(Dp + qt * TROWS + lane, (ZK_LDS void *)(smem + stage + 2 * TILE + 256));
    };

    int fr[4], ft[2][2];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) fr[ks] = frag_row_off(lane, ks);
#pragma unroll
    for (int db = 0; db < 2; db++) {
        ft[db][0] = frag_tr_off(lane, db, 0);
        ft[db][1] = frag_tr_off(lane, db, 1);
    }

    f32x16 dkT[2], dvT[2];
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) dkT[db][r] = dvT[db][r] = 0.0f;

    const int QT0 = CAUSAL ? 2 * kblk : 0; // first query tile that holds a query >= this block's first key
    const int NTQ = T / TROWS - QT0;       // tiles this block streams, u = 0 .. NTQ-1 is query tile QT0 + u
    const int k0w = kblk * 128 + wave * 32; // first key of this wave
#pragma unroll
    for (int u = 0; u < 3; u++)
        if (u < NTQ) stage_tile(QT0 + u, u * STAGE_BWD);
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();

    const f32x16 zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    f32x16 sA, dpA, sB, dpB;
    u32x4 pbA[2], dsA[2], pbB[2], dsB[2]; // P and dS of a sub-tile as bf16 pairs: [16-query half]
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int e = 0; e < 4; e++) pbB[s2][e] = dsB[s2][e] = 0u;
    // register r of a lane's S / dP tile is query 8*(r/4) + 4*hh + r%4 of the sub-tile: the dP accumulators start at that
    // query's -D keep, read from the stage's D row four at a time
    auto dp_start = [&](int stat) {
        f32x4 d[4];
#pragma unroll
        for (int g = 0; g < 4; g++) d[g] = *(const ZK_LDS f32x4 *)(smem + stat + 256 + (8 * g + 4 * hh) * 4);
        f32x16 v;
#pragma unroll
        for (int r = 0; r < 16; r++) v[r] = d[r >> 2][r & 3];
        return v;
    };
    dpA = dp_start(2 * TILE);
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        sA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_row(smem, fr[ks]), kfr[ks], ks == 0 ? zero16 : sA, 0, 0, 0);
        dpA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_row(smem, TILE + fr[ks]), vfr[ks], dpA, 0, 0, 0);
    }

    // One sub-tile. st1: stage and 32-row half that sub-tile j+1's Q / dy rows are read from; st3: the same for
    // sub-tile j-1 (transposed reads); stat, stat1: where the lse and D rows of sub-tiles j and j+1 are; qbase: first
    // query of sub-tile j.
    auto sub = [&](auto mask_, int st1, int st3, int stat, int stat1, int qbase, const f32x16 &sc, const f32x16 &dpc, f32x16 &sn, f32x16 &dpn,
                   const u32x4 (&pbp)[2], const u32x4 (&dsp)[2], u32x4 (&pbn)[2], u32x4 (&dsn)[2]) {
        constexpr bool MASK = decltype(mask_)::value;
        f32x16 dstart; // what sub-tile j+1's dP accumulators start from
        // Issue order, pinned by fences: matrix instruction i, then the LDS reads of the fragment DIST instructions
        // ahead, then slice i of the vector work, written so that no instruction reads the result of the one before
        // it: slice i scales and shifts element i+1 (two fma), exponentiates element i, multiplies element i-1 and
        // packs a finished pair.
        constexpr int DIST = 4;
        bf16x8 frg[16]; // 0..7: transposed dy^T / Q^T fragments of sub-tile j-1 (s2, db, which); 8..15: rows of Q / dy of j+1 (ks, which)
        auto read_frag = [&](int f) {
            if (f < 8) {
                const int s2 = f >> 2, db = (f >> 1) & 1, isq = f & 1;
                const int base = st3 + 16 * s2 * 128 + (isq ? 0 : TILE);
                frg[f] = frag_tr(smem, base + ft[db][0], base + ft[db][1]);
            } else {
                const int ks = (f - 8) >> 1, isdo = f & 1;
                frg[f] = frag_row(smem, st1 + (isdo ? TILE : 0) + fr[ks]);
            }
        };
        auto matrix = [&](int f) {
            if (f < 8) {
                const int s2 = f >> 2, db = (f >> 1) & 1, isq = f & 1;
                if (isq) dkT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frg[f], __builtin_bit_cast(bf16x8, dsp[s2]), dkT[db], 0, 0, 0);
                else dvT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frg[f], __builtin_bit_cast(bf16x8, pbp[s2]), dvT[db], 0, 0, 0);
            } else {
                const int ks = (f - 8) >> 1, isdo = f & 1;
                if (isdo) dpn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frg[f], vfr[ks], ks == 0 ? dstart : dpn, 0, 0, 0);
                else sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frg[f], kfr[ks], ks == 0 ? zero16 : sn, 0, 0, 0);
            }
        };
        // register r of this lane is query qbase + 8*(r/4) + 4*hh + r%4; its lse and D come in groups of four
        f32x4 l2[4];
        auto read_stat = [&](int g) { l2[g] = *(const ZK_LDS f32x4 *)(smem + stat + (8 * g + 4 * hh) * 4); };
        // element r: scale and shift (slot r-1) -> exp2 (slot r) -> product with dP - D keep (slot r+1); a pair is
        // packed one slot after its second product
        float arg[2], pv[4], ds[4];
        auto shift = [&](int r) { arg[r & 1] = __builtin_fmaf(sc[r], c, -l2[r >> 2][r & 3]); };
        auto expo = [&](int r) {
            pv[r & 3] = __builtin_amdgcn_exp2f(arg[r & 1]);
            if (MASK && qbase + 8 * (r >> 2) + 4 * hh + (r & 3) < tk) pv[r & 3] = 0.0f; // query before key
        };
        auto product = [&](int r) { ds[r & 3] = pv[r & 3] * dpc[r]; }; // keep . dS: 1 / keep goes into dK's final scale
        auto pack = [&](int r) { // elements r-1, r (r odd)
            uint32_t w0, w1; // two f32 -> two bf16, round to nearest even; written as instructions so that they stay in their slot
            asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w0) : "v"(pv[(r - 1) & 3]), "v"(pv[r & 3]));
            asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w1) : "v"(ds[(r - 1) & 3]), "v"(ds[r & 3]));
            pbn[r >> 3][(r >> 1) & 3] = w0;
            dsn[r >> 3][(r >> 1) & 3] = w1;
        };
        read_stat(0);
        read_stat(1);
#pragma unroll
        for (int f = 0; f < DIST; f++) read_frag(f);
        __builtin_amdgcn_sched_barrier(0);
        shift(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            matrix(i);
            __builtin_amdgcn_sched_barrier(0);
            if (i + DIST < 16) read_frag(i + DIST);
            if (i == 2) read_stat(2);
            if (i == 4) dstart = dp_start(stat1);
            if (i == 6) read_stat(3);
            if (i > 0) product(i - 1);
            expo(i);
            if (i + 1 < 16) shift(i + 1);
            if (i >= 3 && (i & 1)) pack(i - 2);
            __builtin_amdgcn_sched_barrier(0);
        }
        product(15);
        pack(15);
        // pinned here: left alone, the compiler moves the vector work down to its first use in the next iteration
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) asm volatile("" : "+v"(pbn[s2]), "+v"(dsn[s2]));
    };
    const std::true_type masked;
    const std::false_type plain;
    // tile u: sub-tiles 2u (rows 0..31) and 2u+1. Sub-tile 2u reads the second half of tile u for j+1 and the second
    // half of tile u-1 for j-1 (sub-tile 0: any landed rows, against a zero P); sub-tile 2u+1 reads the first half of
    // tile u+1 (past the end: rows nobody uses the product of) and the first half of tile u.
    int su = 0, sprev = 0; // stages of tile u and of tile u-1
    for (int u = 0; u < NTQ; u++) {
        const int snext = su + STAGE_BWD == NS * STAGE_BWD ? 0 : su + STAGE_BWD;
        const int q0 = (QT0 + u) * TROWS;
        const bool diag = CAUSAL && q0 < k0w + 31; // some query of the tile is before some key of this wave
        if (CAUSAL && diag) sub(masked, su + 32 * 128, sprev + 32 * 128, su + 2 * TILE, su + 2 * TILE + 128, q0, sA, dpA, sB, dpB, pbB, dsB, pbA, dsA);
        else sub(plain, su + 32 * 128, sprev + 32 * 128, su + 2 * TILE, su + 2 * TILE + 128, q0, sA, dpA, sB, dpB, pbB, dsB, pbA, dsA);
        // tile u+1 must have landed, tile u-1 is no longer read: its stage takes tile u+3
        if (u + 2 < NTQ) {
            if (wave < 2) __builtin_amdgcn_s_waitcnt(0x0f70 | 5);
            else __builtin_amdgcn_s_waitcnt(0x0f70 | 4);
        } else __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        if (u + 3 < NTQ) stage_tile(QT0 + u + 3, sprev == su ? 3 * STAGE_BWD : sprev);
        if (CAUSAL && diag) sub(masked, snext, su, su + 2 * TILE + 128, snext + 2 * TILE, q0 + 32, sB, dpB, sA, dpA, pbA, dsA, pbB, dsB);
        else sub(plain, snext, su, su + 2 * TILE + 128, snext + 2 * TILE, q0 + 32, sB, dpB, sA, dpA, pbA, dsA, pbB, dsB);
        sprev = su;
        su = snext;
    }
    // the products of the last sub-tile (second half of the last tile, stage sprev)
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int db = 0; db < 2; db++) {
            const int base = sprev + (32 + 16 * s2) * 128;
            dvT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(smem, base + TILE + ft[db][0], base + TILE + ft[db][1]), __builtin_bit_cast(bf16x8, pbB[s2]), dvT[db], 0, 0, 0);
            dkT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(smem, base + ft[db][0], base + ft[db][1]), __builtin_bit_cast(bf16x8, dsB[s2]), dkT[db], 0, 0, 0);
        }

    // result register r of lane: d = db*32 + 8*(r/4) + 4*hh + r%4, key = lane % 32
    const float ks_ = scale * inv_keep; // dK accumulated keep . dS
    uint16_t *dk = dqkv + ((int64_t)bb * T + tk) * ld + C + h * DH, *dv = dk + C;
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int d = db * 32 + 8 * g + 4 * hh;
            *(u32x2 *)(dk + d) = pack4_trunc(dkT[db][4 * g] * ks_, dkT[db][4 * g + 1] * ks_, dkT[db][4 * g + 2] * ks_, dkT[db][4 * g + 3] * ks_);
            *(u32x2 *)(dv + d) = pack4_trunc(dvT[db][4 * g] * inv_keep, dvT[db][4 * g + 1] * inv_keep, dvT[db][4 * g + 2] * inv_keep, dvT[db][4 * g + 3] * inv_keep);
        }
    }
}

// dQ in the same software pipeline, one workgroup per (batch, head, 128 queries), a wave owns 32 queries and streams key
// tiles in sub-tiles of 32 keys: iteration j issues S^T = K.Q^T and dP^T = V.dy^T of sub-tile j+1 and dQ^T += K^T.dS^T of
// sub-tile j-1 (12 matrix instructions) between the vector work of sub-tile j. A lane owns a query: its lse log2(e) and
// -D keep are scalars, and the dP^T accumulators start at -D keep.
template <bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_k(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ y,
                                                        const uint16_t *__restrict__ dy, const float *__restrict__ lse,
                                                        float *__restrict__ lse2, float *__restrict__ Dn,
                                                        uint16_t *__restrict__ dqkv, int T, int H, float c, float scale,
                                                        float inv_keep) {
    constexpr int NS = 4, STAGE = 2 * TILE; // K tile then V tile
    __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[NS * STAGE];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
    int bh, qblk;
    const int nblk = T / 128;
    if (CAUSAL) { // as in the dK / dV kernel: the last queries (most key tiles) first
        const int BH = (int)gridDim.x / nblk;
        bh = blockIdx.x % BH;
        qblk = nblk - 1 - blockIdx.x / BH;
    } else head_and_block(nblk, bh, qblk);
    {
    const int bb = bh / H, h = bh % H;
    const int64_t C = (int64_t)H * DH, ld = 3 * C;
    const uint16_t *qp = qkv + (int64_t)bb * T * ld + h * DH, *kp = qp + C, *vp = kp + C;
    const int tq = qblk * 128 + wave * 32 + (lane & 31);

    bf16x8 qfr[4], dofr[4]; // B operands: lane -> query, k-slots = dh
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        qfr[ks] = *(const bf16x8 *)(qp + (int64_t)tq * ld + ks * 16 + hh * 8);
        dofr[ks] = *(const bf16x8 *)(dy + ((int64_t)bb * T + tq) * C + h * DH + ks * 16 + hh * 8);
    }
    // D = sum_d dy o y of this lane's query (each half-wave holds half of the row), kept as -D keep; with lse log2(e) it
    // also goes to the workspace, where the dK / dV kernel (launched after this one) reads both
    float dsum = 0.0f;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        const u32x4 o = *(const u32x4 *)(y + ((int64_t)bb * T + tq) * C + h * DH + ks * 16 + hh * 8);
        const u32x4 g = __builtin_bit_cast(u32x4, dofr[ks]);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            dsum = __builtin_fmaf(__uint_as_float(o[i] << 16), __uint_as_float(g[i] << 16), dsum);
            dsum = __builtin_fmaf(__uint_as_float(o[i] & 0xffff0000u), __uint_as_float(g[i] & 0xffff0000u), dsum);
        }
    }
    dsum += xor32(dsum);
    const float l2 = lse[(int64_t)bh * T + tq] * kLog2e, dn = -dsum / inv_keep;
    if (hh == 0) {
        lse2[(int64_t)bh * T + tq] = l2;
        Dn[(int64_t)bh * T + tq] = dn;
    }
    f32x16 dstart;
#pragma unroll
    for (int r = 0; r < 16; r++) dstart[r] = dn;

    uint32_t go[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int row = i * 32 + wave * 8 + (lane >> 3), cc = (lane & 7) ^ tile_f(row);
        go[i] = (uint32_t)(row * ld + cc * 8) * 2;
    }
    auto stage_tile = [&](int kt, int stage) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int rows = (i * 32 + wave * 8) * 128;
            load16_to_lds((const uint8_t *)kp + (int64_t)kt * TROWS * ld * 2 + go[i], (ZK_LDS void *)(smem + stage + rows));
            load16_to_lds((const uint8_t *)vp + (int64_t)kt * TROWS * ld * 2 + go[i], (ZK_LDS void *)(smem + stage + TILE + rows));
        }
    };
    int fr[4], ft[2][2];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) fr[ks] = frag_row_off(lane, ks);
#pragma unroll
    for (int db = 0; db < 2; db++) {
        ft[db][0] = frag_tr_off(lane, db, 0);
        ft[db][1] = frag_tr_off(lane, db, 1);
    }

    f32x16 dqT[2];
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int r = 0; r < 16; r++) dqT[db][r] = 0.0f;

    const int NT = CAUSAL ? 2 * qblk + 2 : T / TROWS;
    const int q0w = qblk * 128 + wave * 32; // first query of this wave
#pragma unroll
    for (int u = 0; u < 3; u++)
        if (u < NT) stage_tile(u, u * STAGE);
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();

    const f32x16 zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    f32x16 sA, dpA, sB, dpB;
    u32x4 dsA[2], dsB[2]; // dS^T of a sub-tile as bf16 pairs: [16-key half]
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int e = 0; e < 4; e++) dsB[s2][e] = 0u;
    dpA = dstart;
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        sA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_row(smem, fr[ks]), qfr[ks], ks == 0 ? zero16 : sA, 0, 0, 0);
        dpA = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_row(smem, TILE + fr[ks]), dofr[ks], dpA, 0, 0, 0);
    }

    // One sub-tile. st1: stage and 32-row half that sub-tile j+1's K / V rows are read from; st3: the same for sub-tile
    // j-1's K rows (transposed reads); kbase: first key of sub-tile j.
    auto sub = [&](auto mask_, int st1, int st3, int kbase, const f32x16 &sc, const f32x16 &dpc, f32x16 &sn, f32x16 &dpn,
                   const u32x4 (&dsp)[2], u32x4 (&dsn)[2]) {
        constexpr bool MASK = decltype(mask_)::value;
        constexpr int DIST = 4;
        bf16x8 frg[12]; // 0..3: K^T fragments of sub-tile j-1 (s2, db); 4..11: rows of K / V of sub-tile j+1 (ks, which)
        auto read_frag = [&](int f) {
            if (f < 4) {
                const int s2 = f >> 1, db = f & 1, base = st3 + 16 * s2 * 128;
                frg[f] = frag_tr(smem, base + ft[db][0], base + ft[db][1]);
            } else {
                const int ks = (f - 4) >> 1, isv = f & 1;
                frg[f] = frag_row(smem, st1 + (isv ? TILE : 0) + fr[ks]);
            }
        };
        auto matrix = [&](int f) {
            if (f < 4) dqT[f & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frg[f], __builtin_bit_cast(bf16x8, dsp[f >> 1]), dqT[f & 1], 0, 0, 0);
            else {
                const int ks = (f - 4) >> 1, isv = f & 1;
                if (isv) dpn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frg[f], dofr[ks], ks == 0 ? dstart : dpn, 0, 0, 0);
                else sn = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frg[f], qfr[ks], ks == 0 ? zero16 : sn, 0, 0, 0);
            }
        };
        // element r (key kbase + 8*(r/4) + 4*hh + r%4): scale and shift -> exp2 -> product with dP - D keep, one step
        // apart, so that no instruction reads the result of the one before it; a pair is packed one step after its
        // second product. 18 steps over the 12 slots behind the matrix instructions.
        float arg[2], pv[4], ds[4];
        auto step = [&](int k) {
            if (k >= 1 && k <= 16) ds[(k - 1) & 3] = pv[(k - 1) & 3] * dpc[k - 1];
            if (k < 16) {
                pv[k & 3] = __builtin_amdgcn_exp2f(arg[k & 1]);
                if (MASK && kbase + 8 * (k >> 2) + 4 * hh + (k & 3) > tq) pv[k & 3] = 0.0f; // key after query
            }
            if (k + 1 < 16) arg[(k + 1) & 1] = __builtin_fmaf(sc[k + 1], c, -l2);
            if (k >= 3 && (k & 1)) { // elements k-3, k-2
                uint32_t w; // two f32 -> two bf16, round to nearest even; written as an instruction so that it stays in its slot
                asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(w) : "v"(ds[(k - 3) & 3]), "v"(ds[(k - 2) & 3]));
                dsn[(k - 2) >> 3][((k - 2) >> 1) & 3] = w;
            }
        };
#pragma unroll
        for (int f = 0; f < DIST; f++) read_frag(f);
        __builtin_amdgcn_sched_barrier(0);
        arg[0] = __builtin_fmaf(sc[0], c, -l2);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 12; i++) {
            matrix(i);
            __builtin_amdgcn_sched_barrier(0);
            if (i + DIST < 12) read_frag(i + DIST);
#pragma unroll
            for (int k = (i * 18) / 12; k < ((i + 1) * 18) / 12; k++) step(k);
            __builtin_amdgcn_sched_barrier(0);
        }
        // pinned here: left alone, the compiler moves the vector work down to its first use in the next iteration
#pragma unroll
        for (int s2 = 0; s2 < 2; s2++) asm volatile("" : "+v"(dsn[s2]));
    };
    const std::true_type masked;
    const std::false_type plain;
    int su = 0, sprev = 0; // stages of tile u and of tile u-1
    for (int u = 0; u < NT; u++) {
        const int snext = su + STAGE == NS * STAGE ? 0 : su + STAGE;
        const bool diag = CAUSAL && u * TROWS + TROWS - 1 > q0w; // some key of the tile is after some query of this wave
        if (CAUSAL && diag) sub(masked, su + 32 * 128, sprev + 32 * 128, u * TROWS, sA, dpA, sB, dpB, dsB, dsA);
        else sub(plain, su + 32 * 128, sprev + 32 * 128, u * TROWS, sA, dpA, sB, dpB, dsB, dsA);
        // tile u+1 must have landed, tile u-1 is no longer read: its stage takes tile u+3
        if (u + 2 < NT) __builtin_amdgcn_s_waitcnt(0x0f70 | 4);
        else __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        if (u + 3 < NT) stage_tile(u + 3, sprev == su ? 3 * STAGE : sprev);
        if (CAUSAL && diag) sub(masked, snext, su, u * TROWS + 32, sB, dpB, sA, dpA, dsA, dsB);
        else sub(plain, snext, su, u * TROWS + 32, sB, dpB, sA, dpA, dsA, dsB);
        sprev = su;
        su = snext;
    }
    // the product of the last sub-tile (second half of the last tile, stage sprev)
#pragma unroll
    for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
        for (int db = 0; db < 2; db++) {
            const int base = sprev + (32 + 16 * s2) * 128;
            dqT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_tr(smem, base + ft[db][0], base + ft[db][1]), __builtin_bit_cast(bf16x8, dsB[s2]), dqT[db], 0, 0, 0);
        }

    const float qs = scale * inv_keep; // dQ accumulated keep . dS
    uint16_t *dq = dqkv + ((int64_t)bb * T + tq) * ld + h * DH;
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            *(u32x2 *)(dq + db * 32 + 8 * g + 4 * hh) =
                pack4_trunc(dqT[db][4 * g] * qs, dqT[db][4 * g + 1] * qs, dqT[db][4 * g + 2] * qs, dqT[db][4 * g + 3] * qs);
    }
}

// ---- general path ---------------------------------------------------------------------------------------
template <int DT> __device__ __forceinline__ float ldf(const void *p, int64_t i) {
    if (DT == DT_F32) return ((const float *)p)[i];
    return bf16_to_f32(((const uint16_t *)p)[i]);
}
template <int DT> __device__ __forceinline__ void stf(void *p, int64_t i, float v) {
    if (DT == DT_F32) ((float *)p)[i] = v;
    else ((uint16_t *)p)[i] = f32_to_bf16_trunc(v);
}

// One wave per (query | key) row `t` of head bh. ROLE 0: dQ row (streams keys); ROLE 1: dK and dV rows
// (streams queries). Partners are taken 64 at a time with lane = partner for the dot products, then
// lane = d for the weighted sums; the weights pass through LDS.
template <int DT, int ROLE>
__global__ __launch_bounds__(64) void attn_bwd_small_k(const void *__restrict__ qkv, const void *__restrict__ y,
                                                       const void *__restrict__ dy, const float *__restrict__ lse,
                                                       void *__restrict__ dqkv, int T, int H, int dh, float scale, float keep,
                                                       int causal) {
    __shared__ float mine[2][256], w0[64], w1[64];
    const int lane = threadIdx.x, t = blockIdx.x, bh = blockIdx.y, bb = bh / H, h = bh % H;
    const int64_t C = (int64_t)H * dh, ld = 3 * C;
    const int64_t rowq = ((int64_t)bb * T + t) * ld + h * dh, rowy = ((int64_t)bb * T + t) * C + h * dh;
    // ROLE 0: mine[0] = q_t, mine[1] = dy_t.  ROLE 1: mine[0] = k_t, mine[1] = v_t.
    for (int d = lane; d < dh; d += 64) {
        mine[0][d] = ldf<DT>(qkv, rowq + (ROLE ? C : 0) + d);
        mine[1][d] = ROLE ? ldf<DT>(qkv, rowq + 2 * C + d) : ldf<DT>(dy, rowy + d);
    }
    __syncthreads();
    float Dt = 0.0f, lse_t = 0.0f;
    if (ROLE == 0) {
        float a = 0.0f;
        for (int d = lane; d < dh; d += 64) a += ldf<DT>(dy, rowy + d) * ldf<DT>(y, rowy + d);
        Dt = wave_allreduce_f32(a, OpAdd());
        lse_t = lse[(int64_t)bh * T + t];
    }
    float acc0[4] = {0, 0, 0, 0}, acc1[4] = {0, 0, 0, 0};
    // causal: a query's partners are the keys 0..t, a key's partners the queries t..T-1
    const int jlo = (causal && ROLE == 1) ? t : 0, jhi = (causal && ROLE == 0) ? t + 1 : T;
    for (int j0 = (jlo / 64) * 64; j0 < jhi; j0 += 64) {
        const int j = j0 + lane;
        float p = 0.0f, ds = 0.0f;
        if (j >= jlo && j < jhi) {
            const int64_t rq = ((int64_t)bb * T + j) * ld + h * dh, ry = ((int64_t)bb * T + j) * C + h * dh;
            float s = 0.0f, dp = 0.0f, Dj = Dt;
            if (ROLE == 0) { // partner j is a key: s = q_t.k_j, dp = dy_t.v_j
                for (int d = 0; d < dh; d++) {
                    s = __builtin_fmaf(mine[0][d], ldf<DT>(qkv, rq + C + d), s);
                    dp = __builtin_fmaf(mine[1][d], ldf<DT>(qkv, rq + 2 * C + d), dp);
                }
                p = expf(s * scale - lse_t);
            } else { // partner j is a query: s = q_j.k_t, dp = dy_j.v_t, D_j = dy_j.y_j
                Dj = 0.0f;
                for (int d = 0; d < dh; d++) {
                    const float g = ldf<DT>(dy, ry + d);
                    s = __builtin_fmaf(ldf<DT>(qkv, rq + d), mine[0][d], s);
                    dp = __builtin_fmaf(g, mine[1][d], dp);
                    Dj = __builtin_fmaf(g, ldf<DT>(y, ry + d), Dj);
                }
                p = expf(s * scale - lse[(int64_t)bh * T + j]);
            }
            ds = p * (dp / keep - Dj);
        }
        __syncthreads();
        w0[lane] = ds;
        w1[lane] = p;
        __syncthreads();
        const int nk = min(64, T - j0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < dh) {
                const int64_t rq = ((int64_t)bb * T + j0) * ld + h * dh + d, ry = ((int64_t)bb * T + j0) * C + h * dh + d;
                float a0 = acc0[i], a1 = acc1[i];
                for (int jj = 0; jj < nk; jj++) {
                    if (ROLE == 0) a0 = __builtin_fmaf(w0[jj], ldf<DT>(qkv, rq + jj * ld + C), a0);    // dq += ds_j k_j
                    else {
                        a0 = __builtin_fmaf(w0[jj], ldf<DT>(qkv, rq + jj * ld), a0);                  // dk += ds_j q_j
                        a1 = __builtin_fmaf(w1[jj], ldf<DT>(dy, ry + jj * C), a1);                    // dv += p_j dy_j
                    }
                }
                acc0[i] = a0;
                acc1[i] = a1;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        if (d < dh) {
            if (ROLE == 0) stf<DT>(dqkv, rowq + d, acc0[i] * scale);
            else {
                stf<DT>(dqkv, rowq + C + d, acc0[i] * scale);
                stf<DT>(dqkv, rowq + 2 * C + d, acc1[i] / keep);
            }
        }
    }
}

} // namespace

uint64_t attention_bwd_workspace_bytes(const Attention &p) {
    return attention_fast_path(p) ? 2 * (uint64_t)p.B * p.H * p.T * 4 : 0; // -D * keep and lse * log2(e)
}

hipError_t attention_bwd(const AttentionBwd &p, hipStream_t st) {
    const Attention &f = p.fwd;
    if (f.B <= 0 || f.T <= 0 || f.H <= 0 || f.dh <= 0) return hipSuccess;
    if (attention_fast_path(f)) {
        if (!p.workspace) return hipErrorInvalidValue;
        float *Dn = (float *)p.workspace, *L2 = Dn + (int64_t)f.B * f.H * f.T;
        const int nblk = f.T / 128;
        dim3 grid((unsigned)(f.B * f.H * nblk)), block(256);
        const float c = f.scale * kLog2e, ik = 1.0f / f.keep;
        // the dQ kernel also leaves -D keep and lse log2(e) of its rows in the workspace for the dK / dV kernel
#define ZK_BWD_DQ(K)                                                                                                  \
    hipLaunchKernelGGL(K, grid, block, 0, st, (const uint16_t *)f.qkv, (const uint16_t *)f.y, (const uint16_t *)p.dy, f.lse, L2, Dn, \
                       (uint16_t *)p.dqkv, f.T, f.H, c, f.scale, ik)
#define ZK_BWD(K)                                                                                                     \
    hipLaunchKernelGGL(K, grid, block, 0, st, (const uint16_t *)f.qkv, (const uint16_t *)p.dy, L2, Dn, (uint16_t *)p.dqkv, f.T, \
                       f.H, c, f.scale, ik)
        if (f.causal) {
            ZK_BWD_DQ(attn_bwd_dq_k<true>);
            ZK_BWD(attn_bwd_dkv_k<true>);
        } else {
            ZK_BWD_DQ(attn_bwd_dq_k<false>);
            ZK_BWD(attn_bwd_dkv_k<false>);
        }
#undef ZK_BWD_DQ
#undef ZK_BWD
        return hipGetLastError();
    }
    if (f.dh > 256 || (int64_t)f.B * f.H > 65535 || (f.dtype != DT_F32 && f.dtype != DT_BF16)) return hipErrorInvalidValue;
    dim3 grid((unsigned)f.T, (unsigned)(f.B * f.H)), block(64);
#define ZK_SMALL(DT, ROLE)                                                                                            \
    hipLaunchKernelGGL((attn_bwd_small_k<DT, ROLE>), grid, block, 0, st, f.qkv, f.y, p.dy, f.lse, p.dqkv, f.T, f.H, f.dh, \
                       f.scale, f.keep, f.causal)
    if (f.dtype == DT_F32) {
        ZK_SMALL(DT_F32, 0);
        ZK_SMALL(DT_F32, 1);
    } else {
        ZK_SMALL(DT_BF16, 0);
        ZK_SMALL(DT_BF16, 1);
    }
#undef ZK_SMALL
    return hipGetLastError();
}

} // namespace zk
