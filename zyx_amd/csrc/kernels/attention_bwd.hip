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
// Matrix-core path (bf16, dh = 64, T % 128 == 0), three launches:
//   attn_bwd_d_k    D[B,H,T] into the program's workspace;
//   attn_bwd_dkv_k  one workgroup per (batch, head, 128 keys), a wave owns 32 keys and streams query
//                   tiles; S = Q.K^T is formed queries x keys so that a lane owns a key column and the
//                   exponentiated / differentiated tiles, packed to bf16, are the B operands of
//                   dV^T += dy^T.P and dK^T += Q^T.dS (dy^T and Q^T come through the transposing LDS read);
//   attn_bwd_dq_k   one workgroup per (batch, head, 128 queries), S^T = K.Q^T keys x queries (a lane owns
//                   a query, lse and D are per-lane scalars), dQ^T += K^T.dS^T.
// No atomics: every output element has one owner, results are reproducible.
//
// attn_bwd_small_*: any dh <= 256 and T, f32 or bf16 storage, f32 arithmetic, one wave per query / key.
#include "attn_common.hpp"
#include "kernels.hpp"

namespace zk {

using namespace attn;

namespace {

constexpr int STAGE_BWD = 2 * TILE + 512; // two tiles + lse*log2(e) [64] + D [64]

// D[bh, t] = sum_d dy[b,t,h,d] * y[b,t,h,d]; 8 lanes per row of 64.
__global__ __launch_bounds__(256) void attn_bwd_d_k(const uint16_t *__restrict__ y, const uint16_t *__restrict__ dy,
                                                    float *__restrict__ D, int64_t rows, int T, int H) {
    const int64_t row = (int64_t)blockIdx.x * 32 + (threadIdx.x >> 3); // row = (b*T + t)*H + h
    const int part = threadIdx.x & 7;
    float a = 0.0f;
    if (row < rows) {
        const u32x4 u = *(const u32x4 *)(y + row * DH + part * 8), v = *(const u32x4 *)(dy + row * DH + part * 8);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            a = __builtin_fmaf(__uint_as_float(u[i] << 16), __uint_as_float(v[i] << 16), a);
            a = __builtin_fmaf(__uint_as_float(u[i] & 0xffff0000u), __uint_as_float(v[i] & 0xffff0000u), a);
        }
    }
    a += dpp_f32<kDppQuadXor1>(a);
    a += dpp_f32<kDppQuadXor2>(a);
    a += dpp_f32<kDppRowHalfMirror>(a);
    if (row < rows && part == 0) {
        const int64_t bt = row / H, h = row % H, b = bt / T, t = bt % T;
        D[(b * H + h) * T + t] = a;
    }
}

// CAUSAL (both kernels below): pairs with key > query carry probability 0. Tiles that hold only such pairs are not
// visited (the workgroup's loop bounds) or not computed (a wave's own keys / queries), and the tiles the diagonal
// crosses zero the masked probabilities, which zeroes dS too. The number of tiles then depends on the block, so a
// workgroup takes blocks j and nblk-1-j one after the other: equal work for every workgroup, on whatever CU.
template <bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_bwd_dkv_k(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ dy,
                                                         const float *__restrict__ lse, const float *__restrict__ D,
                                                         uint16_t *__restrict__ dqkv, int T, int H, float c, float scale,
                                                         float inv_keep) {
    __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[2 * STAGE_BWD];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
    int bh, kblk;
    const int nblk = T / 128;
    head_and_block(CAUSAL ? (nblk + 1) / 2 : nblk, bh, kblk);
    const int blk_first = kblk;
#pragma nounroll
    for (int pass = 0; pass < (CAUSAL ? 2 : 1); pass++) {
    if (CAUSAL && pass) {
        kblk = nblk - 1 - blk_first;
        if (kblk == blk_first) break;
    }
    const int bb = bh / H, h = bh % H;
    const int64_t C = (int64_t)H * DH, ld = 3 * C;
    const uint16_t *qp = qkv + (int64_t)bb * T * ld + h * DH, *kp = qp + C, *vp = kp + C;
    const uint16_t *dop = dy + (int64_t)bb * T * C + h * DH;
    const float *lsep = lse + (int64_t)bh * T, *Dp = D + (int64_t)bh * T;
    const int tk = kblk * 128 + wave * 32 + (lane & 31);

    bf16x8 kfr[4], vfr[4]; // B operands: lane -> key, k-slots = dh
#pragma unroll
    for (int ks = 0; ks < 4; ks++) {
        kfr[ks] = *(const bf16x8 *)(kp + (int64_t)tk * ld + ks * 16 + hh * 8);
        vfr[ks] = *(const bf16x8 *)(vp + (int64_t)tk * ld + ks * 16 + hh * 8);
    }

    u32x4 rq[2], rdo[2];
    float rstat = 0.0f; // threads 0..63: lse of query tid; 64..127: D of query tid - 64
    int sl[2];
    uint32_t gq[2], gdo[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int ch = tid + 256 * i, row = ch >> 3, cc = ch & 7;
        gq[i] = (uint32_t)(row * ld + cc * 8) * 2;
        gdo[i] = (uint32_t)(row * C + cc * 8) * 2;
        sl[i] = tile_slot(row, cc);
    }
    auto gload = [&](int qt) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            rq[i] = *(const u32x4 *)((const uint8_t *)qp + (int64_t)qt * TROWS * ld * 2 + gq[i]);
            rdo[i] = *(const u32x4 *)((const uint8_t *)dop + (int64_t)qt * TROWS * C * 2 + gdo[i]);
        }
        if (tid < 64) rstat = lsep[qt * TROWS + tid] * kLog2e;
        else if (tid < 128) rstat = Dp[qt * TROWS + tid - 64];
    };
    auto lwrite = [&](int stage) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            *(ZK_LDS u32x4 *)(smem + stage + sl[i]) = rq[i];
            *(ZK_LDS u32x4 *)(smem + stage + TILE + sl[i]) = rdo[i];
        }
        if (tid < 128) *(ZK_LDS float *)(smem + stage + 2 * TILE + tid * 4) = rstat;
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

    const int NT = T / TROWS;
    const int QT0 = CAUSAL ? 2 * kblk : 0;        // first query tile that holds a query >= this block's first key
    const int k0w = kblk * 128 + wave * 32;       // first key of this wave
    gload(QT0);
    lwrite(0);
    __syncthreads();
    int stage = 0;
    for (int qt = QT0; qt < NT; qt++) {
        if (qt + 1 < NT) gload(qt + 1);
        const bool diag = CAUSAL && qt * TROWS < k0w + 31; // some query of the tile is before some key of this wave
        if (!CAUSAL || qt * TROWS + TROWS - 1 >= k0w) {
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            f32x16 s, dp;
#pragma unroll
            for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const bf16x8 a = frag_row(smem, stage + qb * 32 * 128 + fr[ks]);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, kfr[ks], s, 0, 0, 0);
            }
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const bf16x8 a = frag_row(smem, stage + TILE + qb * 32 * 128 + fr[ks]);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, vfr[ks], dp, 0, 0, 0);
            }
            // register r of this lane is query qb*32 + 8*(r/4) + 4*hh + r%4
            bf16x8 pb[2], dsb[2];
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                f32x8 p, ds;
#pragma unroll
                for (int g = 0; g < 2; g++) {
                    const int q0 = qb * 32 + 8 * (2 * s2 + g) + 4 * hh;
                    const f32x4 l2 = *(const ZK_LDS f32x4 *)(smem + stage + 2 * TILE + q0 * 4);
                    const f32x4 dd = *(const ZK_LDS f32x4 *)(smem + stage + 2 * TILE + 256 + q0 * 4);
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        const int r = 8 * s2 + 4 * g + j;
                        float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[r], c, -l2[j]));
                        if (CAUSAL && diag && qt * TROWS + q0 + j < tk) pv = 0.0f;
                        p[4 * g + j] = pv;
                        ds[4 * g + j] = pv * __builtin_fmaf(dp[r], inv_keep, -dd[j]);
                    }
                }
                pb[s2] = __builtin_convertvector(p, bf16x8);
                dsb[s2] = __builtin_convertvector(ds, bf16x8);
            }
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                for (int db = 0; db < 2; db++) {
                    const int base = stage + (qb * 32 + 16 * s2) * 128;
                    const bf16x8 doT = frag_tr(smem, base + TILE + ft[db][0], base + TILE + ft[db][1]);
                    dvT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(doT, pb[s2], dvT[db], 0, 0, 0);
                    const bf16x8 qT = frag_tr(smem, base + ft[db][0], base + ft[db][1]);
                    dkT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qT, dsb[s2], dkT[db], 0, 0, 0);
                }
        }
        }
        if (qt + 1 < NT) lwrite(stage ^ STAGE_BWD);
        __syncthreads();
        stage ^= STAGE_BWD;
    }

    // result register r of lane: d = db*32 + 8*(r/4) + 4*hh + r%4, key = lane % 32
    uint16_t *dk = dqkv + ((int64_t)bb * T + tk) * ld + C + h * DH, *dv = dk + C;
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const int d = db * 32 + 8 * g + 4 * hh;
            *(u32x2 *)(dk + d) = pack4_trunc(dkT[db][4 * g] * scale, dkT[db][4 * g + 1] * scale, dkT[db][4 * g + 2] * scale, dkT[db][4 * g + 3] * scale);
            *(u32x2 *)(dv + d) = pack4_trunc(dvT[db][4 * g] * inv_keep, dvT[db][4 * g + 1] * inv_keep, dvT[db][4 * g + 2] * inv_keep, dvT[db][4 * g + 3] * inv_keep);
        }
    }
}

template <bool CAUSAL>
__global__ __launch_bounds__(256, 2) void attn_bwd_dq_k(const uint16_t *__restrict__ qkv, const uint16_t *__restrict__ dy,
                                                        const float *__restrict__ lse, const float *__restrict__ D,
                                                        uint16_t *__restrict__ dqkv, int T, int H, float c, float scale,
                                                        float inv_keep) {
    __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[4 * TILE];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;
    int bh, qblk;
    const int nblk = T / 128;
    head_and_block(CAUSAL ? (nblk + 1) / 2 : nblk, bh, qblk);
    const int blk_first = qblk;
#pragma nounroll
    for (int pass = 0; pass < (CAUSAL ? 2 : 1); pass++) {
    if (CAUSAL && pass) {
        qblk = nblk - 1 - blk_first;
        if (qblk == blk_first) break;
    }
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
    const float l2 = lse[(int64_t)bh * T + tq] * kLog2e, dd = D[(int64_t)bh * T + tq];

    u32x4 rk[2], rv[2];
    int sl[2];
    uint32_t go[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int ch = tid + 256 * i, row = ch >> 3, cc = ch & 7;
        go[i] = (uint32_t)(row * ld + cc * 8) * 2;
        sl[i] = tile_slot(row, cc);
    }
    auto gload = [&](int kt) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            rk[i] = *(const u32x4 *)((const uint8_t *)kp + (int64_t)kt * TROWS * ld * 2 + go[i]);
            rv[i] = *(const u32x4 *)((const uint8_t *)vp + (int64_t)kt * TROWS * ld * 2 + go[i]);
        }
    };
    auto lwrite = [&](int stage) {
#pragma unroll
        for (int i = 0; i < 2; i++) {
            *(ZK_LDS u32x4 *)(smem + stage + sl[i]) = rk[i];
            *(ZK_LDS u32x4 *)(smem + stage + TILE + sl[i]) = rv[i];
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
    gload(0);
    lwrite(0);
    __syncthreads();
    int stage = 0;
    for (int kt = 0; kt < NT; kt++) {
        if (kt + 1 < NT) gload(kt + 1);
        const bool diag = CAUSAL && kt * TROWS + TROWS - 1 > q0w;
        if (!CAUSAL || kt * TROWS <= q0w + 31) {
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            f32x16 s, dp;
#pragma unroll
            for (int r = 0; r < 16; r++) s[r] = dp[r] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const bf16x8 a = frag_row(smem, stage + kb * 32 * 128 + fr[ks]);
                s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qfr[ks], s, 0, 0, 0);
            }
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const bf16x8 a = frag_row(smem, stage + TILE + kb * 32 * 128 + fr[ks]);
                dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, dofr[ks], dp, 0, 0, 0);
            }
            bf16x8 dsb[2];
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                f32x8 ds;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[8 * s2 + e], c, -l2));
                    // register r = 8*s2 + e is key kb*32 + 8*(r/4) + 4*hh + r%4 of the tile
                    if (CAUSAL && diag && kt * TROWS + kb * 32 + 8 * (2 * s2 + (e >> 2)) + 4 * hh + (e & 3) > tq) pv = 0.0f;
                    ds[e] = pv * __builtin_fmaf(dp[8 * s2 + e], inv_keep, -dd);
                }
                dsb[s2] = __builtin_convertvector(ds, bf16x8);
            }
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                for (int db = 0; db < 2; db++) {
                    const int base = stage + (kb * 32 + 16 * s2) * 128;
                    const bf16x8 kT = frag_tr(smem, base + ft[db][0], base + ft[db][1]);
                    dqT[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kT, dsb[s2], dqT[db], 0, 0, 0);
                }
        }
        }
        if (kt + 1 < NT) lwrite(stage ^ (2 * TILE));
        __syncthreads();
        stage ^= 2 * TILE;
    }
    uint16_t *dq = dqkv + ((int64_t)bb * T + tq) * ld + h * DH;
#pragma unroll
    for (int db = 0; db < 2; db++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            *(u32x2 *)(dq + db * 32 + 8 * g + 4 * hh) =
                pack4_trunc(dqT[db][4 * g] * scale, dqT[db][4 * g + 1] * scale, dqT[db][4 * g + 2] * scale, dqT[db][4 * g + 3] * scale);
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
    return attention_fast_path(p) ? (uint64_t)p.B * p.H * p.T * 4 : 0;
}

hipError_t attention_bwd(const AttentionBwd &p, hipStream_t st) {
    const Attention &f = p.fwd;
    if (f.B <= 0 || f.T <= 0 || f.H <= 0 || f.dh <= 0) return hipSuccess;
    if (attention_fast_path(f)) {
        if (!p.workspace) return hipErrorInvalidValue;
        const int64_t rows = (int64_t)f.B * f.T * f.H;
        float *D = (float *)p.workspace;
        hipLaunchKernelGGL(attn_bwd_d_k, dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, st, (const uint16_t *)f.y,
                           (const uint16_t *)p.dy, D, rows, f.T, f.H);
        const int nblk = f.T / 128;
        dim3 grid((unsigned)(f.B * f.H * (f.causal ? (nblk + 1) / 2 : nblk))), block(256);
        const float c = f.scale * kLog2e, ik = 1.0f / f.keep;
#define ZK_BWD(K)                                                                                                     \
    hipLaunchKernelGGL(K, grid, block, 0, st, (const uint16_t *)f.qkv, (const uint16_t *)p.dy, f.lse, D, (uint16_t *)p.dqkv, \
                       f.T, f.H, c, f.scale, ik)
        if (f.causal) {
            ZK_BWD(attn_bwd_dkv_k<true>);
            ZK_BWD(attn_bwd_dq_k<true>);
        } else {
            ZK_BWD(attn_bwd_dkv_k<false>);
            ZK_BWD(attn_bwd_dq_k<false>);
        }
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
