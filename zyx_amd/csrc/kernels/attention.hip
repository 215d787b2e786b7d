// Fused attention core of zyx-nn's CausalSelfAttention (zyx-nn/src/causal_self_attention.rs:36-74):
// y = softmax(scale * q.k^T) / keep . v per head (the reference applies no mask; a causal one is optional), reading q, k, v
// in place from the c_attn output qkv[B, T, 3, H, dh] and writing y[B, T, H*dh], i.e. split / reshape /
// transpose(1,2) before and transpose(1,2) / reshape after are index arithmetic. The [T, T] score
// tensors the reference materialises (q.dot(k.t()), softmax, dropout) never leave registers.
//
// attn_fwd_bf16_k (bf16, dh = 64, T % 128 == 0): one workgroup per (batch, head, 128 queries), 4 waves
// of 32 queries. K and V tiles of 64 keys are loaded straight into LDS (global_load_lds), double buffered. Per tile a wave
// computes S^T = K.Q^T (keys x queries) with v_mfma_f32_32x32x16_bf16, so that every lane owns one
// query column: the running max / sum are per-lane scalars, and the exponentiated tile, packed to
// bf16, already has the register layout of the B operand of O^T += V^T.P^T. V^T fragments come from
// the row-major V tile through the transposing ds_read_b64_tr_b16. Keys are visited in a permuted
// order inside each 32-key block (the order the S^T accumulator registers hold them); P and V use
// the same permutation, and a sum over keys does not depend on it.
//
// attn_small_k: any dh <= 256 and T, f32 or bf16 storage, one wave per query, f32 arithmetic with
// the accurate exponential. Serves the shapes the matrix-core kernel does not take.
#include "dtypes.hpp"
#include "kernels.hpp"
#include "wave.hpp"

namespace zk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define ZK_LDS __attribute__((address_space(3)))

constexpr int QB = 128, KB = 64, DH = 64;
constexpr int TILE = KB * DH * 2;   // one K or V tile: 8 KiB
constexpr int STAGE = 2 * TILE;     // K tile then V tile
constexpr int NSTAGE = 2;           // tiles kt+1 and kt+2 are on their way while tile kt is multiplied
constexpr float kLog2e = 1.44269504088896340736f, kLn2 = 0.69314718055994530942f;
constexpr float kBig = 1.8446744e19f; // 2^64: a block's sum of exponentials beyond this moves the query's reference point

// K tile: [key][16-byte chunk ^ ((key >> 1) & 7)], 128-byte rows: ds_read_b128 of 16 consecutive keys
// at one logical chunk touches 16 different slots modulo 256 bytes.
__device__ __forceinline__ int k_slot(int key, int chunk) { return key * 128 + ((chunk ^ ((key >> 1) & 7)) << 4); }
// V tile: [key][64-byte half ^ ((key >> 1) & 1)][...]: the transposing read of 4 consecutive keys x 32 columns
// (four 64-byte pieces) covers all 64 banks once.
__device__ __forceinline__ int v_slot(int key, int chunk) {
    return key * 128 + (((chunk >> 2) ^ ((key >> 1) & 1)) << 6) + ((chunk & 3) << 4);
}

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// 64 lanes x 16 bytes from global memory straight into LDS at `lds` (wave-uniform byte address) + 16 * lane.
// Written as an instruction, not through the compiler's builtin: for the builtin the compiler waits for every such
// load in flight (vmcnt(0)) before the next LDS read that may touch the same array, which stops a wave for a full
// global-memory latency in every tile although the data it waits for belongs to a later tile. Here completion is
// tracked by hand: callers wait with s_waitcnt vmcnt and a workgroup barrier before anybody reads what was loaded.
// The compiler's own vmcnt bookkeeping stays safe: these loads only ever make the counter larger than it assumes.
__device__ __forceinline__ void load16_to_lds(const void *g, ZK_LDS void *lds) {
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(base), "v"(g) : "memory");
}

// CAUSAL: query t sees keys 0..t. A workgroup then stops at the key tile that holds its last query, a wave leaves out
// tiles that lie wholly after its queries, and the tiles the diagonal crosses get -inf where key > query.
// QW: 32-query blocks per wave (the workgroup takes 128 * QW queries). Every K and V fragment a wave reads from LDS
// serves QW matrix instructions: at QW = 1 the LDS port, which all four SIMDs share, carries 16 KiB per 32 x 64 score
// block and is the busiest unit of the kernel; QW = 2 halves that.
template <bool LSE, bool CAUSAL, int QW>
__global__ __launch_bounds__(256, 2) void attn_fwd_bf16_k(const uint16_t *__restrict__ qkv, uint16_t *__restrict__ y,
                                                          float *__restrict__ lse, int T, int H, float c, float out_scale) {
    constexpr int WQ = 32 * QW, QBW = QB * QW; // queries per wave and per workgroup
    __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[NSTAGE * STAGE];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, hh = lane >> 5;

    // Workgroups whose ids are congruent mod 8 share an XCD (and its L2): give every XCD whole heads, so
    // the K and V of a head are fetched into one L2 only.
    const int QT = T / QBW, BH = (int)gridDim.x / QT; // QT blocks of the grid per head
    int bh, qt;
    if (CAUSAL) {
        // causal work grows with the query block: the blocks with the most key tiles come first in the grid, so that
        // short workgroups fill in behind long ones (ids congruent mod 8 still share a head's XCD when the number of
        // heads is a multiple of 8)
        bh = blockIdx.x % BH;
        qt = QT - 1 - blockIdx.x / BH;
    } else if (BH % 8 == 0) {
        const int x = blockIdx.x & 7, i = blockIdx.x >> 3;
        bh = (i / QT) * 8 + x;
        qt = i % QT;
    } else {
        bh = blockIdx.x / QT;
        qt = blockIdx.x % QT;
    }
    {
    const int bb = bh / H, h = bh % H;
    const int64_t ld = 3 * (int64_t)H * DH;
    const uint16_t *qp = qkv + (int64_t)bb * T * ld + h * DH, *kp = qp + H * DH, *vp = kp + H * DH;
    const int q0w = qt * QBW + wave * WQ; // first query of this wave
    const int tq0 = q0w + (lane & 31);    // this lane's query in block 0; block b: + 32 b

    bf16x8 qf[QW][4]; // B operand of S^T: lane -> query lane % 32, dh = ks*16 + (lane / 32)*8 .. +7
#pragma unroll
    for (int b = 0; b < QW; b++)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) qf[b][ks] = *(const bf16x8 *)(qp + (int64_t)(tq0 + 32 * b) * ld + ks * 16 + hh * 8);

    // staging: direct global -> LDS loads (a wave-load lays 64 x 16 bytes down contiguously: 8 tile rows). The
    // swizzle is applied on the source side: lane l fetches the chunk that belongs at row l/8, physical slot l%8.
    // Wave w issues loads i = 0, 1 of each tile: rows i*32 + w*8 .. +7. No staging registers, no ds_write.
    uint32_t gk[2], gv[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int key = i * 32 + wave * 8 + (lane >> 3), slot = lane & 7;
        const int ck = slot ^ ((key >> 1) & 7);                                   // inverse of k_slot
        const int cv = ((((slot >> 2) ^ ((key >> 1) & 1)) << 2) | (slot & 3));   // inverse of v_slot
        gk[i] = (uint32_t)(key * ld + ck * 8) * 2;
        gv[i] = (uint32_t)(key * ld + cv * 8) * 2;
    }
    auto stage_tile = [&](int kt, int stage) {
        const int64_t base = (int64_t)kt * KB * ld * 2;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int rows = (i * 32 + wave * 8) * 128;
            load16_to_lds((const uint8_t *)kp + base + gk[i], (ZK_LDS void *)(smem + stage + rows));
            load16_to_lds((const uint8_t *)vp + base + gv[i], (ZK_LDS void *)(smem + stage + TILE + rows));
        }
    };

    // fragment offsets inside a stage
    const int kf = (lane & 31) * 128; // + ((chunk ^ key7) << 4), key7 of row lane%32 (+32 leaves it unchanged)
    const int key7 = ((lane & 31) >> 1) & 7;
    int vf[2];
    {
        const int g16 = lane >> 4, r = lane & 15, kr = r >> 2;
#pragma unroll
        for (int db = 0; db < 2; db++)
            vf[db] = TILE + (4 * (g16 >> 1) + kr) * 128 + ((db ^ ((kr >> 1) & 1)) << 6) + ((g16 & 1) * 16 + (r & 3) * 4) * 2;
    }

    f32x16 o[QW][2];
    float m[QW], l[QW];
#pragma unroll
    for (int b = 0; b < QW; b++) {
        m[b] = -INFINITY;
        l[b] = 0.0f;
#pragma unroll
        for (int db = 0; db < 2; db++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[b][db][r] = 0.0f;
    }

    const int NT = CAUSAL ? (qt + 1) * (QBW / KB) : T / KB;
    // A stage_tile is 4 loads per wave; they complete in order, so "at most 4 outstanding" means every tile but the
    // newest has landed. Tiles kt+1 .. kt+NSTAGE-1 are in flight or landed while tile kt is multiplied.
    stage_tile(0, 0);
    if (NSTAGE > 2 && NT > 1) {
        stage_tile(1, STAGE);
        __builtin_amdgcn_s_waitcnt(0x0f74); // vmcnt(4): this wave's part of tile 0 has landed in LDS
    } else {
        __builtin_amdgcn_s_waitcnt(0x0f70);
    }
    __syncthreads();
    int stage = 0, fill = (NSTAGE - 1) * STAGE; // stage of tile kt; the stage last read before the previous barrier
    for (int kt = 0; kt < NT; kt++) {
        if (kt + NSTAGE - 1 < NT) stage_tile(kt + NSTAGE - 1, fill);

        if (!CAUSAL || kt * KB <= q0w + WQ - 1) {
        // causal: the second 32-key block of the tile on the diagonal lies wholly after this wave's queries
        const bool second_live = !CAUSAL || kt * KB + 32 <= q0w + WQ - 1; // uniform over the wave
        f32x16 s[QW][2];
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            if (kb == 1 && !second_live) break;
#pragma unroll
            for (int b = 0; b < QW; b++)
#pragma unroll
                for (int r = 0; r < 16; r++) s[b][kb][r] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const bf16x8 a = *(const ZK_LDS bf16x8 *)(smem + stage + kb * 32 * 128 + kf + (((ks * 2 + hh) ^ key7) << 4));
#pragma unroll
                for (int b = 0; b < QW; b++) s[b][kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[b][ks], s[b][kb], 0, 0, 0);
            }
        }

        if (CAUSAL) {
#pragma unroll
            for (int b = 0; b < QW; b++)
                if (kt * KB + KB - 1 > q0w + 32 * b) { // register r of block kb is key kb*32 + 8*(r/4) + 4*hh + r%4 of the tile
#pragma unroll
                    for (int kb = 0; kb < 2; kb++) {
                        if (kb == 1 && !second_live) break;
#pragma unroll
                        for (int r = 0; r < 16; r++)
                            if (kt * KB + kb * 32 + 8 * (r >> 2) + 4 * hh + (r & 3) > tq0 + 32 * b) s[b][kb][r] = -INFINITY;
                    }
                }
        }
#pragma unroll
        for (int kb = 0; kb < 2; kb++) { // exponentiate one 32-key block, feed it to the matrix pipe, then the next
            if (kb == 1 && !second_live) break;
            // The exponentials are taken against the reference point m the query already has, and checked afterwards:
            // f32 sums and bf16 products carry 2^60 at the same relative precision as 1, so m only has to move when a
            // block's sum leaves that range (or is not a number: the first block of a query, whose m is -inf). Only then
            // is the block's maximum computed, the accumulators rescaled and the block exponentiated again; a query
            // usually sets m once, from the first block it sees, instead of computing a maximum for every block.
            float lt[QW];
            f32x8 p[QW][2];
            auto exponentiate = [&]() {
#pragma unroll
                for (int b = 0; b < QW; b++) {
                    lt[b] = 0.0f;
#pragma unroll
                    for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                        for (int e = 0; e < 8; e++) {
                            p[b][s2][e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[b][kb][8 * s2 + e], c, -m[b]));
                            lt[b] += p[b][s2][e];
                        }
                }
            };
            exponentiate();
            bool redo = false;
#pragma unroll
            for (int b = 0; b < QW; b++) redo |= !(lt[b] < kBig);
            if (__builtin_amdgcn_ballot_w64(redo) != 0) {
#pragma unroll
                for (int b = 0; b < QW; b++) {
                    float bm = s[b][kb][0];
#pragma unroll
                    for (int r = 1; r < 16; r++) bm = fmaxf(bm, s[b][kb][r]);
                    bm = fmaxf(bm, xor32(bm));
                    // a block that lies wholly after its queries (causal) has bm = -inf and changes nothing
                    const float m_new = fmaxf(m[b], bm * c);
                    const float alpha = m[b] == m_new ? 1.0f : __builtin_amdgcn_exp2f(m[b] - m_new);
#pragma unroll
                    for (int db = 0; db < 2; db++)
#pragma unroll
                        for (int r = 0; r < 16; r++) o[b][db][r] *= alpha;
                    l[b] *= alpha;
                    m[b] = m_new;
                }
                exponentiate();
            }
            bf16x8 pf[QW][2];
#pragma unroll
            for (int b = 0; b < QW; b++) {
                l[b] += lt[b];
#pragma unroll
                for (int s2 = 0; s2 < 2; s2++) pf[b][s2] = __builtin_convertvector(p[b][s2], bf16x8);
            }
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
                for (int db = 0; db < 2; db++) {
                    const int off = stage + vf[db] + (kb * 32 + 16 * s2) * 128;
                    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)(smem + off));
                    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)(smem + off + 8 * 128));
                    const bf16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                    for (int b = 0; b < QW; b++) o[b][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[b][s2], o[b][db], 0, 0, 0);
                }
        }
        }

        if (NSTAGE > 2 && kt + 2 < NT) __builtin_amdgcn_s_waitcnt(0x0f74); // this wave's loads of tile kt+1 have landed, kt+2 may be in flight
        else __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        fill = stage;
        stage = stage + STAGE == NSTAGE * STAGE ? 0 : stage + STAGE;
    }

#pragma unroll
    for (int b = 0; b < QW; b++) {
        const int tq = tq0 + 32 * b;
        const float lt = l[b] + xor32(l[b]);
        const float inv = out_scale / lt;
        uint16_t *yp = y + ((int64_t)bb * T + tq) * ((int64_t)H * DH) + h * DH;
#pragma unroll
        for (int db = 0; db < 2; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                uint32_t w0 = (uint32_t)f32_to_bf16_trunc(o[b][db][4 * g + 0] * inv) | ((uint32_t)f32_to_bf16_trunc(o[b][db][4 * g + 1] * inv) << 16);
                uint32_t w1 = (uint32_t)f32_to_bf16_trunc(o[b][db][4 * g + 2] * inv) | ((uint32_t)f32_to_bf16_trunc(o[b][db][4 * g + 3] * inv) << 16);
                u32x2 w = {w0, w1};
                *(u32x2 *)(yp + db * 32 + 8 * g + 4 * hh) = w;
            }
        if (LSE && hh == 0) lse[(int64_t)bh * T + tq] = (m[b] + __builtin_amdgcn_logf(lt)) * kLn2;
    }
    }
}

// One wave per query. Keys are taken 64 at a time (lane = key) for the scores and the
// exponentials, then lane = d for the weighted sum of V rows; p[] and q[] live in LDS.
template <int DT>
__global__ __launch_bounds__(64) void attn_small_k(const void *__restrict__ qkv_, void *__restrict__ y_, float *__restrict__ lse,
                                                   int T, int H, int dh, float scale, float keep, int causal) {
    __shared__ float qs[256], ps[64];
    const int lane = threadIdx.x, t = blockIdx.x, bh = blockIdx.y, bb = bh / H, h = bh % H;
    const int64_t C = (int64_t)H * dh, ld = 3 * C;
    auto ldv = [&](int64_t i) -> float {
        if (DT == DT_F32) return ((const float *)qkv_)[i];
        return bf16_to_f32(((const uint16_t *)qkv_)[i]);
    };
    const int64_t qo = ((int64_t)bb * T + t) * ld + h * dh;
    for (int d = lane; d < dh; d += 64) qs[d] = ldv(qo + d);
    __syncthreads();
    float o[4] = {0.0f, 0.0f, 0.0f, 0.0f}; // d = lane + 64*i
    float m = -INFINITY, l = 0.0f;
    const int Tk = causal ? t + 1 : T; // keys this query sees
    for (int j0 = 0; j0 < Tk; j0 += 64) {
        const int j = j0 + lane;
        float s = -INFINITY;
        if (j < Tk) {
            const int64_t ko = ((int64_t)bb * T + j) * ld + C + h * dh;
            float a = 0.0f;
            for (int d = 0; d < dh; d++) a = __builtin_fmaf(qs[d], ldv(ko + d), a);
            s = a * scale;
        }
        const float m_new = fmaxf(m, wave_allreduce_f32(s, OpMaxF()));
        const float p = j < Tk ? exp_neg(s - m_new) : 0.0f;
        const float alpha = m == -INFINITY ? 0.0f : exp_neg(m - m_new);
        l = l * alpha + wave_allreduce_f32(p, OpAdd());
        m = m_new;
        __syncthreads(); // ps of the previous chunk has been consumed
        ps[lane] = p;
        __syncthreads();
        const int nk = min(64, Tk - j0);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int d = lane + 64 * i;
            if (d < dh) {
                float a = o[i] * alpha;
                const int64_t vo = ((int64_t)bb * T + j0) * ld + 2 * C + h * dh + d;
                for (int jj = 0; jj < nk; jj++) a = __builtin_fmaf(ps[jj], ldv(vo + jj * ld), a);
                o[i] = a;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int d = lane + 64 * i;
        if (d < dh) {
            const float v = (o[i] / l) / keep;
            const int64_t yo = ((int64_t)bb * T + t) * C + h * dh + d;
            if (DT == DT_F32) ((float *)y_)[yo] = v;
            else ((uint16_t *)y_)[yo] = f32_to_bf16_trunc(v);
        }
    }
    if (lse && lane == 0) lse[(int64_t)bh * T + t] = m + logf(l);
}

} // namespace

bool attention_fast_path(const Attention &p) {
    return p.dtype == DT_BF16 && p.dh == DH && p.T % QB == 0 && p.T > 0 && p.scale > 0.0f &&
           (int64_t)p.B * p.H * (p.T / QB) < (1ll << 31) && (int64_t)p.T * 3 * p.H * DH * 2 < (1ll << 31);
}

hipError_t attention_fwd(const Attention &p, hipStream_t st) {
    if (p.B <= 0 || p.T <= 0 || p.H <= 0 || p.dh <= 0) return hipSuccess;
    if (attention_fast_path(p)) {
        // 64 queries per wave where the sequence divides into such workgroups and they still fill the device twice
        const bool wide = !p.causal && p.T % (2 * QB) == 0 && (int64_t)p.B * p.H * (p.T / (2 * QB)) >= 512;
        const int qblocks = p.T / (wide ? 2 * QB : QB);
        dim3 grid((unsigned)(p.B * p.H * qblocks)), block(256);
#define ZK_ATTN(L, CA)                                                                                                \
    do {                                                                                                              \
        if (wide)                                                                                                     \
            hipLaunchKernelGGL((attn_fwd_bf16_k<L, CA, 2>), grid, block, 0, st, (const uint16_t *)p.qkv, (uint16_t *)p.y, p.lse, p.T, \
                               p.H, p.scale * kLog2e, 1.0f / p.keep);                                                 \
        else                                                                                                          \
            hipLaunchKernelGGL((attn_fwd_bf16_k<L, CA, 1>), grid, block, 0, st, (const uint16_t *)p.qkv, (uint16_t *)p.y, p.lse, p.T, \
                               p.H, p.scale * kLog2e, 1.0f / p.keep);                                                 \
    } while (0)
        if (p.lse) {
            if (p.causal) ZK_ATTN(true, true);
            else ZK_ATTN(true, false);
        } else {
            if (p.causal) ZK_ATTN(false, true);
            else ZK_ATTN(false, false);
        }
#undef ZK_ATTN
        return hipGetLastError();
    }
    if (p.dh > 256 || (int64_t)p.B * p.H > 65535 || (p.dtype != DT_F32 && p.dtype != DT_BF16)) return hipErrorInvalidValue;
    dim3 grid((unsigned)p.T, (unsigned)(p.B * p.H)), block(64);
    if (p.dtype == DT_F32)
        hipLaunchKernelGGL(attn_small_k<DT_F32>, grid, block, 0, st, p.qkv, p.y, p.lse, p.T, p.H, p.dh, p.scale, p.keep, p.causal);
    else
        hipLaunchKernelGGL(attn_small_k<DT_BF16>, grid, block, 0, st, p.qkv, p.y, p.lse, p.T, p.H, p.dh, p.scale, p.keep, p.causal);
    return hipGetLastError();
}

} // namespace zk
