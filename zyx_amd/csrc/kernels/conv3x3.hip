// Direct 3 x 3 convolution, bf16 or f32, unit stride, padding 1 (the convolution block of a vision network:
// Tensor::conv, zyx/src/tensor/mod.rs:2583-2680, padding rule zyx/src/kernel/linearize.rs:349-382), on the matrix
// cores without a patch matrix, a padded copy of the input, or a second pass over it; optionally followed by the
// block's 2 x 2 max-pool (Tensor::max_pool, mod.rs:2706-2741) before anything is written. Described for bf16; the f32
// differences are at the kernel.
//
// A workgroup owns R whole output rows of one image (R * W = 448 pixels = 14 MFMA blocks of 32) and 128 output
// channels. It copies the R + 2 input rows of all C channels into LDS once, channel-innermost ([row][col][C], borders
// zero), so that the nine taps are nine shifted views of the same tile: the input operand of tap (ky, kx) and channel
// block cb for pixel (r, c) is the 16 bytes at [r + ky][c + kx][cb*16 + half*8], one ds_read_b128, whatever the shift
// (the pixel stride is padded by 16 bytes, which spreads the 16 lanes of a read phase over all 64 banks). Every input
// element is fetched once and used 9 * 128 times. The weights are re-laid once per launch by a small kernel as
// [tap][C/16][Cout][16], so the weight operand (32 output channels x 16 input channels of one tap) is 1 KiB of
// consecutive bytes read straight from L1 / L2, two k steps ahead of its use.
//
// 4 waves as 2 (pixel halves) x 2 (channel halves), 2 x 7 accumulator tiles of 32 x 32 each = 224 registers, which start
// at the bias. In a tile a lane owns one output channel and 16 pixels in runs of four. The epilogue stages the finished
// tile in LDS (the input tile is dead by then) as [channel][pixel], 8 or 16 bytes per write, and copies it out in 16-byte
// pieces, 896 (bf16) or 1792 (f32) consecutive bytes per channel row of NCHW: the memory pipeline takes one vector
// instruction in about 16 cycles whatever its width, so narrow stores straight from the accumulators cost more than
// the matrix loop.
#include <algorithm>

#include "dtypes.hpp"
#include "kernels.hpp"

namespace zk {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define ZK_LDS __attribute__((address_space(3)))

constexpr int PB = 7;                 // 32-pixel blocks per wave
constexpr int TILE_PIX = 2 * PB * 32; // 448 pixels per workgroup
constexpr int TILE_CO = 128;          // output channels per workgroup
constexpr int STAGE_BYTES = 128 * (TILE_PIX * 2 + 16); // the epilogue's [channel][pixel] copy of the tile (bf16: 128 rows, f32: 64 rows twice)

// w[Cout][C][3][3] -> wt[tap][C/G][Cout][G], G = 16 (bf16) or 8 (f32) channels = the 32 bytes per output channel that one
// k step reads. One thread per (cout, cin): the nine taps of a pair are consecutive, and the G threads of a channel
// block write 32 consecutive bytes of each tap's slice.
template <typename T, int LOG_G>
__global__ __launch_bounds__(256) void conv3x3_weights_k(const T *__restrict__ w, T *__restrict__ wt, int C, int Cout) {
    const int i = blockIdx.x * 256 + threadIdx.x; // = co * C + c
    if (i >= C * Cout) return;
    const int co = i / C, c = i - co * C, cb = c >> LOG_G, ci = c & ((1 << LOG_G) - 1);
    T v[9];
#pragma unroll
    for (int t = 0; t < 9; t++) v[t] = w[(int64_t)i * 9 + t];
#pragma unroll
    for (int t = 0; t < 9; t++) wt[((((int64_t)t * (C >> LOG_G) + cb) * Cout + co) << LOG_G) + ci] = v[t];
}

// floor(q / d) for 0 <= q < 2^22, inv = 1.0f / d: the rounding errors of the reciprocal and of the product are far
// smaller than the distance 0.5 / d of (q + 0.5) / d from the nearest integer
__device__ __forceinline__ int small_div(int q, float inv) { return (int)(((float)q + 0.5f) * inv); }

// The bf16 input tile: rows rb*R - 1 .. rb*R + R of every channel of image n, channel-innermost in LDS, zero outside
// the image. One item = 8 consecutive columns of two neighbouring channels of one row: two 16-byte reads, eight 4-byte
// LDS writes (channel pair packed). The lanes of a wave take 4 neighbouring items of a row for each of 16 channel pairs
// (8 x 8 when C / 2 is not a multiple of 16): the texture unit takes one cache line per cycle, so neighbouring lanes
// share lines, while the writes of one instruction still spread over 32 banks. U items' reads are in flight together.
template <int U>
__device__ __forceinline__ void load_tile_bf16(ZK_LDS uint8_t *smem, const void *x_, int n, int rb, int R, int C, int H, int W,
                                               int PS, int lane, int wave) {
    // Buffer loads with 32-bit byte offsets from the image's first element (conv3x3_direct_ok bounds an image by
    // 2^32 bytes): no 64-bit address arithmetic, and an item outside the image or past the end of the list gets
    // an offset beyond the buffer, for which the load returns zeros without a branch.
    const int Wp = W + 2;
    const int w8 = W >> 3;
    const int C2 = C >> 1, RC = (R + 2) * w8;          // channel pairs; 8-column pieces of one channel's rows
    const int KB = (C2 & 15) ? 3 : 2;                  // log2(items of a row per wave instruction)
    const int k = lane & ((1 << KB) - 1), cp_lo = lane >> KB, cp_lanes = 64 >> KB;
    const int cpblocks = C2 / cp_lanes, groups = (RC + (1 << KB) - 1) >> KB, wave_items = cpblocks * groups;
    const float inv_w8 = 1.0f / (float)w8, inv_cpb = 1.0f / (float)cpblocks;
    const int plane = H * W;
    const uint32_t image_bytes = (uint32_t)C * (uint32_t)plane * 2u;
    const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const uint16_t *)x_ + (int64_t)n * C * plane), 0, (int)image_bytes, 0x00020000);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    for (int t0 = wave_u; t0 < wave_items; t0 += 4 * U) {
        u32x4 va[U], vb[U];
        int dsto[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int t = t0 + 4 * u;                   // uniform over the wave
            const int g = small_div(t, inv_cpb), cpb = t - g * cpblocks;
            const int rc = (g << KB) + k, cp = cpb * cp_lanes + cp_lo;
            const int r = small_div(rc, inv_w8), ch = rc - __mul24(r, w8);
            const int iy = rb * R - 1 + r;
            const bool live = t < wave_items && rc < RC;
            const bool inside = live && iy >= 0 && iy < H;
            const uint32_t off = (uint32_t)(2 * cp * plane + __mul24(iy, W) + ch * 8) * 2u; // (a plane may exceed 24 bits)
            va[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, (int)(inside ? off : 0xfffffff0u), 0, 0));
            vb[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, (int)(inside ? off + (uint32_t)plane * 2u : 0xfffffff0u), 0, 0));
            dsto[u] = live ? __mul24(__mul24(r, Wp) + 1 + ch * 8, PS) + cp * 4 : -1;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (dsto[u] < 0) continue;
            ZK_LDS uint8_t *dst = smem + dsto[u];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                *(ZK_LDS uint32_t *)(dst + (2 * e) * PS) = __builtin_amdgcn_perm(vb[u][e], va[u][e], 0x05040100u);
                *(ZK_LDS uint32_t *)(dst + (2 * e + 1) * PS) = __builtin_amdgcn_perm(vb[u][e], va[u][e], 0x07060302u);
            }
        }
    }
}

// The staged tile ([channel][pixel], TP pixels = whole rows of the image, RS bytes per channel row; 128 channel rows for
// 16-bit output, 64 per pass for 32-bit) leaves for y in 16-byte pieces, or, POOL, through 2 x 2 windows: a channel's
// pooled tile is TP / 4 values, consecutive in the pooled plane, a thread makes 16 bytes of them; the running maximum
// starts at the dtype's lowest finite value and takes the window in row order, like the separate pooling kernel.
template <int TP, bool OUT_BF16, bool POOL>
__device__ __forceinline__ void copy_out(const ZK_LDS uint8_t *smem, void *__restrict__ y, int n, int Cout, int co0, int H, int W,
                                         int rb, int pass, int tid) {
    constexpr int ES = OUT_BF16 ? 2 : 4;
    constexpr int RS = TP * ES + 16;
    constexpr int CPR = TP * ES / 16;
    constexpr int ROWS = OUT_BF16 ? 128 : 64;
    const int64_t plane = (int64_t)H * W;
    if constexpr (POOL) {
        constexpr int PV = TP / 4, VPC = 16 / ES, PCR = PV / VPC;
        const int W2 = W >> 1;
        const float inv_w2 = 1.0f / (float)W2;
        const float lowest = OUT_BF16 ? -3.3895313892515355e38f : -3.4028234663852886e38f;
        const int64_t pplane = plane >> 2;
        uint8_t *ptile = (uint8_t *)y + (((int64_t)n * Cout + co0) * pplane + (int64_t)rb * PV) * ES;
        for (int idx = tid; idx < ROWS * PCR; idx += 256) {
            const int row = idx / PCR, piece = idx - row * PCR;
            const int co = OUT_BF16 ? row : (row >> 5) * 64 + pass * 32 + (row & 31);
            float m[VPC];
            int pr = small_div(piece * VPC, inv_w2), pc = piece * VPC - __mul24(pr, W2); // pooled row, column of value 0
            const ZK_LDS uint8_t *rowp = smem + row * RS + __mul24(2 * pr, W) * ES;
#pragma unroll
            for (int e = 0; e < VPC; e++) {
                const ZK_LDS uint8_t *src = rowp + 2 * pc * ES;
                if (++pc == W2) { // the next value starts the next pooled row
                    pc = 0;
                    rowp += 2 * W * ES;
                }
                float a0, a1, b0, b1;
                if (OUT_BF16) {
                    const uint32_t u0 = *(const ZK_LDS uint32_t *)src, u1 = *(const ZK_LDS uint32_t *)(src + W * ES);
                    a0 = __uint_as_float(u0 << 16), a1 = __uint_as_float(u0 & 0xffff0000u);
                    b0 = __uint_as_float(u1 << 16), b1 = __uint_as_float(u1 & 0xffff0000u);
                } else {
                    const u32x2 u0 = *(const ZK_LDS u32x2 *)src, u1 = *(const ZK_LDS u32x2 *)(src + W * ES);
                    a0 = __uint_as_float(u0[0]), a1 = __uint_as_float(u0[1]), b0 = __uint_as_float(u1[0]), b1 = __uint_as_float(u1[1]);
                }
                m[e] = fmaxf(b1, fmaxf(b0, fmaxf(a1, fmaxf(a0, lowest))));
            }
            u32x4 v;
            if (OUT_BF16) {
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = __builtin_amdgcn_perm(__float_as_uint(m[(2 * e + 1) % VPC]), __float_as_uint(m[(2 * e) % VPC]), 0x07060302u);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = __float_as_uint(m[e % VPC]);
            }
            __builtin_nontemporal_store(v, (u32x4 *)(ptile + (int64_t)co * pplane * ES + piece * 16)); // written once
        }
    } else {
        // the tile's pixels are consecutive in the image plane
        uint8_t *ytile = (uint8_t *)y + (((int64_t)n * Cout + co0) * plane + (int64_t)rb * TP) * ES;
#pragma unroll 4
        for (int idx = tid; idx < ROWS * CPR; idx += 256) {
            const int row = idx / CPR, col = idx - row * CPR;
            const int co = OUT_BF16 ? row : (row >> 5) * 64 + pass * 32 + (row & 31);
            const u32x4 v = *(const ZK_LDS u32x4 *)(smem + row * RS + col * 16);
            __builtin_nontemporal_store(v, (u32x4 *)(ytile + (int64_t)co * plane * ES + col * 16)); // written once
        }
    }
}

// F32_IN: f32 input, weights, bias and output on v_mfma_f32_32x32x2_f32 (a k step is 8 channels of one tap: lane half h
// holds channels 4h .. 4h + 3 of the block, and the j-th of four matrix instructions multiplies channels j and 4 + j);
// otherwise bf16 input on v_mfma_f32_32x32x16_bf16 (a k step is 16 channels of one tap). POOL: the tile leaves through a
// 2 x 2 / stride 2 max-pool (its rows are whole and even in number, so every window lies inside it): y is
// [N, Cout, H / 2, W / 2] and the full-size result never reaches memory.
template <bool F32_IN, bool OUT_BF16, bool RELU, bool POOL>
__global__ __launch_bounds__(256, 1) void conv3x3_k(const void *__restrict__ x_, const void *__restrict__ wt,
                                                    const void *__restrict__ bias, void *__restrict__ y, int C, int H, int W,
                                                    int Cout, int R) {
    static_assert(!(F32_IN && OUT_BF16), "f32 input gives f32 output");
    constexpr int ES_IN = F32_IN ? 4 : 2;
    // A workgroup is alone on its compute unit, one wave per SIMD: nothing hides instruction issue outside the matrix
    // loop, so every phase below is written for a small instruction count (no integer division, no per-element branch).
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const int wm = wave >> 1, wn = wave & 1;
    const int tiles_per_image = H / R;
    const int n = blockIdx.x / tiles_per_image, rb = blockIdx.x - n * tiles_per_image;
    const int co0 = blockIdx.y * TILE_CO;
    const int PS = C * ES_IN + 16;        // bytes between neighbouring pixels in LDS
    const int Wp = W + 2;

    // ---- input tile: rows rb*R - 1 .. rb*R + R of every channel, channel-innermost, zero outside the image ----------
    // One item = 8 consecutive columns of two neighbouring channels of one row: two 16-byte reads, eight 4-byte LDS
    // writes (channel pair packed). The lanes of a wave take 4 neighbouring items of a row for each of 16 channel pairs
    // (8 x 8 when C / 2 is not a multiple of 16): the texture unit takes one cache line per cycle, so neighbouring
    // lanes share lines, while the writes of one instruction still spread over 32 banks (pixels 8 apart are 32 banks
    // apart, 16 channel pairs are 16 consecutive words).
    if constexpr (!F32_IN) {
        load_tile_bf16<9>(smem, x_, n, rb, R, C, H, W, PS, lane, wave);
    } else {
        // f32: one item = 4 consecutive columns of one channel (16 bytes), four 4-byte LDS writes; the lanes of a wave take
        // 4 neighbouring items of a row for each of 16 channels (writes: pixels 4 apart are 16 banks apart for C = 64).
        // (buffer loads with 32-bit byte offsets within the image, as in load_tile_bf16)
        constexpr int U = 12;
        const int w4 = W >> 2, RC = (R + 2) * w4;
        const int k = lane & 3, c_lo = lane >> 2;
        const int cblocks16 = C >> 4, groups = (RC + 3) >> 2, wave_items = cblocks16 * groups;
        const float inv_w4 = 1.0f / (float)w4, inv_cb16 = 1.0f / (float)cblocks16;
        const int plane = H * W;
        const __amdgpu_buffer_rsrc_t xr = __builtin_amdgcn_make_buffer_rsrc(
            (void *)((const float *)x_ + (int64_t)n * C * plane), 0, (int)((uint32_t)C * (uint32_t)plane * 4u), 0x00020000);
        const int wave_u = __builtin_amdgcn_readfirstlane(wave);
        for (int t0 = wave_u; t0 < wave_items; t0 += 4 * U) {
            u32x4 v[U];
            int dsto[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int t = t0 + 4 * u;                   // uniform over the wave
                const int g = small_div(t, inv_cb16), cbk = t - g * cblocks16;
                const int rc = (g << 2) + k, c = cbk * 16 + c_lo;
                const int r = small_div(rc, inv_w4), pc = rc - __mul24(r, w4);
                const int iy = rb * R - 1 + r;
                const bool live = t < wave_items && rc < RC;
                const uint32_t off = (uint32_t)(c * plane + __mul24(iy, W) + pc * 4) * 4u; // (a plane may exceed 24 bits)
                v[u] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(xr, (int)(live && iy >= 0 && iy < H ? off : 0xfffffff0u), 0, 0));
                dsto[u] = live ? __mul24(__mul24(r, Wp) + 1 + pc * 4, PS) + c * 4 : -1;
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (dsto[u] < 0) continue;
                ZK_LDS uint8_t *dst = smem + dsto[u];
#pragma unroll
                for (int e = 0; e < 4; e++) *(ZK_LDS uint32_t *)(dst + e * PS) = v[u][e];
            }
        }
    }
    {
        const int parts = C * ES_IN / 16, edge = (R + 2) * 2 * parts; // columns 0 and W + 1 of every row, 16 bytes at a time
        for (int q = tid; q < edge; q += 256) {
            const int part = q % parts, side = (q / parts) & 1, r = q / parts / 2;
            *(ZK_LDS u32x4 *)(smem + (r * Wp + (side ? W + 1 : 0)) * PS + part * 16) = u32x4{0u, 0u, 0u, 0u};
        }
    }

    // per-lane byte offsets of this wave's pixels (tap 0, channel block 0) and of its weight rows
    int xoff[PB];
    {
        const float inv_w = 1.0f / (float)W;
#pragma unroll
        for (int pb = 0; pb < PB; pb++) {
            const int p = wm * (PB * 32) + pb * 32 + l32, pr = small_div(p, inv_w), pc = p - __mul24(pr, W);
            xoff[pb] = __mul24(__mul24(pr, Wp) + pc, PS) + half * 16;
        }
    }
    const int cblocks = F32_IN ? C >> 3 : C >> 4; // k steps per tap
    // weight fragment of (tap, cb, nb): 16 bytes at ((tap * cblocks + cb) * Cout + co) * 32 + half * 16
    const uint8_t *wlane = (const uint8_t *)wt + ((int64_t)(co0 + wn * 64 + l32)) * 32 + half * 16;
    const int64_t wstep = (int64_t)Cout * 32; // bytes between (tap, cb) slices

    f32x16 acc[2][PB]; // [nb][pb]: rows = pixels, columns = output channels; lane l owns channel l % 32 of block nb
#pragma unroll
    for (int nb = 0; nb < 2; nb++) {
        const int co = co0 + wn * 64 + nb * 32 + l32;
        const float bv = !bias ? 0.0f : F32_IN ? ((const float *)bias)[co] : bf16_to_f32(((const uint16_t *)bias)[co]);
#pragma unroll
        for (int pb = 0; pb < PB; pb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[nb][pb][r] = bv;
    }

    // k step s: tap = s / cblocks, cb = s % cblocks (the order of wt's slices). The weights of a step are requested two
    // steps before their use and the input fragments one step before, each into one of three register sets (the step
    // count 9 * cblocks is a multiple of three), so that a step's matrix instructions never wait for what they read.
    const int steps = 9 * cblocks;
    int tap = 0, cb = 0;
    auto next_toff = [&]() { // tile offset of the next step's tap and channel block (the last step's again past the end)
        const int tp = tap < 9 ? tap : 8, cc = tap < 9 ? cb : cblocks - 1;
        const int ky = tp / 3, kx = tp - ky * 3;
        if (++cb == cblocks) {
            cb = 0;
            tap++;
        }
        return (ky * Wp + kx) * PS + cc * 32;
    };
    auto load_w = [&](u32x4(&wf)[2], int s) {
        const uint8_t *src = wlane + (s < steps ? s : steps - 1) * wstep;
        wf[0] = *(const u32x4 *)src;
        wf[1] = *(const u32x4 *)(src + 32 * 32);
    };
    auto k_step = [&](const u32x4(&wf)[2], const u32x4(&xf)[PB], u32x4(&xnext)[PB]) {
        const int toff = next_toff();
#pragma unroll
        for (int pb = 0; pb < PB; pb++) xnext[pb] = *(const ZK_LDS u32x4 *)(smem + xoff[pb] + toff);
        if constexpr (F32_IN) {
#pragma unroll
            for (int j = 0; j < 4; j++) // j outermost: 14 independent instructions between two on the same accumulator
#pragma unroll
                for (int pb = 0; pb < PB; pb++)
#pragma unroll
                    for (int nb = 0; nb < 2; nb++)
                        acc[nb][pb] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(xf[pb][j]), __uint_as_float(wf[nb][j]), acc[nb][pb], 0, 0, 0);
        } else {
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
#pragma unroll
                for (int nb = 0; nb < 2; nb++)
                    acc[nb][pb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, xf[pb]), __builtin_bit_cast(bf16x8, wf[nb]), acc[nb][pb], 0, 0, 0);
        }
        // issue order: one LDS read of the next step, then this step's share of matrix instructions, seven times
#pragma unroll
        for (int pb = 0; pb < PB; pb++) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, F32_IN ? 8 : 2, 0);
        }
    };
    u32x4 w0[2], w1[2], w2[2], xa[PB], xb[PB], xc[PB];
    load_w(w0, 0);
    load_w(w1, 1);
    __syncthreads(); // the tile is complete
    {
        const int toff = next_toff();
#pragma unroll
        for (int pb = 0; pb < PB; pb++) xa[pb] = *(const ZK_LDS u32x4 *)(smem + xoff[pb] + toff);
    }
    for (int s = 0; s < steps; s += 3) { // the barriers keep the scheduler from sinking a request towards its use
        load_w(w2, s + 2);
        __builtin_amdgcn_sched_barrier(0);
        k_step(w0, xa, xb);
        load_w(w0, s + 3);
        __builtin_amdgcn_sched_barrier(0);
        k_step(w1, xb, xc);
        load_w(w1, s + 4);
        __builtin_amdgcn_sched_barrier(0);
        k_step(w2, xc, xa);
    }

    // ---- epilogue: register r of lane l is pixel 8*(r/4) + 4*(l/32) + r%4 of block pb, channel l%32 of block nb --------
    constexpr int ES = OUT_BF16 ? 2 : 4;          // bytes per output element
    constexpr int RS = TILE_PIX * ES + 16;        // bytes per staged channel row
    constexpr int PASSES = OUT_BF16 ? 1 : 2;      // f32: one channel block (nb) per pass, 64 rows each
    __syncthreads(); // every wave has read its last input fragment
#pragma unroll
    for (int pass = 0; pass < PASSES; pass++) {
        if (pass) __syncthreads(); // the previous pass has been copied out
#pragma unroll
        for (int nb = 0; nb < 2; nb++) {
            if (!OUT_BF16 && nb != pass) continue;
            const int row = OUT_BF16 ? wn * 64 + nb * 32 + l32 : wn * 32 + l32;
            ZK_LDS uint8_t *dst = smem + row * RS + (wm * (PB * 32) + 4 * half) * ES;
#pragma unroll
            for (int pb = 0; pb < PB; pb++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        v[e] = acc[nb][pb][g * 4 + e];
                        asm volatile("" : "+v"(v[e])); // a copy in a vector register, here: the accumulators stay where they are
                        if (RELU) v[e] = (v[e] > 0.0f ? 1.0f : 0.0f) * v[e];
                    }
                    ZK_LDS uint8_t *d = dst + (pb * 32 + g * 8) * ES;
                    if (OUT_BF16) {
                        // truncation to bf16 = the upper halves of the four words
                        u32x2 pk = {__builtin_amdgcn_perm(__float_as_uint(v[1]), __float_as_uint(v[0]), 0x07060302u),
                                    __builtin_amdgcn_perm(__float_as_uint(v[3]), __float_as_uint(v[2]), 0x07060302u)};
                        *(ZK_LDS u32x2 *)d = pk;
                    } else {
                        *(ZK_LDS u32x4 *)d = u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])};
                    }
                    __builtin_amdgcn_sched_barrier(0); // or the scheduler reads all 224 accumulators first and spills
                }
        }
        __syncthreads();
        copy_out<TILE_PIX, OUT_BF16, POOL>(smem, y, n, Cout, co0, H, W, rb, pass, tid);
    }
}

// The same convolution for bf16 input with half the tile, two workgroups to a compute unit: a workgroup's phases
// (fetch the tile, matrix loop, copy out) do not overlap one another, so a second resident workgroup fills the matrix
// pipeline while the first one waits for memory. R * W = 224 pixels x 128 output channels; 4 waves as 2 pixel halves x 2
// channel halves on v_mfma_f32_16x16x32_bf16: 7 pixel blocks x 4 channel blocks of 16 x 16 per wave = 112 accumulator
// registers, and one LDS read still feeds four matrix instructions of 16 cycles (the ratio of the large tile). A k step
// is 32 channels of one tap (C % 32 = 0): lane l holds pixel (or channel) l % 16 and channels 8 * (l / 16) .. + 7 of
// the step; weights re-laid as [tap][C / 32][Cout][32]. Register r of lane l of a block is pixel 4 * (l / 16) + r,
// channel l % 16.
constexpr int SPB = 7;                     // 16-pixel blocks per wave
constexpr int S_TILE_PIX = 2 * SPB * 16;   // 224
constexpr int S_STAGE_BYTES = 128 * (S_TILE_PIX * 2 + 16);
typedef float f32x4a __attribute__((ext_vector_type(4)));

template <bool OUT_BF16, bool RELU, bool POOL, int CB>
__global__ __launch_bounds__(256, 2) void conv3x3_half_k(const void *__restrict__ x_, const void *__restrict__ wt,
                                                         const void *__restrict__ bias, void *__restrict__ y, int C, int H, int W,
                                                         int Cout, int R) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem_raw[];
    ZK_LDS uint8_t *smem = (ZK_LDS uint8_t *)smem_raw;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, quad = lane >> 4, l16 = lane & 15;
    const int wm = wave >> 1, wn = wave & 1;
    const int tiles_per_image = H / R;
    const int n = blockIdx.x / tiles_per_image, rb = blockIdx.x - n * tiles_per_image;
    const int co0 = blockIdx.y * TILE_CO;
    const int PS = C * 2 + 16;
    const int Wp = W + 2;

    {
        const int parts = C * 2 / 16, edge = (R + 2) * 2 * parts; // columns 0 and W + 1 of every row, 16 bytes at a time
        for (int q = tid; q < edge; q += 256) {
            const int part = q % parts, side = (q / parts) & 1, r = q / parts / 2;
            *(ZK_LDS u32x4 *)(smem + (r * Wp + (side ? W + 1 : 0)) * PS + part * 16) = u32x4{0u, 0u, 0u, 0u};
        }
    }

    int xoff[SPB];
    {
        const float inv_w = 1.0f / (float)W;
#pragma unroll
        for (int pb = 0; pb < SPB; pb++) {
            const int p = wm * (SPB * 16) + pb * 16 + l16, pr = small_div(p, inv_w), pc = p - __mul24(pr, W);
            xoff[pb] = __mul24(__mul24(pr, Wp) + pc, PS) + quad * 16;
        }
    }
    const int cblocks = C >> 5; // k steps per tap
    // weight fragment of (tap, cb, nb): 16 bytes at ((tap * cblocks + cb) * Cout + co) * 64 + quad * 16
    // (buffer loads: a fixed 32-bit lane offset plus a scalar offset that moves with the step, so the loads need no
    // address registers of their own, which the allocator would otherwise recycle from a load still in flight and
    // wait for it)
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const uint8_t *)wt + (int64_t)co0 * 64), 0, (int)((int64_t)9 * C * Cout * 2 - (int64_t)co0 * 64), 0x00020000);
    const int wl = (wn * 64 + l16) * 64 + quad * 16;
    const int wstep = Cout * 64;

    f32x4a acc[4][SPB]; // [nb][pb]
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int co = co0 + wn * 64 + nb * 16 + l16;
        const float bv = !bias ? 0.0f : bf16_to_f32(((const uint16_t *)bias)[co]);
#pragma unroll
        for (int pb = 0; pb < SPB; pb++) acc[nb][pb] = f32x4a{bv, bv, bv, bv};
    }

    // k step s: tap = s / cblocks, cb = s % cblocks. The input fragments of a step are read from LDS during the step
    // before, into the other of two register sets; the weights of a step are requested three steps before their use
    // (an L2 round trip is longer than one step's matrix instructions), the first three before the input tile is
    // fetched. CB > 0: C = 32 * CB and the 9 * CB steps are unrolled, so that the tile and weight offsets of a step
    // are constants of the launch and a step is little more than its matrix instructions, seven LDS reads and four
    // loads (one wave per SIMD issues everything in order: at ~90 instructions per step the matrix pipe waited for
    // the scalar bookkeeping of the looping form, 717 cycles per step against 448 of matrix instructions).
    const int steps = 9 * cblocks;
    auto read_x = [&](u32x4(&xf)[SPB], int toff) {
#pragma unroll
        for (int pb = 0; pb < SPB; pb++) xf[pb] = *(const ZK_LDS u32x4 *)(smem + xoff[pb] + toff);
    };
    auto load_w = [&](u32x4(&wf)[4], int s) { // s < steps, uniform
        const int soff = s * wstep;
#pragma unroll
        for (int nb = 0; nb < 4; nb++) wf[nb] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, wl + nb * 16 * 64, soff, 0));
    };
    auto multiply = [&](const u32x4(&wf)[4], const u32x4(&xf)[SPB]) {
#pragma unroll
        for (int pb = 0; pb < SPB; pb++)
#pragma unroll
            for (int nb = 0; nb < 4; nb++)
                acc[nb][pb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xf[pb]), __builtin_bit_cast(bf16x8, wf[nb]), acc[nb][pb], 0, 0, 0);
#pragma unroll
        for (int pb = 0; pb < SPB; pb++) { // issue order: one LDS read of the next step, four matrix instructions
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        }
    };
    u32x4 wq[4][4], xq[2][SPB];
    load_w(wq[0], 0);
    load_w(wq[1], 1);
    load_w(wq[2], 2);
    load_tile_bf16<6>(smem, x_, n, rb, R, C, H, W, PS, lane, wave);
    __syncthreads(); // the tile is complete
    read_x(xq[0], 0);
    if constexpr (CB > 0) {
        constexpr int STEPS = 9 * CB;
        auto toff_of = [&](int s) { // constant folding leaves a few scalar instructions per step
            const int tp = s / CB, cc = s - tp * CB, ky = tp / 3, kx = tp - ky * 3;
            return (ky * Wp + kx) * PS + cc * 64;
        };
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            if (s + 3 < STEPS) load_w(wq[(s + 3) & 3], s + 3);
            __builtin_amdgcn_sched_barrier(0);
            if (s + 1 < STEPS) read_x(xq[(s + 1) & 1], toff_of(s + 1));
            multiply(wq[s & 3], xq[s & 1]);
        }
    } else {
        int cb = 0, kx = 0, ky = 0, toff = 0; // of the step whose fragments are read next
        auto next_toff = [&]() {
            toff += 64;
            if (++cb == cblocks) {
                cb = 0;
                toff += PS - cblocks * 64;
                if (++kx == 3) {
                    kx = 0;
                    toff += (Wp - 3) * PS;
                    ++ky;
                }
            }
            return ky < 3 ? toff : 0; // past the last step: any address inside the tile
        };
        auto k_step = [&](int s, const u32x4(&wf)[4], const u32x4(&xf)[SPB], u32x4(&xnext)[SPB]) {
            read_x(xnext, next_toff());
            multiply(wf, xf);
        };
        auto ahead = [&](u32x4(&wf)[4], int s) { load_w(wf, s < steps ? s : steps - 1); };
        for (int s = 0; s < steps; s += 4) { // the tests on s are uniform
            ahead(wq[3], s + 3);
            __builtin_amdgcn_sched_barrier(0);
            k_step(s, wq[0], xq[0], xq[1]);
            if (s + 1 < steps) {
                ahead(wq[0], s + 4);
                __builtin_amdgcn_sched_barrier(0);
                k_step(s + 1, wq[1], xq[1], xq[0]);
            }
            if (s + 2 < steps) {
                ahead(wq[1], s + 5);
                __builtin_amdgcn_sched_barrier(0);
                k_step(s + 2, wq[2], xq[0], xq[1]);
            }
            if (s + 3 < steps) {
                ahead(wq[2], s + 6);
                __builtin_amdgcn_sched_barrier(0);
                k_step(s + 3, wq[3], xq[1], xq[0]);
            }
        }
    }

    // ---- epilogue ------------------------------------------------------------------------------------------------
    constexpr int ES = OUT_BF16 ? 2 : 4;
    constexpr int RS = S_TILE_PIX * ES + 16;
    constexpr int PASSES = OUT_BF16 ? 1 : 2; // f32: two channel blocks per pass, 64 rows each
    __syncthreads(); // every wave has read its last input fragment
#pragma unroll
    for (int pass = 0; pass < PASSES; pass++) {
        if (pass) __syncthreads(); // the previous pass has been copied out
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            if (!OUT_BF16 && (nb >> 1) != pass) continue;
            const int row = OUT_BF16 ? wn * 64 + nb * 16 + l16 : wn * 32 + (nb & 1) * 16 + l16;
            ZK_LDS uint8_t *dst = smem + row * RS + (wm * (SPB * 16) + 4 * quad) * ES;
#pragma unroll
            for (int pb = 0; pb < SPB; pb++) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[e] = acc[nb][pb][e];
                    if (RELU) v[e] = (v[e] > 0.0f ? 1.0f : 0.0f) * v[e];
                }
                ZK_LDS uint8_t *d = dst + pb * 16 * ES;
                if (OUT_BF16) {
                    u32x2 pk = {__builtin_amdgcn_perm(__float_as_uint(v[1]), __float_as_uint(v[0]), 0x07060302u),
                                __builtin_amdgcn_perm(__float_as_uint(v[3]), __float_as_uint(v[2]), 0x07060302u)};
                    *(ZK_LDS u32x2 *)d = pk;
                } else {
                    *(ZK_LDS u32x4 *)d = u32x4{__float_as_uint(v[0]), __float_as_uint(v[1]), __float_as_uint(v[2]), __float_as_uint(v[3])};
                }
            }
        }
        __syncthreads();
        copy_out<S_TILE_PIX, OUT_BF16, POOL>(smem, y, n, Cout, co0, H, W, rb, pass, tid);
    }
}

int tile_rows(const Conv2d &p) { return p.W > 0 && TILE_PIX % p.W == 0 ? TILE_PIX / p.W : 0; }
int elem_bytes(const Conv2d &p) { return p.dtype == DT_F32 ? 4 : 2; }
uint64_t lds_bytes(const Conv2d &p) { // the input tile, later reused for the staged output tile
    return std::max<uint64_t>((uint64_t)(tile_rows(p) + 2) * (p.W + 2) * (p.C * elem_bytes(p) + 16), STAGE_BYTES);
}
// the half-tile kernel: bf16, 32-channel k steps, whole rows in 224 pixels, two workgroups within a compute unit's LDS
int half_rows(const Conv2d &p) { return p.W > 0 && S_TILE_PIX % p.W == 0 ? S_TILE_PIX / p.W : 0; }
uint64_t half_lds_bytes(const Conv2d &p) {
    return std::max<uint64_t>((uint64_t)(half_rows(p) + 2) * (p.W + 2) * (p.C * 2 + 16), S_STAGE_BYTES);
}
bool half_ok(const Conv2d &p) {
    const int R = half_rows(p);
    return p.dtype == DT_BF16 && p.C % 32 == 0 && R >= 1 && p.H % R == 0 && !(p.pool && R % 2) && half_lds_bytes(p) <= 80 * 1024 &&
           (int64_t)p.N * (p.H / R) < (1ll << 31);
}
} // namespace

bool conv3x3_direct_ok(const Conv2d &p) { // shape only: the same answer at registration and at every launch
    const bool types = (p.dtype == DT_BF16 && (p.out_dtype == DT_BF16 || p.out_dtype == DT_F32)) || (p.dtype == DT_F32 && p.out_dtype == DT_F32);
    const bool common = types && p.KH == 3 && p.KW == 3 && p.sy == 1 && p.sx == 1 && p.dy == 1 && p.dx == 1 && p.py == 1 && p.px == 1 &&
                        p.C >= 16 && p.C % 16 == 0 && p.Cout % TILE_CO == 0 && p.W % 8 == 0 && p.N > 0 && p.H > 0 && p.Cout / TILE_CO <= 65535 &&
                        (int64_t)p.N * p.C * p.H * p.W < (1ll << 31) && (int64_t)p.N * p.Cout * p.H * p.W < (1ll << 40) &&
                        (int64_t)p.C * p.Cout < (1ll << 26) && p.H < (1 << 22) && // row numbers go through 24-bit multiplies
                        (int64_t)p.C * p.H * p.W * elem_bytes(p) < (1ll << 32); // 32-bit byte offsets within an image
    if (!common) return false;
    // the 448-pixel tile, or the 224-pixel one (bf16, C % 32 = 0): whole rows, an even number of them under a fused pool
    // (pooling windows must not straddle two tiles), the tile within LDS
    const int R = tile_rows(p);
    const bool full = R >= 1 && p.H % R == 0 && !(p.pool && R % 2) && lds_bytes(p) <= 160 * 1024 && (int64_t)p.N * (p.H / R) < (1ll << 31);
    return full || half_ok(p);
}

uint64_t conv3x3_scratch_bytes(const Conv2d &p) { return (uint64_t)9 * p.C * p.Cout * elem_bytes(p); }

hipError_t conv3x3_init() {
    // the input tile is larger than the default per-workgroup LDS limit
    hipError_t e = hipSuccess;
#define ZK_V(FI, OB) (const void *)conv3x3_k<FI, OB, false, false>, (const void *)conv3x3_k<FI, OB, true, false>, \
                     (const void *)conv3x3_k<FI, OB, false, true>, (const void *)conv3x3_k<FI, OB, true, true>
    const void *variants[12] = {ZK_V(false, false), ZK_V(false, true), ZK_V(true, false)};
#undef ZK_V
    for (const void *f : variants)
        if (e == hipSuccess) e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
#define ZK_V(OB, CB) (const void *)conv3x3_half_k<OB, false, false, CB>, (const void *)conv3x3_half_k<OB, true, false, CB>, \
                     (const void *)conv3x3_half_k<OB, false, true, CB>, (const void *)conv3x3_half_k<OB, true, true, CB>
    const void *halves[24] = {ZK_V(false, 0), ZK_V(true, 0), ZK_V(false, 2), ZK_V(true, 2), ZK_V(false, 4), ZK_V(true, 4)};
#undef ZK_V
    for (const void *f : halves)
        if (e == hipSuccess) e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 80 * 1024);
    return e;
}

// `wt` holds conv3x3_scratch_bytes(p) bytes for the re-laid weights.
hipError_t conv3x3_direct(const Conv2d &p, void *wt, hipStream_t st) {
    if ((uintptr_t)p.x % 16 || (uintptr_t)p.y % 16 || (uintptr_t)wt % 16) return hipErrorInvalidValue; // pool blocks are 256-byte aligned
    const bool half = half_ok(p); // by shape only: a program's launches all take the same kernel and weight layout
    const int R = half ? half_rows(p) : tile_rows(p);
    const dim3 wgrid((unsigned)((p.C * p.Cout + 255) / 256));
    if (p.weights_ready) {
        // the caller knows that w has not been written since the launch that left its re-laid copy in wt
    } else if (half) hipLaunchKernelGGL((conv3x3_weights_k<uint16_t, 5>), wgrid, dim3(256), 0, st, (const uint16_t *)p.w, (uint16_t *)wt, p.C, p.Cout);
    else if (p.dtype == DT_F32) hipLaunchKernelGGL((conv3x3_weights_k<float, 3>), wgrid, dim3(256), 0, st, (const float *)p.w, (float *)wt, p.C, p.Cout);
    else hipLaunchKernelGGL((conv3x3_weights_k<uint16_t, 4>), wgrid, dim3(256), 0, st, (const uint16_t *)p.w, (uint16_t *)wt, p.C, p.Cout);
    dim3 grid((unsigned)(p.N * (p.H / R)), (unsigned)(p.Cout / TILE_CO));
    const bool out_bf16 = p.out_dtype == DT_BF16;
#define ZK_LAUNCH(FI, OB, RL, PL)                                                                                                 \
    hipLaunchKernelGGL((conv3x3_k<FI, OB, RL, PL>), grid, dim3(256), lds_bytes(p), st, p.x, (const void *)wt, p.bias, p.y, p.C, p.H, \
                       p.W, p.Cout, R)
#define ZK_LAUNCH2(FI, OB)                                                                                                        \
    do {                                                                                                                          \
        if (p.relu && p.pool) ZK_LAUNCH(FI, OB, true, true);                                                                      \
        else if (p.relu) ZK_LAUNCH(FI, OB, true, false);                                                                          \
        else if (p.pool) ZK_LAUNCH(FI, OB, false, true);                                                                          \
        else ZK_LAUNCH(FI, OB, false, false);                                                                                     \
    } while (0)
    if (half) {
#define ZK_HALF_CB(OB, RL, PL, CB)                                                                                                \
    hipLaunchKernelGGL((conv3x3_half_k<OB, RL, PL, CB>), grid, dim3(256), half_lds_bytes(p), st, p.x, (const void *)wt, p.bias, p.y, \
                       p.C, p.H, p.W, p.Cout, R)
#define ZK_HALF(OB, RL, PL)                                                                                                       \
    do {                                                                                                                          \
        if (p.C == 64) ZK_HALF_CB(OB, RL, PL, 2);                                                                                 \
        else if (p.C == 128) ZK_HALF_CB(OB, RL, PL, 4);                                                                           \
        else ZK_HALF_CB(OB, RL, PL, 0);                                                                                           \
    } while (0)
#define ZK_HALF2(OB)                                                                                                              \
    do {                                                                                                                          \
        if (p.relu && p.pool) ZK_HALF(OB, true, true);                                                                            \
        else if (p.relu) ZK_HALF(OB, true, false);                                                                                \
        else if (p.pool) ZK_HALF(OB, false, true);                                                                                \
        else ZK_HALF(OB, false, false);                                                                                           \
    } while (0)
        if (out_bf16) ZK_HALF2(true);
        else ZK_HALF2(false);
#undef ZK_HALF2
#undef ZK_HALF
#undef ZK_HALF_CB
    } else if (p.dtype == DT_F32) ZK_LAUNCH2(true, false);
    else if (out_bf16) ZK_LAUNCH2(false, true);
    else ZK_LAUNCH2(false, false);
#undef ZK_LAUNCH2
#undef ZK_LAUNCH
    return hipGetLastError();
}

} // namespace zk
