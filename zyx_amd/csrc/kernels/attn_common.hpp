// Pieces shared by the attention kernels: vector types, the LDS tile layout and its two fragment reads.
#pragma once
#include "dtypes.hpp"
#include "wave.hpp"

namespace zk {
namespace attn {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
#define ZK_LDS __attribute__((address_space(3)))

constexpr int DH = 64;             // head width of the matrix-core kernels
constexpr int TROWS = 64;          // rows (keys or queries) per staged tile
constexpr int TILE = TROWS * DH * 2; // 8 KiB
constexpr float kLog2e = 1.44269504088896340736f, kLn2 = 0.69314718055994530942f;

// A staged tile is [row][16-byte chunk ^ f(row)] with 128-byte rows, f(row) = row bits (1, 3, 2) as chunk
// bits (2, 1, 0). Both ways of reading it are then conflict-free:
//  * ds_read_b128 of 16 consecutive rows at one logical chunk (an MFMA operand whose 8 k-slots are
//    contiguous in the row): the 8 rows of one parity see 8 different f, and parity picks the other half of
//    the 256-byte bank window;
//  * ds_read_b64_tr_b16 of 4 consecutive rows x 32 columns (an operand transposed on the fly): row bit 1
//    flips the 64-byte half, row bit 0 the 128-byte half, so the four pieces cover all 64 banks once.
__device__ __forceinline__ int tile_f(int row) { return (((row >> 1) & 1) << 2) | (((row >> 3) & 1) << 1) | ((row >> 2) & 1); }
__device__ __forceinline__ int tile_slot(int row, int chunk) { return row * 128 + ((chunk ^ tile_f(row)) << 4); }

// Row-major operand, lane -> row lane%32 of a 32-row block, k-slots = columns ks*16 + (lane/32)*8 .. +7.
// f(row + 16) == f(row), so one offset per ks serves every 16-row multiple: add rows*128.
__device__ __forceinline__ int frag_row_off(int lane, int ks) { return tile_slot(lane & 31, ks * 2 + (lane >> 5)); }
__device__ __forceinline__ bf16x8 frag_row(const ZK_LDS uint8_t *lds, int off) { return *(const ZK_LDS bf16x8 *)(lds + off); }

// Transposed operand, lane -> column db*32 + lane%32, k-slots e = 0..7 = rows base + 8*(e/4) + 4*(lane/32) + e%4
// (base a multiple of 16): the order in which a 32x32 MFMA result holds its rows in registers 8*s2 .. 8*s2+7,
// so a result tile converted to bf16 is directly the other operand. In each group of 16 lanes, lane r
// points at 4 columns of row (r >> 2); the hardware hands lane i column i of those 4 rows. `second` selects
// the rows + 8 (their f differs, so they get an offset of their own).
__device__ __forceinline__ int frag_tr_off(int lane, int db, int second) {
    const int g16 = lane >> 4, r = lane & 15;
    const int row = 4 * (g16 >> 1) + (r >> 2) + 8 * second;
    const int col = db * 32 + (g16 & 1) * 16 + (r & 3) * 4;
    return tile_slot(row, col >> 3) + (col & 7) * 2;
}
__device__ __forceinline__ bf16x8 frag_tr(const ZK_LDS uint8_t *lds, int off_lo, int off_hi) {
    const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)(lds + off_lo));
    const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((ZK_LDS bf16x4 *)(lds + off_hi));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// 4 consecutive result values of a lane as bf16 (truncating store, zyx/src/codegen/c.rs:494-496)
__device__ __forceinline__ u32x2 pack4_trunc(float a, float b, float c, float d) {
    u32x2 w = {(uint32_t)f32_to_bf16_trunc(a) | ((uint32_t)f32_to_bf16_trunc(b) << 16),
               (uint32_t)f32_to_bf16_trunc(c) | ((uint32_t)f32_to_bf16_trunc(d) << 16)};
    return w;
}

// XCD-aware numbering: workgroups with ids congruent mod 8 share an XCD and its L2; hand each XCD whole
// (batch, head) pairs so the tiles every workgroup of a head streams are fetched into one L2 only.
__device__ __forceinline__ void head_and_block(int nblk, int &bh, int &blk) {
    const int BH = (int)gridDim.x / nblk;
    if (BH % 8 == 0) {
        const int x = blockIdx.x & 7, i = blockIdx.x >> 3;
        bh = (i / nblk) * 8 + x;
        blk = i % nblk;
    } else {
        bh = blockIdx.x / nblk;
        blk = blockIdx.x % nblk;
    }
}

} // namespace attn
} // namespace zk
