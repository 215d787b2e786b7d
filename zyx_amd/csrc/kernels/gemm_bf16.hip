// bf16 instances of the LDS-tiled MFMA GEMM (gemm_tiled.inc) and the shape rules both 16-bit dtypes share.
#define ZK_GEMM_F16 false
#include "gemm_tiled.inc"

namespace zk {

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

hipError_t gemm_bf16_init() { return tiled_init(); }

hipError_t gemm_bf16(const GemmBf16 &p, hipStream_t st) {
    if (p.f16) return gemm_f16(p, st);
    return tiled_gemm(p, st);
}

} // namespace zk
