// Recording stand-ins for the hand-written kernel launchers of zyx_amd/csrc/kernels/*.hip (device code, absent from
// a CPU build): each tells the fake runtime which allocations the launch reads and writes and does nothing else.
// Every kind that may own scratch memory asks for some here, whatever the shape, so that the runtime's ordering of
// launches that share a program's scratch is exercised by every such program.
#include "../../zyx_amd/csrc/kernels/kernels.hpp"
#include "fake_hip.h"

namespace zk {

namespace {
constexpr uint64_t kScratch = 4096;
hipError_t rec(hipStream_t st, const char *name, std::initializer_list<const void *> reads, std::initializer_list<const void *> writes) {
    std::vector<FakeAccess> acc;
    for (const void *p : reads) acc.push_back({p, false});
    for (const void *p : writes) acc.push_back({p, true});
    return fakehip_launch(st, name, acc) ? hipSuccess : hipErrorInvalidValue;
}
} // namespace

hipError_t softmax_rows(const SoftmaxRows &p, hipStream_t st) { return rec(st, "softmax_rows", {p.x}, {p.y, p.rowsum, p.arg}); }
hipError_t elementwise(const Elementwise &p, hipStream_t st) { return rec(st, "elementwise", {p.in[0], p.in[1], p.in[2], p.in[3]}, {p.out}); }

bool reduce_shape_ok(int64_t rows, int64_t cols, int) { return rows >= 0 && cols >= 0 && (cols == 0 || rows <= (1ll << 40) / cols); }
// 7777 rows: a shape whose partial results exceed any scratch, for the callers' refusal paths
uint64_t reduce_workspace_bytes(int64_t rows, int64_t cols, int) { return rows == 7777 ? (64ull << 20) : rows > 0 && cols > 0 ? kScratch : 0; }
hipError_t reduce(const Reduce &p, hipStream_t st) { return rec(st, "reduce", {p.x, p.base}, {p.out, p.workspace}); }

bool argmax_shape_ok(int64_t outer, int64_t n, int64_t inner) { return outer >= 0 && n >= 1 && inner >= 0; }
uint64_t argmax_workspace_bytes(int64_t, int64_t, int64_t) { return kScratch; }
hipError_t argmax(const ArgMax &p, hipStream_t st) { return rec(st, "argmax", {p.x}, {p.out, p.workspace}); }

int gemm_bf16_tile_n(int64_t, int64_t) { return 256; }
int gemm_bf16_splits(int64_t, int64_t, int64_t) { return 2; }
uint64_t gemm_bf16_workspace_bytes(int64_t, int64_t, int64_t) { return kScratch; }
bool gemm_bf16_supported(int64_t M, int64_t N, int64_t K) { return M % 256 == 0 && N % 128 == 0 && K % 64 == 0; }
bool gemm_bf16_supported(int64_t M, int64_t N, int64_t K, int, int, int) { return M >= 64 && N >= 64 && K % 64 == 0; }
int64_t gemm_bf16_column_split(int64_t, int64_t, int64_t) { return 0; }
hipError_t gemm_bf16_init() { return hipSuccess; }
hipError_t gemm_f16_init() { return hipSuccess; }
hipError_t gemm_bf16(const GemmBf16 &p, hipStream_t st) { return rec(st, "gemm_bf16", {p.A, p.B, p.bias, p.residual}, {p.C, p.workspace}); }
uint64_t gemm_generic_workspace_bytes(int64_t, int64_t, int64_t, int64_t) { return kScratch; }
hipError_t gemm_generic(const GemmGeneric &p, hipStream_t st) { return rec(st, "gemm_generic", {p.A, p.B, p.bias, p.residual}, {p.C, p.workspace}); }

hipError_t norm_rows(const NormRows &p, hipStream_t st) { return rec(st, "norm_rows", {p.x, p.w, p.b}, {p.y}); }
uint64_t norm_rows_bwd_workspace_bytes(int64_t, int64_t) { return kScratch; }
hipError_t norm_rows_bwd(const NormRowsBwd &p, hipStream_t st) {
    return rec(st, "norm_rows_bwd", {p.x, p.w, p.dy, p.add}, {p.dx, p.dw, p.db, p.workspace});
}

uint64_t conv2d_scratch_bytes(const Conv2d &) { return kScratch; }
hipError_t conv2d(const Conv2d &p, hipStream_t st) { return rec(st, "conv2d", {p.x, p.w, p.bias, p.koff}, {p.y, p.scratch}); }
bool conv3x3_direct_ok(const Conv2d &p) { return p.KH == 3 && p.KW == 3 && p.C % 16 == 0 && p.Cout % 128 == 0; }
uint64_t conv3x3_scratch_bytes(const Conv2d &) { return kScratch; }
hipError_t conv3x3_init() { return hipSuccess; }
hipError_t conv3x3_direct(const Conv2d &p, void *scratch, hipStream_t st) { return rec(st, "conv3x3", {p.x, p.w, p.bias}, {p.y, scratch}); }
hipError_t max_pool2d(const MaxPool2d &p, hipStream_t st) { return rec(st, "max_pool2d", {p.x}, {p.y}); }

hipError_t index_op(const IndexOp &p, hipStream_t st) { return rec(st, "index_op", {p.x, p.idx, p.src}, {p.out}); }
hipError_t copy_range(void *dst, const void *src, uint64_t, hipStream_t st) { return rec(st, "copy_range", {src}, {dst}); }

bool attention_fast_path(const Attention &) { return true; }
hipError_t attention_fwd(const Attention &p, hipStream_t st) { return rec(st, "attention_fwd", {p.qkv}, {p.y, p.lse}); }
uint64_t attention_bwd_workspace_bytes(const Attention &) { return kScratch; }
hipError_t attention_bwd(const AttentionBwd &p, hipStream_t st) {
    return rec(st, "attention_bwd", {p.fwd.qkv, p.fwd.y, p.dy, p.fwd.lse}, {p.dqkv, p.workspace});
}

hipError_t cross_entropy(const CrossEntropy &p, hipStream_t st) { return rec(st, "cross_entropy", {p.x, p.labels}, {p.loss, p.grad, p.mean}); }

hipError_t measure_ceilings(uint64_t, int, Ceilings *out, hipStream_t) {
    *out = Ceilings{};
    return hipSuccess;
}

} // namespace zk
