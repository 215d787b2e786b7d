// Launchers of the hand-written gfx950 kernels. Each takes device pointers that the
// runtime has already bounds-checked against the registered shape, enqueues on the
// given stream and returns the HIP status of the launch.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>

namespace zk {

struct SoftmaxRows {
    int64_t rows, cols;
    int dtype = 2;  // DT_F32 (2), DT_BF16 (0) or DT_F16 (1): storage of x, y and rowsum
    const void *x;
    void *y;        // may be null
    void *rowsum;   // may be null
    int32_t *arg;   // may be null
};
hipError_t softmax_rows(const SoftmaxRows &p, hipStream_t stream);

// Accumulator program over a [rows, cols] view; see zhip_ew_op in include/zyx_hip.h.
struct Elementwise {
    int64_t rows, cols;
    int n_in, n_instr;
    int reg_class;    // DT_F32 or DT_I32
    int need_rowcol;  // some input is a row / column vector
    int in_dtype[4], in_bcast[4];
    int out_dtype;
    uint32_t code[18];
    float consts[8];
    const void *in[4];
    void *out;
};
hipError_t elementwise(const Elementwise &p, hipStream_t stream);
// The same chain as code generated for this one program and compiled at run time (ew_jit.cpp).
struct EwJit;
bool ew_jit_eligible(const Elementwise &p, int *vector_width);
EwJit *ew_jit_compile(const Elementwise &p, std::string &error);
bool ew_jit_can_launch(const EwJit *j, const Elementwise &p);
hipError_t ew_jit_launch(const EwJit *j, const Elementwise &p, hipStream_t stream);
void ew_jit_destroy(EwJit *j);

// Sum / max over the last axis (axis0 == 0) or over axis 0 (axis0 == 1) of x[rows, cols].
struct Reduce {
    int64_t rows, cols;
    int dtype;   // storage dtype of x and out: F32, BF16, F16 (f32 accumulate) or I32
    int op;      // 0 sum, 1 max
    int axis0;
    const void *x;
    void *out;
    void *workspace;           // partial results of the two-stage variants
    uint64_t workspace_bytes;
    float mul = 0.0f, div = 0.0f;   // float dtypes: out = (reduce * mul) / div + base, a 0 / null step is left out
    const void *base = nullptr;     // [len(out)] of the same dtype
};
// rows * cols below 2^40 elements and every grid dimension of the launches within 32 bits
bool reduce_shape_ok(int64_t rows, int64_t cols, int axis0);
uint64_t reduce_workspace_bytes(int64_t rows, int64_t cols, int axis0);
hipError_t reduce(const Reduce &p, hipStream_t stream);

// Index of the maximum along the middle axis of a contiguous x[outer, n, inner] (any axis of a dense tensor), ties to
// the largest index, NaN entries never chosen; out[outer, inner] is i32.
struct ArgMax {
    int64_t outer, n, inner;
    int dtype; // F32, BF16, F16 or I32
    const void *x;
    int32_t *out;
    void *workspace; // argmax_workspace_bytes(outer, n, inner)
    uint64_t workspace_bytes;
};
bool argmax_shape_ok(int64_t outer, int64_t n, int64_t inner);
uint64_t argmax_workspace_bytes(int64_t outer, int64_t n, int64_t inner);
hipError_t argmax(const ArgMax &p, hipStream_t stream);

// Geometry of a zero-padded NCHW input [images, C, Hp, Wp] from which gemm_bf16 gathers the patch matrix of a
// convolution on the fly (khw == 0: not used). Offsets in elements; k = (c*KH + ky)*KW + kx.
struct ConvGather {
    int ohw, ow;        // output pixels per image, per row
    int img, row;       // input elements per image; per output row step (sy * Wp)
    int cs, rs, dx;     // per channel (Hp*Wp), per ky (dy*Wp), per kx (dx)
    uint32_t khw, kw;   // KH*KW, KW
    uint32_t magic_khw, magic_kw; // ceil(2^32 / khw), ceil(2^32 / kw): exact division of k < 2^16 by a multiply-high
};

// C[M,N] = op(A) . op(B) (+ bias[N], + activation) (+ residual[M,N]), bf16 operands, f32 accumulate;
// C and the residual are f32, or bf16 (truncating store) when out_bf16 is set.
// trans_a: A is stored [K,M]; trans_b: B is stored [N,K] (a Linear weight [out,in]).
struct GemmBf16 {
    int64_t M, N, K;
    int trans_a, trans_b;
    int epilogue;      // 0 none, 1 bias, 2 bias+relu, 3 bias+gelu
    int bias_dtype;    // DT_BF16, DT_F16 or DT_F32
    int out_bf16;      // C and the residual are stored in the operands' 16-bit dtype
    int f16;           // operands (and a 16-bit C) are f16 instead of bf16
    int plane; // 0, or C is stored [M / plane, N, plane] (rows of one group of `plane` are contiguous per column)
    int64_t ldn; // 0, or the launch computes N columns of a product ldn columns wide (row stride of C, residual, [K,N] B)
    ConvGather gather; // with plane != 0 and gather.khw != 0: A is the padded input, not a matrix
    const void *A, *B, *bias, *residual; // residual may be null
    void *C;
    void *workspace; // gemm_bf16_workspace_bytes(M, N, K) bytes (split-K partials), may be null when that is 0
};
int gemm_bf16_tile_n(int64_t M, int64_t N);
int gemm_bf16_splits(int64_t M, int64_t N, int64_t K);
uint64_t gemm_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K);
bool gemm_bf16_supported(int64_t M, int64_t N, int64_t K); // every tile whole
bool gemm_bf16_supported(int64_t M, int64_t N, int64_t K, int trans_a, int trans_b, int out_bf16); // edge tiles allowed
int64_t gemm_bf16_column_split(int64_t M, int64_t N, int64_t K);
hipError_t gemm_bf16_init(); // once per device, before the first launch
hipError_t gemm_bf16(const GemmBf16 &p, hipStream_t stream); // either 16-bit dtype (p.f16)
hipError_t gemm_f16_init();
hipError_t gemm_f16(const GemmBf16 &p, hipStream_t stream);

// Any-shape GEMM: dtype F32 / BF16 / F16 operands, f32 accumulate, C stored as F32 or as
// the operand dtype (truncating). `batch` independent products at element strides
// batch_a / batch_b / batch_c. C = alpha * op(A).op(B) (+ bias) (act).
struct GemmGeneric {
    int64_t M, N, K, batch;
    int64_t batch_a, batch_b, batch_c;
    int dtype, out_dtype;
    int trans_a, trans_b;
    int epilogue, bias_dtype;
    float alpha;
    const void *A, *B, *bias, *residual; // residual (dtype out_dtype, [batch, M, N]) may be null
    int residual_is_mask = 0;            // the residual is not added: the result is multiplied by (residual > 0)
    void *C;
    void *workspace;      // gemm_generic_workspace_bytes(M, N, K, batch) bytes, may be null when that is 0
    int splits;           // set by the launcher
    int64_t k_len;        // set by the launcher
};
uint64_t gemm_generic_workspace_bytes(int64_t M, int64_t N, int64_t K, int64_t batch);
hipError_t gemm_generic(const GemmGeneric &p, hipStream_t stream);
// The LDS-tiled f32 kernel (gemm_f32.hip) for whole 64 x 64 x 32 tiles; gemm_generic hands such products over.
bool gemm_f32_tiled_ok(const GemmGeneric &p);
hipError_t gemm_f32_tiled(const GemmGeneric &p, hipStream_t stream);

// LayerNorm (rms == 0) / RMSNorm (rms == 1) over the last axis; w, b may be null.
struct NormRows {
    int64_t rows, cols;
    int dtype; // DT_F32 or DT_BF16 storage of x, w, b, y
    int rms;
    float eps;
    const void *x, *w, *b;
    void *y;
};
hipError_t norm_rows(const NormRows &p, hipStream_t stream);

// Gradients of the above: dx[rows, cols] (+ add, an optional tensor summed into dx: the other branch of a
// residual connection), dw[cols] = sum_rows dy * xhat, db[cols] = sum_rows dy (each optional).
struct NormRowsBwd {
    int64_t rows, cols;
    int dtype, rms;
    float eps;
    const void *x, *w, *dy, *add; // w, add may be null
    void *dx, *dw, *db;           // dw, db may be null
    void *workspace;              // norm_rows_bwd_workspace_bytes(rows, cols)
    uint64_t workspace_bytes;
};
uint64_t norm_rows_bwd_workspace_bytes(int64_t rows, int64_t cols);
hipError_t norm_rows_bwd(const NormRowsBwd &p, hipStream_t stream);

// conv2d forward, NCHW input, weight [Cout, C, KH, KW], groups = 1. koff[k] / kdyx[k] (k = (c,ky,kx)):
// input offset c*H*W + ky*dy*W + kx*dx and the tap displacement (ky*dy) << 16 | (kx*dx), device arrays.
struct Conv2d {
    int N, C, H, W, Cout, KH, KW, OH, OW;
    int sy, sx, py, px, dy, dx;
    int dtype, out_dtype, relu;
    int pool; // 1: y is the 2 x 2 / stride 2 max-pool of the (activated) result; only the direct 3 x 3 kernel does this
    const void *x, *w, *bias;
    void *y;
    const int32_t *koff, *kdyx;
    void *scratch; // conv2d_scratch_bytes(p) bytes when the product runs on the tiled MFMA GEMM, else unused
    bool weights_ready = false; // the direct kernel's re-laid copy of w in `scratch` is current: skip the re-layout launch
};
uint64_t conv2d_scratch_bytes(const Conv2d &p);
hipError_t conv2d(const Conv2d &p, hipStream_t stream);
// Direct 3 x 3 / stride 1 / padding 1 convolution, bf16 or f32, optional fused 2 x 2 max-pool (conv3x3.hip): shapes it takes, bytes for its re-laid weights,
// one-time set-up of the kernel's LDS limit, launch.
bool conv3x3_direct_ok(const Conv2d &p);
uint64_t conv3x3_scratch_bytes(const Conv2d &p);
hipError_t conv3x3_init();
hipError_t conv3x3_direct(const Conv2d &p, void *weights_scratch, hipStream_t stream);

// max-pool over the last two axes of `planes` images [H, W] -> [OH, OW]
struct MaxPool2d {
    int64_t planes;
    int H, W, OH, OW, KH, KW, sy, sx, py, px, dy, dx;
    int dtype;
    const void *x;
    void *y;
};
hipError_t max_pool2d(const MaxPool2d &p, hipStream_t stream);

// gather / index_select / scatter along `axis` of a rank-4 view (leading dims padded with 1).
// gather: x has shape xs, idx (and out) shape os; select: idx is 1-D of length os[axis].
// scatter: self (x) and out have shape xs, idx and src shape os.
struct IndexOp {
    int64_t xs[4], os[4];
    int axis, dtype, idx64, select, scatter;
    const void *x, *idx, *src;
    void *out;
};
hipError_t index_op(const IndexOp &p, hipStream_t stream);
// dst[0, bytes) = src[0, bytes) (ranges must not overlap), as one kernel launch
hipError_t copy_range(void *dst, const void *src, uint64_t bytes, hipStream_t stream);

// Attention core over the packed c_attn output qkv[B, T, 3, H, dh] -> y[B, T, H*dh]:
// y = softmax(scale q k^T) / keep . v per head, no mask. lse[B, H, T] (optional) = ln sum exp(scale q k^T).
struct Attention {
    int B, T, H, dh;
    int dtype; // DT_BF16 or DT_F32 storage of qkv and y
    float scale, keep;
    int causal; // query t attends to keys 0..t only
    const void *qkv;
    void *y;
    float *lse;
};
bool attention_fast_path(const Attention &p);
hipError_t attention_fwd(const Attention &p, hipStream_t stream);
// d(sum(y o dy)) / d(qkv): fwd.y and fwd.lse are the forward's outputs (inputs here), dy[B, T, H*dh] the
// incoming gradient, dqkv[B, T, 3, H, dh] the result. workspace: attention_bwd_workspace_bytes(fwd) bytes.
struct AttentionBwd {
    Attention fwd;
    const void *dy;
    void *dqkv;
    void *workspace;
};
uint64_t attention_bwd_workspace_bytes(const Attention &p);
hipError_t attention_bwd(const AttentionBwd &p, hipStream_t stream);

// What this device sustains right now (ceilings.hip); the layout is zhip_ceilings of include/zyx_hip.h.
struct Ceilings {
    float memcpy_d2d_GBps, copy_kernel_GBps, read_kernel_GBps;
    float mfma_bf16_const_TFLOPs, mfma_bf16_const_MHz, mfma_bf16_const_launch_us;
    float mfma_bf16_random_TFLOPs, mfma_bf16_random_MHz, mfma_bf16_random_launch_us;
};
hipError_t measure_ceilings(uint64_t bytes, int compute_units, Ceilings *out, hipStream_t stream);

// cross_entropy of f32 logits [rows, cols] with i32 class indices; loss / grad may be null.
struct CrossEntropy {
    int64_t rows, cols;
    float gscale;
    const float *x;
    const int32_t *labels;
    float *loss, *grad;
    const float *dense = nullptr; // f32 targets [rows, cols] in place of class indices
    float *mean = nullptr; // [1]: sum(loss) / rows, by a single workgroup (rows <= kCrossEntropyMeanRows)
};
constexpr int64_t kCrossEntropyMeanRows = 4096;
hipError_t cross_entropy(const CrossEntropy &p, hipStream_t stream);

} // namespace zk
