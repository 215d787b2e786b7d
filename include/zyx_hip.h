/*
 * zyx_hip.h -- C ABI of the MI355X (gfx950) HIP backend for zyx.
 *
 * The entry points are what zyx's backend plugin slot for HIP dispatches to: one
 * `zhip_ctx` stands for the `MemoryPool::HIP` + `Device::HIP` pair the reference
 * creates per GPU (zyx/src/backend/hip.rs:122-339, zyx/src/backend/mod.rs:533-1028).
 * Each declaration cites the reference method it replaces (paths relative to the
 * reference checkout). Plain pointers and sizes only; no C++ or torch types.
 *
 * Conventions
 *   - Every function returning int32_t returns a zhip_status: 0 = ok, 1..13 are the
 *     reference's ErrorStatus variants in declaration order (zyx/src/error.rs:125-153).
 *     The message of the last failure on a context is read with zhip_last_error().
 *   - zhip_buf / zhip_prog are slab indices like PoolBufferId / DeviceProgramId
 *     (zyx/src/backend/mod.rs:54-55,121-122; zyx/src/slab.rs): dense, reused after
 *     free, ZHIP_NULL_ID (u32::MAX) = NULL.
 *   - zhip_event is an opaque handle owned by the caller and consumed exactly once.
 *     0 is the null event ("already signalled", the analogue of a null hipEvent_t,
 *     hip.rs:375,396). Wait lists handed to zhip_h2d / zhip_d2h / zhip_launch /
 *     zhip_free are CONSUMED by the call ("a removed event is consumed",
 *     zyx/src/runtime.rs:13-15); the reference's HIP stub leaks them instead.
 *   - Calls may come from any thread; a context serialises them internally (the
 *     reference calls its backends under one global mutex, zyx/src/lib.rs:96).
 *   - Launch argument order: read-only buffers first, then written buffers
 *     (zyx/src/kernel/linearize.rs:138-155; AOT kernels: inputs then outputs,
 *     zyx/src/backend/cblas.rs:260-263, zyx/src/graph/plan.rs:311-327).
 *   - Callers over-allocate by one element / 8 bytes (zyx/src/backend/mod.rs:627,
 *     zyx/src/graph/plan.rs:305); kernels never touch that slack.
 */
#ifndef ZYX_HIP_H
#define ZYX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct zhip_ctx zhip_ctx;
typedef uint32_t zhip_buf;
typedef uint32_t zhip_prog;
typedef uint64_t zhip_event;

#define ZHIP_NULL_ID 0xffffffffu

/* zyx/src/error.rs:125-153 (ErrorStatus), 0 added for success */
enum zhip_status {
    ZHIP_OK = 0,
    ZHIP_DYLIB_NOT_FOUND = 1,
    ZHIP_INITIALIZATION = 2,
    ZHIP_DEINITIALIZATION = 3,
    ZHIP_DEVICE_ENUMERATION = 4,
    ZHIP_DEVICE_QUERY = 5,
    ZHIP_MEMORY_ALLOCATION = 6,
    ZHIP_MEMORY_DEALLOCATION = 7,
    ZHIP_MEMORY_COPY_H2P = 8,
    ZHIP_MEMORY_COPY_P2H = 9,
    ZHIP_INCORRECT_KERNEL_ARG = 10,
    ZHIP_KERNEL_COMPILATION = 11,
    ZHIP_KERNEL_LAUNCH = 12,
    ZHIP_KERNEL_SYNC = 13
};

/* zyx/src/dtype.rs:20-47 (DType discriminants) */
enum zhip_dtype {
    ZHIP_BF16 = 0, ZHIP_F16, ZHIP_F32, ZHIP_F64, ZHIP_U8, ZHIP_U16, ZHIP_U32, ZHIP_U64,
    ZHIP_I8, ZHIP_I16, ZHIP_I32, ZHIP_I64, ZHIP_BOOL, ZHIP_N_DTYPES
};

/* HIPConfig (zyx/src/backend/hip.rs:27-32) + the runtime's debug mask
 * (zyx/src/lib.rs:101-163): bit 0 devices, 5 kernel launches, 6 memory, 7 compile. */
typedef struct zhip_config {
    int32_t device_id;  /* HIP device ordinal; one context per device */
    uint32_t debug;     /* ZYX_DEBUG bitmask */
    uint64_t cache_bytes; /* freed blocks kept for reuse before going back to the driver; 0 = default (1 GiB) */
} zhip_config;

/* DeviceInfo (zyx/src/backend/mod.rs:506-531), filled from the device's properties. */
typedef struct zhip_device_info {
    uint64_t compute;                  /* peak f32 vector flop/s (u128 in the reference) */
    uint64_t max_global_work_dims[3];
    uint32_t max_local_threads;
    uint32_t max_local_work_dims[3];
    uint32_t preferred_vector_size;    /* bytes */
    uint64_t local_mem_size;           /* LDS bytes a workgroup may use */
    uint64_t max_register_bytes;
    uint32_t tensor_cores;             /* MFMA present */
    uint32_t warp_size;                /* 64 */
    uint32_t dtype_capability[ZHIP_N_DTYPES]; /* DTypeCapability bits, mod.rs:440-471 */
    uint32_t has_native_exp2;
    uint32_t n_supported_vec_lens;
    uint32_t supported_vec_lens[4];
    /* not in the reference struct; for reports */
    uint64_t total_bytes;
    uint32_t compute_units;
    uint32_t clock_khz;
    char name[64];
    char arch[32];
} zhip_device_info;

/* Hand-written kernels, registered as AOT programs (the slot cblas/cuDNN fill in the
 * reference: zyx/src/backend/cblas.rs:213-238, zyx/src/backend/cuda.rs:1033-1074). */
enum zhip_kernel_kind {
    /* x[rows,cols] -> y = softmax(x, -1), rowsum = y.sum(-1), arg = y.argmax_axis(-1).
     * dims = {rows, cols}; flags selects outputs (ZHIP_SOFTMAX_*); args: x, then the
     * selected outputs in the order y, rowsum, arg. dtype ZHIP_F32, ZHIP_BF16 or ZHIP_F16 (x, y, rowsum; arg is
     * i32): 16-bit elements widen to f32 registers, y is truncated on store, and the sum and argmax read the stored
     * y, as the C backend's kernels do (zyx/src/codegen/c.rs:456-497).
     * zyx/src/tensor/mod.rs:1457-1461, 2245-2269; zyx/src/tensor/reduce_ops.rs:197-199 */
    ZHIP_K_SOFTMAX_ROWS = 1,
    /* Fused elementwise chain over a [rows, cols] view (dims = {rows, cols}): up to 4
     * inputs, each a full tensor, a [cols] row vector, a [rows] column vector or one
     * scalar, combined by a short accumulator program (zhip_ew_op) whose op semantics are
     * zyx's UOp/BOp tables (zyx/src/kernel/ops.rs:187-261, C meaning
     * zyx/src/codegen/c.rs:290-304,593-611) plus the Tensor-level composites of
     * zyx/src/tensor/elementwise.rs. Float dtypes compute in f32 registers and narrow only
     * on store (bf16 truncates), as the C backend does; I32 computes in int32.
     *   iparams[0] = n_inputs (1..4), iparams[1] = n_instr (1..18),
     *   iparams[2+k] = input k: dtype | (zhip_ew_bcast << 8),
     *   iparams[6+j] = instruction j: op | (src_a << 8) | (src_b << 16),
     *   fparams[0..8] = constants, flags = 0. `dtype` is the register class (ZHIP_F32 or
     *   ZHIP_I32), `out_dtype` the stored dtype. args: inputs in order, then the output. */
    ZHIP_K_ELEMENTWISE = 2,
    /* Reduce over the last axis (flags = 0: x[rows,cols] -> [rows]) or over axis 0
     * (flags = 1: -> [cols]); iparams[0] = 0 sum, 1 max. Accumulates in f32 for float
     * dtypes and i32 for ZHIP_I32, stores as `dtype` (zyx/src/tensor/reduce_ops.rs:45-147,
     * accumulator init zyx/src/kernel/linearize.rs:920-952). Float dtypes may fold the ops that follow a
     * reduce in a training step into its store, each a separate f32 operation in this order:
     * fparams[0] != 0: * fparams[0]; fparams[1] != 0: / fparams[1] (the n of a mean, reduce_ops.rs:62-75);
     * iparams[1] != 0: + base[i], a second input of out's shape and dtype (`p - g * lr` of SGD::update,
     * zyx-optim/src/sgd.rs:77-81, with fparams[0] = -lr and base = p).
     * args: x, (base when iparams[1] != 0), out. */
    ZHIP_K_REDUCE = 3,
    /* C[M,N] = op(A) . op(B) (+ bias[N]) (then ReLU / GELU): Tensor::dot / dot_dtype
     * (zyx/src/tensor/mod.rs:1469-1518) and Linear::forward (zyx-nn/src/linear.rs:38-44),
     * the pattern Graph::match_matmul recognises (zyx/src/vendor/matmul.rs:43-71).
     * dims = {M, N, K, batch (0 = 1)}: `batch` independent dense products laid out back to
     * back; dtype = operand dtype (F32, BF16, F16); out_dtype = dtype of C (F32 or dtype,
     * narrowing stores truncate); flags bit 0: A is stored [K,M], bit 1: B is stored [N,K]
     * (a Linear weight [out,in]);
     * iparams[0] = epilogue: 0 none, 1 + bias, 2 + bias then ReLU, 3 + bias then GELU;
     * iparams[1] = dtype of bias; iparams[2] = 1: a residual[batch, M, N] of dtype out_dtype is
     * added last (the `x + module(x)` of a transformer block, zyx-examples/examples/nanogpt.rs:89-95);
     * iparams[2] = 2: that tensor is a mask instead, the result is multiplied by (mask > 0) last: the
     * gradient of relu = cmpgt(0) * x applied to a product dY . W (zyx/src/tensor/elementwise.rs:289-293,
     * zyx/src/graph/autograd.rs:120-125), with the forward's activations as the mask;
     * fparams[0] = alpha scaling the product (0 = 1).
     * Products and sums are f32. bf16 problems with M, N multiples of 256 and K a multiple of
     * 64 run on the 256x256 LDS-tiled MFMA kernel, the rest on a 64x64 one.
     * args: A, B, (bias when iparams[0] != 0), (residual when iparams[2] != 0), then C. */
    ZHIP_K_GEMM = 4,
    /* y = LayerNorm(x) or RMSNorm(x) over the last axis of x[rows, cols] (dims = {rows, cols},
     * dtype F32 or BF16 for x, weight, bias and y, f32 arithmetic, one narrowing store).
     * flags: ZHIP_NORM_RMS selects RMSNorm, ZHIP_NORM_WEIGHT / ZHIP_NORM_BIAS say which
     * affine operands are passed; fparams[0] = eps. LayerNorm uses the unbiased (n-1)
     * variance, as zyx-nn/src/layer_norm.rs:98-135 does through Tensor::var
     * (zyx/src/tensor/reduce_ops.rs:795-805); RMSNorm is zyx-nn/src/rms_norm.rs:26-32.
     * args: x, (weight[cols]), (bias[cols]), then y. */
    ZHIP_K_NORM_ROWS = 5,
    /* Tensor::cross_entropy of f32 logits[rows, cols] with I32 class indices[rows]
     * (zyx/src/tensor/mod.rs:1639-1655; ln_softmax :1427-1431; one-hot by equal(arange)
     * :1920-1946). flags: ZHIP_CE_LOSS writes the per-sample loss[rows] (ReduceOp::None),
     * ZHIP_CE_GRAD writes d(fparams[0] * sum(loss))/d(logits) = (softmax - onehot) *
     * fparams[0] into grad[rows, cols] (fparams[0] = 1/rows for the Mean reduction),
     * ZHIP_CE_MEAN (rows <= 4096) writes mean[1] = sum(loss) / rows (ReduceOp::Mean) from the same launch.
     * ZHIP_CE_DENSE: the targets are an f32 tensor of the logits' shape instead (the `target` of
     * :1641-1646 when it already has the logits' shape): loss = sum_c -ln_softmax * target,
     * grad = (softmax * sum_c target - target) * fparams[0].
     * args: logits, labels | targets, (loss), (grad), (mean). */
    ZHIP_K_CROSS_ENTROPY = 6,
    /* Tensor::conv for 4-D NCHW input, groups = 1 (zyx/src/tensor/mod.rs:2583-2680; layer
     * zyx-nn/src/conv2d.rs:60-70): y[N,Cout,OH,OW] = x[N,C,H,W] (*) w[Cout,C,KH,KW] (+ bias[Cout])
     * (then ReLU), zero padding, OH = (H + 2*py - dy*(KH-1) - 1) / sy + 1 (OW likewise).
     * dims = {N, C, H, W, Cout, KH, KW}; iparams = {sy, sx, py, px, dy, dx, has_bias, relu, pool};
     * dtype F32 or BF16 for x, w, bias; out_dtype = dtype, or F32 for BF16 operands. Products
     * and sums are f32. pool = 1: y is Tensor::max_pool([2, 2]) of that result (stride 2, no
     * padding; mod.rs:2706-2741), y[N,Cout,OH/2,OW/2], from the same launch; taken for
     * 3x3 / stride 1 / dilation 1 / padding 1 shapes with C % 16 = 0, Cout % 128 = 0, W % 8 = 0,
     * W a divisor of 224 and H a multiple of 448 / W, refused otherwise. args: x, w, (bias), y. */
    ZHIP_K_CONV2D = 7,
    /* Tensor::max_pool over the last two axes (zyx/src/tensor/mod.rs:2706-2741): padding counts
     * as the dtype's lowest value. dims = {planes (product of the leading axes), H, W, KH, KW};
     * iparams = {sy, sx, py, px, dy, dx}; dtype F32 or BF16. args: x, y[planes, OH, OW]. */
    ZHIP_K_MAX_POOL2D = 8,
    /* Tensor::gather / index_select / scatter along one axis, tensors of rank <= 4 given as
     * 4-D shapes with leading 1s (zyx/src/tensor/index_ops.rs:321-445). Negative indices wrap
     * once, indices still out of range read 0 (gather) or are dropped (scatter); scatter adds,
     * duplicates sum in ascending position order, `self` is added last.
     * dims[0..4] = shape of x / self, dims[4..8] = shape of the index tensor (for
     * ZHIP_INDEX_SELECT: shape of the output, the index being 1-D of length dims[4+axis]);
     * iparams[0] = axis (0..3 in the 4-D view), iparams[1] = index dtype (ZHIP_I32 / ZHIP_I64);
     * flags = ZHIP_INDEX_GATHER | ZHIP_INDEX_SELECT | ZHIP_INDEX_SCATTER. dtype: gather and
     * select copy any dtype bit for bit; scatter supports F32, F64, I32, U32, I64, U64.
     * args: gather/select: x, index, out; scatter: self, index, src, out. */
    ZHIP_K_INDEX = 9,
    /* Attention core of CausalSelfAttention::forward (zyx-nn/src/causal_self_attention.rs:36-74) on the
     * c_attn output qkv[B, T, 3*C], C = H*dh: split([c,c,c], 2), reshape [b,t,h,dh], transpose(1,2),
     * att = q.dot(k.t()) * scale, softmax(-1), eval-mode dropout att / (1 - p)
     * (zyx/src/tensor/mod.rs:822-828), att.dot(v), transpose(1,2).reshape([b,t,c]). The reference
     * applies no mask, so none is applied. dims = {B, T, H, dh}; dtype BF16 or F32 (storage of qkv
     * and y, f32 arithmetic); fparams[0] = scale (0 selects 1/sqrt(dh)), fparams[1] = dropout p;
     * flags: ZHIP_ATTN_LSE also writes lse[B, H, T] (f32) = ln sum_j exp(scale q.k_j), which the
     * backward needs; ZHIP_ATTN_CAUSAL: query t attends to keys 0..t only, what a lower-triangular
     * mask filled with -inf before the softmax gives (the reference's module has no such mask; the
     * flag serves models that add one). args: qkv, y[B, T, C], (lse). */
    ZHIP_K_ATTENTION = 10,
    /* Gradient of ZHIP_K_ATTENTION with respect to qkv: what Runtime::gradient
     * (zyx/src/graph/autograd.rs:14-424) builds from the reverse rules of the forward's ops (Mul :120-125,
     * Div :126-134, Exp :87-95, Sub :111-119, the reduce rules :299-379), evaluated in one pass:
     * dV = P^T.dy, dS = Ps o (dy.v^T / (1-p) - rowsum(dy o y)), dQ = scale dS.k, dK = scale dS^T.q, with the
     * probabilities recomputed from lse. dims, dtype, fparams as for ZHIP_K_ATTENTION; flags: ZHIP_ATTN_CAUSAL
     * as in the forward (masked probabilities and their gradients are 0).
     * args: qkv, y, dy[B, T, C], lse[B, H, T] (the forward's inputs and outputs), then dqkv[B, T, 3*C]. */
    ZHIP_K_ATTENTION_BWD = 11,
    /* Gradients of ZHIP_K_NORM_ROWS (LayerNorm zyx-nn/src/layer_norm.rs:98-135, RMSNorm rms_norm.rs:26-32)
     * as Runtime::gradient derives them (zyx/src/graph/autograd.rs:87-134, 299-379), one fused pass per row:
     * LayerNorm dx = rstd (g - mean(g) - xh sum(g xh)/(n-1)), g = dy*w, xh = (x-mean) rstd (the n-1 is the
     * unbiased variance of the forward); RMSNorm dx = r g - r^3 x sum(g x)/n; dw = sum_rows dy*xh,
     * db = sum_rows dy. dims = {rows, cols}; dtype F32 or BF16; fparams[0] = eps; flags: ZHIP_NORM_RMS,
     * ZHIP_NORM_WEIGHT (w is passed and dw is wanted), ZHIP_NORM_BIAS (db is wanted),
     * ZHIP_NORM_ADD (a tensor [rows, cols] that is added to dx: the skip branch of x + f(norm(x))).
     * args: x, (w), dy, (add), then dx, (dw), (db). */
    ZHIP_K_NORM_ROWS_BWD = 12,
    /* Tensor::argmax_axis / argmax (zyx/src/tensor/mod.rs:2228-2269) along one axis of a dense tensor seen as
     * x[outer, n, inner] (outer = product of the axes before it, inner = of those after; argmax() is outer = inner = 1):
     * max_k((x == max_keepdim(x)) * k) as I32, i.e. the LARGEST index among equal maxima; the maximum is a reduce from
     * the dtype's lowest finite value (zyx/src/kernel/linearize.rs:920-952) under fmax, so NaN entries are never
     * chosen and a slice with no candidate gives 0. dims = {outer, n, inner}, n >= 1; dtype F32, BF16, F16 or I32.
     * args: x, out[outer, inner] (I32). */
    ZHIP_K_ARGMAX = 13,
    ZHIP_K_COUNT_
};
#define ZHIP_SOFTMAX_Y 1
#define ZHIP_SOFTMAX_ROWSUM 2
#define ZHIP_SOFTMAX_ARGMAX 4
#define ZHIP_NORM_RMS 1
#define ZHIP_NORM_WEIGHT 2
#define ZHIP_NORM_BIAS 4
#define ZHIP_NORM_ADD 8
#define ZHIP_CE_LOSS 1
#define ZHIP_CE_GRAD 2
#define ZHIP_CE_MEAN 4
#define ZHIP_CE_DENSE 8 /* the second argument is an f32 [rows, cols] target tensor (one-hot or soft labels) */
#define ZHIP_INDEX_GATHER 0
#define ZHIP_INDEX_SELECT 1
#define ZHIP_INDEX_SCATTER 2
#define ZHIP_ATTN_LSE 1
#define ZHIP_ATTN_CAUSAL 2
#define ZHIP_GEMM_TRANS_A 1
#define ZHIP_GEMM_TRANS_B 2

/* Accumulator program of ZHIP_K_ELEMENTWISE. One register `acc`, one saved register `t`.
 * An operand (src_a / src_b) is: 0..3 = input k (read at that point), ZHIP_EW_SRC_T = t,
 * ZHIP_EW_SRC_CONST + k = fparams[k] (converted to the register class). */
enum zhip_ew_op {
    ZHIP_EW_LOAD = 0, /* acc = a */
    ZHIP_EW_SAVE,     /* t = acc */
    /* UOp, acc = op(acc) */
    ZHIP_EW_NEG, ZHIP_EW_BITNOT, ZHIP_EW_EXP, ZHIP_EW_EXP2, ZHIP_EW_LN, ZHIP_EW_LOG2, ZHIP_EW_RECIPROCAL,
    ZHIP_EW_SQRT, ZHIP_EW_SIN, ZHIP_EW_COS, ZHIP_EW_FLOOR, ZHIP_EW_TRUNC, ZHIP_EW_ABS,
    /* BOp, acc = acc op a */
    ZHIP_EW_ADD, ZHIP_EW_SUB, ZHIP_EW_MUL, ZHIP_EW_DIV, ZHIP_EW_POW, ZHIP_EW_MOD, ZHIP_EW_CMPLT, ZHIP_EW_CMPGT,
    ZHIP_EW_CMPGE, ZHIP_EW_MAX, ZHIP_EW_OR, ZHIP_EW_AND, ZHIP_EW_BITXOR, ZHIP_EW_BITOR, ZHIP_EW_BITAND,
    ZHIP_EW_SHL, ZHIP_EW_SHR, ZHIP_EW_NOTEQ, ZHIP_EW_EQ,
    /* operand first: acc = a op acc */
    ZHIP_EW_RSUB, ZHIP_EW_RDIV,
    /* acc = acc != 0 ? a : b   (Tensor::where_ with a true select) */
    ZHIP_EW_WHERE,
    /* acc = acc * a + b        (Op::Mad) */
    ZHIP_EW_MAD,
    /* Tensor-level composites, zyx/src/tensor/elementwise.rs:168-170,289-293,305-307,457-460,585-588 */
    ZHIP_EW_RELU, ZHIP_EW_TANH, ZHIP_EW_GELU, ZHIP_EW_SIGMOID, ZHIP_EW_RSQRT,
    /* Cast to an integer dtype inside a float chain: truncation toward zero (c.rs:243-261) */
    ZHIP_EW_CAST_INT,
    /* acc = d gelu(acc) / d acc: what the reverse rules of zyx/src/graph/autograd.rs:87-134 give for the
     * ops gelu is written in (elementwise.rs:168-170): 0.5(1+t) + 0.5x(1-t^2)*sqrt(2/pi)(1+3*0.044715x^2),
     * t = tanh(sqrt(2/pi)(x+0.044715x^3)) */
    ZHIP_EW_GELU_GRAD,
    ZHIP_EW_OP_COUNT_
};
enum zhip_ew_bcast { ZHIP_EW_FULL = 0, ZHIP_EW_ROW = 1, ZHIP_EW_COL = 2, ZHIP_EW_SCALAR = 3 };
#define ZHIP_EW_SRC_T 0x10
#define ZHIP_EW_SRC_CONST 0x20
#define ZHIP_EW_MAX_INSTR 18

typedef struct zhip_kernel_desc {
    int32_t kind;        /* zhip_kernel_kind */
    int32_t dtype;       /* element dtype of the main operands */
    int32_t out_dtype;   /* result dtype where it may differ */
    int32_t flags;       /* kind specific */
    int64_t dims[8];     /* kind specific sizes, fixed at registration like cblas m,n,k */
    float fparams[8];    /* kind specific scalars */
    int32_t iparams[24]; /* kind specific op codes */
} zhip_kernel_desc;

/* --- linearized kernel IR (what Device::compile receives) ---------------------- */

/* A zyx `Kernel` after linearization is a linear SSA list of `OpNode`s walked from `head` through `next`
 * (zyx/src/kernel/ops.rs:22-147, 353-358). Its image for zhip_compile_ir is
 *     zhip_ir_header | zhip_ir_op[n_ops] in that order | uint32_t extra[n_extra]
 * little endian. `id` is the op's OpId; operands name earlier ids. Ops that only exist before
 * linearization (Move, Reduce) and the tile / tensor-core / assembly ops (Wmma, ReduceTile, MatmulTile,
 * TransposeTile, Asm) have no code here: a kernel holding one is refused with ZHIP_KERNEL_COMPILATION,
 * the answer a backend gives for what it cannot compile (zyx/src/codegen/cuda.rs:56-65).
 *
 *  opcode      dtype   a        b        c       aux                      imm
 *  CONST       yes     -        -        -       -                        value bytes (Constant, dtype.rs)
 *  PARAM       yes     -        -        -       zhip_ir_param_kind       elements the kernel may touch (0 = not checked)
 *  STORAGE     yes     -        -        -       zhip_ir_scope            len
 *  LOAD        -       src      index    -       0 scalar | vector len    -
 *  STORE       -       dst      src      index   0 scalar | vector len    -
 *  CAST        yes     x        -        -       -                        -
 *  UNARY       -       x        -        -       zhip_ir_uop              -
 *  BINARY      -       x        y        -       zhip_ir_bop              -
 *  MAD         -       x        y        z       -                        -
 *  STACK       -       first    count    -       -                        -      (operands = extra[first .. first+count))
 *  DEVECTORIZE -       vec      -        -       lane                     -
 *  INDEX       -       len op   -        -       axis | kind << 8         len for ZHIP_IR_IDX_LOCAL
 *  LOOP        -       len op   -        -       -                        -
 *  IF          -       cond     -        -       -                        -
 *  ENDLOOP, ENDIF, BARRIER: no fields.
 *
 * Kernel arguments are the PARAM ops in list order (zyx/src/codegen/cuda.rs:24-37). Meaning of every op is
 * the C backend's (zyx/src/codegen/c.rs:74-395, 583-612): bf16 / f16 values live in f32 registers, widen on
 * load and truncate on store to global memory; register and local storage of those dtypes holds f32. */
enum zhip_ir_opcode {
    ZHIP_IR_CONST = 0, ZHIP_IR_PARAM, ZHIP_IR_STORAGE, ZHIP_IR_LOAD, ZHIP_IR_STORE, ZHIP_IR_CAST, ZHIP_IR_UNARY,
    ZHIP_IR_BINARY, ZHIP_IR_MAD, ZHIP_IR_STACK, ZHIP_IR_DEVECTORIZE, ZHIP_IR_INDEX, ZHIP_IR_LOOP, ZHIP_IR_ENDLOOP,
    ZHIP_IR_IF, ZHIP_IR_ENDIF, ZHIP_IR_BARRIER,
    /* refused: */
    ZHIP_IR_WMMA, ZHIP_IR_REDUCE_TILE, ZHIP_IR_MATMUL_TILE, ZHIP_IR_TRANSPOSE_TILE, ZHIP_IR_ASM, ZHIP_IR_MOVE, ZHIP_IR_REDUCE
};
/* ParamKind (ops.rs:11-19), MemScope (kernel/mod.rs:203-212), IdxKind (ops.rs:158-166) */
enum zhip_ir_param_kind { ZHIP_IR_VARIABLE = 0, ZHIP_IR_GLOBAL = 1, ZHIP_IR_GLOBAL_MUT = 2 };
enum zhip_ir_scope { ZHIP_IR_SCOPE_GLOBAL = 0, ZHIP_IR_SCOPE_LOCAL = 1, ZHIP_IR_SCOPE_REGISTER = 2, ZHIP_IR_SCOPE_CIRCULAR = 3 };
enum zhip_ir_idx_kind { ZHIP_IR_IDX_GROUP = 0, ZHIP_IR_IDX_LOCAL = 1, ZHIP_IR_IDX_WARP = 2 };
/* UOp (ops.rs:187-213) and BOp (ops.rs:221-260) discriminants */
enum zhip_ir_uop {
    ZHIP_IR_NEG = 0, ZHIP_IR_BITNOT, ZHIP_IR_EXP, ZHIP_IR_EXP2, ZHIP_IR_LN, ZHIP_IR_LOG2, ZHIP_IR_RECIPROCAL, ZHIP_IR_SQRT,
    ZHIP_IR_SIN, ZHIP_IR_COS, ZHIP_IR_FLOOR, ZHIP_IR_TRUNC, ZHIP_IR_ABS
};
enum zhip_ir_bop {
    ZHIP_IR_ADD = 0, ZHIP_IR_SUB, ZHIP_IR_MUL, ZHIP_IR_DIV, ZHIP_IR_POW, ZHIP_IR_MOD, ZHIP_IR_CMPLT, ZHIP_IR_CMPGT,
    ZHIP_IR_CMPGE, ZHIP_IR_MAX, ZHIP_IR_OR, ZHIP_IR_AND, ZHIP_IR_BITXOR, ZHIP_IR_BITOR, ZHIP_IR_BITAND,
    ZHIP_IR_SHL, ZHIP_IR_SHR, ZHIP_IR_NOTEQ, ZHIP_IR_EQ
};
#define ZHIP_IR_MAGIC 0x3152495au /* "ZIR1" */
#define ZHIP_IR_NULL 0xffffffffu  /* OpId::NULL */
#define ZHIP_IR_MAX_PARAMS 32
typedef struct zhip_ir_header {
    uint32_t magic, n_ops, n_extra, reserved;
} zhip_ir_header;
typedef struct zhip_ir_op {
    uint32_t id;
    uint16_t opcode; /* zhip_ir_opcode */
    uint16_t dtype;  /* zhip_dtype where the table says so */
    uint32_t a, b, c, aux;
    uint64_t imm;
} zhip_ir_op;

/* --- host-side random numbers ---------------------------------------------------- */

/* zyx draws every random tensor on the host from one generator (zyx/src/rng.rs: xoshiro256++ seeded by four
 * splitmix64 rounds; default seed 42069, zyx/src/runtime.rs:178) and uploads it. These calls restate it, so seeded
 * inputs match the reference's element for element. No device and no context are involved.
 * zhip_rng_fill draws n elements in order:
 *   ZHIP_RNG_RAND     Tensor::rand (zyx/src/tensor/mod.rs:516-597): F32 in [0, 1] via next_f32 (rng.rs:98-110), or
 *                     the low bytes of one 64-bit draw per element for U8..U64 / I8..I64;
 *   ZHIP_RNG_UNIFORM  Tensor::uniform (mod.rs:637-648), F32: rand * (hi - lo) + lo;
 *   ZHIP_RNG_RANDN    Tensor::randn (mod.rs:603-613), F32: cos(2 pi u0) * sqrt(-2 ln(1 - u1)) over one rand([2, n])
 *                     draw (all u0 first, then all u1), multiplied by hi when hi != 0; cos / ln / sqrt are the host
 *                     libm's (the reference evaluates them on whatever device runs the kernel);
 *   ZHIP_RNG_RANDINT  Tensor::randint (mod.rs:653-660, Rng::range rng.rs:186-208), I32 / I64 in [lo, hi):
 *                     next_u64 % (hi - lo) + lo.
 * Returns ZHIP_INCORRECT_KERNEL_ARG for a dtype the kind does not produce. */
typedef struct zhip_rng { uint64_t s[4]; } zhip_rng;
enum zhip_rng_kind { ZHIP_RNG_RAND = 0, ZHIP_RNG_UNIFORM = 1, ZHIP_RNG_RANDN = 2, ZHIP_RNG_RANDINT = 3 };
void zhip_rng_seed(zhip_rng *rng, uint64_t seed);
uint64_t zhip_rng_next_u64(zhip_rng *rng);
int32_t zhip_rng_fill(zhip_rng *rng, int32_t kind, int32_t dtype, void *out, uint64_t n, double lo, double hi);

/* --- backend lifetime ------------------------------------------------------- */

/* Number of usable GPUs (device enumeration of hip.rs:190-215). */
int32_t zhip_device_count(int32_t *count);
/* initialize_device (hip.rs:122-339): context, pool stream, 8 launch streams. */
int32_t zhip_init(const zhip_config *cfg, zhip_ctx **out);
/* HIPMemoryPool::deinitialize + HIPDevice::deinitialize (hip.rs:341-347, 489-493):
 * drains streams, frees every buffer, program and event. */
int32_t zhip_deinit(zhip_ctx *ctx);
/* Message of the last failed call on ctx (ctx == NULL: last failed zhip_init /
 * zhip_device_count on this thread). BackendError.context, zyx/src/error.rs:107-111. */
const char *zhip_last_error(zhip_ctx *ctx);
/* HIPDevice::info (hip.rs:495-497) */
int32_t zhip_get_device_info(zhip_ctx *ctx, zhip_device_info *info);
/* HIPMemoryPool::free_bytes (hip.rs:350): bookkeeping counter, not a driver query. */
uint64_t zhip_free_bytes(zhip_ctx *ctx);
/* HIPDevice::free_compute (hip.rs:726-728): device-selection weight. */
uint64_t zhip_free_compute(zhip_ctx *ctx);

/* --- memory pool ------------------------------------------------------------ */

/* HIPMemoryPool::allocate (hip.rs:354-370). Fails with ZHIP_MEMORY_ALLOCATION when
 * bytes > free_bytes. *ev is the event the first user must wait on (0 when the
 * block is ready at once). */
int32_t zhip_alloc(zhip_ctx *ctx, uint64_t bytes, zhip_buf *buf, zhip_event *ev);
/* HIPMemoryPool::deallocate (hip.rs:373-385). Consumes evs. */
int32_t zhip_free(zhip_ctx *ctx, zhip_buf buf, const zhip_event *evs, size_t n_evs);
/* MemoryPool::store_variable / get_variable (backend/mod.rs:597-621): scalar kernel
 * arguments live in the buffer id space; value = up to 8 little-endian bytes. */
int32_t zhip_store_variable(zhip_ctx *ctx, int32_t dtype, const uint8_t value[8], zhip_buf *buf);
int32_t zhip_get_variable(zhip_ctx *ctx, zhip_buf buf, int32_t *found, int32_t *dtype, uint8_t value[8]);
/* HIPMemoryPool::host_to_pool (hip.rs:387-409): async; src must stay valid until
 * *ev is synced. Consumes evs. */
int32_t zhip_h2d(zhip_ctx *ctx, const void *src, uint64_t bytes, zhip_buf dst, const zhip_event *evs, size_t n_evs,
                 zhip_event *ev);
/* HIPMemoryPool::pool_to_host (hip.rs:411-434): blocks until the bytes are in dst.
 * Consumes evs. */
int32_t zhip_d2h(zhip_ctx *ctx, zhip_buf src, void *dst, uint64_t bytes, const zhip_event *evs, size_t n_evs);
/* MemoryPool::pool_to_pool with a device source (backend/mod.rs:743-764, todo!() for
 * HIP in the reference): device-to-device copy of `bytes` from src + src_offset to
 * dst + dst_offset inside this pool. Consumes evs. */
int32_t zhip_d2d(zhip_ctx *ctx, zhip_buf src, uint64_t src_offset, zhip_buf dst, uint64_t dst_offset, uint64_t bytes,
                 const zhip_event *evs, size_t n_evs, zhip_event *ev);
/* HIPMemoryPool::sync_events (hip.rs:440-448): wait, then destroy. */
int32_t zhip_sync_events(zhip_ctx *ctx, const zhip_event *evs, size_t n_evs);
/* HIPMemoryPool::release_events (hip.rs:451-458): destroy without waiting. */
int32_t zhip_release_events(zhip_ctx *ctx, const zhip_event *evs, size_t n_evs);
/* Raw device address and size of a buffer (HIPBuffer{ptr,bytes}, hip.rs:85-88), for
 * interop with other code on the same device. */
int32_t zhip_buffer_ptr(zhip_ctx *ctx, zhip_buf buf, void **ptr, uint64_t *bytes);

/* --- device ----------------------------------------------------------------- */

/* AOT registration: validates desc and returns a program id, the role
 * `self.programs.push(..)` plays in CblasDevice::match_graph (cblas.rs:225). */
int32_t zhip_register_kernel(zhip_ctx *ctx, const zhip_kernel_desc *desc, zhip_prog *prog);
/* Device::compile (backend/mod.rs:899-933; the HIP backend's own body is `todo!()`, hip.rs:598-646): turns a
 * linearized kernel (image described above) into HIP source, the way generate_cuda does for CUDA
 * (zyx/src/codegen/cuda.rs:18-396), and compiles it for this device with hiprtc. Grid = the Group index
 * lengths (a constant, or a Variable parameter read at launch: GwsDim, backend/mod.rs:60-98), block = the
 * Local index lengths. A launch takes one argument per PARAM, in order: a zhip_store_variable id for a
 * Variable, a memory buffer otherwise. ZHIP_KERNEL_COMPILATION with the reason in zhip_last_error when the
 * image is malformed, uses an op this backend has no code for, or does not compile. */
int32_t zhip_compile_ir(zhip_ctx *ctx, const void *ir, uint64_t ir_bytes, zhip_prog *prog);
/* Code objects built at run time (zhip_compile_ir, large elementwise chains) are cached like the shared objects of
 * the reference's C backend (zyx/src/backend/c.rs:165-186): in memory for the life of the process and on disk under
 * $ZYX_HIP_CACHE_DIR, else $XDG_CONFIG_HOME/zyx/cache/hip, else $HOME/.config/zyx/cache/hip, keyed by a hash of the
 * source text, the compiler options and the hiprtc version; ZYX_HIP_CACHE=0 switches the disk part off. A file that
 * is truncated or fails its check word is ignored and rebuilt. counts[0..3] = compilations, memory hits, disk hits
 * of this process so far. */
void zhip_compile_cache_stats(uint64_t counts[3]);
/* Source generation alone, no device and no context needed: checks the image and writes the HIP source
 * zhip_compile_ir would compile (ZHIP_OK), or the reason it is refused (ZHIP_KERNEL_COMPILATION), into buf
 * (up to cap - 1 bytes plus a terminator; *len = full length). */
int32_t zhip_ir_generate(const void *ir, uint64_t ir_bytes, char *buf, uint64_t cap, uint64_t *len);
/* The HIP source zhip_compile_ir generated for `prog` (what ZYX_DEBUG=16 prints, hip.rs:560-580): copies up
 * to cap - 1 bytes plus a terminator into buf, *len = full length. Programs registered with
 * zhip_register_kernel have none (*len = 0). */
int32_t zhip_program_source(zhip_ctx *ctx, zhip_prog prog, char *buf, uint64_t cap, uint64_t *len);
/* HIPDevice::launch (hip.rs:654-719). args = inputs then outputs; every argument is
 * checked against the size the program needs before anything is enqueued. Consumes evs. */
int32_t zhip_launch(zhip_ctx *ctx, zhip_prog prog, const zhip_buf *args, size_t n_args, const zhip_event *evs,
                    size_t n_evs, zhip_event *ev);
/* HIPDevice::release (hip.rs:721-724). Refused (ZHIP_INCORRECT_KERNEL_ARG) while a live plan contains the
 * program. Launches of one program that owns scratch memory are ordered among themselves even when their wait
 * lists are unrelated. */
int32_t zhip_release_program(zhip_ctx *ctx, zhip_prog prog);
/* launch_with_timings (zyx/src/kernel/autotune.rs:775-798): launch, sync, host
 * wall-clock nanoseconds -- the value for Node::Kernel.time (graph/mod.rs:177-182). */
int32_t zhip_time_kernel(zhip_ctx *ctx, zhip_prog prog, const zhip_buf *args, size_t n_args, uint64_t *ns);
/* Device-side duration: `iters` back-to-back launches bracketed by HIP events on the
 * stream they run on; *avg_us = mean microseconds per launch. arg_sets > 1 cycles
 * through that many consecutive argument tuples (args holds arg_sets * n_args ids) so
 * successive launches touch different memory. */
int32_t zhip_profile_kernel(zhip_ctx *ctx, zhip_prog prog, const zhip_buf *args, size_t n_args, size_t arg_sets,
                            int32_t iters, float *avg_us);

/* No counterpart in the reference: an entry point for callers that cannot allocate device memory -- code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. It is the ZHIP_K_REDUCE kernel pair
 * (sum: op = 0, max: op = 1; over the last axis: axis0 = 0, over axis 0: axis0 = 1; dtype F32 / BF16 / F16 / I32,
 * no scale / base epilogue) on raw device pointers x[rows, cols] -> out[rows] or out[cols], enqueued on the
 * caller's `stream` (a hipStream_t, NULL = the null stream) of ctx's device; asynchronous, the caller orders it
 * against its other work. The partial results of the two-stage variants go to a 1 MiB array that is part of the
 * library's code object (one copy per GPU, held until the process ends) instead of a per-program allocation:
 * no hipMalloc, hipFree or other allocating routine is called. A shape whose partials need more than 1 MiB is
 * refused with ZHIP_KERNEL_COMPILATION and the needed size in zhip_last_error (register the kernel instead).
 * Results are bit-identical to a ZHIP_K_REDUCE program launched with zhip_launch on the same data. All calls on one
 * GPU share the array: calls that overlap in time on one GPU (different streams, different contexts) race on it,
 * so the caller keeps them in one stream or orders them; nothing in it has to be cleared between calls (every
 * partial a call reads it has written itself). */
int32_t zhip_reduce_static(zhip_ctx *ctx, int32_t dtype, int32_t op, int32_t axis0, int64_t rows, int64_t cols,
                           const void *x, void *out, void *stream);

/* Ceilings measured on this device as it runs now. DeviceInfo.compute (zyx/src/backend/mod.rs:506-531) is a nominal
 * figure; like the reference's autotuner (zyx/src/kernel/autotune.rs:775-798) this call finds out by launching and
 * timing, so that kernel results can be priced against what the part sustains as well as against its data sheet:
 *   memcpy_d2d_GBps   hipMemcpyDtoDAsync of `bytes`, read + written bytes per second;
 *   copy_kernel_GBps  a plain 128-bit streaming copy kernel over the same buffers, read + written;
 *   read_kernel_GBps  a read-only sum over `bytes`;
 *   mfma_bf16_*       one wave per SIMD issuing 4096 v_mfma_f32_32x32x16_bf16 from registers (no memory traffic),
 *                     with constant operands and with uniform(-1, 1) operands that change from instruction to
 *                     instruction (real data draws more power, and the clock follows): TFLOP/s over the in-kernel
 *                     duration, the shader clock read inside the kernel, and the launch-to-launch time in a queue of
 *                     such launches.
 * Allocates 2 x bytes of device memory for the duration of the call (bytes >= 1 MiB); blocks until done. */
typedef struct zhip_ceilings {
    float memcpy_d2d_GBps, copy_kernel_GBps, read_kernel_GBps;
    float mfma_bf16_const_TFLOPs, mfma_bf16_const_MHz, mfma_bf16_const_launch_us;
    float mfma_bf16_random_TFLOPs, mfma_bf16_random_MHz, mfma_bf16_random_launch_us;
} zhip_ceilings;
int32_t zhip_measure_ceilings(zhip_ctx *ctx, uint64_t bytes, zhip_ceilings *out);

/* --- cached execution plans ----------------------------------------------------- */

/* The steady state of Tape::realize / FrozenTape::replay is a fixed list of Launch nodes on
 * fixed buffers (ExecPlan, zyx/src/graph/plan.rs:58-237; replay loop :271-361; plan cache
 * zyx/src/tape.rs:165-181, 299-318). zhip_plan_create records such a list once -- programs
 * in execution order, each with its buffer ids (inputs then outputs), args_flat holding the
 * lists back to back and n_args their lengths -- as a HIP graph on one in-order stream, so a
 * later node sees the results of every earlier one. zhip_plan_launch replays it with one
 * call: it waits for (and consumes) evs, and returns the event of the whole list. Buffers
 * named by a plan must stay alive until zhip_plan_destroy; its programs cannot be released before. */
typedef uint32_t zhip_plan;
int32_t zhip_plan_create(zhip_ctx *ctx, const zhip_prog *progs, const zhip_buf *args_flat, const uint32_t *n_args,
                         size_t n_nodes, zhip_plan *plan);
int32_t zhip_plan_launch(zhip_ctx *ctx, zhip_plan plan, const zhip_event *evs, size_t n_evs, zhip_event *ev);
int32_t zhip_plan_destroy(zhip_ctx *ctx, zhip_plan plan);

#ifdef __cplusplus
}
#endif
#endif /* ZYX_HIP_H */
