"""ctypes front-end of the CPU oracle (``oracle/zyx_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``. The product package ``zyx_amd`` never imports it.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libzyx_oracle.so")

# dtype codes, in the order of zyx/src/dtype.rs:20-47
BF16, F16, F32, F64, U8, U16, U32, U64, I8, I16, I32, I64, BOOL = range(13)

UNARY = dict(neg=0, exp=1, exp2=2, ln=3, log2=4, reciprocal=5, sqrt=6, sin=7, cos=8, floor=9, trunc=10, abs=11,
             relu=32, tanh=33, gelu=34, sigmoid=35, rsqrt=36)
BINARY = dict(add=0, sub=1, mul=2, div=3, pow=4, mod=5, cmplt=6, cmpgt=7, max=8, noteq=9, eq=10, cmpge=11)


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few seconds)."""
    src = os.path.join(_HERE, "zyx_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libzyx_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.zo_rng_next_u64.restype = C.c_uint64
    return _lib


def _p(a: np.ndarray | None):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


_I64 = C.c_int64


class Rng:
    """zyx's xoshiro256++ generator (zyx/src/rng.rs); default seed 42069 (zyx/src/runtime.rs:178)."""

    def __init__(self, seed: int = 42069):
        self._s = (C.c_uint64 * 4)()
        lib().zo_rng_seed(self._s, C.c_uint64(seed))

    def next_u64(self) -> int:
        return lib().zo_rng_next_u64(self._s)

    def rand_u8(self, n: int) -> np.ndarray:
        out = np.empty(n, np.uint8)
        lib().zo_rand_u8(self._s, _p(out), _I64(n))
        return out

    def rand(self, shape) -> np.ndarray:
        out = np.empty(shape, np.float32)
        lib().zo_rand_f32(self._s, _p(out), _I64(out.size))
        return out

    def uniform(self, shape, lo: float, hi: float) -> np.ndarray:
        out = np.empty(shape, np.float32)
        lib().zo_uniform_f32(self._s, _p(out), _I64(out.size), C.c_float(lo), C.c_float(hi))
        return out

    def randn(self, shape, scale: float = 1.0) -> np.ndarray:
        out = np.empty(shape, np.float32)
        lib().zo_randn_f32(self._s, _p(out), _I64(out.size), C.c_float(scale))
        return out

    def randint(self, shape, lo: int, hi: int) -> np.ndarray:
        out = np.empty(shape, np.int32)
        lib().zo_randint_i32(self._s, _p(out), _I64(out.size), _I64(lo), _I64(hi))
        return out


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().zo_f32_to_bf16(_p(x), _p(y), _I64(x.size))
    return y


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.uint16)
    y = np.empty(x.shape, np.float32)
    lib().zo_bf16_to_f32(_p(x), _p(y), _I64(x.size))
    return y


def f32_to_f16(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().zo_f32_to_f16(_p(x), _p(y), _I64(x.size))
    return y


def f16_to_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.uint16)
    y = np.empty(x.shape, np.float32)
    lib().zo_f16_to_f32(_p(x), _p(y), _I64(x.size))
    return y


def _store_dtype(code: int):
    return np.float32 if code == F32 else np.uint16


def unary(op: str, x: np.ndarray, dtype: int = F32) -> np.ndarray:
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    y = np.empty_like(x)
    lib().zo_unary_map(UNARY[op], dtype, _p(x), _p(y), _I64(x.size))
    return y


def binary(op: str, x: np.ndarray, y: np.ndarray, dtype: int = F32) -> np.ndarray:
    """x: [rows, cols] (or any shape, flattened to rows x last); y: same shape, [cols] or scalar."""
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    y = np.ascontiguousarray(y, _store_dtype(dtype))
    cols = x.shape[-1] if x.ndim else 1
    rows = x.size // max(cols, 1)
    if y.size == x.size:
        bc = 0
    elif y.size == 1:
        bc = 2
    else:
        assert y.size == cols, "row-vector broadcast only"
        bc = 1
    z = np.empty_like(x)
    lib().zo_binary_map(BINARY[op], dtype, _p(x), _p(y), _p(z), _I64(rows), _I64(cols), bc)
    return z


def reduce_rows(op: str, x: np.ndarray, dtype: int = F32) -> np.ndarray:
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    rows, cols = x.shape
    y = np.empty(rows, x.dtype)
    lib().zo_reduce_rows(0 if op == "sum" else 1, dtype, _p(x), _p(y), _I64(rows), _I64(cols))
    return y


def reduce_cols(op: str, x: np.ndarray, dtype: int = F32) -> np.ndarray:
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    rows, cols = x.shape
    y = np.empty(cols, x.dtype)
    lib().zo_reduce_cols(0 if op == "sum" else 1, dtype, _p(x), _p(y), _I64(rows), _I64(cols))
    return y


def reduce_rows_i32(op: str, x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.int32)
    rows, cols = x.shape
    y = np.empty(rows, np.int32)
    lib().zo_reduce_rows_i32(0 if op == "sum" else 1, _p(x), _p(y), _I64(rows), _I64(cols))
    return y


def softmax_rows(x: np.ndarray, want_y=True, want_sum=True, want_arg=True, dtype: int = F32):
    """Returns (y, rowsum, argmax) of the reference's softmax -> sum / argmax_axis(-1) chain. dtype BF16 / F16: x, y and
    rowsum are bit patterns (uint16); y is narrowed on store and the sum and argmax read the stored y."""
    if dtype != F32:
        x = np.ascontiguousarray(x, np.uint16)
        rows, cols = x.shape
        y = np.empty_like(x) if want_y else None
        s = np.empty(rows, np.uint16) if want_sum else None
        a = np.empty(rows, np.int32) if want_arg else None
        lib().zo_softmax_rows(dtype, _p(x), _p(y), _p(s), _p(a), _I64(rows), _I64(cols))
        return y, s, a
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    y = np.empty_like(x) if want_y else None
    s = np.empty(rows, np.float32) if want_sum else None
    a = np.empty(rows, np.int32) if want_arg else None
    lib().zo_softmax_rows_f32(_p(x), _p(y), _p(s), _p(a), _I64(rows), _I64(cols))
    return y, s, a


def softmax_rows_f64acc(x: np.ndarray):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    y = np.empty_like(x)
    s = np.empty(rows, np.float32)
    lib().zo_softmax_rows_f64acc(_p(x), _p(y), _p(s), _I64(rows), _I64(cols))
    return y, s


def argmax_rows(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    a = np.empty(rows, np.int32)
    lib().zo_argmax_rows_f32(_p(x), _p(a), _I64(rows), _I64(cols))
    return a


def argmax_axis(x: np.ndarray, axis: int) -> np.ndarray:
    """Tensor::argmax_axis (zyx/src/tensor/mod.rs:2238-2269) for any axis. Float tensors (given as f32 values) go
    through the C row routine on a view with the axis moved last; integer tensors follow the reference's expression
    literally, `max_k((x == max_keepdim(x)) * k)` cast to i32, in numpy integers."""
    x = np.asarray(x)
    axis = axis % x.ndim
    if x.dtype.kind in "iu":
        k = np.arange(x.shape[axis], dtype=np.int64).reshape([-1 if d == axis else 1 for d in range(x.ndim)])
        return ((x == x.max(axis=axis, keepdims=True)) * k).max(axis=axis).astype(np.int32)
    moved = np.moveaxis(x, axis, -1)
    return argmax_rows(np.ascontiguousarray(moved, np.float32).reshape(-1, x.shape[axis])).reshape(moved.shape[:-1])


def matmul(a: np.ndarray, b: np.ndarray, in_dtype: int = F32, out_dtype: int = F32, transb: bool = False,
           transa: bool = False) -> np.ndarray:
    """dot / dot_dtype of zyx/src/tensor/mod.rs:1469-1518 on 2-D operands (a stored [k,m] if transa,
    b stored [n,k] if transb)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    m, k = (a.shape[1], a.shape[0]) if transa else a.shape
    n = b.shape[0] if transb else b.shape[1]
    assert (b.shape[1] if transb else b.shape[0]) == k
    c = np.empty((m, n), _store_dtype(out_dtype))
    lib().zo_matmul_float(in_dtype, out_dtype, _p(a), _p(b), _p(c), _I64(m), _I64(n), _I64(k), int(transb), int(transa))
    return c


def matmul_f64acc(a: np.ndarray, b: np.ndarray, in_dtype: int = F32, transb: bool = False) -> np.ndarray:
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    m, k = a.shape
    n = b.shape[0] if transb else b.shape[1]
    c = np.empty((m, n), np.float64)
    lib().zo_matmul_f64acc(in_dtype, _p(a), _p(b), _p(c), _I64(m), _I64(n), _I64(k), int(transb))
    return c


def matmul_int(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), a.dtype)
    fn = lib().zo_matmul_i64 if a.dtype == np.int64 else lib().zo_matmul_i32
    fn(_p(a), _p(b), _p(c), _I64(m), _I64(n), _I64(k))
    return c


def bias_act(c: np.ndarray, bias: np.ndarray | None, act: str = "none", bias_dtype: int = F32) -> np.ndarray:
    c = np.array(c, np.float32, copy=True, order="C")
    m, n = c.shape
    lib().zo_bias_act_f32(_p(c), _p(None if bias is None else np.ascontiguousarray(bias)), bias_dtype, _I64(m), _I64(n),
                          dict(none=0, relu=1, gelu=2)[act])
    return c


def ew_chain(chain, arrays) -> np.ndarray:
    """Evaluate a `zyx_amd.kernels.Chain` on the CPU with the reference's op semantics."""
    np_store = {F32: np.float32, BF16: np.uint16, F16: np.uint16, I32: np.int32, U8: np.uint8, BOOL: np.uint8}
    n_in = len(chain.inputs)
    arrs = [np.ascontiguousarray(a, np_store[int(chain.inputs[k][0])]) for k, a in enumerate(arrays)]
    in_desc = (C.c_int32 * 4)(*[int(dt) | (bc << 8) for dt, bc in chain.inputs])
    ptrs = (C.c_void_p * 4)(*[a.ctypes.data for a in arrs])
    code = (C.c_uint32 * 18)(*chain.code)
    consts = (C.c_float * 8)(*chain.consts)
    out = np.empty((chain.rows, chain.cols), np_store[int(chain.out_dtype)])
    lib().zo_ew_chain(int(chain.reg), int(chain.out_dtype), n_in, in_desc, ptrs, len(chain.code), code, consts, _p(out),
                      _I64(chain.rows), _I64(chain.cols))
    return out


def layer_norm(x, w=None, b=None, eps: float = 1e-5, dtype: int = F32) -> np.ndarray:
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    rows, cols = x.shape
    y = np.empty_like(x)
    w = None if w is None else np.ascontiguousarray(w, x.dtype)
    b = None if b is None else np.ascontiguousarray(b, x.dtype)
    lib().zo_layer_norm(dtype, _p(x), _p(w), _p(b), _p(y), _I64(rows), _I64(cols), C.c_float(eps))
    return y


def rms_norm(x, w=None, eps: float = 1e-6, dtype: int = F32) -> np.ndarray:
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    rows, cols = x.shape
    y = np.empty_like(x)
    w = None if w is None else np.ascontiguousarray(w, x.dtype)
    lib().zo_rms_norm(dtype, _p(x), _p(w), _p(y), _I64(rows), _I64(cols), C.c_float(eps))
    return y


def cross_entropy(logits, labels, gscale: float | None = None):
    """-> (per-sample loss [rows], grad of gscale*sum(loss) or None)."""
    x = np.ascontiguousarray(logits, np.float32)
    lab = np.ascontiguousarray(labels, np.int32)
    rows, cols = x.shape
    loss = np.empty(rows, np.float32)
    grad = np.empty_like(x) if gscale is not None else None
    lib().zo_cross_entropy(_p(x), _p(lab), _p(loss), _p(grad), _I64(rows), _I64(cols), C.c_float(gscale or 0.0))
    return loss, grad


def mlp_step(x, labels, w1, b1, w2, b2, lr: float):
    """One SGD step of the 2-layer MLP of config 1 (Linear -> ReLU -> Linear -> cross_entropy mean),
    composed from the oracle's primitives in the order zyx's Tape would evaluate them:
      forward  zyx-nn/src/linear.rs:38-44 (x . W^T + b), relu = (x > 0) * x
      backward zyx/src/graph/autograd.rs: Mul :120-125 (relu mask, dot products), Add :111-119 (bias:
               gradient summed over the broadcast batch axis), dot = broadcast-mul + sum(-1)
      update   zyx-optim/src/sgd.rs:77-81 p <- p - g * lr
    Returns (mean loss, new w1, b1, w2, b2, dict of gradients)."""
    n = x.shape[0]
    pre = bias_act(matmul(x, w1, transb=True), b1, "none")
    h = unary("relu", pre)
    logits = bias_act(matmul(h, w2, transb=True), b2, "none")
    loss, dlogits = cross_entropy(logits, labels, 1.0 / n)
    dw2 = matmul(dlogits, h, transa=True)            # [out2, n] . [n, hidden]
    db2 = reduce_cols("sum", dlogits)
    dh = matmul(dlogits, w2)                           # [n, out2] . [out2, hidden]
    dpre = binary("mul", binary("cmpgt", pre, np.float32(0.0)), dh)
    dw1 = matmul(dpre, x, transa=True)
    db1 = reduce_cols("sum", dpre)
    lr32 = np.float32(lr)
    upd = lambda p, g: binary("sub", p, binary("mul", g, lr32))
    grads = dict(w1=dw1, b1=db1, w2=dw2, b2=db2, logits=dlogits)
    mean_loss = np.float32(reduce_rows("sum", loss[None, :])[0] / np.float32(n))
    return mean_loss, upd(w1, dw1), upd(b1[None, :], db1[None, :])[0], upd(w2, dw2), upd(b2[None, :], db2[None, :])[0], grads


def conv2d(x, w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1), relu=False, dtype: int = F32,
           out_dtype: int | None = None) -> np.ndarray:
    """Tensor::conv on NCHW x and weight [Cout, C, KH, KW], groups = 1."""
    out_dtype = dtype if out_dtype is None else out_dtype
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    w = np.ascontiguousarray(w, _store_dtype(dtype))
    b = None if bias is None else np.ascontiguousarray(bias, _store_dtype(dtype))
    n, c, h, wd = x.shape
    co, _, kh, kw = w.shape
    oh = (h + 2 * padding[0] - dilation[0] * (kh - 1) - 1) // stride[0] + 1
    ow = (wd + 2 * padding[1] - dilation[1] * (kw - 1) - 1) // stride[1] + 1
    y = np.empty((n, co, oh, ow), _store_dtype(out_dtype))
    lib().zo_conv2d(dtype, out_dtype, _p(x), _p(w), _p(b), _p(y), _I64(n), _I64(c), _I64(h), _I64(wd), _I64(co), _I64(kh),
                    _I64(kw), stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], int(relu))
    return y


def max_pool2d(x, kernel=(2, 2), stride=(2, 2), padding=(0, 0), dilation=(1, 1), dtype: int = F32) -> np.ndarray:
    x = np.ascontiguousarray(x, _store_dtype(dtype))
    h, wd = x.shape[-2:]
    planes = x.size // (h * wd)
    oh = (h + 2 * padding[0] - dilation[0] * (kernel[0] - 1) - 1) // stride[0] + 1
    ow = (wd + 2 * padding[1] - dilation[1] * (kernel[1] - 1) - 1) // stride[1] + 1
    y = np.empty(x.shape[:-2] + (oh, ow), x.dtype)
    lib().zo_max_pool2d(dtype, _p(x), _p(y), _I64(planes), _I64(h), _I64(wd), _I64(kernel[0]), _I64(kernel[1]), stride[0],
                        stride[1], padding[0], padding[1], dilation[0], dilation[1])
    return y


# ---- gather / scatter / index_select: zyx/src/tensor/index_ops.rs:321-445 (numpy restatement) -------------
def _wrap_index(idx: np.ndarray, dim: int):
    idx = idx.astype(np.int64)
    idx = idx + (idx < 0) * dim          # one wrap: idx + (idx < 0) * dim_size  (:342-343)
    return idx, (idx >= 0) & (idx < dim)  # an index still out of range has an all-zero one-hot (:315-316)


def gather(x: np.ndarray, axis: int, indices: np.ndarray) -> np.ndarray:
    """out[i] = sum_k onehot(idx[i])[k] * x[.., k, ..] over x shrunk to the index tensor's extent."""
    axis %= x.ndim
    idx, ok = _wrap_index(np.asarray(indices), x.shape[axis])
    sl = tuple(slice(None) if d == axis else slice(0, idx.shape[d]) for d in range(x.ndim))
    vals = np.take_along_axis(x[sl], np.where(ok, idx, 0), axis)
    return np.where(ok, vals, np.zeros((), x.dtype)).astype(x.dtype)


def index_select(x: np.ndarray, axis: int, index: np.ndarray) -> np.ndarray:
    axis %= x.ndim
    shape = [1] * x.ndim
    shape[axis] = len(index)
    full = list(x.shape)
    full[axis] = len(index)
    return gather(x, axis, np.broadcast_to(np.asarray(index).reshape(shape), full))


def scatter(x: np.ndarray, axis: int, indices: np.ndarray, src: np.ndarray) -> np.ndarray:
    """self + sum over index positions j (ascending along `axis`) of onehot(idx[.., j, ..]) * src[.., j, ..]."""
    axis %= x.ndim
    idx, ok = _wrap_index(np.asarray(indices), x.shape[axis])
    contrib = np.zeros_like(x)
    grids = np.meshgrid(*[np.arange(n) for n in idx.shape], indexing="ij")
    for j in range(idx.shape[axis]):
        sel = tuple(slice(j, j + 1) if d == axis else slice(None) for d in range(x.ndim))
        tgt = [g[sel] for g in grids]
        tgt[axis] = idx[sel]
        m = ok[sel]
        np.add.at(contrib, tuple(t[m] for t in tgt), np.asarray(src, x.dtype)[sel][m])  # targets are distinct within one j
    return (contrib + x).astype(x.dtype)


# ---- attention: zyx-nn/src/causal_self_attention.rs:36-74 ----------------------------------------------------
def attention(qkv: np.ndarray, n_head: int, scale: float | None = None, dropout_p: float = 0.0, dtype: int = F32,
              want_lse: bool = False, causal: bool = False):
    """Core of CausalSelfAttention::forward on the c_attn output qkv[B,T,3C] -> y[B,T,C] (the reference applies
    no mask). scale defaults to (1/sqrt(dh)) as f32; eval-mode dropout divides the probabilities by 1-p.
    causal: query t sees keys 0..t only (scores of later keys filled with -inf before the softmax)."""
    qkv = np.ascontiguousarray(qkv, _store_dtype(dtype))
    b, t, c3 = qkv.shape
    c = c3 // 3
    dh = c // n_head
    scale = np.float32(1.0 / np.sqrt(float(dh))) if scale is None else np.float32(scale)
    y = np.empty((b, t, c), qkv.dtype)
    lse = np.empty((b, n_head, t), np.float32) if want_lse else None
    lib().zo_attention(dtype, _p(qkv), _p(y), _p(lse), _I64(b), _I64(t), _I64(n_head), _I64(dh), C.c_float(scale),
                       C.c_float(np.float32(1.0) - np.float32(dropout_p)), C.c_int(int(causal)))
    return (y, lse) if want_lse else y


def attention_bwd(qkv: np.ndarray, dy: np.ndarray, n_head: int, scale: float | None = None, dropout_p: float = 0.0,
                  dtype: int = F32, causal: bool = False) -> np.ndarray:
    """d(sum(y * dy)) / d(qkv) for `attention`, f64 arithmetic, stored in `dtype`."""
    qkv = np.ascontiguousarray(qkv, _store_dtype(dtype))
    dy = np.ascontiguousarray(dy, qkv.dtype)
    b, t, c3 = qkv.shape
    dh = c3 // 3 // n_head
    scale = np.float32(1.0 / np.sqrt(float(dh))) if scale is None else np.float32(scale)
    out = np.empty_like(qkv)
    lib().zo_attention_bwd(dtype, _p(qkv), _p(dy), _p(out), _I64(b), _I64(t), _I64(n_head), _I64(dh), C.c_float(scale),
                           C.c_float(np.float32(1.0) - np.float32(dropout_p)), C.c_int(int(causal)))
    return out


def linear(x: np.ndarray, w: np.ndarray, bias: np.ndarray | None = None, dtype: int = F32, act: str = "none") -> np.ndarray:
    """Linear::forward (zyx-nn/src/linear.rs:38-44): x.dot(w^T) + b over the last axis, w stored [out, in]; f32
    registers, one store in `dtype` after the optional activation."""
    lead = x.shape[:-1]
    c = matmul(x.reshape(-1, x.shape[-1]), w, dtype, F32, transb=True)
    if bias is not None or act != "none":
        c = bias_act(c, bias, act, dtype if bias is not None else F32)
    if dtype == BF16:
        c = f32_to_bf16(c)
    elif dtype == F16:
        c = f32_to_f16(c)
    return c.reshape(*lead, w.shape[0])


def causal_self_attention(x, w_attn, w_proj, n_head: int, b_attn=None, b_proj=None, dropout_p: float = 0.0,
                          dtype: int = F32) -> np.ndarray:
    """CausalSelfAttention::forward, tensors materialised (stored in `dtype`) after c_attn, att.dot(v), c_proj."""
    qkv = linear(x, w_attn, b_attn, dtype)
    y = attention(qkv, n_head, None, dropout_p, dtype)
    return linear(y, w_proj, b_proj, dtype)


def norm_bwd(x, dy, w=None, add=None, rms: bool = False, eps: float = 1e-5, dtype: int = F32, want_db: bool = True):
    """Gradients of layer_norm / rms_norm: (dx (+ add), dw or None, db or None)."""
    st = _store_dtype(dtype)
    x = np.ascontiguousarray(x, st)
    rows, cols = x.shape
    dy = np.ascontiguousarray(dy, st)
    w = None if w is None else np.ascontiguousarray(w, st)
    add = None if add is None else np.ascontiguousarray(add, st)
    dx = np.empty_like(x)
    dw = np.empty(cols, st) if w is not None else None
    db = np.empty(cols, st) if want_db and not rms else None
    lib().zo_norm_bwd(dtype, int(rms), _p(x), _p(w), _p(dy), _p(add), _p(dx), _p(dw), _p(db), _I64(rows), _I64(cols),
                      C.c_float(eps))
    return dx, dw, db


# ---- pre-norm transformer block: zyx-examples/examples/nanogpt.rs:41-98 over zyx-nn modules --------------------
def _gelu64(v):
    return 0.5 * v * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (v + 0.044715 * v ** 3)))


def block_forward_f64(p: dict, x: np.ndarray, n_head: int, eps: float = 1e-5, causal: bool = False) -> dict:
    """x[B,T,d] -> every module output of `x + attn(ln_1(x)); x + mlp(ln_2(x))` in f64 (numpy). LayerNorm uses the
    unbiased variance (zyx-nn/src/layer_norm.rs:98-135), attention applies no mask
    (zyx-nn/src/causal_self_attention.rs:36-74), gelu is the tanh form (zyx/src/tensor/elementwise.rs:168-170)."""
    B, T, d = x.shape
    dh = d // n_head
    f = {k: np.asarray(v, np.float64) for k, v in p.items()}

    def ln(v, w, b):
        mu = v.mean(-1, keepdims=True)
        var = ((v - mu) ** 2).sum(-1, keepdims=True) / (d - 1)
        return (v - mu) / np.sqrt(var + eps) * w + b

    s = {"x": np.asarray(x, np.float64)}
    s["n1"] = ln(s["x"], f["ln1_w"], f["ln1_b"])
    s["qkv"] = s["n1"] @ f["attn_w"].T + f["attn_b"]
    q, k, v = [a.reshape(B, T, n_head, dh).transpose(0, 2, 1, 3) for a in np.split(s["qkv"], 3, axis=2)]
    sc = np.einsum("bhtd,bhjd->bhtj", q, k) * float(np.float32(1.0 / np.sqrt(float(dh))))
    if causal:  # not part of the reference's module: scores of later keys filled with -inf (probability 0)
        sc = np.where(np.tril(np.ones((T, T), bool)), sc, -np.inf)
    e = np.exp(sc - sc.max(-1, keepdims=True))
    s["probs"] = e / e.sum(-1, keepdims=True)
    s["att"] = np.einsum("bhtj,bhjd->bhtd", s["probs"], v).transpose(0, 2, 1, 3).reshape(B, T, d)
    s["x2"] = s["x"] + s["att"] @ f["proj_w"].T + f["proj_b"]
    s["n2"] = ln(s["x2"], f["ln2_w"], f["ln2_b"])
    s["h"] = s["n2"] @ f["fc_w"].T + f["fc_b"]
    s["g"] = _gelu64(s["h"])
    s["out"] = s["x2"] + s["g"] @ f["proj2_w"].T + f["proj2_b"]
    return s


def block_backward_f64(p: dict, s: dict, dout: np.ndarray, n_head: int, eps: float = 1e-5) -> dict:
    """Gradients of sum(out * dout) with respect to x and every parameter, given block_forward_f64's outputs `s`:
    Runtime::gradient's reverse rules (zyx/src/graph/autograd.rs:14-424) composed per module."""
    B, T, d = s["x"].shape
    dh = d // n_head
    f = {k: np.asarray(v, np.float64) for k, v in p.items()}
    g = {}
    r2 = lambda a: a.reshape(B * T, -1)

    def ln_bwd(v, w, dy):
        mu = v.mean(-1, keepdims=True)
        rstd = 1.0 / np.sqrt(((v - mu) ** 2).sum(-1, keepdims=True) / (d - 1) + eps)
        xh = (v - mu) * rstd
        gg = dy * w
        dx = rstd * (gg - gg.mean(-1, keepdims=True) - xh * (gg * xh).sum(-1, keepdims=True) / (d - 1))
        return dx, r2(dy * xh).sum(0), r2(dy).sum(0)

    def lin_bwd(name, inp, dy):
        g[name + "_w"] = r2(dy).T @ r2(inp)
        g[name + "_b"] = r2(dy).sum(0)
        return dy @ f[name + "_w"]

    dout = np.asarray(dout, np.float64)
    g["dg"] = lin_bwd("proj2", s["g"], dout)
    hv = s["h"]
    k0 = np.sqrt(2.0 / np.pi)
    t = np.tanh(k0 * (hv + 0.044715 * hv ** 3))
    g["dh"] = g["dg"] * (0.5 * (1 + t) + 0.5 * hv * (1 - t * t) * k0 * (1 + 3 * 0.044715 * hv * hv))
    g["dn2"] = lin_bwd("fc", s["n2"], g["dh"])
    dx, g["ln2_w"], g["ln2_b"] = ln_bwd(s["x2"], f["ln2_w"], g["dn2"])
    g["dx2"] = dout + dx
    g["datt"] = lin_bwd("proj", s["att"], g["dx2"])
    q, k, v = [a.reshape(B, T, n_head, dh).transpose(0, 2, 1, 3) for a in np.split(s["qkv"], 3, axis=2)]
    do = g["datt"].reshape(B, T, n_head, dh).transpose(0, 2, 1, 3)
    ps = s["probs"]
    dps = np.einsum("bhtd,bhjd->bhtj", do, v)
    ds = ps * (dps - (ps * dps).sum(-1, keepdims=True))
    sc = float(np.float32(1.0 / np.sqrt(float(dh))))
    back = lambda a: a.transpose(0, 2, 1, 3).reshape(B, T, d)
    g["dqkv"] = np.concatenate([back(np.einsum("bhtj,bhjd->bhtd", ds, k) * sc), back(np.einsum("bhtj,bhtd->bhjd", ds, q) * sc),
                                back(np.einsum("bhtj,bhtd->bhjd", ps, do))], 2)
    g["dn1"] = lin_bwd("attn", s["n1"], g["dqkv"])
    dx, g["ln1_w"], g["ln1_b"] = ln_bwd(s["x"], f["ln1_w"], g["dn1"])
    g["dx"] = g["dx2"] + dx
    return g


def block_init(d_model: int, n_head: int, seed: int = 42069, std: float = 0.02, mlp_ratio: int = 4) -> dict:
    """Parameters of config 5: Linear weights std * randn, Linear biases zero (nanogpt.rs:121-125), LayerNorm
    weight 1 / bias 0 (zyx-nn/src/layer_norm.rs:52-62), drawn in PARAMS order from one seeded generator."""
    r = Rng(seed)
    d, f = d_model, mlp_ratio * d_model
    z = lambda *s: np.zeros(s, np.float32)
    return dict(ln1_w=np.ones(d, np.float32), ln1_b=z(d), attn_w=r.randn((3 * d, d), std), attn_b=z(3 * d),
                proj_w=r.randn((d, d), std), proj_b=z(d), ln2_w=np.ones(d, np.float32), ln2_b=z(d),
                fc_w=r.randn((f, d), std), fc_b=z(f), proj2_w=r.randn((d, f), std), proj2_b=z(d))
