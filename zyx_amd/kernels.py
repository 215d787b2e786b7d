"""Descriptors of the hand-written kernels (`zhip_kernel_kind` in include/zyx_hip.h) and
thin helpers that replay the reference's realize sequence for one AOT kernel:
allocate stores (+1 trash element), args = loads then stores, launch, keep the event
(zyx/src/runtime.rs:2262-2300, zyx/src/graph/plan.rs:311-327)."""
from __future__ import annotations

import numpy as np

from .backend import DType, Event, HIPDevice, HIPMemoryPool, KernelDesc

K_SOFTMAX_ROWS = 1
SOFTMAX_Y, SOFTMAX_ROWSUM, SOFTMAX_ARGMAX = 1, 2, 4


def softmax_rows_desc(rows: int, cols: int, y=True, rowsum=True, argmax=True, dtype: DType = DType.F32) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_SOFTMAX_ROWS, DType(dtype), DType(dtype)
    d.flags = (SOFTMAX_Y if y else 0) | (SOFTMAX_ROWSUM if rowsum else 0) | (SOFTMAX_ARGMAX if argmax else 0)
    d.dims[0], d.dims[1] = rows, cols
    return d


def to_device(pool: HIPMemoryPool, array: np.ndarray):
    """`Runtime::new_tensor`-style upload: allocate bytes + one trash element, async copy.
    Returns (buffer id, event); `array` must outlive the event."""
    src = np.ascontiguousarray(array)
    buf, ev = pool.allocate(src.nbytes + src.itemsize)
    ev2 = pool.host_to_pool(src, buf, [ev])
    if src is not array:  # a contiguous copy was made: only this frame keeps it alive, so the copy finishes here
        pool.sync_events([ev2])
        ev2 = Event(0)
    return buf, ev2


def to_host(pool: HIPMemoryPool, buf: int, shape, dtype, events=()) -> np.ndarray:
    out = np.empty(shape, dtype)
    pool.pool_to_host(buf, out, list(events))
    return out


def alloc_like(pool: HIPMemoryPool, n_elems: int, itemsize: int):
    return pool.allocate((n_elems + 1) * itemsize)


def softmax_rows(dev: HIPDevice, pool: HIPMemoryPool, x: np.ndarray, y=True, rowsum=True, argmax=True, dtype: DType = DType.F32):
    """Upload x, run the fused kernel, read back (y, rowsum, argmax); entries not asked for are None. bf16 / f16: x, y and
    rowsum are bit patterns (uint16)."""
    st = np.float32 if DType(dtype) == DType.F32 else np.uint16
    x = np.ascontiguousarray(x, st)
    rows, cols = x.shape
    prog = dev.register_kernel(softmax_rows_desc(rows, cols, y, rowsum, argmax, dtype))
    xb, ev = to_device(pool, x)
    waits, outs = [ev], []
    for want, n, isz in ((y, rows * cols, x.itemsize), (rowsum, rows, x.itemsize), (argmax, rows, 4)):
        if want:
            b, e = alloc_like(pool, n, isz)
            outs.append(b)
            waits.append(e)
    done = dev.launch(prog, pool, [xb] + outs, waits)
    res, it = [], iter(outs)
    first = True
    for want, shape, dt in ((y, (rows, cols), st), (rowsum, (rows,), st), (argmax, (rows,), np.int32)):
        if not want:
            res.append(None)
            continue
        res.append(to_host(pool, next(it), shape, dt, [done] if first else []))
        first = False
    for b in [xb] + outs:
        pool.deallocate(b, [])
    dev.release(prog)
    return tuple(res)


# ---- fused elementwise chains (ZHIP_K_ELEMENTWISE) ------------------------------------------
K_ELEMENTWISE = 2
K_REDUCE = 3

EW_OPS = ["load", "save", "neg", "bitnot", "exp", "exp2", "ln", "log2", "reciprocal", "sqrt", "sin", "cos", "floor",
          "trunc", "abs", "add", "sub", "mul", "div", "pow", "mod", "cmplt", "cmpgt", "cmpge", "max", "or", "and",
          "bitxor", "bitor", "bitand", "shl", "shr", "noteq", "eq", "rsub", "rdiv", "where", "mad", "relu", "tanh",
          "gelu", "sigmoid", "rsqrt", "cast_int", "gelu_grad"]
EW_OP = {name: i for i, name in enumerate(EW_OPS)}
EW_FULL, EW_ROW, EW_COL, EW_SCALAR = 0, 1, 2, 3
EW_T = 0x10
EW_CONST = 0x20


class Chain:
    """Builder of an accumulator program: `acc` is threaded through the ops, `t` is one saved
    value. Operands are input indices (from `input()`), `Chain.T`, or constants (`const()`).

        c = Chain(rows, cols)                      # gelu(x + bias)
        x, b = c.input(DType.F32), c.input(DType.F32, EW_ROW)
        c.load(x).add(b).gelu()
    """
    T = EW_T

    def __init__(self, rows: int, cols: int, reg: DType = DType.F32, out_dtype: DType = DType.F32):
        self.rows, self.cols, self.reg, self.out_dtype = rows, cols, DType(reg), DType(out_dtype)
        self.inputs, self.code, self.consts = [], [], []

    def input(self, dtype: DType = DType.F32, bcast: int = EW_FULL) -> int:
        self.inputs.append((DType(dtype), bcast))
        return len(self.inputs) - 1

    def const(self, value: float) -> int:
        value = float(np.float32(value))
        if value not in self.consts:
            self.consts.append(value)
        return EW_CONST + self.consts.index(value)

    def op(self, name: str, a: int = 0, b: int = 0) -> "Chain":
        self.code.append(EW_OP[name] | (a << 8) | (b << 16))
        return self

    def __getattr__(self, name):
        if name in EW_OP:
            return lambda a=0, b=0: self.op(name, a, b)
        raise AttributeError(name)

    def input_elems(self, k: int) -> int:
        bc = self.inputs[k][1]
        return {EW_FULL: self.rows * self.cols, EW_ROW: self.cols, EW_COL: self.rows, EW_SCALAR: 1}[bc]

    def desc(self) -> KernelDesc:
        d = KernelDesc()
        d.kind, d.dtype, d.out_dtype = K_ELEMENTWISE, self.reg, self.out_dtype
        d.dims[0], d.dims[1] = self.rows, self.cols
        d.iparams[0], d.iparams[1] = len(self.inputs), len(self.code)
        for k, (dt, bc) in enumerate(self.inputs):
            d.iparams[2 + k] = int(dt) | (bc << 8)
        for j, ins in enumerate(self.code):
            d.iparams[6 + j] = ins
        for k, v in enumerate(self.consts):
            d.fparams[k] = v
        return d


_NP_STORE = {DType.F32: np.float32, DType.BF16: np.uint16, DType.F16: np.uint16, DType.I32: np.int32,
             DType.U8: np.uint8, DType.Bool: np.uint8}


def run_chain(dev: HIPDevice, pool: HIPMemoryPool, chain: Chain, arrays) -> np.ndarray:
    """Upload the inputs, launch the chain, read the [rows, cols] result back."""
    prog = dev.register_kernel(chain.desc())
    bufs, waits = [], []
    keep = []
    for k, a in enumerate(arrays):
        a = np.ascontiguousarray(a, _NP_STORE[chain.inputs[k][0]])
        assert a.size == chain.input_elems(k)
        keep.append(a)
        b, e = to_device(pool, a)
        bufs.append(b)
        waits.append(e)
    out_np = _NP_STORE[chain.out_dtype]
    ob, e = alloc_like(pool, chain.rows * chain.cols, np.dtype(out_np).itemsize)
    waits.append(e)
    done = dev.launch(prog, pool, bufs + [ob], waits)
    res = to_host(pool, ob, (chain.rows, chain.cols), out_np, [done])
    for b in bufs + [ob]:
        pool.deallocate(b, [])
    dev.release(prog)
    return res


def reduce_desc(rows: int, cols: int, op: str = "sum", axis0: bool = False, dtype: DType = DType.F32, mul: float = 0.0,
                div: float = 0.0, base: bool = False) -> KernelDesc:
    """out = reduce (* mul) (/ div) (+ base); args: x, (base), out."""
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_REDUCE, DType(dtype), DType(dtype)
    d.flags = 1 if axis0 else 0
    d.dims[0], d.dims[1] = rows, cols
    d.iparams[0] = {"sum": 0, "max": 1}[op]
    d.iparams[1] = int(bool(base))
    d.fparams[0], d.fparams[1] = mul, div
    return d


def reduce(dev: HIPDevice, pool: HIPMemoryPool, x: np.ndarray, op: str = "sum", axis0: bool = False,
           dtype: DType = DType.F32, mul: float = 0.0, div: float = 0.0, base: np.ndarray | None = None) -> np.ndarray:
    x = np.ascontiguousarray(x, _NP_STORE[DType(dtype)])
    rows, cols = x.shape
    prog = dev.register_kernel(reduce_desc(rows, cols, op, axis0, dtype, mul, div, base is not None))
    xb, e0 = to_device(pool, x)
    n_out = cols if axis0 else rows
    bufs, waits = [xb], [e0]
    if base is not None:
        bb, eb = to_device(pool, np.ascontiguousarray(base, x.dtype))
        bufs.append(bb)
        waits.append(eb)
    ob, e1 = alloc_like(pool, n_out, x.itemsize)
    done = dev.launch(prog, pool, bufs + [ob], waits + [e1])
    res = to_host(pool, ob, (n_out,), x.dtype, [done])
    for buf in bufs + [ob]:
        pool.deallocate(buf, [])
    dev.release(prog)
    return res


K_ARGMAX = 13


def argmax_desc(outer: int, n: int, inner: int, dtype: DType = DType.F32) -> KernelDesc:
    """Tensor::argmax_axis over the middle axis of a dense [outer, n, inner] view; args: x, out (i32)."""
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_ARGMAX, DType(dtype), DType.I32
    d.dims[0], d.dims[1], d.dims[2] = outer, n, inner
    return d


def argmax_axis(dev: HIPDevice, pool: HIPMemoryPool, x: np.ndarray, axis: int, dtype: DType = DType.F32) -> np.ndarray:
    """x.argmax_axis(axis) (zyx/src/tensor/mod.rs:2238-2243); `x` holds the storage values of `dtype`."""
    x = np.ascontiguousarray(x, _NP_STORE[DType(dtype)])
    axis = axis % x.ndim
    outer, n, inner = int(np.prod(x.shape[:axis], dtype=np.int64)), x.shape[axis], int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    prog = dev.register_kernel(argmax_desc(outer, n, inner, dtype))
    xb, e0 = to_device(pool, x)
    ob, e1 = alloc_like(pool, outer * inner, 4)
    done = dev.launch(prog, pool, [xb, ob], [e0, e1])
    res = to_host(pool, ob, x.shape[:axis] + x.shape[axis + 1:], np.int32, [done])
    pool.deallocate(xb, [])
    pool.deallocate(ob, [])
    dev.release(prog)
    return res


def argmax(dev: HIPDevice, pool: HIPMemoryPool, x: np.ndarray, dtype: DType = DType.F32) -> np.ndarray:
    """x.argmax(): the flattened tensor's arg-max (zyx/src/tensor/mod.rs:2228-2230)."""
    return argmax_axis(dev, pool, np.ascontiguousarray(x).reshape(-1), 0, dtype)


# ---- GEMM (ZHIP_K_GEMM) ----------------------------------------------------------------------
K_GEMM = 4
GEMM_TRANS_A, GEMM_TRANS_B = 1, 2
EPILOGUE = {"none": 0, "bias": 1, "bias_relu": 2, "bias_gelu": 3}


def gemm_desc(m: int, n: int, k: int, dtype: DType = DType.BF16, out_dtype: DType = DType.F32, trans_a=False,
              trans_b=False, epilogue: str = "none", bias_dtype: DType = DType.F32, batch: int = 1,
              alpha: float = 1.0, residual: bool = False) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_GEMM, DType(dtype), DType(out_dtype)
    d.flags = (GEMM_TRANS_A if trans_a else 0) | (GEMM_TRANS_B if trans_b else 0)
    d.dims[0], d.dims[1], d.dims[2], d.dims[3] = m, n, k, batch
    d.iparams[0], d.iparams[1], d.iparams[2] = EPILOGUE[epilogue], int(bias_dtype), 2 if residual == "relu_mask" else int(bool(residual))
    d.fparams[0] = alpha
    return d


def gemm(dev: HIPDevice, pool: HIPMemoryPool, a: np.ndarray, b: np.ndarray, bias: np.ndarray | None = None,
         dtype: DType = DType.BF16, out_dtype: DType = DType.F32, trans_a=False, trans_b=False, epilogue: str = "none",
         bias_dtype: DType = DType.F32, alpha: float = 1.0, residual: np.ndarray | None = None,
         relu_mask: bool = False) -> np.ndarray:
    """a: [M,K] ([K,M] if trans_a), b: [K,N] ([N,K] if trans_b) in their storage dtype; returns C[M,N]
    (+ residual[M,N], stored like C; with relu_mask the result is multiplied by (residual > 0) instead)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    batch = a.shape[0] if a.ndim == 3 else 1
    m, k = (a.shape[-1], a.shape[-2]) if trans_a else a.shape[-2:]
    n = b.shape[-2] if trans_b else b.shape[-1]
    prog = dev.register_kernel(gemm_desc(m, n, k, dtype, out_dtype, trans_a, trans_b, epilogue, bias_dtype, batch, alpha,
                                         "relu_mask" if relu_mask else residual is not None))
    bufs, waits = [], []
    extra = ((np.ascontiguousarray(bias),) if epilogue != "none" else ()) + \
        ((np.ascontiguousarray(residual, _NP_STORE[DType(out_dtype)]),) if residual is not None else ())
    for arr in (a, b) + extra:
        bb, e = to_device(pool, arr)
        bufs.append(bb)
        waits.append(e)
    out_np = _NP_STORE[DType(out_dtype)]
    cb, e = alloc_like(pool, batch * m * n, np.dtype(out_np).itemsize)
    waits.append(e)
    done = dev.launch(prog, pool, bufs + [cb], waits)
    res = to_host(pool, cb, (batch, m, n) if a.ndim == 3 else (m, n), out_np, [done])
    for bb in bufs + [cb]:
        pool.deallocate(bb, [])
    dev.release(prog)
    return res


# ---- LayerNorm / RMSNorm (ZHIP_K_NORM_ROWS), cross entropy (ZHIP_K_CROSS_ENTROPY) --------------------
K_NORM_ROWS, K_CROSS_ENTROPY = 5, 6
NORM_RMS, NORM_WEIGHT, NORM_BIAS = 1, 2, 4
CE_LOSS, CE_GRAD, CE_MEAN, CE_DENSE = 1, 2, 4, 8


def norm_rows_desc(rows: int, cols: int, rms=False, weight=True, bias=True, eps=1e-5, dtype: DType = DType.F32) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_NORM_ROWS, DType(dtype), DType(dtype)
    d.flags = (NORM_RMS if rms else 0) | (NORM_WEIGHT if weight else 0) | (NORM_BIAS if bias and not rms else 0)
    d.dims[0], d.dims[1] = rows, cols
    d.fparams[0] = eps
    return d


def norm_rows(dev: HIPDevice, pool: HIPMemoryPool, x, w=None, b=None, rms=False, eps=1e-5, dtype: DType = DType.F32):
    """LayerNorm::forward / RMSNorm::forward over the last axis of x[rows, cols]."""
    st = _NP_STORE[DType(dtype)]
    x = np.ascontiguousarray(x, st)
    rows, cols = x.shape
    prog = dev.register_kernel(norm_rows_desc(rows, cols, rms, w is not None, b is not None, eps, dtype))
    bufs, waits = [], []
    for arr in [x] + [np.ascontiguousarray(a, st) for a in (w, b) if a is not None]:
        bb, e = to_device(pool, arr)
        bufs.append(bb)
        waits.append(e)
    yb, e = alloc_like(pool, rows * cols, x.itemsize)
    done = dev.launch(prog, pool, bufs + [yb], waits + [e])
    y = to_host(pool, yb, (rows, cols), st, [done])
    for bb in bufs + [yb]:
        pool.deallocate(bb, [])
    dev.release(prog)
    return y


def cross_entropy_desc(rows: int, cols: int, loss=True, grad=False, gscale: float = 1.0, mean=False, dense=False) -> KernelDesc:
    """args: logits, labels (dense: f32 targets[rows, cols]), (loss[rows]), (grad[rows, cols]), (mean[1])."""
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_CROSS_ENTROPY, DType.F32, DType.F32
    d.flags = (CE_LOSS if loss else 0) | (CE_GRAD if grad else 0) | (CE_MEAN if mean else 0) | (CE_DENSE if dense else 0)
    d.dims[0], d.dims[1] = rows, cols
    d.fparams[0] = gscale
    return d


def cross_entropy(dev: HIPDevice, pool: HIPMemoryPool, logits, labels, grad_scale=None, mean=False, dense=False):
    """-> (per-sample loss, grad or None); grad = d(grad_scale * sum(loss)) / d(logits). With mean=True a third
    value, the batch mean from the same launch. dense: `labels` is an f32 target tensor of the logits' shape."""
    x = np.ascontiguousarray(logits, np.float32)
    lab = np.ascontiguousarray(labels, np.float32 if dense else np.int32)
    rows, cols = x.shape
    if dense and lab.shape != x.shape:
        raise ValueError("dense targets have the logits' shape")
    prog = dev.register_kernel(cross_entropy_desc(rows, cols, True, grad_scale is not None, grad_scale or 0.0, mean, dense))
    xb, e0 = to_device(pool, x)
    lb, e1 = to_device(pool, lab)
    ob, e2 = alloc_like(pool, rows, 4)
    outs, waits = [ob], [e0, e1, e2]
    if grad_scale is not None:
        gb, e3 = alloc_like(pool, rows * cols, 4)
        outs.append(gb)
        waits.append(e3)
    if mean:
        mb, e4 = alloc_like(pool, 1, 4)
        outs.append(mb)
        waits.append(e4)
    done = dev.launch(prog, pool, [xb, lb] + outs, waits)
    loss = to_host(pool, ob, (rows,), np.float32, [done])
    grad = to_host(pool, outs[1], (rows, cols), np.float32) if grad_scale is not None else None
    mean_v = to_host(pool, outs[-1], (1,), np.float32) if mean else None
    for bb in [xb, lb] + outs:
        pool.deallocate(bb, [])
    dev.release(prog)
    return (loss, grad, mean_v) if mean else (loss, grad)


# ---- conv2d / max_pool2d (ZHIP_K_CONV2D, ZHIP_K_MAX_POOL2D) ---------------------------------------------
K_CONV2D, K_MAX_POOL2D = 7, 8


def conv_out(size: int, k: int, stride: int, pad: int, dil: int) -> int:
    return (size + 2 * pad - dil * (k - 1) - 1) // stride + 1


def conv2d_desc(n, c, h, w, cout, kh, kw, stride=(1, 1), padding=(0, 0), dilation=(1, 1), bias=False, relu=False,
                dtype: DType = DType.F32, out_dtype: DType | None = None, pool=False) -> KernelDesc:
    """pool: the launch also applies max_pool([2, 2]) and writes only the pooled [n, cout, oh / 2, ow / 2] result
    (shapes of the direct 3 x 3 kernel; registration refuses others)."""
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_CONV2D, DType(dtype), DType(dtype if out_dtype is None else out_dtype)
    for i, v in enumerate((n, c, h, w, cout, kh, kw)):
        d.dims[i] = v
    for i, v in enumerate((stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1], int(bias), int(relu), int(pool))):
        d.iparams[i] = v
    return d


def max_pool2d_desc(planes, h, w, kernel=(2, 2), stride=(2, 2), padding=(0, 0), dilation=(1, 1),
                    dtype: DType = DType.F32) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_MAX_POOL2D, DType(dtype), DType(dtype)
    for i, v in enumerate((planes, h, w, kernel[0], kernel[1])):
        d.dims[i] = v
    for i, v in enumerate((stride[0], stride[1], padding[0], padding[1], dilation[0], dilation[1])):
        d.iparams[i] = v
    return d


def conv2d(dev: HIPDevice, pool: HIPMemoryPool, x, w, bias=None, stride=(1, 1), padding=(0, 0), dilation=(1, 1),
           relu=False, dtype: DType = DType.F32, out_dtype: DType | None = None, pool_kernel=None, fused_pool=False):
    """Conv2d::forward (+ ReLU) and optionally max_pool(pool_kernel, stride = kernel) as two launches whose
    second waits on the first's event. Returns y, or (y, pooled). fused_pool: one launch that returns only the
    2 x 2 pooled result."""
    st = _NP_STORE[DType(dtype)]
    out_dtype = DType(dtype if out_dtype is None else out_dtype)
    x, w = np.ascontiguousarray(x, st), np.ascontiguousarray(w, st)
    n, c, h, wd = x.shape
    co, _, kh, kw = w.shape
    oh, ow = conv_out(h, kh, stride[0], padding[0], dilation[0]), conv_out(wd, kw, stride[1], padding[1], dilation[1])
    prog = dev.register_kernel(conv2d_desc(n, c, h, wd, co, kh, kw, stride, padding, dilation, bias is not None, relu,
                                           dtype, out_dtype, pool=fused_pool))
    if fused_pool:
        oh, ow = oh // 2, ow // 2
    bufs, waits = [], []
    for arr in (x, w) + ((np.ascontiguousarray(bias, st),) if bias is not None else ()):
        bb, e = to_device(pool, arr)
        bufs.append(bb)
        waits.append(e)
    out_np = _NP_STORE[out_dtype]
    yb, e = alloc_like(pool, n * co * oh * ow, np.dtype(out_np).itemsize)
    done = dev.launch(prog, pool, bufs + [yb], waits + [e])
    progs, extra = [prog], []
    if pool_kernel is not None:
        ph, pw = conv_out(oh, pool_kernel[0], pool_kernel[0], 0, 1), conv_out(ow, pool_kernel[1], pool_kernel[1], 0, 1)
        pprog = dev.register_kernel(max_pool2d_desc(n * co, oh, ow, pool_kernel, pool_kernel, dtype=out_dtype))
        pb, e = alloc_like(pool, n * co * ph * pw, np.dtype(out_np).itemsize)
        pdone = dev.launch(pprog, pool, [yb, pb], [done, e])
        pooled = to_host(pool, pb, (n, co, ph, pw), out_np, [pdone])
        y = to_host(pool, yb, (n, co, oh, ow), out_np)
        progs.append(pprog)
        extra.append(pb)
    else:
        y = to_host(pool, yb, (n, co, oh, ow), out_np, [done])
    for bb in bufs + [yb] + extra:
        pool.deallocate(bb, [])
    for pr in progs:
        dev.release(pr)
    return (y, pooled) if pool_kernel is not None else y


def max_pool2d(dev: HIPDevice, pool: HIPMemoryPool, x, kernel=(2, 2), stride=(2, 2), padding=(0, 0), dilation=(1, 1),
               dtype: DType = DType.F32):
    st = _NP_STORE[DType(dtype)]
    x = np.ascontiguousarray(x, st)
    h, wd = x.shape[-2:]
    planes = x.size // (h * wd)
    oh, ow = conv_out(h, kernel[0], stride[0], padding[0], dilation[0]), conv_out(wd, kernel[1], stride[1], padding[1], dilation[1])
    prog = dev.register_kernel(max_pool2d_desc(planes, h, wd, kernel, stride, padding, dilation, dtype))
    xb, e0 = to_device(pool, x)
    yb, e1 = alloc_like(pool, planes * oh * ow, x.itemsize)
    done = dev.launch(prog, pool, [xb, yb], [e0, e1])
    y = to_host(pool, yb, x.shape[:-2] + (oh, ow), st, [done])
    pool.deallocate(xb, [])
    pool.deallocate(yb, [])
    dev.release(prog)
    return y


# ---- gather / index_select / scatter (ZHIP_K_INDEX) ----------------------------------------------------------
K_INDEX = 9
INDEX_GATHER, INDEX_SELECT, INDEX_SCATTER = 0, 1, 2
_DT_OF_NP = {np.dtype(np.float32): DType.F32, np.dtype(np.float64): DType.F64, np.dtype(np.int32): DType.I32,
             np.dtype(np.int64): DType.I64, np.dtype(np.uint8): DType.U8, np.dtype(np.uint16): DType.U16,
             np.dtype(np.uint32): DType.U32, np.dtype(np.uint64): DType.U64, np.dtype(np.int8): DType.I8,
             np.dtype(np.int16): DType.I16, np.dtype(np.bool_): DType.Bool}


def _pad4(shape):
    assert len(shape) <= 4, "rank <= 4"
    return (1,) * (4 - len(shape)) + tuple(shape)


def index_desc(mode: int, x_shape, idx_shape, axis: int, dtype: DType, idx_dtype: DType = DType.I32) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype, d.flags = K_INDEX, DType(dtype), DType(dtype), mode
    rank = len(x_shape)
    for i, v in enumerate(_pad4(x_shape) + _pad4(idx_shape)):
        d.dims[i] = v
    d.iparams[0], d.iparams[1] = (axis % rank) + (4 - rank), int(idx_dtype)
    return d


def _index_run(dev, pool, desc, arrays, out_shape, out_np):
    prog = dev.register_kernel(desc)
    bufs, waits = [], []
    for a in arrays:
        b, e = to_device(pool, a)
        bufs.append(b)
        waits.append(e)
    n = int(np.prod(out_shape))
    ob, e = alloc_like(pool, n, np.dtype(out_np).itemsize)
    done = dev.launch(prog, pool, bufs + [ob], waits + [e])
    out = to_host(pool, ob, out_shape, out_np, [done])
    for b in bufs + [ob]:
        pool.deallocate(b, [])
    dev.release(prog)
    return out


def _as_index(indices):
    idx = np.ascontiguousarray(indices)
    if idx.dtype == np.int64:
        return idx, DType.I64
    return np.ascontiguousarray(idx, np.int32), DType.I32  # unsigned / narrow index dtypes widen losslessly


def gather(dev: HIPDevice, pool: HIPMemoryPool, x, axis: int, indices):
    """Tensor::gather (zyx/src/tensor/index_ops.rs:321-361)."""
    x = np.ascontiguousarray(x)
    idx, idt = _as_index(indices)
    if x.ndim != idx.ndim:
        raise ValueError(f"self.rank({x.ndim}) != indices.rank({idx.ndim})")
    return _index_run(dev, pool, index_desc(INDEX_GATHER, x.shape, idx.shape, axis, _DT_OF_NP[x.dtype], idt), [x, idx],
                      idx.shape, x.dtype)


def index_select(dev: HIPDevice, pool: HIPMemoryPool, x, axis: int, index):
    """Tensor::index_select (index_ops.rs:431-445): 1-D index along `axis`."""
    x = np.ascontiguousarray(x)
    idx, idt = _as_index(index)
    out_shape = list(x.shape)
    out_shape[axis % x.ndim] = idx.shape[0]
    return _index_run(dev, pool, index_desc(INDEX_SELECT, x.shape, out_shape, axis, _DT_OF_NP[x.dtype], idt), [x, idx],
                      tuple(out_shape), x.dtype)


def scatter(dev: HIPDevice, pool: HIPMemoryPool, x, axis: int, indices, src):
    """Tensor::scatter (index_ops.rs:376-425): adds src into self at the indexed positions."""
    x = np.ascontiguousarray(x)
    idx, idt = _as_index(indices)
    src = np.ascontiguousarray(src, x.dtype)
    if x.ndim != idx.ndim:
        raise ValueError(f"self.rank({x.ndim}) != indices.rank({idx.ndim})")
    if idx.shape != src.shape:
        raise ValueError(f"indices shape {idx.shape} != src shape {src.shape}")
    return _index_run(dev, pool, index_desc(INDEX_SCATTER, x.shape, idx.shape, axis, _DT_OF_NP[x.dtype], idt),
                      [x, idx, src], x.shape, x.dtype)


# ---- attention core (ZHIP_K_ATTENTION) -----------------------------------------------------------------------
K_ATTENTION = 10
ATTN_LSE, ATTN_CAUSAL = 1, 2


def attention_desc(b: int, t: int, n_head: int, dh: int, dtype: DType = DType.BF16, scale: float = 0.0,
                   dropout_p: float = 0.0, lse: bool = False, causal: bool = False) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_ATTENTION, DType(dtype), DType(dtype)
    d.flags = (ATTN_LSE if lse else 0) | (ATTN_CAUSAL if causal else 0)
    d.dims[0], d.dims[1], d.dims[2], d.dims[3] = b, t, n_head, dh
    d.fparams[0], d.fparams[1] = scale, dropout_p
    return d


def attention(dev: HIPDevice, pool: HIPMemoryPool, qkv, n_head: int, dtype: DType = DType.BF16, scale: float = 0.0,
              dropout_p: float = 0.0, want_lse: bool = False, causal: bool = False):
    """Core of CausalSelfAttention::forward (zyx-nn/src/causal_self_attention.rs:36-74) on the c_attn output
    qkv[B,T,3C] (bf16 bit patterns as uint16, or float32) -> y[B,T,C] (, lse[B,H,T])."""
    qkv = np.ascontiguousarray(qkv)
    b, t, c3 = qkv.shape
    c = c3 // 3
    prog = dev.register_kernel(attention_desc(b, t, n_head, c // n_head, dtype, scale, dropout_p, want_lse, causal))
    xb, e0 = to_device(pool, qkv)
    yb, e1 = alloc_like(pool, b * t * c, qkv.dtype.itemsize)
    bufs, waits = [xb, yb], [e0, e1]
    if want_lse:
        lb, e2 = alloc_like(pool, b * n_head * t, 4)
        bufs.append(lb)
        waits.append(e2)
    done = dev.launch(prog, pool, bufs, waits)
    y = to_host(pool, yb, (b, t, c), qkv.dtype, [done])
    out = (y, to_host(pool, bufs[2], (b, n_head, t), np.float32, [])) if want_lse else y
    for buf in bufs:
        pool.deallocate(buf, [])
    dev.release(prog)
    return out


K_ATTENTION_BWD = 11


def attention_bwd_desc(b: int, t: int, n_head: int, dh: int, dtype: DType = DType.BF16, scale: float = 0.0,
                       dropout_p: float = 0.0, causal: bool = False) -> KernelDesc:
    d = attention_desc(b, t, n_head, dh, dtype, scale, dropout_p, causal=causal)
    d.kind = K_ATTENTION_BWD
    return d


def attention_bwd(dev: HIPDevice, pool: HIPMemoryPool, qkv, y, dy, lse, n_head: int, dtype: DType = DType.BF16,
                  scale: float = 0.0, dropout_p: float = 0.0, causal: bool = False):
    """Gradient of `attention` with respect to qkv given dy; y and lse are the forward's outputs."""
    qkv = np.ascontiguousarray(qkv)
    b, t, c3 = qkv.shape
    prog = dev.register_kernel(attention_bwd_desc(b, t, n_head, c3 // 3 // n_head, dtype, scale, dropout_p, causal))
    bufs, waits = [], []
    for a in (qkv, np.ascontiguousarray(y, qkv.dtype), np.ascontiguousarray(dy, qkv.dtype), np.ascontiguousarray(lse, np.float32)):
        buf, e = to_device(pool, a)
        bufs.append(buf)
        waits.append(e)
    ob, e = alloc_like(pool, qkv.size, qkv.dtype.itemsize)
    done = dev.launch(prog, pool, bufs + [ob], waits + [e])
    out = to_host(pool, ob, qkv.shape, qkv.dtype, [done])
    for buf in bufs + [ob]:
        pool.deallocate(buf, [])
    dev.release(prog)
    return out


# ---- gradients of LayerNorm / RMSNorm (ZHIP_K_NORM_ROWS_BWD) -------------------------------------------------
K_NORM_ROWS_BWD = 12
NORM_ADD = 8


def norm_rows_bwd_desc(rows: int, cols: int, rms=False, weight=True, bias=True, add=False, eps=1e-5,
                       dtype: DType = DType.F32) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_NORM_ROWS_BWD, DType(dtype), DType(dtype)
    d.flags = (NORM_RMS if rms else 0) | (NORM_WEIGHT if weight else 0) | (NORM_BIAS if bias and not rms else 0) | \
        (NORM_ADD if add else 0)
    d.dims[0], d.dims[1] = rows, cols
    d.fparams[0] = eps
    return d


def norm_rows_bwd(dev: HIPDevice, pool: HIPMemoryPool, x, dy, w=None, add=None, rms=False, want_db=True, eps=1e-5,
                  dtype: DType = DType.F32):
    """Gradients of LayerNorm / RMSNorm: returns (dx (+ add), dw or None, db or None)."""
    st = _NP_STORE[DType(dtype)]
    x = np.ascontiguousarray(x, st)
    rows, cols = x.shape
    want_db = want_db and not rms
    prog = dev.register_kernel(norm_rows_bwd_desc(rows, cols, rms, w is not None, want_db, add is not None, eps, dtype))
    ins = [x] + ([np.ascontiguousarray(w, st)] if w is not None else []) + [np.ascontiguousarray(dy, st)] + \
        ([np.ascontiguousarray(add, st)] if add is not None else [])
    bufs, waits = [], []
    for arr in ins:
        bb, e = to_device(pool, arr)
        bufs.append(bb)
        waits.append(e)
    outs = [(rows, cols)] + ([(cols,)] if w is not None else []) + ([(cols,)] if want_db else [])
    obufs = []
    for shp in outs:
        ob, e = alloc_like(pool, int(np.prod(shp)), x.itemsize)
        obufs.append(ob)
        waits.append(e)
    done = dev.launch(prog, pool, bufs + obufs, waits)
    res = [to_host(pool, ob, shp, st, [done] if i == 0 else []) for i, (ob, shp) in enumerate(zip(obufs, outs))]
    for bb in bufs + obufs:
        pool.deallocate(bb, [])
    dev.release(prog)
    dx = res[0]
    dw = res[1] if w is not None else None
    db = res[-1] if want_db else None
    return dx, dw, db
