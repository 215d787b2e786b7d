"""Graph nodes, reverse-mode differentiation and lowering to generated kernels.

The node kinds are the ones `Runtime::gradient` differentiates (zyx/src/graph/autograd.rs:14-424; `Node` in
zyx/src/graph/mod.rs): Leaf, Const, Unary, Binary, Cast, Reshape, Expand, Permute, Flip, Reduce. `Graph.gradient`
applies that function's rules node by node, including the rules the reference keeps as comments beside a `todo!()`
(Reshape :183-194, Expand :195-242, Reduce sum :269-295, Reduce max :299-379: every tied maximum receives the
full gradient). `lower` turns the nodes to compute into kernels in the linearized-kernel image `Device::compile`
takes: one thread per output element, movement ops folded into the index arithmetic of the loads, a reduce as one
serial loop per output element with its accumulator in a register (zyx/src/kernel/linearize.rs:920-952) -- the kernel
the reference generates before any optimisation pass. `Tape` runs them on a HIP device.

Conventions where the graph leaves the dtype open (`Graph::dtype` returns x's dtype for every Binary, graph/mod.rs:
1113-1134, and scalars broadcast implicitly, :1759-1769): a comparison or logical op yields Bool; when the operands
of a Binary differ in dtype, a Const or Bool operand is converted to the other operand's dtype, otherwise y to x's.
"""
from __future__ import annotations

import dataclasses
from typing import Sequence

import numpy as np

from .backend import DType
from .ir import BOp, Kernel, MemScope, ParamKind, UOp

_BOOL_OPS = (BOp.Cmplt, BOp.Cmpgt, BOp.Cmpge, BOp.NotEq, BOp.Eq, BOp.Or, BOp.And)
_NO_GRAD_BOPS = _BOOL_OPS + (BOp.BitXor, BOp.BitOr, BOp.BitAnd, BOp.BitShiftLeft, BOp.BitShiftRight)
_NP = {DType.BF16: np.uint16, DType.F16: np.float16, DType.F32: np.float32, DType.F64: np.float64, DType.U8: np.uint8,
       DType.U16: np.uint16, DType.U32: np.uint32, DType.U64: np.uint64, DType.I8: np.int8, DType.I16: np.int16,
       DType.I32: np.int32, DType.I64: np.int64, DType.Bool: np.uint8}


def storage_dtype(dtype: DType):
    """numpy type of a buffer of this dtype (bf16 travels as its 16 bits)."""
    return _NP[DType(dtype)]


def min_constant(dtype: DType):
    """Neutral element of a max reduce: the lowest finite value (zyx/src/dtype.rs:207-224), not -inf."""
    dtype = DType(dtype)
    if dtype in (DType.BF16, DType.F32):
        return -3.4028234663852886e38 if dtype == DType.F32 else -3.3895313892515355e38
    if dtype == DType.F16:
        return -65504.0
    if dtype == DType.F64:
        return -1.7976931348623157e308
    if dtype == DType.Bool:
        return 0
    return int(np.iinfo(_NP[dtype]).min)


@dataclasses.dataclass(frozen=True)
class Node:
    kind: str                 # leaf const unary binary cast reshape expand permute flip reduce
    dtype: DType
    shape: tuple
    src: tuple = ()           # operand node ids
    op: int | None = None     # UOp / BOp (reduce: BOp.Add or BOp.Max)
    arg: object = None        # const value / axes


def _numel(shape) -> int:
    n = 1
    for d in shape:
        n *= int(d)
    return n


class Graph:
    def __init__(self):
        self.nodes: list[Node] = []
        self.convs: dict[int, dict] = {}  # result node of `conv` -> its operands and parameters
        self.pools: dict[int, dict] = {}  # result node of a 2-D `max_pool` -> its operand and parameters
        # Module-level expressions the hand-written kernels compute whole (`layer_norm`, `rms_norm`, `self_attention`):
        # result node -> dict(kind, inputs, params). The reverse pass differentiates such an expression as a unit (the
        # same primitive rules, applied to its own nodes only) and notes the gradient nodes in `fused_bwd`, so that the
        # lowering can hand forward and backward to one launch each.
        self.composites: dict[int, dict] = {}
        self.fused_bwd: dict[int, dict] = {}   # gradient node of a composite's input -> dict(kind, fwd, dy, inputs, grads, params)

    def _push(self, node: Node) -> int:
        self.nodes.append(node)
        return len(self.nodes) - 1

    def __getitem__(self, i: int) -> Node:
        return self.nodes[i]

    # -- nodes --------------------------------------------------------------------------------------------------
    def leaf(self, shape, dtype: DType) -> int:
        return self._push(Node("leaf", DType(dtype), tuple(int(d) for d in shape)))

    def const(self, value, dtype: DType) -> int:
        return self._push(Node("const", DType(dtype), (), arg=value))

    def unary(self, x: int, uop: UOp) -> int:
        n = self[x]
        return self._push(Node("unary", n.dtype, n.shape, (x,), UOp(uop)))

    def binary(self, x: int, y: int, bop: BOp) -> int:
        bop = BOp(bop)
        nx, ny = self[x], self[y]
        if nx.shape != ny.shape and nx.shape != () and ny.shape != ():
            raise ValueError(f"binary operands have shapes {nx.shape} and {ny.shape}: only scalars broadcast implicitly")
        shape = nx.shape if nx.shape != () else ny.shape
        return self._push(Node("binary", DType.Bool if bop in _BOOL_OPS else self.operand_dtype(x, y), shape, (x, y), bop))

    def operand_dtype(self, x: int, y: int) -> DType:
        """The dtype both operands of a Binary are brought to (module docstring)."""
        nx, ny = self[x], self[y]

        def yields(n: Node) -> int:
            return 2 if n.dtype == DType.Bool else (1 if n.kind == "const" else 0)

        return ny.dtype if yields(ny) < yields(nx) else nx.dtype

    def cast(self, x: int, dtype: DType) -> int:
        return self._push(Node("cast", DType(dtype), self[x].shape, (x,)))

    def reshape(self, x: int, shape) -> int:
        shape = tuple(int(d) for d in shape)
        if _numel(shape) != _numel(self[x].shape):
            raise ValueError(f"cannot reshape {self[x].shape} to {shape}")
        return x if shape == self[x].shape else self._push(Node("reshape", self[x].dtype, shape, (x,)))

    def expand(self, x: int, shape) -> int:
        """Right-aligned broadcast: dims of size 1 stretch, missing leading dims are added."""
        shape, xs = tuple(int(d) for d in shape), self[x].shape
        pad = len(shape) - len(xs)
        if pad < 0 or any(d != 1 and d != shape[pad + i] for i, d in enumerate(xs)):
            raise ValueError(f"cannot expand {xs} to {shape}")
        return x if shape == xs else self._push(Node("expand", self[x].dtype, shape, (x,)))

    def permute(self, x: int, axes) -> int:
        xs = self[x].shape
        axes = tuple(int(a) % len(xs) for a in axes)
        if sorted(axes) != list(range(len(xs))):
            raise ValueError(f"{axes} is not a permutation of the axes of {xs}")
        return self._push(Node("permute", self[x].dtype, tuple(xs[a] for a in axes), (x,), arg=axes))

    def flip(self, x: int, axes) -> int:
        xs = self[x].shape
        return self._push(Node("flip", self[x].dtype, xs, (x,), arg=tuple(sorted({int(a) % len(xs) for a in axes}))))

    @staticmethod
    def _axis(axis: int, rank: int) -> int:
        axis = int(axis)
        if not -rank <= axis < rank:
            raise ValueError(f"axis {axis} out of range for rank {rank}")
        return axis % rank

    def pad(self, x: int, axis: int, lp: int, length: int) -> int:
        """`Node::Pad { x, axis, lp, len }` (zyx/src/graph/mod.rs:118-127): element i of `axis` is x[i - lp] where that
        exists and 0 elsewhere; `length` is the new extent of the axis. A negative `lp` drops leading elements, a
        `length` short of lp + the old extent drops trailing ones (`Tensor::pad_axis`, zyx/src/tensor/mod.rs:1126-1138)."""
        xs = self[x].shape
        axis = self._axis(axis, len(xs))
        lp, length = int(lp), int(length)
        if length < 1 or lp + xs[axis] <= 0 or lp >= length:
            raise ValueError(f"padding lp={lp}, len={length} leaves nothing of an axis of extent {xs[axis]}")
        if lp == 0 and length == xs[axis]:
            return x
        return self._push(Node("pad", self[x].dtype, xs[:axis] + (length,) + xs[axis + 1:], (x,), arg=(axis, lp)))

    def narrow(self, x: int, axis: int, start: int, length: int) -> int:
        """`Node::Narrow { x, axis, start, len }` (zyx/src/graph/mod.rs:132-137): elements start .. start + len of `axis`."""
        xs = self[x].shape
        axis = self._axis(axis, len(xs))
        start, length = int(start), int(length)
        if start < 0 or length < 1 or start + length > xs[axis]:
            raise ValueError(f"cannot narrow an axis of extent {xs[axis]} to [{start}, {start + length})")
        if start == 0 and length == xs[axis]:
            return x
        return self._push(Node("narrow", self[x].dtype, xs[:axis] + (length,) + xs[axis + 1:], (x,), arg=(axis, start)))

    def reduce(self, x: int, rop: BOp, axes) -> int:
        """Reduced dims are dropped; reducing every axis leaves shape [1]."""
        rop, xs = BOp(rop), self[x].shape
        if rop not in (BOp.Add, BOp.Max):
            raise ValueError("reduce ops are Add and Max")
        axes = tuple(sorted({int(a) % len(xs) for a in axes}))
        shape = tuple(d for i, d in enumerate(xs) if i not in axes) or (1,)
        return self._push(Node("reduce", self[x].dtype, shape, (x,), rop, axes))

    # -- tensor-level compositions the reference builds from those nodes -------------------------------------------
    def broadcast(self, x: int, shape) -> int:
        """`Tensor::broadcast` for one side: pad the shape with leading 1s, then expand."""
        xs = self[x].shape
        if xs == ():
            return self.expand(x, shape)
        return self.expand(self.reshape(x, (1,) * (len(shape) - len(xs)) + xs), shape)

    def binary_b(self, x: int, y: int, bop: BOp) -> int:
        """Binary after numpy-style broadcasting of both operands."""
        xs, ys = self[x].shape, self[y].shape
        if xs != ys and xs != () and ys != ():
            shape = tuple(np.broadcast_shapes(xs, ys))
            x, y = self.broadcast(x, shape), self.broadcast(y, shape)
        return self.binary(x, y, bop)

    def relu(self, x: int) -> int:
        """`self.cmpgt(0) * self` (zyx/src/tensor/elementwise.rs:289-293)."""
        return self.binary(self.binary(x, self.const(0, self[x].dtype), BOp.Cmpgt), x, BOp.Mul)

    def tanh(self, x: int) -> int:
        """`e = (x + x).exp(); (e - 1) / (e + 1)` (zyx/src/tensor/elementwise.rs:585-588)."""
        dt = self[x].dtype
        e = self.unary(self.binary(x, x, BOp.Add), UOp.Exp)
        return self.binary(self.binary(e, self.const(1, dt), BOp.Sub), self.binary(e, self.const(1, dt), BOp.Add), BOp.Div)

    def gelu(self, x: int) -> int:
        """`x * 0.5 * (tanh((x + x * x * x * 0.044715) * sqrt(2 / pi)) + 1)` (zyx/src/tensor/elementwise.rs:168-170)."""
        dt = self[x].dtype
        cube = self.binary(self.binary(self.binary(x, x, BOp.Mul), x, BOp.Mul), self.const(0.044715, dt), BOp.Mul)
        inner = self.binary(self.binary(x, cube, BOp.Add), self.const(float(np.sqrt(np.float32(2.0) / np.float32(np.pi))), dt), BOp.Mul)
        return self.binary(self.binary(x, self.const(0.5, dt), BOp.Mul), self.binary(self.tanh(inner), self.const(1, dt), BOp.Add), BOp.Mul)

    def t(self, x: int) -> int:
        r = len(self[x].shape)
        return x if r < 2 else self.permute(x, tuple(range(r - 2)) + (r - 1, r - 2))

    def dot(self, x: int, y: int) -> int:
        """`Tensor::dot` (zyx/src/tensor/mod.rs:1469-1490): x[.., m, 1, k] * y^T[.., 1, n, k], summed over k."""
        yt = self.t(y)
        xs, ys = self[x].shape, self[yt].shape
        if xs[-1] != ys[-1]:
            raise ValueError(f"cannot dot tensors with shapes {xs} and {self[y].shape}")
        x3 = self.reshape(x, xs[:-1] + (1, xs[-1]))
        y3 = self.reshape(yt, ys[:-2] + (1,) + ys[max(len(ys) - 2, 0):])
        prod = self.binary_b(x3, y3, BOp.Mul)
        s = self.reduce(prod, BOp.Add, [-1])
        return self.reshape(s, xs[:-1] + (ys[-2] if len(ys) > 1 else 1,))

    def reduce_keepdim(self, x: int, rop: BOp, axes) -> int:
        xs = self[x].shape
        axes = [int(a) % len(xs) for a in axes] or list(range(len(xs)))
        return self.reshape(self.reduce(x, rop, axes), tuple(1 if i in axes else d for i, d in enumerate(xs)))

    def softmax(self, x: int, axes) -> int:
        """`e = (x - max_keepdim).exp(); e / e.sum_keepdim` (zyx/src/tensor/mod.rs:1457-1461)."""
        e = self.unary(self.binary_b(x, self.reduce_keepdim(x, BOp.Max, axes), BOp.Sub), UOp.Exp)
        return self.binary_b(e, self.reduce_keepdim(e, BOp.Add, axes), BOp.Div)

    def ln_softmax(self, x: int, axes) -> int:
        """`m = x - max_keepdim; m - m.exp().sum_keepdim.ln()` (zyx/src/tensor/mod.rs:1427-1431)."""
        m = self.binary_b(x, self.reduce_keepdim(x, BOp.Max, axes), BOp.Sub)
        return self.binary_b(m, self.unary(self.reduce_keepdim(self.unary(m, UOp.Exp), BOp.Add, axes), UOp.Ln), BOp.Sub)

    def dropout(self, x: int, probability: float, uniform: int | None = None) -> int:
        """`Tensor::dropout` (zyx/src/tensor/mod.rs:822-828). Training (`uniform` = the tensor `Tensor::rand` would
        draw, same shape and dtype as x): `probability.cmplt(uniform) * x`, without rescaling; evaluation:
        `x / (1 - probability)`."""
        dt = self[x].dtype
        if uniform is None:
            return self.binary(x, self.const(1.0 - probability, dt), BOp.Div)
        return self.binary(self.binary(self.const(probability, dt), uniform, BOp.Cmplt), x, BOp.Mul)

    def sum_all(self, x: int) -> int:
        return self.reduce(x, BOp.Add, range(len(self[x].shape)))

    def max_all(self, x: int) -> int:
        return self.reduce(x, BOp.Max, range(len(self[x].shape)))

    def mean(self, x: int, axes=()) -> int:
        """`sum(axes) / n` with n the number of elements reduced, as a constant of x's dtype (`ReduceOp::Mean`,
        zyx/src/tensor/reduce_ops.rs:102-110); no axes: all of them."""
        xs = self[x].shape
        axes = [self._axis(a, len(xs)) for a in axes] or list(range(len(xs)))
        n = _numel([xs[a] for a in axes])
        return self.binary(self.reduce(x, BOp.Add, axes), self.const(n, self[x].dtype), BOp.Div)

    def var(self, x: int, axes, correction: int = 1, keepdim: bool = False) -> int:
        """`ReduceOp::Var` (zyx/src/tensor/reduce_ops.rs:111-123): `d = x - mean_keepdim(x); sum(d * d) / (n - correction)`."""
        xs = self[x].shape
        axes = [self._axis(a, len(xs)) for a in axes] or list(range(len(xs)))
        n = _numel([xs[a] for a in axes])
        dt = self[x].dtype
        mean = self.binary(self.reduce_keepdim(x, BOp.Add, axes), self.const(n, dt), BOp.Div)
        d = self.binary_b(x, mean, BOp.Sub)
        sq = self.binary(d, d, BOp.Mul)
        red = self.reduce_keepdim(sq, BOp.Add, axes) if keepdim else self.reduce(sq, BOp.Add, axes)
        return self.binary(red, self.const(n - correction, dt), BOp.Div)

    def layer_norm(self, x: int, weight: int | None = None, bias: int | None = None, eps: float = 1e-5) -> int:
        """`LayerNorm::forward` over the last axis (zyx-nn/src/layer_norm.rs:98-135): `(x - mean) / sqrt(var + eps)`
        (`var_keepdim`, correction 1), then `* weight`, `+ bias`."""
        dt, n = self[x].dtype, self[x].shape[-1]
        mean = self.binary(self.reduce_keepdim(x, BOp.Add, [-1]), self.const(n, dt), BOp.Div)
        variance = self.var(x, [-1], 1, keepdim=True)
        out = self.binary_b(self.binary_b(x, mean, BOp.Sub),
                            self.unary(self.binary(variance, self.const(eps, dt), BOp.Add), UOp.Sqrt), BOp.Div)
        if weight is not None:
            out = self.binary_b(out, weight, BOp.Mul)
        if bias is not None:
            out = self.binary_b(out, bias, BOp.Add)
        self.composites[out] = dict(kind="layer_norm", inputs=(x, weight, bias), params=dict(eps=float(eps)))
        return out

    def rms_norm(self, x: int, scale: int, eps: float = 1e-6) -> int:
        """`RMSNorm::forward` (zyx-nn/src/rms_norm.rs:26-32): `x * (mean_keepdim(x * x, [-1]) + eps).rsqrt() * scale`,
        rsqrt being `reciprocal().sqrt()` (zyx/src/tensor/elementwise.rs:305-307)."""
        dt, n = self[x].dtype, self[x].shape[-1]
        ms = self.binary(self.reduce_keepdim(self.binary(x, x, BOp.Mul), BOp.Add, [-1]), self.const(n, dt), BOp.Div)
        r = self.unary(self.unary(self.binary(ms, self.const(eps, dt), BOp.Add), UOp.Reciprocal), UOp.Sqrt)
        out = self.binary_b(self.binary_b(x, r, BOp.Mul), scale, BOp.Mul)
        self.composites[out] = dict(kind="rms_norm", inputs=(x, scale, None), params=dict(eps=float(eps)))
        return out

    def self_attention(self, qkv: int, n_head: int) -> int:
        """The core of `CausalSelfAttention::forward` between c_attn and c_proj (zyx-nn/src/causal_self_attention.rs:
        39-69; the reference applies no mask and, in evaluation, no dropout): qkv[B, T, 3C] is split along the last axis,
        each part viewed as [B, H, T, C / H], `softmax(q . k^T * scale, [-1]) . v`, back to [B, T, C]."""
        b, t, c3 = self[qkv].shape
        c = c3 // 3
        if c * 3 != c3 or c % n_head:
            raise ValueError(f"qkv of shape {self[qkv].shape} does not split into 3 x {n_head} heads")
        dh, dt = c // n_head, self[qkv].dtype
        q, k, v = (self.permute(self.reshape(self.narrow(qkv, 2, i * c, c), (b, t, n_head, dh)), (0, 2, 1, 3)) for i in range(3))
        scale = float(np.float32(1.0 / np.sqrt(float(dh))))
        att = self.softmax(self.binary(self.dot(q, self.t(k)), self.const(scale, dt), BOp.Mul), [-1])
        y = self.reshape(self.permute(self.dot(att, v), (0, 2, 1, 3)), (b, t, c))
        self.composites[y] = dict(kind="attention", inputs=(qkv,), params=dict(n_head=int(n_head), scale=scale))
        return y

    def cross_entropy(self, logits: int, target: int, reduction: str = "mean") -> int:
        """`Tensor::cross_entropy` (zyx/src/tensor/mod.rs:1639-1655) for a target of the logits' shape (one-hot or soft
        labels): `(-ln_softmax(logits, [classes]) * target).sum([classes])`, then the mean, the sum, or nothing;
        the class axis is 0 for 1-D logits and 1 otherwise."""
        if self[logits].shape != self[target].shape:
            raise ValueError(f"target shape {self[target].shape} is not the logits' {self[logits].shape}")
        cd = 0 if len(self[logits].shape) <= 1 else 1
        per_sample = self.reduce(self.binary(self.unary(self.ln_softmax(logits, [cd]), UOp.Neg), target, BOp.Mul), BOp.Add, [cd])
        if reduction == "mean":
            return self.mean(per_sample)
        if reduction == "sum":
            return self.sum_all(per_sample)
        if reduction == "none":
            return per_sample
        raise ValueError("invalid reduction for cross_entropy, expected mean, sum or none")

    # -- padding, slicing, pooling and convolution as the reference composes them ----------------------------------
    def pad_zeros(self, x: int, padding) -> int:
        """`Tensor::pad_zeros` (zyx/src/tensor/mod.rs:1161-1179): `padding[i] = (left, right)` for axis i, first axis
        first; negative amounts crop."""
        for axis, (l, r) in enumerate(padding):
            if l or r:
                x = self.pad(x, axis, l, self[x].shape[axis] + l + r)
        return x

    def rpad_zeros(self, x: int, padding) -> int:
        """`Tensor::rpad_zeros` (mod.rs:1202-1222): the first pair pads the LAST axis."""
        padding = list(padding)
        rank = len(self[x].shape)
        return self.pad_zeros(x, ([(0, 0)] * (rank - len(padding)) + padding[::-1]))

    def pad_value(self, x: int, padding, value) -> int:
        """`Tensor::pad` (mod.rs:1257-1275): `pad_zeros(x) + pad_zeros(ones).where_(zeros, value)`, where_ being
        `m * a + (1 - m) * b` (mod.rs:1617-1624)."""
        dt, xs = self[x].dtype, self[x].shape
        m = self.pad_zeros(self.expand(self.const(1, dt), xs), padding)
        shape = self[m].shape
        zeros, val = self.expand(self.const(0, dt), shape), self.expand(self.const(value, dt), shape)
        one_minus = self.binary(self.expand(self.const(1, dt), shape), m, BOp.Sub)
        filler = self.binary(self.binary(m, zeros, BOp.Mul), self.binary(one_minus, val, BOp.Mul), BOp.Add)
        return self.binary(self.pad_zeros(x, padding), filler, BOp.Add)

    def slice(self, x: int, ranges) -> int:
        """`Tensor::slice` with plain `start..stop` ranges for the leading axes."""
        for axis, (start, stop) in enumerate(ranges):
            x = self.narrow(x, axis, start, stop - start)
        return x

    def repeat(self, x: int, repeats) -> int:
        """`Tensor::repeat` (mod.rs:2766-2783): reshape to [1, d]..., expand to [r, d]..., reshape to [r * d]...."""
        repeats, xs = [int(r) for r in repeats], self[x].shape
        base = (1,) * (len(repeats) - len(xs)) + xs
        x = self.reshape(x, [v for d in base for v in (1, d)])
        x = self.expand(x, [v for r, d in zip(repeats, base) for v in (r, d)])
        return self.reshape(x, [r * d for r, d in zip(repeats, base)])

    def pool(self, x: int, kernel, stride=1, dilation=1) -> int:
        """`Tensor::pool` (mod.rs:2442-2544): the trailing len(kernel) axes [.., i..] become [.., o.., k..] windows,
        by repeat / slice / reshape only (no gather): element [.., o, k] is x[.., o * s + k * d]."""
        k_ = [int(k) for k in kernel]
        nk = len(k_)
        s_ = [int(stride)] * nk if np.isscalar(stride) else [int(v) for v in stride]
        d_ = [int(dilation)] * nk if np.isscalar(dilation) else [int(v) for v in dilation]
        if len(s_) == 1: s_ = s_ * nk
        if len(d_) == 1: d_ = d_ * nk
        shape = self[x].shape
        lead = list(shape[:len(shape) - nk])
        i_ = list(shape[len(shape) - nk:])
        o_ = [-(-(i - d * (k - 1)) // s) for i, d, k, s in zip(i_, d_, k_, s_)]
        full = [(0, d) for d in lead]
        x = self.repeat(x, [1] * len(lead) + [-(-(k * (i + d)) // i) for k, i, d in zip(k_, i_, d_)])
        x = self.slice(x, full + [(0, k * (i + d)) for k, i, d in zip(k_, i_, d_)])
        x = self.reshape(x, lead + [v for k, i, d in zip(k_, i_, d_) for v in (k, i + d)])
        x = self.slice(x, full + [r for k, o, s in zip(k_, o_, s_) for r in ((0, k), (0, o * s))])
        x = self.reshape(x, lead + [v for k, o, s in zip(k_, o_, s_) for v in (k, o, s)])
        x = self.slice(x, full + [r for k, o in zip(k_, o_) for r in ((0, k), (0, o), (0, 1))])
        x = self.reshape(x, lead + [v for k, o in zip(k_, o_) for v in (k, o)])
        n = len(lead)
        return self.permute(x, list(range(n)) + [n + 2 * i + 1 for i in range(nk)] + [n + 2 * i for i in range(nk)])

    def conv(self, x: int, w: int, bias: int | None = None, groups: int = 1, stride=1, dilation=1, padding=0) -> int:
        """`Tensor::conv` (mod.rs:2583-2680): pad, pool into windows, broadcast against the reshaped weight, sum over
        (cin, kernel). `padding`: one amount, one per spatial axis (both sides), 2 * nk amounts running from the last axis
        to the first as (before, after, before, after, ...) like the reference's, or one (before, after) pair per spatial
        axis, first axis first. The result node is remembered in `self.convs` with its operands and parameters, so that a 2-D
        convolution can be handed to the hand-written kernel as a whole (`match_conv`)."""
        xs, ws = self[x].shape, self[w].shape
        bs, cin_, (cout, cin), hw = xs[0], xs[1], ws[:2], list(ws[2:])
        nk = len(hw)
        if groups * cin != cin_ or len(xs) != len(ws):
            raise ValueError(f"input shape {xs} does not match the weights {ws}")
        if not np.isscalar(padding) and all(not np.isscalar(q) for q in padding):
            # (before, after) per spatial axis, first axis first
            if len(padding) != nk or any(len(q) != 2 for q in padding):
                raise ValueError(f"padding {padding} does not name {nk} (before, after) pairs")
            padding = [int(v) for q in reversed(list(padding)) for v in q]
        pads = [int(padding)] * (2 * nk) if np.isscalar(padding) else [int(v) for v in padding]
        if len(pads) == nk:  # one amount per spatial axis, both sides
            pads = [v for q in pads for v in (q, q)][::-1]
        elif len(pads) == 1:
            pads = pads * (2 * nk)
        stride = [int(stride)] * nk if np.isscalar(stride) else [int(v) for v in stride]
        dilation = [int(dilation)] * nk if np.isscalar(dilation) else [int(v) for v in dilation]
        px = self.rpad_zeros(x, [(pads[2 * i], pads[2 * i + 1]) for i in range(nk)])
        pooled = self.pool(px, hw, stride, dilation)
        rcout = cout // groups
        oyx = list(self[pooled].shape[2:2 + nk])
        t = self.reshape(pooled, [bs, groups, cin, 1] + oyx + hw)
        t = self.expand(t, [bs, groups, cin, rcout] + oyx + hw)
        t = self.permute(t, [0, 1, 3] + [4 + i for i in range(nk)] + [2] + [4 + nk + i for i in range(nk)])
        wr = self.reshape(w, [1, groups, rcout] + [1] * nk + [cin] + hw)
        prod = self.binary_b(t, wr, BOp.Mul)
        rank = len(self[prod].shape)
        out = self.reshape(self.reduce(prod, BOp.Add, [rank - 1 - i for i in range(nk + 1)]), [bs, cout] + oyx)
        core = out
        if bias is not None:
            out = self.binary_b(out, self.reshape(bias, [1, cout] + [1] * nk), BOp.Add)
        if nk == 2 and groups == 1:
            # rpad_zeros pairs run last axis first: (left, right) of W, then (top, bottom) of H
            info = dict(x=x, w=w, bias=bias, stride=tuple(stride), dilation=tuple(dilation), padding=(pads[2], pads[0]),
                        symmetric=pads[0] == pads[1] and pads[2] == pads[3], core=core)
            self.convs[out] = info
        return out

    def max_pool(self, x: int, kernel, stride=None, dilation=1, padding=None) -> int:
        """`Tensor::max_pool` (mod.rs:2706-2741): pad the trailing axes with the dtype's lowest value, pool, maximum over
        the window axes. `padding[i] = (before, after)` for the i-th of the trailing axes, first of them first."""
        nk = len(kernel)
        stride = list(kernel) if stride is None else stride
        rank = len(self[x].shape)
        orig = x
        if padding is not None and any(l or r for l, r in padding):
            x = self.pad_value(x, [(0, 0)] * (rank - nk) + list(padding), min_constant(self[x].dtype))
        pooled = self.pool(x, kernel, stride, dilation)
        prank = len(self[pooled].shape)
        out = self.reduce(pooled, BOp.Max, range(prank - nk, prank))
        if nk == 2:
            pads = [(0, 0), (0, 0)] if padding is None else [tuple(q) for q in padding]
            s2 = [int(stride)] * 2 if np.isscalar(stride) else [int(v) for v in stride]
            d2 = [int(dilation)] * 2 if np.isscalar(dilation) else [int(v) for v in dilation]
            if all(l == r for l, r in pads):
                self.pools[out] = dict(x=orig, kernel=tuple(int(k) for k in kernel), stride=tuple(s2), dilation=tuple(d2),
                                       padding=(pads[0][0], pads[1][0]))
        return out

    # -- reverse mode ---------------------------------------------------------------------------------------------
    def _grad_order(self, target: int, sources: set) -> list:
        """Nodes between the sources and the target, target first (`Graph::build_topo`, autograd.rs:427-493):
        operands of comparison, logical and bit ops are not followed."""
        needs: dict[int, bool] = {}

        def visit(i: int) -> bool:
            if i in needs:
                return needs[i]
            n = self[i]
            blocked = n.kind == "binary" and n.op in _NO_GRAD_BOPS
            dep = False
            if not blocked:
                for s in n.src:
                    dep = (visit(s) or s in sources) or dep
            needs[i] = dep
            return dep

        import sys
        old = sys.getrecursionlimit()
        sys.setrecursionlimit(max(old, 10000 + 4 * len(self.nodes)))
        try:
            visit(target)
        finally:
            sys.setrecursionlimit(old)
        # node ids are topological (operands are created before their users): descending id = reverse topological
        return sorted((i for i, d in needs.items() if d), reverse=True)

    def gradient(self, target: int, sources: Sequence[int], seed: int | None = None, _inside: int | None = None) -> list:
        """d target / d source for every source, as new nodes (`Runtime::gradient`, autograd.rs:14-424). The seed is
        1 in the target's dtype (or the node `seed`, of the target's shape: the gradient arriving from above); a source
        the target does not depend on gets zeros of its shape and dtype."""
        src_set = set(sources)
        grads: dict[int, int] = {target: self.expand(self.const(1, self[target].dtype), self[target].shape) if seed is None else seed}
        order = self._grad_order(target, src_set)
        wanted = set(order) | src_set

        def acc(x: int, g: int):
            if x in wanted:
                grads[x] = self.binary(grads[x], g, BOp.Add) if x in grads else g

        for cid in order:
            if cid not in grads:
                continue
            grad, n = grads[cid], self[cid]
            comp = self.composites.get(cid)
            if comp is not None and cid != _inside:
                # a module-level expression: the same rules, applied to its own nodes with the arriving gradient as seed
                ins = [i for i in comp["inputs"] if i is not None]
                gs = self.gradient(cid, ins, seed=grad, _inside=cid)
                record = dict(kind=comp["kind"], fwd=cid, dy=grad, inputs=comp["inputs"], grads=dict(zip(ins, gs)), params=comp["params"])
                for i, gi in zip(ins, gs):
                    self.fused_bwd[gi] = record
                    acc(i, gi)
                continue
            if n.kind == "unary":
                (x,) = n.src
                u = n.op
                if u == UOp.Neg:
                    acc(x, self.unary(grad, UOp.Neg))
                elif u == UOp.Reciprocal:  # -z^2 * grad
                    acc(x, self.binary(grad, self.unary(self.binary(cid, cid, BOp.Mul), UOp.Neg), BOp.Mul))
                elif u == UOp.Exp2:
                    acc(x, self.binary(grad, self.binary(cid, self.const(np.log(2.0), DType.F64), BOp.Mul), BOp.Mul))
                elif u == UOp.Log2:
                    acc(x, self.binary(grad, self.binary(x, self.const(np.log(2.0), DType.F64), BOp.Mul), BOp.Div))
                elif u == UOp.Sqrt:
                    acc(x, self.binary(grad, self.binary(cid, self.const(2, DType.I32), BOp.Mul), BOp.Div))
                elif u == UOp.Sin:
                    acc(x, self.binary(grad, self.unary(x, UOp.Cos), BOp.Mul))
                elif u == UOp.Cos:
                    acc(x, self.binary(grad, self.unary(self.unary(x, UOp.Sin), UOp.Neg), BOp.Mul))
                elif u == UOp.Exp:
                    acc(x, self.binary(grad, self.unary(x, UOp.Exp), BOp.Mul))
                elif u == UOp.Ln:
                    acc(x, self.binary(grad, x, BOp.Div))
                elif u == UOp.Abs:  # grad * ((x > 0) * 1 + (x < 0) * -1); the constants take x's dtype so the sign survives
                    zero, one, neg = (self.const(c, n.dtype) for c in (0, 1, -1))
                    pos = self.binary(self.binary(x, zero, BOp.Cmpgt), one, BOp.Mul)
                    ngt = self.binary(self.binary(x, zero, BOp.Cmplt), neg, BOp.Mul)
                    acc(x, self.binary(grad, self.binary(pos, ngt, BOp.Add), BOp.Mul))
                # Floor, Trunc, BitNot: no gradient
            elif n.kind == "binary":
                x, y = n.src
                b = n.op
                if b == BOp.Add:
                    acc(x, grad)
                    acc(y, grad)
                elif b == BOp.Sub:
                    acc(x, grad)
                    acc(y, self.unary(grad, UOp.Neg))
                elif b == BOp.Mul:
                    # 1 * v is v: the product with a gradient that is all ones (the seed seen through views) is not materialised
                    def times(v):
                        if _const_value(self, grad) == 1 and self[v].shape == self[grad].shape and self[v].dtype == n.dtype:
                            return v
                        return self.binary(grad, v, BOp.Mul)
                    acc(x, times(y))
                    acc(y, times(x))
                elif b == BOp.Div:
                    acc(x, self.binary(grad, y, BOp.Div))
                    x_mul = self.binary(self.unary(grad, UOp.Neg), x, BOp.Mul)
                    acc(y, self.binary(x_mul, self.binary(y, y, BOp.Mul), BOp.Div))
                elif b == BOp.Pow:
                    y_1 = self.binary(y, self.const(1, DType.U8), BOp.Sub)
                    y_mul = self.binary(y, self.binary(x, y_1, BOp.Pow), BOp.Mul)
                    acc(x, self.binary(grad, y_mul, BOp.Mul))
                    acc(y, self.binary(grad, self.binary(cid, self.unary(x, UOp.Ln), BOp.Mul), BOp.Mul))
                elif b == BOp.Mod:
                    acc(x, grad)
                    floored = self.unary(self.binary(x, y, BOp.Div), UOp.Floor)
                    acc(y, self.binary(self.unary(floored, UOp.Neg), grad, BOp.Mul))
                elif b == BOp.Max:  # strict comparisons: neither side of a tie receives anything
                    acc(x, self.binary(grad, self.binary(x, y, BOp.Cmpgt), BOp.Mul))
                    acc(y, self.binary(grad, self.binary(x, y, BOp.Cmplt), BOp.Mul))
            elif n.kind == "cast":
                acc(n.src[0], self.cast(grad, self[n.src[0]].dtype))
            elif n.kind == "reshape":
                acc(n.src[0], self.reshape(grad, self[n.src[0]].shape))
            elif n.kind == "expand":
                x = n.src[0]
                xs = self[x].shape
                pad = len(n.shape) - len(xs)
                axes = list(range(pad)) + [pad + i for i, d in enumerate(xs) if d == 1 and n.shape[pad + i] > 1]
                g = grad if not axes else self.reshape(self.reduce(grad, BOp.Add, axes), xs)
                acc(x, g)
            elif n.kind == "permute":
                inv = [0] * len(n.arg)
                for i, a in enumerate(n.arg):
                    inv[a] = i
                acc(n.src[0], self.permute(grad, inv))
            elif n.kind == "flip":
                acc(n.src[0], self.flip(grad, n.arg))
            elif n.kind == "pad":
                # `todo!()` in the reference (autograd.rs:252-254). The padding received no contribution from x and
                # cropped elements none from the result: the gradient is the same window moved back, i.e. a Pad by -lp
                # to x's extent.
                axis, lp = n.arg
                acc(n.src[0], self.pad(grad, axis, -lp, self[n.src[0]].shape[axis]))
            elif n.kind == "narrow":
                # `todo!()` in the reference (autograd.rs:255-257): zeros around the window that was kept
                axis, start = n.arg
                acc(n.src[0], self.pad(grad, axis, start, self[n.src[0]].shape[axis]))
            elif n.kind == "reduce":
                x = n.src[0]
                xs = self[x].shape
                keep = tuple(1 if i in n.arg else d for i, d in enumerate(xs))
                grad_e = self.expand(self.reshape(grad, keep), xs)
                if n.op == BOp.Add:
                    acc(x, grad_e)
                else:  # (1 - (x < max)) * grad
                    z_b = self.expand(self.reshape(cid, keep), xs)
                    cmp_f = self.cast(self.binary(x, z_b, BOp.Cmplt), self[x].dtype)
                    one_e = self.expand(self.const(1, self[x].dtype), xs)
                    acc(x, self.binary(self.binary(one_e, cmp_f, BOp.Sub), grad_e, BOp.Mul))
        out = []
        for s in sources:
            if s in grads:
                g = grads[s]
                if self[g].dtype != self[s].dtype:
                    g = self.cast(g, self[s].dtype)
                out.append(g)
            else:
                out.append(self.expand(self.const(0, self[s].dtype), self[s].shape))
        return out


# ---- matching: products summed over shared axes -> the hand-written GEMM -------------------------------------------------

@dataclasses.dataclass
class Contraction:
    """`out[batch, m, n] = sum_k a . b` found in the graph: `a` and `b` are the nodes whose buffers the GEMM reads in
    place (`[batch, m, k]`, or `[batch, k, m]` with trans_a; `[batch, k, n]`, or `[batch, n, k]` with trans_b)."""
    a: int
    b: int
    out: int
    m: int
    n: int
    k: int
    batch: int
    trans_a: bool
    trans_b: bool
    dtype: DType
    fallback: object = None   # the generated kernel for the same node, reading the same operand buffers (set by `lower`)
    # what the GEMM's epilogue applies before it stores (found by `match_linear`): out = act(alpha * product + bias),
    # then + residual, or * (residual > 0)
    epilogue: str = "none"    # "none" | "bias" | "bias_relu" | "bias_gelu"
    bias: int | None = None
    alpha: float = 1.0
    residual: int | None = None
    relu_mask: bool = False   # the residual operand is a relu's input or output: multiply by (residual > 0)
    mask_node: int | None = None  # the `v > 0` node of a relu folded into the epilogue (its v is never stored)


def _reshape_strides(old_shape, old_strides, new_shape):
    """Strides of `new_shape` over the same elements, or None when the reshape needs a copy. Dims of extent 1 carry
    stride 0; a group of old dims can be split or merged only where it is contiguous in itself."""
    old = [(d, st) for d, st in zip(old_shape, old_strides) if d != 1]
    new_strides = [0] * len(new_shape)
    oi = ni = 0
    while ni < len(new_shape):
        if new_shape[ni] == 1:
            ni += 1
            continue
        if oi >= len(old):
            return None
        np_, op_, nj, oj = new_shape[ni], old[oi][0], ni + 1, oi + 1
        while np_ != op_:
            if np_ < op_:
                if nj >= len(new_shape):
                    return None
                np_ *= new_shape[nj]
                nj += 1
            else:
                if oj >= len(old):
                    return None
                op_ *= old[oj][0]
                oj += 1
        if any(old[t][1] != old[t + 1][1] * old[t + 1][0] for t in range(oi, oj - 1)):
            return None
        st = old[oj - 1][1]
        for t in range(nj - 1, ni - 1, -1):
            if new_shape[t] != 1:
                new_strides[t] = st
                st *= new_shape[t]
        ni, oi = nj, oj
    return new_strides if oi == len(old) else None


def _contiguous(shape):
    st, out = 1, []
    for d in reversed(shape):
        out.append(0 if d == 1 else st)
        st *= d
    return out[::-1]


def view_of(graph: Graph, nid: int):
    """(base node, element strides of every dim of `nid` in the base's row-major buffer): looks through Permute,
    Expand and every Reshape that needs no copy. Anything else -- including a Flip -- is a base itself."""
    n = graph[nid]
    if n.kind == "permute":
        base, st = view_of(graph, n.src[0])
        return base, [st[a] for a in n.arg]
    if n.kind == "expand":
        base, st = view_of(graph, n.src[0])
        pad = len(n.shape) - len(st)
        return base, [0] * pad + [0 if graph[n.src[0]].shape[i] == 1 else v for i, v in enumerate(st)]
    if n.kind == "reshape":
        base, st = view_of(graph, n.src[0])
        new = _reshape_strides(graph[n.src[0]].shape, st, n.shape)
        if new is not None:
            return base, new
    return nid, _contiguous(n.shape)


def match_contraction(graph: Graph, nid: int):
    """`Graph::match_matmul` (zyx/src/vendor/matmul.rs:41-71) generalised from the canonical `dot` form to every
    Reduce(Add) over a Mul of two views: the forward product, both backward products (which autograd leaves as
    sums over the m or the n axis of the same broadcast product) and batched products. Returns None when the node is
    not such a product or its operands would need a copy first."""
    r = graph[nid]
    if r.kind != "reduce" or r.op != BOp.Add or r.dtype not in (DType.F32, DType.BF16, DType.F16):
        return None
    p = graph[r.src[0]]
    if p.kind != "binary" or p.op != BOp.Mul or any(graph[s].dtype != r.dtype for s in p.src):
        return None
    (xa, sa), (xb, sb) = view_of(graph, p.src[0]), view_of(graph, p.src[1])
    if graph[p.src[0]].shape != p.shape or graph[p.src[1]].shape != p.shape:
        return None  # a scalar operand
    groups = {"batch": [], "m": [], "n": [], "k": []}
    order = []
    for d, ext in enumerate(p.shape):
        if ext == 1:
            continue
        ina, inb, red = sa[d] != 0, sb[d] != 0, d in r.arg
        kind = "k" if (red and ina and inb) else None if red else "batch" if (ina and inb) else "m" if ina else "n" if inb else None
        if kind is None:
            return None
        groups[kind].append(d)
        if not red and (not order or order[-1] != kind):
            order.append(kind)
    if not groups["k"] or order not in (["batch", "m", "n"], ["batch", "n", "m"], ["m", "n"], ["n", "m"], ["batch", "m"], ["batch", "n"],
                                        ["m"], ["n"], ["batch"], []):
        return None
    if order and order[-1] == "m" and "n" in order:  # out is [.., n, m]: compute the transposed product
        xa, sa, xb, sb = xb, sb, xa, sa
        groups["m"], groups["n"] = groups["n"], groups["m"]

    def merged(dims, strides):
        """(extent, stride) of a group of dims seen as one, or None."""
        if not dims:
            return 1, 0
        if any(strides[dims[i]] != strides[dims[i + 1]] * p.shape[dims[i + 1]] for i in range(len(dims) - 1)):
            return None
        return _numel([p.shape[d] for d in dims]), strides[dims[-1]]

    parts = {}
    for name in ("batch", "m", "n", "k"):
        for tag, st in (("a", sa), ("b", sb)):
            if (name, tag) in (("n", "a"), ("m", "b")):
                continue
            got = merged(groups[name], st)
            if got is None:
                return None
            parts[name, tag] = got
    batch, m, n, k = parts["batch", "a"][0], parts["m", "a"][0], parts["n", "b"][0], parts["k", "a"][0]
    if batch * m * n == 1:
        return None  # an inner product of two vectors: one output element is a reduce, not a GEMM

    def layout(rows, row_st, cols, col_st, batch_st, base):
        """False: [rows, cols] row-major; True: [cols, rows]; None: neither."""
        if _numel(graph[base].shape) != batch * rows * cols or (batch > 1 and batch_st != rows * cols):
            return None
        if (cols == 1 or col_st == 1) and (rows == 1 or row_st == cols):
            return False
        if (rows == 1 or row_st == 1) and (cols == 1 or col_st == rows):
            return True
        return None

    ta = layout(m, parts["m", "a"][1], k, parts["k", "a"][1], parts["batch", "a"][1], xa)
    tb = layout(k, parts["k", "b"][1], n, parts["n", "b"][1], parts["batch", "b"][1], xb)
    if ta is None or tb is None:
        return None
    return Contraction(xa, xb, nid, m, n, k, batch, ta, tb, r.dtype)


@dataclasses.dataclass
class SoftmaxRows:
    """`out[rows, cols] = softmax(x, last axis)` found in the graph; `x` is the node whose buffer the fused kernel reads."""
    x: int
    out: int
    rows: int
    cols: int


def _keepdim_reduce_of(graph: Graph, nid: int, rop: BOp, src: int):
    """True when `nid` is `src` reduced with `rop` over its last axis and broadcast back to src's shape."""
    base, st = view_of(graph, nid)
    b, shape = graph[base], graph[src].shape
    return (b.kind == "reduce" and b.op == rop and b.src[0] == src and b.arg == (len(shape) - 1,)
            and graph[nid].shape == shape and st == _contiguous(shape[:-1]) + [0])


def match_softmax(graph: Graph, nid: int):
    """`e = exp(x - max_keepdim(x)); e / sum_keepdim(e)` over the last axis (`Tensor::softmax`,
    zyx/src/tensor/mod.rs:1457-1461) in f32: the shape the fused row-softmax kernel computes in one pass."""
    n = graph[nid]
    if n.kind != "binary" or n.op != BOp.Div or n.dtype != DType.F32 or len(n.shape) < 1 or n.shape[-1] < 2:
        return None
    e, den = n.src
    ne = graph[e]
    if ne.kind != "unary" or ne.op != UOp.Exp or ne.dtype != DType.F32 or not _keepdim_reduce_of(graph, den, BOp.Add, e):
        return None
    d = graph[ne.src[0]]
    if d.kind != "binary" or d.op != BOp.Sub or graph[d.src[0]].dtype != DType.F32:
        return None
    x, mx = d.src
    if graph[x].shape != n.shape or not _keepdim_reduce_of(graph, mx, BOp.Max, x):
        return None
    base, st = view_of(graph, x)
    if st != _contiguous(n.shape) or _numel(graph[base].shape) != _numel(n.shape):
        base = x  # not a plain view of a whole buffer: x gets its own
    return SoftmaxRows(base, nid, _numel(n.shape[:-1]), n.shape[-1])


@dataclasses.dataclass
class RowColReduce:
    """`out = reduce(x)` over the last axis (x seen as [rows, cols] -> [rows]) or over the leading axis (-> [cols]) of a
    tensor that already has a buffer: the shapes the two-stage reduce kernel takes."""
    x: int
    out: int
    rows: int
    cols: int
    axis0: bool
    op: str
    dtype: DType
    mul: float = 0.0          # out = reduce * mul + base when a base is named (`base - reduce * c` is mul = -c)
    base: int | None = None


def match_reduce(graph: Graph, nid: int, stored) -> RowColReduce | None:
    """A Reduce(Add | Max) whose operand is a plain view of a whole buffer that exists already (a leaf or a node in
    `stored`: an operand that is an expression stays fused into the generated reduce), reduced over its trailing axes
    or over its leading axes, with enough elements per result for the tree-shaped kernel to pay."""
    r = graph[nid]
    if r.kind != "reduce" or r.dtype not in (DType.F32, DType.BF16, DType.F16, DType.I32):
        return None
    x = r.src[0]
    xs = graph[x].shape
    base, st = view_of(graph, x)
    if st != _contiguous(xs) or _numel(graph[base].shape) != _numel(xs) or not (graph[base].kind == "leaf" or base in stored):
        return None
    k, n = len(r.arg), len(xs)
    if r.arg == tuple(range(n - k, n)):
        rows, cols, axis0 = _numel(xs[:n - k]), _numel(xs[n - k:]), False
    elif r.arg == tuple(range(k)):
        rows, cols, axis0 = _numel(xs[:k]), _numel(xs[k:]), True
    else:
        return None
    if (rows if axis0 else cols) < 256:
        return None  # short reductions: one serial loop per result is as good and needs no second launch
    return RowColReduce(base, nid, rows, cols, axis0, "sum" if r.op == BOp.Add else "max", r.dtype)


@dataclasses.dataclass
class Conv2dMatch:
    """`out = conv(x, w) (+ bias) (then relu)` for NCHW x and [Cout, C, KH, KW] w, groups = 1, equal padding on both sides
    of an axis: what ZHIP_K_CONV2D computes in one launch. x, w, bias are the nodes whose buffers it reads."""
    x: int
    w: int
    bias: int | None
    out: int
    dims: tuple      # N, C, H, W, Cout, KH, KW
    stride: tuple
    padding: tuple
    dilation: tuple
    relu: bool
    dtype: DType
    fallback: object = None


@dataclasses.dataclass
class MaxPoolMatch:
    """`out = max_pool(x)` over the last two axes (ZHIP_K_MAX_POOL2D)."""
    x: int
    out: int
    planes: int
    hw: tuple
    kernel: tuple
    stride: tuple
    padding: tuple
    dilation: tuple
    dtype: DType


def _is_relu_of(graph: Graph, nid: int):
    """The node x when `nid` is `x.cmpgt(0) * x` (`Tensor::relu`, zyx/src/tensor/elementwise.rs:289-293), else None."""
    n = graph[nid]
    if n.kind != "binary" or n.op != BOp.Mul:
        return None
    c, x = graph[n.src[0]], n.src[1]
    if c.kind == "binary" and c.op == BOp.Cmpgt and c.src[0] == x:
        z = graph[c.src[1]]
        if z.kind == "const" and z.arg == 0:
            return x
    return None


def match_conv(graph: Graph, nid: int, users: dict | None = None) -> Conv2dMatch | None:
    """A node `Graph.conv` built, or the `relu` of one whose only consumers are that relu's two nodes (`users`: node ->
    its consumers among the nodes being computed, -1 standing for the caller; without it no relu is folded in). The composition of pads, window
    views and the broadcast product is recognised by where it came from rather than by its thirty-odd movement nodes:
    `Graph.conv` notes operands and parameters next to the node it returns."""
    relu, c = False, nid
    inner = _is_relu_of(graph, nid)
    if inner is not None and inner in graph.convs and users is not None and users.get(inner, set()) == {graph[nid].src[0], nid}:
        relu, c = True, inner
    info = graph.convs.get(c)
    if info is None or not info["symmetric"] or graph[nid].dtype not in (DType.F32, DType.BF16):
        return None
    xs, ws = graph[info["x"]].shape, graph[info["w"]].shape
    return Conv2dMatch(info["x"], info["w"], info["bias"], nid, (xs[0], xs[1], xs[2], xs[3], ws[0], ws[2], ws[3]), info["stride"],
                       info["padding"], info["dilation"], relu, graph[nid].dtype)


def consumers(graph: Graph, outputs: Sequence[int], stored=()) -> dict:
    """node -> the nodes that read it, among those `outputs` are computed from (not looking behind stored nodes)."""
    users: dict[int, set] = {o: {-1} for o in outputs}  # the caller reads the outputs
    seen, stack = set(stored), list(outputs)
    while stack:
        i = stack.pop()
        if i in seen:
            continue
        seen.add(i)
        for s in graph[i].src:
            users.setdefault(s, set()).add(i)
            stack.append(s)
    return users


def match_max_pool(graph: Graph, nid: int) -> MaxPoolMatch | None:
    info = graph.pools.get(nid)
    if info is None or graph[nid].dtype not in (DType.F32, DType.BF16):
        return None
    xs = graph[info["x"]].shape
    return MaxPoolMatch(info["x"], nid, _numel(xs[:-2]), (xs[-2], xs[-1]), info["kernel"], info["stride"], info["padding"],
                        info["dilation"], graph[nid].dtype)




# ---- matching by template: an expression has the shape of one the builders above produce -----------------------------

def same_tree(graph: Graph, nid: int, tgraph: Graph, tid: int, bind: dict) -> bool:
    """True when the expression below `nid` is, node for node, the expression below `tid` of `tgraph`; the leaves of
    the template stand for any node of their shape and dtype. `bind` (template node -> graph node) is extended; a
    template node reached twice has to meet the same graph node both times."""
    todo = [(nid, tid)]
    while todo:
        a, t = todo.pop()
        if t in bind:
            if bind[t] != a:
                return False
            continue
        na, nt = graph[a], tgraph[t]
        if na.shape != nt.shape or na.dtype != nt.dtype:
            return False
        if nt.kind != "leaf":
            if na.kind != nt.kind or na.op != nt.op or len(na.src) != len(nt.src) or na.arg != nt.arg:
                return False
            todo.extend(zip(na.src, nt.src))
        bind[t] = a
    return True


_TEMPLATES: dict = {}


def _template(key, build):
    """Templates are built once per (kind, shape, dtype, ...)."""
    if key not in _TEMPLATES:
        if len(_TEMPLATES) > 256:
            _TEMPLATES.clear()
        t = Graph()
        _TEMPLATES[key] = (t, build(t))
    return _TEMPLATES[key]


def _is_gelu_of(graph: Graph, nid: int):
    """The node x when `nid` is `Graph.gelu(x)`, else None."""
    n = graph[nid]
    if n.kind != "binary" or n.op != BOp.Mul or n.dtype not in (DType.F32, DType.BF16, DType.F16):
        return None

    def build(t):
        x = t.leaf(n.shape, n.dtype)
        return x, t.gelu(x)

    t, (x, root) = _template(("gelu", n.shape, n.dtype), build)
    bind: dict = {}
    return bind[x] if same_tree(graph, nid, t, root, bind) else None


def _interior(graph: Graph, root: int, stop: int) -> set:
    """Nodes strictly between `root` and `stop` (the expression of root in terms of stop)."""
    seen, stack = set(), [root]
    while stack:
        i = stack.pop()
        for s_ in graph[i].src:
            if s_ != stop and s_ not in seen and graph[s_].kind != "const":
                seen.add(s_)
                stack.append(s_)
    return seen


def _plain(graph: Graph, nid: int):
    """The node whose buffer holds `nid` element for element (reshapes and permutes that keep the linear order), or
    None when `nid` is a strided or broadcast view."""
    base, st = view_of(graph, nid)
    shape = graph[nid].shape
    if _numel(graph[base].shape) != _numel(shape):
        return None
    want = _contiguous(shape)
    return base if all(d == 1 or a == b for d, a, b in zip(shape, st, want)) else None


def _row_vector(graph: Graph, nid: int):
    """The [n] node that `nid` ([.., n]) repeats along all its leading axes, or None."""
    base, st = view_of(graph, nid)
    shape = graph[nid].shape
    if not shape or _numel(graph[base].shape) != shape[-1] or shape[-1] == 1:
        return None
    if st[-1] != 1 or any(d != 1 and v != 0 for d, v in zip(shape[:-1], st[:-1])):
        return None
    return base


def _const_value(graph: Graph, nid: int):
    """The scalar a node broadcasts, or None."""
    base, _ = view_of(graph, nid)
    n = graph[base]
    return n.arg if n.kind == "const" else None


def match_linear(graph: Graph, nid: int, users: dict, relu_mask: dict):
    """A product summed over shared axes together with what the GEMM kernel's epilogue can apply to it on the way out
    (`Linear::forward` zyx-nn/src/linear.rs:38-44 with the activation behind it, and the three products of its reverse
    pass with the SGD step zyx-optim/src/sgd.rs:45-84 behind them):
      act(product + bias)            act = relu | gelu | nothing, bias repeated along the rows
      w - product * c                a parameter update: alpha = -c, residual = w
      product * (v > 0)              the reverse of a relu: residual = v (or relu(v) where only that is stored)
    `users`: node -> consumers among the nodes being computed; an inner node folded away must have no other reader.
    Returns a `Contraction` whose `out` is `nid`, or None."""
    n = graph[nid]
    if n.dtype not in (DType.F32, DType.BF16, DType.F16) or n.kind not in ("binary", "reduce", "reshape", "permute"):
        return None

    def only_reader(node, *readers):
        return users.get(node, set()) <= set(readers)

    def product(node, reader):
        """The Contraction of the reduce that `node` shows element for element, if `reader` alone reads it."""
        base = _plain(graph, node)
        if base is None or graph[base].kind != "reduce":
            return None
        chain, i = [], node
        while i != base:  # the views between node and the reduce: each read by the next only
            chain.append(i)
            i = graph[i].src[0]
        chain.append(base)
        for j, v in enumerate(chain):
            if not only_reader(v, reader if j == 0 else chain[j - 1]):
                return None
        return match_contraction(graph, base)

    cur, act, mask_node = nid, None, None
    v = _is_relu_of(graph, cur)
    if v is not None and users.get(v, set()) == {graph[cur].src[0], cur}:
        act, mask_node, cur = "relu", graph[cur].src[0], v
    else:
        v = _is_gelu_of(graph, cur)
        if v is not None:
            inner = _interior(graph, cur, v)
            if all(users.get(i, set()) <= inner | {cur} for i in inner | {v}):
                act, cur = "gelu", v
    c = graph[cur]
    if c.kind == "binary" and c.op == BOp.Add:
        for core, other in (c.src, c.src[::-1]):
            bias = _row_vector(graph, other)
            if bias is None or graph[bias].dtype != n.dtype:
                continue
            m = product(core, cur)
            if m is not None and m.batch == 1 and _numel(graph[bias].shape) == m.n:
                m.out, m.bias, m.mask_node = nid, bias, mask_node
                m.epilogue = {None: "bias", "relu": "bias_relu", "gelu": "bias_gelu"}[act]
                return m
        if act is None:  # (product + bias) + a tensor of the result's shape: the skip connection around a Linear
            for inner, res in (c.src, c.src[::-1]):
                rb, ni = _plain(graph, res), graph[inner]
                if rb is None or graph[rb].dtype != n.dtype or ni.kind != "binary" or ni.op != BOp.Add or not only_reader(inner, cur):
                    continue
                for core, other in (ni.src, ni.src[::-1]):
                    bias = _row_vector(graph, other)
                    if bias is None or graph[bias].dtype != n.dtype:
                        continue
                    m = product(core, inner)
                    if m is not None and m.batch == 1 and _numel(graph[bias].shape) == m.n:
                        m.out, m.bias, m.epilogue, m.residual = nid, bias, "bias", rb
                        return m
        return None
    if act is not None:
        return None  # an activation straight on a product: the kernel has no such epilogue
    if c.kind == "binary" and c.op == BOp.Sub:
        w, scaled = c.src
        sc = graph[scaled]
        wb = _plain(graph, w)
        if wb is None or sc.kind != "binary" or sc.op != BOp.Mul:
            return None
        for core, other in (sc.src, sc.src[::-1]):
            k = _const_value(graph, other)
            if k is None or not only_reader(scaled, cur):
                continue
            m = product(core, scaled)
            if m is not None and m.batch == 1:
                m.out, m.alpha, m.residual = nid, -float(k), wb
                return m
        return None
    if c.kind == "binary" and c.op == BOp.Mul:
        for core, other in (c.src, c.src[::-1]):
            o = graph[other]
            if o.kind != "binary" or o.op != BOp.Cmpgt or _const_value(graph, o.src[1]) != 0:
                continue
            shown = relu_mask.get(other)
            if shown is None:  # relu(v) > 0 is v > 0: where the relu itself is computed, read that
                shown = next((r for r in users.get(o.src[0], ()) if r >= 0 and _is_relu_of(graph, r) == o.src[0]), o.src[0])
            vb = _plain(graph, shown)
            if vb is None or graph[vb].dtype != n.dtype:
                continue
            m = product(core, cur)
            if m is not None and m.batch == 1:
                m.out, m.residual, m.relu_mask = nid, vb, True
                return m
    return None


def match_reduce_update(graph: Graph, nid: int, users: dict) -> RowColReduce | None:
    """`b - reduce(x) * c` with x a whole buffer that exists (a bias update, zyx-optim/src/sgd.rs:45-84 applied to
    the column sums the reverse pass of a broadcast bias leaves): one launch of the reduce kernel with its scale and
    base operands, whatever the length of the reduction."""
    n = graph[nid]
    if n.kind != "binary" or n.op != BOp.Sub or n.dtype != DType.F32:
        return None
    b, scaled = n.src
    bb, sc = _plain(graph, b), graph[scaled]
    if bb is None or sc.kind != "binary" or sc.op != BOp.Mul:
        return None
    if not users.get(scaled, set()) <= {nid}:
        return None
    for core, other in (sc.src, sc.src[::-1]):
        k = _const_value(graph, other)
        base = _plain(graph, core)
        if k is None or base is None or graph[base].kind != "reduce" or graph[base].op != BOp.Add:
            continue
        r = graph[base]
        x = r.src[0]
        xs = graph[x].shape
        xb = _plain(graph, x)
        if xb is None:
            continue
        kk, rank = len(r.arg), len(xs)
        if r.arg == tuple(range(rank - kk, rank)):
            rows, cols, axis0 = _numel(xs[:rank - kk]), _numel(xs[rank - kk:]), False
        elif r.arg == tuple(range(kk)):
            rows, cols, axis0 = _numel(xs[:kk]), _numel(xs[kk:]), True
        else:
            continue
        return RowColReduce(xb, nid, rows, cols, axis0, "sum", r.dtype, mul=-float(k), base=bb)
    return None


@dataclasses.dataclass
class CrossEntropyMatch:
    """`Graph.cross_entropy(x, target, "mean")` and / or its gradient with respect to x, found in the graph: one launch
    of ZHIP_K_CROSS_ENTROPY with dense targets writes both."""
    x: int
    target: int
    rows: int
    cols: int
    gscale: float
    grad: int | None = None
    mean: int | None = None

    @property
    def out(self):
        return self.grad if self.grad is not None else self.mean


def _ce_template(rows: int, cols: int, reduction: str):
    def build(t):
        x, y = t.leaf((rows, cols), DType.F32), t.leaf((rows, cols), DType.F32)
        loss = t.cross_entropy(x, y, reduction)
        (gx,) = t.gradient(loss, [x])
        return x, y, loss, gx

    return _template(("ce", rows, cols, reduction), build)


def scan_cross_entropy(graph: Graph, nodes) -> dict:
    """node -> CrossEntropyMatch for the mean cross-entropy losses among `nodes` and the gradients the reverse rules
    derive from such a loss (mean or sum) for its logits. The gradient's template is what `Graph.gradient` makes of
    the template loss: the same rules applied to the same expression give the same expression, so the comparison is
    node for node. A loss and a gradient over the same logits and target share one match (one launch)."""
    found: dict[tuple, CrossEntropyMatch] = {}
    by_node: dict[int, CrossEntropyMatch] = {}
    for nid in nodes:
        n = graph[nid]
        if n.dtype != DType.F32 or n.kind != "binary":
            continue
        if n.shape == (1,) and n.op == BOp.Div:
            r = graph[n.src[0]]
            per = graph[r.src[0]] if r.kind == "reduce" and r.src else None
            prod = graph[per.src[0]] if per is not None and per.kind == "reduce" else None
            if prod is None or len(prod.shape) != 2:
                continue
            rows, cols = prod.shape
            t, (tx, ty, tloss, _) = _ce_template(rows, cols, "mean")
            bind: dict = {}
            if same_tree(graph, nid, t, tloss, bind):
                m = found.setdefault((bind[tx], bind[ty]), CrossEntropyMatch(bind[tx], bind[ty], rows, cols, 1.0 / rows))
                if m.mean is None:
                    m.mean = nid
                    by_node[nid] = m
        elif len(n.shape) == 2:
            rows, cols = n.shape
            for reduction, gscale in (("mean", 1.0 / rows), ("sum", 1.0)):
                t, (tx, ty, _, tgx) = _ce_template(rows, cols, reduction)
                if graph[nid].op != t[tgx].op:
                    continue
                bind = {}
                if same_tree(graph, nid, t, tgx, bind) and tx in bind and ty in bind:
                    m = found.setdefault((bind[tx], bind[ty]), CrossEntropyMatch(bind[tx], bind[ty], rows, cols, gscale))
                    if m.grad is None and m.gscale == gscale:
                        m.grad = nid
                        by_node[nid] = m
                    break
    return by_node


@dataclasses.dataclass
class NormRowsMatch:
    """`out = layer_norm(x, w, b)` or `rms_norm(x, scale)` over the last axis (ZHIP_K_NORM_ROWS)."""
    x: int
    w: int | None
    b: int | None
    out: int
    rows: int
    cols: int
    rms: bool
    eps: float
    dtype: DType


@dataclasses.dataclass
class NormBwdMatch:
    """The gradients of a norm with respect to x, weight and bias for the arriving gradient dy, optionally with the
    gradient of a skip branch added to dx in the same pass (ZHIP_K_NORM_ROWS_BWD). `dx`, `dw`, `db`: the nodes that
    receive the results (None: not asked for)."""
    x: int
    w: int | None
    dy: int
    add: int | None
    dx: int
    dw: int | None
    db: int | None
    rows: int
    cols: int
    rms: bool
    eps: float
    dtype: DType

    @property
    def out(self):
        return self.dx


@dataclasses.dataclass
class AttentionMatch:
    """`y = self_attention(qkv)` (ZHIP_K_ATTENTION); `lse`: the launch also leaves the row log-sum-exps the backward
    kernel reads, in a buffer that belongs to `out` and is no graph node."""
    qkv: int
    out: int
    dims: tuple      # B, T, H, dh
    scale: float
    lse: bool
    dtype: DType


@dataclasses.dataclass
class AttentionBwdMatch:
    """d qkv of `self_attention` for the arriving gradient dy (ZHIP_K_ATTENTION_BWD): reads qkv, the forward's y and
    row log-sum-exps."""
    qkv: int
    y: int
    dy: int
    out: int
    dims: tuple
    scale: float
    dtype: DType


def _rows_cols(shape):
    return _numel(shape[:-1]), shape[-1]


def match_norm(graph: Graph, nid: int) -> NormRowsMatch | None:
    comp = graph.composites.get(nid)
    if comp is None or comp["kind"] not in ("layer_norm", "rms_norm") or graph[nid].dtype not in (DType.F32, DType.BF16):
        return None
    x, w, b = comp["inputs"]
    cols = graph[nid].shape[-1]
    if any(v is not None and (_numel(graph[v].shape) != cols or graph[v].dtype != graph[nid].dtype) for v in (w, b)):
        return None
    rows, cols = _rows_cols(graph[nid].shape)
    return NormRowsMatch(x, w, b, nid, rows, cols, comp["kind"] == "rms_norm", comp["params"]["eps"], graph[nid].dtype)


def match_norm_bwd(graph: Graph, nid: int, users: dict) -> NormBwdMatch | None:
    """`nid` is one of the gradients a norm's reverse pass produced, or the sum of its dx and one other gradient of
    the same tensor (the skip branch of a pre-norm block) where nothing else reads dx."""
    n = graph[nid]
    rec, add, dx_node = graph.fused_bwd.get(nid), None, None
    if rec is None and n.kind == "binary" and n.op == BOp.Add:
        for a, other in (n.src, n.src[::-1]):
            r = graph.fused_bwd.get(a)
            if r is not None and r["kind"] in ("layer_norm", "rms_norm") and r["grads"].get(r["inputs"][0]) == a \
                    and users.get(a, set()) <= {nid} and graph[other].shape == n.shape:
                rec, add, dx_node = r, other, nid
                break
    if rec is None or rec["kind"] not in ("layer_norm", "rms_norm") or n.dtype not in (DType.F32, DType.BF16):
        return None
    x, w, b = rec["inputs"]
    gx = rec["grads"][x]
    if dx_node is None:  # reached through dw or db: dx goes where it would go when reached through itself
        dx_node = gx
        readers = users.get(gx, set())
        if len(readers) == 1:
            (u,) = readers
            if u >= 0 and graph[u].kind == "binary" and graph[u].op == BOp.Add and gx in graph[u].src and graph[u].shape == graph[gx].shape \
                    and graph[u].src[0] != graph[u].src[1]:
                dx_node, add = u, [v for v in graph[u].src if v != gx][0]

    def wanted(v):
        return v is not None and (rec["grads"][v] in users or rec["grads"][v] == nid)

    rows, cols = _rows_cols(graph[x].shape)
    return NormBwdMatch(x, w, rec["dy"], add, dx_node, rec["grads"][w] if wanted(w) else None, rec["grads"][b] if wanted(b) else None,
                        rows, cols, rec["kind"] == "rms_norm", rec["params"]["eps"], n.dtype)


def match_attention(graph: Graph, nid: int, users: dict) -> AttentionMatch | None:
    comp = graph.composites.get(nid)
    if comp is None or comp["kind"] != "attention" or graph[nid].dtype not in (DType.F32, DType.BF16):
        return None
    (qkv,) = comp["inputs"]
    b, t, c = graph[nid].shape
    h = comp["params"]["n_head"]
    gq = None
    for g_, rec in graph.fused_bwd.items():  # does a backward of this forward belong to what is being computed?
        if rec["fwd"] == nid and (g_ in users):
            gq = g_
    return AttentionMatch(qkv, nid, (b, t, h, c // h), comp["params"]["scale"], gq is not None, graph[nid].dtype)


def match_attention_bwd(graph: Graph, nid: int) -> AttentionBwdMatch | None:
    rec = graph.fused_bwd.get(nid)
    if rec is None or rec["kind"] != "attention" or graph[nid].dtype not in (DType.F32, DType.BF16):
        return None
    (qkv,) = rec["inputs"]
    b, t, c = graph[rec["fwd"]].shape
    h = rec["params"]["n_head"]
    return AttentionBwdMatch(qkv, rec["fwd"], rec["dy"], nid, (b, t, h, c // h), rec["params"]["scale"], graph[nid].dtype)


def match_operands(m) -> tuple:
    """Nodes whose buffers a matched kernel reads, in argument order."""
    if isinstance(m, NormRowsMatch):
        return (m.x,) + tuple(v for v in (m.w, m.b) if v is not None)
    if isinstance(m, NormBwdMatch):
        return (m.x,) + ((m.w,) if m.w is not None else ()) + (m.dy,) + ((m.add,) if m.add is not None else ())
    if isinstance(m, AttentionMatch):
        return (m.qkv,)
    if isinstance(m, AttentionBwdMatch):
        return (m.qkv, m.y, m.dy)
    if isinstance(m, Contraction):
        return (m.a, m.b) + ((m.bias,) if m.bias is not None else ()) + ((m.residual,) if m.residual is not None else ())
    if isinstance(m, RowColReduce):
        return (m.x,) + ((m.base,) if m.base is not None else ())
    if isinstance(m, CrossEntropyMatch):
        return (m.x, m.target)
    if isinstance(m, Conv2dMatch):
        return (m.x, m.w) + ((m.bias,) if m.bias is not None else ())
    return (m.x,)


MATCHED = (Contraction, SoftmaxRows, RowColReduce, Conv2dMatch, MaxPoolMatch, CrossEntropyMatch, NormRowsMatch, NormBwdMatch,
           AttentionMatch, AttentionBwdMatch)


# ---- lowering ---------------------------------------------------------------------------------------------------------

@dataclasses.dataclass
class Alias:
    """`out` shows `base` element for element (a reshape, or permutes that cancel): it shares base's buffer."""
    out: int
    base: int


@dataclasses.dataclass
class LoweredKernel:
    image: bytes
    inputs: list      # node ids of the buffers read, in parameter order
    output: int       # node id of the buffer written
    elements: int
    more_outputs: tuple = ()  # further buffers written, after `output` in the argument list


class _V:
    """An index value that lives in an IR op (Python ints stand for constants and are folded)."""
    __slots__ = ("id",)

    def __init__(self, op_id: int):
        self.id = op_id


class _Emitter:
    LOCAL = 64

    def __init__(self, graph: Graph, stored: set):
        self.g, self.stored = graph, stored
        self.relu_mask: dict[int, int] = {}  # `v > 0` node of a relu whose v is not stored -> the stored relu(v)
        self.inline: set = set()  # reduces computed inside the kernel of the one expression that reads them element for element

    # index arithmetic with constant folding
    def _ix(self, v):
        if isinstance(v, _V):
            return v.id
        if v not in self.consts:
            self.consts[v] = self.k.const_idx(v)
        return self.consts[v]

    def _op(self, a, b, bop, fold):
        if not isinstance(a, _V) and not isinstance(b, _V):
            return fold(a, b)
        return _V(self.k.binary(self._ix(a), self._ix(b), bop))

    def add(self, a, b):
        if not isinstance(a, _V) and a == 0: return b
        if not isinstance(b, _V) and b == 0: return a
        return self._op(a, b, BOp.Add, lambda p, q: p + q)

    def mul(self, a, c: int):
        if c == 1: return a
        if c == 0: return 0
        return self._op(a, c, BOp.Mul, lambda p, q: p * q)

    def div(self, a, c: int):
        return a if c == 1 else self._op(a, c, BOp.Div, lambda p, q: p // q)

    def mod(self, a, c: int):
        return 0 if c == 1 else self._op(a, c, BOp.Mod, lambda p, q: p % q)

    def ravel(self, idx, shape):
        lin, stride = 0, 1
        for i, d in zip(reversed(idx), reversed(shape)):
            lin = self.add(lin, self.mul(i, stride))
            stride *= d
        return lin

    def unravel(self, lin, shape):
        """lin < numel(shape) for every caller, so the first component of extent > 1 needs no remainder."""
        idx, total = [], _numel(shape)
        remaining = total
        for d in shape:
            stride = remaining // d
            if d == 1:
                idx.append(0)
            else:
                q = self.div(lin, stride)
                idx.append(q if remaining == total else self.mod(q, d))
            remaining = stride
        return idx

    # expression emission -----------------------------------------------------------------------------------------
    def value(self, nid: int, idx: list, root: bool = False):
        """IR op holding element `idx` of node `nid`."""
        key = (nid, tuple(i.id if isinstance(i, _V) else ("c", i) for i in idx))
        if key in self.memo:
            return self.memo[key]
        n, k = self.g[nid], self.k
        if (n.kind == "leaf" or nid in self.stored) and not root:
            v = k.load(self.params[nid], self._ix(self.ravel(idx, n.shape)))
        elif n.kind == "reduce":
            v = self._reduce(n, idx)
        elif n.kind == "const":
            v = k.const(n.arg, n.dtype)
        elif n.kind == "unary":
            v = k.unary(self.value(n.src[0], idx), n.op)
        elif n.kind == "binary":
            x, y = n.src
            x = self.relu_mask.get(nid, x)
            dt = self.g.operand_dtype(x, y)
            v = k.binary(self.operand(x, idx, dt), self.operand(y, idx, dt), n.op)
        elif n.kind == "cast":
            v = k.cast(self.value(n.src[0], idx), n.dtype)
        elif n.kind == "reshape":
            v = self.value(n.src[0], self.unravel(self.ravel(idx, n.shape), self.g[n.src[0]].shape))
        elif n.kind == "expand":
            xs = self.g[n.src[0]].shape
            pad = len(n.shape) - len(xs)
            v = self.value(n.src[0], [0 if d == 1 else idx[pad + i] for i, d in enumerate(xs)])
        elif n.kind == "permute":
            x_idx = [0] * len(idx)
            for i, a in enumerate(n.arg):
                x_idx[a] = idx[i]
            v = self.value(n.src[0], x_idx)
        elif n.kind == "narrow":
            axis, start = n.arg
            x_idx = list(idx)
            x_idx[axis] = self.add(idx[axis], start)
            v = self.value(n.src[0], x_idx)
        elif n.kind == "pad":
            # the reference's rule (zyx/src/kernel/linearize.rs:349-382): pc = (0 <= j < extent); the load happens at
            # pc * j and its value is multiplied by pc
            axis, lp = n.arg
            ext = self.g[n.src[0]].shape[axis]
            i = idx[axis]
            x_idx = list(idx)
            if not isinstance(i, _V):
                j = i - lp
                if 0 <= j < ext:
                    x_idx[axis] = j
                    v = self.value(n.src[0], x_idx)
                else:
                    v = k.const(0, n.dtype)
            else:
                j = self.add(i, -lp) if lp <= 0 else _V(k.sub(i.id, self._ix(lp)))
                inside = None
                if lp > 0:
                    inside = k.cmpge(j.id, self._ix(0))
                if n.shape[axis] - lp > ext:
                    hi = k.cmplt(j.id, self._ix(ext))
                    inside = hi if inside is None else k.and_(inside, hi)
                if inside is None:  # a pure crop: every index of the result exists in x
                    x_idx[axis] = j
                    v = self.value(n.src[0], x_idx)
                else:
                    pc_i = k.cast(inside, DType.I64)
                    x_idx[axis] = _V(k.mul(j.id, pc_i))
                    v = k.binary(self.value(n.src[0], x_idx), k.cast(inside, n.dtype), BOp.Mul)
        elif n.kind == "flip":
            x_idx = list(idx)
            for a in n.arg:
                i = idx[a]
                x_idx[a] = n.shape[a] - 1 - i if not isinstance(i, _V) else _V(k.sub(self._ix(n.shape[a] - 1), i.id))
            v = self.value(n.src[0], x_idx)
        else:
            raise ValueError(f"node kind {n.kind} cannot be computed inside an expression")
        self.memo[key] = v
        return v

    def operand(self, nid: int, idx: list, dtype: DType):
        n = self.g[nid]
        if n.dtype == dtype:
            return self.value(nid, idx if n.shape != () else [])
        if n.kind == "const":
            return self.k.const(n.arg, dtype)
        return self.k.cast(self.value(nid, idx if n.shape != () else []), dtype)

    def _inputs(self, nid: int, root: bool, seen: set, order: list):
        n = self.g[nid]
        if (n.kind == "leaf" or nid in self.stored) and not root:
            if nid not in seen:
                seen.add(nid)
                order.append(nid)
            return
        for i, s in enumerate(n.src):
            self._inputs(self.relu_mask.get(nid, s) if i == 0 else s, False, seen, order)

    def _reduce(self, n, idx):
        """Element `idx` of a Reduce as one serial loop with a register accumulator, where it is asked for. What the loop
        body defines stays inside the loop: the memo and the constant table are put back afterwards."""
        k = self.k
        x = n.src[0]
        xs = self.g[x].shape
        red = [xs[a] for a in n.arg]
        zero = self._ix(0)
        accu = k.storage(n.dtype, MemScope.Register, 1)
        k.store(accu, k.const(0 if n.op == BOp.Add else min_constant(n.dtype), n.dtype), zero)
        r = _V(k.loop(self._ix(_numel(red))))
        outer_consts, outer_memo = dict(self.consts), dict(self.memo)
        r_idx = self.unravel(r, red)
        kept = iter(idx if len(n.arg) < len(xs) else [])
        x_idx = [r_idx[n.arg.index(i)] if i in n.arg else next(kept) for i in range(len(xs))]
        v = self.value(x, x_idx)
        k.store(accu, k.binary(v, k.load(accu, zero), n.op), zero)  # x (op) acc, linearize.rs:943-946
        k.end_loop()
        self.consts, self.memo = outer_consts, outer_memo
        return k.load(accu, zero)

    def kernel(self, nid: int) -> LoweredKernel:
        n = self.g[nid]
        self.k = k = Kernel()
        self.consts, self.memo = {}, {}
        inputs: list = []
        self._inputs(nid, True, set(), inputs)
        self.params = {i: k.param(self.g[i].dtype, ParamKind.Global, max(_numel(self.g[i].shape), 1)) for i in inputs}
        total = max(_numel(n.shape), 1)
        out = k.param(n.dtype, ParamKind.GlobalMut, total)
        local = self.LOCAL if total >= self.LOCAL else 1
        groups = (total + local - 1) // local
        gid = _V(k.group_index(0, k.const_idx(groups)))
        lin = gid if local == 1 else self.add(self.mul(gid, local), _V(k.local_index(0, local)))
        guarded = groups * local != total
        if guarded:
            k.if_(k.cmplt(self._ix(lin), self._ix(total)))
            self.consts = {}  # constants created from here on live inside the If
        idx = self.unravel(lin, n.shape) if n.shape else []
        v = self._reduce(n, idx) if n.kind == "reduce" else self.value(nid, idx, root=True)
        k.store(out, v, self._ix(lin))
        if guarded:
            k.end_if()
        return LoweredKernel(k.to_bytes(), inputs, nid, total)


def lower(graph: Graph, outputs: Sequence[int], stored: Sequence[int] = (), match: bool = False) -> list:
    """Kernels that compute `outputs`, in execution order. Leaves and the nodes in `stored` already have buffers;
    every Reduce on the way and every output gets one (and is appended to the schedule once). With `match`, a Reduce
    that `match_contraction` recognises is scheduled as a `Contraction` (its operands get buffers first) with the
    generated kernel kept beside it as `.fallback`, so the caller can let the two compete on measured time the way
    kernel nodes compete in the reference's graph (zyx/src/backend/cblas.rs:227-236); a softmax over the last axis is
    scheduled as a `SoftmaxRows` (one fused pass in place of two reduces and a map: no competition needed)."""
    have = set(stored)
    emitter = _Emitter(graph, have)
    schedule: list = []
    users = consumers(graph, outputs, stored)
    losses = scan_cross_entropy(graph, [i for i in users if i >= 0] + list(outputs)) if match else {}

    def find(nid: int):
        return (losses.get(nid) or match_norm(graph, nid) or match_norm_bwd(graph, nid, users) or match_attention(graph, nid, users)
                or match_attention_bwd(graph, nid) or match_conv(graph, nid, users) or match_max_pool(graph, nid)
                or match_linear(graph, nid, users, emitter.relu_mask) or match_contraction(graph, nid)
                or match_softmax(graph, nid) or match_reduce_update(graph, nid, users) or match_reduce(graph, nid, have))

    def need(nid: int, root: bool, via: int | None = None):
        """via: the node that reads `nid` when every node between the kernel's root and `nid` keeps the element order
        (unary, cast, reshape, binary with an operand of its own shape), else None."""
        n = graph[nid]
        if n.kind == "leaf" or nid in have or nid in emitter.inline:
            return
        if match:
            # A convolution or a Linear read only by its relu is never stored: the relu's launch computes both, and the
            # relu's mask `v > 0`, which the reverse pass reads, is taken from the relu's result (`relu(v) > 0` is `v > 0`).
            for r in users.get(nid, ()):
                if r >= 0 and _is_relu_of(graph, r) == nid:
                    m = match_conv(graph, r, users) or match_linear(graph, r, users, emitter.relu_mask)
                    if m is not None and (getattr(m, "relu", False) or getattr(m, "mask_node", None) is not None):
                        need(r, True)
                        return
        c = find(nid) if match else None
        if c is None and match and root:
            base = _plain(graph, nid)
            if base is not None and base != nid and graph[base].kind != "const":
                need(base, True)
                schedule.append(Alias(nid, base))
                have.add(nid)
                return
        if c is not None:
            for attr in ("x", "w", "b", "dy", "add", "qkv", "bias", "residual", "target", "base"):
                v = getattr(c, attr, None)  # an operand that only re-views a tensor reads that tensor's buffer
                if isinstance(v, int) and not isinstance(c, (Conv2dMatch, MaxPoolMatch)):
                    shown = _plain(graph, v)
                    if shown is not None and graph[shown].kind != "const":
                        setattr(c, attr, shown)
            for s in match_operands(c):
                need(s, True)
            if isinstance(c, Contraction) and c.epilogue == "none" and c.residual is None:
                c.fallback = emitter.kernel(nid)
            if isinstance(c, Conv2dMatch) and c.relu:
                emitter.relu_mask[graph[nid].src[0]] = nid
            if isinstance(c, Contraction) and c.mask_node is not None:
                emitter.relu_mask[c.mask_node] = nid
            schedule.append(c)
            outs = (c.grad, c.mean) if isinstance(c, CrossEntropyMatch) else (c.dx, c.dw, c.db) if isinstance(c, NormBwdMatch) else (nid,)
            have.update(i for i in outs if i is not None)
            return
        if n.kind == "reduce" and not root and via is not None and users.get(nid, set()) == {via}:
            # read once, element for element, by an expression whose thread i wants exactly element i: the loop runs
            # inside that expression's kernel and the reduce gets no buffer and no launch of its own
            emitter.inline.add(nid)
            for s in n.src:
                need(s, False)
            return
        for s in n.src:
            keeps = (n.kind in ("unary", "cast", "reshape") or (n.kind == "binary" and graph[s].shape == n.shape)) and n.kind != "reduce"
            reader = nid if keeps and (root or via is not None) else None
            if reader is not None and graph[s].kind in ("reshape", "permute"):
                # a chain of views that shows a reduce element for element (transposes that cancel): same thing
                b = _plain(graph, s)
                if b is not None and b != s and graph[b].kind == "reduce" and b not in have and b not in emitter.inline:
                    chain, i = [], s
                    while i != b:
                        chain.append(i)
                        i = graph[i].src[0]
                    if all(users.get(c, set()) == {r} for c, r in zip(chain + [b], [nid] + chain)) and not (match and find(b) is not None):
                        emitter.inline.add(b)
                        for q in graph[b].src:
                            need(q, False)
                        continue
            need(s, False, reader)
        if root or n.kind == "reduce":
            schedule.append(emitter.kernel(nid))
            have.add(nid)

    import sys
    old = sys.getrecursionlimit()
    sys.setrecursionlimit(max(old, 10000 + 4 * len(graph.nodes)))
    try:
        for o in outputs:
            need(o, True)
    finally:
        sys.setrecursionlimit(old)
    return schedule


# ---- device -----------------------------------------------------------------------------------------------------------

class Tape:
    """Tensors of one graph on a HIP device: leaves are uploaded, `realize` lowers, compiles (once per distinct
    kernel) and launches, `numpy` downloads. The analogue of `Tape::new` / `gradient` / `realize`
    (zyx/tests/11_autograd.rs uses them throughout)."""

    def __init__(self, device, pool, match=False):
        """match: True -- products summed over shared axes run on the hand-written GEMM instead of a generated
        kernel; "time" -- both are timed once per distinct product (`zhip_time_kernel`, the clock the reference's
        autotuner uses, zyx/src/kernel/autotune.rs:775-798) and the faster one runs, as kernel nodes compete on
        `time` in the reference's graph."""
        self.dev, self.pool, self.graph, self.match = device, pool, Graph(), match
        self.matched = 0          # launches that went to a hand-written kernel
        self.timings: list = []   # (match, ns of the hand-written kernel, ns of the generated kernel)
        self._choice: dict = {}
        self._buf: dict[int, int] = {}
        self._ev: dict[int, object] = {}
        self._programs: dict[bytes, int] = {}
        self._keep: list = []
        self._last = None  # event of the most recent launch: launches form one chain
        self._plans: list = []
        self._spare: list = []  # second buffers of the input leaves of plans

    def tensor(self, array, dtype: DType) -> int:
        a = np.ascontiguousarray(array, storage_dtype(dtype))
        nid = self.graph.leaf(a.shape, dtype)
        self._alloc(nid)
        self._keep.append(a)  # the source of an upload stays valid until its event is synced
        self._ev[nid] = self.pool.host_to_pool(a, self._buf[nid], [self._ev.pop(nid)])
        return nid

    def _alloc(self, nid: int):
        n = self.graph[nid]
        buf, ev = self.pool.allocate(max(_numel(n.shape), 1) * np.dtype(storage_dtype(n.dtype)).itemsize)
        self._buf[nid], self._ev[nid] = buf, ev

    def gradient(self, target: int, sources: Sequence[int]) -> list:
        return self.graph.gradient(target, sources)

    def _aux(self, key, nbytes: int):
        """A buffer that belongs to a matched kernel and is no graph node (row log-sum-exps, an unwanted output)."""
        if key not in self._buf:
            buf, ev = self.pool.allocate(max(int(nbytes), 1))
            self._buf[key], self._ev[key] = buf, ev
        return key

    def realize(self, nodes: Sequence[int]):
        for kern in lower(self.graph, [n for n in nodes if n not in self._buf], stored=[n for n in self._buf if isinstance(n, int)], match=self.match):
            if isinstance(kern, Alias):
                self._buf[kern.out] = self._buf[kern.base]
                continue
            if isinstance(kern, MATCHED):
                kern = self._matched_or_generated(kern)
            prog = self._programs.get(kern.image)
            if prog is None:
                prog = self._programs[kern.image] = self.dev.compile(kern.image)
            for o in (kern.output,) + tuple(kern.more_outputs):
                if o not in self._buf:
                    self._alloc(o)
            # A launch consumes the events it waits for, and it waits for everything outstanding: the launch before it
            # and every upload, copy or allocation whose event nobody has consumed yet (after `write` / `assign` the
            # chain of launches continues in such an event, not in `_last`). The launches thus form one chain, and a
            # buffer whose event an earlier launch consumed is ready for all later ones too.
            waits = list(self._ev.values())
            self._ev.clear()
            if self._last is not None:
                waits.append(self._last)
            self._last = self.dev.launch(prog, self.pool, [self._buf[i] for i in kern.inputs + [kern.output] + list(kern.more_outputs)], waits)

    def plan(self, nodes: Sequence[int], updates: dict | None = None, inputs: Sequence[int] = ()) -> "TapePlan":
        """The schedule of `nodes` as one cached plan (a HIP graph): the analogue of the reference's plan cache
        (zyx/src/graph/plan.rs:58-237). Leaves may be rewritten with `write` between launches; every launch
        recomputes all the plan's nodes from the leaves' current contents.

        updates: {leaf: node} -- after every launch the leaf holds what the launch computed for the node
        (`Tensor::assign` of every updated parameter, as an optimizer step ends: zyx-optim/src/sgd.rs:45-84), without
        a copy: a kernel's outputs never alias its inputs, so the plan exists twice, over the two buffers of each pair
        in either role, and the pairs swap after each launch. Between launches the node's own value is the leaf's
        previous one.

        inputs: leaves the caller rewrites before every launch (the batch). Each gets a second buffer and the two
        copies of the plan read them alternately, so `write` fills the one the running launch does not read and the
        upload of the next batch overlaps the current step."""
        updates = dict(updates or {})
        for leaf in inputs:
            if self.graph[leaf].kind != "leaf" or leaf in updates:
                raise ValueError("inputs are leaves that no update writes")
        for leaf, node in updates.items():
            a, b = self.graph[leaf], self.graph[node]
            if a.kind != "leaf" or a.shape != b.shape or a.dtype != b.dtype or node not in nodes or self.graph[node].kind == "leaf":
                raise ValueError("updates map leaves to nodes of the plan with the leaf's shape and dtype")
        if self.match == "time":
            self.realize(nodes)  # settles which candidate each product runs on; the plan reuses the buffers
        self.sync()
        launches = []
        stored = [n for n in self._buf if isinstance(n, int) and self.graph[n].kind == "leaf"]  # everything else is computed by the plan
        for kern in lower(self.graph, list(nodes), stored=stored, match=bool(self.match)):
            if isinstance(kern, Alias):
                if kern.out in updates.values():
                    raise ValueError("an update has to be computed, not a view of another tensor")
                self._buf[kern.out] = self._buf[kern.base]
                continue
            if isinstance(kern, MATCHED):
                kern = self._matched_or_generated(kern)
            prog = self._programs.get(kern.image)
            if prog is None:
                prog = self._programs[kern.image] = self.dev.compile(kern.image)
            outs = [kern.output] + list(kern.more_outputs)
            for o in outs:
                if o not in self._buf:
                    self._alloc(o)
            launches.append((prog, [self._buf[i] for i in kern.inputs + outs]))
        self.sync()
        ids = [self.dev.create_plan(launches)]
        pairs = dict(updates)
        for leaf in inputs:  # the alternate of an input leaf is a buffer of its own, filled by the next `write`
            n = self.graph[leaf]
            buf, ev = self.pool.allocate(max(_numel(n.shape), 1) * np.dtype(storage_dtype(n.dtype)).itemsize)
            self.pool.sync_events([ev])
            pairs[leaf] = ("alt", buf)
            self._spare.append(buf)
        if pairs:
            swap = {}
            for leaf, other in pairs.items():
                ob = other[1] if isinstance(other, tuple) else self._buf[other]
                swap[self._buf[leaf]], swap[ob] = ob, self._buf[leaf]
            ids.append(self.dev.create_plan([(prog, [swap.get(b, b) for b in bufs]) for prog, bufs in launches]))
        return TapePlan(self, ids, len(launches), pairs)

    def write(self, leaf: int, array):
        """New contents for a leaf (same shape and dtype); later launches read them."""
        n = self.graph[leaf]
        a = np.ascontiguousarray(array, storage_dtype(n.dtype))
        if n.kind != "leaf" or a.shape != n.shape:
            raise ValueError("write takes a leaf and an array of its shape")
        self._keep.append(a)
        if len(self._keep) > 1024:  # bound the host arrays kept alive: after a sync none is still being read
            self.sync()
            self._keep.append(a)
        # No wait for the launch in flight: the runtime orders a copy after every earlier access of its destination by
        # itself, and a launch that does not touch this buffer has no reason to hold the upload back.
        waits = [self._ev.pop(leaf)] if leaf in self._ev else []
        self._ev[leaf] = self.pool.host_to_pool(a, self._buf[leaf], waits)

    def assign(self, leaf: int, node: int):
        """leaf <- node, device to device (`Tensor::assign` of an updated parameter): later launches read the new
        contents."""
        a, b = self.graph[leaf], self.graph[node]
        if a.kind != "leaf" or a.shape != b.shape or a.dtype != b.dtype or node not in self._buf:
            raise ValueError("assign takes a leaf and a realised node of the same shape and dtype")
        waits = [self._ev.pop(i) for i in (leaf, node) if i in self._ev]
        if self._last is not None:
            waits.append(self._last)
            self._last = None
        nbytes = max(_numel(a.shape), 1) * np.dtype(storage_dtype(a.dtype)).itemsize
        self._ev[leaf] = self.pool.copy_range(self._buf[node], 0, self._buf[leaf], 0, nbytes, waits)

    def _matched_or_generated(self, c) -> LoweredKernel:
        from .kernels import (attention_bwd_desc, attention_desc, conv2d_desc, cross_entropy_desc, gemm_desc, max_pool2d_desc,
                              norm_rows_bwd_desc, norm_rows_desc, reduce_desc, softmax_rows_desc)
        more = ()
        isz = np.dtype(storage_dtype(c.dtype)).itemsize if hasattr(c, "dtype") else 4
        if isinstance(c, NormRowsMatch):
            desc = norm_rows_desc(c.rows, c.cols, c.rms, c.w is not None, c.b is not None, c.eps, c.dtype)
            inputs, elements = list(match_operands(c)), c.rows * c.cols
        elif isinstance(c, NormBwdMatch):
            want_db = c.db is not None and not c.rms
            desc = norm_rows_bwd_desc(c.rows, c.cols, c.rms, c.w is not None, want_db, c.add is not None, c.eps, c.dtype)
            inputs, elements = list(match_operands(c)), c.rows * c.cols
            if c.w is not None:  # the kernel writes dw whenever there is a weight
                more += (c.dw if c.dw is not None else self._aux(("dw", c.dx), c.cols * isz),)
            if want_db:
                more += (c.db,)
        elif isinstance(c, AttentionMatch):
            b_, t_, h_, dh_ = c.dims
            desc = attention_desc(b_, t_, h_, dh_, c.dtype, c.scale, 0.0, c.lse, False)
            inputs, elements = [c.qkv], b_ * t_ * h_ * dh_
            if c.lse:
                more = (self._aux(("lse", c.out), b_ * h_ * t_ * 4),)
        elif isinstance(c, AttentionBwdMatch):
            b_, t_, h_, dh_ = c.dims
            desc = attention_bwd_desc(b_, t_, h_, dh_, c.dtype, c.scale, 0.0, False)
            inputs, elements = [c.qkv, c.y, c.dy, ("lse", c.y)], 3 * b_ * t_ * h_ * dh_
            if ("lse", c.y) not in self._buf:
                raise RuntimeError("the attention forward of this backward was realised without its row log-sum-exps")
        elif isinstance(c, Conv2dMatch):
            n_, c_, h, w, co, kh, kw = c.dims
            desc = conv2d_desc(n_, c_, h, w, co, kh, kw, c.stride, c.padding, c.dilation, c.bias is not None, c.relu, c.dtype)
            inputs, elements = list(match_operands(c)), _numel(self.graph[c.out].shape)
        elif isinstance(c, MaxPoolMatch):
            desc = max_pool2d_desc(c.planes, c.hw[0], c.hw[1], c.kernel, c.stride, c.padding, c.dilation, c.dtype)
            inputs, elements = [c.x], _numel(self.graph[c.out].shape)
        elif isinstance(c, Contraction):
            bias_dtype = self.graph[c.bias].dtype if c.bias is not None else DType.F32
            desc = gemm_desc(c.m, c.n, c.k, c.dtype, c.dtype, c.trans_a, c.trans_b, c.epilogue, bias_dtype, c.batch, c.alpha,
                             "relu_mask" if c.relu_mask else c.residual is not None)
            inputs, elements = list(match_operands(c)), c.batch * c.m * c.n
        elif isinstance(c, RowColReduce):
            desc = reduce_desc(c.rows, c.cols, c.op, c.axis0, c.dtype, mul=c.mul, base=c.base is not None)
            inputs, elements = list(match_operands(c)), c.cols if c.axis0 else c.rows
        elif isinstance(c, CrossEntropyMatch):
            desc = cross_entropy_desc(c.rows, c.cols, False, c.grad is not None, c.gscale, c.mean is not None, dense=True)
            inputs, elements = [c.x, c.target], c.rows * c.cols if c.grad is not None else 1
            more = (c.mean,) if c.grad is not None and c.mean is not None else ()
        else:
            desc = softmax_rows_desc(c.rows, c.cols, y=True, rowsum=False, argmax=False)
            inputs, elements = [c.x], c.rows * c.cols
        key = bytes(desc)
        if key not in self._programs:
            self._programs[key] = self.dev.register_kernel(desc)
        gemm = LoweredKernel(key, inputs, c.out, elements, more)
        if self.match == "time" and isinstance(c, Contraction) and c.fallback is not None:
            pair = (key, c.fallback.image)
            if pair not in self._choice:
                if c.fallback.image not in self._programs:
                    self._programs[c.fallback.image] = self.dev.compile(c.fallback.image)
                self._alloc(c.out)
                self.sync()  # the operands are complete and the new buffer exists
                ns = []
                for k in (gemm, c.fallback):
                    args = [self._buf[i] for i in k.inputs] + [self._buf[c.out]]
                    ns.append(min(self.dev.time_kernel(self._programs[k.image], args) for _ in range(3)))
                self.timings.append((c, ns[0], ns[1]))
                self._choice[pair] = ns[0] <= ns[1]
            if not self._choice[pair]:
                return c.fallback
        self.matched += 1
        return gemm

    def numpy(self, nid: int) -> np.ndarray:
        if nid not in self._buf:
            self.realize([nid])
        n = self.graph[nid]
        out = np.empty(n.shape if n.shape else (1,), storage_dtype(n.dtype))
        self.sync()
        self.pool.pool_to_host(self._buf[nid], out, [])
        return out.reshape(n.shape)

    def sync(self):
        evs = list(self._ev.values()) + ([self._last] if self._last is not None else [])
        self._ev.clear()
        self._last = None
        if evs:
            self.pool.sync_events(evs)
        self._keep.clear()

    def close(self):
        self.sync()
        for pl in self._plans:
            self.dev.destroy_plan(pl)
        self._plans.clear()
        for prog in self._programs.values():
            self.dev.release(prog)
        for buf in sorted(set(self._buf.values()) | set(self._spare)):  # aliases share a buffer
            self.pool.deallocate(buf, [])
        self._spare.clear()
        self._programs.clear()
        self._buf.clear()


class TapePlan:
    """A realised schedule kept as one replayable unit; `launch` runs it after everything the tape has outstanding."""

    def __init__(self, tape: Tape, plan_ids: list, launches: int, updates: dict | None = None):
        self.tape, self.ids, self.launches, self.updates = tape, plan_ids, launches, dict(updates or {})
        self._parity = 0
        tape._plans.extend(plan_ids)

    def launch(self):
        t = self.tape
        waits = list(t._ev.values()) + ([t._last] if t._last is not None else [])
        t._ev.clear()
        t._last = t.dev.launch_plan(self.ids[self._parity], waits)
        if self.updates:
            for leaf, other in self.updates.items():
                if isinstance(other, tuple):  # an input leaf: the next `write` goes to the buffer this launch does not read
                    spare = other[1]
                    self.updates[leaf] = ("alt", t._buf[leaf])
                    t._spare[t._spare.index(spare)] = t._buf[leaf]
                    t._buf[leaf] = spare
                else:
                    t._buf[leaf], t._buf[other] = t._buf[other], t._buf[leaf]
            self._parity ^= 1
