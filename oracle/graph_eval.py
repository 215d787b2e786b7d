"""TEST INFRASTRUCTURE, not product code: evaluates a graph of zyx node kinds (Leaf, Const, Unary, Binary, Cast,
Reshape, Expand, Permute, Flip, Pad, Narrow, Reduce -- zyx/src/graph/mod.rs `Node`) with numpy, node by node, as the checker for
the kernels the HIP backend generates from such a graph.

Element arithmetic is the C backend's (oracle/ir_interp.py `unary` / `binary` / `_c_cast`, which restate
zyx/src/codegen/c.rs:290-304, 583-612); movement ops are numpy's reshape / broadcast_to / transpose / flip; a reduce
accumulates serially, `acc = x (op) acc`, over the reduced dims in row-major order starting from 0 or the lowest
finite value (zyx/src/kernel/linearize.rs:920-952). Operands of a Binary that differ in dtype: a Bool operand is
converted to the other's dtype, else a Const to the other's, else y to x's. Values of the 16-bit float dtypes are
held as f32, as in registers.

Pinned in tests/test_graph_oracle.py by the golden gradients of zyx/tests/11_autograd.rs (evaluated through this
file), numpy closed forms and finite differences.
"""
from __future__ import annotations

import numpy as np

from . import ir_interp as I

_BOOL_OPS = (6, 7, 8, 10, 11, 17, 18)


def _reg(dt):
    return I._REG[int(dt)]


def _convert(v, src, dst):
    src, dst = int(src), int(dst)
    if src == dst:
        return v
    if dst in (I.BF16, I.F16):
        return v.astype(np.float32)
    return I._c_cast(v, dst)


def _lowest(dt):
    dt = int(dt)
    if dt == I.F32: return np.float32(-3.4028234663852886e38)
    if dt == I.BF16: return np.float32(-3.3895313892515355e38)
    if dt == I.F16: return np.float32(-65504.0)
    if dt == I.F64: return np.float64(-1.7976931348623157e308)
    if dt == I.BOOL: return np.uint8(0)
    return np.iinfo(_reg(dt)).min


def evaluate(nodes, leaves: dict, wanted) -> dict:
    """`nodes`: sequence of objects with kind / dtype / shape / src / op / arg; `leaves`: node id -> numpy array in
    register format (f32 for bf16 / f16 leaves). Returns node id -> array for every id in `wanted`."""
    done: dict[int, np.ndarray] = {}

    def softness(n):
        return 2 if int(n.dtype) == I.BOOL else (1 if n.kind == "const" else 0)

    def ev(i: int) -> np.ndarray:
        stack = [i]
        while stack:
            j = stack[-1]
            if j in done:
                stack.pop()
                continue
            n = nodes[j]
            missing = [s for s in n.src if s not in done]
            if missing:
                stack.extend(missing)
                continue
            stack.pop()
            done[j] = one(j, n)
        return done[i]

    def one(j, n):
        dt = int(n.dtype)
        if n.kind == "leaf":
            return np.asarray(leaves[j]).astype(_reg(dt)).reshape(n.shape)
        if n.kind == "const":
            if dt in (I.BF16,):
                return I.bf16_bits_to_f32(I.f32_to_bf16_bits(np.array(n.arg, np.float32)))
            return np.array(n.arg).astype(_reg(dt)) if dt not in (I.F16,) else np.array(n.arg, np.float16).astype(np.float32)
        x = done[n.src[0]]
        xn = nodes[n.src[0]]
        if n.kind == "unary":
            return I.unary(int(n.op), x, int(xn.dtype)).reshape(n.shape)
        if n.kind == "binary":
            yn, y = nodes[n.src[1]], done[n.src[1]]
            common = int(yn.dtype) if softness(yn) < softness(xn) else int(xn.dtype)
            xv = const_in(xn, common) if xn.kind == "const" else _convert(x, xn.dtype, common)
            yv = const_in(yn, common) if yn.kind == "const" else _convert(y, yn.dtype, common)
            xv, yv = np.broadcast_arrays(xv, yv)
            return I.binary(int(n.op), xv, yv, common).reshape(n.shape)
        if n.kind == "cast":
            return _convert(x, xn.dtype, dt)
        if n.kind == "reshape":
            return x.reshape(n.shape)
        if n.kind == "expand":
            return np.broadcast_to(x, n.shape)
        if n.kind == "permute":
            return np.transpose(x, n.arg)
        if n.kind == "flip":
            return np.flip(x, n.arg)
        if n.kind == "narrow":  # Node::Narrow: elements start .. start + len of one axis
            axis, start = n.arg
            return x[(slice(None),) * axis + (slice(start, start + n.shape[axis]),)]
        if n.kind == "pad":  # Node::Pad: element i of the axis is x[i - lp] where that exists, else 0
            axis, lp = n.arg
            out = np.zeros(n.shape, x.dtype)
            lo, hi = max(0, lp), min(n.shape[axis], lp + x.shape[axis])  # positions of the result that come from x
            pre = (slice(None),) * axis
            out[pre + (slice(lo, hi),)] = x[pre + (slice(lo - lp, hi - lp),)]
            return out
        if n.kind == "reduce":
            axes = tuple(n.arg)
            keep = [a for a in range(x.ndim) if a not in axes]
            moved = np.transpose(x, keep + list(axes)).reshape(int(np.prod([x.shape[a] for a in keep], dtype=np.int64)), -1)
            acc = np.full(moved.shape[0], 0 if int(n.op) == 0 else _lowest(dt), _reg(dt))
            for r in range(moved.shape[1]):
                acc = I.binary(int(n.op), np.ascontiguousarray(moved[:, r]), acc, dt)
            return acc.reshape(n.shape)
        raise ValueError(n.kind)

    def const_in(n, dt):
        """A constant takes the other operand's dtype directly (no intermediate rounding in its own)."""
        if dt == I.BF16:
            return I.bf16_bits_to_f32(I.f32_to_bf16_bits(np.array(n.arg, np.float32)))
        if dt == I.F16:
            return np.array(n.arg, np.float16).astype(np.float32)
        return np.array(n.arg).astype(_reg(dt))

    return {w: np.ascontiguousarray(ev(w)) for w in wanted}
