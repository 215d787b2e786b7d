"""Linearized kernels in the shape zyx's own passes leave them, built by hand with zyx_amd.ir for the tests of the
generic-kernel path (the reference's lowering itself is Rust and cannot run here). Patterns follow:
reduce accumulators zyx/src/kernel/linearize.rs:920-952, masked (padded) loads linearize.rs:349-382, group / local
index split and local-memory tree reduction zyx/src/kernel/local_reduce.rs, vector loads zyx/src/kernel/vectorize.rs,
dynamic group counts zyx/src/backend/mod.rs:60-98."""
from __future__ import annotations

import numpy as np

from zyx_amd import DType
from zyx_amd.ir import BOp, Kernel, MemScope, ParamKind, UOp


def _acc(k: Kernel, dtype: DType, init):
    """Register accumulator: Storage[1], store of the neutral element (linearize.rs:930-940)."""
    zero = k.const_idx(0)
    init = k.const(init, dtype)
    acc = k.storage(dtype, MemScope.Register, 1)
    k.store(acc, init, zero)
    return acc, zero


def _accumulate(k: Kernel, acc, zero, x, bop: BOp):
    """acc = x (op) acc, in that operand order (linearize.rs:943-946)."""
    cur = k.load(acc, zero)
    k.store(acc, k.binary(x, cur, bop), zero)


def elementwise(n_groups: int, local: int, uops=(), in_dtype=DType.F32, out_dtype=DType.F32, **kw) -> Kernel:
    """y[i] = uops(...(x[i])) for i = group * local + lane; loads widen, the store truncates (16-bit floats)."""
    k = Kernel(**kw)
    x = k.param(in_dtype, ParamKind.Global, n_groups * local)
    y = k.param(out_dtype, ParamKind.GlobalMut, n_groups * local)
    g = k.group_index(0, k.const_idx(n_groups))
    l = k.local_index(0, local)
    i = k.add(k.mul(g, k.const_idx(local)), l)
    v = k.load(x, i)
    for u in uops:
        v = k.unary(v, u)
    if in_dtype != out_dtype:
        v = k.cast(v, out_dtype)
    k.store(y, v, i)
    return k


def binary_table(n: int, dtype: DType, bop: BOp) -> Kernel:
    """z[i] = x[i] (op) y[i]; comparisons store their Bool as one byte."""
    k = Kernel()
    x = k.param(dtype, ParamKind.Global, n)
    y = k.param(dtype, ParamKind.Global, n)
    out_dt = DType.Bool if bop in (BOp.Cmplt, BOp.Cmpgt, BOp.Cmpge, BOp.NotEq, BOp.Eq, BOp.Or, BOp.And) else dtype
    z = k.param(out_dt, ParamKind.GlobalMut, n)
    i = k.group_index(0, k.const_idx(n))
    k.store(z, k.binary(k.load(x, i), k.load(y, i), bop), i)
    return k


def unary_table(n: int, dtype: DType, uop: UOp) -> Kernel:
    k = Kernel()
    x = k.param(dtype, ParamKind.Global, n)
    z = k.param(dtype, ParamKind.GlobalMut, n)
    i = k.group_index(0, k.const_idx(n))
    k.store(z, k.unary(k.load(x, i), uop), i)
    return k


def cast_table(n: int, src: DType, dst: DType) -> Kernel:
    k = Kernel()
    x = k.param(src, ParamKind.Global, n)
    z = k.param(dst, ParamKind.GlobalMut, n)
    i = k.group_index(0, k.const_idx(n))
    k.store(z, k.cast(k.load(x, i), dst), i)
    return k


def matmul(m: int, n: int, kk: int, dtype=DType.F32, out_dtype=DType.F32, use_mad=False, local=(1, 1), **kw) -> Kernel:
    """C[i, j] = sum_k A[i, k] * B[k, j], one thread per element, serial k (what `x.dot(y)` lowers to before any
    optimisation pass): groups (m / lx, n / ly), locals (lx, ly)."""
    lx, ly = local
    assert m % lx == 0 and n % ly == 0
    k = Kernel(**kw)
    a = k.param(dtype, ParamKind.Global, m * kk)
    b = k.param(dtype, ParamKind.Global, kk * n)
    c = k.param(out_dtype, ParamKind.GlobalMut, m * n)
    gi = k.group_index(0, k.const_idx(m // lx))
    gj = k.group_index(1, k.const_idx(n // ly))
    i, j = gi, gj
    if lx > 1:
        i = k.add(k.mul(gi, k.const_idx(lx)), k.local_index(0, lx))
    if ly > 1:
        j = k.add(k.mul(gj, k.const_idx(ly)), k.local_index(1, ly))
    acc, zero = _acc(k, dtype, 0)
    ck, cn = k.const_idx(kk), k.const_idx(n)
    r = k.loop(ck)
    av = k.load(a, k.add(k.mul(i, ck), r))
    bv = k.load(b, k.add(k.mul(r, cn), j))
    if use_mad:
        cur = k.load(acc, zero)
        k.store(acc, k.mad(av, bv, cur), zero)
    else:
        _accumulate(k, acc, zero, k.mul(av, bv), BOp.Add)
    k.end_loop()
    out = k.load(acc, zero)
    if out_dtype != dtype:
        out = k.cast(out, out_dtype)
    k.store(c, out, k.add(k.mul(i, cn), j))
    return k


def softmax_rows(rows: int, cols: int, **kw) -> Kernel:
    """softmax over the last axis as three serial reduce / map loops per row (x.softmax([-1]) unfused:
    m = max(x); e = exp(x - m); s = sum(e); y = e / s), one group per row, max accumulator starting at f32::MIN."""
    k = Kernel(**kw)
    x = k.param(DType.F32, ParamKind.Global, rows * cols)
    y = k.param(DType.F32, ParamKind.GlobalMut, rows * cols)
    g = k.group_index(0, k.const_idx(rows))
    cc = k.const_idx(cols)
    base = k.mul(g, cc)
    mx, zero = _acc(k, DType.F32, -3.4028234663852886e38)
    r = k.loop(cc)
    _accumulate(k, mx, zero, k.load(x, k.add(base, r)), BOp.Max)
    k.end_loop()
    m = k.load(mx, zero)
    sm, zero2 = _acc(k, DType.F32, 0.0)
    r = k.loop(cc)
    e = k.unary(k.sub(k.load(x, k.add(base, r)), m), UOp.Exp)
    _accumulate(k, sm, zero2, e, BOp.Add)
    k.end_loop()
    s = k.load(sm, zero2)
    r = k.loop(cc)
    idx = k.add(base, r)
    e = k.unary(k.sub(k.load(x, idx), m), UOp.Exp)
    k.store(y, k.div(e, s), idx)
    k.end_loop()
    return k


def row_sum_local(rows: int, cols: int, local: int = 256, dtype=DType.F32) -> Kernel:
    """s[row] = sum of the row: each of `local` threads sums a strided slice serially, then a tree reduction through
    local memory with a barrier per level and `If lane < stride` (kernel/local_reduce.rs)."""
    assert cols % local == 0 and local & (local - 1) == 0
    k = Kernel()
    x = k.param(dtype, ParamKind.Global, rows * cols)
    s = k.param(dtype, ParamKind.GlobalMut, rows)
    g = k.group_index(0, k.const_idx(rows))
    l = k.local_index(0, local)
    tile = k.storage(dtype, MemScope.Local, local)
    acc, zero = _acc(k, dtype, 0)
    cl = k.const_idx(local)
    base = k.mul(g, k.const_idx(cols))
    r = k.loop(k.const_idx(cols // local))
    _accumulate(k, acc, zero, k.load(x, k.add(base, k.add(k.mul(r, cl), l))), BOp.Add)
    k.end_loop()
    k.store(tile, k.load(acc, zero), l)
    stride = local // 2
    while stride >= 1:
        k.barrier()
        cs = k.const_idx(stride)
        k.if_(k.cmplt(l, cs))
        k.store(tile, k.add(k.load(tile, l), k.load(tile, k.add(l, cs))), l)
        k.end_if()
        stride //= 2
    k.barrier()
    k.if_(k.binary(l, k.const_idx(0), BOp.Eq))
    k.store(s, k.load(tile, zero), g)
    k.end_if()
    return k


def padded_copy(n: int, pad_left: int, pad_right: int) -> Kernel:
    """y = x.pad(pad_left, pad_right) on one axis: the load index is shifted, bounds give a Bool that zeroes both
    the offset and the value (linearize.rs:349-382, after the scalar autocast of the mask)."""
    total = n + pad_left + pad_right
    k = Kernel()
    x = k.param(DType.F32, ParamKind.Global, n)
    y = k.param(DType.F32, ParamKind.GlobalMut, total)
    i = k.group_index(0, k.const_idx(total))
    idx = k.sub(i, k.const_idx(pad_left))
    pc = k.and_(k.cmplt(idx, k.const_idx(n)), k.and_(k.cmpge(idx, k.const_idx(0)), k.const(1, DType.Bool)))
    off = k.mul(k.cast(pc, DType.I64), idx)
    v = k.load(x, off)
    k.store(y, k.mul(k.cast(pc, DType.F32), v), i)
    return k


def vector_axpy(n_groups: int, local: int, vlen: int, dtype=DType.F32) -> Kernel:
    """z = a * x + y with Vector(vlen) loads and stores, one lane pulled out and put back through
    Devectorize / Stack (kernel/vectorize.rs); a is a Variable parameter."""
    k = Kernel()
    a = k.param(DType.F32, ParamKind.Variable)
    x = k.param(dtype, ParamKind.Global, n_groups * local * vlen)
    y = k.param(dtype, ParamKind.Global, n_groups * local * vlen)
    z = k.param(dtype, ParamKind.GlobalMut, n_groups * local * vlen)
    g = k.group_index(0, k.const_idx(n_groups))
    l = k.local_index(0, local)
    i = k.mul(k.add(k.mul(g, k.const_idx(local)), l), k.const_idx(vlen))
    av = k.load(a, k.const_idx(0))
    xv, yv = k.load(x, i, vlen), k.load(y, i, vlen)
    lanes = [k.add(k.mul(av, k.devectorize(xv, j)), k.devectorize(yv, j)) for j in range(vlen)]
    k.store(z, k.stack(lanes), i, vlen)
    return k


def vector_scale(n_groups: int, local: int, vlen: int, dtype=DType.F32) -> Kernel:
    """y = 2 * x + 1 on whole vectors: vector (op) scalar constant broadcasts the constant."""
    k = Kernel()
    x = k.param(dtype, ParamKind.Global, n_groups * local * vlen)
    y = k.param(dtype, ParamKind.GlobalMut, n_groups * local * vlen)
    g = k.group_index(0, k.const_idx(n_groups))
    l = k.local_index(0, local)
    i = k.mul(k.add(k.mul(g, k.const_idx(local)), l), k.const_idx(vlen))
    v = k.load(x, i, vlen)
    v = k.add(k.mul(v, k.const(2.0, dtype)), k.const(1.0, dtype))
    k.store(y, v, i, vlen)
    return k


def dynamic_rows(cols: int) -> Kernel:
    """y[r, :] = x[r, :] + r with the row count a Variable parameter that is also the group count (GwsDim::Param)."""
    k = Kernel()
    rows = k.param(DType.I64, ParamKind.Variable)
    x = k.param(DType.F32, ParamKind.Global)
    y = k.param(DType.F32, ParamKind.GlobalMut)
    g = k.group_index(0, rows)
    l = k.local_index(0, cols)
    i = k.add(k.mul(g, k.const_idx(cols)), l)
    k.store(y, k.add(k.load(x, i), k.cast(g, DType.F32)), i)
    return k


def ragged_loop(rows: int) -> Kernel:
    """s[r] = sum_{j < len[r]} x[r * 64 + j]: a loop whose length is loaded per thread, so neighbouring threads run
    different trip counts."""
    k = Kernel()
    ln = k.param(DType.I32, ParamKind.Global, rows)
    x = k.param(DType.F32, ParamKind.Global, rows * 64)
    s = k.param(DType.F32, ParamKind.GlobalMut, rows)
    g = k.group_index(0, k.const_idx(rows // 32))
    l = k.local_index(0, 32)
    r = k.add(k.mul(g, k.const_idx(32)), l)
    acc, zero = _acc(k, DType.F32, 0.0)
    j = k.loop(k.cast(k.load(ln, r), DType.I64))
    _accumulate(k, acc, zero, k.load(x, k.add(k.mul(r, k.const_idx(64)), j)), BOp.Add)
    k.end_loop()
    k.store(s, k.load(acc, zero), r)
    return k
