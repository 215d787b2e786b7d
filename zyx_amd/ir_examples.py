"""Linearized kernels in the optimised shape zyx's passes aim for (local reduce zyx/src/kernel/local_reduce.rs,
vector loads zyx/src/kernel/vectorize.rs, register blocking zyx/src/kernel/coarsen.rs), written with zyx_amd.ir:
the benchmarks time them to show what the generic-kernel path reaches on memory-bound work."""
from __future__ import annotations

from .backend import DType
from .ir import BOp, Kernel, MemScope, ParamKind, UOp

LOG2_E = 1.4426950408889634


def _tree(k: Kernel, tile, lane, local: int, bop: BOp):
    """Tree reduction of tile[0..local) into tile[0], a barrier per level."""
    stride = local // 2
    while stride >= 1:
        k.barrier()
        cs = k.const_idx(stride)
        k.if_(k.cmplt(lane, cs))
        k.store(tile, k.binary(k.load(tile, lane), k.load(tile, k.add(lane, cs)), bop), lane)
        k.end_if()
        stride //= 2
    k.barrier()


def softmax_rows_local(rows: int, cols: int, local: int = 256, vlen: int = 4) -> Kernel:
    """y = softmax(x) over the last axis, f32: one group per row, the row held in registers (cols / local values per
    thread, loaded as vectors), maximum and sum reduced through local memory. exp(v - m) is exp2((v - m) * log2 e),
    the rewrite zyx applies when the device reports a native exp2 (kernel/autotune.rs:578-584)."""
    per = cols // (local * vlen)
    assert per * local * vlen == cols and local & (local - 1) == 0
    k = Kernel()
    x = k.param(DType.F32, ParamKind.Global, rows * cols)
    y = k.param(DType.F32, ParamKind.GlobalMut, rows * cols)
    g = k.group_index(0, k.const_idx(rows))
    lane = k.local_index(0, local)
    tile = k.storage(DType.F32, MemScope.Local, local)
    regs = k.storage(DType.F32, MemScope.Register, per * vlen)
    zero, cper, cv = k.const_idx(0), k.const_idx(per), k.const_idx(vlen)
    base = k.mul(g, k.const_idx(cols))
    step = k.const_idx(local * vlen)
    lane_off = k.mul(lane, cv)

    acc = k.storage(DType.F32, MemScope.Register, 1)
    k.store(acc, k.const(-3.4028234663852886e38, DType.F32), zero)
    r = k.loop(cper)
    v = k.load(x, k.add(base, k.add(k.mul(r, step), lane_off)), vlen)
    k.store(regs, v, k.mul(r, cv), vlen)
    for j in range(vlen):
        k.store(acc, k.max(k.devectorize(v, j), k.load(acc, zero)), zero)
    k.end_loop()
    k.store(tile, k.load(acc, zero), lane)
    _tree(k, tile, lane, local, BOp.Max)
    m = k.load(tile, zero)
    k.barrier()

    k.store(acc, k.const(0.0, DType.F32), zero)
    log2e = k.const(LOG2_E, DType.F32)
    r = k.loop(cper)
    v = k.load(regs, k.mul(r, cv), vlen)
    e = k.unary(k.mul(k.sub(v, m), log2e), UOp.Exp2)
    k.store(regs, e, k.mul(r, cv), vlen)
    for j in range(vlen):
        k.store(acc, k.add(k.devectorize(e, j), k.load(acc, zero)), zero)
    k.end_loop()
    k.store(tile, k.load(acc, zero), lane)
    _tree(k, tile, lane, local, BOp.Add)
    inv = k.unary(k.load(tile, zero), UOp.Reciprocal)

    r = k.loop(cper)
    v = k.load(regs, k.mul(r, cv), vlen)
    k.store(y, k.mul(v, inv), k.add(base, k.add(k.mul(r, step), lane_off)), vlen)
    k.end_loop()
    return k


def scaled_exp2(n: int, dtype: DType = DType.F32, local: int = 256, vlen: int = 4, per: int = 4) -> Kernel:
    """y = exp2(x) * 2 + 1 elementwise, `per` vectors of `vlen` elements per thread."""
    chunk = local * vlen * per
    assert n % chunk == 0
    k = Kernel()
    x = k.param(dtype, ParamKind.Global, n)
    y = k.param(dtype, ParamKind.GlobalMut, n)
    g = k.group_index(0, k.const_idx(n // chunk))
    lane = k.local_index(0, local)
    base = k.add(k.mul(g, k.const_idx(chunk)), k.mul(lane, k.const_idx(vlen)))
    r = k.loop(k.const_idx(per))
    i = k.add(base, k.mul(r, k.const_idx(local * vlen)))
    v = k.unary(k.load(x, i, vlen), UOp.Exp2)
    k.store(y, k.add(k.mul(v, k.const(2.0, dtype)), k.const(1.0, dtype)), i, vlen)
    k.end_loop()
    return k
