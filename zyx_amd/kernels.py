"""Descriptors of the hand-written kernels (`zhip_kernel_kind` in include/zyx_hip.h) and
thin helpers that replay the reference's realize sequence for one AOT kernel:
allocate stores (+1 trash element), args = loads then stores, launch, keep the event
(zyx/src/runtime.rs:2262-2300, zyx/src/graph/plan.rs:311-327)."""
from __future__ import annotations

import numpy as np

from .backend import DType, Event, HIPDevice, HIPMemoryPool, KernelDesc

K_SOFTMAX_ROWS = 1
SOFTMAX_Y, SOFTMAX_ROWSUM, SOFTMAX_ARGMAX = 1, 2, 4


def softmax_rows_desc(rows: int, cols: int, y=True, rowsum=True, argmax=True) -> KernelDesc:
    d = KernelDesc()
    d.kind, d.dtype, d.out_dtype = K_SOFTMAX_ROWS, DType.F32, DType.F32
    d.flags = (SOFTMAX_Y if y else 0) | (SOFTMAX_ROWSUM if rowsum else 0) | (SOFTMAX_ARGMAX if argmax else 0)
    d.dims[0], d.dims[1] = rows, cols
    return d


def to_device(pool: HIPMemoryPool, array: np.ndarray):
    """`Runtime::new_tensor`-style upload: allocate bytes + one trash element, async copy.
    Returns (buffer id, event); `array` must outlive the event."""
    array = np.ascontiguousarray(array)
    buf, ev = pool.allocate(array.nbytes + array.itemsize)
    ev2 = pool.host_to_pool(array, buf, [ev])
    return buf, ev2


def to_host(pool: HIPMemoryPool, buf: int, shape, dtype, events=()) -> np.ndarray:
    out = np.empty(shape, dtype)
    pool.pool_to_host(buf, out, list(events))
    return out


def alloc_like(pool: HIPMemoryPool, n_elems: int, itemsize: int):
    return pool.allocate((n_elems + 1) * itemsize)


def softmax_rows(dev: HIPDevice, pool: HIPMemoryPool, x: np.ndarray, y=True, rowsum=True, argmax=True):
    """Upload x, run the fused kernel, read back (y, rowsum, argmax); entries not asked for are None."""
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = x.shape
    prog = dev.register_kernel(softmax_rows_desc(rows, cols, y, rowsum, argmax))
    xb, ev = to_device(pool, x)
    waits, outs = [ev], []
    for want, n, isz in ((y, rows * cols, 4), (rowsum, rows, 4), (argmax, rows, 4)):
        if want:
            b, e = alloc_like(pool, n, isz)
            outs.append(b)
            waits.append(e)
    done = dev.launch(prog, pool, [xb] + outs, waits)
    res, it = [], iter(outs)
    first = True
    for want, shape, dt in ((y, (rows, cols), np.float32), (rowsum, (rows,), np.float32), (argmax, (rows,), np.int32)):
        if not want:
            res.append(None)
            continue
        res.append(to_host(pool, next(it), shape, dt, [done] if first else []))
        first = False
    for b in [xb] + outs:
        pool.deallocate(b, [])
    dev.release(prog)
    return tuple(res)
