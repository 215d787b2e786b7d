"""zhip_reduce_static, the entry point that allocates nothing, against the ZHIP_K_REDUCE program launched through
zhip_launch on the same data: bit-identical, on two calls in a row that share the library's static scratch array
(the second with a smaller input), on the null stream and on a stream of the caller's."""
import ctypes as C

import numpy as np
import pytest

import zyx_amd
from zyx_amd import kernels
from zyx_amd.backend import DType

pytestmark = pytest.mark.gpu

_NP = {DType.F32: np.float32, DType.I32: np.int32, DType.BF16: np.uint16}


def _hip_runtime():
    # the HIP runtime the backend library is linked against is already mapped: this only looks it up
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    return hip


def _static_reduce(dev, pool, hip, x, dtype, op, axis0, stream):
    rows, cols = x.shape
    n_out = cols if axis0 else rows
    xb, ev = kernels.to_device(pool, x)
    ob, ev2 = kernels.alloc_like(pool, n_out, x.itemsize)
    pool.sync_events([ev, ev2])  # inputs resident before the caller's stream touches them
    xp, _ = pool.buffer_ptr(xb)
    op_, _ = pool.buffer_ptr(ob)
    dev.reduce_static(dtype, {"sum": 0, "max": 1}[op], axis0, rows, cols, xp, op_, stream or 0)
    assert hip.hipStreamSynchronize(C.c_void_p(stream)) == 0
    res = kernels.to_host(pool, ob, (n_out,), x.dtype)
    pool.deallocate(xb, [])
    pool.deallocate(ob, [])
    return res


CASES = [
    # (dtype, op, axis0, first shape, second (smaller) shape): every shape takes the two-stage path, i.e. the scratch
    (DType.F32, "sum", True, (8192, 1024), (1024, 512)),
    (DType.F32, "max", True, (4096, 768), (512, 260)),
    (DType.I32, "sum", True, (2048, 1000), (640, 333)),
    (DType.F32, "sum", False, (4, 65536), (2, 16384)),
    (DType.BF16, "sum", False, (16, 32768), (3, 8200)),
    (DType.I32, "max", False, (1, 1 << 20), (5, 8192)),
]


def _data(rng, shape, dtype):
    if dtype == DType.I32:
        return rng.integers(-1000, 1000, size=shape, dtype=np.int32)
    x = rng.standard_normal(shape).astype(np.float32)
    if dtype == DType.BF16:
        return (x.view(np.uint32) >> 16).astype(np.uint16)
    return x


@pytest.mark.parametrize("dtype,op,axis0,big,small", CASES)
def test_two_calls_share_the_scratch(hip, dtype, op, axis0, big, small):
    dev, pool = hip
    rt = _hip_runtime()
    stream = C.c_void_p()
    assert rt.hipStreamCreate(C.byref(stream)) == 0
    try:
        rng = np.random.default_rng(7)
        for shape, st in ((big, None), (small, stream.value), (small, None)):
            x = _data(rng, shape, dtype)
            want = kernels.reduce(dev, pool, x, op, axis0, dtype)
            got = _static_reduce(dev, pool, rt, x, dtype, op, axis0, st)
            assert got.dtype == want.dtype and np.array_equal(got.view(np.uint8), want.view(np.uint8)), (shape, st)
    finally:
        rt.hipStreamDestroy(stream)


def test_single_stage_shapes_and_empty(hip):
    dev, pool = hip
    rt = _hip_runtime()
    rng = np.random.default_rng(8)
    for shape, axis0 in (((300, 77), False), ((33, 4096), True), ((5, 0), False)):
        x = _data(rng, shape, DType.F32).reshape(shape)
        want = kernels.reduce(dev, pool, x, "sum", axis0, DType.F32)
        got = _static_reduce(dev, pool, rt, x, DType.F32, "sum", axis0, None)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_null_pointers_and_unsupported_dtypes_are_refused(hip):
    """Nothing is launched for a call that cannot be right. Only null pointers are used here: a made-up non-null
    pointer would fault the device if a refusal ever went missing. (No shape the reduce planner produces needs more
    than the 1 MiB of static scratch any more -- its partials are bounded by two workgroups per compute unit -- so that
    refusal is exercised on the CPU, against the host model of the runtime: tests/fakehip/harness.cpp.)"""
    dev, pool = hip
    with pytest.raises(zyx_amd.BackendError) as ei:
        dev.reduce_static(DType.F32, 0, True, 256, 4096, 0, 0, 0)
    assert ei.value.status == zyx_amd.ErrorStatus.IncorrectKernelArg and "null" in ei.value.context
    with pytest.raises(zyx_amd.BackendError) as ei:
        dev.reduce_static(DType.F64, 0, True, 4, 4, 0, 0, 0)
    assert ei.value.status == zyx_amd.ErrorStatus.KernelCompilation
