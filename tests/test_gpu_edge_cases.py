"""Empty and degenerate shapes through every kernel kind of the C ABI: nothing may fault, outputs of empty
problems are empty, and one-element problems agree with the oracle. The reference's tensors may have zero-sized
axes (zyx/tests/05_misc.rs, 04_reduce.rs exercise reshapes and reductions down to single elements)."""
import numpy as np
import pytest

from zyx_amd import BackendError, DType, ErrorStatus
from zyx_amd import kernels as K

pytestmark = pytest.mark.gpu


def _buf(pool, nbytes):
    b, e = pool.allocate(nbytes + 8)
    pool.sync_events([e])
    return b


def test_empty_problems_launch_and_finish(hip):
    dev, pool = hip
    chain = K.Chain(0, 16)
    chain.load(chain.input()).relu()
    cases = [
        (K.softmax_rows_desc(0, 128), 4), (chain.desc(), 2), (K.reduce_desc(0, 64, "sum"), 2),
        (K.reduce_desc(0, 64, "sum", axis0=True), 2), (K.norm_rows_desc(0, 256), 4),
        (K.norm_rows_bwd_desc(0, 256, add=True), 7), (K.cross_entropy_desc(0, 10, True, True, 1.0), 4),
        (K.attention_desc(0, 128, 2, 64, DType.BF16, lse=True), 3), (K.attention_bwd_desc(0, 128, 2, 64, DType.BF16), 5),
        (K.conv2d_desc(0, 3, 8, 8, 4, 3, 3, padding=(1, 1)), 3), (K.max_pool2d_desc(0, 8, 8), 2),
        (K.index_desc(K.INDEX_GATHER, (0, 5), (0, 3), 1, DType.F32), 3),
    ]
    bufs = [_buf(pool, 1 << 16) for _ in range(7)]
    for desc, n_args in cases:
        prog = dev.register_kernel(desc)
        pool.sync_events([dev.launch(prog, pool, bufs[:n_args], [])])
        dev.release(prog)
    for b in bufs:
        pool.deallocate(b, [])


def test_degenerate_gemm_shapes_are_refused_or_empty(hip):
    dev, pool = hip
    for m, n, k in [(0, 4, 4), (4, 0, 4), (4, 4, 0)]:
        with pytest.raises(BackendError) as ei:
            dev.register_kernel(K.gemm_desc(m, n, k, DType.F32, DType.F32))
        assert ei.value.status == ErrorStatus.KernelCompilation


def test_single_element_problems(hip, oracle):
    dev, pool = hip
    x = np.array([[3.5]], np.float32)
    y, s, a = K.softmax_rows(dev, pool, x)
    assert y.tolist() == [[1.0]] and s.tolist() == [1.0] and a.tolist() == [0]
    assert K.reduce(dev, pool, x, "max").tolist() == [3.5] and K.reduce(dev, pool, x, "sum", axis0=True).tolist() == [3.5]
    assert K.gemm(dev, pool, x, np.array([[2.0]], np.float32), dtype=DType.F32).tolist() == [[7.0]]
    qkv = np.array([[[1.0, 2.0, 5.0]]], np.float32)  # one token, one head of width 1: softmax over one key is 1 -> y = v
    assert K.attention(dev, pool, qkv, 1, DType.F32).tolist() == [[[5.0]]]
    assert K.gather(dev, pool, np.array([7], np.int32), 0, np.array([0])).tolist() == [7]
    w = np.array([[[[2.0]]]], np.float32)
    assert K.conv2d(dev, pool, np.array([[[[3.0]]]], np.float32), w).tolist() == [[[[6.0]]]]
    ln = K.norm_rows(dev, pool, np.array([[1.0, 3.0]], np.float32))  # n-1 variance of (1, 3) is 2
    assert np.allclose(ln, oracle.layer_norm(np.array([[1.0, 3.0]], np.float32)), rtol=1e-6)


def test_ragged_shapes_next_to_the_fast_paths(hip, oracle):
    """One element off the shapes the specialised kernels take: the general kernels must pick them up."""
    dev, pool = hip
    r = oracle.Rng(1)
    a, b = oracle.f32_to_bf16(r.uniform((257, 65), -1, 1)), oracle.f32_to_bf16(r.uniform((65, 129), -1, 1))
    want = oracle.bf16_to_f32(a).astype(np.float64) @ oracle.bf16_to_f32(b).astype(np.float64)
    assert np.allclose(K.gemm(dev, pool, a, b), want, rtol=1e-3, atol=1e-4)
    x = r.randn((3, 4097))
    y, s, arg = K.softmax_rows(dev, pool, x)
    ry, rs, ra = oracle.softmax_rows(x)
    assert np.allclose(y, ry, rtol=2e-5, atol=1e-9) and np.array_equal(arg, ra)
    xn = r.randn((5, 1025))
    assert np.allclose(K.norm_rows(dev, pool, xn), oracle.layer_norm(xn), rtol=1e-5, atol=1e-5)
    qkv = oracle.f32_to_bf16(r.randn((1, 129, 3 * 64)))
    got = oracle.bf16_to_f32(K.attention(dev, pool, qkv, 1))
    ref = oracle.bf16_to_f32(oracle.attention(qkv, 1, dtype=oracle.BF16))
    assert np.all(np.abs(got - ref) <= 2.0 ** -6 * np.abs(ref) + 3e-3)


def test_shapes_whose_byte_counts_would_overflow_are_refused(hip):
    """Every tensor of a kernel stays below 2^40 elements: a descriptor whose sizes would wrap the 64-bit byte counts
    (and so pass the buffer-size check of a launch) is refused at registration."""
    from zyx_amd import BackendError, ErrorStatus, KernelDesc
    from zyx_amd import kernels as K
    dev, pool = hip
    big = 1 << 62

    def refused(d):
        with pytest.raises(BackendError) as e:
            dev.release(dev.register_kernel(d))
        assert e.value.status == ErrorStatus.KernelCompilation

    for m, n, k in ((64, big, 64), (64, 64, big), (1 << 21, 1 << 21, 64), (64, (1 << 31), 64)):
        refused(K.gemm_desc(m, n, k, DType.F32, DType.F32))
    d = K.gemm_desc(64, 64, 64, DType.F32, DType.F32)
    d.dims[3] = 1 << 20
    refused(d)
    d = K.conv2d_desc(1, 3, 8, 8, 4, 3, 3) if hasattr(K, "conv2d_desc") else None
    if d is not None:
        for idx, val in ((0, big), (4, big), (4, 1 << 33), (5, 1 << 40), (1, 1 << 30)):
            e = KernelDesc.from_buffer_copy(bytes(d))
            e.dims[idx] = val
            refused(e)
    d = K.max_pool2d_desc(4, 8, 8) if hasattr(K, "max_pool2d_desc") else None
    if d is not None:
        e = KernelDesc.from_buffer_copy(bytes(d))
        e.dims[0] = big
        refused(e)
    d = K.attention_desc(1, 16, 2, 8, DType.F32)
    for idx, val in ((2, big), (0, 1 << 40), (2, 70000)):
        e = KernelDesc.from_buffer_copy(bytes(d))
        e.dims[idx] = val
        refused(e)
    # padding / dilation / stride near 2^31 must be refused, not wrap the output-size arithmetic
    for ip, val in ((2, (1 << 31) - 1), (3, 1 << 30), (4, 1 << 30), (0, 1 << 30)):
        e = K.conv2d_desc(1, 3, 8, 8, 4, 3, 3)
        e.iparams[ip] = val
        refused(e)
        e = K.max_pool2d_desc(4, 8, 8)
        e.iparams[ip] = val
        refused(e)
    # a last-axis reduce with more (row, segment) items than a 32-bit grid of 4-item workgroups holds
    refused(K.reduce_desc(1 << 34, 1, "sum"))
    refused(K.reduce_desc(1 << 34, 0, "sum"))
    dev.release(dev.register_kernel(K.reduce_desc(1 << 32, 1, "sum")))  # 2^30 workgroups: fits
