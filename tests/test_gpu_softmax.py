"""Parity of the fused softmax + row-sum + row-argmax HIP kernel with the CPU oracle.

Mirrors the reference's softmax / argmax tests (zyx/tests/05_misc.rs:664-683, 1049-1070;
zyx/tests/08_indexing.rs:630-694; zyx/tests/07_realize.rs:264-363) through the C ABI.
Tolerances (f32, relative 1e-5 as the north star states; +1e-37 absolute for results in
the subnormal range, which the hardware exp2 flushes); argmax bit-exact.

Two oracles are used for the float outputs:
  * the f64-accumulated oracle (what the mathematics fixes): GPU must be within 1e-5;
  * the reference-order oracle (serial f32 register accumulator, as zyx's C backend
    emits): its own 4096-term serial sum drifts up to 1.3e-5 from the exact value on the
    config-2 input (measured in test_config2_full_size), and the reference's autotuner may
    reassociate that loop anyway, so the GPU must be within 1e-5 PLUS that oracle's own
    distance to the f64 result, element by element.
"""
import numpy as np
import pytest

from zyx_amd import BackendError, ErrorStatus, kernels

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-37


def assert_close(got, want, rtol=RTOL, atol=ATOL, slack=0.0):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    bad = err > rtol * np.abs(want) + atol + slack
    assert not bad.any(), f"max rel err {np.max(err / (np.abs(want) + 1e-300)):.3e} at {np.argwhere(bad)[:4].tolist()}"


def run_and_check(hip, oracle, x):
    dev, pool = hip
    y, s, a = kernels.softmax_rows(dev, pool, x)
    yo, so, ao = oracle.softmax_rows(x)
    y64, s64 = oracle.softmax_rows_f64acc(x)
    assert_close(y, y64)
    assert_close(s, s64)
    assert_close(y, yo, slack=np.abs(yo.astype(np.float64) - y64))
    assert_close(s, so, slack=np.abs(so.astype(np.float64) - s64))
    assert np.array_equal(a, ao)
    return y, s, a


def test_reference_goldens(hip, oracle):
    dev, pool = hip
    y, _, a = kernels.softmax_rows(dev, pool, np.array([[2.0, 4.0, 3.0], [4.0, 2.0, 3.0]], np.float32))
    assert_close(y, [[0.090030566, 0.6652409, 0.24472846], [0.6652409, 0.090030566, 0.24472846]], rtol=1e-6)
    assert a.tolist() == [1, 0]
    y, _, _ = kernels.softmax_rows(dev, pool, np.array([[2.0, 4.0, 3.0, 4.0, 2.0, 3.0]], np.float32))
    assert_close(y, [[0.045015287, 0.33262047, 0.12236424, 0.33262047, 0.045015287, 0.12236424]], rtol=1e-6)


def test_config2_full_size(hip, oracle):
    """The headline benchmark shape: f32 8192x4096 drawn N(0, 3^2), seeded with zyx's generator."""
    x = oracle.Rng(42069).randn((8192, 4096), 3.0)
    y, s, a = run_and_check(hip, oracle, x)
    yo, _, _ = oracle.softmax_rows(x)
    y64, _ = oracle.softmax_rows_f64acc(x)
    drift = np.max(np.abs(yo - y64) / y64.clip(1e-300))
    assert 1e-6 < drift < 5e-5  # the reference-order sum itself is only good to ~1e-5 here
    # size-independent properties
    assert np.all(np.abs(s - 1.0) < 1e-5)
    assert np.array_equal(a, x.argmax(1))
    assert np.all(y >= 0) and np.all(y <= 1)
    # monotone: order of y follows order of x inside a row
    r = 17
    order = np.argsort(x[r], kind="stable")
    assert np.all(np.diff(y[r][order]) >= 0)


@pytest.mark.parametrize("shape", [(1, 1), (3, 4), (5, 10), (64, 10), (7, 252), (33, 256), (9, 1000), (130, 1024),
                                   (17, 2048), (6, 4092), (5, 4096), (3, 4097), (4, 5000), (2, 16384), (1, 100003),
                                   (2048, 320), (1025, 12),
                                   # rows held in the registers of 4, 8 or 16 waves: whole and ragged last parts
                                   (3, 8192), (5, 8188), (3, 4100), (2, 12292), (3, 32768), (2, 20484), (2, 32772),
                                   (1030, 3072), (1025, 2052), (1024, 4092)])
def test_shapes(hip, oracle, shape):
    x = oracle.Rng(shape[0] * 131 + shape[1]).randn(shape, 3.0)
    run_and_check(hip, oracle, x)


def test_ties_pick_largest_index(hip, oracle):
    # tensor/mod.rs:2262-2266: max_k((y == max) * k)
    x = np.zeros((6, 512), np.float32)
    x[1, [3, 400]] = 5.0
    x[2, :] = -7.25
    x[3, [0]] = 1.0
    x[4, [511, 510]] = 2.0
    x[5, 100:200] = 9.0
    y, s, a = run_and_check(hip, oracle, x)
    assert a.tolist() == [511, 400, 511, 0, 511, 199]
    x = np.zeros((3, 7), np.float32)  # generic (unaligned) path
    x[1, [2, 5]] = 1.0
    x[2, 6] = -1.0
    _, _, a = run_and_check(hip, oracle, x)
    assert a.tolist() == [6, 5, 5]


def test_large_magnitudes(hip, oracle):
    r = oracle.Rng(3)
    x = r.randn((16, 4096), 30.0)      # differences up to ~ -250: many results underflow
    run_and_check(hip, oracle, x)
    x = r.randn((16, 1024), 1e-3) + 1e4  # large common offset is removed by the max
    run_and_check(hip, oracle, x)


@pytest.mark.parametrize("cols", [4096, 1000, 333, 8192])
def test_masked_entries(hip, oracle, cols):
    """-inf entries (a masked_fill before the softmax) give exactly 0 and take no part in the sum, as exp(-inf) = 0
    does in the C backend; the extremes of the finite range behave the same way; a NaN poisons its own row only;
    a row that is -inf throughout is 0 / 0 = NaN on both sides (the max reduce starts from the lowest finite value)."""
    r = oracle.Rng(11)
    x = r.randn((12, cols), 2.0)
    x[0, ::3] = -np.inf
    x[1, 1:] = -np.inf                       # a single live entry
    x[2, : cols // 2] = -3.0e38              # x - max overflows to -inf
    x[3, 5] = 3.0e38
    x[3, 7] = -3.0e38
    x[4, :] = -np.inf
    x[5, 9] = np.nan
    dev, pool = hip
    y, s, a = kernels.softmax_rows(dev, pool, x)
    yo, so, ao = oracle.softmax_rows(x)
    fin = [0, 1, 2, 3] + list(range(6, 12))
    assert not np.isnan(y[fin]).any() and (y[0, ::3] == 0).all() and y[1, 0] == 1.0 and (y[1, 1:] == 0).all()
    assert (y[2, : cols // 2] == 0).all() and y[3, 5] == 1.0 and y[3, 7] == 0
    assert_close(y[fin], yo[fin], slack=1e-6 * np.abs(yo[fin]))
    assert_close(s[fin], so[fin], slack=2e-6)
    assert np.array_equal(a[fin], ao[fin])
    assert np.isnan(y[4]).all() and np.isnan(yo[4]).all() and np.isnan(y[5]).all() and np.isnan(yo[5]).all()


@pytest.mark.parametrize("flags", [(True, False, False), (False, True, False), (False, False, True),
                                   (True, True, False), (True, False, True), (False, True, True)])
@pytest.mark.parametrize("shape", [(37, 4096), (5, 333)])
def test_output_subsets(hip, oracle, flags, shape):
    dev, pool = hip
    x = oracle.Rng(9).randn(shape, 3.0)
    got = kernels.softmax_rows(dev, pool, x, *flags)
    want = oracle.softmax_rows(x)
    for g, w, f in zip(got, want, flags):
        assert (g is not None) == f
        if f and w.dtype == np.int32:
            assert np.array_equal(g, w)
        elif f:
            assert_close(g, w, rtol=2e-5)  # vs the serial-f32 oracle, see module docstring


def test_empty(hip):
    dev, pool = hip
    y, s, a = kernels.softmax_rows(dev, pool, np.zeros((0, 16), np.float32))
    assert y.shape == (0, 16) and s.shape == (0,) and a.shape == (0,)


def test_undersized_argument_is_rejected(hip):
    """Launch arguments are checked on the host before anything is enqueued."""
    dev, pool = hip
    prog = dev.register_kernel(kernels.softmax_rows_desc(8, 64))
    x, e1 = pool.allocate(8 * 64 * 4)
    y, e2 = pool.allocate(8 * 64 * 4 - 4)  # one element short
    s, e3 = pool.allocate(8 * 4)
    a, e4 = pool.allocate(8 * 4)
    with pytest.raises(BackendError) as ei:
        dev.launch(prog, pool, [x, y, s, a], [e1, e2, e3, e4])
    assert ei.value.status == ErrorStatus.IncorrectKernelArg
    with pytest.raises(BackendError) as ei:
        dev.launch(prog, pool, [x, s, a], [])
    assert ei.value.status == ErrorStatus.IncorrectKernelArg
    for b in (x, y, s, a):
        pool.deallocate(b, [])
    dev.release(prog)


# ---- 16-bit storage -----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["bf16", "f16"])
@pytest.mark.parametrize("shape", [(1, 1), (5, 10), (64, 252), (33, 256), (9, 1000), (130, 1024), (6, 4092), (5, 4096), (3, 4097),
                                   (2, 16384), (2048, 320),
                                   (1025, 1024), (1024, 2048), (2050, 4096), (1027, 8192),  # rows split over the waves of a workgroup
                                   (3, 8192), (5, 8184), (2, 12296), (3, 32768), (2, 50264), (2, 65536), (3, 4104)])  # rows in the registers of 8 or 16 waves
def test_sixteen_bit_storage(hip, oracle, shape, dt):
    """bf16 / f16 rows: elements widen to f32 registers, y is truncated on store, the row sum and the argmax read the stored
    y (zyx/src/codegen/c.rs:456-497, 491-496). Against the oracle's restatement: the device's exp differs from expf in the
    last bits of an f32, which can move a truncated y by one unit of its last place; the argmax follows the stored y."""
    from zyx_amd import DType
    dev, pool = hip
    code, dtype, to16, to32, ulp = ((oracle.BF16, DType.BF16, oracle.f32_to_bf16, oracle.bf16_to_f32, 2.0 ** -7) if dt == "bf16" else
                                    (oracle.F16, DType.F16, oracle.f32_to_f16, oracle.f16_to_f32, 2.0 ** -10))
    x = to16(oracle.Rng(shape[0] * 7 + shape[1]).randn(shape, 3.0))
    y, s, a = kernels.softmax_rows(dev, pool, x, dtype=dtype)
    yo, so, ao = oracle.softmax_rows(x, dtype=code)
    yf, yof = to32(y).astype(np.float64), to32(yo).astype(np.float64)
    close = np.abs(yf - yof) <= ulp * yof + (1e-37 if dt == "bf16" else 6e-8)  # at most one step (f16: one subnormal step)
    if dt == "f16":
        # the reference's f32 -> f16 conversion gives 0 below 2^-14 (no subnormals): a y whose f32 value lies within a few
        # ulps of 2^-14 is stored as 2^-14 by one side and as 0 by the other
        cliff = ((yf == 0) & (yof == 2.0 ** -14)) | ((yof == 0) & (yf == 2.0 ** -14))
        assert cliff.sum() <= max(1, y.size // 100000)
        close |= cliff
    assert np.all(close)
    assert np.mean(y == yo) > 0.98
    # the row sum of the stored values, itself stored truncated: a few steps of the 16-bit format around the oracle's
    assert np.all(np.abs(to32(s).astype(np.float64) - to32(so)) <= 4 * ulp)
    exact = to32(y).astype(np.float32).sum(1, dtype=np.float64)
    assert np.all(np.abs(to32(s) - exact) <= 2 * ulp * exact + 1e-3 * ulp)
    # argmax: the largest column among the maxima of the device's own stored row
    yf32 = to32(y)
    want = np.array([np.flatnonzero(r == r.max())[-1] for r in yf32], np.int32)
    assert np.array_equal(a, want)
    assert np.mean(a == ao) > 0.95


def test_sixteen_bit_descriptor_is_checked(hip):
    from zyx_amd import DType
    dev, _ = hip
    d = kernels.softmax_rows_desc(4, 8, dtype=DType.F64)
    with pytest.raises(BackendError) as e:
        dev.register_kernel(d)
    assert e.value.status == ErrorStatus.KernelCompilation
