"""Row / column sum and max on the GPU vs the CPU oracle; integer cases replay the
reference's closed-form tests (zyx/tests/04_reduce.rs:7-175) bit-exactly.

Float tolerance: the GPU folds in a tree, the reference serially; both are compared with
the f64 sum at 1e-5 of sum(|x|) (the bound both orders satisfy), and max is exact.
"""
import numpy as np
import pytest

from zyx_amd import BackendError, DType
from zyx_amd.kernels import argmax_desc, reduce

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (3, 5), (8, 4096), (1, 131072), (1, 1 << 22), (4096, 512), (100, 1000), (513, 257), (70000, 12),
          (2, 100003), (64, 128), (64, 10), (8192, 4096), (2048, 2050), (2100, 2500), (2048, 16384),
          (2047, 4096), (2048, 3072), (2049, 6140), (2048, 6144)]  # either side of the rows-per-workgroup and waves-per-row switches


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("axis0", [False, True])
def test_float_sum_max(hip, oracle, shape, axis0):
    dev, pool = hip
    x = oracle.Rng(shape[0] * 7 + shape[1]).randn(shape, 2.0)
    xd = x.astype(np.float64)
    ax = 0 if axis0 else 1
    got = reduce(dev, pool, x, "sum", axis0)
    want = xd.sum(ax)
    bound = 1e-5 * np.abs(xd).sum(ax) + 1e-30
    assert np.all(np.abs(got - want) <= bound), np.max(np.abs(got - want) / bound)
    ref = (oracle.reduce_cols if axis0 else oracle.reduce_rows)("sum", x)
    assert np.all(np.abs(ref - want) <= bound * 4)  # the serial reference order obeys the same kind of bound
    assert np.array_equal(reduce(dev, pool, x, "max", axis0), x.max(ax))


def test_reference_int_goldens(hip, oracle):
    dev, pool = hip
    assert reduce(dev, pool, np.ones((8, 4096), np.int32), "sum", False, DType.I32).tolist() == [4096] * 8
    assert reduce(dev, pool, np.ones((1, 131072), np.int32), "sum", False, DType.I32).tolist() == [131072]
    x = (np.arange(4 * 1024 * 512) % 10).astype(np.int32).reshape(4 * 1024, 512)
    for axis0 in (False, True):
        assert np.array_equal(reduce(dev, pool, x, "sum", axis0, DType.I32), x.sum(0 if axis0 else 1))
        assert np.array_equal(reduce(dev, pool, x, "max", axis0, DType.I32), x.max(0 if axis0 else 1))
    rng = np.random.default_rng(1)
    big = rng.integers(-2**31, 2**31, size=(300, 999), dtype=np.int64).astype(np.int32)
    assert np.array_equal(reduce(dev, pool, big, "sum", False, DType.I32), oracle.reduce_rows_i32("sum", big))  # wraps
    assert np.array_equal(reduce(dev, pool, big, "max", True, DType.I32), big.max(0))


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16])
def test_16bit_inputs_accumulate_in_f32(hip, oracle, dt):
    dev, pool = hip
    conv = oracle.f32_to_bf16 if dt == DType.BF16 else oracle.f32_to_f16
    back = oracle.bf16_to_f32 if dt == DType.BF16 else oracle.f16_to_f32
    code = oracle.BF16 if dt == DType.BF16 else oracle.F16
    x = conv(oracle.Rng(5).randn((96, 2048)))
    for axis0 in (False, True):
        got = back(reduce(dev, pool, x, "sum", axis0, dt))
        ref = back((oracle.reduce_cols if axis0 else oracle.reduce_rows)("sum", x, code))
        # both truncate an f32 sum to 16 bits: results agree to one unit in the last 16-bit place
        ulp = 2.0 ** (np.floor(np.log2(np.abs(ref) + 1e-30)) - (7 if dt == DType.BF16 else 10))
        assert np.all(np.abs(got - ref) <= ulp + 1e-6)
        assert np.array_equal(reduce(dev, pool, x, "max", axis0, dt),
                              (oracle.reduce_cols if axis0 else oracle.reduce_rows)("max", x, code))


@pytest.mark.parametrize("cols", [4096, 4100, 4103, 12296])
def test_rows_shared_by_a_workgroup(hip, oracle, cols):
    """Many rows of 8-64 KiB: four waves take a quarter of the row each. Integer sums (wrapping) and maxima are exact
    whatever the split; 16-bit rows whose quarters are not whole 16-byte pieces take the narrower loads."""
    dev, pool = hip
    rng = np.random.default_rng(cols)
    x = rng.integers(-2**31, 2**31, size=(2048, cols), dtype=np.int64).astype(np.int32)
    assert np.array_equal(reduce(dev, pool, x, "sum", False, DType.I32), oracle.reduce_rows_i32("sum", x))
    assert np.array_equal(reduce(dev, pool, x, "max", False, DType.I32), x.max(1))
    xb = oracle.f32_to_bf16(oracle.Rng(cols).randn((2048, cols)))
    assert np.array_equal(reduce(dev, pool, xb, "max", False, DType.BF16), oracle.reduce_rows("max", xb, oracle.BF16))
    got = oracle.bf16_to_f32(reduce(dev, pool, xb, "sum", False, DType.BF16))
    ref = oracle.bf16_to_f32(oracle.reduce_rows("sum", xb, oracle.BF16))
    ulp = 2.0 ** (np.floor(np.log2(np.abs(ref) + 1e-30)) - 7)
    assert np.all(np.abs(got - ref) <= ulp + 1e-4 * np.sqrt(cols))


def test_empty_axes(hip):
    dev, pool = hip
    assert reduce(dev, pool, np.zeros((4, 0), np.float32), "sum").tolist() == [0.0] * 4
    assert reduce(dev, pool, np.zeros((0, 4), np.float32), "sum").shape == (0,)
    assert np.all(reduce(dev, pool, np.zeros((4, 0), np.float32), "max") == np.float32(-3.4028235e38))


@pytest.mark.parametrize("shape,axis0", [((64, 10), True), ((64, 128), True), ((1, 64), False), ((4096, 512), True), ((300, 1000), False),
                                         ((2, 100003), False), ((70000, 12), True)])
def test_scaled_sum_onto_a_base(hip, oracle, shape, axis0):
    """The ops that follow a reduce in a training step folded into its store: (sum * mul) / div + base, each one
    f32 operation in that order -- bit-identical to applying them to the plain kernel's result (`p - g * lr` is
    `g * -lr + p` exactly; a mean divides by n)."""
    dev, pool = hip
    x = oracle.Rng(shape[0] + shape[1]).randn(shape, 1.5)
    n_out = shape[1] if axis0 else shape[0]
    base = oracle.Rng(9).randn((n_out,), 1.0)
    plain = reduce(dev, pool, x, "sum", axis0)
    lr = np.float32(0.01)
    assert np.array_equal(reduce(dev, pool, x, "sum", axis0, mul=-float(lr), base=base), base - plain * lr)
    assert np.array_equal(reduce(dev, pool, x, "sum", axis0, div=float(shape[0])), plain / np.float32(shape[0]))
    assert np.array_equal(reduce(dev, pool, x, "sum", axis0, mul=3.0, div=7.0, base=base), plain * np.float32(3) / np.float32(7) + base)
    assert np.array_equal(reduce(dev, pool, x, "max", axis0, base=base), x.max(0 if axis0 else 1) + base)
    xb = oracle.f32_to_bf16(x)
    got = reduce(dev, pool, xb, "sum", axis0, DType.BF16, mul=0.5, base=oracle.f32_to_bf16(base))
    acc = oracle.bf16_to_f32(reduce(dev, pool, xb, "sum", axis0, DType.BF16))  # stored sum: one truncation early
    want = oracle.bf16_to_f32(xb).astype(np.float64).sum(0 if axis0 else 1) * 0.5 + oracle.bf16_to_f32(oracle.f32_to_bf16(base))
    assert np.all(np.abs(oracle.bf16_to_f32(got) - want) <= 2.0 ** -7 * np.abs(want) + 1e-4 * np.abs(oracle.bf16_to_f32(xb)).sum(0 if axis0 else 1))


def test_scale_is_refused_for_integers(hip):
    from zyx_amd import BackendError
    from zyx_amd.kernels import reduce_desc
    dev, pool = hip
    with pytest.raises(BackendError):
        dev.register_kernel(reduce_desc(4, 4, "sum", False, DType.I32, mul=2.0))


# ---- argmax_axis (zyx/src/tensor/mod.rs:2238-2269) -------------------------------------------------------------
def test_argmax_reference_goldens(hip):
    """zyx/tests/08_indexing.rs:630-694 on the device, as i32 tensors (what the reference builds) and as f32."""
    from zyx_amd.kernels import argmax, argmax_axis
    dev, pool = hip
    for dt, np_dt in ((DType.I32, np.int32), (DType.F32, np.float32)):
        am = lambda x, ax: argmax_axis(dev, pool, np.array(x, np_dt), ax, dt).tolist()
        assert am([1, 3, 2, 5], 0) == 3 or am([1, 3, 2, 5], 0) == [3]
        x2 = [[1, 3, 2], [4, 6, 5], [7, 9, 8]]
        assert argmax(dev, pool, np.array(x2, np_dt), dt).item() == 7
        assert am(x2, 0) == [2, 2, 2] and am(x2, 1) == [1, 1, 1]
        xn = [[-1, -3, -2], [-4, -6, -5]]
        assert argmax(dev, pool, np.array(xn, np_dt), dt).item() == 0
        assert am(xn, 0) == [0, 0, 0] and am(xn, 1) == [0, 0]
        assert am([[42]], 0) == [0] and am([[42]], 1) == [0]
        x3 = [[[1, 5, 2], [4, 0, 3]], [[7, 2, 6], [1, 8, 0]]]
        assert am(x3, 0) == [[1, 0, 1], [0, 1, 0]] and am(x3, 1) == [[1, 0, 1], [0, 1, 0]] and am(x3, 2) == [[1, 0], [0, 1]]


@pytest.mark.parametrize("shape,axis", [((8192, 4096), 1), ((8192, 4096), 0), ((3, 70000), 1), ((1, 1 << 21), 1),
                                        ((5, 777, 33), 1), ((2, 9000, 3), 1), ((64, 10), 1), ((7, 5, 260), 0),
                                        ((300, 1001), 1), ((4097, 2), 0)])
def test_argmax_axis_matches_oracle(hip, oracle, shape, axis):
    """Bit-exact arg-max on every layout the kernels split differently (one wave per row, segmented rows, strided
    axis with and without chunks), with many ties (values drawn from 12 levels) and without."""
    from zyx_amd.kernels import argmax_axis
    dev, pool = hip
    rng = np.random.default_rng(sum(shape) + axis)
    ties = rng.integers(-6, 6, size=shape).astype(np.int32)
    assert np.array_equal(argmax_axis(dev, pool, ties, axis, DType.I32), oracle.argmax_axis(ties, axis))
    assert np.array_equal(argmax_axis(dev, pool, ties.astype(np.float32), axis, DType.F32), oracle.argmax_axis(ties.astype(np.float32), axis))
    x = rng.standard_normal(shape).astype(np.float32)
    assert np.array_equal(argmax_axis(dev, pool, x, axis, DType.F32), oracle.argmax_axis(x, axis))
    xb = oracle.f32_to_bf16(x)  # storage bits; many ties after truncation
    assert np.array_equal(argmax_axis(dev, pool, xb, axis, DType.BF16), oracle.argmax_axis(oracle.bf16_to_f32(xb), axis))


def test_argmax_skips_nan_and_handles_lowest(hip, oracle):
    from zyx_amd.kernels import argmax_axis
    dev, pool = hip
    x = np.array([[np.nan, 1.0, np.nan, 1.0, 0.5], [np.nan] * 5, [-np.inf] * 5, [-3.4028235e38, -np.inf, -3.4028235e38, -np.inf, -np.inf],
                  [0.0, -0.0, 0.0, -0.0, -1.0]], np.float32)
    got = argmax_axis(dev, pool, x, 1, DType.F32)
    # fmax skips a NaN and a NaN equals nothing: the expression's IEEE reading. (The reference's C backend compiles
    # with -ffast-math, which leaves NaN handling unspecified; the CPU oracle, built with the same flags, is therefore
    # only consulted on the NaN-free rows.)
    assert got.tolist() == [3, 0, 0, 2, 3]
    assert np.array_equal(got[2:], oracle.argmax_axis(x[2:], 1))
    with pytest.raises(BackendError):
        dev.register_kernel(argmax_desc(4, 0, 4))
