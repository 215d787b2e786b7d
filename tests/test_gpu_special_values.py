"""Infinities, NaN, signed zeros and the ends of the finite range through the hand-written kernels, against the CPU
oracle on the same inputs. What is compared is the class of every result (finite / +inf / -inf / NaN) element by
element, and the value where it is finite (1e-5 relative); the C backend's meaning is the oracle's: `fmax` ignores
a NaN operand (zyx/src/codegen/c.rs:600), sums propagate it, a max reduce starts from the lowest finite value
(zyx/src/dtype.rs:207-224), exp(-inf) is 0."""
import numpy as np
import pytest

from zyx_amd import DType
from zyx_amd.kernels import cross_entropy, gemm, norm_rows, reduce

pytestmark = pytest.mark.gpu


def same_class_and_value(got, want, rtol=1e-5, atol=0.0):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want)), np.argwhere(np.isnan(got) != np.isnan(want))[:4].tolist()
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf]) and not np.isinf(got[~inf & ~np.isnan(want)]).any()
    fin = np.isfinite(want)
    np.testing.assert_allclose(got[fin], want[fin], rtol=rtol, atol=atol)


def poisoned(oracle, shape, seed):
    x = oracle.Rng(seed).randn(shape, 2.0)
    rows, cols = shape
    x[0, 1 % cols] = np.inf
    x[1 % rows, 0] = -np.inf
    x[2 % rows, cols // 2] = np.nan
    x[3 % rows, :] = -np.inf
    x[4 % rows, cols - 1] = 3.0e38
    x[4 % rows, cols // 3] = 3.0e38     # the sum of the two overflows
    x[5 % rows, 0] = -0.0
    x[6 % rows, cols // 2] = 1e-45      # subnormal
    return x


@pytest.mark.parametrize("shape", [(8, 4096), (70, 100), (300, 257), (16, 70000)])
@pytest.mark.parametrize("axis0", [False, True])
def test_reductions(hip, oracle, shape, axis0):
    dev, pool = hip
    x = poisoned(oracle, shape, 5)
    ref = oracle.reduce_cols if axis0 else oracle.reduce_rows
    # sums: the tree order differs from the serial one, so finite sums are compared at 1e-5 of sum |x| over finite entries
    got, want = reduce(dev, pool, x, "sum", axis0), ref("sum", x)
    bound = 1e-5 * np.where(np.isfinite(x), np.abs(x), 0).astype(np.float64).sum(0 if axis0 else 1).max()
    same_class_and_value(got, want, rtol=1e-5, atol=bound)
    # max: exact, NaN ignored, a row of -inf gives the lowest finite value it started from
    got, want = reduce(dev, pool, x, "max", axis0), ref("max", x)
    assert np.array_equal(got, want, equal_nan=True)
    if not axis0:
        assert got[3 % shape[0]] == np.float32(-3.4028234663852886e38) and got[2 % shape[0]] == np.nanmax(x[2 % shape[0]])


@pytest.mark.parametrize("shape", [(8, 1024), (9, 1000), (7, 4096)])
def test_norm_rows(hip, oracle, shape):
    """A row holding an infinity or a NaN comes out NaN in every column; rows next to it are untouched."""
    dev, pool = hip
    x = poisoned(oracle, shape, 6)
    x[4, :] = oracle.Rng(1).randn((shape[1],), 1.0)  # the overflowing pair is exercised by the reductions
    w, b = oracle.Rng(2).randn(shape[1]), oracle.Rng(3).randn(shape[1])
    same_class_and_value(norm_rows(dev, pool, x, w, b), oracle.layer_norm(x, w, b), rtol=2e-5, atol=1e-6)
    same_class_and_value(norm_rows(dev, pool, x, w, rms=True, eps=1e-6), oracle.rms_norm(x, w, 1e-6), rtol=2e-5, atol=1e-6)
    big = np.full(shape, 1.5e19, np.float32)  # squares overflow f32
    big[0, ::2] = -1.5e19
    same_class_and_value(norm_rows(dev, pool, big, w, rms=True, eps=1e-6), oracle.rms_norm(big, w, 1e-6))


def test_cross_entropy(hip, oracle):
    """-inf logits of classes other than the label take no part (their softmax is 0); a -inf logit at the label is an
    infinite loss; an infinite or NaN logit makes its row NaN."""
    dev, pool = hip
    x = oracle.Rng(4).randn((6, 10), 2.0)
    lab = np.array([1, 2, 3, 4, 5, 6], np.int32)
    x[0, 5:] = -np.inf
    x[1, 2] = -np.inf
    x[2, 0] = np.inf
    x[3, 9] = np.nan
    x[4, :] = -np.inf
    loss, grad = cross_entropy(dev, pool, x, lab, 1.0)
    wl, wg = oracle.cross_entropy(x, lab, 1.0)
    same_class_and_value(loss, wl, atol=1e-6)
    same_class_and_value(grad, wg, atol=1e-7)
    assert np.isfinite(loss[0]) and (grad[0, 5:] == 0).all() and loss[1] == np.inf


@pytest.mark.parametrize("dtype", [DType.F32, DType.BF16])
@pytest.mark.parametrize("mnk", [(64, 48, 32), (256, 256, 128)])
def test_gemm(hip, oracle, dtype, mnk):
    """inf and NaN operands reach exactly the rows and columns of C they touch (inf * 0 = NaN included), through the
    general kernel and the LDS-tiled bf16 one."""
    dev, pool = hip
    m, n, k = mnk
    r = oracle.Rng(7)
    a, b = r.randn((m, k)), r.randn((k, n))
    a[1, 3] = np.inf
    a[2, 5] = np.nan
    a[3, 7] = -np.inf
    b[3, 4] = 0.0          # inf * 0 in C[1, 4]
    b[9, 6] = np.inf
    b[11, :] = 0.0
    a[5, 11] = np.inf      # a whole row of C becomes NaN
    if dtype == DType.BF16:
        a, b = oracle.f32_to_bf16(a), oracle.f32_to_bf16(b)
    got = gemm(dev, pool, a, b, dtype=dtype, out_dtype=DType.F32)
    want = oracle.matmul(a, b, oracle.BF16 if dtype == DType.BF16 else oracle.F32, oracle.F32)
    # inf - inf inside a sum depends on nothing but the operands present, so classes agree whatever the order
    same_class_and_value(got, want, rtol=1e-4, atol=1e-4)
    assert np.isnan(got[1, 4]) and np.isnan(got[2]).all() and np.isnan(got[5]).all() and np.isfinite(got[10]).sum() >= n - 1
