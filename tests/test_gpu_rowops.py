"""LayerNorm / RMSNorm / cross entropy on the GPU vs the CPU oracle and the reference's goldens
(zyx/tests/05_misc.rs:702-730 layer_norm, :1199-1214 cross_entropy). f32 tolerance 1e-5 relative
to the row's scale (a normalised row has cancelling entries near zero, so the bound is
rel 1e-5 * max(|want|, rms of the row))."""
import numpy as np
import pytest

from zyx_amd import DType
from zyx_amd.kernels import cross_entropy, norm_rows

pytestmark = pytest.mark.gpu


def close_rows(got, want, rtol=1e-5):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    scale = np.maximum(np.abs(want), np.sqrt((want**2).mean(-1, keepdims=True)))
    assert np.all(np.abs(got - want) <= rtol * scale + 1e-30), np.max(np.abs(got - want) / (scale + 1e-30))


def test_layer_norm_reference_golden(hip):
    dev, pool = hip
    x = np.array([[3, 5, 2, 1], [6, 1, 4, 2]], np.float32)
    y = norm_rows(dev, pool, x, w=np.array([4, 5, 1, 2], np.float32), eps=0.00001)
    np.testing.assert_allclose(y, [[0.585539, 6.587314, -0.439154, -2.049387], [4.960858, -5.073606, 0.338240, -1.127468]],
                               rtol=2e-6)


@pytest.mark.parametrize("shape", [(8192, 1024), (5, 7), (33, 1000), (4, 4096), (3, 5001), (1, 2), (64, 256), (7, 512), (9, 2048),
                                   # widths held in the registers of 1 .. 16 waves, whole and ragged last parts
                                   (130, 768), (33, 1280), (9, 3072), (5, 5120), (3, 8192), (4, 16384), (2, 12292), (1025, 772),
                                   (7, 260), (6, 1028), (3, 2052), (2, 16388)])
@pytest.mark.parametrize("rms", [False, True])
def test_norms_f32(hip, oracle, shape, rms):
    dev, pool = hip
    r = oracle.Rng(shape[1])
    x, w, b = r.randn(shape, 2.0) + np.float32(0.5), r.randn(shape[1]), r.randn(shape[1])
    if rms:
        close_rows(norm_rows(dev, pool, x, w, rms=True, eps=1e-6), oracle.rms_norm(x, w, 1e-6))
        close_rows(norm_rows(dev, pool, x, None, rms=True, eps=1e-6), oracle.rms_norm(x, None, 1e-6))
    else:
        close_rows(norm_rows(dev, pool, x, w, b), oracle.layer_norm(x, w, b))
        close_rows(norm_rows(dev, pool, x, w, None), oracle.layer_norm(x, w, None))
        close_rows(norm_rows(dev, pool, x), oracle.layer_norm(x))
        xd = x.astype(np.float64)  # what the mathematics fixes: unbiased variance
        want = (xd - xd.mean(1, keepdims=True)) / np.sqrt(xd.var(1, ddof=1, keepdims=True) + 1e-5)
        close_rows(norm_rows(dev, pool, x), want)


@pytest.mark.parametrize("shape", [(64, 1024), (130, 768), (33, 1544), (9, 3072), (5, 5120), (3, 8200), (4, 16384), (2, 12292),
                                   (7, 260), (6, 1028), (1025, 776), (3, 4100), (5, 1001)])
@pytest.mark.parametrize("rms", [False, True])
def test_norms_bf16(hip, oracle, rms, shape):
    """bf16 storage: f32 arithmetic, one truncating store -> at most one bf16 unit from the oracle. Widths of a
    multiple of 8 (16-byte vectors), of 4 only (8-byte vectors) and of neither, over 1-16 waves per row."""
    dev, pool = hip
    r = oracle.Rng(3)
    cols = shape[1]
    x, w, b = (oracle.f32_to_bf16(a) for a in (r.randn(shape), r.randn(cols), r.randn(cols)))
    if rms:
        got, want = norm_rows(dev, pool, x, w, rms=True, eps=1e-6, dtype=DType.BF16), oracle.rms_norm(x, w, 1e-6, oracle.BF16)
    else:
        got, want = norm_rows(dev, pool, x, w, b, dtype=DType.BF16), oracle.layer_norm(x, w, b, 1e-5, oracle.BF16)
    # one bf16 unit, or, where norm * w and b cancel, the f32 rounding of the two terms
    gf, wf = oracle.bf16_to_f32(got).astype(np.float64), oracle.bf16_to_f32(want).astype(np.float64)
    bad = (np.abs(got.astype(np.int32) - want.astype(np.int32)) > 1) & (np.abs(gf - wf) > 1e-5)
    assert not bad.any(), (int(bad.sum()), gf[bad][:4], wf[bad][:4])
    assert np.mean(got == want) > 0.98


def test_cross_entropy(hip, oracle):
    dev, pool = hip
    loss, _ = cross_entropy(dev, pool, np.array([[2, 3, 4], [5, 6, 7]], np.float32), np.array([1, 2], np.int32))
    np.testing.assert_allclose(loss, [1.407606, 0.407606], rtol=2e-6)
    r = oracle.Rng(8)
    for rows, cols in ((64, 10), (1, 1), (300, 1000), (7, 65)):
        x, lab = r.randn((rows, cols), 3.0), r.randint(rows, 0, cols)
        loss, grad = cross_entropy(dev, pool, x, lab, 1.0 / rows)
        wl, wg = oracle.cross_entropy(x, lab, 1.0 / rows)
        np.testing.assert_allclose(loss, wl, rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(grad, wg, rtol=1e-5, atol=1e-9)
        assert np.all(np.abs(grad.sum(1)) < 1e-6)  # softmax - onehot sums to zero in every row
    # labels outside the class range match no class: zero loss, gradient = softmax * scale
    x = r.randn((2, 5))
    loss, grad = cross_entropy(dev, pool, x, np.array([-1, 5], np.int32), 1.0)
    assert loss.tolist() == [0.0, 0.0]
    np.testing.assert_allclose(grad.sum(1), [1.0, 1.0], rtol=1e-6)


@pytest.mark.parametrize("shape", [(5, 2052), (3, 2049), (9, 4096), (3, 4097), (4, 8192), (2, 8190), (3, 16384), (2, 20000),
                                   (2, 32768), (2, 40001), (3, 50257), (1, 65536), (2, 65535), (300, 3000)])
def test_cross_entropy_many_classes(hip, oracle, shape):
    """Rows of 2049-65536 classes are read once by a workgroup of 4-16 waves (16-byte vectors when the class count is
    a multiple of 4, single values otherwise); same bar as the one-wave-per-row kernel."""
    dev, pool = hip
    rows, cols = shape
    r = oracle.Rng(cols)
    x, lab = r.randn(shape, 3.0), r.randint(rows, 0, cols)
    lab[0] = cols - 1
    if rows > 1:
        lab[1] = -1   # matches no class: zero loss, gradient = softmax * scale
    loss, grad = cross_entropy(dev, pool, x, lab, 1.0 / rows)
    wl, wg = oracle.cross_entropy(x, lab, 1.0 / rows)
    # the oracle adds a row's exp terms one after the other in f32: its sum, the divisor of every gradient, carries an
    # error that grows with the row length (measured 5e-5 at 65536 classes); the kernel's sum is a tree
    tol = 1e-5 * max(1.0, cols / 4096)
    np.testing.assert_allclose(loss, wl, rtol=1e-5, atol=tol)
    np.testing.assert_allclose(grad, wg, rtol=tol, atol=1e-9)
    s = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))   # against the sum in f64: the usual bar
    wg64 = (s / s.sum(1, keepdims=True) - (np.arange(cols)[None, :] == lab[:, None])) / rows
    np.testing.assert_allclose(grad, wg64, rtol=1e-5, atol=1e-9)
    live = lab >= 0
    assert np.all(np.abs(grad[live].astype(np.float64).sum(1)) < 1e-6)
    loss_only, none = cross_entropy(dev, pool, x, lab, None)
    assert none is None and np.array_equal(loss_only, loss)


# ---- gradients of the norms ---------------------------------------------------------------------------------
@pytest.mark.parametrize("shape", [(5, 9), (64, 128), (130, 1024), (3, 1000), (2100, 64), (64, 256), (7, 512), (9, 2048),
                                   (8192, 1024), (4099, 1024), (2051, 512),  # several rows per wave: rows fetched ahead
                                   # widths that are not 256 * 2^n, with lanes past the end of the row
                                   (4100, 768), (2049, 1280), (300, 1536), (37, 1800), (5, 2044), (7, 260), (600, 772), (3, 4),
                                   (1030, 520), (9, 2052)])
@pytest.mark.parametrize("rms", [False, True])
def test_norm_backward_f32(hip, oracle, shape, rms):
    from zyx_amd.kernels import norm_rows_bwd
    dev, pool = hip
    rows, cols = shape
    r = oracle.Rng(rows + cols)
    x, dy, add, w = r.randn(shape), r.randn(shape), r.randn(shape), r.randn((cols,))
    eps = 1e-6 if rms else 1e-5
    for use_w, use_add in ((True, True), (False, False)):
        got = norm_rows_bwd(dev, pool, x, dy, w if use_w else None, add if use_add else None, rms=rms, eps=eps)
        want = oracle.norm_bwd(x, dy, w if use_w else None, add if use_add else None, rms=rms, eps=eps)
        # dx: sums of `cols` terms of size |g|; dw/db: sums of `rows` terms
        assert np.allclose(got[0], want[0], rtol=1e-5, atol=1e-5 * np.sqrt(cols))
        for g, wv in zip(got[1:], want[1:]):
            assert (g is None) == (wv is None)
            if g is not None:
                assert np.allclose(g, wv, rtol=1e-5, atol=2e-6 * rows)


@pytest.mark.parametrize("shape", [(8192, 1024), (4100, 768), (1000, 1288), (300, 2040)])
def test_norm_backward_bf16_rows(hip, oracle, shape):
    """Rows of 1024 bf16 as in config 5 (8192 rows), and widths with lanes past the end of the row: f32 arithmetic,
    one truncating bf16 store."""
    from zyx_amd.kernels import norm_rows_bwd
    from zyx_amd import DType
    dev, pool = hip
    r = oracle.Rng(9)
    x, dy, add = [oracle.f32_to_bf16(r.randn(shape)) for _ in range(3)]
    w = oracle.f32_to_bf16(1.0 + 0.1 * r.randn((shape[1],)))
    got = norm_rows_bwd(dev, pool, x, dy, w, add, dtype=DType.BF16)
    want = oracle.norm_bwd(x, dy, w, add, dtype=oracle.BF16)
    col = float(np.sqrt(shape[0]))   # column sums of `rows` N(0,1) terms are ~sqrt(rows) in size
    for g, wv, scale in zip(got, want, (1.0, col, col)):
        gf, wf = oracle.bf16_to_f32(g).astype(np.float64), oracle.bf16_to_f32(wv).astype(np.float64)
        assert np.all(np.abs(gf - wf) <= 2.0 ** -7 * np.abs(wf) + 1e-4 * scale)


@pytest.mark.parametrize("shape", [(64, 10), (1, 3), (333, 1000), (4096, 17)])
def test_cross_entropy_with_batch_mean(hip, oracle, shape):
    """ZHIP_CE_MEAN: loss, gradient and the batch mean from one launch; rows and gradient equal the plain kernel's
    bit for bit, the mean is sum(loss) / rows to summation order."""
    dev, pool = hip
    r = oracle.Rng(shape[0])
    x, lab = r.randn(shape, 3.0), r.randint(shape[0], 0, shape[1])
    loss, grad = cross_entropy(dev, pool, x, lab, 1.0 / shape[0])
    loss2, grad2, mean = cross_entropy(dev, pool, x, lab, 1.0 / shape[0], mean=True)
    assert np.array_equal(loss, loss2) and np.array_equal(grad, grad2)
    np.testing.assert_allclose(mean, [loss.astype(np.float64).mean()], rtol=2e-6)


def test_cross_entropy_mean_row_limit(hip):
    from zyx_amd import BackendError
    from zyx_amd.kernels import cross_entropy_desc
    dev, pool = hip
    with pytest.raises(BackendError):
        dev.register_kernel(cross_entropy_desc(4097, 10, True, False, 1.0, mean=True))
