"""conv2d (+bias, +ReLU) and max-pool on the GPU vs the CPU oracle. f32: 1e-5 relative to
sum |x w| over the receptive field (the scale of any summation order's rounding); bf16: the
f32 sum is truncated to bf16, so results agree to one bf16 unit (plus 1e-3 of that scale).
Max-pool is exact. Goldens: zyx/tests/05_misc.rs:880-888 (conv1), :85-109 (test_max_pool)."""
import numpy as np
import pytest

from zyx_amd import DType
from zyx_amd.kernels import conv2d, max_pool2d

pytestmark = pytest.mark.gpu


def test_reference_goldens(hip):
    dev, pool = hip
    t = np.arange(9, dtype=np.float32).reshape(1, 1, 3, 3)
    assert conv2d(dev, pool, t, np.ones((1, 1, 2, 2), np.float32)).tolist() == [[[[8.0, 12.0], [20.0, 24.0]]]]
    x = np.arange(1, 17, dtype=np.float32).reshape(1, 1, 4, 4)
    assert max_pool2d(dev, pool, x).tolist() == [[[[6.0, 8.0], [14.0, 16.0]]]]


CASES = [
    # n, c, h, w, cout, kh, kw, stride, pad, dil
    (2, 3, 9, 11, 4, 3, 2, (1, 1), (1, 1), (1, 1)),
    (2, 3, 9, 11, 4, 3, 2, (2, 1), (0, 2), (1, 1)),
    (1, 5, 12, 10, 70, 3, 3, (1, 2), (2, 1), (2, 2)),
    (3, 16, 14, 14, 33, 1, 1, (1, 1), (0, 0), (1, 1)),
    (2, 64, 28, 28, 128, 3, 3, (1, 1), (1, 1), (1, 1)),
    (1, 7, 5, 5, 3, 5, 5, (1, 1), (2, 2), (1, 1)),
]


@pytest.mark.parametrize("case", CASES)
def test_conv_f32(hip, oracle, case):
    dev, pool = hip
    n, c, h, w, co, kh, kw, stride, pad, dil = case
    r = oracle.Rng(c * 100 + co)
    x, wt, b = r.randn((n, c, h, w)), r.randn((co, c, kh, kw), float(np.sqrt(2.0 / (c * kh * kw)))), r.randn(co, 0.1)
    for bias, relu in ((None, False), (b, False), (b, True)):
        got = conv2d(dev, pool, x, wt, bias, stride, pad, dil, relu)
        want = oracle.conv2d(x, wt, bias, stride, pad, dil, relu)
        mag = oracle.conv2d(np.abs(x), np.abs(wt), None if bias is None else np.abs(b), stride, pad, dil)
        assert got.shape == want.shape
        assert np.all(np.abs(got - want) <= 2e-5 * mag + 1e-30), np.max(np.abs(got - want) / (mag + 1e-30))


def test_conv_relu_pool_config4_slice(hip, oracle):
    """Config 4 geometry (C=64, 56x56, 3x3, 128 output channels, stride 1, pad 1, Kaiming-normal
    weights, ReLU, 2x2 max-pool) on a batch of 2 -- the oracle needs ~0.5 s per image."""
    dev, pool = hip
    r = oracle.Rng(42069)
    x, wt = r.randn((2, 64, 56, 56)), r.randn((128, 64, 3, 3), float(np.sqrt(2.0 / 576)))
    y, pooled = conv2d(dev, pool, x, wt, None, (1, 1), (1, 1), (1, 1), relu=True, pool_kernel=(2, 2))
    want = oracle.conv2d(x, wt, None, (1, 1), (1, 1), (1, 1), relu=True)
    mag = oracle.conv2d(np.abs(x), np.abs(wt), None, (1, 1), (1, 1), (1, 1))
    assert np.all(np.abs(y - want) <= 2e-5 * mag)
    assert np.array_equal(pooled, oracle.max_pool2d(y))  # pooling the GPU's own conv output is exact
    assert pooled.shape == (2, 128, 28, 28) and pooled.min() >= 0


def test_conv_full_batch_linearity(hip, oracle):
    """Full config-4 size (N=32): checked through properties instead of the CPU oracle --
    conv(x, w1 + w2) == conv(x, w1) + conv(x, w2) and batch independence."""
    dev, pool = hip
    r = oracle.Rng(1)
    x = r.randn((32, 64, 56, 56))
    w1, w2 = r.randn((128, 64, 3, 3), 0.05), r.randn((128, 64, 3, 3), 0.05)
    y1 = conv2d(dev, pool, x, w1, None, (1, 1), (1, 1))
    y2 = conv2d(dev, pool, x, w2, None, (1, 1), (1, 1))
    y12 = conv2d(dev, pool, x, w1 + w2, None, (1, 1), (1, 1))
    assert y12.shape == (32, 128, 56, 56)
    assert np.allclose(y12, y1 + y2, rtol=1e-4, atol=2e-4)
    ysub = conv2d(dev, pool, x[5:7], w1, None, (1, 1), (1, 1))
    assert np.array_equal(ysub, y1[5:7])


def test_conv_bf16(hip, oracle):
    dev, pool = hip
    r = oracle.Rng(3)
    x, wt, b = (oracle.f32_to_bf16(a) for a in (r.randn((2, 16, 20, 20)), r.randn((24, 16, 3, 3), 0.1), r.randn(24, 0.1)))
    got = conv2d(dev, pool, x, wt, b, (1, 1), (1, 1), (1, 1), relu=True, dtype=DType.BF16)
    want = oracle.conv2d(x, wt, b, (1, 1), (1, 1), (1, 1), True, oracle.BF16)
    g, wv = oracle.bf16_to_f32(got), oracle.bf16_to_f32(want)
    mag = oracle.conv2d(np.abs(oracle.bf16_to_f32(x)), np.abs(oracle.bf16_to_f32(wt)), np.abs(oracle.bf16_to_f32(b)), (1, 1), (1, 1))
    assert np.all(np.abs(g - wv) <= 2.0 ** -7 * np.abs(wv) + 1e-3 * mag)
    got32 = conv2d(dev, pool, x, wt, None, (1, 1), (1, 1), (1, 1), dtype=DType.BF16, out_dtype=DType.F32)
    want32 = oracle.conv2d(x, wt, None, (1, 1), (1, 1), (1, 1), False, oracle.BF16, oracle.F32)
    assert np.all(np.abs(got32 - want32) <= 1e-3 * np.abs(want32) + 2e-5 * mag)


@pytest.mark.parametrize("args", [((2, 2), (2, 2), (0, 0), (1, 1)), ((3, 3), (2, 2), (1, 1), (1, 1)),
                                  ((3, 2), (1, 2), (1, 0), (2, 1)), ((1, 1), (1, 1), (0, 0), (1, 1))])
def test_max_pool(hip, oracle, args):
    dev, pool = hip
    x = oracle.Rng(2).randn((3, 5, 17, 23))
    assert np.array_equal(max_pool2d(dev, pool, x, *args), oracle.max_pool2d(x, *args))
    xb = oracle.f32_to_bf16(x)
    assert np.array_equal(max_pool2d(dev, pool, xb, *args, dtype=DType.BF16), oracle.max_pool2d(xb, *args, dtype=oracle.BF16))


@pytest.mark.parametrize("case", [
    # (N, C, H, W, Cout, k, stride, pad, dilation): pixels % 256 == 0, Cout % 128 == 0, C*k*k % 64 == 0 -> patches + tiled GEMM
    (4, 64, 16, 16, 128, 3, 1, 1, 1), (2, 64, 32, 32, 256, 1, 1, 0, 1), (8, 16, 16, 16, 128, 2, 2, 0, 1), (1, 64, 34, 34, 128, 3, 2, 1, 2)])
@pytest.mark.parametrize("bias,relu", [(True, True), (False, True), (True, False), (False, False)])
def test_conv_bf16_on_the_tiled_gemm(hip, oracle, case, bias, relu):
    dev, pool = hip
    n, c, h, w, co, k, s, p, d = case
    r = oracle.Rng(n + c + k)
    x, wt = oracle.f32_to_bf16(r.randn((n, c, h, w))), oracle.f32_to_bf16(r.randn((co, c, k, k), 0.1))
    b = oracle.f32_to_bf16(r.randn(co, 0.5)) if bias else None
    args = ((s, s), (p, p), (d, d))
    mag = oracle.conv2d(np.abs(oracle.bf16_to_f32(x)), np.abs(oracle.bf16_to_f32(wt)), None if b is None else np.abs(oracle.bf16_to_f32(b)), *args)
    got = conv2d(dev, pool, x, wt, b, *args, relu=relu, dtype=DType.BF16)
    want = oracle.conv2d(x, wt, b, *args, relu, oracle.BF16)
    assert got.shape == want.shape and (got.shape[0] * got.shape[2] * got.shape[3]) % 256 == 0
    g, wv = oracle.bf16_to_f32(got), oracle.bf16_to_f32(want)
    # the oracle stores the 16-bit sum (truncating) before a second kernel adds the bias; the GPU adds the bias in
    # the same kernel and stores once: they differ by up to one bf16 unit of the pre-bias value
    pre = np.abs(wv) + (np.abs(oracle.bf16_to_f32(b)).reshape(1, -1, 1, 1) if bias else 0.0)
    assert np.all(np.abs(g - wv) <= 2.0 ** -7 * pre + 1e-3 * mag)
    got32 = conv2d(dev, pool, x, wt, b, *args, relu=relu, dtype=DType.BF16, out_dtype=DType.F32)
    want32 = oracle.conv2d(x, wt, b, *args, relu, oracle.BF16, oracle.F32)
    assert np.all(np.abs(got32 - want32) <= 1e-3 * np.abs(want32) + 2e-5 * mag)
    # identical arithmetic before the store: the bf16 result is the truncation of the f32 one
    assert np.array_equal(got, oracle.f32_to_bf16(got32))


def test_config4_bf16_full_size(hip, oracle):
    """N=32, C=64, 56x56, 3x3 -> 128, pad 1, ReLU, then 2x2 max-pool, bf16 storage: 4 images against the oracle,
    all of it through linearity in the weights (ReLU off) and batch independence."""
    dev, pool = hip
    r = oracle.Rng(42069)
    x = oracle.f32_to_bf16(r.randn((32, 64, 56, 56)))
    w1 = oracle.f32_to_bf16(r.randn((128, 64, 3, 3), float(np.sqrt(2.0 / 576))))
    y, pooled = conv2d(dev, pool, x, w1, None, (1, 1), (1, 1), relu=True, dtype=DType.BF16, pool_kernel=(2, 2))
    assert y.shape == (32, 128, 56, 56) and pooled.shape == (32, 128, 28, 28)
    sel = [0, 11, 31]
    want = oracle.bf16_to_f32(oracle.conv2d(x[sel], w1, None, (1, 1), (1, 1), (1, 1), True, oracle.BF16))
    mag = oracle.conv2d(np.abs(oracle.bf16_to_f32(x[sel])), np.abs(oracle.bf16_to_f32(w1)), None, (1, 1), (1, 1))
    assert np.all(np.abs(oracle.bf16_to_f32(y[sel]) - want) <= 2.0 ** -7 * np.abs(want) + 1e-3 * mag)
    assert np.array_equal(pooled, oracle.max_pool2d(y, dtype=oracle.BF16))
    # f32 results of bf16 operands are linear in the weights up to f32 summation error
    w2 = oracle.f32_to_bf16(r.randn((128, 64, 3, 3), 0.05))
    w12 = oracle.f32_to_bf16(oracle.bf16_to_f32(w1) * 0.5)  # exact in bf16
    ya = conv2d(dev, pool, x, w1, None, (1, 1), (1, 1), dtype=DType.BF16, out_dtype=DType.F32)
    yb = conv2d(dev, pool, x, w12, None, (1, 1), (1, 1), dtype=DType.BF16, out_dtype=DType.F32)
    assert np.array_equal(yb, ya * 0.5)  # scaling the weights by a power of two scales every product exactly
    assert np.array_equal(conv2d(dev, pool, x[7:15], w2, None, (1, 1), (1, 1), dtype=DType.BF16, out_dtype=DType.F32),
                          conv2d(dev, pool, x, w2, None, (1, 1), (1, 1), dtype=DType.BF16, out_dtype=DType.F32)[7:15])


@pytest.mark.parametrize("geom", [
    # (x shape, weight shape, stride, padding, dilation): shapes whose patch rows the GEMM gathers itself (unit
    # column stride, output rows of 8k pixels); dilation, row stride, asymmetric padding, 1x1 and 5x5 windows
    ((4, 64, 24, 24), (128, 64, 3, 3), (1, 1), (2, 2), (2, 2)), ((4, 64, 32, 16), (128, 64, 3, 3), (2, 1), (1, 1), (1, 1)),
    ((2, 64, 8, 32), (256, 64, 1, 1), (1, 1), (0, 0), (1, 1)), ((1, 64, 16, 20), (128, 64, 5, 5), (1, 1), (2, 0), (1, 1)),
    ((8, 32, 9, 16), (128, 32, 2, 1), (1, 1), (0, 0), (1, 1)), ((2, 64, 17, 25), (128, 64, 2, 2), (1, 1), (0, 0), (1, 1))])
def test_conv_bf16_gathered_by_the_gemm(hip, oracle, geom):
    dev, pool = hip
    xs, ws, stride, pad, dil = geom
    r = oracle.Rng(sum(xs))
    x, wt, b = oracle.f32_to_bf16(r.randn(xs)), oracle.f32_to_bf16(r.randn(ws, 0.1)), oracle.f32_to_bf16(r.randn(ws[0], 0.5))
    got32 = conv2d(dev, pool, x, wt, b, stride, pad, dil, relu=True, dtype=DType.BF16, out_dtype=DType.F32)
    want32 = oracle.conv2d(x, wt, b, stride, pad, dil, True, oracle.BF16, oracle.F32)
    mag = oracle.conv2d(np.abs(oracle.bf16_to_f32(x)), np.abs(oracle.bf16_to_f32(wt)), np.abs(oracle.bf16_to_f32(b)), stride, pad, dil)
    assert got32.shape == want32.shape and got32.shape[3] % 8 == 0 and (got32.shape[0] * got32.shape[2] * got32.shape[3]) % 256 == 0
    assert np.all(np.abs(got32 - want32) <= 1e-3 * np.abs(want32) + 2e-5 * mag)


@pytest.mark.parametrize("shape", [(2, 3, 8, 8), (32, 128, 56, 56), (1, 5, 17, 24), (3, 2, 2, 16), (1, 1, 9, 40)])
def test_max_pool_2x2_fast_path(hip, oracle, shape):
    """2 x 2 / stride 2 windows over rows of a multiple of 8 elements take the vectorised kernel: exact against the
    oracle, including odd heights, a NaN beside numbers (ignored by fmax) and -inf (the running maximum starts at the
    lowest finite value, which a window of -inf therefore returns). A window of NaN only is left out: the reference
    compiles its kernels with -ffast-math, under which fmax of two NaN-free-by-assumption operands is whatever the
    compiler picked."""
    dev, pool = hip
    x = oracle.Rng(shape[2] * shape[3]).randn(shape, 3.0)
    x[0, 0, 0, 0] = np.nan
    x[0, 0, 0, 4:6] = -np.inf
    x[0, 0, 1, 4:6] = -np.inf                # a window of -inf only
    x[-1, -1, 1, -1] = np.inf
    args = ((2, 2), (2, 2), (0, 0), (1, 1))
    got, want = max_pool2d(dev, pool, x, *args), oracle.max_pool2d(x, *args)
    assert np.array_equal(got, want) and got[0, 0, 0, 2] == np.float32(-3.4028234663852886e38)
    xb = oracle.f32_to_bf16(x)
    assert np.array_equal(max_pool2d(dev, pool, xb, *args, dtype=DType.BF16), oracle.max_pool2d(xb, *args, dtype=oracle.BF16))


@pytest.mark.parametrize("shape", [(2, 16, 16, 56, 128), (1, 64, 56, 56, 128), (3, 32, 28, 16, 256), (2, 48, 8, 112, 128), (1, 16, 56, 8, 128),
                                   (2, 64, 16, 28, 128), (1, 96, 8, 56, 128), (1, 32, 2, 224, 128), (1, 128, 28, 16, 128),
                                   (2, 64, 28, 56, 128), (1, 32, 3, 224, 128),  # heights only the 224-pixel tile divides
                                   (1, 128, 8, 56, 128)])  # 128 channels at this width fit the 448-pixel tile's LDS only
@pytest.mark.parametrize("bias,relu", [(True, True), (False, False)])
def test_conv3x3_direct_bf16(hip, oracle, shape, bias, relu):
    """3 x 3 / stride 1 / padding 1 bf16 shapes whose rows tile into 448-pixel blocks take the direct kernel (input
    tile in LDS, nine shifted views, no patch matrix; 224-pixel tiles on 16 x 16 x 32 matrix instructions when the
    channel count is a multiple of 32 -- an odd and an even number of 32-channel steps, 1 to 14 rows per tile -- and
    448-pixel tiles otherwise): against the oracle, bf16 and f32 results, first / last rows and
    columns (the zero border) included; the f32 result is also checked against the f64 convolution."""
    dev, pool = hip
    n, c, h, w, co = shape
    r = oracle.Rng(n * 1000 + c + w)
    x, wt = oracle.f32_to_bf16(r.randn((n, c, h, w))), oracle.f32_to_bf16(r.randn((co, c, 3, 3), 0.1))
    b = oracle.f32_to_bf16(r.randn(co, 0.1)) if bias else None
    mag = oracle.conv2d(np.abs(oracle.bf16_to_f32(x)), np.abs(oracle.bf16_to_f32(wt)), None if b is None else np.abs(oracle.bf16_to_f32(b)), (1, 1), (1, 1))
    got32 = conv2d(dev, pool, x, wt, b, (1, 1), (1, 1), (1, 1), relu=relu, dtype=DType.BF16, out_dtype=DType.F32)
    want32 = oracle.conv2d(x, wt, b, (1, 1), (1, 1), (1, 1), relu, oracle.BF16, oracle.F32)
    assert np.all(np.abs(got32 - want32) <= 1e-3 * np.abs(want32) + 2e-5 * mag)
    got = conv2d(dev, pool, x, wt, b, (1, 1), (1, 1), (1, 1), relu=relu, dtype=DType.BF16)
    want = oracle.conv2d(x, wt, b, (1, 1), (1, 1), (1, 1), relu, oracle.BF16)
    g, wv = oracle.bf16_to_f32(got), oracle.bf16_to_f32(want)
    assert np.all(np.abs(g - wv) <= 2.0 ** -7 * np.abs(wv) + 1e-3 * mag)
    # borders: a ones image with ones weights counts the taps inside the image
    ones_x, ones_w = oracle.f32_to_bf16(np.ones((1, c, h, w), np.float32)), oracle.f32_to_bf16(np.ones((co, c, 3, 3), np.float32))
    cnt = conv2d(dev, pool, ones_x, ones_w, None, (1, 1), (1, 1), (1, 1), dtype=DType.BF16, out_dtype=DType.F32)
    taps = np.full((h, w), 9.0)
    taps[0, :] = taps[-1, :] = 6
    taps[:, 0] = taps[:, -1] = 6
    taps[0, 0] = taps[0, -1] = taps[-1, 0] = taps[-1, -1] = 4
    assert np.array_equal(cnt[0, 0], taps * c) and np.array_equal(cnt[0, -1], taps * c)


@pytest.mark.parametrize("shape", [(2, 16, 16, 56, 128), (1, 64, 56, 56, 128), (3, 32, 28, 16, 256), (2, 48, 8, 112, 128), (1, 16, 56, 8, 128)])
@pytest.mark.parametrize("bias,relu", [(True, True), (False, False)])
def test_conv3x3_direct_f32(hip, oracle, shape, bias, relu):
    """The same direct kernel on f32 data (v_mfma_f32_32x32x2_f32): 2e-5 of the magnitude sum against the oracle (the
    order of the k sum differs), zero borders by tap counting, and linearity in the input."""
    dev, pool = hip
    n, c, h, w, co = shape
    r = oracle.Rng(n * 2000 + c + w)
    x, wt = r.randn((n, c, h, w)), r.randn((co, c, 3, 3), 0.1)
    b = r.randn(co, 0.1) if bias else None
    args = ((1, 1), (1, 1), (1, 1))
    mag = oracle.conv2d(np.abs(x), np.abs(wt), None if b is None else np.abs(b), *args)
    got = conv2d(dev, pool, x, wt, b, *args, relu=relu)
    want = oracle.conv2d(x, wt, b, *args, relu)
    assert got.dtype == np.float32 and np.all(np.abs(got - want) <= 2e-5 * mag + 1e-30), np.max(np.abs(got - want) / (mag + 1e-30))
    cnt = conv2d(dev, pool, np.ones((1, c, h, w), np.float32), np.ones((co, c, 3, 3), np.float32), None, *args)
    taps = np.full((h, w), 9.0)
    taps[0, :] = taps[-1, :] = 6
    taps[:, 0] = taps[:, -1] = 6
    taps[0, 0] = taps[0, -1] = taps[-1, 0] = taps[-1, -1] = 4
    assert np.array_equal(cnt[0, 0], taps * c) and np.array_equal(cnt[0, -1], taps * c)
    if not relu and b is None:
        x2 = r.randn((n, c, h, w))
        both = conv2d(dev, pool, x + x2, wt, None, *args)
        assert np.allclose(both, got + conv2d(dev, pool, x2, wt, None, *args), rtol=1e-4, atol=2e-4)


@pytest.mark.parametrize("shape", [(2, 16, 16, 56, 128), (2, 64, 56, 56, 128), (3, 32, 28, 16, 256), (2, 48, 8, 112, 128)])
@pytest.mark.parametrize("dtype", ["f32", "bf16", "bf16->f32"])
def test_conv3x3_fused_max_pool(hip, oracle, shape, dtype):
    """conv + bias + ReLU + 2 x 2 max-pool in one launch (only the pooled tensor is written) equals the two-launch
    result bit for bit, and the oracle's pooled convolution within the convolution's tolerance; without ReLU negative
    maxima survive. A shape whose tiles hold an odd number of rows is refused."""
    dev, pool = hip
    n, c, h, w, co = shape
    r = oracle.Rng(n * 3000 + c + w)
    x, wt, b = r.randn((n, c, h, w)), r.randn((co, c, 3, 3), 0.1), r.randn(co, 0.1)
    dt = DType.F32 if dtype == "f32" else DType.BF16
    odt = DType.BF16 if dtype == "bf16" else DType.F32
    if dt == DType.BF16:
        x, wt, b = oracle.f32_to_bf16(x), oracle.f32_to_bf16(wt), oracle.f32_to_bf16(b)
    args = ((1, 1), (1, 1), (1, 1))
    for relu in (True, False):
        y, pooled = conv2d(dev, pool, x, wt, b, *args, relu=relu, dtype=dt, out_dtype=odt, pool_kernel=(2, 2))
        fused = conv2d(dev, pool, x, wt, b, *args, relu=relu, dtype=dt, out_dtype=odt, fused_pool=True)
        assert fused.shape == (n, co, h // 2, w // 2) and fused.dtype == pooled.dtype
        assert np.array_equal(fused, pooled)
        ref = y.reshape(n, co, h // 2, 2, w // 2, 2)
        ref = oracle.bf16_to_f32(ref) if odt == DType.BF16 else ref
        got = oracle.bf16_to_f32(fused) if odt == DType.BF16 else fused
        assert np.array_equal(got, ref.max(axis=(3, 5)))
        if not relu:
            assert (got < 0).any()
    if dtype == "f32" and shape == (2, 16, 16, 56, 128):
        xf = oracle.Rng(1).randn((1, 16, 4, 56))
        with pytest.raises(Exception):  # 448 / 56 = 8 rows per tile, H = 4 is not a multiple
            conv2d(dev, pool, xf, wt, b, *args, relu=True, fused_pool=True)
        xf = oracle.Rng(1).randn((1, 16, 8, 56))
        want = oracle.max_pool2d(oracle.conv2d(xf, wt, b, *args, True), (2, 2), (2, 2), (0, 0), (1, 1))
        mag = oracle.max_pool2d(oracle.conv2d(np.abs(xf), np.abs(wt), np.abs(b), *args), (2, 2), (2, 2), (0, 0), (1, 1))
        got = conv2d(dev, pool, xf, wt, b, *args, relu=True, fused_pool=True)
        assert np.all(np.abs(got - want) <= 2e-5 * mag)
        with pytest.raises(Exception):  # W = 448: one row per tile
            conv2d(dev, pool, np.zeros((1, 16, 2, 448), np.float32), wt, b, *args, fused_pool=True)


def test_relaid_weights_follow_every_write_of_the_weight_buffer(hip, oracle):
    """The direct 3 x 3 kernel keeps a re-laid copy of its weights in the program's scratch and makes it again only when
    the weight buffer has been written since (host upload, device copy, another launch's output) or another buffer is
    passed: launches with unchanged weights give the same bits, every change of the weights shows in the next launch,
    whichever way it was made, inside a plan too."""
    from zyx_amd import kernels as K
    dev, pool = hip
    r = oracle.Rng(7)
    n, c, hw, co = 1, 64, 56, 128
    x = r.randn((n, c, hw, hw))
    w1, w2 = r.randn((co, c, 3, 3), 0.05), r.randn((co, c, 3, 3), 0.05)
    prog = dev.register_kernel(K.conv2d_desc(n, c, hw, hw, co, 3, 3, (1, 1), (1, 1), (1, 1), False, False, DType.F32))
    xb, e0 = K.to_device(pool, x)
    wa, e1 = K.to_device(pool, w1)
    wb, e2 = K.to_device(pool, w2)
    yb, e3 = K.alloc_like(pool, n * co * hw * hw, 4)
    pool.sync_events([e0, e1, e2, e3])

    def run(wbuf):
        ev = dev.launch(prog, pool, [xb, wbuf, yb], [])
        return K.to_host(pool, yb, (n, co, hw, hw), np.float32, [ev])

    y1 = run(wa)
    assert np.array_equal(run(wa), y1)                       # copy kept
    y2 = run(wb)                                             # another buffer
    assert not np.array_equal(y2, y1) and np.array_equal(run(wb), y2)
    assert np.array_equal(run(wa), y1)                       # and back
    pool.sync_events([pool.host_to_pool(np.ascontiguousarray(w2, np.float32), wa, [])])
    assert np.array_equal(run(wa), y2)                       # same buffer, new contents from the host
    pool.sync_events([pool.host_to_pool(np.ascontiguousarray(w1, np.float32), wb, [])])
    pool.sync_events([pool.copy_range(wb, 0, wa, 0, w1.size * 4, [])])
    assert np.array_equal(run(wa), y1)                       # new contents by a device copy
    plan = dev.create_plan([(prog, [xb, wb, yb])])           # a plan re-lays from its own weights every time
    pool.sync_events([dev.launch_plan(plan, [])])
    assert np.array_equal(K.to_host(pool, yb, (n, co, hw, hw), np.float32), y1)   # wb holds w1 now
    assert np.array_equal(run(wa), y1)
    pool.sync_events([pool.host_to_pool(np.ascontiguousarray(w2, np.float32), wb, [])])
    pool.sync_events([dev.launch_plan(plan, [])])
    assert np.array_equal(K.to_host(pool, yb, (n, co, hw, hw), np.float32), y2)
    assert np.array_equal(run(wa), y1)                       # the plan's re-layout does not pass for wa's
    want = oracle.conv2d(x, w1, None, (1, 1), (1, 1), (1, 1))
    mag = oracle.conv2d(np.abs(x), np.abs(w1), None, (1, 1), (1, 1), (1, 1))
    assert np.all(np.abs(y1 - want) <= 2e-5 * mag)
    dev.destroy_plan(plan)
    dev.release(prog)
    for b_ in (xb, wa, wb, yb):
        pool.deallocate(b_, [])
