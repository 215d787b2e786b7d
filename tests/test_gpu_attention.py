"""Attention core on the GPU against the oracle (zyx-nn/src/causal_self_attention.rs:36-74 restated) and the
reference's goldens (zyx/tests/05_misc.rs:1073-1163, zyx-nn/src/causal_self_attention.rs:78-158).

Tolerances: f32 storage 1e-5 relative to max(|y|, sum_j p_j |v_j|) =: mag. bf16 storage: 1e-3 * mag (north star
for f32-accumulated bf16 matrix products) + 2^-9 * mag (the probabilities enter att.dot(v) as bf16 values, as the
reference's bf16 `att` tensor does; round-to-nearest moves each by at most half a bf16 ulp, which is 2^-8 relative in
the worst case and averages below 2^-9 over rows of many comparable terms: the test whose rows are carried by a few
keys uses 2^-8) + 2^-7 * |y| (the truncating bf16 store of y)."""
import numpy as np
import pytest

from zyx_amd import DType
from zyx_amd.kernels import attention

pytestmark = pytest.mark.gpu


def sdpa64(qkv, n_head, scale=None, p=0.0, causal=False):
    b, t, c3 = qkv.shape
    dh = c3 // 3 // n_head
    q, k, v = [a.reshape(b, t, n_head, dh).transpose(0, 2, 1, 3) for a in np.split(qkv.astype(np.float64), 3, axis=2)]
    s = np.einsum("bhtd,bhjd->bhtj", q, k) * float(np.float32(1 / np.sqrt(dh)) if scale is None else scale)
    if causal:
        s = np.where(np.tril(np.ones((t, t), bool)), s, -np.inf)  # masked_fill(-inf) above the diagonal
    m = s.max(-1, keepdims=True)
    e = np.exp(s - m)
    pr = e / e.sum(-1, keepdims=True) / (1.0 - p)
    y = np.einsum("bhtj,bhjd->bhtd", pr, v).transpose(0, 2, 1, 3).reshape(b, t, c3 // 3)
    mag = np.einsum("bhtj,bhjd->bhtd", pr, np.abs(v)).transpose(0, 2, 1, 3).reshape(b, t, c3 // 3)
    return y, mag, (m + np.log(e.sum(-1, keepdims=True)))[..., 0]


def test_reference_goldens_f32(hip, oracle):
    dev, pool = hip
    w = np.array([[3, 1, 2, 3, 1, 2, 5, 4, 2, 3, 1, 3], [1, 1, 2, 3, 1, 2, 5, 4, 2, 3, 1, 3],
                  [3, 1, 5, 3, 1, 2, 5, 4, 2, 3, 1, 3], [3, 1, 2, 3, 1, 2, 5, 8, 2, 3, 1, 3]], np.float32).T
    x = np.array([[[1, 0, 4, 2], [2, 5, 0, 1], [0, 8, 1, 0], [5, 1, 0, 0]]], np.float32)
    y = attention(dev, pool, oracle.linear(x, w), 4, DType.F32)
    assert np.allclose(y, np.tile(np.array([18, 27, 9, 24], np.float32), (1, 4, 1)), rtol=1e-5)


@pytest.mark.parametrize("shape", [(1, 3, 2, 2), (2, 7, 3, 5), (1, 64, 1, 64), (2, 65, 2, 80), (1, 200, 2, 130), (3, 129, 4, 16)])
@pytest.mark.parametrize("p", [0.0, 0.25])
def test_small_kernel_f32(hip, oracle, shape, p):
    dev, pool = hip
    b, t, h, dh = shape
    qkv = oracle.Rng(t + dh).randn((b, t, 3 * h * dh))
    y, lse = attention(dev, pool, qkv, h, DType.F32, dropout_p=p, want_lse=True)
    want, mag, lse64 = sdpa64(qkv, h, p=p)
    assert np.all(np.abs(y - want) <= 1e-5 * np.maximum(np.abs(want), mag) + 1e-7)
    assert np.allclose(lse, lse64, rtol=1e-5, atol=1e-5)
    ref, ref_lse = oracle.attention(qkv, h, dropout_p=p, want_lse=True)  # the reference's serial f32 order
    assert np.all(np.abs(y - ref) <= 2e-5 * np.maximum(np.abs(want), mag) + 1e-7)


def bf16_close(oracle, got_bits, want, mag):
    got = oracle.bf16_to_f32(got_bits).astype(np.float64)
    return np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + (1e-3 + 2.0 ** -9) * mag


@pytest.mark.parametrize("shape", [(1, 128, 1, 64), (2, 256, 3, 64), (1, 1024, 2, 64), (8, 128, 8, 64)])
def test_mfma_kernel_bf16(hip, oracle, shape):
    dev, pool = hip
    b, t, h, dh = shape
    qkv = oracle.f32_to_bf16(oracle.Rng(t + b).randn((b, t, 3 * h * dh)))
    y, lse = attention(dev, pool, qkv, h, DType.BF16, want_lse=True)
    want, mag, lse64 = sdpa64(oracle.bf16_to_f32(qkv), h)
    assert np.all(bf16_close(oracle, y, want, mag))
    assert np.allclose(lse, lse64, rtol=1e-4, atol=1e-4)
    ref = oracle.bf16_to_f32(oracle.attention(qkv, h, dtype=oracle.BF16)).astype(np.float64)  # serial f32, truncating store
    assert np.all(np.abs(oracle.bf16_to_f32(y) - ref) <= 2.0 ** -6 * np.abs(want) + (1e-3 + 2.0 ** -9) * mag)


def test_bf16_ragged_shapes_take_the_general_kernel(hip, oracle):
    dev, pool = hip
    for b, t, h, dh in [(2, 100, 2, 64), (1, 128, 2, 32)]:
        qkv = oracle.f32_to_bf16(oracle.Rng(t).randn((b, t, 3 * h * dh)))
        y = attention(dev, pool, qkv, h, DType.BF16, dropout_p=0.1)
        want, mag, _ = sdpa64(oracle.bf16_to_f32(qkv), h, p=float(np.float32(1) - (np.float32(1) - np.float32(0.1))))
        assert np.all(bf16_close(oracle, y, want, mag))


def test_structured_inputs_bf16(hip, oracle):
    """Cases with closed forms: identical keys give the mean of V; one dominant key selects its V row."""
    dev, pool = hip
    b, t, h, dh = 1, 256, 2, 64
    rng = np.random.default_rng(3)
    q = rng.standard_normal((b, t, h * dh)).astype(np.float32)
    k = np.tile(rng.standard_normal((b, 1, h * dh)).astype(np.float32), (1, t, 1))
    v = rng.integers(-8, 9, size=(b, t, h * dh)).astype(np.float32)
    y = oracle.bf16_to_f32(attention(dev, pool, oracle.f32_to_bf16(np.concatenate([q, k, v], 2)), h))
    assert np.allclose(y, np.broadcast_to(v.mean(1, keepdims=True), v.shape), rtol=2.0 ** -7, atol=1e-3)
    k = np.zeros((b, t, h * dh), np.float32)
    k[:, 77, :] = 16.0
    q = np.full((b, t, h * dh), 2.0, np.float32)  # score of key 77: 64*32/8 = 256, others 0
    y = oracle.bf16_to_f32(attention(dev, pool, oracle.f32_to_bf16(np.concatenate([q, k, v], 2)), h))
    assert np.array_equal(y, np.broadcast_to(v[:, 77:78, :], v.shape))


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(1, 512, 2, 64), (8, 256, 64, 64)])  # 32 and 64 queries per wave
def test_scores_that_keep_growing_bf16(hip, oracle, shape, causal):
    """Scores rise by ~37 (in powers of two) from one block of 32 keys to the next, so the reference point of the
    running exponentials has to move several times inside a row, and every probability but the last few underflows."""
    dev, pool = hip
    b, t, h, dh = shape
    rng = np.random.default_rng(t + h)
    q = (1.0 + 0.1 * rng.standard_normal((b, t, h * dh))).astype(np.float32)
    k = np.broadcast_to((0.1 * np.arange(t, dtype=np.float32))[None, :, None], (b, t, h * dh))
    v = rng.standard_normal((b, t, h * dh)).astype(np.float32)
    # packed layout [B, T, 3, H, dh]
    qkv = oracle.f32_to_bf16(np.stack([q.reshape(b, t, h, dh), k.reshape(b, t, h, dh), v.reshape(b, t, h, dh)], 2).reshape(b, t, 3 * h * dh))
    y, lse = attention(dev, pool, qkv, h, DType.BF16, want_lse=True, causal=causal)
    want, mag, lse64 = sdpa64(oracle.bf16_to_f32(qkv), h, causal=causal)
    got = oracle.bf16_to_f32(y).astype(np.float64)
    assert np.all(np.isfinite(got)) and np.all(np.isfinite(lse))
    # a handful of keys carry each row here, so the roundings of their probabilities to bf16 do not average out: the
    # bar is the worst case of round-to-nearest on 8 significant bits, 2^-8 * mag, instead of the 2^-9 that rows of
    # many comparable terms are held to
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + (1e-3 + 2.0 ** -8) * mag)
    assert np.allclose(lse, lse64, rtol=1e-4, atol=1e-4)


def test_config5_attention_full_size(hip, oracle):
    """B=8, T=1024, 16 heads x 64, bf16: every element against the C oracle (f32 registers, serial sums) and
    2 heads against the f64 textbook form."""
    dev, pool = hip
    r = oracle.Rng(42069)
    qkv = oracle.f32_to_bf16(r.randn((8, 1024, 3072)))
    y, lse = attention(dev, pool, qkv, 16, want_lse=True)
    ref, ref_lse = oracle.attention(qkv, 16, dtype=oracle.BF16, want_lse=True)
    yf, rf = oracle.bf16_to_f32(y), oracle.bf16_to_f32(ref)
    # mag = sum_j p_j |v_j| stays near E|v| ~ 0.8 for these inputs, so (1e-3 + 2^-9) * mag < 3e-3
    assert np.all(np.abs(yf - rf) <= 2.0 ** -6 * np.abs(rf) + 3e-3)
    assert np.allclose(lse, ref_lse, rtol=1e-4, atol=1e-4)
    sub = np.ascontiguousarray(qkv.reshape(8, 1024, 3, 16, 64)[:1, :, :, :2, :]).reshape(1, 1024, 3 * 128)
    want, mag, _ = sdpa64(oracle.bf16_to_f32(sub), 2)
    got = y.reshape(8, 1024, 16, 64)[:1, :, :2, :].reshape(1, 1024, 128)
    assert np.all(bf16_close(oracle, got, want, mag))


# ---- backward ---------------------------------------------------------------------------------------------------
from zyx_amd.kernels import attention_bwd


def grad64(qkv, dy, n_head, p=0.0, causal=False, with_ymag=False):
    """Textbook gradient in f64 (numpy), with the magnitude sums the tolerances are relative to. with_ymag also
    returns how far one unit of relative error in every stored y element moves dq and dk: the backward reads y as
    the forward stored it (D = rowsum(dy o y)), so a bf16 y brings 2^-7 of sum_d |dy_d y_d| into every dS of its row."""
    b, t, c3 = qkv.shape
    dh = c3 // 3 // n_head
    sc = float(np.float32(1 / np.sqrt(dh)))
    q, k, v = [a.reshape(b, t, n_head, dh).transpose(0, 2, 1, 3) for a in np.split(qkv.astype(np.float64), 3, axis=2)]
    do = dy.astype(np.float64).reshape(b, t, n_head, dh).transpose(0, 2, 1, 3)
    s = np.einsum("bhtd,bhjd->bhtj", q, k) * sc
    if causal:
        s = np.where(np.tril(np.ones((t, t), bool)), s, -np.inf)
    e = np.exp(s - s.max(-1, keepdims=True))
    ps = e / e.sum(-1, keepdims=True)
    dps = np.einsum("bhtd,bhjd->bhtj", do, v) / (1 - p)
    ds = ps * (dps - (ps * dps).sum(-1, keepdims=True))
    ads = ps * (np.abs(dps) + (ps * np.abs(dps)).sum(-1, keepdims=True))
    back = lambda a: a.transpose(0, 2, 1, 3).reshape(b, t, n_head * dh)
    g = np.concatenate([back(np.einsum("bhtj,bhjd->bhtd", ds, k) * sc), back(np.einsum("bhtj,bhtd->bhjd", ds, q) * sc),
                        back(np.einsum("bhtj,bhtd->bhjd", ps, do) / (1 - p))], 2)
    mag = np.concatenate([back(np.einsum("bhtj,bhjd->bhtd", ads, np.abs(k)) * sc), back(np.einsum("bhtj,bhtd->bhjd", ads, np.abs(q)) * sc),
                          back(np.einsum("bhtj,bhtd->bhjd", ps, np.abs(do)) / (1 - p))], 2)
    if with_ymag:
        y = np.einsum("bhtj,bhjd->bhtd", ps, v) / (1 - p)
        ey = ps * (np.abs(do) * np.abs(y)).sum(-1, keepdims=True)
        zeros = np.zeros((b, t, n_head * dh))
        ymag = np.concatenate([back(np.einsum("bhtj,bhjd->bhtd", ey, np.abs(k)) * sc), back(np.einsum("bhtj,bhtd->bhjd", ey, np.abs(q)) * sc), zeros], 2)
        return g, mag, ymag
    return g, mag


@pytest.mark.parametrize("shape", [(1, 3, 2, 2), (2, 7, 3, 5), (2, 65, 2, 80), (1, 130, 2, 130)])
@pytest.mark.parametrize("p", [0.0, 0.25])
def test_backward_small_kernel_f32(hip, oracle, shape, p):
    dev, pool = hip
    b, t, h, dh = shape
    qkv = oracle.Rng(t + dh).randn((b, t, 3 * h * dh))
    dy = oracle.Rng(t).randn((b, t, h * dh))
    y, lse = attention(dev, pool, qkv, h, DType.F32, dropout_p=p, want_lse=True)
    got = attention_bwd(dev, pool, qkv, y, dy, lse, h, DType.F32, dropout_p=p)
    keep = float(np.float32(1) - np.float32(p))
    want, mag = grad64(qkv, dy, h, 1 - keep)
    assert np.all(np.abs(got - want) <= 2e-5 * mag + 1e-7)
    assert np.all(np.abs(got - oracle.attention_bwd(qkv, dy, h, dropout_p=p)) <= 2e-5 * mag + 1e-7)


@pytest.mark.parametrize("shape", [(1, 128, 1, 64), (2, 256, 3, 64), (1, 512, 8, 64)])
def test_backward_mfma_kernel_bf16(hip, oracle, shape):
    """bf16 operands (P, dS, dy, q, k, v are bf16 matrix-core operands): 1e-3 of the magnitude sum for the f32
    accumulation, 2^-8 of it for operand rounding of P / dS, one bf16 ulp for the truncating store."""
    dev, pool = hip
    b, t, h, dh = shape
    qkv = oracle.f32_to_bf16(oracle.Rng(t + b).randn((b, t, 3 * h * dh)))
    dy = oracle.f32_to_bf16(oracle.Rng(t).randn((b, t, h * dh)))
    y, lse = attention(dev, pool, qkv, h, DType.BF16, want_lse=True)
    got = oracle.bf16_to_f32(attention_bwd(dev, pool, qkv, y, dy, lse, h, DType.BF16)).astype(np.float64)
    want, mag = grad64(oracle.bf16_to_f32(qkv), oracle.bf16_to_f32(dy), h)
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + (1e-3 + 2.0 ** -8) * mag)
    # the same through the general kernel (a shape the matrix-core path does not take) agrees as well
    if t == 128:
        y2, lse2 = attention(dev, pool, qkv[:, :100], h, DType.BF16, want_lse=True)
        got2 = oracle.bf16_to_f32(attention_bwd(dev, pool, qkv[:, :100], y2, dy[:, :100], lse2, h, DType.BF16)).astype(np.float64)
        want2, mag2 = grad64(oracle.bf16_to_f32(qkv[:, :100]), oracle.bf16_to_f32(dy[:, :100]), h)
        assert np.all(np.abs(got2 - want2) <= 2.0 ** -7 * np.abs(want2) + 2e-3 * mag2)


def test_config5_attention_backward_full_size(hip, oracle):
    """B=8, T=1024, 16 x 64 bf16: two (batch, head) pairs against the f64 gradient; all of it through
    d/dv linearity: sum_t dV[t] equals sum over queries of P^T dy, i.e. column sums of dV per head equal
    column sums of dy per head (rows of P sum to one)."""
    dev, pool = hip
    qkv = oracle.f32_to_bf16(oracle.Rng(42069).randn((8, 1024, 3072)))
    dy = oracle.f32_to_bf16(oracle.Rng(7).randn((8, 1024, 1024)))
    y, lse = attention(dev, pool, qkv, 16, want_lse=True)
    got = oracle.bf16_to_f32(attention_bwd(dev, pool, qkv, y, dy, lse, 16))
    dv_sum = got[:, :, 2048:].astype(np.float64).sum(1)
    dy_sum = oracle.bf16_to_f32(dy).astype(np.float64).sum(1)
    assert np.all(np.abs(dv_sum - dy_sum) <= 2.0 ** -7 * np.abs(oracle.bf16_to_f32(dy)).astype(np.float64).sum(1))
    for bsel, hsel in [(0, 0), (7, 15)]:
        cols = np.concatenate([np.arange(64) + 1024 * i + 64 * hsel for i in range(3)])
        sub, dsub = qkv[bsel:bsel + 1][:, :, cols], dy[bsel:bsel + 1, :, 64 * hsel:64 * hsel + 64]
        want, mag = grad64(oracle.bf16_to_f32(sub), oracle.bf16_to_f32(dsub), 1)
        g = got[bsel:bsel + 1][:, :, cols].astype(np.float64)
        assert np.all(np.abs(g - want) <= 2.0 ** -7 * np.abs(want) + (1e-3 + 2.0 ** -8) * mag)


# ---- causal mask --------------------------------------------------------------------------------------------------
# The reference's module applies no mask (zyx-nn/src/causal_self_attention.rs:57-62); the flag is checked against the
# textbook masked softmax in f64 and against the oracle's serial loops over the keys 0..t.

@pytest.mark.parametrize("shape", [(1, 3, 2, 2), (2, 7, 3, 5), (1, 64, 1, 64), (2, 65, 2, 80), (1, 200, 2, 130), (3, 129, 4, 16)])
@pytest.mark.parametrize("p", [0.0, 0.25])
def test_causal_small_kernel_f32(hip, oracle, shape, p):
    dev, pool = hip
    b, t, h, dh = shape
    qkv = oracle.Rng(t + dh).randn((b, t, 3 * h * dh))
    y, lse = attention(dev, pool, qkv, h, DType.F32, dropout_p=p, want_lse=True, causal=True)
    want, mag, lse64 = sdpa64(qkv, h, p=p, causal=True)
    assert np.all(np.abs(y - want) <= 1e-5 * np.maximum(np.abs(want), mag) + 1e-7)
    assert np.allclose(lse, lse64, rtol=1e-5, atol=1e-5)
    ref = oracle.attention(qkv, h, dropout_p=p, causal=True)
    assert np.all(np.abs(y - ref) <= 2e-5 * np.maximum(np.abs(want), mag) + 1e-7)
    # the first query sees one key: its row is v_0 / keep exactly
    v0 = qkv[:, 0, 2 * h * dh:]
    assert np.allclose(y[:, 0], v0 / (np.float32(1) - np.float32(p)), rtol=1e-6, atol=0)
    dy = oracle.Rng(t).randn((b, t, h * dh))
    got = attention_bwd(dev, pool, qkv, y, dy, lse, h, DType.F32, dropout_p=p, causal=True)
    keep = float(np.float32(1) - np.float32(p))
    gwant, gmag = grad64(qkv, dy, h, 1 - keep, causal=True)
    assert np.all(np.abs(got - gwant) <= 2e-5 * gmag + 1e-7)
    assert np.all(np.abs(got - oracle.attention_bwd(qkv, dy, h, dropout_p=p, causal=True)) <= 2e-5 * gmag + 1e-7)


@pytest.mark.parametrize("shape", [(1, 128, 1, 64), (2, 256, 3, 64), (1, 1024, 2, 64), (8, 384, 8, 64)])
def test_causal_mfma_kernels_bf16(hip, oracle, shape):
    dev, pool = hip
    b, t, h, dh = shape
    qkv = oracle.f32_to_bf16(oracle.Rng(t + b).randn((b, t, 3 * h * dh)))
    dy = oracle.f32_to_bf16(oracle.Rng(t).randn((b, t, h * dh)))
    y, lse = attention(dev, pool, qkv, h, DType.BF16, want_lse=True, causal=True)
    want, mag, lse64 = sdpa64(oracle.bf16_to_f32(qkv), h, causal=True)
    assert np.all(bf16_close(oracle, y, want, mag))
    assert np.allclose(lse, lse64, rtol=1e-4, atol=1e-4)
    assert np.array_equal(y[:, 0], qkv[:, 0, 2 * h * dh:])         # one visible key: y_0 = v_0, bit for bit
    y_nolse = attention(dev, pool, qkv, h, DType.BF16, causal=True)
    assert np.array_equal(y_nolse, y)
    got = oracle.bf16_to_f32(attention_bwd(dev, pool, qkv, y, dy, lse, h, DType.BF16, causal=True)).astype(np.float64)
    # early queries see few keys: their y is as large as v, and its truncating bf16 store is felt in D = rowsum(dy o y)
    gwant, gmag, ymag = grad64(oracle.bf16_to_f32(qkv), oracle.bf16_to_f32(dy), h, causal=True, with_ymag=True)
    assert np.all(np.abs(got - gwant) <= 2.0 ** -7 * np.abs(gwant) + (1e-3 + 2.0 ** -8) * gmag + 2.0 ** -7 * ymag)
    if t <= 256:
        ref = oracle.bf16_to_f32(oracle.attention(qkv, h, dtype=oracle.BF16, causal=True)).astype(np.float64)
        assert np.all(np.abs(oracle.bf16_to_f32(y) - ref) <= 2.0 ** -6 * np.abs(want) + (1e-3 + 2.0 ** -9) * mag)
