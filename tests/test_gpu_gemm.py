"""bf16 MFMA GEMM vs the CPU oracle. Tolerance: 1e-3 relative to the f32-accumulated result
(north star), measured against sum_k |a_k b_k| so cancelling sums do not inflate it; the
f64-accumulated oracle anchors both."""
import numpy as np
import pytest

from zyx_amd import DType
from zyx_amd.kernels import gemm

pytestmark = pytest.mark.gpu


def make(oracle, m, n, k, seed, trans_a=False, trans_b=False):
    r = oracle.Rng(seed)
    a = oracle.f32_to_bf16(r.uniform((k, m) if trans_a else (m, k), -1, 1))
    b = oracle.f32_to_bf16(r.uniform((n, k) if trans_b else (k, n), -1, 1))
    return a, b


def reference(oracle, a, b, trans_a, trans_b):
    af, bf = oracle.bf16_to_f32(a).astype(np.float64), oracle.bf16_to_f32(b).astype(np.float64)
    af = af.T if trans_a else af
    bf = bf.T if trans_b else bf
    return af @ bf, np.abs(af) @ np.abs(bf)


@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", [(256, 256, 64), (256, 512, 128), (512, 256, 576), (1024, 2048, 512), (256, 384, 256), (3072, 4096, 256)])
def test_bf16_gemm_layouts(hip, oracle, mnk, trans_a, trans_b):
    dev, pool = hip
    m, n, k = mnk
    a, b = make(oracle, m, n, k, m + n + k, trans_a, trans_b)
    got = gemm(dev, pool, a, b, trans_a=trans_a, trans_b=trans_b)
    want, mag = reference(oracle, a, b, trans_a, trans_b)
    assert np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-5 * mag), np.max(np.abs(got - want) / (mag + 1e-30))
    # the same product in the reference's serial f32 order is no closer to the exact value
    if m * n * k <= 256 * 512 * 128 and not trans_a:
        ser = oracle.matmul(a, b, oracle.BF16, oracle.F32, transb=trans_b)
        assert np.all(np.abs(got - ser) <= 1e-3 * np.abs(want) + 2e-5 * mag)


def test_identity_and_exactness(hip, oracle):
    """Small integers are exact in bf16 and in f32 sums: the product must be bit-exact."""
    dev, pool = hip
    rng = np.random.default_rng(0)
    a = rng.integers(-4, 5, size=(256, 128)).astype(np.float32)
    b = rng.integers(-4, 5, size=(128, 256)).astype(np.float32)
    got = gemm(dev, pool, oracle.f32_to_bf16(a), oracle.f32_to_bf16(b))
    assert np.array_equal(got, a @ b)
    eye = np.eye(256, dtype=np.float32)
    x = oracle.f32_to_bf16(oracle.Rng(1).randn((256, 256)))
    assert np.array_equal(gemm(dev, pool, x, oracle.f32_to_bf16(eye)), oracle.bf16_to_f32(x))
    assert np.array_equal(gemm(dev, pool, oracle.f32_to_bf16(eye), x), oracle.bf16_to_f32(x))


def test_config3_full_size(hip, oracle):
    """Benchmark configuration 3: A, B uniform(-1,1) truncated to bf16, 4096^3, f32 out. The full
    oracle product takes minutes on the CPU, so 64 rows x 4096 columns are checked against
    the f64-accumulated oracle and the rest through linearity: C . v == A . (B . v)."""
    dev, pool = hip
    a, b = make(oracle, 4096, 4096, 4096, 42069)
    got = gemm(dev, pool, a, b)
    rows = np.arange(0, 4096, 64)
    af, bf = oracle.bf16_to_f32(a).astype(np.float64), oracle.bf16_to_f32(b).astype(np.float64)
    want = af[rows] @ bf
    mag = np.abs(af[rows]) @ np.abs(bf)
    assert np.all(np.abs(got[rows] - want) <= 1e-3 * np.abs(want) + 1e-5 * mag)
    v = np.random.default_rng(1).standard_normal(4096)
    lhs, rhs = got.astype(np.float64) @ v, af @ (bf @ v)
    assert np.all(np.abs(lhs - rhs) <= 1e-4 * (np.abs(af) @ (np.abs(bf) @ np.abs(v))))


def test_config3_full_size_bias_gelu(hip, oracle):
    """Benchmark configuration 3 with its epilogue, gelu(A.B + bias) at 4096^3: the pre-activations have a standard
    deviation of ~21, so most outputs lie where the reference's tanh = (e^2z - 1) / (e^2z + 1) has overflowed
    (z > ~44, i.e. x > ~10: inf / inf, unspecified under its -ffast-math) or underflowed. The kernel saturates there
    (gelu(x) -> x, resp. -> 0); everywhere it must be finite and match the formula of
    zyx/src/tensor/elementwise.rs:168-170 evaluated in f64 on the f64-accumulated product of sampled rows."""
    dev, pool = hip
    a, b = make(oracle, 4096, 4096, 4096, 42069)
    bias = oracle.f32_to_bf16(oracle.Rng(7).uniform(4096, -1 / 64, 1 / 64))
    got = gemm(dev, pool, a, b, bias, epilogue="bias_gelu", bias_dtype=DType.BF16)
    assert np.all(np.isfinite(got))
    rows = np.arange(5, 4096, 64)
    af, bf = oracle.bf16_to_f32(a).astype(np.float64), oracle.bf16_to_f32(b).astype(np.float64)
    pre = af[rows] @ bf + oracle.bf16_to_f32(bias).astype(np.float64)[None, :]
    mag = np.abs(af[rows]) @ np.abs(bf)
    want = 0.5 * pre * (1 + np.tanh(np.sqrt(2 / np.pi) * (pre + 0.044715 * pre ** 3)))
    # |gelu'| <= 1.13: the product's summation-order error (1e-5 of sum |a b|) passes through at most that much
    assert np.all(np.abs(got[rows] - want) <= 1e-3 * np.abs(want) + 2e-5 * mag + 1e-6)
    hi, lo = pre > 10, pre < -10
    assert hi.sum() > 1000 and lo.sum() > 1000  # the sample does reach both saturated regions
    assert np.all(np.abs(got[rows][hi] - pre[hi]) <= 2e-5 * mag[hi] + 1e-3 * np.abs(pre[hi]))
    assert np.all(np.abs(got[rows][lo]) <= 1e-6)


# ---- general kernel: f32, ragged shapes, narrow outputs, batches -------------------------------------

def test_reference_matmul_goldens(hip):
    # zyx/tests/05_misc.rs:201-208 (matmul_2) on f32 registers, and 09_graph.rs:43-51
    dev, pool = hip
    x = np.array([[2, 4, 3], [1, 5, 1]], np.float32)
    y = np.array([[2, 4], [3, 1], [5, 1]], np.float32)
    assert gemm(dev, pool, x, y, dtype=DType.F32).tolist() == [[31, 15], [22, 10]]


@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", [(1, 1, 1), (64, 128, 784), (64, 10, 128), (128, 784, 64), (10, 128, 64), (56, 5, 12),
                                 (315, 76, 243), (574, 97, 705), (1024, 1024, 1024)])
def test_f32_gemm_any_shape(hip, oracle, mnk, trans_a, trans_b):
    """f32: relative 1e-5 against the f64-accumulated product (measured against sum |a b|, the
    scale rounding errors of any summation order are proportional to); sizes include the
    reference's matmul_1 sweep corners (05_misc.rs:210-237) and the config-1 MLP products."""
    dev, pool = hip
    m, n, k = mnk
    r = oracle.Rng(m * 31 + n * 7 + k)
    a = r.uniform((k, m) if trans_a else (m, k), -1, 1)
    b = r.uniform((n, k) if trans_b else (k, n), -1, 1)
    got = gemm(dev, pool, a, b, dtype=DType.F32, trans_a=trans_a, trans_b=trans_b)
    ad, bd = a.astype(np.float64), b.astype(np.float64)
    ad, bd = (ad.T if trans_a else ad), (bd.T if trans_b else bd)
    want, mag = ad @ bd, np.abs(ad) @ np.abs(bd)
    assert np.all(np.abs(got - want) <= 1e-5 * mag + 1e-30), np.max(np.abs(got - want) / (mag + 1e-30))
    if m * n * k <= 64 * 128 * 784 and not trans_a:
        ser = oracle.matmul(a, b, oracle.F32, oracle.F32, transb=trans_b)  # the reference's serial order
        assert np.all(np.abs(got - ser) <= 2e-5 * mag + 1e-30)


def test_f32_integer_products_are_exact(hip):
    """Integer-valued f32 operands (the reference's i+j / i-j matrices): every partial sum is
    exact in f32, so any summation order must give the exact integer result."""
    dev, pool = hip
    m, k, n = 315, 243, 76
    x = (np.arange(m)[:, None] + np.arange(k)[None, :]).astype(np.float32) % 16
    y = (np.arange(k)[:, None] - np.arange(n)[None, :]).astype(np.float32) % 8
    assert np.array_equal(gemm(dev, pool, x, y, dtype=DType.F32), x @ y)


@pytest.mark.parametrize("epilogue", ["bias", "bias_relu", "bias_gelu"])
def test_linear_epilogues(hip, oracle, epilogue):
    dev, pool = hip
    r = oracle.Rng(77)
    x, w, b = r.randn((64, 784)), r.uniform((128, 784), -0.05, 0.05), r.uniform(128, -0.05, 0.05)
    got = gemm(dev, pool, x, w, b, dtype=DType.F32, trans_b=True, epilogue=epilogue)  # Linear: x . W^T + b
    lin = oracle.matmul(x, w, oracle.F32, oracle.F32, transb=True)
    want = oracle.bias_act(lin, b, {"bias": "none", "bias_relu": "relu", "bias_gelu": "gelu"}[epilogue])
    mag = np.abs(x) @ np.abs(w.T) + np.abs(b)
    assert np.all(np.abs(got - want) <= 2e-5 * mag)
    # bf16 operands, bf16 bias, big-tile kernel and general kernel give the same epilogue
    xb, wb, bb = oracle.f32_to_bf16(r.randn((256, 128))), oracle.f32_to_bf16(r.uniform((256, 128), -0.1, 0.1)), \
        oracle.f32_to_bf16(r.uniform(256, -1, 1))
    got = gemm(dev, pool, xb, wb, bb, trans_b=True, epilogue=epilogue, bias_dtype=DType.BF16)
    lin = oracle.matmul_f64acc(xb, wb, oracle.BF16, transb=True).astype(np.float32)
    want = oracle.bias_act(lin, bb, {"bias": "none", "bias_relu": "relu", "bias_gelu": "gelu"}[epilogue], oracle.BF16)
    assert np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-4)


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16])
def test_16bit_ragged_and_narrow_store(hip, oracle, dt):
    """`dot` on 16-bit tensors stores the f32 sum truncated to the operand dtype
    (zyx/src/tensor/reduce_ops.rs:134-136, zyx/src/codegen/c.rs:494-496); includes the
    reference's bf16_matmul_1 shape 17x2x19 (zyx/tests/10_bf16.rs:160-198)."""
    dev, pool = hip
    conv = oracle.f32_to_bf16 if dt == DType.BF16 else oracle.f32_to_f16
    back = oracle.bf16_to_f32 if dt == DType.BF16 else oracle.f16_to_f32
    code = oracle.BF16 if dt == DType.BF16 else oracle.F16
    m, k, n = 17, 2, 19
    xf = np.fromfunction(lambda i, j: np.fmod(i + j, 10.0), (m, k)).astype(np.float32)
    yf = np.fromfunction(lambda i, j: np.fmod(i - j, 10.0), (k, n)).astype(np.float32)
    got = gemm(dev, pool, conv(xf), conv(yf), dtype=dt, out_dtype=dt)
    assert np.array_equal(got, oracle.matmul(conv(xf), conv(yf), code, code))  # small ints: exact, then truncated
    r = oracle.Rng(5)
    a, b = conv(r.uniform((100, 333), -1, 1)), conv(r.uniform((333, 77), -1, 1))
    got = back(gemm(dev, pool, a, b, dtype=dt, out_dtype=dt))
    want = oracle.matmul_f64acc(a, b, code)
    assert np.all(np.abs(got - want) <= (2 ** -7 if dt == DType.BF16 else 2 ** -10) * np.abs(want) + 1e-4 * (np.abs(back(a)) @ np.abs(back(b))))


def test_batched_and_scaled(hip, oracle):
    """Batched product with alpha: the q . k^T * scale of attention (zyx-nn/src/causal_self_attention.rs:57-60)."""
    dev, pool = hip
    r = oracle.Rng(9)
    q, k = r.randn((6, 40, 64)), r.randn((6, 50, 64))
    got = gemm(dev, pool, q, k, dtype=DType.F32, trans_b=True, alpha=0.125)
    want = np.einsum("bik,bjk->bij", q.astype(np.float64), k.astype(np.float64)) * 0.125
    assert got.shape == (6, 40, 50)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("mnk", [(256, 512, 128), (100, 70, 50), (256, 256, 1024), (512, 256, 4096)])
@pytest.mark.parametrize("epilogue", ["none", "gelu"])
def test_bf16_output_and_residual(hip, oracle, mnk, epilogue):
    """bf16 C with the truncating store, and the fused residual add (x + Linear(x)): both kernels."""
    dev, pool = hip
    m, n, k = mnk
    a, b = make(oracle, m, n, k, 11, trans_b=True)
    r = oracle.Rng(5)
    bias = oracle.f32_to_bf16(r.uniform((n,), -1, 1))
    res = oracle.f32_to_bf16(r.randn((m, n)))
    kw = dict(bias=bias, epilogue="bias" if epilogue == "none" else "bias_gelu", bias_dtype=DType.BF16, trans_b=True)
    want, mag = reference(oracle, a, b, False, True)
    want = want + oracle.bf16_to_f32(bias).astype(np.float64)
    if epilogue == "gelu":
        want = 0.5 * want * (1 + np.tanh(np.sqrt(2 / np.pi) * (want + 0.044715 * want ** 3)))
    for residual in (None, res):
        w = want + (oracle.bf16_to_f32(res).astype(np.float64) if residual is not None else 0.0)
        got32 = gemm(dev, pool, a, b, out_dtype=DType.F32, residual=None if residual is None else oracle.bf16_to_f32(res), **kw)
        assert np.all(np.abs(got32 - w) <= 1e-3 * np.abs(w) + 2e-5 * mag + 1e-6)
        got16 = gemm(dev, pool, a, b, out_dtype=DType.BF16, residual=residual, **kw)
        # the bf16 result is the truncation of the f32 one (identical arithmetic before the store)
        assert np.array_equal(got16, oracle.f32_to_bf16(got32))


# ---- edge tiles of the big-tile kernel ------------------------------------------------------------------

def _guarded_gemm(dev, pool, a, b, m, n, k, out_dtype, extra=(), **desc_kw):
    """Runs one bf16 product into a result buffer followed by 4096 sentinel elements; returns (C, sentinels)."""
    from zyx_amd.kernels import gemm_desc, to_device, to_host
    prog = dev.register_kernel(gemm_desc(m, n, k, DType.BF16, out_dtype, **desc_kw))
    np_out = np.uint16 if out_dtype == DType.BF16 else np.float32
    bufs, waits = [], []
    for arr in (a, b) + tuple(extra):
        bb, e = to_device(pool, arr)
        bufs.append(bb)
        waits.append(e)
    guard = np.full(m * n + 4096, 0x7fc1 if out_dtype == DType.BF16 else np.float32(-12345.5), np_out)
    cb, e = to_device(pool, guard)
    waits.append(e)
    done = dev.launch(prog, pool, bufs + [cb], waits)
    res = to_host(pool, cb, (m * n + 4096,), np_out, [done])
    for bb in bufs + [cb]:
        pool.deallocate(bb, [])
    dev.release(prog)
    return res[:m * n].reshape(m, n), (res[m * n:], guard[m * n:])


@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", [(264, 136, 64), (64, 64, 128), (200, 328, 192), (1000, 1000, 256), (520, 72, 1024),
                                 (776, 2056, 128), (2048, 50264, 64)])
def test_bf16_edge_tiles(hip, oracle, mnk, trans_a, trans_b):
    """M and N that are not multiples of the tile: the edge tiles' clamped loads must not leak into stored
    elements and their masked stores must not touch anything past row M - 1 or column N - 1 (the last shape
    is a vocabulary projection; (520, 72, 1024) also takes the split-K path)."""
    dev, pool = hip
    m, n, k = mnk
    a, b = make(oracle, m, n, k, m * 3 + n + k, trans_a, trans_b)
    got, (tail, guard) = _guarded_gemm(dev, pool, a, b, m, n, k, DType.F32, trans_a=trans_a, trans_b=trans_b)
    assert np.array_equal(tail, guard)
    want, mag = reference(oracle, a, b, trans_a, trans_b)
    assert np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-5 * mag), np.max(np.abs(got - want) / (mag + 1e-30))


@pytest.mark.parametrize("mnk", [(300, 200, 128), (1000, 72, 64), (72, 1000, 256), (257, 258, 64), (130, 66, 2048)])
@pytest.mark.parametrize("epilogue", ["bias", "bias_relu", "bias_gelu"])
def test_bf16_edge_tiles_linear(hip, oracle, mnk, epilogue):
    """Linear layers of ragged width (x . W^T + b, activation, + residual) with f32 and bf16 results; the bf16
    result must be the truncation of the f32 one, edge tiles included (N here is even, not always a multiple of 8)."""
    dev, pool = hip
    m, n, k = mnk
    a, b = make(oracle, m, n, k, 13, trans_b=True)
    r = oracle.Rng(6)
    bias = oracle.f32_to_bf16(r.uniform((n,), -1, 1))
    res = oracle.f32_to_bf16(r.randn((m, n)))
    want, mag = reference(oracle, a, b, False, True)
    want = want + oracle.bf16_to_f32(bias).astype(np.float64)
    if epilogue == "bias_relu":
        want = np.maximum(want, 0.0)
    if epilogue == "bias_gelu":
        want = 0.5 * want * (1 + np.tanh(np.sqrt(2 / np.pi) * (want + 0.044715 * want ** 3)))
    kw = dict(trans_b=True, epilogue=epilogue, bias_dtype=DType.BF16)
    for residual in (False, True):
        w = want + (oracle.bf16_to_f32(res).astype(np.float64) if residual else 0.0)
        got32, (tail, guard) = _guarded_gemm(dev, pool, a, b, m, n, k, DType.F32,
                                             (bias,) + ((oracle.bf16_to_f32(res),) if residual else ()), residual=residual, **kw)
        assert np.array_equal(tail, guard)
        assert np.all(np.abs(got32 - w) <= 1e-3 * np.abs(w) + 2e-5 * mag + 1e-6)
        got16, (tail, guard) = _guarded_gemm(dev, pool, a, b, m, n, k, DType.BF16, (bias,) + ((res,) if residual else ()),
                                             residual=residual, **kw)
        assert np.array_equal(tail, guard)
        assert np.array_equal(got16, oracle.f32_to_bf16(got32))


@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
def test_bf16_column_blocks(hip, oracle, trans_a, trans_b):
    """4096 x 6144: 384 wide tiles would fill one and a half rounds of the 256 CUs, so the product is launched as two
    blocks of columns (4096 of wide tiles, 2048 of narrow ones) that share A and write one C: every layout, with
    bias + residual, f32 and bf16 results."""
    dev, pool = hip
    m, n, k = 4096, 6144, 64
    a, b = make(oracle, m, n, k, 77, trans_a, trans_b)
    r = oracle.Rng(78)
    bias = oracle.f32_to_bf16(r.uniform((n,), -1, 1))
    res = oracle.f32_to_bf16(r.randn((m, n)))
    want, mag = reference(oracle, a, b, trans_a, trans_b)
    got = gemm(dev, pool, a, b, trans_a=trans_a, trans_b=trans_b)
    assert np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-5 * mag)
    w = want + oracle.bf16_to_f32(bias).astype(np.float64) + oracle.bf16_to_f32(res).astype(np.float64)
    kw = dict(bias=bias, epilogue="bias", bias_dtype=DType.BF16, trans_a=trans_a, trans_b=trans_b)
    got32 = gemm(dev, pool, a, b, out_dtype=DType.F32, residual=oracle.bf16_to_f32(res), **kw)
    assert np.all(np.abs(got32 - w) <= 1e-3 * np.abs(w) + 2e-5 * mag + 1e-6)
    got16 = gemm(dev, pool, a, b, out_dtype=DType.BF16, residual=res, **kw)
    assert np.array_equal(got16, oracle.f32_to_bf16(got32))


@pytest.mark.parametrize("dtype", [DType.F32, DType.BF16])
@pytest.mark.parametrize("mnk", [(64, 128, 10), (70, 33, 45), (256, 512, 64), (1000, 300, 96)])
def test_relu_mask_epilogue(hip, oracle, dtype, mnk):
    """C = (mask > 0) * (A . B): the gradient of relu folded into the product that feeds it; equal, bit for bit, to
    masking the plain product afterwards (small, general and split-K paths)."""
    dev, pool = hip
    m, n, k = mnk
    r = oracle.Rng(m + n)
    a, b, mask = r.randn((m, k)), r.randn((k, n)), r.randn((m, n))
    mask[0, :] = 0.0
    mask[1, 0] = -0.0
    if dtype == DType.BF16:
        a, b = oracle.f32_to_bf16(a), oracle.f32_to_bf16(b)
    plain = gemm(dev, pool, a, b, dtype=dtype, out_dtype=DType.F32)
    got = gemm(dev, pool, a, b, dtype=dtype, out_dtype=DType.F32, residual=mask, relu_mask=True)
    want = (mask > 0).astype(np.float32) * plain
    if dtype == DType.F32:
        assert np.array_equal(got, want)
    else:  # the unmasked bf16 product may run on the LDS-tiled kernel, which sums in another order
        np.testing.assert_allclose(got, want, rtol=0, atol=2e-6 * np.abs(plain).max() * np.sqrt(k))
        assert np.array_equal(got == 0, want == 0)
    assert (got[0] == 0).all() and got[1, 0] == 0


# ---- f16 on the LDS-tiled kernel (v_mfma_f32_32x32x16_f16) -----------------------------------------------------------

def _f16_operands(oracle, m, n, k, seed, trans_a, trans_b):
    r = oracle.Rng(seed)
    a = oracle.f32_to_f16(r.uniform((k, m) if trans_a else (m, k), -1, 1))
    b = oracle.f32_to_f16(r.uniform((n, k) if trans_b else (k, n), -1, 1))
    af, bf = oracle.f16_to_f32(a).astype(np.float64), oracle.f16_to_f32(b).astype(np.float64)
    af, bf = (af.T if trans_a else af), (bf.T if trans_b else bf)
    return a, b, af @ bf, np.abs(af) @ np.abs(bf)


@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", [(256, 256, 64), (512, 256, 576), (1024, 2048, 512), (256, 384, 256), (264, 136, 64), (1000, 1000, 256),
                                 (256, 256, 4096)])
def test_f16_tiled_gemm_layouts(hip, oracle, mnk, trans_a, trans_b):
    """Whole tiles, edge tiles, the 128-wide tile and split-K, all four layouts; 1e-3 of the f32-accumulated product."""
    dev, pool = hip
    m, n, k = mnk
    a, b, want, mag = _f16_operands(oracle, m, n, k, m + 3 * n + k, trans_a, trans_b)
    got = gemm(dev, pool, a, b, dtype=DType.F16, trans_a=trans_a, trans_b=trans_b)
    assert np.all(np.abs(got - want) <= 1e-3 * np.abs(want) + 1e-5 * mag), np.max(np.abs(got - want) / (mag + 1e-30))


def test_f16_small_integers_are_exact(hip, oracle):
    dev, pool = hip
    rng = np.random.default_rng(2)
    a = rng.integers(-4, 5, size=(256, 192)).astype(np.float32)
    b = rng.integers(-4, 5, size=(192, 256)).astype(np.float32)
    assert np.array_equal(gemm(dev, pool, oracle.f32_to_f16(a), oracle.f32_to_f16(b), dtype=DType.F16), a @ b)


@pytest.mark.parametrize("mnk", [(256, 512, 128), (512, 256, 4096), (300, 200, 128)])
@pytest.mark.parametrize("epilogue", ["bias", "bias_relu", "bias_gelu"])
def test_f16_epilogues_result_and_residual(hip, oracle, mnk, epilogue):
    """Linear (weights [out, in]) with f16 bias, activation, f16 result by the C backend's truncating store
    (zyx/src/codegen/c.rs:475-490) and the fused residual add."""
    dev, pool = hip
    m, n, k = mnk
    a, b, want, mag = _f16_operands(oracle, m, n, k, 17, False, True)
    r = oracle.Rng(6)
    bias, res = oracle.f32_to_f16(r.uniform((n,), -1, 1)), oracle.f32_to_f16(r.randn((m, n)))
    want = want + oracle.f16_to_f32(bias).astype(np.float64)
    if epilogue == "bias_relu":
        want = np.maximum(want, 0.0)
    if epilogue == "bias_gelu":
        want = 0.5 * want * (1 + np.tanh(np.sqrt(2 / np.pi) * (want + 0.044715 * want ** 3)))
    kw = dict(bias=bias, epilogue=epilogue, bias_dtype=DType.F16, trans_b=True, dtype=DType.F16)
    for residual in (None, res):
        w = want + (oracle.f16_to_f32(res).astype(np.float64) if residual is not None else 0.0)
        got32 = gemm(dev, pool, a, b, out_dtype=DType.F32, residual=None if residual is None else oracle.f16_to_f32(res), **kw)
        assert np.all(np.abs(got32 - w) <= 1e-3 * np.abs(w) + 2e-5 * mag + 1e-6)
        got16 = gemm(dev, pool, a, b, out_dtype=DType.F16, residual=residual, **kw)
        assert np.array_equal(got16, oracle.f32_to_f16(got32))  # the f16 result is the f32 one truncated


# ---- f32 on the LDS-tiled kernel (v_mfma_f32_32x32x2_f32) ------------------------------------------------------------

@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
@pytest.mark.parametrize("mnk", [(1024, 1024, 1024), (512, 1024, 96), (2048, 2048, 64), (768, 640, 224), (4096, 128, 32)])
def test_f32_tiled_gemm(hip, oracle, mnk, trans_a, trans_b):
    """zyx/tests/05_misc.rs:820-842 multiplies 1024^3 in f32 against a textbook sgemm: here against the f64-accumulated
    product at 1e-5 of sum |a b|, on both tile sizes (128 x 128 when the grid is large, 64 x 64 otherwise)."""
    dev, pool = hip
    m, n, k = mnk
    r = oracle.Rng(m + n * 3 + k * 7)
    a = r.uniform((k, m) if trans_a else (m, k), -1, 1)
    b = r.uniform((n, k) if trans_b else (k, n), -1, 1)
    got = gemm(dev, pool, a, b, dtype=DType.F32, trans_a=trans_a, trans_b=trans_b)
    ad, bd = a.astype(np.float64), b.astype(np.float64)
    ad, bd = (ad.T if trans_a else ad), (bd.T if trans_b else bd)
    want, mag = ad @ bd, np.abs(ad) @ np.abs(bd)
    assert np.all(np.abs(got - want) <= 1e-5 * mag + 1e-30), np.max(np.abs(got - want) / (mag + 1e-30))


def test_f32_tiled_integer_products_and_epilogues(hip, oracle):
    dev, pool = hip
    rng = np.random.default_rng(4)
    a = rng.integers(-8, 9, size=(1024, 512)).astype(np.float32)
    b = rng.integers(-8, 9, size=(512, 1024)).astype(np.float32)
    assert np.array_equal(gemm(dev, pool, a, b, dtype=DType.F32), a @ b)  # exact in f32 whatever the order
    r = oracle.Rng(12)
    x, w, bias = r.randn((1024, 256)), r.uniform((1024, 256), -0.06, 0.06), r.uniform(1024, -0.06, 0.06)
    res = r.randn((1024, 1024))
    lin = x.astype(np.float64) @ w.astype(np.float64).T + bias
    mag = np.abs(x) @ np.abs(w.T) + np.abs(bias)
    for epi, f in (("bias", lambda v: v), ("bias_relu", lambda v: np.maximum(v, 0)),
                   ("bias_gelu", lambda v: 0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3))))):
        got = gemm(dev, pool, x, w, bias, dtype=DType.F32, trans_b=True, epilogue=epi, residual=res)
        assert np.all(np.abs(got - (f(lin) + res)) <= 2e-5 * mag + 1e-6), epi
    mask = gemm(dev, pool, x, w, dtype=DType.F32, trans_b=True, residual=res, relu_mask=True)
    assert np.all(np.abs(mask - (x.astype(np.float64) @ w.astype(np.float64).T) * (res > 0)) <= 2e-5 * mag)
