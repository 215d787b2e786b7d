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
@pytest.mark.parametrize("mnk", [(256, 256, 64), (256, 512, 128), (512, 256, 576), (1024, 2048, 512)])
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
    """BASELINE config 3: A, B uniform(-1,1) truncated to bf16, 4096^3, f32 out. The full
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
