"""The oracle's chain evaluator must agree with its own primitive-op tables (which the
reference goldens pin) and with closed forms; the chain encoding itself is this build's."""
import numpy as np

from zyx_amd import DType
from zyx_amd.kernels import EW_COL, EW_ROW, EW_SCALAR, Chain


def test_chain_matches_primitive_tables(oracle):
    r = oracle.Rng(4)
    x, y = r.randn((5, 12)), r.randn((5, 12))
    for name in ["neg", "exp", "exp2", "sin", "cos", "floor", "trunc", "abs", "relu", "tanh", "gelu", "sigmoid"]:
        c = Chain(5, 12)
        c.load(c.input()).op(name)
        assert np.array_equal(oracle.ew_chain(c, [x]), oracle.unary(name, x)), name
    for name in ["add", "sub", "mul", "div", "cmplt", "cmpgt", "max", "eq", "noteq"]:
        c = Chain(5, 12)
        a, b = c.input(), c.input()
        c.load(a).op(name, b)
        assert np.array_equal(oracle.ew_chain(c, [x, y]), oracle.binary(name, x, y)), name


def test_chain_broadcasts_and_composites(oracle):
    r = oracle.Rng(8)
    x, bias, col, s = r.randn((6, 8)), r.randn(8), r.randn(6), r.randn(1)
    c = Chain(6, 8)
    ix, ib, ic, is_ = c.input(), c.input(DType.F32, EW_ROW), c.input(DType.F32, EW_COL), c.input(DType.F32, EW_SCALAR)
    c.load(ix).add(ib).mul(ic).sub(is_).save().mul(c.const(0.5)).rsub(Chain.T)
    t = (x + bias[None, :]) * col[:, None] - s[0]
    assert np.allclose(oracle.ew_chain(c, [x, bias, col, s]), t - t * np.float32(0.5), rtol=1e-6, atol=1e-7)
    # where / mad
    c = Chain(6, 8)
    ix, iy = c.input(), c.input()
    c.load(ix).cmpgt(c.const(0.0)).where(iy, c.const(-1.0))
    assert np.array_equal(oracle.ew_chain(c, [x, x * 2]), np.where(x > 0, x * 2, np.float32(-1)))
    # SGD step p - g*lr (zyx-optim/src/sgd.rs:77-81)
    c = Chain(6, 8)
    ip, ig = c.input(), c.input()
    c.load(ig).mul(c.const(0.01)).rsub(ip)
    assert np.array_equal(oracle.ew_chain(c, [x, x * 3]), x - (x * 3) * np.float32(0.01))


def test_chain_int_registers_and_stores(oracle):
    a = np.array([[7, -7, 2**31 - 1, -5]], np.int32)
    b = np.array([[2, 2, 1, -3]], np.int32)
    c = Chain(1, 4, DType.I32, DType.I32)
    ia, ib = c.input(DType.I32), c.input(DType.I32)
    c.load(ia).add(ib)
    assert oracle.ew_chain(c, [a, b]).tolist() == [[9, -5, -(2**31), -8]]  # wraps
    c = Chain(1, 4, DType.I32, DType.I32)
    ia, ib = c.input(DType.I32), c.input(DType.I32)
    c.load(ia).div(ib)
    assert oracle.ew_chain(c, [a, b]).tolist() == [[3, -3, 2**31 - 1, 1]]  # C truncation
    c = Chain(1, 4, DType.I32, DType.I32)
    ia, ib = c.input(DType.I32), c.input(DType.I32)
    c.load(ia).mod(ib)
    assert oracle.ew_chain(c, [a, b]).tolist() == [[1, -1, 0, -2]]
    # float -> bf16 store truncates; float -> i32 store truncates toward zero
    x = np.array([[1.0 + 2**-8 + 2**-9, -2.75, 3.99, -0.5]], np.float32)
    c = Chain(1, 4, DType.F32, DType.BF16)
    c.load(c.input())
    assert np.array_equal(oracle.ew_chain(c, [x]), oracle.f32_to_bf16(x))
    c = Chain(1, 4, DType.F32, DType.I32)
    c.load(c.input())
    assert oracle.ew_chain(c, [x]).tolist() == [[1, -2, 3, 0]]


def test_gelu_grad_matches_finite_differences(oracle):
    """gelu_grad is the derivative of the oracle's own gelu: central differences in f64 of the reference's
    expression (zyx/src/tensor/elementwise.rs:168-170) pin the formula; a wrong cubic coefficient (0.134145 =
    3 * 0.044715) or a missing (1 - t^2) factor fails it."""
    from zyx_amd.kernels import Chain
    x = np.linspace(-6, 6, 1001).astype(np.float32).reshape(1, -1)
    c = Chain(1, x.size)
    c.load(c.input()).gelu_grad()
    got = oracle.ew_chain(c, [x])
    f = lambda v: 0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3)))
    x64 = x.astype(np.float64)
    num = (f(x64 + 1e-6) - f(x64 - 1e-6)) / 2e-6
    assert np.allclose(got, num, rtol=1e-5, atol=2e-6)
    big = np.array([[50.0, -50.0, 1e4, -1e4]], np.float32)  # saturated tanh: slope 1 and 0
    c2 = Chain(1, 4)
    c2.load(c2.input()).gelu_grad()
    assert oracle.ew_chain(c2, [big]).tolist() == [[1.0, 0.0, 1.0, 0.0]]
