"""Fused elementwise chains on the GPU vs the CPU oracle (zyx/tests/01_unary.rs,
02_binary.rs, 10_bf16.rs are the reference's tests for the same ops).

Tolerance: f32 relative 1e-5. Ops the reference builds from exp with a cancelling
add/subtract (tanh = (e^2x-1)/(e^2x+1), gelu's x/2 * (1+tanh), sigmoid) carry the rounding
of a value near 1 (ulp 6e-8..1.2e-7) as ABSOLUTE error, scaled by |x|/2 in gelu: two
implementations of exp that differ by one ulp differ by that much, so those ops add
2.4e-7 * max(1,|x|) absolute (4 ulp(1.0) * |x|/2). Integer and comparison results are bit-exact.
"""
import numpy as np
import pytest

from zyx_amd import BackendError, DType, ErrorStatus
from zyx_amd.kernels import EW_COL, EW_ROW, EW_SCALAR, Chain, run_chain

pytestmark = pytest.mark.gpu


def close(got, want, rtol=1e-5, atol=0.0):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    err = np.abs(got - want)
    ok = (err <= rtol * np.abs(want) + atol) | (np.isnan(got) & np.isnan(want)) | (got == want)
    assert ok.all(), f"max err {np.nanmax(err):.3e}, first bad {np.argwhere(~ok)[:3].tolist()}"


UNARY_POS = {"ln", "log2", "sqrt", "rsqrt", "reciprocal"}


@pytest.mark.parametrize("name", ["neg", "exp", "exp2", "ln", "log2", "reciprocal", "sqrt", "sin", "cos", "floor",
                                  "trunc", "abs", "relu", "tanh", "gelu", "sigmoid", "rsqrt"])
@pytest.mark.parametrize("shape", [(64, 1024), (3, 7)])
def test_unary(hip, oracle, name, shape):
    dev, pool = hip
    x = oracle.Rng(len(name)).randn(shape, 3.0)
    if name in UNARY_POS:
        x = np.abs(x) + np.float32(1e-3)
    c = Chain(*shape)
    c.load(c.input()).op(name)
    atol = 2.4e-7 * np.maximum(1.0, np.abs(x)) if name in ("tanh", "gelu", "sigmoid") else 0.0
    want = oracle.ew_chain(c, [x])
    if name in ("tanh", "gelu"):
        # The reference's tanh is inf/inf = NaN once exp(2z) overflows f32 (z > 44.36, i.e.
        # x > ~10 for gelu); the kernel saturates instead (tanh -> 1). Parity is asserted
        # where the reference is finite, saturation where it is not.
        over = np.isnan(want)
        assert np.all(x[over] > 9.0)
        want = np.where(over, x if name == "gelu" else np.float32(1.0), want)
    close(run_chain(dev, pool, c, [x]), want, atol=atol)


def test_reference_unary_goldens(hip):
    # zyx/tests/01_unary.rs:9-16 (relu_1), :652-657 (tanh_2)
    dev, pool = hip
    data = np.array([[-3.285, 0.001, 1.780, 5.675, -8.521, -0.456, 1.215, -3.474, -4.128, -7.657]], np.float32)
    c = Chain(1, 10)
    c.load(c.input()).relu()
    assert np.array_equal(run_chain(dev, pool, c, [data]),
                          np.array([[0.0, 0.001, 1.780, 5.675, 0.0, 0.0, 1.215, 0.0, 0.0, 0.0]], np.float32))
    c = Chain(2, 3)
    c.load(c.input()).tanh()
    close(run_chain(dev, pool, c, [np.array([[2, 4, 1], [5, 4, 1]], np.float32)]),
          [[0.964028, 0.999329, 0.761594], [0.999909, 0.999329, 0.761594]], rtol=2e-6)


@pytest.mark.parametrize("name", ["add", "sub", "mul", "div", "max", "cmplt", "cmpgt", "cmpge", "eq", "noteq", "pow",
                                  "mod", "rsub", "rdiv", "or", "and"])
def test_binary_and_broadcast(hip, oracle, name):
    dev, pool = hip
    r = oracle.Rng(17)
    x = r.randn((33, 256), 3.0)
    if name == "pow":
        x = np.abs(x) + np.float32(0.1)
    for bc, y in ((0, r.randn((33, 256), 3.0)), (EW_ROW, r.randn(256, 3.0)), (EW_COL, r.randn(33, 3.0)),
                  (EW_SCALAR, r.randn(1, 3.0))):
        if name in ("mod", "div", "rdiv"):
            y = np.where(np.abs(y) < 1.0, np.float32(1.5), y).astype(np.float32)
        c = Chain(33, 256)
        a, b = c.input(), c.input(DType.F32, bc)
        c.load(a).op(name, b)
        close(run_chain(dev, pool, c, [x, y]), oracle.ew_chain(c, [x, y]), rtol=3e-5 if name == "pow" else 1e-5)


def test_fused_chains_from_the_configs(hip, oracle):
    dev, pool = hip
    r = oracle.Rng(23)
    # Linear epilogue gelu(x + bias) (zyx-nn/src/linear.rs:38-44 + elementwise.rs:168-170)
    x, bias = r.randn((512, 1024), 2.0), r.uniform(1024, -1, 1)
    c = Chain(512, 1024)
    ix, ib = c.input(), c.input(DType.F32, EW_ROW)
    c.load(ix).add(ib).gelu()
    close(run_chain(dev, pool, c, [x, bias]), oracle.ew_chain(c, [x, bias]), atol=2.4e-7 * np.maximum(1, np.abs(x) + 1))
    # relu backward: dy * (x > 0)  (autograd rule for cmpgt*mul, graph/autograd.rs:120-125)
    dy = r.randn((512, 1024))
    c = Chain(512, 1024)
    ix, idy = c.input(), c.input()
    c.load(ix).cmpgt(c.const(0.0)).mul(idy)
    assert np.array_equal(run_chain(dev, pool, c, [x, dy]), oracle.ew_chain(c, [x, dy]))
    # SGD: p - g * lr  (zyx-optim/src/sgd.rs:77-81)
    c = Chain(512, 1024)
    ip, ig = c.input(), c.input()
    c.load(ig).mul(c.const(0.01)).rsub(ip)
    got = run_chain(dev, pool, c, [x, dy])
    close(got, oracle.ew_chain(c, [x, dy]), rtol=1e-6)
    # residual add + scale with a saved temporary
    c = Chain(512, 1024)
    ix, idy = c.input(), c.input()
    c.load(ix).add(idy).save().mul(Chain.T).mad(c.const(0.5), Chain.T)
    close(run_chain(dev, pool, c, [x, dy]), oracle.ew_chain(c, [x, dy]), rtol=1e-6)


@pytest.mark.parametrize("dt", [DType.BF16, DType.F16])
def test_16bit_storage(hip, oracle, dt):
    """bf16/f16 widen on load, compute in f32, truncate on store (zyx/src/codegen/c.rs:456-497)."""
    dev, pool = hip
    r = oracle.Rng(31)
    conv = oracle.f32_to_bf16 if dt == DType.BF16 else oracle.f32_to_f16
    x, y = conv(r.randn((40, 512), 2.0)), conv(r.randn((40, 512), 2.0))
    for shape in ((40, 512), (5, 4093 - 1)):  # vector and scalar paths
        n = shape[0] * shape[1]
        xa, ya = x.reshape(-1)[:n].reshape(shape), y.reshape(-1)[:n].reshape(shape)
        c = Chain(shape[0], shape[1], DType.F32, dt)
        a, b = c.input(dt), c.input(dt)
        c.load(a).mul(b).add(a)
        assert np.array_equal(run_chain(dev, pool, c, [xa, ya]), oracle.ew_chain(c, [xa, ya]))
    # cast f32 -> 16 bit and back
    xf = r.randn((7, 64), 100.0)
    c = Chain(7, 64, DType.F32, dt)
    c.load(c.input())
    assert np.array_equal(run_chain(dev, pool, c, [xf]), conv(xf))


def test_int_registers_bit_exact(hip, oracle):
    dev, pool = hip
    rng = np.random.default_rng(0)
    a = rng.integers(-2**31, 2**31, size=(37, 128), dtype=np.int64).astype(np.int32)
    b = rng.integers(-2**31, 2**31, size=(37, 128), dtype=np.int64).astype(np.int32)
    b[0, :8] = [0, -1, 1, 2, -2, 0, -1, 7]
    a[0, :2] = [-2**31, -2**31]
    for name in ["add", "sub", "mul", "div", "mod", "max", "cmplt", "cmpgt", "cmpge", "eq", "noteq", "bitxor", "bitor",
                 "bitand", "shl", "shr", "rsub", "or", "and"]:
        c = Chain(37, 128, DType.I32, DType.I32)
        ia, ib = c.input(DType.I32), c.input(DType.I32)
        c.load(ia).op(name, ib)
        assert np.array_equal(run_chain(dev, pool, c, [a, b]), oracle.ew_chain(c, [a, b])), name
    for name in ["neg", "bitnot", "abs", "relu"]:
        c = Chain(37, 128, DType.I32, DType.I32)
        c.load(c.input(DType.I32)).op(name)
        assert np.array_equal(run_chain(dev, pool, c, [a]), oracle.ew_chain(c, [a])), name
    # one-hot mask (Tensor::one_hot = equal(arange)) stored as u8/bool
    labels = rng.integers(0, 10, size=(64,)).astype(np.int32)
    c = Chain(64, 10, DType.I32, DType.U8)
    il, ia = c.input(DType.I32, EW_COL), c.input(DType.I32, EW_ROW)
    c.load(il).eq(ia)
    got = run_chain(dev, pool, c, [labels, np.arange(10, dtype=np.int32)])
    assert np.array_equal(got, (labels[:, None] == np.arange(10)[None, :]).astype(np.uint8))


def test_float_to_int_store_truncates(hip, oracle):
    dev, pool = hip
    x = np.array([[1.9, -2.75, 3.99, -0.5, 1e6, -1e6, 0.0, 123456.7]], np.float32)
    c = Chain(1, 8, DType.F32, DType.I32)
    c.load(c.input())
    assert run_chain(dev, pool, c, [x]).tolist() == [[1, -2, 3, 0, 1000000, -1000000, 0, 123456]]


def test_bad_programs_are_refused(hip):
    dev, pool = hip
    c = Chain(4, 4)
    c.load(c.input()).op("bitxor", 0)  # int-only op on float registers
    with pytest.raises(BackendError) as ei:
        dev.register_kernel(c.desc())
    assert ei.value.status == ErrorStatus.KernelCompilation
    c = Chain(4, 4)
    c.load(c.input()).add(3)  # operand 3 does not exist
    with pytest.raises(BackendError):
        dev.register_kernel(c.desc())
    c = Chain(4, 4)
    c.exp()  # must start with LOAD
    c.input()
    with pytest.raises(BackendError):
        dev.register_kernel(c.desc())


def test_large_tensor_grid_stride(hip, oracle):
    dev, pool = hip
    x = oracle.Rng(41).randn((4096, 8192))
    c = Chain(4096, 8192)
    c.load(c.input()).mul(c.const(2.0)).add(c.const(1.0))
    assert np.array_equal(run_chain(dev, pool, c, [x]), x * np.float32(2) + np.float32(1))


def test_gelu_grad_chain(hip, oracle):
    """dh = dg * gelu'(h), the chain the MLP backward of a transformer block launches (bf16 storage)."""
    from zyx_amd import DType
    from zyx_amd.kernels import Chain, run_chain
    dev, pool = hip
    r = oracle.Rng(3)
    h = r.randn((64, 512), 3.0)
    dg = r.randn((64, 512))
    c = Chain(64, 512)
    hi, gi = c.input(DType.F32), c.input(DType.F32)
    c.load(hi).gelu_grad().mul(gi)
    got, want = run_chain(dev, pool, c, [h, dg]), oracle.ew_chain(c, [h, dg])
    assert np.all(np.abs(got - want) <= 1e-5 * np.abs(want) + 1e-6 * np.abs(dg))
    cb = Chain(64, 512, out_dtype=DType.BF16)
    hi, gi = cb.input(DType.BF16), cb.input(DType.BF16)
    cb.load(hi).gelu_grad().mul(gi)
    hb, gb = oracle.f32_to_bf16(h), oracle.f32_to_bf16(dg)
    got, want = run_chain(dev, pool, cb, [hb, gb]), oracle.ew_chain(cb, [hb, gb])
    assert np.all(np.abs(oracle.bf16_to_f32(got) - oracle.bf16_to_f32(want)) <= 2.0 ** -7 * np.abs(oracle.bf16_to_f32(want)) + 1e-6)


# ---- chains above the size threshold run as code generated and compiled for that one program ----------------
BIG = (1024, 2048)  # 2 Mi elements: above the default threshold of 1 Mi


def _big_inputs(oracle, seed=0):
    r = oracle.Rng(seed)
    return r.randn(BIG, 2.0), r.randn(BIG), r.randn((BIG[1],)), r.randn((BIG[0],))


def test_generated_chain_f32_all_operand_kinds(hip, oracle):
    from zyx_amd import DType
    from zyx_amd.kernels import Chain, EW_ROW, EW_COL, EW_SCALAR, run_chain
    dev, pool = hip
    x, y, rowv, colv = _big_inputs(oracle)
    c = Chain(*BIG)
    ix, iy, ir, ic = c.input(), c.input(), c.input(DType.F32, EW_ROW), c.input(DType.F32, EW_COL)
    c.load(ix).mul(iy).save().add(ir).max(ic).mad(Chain.T, c.const(0.25)).relu().sub(c.const(1.5))
    got, want = run_chain(dev, pool, c, [x, y, rowv, colv]), oracle.ew_chain(c, [x, y, rowv, colv])
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    c = Chain(*BIG)
    ix, isc = c.input(), c.input(DType.F32, EW_SCALAR)
    c.load(ix).cmplt(isc).where(c.const(2.0), ix)
    s = np.array([0.3], np.float32)
    assert np.array_equal(run_chain(dev, pool, c, [x, s]), oracle.ew_chain(c, [x, s]))


@pytest.mark.parametrize("op", ["gelu", "gelu_grad", "tanh", "sigmoid", "exp", "rsqrt", "neg", "abs"])
def test_generated_unary_bf16(hip, oracle, op):
    from zyx_amd import DType
    from zyx_amd.kernels import Chain, run_chain
    dev, pool = hip
    x = oracle.f32_to_bf16(np.abs(_big_inputs(oracle, 1)[0]) + 0.01 if op == "rsqrt" else _big_inputs(oracle, 1)[0])
    c = Chain(*BIG, out_dtype=DType.BF16)
    getattr(c.load(c.input(DType.BF16)), op)()
    got, want = oracle.bf16_to_f32(run_chain(dev, pool, c, [x])), oracle.bf16_to_f32(oracle.ew_chain(c, [x]))
    # one truncating store apart at most; the absolute term covers the tails, where the reference's own expression
    # rounds 1 + tanh to 0 (gelu'(-5.06) = -1.03e-6 comes out as 0 there, the kernel returns the value itself)
    ok = np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + (2e-6 if op == "gelu_grad" else 1e-6)
    assert np.all(ok | (np.isnan(want) & (np.isnan(got) | np.isfinite(got))))


def test_generated_mixed_dtypes_and_int_chain(hip, oracle):
    from zyx_amd import DType
    from zyx_amd.kernels import Chain, EW_ROW, run_chain
    dev, pool = hip
    x, y, rowv, _ = _big_inputs(oracle, 2)
    # f32 master weights - lr * bf16 gradient -> f16 copy: three storage dtypes in one chain
    c = Chain(*BIG, out_dtype=DType.F16)
    ip, ig = c.input(DType.F32), c.input(DType.BF16)
    c.load(ig).mul(c.const(0.01)).rsub(ip)
    g = oracle.f32_to_bf16(y)
    assert np.array_equal(run_chain(dev, pool, c, [x, g]), oracle.ew_chain(c, [x, g]))
    # int32 registers, u8 and i32 operands, row-broadcast i32, u8 result
    rng = np.random.default_rng(0)
    a = rng.integers(0, 256, BIG).astype(np.uint8)
    b = rng.integers(-1000, 1000, BIG).astype(np.int32)
    r = rng.integers(1, 9, BIG[1]).astype(np.int32)
    ci = Chain(*BIG, reg=DType.I32, out_dtype=DType.U8)
    ia, ib, ir = ci.input(DType.U8), ci.input(DType.I32), ci.input(DType.I32, EW_ROW)
    ci.load(ia).mul(ib).div(ir).bitxor(ib).shr(ci.const(3.0)).bitand(ci.const(255.0))
    assert np.array_equal(run_chain(dev, pool, ci, [a, b, r]), oracle.ew_chain(ci, [a, b, r]))
    ci = Chain(*BIG, reg=DType.I32, out_dtype=DType.I32)
    ia, ib = ci.input(DType.I32), ci.input(DType.I32)
    ci.load(ia).mod(ib).save().cmplt(ci.const(0.0)).where(ib, ci.const(0.0)).add(Chain.T)
    b2 = rng.integers(-7, 8, BIG).astype(np.int32)
    assert np.array_equal(run_chain(dev, pool, ci, [b, b2]), oracle.ew_chain(ci, [b, b2]))
