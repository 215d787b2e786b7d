"""Pins oracle/ir_interp.py (the checker for generated kernels): the reference's golden values computed through
linearized kernels, bit-for-bit agreement with the C oracle's serial loops (itself pinned to the goldens in
test_oracle_goldens.py), exhaustive 8-bit tables of the integer ops against Python integers, closed forms."""
import json
import os
import struct

import numpy as np
import pytest

import ir_kernels as K
from oracle import ir_interp
from zyx_amd import DType
from zyx_amd.ir import BOp, UOp

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def run(kernel, *args):
    ir_interp.run(kernel.to_bytes(), list(args))


def ulps(a, b):
    a, b = np.asarray(a, np.float32), np.asarray(b, np.float32)
    ia, ib = a.view(np.int32).astype(np.int64), b.view(np.int32).astype(np.int64)
    ia, ib = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia), np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    return np.abs(ia - ib)


def test_reference_matmul_goldens():
    # zyx/tests/05_misc.rs:201-208 (matmul_2)
    x = np.array([[2, 4, 3], [1, 5, 1]], np.float32)
    y = np.array([[2, 4], [3, 1], [5, 1]], np.float32)
    z = np.zeros((2, 2), np.float32)
    run(K.matmul(2, 2, 3), x, y, z)
    assert z.tolist() == [[31, 15], [22, 10]]
    xi, yi, zi = x.astype(np.int32), y.astype(np.int32), np.zeros((2, 2), np.int32)
    run(K.matmul(2, 2, 3, DType.I32, DType.I32), xi, yi, zi)
    assert zi.tolist() == [[31, 15], [22, 10]]
    # the i64 fixture the reference's own test loads (zyx/tests/xyz2.safetensors)
    with open(os.path.join(GOLD, "xyz2.safetensors"), "rb") as f:
        n = struct.unpack("<Q", f.read(8))[0]
        hdr = json.loads(f.read(n))
        blob = f.read()
    t = {k: np.frombuffer(blob[d["data_offsets"][0]:d["data_offsets"][1]], "<i8").reshape(d["shape"]).copy()
         for k, d in hdr.items() if k != "__metadata__"}
    (m, kk), n_ = t["x"].shape, t["y"].shape[1]
    z = np.zeros((m, n_), np.int64)
    run(K.matmul(m, n_, kk, DType.I64, DType.I64, use_mad=True), t["x"], t["y"], z)
    assert np.array_equal(z, t["z"])


@pytest.mark.parametrize("mnk,local", [((56, 5, 12), (1, 1)), ((64, 16, 97), (8, 4)), ((17, 19, 2), (1, 1))])
def test_matmul_is_the_c_oracles_serial_loop(oracle, mnk, local):
    m, n, k = mnk
    r = oracle.Rng(m + n + k)
    a, b = r.uniform((m, k), -1, 1), r.uniform((k, n), -1, 1)
    c = np.zeros((m, n), np.float32)
    run(K.matmul(m, n, k, local=local, first_id=7, id_step=3), a, b, c)
    assert np.array_equal(c, oracle.matmul(a, b, oracle.F32, oracle.F32))
    # bf16 storage: widening loads, f32 accumulation, truncating store (zyx/tests/10_bf16.rs:160-198 is the 17x2x19 case)
    ab, bb = oracle.f32_to_bf16(a), oracle.f32_to_bf16(b)
    cb = np.zeros((m, n), np.uint16)
    run(K.matmul(m, n, k, DType.BF16, DType.BF16, local=local), ab, bb, cb)
    assert np.array_equal(cb, oracle.matmul(ab, bb, oracle.BF16, oracle.BF16))


def test_softmax_goldens_and_c_oracle(oracle):
    # zyx/tests/05_misc.rs:664-683
    x = np.array([[2.0, 4.0, 3.0], [4.0, 2.0, 3.0]], np.float32)
    y = np.zeros_like(x)
    run(K.softmax_rows(2, 3), x, y)
    assert np.allclose(y, [[0.090030566, 0.6652409, 0.24472846], [0.6652409, 0.090030566, 0.24472846]], rtol=1e-6)
    x = (3 * oracle.Rng(5).randn((64, 333))).astype(np.float32)
    y = np.zeros_like(x)
    run(K.softmax_rows(64, 333), x, y)
    want, _, _ = oracle.softmax_rows(x)
    # same serial loops; exp through double here, the compiler's (vectorised) expf there: a few ulp apart, and both
    # within 1e-5 (serial f32 sums of 333 terms) of the double-precision rows
    assert ulps(y, want).max() <= 8
    y64, _ = oracle.softmax_rows_f64acc(x)
    assert np.allclose(y, y64, rtol=1e-5, atol=0)


@pytest.mark.parametrize("uop,name", [(UOp.Neg, "neg"), (UOp.Exp, "exp"), (UOp.Exp2, "exp2"), (UOp.Ln, "ln"), (UOp.Log2, "log2"),
                                      (UOp.Reciprocal, "reciprocal"), (UOp.Sqrt, "sqrt"), (UOp.Sin, "sin"), (UOp.Cos, "cos"),
                                      (UOp.Floor, "floor"), (UOp.Trunc, "trunc"), (UOp.Abs, "abs")])
def test_unary_ops_match_the_c_oracle(oracle, uop, name):
    x = oracle.Rng(int(uop) + 1).uniform(4096, -8, 8)
    if uop in (UOp.Ln, UOp.Log2, UOp.Sqrt):
        x = np.abs(x) + np.float32(1e-3)
    y = np.zeros_like(x)
    run(K.unary_table(4096, DType.F32, uop), x, y)
    want = oracle.unary(name, x)
    if uop in (UOp.Neg, UOp.Reciprocal, UOp.Sqrt, UOp.Floor, UOp.Trunc, UOp.Abs):
        assert np.array_equal(y, want)
    else:  # the C oracle's float entry points (a few ulp when vectorised) against double evaluation narrowed once
        assert ulps(y, want).max() <= 4
        ref = {UOp.Exp: np.exp, UOp.Exp2: np.exp2, UOp.Ln: np.log, UOp.Log2: np.log2, UOp.Sin: np.sin, UOp.Cos: np.cos}[uop]
        assert np.array_equal(y, ref(x.astype(np.float64)).astype(np.float32))


@pytest.mark.parametrize("bop,name", [(BOp.Add, "add"), (BOp.Sub, "sub"), (BOp.Mul, "mul"), (BOp.Div, "div"), (BOp.Mod, "mod"),
                                      (BOp.Max, "max"), (BOp.Cmplt, "cmplt"), (BOp.Cmpgt, "cmpgt"), (BOp.Cmpge, "cmpge"),
                                      (BOp.NotEq, "noteq"), (BOp.Eq, "eq")])
def test_float_binary_ops_match_the_c_oracle(oracle, bop, name):
    r = oracle.Rng(int(bop) + 40)
    x, y = r.uniform(2048, -9, 9), r.uniform(2048, -9, 9)
    y[::7] = x[::7]
    if bop == BOp.Mod:  # (int)y == 0 is a division by zero in C: the reference's loop would trap
        y = np.where(np.abs(y) < 1, np.float32(2.5), y)
    want = oracle.binary(name, x, y)
    boolean = bop in (BOp.Cmplt, BOp.Cmpgt, BOp.Cmpge, BOp.NotEq, BOp.Eq)
    z = np.zeros(2048, np.uint8 if boolean else np.float32)
    run(K.binary_table(2048, DType.F32, bop), x, y, z)
    assert np.array_equal(z.astype(np.float32), want)


def _c_div(a, b):
    q = abs(a) // abs(b)
    return q if (a < 0) == (b < 0) else -q


@pytest.mark.parametrize("dtype,np_t", [(DType.I8, np.int8), (DType.U8, np.uint8)])
def test_integer_ops_exhaustive_8_bit(dtype, np_t):
    """Every pair of 8-bit values against Python integer arithmetic wrapped to 8 bits: wrap-around add / sub / mul,
    truncating division (0 for a zero divisor), (int)x % (int)y, max, bit operations, shifts modulo the width."""
    lo, hi = (-128, 128) if np_t == np.int8 else (0, 256)
    a, b = np.meshgrid(np.arange(lo, hi), np.arange(lo, hi), indexing="ij")
    x, y = a.reshape(-1).astype(np_t), b.reshape(-1).astype(np_t)

    def wrap(v):
        v &= 0xFF
        return v - 256 if (np_t == np.int8 and v >= 128) else v

    def c_mod(p, q):
        return 0 if q in (0, -1) else p - q * _c_div(p, q)

    table = {
        BOp.Add: lambda p, q: wrap(p + q), BOp.Sub: lambda p, q: wrap(p - q), BOp.Mul: lambda p, q: wrap(p * q),
        BOp.Div: lambda p, q: 0 if q == 0 else wrap(_c_div(p, q)), BOp.Mod: lambda p, q: wrap(c_mod(p, q)),
        BOp.Max: max, BOp.BitXor: lambda p, q: wrap(p ^ q), BOp.BitOr: lambda p, q: wrap(p | q), BOp.BitAnd: lambda p, q: wrap(p & q),
        BOp.BitShiftLeft: lambda p, q: wrap(p << (q & 7)), BOp.BitShiftRight: lambda p, q: wrap(p >> (q & 7)),
    }
    for bop, fn in table.items():
        z = np.zeros(x.size, np_t)
        run(K.binary_table(x.size, dtype, bop), x, y, z)
        want = np.array([fn(int(p), int(q)) for p, q in zip(x[::1], y[::1])], np.int64).astype(np_t)
        assert np.array_equal(z, want), bop
    for bop, fn in {BOp.Cmplt: lambda p, q: p < q, BOp.Cmpge: lambda p, q: p >= q, BOp.Eq: lambda p, q: p == q,
                    BOp.Or: lambda p, q: bool(p) or bool(q), BOp.And: lambda p, q: bool(p) and bool(q)}.items():
        z = np.zeros(x.size, np.uint8)
        run(K.binary_table(x.size, dtype, bop), x, y, z)
        assert np.array_equal(z, np.array([fn(int(p), int(q)) for p, q in zip(x, y)], np.uint8)), bop
    for uop, fn in {UOp.Neg: lambda p: wrap(-p), UOp.BitNot: lambda p: wrap(~p), UOp.Abs: lambda p: wrap(abs(p))}.items():
        v = np.arange(lo, hi).astype(np_t)
        z = np.zeros_like(v)
        run(K.unary_table(v.size, dtype, uop), v, z)
        assert np.array_equal(z, np.array([fn(int(p)) for p in v], np.int64).astype(np_t)), uop


def test_casts_and_16_bit_stores(oracle):
    x = np.array([0.0, 0.5, -0.5, 1.0, -1.0, 1.9, -1.9, 255.9, 256.0, 300.7, -129.2, 65535.6, 1e6, -1e6], np.float32)
    z = np.zeros(x.size, np.int32)
    run(K.cast_table(x.size, DType.F32, DType.I32), x, z)
    assert z.tolist() == [int(v) for v in x]                      # truncation toward zero
    zb = np.zeros(x.size, np.uint8)
    run(K.cast_table(x.size, DType.F32, DType.Bool), x, zb)       # (uint8_t)x, not x != 0 (c.rs:243-261, 618)
    assert zb.tolist() == [int(v) & 0xFF for v in x]
    i = np.array([-1, 0, 1, 127, 128, 255, 256, -129, 2**31 - 1, -2**31], np.int32)
    z8 = np.zeros(i.size, np.int8)
    run(K.cast_table(i.size, DType.I32, DType.I8), i, z8)
    assert np.array_equal(z8, i.astype(np.int8))
    zf = np.zeros(i.size, np.float32)
    run(K.cast_table(i.size, DType.I32, DType.F32), i, zf)
    assert np.array_equal(zf, i.astype(np.float32))
    # stores to bf16 / f16 truncate (f16: overflow to inf, subnormal results flushed): the pinned C conversions
    v = np.concatenate([oracle.Rng(3).uniform(2000, -70000, 70000), np.array([1e-9, -1e-9, 6e-8, 65504.0, 65520.0, 1e-5, np.inf, -np.inf], np.float32)])
    v = np.resize(v, 2048).astype(np.float32)
    hb = np.zeros(2048, np.uint16)
    run(K.elementwise(8, 256, (), DType.F32, DType.BF16), v, hb)
    assert np.array_equal(hb, oracle.f32_to_bf16(v))
    hf = np.zeros(2048, np.uint16)
    run(K.elementwise(8, 256, (), DType.F32, DType.F16), v, hf)
    assert np.array_equal(hf, oracle.f32_to_f16(v).view(np.uint16))
    back = np.zeros(2048, np.float32)
    run(K.elementwise(8, 256, (), DType.F16, DType.F32), hf, back)
    assert np.array_equal(back, oracle.f16_to_f32(hf.view(oracle.f32_to_f16(v).dtype)))


def test_local_reduce_padding_vectors_and_dynamic_shapes(oracle):
    r = oracle.Rng(11)
    # integer-valued data: every order of summation gives the same f32, so the tree must equal numpy's sum exactly
    x = np.floor(r.uniform((6, 1024), -50, 50)).astype(np.float32)
    s = np.zeros(6, np.float32)
    run(K.row_sum_local(6, 1024, 256), x, s)
    assert np.array_equal(s, x.sum(axis=1))
    # general data: the same strided-serial then pairwise order, written out with numpy
    x = r.randn((3, 512))
    s = np.zeros(3, np.float32)
    run(K.row_sum_local(3, 512, 128), x, s)
    part = np.zeros((3, 128), np.float32)
    for j in range(4):
        part = x[:, j * 128:(j + 1) * 128] + part
    st = 64
    while st >= 1:
        part[:, :st] = part[:, :st] + part[:, st:2 * st]
        st //= 2
    assert np.array_equal(s, part[:, 0])

    x = r.randn(37)
    y = np.full(37 + 5 + 9, np.nan, np.float32)
    run(K.padded_copy(37, 5, 9), x, y)
    assert np.array_equal(y, np.pad(x, (5, 9)))

    for vlen in (2, 4, 8):
        n = 3 * 64 * vlen
        a, b = r.randn(n), r.randn(n)
        z = np.zeros(n, np.float32)
        run(K.vector_axpy(3, 64, vlen), np.float32(1.7), a, b, z)
        assert np.array_equal(z, np.float32(1.7) * a + b)
        run(K.vector_scale(3, 64, vlen), a, z)
        assert np.array_equal(z, a * np.float32(2) + np.float32(1))

    for rows in (1, 5, 0):
        x = r.randn((max(rows, 1), 64))
        y = np.zeros_like(x)
        run(K.dynamic_rows(64), rows, x, y)
        want = np.zeros_like(x)
        want[:rows] = x[:rows] + np.arange(rows, dtype=np.float32)[:, None]
        assert np.array_equal(y, want)

    ln = (np.arange(64) * 7 % 65).astype(np.int32)
    x = r.randn((64, 64))
    s = np.zeros(64, np.float32)
    run(K.ragged_loop(64), ln, x, s)
    want = np.zeros(64, np.float32)
    for j in range(64):
        want = np.where(j < ln, x[:, j] + want, want)
    assert np.array_equal(s, want)


def test_mad_rounds_once():
    # 1 + 2^-12 squared is 1 + 2^-11 + 2^-24: a separate multiply drops the last term before the subtraction sees it
    x = np.array([1 + 2.0 ** -12], np.float32)
    assert ir_interp.mad(x, x, np.array([-(1 + 2.0 ** -11)], np.float32), ir_interp.F32)[0] == np.float32(2.0 ** -24)
    assert (x * x - np.float32(1 + 2.0 ** -11))[0] == 0.0
