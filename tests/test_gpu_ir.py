"""Generic kernels on the GPU: Device::compile on the image of a linearized kernel, launched through the C ABI and
compared with the CPU interpreter of the same image (oracle/ir_interp.py). Bar: bit-exact for integer ops, casts,
16-bit stores and every kernel made of + - * / max, comparisons and loads / stores only (no contraction, same
serial order); kernels with exp / log / sin / cos within 1e-5 relative (the device's float entry points against
double evaluation), Mad within one rounding of the separate multiply-add."""
import numpy as np
import pytest

import ir_kernels as K
from oracle import ir_interp
from zyx_amd import BackendError, DType, ErrorStatus
from zyx_amd import ir
from zyx_amd.ir import BOp, ParamKind, UOp
from zyx_amd.kernels import to_device, to_host

pytestmark = pytest.mark.gpu


def both(hip, kernel, args, plan=False):
    """Runs the image on the GPU and in the interpreter; returns [(gpu, cpu)] for every GlobalMut argument."""
    dev, pool = hip
    img = kernel.to_bytes()
    params = [o for o in kernel.ops if o.opcode == ir.Opcode.PARAM]
    assert len(params) == len(args)
    prog = dev.compile(img)
    bufs, waits, outs = [], [], []
    for p, a in zip(params, args):
        if p.aux == ParamKind.Variable:
            bufs.append(pool.store_variable(DType(p.dtype), a))
        else:
            b, e = to_device(pool, a)
            bufs.append(b)
            waits.append(e)
    if plan:
        pool.sync_events(waits)
        pl = dev.create_plan([(prog, bufs)])
        done = dev.launch_plan(pl, [])
    else:
        done = dev.launch(prog, pool, bufs, waits)
    cpu_args = [a.copy() if isinstance(a, np.ndarray) else a for a in args]
    ir_interp.run(img, cpu_args)
    res = []
    pool.sync_events([done])
    for p, a, b, ca in zip(params, args, bufs, cpu_args):
        if p.aux == ParamKind.GlobalMut:
            res.append((to_host(pool, b, a.shape, a.dtype, []), ca))
    if plan:
        dev.destroy_plan(pl)
    for b in bufs:
        pool.deallocate(b, [])
    dev.release(prog)
    return res


def exact(pairs):
    for g, c in pairs:
        assert np.array_equal(g, c, equal_nan=True), np.flatnonzero(g.reshape(-1) != c.reshape(-1))[:8]


@pytest.mark.parametrize("mnk,local", [((56, 5, 12), (1, 1)), ((64, 16, 97), (8, 4)), ((128, 128, 64), (16, 16)), ((17, 19, 2), (1, 1))])
def test_matmul_kernels(hip, oracle, mnk, local):
    m, n, k = mnk
    r = oracle.Rng(m + n + k)
    a, b = r.uniform((m, k), -1, 1), r.uniform((k, n), -1, 1)
    (g, c), = both(hip, K.matmul(m, n, k, local=local, first_id=7, id_step=3), [a, b, np.zeros((m, n), np.float32)])
    assert np.array_equal(g, c) and np.array_equal(g, oracle.matmul(a, b, oracle.F32, oracle.F32))
    ab, bb = oracle.f32_to_bf16(a), oracle.f32_to_bf16(b)
    (g, c), = both(hip, K.matmul(m, n, k, DType.BF16, DType.BF16, local=local), [ab, bb, np.zeros((m, n), np.uint16)])
    assert np.array_equal(g, c) and np.array_equal(g, oracle.matmul(ab, bb, oracle.BF16, oracle.BF16))
    ai, bi = r.randint((m, k), -100, 100).astype(np.int64), r.randint((k, n), -100, 100).astype(np.int64)
    (g, c), = both(hip, K.matmul(m, n, k, DType.I64, DType.I64, use_mad=True, local=local), [ai, bi, np.zeros((m, n), np.int64)])
    assert np.array_equal(g, c) and np.array_equal(g, ai @ bi)
    # Mad on floats is one rounding per step on the GPU and (through double) in the interpreter
    (g, c), = both(hip, K.matmul(m, n, k, use_mad=True, local=local), [a, b, np.zeros((m, n), np.float32)])
    mag = np.abs(a) @ np.abs(b)
    assert np.all(np.abs(g - c) <= 1e-6 * mag)


def test_reference_goldens_on_the_device(hip):
    # zyx/tests/05_misc.rs:201-208 and :664-683
    x = np.array([[2, 4, 3], [1, 5, 1]], np.float32)
    y = np.array([[2, 4], [3, 1], [5, 1]], np.float32)
    (g, _), = both(hip, K.matmul(2, 2, 3), [x, y, np.zeros((2, 2), np.float32)])
    assert g.tolist() == [[31, 15], [22, 10]]
    x = np.array([[2.0, 4.0, 3.0], [4.0, 2.0, 3.0]], np.float32)
    (g, _), = both(hip, K.softmax_rows(2, 3), [x, np.zeros_like(x)])
    assert np.allclose(g, [[0.090030566, 0.6652409, 0.24472846], [0.6652409, 0.090030566, 0.24472846]], rtol=1e-6)


def test_softmax_kernel(hip, oracle):
    x = (3 * oracle.Rng(5).randn((256, 333))).astype(np.float32)
    (g, c), = both(hip, K.softmax_rows(256, 333), [x, np.zeros_like(x)])
    assert np.allclose(g, c, rtol=1e-5, atol=0)
    y64, _ = oracle.softmax_rows_f64acc(x)
    assert np.allclose(g, y64, rtol=1e-5, atol=0)


@pytest.mark.parametrize("uop", list(UOp))
def test_float_unary_ops(hip, oracle, uop):
    if uop == UOp.BitNot:
        pytest.skip("no meaning on floats")
    x = oracle.Rng(int(uop) + 1).uniform(8192, -8, 8)
    if uop in (UOp.Ln, UOp.Log2, UOp.Sqrt):
        x = np.abs(x) + np.float32(1e-3)
    (g, c), = both(hip, K.unary_table(8192, DType.F32, uop), [x, np.zeros_like(x)])
    if uop in (UOp.Neg, UOp.Reciprocal, UOp.Sqrt, UOp.Floor, UOp.Trunc, UOp.Abs):
        assert np.array_equal(g, c)        # IEEE operations: correctly rounded on both sides
    else:
        assert np.all(np.abs(g - c) <= 1e-5 * np.abs(c) + 1e-6)
    xd = x.astype(np.float64)
    (g, c), = both(hip, K.unary_table(8192, DType.F64, uop), [xd, np.zeros_like(xd)])
    assert np.allclose(g, c, rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("bop", [BOp.Add, BOp.Sub, BOp.Mul, BOp.Div, BOp.Mod, BOp.Max, BOp.Cmplt, BOp.Cmpgt, BOp.Cmpge,
                                 BOp.NotEq, BOp.Eq, BOp.Or, BOp.And, BOp.Pow])
def test_float_binary_ops(hip, oracle, bop):
    r = oracle.Rng(int(bop) + 40)
    x, y = r.uniform(4096, -9, 9), r.uniform(4096, -9, 9)
    y[::7] = x[::7]
    x[::11] = 0
    boolean = bop in (BOp.Cmplt, BOp.Cmpgt, BOp.Cmpge, BOp.NotEq, BOp.Eq, BOp.Or, BOp.And)
    if bop == BOp.Pow:
        x = np.abs(x) + np.float32(0.1)
    (g, c), = both(hip, K.binary_table(4096, DType.F32, bop), [x, y, np.zeros(4096, np.uint8 if boolean else np.float32)])
    if bop == BOp.Pow:
        assert np.allclose(g, c, rtol=1e-5)
    else:
        assert np.array_equal(g, c)


@pytest.mark.parametrize("dtype,np_t", [(DType.I8, np.int8), (DType.U8, np.uint8)])
def test_integer_ops_exhaustive_8_bit(hip, dtype, np_t):
    lo, hi = (-128, 128) if np_t == np.int8 else (0, 256)
    a, b = np.meshgrid(np.arange(lo, hi), np.arange(lo, hi), indexing="ij")
    x, y = a.reshape(-1).astype(np_t), b.reshape(-1).astype(np_t)
    for bop in (BOp.Add, BOp.Sub, BOp.Mul, BOp.Div, BOp.Mod, BOp.Max, BOp.BitXor, BOp.BitOr, BOp.BitAnd, BOp.BitShiftLeft,
                BOp.BitShiftRight, BOp.Cmplt, BOp.Cmpge, BOp.Eq, BOp.Or, BOp.And):
        boolean = bop in (BOp.Cmplt, BOp.Cmpge, BOp.Eq, BOp.Or, BOp.And)
        exact(both(hip, K.binary_table(x.size, dtype, bop), [x, y, np.zeros(x.size, np.uint8 if boolean else np_t)]))
    v = np.arange(lo, hi).astype(np_t)
    for uop in (UOp.Neg, UOp.BitNot, UOp.Abs):
        exact(both(hip, K.unary_table(v.size, dtype, uop), [v, np.zeros_like(v)]))


@pytest.mark.parametrize("dtype,np_t", [(DType.I32, np.int32), (DType.U32, np.uint32), (DType.I64, np.int64), (DType.U64, np.uint64),
                                        (DType.I16, np.int16), (DType.U16, np.uint16)])
def test_wide_integer_ops(hip, dtype, np_t):
    rng = np.random.default_rng(int(dtype))
    info = np.iinfo(np_t)
    x = rng.integers(info.min, info.max, 4096, dtype=np_t, endpoint=True)
    y = rng.integers(info.min, info.max, 4096, dtype=np_t, endpoint=True)
    y[::5] = rng.integers(0, 70, y[::5].size).astype(np_t)
    x[:4] = [info.min, info.max, 0, info.min]
    y[:4] = [info.max, info.min, 0, np_t(-1) if info.min < 0 else 1]
    for bop in (BOp.Add, BOp.Sub, BOp.Mul, BOp.Div, BOp.Max, BOp.BitXor, BOp.BitShiftLeft, BOp.BitShiftRight, BOp.Cmplt, BOp.NotEq):
        boolean = bop in (BOp.Cmplt, BOp.NotEq)
        exact(both(hip, K.binary_table(4096, dtype, bop), [x, y, np.zeros(4096, np.uint8 if boolean else np_t)]))


def test_casts_and_16_bit_stores(hip, oracle):
    x = np.array([0.0, 0.5, -0.5, 1.0, -1.0, 1.9, -1.9, 255.9, 256.0, 300.7, -129.2, 65535.6, 1e6, -1e6, 3.0, 77.0], np.float32)
    exact(both(hip, K.cast_table(x.size, DType.F32, DType.I32), [x, np.zeros(x.size, np.int32)]))
    exact(both(hip, K.cast_table(x.size, DType.F32, DType.Bool), [x, np.zeros(x.size, np.uint8)]))
    i = np.array([-1, 0, 1, 127, 128, 255, 256, -129, 2**31 - 1, -2**31], np.int32)
    exact(both(hip, K.cast_table(i.size, DType.I32, DType.I8), [i, np.zeros(i.size, np.int8)]))
    exact(both(hip, K.cast_table(i.size, DType.I32, DType.F32), [i, np.zeros(i.size, np.float32)]))
    exact(both(hip, K.cast_table(i.size, DType.I32, DType.I64), [i, np.zeros(i.size, np.int64)]))
    exact(both(hip, K.cast_table(i.size, DType.I32, DType.F64), [i, np.zeros(i.size, np.float64)]))
    v = np.concatenate([oracle.Rng(3).uniform(2000, -70000, 70000),
                        np.array([1e-9, -1e-9, 6e-8, 65504.0, 65520.0, 1e-5, np.inf, -np.inf], np.float32)])
    v = np.resize(v, 2048).astype(np.float32)
    (g, c), = both(hip, K.elementwise(8, 256, (), DType.F32, DType.BF16), [v, np.zeros(2048, np.uint16)])
    assert np.array_equal(g, c) and np.array_equal(g, oracle.f32_to_bf16(v))
    (g, c), = both(hip, K.elementwise(8, 256, (), DType.F32, DType.F16), [v, np.zeros(2048, np.uint16)])
    assert np.array_equal(g, c) and np.array_equal(g, oracle.f32_to_f16(v).view(np.uint16))
    exact(both(hip, K.elementwise(8, 256, (UOp.Neg,), DType.F16, DType.F32), [g, np.zeros(2048, np.float32)]))
    exact(both(hip, K.elementwise(8, 256, (UOp.Abs, UOp.Sqrt), DType.BF16, DType.BF16), [oracle.f32_to_bf16(v), np.zeros(2048, np.uint16)]))


def test_local_memory_reduction_with_barriers(hip, oracle):
    r = oracle.Rng(11)
    x = r.randn((300, 2048))
    (g, c), = both(hip, K.row_sum_local(300, 2048, 256), [x, np.zeros(300, np.float32)])
    assert np.array_equal(g, c)                    # same strided-serial, then pairwise order
    assert np.allclose(g, x.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-4)
    xi = np.floor(r.uniform((64, 1024), -50, 50)).astype(np.float32)
    (g, _), = both(hip, K.row_sum_local(64, 1024, 64), [xi, np.zeros(64, np.float32)])
    assert np.array_equal(g, xi.sum(axis=1))
    xb = oracle.f32_to_bf16(x[:32, :512])          # bf16 in global memory, f32 in the local tile
    exact(both(hip, K.row_sum_local(32, 512, 128, DType.BF16), [xb, np.zeros(32, np.uint16)]))


def test_padding_masks_vectors_variables(hip, oracle):
    r = oracle.Rng(12)
    x = r.randn(1000)
    (g, c), = both(hip, K.padded_copy(1000, 33, 91), [x, np.full(1000 + 33 + 91, np.nan, np.float32)])
    assert np.array_equal(g, c) and np.array_equal(g, np.pad(x, (33, 91)))
    for vlen in (2, 4, 8, 16):
        n = 40 * 64 * vlen
        a, b = r.randn(n), r.randn(n)
        (g, c), = both(hip, K.vector_axpy(40, 64, vlen), [np.float32(1.7), a, b, np.zeros(n, np.float32)])
        assert np.array_equal(g, c) and np.array_equal(g, np.float32(1.7) * a + b)
        exact(both(hip, K.vector_scale(40, 64, vlen), [a, np.zeros(n, np.float32)]))
        ab = oracle.f32_to_bf16(a)
        exact(both(hip, K.vector_axpy(40, 64, vlen, DType.BF16), [np.float32(-0.3), ab, oracle.f32_to_bf16(b), np.zeros(n, np.uint16)]))
        exact(both(hip, K.vector_scale(40, 64, vlen, DType.F16), [oracle.f32_to_f16(a).view(np.uint16), np.zeros(n, np.uint16)]))


def test_group_count_from_a_variable_and_ragged_loops(hip, oracle):
    r = oracle.Rng(13)
    for rows in (1, 5, 777, 0):
        x = r.randn((max(rows, 1), 64))
        (g, c), = both(hip, K.dynamic_rows(64), [rows, x, np.zeros_like(x)])
        assert np.array_equal(g, c)
        if rows:
            assert np.array_equal(g[:rows], x[:rows] + np.arange(rows, dtype=np.float32)[:, None])
    ln = (np.arange(256) * 7 % 65).astype(np.int32)
    x = r.randn((256, 64))
    (g, c), = both(hip, K.ragged_loop(256), [ln, x, np.zeros(256, np.float32)])
    assert np.array_equal(g, c)


def test_generated_kernels_in_plans_and_errors(hip, oracle):
    dev, pool = hip
    assert not dev.aot_only()
    r = oracle.Rng(14)
    a, b = r.uniform((64, 97), -1, 1), r.uniform((97, 16), -1, 1)
    (g, c), = both(hip, K.matmul(64, 16, 97, local=(8, 4)), [a, b, np.zeros((64, 16), np.float32)], plan=True)
    assert np.array_equal(g, c)
    k = K.elementwise(4, 64)
    prog = dev.compile(k.to_bytes())
    assert "zir_kernel" in dev.program_source(prog)
    x, e1 = to_device(pool, np.zeros(256, np.float32))
    small, e2 = pool.allocate(16)
    var = pool.store_variable(DType.I64, 3)
    pool.sync_events([e1, e2])
    for args in ([x], [x, small], [x, var], [var, x]):       # wrong count, too small, a variable where memory is due
        with pytest.raises(BackendError) as e:
            dev.launch(prog, pool, args, [])
        assert e.value.status == ErrorStatus.IncorrectKernelArg
    dev.release(prog)
    prog = dev.compile(K.dynamic_rows(64).to_bytes())
    y, e3 = pool.allocate(64 * 4 * 4)
    pool.sync_events([e3])
    with pytest.raises(BackendError) as e:                   # memory where the Variable is due
        dev.launch(prog, pool, [x, x, y], [])
    assert e.value.status == ErrorStatus.IncorrectKernelArg
    bad = pool.store_variable(DType.I32, 3)                  # a Variable of another dtype
    with pytest.raises(BackendError) as e:
        dev.launch(prog, pool, [bad, x, y], [])
    assert e.value.status == ErrorStatus.IncorrectKernelArg
    huge = pool.store_variable(DType.I64, 2**40)             # more groups than the device can launch
    with pytest.raises(BackendError) as e:
        dev.launch(prog, pool, [huge, x, y], [])
    assert e.value.status == ErrorStatus.KernelLaunch
    dev.release(prog)
    for b in (x, small, var, y, bad, huge):
        pool.deallocate(b, [])
    with pytest.raises(BackendError) as e:
        dev.compile(b"\x00" * 16)
    assert e.value.status == ErrorStatus.KernelCompilation


def test_optimised_example_kernels(hip, oracle):
    """The benchmark's generated kernels: parity with the interpreter at a small size, and at the benchmark's size
    against the double-precision rows and the invariants (rows sum to 1, argmax preserved)."""
    from zyx_amd import ir_examples
    dev, pool = hip
    x = (3 * oracle.Rng(21).randn((16, 1024))).astype(np.float32)
    (g, c), = both(hip, ir_examples.softmax_rows_local(16, 1024, 64, 4), [x, np.zeros_like(x)])
    assert np.allclose(g, c, rtol=1e-5, atol=1e-37)
    x = (3 * oracle.Rng(22).randn((8192, 4096))).astype(np.float32)
    prog = dev.compile(ir_examples.softmax_rows_local(8192, 4096).to_bytes())
    xb, e1 = to_device(pool, x)
    yb, e2 = pool.allocate(x.nbytes)
    y = to_host(pool, yb, x.shape, np.float32, [dev.launch(prog, pool, [xb, yb], [e1, e2])])
    y64, _ = oracle.softmax_rows_f64acc(x)
    assert np.allclose(y, y64, rtol=1e-5, atol=1e-37)
    assert np.allclose(y.sum(axis=1, dtype=np.float64), 1.0, atol=1e-5) and np.array_equal(y.argmax(1), x.argmax(1))
    dev.release(prog)
    for b in (xb, yb):
        pool.deallocate(b, [])
    for dt, vlen in ((DType.F32, 4), (DType.BF16, 8)):
        n = 1 << 16
        v = oracle.Rng(23).uniform(n, -4, 4)
        arr = v if dt == DType.F32 else oracle.f32_to_bf16(v)
        (g, c), = both(hip, ir_examples.scaled_exp2(n, dt, vlen=vlen), [arr, np.zeros_like(arr)])
        gf, cf = (g, c) if dt == DType.F32 else (oracle.bf16_to_f32(g), oracle.bf16_to_f32(c))
        assert np.all(np.abs(gf - cf) <= (1e-5 if dt == DType.F32 else 2.0 ** -7) * np.abs(cf))


def test_autotune_call_sequence(hip):
    """What zyx's autotuner does with a candidate kernel (zyx/src/kernel/autotune.rs:358-430, 775-798): buffers of
    ones plus one spare element, dynamic dimensions stored as 42, compile, a timed launch, release."""
    dev, pool = hip
    k = K.dynamic_rows(64)
    rows = pool.store_variable(DType.I64, 42)
    x, e1 = to_device(pool, np.ones(42 * 64 + 1, np.float32))
    y, e2 = to_device(pool, np.ones(42 * 64 + 1, np.float32))
    pool.sync_events([e1, e2])
    prog = dev.compile(k.to_bytes())
    ns = dev.time_kernel(prog, [rows, x, y])
    assert 0 < ns < 1e9
    got = to_host(pool, y, (42 * 64 + 1,), np.float32, [])
    assert np.array_equal(got[:-1].reshape(42, 64), 1.0 + np.arange(42, dtype=np.float32)[:, None] * np.ones((1, 64), np.float32))
    assert got[-1] == 1.0          # the spare element is not touched
    us = dev.profile_kernel(prog, [[rows, x, y]], 5)
    assert us > 0
    dev.release(prog)
    for b in (rows, x, y):
        pool.deallocate(b, [])


def test_reference_integer_matmuls_on_the_device(hip):
    """Integer products are bit-exact on the GPU: the reference's i64 fixture (zyx/tests/xyz2.safetensors,
    zyx/tests/05_misc.rs:639-661: x[256,512] . y[512,368] == z) and the closed-form i32 sweep of matmul_1
    (05_misc.rs:210-237: x[i][j] = i + j, y[i][j] = i - j), through generated matmul kernels."""
    import os
    from zyx_amd import safetensors_io
    t = safetensors_io.load(os.path.join(os.path.dirname(__file__), "golden", "xyz2.safetensors"))
    x, y, z = (np.ascontiguousarray(t[k][1]) for k in "xyz")
    assert x.dtype == np.int64 and x.shape == (256, 512) and y.shape == (512, 368)
    for local in ((16, 16), (1, 1)):
        (g, _), = both(hip, K.matmul(256, 368, 512, DType.I64, DType.I64, use_mad=True, local=local),
                       [x, y, np.zeros((256, 368), np.int64)])
        assert g.dtype == np.int64 and np.array_equal(g, z)
    for m in range(56, 576, 259):
        for k in range(12, 890, 231):
            for n in range(5, 97, 71):
                a = (np.arange(m)[:, None] + np.arange(k)[None, :]).astype(np.int32)
                b = (np.arange(k)[:, None] - np.arange(n)[None, :]).astype(np.int32)
                want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.int32)  # wraps like i32 accumulation
                (g, c), = both(hip, K.matmul(m, n, k, DType.I32, DType.I32), [a, b, np.zeros((m, n), np.int32)])
                assert np.array_equal(g, want) and np.array_equal(c, want), (m, k, n)


def test_compiled_code_is_cached_in_memory_and_on_disk(hip, tmp_path):
    """The reference's C backend keeps what it compiled on disk by kernel hash (zyx/src/backend/c.rs:165-186); here
    the code object of a generated kernel is found again in memory by the same process and on disk by another one,
    and a damaged cache file is rebuilt."""
    import os
    import subprocess
    import sys
    import time
    from zyx_amd import backend
    dev, pool = hip
    old = os.environ.get("ZYX_HIP_CACHE_DIR")
    os.environ["ZYX_HIP_CACHE_DIR"] = str(tmp_path)
    try:
        kernel = K.elementwise(977, 64, [UOp.Exp2, UOp.Sin, UOp.Neg])  # a shape no other test compiles
        img = kernel.to_bytes()
        s0 = backend.compile_cache_stats()
        t0 = time.perf_counter()
        p1 = dev.compile(img)
        t1 = time.perf_counter()
        p2 = dev.compile(img)
        t2 = time.perf_counter()
        s1 = backend.compile_cache_stats()
        assert s1["compiled"] == s0["compiled"] + 1 and s1["memory_hits"] == s0["memory_hits"] + 1
        assert t2 - t1 < 0.05 and t2 - t1 < t1 - t0
        files = [f for f in os.listdir(tmp_path) if f.endswith(".hsaco")]
        assert len(files) == 1
        dev.release(p1)
        dev.release(p2)
        # another process finds the file; after the file is cut short it compiles again and repairs it
        child = ("import sys, numpy as np; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
                 "import zyx_amd, ir_kernels as K\n"
                 "from zyx_amd import backend\n"
                 "from zyx_amd.ir import UOp\n"
                 "pools, devs = zyx_amd.initialize_device(zyx_amd.HIPConfig(device_ids=[0]))\n"
                 "devs[0].compile(K.elementwise(977, 64, [UOp.Exp2, UOp.Sin, UOp.Neg]).to_bytes())\n"
                 "s = backend.compile_cache_stats(); print(s['compiled'], s['disk_hits'])\n"
                 "pools[0].deinitialize()\n") % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                                                os.path.dirname(os.path.abspath(__file__)))
        out = subprocess.run([sys.executable, "-c", child], capture_output=True, text=True, timeout=100, env=dict(os.environ))
        assert out.returncode == 0, out.stderr[-2000:]
        assert out.stdout.split()[-2:] == ["0", "1"]
        path = os.path.join(tmp_path, files[0])
        whole = open(path, "rb").read()
        open(path, "wb").write(whole[:len(whole) // 2])
        out = subprocess.run([sys.executable, "-c", child], capture_output=True, text=True, timeout=100, env=dict(os.environ))
        assert out.returncode == 0, out.stderr[-2000:]
        assert out.stdout.split()[-2:] == ["1", "0"]
        assert len(open(path, "rb").read()) >= len(whole) // 2 + 1 and not [f for f in os.listdir(tmp_path) if ".tmp" in f]
    finally:
        if old is None:
            del os.environ["ZYX_HIP_CACHE_DIR"]
        else:
            os.environ["ZYX_HIP_CACHE_DIR"] = old
