"""The pool / device calls of the HIP backend slot, exercised the way the reference's runtime
drives them (zyx/src/runtime.rs:2075-2308, zyx/src/graph/plan.rs:271-361) on a real GPU."""
import numpy as np
import pytest

from zyx_amd import BackendError, DType, ErrorStatus, Event, kernels

pytestmark = pytest.mark.gpu


def test_device_info(hip):
    dev, pool = hip
    info = dev.info()
    assert info.arch.startswith("gfx950")
    assert info.warp_size == 64 and info.tensor_cores and info.has_native_exp2
    assert info.max_local_threads == 1024 and info.preferred_vector_size == 16
    assert not dev.aot_only() and dev.memory_pool_id() == 0
    assert dev.free_compute() > 10 * 2**40  # must outrank the C backend's weight (c.rs:120)
    assert pool.free_bytes() > 100 * 2**30


def test_alloc_copy_roundtrip_and_accounting(hip):
    dev, pool = hip
    before = pool.free_bytes()
    data = np.arange(100003, dtype=np.int32)
    buf, ev = pool.allocate(data.nbytes + 8)
    assert pool.free_bytes() == before - (data.nbytes + 8)
    ev2 = pool.host_to_pool(data, buf, [ev])
    out = np.empty_like(data)
    pool.pool_to_host(buf, out, [ev2])
    assert np.array_equal(out, data)
    pool.deallocate(buf, [])
    assert pool.free_bytes() == before


def test_ids_are_reused_lowest_first(hip):
    dev, pool = hip
    ids = [pool.allocate(1024)[0] for _ in range(4)]
    pool.deallocate(ids[1], [])
    pool.deallocate(ids[2], [])
    again = pool.allocate(64)[0]
    assert again == ids[1]
    for b in (ids[0], ids[3], again):
        pool.deallocate(b, [])


def test_oversized_allocation_fails(hip):
    dev, pool = hip
    with pytest.raises(BackendError) as ei:
        pool.allocate(pool.free_bytes() + 1)
    assert ei.value.status == ErrorStatus.MemoryAllocation and "Allocation failure" in ei.value.context


def test_variables_live_in_buffer_id_space(hip):
    dev, pool = hip
    v = pool.store_variable(DType.I64, 42)
    f = pool.store_variable(DType.F32, 0.5)
    m, ev = pool.allocate(64)
    assert pool.get_variable(v) == (DType.I64, 42)
    assert pool.get_variable(f) == (DType.F32, 0.5)
    assert pool.get_variable(m) is None
    assert len({v, f, m}) == 3
    prog = dev.register_kernel(kernels.softmax_rows_desc(1, 4, True, False, False))
    with pytest.raises(BackendError) as ei:  # a scalar where memory is expected
        dev.launch(prog, pool, [m, v], [ev])
    assert ei.value.status == ErrorStatus.IncorrectKernelArg
    dev.release(prog)
    for b in (v, f, m):
        pool.deallocate(b, [])


def test_events_are_consumed_once(hip):
    dev, pool = hip
    data = np.ones(1024, np.float32)
    buf, ev = pool.allocate(data.nbytes + 4)
    e = pool.host_to_pool(data, buf, [ev])
    pool.sync_events([e])
    with pytest.raises(BackendError) as ei:
        pool.sync_events([e])  # stale handle: an error, never a crash
    assert ei.value.status == ErrorStatus.KernelSync
    pool.sync_events([Event(0)])  # the null event is always signalled
    e = pool.host_to_pool(data, buf, [])
    pool.release_events([e])
    pool.deallocate(buf, [])


def test_malformed_ir_is_refused(hip):
    dev, pool = hip
    with pytest.raises(BackendError) as ei:
        dev.compile(b"\x00" * 16)
    assert ei.value.status == ErrorStatus.KernelCompilation


def test_dependent_launch_chain_and_block_reuse(hip, oracle):
    """softmax(softmax(x)) through freed-and-reused blocks: the second launch must see the first's output."""
    dev, pool = hip
    x = oracle.Rng(1).randn((512, 1024), 3.0)
    prog = dev.register_kernel(kernels.softmax_rows_desc(512, 1024, True, False, False))
    want = oracle.softmax_rows(oracle.softmax_rows(x)[0])[0]
    for _ in range(3):
        xb, e0 = kernels.to_device(pool, x)
        y1, e1 = pool.allocate(x.nbytes + 4)
        l1 = dev.launch(prog, pool, [xb, y1], [e0, e1])
        y2, e2 = pool.allocate(x.nbytes + 4)
        l2 = dev.launch(prog, pool, [y1, y2], [l1, e2])
        got = kernels.to_host(pool, y2, x.shape, np.float32, [l2])
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-37)
        for b in (xb, y1, y2):
            pool.deallocate(b, [])
    dev.release(prog)


def test_timer_and_profile(hip, oracle):
    dev, pool = hip
    x = oracle.Rng(2).randn((1024, 4096), 3.0)
    prog = dev.register_kernel(kernels.softmax_rows_desc(1024, 4096))
    xb, e0 = kernels.to_device(pool, x)
    outs = [pool.allocate(n)[0] for n in (x.nbytes + 4, 1024 * 4 + 4, 1024 * 4 + 4)]
    pool.sync_events([e0])
    ns = dev.time_kernel(prog, [xb] + outs)
    us = dev.profile_kernel(prog, [[xb] + outs], 10)
    assert 0 < us < 1e4 and ns > 0
    for b in [xb] + outs:
        pool.deallocate(b, [])
    dev.release(prog)


def test_plan_keeps_its_programs_alive(hip, oracle):
    """A plan's graph holds its programs' kernels and scratch: releasing one while the plan lives is refused."""
    from zyx_amd import BackendError, ErrorStatus
    from zyx_amd.kernels import reduce_desc, to_device, alloc_like, to_host
    dev, pool = hip
    x = oracle.Rng(8).randn((4096, 512))
    prog = dev.register_kernel(reduce_desc(4096, 512, "sum", axis0=True))  # two-stage: owns a workspace
    xb, e0 = to_device(pool, x)
    ob, e1 = alloc_like(pool, 512, 4)
    pool.sync_events([e0, e1])
    plan = dev.create_plan([(prog, [xb, ob])])
    with pytest.raises(BackendError) as ei:
        dev.release(prog)
    assert ei.value.status == ErrorStatus.IncorrectKernelArg and "live plan" in ei.value.context
    done = dev.launch_plan(plan, [])
    got = to_host(pool, ob, (512,), np.float32, [done])
    assert np.allclose(got, x.astype(np.float64).sum(0), rtol=1e-5, atol=1e-4)
    dev.destroy_plan(plan)
    dev.release(prog)
    for b in (xb, ob):
        pool.deallocate(b, [])


def test_launches_of_one_program_do_not_overlap_on_its_workspace(hip, oracle):
    """Independent wait lists send launches to different streams; a program with scratch memory (two-stage
    column sum here) must still run them one after the other. Many rounds, every result checked."""
    from zyx_amd.kernels import reduce_desc, to_device, alloc_like, to_host
    dev, pool = hip
    r = oracle.Rng(9)
    xs = [r.randn((8192, 256)) for _ in range(4)]
    want = [x.astype(np.float64).sum(0) for x in xs]
    prog = dev.register_kernel(reduce_desc(8192, 256, "sum", axis0=True))
    bufs = []
    for x in xs:
        xb, e = to_device(pool, x)
        ob, e2 = alloc_like(pool, 256, 4)
        pool.sync_events([e, e2])
        bufs.append((xb, ob))
    for _ in range(20):
        evs = [dev.launch(prog, pool, [xb, ob], []) for xb, ob in bufs]  # empty wait lists: round-robin streams
        for (xb, ob), ev, w in zip(bufs, evs, want):
            assert np.allclose(to_host(pool, ob, (256,), np.float32, [ev]), w, rtol=1e-5, atol=2e-4)
    dev.release(prog)
    for xb, ob in bufs:
        pool.deallocate(xb, [])
        pool.deallocate(ob, [])


def test_calls_from_several_threads(hip, oracle):
    """zyx calls its backends from whichever user thread holds the runtime mutex (zyx/src/lib.rs:96): the library is
    not thread-affine. Four threads each upload, launch a softmax of their own data and read it back, 20 times."""
    import threading
    from zyx_amd.kernels import softmax_rows
    dev, pool = hip
    errors = []

    def work(seed):
        try:
            x = (3 * oracle.Rng(seed).randn((64, 512))).astype(np.float32)
            want, _, want_arg = oracle.softmax_rows(x)
            for _ in range(20):
                y, s, a = softmax_rows(dev, pool, x)
                assert np.allclose(y, want, rtol=1e-5, atol=1e-37) and np.array_equal(a, want_arg)
        except Exception as e:  # surfaced in the main thread below
            errors.append(repr(e))

    threads = [threading.Thread(target=work, args=(100 + i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_device_to_device_ranges(hip):
    """zhip_d2d: aligned and unaligned ranges, a move inside one buffer (disjoint and overlapping), a large one, and
    the bounds errors; the bytes around the destination range stay as they were."""
    dev, pool = hip
    rng = np.random.default_rng(3)
    src = rng.integers(0, 256, 9 << 20, dtype=np.uint8)
    sb, e0 = pool.allocate(src.nbytes)
    db, e1 = pool.allocate(src.nbytes)
    pool.sync_events([pool.host_to_pool(src, sb, [e0]), pool.host_to_pool(np.zeros_like(src), db, [e1])])
    want = np.zeros_like(src)
    for s_off, d_off, n in ((0, 0, 4096), (16, 64, 200704), (3, 5, 1001), (7, 1 << 20, 123457), (1 << 20, 2 << 20, 5 << 20),
                            (100, 8 << 20, 0)):
        ev = pool.copy_range(sb, s_off, db, d_off, n, [])
        pool.sync_events([ev])
        want[d_off:d_off + n] = src[s_off:s_off + n]
    got = np.empty_like(src)
    pool.pool_to_host(db, got, [])
    assert np.array_equal(got, want)
    # inside one buffer: disjoint (copy kernel) and overlapping forward (the runtime's copy: memmove is not promised,
    # so only the non-overlapping part is checked)
    pool.sync_events([pool.copy_range(sb, 0, sb, 4 << 20, 1 << 20, [])])
    pool.pool_to_host(sb, got, [])
    assert np.array_equal(got[4 << 20:5 << 20], src[:1 << 20]) and np.array_equal(got[:4 << 20], src[:4 << 20])
    for bad in ((0, 0, src.nbytes + 1), (src.nbytes, 0, 1), (0, src.nbytes - 3, 4)):
        with pytest.raises(BackendError):
            pool.copy_range(sb, bad[0], db, bad[1], bad[2], [])
    pool.deallocate(sb, [])
    pool.deallocate(db, [])
