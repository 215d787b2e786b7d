#!/usr/bin/env python3
"""Benchmark of the HIP backend's hot path on one MI355X.

Workload (benchmark configuration 2): fused row softmax + row-sum + row-argmax over an f32
8192x4096 tensor, inputs resident in HBM. A "step" is one launch of the fused kernel
through the C ABI (zhip_launch) on one buffer set; buffer sets rotate so no step finds
its input in the 256 MB Infinity Cache left by the previous one.

Prints one JSON line: whole-job GB/s (algorithmic bytes / wall time of K steps), plus
  roofline     -- the kernel's own duration from HIP events on its launch stream
  cpu_baseline -- the CPU oracle (restated zyx C backend) timed on the host cores
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from zyx_amd.rng import Rng  # zyx's own generator (zyx/src/rng.rs): every input below is drawn from it, outside the timed regions

ROWS, COLS = 8192, 4096
# x read once + y written once + rowsum and argmax written once
ALGO_BYTES = ROWS * COLS * 4 * 2 + 2 * ROWS * 4
HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published
N_SETS = 4              # 4 x 268 MB working set > Infinity Cache
# HBM bytes per launch of the fused kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled
# by the same counter's reading for a plain copy kernel of known size in the same run
# (profiles/softmax_rows_f32_8192x4096.md): 134,262,878 B fetched + 134,739,929 B written.
TRAFFIC_BYTES = 269002807


def measured_ceilings(dev, nbytes: int = 1 << 30):
    """What this device sustains right now, beside the published peaks the roofline fractions are quoted against:
    hipMemcpy device to device and a float4 copy kernel over `nbytes` (bytes read + written per second), a read-only
    kernel (bytes read), and a register-resident v_mfma_f32_32x32x16_bf16 loop on all compute units with constant
    operands (the clock holds) and with random ones (the power limit lowers it): rate, average clock, launch time."""
    c = dev.measure_ceilings(nbytes)
    c["bytes"] = nbytes
    c["frac_of_8TB/s"] = {k: round(c[k] / HBM_PEAK_GBPS, 4) for k in ("memcpy_d2d_GBps", "copy_kernel_GBps", "read_kernel_GBps")}
    c["frac_of_2.5PF"] = {k: round(c[k] / 2500.0, 4) for k in ("mfma_bf16_const_TFLOPs", "mfma_bf16_random_TFLOPs")}
    return c


def cpu_baseline(x: np.ndarray, budget_s: float = 10.0):
    import oracle

    oracle.build()
    threads = len(os.sched_getaffinity(0))
    threads = int(os.environ.get("OMP_NUM_THREADS", threads))
    oracle.softmax_rows(x[:64])  # load + warm
    reps, t0 = 0, time.perf_counter()
    best = float("inf")
    while True:
        t1 = time.perf_counter()
        oracle.softmax_rows(x)
        dt = time.perf_counter() - t1
        best = min(best, dt)
        reps += 1
        if time.perf_counter() - t0 > budget_s or reps >= 40:
            break
    return {"value": ALGO_BYTES / best / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"full {ROWS}x{COLS} f32 workload, min of {reps} passes of the OpenMP C oracle "
                      f"(serial per-row loops as zyx's C backend emits), {best * 1e3:.1f} ms/pass"}


def extra_gemm(dev, pool, kernels, steps=100, warmup=200):
    """Config 3: bf16 4096^3 GEMM (f32 accumulate), raw and with the fused bias+GELU epilogue."""
    n = 4096
    rng = Rng(1)
    trunc = lambda a: (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)  # bf16 by truncation, as zyx does
    a, b = trunc(rng.uniform((n, n), -1, 1)), trunc(rng.uniform((n, n), -1, 1))
    bias = trunc(rng.uniform(n, -1 / 64, 1 / 64))
    ab, e1 = kernels.to_device(pool, a)
    bb, e2 = kernels.to_device(pool, b)
    biasb, e3 = kernels.to_device(pool, bias)
    cb, e4 = pool.allocate(n * n * 4 + 4)
    pool.sync_events([e1, e2, e3, e4])
    out = {}
    for name, epi in (("nn", "none"), ("nn_bias_gelu", "bias_gelu")):
        prog = dev.register_kernel(kernels.gemm_desc(n, n, n, epilogue=epi, bias_dtype=zyx_dtype_bf16()))
        args = [ab, bb] + ([biasb] if epi != "none" else []) + [cb]
        dev.profile_kernel(prog, [args], warmup)  # also lets the clocks settle
        us = dev.profile_kernel(prog, [args], steps)
        tf = 2.0 * n**3 / us / 1e6
        out[name] = {"avg_launch_us": round(us, 2), "TFLOP/s": round(tf, 1), "frac_of_2.5PF_bf16_peak": round(tf / 2500.0, 4)}
        dev.release(prog)
    for b_ in (ab, bb, biasb, cb):
        pool.deallocate(b_, [])
    # the other operand dtypes of Tensor::dot: f16 on the same LDS-tiled kernel, f32 (what the reference's own AOT
    # matchers claim, zyx/src/backend/cblas.rs:265-268; zyx/tests/05_misc.rs:820-842 multiplies 1024^3) at 1024^3 and 4096^3
    import zyx_amd
    to_f16 = lambda x: x.astype(np.float16).view(np.uint16)
    for name, dt, n2, peak, conv in (("f16_4096", zyx_amd.DType.F16, 4096, 2500.0, to_f16),
                                     ("f32_1024", zyx_amd.DType.F32, 1024, 157.3, lambda x: x),
                                     ("f32_4096", zyx_amd.DType.F32, 4096, 157.3, lambda x: x)):
        a2, b2 = conv(rng.uniform((n2, n2), -1, 1)), conv(rng.uniform((n2, n2), -1, 1))
        ab, e1 = kernels.to_device(pool, a2)
        bb, e2 = kernels.to_device(pool, b2)
        cb, e3 = pool.allocate(n2 * n2 * 4 + 4)
        pool.sync_events([e1, e2, e3])
        prog = dev.register_kernel(kernels.gemm_desc(n2, n2, n2, dtype=dt))
        dev.profile_kernel(prog, [[ab, bb, cb]], max(20, warmup // 4))
        us = dev.profile_kernel(prog, [[ab, bb, cb]], max(10, steps // 4))
        tf = 2.0 * n2**3 / us / 1e6
        out[name] = {"avg_launch_us": round(us, 2), "TFLOP/s": round(tf, 1), "peak_TFLOP/s": peak, "frac_of_peak": round(tf / peak, 4)}
        dev.release(prog)
        for b_ in (ab, bb, cb):
            pool.deallocate(b_, [])
    return out


def extra_conv(dev, pool, kernels, steps=50, warmup=50):
    """Config 4: conv2d N=32 C=64 56x56, 3x3 -> 128 channels, stride 1 pad 1 (+ ReLU), then 2x2 max-pool."""
    import zyx_amd
    N, C, HW, CO = 32, 64, 56, 128
    flop = 2.0 * N * CO * HW * HW * C * 9
    rng = Rng(4)
    out = {}
    for name, dt, isz in (("f32", zyx_amd.DType.F32, 4), ("bf16", zyx_amd.DType.BF16, 2)):
        x = rng.randn((N, C, HW, HW))
        w = rng.randn((CO, C, 3, 3), float(np.sqrt(2.0 / 576)))
        if isz == 2:
            x, w = [(a.view(np.uint32) >> 16).astype(np.uint16) for a in (x, w)]
        xb, e1 = kernels.to_device(pool, x)
        wb, e2 = kernels.to_device(pool, w)
        yb, e3 = kernels.alloc_like(pool, N * CO * HW * HW, isz)
        pb, e4 = kernels.alloc_like(pool, N * CO * (HW // 2) ** 2, isz)
        pool.sync_events([e1, e2, e3, e4])
        conv = dev.register_kernel(kernels.conv2d_desc(N, C, HW, HW, CO, 3, 3, padding=(1, 1), relu=True, dtype=dt))
        mp = dev.register_kernel(kernels.max_pool2d_desc(N * CO, HW, HW, dtype=dt))
        dev.profile_kernel(conv, [[xb, wb, yb]], warmup)
        us = dev.profile_kernel(conv, [[xb, wb, yb]], steps)
        dev.profile_kernel(mp, [[yb, pb]], warmup)
        us_p = dev.profile_kernel(mp, [[yb, pb]], steps)
        fused = dev.register_kernel(kernels.conv2d_desc(N, C, HW, HW, CO, 3, 3, padding=(1, 1), relu=True, dtype=dt, pool=True))
        dev.profile_kernel(fused, [[xb, wb, pb]], warmup)
        us_f = dev.profile_kernel(fused, [[xb, wb, pb]], steps)
        dev.release(fused)
        pool_bytes = (N * CO * HW * HW + N * CO * (HW // 2) ** 2) * isz
        peak = 157.3 if isz == 4 else 2500.0
        out[name] = {"conv_relu_us": round(us, 2), "conv_TFLOP/s": round(flop / us / 1e6, 1),
                     "conv_frac_of_peak": round(flop / us / 1e6 / peak, 4), "peak_TFLOP/s": peak,
                     "max_pool_us": round(us_p, 2), "max_pool_GB/s": round(pool_bytes / us_p / 1e3, 1),
                     "conv_relu_pool_one_launch_us": round(us_f, 2), "conv_relu_pool_two_launches_us": round(us + us_p, 2)}
        dev.release(conv)
        dev.release(mp)
        for b_ in (xb, wb, yb, pb):
            pool.deallocate(b_, [])
    return out


def extra_streaming(dev, pool, kernels, steps=20, warmup=5):
    """Memory-bound kernels at the transformer block's shapes: fused elementwise chains, column / row reductions,
    LayerNorm forward and backward. GB/s = (bytes of every input + output tensor, each once) / kernel time. Every kernel
    runs over rotating sets of buffers that together exceed 1 GiB, so that no launch finds its operands in the 256 MB
    Infinity Cache the launch before left behind (the same rule as the headline leg)."""
    import zyx_amd
    M, F, D = 8192, 4096, 1024
    rng = Rng(3)
    out = {}
    WORKING_SET = 1 << 30

    def dev_arr(a, dt):
        if dt == zyx_amd.DType.BF16:
            a = (a.view(np.uint32) >> 16).astype(np.uint16)
        b, e = kernels.to_device(pool, a)
        pool.sync_events([e])
        return b

    def out_arr(n, isz):
        b, e = kernels.alloc_like(pool, n, isz)
        pool.sync_events([e])
        return b

    def timeit(name, desc, make_args, nbytes):
        """make_args() allocates one set of argument buffers (inputs filled); nbytes = bytes one launch moves."""
        sets = [make_args() for _ in range(max(2, -(-WORKING_SET // nbytes)))]
        prog = dev.register_kernel(desc)
        dev.profile_kernel(prog, sets, max(warmup, len(sets)))
        us = dev.profile_kernel(prog, sets, max(steps, 2 * len(sets)))
        out[name] = {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1), "frac_of_8TB/s": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                     "buffer_sets": len(sets)}
        dev.release(prog)
        for b_ in {b for s_ in sets for b in s_}:
            pool.deallocate(b_, [])

    for dt, isz, tag in ((zyx_amd.DType.BF16, 2, "bf16"), (zyx_amd.DType.F32, 4, "f32")):
        big, row = rng.randn((M, F)), rng.randn((M, D))
        vec = rng.randn((D,))
        full = lambda: dev_arr(big, dt)
        c = kernels.Chain(M, F, out_dtype=dt)
        c.load(c.input(dt))
        timeit(f"copy_{tag}_8192x4096", c.desc(), lambda: [full(), out_arr(M * F, isz)], 2 * M * F * isz)  # the streaming ceiling of this part
        c = kernels.Chain(M, F, out_dtype=dt)
        c.load(c.input(dt)).gelu()
        timeit(f"gelu_{tag}_8192x4096", c.desc(), lambda: [full(), out_arr(M * F, isz)], 2 * M * F * isz)
        c = kernels.Chain(M, F, out_dtype=dt)
        a, b = c.input(dt), c.input(dt)
        c.load(a).gelu_grad().mul(b)
        timeit(f"gelu_grad_mul_{tag}_8192x4096", c.desc(), lambda: [full(), full(), out_arr(M * F, isz)], 3 * M * F * isz)
        c = kernels.Chain(M, F, out_dtype=dt)
        a, b = c.input(dt), c.input(dt)
        c.load(a).add(b)
        timeit(f"add_{tag}_8192x4096", c.desc(), lambda: [full(), full(), out_arr(M * F, isz)], 3 * M * F * isz)
        # the fused softmax (y, row sum, arg-max) on this storage type: x read once, y written once
        timeit(f"softmax_{tag}_8192x4096", kernels.softmax_rows_desc(M, F, dtype=dt),
               lambda: [full(), out_arr(M * F, isz), out_arr(M, isz), out_arr(M, 4)], 2 * M * F * isz + M * (isz + 4))
        timeit(f"colsum_{tag}_8192x4096", kernels.reduce_desc(M, F, "sum", axis0=True, dtype=dt), lambda: [full(), out_arr(F, isz)], M * F * isz)
        timeit(f"rowsum_{tag}_8192x4096", kernels.reduce_desc(M, F, "sum", dtype=dt), lambda: [full(), out_arr(M, isz)], M * F * isz)
        c = kernels.Chain(M, D, out_dtype=dt)
        c.load(c.input(dt))
        timeit(f"copy_{tag}_8192x1024", c.desc(), lambda: [dev_arr(row, dt), out_arr(M * D, isz)], 2 * M * D * isz)  # what a launch this small can reach
        w, bb = dev_arr(vec, dt), dev_arr(vec, dt)  # the affine parameters are shared by every set, as in a model
        timeit(f"layernorm_{tag}_8192x1024", kernels.norm_rows_desc(M, D, dtype=dt), lambda: [dev_arr(row, dt), w, bb, out_arr(M * D, isz)], 2 * M * D * isz)
        w, bb = dev_arr(vec, dt), dev_arr(vec, dt)
        timeit(f"layernorm_bwd_{tag}_8192x1024", kernels.norm_rows_bwd_desc(M, D, add=True, dtype=dt),
               lambda: [dev_arr(row, dt), w, dev_arr(row, dt), dev_arr(row, dt), out_arr(M * D, isz), out_arr(D, isz), out_arr(D, isz)], 4 * M * D * isz)
        # a width that is not 256 * 2^n: rows with lanes past their end
        D2 = 768
        row2, vec2 = rng.randn((M, D2)), rng.randn((D2,))
        w, bb = dev_arr(vec2, dt), dev_arr(vec2, dt)
        timeit(f"layernorm_{tag}_8192x768", kernels.norm_rows_desc(M, D2, dtype=dt), lambda: [dev_arr(row2, dt), w, bb, out_arr(M * D2, isz)], 2 * M * D2 * isz)
        w = dev_arr(vec2, dt)
        timeit(f"layernorm_bwd_{tag}_8192x768", kernels.norm_rows_bwd_desc(M, D2, add=True, dtype=dt),
               lambda: [dev_arr(row2, dt), w, dev_arr(row2, dt), dev_arr(row2, dt), out_arr(M * D2, isz), out_arr(D2, isz), out_arr(D2, isz)], 4 * M * D2 * isz)
    # cross-entropy (loss + gradient) over a language model's vocabulary: logits read once, gradient written once
    R, V = 2048, 32000
    logits, labels = rng.randn((R, V)), rng.randint((R,), 0, V).astype(np.int32)

    def ce_args():
        lb, e = kernels.to_device(pool, labels)
        pool.sync_events([e])
        return [dev_arr(logits, zyx_amd.DType.F32), lb, out_arr(R, 4), out_arr(R * V, 4)]
    timeit("cross_entropy_f32_2048x32000", kernels.cross_entropy_desc(R, V, True, True, 1.0 / R), ce_args, 2 * R * V * 4 + R * 8)
    return out


def extra_graph(dev, pool, steps=60, warmup=10):
    """Config 1 through the generic path: the training step written as graph nodes (zyx_amd/graph.py), differentiated
    by the reverse rules, lowered to generated kernels (products optionally matched to the GEMM kernel), kept as one
    plan; per step two host writes (batch, one-hot labels), one plan launch, four device-side parameter assignments."""
    import zyx_amd
    from zyx_amd.graph import Tape
    from zyx_amd.ir import BOp, UOp
    F32 = zyx_amd.DType.F32
    B, NIN, H, NOUT, LR = 64, 784, 128, 10, 0.01
    out = {}
    for match, in_place in ((False, False), (True, False), (True, True)):
        rng = Rng(42069)  # the same parameters and batches for all runs
        tape = Tape(dev, pool, match=match)
        g = tape.graph
        k1, k2 = 1 / np.sqrt(NIN), 1 / np.sqrt(H)
        x, onehot = tape.tensor(np.zeros((B, NIN)), F32), tape.tensor(np.zeros((B, NOUT)), F32)
        params = [tape.tensor(rng.uniform((H, NIN), -k1, k1), F32), tape.tensor(rng.uniform((H,), -k1, k1), F32),
                  tape.tensor(rng.uniform((NOUT, H), -k2, k2), F32), tape.tensor(rng.uniform((NOUT,), -k2, k2), F32)]
        h = g.relu(g.binary_b(g.dot(x, g.t(params[0])), params[1], BOp.Add))
        logits = g.binary_b(g.dot(h, g.t(params[2])), params[3], BOp.Add)
        loss = g.cross_entropy(logits, onehot, "mean")
        lr = g.const(LR, F32)
        new = [g.binary(p, g.binary(gr, lr, BOp.Mul), BOp.Sub) for p, gr in zip(params, tape.gradient(loss, params))]
        t0 = time.perf_counter()
        plan = tape.plan(new + [loss], updates=dict(zip(params, new)) if in_place else None, inputs=[x, onehot] if in_place else ())
        build_ms = (time.perf_counter() - t0) * 1e3
        xs = rng.randn((steps + warmup, B, NIN))
        hot = np.eye(NOUT, dtype=np.float32)[rng.randint((steps + warmup, B), 0, NOUT)]
        for i in range(steps + warmup):
            if i == warmup:
                tape.sync()
                t0 = time.perf_counter()
            tape.write(x, xs[i])
            tape.write(onehot, hot[i])
            plan.launch()
            if not in_place:
                for p, n in zip(params, new):
                    tape.assign(p, n)
        final = float(tape.numpy(loss)[0])
        sps = steps / (time.perf_counter() - t0)
        out["matched_updates_in_place" if in_place else "matched_to_kernels" if match else "generated_kernels_only"] = {
            "steps_per_s": round(sps, 1), "launches_per_step": plan.launches, "lower_and_compile_ms": round(build_ms, 1),
            "final_loss": round(final, 5)}
        tape.close()
    return out


def extra_ir(dev, pool, kernels, steps=20, warmup=5):
    """Kernels generated at run time from a linearized zyx kernel (Device::compile): the config-2 softmax rows written
    as such a kernel (row in registers, local-memory reductions) beside the hand-written one, and an elementwise map."""
    import zyx_amd
    from zyx_amd import ir_examples
    rng = Rng(4)
    out = {}
    x = rng.randn((ROWS, COLS), 3.0)
    sets, pending = [], []
    for _ in range(N_SETS):  # rotating buffer sets, like the headline run: no launch finds its rows in the cache
        xb, e1 = kernels.to_device(pool, x)
        yb, e2 = kernels.alloc_like(pool, ROWS * COLS, 4)
        sets.append([xb, yb])
        pending += [e1, e2]
    pool.sync_events(pending)

    def timeit(name, prog, nbytes):
        dev.profile_kernel(prog, sets, warmup)
        us = dev.profile_kernel(prog, sets, steps)
        out[name] = {"us": round(us, 2), "GB/s": round(nbytes / us / 1e3, 1), "frac_of_8TB/s": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}

    import time
    t0 = time.perf_counter()
    prog = dev.compile(ir_examples.softmax_rows_local(ROWS, COLS).to_bytes())
    out["compile_ms_softmax"] = round((time.perf_counter() - t0) * 1e3, 1)
    timeit(f"generated_softmax_f32_{ROWS}x{COLS}", prog, 2 * ROWS * COLS * 4)
    y = kernels.to_host(pool, sets[0][1], (ROWS, COLS), np.float32)
    e = np.exp(x[:8].astype(np.float64) - x[:8].max(1, keepdims=True))
    assert np.allclose(y[:8], e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-37), "generated softmax is wrong"
    dev.release(prog)
    hand = dev.register_kernel(kernels.softmax_rows_desc(ROWS, COLS, True, False, False))
    timeit(f"handwritten_softmax_f32_{ROWS}x{COLS}", hand, 2 * ROWS * COLS * 4)
    dev.release(hand)
    for dt, isz, tag in ((zyx_amd.DType.F32, 4, "f32"), (zyx_amd.DType.BF16, 2, "bf16")):
        n = ROWS * COLS
        prog = dev.compile(ir_examples.scaled_exp2(n, dt, vlen=4 if isz == 4 else 8).to_bytes())
        timeit(f"generated_exp2_scale_{tag}_{n}", prog, 2 * n * isz)
        dev.release(prog)
    for st in sets:
        for b in st:
            pool.deallocate(b, [])
    return out


def extra_attention(dev, pool, kernels, steps=30, warmup=10):
    """Config 5's attention core alone: B=8, T=1024, 16 heads x 64, bf16. FLOPs: 4*B*H*T*T*dh forward (QK^T, PV),
    10*B*H*T*T*dh backward (5 products; the two-kernel backward recomputes QK^T and dy.V^T, not counted)."""
    import zyx_amd
    B, T, H, DH = 8, 1024, 16, 64
    rng = Rng(6)
    trunc = lambda a: (a.view(np.uint32) >> 16).astype(np.uint16)
    qkv = trunc(rng.randn((B, T, 3 * H * DH)))
    dy = trunc(rng.randn((B, T, H * DH)))
    xb, e0 = kernels.to_device(pool, qkv)
    db, e1 = kernels.to_device(pool, dy)
    yb, e2 = kernels.alloc_like(pool, B * T * H * DH, 2)
    lb, e3 = kernels.alloc_like(pool, B * H * T, 4)
    gb, e4 = kernels.alloc_like(pool, B * T * 3 * H * DH, 2)
    pool.sync_events([e0, e1, e2, e3, e4])
    res = {}
    # causal: the T(T+1)/2 visible (query, key) pairs are what is counted
    for tag, causal, pairs in (("", False, float(T) * T), ("causal_", True, T * (T + 1) / 2.0)):
        fwd = dev.register_kernel(kernels.attention_desc(B, T, H, DH, zyx_amd.DType.BF16, lse=True, causal=causal))
        bwd = dev.register_kernel(kernels.attention_bwd_desc(B, T, H, DH, zyx_amd.DType.BF16, causal=causal))
        for name, prog, args, flop in ((tag + "forward", fwd, [xb, yb, lb], 4.0 * B * H * pairs * DH),
                                       (tag + "backward", bwd, [xb, yb, db, lb, gb], 10.0 * B * H * pairs * DH)):
            dev.profile_kernel(prog, [args], warmup)
            us = dev.profile_kernel(prog, [args], steps)
            res[name] = {"us": round(us, 2), "TFLOP/s": round(flop / us / 1e6, 1), "frac_of_2.5PF_bf16_peak": round(flop / us / 1e6 / 2500.0, 4)}
        dev.release(fwd)
        dev.release(bwd)
    for b_ in (xb, db, yb, lb, gb):
        pool.deallocate(b_, [])
    return res


def extra_block(dev, pool, steps=20, warmup=5, cpu=True):
    """Config 5: pre-norm transformer block B=8 T=1024 d=1024 16 heads, bf16, forward and forward + backward, each
    one cached plan launch (8 and 24 kernels). FLOPs counted: the matrix products only (240.5 GFLOP forward)."""
    import zyx_amd
    from zyx_amd.block import TransformerBlock
    B, T, D, H = 8, 1024, 1024, 16
    fwd_flop = 2.0 * B * T * (3 * D * D + D * D + 8 * D * D) + 4.0 * B * H * T * T * (D // H)
    blk = TransformerBlock(dev, pool, B, T, D, H, zyx_amd.DType.BF16)
    trunc = lambda a: (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    # config 5's parameters: Linear weights 0.02 * randn and zero biases (nanogpt.rs:121-125), LayerNorm weight 1 / bias 0
    prng = Rng(42069)
    w = lambda *shape: prng.randn(shape, 0.02)
    z = lambda n: np.zeros(n, np.float32)
    params = dict(ln1_w=np.ones(D, np.float32), ln1_b=z(D), attn_w=w(3 * D, D), attn_b=z(3 * D), proj_w=w(D, D), proj_b=z(D),
                  ln2_w=np.ones(D, np.float32), ln2_b=z(D), fc_w=w(4 * D, D), fc_b=z(4 * D), proj2_w=w(D, 4 * D), proj2_b=z(D))
    blk.set_params({k: trunc(v) for k, v in params.items()})
    rng = Rng(5)
    x = rng.randn((B * T, D))
    blk.write("x", trunc(x))
    blk.write("dout", trunc(np.ones((B * T, D), np.float32)))
    res = {"kernels_forward": len(blk.forward_nodes), "kernels_forward_backward": len(blk.forward_nodes) + len(blk.backward_nodes)}
    for name, fn, flop in (("forward", blk.forward, fwd_flop), ("forward_backward", blk.forward_backward, 3 * fwd_flop),
                           ("forward_backward_launch_by_launch", blk.forward_backward_unplanned, 3 * fwd_flop)):
        for _ in range(warmup):
            fn()
        blk.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        blk.sync()
        ms = (time.perf_counter() - t0) / steps * 1e3
        res[name] = {"ms": round(ms, 3), "TFLOP/s": round(flop / ms / 1e9, 1), "frac_of_2.5PF_bf16_peak": round(flop / ms / 1e9 / 2500.0, 4)}
    blk.close()
    if cpu:
        import oracle  # the CPU comparison leg only
        # one attention head pair and 64 rows of each Linear on the host cores, scaled to the whole forward
        sub = trunc(rng.randn((1, T, 3 * 128)))
        t0 = time.perf_counter()
        oracle.attention(sub, 2, dtype=oracle.BF16)
        t_att = (time.perf_counter() - t0) * (B * H / 2)
        rows = trunc(x[:64])
        t0 = time.perf_counter()
        for w in ("attn_w", "proj_w", "fc_w"):
            oracle.linear(rows, trunc(params[w]), dtype=oracle.BF16)
        oracle.linear(trunc(rng.randn((64, 4 * D))), trunc(params["proj2_w"]), dtype=oracle.BF16)
        t_lin = (time.perf_counter() - t0) * (B * T / 64)
        res["cpu_oracle_forward_s_extrapolated"] = round(t_att + t_lin, 2)
        res["cpu_sample"] = "2 of 128 (batch, head) attention problems and 64 of 8192 rows of the four Linear layers"
    return res


def zyx_dtype_bf16():
    import zyx_amd
    return zyx_amd.DType.BF16


def extra_mlp(dev, pool, steps=100, cpu=True):
    """Config 1: MLP 784->128->10, batch 64, SGD 0.01, 100 steps; steps 10..99 timed. GPU: per step two
    device-to-device batch copies out of the resident dataset and one cached plan launch (8 launch nodes: the weight
    updates ride in the weight-gradient GEMMs' epilogues, the bias updates in their column sums, the loss mean in the
    cross-entropy launch, the ReLU gradient in the epilogue of the product that feeds it)."""
    from zyx_amd.training import MLPTrainStep
    B, NIN, H, NOUT, LR = 64, 784, 128, 10, 0.01
    rng = Rng(42069)
    k1, k2 = 1 / np.sqrt(NIN), 1 / np.sqrt(H)
    w1, b1 = rng.uniform((H, NIN), -k1, k1), rng.uniform(H, -k1, k1)
    w2, b2 = rng.uniform((NOUT, H), -k2, k2), rng.uniform(NOUT, -k2, k2)
    xs = rng.randn((steps, B, NIN))
    ys = rng.randint((steps, B), 0, NOUT)
    m = MLPTrainStep(dev, pool, B, NIN, H, NOUT, LR, fused_update=True)
    m.set_params(w1, b1, w2, b2)
    from zyx_amd import kernels as K
    xb, e1 = K.to_device(pool, xs)  # the whole synthetic dataset is resident in HBM before timing
    yb, e2 = K.to_device(pool, ys)
    pool.sync_events([e1, e2])
    t0 = None
    for i in range(steps):
        if i == 10:
            pool.sync_events(m._pending)
            m._pending = []
            t0 = time.perf_counter()
        m.set_batch_from_device(xb, yb, i)
        m.step()
    final = m.mean_loss()  # blocks until the last step is done
    gpu_sps = (steps - 10) / (time.perf_counter() - t0)
    n_nodes = len(m.nodes)
    m.close()
    pool.deallocate(xb, [])
    pool.deallocate(yb, [])
    res = {"gpu_steps_per_s": round(gpu_sps, 1), "launches_per_step": n_nodes, "final_loss": round(final, 5)}
    if cpu:
        import oracle
        p = (w1, b1, w2, b2)
        for i in range(steps):
            if i == 10:
                t0 = time.perf_counter()
            loss, *p, _ = oracle.mlp_step(xs[i], ys[i], *p, LR)
            p = tuple(p)
        res["cpu_oracle_steps_per_s"] = round((steps - 10) / (time.perf_counter() - t0), 1)
        res["cpu_final_loss"] = round(float(loss), 5)
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="only the headline workload (used for profiling)")
    ap.add_argument("--gemm-only", action="store_true",
                    help="run only the config-3 GEMM leg and print its numbers (used for profiling that kernel)")
    ap.add_argument("--conv-only", action="store_true", help="run only the config-4 conv + max-pool leg")
    ap.add_argument("--block-only", action="store_true", help="run only the config-5 transformer block leg")
    ap.add_argument("--mlp-only", action="store_true", help="run only the config-1 MLP training leg")
    ap.add_argument("--streaming-only", action="store_true", help="run only the memory-bound kernel leg")
    ap.add_argument("--attention-only", action="store_true", help="run only the attention core leg")
    ap.add_argument("--ir-only", action="store_true", help="run only the generated-kernel leg")
    ap.add_argument("--graph-only", action="store_true", help="run only the config-1 training step through the graph path")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="run only the ceiling probes (hipMemcpy device to device, copy and read-only kernels, bf16 "
                         "matrix-instruction loops on constant and on random operands) and print them")
    ap.add_argument("--counters", action="store_true",
                    help="short run for `rocprofv3 --pmc`: a few launches of the fused kernel and of a plain copy "
                         "kernel over the same 8192x4096 f32 tensor (known traffic: 134217728 B read + written), "
                         "then exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend drives one GPU per context and this build measures one GPU only; "
                 "run with --gpus 1")

    import zyx_amd
    from zyx_amd import kernels

    pools, devices = zyx_amd.initialize_device(zyx_amd.HIPConfig(device_ids=[0]))
    pool, dev = pools[0], devices[0]
    info = dev.info()

    if args.mfma_ceiling:
        print(json.dumps({"measured_ceilings": measured_ceilings(dev)}))
        pool.deinitialize()
        return

    if args.gemm_only:
        res = extra_gemm(dev, pool, kernels, steps=args.steps, warmup=max(args.warmup, 100))
        res["measured_ceilings"] = measured_ceilings(dev)
        print(json.dumps({"config3_gemm_bf16_4096": res}))
        pool.deinitialize()
        return

    if args.conv_only or args.block_only or args.streaming_only or args.attention_only or args.mlp_only or args.ir_only or args.graph_only:
        if args.mlp_only:
            res = {"config1_mlp_train": extra_mlp(dev, pool, cpu=not args.no_cpu)}
        elif args.conv_only:
            res = {"config4_conv_relu_pool": extra_conv(dev, pool, kernels)}
        elif args.streaming_only:
            res = {"memory_bound_kernels": extra_streaming(dev, pool, kernels)}
        elif args.attention_only:
            res = {"config5_attention_core": extra_attention(dev, pool, kernels)}
        elif args.ir_only:
            res = {"generated_kernels": extra_ir(dev, pool, kernels)}
        elif args.graph_only:
            res = {"config1_mlp_train_graph_path": extra_graph(dev, pool)}
        else:
            res = {"config5_transformer_block": extra_block(dev, pool, steps=args.steps if args.steps != 200 else 20, cpu=not args.no_cpu)}
        print(json.dumps(res))
        pool.deinitialize()
        return

    rng = Rng(42069)
    x = rng.randn((ROWS, COLS), 3.0)

    prog = dev.register_kernel(kernels.softmax_rows_desc(ROWS, COLS))
    sets, pending = [], []
    for _ in range(N_SETS):
        xb, ev = kernels.to_device(pool, x)
        pending.append(ev)
        outs = []
        for n in (ROWS * COLS, ROWS, ROWS):
            b, e = kernels.alloc_like(pool, n, 4)
            outs.append(b)
            pending.append(e)
        sets.append([xb] + outs)
    pool.sync_events(pending)

    def run(n):
        # each step waits on the previous one: the chain stays on one in-order launch stream, so
        # a profiler sees back-to-back, non-overlapping dispatches
        ev = []
        for i in range(n):
            ev = [dev.launch(prog, pool, sets[i % N_SETS], ev)]
        pool.sync_events(ev)

    if args.counters:
        copy = kernels.Chain(ROWS, COLS)
        copy.load(copy.input())
        cprog = dev.register_kernel(copy.desc())
        ev = []
        for i in range(5):
            ev = [dev.launch(prog, pool, sets[i % N_SETS], ev)]
        for i in range(5):
            ev = [dev.launch(cprog, pool, [sets[i % N_SETS][0], sets[(i + 1) % N_SETS][1]], ev)]
        pool.sync_events(ev)
        print(json.dumps({"counters_run": True, "softmax_launches": 5, "copy_launches": 5,
                          "copy_bytes_read": ROWS * COLS * 4, "copy_bytes_written": ROWS * COLS * 4}))
        pool.deinitialize()
        return

    run(args.warmup)
    t0 = time.perf_counter()
    run(args.steps)
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = ALGO_BYTES * args.steps / wall / 1e9

    # the kernel's own duration: HIP events on the stream it is launched on
    dev.profile_kernel(prog, sets, max(args.warmup, N_SETS))
    us = dev.profile_kernel(prog, sets, args.steps)
    achieved = ALGO_BYTES / (us * 1e-6) / 1e9

    # spot check that the timed kernel produced the right thing (first rows, numpy float64)
    y = kernels.to_host(pool, sets[0][1], (ROWS, COLS), np.float32)
    e = np.exp(x[:8].astype(np.float64) - x[:8].max(1, keepdims=True))
    assert np.allclose(y[:8], e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-37), "bench output is wrong"

    out = {
        "metric": "fused_softmax_rowsum_argmax_f32_GBps", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"config 2: fused row softmax + row-sum + row-argmax, f32 {ROWS}x{COLS}, N(0,3^2), "
                               f"{N_SETS} rotating buffer sets resident in HBM",
                   "algorithmic_bytes_per_step": ALGO_BYTES, "device": info.name, "arch": info.arch,
                   "compute_units": info.compute_units},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": TRAFFIC_BYTES,
                     "kernel": "softmax_rows_split_k<4, 4>", "avg_launch_us": round(us, 3)},
    }
    for s in sets:
        for b in s:
            pool.deallocate(b, [])
    dev.release(prog)
    ceil = measured_ceilings(dev)
    out["config"]["measured_ceilings"] = ceil
    out["roofline"]["frac_of_measured_copy_kernel"] = round(achieved / ceil["copy_kernel_GBps"], 4) if ceil["copy_kernel_GBps"] else None
    if not args.no_extra:
        # other configs of the same backend, reported beside the headline (not part of `value`)
        out["extra"] = {"config3_gemm_bf16_4096": extra_gemm(dev, pool, kernels),
                        "config1_mlp_train": extra_mlp(dev, pool, cpu=not args.no_cpu),
                        "config4_conv_relu_pool": extra_conv(dev, pool, kernels),
                        "config5_attention_core": extra_attention(dev, pool, kernels),
                        "config5_transformer_block": extra_block(dev, pool, cpu=not args.no_cpu),
                        "memory_bound_kernels": extra_streaming(dev, pool, kernels),
                        "generated_kernels": extra_ir(dev, pool, kernels),
                        "config1_mlp_train_graph_path": extra_graph(dev, pool)}
    pool.deinitialize()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(x)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
