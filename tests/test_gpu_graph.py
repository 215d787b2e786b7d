"""zyx_amd.graph on the GPU: graphs and their gradients realised by `Tape` (lowered kernels compiled and launched
through the C ABI) against the CPU evaluation of the same graph (oracle/graph_eval.py) and the gradients
zyx/tests/11_autograd.rs asserts. Bar: bit-exact for integer graphs and for float graphs made of + - * / max,
comparisons, casts and movement ops (same serial order, no contraction); within 1e-5 relative (f32) / 1e-12 (f64)
where exp / log / sin / cos / pow / sqrt are involved."""
import numpy as np
import pytest

from graph_cases import CASES, mixed_graph, mlp_graph
from oracle import graph_eval
from zyx_amd import DType
from zyx_amd.graph import Tape, storage_dtype
from zyx_amd.ir import BOp, UOp

pytestmark = pytest.mark.gpu

_EXACT_UOPS = (UOp.Neg, UOp.Reciprocal, UOp.Floor, UOp.Trunc, UOp.Abs, UOp.BitNot)


def on_device(hip, build, *args, **kw):
    dev, pool = hip
    tape, leaves = Tape(dev, pool), {}

    def leaf(array, dtype):
        a = np.ascontiguousarray(np.asarray(array).astype(storage_dtype(dtype)))
        nid = tape.tensor(a, dtype)
        leaves[nid] = a
        return nid

    return tape, leaves, build(tape.graph, leaf, *args, **kw)


def is_exact(g, nodes):
    """No transcendental op anywhere below these nodes."""
    seen, stack = set(), list(nodes)
    while stack:
        i = stack.pop()
        if i in seen:
            continue
        seen.add(i)
        n = g[i]
        if (n.kind == "unary" and n.op not in _EXACT_UOPS) or (n.kind == "binary" and n.op == BOp.Pow):
            return False
        stack.extend(n.src)
    return True


def compare(tape, leaves, nodes, rtol):
    g = tape.graph
    want = graph_eval.evaluate(g.nodes, leaves, nodes)
    tape.realize(nodes)
    for nid in nodes:
        got = tape.numpy(nid)
        assert got.dtype == want[nid].dtype and got.shape == want[nid].shape
        if is_exact(g, [nid]):
            assert np.array_equal(got, want[nid], equal_nan=True), nid
        else:
            np.testing.assert_allclose(got, want[nid], rtol=rtol, atol=0)
    return want


@pytest.mark.parametrize("name,build", CASES, ids=[c[0] for c in CASES])
def test_reference_gradients(hip, name, build):
    tape, leaves, (target, sources, expected) = on_device(hip, build)
    try:
        grads = tape.gradient(target, sources)
        f64 = any(tape.graph[s].dtype == DType.F64 for s in sources)
        compare(tape, leaves, grads + [target], 1e-12 if f64 else 1e-5)
        for gid, src, exp in zip(grads, sources, expected):
            if exp is None:
                continue
            got = tape.numpy(gid)
            if tape.graph[src].dtype in (DType.F32, DType.F64):
                np.testing.assert_allclose(got, exp, rtol=1e-12 if f64 else 1e-5, atol=0)
            else:
                assert got.tolist() == np.asarray(exp).tolist()
    finally:
        tape.close()


@pytest.mark.parametrize("dtype,rtol", [(DType.F64, 1e-11), (DType.F32, 2e-4)])
def test_every_rule(hip, dtype, rtol):
    """f32: the loss sums exponentials of sines of products, so a few ulp in one function move the result by more
    than 1e-5 of some gradient entries that cancel; the f64 run holds the tight bar."""
    tape, leaves, (loss, sources) = on_device(hip, mixed_graph, dtype=dtype)
    try:
        grads = tape.gradient(loss, sources)
        compare(tape, leaves, grads + [loss], rtol)
    finally:
        tape.close()


@pytest.mark.parametrize("shape", [dict(batch=8, n_in=12, hidden=16, n_out=5), dict(batch=64, n_in=784, hidden=128, n_out=10)])
def test_mlp_gradients(hip, shape):
    """zz_bw_relu_matmul (11_autograd.rs:908-927), at a small size and at the size of the MNIST network: gradients
    of sum(logits) and one SGD step `w - g * lr` realised on the device, against the evaluation of the same graph
    (exact: only + * and comparisons) and the closed-form backward products in f64."""
    tape, leaves, (loss, sources, (x, w1, b1, w2, b2)) = on_device(hip, mlp_graph, **shape)
    try:
        g = tape.graph
        grads = tape.gradient(loss, sources)
        lr = g.const(0.01, DType.F32)
        new = [g.binary(s, g.binary(gr, lr, BOp.Mul), BOp.Sub) for s, gr in zip(sources, grads)]
        want = compare(tape, leaves, grads + new + [loss], 1e-5)
        X, W1, B1, W2 = (leaves[i].astype(np.float64) for i in (x, w1, b1, w2))
        pre = X @ W1.T + B1
        dh = (np.ones((X.shape[0], W2.shape[0])) @ W2) * (pre > 0)
        ref = [dh.T @ X, dh.sum(0), np.ones((W2.shape[0], X.shape[0])) @ np.maximum(pre, 0), np.full(W2.shape[0], X.shape[0])]
        for gid, r in zip(grads, ref):
            np.testing.assert_allclose(tape.numpy(gid), r, rtol=1e-4, atol=1e-4 * np.abs(r).max())
    finally:
        tape.close()


def test_movement_and_reduce_at_size(hip):
    """Index arithmetic of every movement op and both reduces on tensors of a few hundred thousand elements."""
    dev, pool = hip
    tape = Tape(dev, pool)
    try:
        r = np.random.default_rng(5)
        g = tape.graph
        xa = r.integers(-100, 100, (37, 129, 65)).astype(np.int32)
        x = tape.tensor(xa, DType.I32)
        a = g.flip(g.permute(x, [2, 0, 1]), [0, 2])                       # [65, 37, 129]
        b = g.reduce(a, BOp.Add, [1])                                     # [65, 129]
        c = g.reduce(g.binary(a, g.expand(g.reshape(b, [65, 1, 129]), [65, 37, 129]), BOp.Mul), BOp.Max, [0, 2])  # [37]
        d = g.expand(g.reshape(c, [37, 1]), [3, 37, 5])
        tape.realize([a, b, c, d])
        A = np.flip(np.transpose(xa, (2, 0, 1)), (0, 2))
        B = A.sum(1, dtype=np.int32)
        Cc = (A * B[:, None, :]).max((0, 2))
        assert np.array_equal(tape.numpy(a), A) and np.array_equal(tape.numpy(b), B)
        assert np.array_equal(tape.numpy(c), Cc)
        assert np.array_equal(tape.numpy(d), np.broadcast_to(Cc.reshape(37, 1), (3, 37, 5)))
    finally:
        tape.close()


def test_programs_are_compiled_once(hip):
    dev, pool = hip
    tape = Tape(dev, pool)
    try:
        g = tape.graph
        xs = [tape.tensor(np.full(100, i, np.float32), DType.F32) for i in range(4)]
        outs = [g.binary(x, g.const(2.0, DType.F32), BOp.Mul) for x in xs]
        tape.realize(outs)
        assert len(tape._programs) == 1
        assert [tape.numpy(o)[0] for o in outs] == [0.0, 2.0, 4.0, 6.0]
    finally:
        tape.close()


@pytest.mark.parametrize("causal,p", [(False, 0.0), (True, 0.25)])
def test_fused_attention_against_the_graph_path(hip, causal, p):
    """Two independent routes on the device: the fused attention kernels (forward + backward) and the same maths
    as graph nodes differentiated by the reverse rules and run as generated kernels. f32 both; they sum in
    different orders, so the bar is 1e-5 of the largest magnitude of each tensor."""
    from graph_cases import attention_graph
    from zyx_amd import kernels as K
    dev, pool = hip
    tape, leaves, (loss, sources, (y, arrs)) = on_device(hip, attention_graph, causal=causal, p=p)
    try:
        grads = tape.gradient(loss, sources)
        tape.realize(grads + [y])
        b, h, t, dh = arrs["q"].shape
        pack = lambda a: np.ascontiguousarray(a.transpose(0, 2, 1, 3).reshape(b, t, h * dh))  # [B,H,T,dh] -> [B,T,C]
        qkv = np.concatenate([pack(arrs[n]) for n in ("q", "k", "v")], 2).astype(np.float32)
        y_f, lse = K.attention(dev, pool, qkv, h, DType.F32, dropout_p=p, want_lse=True, causal=causal)
        dqkv = K.attention_bwd(dev, pool, qkv, y_f, pack(arrs["dy"]).astype(np.float32), lse, h, DType.F32, dropout_p=p, causal=causal)
        y_g = pack(tape.numpy(y))
        np.testing.assert_allclose(y_f, y_g, rtol=0, atol=1e-5 * np.abs(y_g).max())
        for i, gid in enumerate(grads):
            g_g = pack(tape.numpy(gid))
            np.testing.assert_allclose(dqkv[:, :, i * h * dh:(i + 1) * h * dh], g_g, rtol=0, atol=2e-5 * np.abs(g_g).max())
    finally:
        tape.close()


@pytest.mark.parametrize("dtype,rtol", [(DType.F64, 1e-10), (DType.F32, 1e-4)])
def test_attention_with_training_dropout(hip, dtype, rtol):
    """Training-mode dropout inside attention (`probability.cmplt(rand) * att`, tensor/mod.rs:822-828) through the
    graph path, forward and gradients, against the CPU evaluation of the same graph."""
    from graph_cases import attention_graph
    tape, leaves, (loss, sources, (y, arrs)) = on_device(hip, attention_graph, causal=True, p=0.3, training=True, dtype=dtype)
    try:
        grads = tape.gradient(loss, sources)
        nodes = grads + [y]
        want = graph_eval.evaluate(tape.graph.nodes, leaves, nodes)
        tape.realize(nodes)
        for nid in nodes:
            np.testing.assert_allclose(tape.numpy(nid), want[nid], rtol=0, atol=rtol * np.abs(want[nid]).max())
    finally:
        tape.close()


# ---- products matched to the hand-written GEMM ---------------------------------------------------------------------------

def _dense_mlp(g, leaf, **shape):
    loss, sources, leaves5 = mlp_graph(g, leaf, **shape)
    logits = g[loss].src[0]
    return g.sum_all(g.binary(logits, logits, BOp.Mul)), sources, leaves5


def matched_tape(hip, build, match=True, **kw):
    dev, pool = hip
    tape, leaves = Tape(dev, pool, match=match), {}

    def leaf(array, dtype):
        a = np.ascontiguousarray(np.asarray(array).astype(storage_dtype(dtype)))
        nid = tape.tensor(a, dtype)
        leaves[nid] = a
        return nid

    return tape, leaves, build(tape.graph, leaf, **kw)


def test_mlp_products_run_on_the_gemm_kernel(hip):
    """The MNIST-size network with a dense upstream gradient: the two forward and the three backward products are
    launched as GEMMs reading the operands in place (weights [out, in], x and dY through trans_a); f32, bar 1e-5 of
    each tensor's magnitude against the CPU evaluation of the graph (the GEMM sums in another order)."""
    tape, leaves, (loss, sources, _) = matched_tape(hip, _dense_mlp, batch=64, n_in=784, hidden=128, n_out=10)
    try:
        grads = tape.gradient(loss, sources)
        want = graph_eval.evaluate(tape.graph.nodes, leaves, grads + [loss])
        tape.realize(grads + [loss])
        assert tape.matched == 5
        for nid in grads + [loss]:
            np.testing.assert_allclose(tape.numpy(nid), want[nid], rtol=0, atol=1e-5 * np.abs(want[nid]).max())
    finally:
        tape.close()


@pytest.mark.parametrize("causal", [False, True])
def test_attention_products_run_on_the_batched_gemm(hip, causal):
    from graph_cases import attention_graph
    tape, leaves, (loss, sources, (y, _)) = matched_tape(hip, attention_graph, causal=causal, p=0.1, t=40, dh=16)
    try:
        grads = tape.gradient(loss, sources)
        want = graph_eval.evaluate(tape.graph.nodes, leaves, grads + [y])
        tape.realize(grads + [y])
        assert tape.matched == 7   # six batched products and the softmax over keys
        for nid in grads + [y]:
            np.testing.assert_allclose(tape.numpy(nid), want[nid], rtol=0, atol=3e-5 * np.abs(want[nid]).max())
    finally:
        tape.close()


def test_gemm_and_generated_kernel_compete_on_time(hip):
    """A 512^3 product: both candidates are timed with the autotuner's clock and the GEMM wins by a wide margin (the
    generated kernel is one serial loop per output element)."""
    def build(g, leaf):
        r = np.random.default_rng(9)
        a, b = leaf(r.standard_normal((512, 512)), DType.F32), leaf(r.standard_normal((512, 512)), DType.F32)
        return g.dot(a, b), (a, b)

    tape, leaves, (out, (a, b)) = matched_tape(hip, build, match="time")
    try:
        tape.realize([out])
        (c, t_gemm, t_gen), = tape.timings
        assert (c.m, c.n, c.k, c.trans_a, c.trans_b) == (512, 512, 512, False, False)
        assert t_gemm < t_gen and tape.matched == 1
        ref = leaves[a].astype(np.float64) @ leaves[b].astype(np.float64)
        np.testing.assert_allclose(tape.numpy(out), ref, rtol=0, atol=1e-5 * np.abs(ref).max())
        print(f"512^3 f32: GEMM {t_gemm / 1e3:.1f} us, generated kernel {t_gen / 1e3:.1f} us")
    finally:
        tape.close()


def test_softmax_runs_on_the_fused_kernel(hip):
    """`Tensor::softmax` over the last axis of a graph tensor is launched as the fused row-softmax kernel (one pass)
    in place of two reduces and a map; f32 within 2e-6 relative of the CPU evaluation (exp and summation order)."""
    def build(g, leaf):
        x = leaf(3 * np.random.default_rng(4).standard_normal((4, 128, 4096)), DType.F32)
        return g.softmax(x, [-1]), x

    tape, leaves, (sm, x) = matched_tape(hip, build)
    try:
        tape.realize([sm])
        assert tape.matched == 1 and len(tape._programs) == 1
        got = tape.numpy(sm)
        xv = leaves[x].astype(np.float64)
        e = np.exp(xv - xv.max(-1, keepdims=True))
        np.testing.assert_allclose(got, e / e.sum(-1, keepdims=True), rtol=2e-6, atol=1e-12)
    finally:
        tape.close()


@pytest.mark.parametrize("match", [False, True])
def test_training_steps_as_a_cached_plan(hip, oracle, match):
    """Twelve SGD steps of the MNIST-size network: the whole step (forward, cross entropy, gradients by the reverse
    rules, updates) is lowered once, kept as one plan and replayed; new batches are written into the leaves and the
    updated parameters assigned back on the device. Loss curve and final parameters against the CPU oracle's
    training step on the same data."""
    from graph_cases import mlp_training_graph
    tape, leaves, (loss, new, params, (x, onehot)) = matched_tape(hip, mlp_training_graph, match=match)
    try:
        plan = tape.plan(new + [loss])
        r = np.random.default_rng(11)
        p = [leaves[i].copy() for i in params]
        for step in range(12):
            xs = r.standard_normal((64, 784)).astype(np.float32)
            lab = r.integers(0, 10, 64).astype(np.int32)
            tape.write(x, xs)
            tape.write(onehot, np.eye(10, dtype=np.float32)[lab])
            plan.launch()
            got_loss = tape.numpy(loss)
            for leaf_id, n in zip(params, new):
                tape.assign(leaf_id, n)
            want_loss, *p, _ = oracle.mlp_step(xs, lab, *p, 0.01)
            np.testing.assert_allclose(got_loss, [want_loss], rtol=2e-5)
        for leaf_id, w in zip(params, p):
            np.testing.assert_allclose(tape.numpy(leaf_id), w, rtol=1e-4, atol=1e-6)
        assert (tape.matched >= 5) == bool(match)
        print(f"match={match}: {plan.launches} launches per step")
    finally:
        tape.close()


def test_training_steps_with_fused_launches_and_in_place_updates(hip, oracle):
    """The same twelve steps with every matcher on and the parameter updates declared to the plan: eight launches per
    step (the list zyx_amd/training.py writes by hand), no copies between steps; loss curve and final parameters
    against the CPU oracle's training step."""
    from graph_cases import mlp_training_graph
    tape, leaves, (loss, new, params, (x, onehot)) = matched_tape(hip, mlp_training_graph, match=True)
    try:
        plan = tape.plan(new + [loss], updates=dict(zip(params, new)), inputs=[x, onehot])
        assert plan.launches == 8 and tape.matched == 8
        r = np.random.default_rng(11)
        p = [leaves[i].copy() for i in params]
        for step in range(12):
            xs = r.standard_normal((64, 784)).astype(np.float32)
            lab = r.integers(0, 10, 64).astype(np.int32)
            tape.write(x, xs)
            tape.write(onehot, np.eye(10, dtype=np.float32)[lab])
            plan.launch()
            want_loss, *p, _ = oracle.mlp_step(xs, lab, *p, 0.01)
            if step % 5 == 0 or step == 11:
                np.testing.assert_allclose(tape.numpy(loss), [want_loss], rtol=2e-5)
                for leaf_id, w in zip(params, p):  # the leaves hold the updated parameters after every launch
                    np.testing.assert_allclose(tape.numpy(leaf_id), w, rtol=1e-4, atol=1e-6)
        with pytest.raises(ValueError):
            tape.plan(new + [loss], updates={params[0]: new[1]})
    finally:
        tape.close()


def test_cross_entropy_with_dense_targets(hip, oracle):
    """ZHIP_K_CROSS_ENTROPY with an f32 target tensor: one-hot targets give what class indices give; soft targets give
    -sum(ln_softmax * t) and (softmax * sum t - t) * scale."""
    from zyx_amd import kernels
    dev, pool = hip
    r = np.random.default_rng(3)
    for rows, cols in ((64, 10), (33, 1000), (5, 1)):
        X = (r.standard_normal((rows, cols)) * 3).astype(np.float32)
        lab = r.integers(0, cols, rows).astype(np.int32)
        l0, g0, m0 = kernels.cross_entropy(dev, pool, X, lab, 1.0 / rows, mean=True)
        l1, g1, m1 = kernels.cross_entropy(dev, pool, X, np.eye(cols, dtype=np.float32)[lab], 1.0 / rows, mean=True, dense=True)
        np.testing.assert_allclose(l1, l0, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(g1, g0, rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(m1, m0, rtol=1e-6)
        T = r.random((rows, cols)).astype(np.float32)
        l2, g2 = kernels.cross_entropy(dev, pool, X, T, 0.5, dense=True)
        x64 = X.astype(np.float64)
        m = x64 - x64.max(1, keepdims=True)
        ls = m - np.log(np.exp(m).sum(1, keepdims=True))
        np.testing.assert_allclose(l2, (-ls * T).sum(1), rtol=2e-5, atol=1e-6)
        np.testing.assert_allclose(g2, (np.exp(ls) * T.sum(1, keepdims=True) - T) * 0.5, rtol=2e-5, atol=1e-6)


def test_long_reductions_run_on_the_reduce_kernel(hip):
    """Row sums, a maximum over the trailing axes and an integer column sum of tensors with buffers are launched as
    the two-stage reduce kernel; integers and maxima exact, float sums to 1e-5 of sum |x|."""
    def build(g, leaf):
        r = np.random.default_rng(8)
        x = leaf(r.standard_normal((64, 16, 4096)), DType.F32)
        y = leaf(r.integers(-100, 100, (5000, 33)), DType.I32)
        return (g.reduce(x, BOp.Add, [2]), g.reduce(x, BOp.Max, [1, 2]), g.reduce(y, BOp.Add, [0])), (x, y)

    tape, leaves, ((rs, mx, cs), (x, y)) = matched_tape(hip, build)
    try:
        tape.realize([rs, mx, cs])
        assert tape.matched == 3
        xv = leaves[x].astype(np.float64)
        np.testing.assert_allclose(tape.numpy(rs), xv.sum(2), rtol=0, atol=1e-5 * np.abs(xv).sum(2).max())
        assert np.array_equal(tape.numpy(mx), leaves[x].max((1, 2))) and np.array_equal(tape.numpy(cs), leaves[y].sum(0, dtype=np.int32))
    finally:
        tape.close()


def test_launch_chain_survives_a_write_to_an_unrelated_leaf(hip):
    """realize -> write of a leaf the next kernel does not read -> realize of a dependant of the first result: the
    second launch must still be ordered after the first (the chain continues in the copy's event). A long serial
    reduce makes the first kernel slow enough that an unordered second launch would read unfinished data."""
    dev, pool = hip
    tape = Tape(dev, pool)
    try:
        g = tape.graph
        n = 1 << 22
        xa = np.arange(n, dtype=np.int32).reshape(4, n // 4) % 1000
        x = tape.tensor(xa, DType.I32)
        other = tape.tensor(np.zeros(16, np.int32), DType.I32)
        other2 = tape.tensor(np.zeros(16, np.int32), DType.I32)
        keep = g.binary(other, g.const(0, DType.I32), BOp.Add)
        tape.realize([keep])
        for rep in range(3):
            a = g.reduce(g.binary(x, g.const(rep, DType.I32), BOp.Add), BOp.Add, [1])   # 4 serial sums of a million terms each
            base = (xa + rep).sum(1, dtype=np.int32)
            tape.realize([a])
            tape.write(other, np.full(16, rep, np.int32))     # pool-stream copy between the two launches
            b = g.binary(a, g.const(2 + rep, DType.I32), BOp.Mul)
            tape.realize([b])
            tape.assign(other2, keep)                          # a device-side copy between the next two
            c = g.binary(b, g.const(1, DType.I32), BOp.Add)
            tape.realize([c])
            assert np.array_equal(tape.numpy(c), base * (2 + rep) + 1)
            assert np.array_equal(tape.numpy(b), base * (2 + rep))
        assert tape.numpy(other).tolist() == [2] * 16
    finally:
        tape.close()
