"""zyx_amd.graph on the CPU: the reverse rules against the gradients zyx/tests/11_autograd.rs asserts, finite
differences and closed forms (evaluated by oracle/graph_eval.py), and the lowered kernels executed by the kernel
interpreter (oracle/ir_interp.py) against that evaluation, bit for bit."""
import numpy as np
import pytest

from graph_cases import CASES, mixed_graph, mlp_graph
from oracle import graph_eval, ir_interp
from zyx_amd import DType
from zyx_amd.graph import (Alias, AttentionBwdMatch, AttentionMatch, Contraction, Conv2dMatch, CrossEntropyMatch, Graph, NormBwdMatch, NormRowsMatch, MaxPoolMatch, RowColReduce, SoftmaxRows, lower, match_reduce, match_softmax, match_contraction, storage_dtype, view_of)
from zyx_amd.ir import BOp, UOp

_FLOAT = (DType.F32, DType.F64)


def _build(build, *args, **kw):
    g, leaves = Graph(), {}

    def leaf(array, dtype):
        a = np.ascontiguousarray(np.asarray(array).astype(storage_dtype(dtype)))
        nid = g.leaf(a.shape, dtype)
        leaves[nid] = a
        return nid

    return g, leaves, build(g, leaf, *args, **kw)


def conv_textbook(x, w, bias, stride, dilation, padding):
    """y[n,o,i,j] = bias[o] + sum_{c,p,q} xpad[n,c,i*sh + p*dh, j*sw + q*dw] * w[o,c,p,q], in f64; padding = [(top, bottom),
    (left, right)]."""
    x, w = np.asarray(x, np.float64), np.asarray(w, np.float64)
    xp = np.pad(x, [(0, 0), (0, 0), tuple(padding[0]), tuple(padding[1])])
    (sh, sw), (dh, dw) = stride, dilation
    co, _, kh, kw = w.shape
    oh = (xp.shape[2] - dh * (kh - 1) - 1) // sh + 1
    ow = (xp.shape[3] - dw * (kw - 1) - 1) // sw + 1
    y = np.zeros((x.shape[0], co, oh, ow))
    for p in range(kh):
        for q in range(kw):
            win = xp[:, :, p * dh: p * dh + (oh - 1) * sh + 1: sh, q * dw: q * dw + (ow - 1) * sw + 1: sw]
            y += np.einsum("ncij,oc->noij", win, w[:, :, p, q])
    return y if bias is None else y + np.asarray(bias, np.float64).reshape(1, -1, 1, 1)


def max_pool_textbook(x, kernel, stride, dilation, padding):
    """x: [planes, h, w]; padding = (ph, pw) on both sides with -inf."""
    xp = np.pad(x, [(0, 0), (padding[0],) * 2, (padding[1],) * 2], constant_values=-np.inf)
    oh = (xp.shape[1] - dilation[0] * (kernel[0] - 1) - 1) // stride[0] + 1
    ow = (xp.shape[2] - dilation[1] * (kernel[1] - 1) - 1) // stride[1] + 1
    y = np.full((x.shape[0], oh, ow), -np.inf, x.dtype)
    for p in range(kernel[0]):
        for q in range(kernel[1]):
            y = np.maximum(y, xp[:, p * dilation[0]: p * dilation[0] + (oh - 1) * stride[0] + 1: stride[0],
                                 q * dilation[1]: q * dilation[1] + (ow - 1) * stride[1] + 1: stride[1]])
    return y


def run_lowered(g, leaves, outputs, match=False, seen=None):
    """Executes the schedule with the kernel interpreter; buffers are flat arrays in storage format. A matched
    product is computed the way the GEMM kernel reads its operands: in place, [batch, m, k] or [batch, k, m]
    (trans_a) times [batch, k, n] or [batch, n, k] (trans_b), written as [batch, m, n]."""
    bufs = {i: a.reshape(-1).copy() for i, a in leaves.items()}
    for kern in lower(g, outputs, match=match):
        if isinstance(kern, Alias):
            bufs[kern.out] = bufs[kern.base]
            continue
        if isinstance(kern, Contraction):
            A = bufs[kern.a].reshape((kern.batch, kern.k, kern.m) if kern.trans_a else (kern.batch, kern.m, kern.k))
            B = bufs[kern.b].reshape((kern.batch, kern.n, kern.k) if kern.trans_b else (kern.batch, kern.k, kern.n))
            A = A.transpose(0, 2, 1) if kern.trans_a else A
            B = B.transpose(0, 2, 1) if kern.trans_b else B
            acc = np.matmul(A.astype(np.float64), B.astype(np.float64)) * np.float64(np.float32(kern.alpha))
            if kern.bias is not None:
                acc = acc + bufs[kern.bias].astype(np.float64).reshape(1, 1, -1)
            if kern.epilogue == "bias_relu":
                acc = np.maximum(acc, 0)
            elif kern.epilogue == "bias_gelu":
                acc = acc * 0.5 * (np.tanh((acc + acc ** 3 * 0.044715) * np.sqrt(2 / np.pi)) + 1)
            if kern.residual is not None:
                res = bufs[kern.residual].astype(np.float64).reshape(acc.shape)
                acc = acc * (res > 0) if kern.relu_mask else acc + res
            bufs[kern.out] = acc.astype(A.dtype).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, NormRowsMatch):
            x = bufs[kern.x].reshape(kern.rows, kern.cols).astype(np.float64)
            if kern.rms:
                y = x * np.sqrt(1.0 / ((x * x).mean(1, keepdims=True) + kern.eps))
            else:
                y = (x - x.mean(1, keepdims=True)) / np.sqrt(x.var(1, ddof=1, keepdims=True) + kern.eps)
            if kern.w is not None:
                y = y * bufs[kern.w].astype(np.float64).reshape(1, -1)
            if kern.b is not None:
                y = y + bufs[kern.b].astype(np.float64).reshape(1, -1)
            bufs[kern.out] = y.astype(bufs[kern.x].dtype).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, NormBwdMatch):
            x = bufs[kern.x].reshape(kern.rows, kern.cols).astype(np.float64)
            dy = bufs[kern.dy].reshape(kern.rows, kern.cols).astype(np.float64)
            gg = dy * bufs[kern.w].astype(np.float64).reshape(1, -1) if kern.w is not None else dy
            n = kern.cols
            if kern.rms:
                r = np.sqrt(1.0 / ((x * x).mean(1, keepdims=True) + kern.eps))
                xh = x * r
                dx = r * gg - r ** 3 * x * (gg * x).sum(1, keepdims=True) / n
            else:
                r = 1.0 / np.sqrt(x.var(1, ddof=1, keepdims=True) + kern.eps)
                xh = (x - x.mean(1, keepdims=True)) * r
                dx = r * (gg - gg.mean(1, keepdims=True) - xh * (gg * xh).sum(1, keepdims=True) / (n - 1))
            if kern.add is not None:
                dx = dx + bufs[kern.add].reshape(kern.rows, kern.cols).astype(np.float64)
            st = bufs[kern.x].dtype
            bufs[kern.dx] = dx.astype(st).reshape(-1)
            if kern.dw is not None:
                bufs[kern.dw] = (dy * xh).sum(0).astype(st)
            if kern.db is not None:
                bufs[kern.db] = dy.sum(0).astype(st)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, (AttentionMatch, AttentionBwdMatch)):
            b_, t_, h_, dh_ = kern.dims
            qkv = bufs[kern.qkv].reshape(b_, t_, 3, h_, dh_).astype(np.float64)
            q, k, v = (qkv[:, :, i].transpose(0, 2, 1, 3) for i in range(3))
            sc = np.einsum("bhtd,bhsd->bhts", q, k) * kern.scale
            p = np.exp(sc - sc.max(-1, keepdims=True))
            p /= p.sum(-1, keepdims=True)
            if isinstance(kern, AttentionMatch):
                y = np.einsum("bhts,bhsd->bhtd", p, v).transpose(0, 2, 1, 3).reshape(b_, t_, h_ * dh_)
                bufs[kern.out] = y.astype(bufs[kern.qkv].dtype).reshape(-1)
            else:
                dy = bufs[kern.dy].reshape(b_, t_, h_, dh_).astype(np.float64).transpose(0, 2, 1, 3)
                dv = np.einsum("bhts,bhtd->bhsd", p, dy)
                dp = np.einsum("bhtd,bhsd->bhts", dy, v)
                ds = p * (dp - (dp * p).sum(-1, keepdims=True)) * kern.scale
                dq, dk = np.einsum("bhts,bhsd->bhtd", ds, k), np.einsum("bhts,bhtd->bhsd", ds, q)
                out = np.stack([a.transpose(0, 2, 1, 3) for a in (dq, dk, dv)], 2).reshape(b_, t_, 3 * h_ * dh_)
                bufs[kern.out] = out.astype(bufs[kern.qkv].dtype).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, CrossEntropyMatch):
            x = bufs[kern.x].reshape(kern.rows, kern.cols).astype(np.float64)
            t = bufs[kern.target].reshape(kern.rows, kern.cols).astype(np.float64)
            m = x - x.max(1, keepdims=True)
            ls = m - np.log(np.exp(m).sum(1, keepdims=True))
            if kern.mean is not None:
                bufs[kern.mean] = np.array([(-ls * t).sum(1).mean()], np.float32)
            if kern.grad is not None:
                bufs[kern.grad] = ((np.exp(ls) * t.sum(1, keepdims=True) - t) * kern.gscale).astype(np.float32).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, RowColReduce):
            x = bufs[kern.x].reshape(kern.rows, kern.cols)
            f = np.sum if kern.op == "sum" else np.max
            red = f(x.astype(np.float64) if x.dtype.kind == "f" else x, axis=0 if kern.axis0 else 1)
            if kern.base is not None:
                red = red * np.float64(np.float32(kern.mul)) + bufs[kern.base].astype(np.float64).reshape(-1)
            bufs[kern.out] = red.astype(x.dtype).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, SoftmaxRows):
            x = bufs[kern.x].reshape(kern.rows, kern.cols).astype(np.float64)
            e = np.exp(x - x.max(1, keepdims=True))
            bufs[kern.out] = (e / e.sum(1, keepdims=True)).astype(np.float32).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, Conv2dMatch):
            n, c, h, w, co, kh, kw = kern.dims
            y = conv_textbook(bufs[kern.x].reshape(n, c, h, w), bufs[kern.w].reshape(co, c, kh, kw),
                              None if kern.bias is None else bufs[kern.bias], kern.stride, kern.dilation,
                              [(kern.padding[0],) * 2, (kern.padding[1],) * 2])
            bufs[kern.out] = (np.maximum(y, 0) if kern.relu else y).astype(np.float32).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        if isinstance(kern, MaxPoolMatch):
            x = bufs[kern.x].reshape(kern.planes, *kern.hw)
            bufs[kern.out] = max_pool_textbook(x, kern.kernel, kern.stride, kern.dilation, kern.padding).reshape(-1)
            if seen is not None:
                seen.append(kern)
            continue
        out = np.zeros(kern.elements, storage_dtype(g[kern.output].dtype))
        ir_interp.run(kern.image, [bufs[i] for i in kern.inputs] + [out])
        bufs[kern.output] = out
    return {o: bufs[o].reshape(g[o].shape) for o in outputs}


@pytest.mark.parametrize("name,build", CASES, ids=[c[0] for c in CASES])
def test_reference_gradients(name, build):
    g, leaves, (target, sources, expected) = _build(build)
    grads = g.gradient(target, sources)
    want = graph_eval.evaluate(g.nodes, leaves, grads + [target])
    for gid, src, exp in zip(grads, sources, expected):
        assert g[gid].shape == g[src].shape and g[gid].dtype == g[src].dtype
        if exp is None:
            continue
        if g[src].dtype in _FLOAT:
            np.testing.assert_allclose(want[gid], exp, rtol=2e-7 if g[src].dtype == DType.F32 else 1e-12, atol=0)
        else:
            assert want[gid].tolist() == np.asarray(exp).tolist()
    got = run_lowered(g, leaves, grads + [target])
    for gid in grads + [target]:
        assert got[gid].dtype == want[gid].dtype
        assert np.array_equal(got[gid], want[gid], equal_nan=True), (name, gid)


def _loss(build, leaves_override, **kw):
    g, leaves, out = _build(build, **kw)
    leaves.update(leaves_override)
    return float(graph_eval.evaluate(g.nodes, leaves, [out[0]])[out[0]].reshape(-1)[0])


def test_every_rule_against_finite_differences():
    g, leaves, (loss, sources) = _build(mixed_graph)
    grads = g.gradient(loss, sources)
    got = graph_eval.evaluate(g.nodes, leaves, grads)
    low = run_lowered(g, leaves, grads)
    for gid, src in zip(grads, sources):
        assert np.array_equal(low[gid], got[gid])
        base = leaves[src]
        num = np.zeros_like(base)
        for i in np.ndindex(base.shape):
            h = 1e-6
            up, dn = base.copy(), base.copy()
            up[i] += h
            dn[i] -= h
            num[i] = (_loss(mixed_graph, {src: up}) - _loss(mixed_graph, {src: dn})) / (2 * h)
        np.testing.assert_allclose(got[gid], num, rtol=2e-6, atol=1e-8)


def test_max_ties():
    """Reduce max: every tied maximum receives the full gradient (mask 1 - (x < max), autograd.rs:330-352); binary
    Max: strict comparisons on both sides, so a tie passes nothing (:155-162)."""
    g = Graph()
    x = g.leaf((2, 3), DType.F32)
    y = g.leaf((2, 3), DType.F32)
    leaves = {x: np.array([[1, 5, 5], [7, 7, 7]], np.float32), y: np.array([[1, 9, 5], [0, 7, 8]], np.float32)}
    r = g.reduce(x, BOp.Max, [1])
    (gr,) = g.gradient(r, [x])
    m = g.binary(x, y, BOp.Max)
    gx, gy = g.gradient(m, [x, y])
    got = run_lowered(g, leaves, [gr, gx, gy, r])
    assert got[r].tolist() == [5, 7]
    assert got[gr].tolist() == [[0, 1, 1], [1, 1, 1]]
    assert got[gx].tolist() == [[0, 0, 0], [1, 0, 0]]
    assert got[gy].tolist() == [[0, 1, 0], [0, 0, 1]]


def test_mlp_gradients_closed_form():
    g, leaves, (loss, sources, (x, w1, b1, w2, b2)) = _build(mlp_graph)
    grads = g.gradient(loss, sources)
    got = run_lowered(g, leaves, grads + [loss])
    X, W1, B1, W2 = (leaves[i].astype(np.float64) for i in (x, w1, b1, w2))
    pre = X @ W1.T + B1
    h = np.maximum(pre, 0)
    dlogits = np.ones((X.shape[0], W2.shape[0]))
    dh = (dlogits @ W2) * (pre > 0)
    want = [dh.T @ X, dh.sum(0), dlogits.T @ h, dlogits.sum(0)]
    for gid, w in zip(grads, want):
        np.testing.assert_allclose(got[gid], w, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(got[loss], [(h @ W2.T + leaves[b2]).sum()], rtol=1e-5)


def test_unrelated_source_and_dtype_of_gradient():
    g = Graph()
    x, y = g.leaf((3,), DType.F32), g.leaf((2, 2), DType.I32)
    z = g.unary(x, UOp.Exp)
    gx, gy = g.gradient(z, [x, y])
    got = run_lowered(g, {x: np.zeros(3, np.float32), y: np.zeros((2, 2), np.int32)}, [gx, gy])
    assert got[gy].dtype == np.int32 and got[gy].tolist() == [[0, 0], [0, 0]]
    assert got[gx].tolist() == [1, 1, 1]
    # a cast on the way: the gradient returns in the source's dtype
    c = g.cast(y, DType.F32)
    s = g.sum_all(g.binary(c, c, BOp.Mul))
    (gc,) = g.gradient(s, [y])
    got = run_lowered(g, {y: np.array([[1, 2], [3, 4]], np.int32)}, [gc])
    assert got[gc].dtype == np.int32 and got[gc].tolist() == [[2, 4], [6, 8]]


@pytest.mark.parametrize("n", [1, 63, 64, 65, 130, 4097])
def test_lowered_sizes_and_movement(n):
    """Thread guard for sizes that are not a multiple of the workgroup, and the index arithmetic of every movement op."""
    r = np.random.default_rng(n)
    g = Graph()
    x = g.leaf((n, 3), DType.I32)
    leaves = {x: r.integers(-50, 50, (n, 3)).astype(np.int32)}
    a = g.flip(g.permute(x, [1, 0]), [1])                       # [3, n]
    b = g.expand(g.reshape(a, [3, 1, n]), [3, 2, n])            # [3, 2, n]
    c = g.reduce(b, BOp.Add, [1])                               # [3, n]
    d = g.reduce(g.binary(c, a, BOp.Mul), BOp.Max, [0])         # [n]
    e = g.reduce(b, BOp.Add, [0, 2])                            # [2]
    got = run_lowered(g, leaves, [a, b, c, d, e])
    A = np.flip(leaves[x].T, 1)
    B = np.broadcast_to(A.reshape(3, 1, n), (3, 2, n))
    assert np.array_equal(got[a], A) and np.array_equal(got[b], B)
    assert np.array_equal(got[c], B.sum(1)) and np.array_equal(got[d], (B.sum(1) * A).max(0))
    assert np.array_equal(got[e], B.sum((0, 2)))


def test_schedule_shape():
    """One kernel per requested output and per reduce; read-only parameters come first, in first-use order."""
    g = Graph()
    x, y = g.leaf((4, 4), DType.F32), g.leaf((4, 4), DType.F32)
    s = g.reduce(g.binary(y, x, BOp.Mul), BOp.Add, [1])
    out = g.binary_b(g.unary(x, UOp.Exp), g.reshape(s, [4, 1]), BOp.Div)
    ks = lower(g, [out])
    assert [k.output for k in ks] == [s, out]
    assert ks[0].inputs == [y, x] and ks[1].inputs == [x, s]
    ops, _ = ir_interp.parse(ks[1].image)
    params = [o for o in ops if o[1] == ir_interp.PARAM]
    assert [p[6] for p in params] == [ir_interp.GLOBAL, ir_interp.GLOBAL, ir_interp.GLOBAL_MUT]
    # nodes that already have a buffer are not computed again
    assert [k.output for k in lower(g, [out], stored=[s])] == [out]


def test_shape_errors():
    g = Graph()
    x = g.leaf((2, 3), DType.F32)
    for bad in (lambda: g.reshape(x, [4]), lambda: g.expand(x, [2, 4]), lambda: g.permute(x, [0, 0]),
                lambda: g.binary(x, g.leaf((3, 2), DType.F32), BOp.Add), lambda: g.reduce(x, BOp.Mul, [0]),
                lambda: g.dot(x, g.leaf((2, 3), DType.F32))):
        with pytest.raises(ValueError):
            bad()


def test_lowered_kernels_are_accepted_by_the_source_generator():
    """Every image the lowering produces for the reference's cases turns into HIP source (no GPU needed); the
    largest one is also compiled for gfx950 when hipcc is present."""
    import os, shutil, subprocess, tempfile
    from zyx_amd.backend import generate_source
    biggest = ""
    for name, build in CASES + [("mixed", lambda g, leaf: mixed_graph(g, leaf) + ([None] * 3,))]:
        g, leaves, (target, sources, _) = _build(build)
        for kern in lower(g, g.gradient(target, sources) + [target]):
            src = generate_source(kern.image)
            assert "zir_kernel" in src
            biggest = max(biggest, src, key=len)
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "k.hip")
        open(path, "w").write(biggest)
        r = subprocess.run([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fwrapv", "-Xclang",
                            "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-include",
                            "hip/hip_runtime.h", "-c", path, "-o", os.path.join(d, "k.o")],
                           capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr[-2000:]


def test_softmax_and_dropout_compositions():
    """softmax golden of zyx/tests/05_misc.rs:664-683 through the graph; training-mode dropout keeps x where
    p < u without rescaling, evaluation divides by 1 - p (tensor/mod.rs:822-828)."""
    g = Graph()
    x = g.leaf((1, 3), DType.F32)
    u = g.leaf((1, 3), DType.F32)
    leaves = {x: np.array([[2, 4, 3]], np.float32), u: np.array([[0.1, 0.25, 0.9]], np.float32)}
    sm, ls = g.softmax(x, [-1]), g.ln_softmax(x, [-1])
    tr, evl = g.dropout(x, 0.25, u), g.dropout(x, 0.25)
    got = run_lowered(g, leaves, [sm, ls, tr, evl])
    np.testing.assert_allclose(got[sm], [[0.090030566, 0.6652409, 0.24472846]], rtol=1e-6)
    np.testing.assert_allclose(np.exp(got[ls]), got[sm], rtol=1e-6)
    assert got[tr].tolist() == [[0, 0, 3]]
    assert np.array_equal(got[evl], np.array([[2, 4, 3]], np.float32) / np.float32(0.75))


@pytest.mark.parametrize("causal,p,training", [(False, 0.0, False), (True, 0.25, False), (True, 0.3, True)])
def test_attention_graph_gradients(causal, p, training):
    """The attention core built from graph nodes and differentiated by the reverse rules, against the textbook
    forward and backward in f64 (with the dropout mask applied after the softmax, as the reference orders them)."""
    from graph_cases import attention_graph
    g, leaves, (loss, sources, (y, arrs)) = _build(attention_graph, causal=causal, p=p, training=training, dtype=DType.F64)
    grads = g.gradient(loss, sources)
    got = graph_eval.evaluate(g.nodes, leaves, grads + [y])
    q, k, v, dy = (arrs[n] for n in ("q", "k", "v", "dy"))
    t, dh = q.shape[2], q.shape[3]
    sc = float(np.float32(1 / np.sqrt(dh)))
    s = np.einsum("bhtd,bhjd->bhtj", q, k) * sc
    if causal:
        s = np.where(np.tril(np.ones((t, t), bool)), s, -np.inf)
    e = np.exp(s - s.max(-1, keepdims=True))
    ps = e / e.sum(-1, keepdims=True)
    keep = (p < arrs["u"]).astype(np.float64) if training else np.full_like(ps, 1 / (1 - p))
    pd = ps * keep
    np.testing.assert_allclose(got[y], np.einsum("bhtj,bhjd->bhtd", pd, v), rtol=1e-11, atol=1e-13)
    dpd = np.einsum("bhtd,bhjd->bhtj", dy, v) * keep
    ds = ps * (dpd - (ps * dpd).sum(-1, keepdims=True))
    want = [np.einsum("bhtj,bhjd->bhtd", ds, k) * sc, np.einsum("bhtj,bhtd->bhjd", ds, q) * sc, np.einsum("bhtj,bhtd->bhjd", pd, dy)]
    for gid, w in zip(grads, want):
        np.testing.assert_allclose(got[gid], w, rtol=1e-9, atol=1e-12)


# ---- products matched to the GEMM kernel -----------------------------------------------------------------------------

def test_views_and_reshape_strides():
    g = Graph()
    x = g.leaf((4, 6, 5), DType.F32)
    assert view_of(g, g.permute(x, [2, 0, 1])) == (x, [1, 30, 5])
    assert view_of(g, g.reshape(x, [24, 5])) == (x, [5, 1])
    assert view_of(g, g.reshape(x, [2, 2, 3, 2, 5])) == (x, [60, 30, 10, 5, 1])
    assert view_of(g, g.expand(g.reshape(x, [4, 1, 6, 5]), [4, 7, 6, 5])) == (x, [30, 0, 5, 1])
    assert view_of(g, g.reshape(g.permute(x, [1, 0, 2]), [6, 20]))[0] != x      # merging permuted dims needs a copy
    t = g.reshape(g.permute(x, [1, 0, 2]), [6, 4, 1, 5])
    assert view_of(g, t) == (x, [5, 30, 0, 1])                                  # inserting a 1 into permuted dims does not
    assert view_of(g, g.flip(x, [0]))[0] != x


def _mlp_sq(g, leaf):
    loss, sources, leaves5 = mlp_graph(g, leaf)
    logits = g[loss].src[0]
    return g.sum_all(g.binary(logits, logits, BOp.Mul)), sources, leaves5


def test_matched_products_of_an_mlp():
    """Forward products x.W^T, and with a loss that gives a dense upstream gradient all three backward products
    (dY^T.X read through trans_a, dY.W) are recognised; results agree with the unmatched schedule."""
    g, leaves, (loss, sources, _) = _build(_mlp_sq)
    grads = g.gradient(loss, sources)
    seen = []
    got = run_lowered(g, leaves, grads + [loss], match=True, seen=seen)
    want = run_lowered(g, leaves, grads + [loss])
    shapes = sorted((c.m, c.n, c.k, c.trans_a, c.trans_b) for c in seen)
    assert shapes == sorted([(8, 16, 12, False, True), (8, 5, 16, False, True),      # x.W1^T, h.W2^T
                             (8, 16, 5, False, False),                               # dh = dlogits.W2
                             (5, 16, 8, True, False), (16, 12, 8, True, False)])     # dW2 = dlogits^T.h, dW1 = dpre^T.x
    for nid in grads + [loss]:
        np.testing.assert_allclose(got[nid], want[nid], rtol=2e-5, atol=1e-5)


@pytest.mark.parametrize("causal", [False, True])
def test_matched_products_of_attention(causal):
    from graph_cases import attention_graph
    g, leaves, (loss, sources, (y, _)) = _build(attention_graph, causal=causal, p=0.1)
    grads = g.gradient(loss, sources)
    seen = []
    got = run_lowered(g, leaves, grads + [y], match=True, seen=seen)
    want = run_lowered(g, leaves, grads + [y])
    gemms = [c for c in seen if isinstance(c, Contraction)]
    assert len(gemms) == 6 and all(c.batch == 4 for c in gemms)   # q.k^T, att.v and the four backward products
    (sm,) = [c for c in seen if isinstance(c, SoftmaxRows)]
    assert (sm.rows, sm.cols) == (2 * 2 * 24, 24)
    for nid in grads + [y]:
        np.testing.assert_allclose(got[nid], want[nid], rtol=0, atol=2e-5 * np.abs(want[nid]).max())


def test_products_that_are_not_matched():
    g = Graph()
    xi, yi = g.leaf((4, 3), DType.I32), g.leaf((3, 5), DType.I32)
    assert match_contraction(g, g[g.dot(xi, yi)].src[0] if g[g.dot(xi, yi)].kind == "reshape" else g.dot(xi, yi)) is None  # integers
    x, y = g.leaf((4, 3), DType.F32), g.leaf((3, 5), DType.F32)
    prod = g.binary(g.expand(g.reshape(x, [4, 1, 3]), [4, 5, 3]), g.expand(g.reshape(g.t(y), [1, 5, 3]), [4, 5, 3]), BOp.Mul)
    assert match_contraction(g, g.reduce(prod, BOp.Add, [2])) is not None
    assert match_contraction(g, g.reduce(prod, BOp.Max, [2])) is None               # not a sum
    assert match_contraction(g, g.reduce(prod, BOp.Add, [1])) is None               # sums an axis only one side has
    assert match_contraction(g, g.reduce(g.binary(prod, prod, BOp.Add), BOp.Add, [2])) is None
    fl = g.binary(g.expand(g.reshape(g.flip(x, [1]), [4, 1, 3]), [4, 5, 3]), g.expand(g.reshape(g.t(y), [1, 5, 3]), [4, 5, 3]), BOp.Mul)
    c = match_contraction(g, g.reduce(fl, BOp.Add, [2]))
    assert c is not None and g[c.a].kind == "flip"                                  # the flipped operand is copied first


def test_softmax_match():
    g = Graph()
    x = g.leaf((3, 5, 7), DType.F32)
    sm = g.softmax(x, [-1])
    m = match_softmax(g, sm)
    assert (m.x, m.rows, m.cols) == (x, 15, 7)
    assert match_softmax(g, g.softmax(x, [1])) is None                       # not the last axis
    assert match_softmax(g, g.softmax(x, [1, 2])) is None                    # two axes
    assert match_softmax(g, g.ln_softmax(x, [-1])) is None
    h = g.leaf((3, 5, 7), DType.F64)
    assert match_softmax(g, g.softmax(h, [-1])) is None                      # f32 only
    y = g.unary(g.permute(x, [1, 0, 2]), UOp.Neg)                            # an expression: gets its own buffer
    m = match_softmax(g, g.softmax(y, [-1]))
    assert m.x == y and (m.rows, m.cols) == (15, 7)
    p = g.permute(x, [1, 0, 2])                                              # a permuted view is not row-contiguous
    assert match_softmax(g, g.softmax(p, [-1])).x == p
    # e / sum(e) where e is not exp(x - max): no match
    e = g.unary(x, UOp.Exp)
    assert match_softmax(g, g.binary_b(e, g.reduce_keepdim(e, BOp.Add, [-1]), BOp.Div)) is None
    leaves = {x: np.random.default_rng(2).standard_normal((3, 5, 7)).astype(np.float32)}
    seen = []
    got = run_lowered(g, leaves, [sm], match=True, seen=seen)
    assert len(seen) == 1
    np.testing.assert_allclose(got[sm], run_lowered(g, leaves, [sm])[sm], rtol=1e-6)


def test_reduce_match():
    """Long reductions over the trailing or the leading axes of a tensor that has a buffer go to the reduce kernel;
    short ones, middle axes and operands that are expressions stay generated (fused)."""
    g = Graph()
    x = g.leaf((6, 4, 512), DType.F32)
    m = match_reduce(g, g.reduce(x, BOp.Add, [2]), set())
    assert (m.x, m.rows, m.cols, m.axis0, m.op) == (x, 24, 512, False, "sum")
    m = match_reduce(g, g.reduce(x, BOp.Max, [1, 2]), set())
    assert (m.rows, m.cols, m.axis0, m.op) == (6, 2048, False, "max")
    y = g.leaf((300, 7, 3), DType.I32)
    m = match_reduce(g, g.reduce(g.reshape(y, [300, 21]), BOp.Add, [0]), set())
    assert (m.x, m.rows, m.cols, m.axis0) == (y, 300, 21, True)
    assert match_reduce(g, g.reduce(x, BOp.Add, [1]), set()) is None                      # a middle axis
    assert match_reduce(g, g.reduce(x, BOp.Add, [0]), set()) is None                      # 6 elements per result
    e = g.unary(x, UOp.Exp)
    assert match_reduce(g, g.reduce(e, BOp.Add, [2]), set()) is None                      # an expression: stays fused
    assert match_reduce(g, g.reduce(e, BOp.Add, [2]), {e}) is not None                    # unless it has a buffer anyway
    assert match_reduce(g, g.reduce(g.permute(x, [1, 0, 2]), BOp.Add, [2]), set()) is None
    leaves = {x: np.random.default_rng(1).standard_normal((6, 4, 512)).astype(np.float32),
              y: np.random.default_rng(2).integers(-9, 9, (300, 7, 3)).astype(np.int32)}
    outs = [g.reduce(x, BOp.Add, [2]), g.reduce(x, BOp.Max, [1, 2]), g.reduce(g.reshape(y, [300, 21]), BOp.Add, [0])]
    seen = []
    got, want = run_lowered(g, leaves, outs, match=True, seen=seen), run_lowered(g, leaves, outs)
    assert len(seen) == 3
    np.testing.assert_allclose(got[outs[0]], want[outs[0]], rtol=1e-5, atol=1e-5)
    assert np.array_equal(got[outs[1]], want[outs[1]]) and np.array_equal(got[outs[2]], want[outs[2]])
