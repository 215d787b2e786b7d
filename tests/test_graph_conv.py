"""Pad / Narrow nodes and the pool, conv and max_pool compositions of zyx_amd.graph on the CPU: the values the
reference's tests assert (zyx/tests/05_misc.rs:83-109 max_pool, :371-382 pool, :880-888 conv1), a textbook convolution,
reverse rules against central differences and closed forms, and the lowered kernels (kernel interpreter) against the
node-by-node evaluation, bit for bit."""
import numpy as np
import pytest

from oracle import graph_eval
from test_graph_oracle import conv_textbook, max_pool_textbook, run_lowered
from zyx_amd import DType
from zyx_amd.graph import Conv2dMatch, Graph, LoweredKernel, MaxPoolMatch, lower
from zyx_amd.ir import BOp


def _eval(g, leaves, outs):
    return graph_eval.evaluate(g.nodes, leaves, outs)


def test_pool_golden():
    g = Graph()
    x = g.leaf((3, 3), DType.I32)
    p = g.pool(x, (2, 2), 1, 1)
    leaves = {x: np.arange(9, dtype=np.int32).reshape(3, 3)}
    want = [[[[0, 1], [3, 4]], [[1, 2], [4, 5]]], [[[3, 4], [6, 7]], [[4, 5], [7, 8]]]]
    assert _eval(g, leaves, [p])[p].tolist() == want
    assert run_lowered(g, leaves, [p])[p].tolist() == want


def test_conv1_golden():
    g = Graph()
    t, w = g.leaf((1, 1, 3, 3), DType.F32), g.leaf((1, 1, 2, 2), DType.F32)
    c = g.conv(t, w, None, stride=1, dilation=1, padding=0)
    leaves = {t: np.arange(9, dtype=np.float32).reshape(1, 1, 3, 3), w: np.ones((1, 1, 2, 2), np.float32)}
    want = [[[[8.0, 12.0], [20.0, 24.0]]]]
    assert _eval(g, leaves, [c])[c].tolist() == want
    assert run_lowered(g, leaves, [c])[c].tolist() == want
    assert run_lowered(g, leaves, [c], match=True)[c].tolist() == want


def test_max_pool_golden():
    g = Graph()
    x = g.leaf((4, 4), DType.F32)
    p = g.max_pool(x, (2, 2), (2, 2), (1, 1), [(0, 0), (0, 0)])
    leaves = {x: np.arange(1, 17, dtype=np.float32).reshape(4, 4)}
    want = [[6.0, 8.0], [14.0, 16.0]]
    assert _eval(g, leaves, [p])[p].tolist() == want
    assert run_lowered(g, leaves, [p])[p].tolist() == want
    seen = []
    assert run_lowered(g, leaves, [p], match=True, seen=seen)[p].tolist() == want
    assert [type(k) for k in seen] == [MaxPoolMatch]


def test_pad_and_narrow_values_and_errors():
    g = Graph()
    x = g.leaf((2, 3), DType.I32)
    X = np.arange(6, dtype=np.int32).reshape(2, 3)
    a = g.pad_zeros(x, [(1, 2), (0, 1)])          # grows both axes
    b = g.pad_zeros(x, [(0, 0), (-1, 2)])         # crops on the left, grows on the right
    c = g.narrow(x, 1, 1, 2)
    d = g.slice(x, [(1, 2), (0, 2)])
    e = g.pad_value(x, [(0, 0), (1, 0)], -7)
    outs = [a, b, c, d, e]
    want = _eval(g, {x: X}, outs)
    assert want[a].tolist() == np.pad(X, [(1, 2), (0, 1)]).tolist()
    assert want[b].tolist() == np.pad(X[:, 1:], [(0, 0), (0, 2)]).tolist()
    assert want[c].tolist() == X[:, 1:3].tolist() and want[d].tolist() == X[1:2, 0:2].tolist()
    assert want[e].tolist() == np.pad(X, [(0, 0), (1, 0)], constant_values=-7).tolist()
    got = run_lowered(g, {x: X}, outs)
    for o in outs:
        assert np.array_equal(got[o], want[o])
    with pytest.raises(ValueError):
        g.narrow(x, 1, 2, 2)
    with pytest.raises(ValueError):
        g.narrow(x, 2, 0, 1)
    with pytest.raises(ValueError):
        g.pad(x, 0, -2, 0)


@pytest.mark.parametrize("stride,dilation,padding", [((1, 1), (1, 1), 0), ((1, 1), (1, 1), 1), ((2, 1), (1, 2), (1, 2)),
                                                       ((2, 3), (2, 1), [(1, 0), (2, 1)]), ((3, 3), (1, 1), 2)])
def test_conv_is_the_textbook_convolution(stride, dilation, padding):
    rng = np.random.default_rng(3)
    X = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    W = rng.standard_normal((4, 3, 3, 2)).astype(np.float32)
    Bv = rng.standard_normal(4).astype(np.float32)
    g = Graph()
    x, w, b = g.leaf(X.shape, DType.F32), g.leaf(W.shape, DType.F32), g.leaf(Bv.shape, DType.F32)
    c = g.conv(x, w, b, stride=stride, dilation=dilation, padding=padding)
    leaves = {x: X, w: W, b: Bv}
    pads = [(padding, padding)] * 2 if np.isscalar(padding) else [(q, q) if np.isscalar(q) else q for q in padding]
    want = conv_textbook(X, W, Bv, stride, dilation, pads)
    got = _eval(g, leaves, [c])[c]
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)
    assert np.array_equal(run_lowered(g, leaves, [c])[c], got)
    kinds = [type(k) for k in lower(g, [c], match=True)]
    symmetric = all(l == r for l, r in pads)
    assert kinds == ([Conv2dMatch] if symmetric else [LoweredKernel, LoweredKernel][:len(kinds)])


def _conv_net(g, leaf, dtype=DType.F64, seed=5, pool_pad=None):
    rng = np.random.default_rng(seed)
    x = leaf(rng.standard_normal((2, 2, 6, 5)), dtype)
    w = leaf(rng.standard_normal((3, 2, 3, 3)) * 0.5, dtype)
    b = leaf(rng.standard_normal(3), dtype)
    t = leaf(rng.standard_normal((2, 3, 3, 2 if pool_pad is None else 3)), dtype)
    h = g.relu(g.conv(x, w, b, stride=1, dilation=1, padding=1))
    p = g.max_pool(h, (2, 2), None, 1, pool_pad)
    loss = g.reduce(g.binary(p, t, BOp.Mul), BOp.Add, range(4))
    return loss, [x, w, b], p


def _build(build, **kw):
    g, leaves = Graph(), {}

    def leaf(array, dtype):
        from zyx_amd.graph import storage_dtype
        a = np.ascontiguousarray(np.asarray(array).astype(storage_dtype(dtype)))
        nid = g.leaf(a.shape, dtype)
        leaves[nid] = a
        return nid

    return g, leaves, build(g, leaf, **kw)


@pytest.mark.parametrize("pool_pad", [None, [(0, 0), (1, 1)]])
def test_conv_relu_pool_gradients_against_central_differences(pool_pad):
    g, leaves, (loss, sources, _) = _build(_conv_net, pool_pad=pool_pad)
    grads = g.gradient(loss, sources)
    got = _eval(g, leaves, grads)
    low = run_lowered(g, leaves, grads)

    def value(override):
        g2, l2, (loss2, _, _) = _build(_conv_net, pool_pad=pool_pad)
        l2.update(override)
        return float(_eval(g2, l2, [loss2])[loss2].reshape(-1)[0])

    for gid, src in zip(grads, sources):
        assert np.array_equal(low[gid], got[gid])
        base, num = leaves[src], np.zeros_like(leaves[src])
        for i in np.ndindex(base.shape):
            up, dn = base.copy(), base.copy()
            up[i] += 1e-6
            dn[i] -= 1e-6
            num[i] = (value({src: up}) - value({src: dn})) / 2e-6
        np.testing.assert_allclose(got[gid], num, rtol=1e-5, atol=1e-7)


def test_conv_weight_backward_closed_form():
    """The shape of zyx-nn/tests/conv_backward.rs:50-63 (conv 3 -> 16, 3 x 3, padding 1, no bias, loss = sum of the
    output) at a smaller batch: dL/dw[o,c,p,q] is the sum of the padded input over the window positions tap (p, q)
    visits, the same for every o; dL/dx[n,c,y,x] is the sum of the weights of the taps that reach (y, x)."""
    rng = np.random.default_rng(9)
    X = rng.random((4, 3, 8, 8)).astype(np.float32)
    W = rng.standard_normal((16, 3, 3, 3)).astype(np.float32)
    g = Graph()
    x, w = g.leaf(X.shape, DType.F32), g.leaf(W.shape, DType.F32)
    loss = g.reduce(g.conv(x, w, None, padding=1), BOp.Add, range(4))
    gw, gx = g.gradient(loss, [w, x])
    got = run_lowered(g, {x: X, w: W}, [gw, gx])
    xp = np.pad(X.astype(np.float64), [(0, 0), (0, 0), (1, 1), (1, 1)])
    dw = np.array([[[xp[:, c, p:p + 8, q:q + 8].sum() for q in range(3)] for p in range(3)] for c in range(3)])
    np.testing.assert_allclose(got[gw], np.broadcast_to(dw, (16, 3, 3, 3)), rtol=2e-6)
    dx = conv_textbook(np.ones((1, 16, 8, 8)), W.transpose(1, 0, 2, 3)[:, :, ::-1, ::-1], None, (1, 1), (1, 1), [(1, 1), (1, 1)])
    np.testing.assert_allclose(got[gx], np.broadcast_to(dx, X.shape), rtol=1e-5, atol=1e-6)


def test_matched_conv_relu_pool_and_its_backward():
    """With matching on, conv + relu is one Conv2dMatch (the convolution itself is never stored; the reverse pass takes
    the relu mask from the relu's result), max_pool one MaxPoolMatch, and the gradients equal the unmatched ones."""
    g, leaves, (loss, sources, pooled) = _build(_conv_net, dtype=DType.F32)
    grads = g.gradient(loss, sources)
    outs = grads + [pooled]
    want = _eval(g, leaves, outs)
    seen = []
    got = run_lowered(g, leaves, outs, match=True, seen=seen)
    convs = [k for k in seen if isinstance(k, Conv2dMatch)]
    assert len(convs) == 1 and convs[0].relu and convs[0].bias is not None and convs[0].padding == (1, 1)
    assert sum(isinstance(k, MaxPoolMatch) for k in seen) == 1
    for o in outs:
        np.testing.assert_allclose(got[o], want[o], rtol=1e-5, atol=1e-5)


def test_relu_is_not_folded_when_the_convolution_is_read_elsewhere():
    g, leaves, (loss, sources, pooled) = _build(_conv_net, dtype=DType.F32)
    conv = next(iter(g.convs))
    seen = []
    run_lowered(g, leaves, [pooled, conv], match=True, seen=seen)
    convs = [k for k in seen if isinstance(k, Conv2dMatch)]
    assert len(convs) == 1 and not convs[0].relu and convs[0].out == conv


def test_max_pool_textbook_helper_matches_graph():
    rng = np.random.default_rng(2)
    X = rng.standard_normal((3, 7, 9)).astype(np.float32)
    g = Graph()
    x = g.leaf(X.shape, DType.F32)
    p = g.max_pool(x, (3, 2), (2, 1), (1, 2), [(1, 1), (2, 2)])
    got = _eval(g, {x: X}, [p])[p]
    assert np.array_equal(got, max_pool_textbook(X, (3, 2), (2, 1), (1, 2), (1, 2)))
    assert np.array_equal(run_lowered(g, {x: X}, [p])[p], got)
