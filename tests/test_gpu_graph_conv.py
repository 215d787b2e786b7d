"""Pad / Narrow nodes and the convolution compositions of zyx_amd.graph on the GPU through `Tape`: generated kernels
against the CPU evaluation of the same graph (oracle/graph_eval.py) bit for bit, the matched path (conv + relu on
ZHIP_K_CONV2D, max_pool on ZHIP_K_MAX_POOL2D, reverse pass on generated kernels) against it within 1e-5, and the
conv -> relu -> max_pool block of the benchmark geometry (64 -> 128 channels, 56 x 56, 3 x 3, padding 1), forward and
backward, against a textbook convolution and its textbook adjoints computed with BLAS on the host."""
import numpy as np
import pytest

from oracle import graph_eval
from test_graph_conv import _conv_net
from test_graph_oracle import conv_textbook
from zyx_amd import DType
from zyx_amd.graph import Tape, storage_dtype
from zyx_amd.ir import BOp

pytestmark = pytest.mark.gpu


def _on_device(hip, build, match=False, **kw):
    dev, pool = hip
    tape, leaves = Tape(dev, pool, match=match), {}

    def leaf(array, dtype):
        a = np.ascontiguousarray(np.asarray(array).astype(storage_dtype(dtype)))
        nid = tape.tensor(a, dtype)
        leaves[nid] = a
        return nid

    return tape, leaves, build(tape.graph, leaf, **kw)


@pytest.mark.parametrize("dtype", [DType.F32, DType.F64])
@pytest.mark.parametrize("pool_pad", [None, [(0, 0), (1, 1)]])
def test_generated_conv_relu_pool_and_gradients(hip, dtype, pool_pad):
    tape, leaves, (loss, sources, pooled) = _on_device(hip, _conv_net, dtype=dtype, pool_pad=pool_pad)
    grads = tape.gradient(loss, sources)
    nodes = [pooled, loss] + grads
    want = graph_eval.evaluate(tape.graph.nodes, leaves, nodes)
    tape.realize(nodes)
    for nid in nodes:
        got = tape.numpy(nid)
        assert got.dtype == want[nid].dtype and np.array_equal(got, want[nid]), nid
    tape.close()


def test_pad_narrow_values_on_the_device(hip):
    dev, pool = hip
    tape = Tape(dev, pool)
    X = np.arange(2 * 3 * 5, dtype=np.int32).reshape(2, 3, 5)
    x = tape.tensor(X, DType.I32)
    g = tape.graph
    a = g.pad_zeros(x, [(1, 2), (0, 0), (0, 3)])
    b = g.pad_zeros(x, [(0, 0), (-1, 2), (-2, -1)])
    c = g.narrow(x, 2, 1, 3)
    d = g.pad_value(x, [(0, 0), (1, 1), (2, 0)], -9)
    e = g.repeat(x, [2, 1, 3])
    tape.realize([a, b, c, d, e])
    assert np.array_equal(tape.numpy(a), np.pad(X, [(1, 2), (0, 0), (0, 3)]))
    assert np.array_equal(tape.numpy(b), np.pad(X[:, 1:, 2:4], [(0, 0), (0, 2), (0, 0)]))
    assert np.array_equal(tape.numpy(c), X[:, :, 1:4])
    assert np.array_equal(tape.numpy(d), np.pad(X, [(0, 0), (1, 1), (2, 0)], constant_values=-9))
    assert np.array_equal(tape.numpy(e), np.tile(X, [2, 1, 3]))
    tape.close()


def test_matched_conv_relu_pool_and_gradients(hip):
    tape, leaves, (loss, sources, pooled) = _on_device(hip, _conv_net, match=True, dtype=DType.F32)
    grads = tape.gradient(loss, sources)
    nodes = [pooled, loss] + grads
    want = graph_eval.evaluate(tape.graph.nodes, leaves, nodes)
    tape.realize(nodes)
    assert tape.matched >= 2  # conv + relu and max_pool went to the hand-written kernels
    for nid in nodes:
        np.testing.assert_allclose(tape.numpy(nid), want[nid], rtol=1e-5, atol=1e-5)
    tape.close()


def _block(g, leaf, n, c, hw, cout, seed=11):
    rng = np.random.default_rng(seed)
    x = leaf(rng.standard_normal((n, c, hw, hw)), DType.F32)
    w = leaf(rng.standard_normal((cout, c, 3, 3)) * np.sqrt(2.0 / (c * 9)), DType.F32)  # Kaiming-normal, fan-in
    b = leaf(rng.standard_normal(cout) * 0.1, DType.F32)
    t = leaf(rng.standard_normal((n, cout, hw // 2, hw // 2)), DType.F32)
    r = g.relu(g.conv(x, w, b, stride=1, dilation=1, padding=1))
    p = g.max_pool(r, (2, 2))
    loss = g.reduce(g.binary(p, t, BOp.Mul), BOp.Add, range(4))
    return (x, w, b, t), r, p, loss


@pytest.mark.parametrize("n,match", [(2, False), (32, True)])
def test_benchmark_conv_block_forward_and_backward(hip, n, match):
    """n = 32 is the benchmark's batch. The forward is checked against a textbook convolution; the reverse pass
    against the textbook adjoints of max_pool, relu and the convolution evaluated on the forward the device produced
    (the pooling and relu masks of a nearly tied or nearly zero activation would otherwise depend on the last bit of
    the forward)."""
    c, hw, cout = 64, 56, 128
    tape, leaves, ((x, w, b, t), r, p, loss) = _on_device(hip, _block, match=match, n=n, c=c, hw=hw, cout=cout)
    gx, gw, gb = tape.gradient(loss, [x, w, b])
    tape.realize([r, p, loss, gx, gw, gb])
    if match:
        assert tape.matched >= 2
    X, W, Bv, T = (leaves[i] for i in (x, w, b, t))
    R, P = tape.numpy(r), tape.numpy(p)
    # forward, first two images against the f64 textbook
    want = np.maximum(conv_textbook(X[:2], W, Bv, (1, 1), (1, 1), [(1, 1), (1, 1)]), 0)
    np.testing.assert_allclose(R[:2], want, rtol=1e-4, atol=1e-4)
    assert np.array_equal(P, R.reshape(n, cout, hw // 2, 2, hw // 2, 2).max(axis=(3, 5)))
    terms = P.astype(np.float64) * T  # signs cancel: the bar is relative to the magnitude summed
    np.testing.assert_allclose(tape.numpy(loss)[0], terms.sum(), rtol=0, atol=2e-6 * np.abs(terms).sum())
    # reverse: every tied maximum of a window receives the gradient (zyx/src/autograd.rs:330-352), relu passes where
    # its input was positive, which is where its output is
    up = lambda a: np.repeat(np.repeat(a, 2, axis=2), 2, axis=3)
    dC = (up(T) * (R == up(P)) * (R > 0)).astype(np.float32)
    np.testing.assert_allclose(tape.numpy(gb), dC.sum(axis=(0, 2, 3), dtype=np.float64), rtol=0,
                               atol=1e-5 * np.abs(dC).sum(axis=(0, 2, 3), dtype=np.float64).max())  # serial f32 sums of mixed signs
    Xp = np.pad(X, [(0, 0), (0, 0), (1, 1), (1, 1)])
    dW = np.empty_like(W)
    dXp = np.zeros(Xp.shape, np.float64)
    dC2 = np.ascontiguousarray(dC.transpose(1, 0, 2, 3).reshape(cout, -1))  # [o, (n, i, j)]
    for pp in range(3):
        for q in range(3):
            win = np.ascontiguousarray(Xp[:, :, pp:pp + hw, q:q + hw].transpose(0, 2, 3, 1).reshape(-1, c))  # [(n, i, j), c]
            dW[:, :, pp, q] = dC2 @ win
            back = (dC2.T @ W[:, :, pp, q]).reshape(n, hw, hw, c).transpose(0, 3, 1, 2)
            dXp[:, :, pp:pp + hw, q:q + hw] += back
    np.testing.assert_allclose(tape.numpy(gw), dW, rtol=2e-3, atol=2e-3 * np.abs(dW).max())
    np.testing.assert_allclose(tape.numpy(gx), dXp[:, :, 1:-1, 1:-1], rtol=1e-3, atol=1e-4)
    tape.close()
