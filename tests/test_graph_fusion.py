"""The matchers that turn a training step written as graph nodes into the fused launch list (zyx_amd.graph.lower with
match=True), on the CPU: which kernels the schedule holds, and that executing it (products, reductions and the
cross-entropy computed by numpy the way the hand-written kernels define them) gives what the node-by-node evaluation
of the same graph gives (oracle/graph_eval.py)."""
import numpy as np
import pytest

from graph_cases import mlp_training_graph
from oracle import graph_eval
from test_graph_oracle import _build, run_lowered
from zyx_amd import DType
from zyx_amd.graph import (Contraction, CrossEntropyMatch, Graph, LoweredKernel, RowColReduce, lower, same_tree,
                           scan_cross_entropy)
from zyx_amd.ir import BOp, UOp

F32 = DType.F32


def test_mlp_training_step_is_eight_launches():
    g, leaves, (loss, new, params, (x, onehot)) = _build(mlp_training_graph, batch=16, n_in=24, hidden=32, n_out=10)
    rng = np.random.default_rng(0)
    leaves[x] = rng.standard_normal((16, 24)).astype(np.float32)
    leaves[onehot] = np.eye(10, dtype=np.float32)[rng.integers(0, 10, 16)]
    outs = new + [loss]
    sched = lower(g, outs, match=True)
    kinds = [(type(k).__name__, getattr(k, "epilogue", None), getattr(k, "residual", None) is not None,
              getattr(k, "relu_mask", None), getattr(k, "base", None) is not None) for k in sched]
    assert kinds == [
        ("Contraction", "bias_relu", False, False, False),   # h = relu(x . W1^T + b1)
        ("Contraction", "bias", False, False, False),        # logits = h . W2^T + b2
        ("CrossEntropyMatch", None, False, None, False),     # loss (mean) and dlogits
        ("Contraction", "none", True, True, False),          # dpre = (h > 0) * (dlogits . W2)
        ("Contraction", "none", True, False, False),         # W1 - (dpre^T . x) * lr
        ("RowColReduce", None, False, None, True),           # b1 - colsum(dpre) * lr
        ("Contraction", "none", True, False, False),         # W2 - (dlogits^T . h) * lr
        ("RowColReduce", None, False, None, True),           # b2 - colsum(dlogits) * lr
    ]
    ce = sched[2]
    assert ce.grad is not None and ce.mean == loss and ce.gscale == 1.0 / 16 and ce.target == onehot
    assert sched[4].alpha == -0.01 and sched[4].residual == params[0] and sched[6].residual == params[2]
    assert sched[5].mul == -0.01 and sched[5].base == params[1] and sched[5].axis0
    want = graph_eval.evaluate(g.nodes, leaves, outs)
    got = run_lowered(g, leaves, outs, match=True)
    for o in outs:
        np.testing.assert_allclose(got[o], want[o], rtol=2e-5, atol=2e-6)


def test_soft_targets_sum_reduction_and_lone_outputs():
    rng = np.random.default_rng(1)
    X = rng.standard_normal((6, 7)).astype(np.float32)
    T = rng.random((6, 7)).astype(np.float32)
    for reduction, want_loss_match in (("mean", True), ("sum", False)):
        g = Graph()
        x, t = g.leaf(X.shape, F32), g.leaf(T.shape, F32)
        z = g.binary(x, g.const(1.5, F32), BOp.Mul)  # the logits are an expression, not a leaf
        loss = g.cross_entropy(z, t, reduction)
        (gz,) = g.gradient(loss, [z])
        (gx,) = g.gradient(loss, [x])
        leaves = {x: X, t: T}
        for outs in ([loss, gx], [gx], [loss]):
            seen = []
            got = run_lowered(g, leaves, outs, match=True, seen=seen)
            want = graph_eval.evaluate(g.nodes, leaves, outs)
            ces = [k for k in seen if isinstance(k, CrossEntropyMatch)]
            assert len(ces) == (1 if (gx in outs or want_loss_match) else 0)
            if ces:
                assert ces[0].x == z and ces[0].target == t
                assert (ces[0].grad is not None) == (gx in outs)
                assert (ces[0].mean is not None) == (loss in outs and want_loss_match)
            for o in outs:
                np.testing.assert_allclose(got[o], want[o], rtol=2e-5, atol=2e-6)
        del gz


def test_cross_entropy_value_and_gradient_closed_form():
    rng = np.random.default_rng(2)
    X = rng.standard_normal((5, 4)).astype(np.float32) * 3
    labels = rng.integers(0, 4, 5)
    T = np.eye(4, dtype=np.float32)[labels]
    g = Graph()
    x, t = g.leaf(X.shape, F32), g.leaf(T.shape, F32)
    loss = g.cross_entropy(x, t, "mean")
    (gx,) = g.gradient(loss, [x])
    got = graph_eval.evaluate(g.nodes, {x: X, t: T}, [loss, gx])
    x64 = X.astype(np.float64)
    p = np.exp(x64 - x64.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    np.testing.assert_allclose(got[loss][0], -np.log(p[np.arange(5), labels]).mean(), rtol=1e-6)
    np.testing.assert_allclose(got[gx], (p - T) / 5, rtol=1e-5, atol=1e-7)
    with pytest.raises(ValueError):
        g.cross_entropy(x, g.leaf((5,), F32))
    with pytest.raises(ValueError):
        g.cross_entropy(x, t, "median")


def test_something_that_only_resembles_a_cross_entropy_is_left_alone():
    g = Graph()
    x, t = g.leaf((6, 7), F32), g.leaf((6, 7), F32)
    # ln_softmax over the other axis; a different divisor
    a = g.mean(g.reduce(g.binary(g.unary(g.ln_softmax(x, [0]), UOp.Neg), t, BOp.Mul), BOp.Add, [1]))
    b = g.binary(g.sum_all(g.reduce(g.binary(g.unary(g.ln_softmax(x, [1]), UOp.Neg), t, BOp.Mul), BOp.Add, [1])),
                 g.const(7, F32), BOp.Div)
    assert scan_cross_entropy(g, range(len(g.nodes))) == {}
    c = g.cross_entropy(x, t)
    assert list(scan_cross_entropy(g, range(len(g.nodes)))) == [c]
    del a, b


def test_same_tree_binds_consistently():
    t = Graph()
    u = t.leaf((3,), F32)
    troot = t.binary(u, u, BOp.Mul)
    g = Graph()
    p, q = g.leaf((3,), F32), g.leaf((3,), F32)
    assert same_tree(g, g.binary(p, p, BOp.Mul), t, troot, {})
    assert not same_tree(g, g.binary(p, q, BOp.Mul), t, troot, {})
    assert not same_tree(g, g.binary(p, p, BOp.Add), t, troot, {})


def _linear_gelu(g, leaf, training):
    rng = np.random.default_rng(5)
    x = leaf(rng.standard_normal((8, 12)), F32)
    w, b = leaf(rng.standard_normal((16, 12)) * 0.3, F32), leaf(rng.standard_normal(16), F32)
    y = g.gelu(g.binary_b(g.dot(x, g.t(w)), b, BOp.Add))
    if not training:
        return [y], (x, w, b)
    loss = g.sum_all(g.binary(y, y, BOp.Mul))
    return [y] + g.gradient(loss, [w, b]), (x, w, b)


@pytest.mark.parametrize("training", [False, True])
def test_gelu_is_folded_only_where_nothing_reads_its_input(training):
    g, leaves, (outs, _) = _build(_linear_gelu, training=training)
    seen = []
    got = run_lowered(g, leaves, outs, match=True, seen=seen)
    want = graph_eval.evaluate(g.nodes, leaves, outs)
    first = next(k for k in seen if isinstance(k, Contraction))
    assert first.epilogue == ("bias" if training else "bias_gelu")  # the reverse pass reads the pre-activation
    for o in outs:
        np.testing.assert_allclose(got[o], want[o], rtol=1e-4, atol=1e-5)


def test_folded_relu_is_the_only_thing_stored():
    """h = relu(x . W^T + b) with a reverse pass: the pre-activation gets no buffer; every generated kernel that needs
    its sign reads h."""
    g, leaves, (loss, new, params, (x, onehot)) = _build(mlp_training_graph, batch=8, n_in=6, hidden=5, n_out=3)
    sched = lower(g, new + [loss], match=True)
    h = sched[0].out
    pre = g[h].src[1]
    stored = {k.out if not isinstance(k, LoweredKernel) else k.output for k in sched}
    assert pre not in stored and h in stored
    assert sched[3].relu_mask and sched[3].residual == h


def test_transformer_block_lowers_to_the_module_level_launches():
    """The block of zyx_amd/block.py written as graph nodes: with matching on, forward and backward come out as the
    launches that file lists by hand (norms, products with their epilogues, attention, column sums, the two norm
    backward passes with the skip gradient added in) plus generated elementwise kernels for gelu and gelu'."""
    from graph_cases import BLOCK_PARAMS, block_graph
    from zyx_amd.graph import AttentionBwdMatch, AttentionMatch, NormBwdMatch, NormRowsMatch
    g, leaves, (out, loss, P, xl, dl) = _build(block_graph)
    grads = g.gradient(loss, [P[n] for n in BLOCK_PARAMS] + [xl])
    outs = [out] + grads
    seen = []
    got = run_lowered(g, leaves, outs, match=True, seen=seen)
    want = graph_eval.evaluate(g.nodes, leaves, outs)
    for o in outs:
        np.testing.assert_allclose(got[o], want[o], rtol=2e-4, atol=2e-5)
    from zyx_amd.graph import Alias
    kinds = [type(k).__name__ for k in lower(g, outs, match=True) if not isinstance(k, Alias)]
    count = {k: kinds.count(k) for k in set(kinds)}
    assert len(kinds) == 24                 # 8 forward + 16 backward: the list zyx_amd/block.py writes by hand
    assert count["NormRowsMatch"] == 2 and count["NormBwdMatch"] == 2 and count["AttentionMatch"] == 1 and count["AttentionBwdMatch"] == 1
    assert count["Contraction"] == 12       # 4 Linear forward, 4 x (dW, dX) backward
    assert count.get("RowColReduce", 0) + count["LoweredKernel"] == 4 + 2   # the bias gradients' column sums; gelu and gelu'
    fwd = [k for k in seen if isinstance(k, Contraction) and k.epilogue == "bias"]
    assert sum(k.residual is not None for k in fwd) == 2          # both skip connections ride on a Linear's epilogue
    nb = [k for k in seen if isinstance(k, NormBwdMatch)]
    assert all(k.add is not None and k.dw is not None and k.db is not None for k in nb)
    assert [k.lse for k in seen if isinstance(k, AttentionMatch)] == [True]
    # forward alone: no row log-sum-exps asked of the attention kernel
    assert [k.lse for k in lower(g, [out], match=True) if isinstance(k, AttentionMatch)] == [False]
    # ... and gelu, whose input nothing reads any more, folds into the product before it: 7 launches
    assert len([k for k in lower(g, [out], match=True) if not isinstance(k, Alias)]) == 7


def test_norm_composites_against_closed_forms():
    rng = np.random.default_rng(4)
    X, W, T = rng.standard_normal((5, 12)), rng.standard_normal(12), rng.standard_normal((5, 12))
    g = Graph()
    x, w, t = (g.leaf(a.shape, DType.F64) for a in (X, W, T))
    y = g.rms_norm(x, w)
    (gx, gw) = g.gradient(g.sum_all(g.binary(y, t, BOp.Mul)), [x, w])
    got = graph_eval.evaluate(g.nodes, {x: X, w: W, t: T}, [y, gx, gw])
    r = np.sqrt(1.0 / ((X * X).mean(1, keepdims=True) + 1e-6))
    np.testing.assert_allclose(got[y], X * r * W, rtol=1e-12)
    gg = T * W
    np.testing.assert_allclose(got[gx], r * gg - r ** 3 * X * (gg * X).sum(1, keepdims=True) / 12, rtol=1e-10)
    np.testing.assert_allclose(got[gw], (T * X * r).sum(0), rtol=1e-10)
    seen = []
    low = run_lowered(g, {x: X.astype(np.float32), w: W.astype(np.float32), t: T.astype(np.float32)}, [y, gx, gw], match=True, seen=seen)
    assert seen == []  # f64 graphs stay on generated kernels
    del low
