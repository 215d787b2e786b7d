"""Graphs with known gradients, shared by the CPU and the GPU tests of zyx_amd.graph: the cases of
zyx/tests/11_autograd.rs with the values that file asserts, rebuilt node by node the way the reference's tensor
methods compose them (relu = cmpgt * x, dot = reshape / expand / mul / sum, broadcasting = reshape + expand).

A case is `(name, build)`; `build(g, leaf)` creates leaves through `leaf(array, dtype)` and returns
`(target, sources, expected)` with one expected array per source (None: only checked against the CPU evaluation)."""
from __future__ import annotations

import numpy as np

from zyx_amd import DType
from zyx_amd.ir import BOp, UOp

F32, F64, I32 = DType.F32, DType.F64, DType.I32
f32 = np.float32


def _unary_case(uop, data, expected, dtype=F32):
    def build(g, leaf):
        x = leaf(np.array(data), dtype)
        return g.unary(x, uop), [x], [np.array(expected)]
    return build


def _binary_case(bop, xd, yd, ex, ey, dtype=F32):
    def build(g, leaf):
        x, y = leaf(np.array(xd), dtype), leaf(np.array(yd), dtype)
        return g.binary(x, y, bop), [x, y], [None if ex is None else np.array(ex), None if ey is None else np.array(ey)]
    return build


def _relu_2(g, leaf):  # grad_relu_2 :18-27
    x = leaf(np.array([3, -2, 0]), I32)
    return g.relu(x), [x], [np.array([1, 0, 0])]


def _reshape(g, leaf):  # grad_reshape :295-304
    x = leaf(np.array([[4], [3], [1]]), I32)
    return g.reshape(x, [1, 3, 1, 1]), [x], [np.array([[1], [1], [1]])]


def _expand_1(g, leaf):  # grad_expand_1 :307-316
    x = leaf(np.array([[4], [3], [1]]), I32)
    return g.expand(x, [3, 4]), [x], [np.array([[4], [4], [4]])]


def _expand_2(g, leaf):  # grad_expand_2 :319-328
    x = leaf(np.array([4, 3, 1]), I32)
    return g.expand(g.reshape(x, [3, 1]), [3, 4]), [x], [np.array([4, 4, 4])]


def _permute(g, leaf):  # grad_permute :331-340
    x = leaf(np.array([[4], [3], [1]]), I32)
    return g.permute(x, [1, 0]), [x], [np.array([[1], [1], [1]])]


def _flip(g, leaf):  # grad_flip :343-352
    x = leaf(np.array([[4, 5], [3, 1]]), I32)
    return g.flip(x, [0, 1]), [x], [np.array([[1, 1], [1, 1]])]


def _dot(g, leaf):  # grad_dot :355-367
    x, y = leaf(np.array([2, 3, 1]), I32), leaf(np.array([[2], [3], [1]]), I32)
    return g.dot(x, y), [x, y], [np.array([2, 3, 1]), np.array([[2], [3], [1]])]


def _linear_1(g, leaf):  # grad_linear_1 :370-388
    x = leaf(np.array([2, 3, 1]), I32)
    w = leaf(np.array([2, 3, 1, 4, 5, 1, 6, 2, 3, 1, 6, 2, 4, 1, 4]).reshape(3, 5), I32)
    b = leaf(np.array([4, 1, 5, 7, 6]), I32)
    z = g.binary_b(g.dot(x, w), b, BOp.Add)
    return z, [w, b], [np.array([[2] * 5, [3] * 5, [1] * 5]), np.array([1] * 5)]


def _mse(g, leaf):  # grad_mse :391-407
    x, y = leaf(np.array([2, 3, 1]), F32), leaf(np.array([5, 1, 1]), F32)
    z = g.binary(x, y, BOp.Sub)
    return g.binary(z, z, BOp.Mul), [x, y], [np.array([-6, 4, 0]), np.array([6, -4, 0])]


def _linear_2(g, leaf):  # grad_linear_2 :410-466 (exact integers)
    x, y = leaf(np.array([2, 3, 1]), I32), leaf(np.array([5, 4, 5, 2]), I32)
    w1 = leaf(np.array([2, 3, 1, 4, 5, 1, 6, 2, 3, 1, 6, 2, 4, 1, 4]).reshape(3, 5), I32)
    b1 = leaf(np.array([4, 1, 5, 7, 6]), I32)
    w2 = leaf(np.array([2, 3, 1, 4, 5, 1, 6, 2, 3, 1, 6, 2, 4, 1, 4, 5, 1, 2, 4, 1]).reshape(5, 4), I32)
    b2 = leaf(np.array([4, 1, 5, 7]), I32)
    h = g.relu(g.binary_b(g.dot(x, w1), b1, BOp.Add))
    o = g.binary_b(g.binary_b(g.dot(h, w2), b2, BOp.Add), y, BOp.Sub)
    loss = g.sum_all(g.binary(o, o, BOp.Mul))
    return loss, [w1, b1, w2, b2], [
        np.array([[11528, 21316, 18580, 19872, 11476], [17292, 31974, 27870, 29808, 17214], [5764, 10658, 9290, 9936, 5738]]),
        np.array([5764, 10658, 9290, 9936, 5738]),
        np.array([[11628, 5542, 16082, 10506], [18468, 8802, 25542, 16686], [11628, 5542, 16082, 10506],
                  [17100, 8150, 23650, 15450], [15732, 7498, 21758, 14214]]),
        np.array([684, 326, 946, 618])]


def _t7(g, leaf):  # grad_t7 :486-499: the target is its own source
    x = leaf(np.linspace(0, 1, 800).reshape(8, 10, 10), F32)
    z = g.sum_all(x)
    return z, [z], [np.array([1.0])]


def _sum(g, leaf):  # grad_sum :694-706
    x = leaf(np.array([1, 2, 3]), F32)
    return g.sum_all(x), [x], [np.ones(3)]


def _max_1(g, leaf):  # grad_max_1 :709-722
    x = leaf(np.array([1, 3, 2]), F32)
    return g.max_all(x), [x], [np.array([0, 1, 0])]


def _cmplt_none(g, leaf):  # grad_cmplt_none :725-737
    x, y = leaf(np.array([1, 2, 3]), F32), leaf(np.array([2, 2, 2]), F32)
    return g.binary(x, y, BOp.Cmplt), [x], [np.zeros(3)]


def _maximum(g, leaf):  # grad_maximum :740-755
    x, y = leaf(np.array([1, 5, 2]), F32), leaf(np.array([2, 3, 3]), F32)
    return g.binary(x, y, BOp.Max), [x], [np.array([0, 1, 0])]


def _cmpgt_source(g, leaf):  # grad_cmpgt_source :796-824
    x, th, w = leaf(np.array([1, 2, 3]), F32), leaf(np.array([2]), F32), leaf(np.array([1, 1, 1]), F32)
    spike = g.cast(g.binary_b(x, th, BOp.Cmpgt), F32)
    loss = g.sum_all(g.binary(spike, w, BOp.Mul))
    return loss, [x, w], [np.zeros(3), np.array([0, 0, 1])]


_D = [0.5, 1.5, -0.5, -1.5, 0.1, 0.9, -0.1, -0.9, 2.3, -2.3]
CASES = [
    ("relu_2", _relu_2),
    ("reciprocal", _unary_case(UOp.Reciprocal, [3, 2, 4], [-0.11111111, -0.25, -0.0625])),                    # :30-39
    ("exp2", _unary_case(UOp.Exp2, [1, 2, 0.5], [f32(2) ** f32(v) * f32(np.log(2)) for v in (1, 2, 0.5)])),  # :42-53
    ("reciprocal_f64", _unary_case(UOp.Reciprocal, [2.0, -1.0, 0.5], [-0.25, -1.0, -4.0], F64)),              # :56-81
    ("floor", _unary_case(UOp.Floor, _D, [0.0] * 10, F64)),                                                   # :98-110
    ("trunc", _unary_case(UOp.Trunc, _D, [0.0] * 10, F64)),                                                   # :113-125
    ("pow_2", _binary_case(BOp.Pow, [2, 3, 4], [3, 2, 0.5], [12, 6, 0.25],
                           [f32(8) * np.log(f32(2)), f32(9) * np.log(f32(3)), f32(2) * np.log(f32(4))])),    # :128-162
    ("pow_3", _binary_case(BOp.Pow, [1.5, 2.3, 5.7], [0.7, 1.2, 0.3],
                           [y * x ** (y - 1) for x, y in zip((1.5, 2.3, 5.7), (0.7, 1.2, 0.3))],
                           [x ** y * np.log(x) for x, y in zip((1.5, 2.3, 5.7), (0.7, 1.2, 0.3))], F64)),     # :165-205
    ("cos_2", _unary_case(UOp.Cos, [3, 2, 4], [-0.14112, -0.9092974, 0.7568025])),                            # :208-217
    ("add_1", _binary_case(BOp.Add, [3, 2, 4], [3, 1, 5], [1, 1, 1], [1, 1, 1], I32)),                        # :220-232
    ("sub", _binary_case(BOp.Sub, [3, 2, 4], [3, 1, 5], [1, 1, 1], [-1, -1, -1], I32)),                       # :235-247
    ("mul", _binary_case(BOp.Mul, [3, 2, 4], [3, 1, 5], [3, 1, 5], [3, 2, 4], I32)),                          # :250-262
    ("div_1", _binary_case(BOp.Div, [3, 2, 4], [3, 1, 5], [0.33333334, 1, 0.2], [-0.33333334, -2, -0.16])),  # :265-277
    ("pow", _binary_case(BOp.Pow, [3, 2, 4], [3, 1, 5], [27, 1, 1280], [29.66253, 1.3862944, 1419.5654])),   # :280-292
    ("reshape", _reshape), ("expand_1", _expand_1), ("expand_2", _expand_2), ("permute", _permute), ("flip", _flip),
    ("dot", _dot), ("linear_1", _linear_1), ("mse", _mse), ("linear_2", _linear_2), ("t7", _t7),
    ("add_2", _binary_case(BOp.Add, [1, 2, 3], [4, 5, 6], [1, 1, 1], None)),                                  # :502-516
    ("sub_2", _binary_case(BOp.Sub, [1, 2, 3], [4, 5, 6], [1, 1, 1], None)),                                  # :519-532
    ("mul_2", _binary_case(BOp.Mul, [1, 2, 3], [4, 5, 6], [4, 5, 6], None)),                                  # :535-548
    ("div_2", _binary_case(BOp.Div, [2, 4, 6], [1, 2, 3], [1.0, 0.5, f32(1) / f32(3)], None)),                # :551-565
    ("pow_4", _binary_case(BOp.Pow, [1, 2, 3], [2, 2, 2], [2, 4, 6], None)),                                  # :568-581
    ("neg", _unary_case(UOp.Neg, [1, -2, 3], [-1, -1, -1])),                                                  # :584-596
    ("log2", _unary_case(UOp.Log2, [1, 2, 4], [1 / (f32(v) * f32(np.log(2))) for v in (1, 2, 4)])),           # :599-611
    ("ln", _unary_case(UOp.Ln, [1, 2, 4], [1, 0.5, 0.25])),                                                   # :614-626
    ("reciprocal_3", _unary_case(UOp.Reciprocal, [1, 2, 4], [-1, -0.25, -0.0625])),                           # :629-642
    ("sqrt", _unary_case(UOp.Sqrt, [1, 4, 9], [0.5, 0.25, f32(1) / f32(6)])),                                 # :645-658
    ("sin_1", _unary_case(UOp.Sin, [0, 1, 2], np.cos(np.array([0, 1, 2], f32)))),                            # :661-676
    ("cos", _unary_case(UOp.Cos, [0, 1, 2], -np.sin(np.array([0, 1, 2], f32)))),                             # :679-691
    ("sum", _sum), ("max_1", _max_1), ("cmplt_none", _cmplt_none), ("maximum", _maximum),
    ("cmpgt_source", _cmpgt_source),
]


# ---- seeded graphs for finite differences and device parity ----------------------------------------------------------

def mixed_graph(g, leaf, seed=0, dtype=F64):
    """Every differentiable node kind in one scalar loss over small tensors with values away from the kinks."""
    r = np.random.default_rng(seed)
    a = leaf(r.uniform(0.5, 2.0, (3, 4)), dtype)
    b = leaf(r.uniform(0.5, 2.0, (4,)), dtype)
    c = leaf(r.uniform(-1.0, 1.0, (4, 3)), dtype)
    u = g.binary_b(a, b, BOp.Mul)                                  # broadcast row vector
    u = g.binary(g.unary(u, UOp.Sqrt), g.unary(a, UOp.Ln), BOp.Add)
    u = g.binary(u, g.unary(g.unary(a, UOp.Exp2), UOp.Reciprocal), BOp.Sub)
    v = g.dot(u, c)                                                # [3, 3]
    v = g.binary(g.unary(v, UOp.Sin), g.unary(g.permute(v, [1, 0]), UOp.Cos), BOp.Mul)
    v = g.binary(v, g.flip(v, [0]), BOp.Add)
    w = g.binary(g.unary(g.reshape(v, [9]), UOp.Exp), g.const(3.0, dtype), BOp.Div)
    m = g.reduce(g.binary_b(a, g.reshape(g.reduce(c, BOp.Max, [1]), [1, 4]), BOp.Max), BOp.Max, [0])   # [4]
    p = g.binary(g.unary(g.unary(b, UOp.Neg), UOp.Abs), g.unary(b, UOp.Log2), BOp.Pow)
    loss = g.binary(g.sum_all(w), g.sum_all(g.binary(m, p, BOp.Mul)), BOp.Add)
    return loss, [a, b, c]


def mlp_graph(g, leaf, batch=8, n_in=12, hidden=16, n_out=5, seed=1, dtype=F32):
    """zz_bw_relu_matmul :908-927 at a small size: two Linear layers ([out, in] weights), relu, loss = sum of logits."""
    r = np.random.default_rng(seed)
    x = leaf(r.standard_normal((batch, n_in)), dtype)
    w1, b1 = leaf(r.standard_normal((hidden, n_in)), dtype), leaf(r.standard_normal((hidden,)), dtype)
    w2, b2 = leaf(r.standard_normal((n_out, hidden)), dtype), leaf(r.standard_normal((n_out,)), dtype)
    l1 = g.relu(g.binary_b(g.dot(x, g.t(w1)), b1, BOp.Add))
    logits = g.binary_b(g.dot(l1, g.t(w2)), b2, BOp.Add)
    return g.sum_all(logits), [w1, b1, w2, b2], (x, w1, b1, w2, b2)


def attention_graph(g, leaf, b=2, h=2, t=24, dh=8, seed=3, causal=False, p=0.0, training=False, dtype=F32):
    """Core of CausalSelfAttention::forward (zyx-nn/src/causal_self_attention.rs:50-70) as graph nodes: scores
    q.k^T * scale, optional additive mask (0 / -inf above the diagonal), softmax over keys, dropout (evaluation
    scale, or the training mask from a uniform tensor), . v. Loss = sum(y * dy) so that d loss / d(q, k, v) is the
    backward of the fused kernel for the upstream gradient dy. Returns (loss, [q, k, v], (y, arrays))."""
    r = np.random.default_rng(seed)
    arrs = {n: r.standard_normal((b, h, t, dh)) for n in ("q", "k", "v", "dy")}
    q, k, v, dy = (leaf(arrs[n], dtype) for n in ("q", "k", "v", "dy"))
    att = g.binary(g.dot(q, g.t(k)), g.const(float(np.float32(1.0 / np.sqrt(dh))), dtype), BOp.Mul)
    if causal:
        mask = leaf(np.where(np.tril(np.ones((t, t), bool)), 0.0, -np.inf), dtype)
        att = g.binary_b(att, mask, BOp.Add)
    att = g.softmax(att, [-1])
    if training:
        arrs["u"] = r.uniform(0, 1, (b, h, t, t))
        att = g.dropout(att, p, leaf(arrs["u"], dtype))
    elif p:
        att = g.dropout(att, p)
    y = g.dot(att, v)
    loss = g.sum_all(g.binary(y, dy, BOp.Mul))
    return loss, [q, k, v], (y, arrs)


def mlp_training_graph(g, leaf, batch=64, n_in=784, hidden=128, n_out=10, lr=0.01, seed=4):
    """The MNIST network's training step as one graph (zyx/tests/mnist.rs:54-66): Linear, relu, Linear,
    cross_entropy(one_hot(labels), Mean) (tensor/mod.rs:1639-1655),
    gradients by the reverse rules, `w - g * lr`. Returns (loss, new parameters, parameter leaves, (x, onehot))."""
    r = np.random.default_rng(seed)
    k1, k2 = 1 / np.sqrt(n_in), 1 / np.sqrt(hidden)
    x = leaf(np.zeros((batch, n_in)), F32)
    onehot = leaf(np.zeros((batch, n_out)), F32)
    w1, b1 = leaf(r.uniform(-k1, k1, (hidden, n_in)), F32), leaf(r.uniform(-k1, k1, (hidden,)), F32)
    w2, b2 = leaf(r.uniform(-k2, k2, (n_out, hidden)), F32), leaf(r.uniform(-k2, k2, (n_out,)), F32)
    h = g.relu(g.binary_b(g.dot(x, g.t(w1)), b1, BOp.Add))
    logits = g.binary_b(g.dot(h, g.t(w2)), b2, BOp.Add)
    loss = g.cross_entropy(logits, onehot, "mean")
    params = [w1, b1, w2, b2]
    grads = g.gradient(loss, params)
    lr_c = g.const(lr, F32)
    new = [g.binary(p, g.binary(gr, lr_c, BOp.Mul), BOp.Sub) for p, gr in zip(params, grads)]
    return loss, new, params, (x, onehot)


BLOCK_PARAMS = ("ln1_w", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b", "ln2_w", "ln2_b", "fc_w", "fc_b", "proj2_w", "proj2_b")


def block_graph(g, leaf, b=2, t=16, d=32, n_head=4, dtype=F32, seed=7, params=None, x=None, dout=None):
    """One pre-norm transformer block `x = x + attn(ln_1(x)); x = x + mlp(ln_2(x))` (zyx-examples/examples/nanogpt.rs:
    68-98) from zyx-nn modules written as graph nodes: LayerNorm, CausalSelfAttention (c_attn Linear, the attention
    core, c_proj Linear), MLP = Linear d -> 4d, gelu, Linear 4d -> d; rows are (batch, position) pairs. The loss is
    sum(out * dout), so the gradients are those of the block for the upstream gradient dout.
    Returns (out, loss, parameter leaves by name, x leaf, dout leaf)."""
    r = np.random.default_rng(seed)
    f = 4 * d
    shapes = dict(ln1_w=(d,), ln1_b=(d,), attn_w=(3 * d, d), attn_b=(3 * d,), proj_w=(d, d), proj_b=(d,),
                  ln2_w=(d,), ln2_b=(d,), fc_w=(f, d), fc_b=(f,), proj2_w=(d, f), proj2_b=(d,))
    if params is None:
        params = {n: (1.0 + 0.1 * r.standard_normal(s)) if n in ("ln1_w", "ln2_w") else 0.02 * r.standard_normal(s) if n.endswith("_w")
                  else 0.01 * r.standard_normal(s) for n, s in shapes.items()}
    P = {n: leaf(np.asarray(params[n]).reshape(shapes[n]), dtype) for n in BLOCK_PARAMS}
    xl = leaf(r.standard_normal((b, t, d)) if x is None else x, dtype)
    dl = leaf(r.standard_normal((b, t, d)) if dout is None else dout, dtype)

    def linear(v, w, bias):  # zyx-nn/src/linear.rs:38-44
        return g.binary_b(g.dot(v, g.t(P[w])), P[bias], BOp.Add)

    n1 = g.layer_norm(xl, P["ln1_w"], P["ln1_b"])
    att = g.self_attention(linear(n1, "attn_w", "attn_b"), n_head)
    x2 = g.binary(linear(att, "proj_w", "proj_b"), xl, BOp.Add)
    n2 = g.layer_norm(x2, P["ln2_w"], P["ln2_b"])
    hid = g.gelu(linear(n2, "fc_w", "fc_b"))
    out = g.binary(linear(hid, "proj2_w", "proj2_b"), x2, BOp.Add)
    loss = g.sum_all(g.binary(out, dl, BOp.Mul))
    return out, loss, P, xl, dl
