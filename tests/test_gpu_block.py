"""Pre-norm transformer block (config 5: LayerNorm, attention, 4x MLP, forward + backward) on the GPU.

Two kinds of check. Launch by launch: every kernel of the plan is compared with the oracle's op evaluated on the
inputs the GPU itself gave that kernel (so one bf16 truncating store and one kernel's arithmetic separate the two).
End to end: outputs and gradients against the f64 block (oracle.block_forward_f64 / block_backward_f64, pinned by
finite differences), where the bf16 stores of ~20 chained tensors accumulate, with a correspondingly looser bound.

bf16 tolerance per launch: 2^-7 |want| (truncating store) + 1e-3 * mag (f32-accumulated bf16 products, north star),
mag = the sum of absolute values of the terms of each output element.
"""
import numpy as np
import pytest

from zyx_amd import DType
from zyx_amd.block import PARAMS, TransformerBlock

pytestmark = pytest.mark.gpu


def test_block_with_causal_mask(hip, oracle):
    """The mask the reference's module lacks (a flag of the attention launches): f32 on the general kernels and bf16
    on the matrix-core kernels against the masked f64 block."""
    B, T, d, H = 2, 5, 8, 2
    blk, p, x, dout = make_block(hip, oracle, B, T, d, H, DType.F32, std=0.3, causal=True)
    blk.forward_backward()
    s = oracle.block_forward_f64(p, x.reshape(B, T, d), H, causal=True)
    g = oracle.block_backward_f64(p, s, dout.reshape(B, T, d), H)
    assert np.allclose(blk.read("out").reshape(B, T, d), s["out"], rtol=1e-4, atol=1e-5)
    assert np.allclose(blk.read("dx").reshape(B, T, d), g["dx"], rtol=1e-4, atol=2e-5)
    for n in PARAMS:
        assert np.allclose(blk.read("d_" + n), g[n], rtol=1e-4, atol=2e-5), n
    blk.close()
    B, T, d, H = 2, 256, 256, 4
    blk, p, x, dout = make_block(hip, oracle, B, T, d, H, DType.BF16, std=0.05, causal=True)
    blk.forward_backward()
    pf = {k: f64(oracle, v) for k, v in p.items()}
    s = oracle.block_forward_f64(pf, f64(oracle, x).reshape(B, T, d), H, causal=True)
    g = oracle.block_backward_f64(pf, s, f64(oracle, dout).reshape(B, T, d), H)
    rel = lambda got, want: np.abs(f64(oracle, got).reshape(want.shape) - want).max() / np.abs(want).max()
    assert rel(blk.read("att"), s["att"]) < 0.02 and rel(blk.read("out"), s["out"]) < 0.02
    assert rel(blk.read("dx"), g["dx"]) < 0.03
    for n in PARAMS:
        assert rel(blk.read("d_" + n), g[n]) < 0.03, n
    blk.close()


def f64(oracle, a):
    return (oracle.bf16_to_f32(a) if a.dtype == np.uint16 else a).astype(np.float64)


def close_bf16(oracle, got, want, mag, extra=0.0):
    return np.abs(f64(oracle, got) - want) <= 2.0 ** -7 * np.abs(want) + (1e-3 + extra) * mag + 1e-30


def make_block(hip, oracle, B, T, d, H, dtype, seed=1, std=0.02, causal=False):
    dev, pool = hip
    blk = TransformerBlock(dev, pool, B, T, d, H, dtype, causal=causal)
    p = oracle.block_init(d, H, seed, std)
    r = oracle.Rng(seed + 1)
    # non-trivial affine parts and biases so that every gradient path is exercised
    for k in ("ln1_w", "ln2_w"):
        p[k] = (1.0 + 0.1 * r.randn(p[k].shape)).astype(np.float32)
    for k in ("ln1_b", "ln2_b", "attn_b", "proj_b", "fc_b", "proj2_b"):
        p[k] = (0.1 * r.randn(p[k].shape)).astype(np.float32)
    x, dout = r.randn((B * T, d)), r.randn((B * T, d))
    conv = oracle.f32_to_bf16 if dtype == DType.BF16 else (lambda a: a)
    p = {k: conv(v) for k, v in p.items()}
    x, dout = conv(x), conv(dout)
    blk.set_params(p)
    blk.write("x", x)
    blk.write("dout", dout)
    return blk, p, x, dout


def check_launches(oracle, blk, p, B, T, d, H):
    """Every launch against the oracle's op on the GPU's own inputs (bf16 storage)."""
    o, BF = oracle, oracle.BF16
    t = {n: blk.read(n) for n in ("x", "n1", "qkv", "att", "lse", "x2", "n2", "h", "g", "out", "dout", "dg", "dh", "dn2", "dx2",
                                  "datt", "dqkv", "dn1", "dx")}
    gr = {n: blk.read("d_" + n) for n in PARAMS}
    F = lambda a: f64(o, a)
    ulp = lambda got, want, atol: np.abs(F(got) - F(want)) <= 2.0 ** -7 * np.abs(F(want)) + atol

    def linear_ok(out, inp, w, b, res=None):
        want = F(inp) @ F(w).T + F(b) + (F(res) if res is not None else 0.0)
        mag = np.abs(F(inp)) @ np.abs(F(w)).T + np.abs(F(b)) + (np.abs(F(res)) if res is not None else 0.0)
        return np.all(close_bf16(o, out, want, mag))

    def products_ok(out, a, b):  # out = a . b in f64
        return np.all(close_bf16(o, out, F(a) @ F(b), np.abs(F(a)) @ np.abs(F(b))))

    # forward
    assert np.all(ulp(t["n1"], o.layer_norm(t["x"], p["ln1_w"], p["ln1_b"], dtype=BF), 1e-5))
    assert linear_ok(t["qkv"], t["n1"], p["attn_w"], p["attn_b"])
    ref_att, ref_lse = o.attention(t["qkv"].reshape(B, T, 3 * d), H, dtype=BF, want_lse=True)
    qf = F(t["qkv"]).reshape(B, T, 3, H, d // H)
    vmag = np.abs(qf[:, :, 2]).max()
    assert np.all(np.abs(F(t["att"]) - F(ref_att).reshape(B * T, d)) <= 2.0 ** -6 * np.abs(F(ref_att).reshape(B * T, d)) + 3e-3 * vmag)
    assert np.allclose(t["lse"], ref_lse, rtol=1e-4, atol=1e-4)
    assert linear_ok(t["x2"], t["att"], p["proj_w"], p["proj_b"], t["x"])
    assert np.all(ulp(t["n2"], o.layer_norm(t["x2"], p["ln2_w"], p["ln2_b"], dtype=BF), 1e-5))
    assert linear_ok(t["h"], t["n2"], p["fc_w"], p["fc_b"])
    assert np.all(ulp(t["g"], o.unary("gelu", t["h"], BF), 1e-6))
    assert linear_ok(t["out"], t["g"], p["proj2_w"], p["proj2_b"], t["x2"])
    # backward
    colsum_ok = lambda out, a: np.all(close_bf16(o, out, F(a).sum(0), np.abs(F(a)).sum(0)))
    assert colsum_ok(gr["proj2_b"], t["dout"]) and products_ok(gr["proj2_w"], t["dout"].T, t["g"]) and products_ok(t["dg"], t["dout"], p["proj2_w"])
    from zyx_amd.kernels import Chain
    c = Chain(*t["h"].shape, out_dtype=DType.BF16)
    ih, ig = c.input(DType.BF16), c.input(DType.BF16)
    c.load(ih).gelu_grad().mul(ig)
    assert np.all(ulp(t["dh"], o.ew_chain(c, [t["h"], t["dg"]]), 1e-6))
    assert colsum_ok(gr["fc_b"], t["dh"]) and products_ok(gr["fc_w"], t["dh"].T, t["n2"]) and products_ok(t["dn2"], t["dh"], p["fc_w"])
    rows = t["x"].shape[0]
    for dxn, xn, wn, dyn, addn, gw, gb in (("dx2", "x2", "ln2_w", "dn2", "dout", "ln2_w", "ln2_b"), ("dx", "x", "ln1_w", "dn1", "dx2", "ln1_w", "ln1_b")):
        wdx, wdw, wdb = o.norm_bwd(t[xn], t[dyn], p[wn], t[addn], dtype=BF)
        scale = np.abs(F(t[dyn])).max()
        assert np.all(ulp(t[dxn], wdx, 1e-4 * scale))
        assert np.all(ulp(gr[gw], wdw, 1e-4 * scale * np.sqrt(rows) * 4)) and np.all(ulp(gr[gb], wdb, 1e-4 * scale * np.sqrt(rows) * 4))
    assert colsum_ok(gr["proj_b"], t["dx2"]) and products_ok(gr["proj_w"], t["dx2"].T, t["att"]) and products_ok(t["datt"], t["dx2"], p["proj_w"])
    want = F(o.attention_bwd(t["qkv"].reshape(B, T, 3 * d), t["datt"].reshape(B, T, d), H, dtype=BF)).reshape(B * T, 3 * d)
    gscale = np.abs(F(t["datt"])).max() * max(1.0, np.abs(qf).max())
    assert np.all(np.abs(F(t["dqkv"]) - want) <= 2.0 ** -6 * np.abs(want) + 6e-3 * gscale)
    assert colsum_ok(gr["attn_b"], t["dqkv"]) and products_ok(gr["attn_w"], t["dqkv"].T, t["n1"]) and products_ok(t["dn1"], t["dqkv"], p["attn_w"])
    return t, gr


def test_block_bf16_every_launch_and_end_to_end(hip, oracle):
    B, T, d, H = 2, 128, 256, 4
    blk, p, x, dout = make_block(hip, oracle, B, T, d, H, DType.BF16, std=0.05)
    blk.forward_backward()
    t, gr = check_launches(oracle, blk, p, B, T, d, H)
    # the unplanned launch list gives the same bits as the captured plan
    blk.forward_backward_unplanned()
    assert np.array_equal(blk.read("dx"), t["dx"]) and np.array_equal(blk.read("d_attn_w"), gr["attn_w"])
    # end to end against f64: ~20 chained bf16 tensors, each store truncating up to 2^-7
    pf = {k: f64(oracle, v) for k, v in p.items()}
    s = oracle.block_forward_f64(pf, f64(oracle, x).reshape(B, T, d), H)
    g = oracle.block_backward_f64(pf, s, f64(oracle, dout).reshape(B, T, d), H)
    rel = lambda got, want: np.abs(f64(oracle, got).reshape(want.shape) - want).max() / np.abs(want).max()
    assert rel(t["out"], s["out"]) < 0.02
    assert rel(t["dx"], g["dx"]) < 0.03
    for n in PARAMS:
        assert rel(gr[n], g[n]) < 0.03, n
    blk.close()


def test_block_f32_small_uses_general_kernels(hip, oracle):
    B, T, d, H = 2, 5, 8, 2
    blk, p, x, dout = make_block(hip, oracle, B, T, d, H, DType.F32, std=0.3)
    blk.forward_backward()
    s = oracle.block_forward_f64(p, x.reshape(B, T, d), H)
    g = oracle.block_backward_f64(p, s, dout.reshape(B, T, d), H)
    assert np.allclose(blk.read("out").reshape(B, T, d), s["out"], rtol=1e-4, atol=1e-5)
    assert np.allclose(blk.read("dx").reshape(B, T, d), g["dx"], rtol=1e-4, atol=2e-5)
    for n in PARAMS:
        assert np.allclose(blk.read("d_" + n), g[n], rtol=1e-4, atol=2e-5), n
    blk.forward()
    assert np.allclose(blk.read("out").reshape(B, T, d), s["out"], rtol=1e-4, atol=1e-5)
    blk.close()


def test_config5_block_full_size(hip, oracle):
    """B=8, T=1024, d=1024, 16 heads, bf16, weights 0.02 * randn, loss = sum(out) (dout = 1): sampled rows of every
    launch against f64 products of the GPU's own inputs, and column-sum identities over whole tensors."""
    dev, pool = hip
    B, T, d, H = 8, 1024, 1024, 16
    blk = TransformerBlock(dev, pool, B, T, d, H, DType.BF16)
    p = {k: oracle.f32_to_bf16(v) for k, v in oracle.block_init(d, H).items()}
    blk.set_params(p)
    x = oracle.f32_to_bf16(oracle.Rng(5).randn((B * T, d)))
    blk.write("x", x)
    blk.write("dout", oracle.f32_to_bf16(np.ones((B * T, d), np.float32)))
    blk.forward_backward()
    F = lambda a: f64(oracle, a)
    rows = np.arange(7, B * T, 611)
    t = {n: blk.read(n) for n in ("n1", "qkv", "att", "x2", "n2", "h", "g", "out", "dg", "dh", "dn2", "dx2", "datt", "dqkv", "dn1", "dx")}

    def lin(out, inp, w, b, res=None):
        want = F(t[inp][rows]) @ F(p[w]).T + F(p[b]) + (F(res[rows]) if res is not None else 0.0)
        mag = np.abs(F(t[inp][rows])) @ np.abs(F(p[w])).T + np.abs(F(p[b])) + (np.abs(F(res[rows])) if res is not None else 0.0)
        assert np.all(close_bf16(oracle, t[out][rows], want, mag)), out

    assert np.all(np.abs(F(t["n1"][rows]) - F(oracle.layer_norm(x[rows], p["ln1_w"], p["ln1_b"], dtype=oracle.BF16))) <= 2.0 ** -7 * np.abs(F(t["n1"][rows])) + 1e-5)
    lin("qkv", "n1", "attn_w", "attn_b")
    ref = oracle.attention(t["qkv"].reshape(B, T, 3 * d), H, dtype=oracle.BF16)
    vmax = np.abs(F(t["qkv"])[:, 2 * d:]).max()
    assert np.all(np.abs(F(t["att"]) - F(ref).reshape(B * T, d)) <= 2.0 ** -6 * np.abs(F(ref).reshape(B * T, d)) + 3e-3 * vmax)
    lin("x2", "att", "proj_w", "proj_b", x)
    lin("h", "n2", "fc_w", "fc_b")
    lin("out", "g", "proj2_w", "proj2_b", t["x2"])
    # backward products on sampled rows: dX = dY . W
    for out, dy, w in (("dg", None, "proj2_w"), ("dn2", "dh", "fc_w"), ("datt", "dx2", "proj_w"), ("dn1", "dqkv", "attn_w")):
        dyv = np.ones((len(rows), d)) if dy is None else F(t[dy][rows])
        assert np.all(close_bf16(oracle, t[out][rows], dyv @ F(p[w]), np.abs(dyv) @ np.abs(F(p[w])))), out
    # weight gradients on sampled output rows: dW[r, :] = sum_m dY[m, r] X[m, :]
    for name, dy, inp in (("fc_w", "dh", "n2"), ("attn_w", "dqkv", "n1"), ("proj_w", "dx2", "att")):
        got = blk.read("d_" + name)
        sel = np.arange(3, got.shape[0], got.shape[0] // 8)
        want = F(t[dy][:, sel]).T @ F(t[inp])
        mag = np.abs(F(t[dy][:, sel])).T @ np.abs(F(t[inp]))
        assert np.all(close_bf16(oracle, got[sel], want, mag)), name
    # bias gradients are column sums of the tensors they were reduced from
    for name, src in (("fc_b", "dh"), ("attn_b", "dqkv"), ("proj_b", "dx2")):
        want, mag = F(t[src]).sum(0), np.abs(F(t[src])).sum(0)
        assert np.all(close_bf16(oracle, blk.read("d_" + name), want, mag)), name
    assert np.all(f64(oracle, blk.read("d_proj2_b")) == B * T)  # column sums of ones: 8192, exact in bf16
    # rows of softmax sum to one: column sums of dV per head equal those of datt (d/dv linearity)
    dv = F(t["dqkv"])[:, 2 * d:].reshape(B, T, d).sum(1)
    da = F(t["datt"]).reshape(B, T, d)
    assert np.all(np.abs(dv - da.sum(1)) <= 2.0 ** -6 * np.abs(da).sum(1) + 1e-6)
    blk.close()


@pytest.mark.parametrize("dtype", [DType.BF16, DType.F32])
def test_block_written_as_graph_nodes_gives_the_hand_written_launch_list(hip, oracle, dtype):
    """The same block built from graph nodes (layer_norm, Linear, self_attention, gelu, skip connections), its
    gradients taken by the reverse rules and everything lowered with matching on: 24 launches like the list in
    zyx_amd/block.py, the same kernel kinds, and the results of that list. bf16: the two paths share every
    hand-written kernel and differ in gelu / gelu' (generated from the expression here, one fused op there): both
    store bf16, so values agree to a few bf16 steps of the tensors they go through; bit equality is asserted where
    only shared kernels are involved (n1, qkv, att, x2, n2, h)."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    from graph_cases import BLOCK_PARAMS, block_graph
    from zyx_amd.graph import Alias, Tape, lower, storage_dtype
    dev, pool = hip
    B, T, d, H = 2, 128, 256, 4
    blk, p, x, dout = make_block(hip, oracle, B, T, d, H, dtype, std=0.05)
    blk.forward_backward()
    tape, leaves = Tape(dev, pool, match=True), {}

    def leaf(array, dt):
        a = np.ascontiguousarray(array)
        nid = tape.tensor(a, dt)
        leaves[nid] = a
        return nid

    g = tape.graph
    out, loss, P, xl, dl = block_graph(g, leaf, B, T, d, H, dtype, params=p, x=x.reshape(B, T, d), dout=dout.reshape(B, T, d))
    grads = tape.gradient(loss, [P[n] for n in BLOCK_PARAMS] + [xl])
    nodes = [out] + grads
    sched = [k for k in lower(g, nodes, stored=list(leaves), match=True) if not isinstance(k, Alias)]
    assert len(sched) == len(blk.forward_nodes) + len(blk.backward_nodes) == 24
    tape.realize(nodes)
    assert tape.matched == 24 - 2 if dtype == DType.BF16 else tape.matched >= 18  # all but gelu and gelu' (f32 at this size: short column sums are generated too)
    F = lambda a: f64(oracle, np.asarray(a))
    inter = {"n1": None, "qkv": None, "att": None, "x2": None, "n2": None, "h": None}
    comps = [k for k, v in g.composites.items()]
    by_name = {"n1": comps[0], "att": comps[1], "n2": comps[2]}
    for name, nid in by_name.items():
        assert np.array_equal(tape.numpy(nid).reshape(-1), blk.read(name).reshape(-1)), name
    scale = lambda a: np.abs(F(a)).max()
    got_out, want_out = tape.numpy(out).reshape(B * T, d), blk.read("out")
    assert np.abs(F(got_out) - F(want_out)).max() <= 2.0 ** -6 * scale(want_out)
    for n, gid in zip(list(BLOCK_PARAMS) + ["x"], grads):
        want = blk.read("dx" if n == "x" else "d_" + n)
        got = tape.numpy(gid).reshape(want.shape)
        assert np.abs(F(got) - F(want)).max() <= 2.0 ** -5 * scale(want), n
    del inter
    tape.close()
    blk.close()
