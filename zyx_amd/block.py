"""The launch list of one pre-norm transformer block, forward and backward, as zyx's Tape would hand it to
the device once its plan is cached (zyx/src/tape.rs:141-202 -> zyx/src/graph/plan.rs:271-361).

The block is `x = x + attn(ln_1(x)); x = x + mlp(ln_2(x))` of zyx-examples/examples/nanogpt.rs:68-98 built from
zyx-nn modules: LayerNorm (zyx-nn/src/layer_norm.rs:98-135), CausalSelfAttention
(zyx-nn/src/causal_self_attention.rs:36-74: c_attn Linear d -> 3d, per-head softmax(q k^T / sqrt(dh)) v with no
mask -- `causal=True` adds the lower-triangular one --, c_proj Linear d -> d), MLP = Linear d -> 4d, gelu, Linear 4d -> d (nanogpt.rs:41-66), Linear weights stored
[out, in] (zyx-nn/src/linear.rs:24-44). Every tensor a module returns is stored once in `dtype` (bf16 stores
truncate); arithmetic inside a kernel is f32.

Forward, 8 launches:
    n1  = LayerNorm(x)                          row kernel
    qkv = n1 . W_attn^T + b_attn                GEMM, bias epilogue
    att = attention(qkv) (+ lse)                fused attention
    x2  = att . W_proj^T + b_proj + x           GEMM, bias + residual epilogue
    n2  = LayerNorm(x2)                         row kernel
    h   = n2 . W_fc^T + b_fc                    GEMM, bias epilogue
    g   = gelu(h)                               elementwise chain
    out = g . W_proj2^T + b_proj2 + x2          GEMM, bias + residual epilogue
Backward of `sum(out * dout)` (Runtime::gradient, zyx/src/graph/autograd.rs:14-424, evaluated with one fused
kernel per module-level rule), 16 launches: for every Linear dW = dY^T . X (GEMM, A transposed), db = column sum
of dY, dX = dY . W (GEMM); gelu' chain; LayerNorm backward with the skip branch added in the same pass;
attention backward.
"""
from __future__ import annotations

import numpy as np

from . import kernels as K
from .backend import DType, HIPDevice, HIPMemoryPool

PARAMS = ("ln1_w", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b", "ln2_w", "ln2_b", "fc_w", "fc_b", "proj2_w", "proj2_b")


class TransformerBlock:
    def __init__(self, dev: HIPDevice, pool: HIPMemoryPool, batch: int, seq: int, d_model: int, n_head: int,
                 dtype: DType = DType.BF16, eps: float = 1e-5, dropout_p: float = 0.0, mlp_ratio: int = 4,
                 causal: bool = False):
        self.dev, self.pool, self.dtype = dev, pool, DType(dtype)
        self.batch, self.seq, self.d, self.n_head, self.hidden = batch, seq, d_model, n_head, mlp_ratio * d_model
        self.np_dtype = np.uint16 if self.dtype == DType.BF16 else np.float32
        isz = np.dtype(self.np_dtype).itemsize
        m, d, f, dt = batch * seq, d_model, self.hidden, self.dtype
        self._bufs, self._progs, self.shapes = {}, [], {}
        self._pending = []

        def buf(name, shape, itemsize=isz):
            b, ev = pool.allocate((int(np.prod(shape)) + 1) * itemsize)  # + one trash element, as zyx's Allocate node does
            pool.sync_events([ev])
            self._bufs[name], self.shapes[name] = b, tuple(shape)
            return b

        def prog(desc):
            p = dev.register_kernel(desc)
            self._progs.append(p)
            return p

        self.param_shapes = dict(ln1_w=(d,), ln1_b=(d,), attn_w=(3 * d, d), attn_b=(3 * d,), proj_w=(d, d), proj_b=(d,),
                                 ln2_w=(d,), ln2_b=(d,), fc_w=(f, d), fc_b=(f,), proj2_w=(d, f), proj2_b=(d,))
        P = {n: buf(n, s) for n, s in self.param_shapes.items()}
        G = {n: buf("d_" + n, s) for n, s in self.param_shapes.items()}
        x, n1, qkv, att = buf("x", (m, d)), buf("n1", (m, d)), buf("qkv", (m, 3 * d)), buf("att", (m, d))
        lse = buf("lse", (batch, n_head, seq), 4)
        x2, n2, h, g, out = buf("x2", (m, d)), buf("n2", (m, d)), buf("h", (m, f)), buf("g", (m, f)), buf("out", (m, d))
        dout, dg, dh, dn2, dx2 = buf("dout", (m, d)), buf("dg", (m, f)), buf("dh", (m, f)), buf("dn2", (m, d)), buf("dx2", (m, d))
        datt, dqkv, dn1, dx = buf("datt", (m, d)), buf("dqkv", (m, 3 * d)), buf("dn1", (m, d)), buf("dx", (m, d))

        gelu = K.Chain(m, f, out_dtype=dt)
        gelu.load(gelu.input(dt)).gelu()
        gelu_bwd = K.Chain(m, f, out_dtype=dt)
        ih, ig = gelu_bwd.input(dt), gelu_bwd.input(dt)
        gelu_bwd.load(ih).gelu_grad().mul(ig)

        def linear(rows, n_out, n_in, residual=False):
            return prog(K.gemm_desc(rows, n_out, n_in, dt, dt, trans_b=True, epilogue="bias", bias_dtype=dt, residual=residual))

        ln = prog(K.norm_rows_desc(m, d, eps=eps, dtype=dt))
        ln_bwd = prog(K.norm_rows_bwd_desc(m, d, add=True, eps=eps, dtype=dt))
        ln_bwd2 = prog(K.norm_rows_bwd_desc(m, d, add=True, eps=eps, dtype=dt))  # own workspace: a program's scratch is per program
        dh_ = d // n_head
        self.forward_nodes = [
            (ln, [x, P["ln1_w"], P["ln1_b"], n1]),
            (linear(m, 3 * d, d), [n1, P["attn_w"], P["attn_b"], qkv]),
            (prog(K.attention_desc(batch, seq, n_head, dh_, dt, dropout_p=dropout_p, lse=True, causal=causal)), [qkv, att, lse]),
            (linear(m, d, d, residual=True), [att, P["proj_w"], P["proj_b"], x, x2]),
            (ln, [x2, P["ln2_w"], P["ln2_b"], n2]),
            (linear(m, f, d), [n2, P["fc_w"], P["fc_b"], h]),
            (prog(gelu.desc()), [h, g]),
            (linear(m, d, f, residual=True), [g, P["proj2_w"], P["proj2_b"], x2, out]),
        ]

        def colsum(cols):
            return prog(K.reduce_desc(m, cols, "sum", axis0=True, dtype=dt))

        def dweight(n_out, n_in):   # dW[out, in] = dY[m, out]^T . X[m, in]
            return prog(K.gemm_desc(n_out, n_in, m, dt, dt, trans_a=True))

        def dinput(n_out, n_in):    # dX[m, in] = dY[m, out] . W[out, in]
            return prog(K.gemm_desc(m, n_in, n_out, dt, dt))

        cs_d = colsum(d)
        self.backward_nodes = [
            (cs_d, [dout, G["proj2_b"]]),
            (dweight(d, f), [dout, g, G["proj2_w"]]),
            (dinput(d, f), [dout, P["proj2_w"], dg]),
            (prog(gelu_bwd.desc()), [h, dg, dh]),
            (colsum(f), [dh, G["fc_b"]]),
            (dweight(f, d), [dh, n2, G["fc_w"]]),
            (dinput(f, d), [dh, P["fc_w"], dn2]),
            (ln_bwd, [x2, P["ln2_w"], dn2, dout, dx2, G["ln2_w"], G["ln2_b"]]),
            (cs_d, [dx2, G["proj_b"]]),
            (dweight(d, d), [dx2, att, G["proj_w"]]),
            (dinput(d, d), [dx2, P["proj_w"], datt]),
            (prog(K.attention_bwd_desc(batch, seq, n_head, dh_, dt, dropout_p=dropout_p, causal=causal)), [qkv, att, datt, lse, dqkv]),
            (colsum(3 * d), [dqkv, G["attn_b"]]),
            (dweight(3 * d, d), [dqkv, n1, G["attn_w"]]),
            (dinput(3 * d, d), [dqkv, P["attn_w"], dn1]),
            (ln_bwd2, [x, P["ln1_w"], dn1, dx2, dx, G["ln1_w"], G["ln1_b"]]),
        ]
        self._plan_fwd = dev.create_plan(self.forward_nodes)
        self._plan_all = dev.create_plan(self.forward_nodes + self.backward_nodes)

    # -- host <-> device ------------------------------------------------------------------------
    def write(self, name: str, array):
        a = np.ascontiguousarray(array, self.np_dtype).reshape(self.shapes[name])
        self.pool.sync_events(self._pending)  # the previous launch may still read the buffer
        self._pending = []
        self.pool.sync_events([self.pool.host_to_pool(a, self._bufs[name], [])])

    def set_params(self, params: dict):
        for n in PARAMS:
            self.write(n, params[n])

    def read(self, name: str) -> np.ndarray:
        out = np.empty(self.shapes[name], np.float32 if name == "lse" else self.np_dtype)
        self.pool.pool_to_host(self._bufs[name], out, self._pending)
        self._pending = []
        return out

    def buffer(self, name: str) -> int:
        return self._bufs[name]

    # -- launches ---------------------------------------------------------------------------------
    def forward(self):
        self._pending = [self.dev.launch_plan(self._plan_fwd, self._pending)]

    def forward_backward(self):
        """Forward, then the gradient of sum(out * dout) with respect to x and every parameter: one plan launch."""
        self._pending = [self.dev.launch_plan(self._plan_all, self._pending)]

    def forward_backward_unplanned(self):
        ev = self._pending
        for p, bufs in self.forward_nodes + self.backward_nodes:
            ev = [self.dev.launch(p, self.pool, bufs, ev)]
        self._pending = ev

    def sync(self):
        self.pool.sync_events(self._pending)
        self._pending = []

    def close(self):
        self.sync()
        self.dev.destroy_plan(self._plan_fwd)
        self.dev.destroy_plan(self._plan_all)
        for p in self._progs:
            self.dev.release(p)
        for b in self._bufs.values():
            self.pool.deallocate(b, [])
