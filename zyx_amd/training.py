"""The launch list of one training step of the two-layer MLP (Linear -> ReLU -> Linear ->
cross_entropy mean, SGD), as zyx's Tape would hand it to the device once its plan is cached
(zyx/src/tape.rs:141-202 -> zyx/src/graph/plan.rs:271-361): buffers allocated once, then the
same Launch nodes every step. Model and loop follow zyx/tests/mnist.rs:54-66 and the README
training loop (784 -> 128 -> 10, batch 64, lr 0.01); layers are zyx-nn Linear
(zyx-nn/src/linear.rs:24-44, weight stored [out, in]), the update is zyx-optim SGD without
momentum (zyx-optim/src/sgd.rs:45-84).

Per step the device runs 15 kernels:
  forward   h = relu(x . W1^T + b1)                     GEMM, bias+ReLU epilogue
            logits = h . W2^T + b2                       GEMM, bias epilogue
  loss      per-sample cross entropy + dlogits           fused row kernel
            mean loss                                    row reduce + scale
  backward  dW2 = dlogits^T . h, db2 = colsum(dlogits)   GEMM (A transposed), column reduce
            dh = dlogits . W2                            GEMM
            dpre = (h > 0) * dh                          elementwise chain
            dW1 = dpre^T . x, db1 = colsum(dpre)         GEMM (A transposed), column reduce
  update    p <- p - g * lr for W1, b1, W2, b2           4 elementwise chains
"""
from __future__ import annotations

import numpy as np

from . import kernels as K
from .backend import DType, HIPDevice, HIPMemoryPool


class MLPTrainStep:
    def __init__(self, dev: HIPDevice, pool: HIPMemoryPool, batch: int, n_in: int, hidden: int, n_out: int, lr: float,
                 fused_update: bool = False):
        """fused_update: the weight-gradient GEMMs write `w - lr * dW` directly (alpha = -lr, the old weight as the
        fused residual operand), so dW1 / dW2 are never materialised and two update launches disappear."""
        self.dev, self.pool = dev, pool
        self.shape = (batch, n_in, hidden, n_out)
        f32 = DType.F32
        self._bufs, self._progs = {}, []

        def buf(name, elems, itemsize=4):
            b, ev = pool.allocate((elems + 1) * itemsize)  # + one trash element, as zyx's Allocate node does
            pool.sync_events([ev])
            self._bufs[name] = b
            return b

        def prog(desc):
            p = dev.register_kernel(desc)
            self._progs.append(p)
            return p

        x, y = buf("x", batch * n_in), buf("labels", batch)
        x2, y2 = buf("x2", batch * n_in), buf("labels2", batch)  # the batch of the other plan (see below)
        w1, b1, w2, b2 = buf("w1", hidden * n_in), buf("b1", hidden), buf("w2", n_out * hidden), buf("b2", n_out)
        h, logits = buf("h", batch * hidden), buf("logits", batch * n_out)
        loss, mean_loss, dlogits = buf("loss", batch), buf("mean_loss", 1), buf("dlogits", batch * n_out)
        dw2, db2, dh, dpre = buf("dw2", n_out * hidden), buf("db2", n_out), buf("dh", batch * hidden), buf("dpre", batch * hidden)
        dw1, db1, loss_sum = buf("dw1", hidden * n_in), buf("db1", hidden), buf("loss_sum", 1)
        nw1, nb1, nw2, nb2 = buf("nw1", hidden * n_in), buf("nb1", hidden), buf("nw2", n_out * hidden), buf("nb2", n_out)

        relu_bwd = K.Chain(batch, hidden)
        ih, idh = relu_bwd.input(), relu_bwd.input()
        relu_bwd.load(ih).cmpgt(relu_bwd.const(0.0)).mul(idh)
        scale = K.Chain(1, 1)
        scale.load(scale.input()).div(scale.const(float(batch)))

        def sgd(rows, cols):
            c = K.Chain(rows, cols)
            ip, ig = c.input(), c.input()
            c.load(ig).mul(c.const(lr)).rsub(ip)
            return prog(c.desc())

        if fused_update:
            dw2_node = (prog(K.gemm_desc(n_out, hidden, batch, f32, f32, trans_a=True, alpha=-lr, residual=True)), [dlogits, h, w2, nw2])
            dw1_node = (prog(K.gemm_desc(hidden, n_in, batch, f32, f32, trans_a=True, alpha=-lr, residual=True)), [dpre, x, w1, nw1])
        else:
            dw2_node = (prog(K.gemm_desc(n_out, hidden, batch, f32, f32, trans_a=True)), [dlogits, h, dw2])
            dw1_node = (prog(K.gemm_desc(hidden, n_in, batch, f32, f32, trans_a=True)), [dpre, x, dw1])
        nodes = [
            (prog(K.gemm_desc(batch, hidden, n_in, f32, f32, trans_b=True, epilogue="bias_relu")), [x, w1, b1, h]),
            (prog(K.gemm_desc(batch, n_out, hidden, f32, f32, trans_b=True, epilogue="bias")), [h, w2, b2, logits]),
        ] + ([(prog(K.cross_entropy_desc(batch, n_out, True, True, 1.0 / batch, mean=True)), [logits, y, loss, dlogits, mean_loss])]
             if fused_update and batch <= 4096 else
             [(prog(K.cross_entropy_desc(batch, n_out, True, True, 1.0 / batch)), [logits, y, loss, dlogits]),
              (prog(K.reduce_desc(1, batch, "sum")), [loss, loss_sum]), (prog(scale.desc()), [loss_sum, mean_loss])]) + [
            dw2_node,
            # bias gradients are column sums; the fused form stores b - lr * sum straight into the new bias
            (prog(K.reduce_desc(batch, n_out, "sum", axis0=True, mul=-lr, base=True)), [dlogits, b2, nb2]) if fused_update else
            (prog(K.reduce_desc(batch, n_out, "sum", axis0=True)), [dlogits, db2]),
        ] + ([(prog(K.gemm_desc(batch, hidden, n_out, f32, f32, residual="relu_mask")), [dlogits, w2, h, dpre])] if fused_update else
             [(prog(K.gemm_desc(batch, hidden, n_out, f32, f32)), [dlogits, w2, dh]), (prog(relu_bwd.desc()), [h, dh, dpre])]) + [
            dw1_node,
            (prog(K.reduce_desc(batch, hidden, "sum", axis0=True, mul=-lr, base=True)), [dpre, b1, nb1]) if fused_update else
            (prog(K.reduce_desc(batch, hidden, "sum", axis0=True)), [dpre, db1]),
        ] + ([] if fused_update else [(sgd(hidden, n_in), [w1, dw1, nw1]), (sgd(n_out, hidden), [w2, dw2, nw2]),
                                      (sgd(1, hidden), [b1, db1, nb1]), (sgd(1, n_out), [b2, db2, nb2])])
        # the updated parameters are written to fresh buffers (a kernel's outputs never alias its
        # inputs); the two parameter sets swap roles every step, so two plans alternate. Each plan also reads its
        # own batch buffers: the next batch is copied in while the current step still runs.
        swap = {w1: nw1, b1: nb1, w2: nw2, b2: nb2, nw1: w1, nb1: b1, nw2: w2, nb2: b2, x: x2, y: y2}
        nodes_b = [(p, [swap.get(b, b) for b in bufs]) for p, bufs in nodes]
        self.nodes = nodes
        self._plans = [dev.create_plan(nodes), dev.create_plan(nodes_b)]
        self._param_sets = [dict(w1=w1, b1=b1, w2=w2, b2=b2), dict(w1=nw1, b1=nb1, w2=nw2, b2=nb2)]
        self._batch_bufs = [(x, y), (x2, y2)]
        self._cur = 0
        self._plan_ev = [None, None]  # event of the last launch of each plan, until something waits for it
        self._copy_ev = []            # uploads of the batch the next step reads
        self._batch_no = 0            # batches set so far, and which of them each pair of batch buffers holds
        self._holds = [0, 0]
        self._host = [None, None]     # host arrays of the batch last uploaded into each pair of batch buffers

    @property
    def _pending(self):
        """Every event the host has to wait for before it touches a buffer of the step."""
        return self._copy_ev + [e for e in self._plan_ev if e is not None]

    @_pending.setter
    def _pending(self, events):
        assert not events, "outstanding events are tracked per plan; only clearing is supported"
        self._copy_ev, self._plan_ev = [], [None, None]

    def _take_plan_event(self, parity: int):
        ev, self._plan_ev[parity] = self._plan_ev[parity], None
        return [ev] if ev is not None else []

    # -- host <-> device ------------------------------------------------------------------------
    def set_params(self, w1, b1, w2, b2):
        self._cur = 0
        evs = [self.pool.host_to_pool(np.ascontiguousarray(a, np.float32), self._param_sets[0][n], [])
               for n, a in (("w1", w1), ("b1", b1), ("w2", w2), ("b2", b2))]
        self.pool.sync_events(evs)

    def set_batch(self, x, labels):
        """Uploads into this step's pair of batch buffers once the step before the previous one, which read them, is
        done. That step also waited for its own uploads, so the host arrays they came from are free to drop here and
        not before: a source of host_to_pool must outlive the copy."""
        xb, yb = self._batch_bufs[self._cur]
        if self._copy_ev:  # a batch that no step consumed
            self.pool.sync_events(self._copy_ev)
        self.pool.sync_events(self._take_plan_event(self._cur))
        self._host[self._cur] = (np.ascontiguousarray(x, np.float32), np.ascontiguousarray(labels, np.int32))
        e1 = self.pool.host_to_pool(self._host[self._cur][0], xb, [])
        e2 = self.pool.host_to_pool(self._host[self._cur][1], yb, [])
        self._copy_ev = [e1, e2]
        self._batch_no += 1
        self._holds[self._cur] = self._batch_no

    def set_batch_from_device(self, x_buf: int, y_buf: int, index: int):
        """Batch `index` of a dataset already resident in the pool (x_buf f32 [n, batch, n_in], y_buf i32
        [n, batch]): two device-to-device range copies, as Tensor::index_select feeds batches in
        zyx-examples/examples/mnist.rs:62-64."""
        b, n_in, _, _ = self.shape
        xb, yb = self._batch_bufs[self._cur]
        if self._copy_ev:
            self.pool.sync_events(self._copy_ev)
        e1 = self.pool.copy_range(x_buf, index * b * n_in * 4, xb, 0, b * n_in * 4, self._take_plan_event(self._cur))
        e2 = self.pool.copy_range(y_buf, index * b * 4, yb, 0, b * 4, [])
        self._copy_ev = [e1, e2]
        self._batch_no += 1
        self._holds[self._cur] = self._batch_no

    def _same_batch_again(self):
        """A step without a new batch reads the last one: it is copied over from the other plan's buffers."""
        if self._holds[self._cur] == self._batch_no:
            return
        b, n_in, _, _ = self.shape
        (sx, sy), (dx, dy) = self._batch_bufs[self._cur ^ 1], self._batch_bufs[self._cur]
        e1 = self.pool.copy_range(sx, 0, dx, 0, b * n_in * 4, self._copy_ev + self._take_plan_event(self._cur))
        e2 = self.pool.copy_range(sy, 0, dy, 0, b * 4, [])  # the pool's copies run in order
        self._copy_ev = [e1, e2]
        self._holds[self._cur] = self._batch_no

    def step(self):
        """One forward + backward + update: a single plan launch."""
        self._same_batch_again()
        old = self._take_plan_event(self._cur)  # only there when the batch buffers were not written since
        ev = self.dev.launch_plan(self._plans[self._cur], self._copy_ev + old)
        self._copy_ev = []
        self._plan_ev[self._cur] = ev
        self._cur ^= 1

    def step_unplanned(self):
        """The same list issued node by node through HIPDevice::launch (no cached plan)."""
        self._same_batch_again()
        nodes = self.nodes if self._cur == 0 else None
        if nodes is None:
            cur, oth = self._param_sets[1], self._param_sets[0]
            swap = {**{oth[k]: cur[k] for k in cur}, **{cur[k]: oth[k] for k in cur}}
            swap.update(zip(self._batch_bufs[0], self._batch_bufs[1]))
            nodes = [(p, [swap.get(b, b) for b in bufs]) for p, bufs in self.nodes]
        ev = self._pending  # launch by launch: simply after everything outstanding
        self._pending = []
        for p, bufs in nodes:
            ev = [self.dev.launch(p, self.pool, bufs, ev)]
        self._plan_ev[self._cur] = ev[0]
        self._cur ^= 1

    def read(self, name: str, shape) -> np.ndarray:
        params = self._param_sets[self._cur]
        out = np.empty(shape, np.int32 if name == "labels" else np.float32)
        last = self._batch_bufs[self._cur ^ 1]  # the batch the most recent step read
        src = params.get(name, {"x": last[0], "labels": last[1]}.get(name, self._bufs.get(name)))
        self.pool.pool_to_host(src, out, self._pending)
        self._pending = []
        return out

    def mean_loss(self) -> float:
        return float(self.read("mean_loss", (1,))[0])

    def close(self):
        self.pool.sync_events(self._pending)
        self._pending = []
        for pl in self._plans:
            self.dev.destroy_plan(pl)
        for p in self._progs:
            self.dev.release(p)
        for b in self._bufs.values():
            self.pool.deallocate(b, [])
