"""Config 1: two-layer MLP 784 -> 128 -> 10 (ReLU, f32, bias), SGD lr 0.01, batch 64 of seeded
N(0,1) inputs with uniform labels, 100 steps -- the GPU launch list against the CPU oracle on
identical data. Tolerance: the loss curve and the final parameters to 1e-4 relative (f32 sums in
different orders, compounded over 100 dependent steps; a single step agrees to 1e-5)."""
import numpy as np
import pytest

from zyx_amd.training import MLPTrainStep

pytestmark = pytest.mark.gpu

B, NIN, H, NOUT, LR = 64, 784, 128, 10, 0.01


def init(oracle, seed=42069):
    r = oracle.Rng(seed)
    k1, k2 = 1.0 / np.sqrt(NIN), 1.0 / np.sqrt(H)  # zyx-nn/src/linear.rs:24-33
    return r, r.uniform((H, NIN), -k1, k1), r.uniform(H, -k1, k1), r.uniform((NOUT, H), -k2, k2), r.uniform(NOUT, -k2, k2)


def test_single_step_gradients_and_update(hip, oracle):
    dev, pool = hip
    r, w1, b1, w2, b2 = init(oracle)
    x, lab = r.randn((B, NIN)), r.randint(B, 0, NOUT)
    loss, nw1, nb1, nw2, nb2, g = oracle.mlp_step(x, lab, w1, b1, w2, b2, LR)
    m = MLPTrainStep(dev, pool, B, NIN, H, NOUT, LR)
    m.set_params(w1, b1, w2, b2)
    m.set_batch(x, lab)
    m.step()
    assert abs(m.mean_loss() - loss) <= 1e-5 * abs(loss)
    for name, shape, want in (("dw1", (H, NIN), g["w1"]), ("db1", (H,), g["b1"]), ("dw2", (NOUT, H), g["w2"]),
                              ("db2", (NOUT,), g["b2"]), ("dlogits", (B, NOUT), g["logits"])):
        got = m.read(name, shape)
        scale = np.abs(want).max()
        assert np.all(np.abs(got - want) <= 1e-5 * scale + 1e-9), (name, np.abs(got - want).max() / scale)
    for name, shape, want in (("w1", (H, NIN), nw1), ("b1", (H,), nb1), ("w2", (NOUT, H), nw2), ("b2", (NOUT,), nb2)):
        np.testing.assert_allclose(m.read(name, shape), want, rtol=1e-6, atol=1e-8)
    m.close()


@pytest.mark.parametrize("fused_update", [False, True])
def test_100_steps_loss_curve(hip, oracle, fused_update):
    """fused_update: w - lr * dW is formed in the weight-gradient GEMM's epilogue instead of a separate launch."""
    dev, pool = hip
    r, w1, b1, w2, b2 = init(oracle)
    m = MLPTrainStep(dev, pool, B, NIN, H, NOUT, LR, fused_update=fused_update)
    m.set_params(w1, b1, w2, b2)
    gpu_losses, cpu_losses = [], []
    for step in range(100):
        x, lab = r.randn((B, NIN)), r.randint(B, 0, NOUT)
        loss, w1, b1, w2, b2, _ = oracle.mlp_step(x, lab, w1, b1, w2, b2, LR)
        cpu_losses.append(loss)
        m.set_batch(x, lab)
        if step % 2:
            m.step()
        else:
            m.step_unplanned()  # the same nodes through plain launches must give the same result
        gpu_losses.append(m.mean_loss())
    np.testing.assert_allclose(gpu_losses, cpu_losses, rtol=1e-4)
    np.testing.assert_allclose(m.read("w1", (H, NIN)), w1, rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(m.read("w2", (NOUT, H)), w2, rtol=1e-4, atol=1e-6)
    assert 2.0 < gpu_losses[0] < 2.8  # ~ln(10) at initialisation
    m.close()


def test_plan_replays_are_stable(hip, oracle):
    """A cached plan replayed many times with host work in between keeps giving the eager result."""
    dev, pool = hip
    r, w1, b1, w2, b2 = init(oracle, 7)
    x, lab = r.randn((B, NIN)), r.randint(B, 0, NOUT)
    a, b = MLPTrainStep(dev, pool, B, NIN, H, NOUT, LR), MLPTrainStep(dev, pool, B, NIN, H, NOUT, LR)
    a.set_params(w1, b1, w2, b2)
    b.set_params(w1, b1, w2, b2)
    for _ in range(12):
        a.set_batch(x, lab)
        b.set_batch(x, lab)
        a.step()
        b.step_unplanned()
        assert a.mean_loss() == b.mean_loss()
        assert np.array_equal(a.read("w1", (H, NIN)), b.read("w1", (H, NIN)))
    a.close()
    b.close()
