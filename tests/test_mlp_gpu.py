"""GPU parity of the MLP train step (the MLP configuration) against the numpy model.

Protocols follow /root/reference/test_autograd.py: loss within 2e-3 and gradients
within 2e-2 relative of an independent float32 model (:78-103), AdamW overfits one
batch (:152-166); plus the loss *curve* of the recorded TrainStep against the
numpy model that rounds where the device rounds.
"""

import numpy as np
import pytest

from oracle import ref_mlp
from tests.mlp_harness import build_pair, run_curve, upload_batch

pytestmark = pytest.mark.gpu


def relerr(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-8))


@pytest.mark.parametrize("fuse", ["separate passes", "epilogues", "epilogues + column sums"])
@pytest.mark.parametrize("act", ["gelu", "relu"])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_loss_and_gradients(dev, act, dtype, fuse):
    """Two hidden layers, so that a dX GEMM with the activation derivative (and the bias
    column sums) of the layer below in its epilogue is on the path when fused."""
    batch, n_in, n_hid, n_cls, pad = 16, 32, 16, 4, 16
    ctx, model, ref = build_pair(dev, batch, (n_in, n_hid, n_hid), n_cls, pad, act, dtype, seed=0,
                                 fuse_bias=fuse != "separate passes", fuse_colsum=fuse.endswith("sums"))
    try:
        xb, yb, xf, y = upload_batch(ctx, batch, n_in, n_cls, 0, dtype)
        loss = model.forward_backward(xb, yb)
        # independent float32 model (no 16-bit rounding): the reference's tolerances
        pure = ref_mlp.RefMLP((n_in, n_hid, n_hid), n_cls, pad, act=act, pure_f32=True)
        pure.set_params(ref.W, ref.b)
        ploss, dW, db = pure.loss_and_grads(xf, y)
        tol_loss, tol_grad = (2e-3, 2e-2) if dtype == "f16" else (2e-2, 6e-2)   # bf16 has 3 fewer mantissa bits
        assert abs(loss - ploss) < tol_loss
        for layer, gw, gb in zip(model.layers, dW, db):
            assert relerr(layer.W.grad_numpy(), gw) < tol_grad
            assert relerr(layer.b.grad_numpy(), gb) < tol_grad
        # the model that rounds where the device rounds agrees far more tightly
        rloss, rW, rb = ref.loss_and_grads(xf, y)
        assert abs(loss - rloss) < 2e-5
        for layer, gw, gb in zip(model.layers, rW, rb):
            assert relerr(layer.W.grad_numpy(), gw) < 2e-3
            assert relerr(layer.b.grad_numpy(), gb) < 2e-3
    finally:
        ctx.destroy()


@pytest.mark.parametrize("fuse_bias", [False, True])
def test_baseline_config_loss_curve(dev, fuse_bias):
    """784 -> 512 -> 512 -> 10, ReLU, batch 128, AdamW lr 1e-3: 100 recorded steps."""
    got, want = run_curve(dev, steps=100, batch=128, sizes=(784, 512, 512), n_classes=10, pad=10,
                          act="relu", dtype="f16", fuse_bias=fuse_bias, recorded=True)
    assert np.isfinite(got).all()
    # Early steps agree to the reference's loss tolerance (test_autograd.py:90).
    # Later the two trajectories separate slowly: Adam's normalised update turns
    # one-ulp differences in a gradient into different 16-bit roundings of the
    # weights, so the bound widens with the step count.
    assert np.abs(got[:5] - want[:5]).max() < 2e-3, f"early drift {np.abs(got[:5] - want[:5]).max()}"
    assert np.abs(got - want).max() < 3e-2, f"max drift {np.abs(got - want).max()}"
    assert got[-1] < 0.5 * got[0], "not learning"


@pytest.mark.parametrize("fuse_bias,fuse_colsum", [(False, False), (True, False), (True, True)])
def test_reference_variant_loss_curve(dev, fuse_bias, fuse_colsum):
    """What examples.mnist --synthetic actually runs (mnist.py:124-128, 146-147):
    784 zero-padded to 1024 -> 256 -> 16 (10 real classes), GELU; with fuse_bias the
    bias, GELU and narrowing happen in the forward GEMM's epilogue and GELU' in the head's
    dX epilogue, with fuse_colsum the hidden layer's bias gradient too."""
    got, want = run_curve(dev, steps=60, batch=128, sizes=(1024, 256), n_classes=10, pad=16,
                          act="gelu", dtype="f16", fuse_bias=fuse_bias, recorded=True, fuse_colsum=fuse_colsum)
    assert np.abs(got[:5] - want[:5]).max() < 2e-3
    assert np.abs(got - want).max() < 3e-2


def test_eager_equals_recorded(dev):
    a, _ = run_curve(dev, steps=8, batch=32, sizes=(64, 48), n_classes=10, pad=10, act="relu", recorded=True)
    b, _ = run_curve(dev, steps=8, batch=32, sizes=(64, 48), n_classes=10, pad=10, act="relu", recorded=False)
    assert np.abs(a - b).max() < 1e-6


def test_adamw_overfits_one_batch(dev):
    got, _ = run_curve(dev, steps=200, batch=32, sizes=(64, 32), n_classes=8, pad=16, act="gelu", lr=3e-3)
    assert got[-1] < 0.2 * got[0]


def test_graph_replay_sees_new_inputs(dev):
    """A recorded step must read the batch the CPU wrote into mapped memory
    after recording (autograd.py:346-366)."""
    from vkgrad_amd.autograd import AdamW, TrainStep
    batch, sizes, n_cls = 32, (64, 48), 10
    ctx, model, ref = build_pair(dev, batch, sizes, n_cls, 10, "relu", "f16")
    try:
        xb, yb, xf, y = upload_batch(ctx, batch, sizes[0], n_cls, 0, "f16")
        opt = AdamW(ctx, model.params(), lr=0.0)       # lr 0: parameters stay put
        step = TrainStep(model, opt, xb, yb)
        l0, _ = step()
        xs2, xf2, y2 = ref_mlp.synthetic_batch(batch, sizes[0], n_cls, seed=5)
        xb.array(np.float16, xs2.shape)[:] = xs2
        yb.array(np.uint32, (batch,))[:] = y2
        l1, _ = step()
        want0, _, _ = ref.loss_and_grads(xf, y)
        want1, _, _ = ref.loss_and_grads(xf2, y2)
        assert abs(l0 - want0) < 2e-5 and abs(l1 - want1) < 2e-5 and abs(l0 - l1) > 1e-4
    finally:
        ctx.destroy()


@pytest.mark.parametrize("dirty", [False, True])
def test_gradient_accumulation_equals_one_large_batch(dev, dirty):
    """GradAccum over N micro-batches of B rows against the device's own batch of N*B rows
    (test_accum.py:1-9, 139-168: relative error below 2e-2, also when the accumulator holds
    stale values before it is zeroed), and one optimiser step from each lands on the same
    weights."""
    from vkgrad_amd.autograd import MLP, AdamW, Ctx
    from vkgrad_amd.dataparallel import GradAccum
    B, N, in_f, hidden, n_cls = 16, 4, 64, 32, 8
    rng = np.random.default_rng(3)
    data = rng.standard_normal((B * N, in_f)).astype(np.float16)
    labels = rng.integers(0, n_cls, B * N).astype(np.uint32)

    def build(batch):
        ctx = Ctx(dev)
        model = MLP(ctx, batch, [in_f, hidden], n_cls, pad_classes=16)
        r = np.random.default_rng(7)                      # identical weights however the batch is split
        for p in model.params():
            p.set(r.standard_normal(p.shape).astype(np.float32) * 0.05)
        xb, yb = ctx.buf(batch * in_f * 2, "shared"), ctx.buf(batch * 4, "shared")
        return ctx, model, xb, yb

    def feed(xb, yb, rows, lo):
        xb.array(np.float16, (rows, in_f))[:] = data[lo:lo + rows]
        yb.array(np.uint32, (rows,))[:] = labels[lo:lo + rows]
        xb.flush()
        yb.flush()

    ctx, model, xb, yb = build(B)
    ctx2, big, xb2, yb2 = build(B * N)
    try:
        params = list(model.params())
        opt = AdamW(ctx, params, lr=1e-3)
        ga = GradAccum(ctx, params, accum=N)
        assert ga.total == sum(p.n for p in params) and ga.offsets[1] == params[0].n
        if dirty:
            ga.arena.upload(np.random.default_rng(11).standard_normal(ga.total).astype(np.float32))
            assert np.abs(ga.arena.download(np.float32, (ga.total,))).max() > 0.5
        g_zero, g_micro, g_apply = dev.graph("zero"), dev.graph("micro"), dev.graph("apply")
        ga.record_zero(g_zero)
        model.record(xb, yb, g_micro)
        ga.record_push(g_micro)
        ga.record_apply(g_apply, opt)
        for g in (g_zero, g_micro, g_apply):
            g.finish()
        g_zero.submit()
        for i in range(N):
            feed(xb, yb, B, i * B)
            g_micro.submit()
        summed = ga.arena.download(np.float32, (ga.total,))
        opt.advance()
        g_apply.submit()

        params2 = list(big.params())
        opt2 = AdamW(ctx2, params2, lr=1e-3)
        feed(xb2, yb2, B * N, 0)
        big.forward_backward(xb2, yb2)
        want = np.concatenate([p.grad_numpy().reshape(-1) for p in params2])
        assert relerr(summed / N, want) < 2e-3            # the reference allows 2e-2 and measures 8.8e-06
        pulled = np.concatenate([p.grad_numpy().reshape(-1) for p in params])
        assert np.allclose(pulled, summed / N, rtol=1e-6, atol=0)
        opt2.step()
        for p, p2 in zip(params, params2):
            assert np.abs(p.numpy() - p2.numpy()).max() < 3e-4, p.name   # |update| is about lr = 1e-3
        for g in (g_zero, g_micro, g_apply):
            g.destroy()
        ga.destroy()
    finally:
        ctx.destroy()
        ctx2.destroy()
