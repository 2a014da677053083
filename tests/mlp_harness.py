"""Drives the device MLP (vkgrad_amd.autograd) and the numpy model side by side."""

import numpy as np

from oracle import ref_mlp


def build_pair(dev, batch, sizes, n_classes, pad, act="gelu", dtype="f16", seed=0, fuse_bias=False,
               bias_std=0.1, fuse_colsum=False):
    from vkgrad_amd.autograd import MLP, Ctx
    ctx = Ctx(dev, dtype=dtype, fuse_bias=fuse_bias, fuse_colsum=fuse_colsum)
    model = MLP(ctx, batch, list(sizes), n_classes, pad_classes=pad, activation=act)
    Ws, bs = ref_mlp.he_init(list(sizes) + [pad], seed)
    rng = np.random.default_rng(seed + 77)
    # non-zero, per-column-distinct biases so a skipped bias add shows
    bs = [(rng.standard_normal(b.shape) * bias_std).astype(np.float32) for b in bs]
    for layer, W, b in zip(model.layers, Ws, bs):
        layer.W.set(W)
        layer.b.set(b)
    ref = ref_mlp.RefMLP(sizes, n_classes, pad, act=act, dtype=dtype)
    ref.set_params(Ws, bs)
    return ctx, model, ref


def upload_batch(ctx, batch, n_in, n_classes, seed, dtype):
    xs, xf, y = ref_mlp.synthetic_batch(batch, n_in, n_classes, seed, dtype)
    xb = ctx.buf(xs.nbytes, "shared")
    xb.array(xs.dtype, xs.shape)[:] = xs
    yb = ctx.buf(batch * 4, "shared")
    yb.array(np.uint32, (batch,))[:] = y
    return xb, yb, xf, y


def run_curve(dev, steps=20, batch=128, sizes=(784, 512, 512), n_classes=10, pad=10, act="relu",
              dtype="f16", fuse_bias=False, recorded=True, lr=1e-3, fuse_colsum=False):
    """Train both models on one fixed synthetic batch; returns (device losses, numpy losses)."""
    from vkgrad_amd.autograd import AdamW, TrainStep
    ctx, model, ref = build_pair(dev, batch, sizes, n_classes, pad, act, dtype, fuse_bias=fuse_bias,
                                 fuse_colsum=fuse_colsum)
    try:
        xb, yb, xf, y = upload_batch(ctx, batch, sizes[0], n_classes, 0, dtype)
        opt = AdamW(ctx, model.params(), lr=lr)
        got, want = [], []
        if recorded:
            step = TrainStep(model, opt, xb, yb)
            for _ in range(steps):
                loss, _ = step()
                got.append(loss)
        else:
            for _ in range(steps):
                got.append(model.forward_backward(xb, yb))
                opt.step()
        for _ in range(steps):
            want.append(ref.train_step(xf, y, lr=lr))
        return np.array(got), np.array(want)
    finally:
        ctx.destroy()


def smoke_train_steps(dev, steps=5):
    got, want = run_curve(dev, steps=steps, batch=32, sizes=(64, 48), n_classes=10, pad=10, act="relu")
    return float(np.abs(got - want).max())
