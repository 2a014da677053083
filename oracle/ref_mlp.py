"""numpy model of the MLP train step.  TEST INFRASTRUCTURE ONLY.

Restates, with the same mixed precision as the device path, the reference's
training step for `examples.mnist` (/root/reference/examples/mnist.py:124-177):

  forward    Linear.forward   autograd.py:186-200   acc = x16 @ w16 (f32), z = acc + b,
                                                     y16 = narrow(act(z))        kernels.py:709-718, 742-749
  loss       softmax_ce       kernels.py:766-791     mean over rows; classes >= n_classes masked
  backward   Linear.backward  autograd.py:202-228    g = dout * act'(z), dW = x16^T @ g16, db = colsum(g32),
                                                     dx = g16 @ w16^T              kernels.py:721-729, 753-761
  optimiser  AdamW            autograd.py:304-343 + kernels.py:832-851 (t advanced before the step,
                                                     bias corrections 1 - beta^max(t,1), 16-bit mirror refreshed)

Every tensor the device rounds to 16 bits is rounded here at the same point, and
all arithmetic is float32, so the two loss curves agree to float32 noise rather
than to mixed-precision noise.  `pure_f32=True` drops the roundings and gives
the independent float32 model of test_autograd.py:21-46 instead.

Pinned by tests/test_oracle.py: finite differences of the loss against the
analytic gradients (float64 run of the same code), the closed form of the first
AdamW step (|dw| = lr * (1 + wd*|w|) to first order), and softmax-CE row sums.
"""

import numpy as np

from .ref_gemm import round_to, widen

GELU_C = np.float32(0.7978845608028654)


def gelu(x):
    x = x.astype(np.float32, copy=False) if x.dtype != np.float64 else x
    c = x.dtype.type(0.7978845608028654)
    return x.dtype.type(0.5) * x * (x.dtype.type(1.0) + np.tanh(c * (x + x.dtype.type(0.044715) * x * x * x)))


def dgelu(x):
    c = x.dtype.type(0.7978845608028654)
    t = np.tanh(c * (x + x.dtype.type(0.044715) * x * x * x))
    sech2 = x.dtype.type(1.0) - t * t
    return (x.dtype.type(0.5) * (x.dtype.type(1.0) + t)
            + x.dtype.type(0.5) * x * sech2 * c * (x.dtype.type(1.0) + x.dtype.type(3.0 * 0.044715) * x * x))


def act_fn(x, act):
    return gelu(x) if act == "gelu" else np.maximum(x, x.dtype.type(0))


def dact_fn(x, act):
    return dgelu(x) if act == "gelu" else (x > 0).astype(x.dtype)


class RefMLP:
    """sizes = [in, h1, ..., h_last]; a linear head to `pad_classes` follows."""

    def __init__(self, sizes, n_classes, pad_classes, act="gelu", dtype="f16", pure_f32=False,
                 ftype=np.float32):
        self.sizes = list(sizes) + [pad_classes]
        self.n_classes, self.pad = n_classes, pad_classes
        self.act, self.dtype, self.pure, self.ft = act, dtype, pure_f32, ftype
        self.W = [None] * (len(self.sizes) - 1)
        self.b = [None] * (len(self.sizes) - 1)
        self.t = 0
        self.m = None
        self.v = None

    # -- rounding points ---------------------------------------------------
    def r16(self, x):
        if self.pure:
            return x
        return widen(round_to(x.astype(np.float32), self.dtype), self.dtype).astype(self.ft)

    def set_params(self, Ws, bs):
        self.W = [np.array(w, dtype=self.ft) for w in Ws]
        self.b = [np.array(b, dtype=self.ft) for b in bs]
        self.m = [np.zeros_like(p) for p in self.W + self.b]
        self.v = [np.zeros_like(p) for p in self.W + self.b]
        self.t = 0

    def forward(self, x16):
        """x16: float array holding 16-bit-exact inputs.  Returns logits (B, pad)."""
        h = np.asarray(x16, dtype=self.ft)
        self.xs, self.zs = [], []
        nl = len(self.W)
        for i in range(nl):
            self.xs.append(h)
            z = h @ self.r16(self.W[i]) + self.b[i]
            self.zs.append(z)
            h = self.r16(act_fn(z, self.act)) if i < nl - 1 else z
        return h

    def loss_and_grads(self, x16, y):
        ft = self.ft
        logits = self.forward(x16)
        B = logits.shape[0]
        valid = logits[:, :self.n_classes]
        mx = valid.max(1, keepdims=True)
        s = np.exp(valid - mx).sum(1, keepdims=True)
        logZ = mx + np.log(s)
        rows = (logZ[:, 0] - valid[np.arange(B), y]).astype(ft)
        loss = float(rows.mean())
        dlog = np.zeros_like(logits)
        onehot = np.zeros_like(valid)
        onehot[np.arange(B), y] = 1
        dlog[:, :self.n_classes] = (np.exp(valid - logZ) - onehot) * ft(1.0 / B)
        g32 = dlog
        g16 = self.r16(dlog)
        nl = len(self.W)
        dW, db = [None] * nl, [None] * nl
        for i in reversed(range(nl)):
            if i < nl - 1:
                g32 = g32 * dact_fn(self.zs[i], self.act)
                g16 = self.r16(g32)
            dW[i] = self.xs[i].T @ g16
            db[i] = g32.sum(0)
            if i > 0:
                g32 = g16 @ self.r16(self.W[i]).T
        return loss, dW, db

    def adamw_step(self, dW, db, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, wd=0.01):
        ft = self.ft
        self.t += 1
        bc1 = ft(np.float32(1 - b1 ** max(self.t, 1)))
        bc2 = ft(np.float32(1 - b2 ** max(self.t, 1)))
        lr, b1, b2, eps = ft(np.float32(lr)), ft(np.float32(b1)), ft(np.float32(b2)), ft(np.float32(eps))
        params = self.W + self.b
        grads = dW + db
        nW = len(self.W)
        for i, (p, g) in enumerate(zip(params, grads)):
            decay = ft(np.float32(wd)) if i < nW else ft(0)
            self.m[i] = b1 * self.m[i] + (ft(1) - b1) * g
            self.v[i] = b2 * self.v[i] + (ft(1) - b2) * g * g
            mh = self.m[i] / bc1
            vh = self.v[i] / bc2
            p -= lr * (mh / (np.sqrt(vh) + eps) + decay * p)

    def train_step(self, x16, y, **hp):
        loss, dW, db = self.loss_and_grads(x16, y)
        self.adamw_step(dW, db, **hp)
        return loss


def he_init(sizes_full, seed):
    """He-normal weights (autograd.py:173) from one seeded generator; zero biases."""
    rng = np.random.default_rng(seed)
    Ws, bs = [], []
    for fin, fout in zip(sizes_full[:-1], sizes_full[1:]):
        Ws.append((rng.standard_normal((fin, fout)) * np.sqrt(2.0 / fin)).astype(np.float32))
        bs.append(np.zeros(fout, np.float32))
    return Ws, bs


def synthetic_batch(batch, n_in, n_classes, seed=0, dtype="f16"):
    """Inputs of the MLP configuration: x uniform[0,1) rounded to the 16-bit type,
    integer labels uniform over the classes."""
    rng = np.random.default_rng(seed)
    x = rng.random((batch, n_in), dtype=np.float32)
    y = rng.integers(0, n_classes, batch).astype(np.uint32)
    xs = round_to(x, dtype)
    return xs, widen(xs, dtype), y
