"""Tape autograd call sites of the GEMM path: Ctx, Param, Linear, MLP, AdamW, TrainStep.

Same classes, arguments and tensor semantics as the reference
(/root/reference/autograd.py:22-41 pick_config, 44-108 Ctx, 111-156 Param,
159-228 Linear, 231-301 MLP, 304-343 AdamW, 346-366 TrainStep).  Three GEMMs
per Linear, in the reference's storage convention (W is in_f x out_f):

    forward  acc = x @ W           (F,F)  m=batch, n=out_f, k=in_f
    dW       g32 = x^T @ dz        (T,F)  m=in_f,  n=out_f, k=batch
    dX       dx  = dz @ W^T        (F,T)  m=batch, n=in_f,  k=out_f

Extensions (all off by default keep the reference's exact kernel sequence):
    Ctx(dtype="bf16")        16-bit type of activations and weight mirrors
    Ctx(fuse_bias=True)      bias, activation and 16-bit narrowing in the forward GEMM's epilogue
    MLP(activation="relu")   ReLU instead of GELU in hidden layers
    Linear.backward(accumulate=True)   dW += (beta=1 epilogue), db +=
"""

import os
import zlib

import numpy as np

from .kernels import CONFIGS, Matmul, autotune_matmul, lookup_tuned, make_kernels
from .vk import VkError


def pick_config(m, n, k, trans_a=False, trans_b=False, min_groups=256):
    """Tile chosen without benchmarking (autograd.py:22-41): the largest tile
    area that still gives min_groups workgroups (one per CU of an MI355X).  The
    reference only considers tiles that divide the shape; ragged shapes are
    legal here, so "divides" becomes "wastes under half of the tile grid on
    padding".  Returns the tile id.  The library's own picker (mg_pick) prices
    the same trade-off with K splits as well; this restatement exists for
    callers that used the reference function directly."""
    best = None
    for t in CONFIGS:
        gm, gn = -(-m // t["bm"]), -(-n // t["bn"])
        groups = gm * gn
        useful = (m * n) / (gm * t["bm"] * gn * t["bn"])
        score = (useful >= 0.5, groups >= min_groups, t["bm"] * t["bn"], groups)
        if best is None or score > best[0]:
            best = (score, t["id"])
    if best is None:
        raise VkError(f"no matmul tile fits {m}x{n}x{k}")
    return best[1]


class Ctx:
    """Owns the device, the elementwise kernels and a matmul cache keyed by shape."""

    def __init__(self, dev, tune=False, scalar_only=None, *, dtype="f16", fuse_bias=False, fuse_colsum=False):
        """fuse_bias: bias, activation and narrowing (forward) and the activation derivative
        (backward) run in the GEMM epilogues instead of separate passes.  fuse_colsum (with
        fuse_bias): the bias gradients of the hidden layers are summed in the same backward
        epilogue with float atomics - one pass less, last bits not reproducible."""
        if scalar_only:
            raise VkError("there is no scalar GEMM path on MI355X: MFMA is always present")
        self.dev = dev
        self.dtype = dtype
        self.fuse_bias = fuse_bias
        self.fuse_colsum = bool(fuse_colsum and fuse_bias)
        self.K = make_kernels(dev, dtype)
        self.tune = tune
        self.scalar_only = False
        self._mm = {}
        self._owned = []

    def matmul(self, m, n, k, trans_a=False, trans_b=False, batched=False, nbatch=1):
        key = (m, n, k, trans_a, trans_b, batched, nbatch)
        if key not in self._mm:
            if self.tune:
                mm, _ = autotune_matmul(self.dev, m, n, k, trans_a, trans_b, batched=batched,
                                        nbatch=nbatch, dtype=self.dtype)
            else:
                e = lookup_tuned(self.dev.name, m, n, k, trans_a, trans_b, self.dtype, batched, nbatch)
                if e is not None:
                    mm = Matmul(self.dev, trans_a=trans_a, trans_b=trans_b, batched=batched,
                                tile=e["tile_id"], dtype=self.dtype, split_k=e.get("split_k", 0),
                                group_m=e.get("group_m", 0), atomic_split=e.get("atomic_split", False))
                else:
                    mm = Matmul(self.dev, trans_a=trans_a, trans_b=trans_b, batched=batched,
                                dtype=self.dtype)
            self._mm[key] = mm
        return self._mm[key]

    def buf(self, nbytes, kind="device"):
        b = self.dev.buffer(nbytes, kind)
        self._owned.append(b)
        return b

    def zeros(self, n_floats):
        b = self.buf(n_floats * 4, "device")
        self.K["zero"]([b], n_floats)
        return b

    def destroy(self):
        for m in self._mm.values():
            m.destroy()
        for k in self.K.values():
            k.destroy()
        for b in self._owned:
            b.destroy()
        self._mm.clear()
        self._owned.clear()


class Param:
    """f32 master, 16-bit mirror for the matmul, f32 grad, Adam moments (autograd.py:111-156).

    The reference keeps the master in host-cached mapped memory, which on its APU is the
    same DRAM the GPU uses; on a discrete card the optimiser (and the bias read of a GEMM
    epilogue) would cross PCIe for every element, so the master lives in HBM and numpy() /
    set() copy."""

    def __init__(self, ctx, shape, init=None, name="", no_decay=False):
        self.ctx = ctx
        self.shape = shape
        self.n = int(np.prod(shape))
        self.name = name
        self.no_decay = no_decay
        self.w32 = ctx.buf(self.n * 4, "device")
        self.w16 = ctx.buf(self.n * 2, "device")
        self.g32 = ctx.buf(self.n * 4, "device")
        self.m = ctx.zeros(self.n)
        self.v = ctx.zeros(self.n)
        self.set(np.zeros(shape, np.float32) if init is None else init)

    def sync16(self):
        self.ctx.K["cast16"]([self.w32, self.w16], self.n)

    def numpy(self):
        """A host copy of the master weights."""
        return self.w32.download(np.float32, self.shape)

    def set(self, arr):
        self.w32.upload(np.ascontiguousarray(np.broadcast_to(np.asarray(arr, np.float32), self.shape)))
        self.sync16()

    def grad_numpy(self):
        """Copy the gradient back for checking."""
        return self.g32.download(np.float32, self.shape)


def _seed(name):
    # the reference seeds from hash(name), which Python randomises per process
    # (autograd.py:172); crc32 is stable
    return zlib.crc32(name.encode()) & 0xFFFFFFFF


class Linear:
    """y = act(x @ W + b), or the same without the activation."""

    def __init__(self, ctx, batch, in_f, out_f, activation=True, need_dx=True, name="", act="gelu"):
        self.ctx, self.name = ctx, name
        self.batch, self.in_f, self.out_f = batch, in_f, out_f
        self.activation = activation
        if act not in ("gelu", "relu"):
            raise VkError(f"unknown activation {act!r}")
        self.act = act
        self.need_dx = need_dx
        rng = np.random.default_rng(_seed(name))
        w = (rng.standard_normal((in_f, out_f)) * np.sqrt(2.0 / in_f)).astype(np.float32)
        self.W = Param(ctx, (in_f, out_f), w, name + ".W")
        self.b = Param(ctx, (out_f,), np.zeros(out_f, np.float32), name + ".b", no_decay=True)

        self.acc = ctx.buf(batch * out_f * 4)
        self.z = ctx.buf(batch * out_f * 4)
        self.y16 = ctx.buf(batch * out_f * 2)
        self.dz16 = ctx.buf(batch * out_f * 2)
        self.dz32 = ctx.buf(batch * out_f * 4)
        self.dx32 = ctx.buf(batch * in_f * 4) if need_dx else None
        self.x16 = None
        self._dz_ready = False   # set by the layer above when its dX epilogue wrote dz16 / dz32
        self._db_ready = False   # ... and when it also summed this layer's bias gradient

    def forward(self, x16, tape, graph=None):
        c, K = self.ctx, self.ctx.K
        self.x16 = x16
        n = self.batch * self.out_f
        mm = c.matmul(self.batch, self.out_f, self.in_f)
        if c.fuse_bias:
            # z = x @ W + b straight out of the GEMM epilogue, and with an activation
            # also y16 = narrow(act(z)): no separate pass over the (batch x out_f) tensor
            if self.activation:
                mm(x16, self.W.w16, self.z, self.batch, self.out_f, self.in_f, graph=graph, bias=self.b.w32,
                   act=self.act, y16=self.y16)
                out = self.y16
            else:
                mm(x16, self.W.w16, self.z, self.batch, self.out_f, self.in_f, graph=graph, bias=self.b.w32)
                out = self.z
        else:
            mm(x16, self.W.w16, self.acc, self.batch, self.out_f, self.in_f, graph=graph)
            if self.activation:
                K["bias_" + self.act]([self.acc, self.b.w32, self.z, self.y16], n, self.out_f, graph=graph)
                out = self.y16
            else:
                K["bias"]([self.acc, self.b.w32, self.z], n, self.out_f, graph=graph)
                out = self.z
        tape.append(self.backward)
        return out

    def backward(self, dout16, dout32, graph=None, accumulate=False, below=None):
        """`below`: the Linear whose output this layer consumed.  Under fuse_bias, when
        that layer has an activation, this layer's dX GEMM multiplies by act'(below.z) in
        its epilogue and writes below.dz16 / below.dz32 itself: the separate
        activation-backward pass of the reference (autograd.py:204-207) disappears, and
        (below.dz16, below.dz32) is returned in place of dX."""
        c, K = self.ctx, self.ctx.K
        n = self.batch * self.out_f
        if self.activation and self._dz_ready:
            self._dz_ready = False
            g16, g32 = self.dz16, self.dz32
        elif self.activation:
            K["bias_" + self.act + "_bwd"]([dout32, self.z, self.dz16, self.dz32], n, graph=graph)
            g16, g32 = self.dz16, self.dz32
        else:
            g16, g32 = dout16, dout32

        # dW = X^T @ dZ.  X is stored batch x in_f, which is K x M: trans_a.
        c.matmul(self.in_f, self.out_f, self.batch, trans_a=True)(
            self.x16, g16, self.W.g32, self.in_f, self.out_f, self.batch, graph=graph,
            accumulate=accumulate)
        if self._db_ready:
            self._db_ready = False
        else:
            K["col_sum_acc" if accumulate else "col_sum"]([g32, self.b.g32], self.out_f, self.batch, graph=graph)

        if not self.need_dx:
            return None, None
        # dX = dZ @ W^T.  W is stored in_f x out_f, which is N x K: trans_b.
        mm = c.matmul(self.batch, self.in_f, self.out_f, trans_b=True)
        if (c.fuse_bias and below is not None and below.activation
                and (below.batch, below.out_f) == (self.batch, self.in_f)):
            if c.fuse_colsum:
                # db of the layer below comes out of the same epilogue; dz32 is then not needed
                if not accumulate:
                    K["zero"]([below.b.g32], below.out_f, graph=graph)
                mm(g16, self.W.w16, None, self.batch, self.in_f, self.out_f, graph=graph,
                   act=below.act + "_grad", z=below.z, y16=below.dz16, colsum=below.b.g32)
                below._db_ready = True
            else:
                mm(g16, self.W.w16, below.dz32, self.batch, self.in_f, self.out_f, graph=graph,
                   act=below.act + "_grad", z=below.z, y16=below.dz16)
            below._dz_ready = True
            return below.dz16, below.dz32
        mm(g16, self.W.w16, self.dx32, self.batch, self.in_f, self.out_f, graph=graph)
        return None, self.dx32


class MLP:
    """Hidden layers use the activation; the head is linear and feeds softmax + CE.
    Classes beyond n_classes (padding) are masked inside the softmax kernel.  The
    reference pads the class count to a tile multiple (autograd.py:234-240);
    ragged N is legal here, so pad_classes may equal n_classes."""

    def __init__(self, ctx, batch, sizes, n_classes, pad_classes=16, activation="gelu"):
        if pad_classes < n_classes:
            raise VkError(f"pad_classes {pad_classes} < n_classes {n_classes}")
        self.ctx, self.batch = ctx, batch
        self.n_classes, self.pad = n_classes, pad_classes
        self.layers = []
        for i in range(len(sizes) - 1):
            self.layers.append(Linear(ctx, batch, sizes[i], sizes[i + 1], activation=True,
                                      need_dx=(i > 0), name=f"fc{i}", act=activation))
        self.layers.append(Linear(ctx, batch, sizes[-1], pad_classes, activation=False,
                                  need_dx=True, name="head", act=activation))
        self.dlog16 = ctx.buf(batch * pad_classes * 2)
        self.dlog32 = ctx.buf(batch * pad_classes * 4)
        self.loss = ctx.buf(batch * 4, "cached")
        self._stage = {}   # HBM copies of host-mapped inputs, by buffer

    def params(self):
        for l in self.layers:
            yield l.W
            yield l.b

    def logits(self, x16, tape=None, graph=None):
        h = x16
        for l in self.layers:
            h = l.forward(h, tape if tape is not None else [], graph=graph)
        return h

    def _staged(self, buf, graph):
        """A buffer the CPU writes between replays (host-mapped, vk.py:583-590) is copied
        into HBM by the step's first kernels: the GEMMs that read the batch twice (forward
        and dW of the first layer) then do not fetch it over PCIe."""
        if not buf.host_visible:
            return buf
        dev_copy = self._stage.get(id(buf))
        if dev_copy is None:
            dev_copy = self._stage[id(buf)] = self.ctx.buf((buf.size + 3) // 4 * 4, "device")
        self.ctx.K["copy"]([buf, dev_copy], buf.size // 4 * 4, graph=graph)
        return dev_copy

    def record(self, x16, labels_buf, graph, accumulate=False):
        K = self.ctx.K
        tape = []
        x16, labels_buf = self._staged(x16, graph), self._staged(labels_buf, graph)
        logits = self.logits(x16, tape, graph=graph)
        K["softmax_ce"]([logits, labels_buf, self.dlog16, self.dlog32, self.loss],
                        self.batch, self.pad, self.n_classes, graph=graph)
        g16, g32 = self.dlog16, self.dlog32
        for i in reversed(range(len(tape))):
            g16, g32 = tape[i](g16, g32, graph=graph, accumulate=accumulate,
                               below=self.layers[i - 1] if i > 0 else None)

    def read_loss(self):
        self.loss.invalidate()
        return float(self.loss.array(np.float32, (self.batch,)).mean())

    def forward_backward(self, x16, labels_buf, accumulate=False):
        """Eager: one synchronous launch per kernel."""
        K = self.ctx.K
        tape = []
        logits = self.logits(x16, tape)
        K["softmax_ce"]([logits, labels_buf, self.dlog16, self.dlog32, self.loss],
                        self.batch, self.pad, self.n_classes)
        loss = self.read_loss()
        g16, g32 = self.dlog16, self.dlog32
        for i in reversed(range(len(tape))):
            g16, g32 = tape[i](g16, g32, accumulate=accumulate, below=self.layers[i - 1] if i > 0 else None)
        return loss

    def predict(self, x16):
        logits = self.logits(x16)
        out = logits.download(np.float32, (self.batch, self.pad))[:, :self.n_classes]
        return out.argmax(1).copy()


class AdamW:
    """One fused kernel per parameter (autograd.py:304-343); step-varying
    scalars live in a mapped buffer so a recorded step stays valid."""

    def __init__(self, ctx, params, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, wd=0.01):
        self.ctx, self.params = ctx, list(params)
        self.lr, self.b1, self.b2, self.eps, self.wd = lr, b1, b2, eps, wd
        self.t = 0
        self.hp = ctx.buf(8 * 4, "shared")
        self.hpv = self.hp.array(np.float32)
        # the kernels read the scalars from HBM: one staging copy per step instead of a
        # PCIe read of the mapped buffer from every wavefront of every parameter's kernel
        self.hp_dev = ctx.buf(8 * 4, "device")
        self._set_hp(lr)

    def _set_hp(self, lr):
        bc1 = 1 - self.b1 ** max(self.t, 1)
        bc2 = 1 - self.b2 ** max(self.t, 1)
        self.hpv[:6] = [lr, self.b1, self.b2, bc1, bc2, self.eps]
        self.hp.flush()

    def advance(self, lr=None):
        self.t += 1
        self._set_hp(self.lr if lr is None else lr)

    def record(self, graph):
        k = self.ctx.K["adamw"]
        self.ctx.K["copy"]([self.hp, self.hp_dev], 8 * 4, graph=graph)
        for p in self.params:
            wd = 0.0 if p.no_decay else self.wd
            k([p.w32, p.g32, p.m, p.v, p.w16, self.hp_dev], p.n, wd, graph=graph)

    def step(self, lr=None):
        self.advance(lr)
        k = self.ctx.K["adamw"]
        self.ctx.K["copy"]([self.hp, self.hp_dev], 8 * 4)
        for p in self.params:
            wd = 0.0 if p.no_decay else self.wd
            k([p.w32, p.g32, p.m, p.v, p.w16, self.hp_dev], p.n, wd)


class TrainStep:
    """The whole step recorded once and replayed (autograd.py:346-366)."""

    def __init__(self, model, opt, xbuf, ybuf):
        self.model, self.opt = model, opt
        self.graph = model.ctx.dev.graph("train_step")
        model.record(xbuf, ybuf, self.graph)
        opt.record(self.graph)
        self.graph.finish()
        self.n_dispatch = self.graph.n_dispatch

    def __call__(self, lr=None):
        self.opt.advance(lr)
        dt = self.graph.submit()
        return self.model.read_loss(), dt
