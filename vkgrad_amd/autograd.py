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

import ctypes as C
import os
import zlib

import numpy as np

from . import _lib as L
from .kernels import CONFIGS, Elementwise, Matmul, autotune_matmul, lookup_tuned, make_kernels
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
        if t["name"].startswith(("mv_", "ms_")):
            continue   # the skinny-M streams serve one layout and few rows; the library's picker knows when
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
                                group_m=e.get("group_m", 0), atomic_split=e.get("atomic_split", False),
                                xcd_rotate=e.get("xcd_rotate"))
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
    """One dense layer, y = act(x @ W + b) or, with activation=False, z = x @ W + b.

    Buffers: `z` pre-activation (f32), `y16` activated output in the GEMM operand type,
    `dz16` / `dz32` gradient w.r.t. z in both precisions, `dx32` gradient w.r.t. the input.
    Two schedules (`ctx.fuse_bias`): separate passes as the reference issues them
    (autograd.py:186-228), or the same arithmetic inside GEMM epilogues."""

    ACTS = ("gelu", "relu")

    def __init__(self, ctx, batch, in_f, out_f, activation=True, need_dx=True, name="", act="gelu"):
        if act not in self.ACTS:
            raise VkError(f"unknown activation {act!r}")
        self.ctx, self.name, self.act = ctx, name, act
        self.batch, self.in_f, self.out_f = batch, in_f, out_f
        self.activation, self.need_dx = activation, need_dx
        he = np.random.default_rng(_seed(name)).standard_normal((in_f, out_f)) * np.sqrt(2.0 / in_f)
        self.W = Param(ctx, (in_f, out_f), he.astype(np.float32), name + ".W")
        self.b = Param(ctx, (out_f,), np.zeros(out_f, np.float32), name + ".b", no_decay=True)
        out_elems = batch * out_f
        self.acc, self.z, self.dz32 = (ctx.buf(out_elems * 4) for _ in range(3))
        self.y16, self.dz16 = ctx.buf(out_elems * 2), ctx.buf(out_elems * 2)
        self.dx32 = ctx.buf(batch * in_f * 4) if need_dx else None
        self.x16 = None
        # set by the layer above when its dX epilogue already produced this layer's dz (and db)
        self._dz_ready = self._db_ready = False

    # -- forward -------------------------------------------------------------------------
    def forward(self, x16, tape, graph=None):
        self.x16 = x16
        ctx, B, N, K = self.ctx, self.batch, self.out_f, self.in_f
        gemm = ctx.matmul(B, N, K)
        if ctx.fuse_bias:
            # bias (and activation + narrowing) leave the GEMM's epilogue: no pass over (B, N) after it
            extra = dict(act=self.act, y16=self.y16) if self.activation else {}
            gemm(x16, self.W.w16, self.z, B, N, K, graph=graph, bias=self.b.w32, **extra)
        else:
            gemm(x16, self.W.w16, self.acc, B, N, K, graph=graph)
            if self.activation:
                ctx.K["bias_" + self.act]([self.acc, self.b.w32, self.z, self.y16], B * N, N, graph=graph)
            else:
                ctx.K["bias"]([self.acc, self.b.w32, self.z], B * N, N, graph=graph)
        tape.append(self.backward)
        return self.y16 if self.activation else self.z

    # -- backward ------------------------------------------------------------------------
    def _grad_wrt_z(self, dout16, dout32, graph):
        """(16-bit, f32) gradient w.r.t. this layer's pre-activation."""
        if not self.activation:
            return dout16, dout32
        if self._dz_ready:
            self._dz_ready = False
        else:
            self.ctx.K["bias_" + self.act + "_bwd"]([dout32, self.z, self.dz16, self.dz32], self.batch * self.out_f,
                                                    graph=graph)
        return self.dz16, self.dz32

    def backward(self, dout16, dout32, graph=None, accumulate=False, below=None):
        """dout16 / dout32: dLoss/dOutput in both precisions (16-bit for the GEMMs, f32 for the
        activation derivative and the bias sum).  Returns (g16, g32) for the layer below.

        `below`: the Linear whose output this layer consumed.  Under fuse_bias, when it has an
        activation, this layer's dX GEMM multiplies by act'(below.z) in its epilogue and writes
        below.dz16 / below.dz32 itself (with fuse_colsum also below's bias gradient), so the
        separate activation-backward pass of the reference (autograd.py:204-207) disappears;
        (below.dz16, below.dz32) is then returned in place of (None, dx32)."""
        ctx, B, N, K = self.ctx, self.batch, self.out_f, self.in_f
        g16, g32 = self._grad_wrt_z(dout16, dout32, graph)
        # dW = x^T g : x is stored (B, K), i.e. (contraction, M) -> trans_a
        ctx.matmul(K, N, B, trans_a=True)(self.x16, g16, self.W.g32, K, N, B, graph=graph, accumulate=accumulate)
        if self._db_ready:
            self._db_ready = False
        else:
            ctx.K["col_sum_acc" if accumulate else "col_sum"]([g32, self.b.g32], N, B, graph=graph)
        if not self.need_dx:
            return None, None
        # dX = g W^T : W is stored (K, N), i.e. (N_out, contraction) -> trans_b
        dx_gemm = ctx.matmul(B, K, N, trans_b=True)
        fuse_down = (ctx.fuse_bias and below is not None and below.activation
                     and (below.batch, below.out_f) == (B, K))
        if not fuse_down:
            dx_gemm(g16, self.W.w16, self.dx32, B, K, N, graph=graph)
            return None, self.dx32
        epilogue = dict(act=below.act + "_grad", z=below.z, y16=below.dz16)
        if ctx.fuse_colsum:
            # below's bias gradient comes out of the same epilogue; its f32 dz is then not needed
            if not accumulate:
                ctx.K["zero"]([below.b.g32], below.out_f, graph=graph)
            dx_gemm(g16, self.W.w16, None, B, K, N, graph=graph, colsum=below.b.g32, **epilogue)
            below._db_ready = True
        else:
            dx_gemm(g16, self.W.w16, below.dz32, B, K, N, graph=graph, **epilogue)
        below._dz_ready = True
        return below.dz16, below.dz32


class MLP:
    """Hidden layers with an activation, a linear head, softmax cross-entropy.  Classes
    beyond n_classes are padding and masked inside the loss kernel.  The reference pads the
    class count to a tile multiple (autograd.py:234-240); ragged N is legal here, so
    pad_classes may equal n_classes."""

    def __init__(self, ctx, batch, sizes, n_classes, pad_classes=16, activation="gelu"):
        if pad_classes < n_classes:
            raise VkError(f"pad_classes {pad_classes} < n_classes {n_classes}")
        self.ctx, self.batch = ctx, batch
        self.n_classes, self.pad = n_classes, pad_classes
        widths = list(sizes) + [pad_classes]
        last = len(widths) - 2
        # hidden layers fc0, fc1, ... then the linear head; the first layer's input needs no gradient
        self.layers = [Linear(ctx, batch, widths[i], widths[i + 1], activation=i < last, need_dx=i > 0 or i == last,
                              name="head" if i == last else f"fc{i}", act=activation)
                       for i in range(last + 1)]
        self.dlog16 = ctx.buf(batch * pad_classes * 2)
        self.dlog32 = ctx.buf(batch * pad_classes * 4)
        self.loss = ctx.buf(batch * 4, "cached")
        self._stage = {}   # HBM copies of host-mapped inputs, by buffer

    def params(self):
        for layer in self.layers:
            yield from (layer.W, layer.b)

    def logits(self, x16, tape=None, graph=None):
        tape = [] if tape is None else tape
        out = x16
        for layer in self.layers:
            out = layer.forward(out, tape, graph=graph)
        return out

    def _staged(self, buf, graph):
        """A buffer the CPU writes between replays (host-mapped, vk.py:583-590) is copied
        into HBM by the step's first kernels: the GEMMs that read the batch twice (forward
        and dW of the first layer) then do not fetch it over PCIe."""
        if not buf.host_visible:
            return buf
        if id(buf) not in self._stage:
            self._stage[id(buf)] = self.ctx.buf((buf.size + 3) // 4 * 4, "device")
        self.ctx.K["copy"]([buf, self._stage[id(buf)]], buf.size // 4 * 4, graph=graph)
        return self._stage[id(buf)]

    def _loss_and_backward(self, x16, labels_buf, graph, accumulate, after_loss=None):
        tape = []
        logits = self.logits(x16, tape, graph=graph)
        self.ctx.K["softmax_ce"]([logits, labels_buf, self.dlog16, self.dlog32, self.loss],
                                 self.batch, self.pad, self.n_classes, graph=graph)
        result = after_loss() if after_loss is not None else None
        grads = (self.dlog16, self.dlog32)
        for depth in range(len(tape) - 1, -1, -1):
            grads = tape[depth](*grads, graph=graph, accumulate=accumulate,
                                below=self.layers[depth - 1] if depth else None)
        return result

    def record(self, x16, labels_buf, graph, accumulate=False):
        self._loss_and_backward(self._staged(x16, graph), self._staged(labels_buf, graph), graph, accumulate)

    def read_loss(self):
        self.loss.invalidate()
        return float(self.loss.array(np.float32, (self.batch,)).mean())

    def forward_backward(self, x16, labels_buf, accumulate=False):
        """Eager: one synchronous launch per kernel; returns the loss."""
        return self._loss_and_backward(x16, labels_buf, None, accumulate, after_loss=self.read_loss)

    def predict(self, x16):
        scores = self.logits(x16).download(np.float32, (self.batch, self.pad))
        return scores[:, :self.n_classes].argmax(1).copy()


class AdamW:
    """Decoupled-weight-decay Adam, one fused kernel per parameter (autograd.py:304-343).
    The scalars that change from step to step (learning rate, bias corrections) sit in a
    mapped buffer the CPU rewrites, so a recorded step stays valid; the kernels read an HBM
    copy of it made by the step's first launch instead of reaching over PCIe from every
    wavefront."""

    def __init__(self, ctx, params, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, wd=0.01):
        self.ctx, self.params = ctx, list(params)
        self.lr, self.b1, self.b2, self.eps, self.wd = lr, b1, b2, eps, wd
        self.t = 0
        self.hp = ctx.buf(8 * 4, "shared")
        self.hpv = self.hp.array(np.float32)
        self.hp_dev = ctx.buf(8 * 4, "device")
        self._table_dev, self._blocks = None, 0
        self._set_hp(lr)

    def _set_hp(self, lr):
        t = max(self.t, 1)
        self.hpv[:6] = [lr, self.b1, self.b2, 1 - self.b1 ** t, 1 - self.b2 ** t, self.eps]
        self.hp.flush()

    def advance(self, lr=None):
        """Count a step and publish its scalars (call before replaying a recorded step)."""
        self.t += 1
        self._set_hp(self.lr if lr is None else lr)

    def _table(self):
        """Device table of (w, g, m, v, w16, n, first workgroup, weight decay) per parameter for
        the one-launch update; a workgroup covers 1024 elements."""
        if self._table_dev is None:
            entries = (L.AdamWEntry * len(self.params))()
            blocks = 0
            for e, p in zip(entries, self.params):
                e.w, e.g, e.m, e.v, e.w16 = p.w32.ptr, p.g32.ptr, p.m.ptr, p.v.ptr, p.w16.ptr
                e.n, e.first_block, e.wd = p.n, blocks, 0.0 if p.no_decay else self.wd
                e.vec = int(all(ptr % 16 == 0 for ptr in (e.w, e.g, e.m, e.v)) and e.w16 % 8 == 0)
                blocks += -(-p.n // 1024)
            self._table_dev = self.ctx.buf(C.sizeof(entries), "device")
            self._table_dev.upload(np.frombuffer(entries, dtype=np.uint8))
            self._blocks = blocks
        return self._table_dev

    def record(self, graph):
        """Stage the step's scalars into HBM, then update every parameter in one launch (the
        reference launches the kernel once per parameter, autograd.py:331-343)."""
        ctx = self.ctx
        ctx.K["copy"]([self.hp, self.hp_dev], 8 * 4, graph=graph)
        table, lib, dt = self._table(), ctx.dev._lib, L.DTYPES[ctx.dtype]
        n, blocks = len(self.params), self._blocks

        def launch(lib, mg, ptrs, _n):
            return lib.mg_ew_adamw_multi(mg, ptrs[0], n, blocks, ptrs[1], dt)

        Elementwise(ctx.dev, "adamw_multi", launch)([table, self.hp_dev], n, graph=graph)

    def step(self, lr=None):
        self.advance(lr)
        self.record(None)


class TrainStep:
    """Forward, loss, backward and optimiser recorded once, replayed per step
    (autograd.py:346-366); call it after writing the batch into the mapped input buffers."""

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
