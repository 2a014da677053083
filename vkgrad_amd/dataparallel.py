"""Gradient accumulation over micro-batches on one device: `GradAccum` with the
reference's methods (/root/reference/dataparallel.py:153-207) and its three
single-writer kernels `add`, `zero`, `pull` (dataparallel.py:47-73).

Each micro-batch adds its gradients into one flat f32 accumulator laid out
parameter after parameter; the optimiser then steps once from the scaled sum
(scale 1/accum, so that N micro-batches of B rows equal one batch of N*B,
dataparallel.py:63-68).  The accumulator lives in HBM and the adds are plain
read-modify-writes: one writer, no atomics.

The exchange between several devices through a shared host arena (`HostArena`,
`Replica`, the atomic `push`) is not part of this library: it runs on one GPU.
Where the model is built from `autograd.Linear`, `backward(..., accumulate=True)`
is the cheaper way to the same sum - the dW GEMMs add into the gradient buffers
themselves (beta = 1) and no accumulator pass exists at all.
"""

from .kernels import Elementwise
from .vk import VkError


def make_reduce_kernels(dev):
    """`add`: arena[off + i] += g[i]; `zero`: arena[i] = 0; `pull`: g[i] = arena[off + i] * scale.
    Buffers and arguments as in the reference: add([g, arena], n, off), zero([arena], n),
    pull([arena, g], n, off, scale)."""
    K = {}
    K["add"] = Elementwise(dev, "grad_add", lambda lib, ctx, p, n, off:
                           lib.mg_ew_grad_add(ctx, p[1] + 4 * int(off), p[0], n))
    K["zero"] = Elementwise(dev, "arena_zero", lambda lib, ctx, p, n: lib.mg_ew_zero(ctx, p[0], n))
    K["pull"] = Elementwise(dev, "grad_pull", lambda lib, ctx, p, n, off, scale:
                            lib.mg_ew_scale_copy(ctx, p[1], p[0] + 4 * int(off), n, float(scale)))
    return K


class GradAccum:
    def __init__(self, ctx, params, accum=1):
        if accum < 1:
            raise VkError(f"accum must be >= 1, got {accum}")
        self.ctx, self.params, self.accum = ctx, list(params), accum
        self.K = make_reduce_kernels(ctx.dev)
        self.offsets, total = [], 0
        for p in self.params:
            self.offsets.append(total)
            total += p.n
        self.total = total
        self.arena = ctx.buf(total * 4, "device")

    def record_push(self, graph):
        """Add the gradients of the micro-batch just computed into the accumulator."""
        for p, off in zip(self.params, self.offsets):
            self.K["add"]([p.g32, self.arena], p.n, off, graph=graph)

    def record_zero(self, graph):
        self.K["zero"]([self.arena], self.total, graph=graph)

    def record_apply(self, graph, opt, scale=None):
        """Summed gradients back into every parameter's g32, times `scale` (default
        1 / accum), and one optimiser step from them."""
        factor = (1.0 / self.accum) if scale is None else scale
        for p, off in zip(self.params, self.offsets):
            self.K["pull"]([self.arena, p.g32], p.n, off, factor, graph=graph)
        opt.record(graph)

    def destroy(self):
        for k in self.K.values():
            k.destroy()
