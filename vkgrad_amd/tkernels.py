"""Transformer row kernels by the reference's names and call shapes
(/root/reference/tkernels.py:16-389): `TK[name](buffers, n, *args, graph=None)`.

Row kernels keep the reference's dispatch convention `n = rows *
dev.row_subgroup_size` (tkernels.py:96-104; transformer.py:57-59): one wavefront
of the device's width (64 lanes here) works on a row.  The two column-sum
entries keep their (NCHUNK * ncol, ncol, nrow, nchunk) arguments; the chunking
itself is the library's business and `nchunk` is ignored.
"""

import time

from . import _lib as L
from .kernels import _check
from .vk import VkError


class RowKernel:
    """One kernel; buffers may contain None where the C entry point takes an
    optional pointer."""

    def __init__(self, dev, name, launch):
        self.dev, self.name, self._launch = dev, name, launch

    def __call__(self, buffers, n, *args, repeat=1, graph=None):
        lib, ctx = self.dev._lib, self.dev._ctx
        if any(b is not None and b.ptr is None for b in buffers):
            raise VkError(f"{self.name}: a buffer was destroyed")
        ptrs = [None if b is None else b.ptr for b in buffers]

        def launch():
            _check(self._launch(lib, ctx, ptrs, int(n), *args), self.name)

        if graph is not None:
            graph.record(launch, [b for b in buffers if b is not None], name=self.name)
            return 0.0
        t0 = time.perf_counter()
        for _ in range(repeat):
            launch()
        _check(lib.mg_sync(ctx), self.name)
        return time.perf_counter() - t0

    def destroy(self):
        pass


def make_transformer_kernels(dev, dtype="f16"):
    dt = L.DTYPES[dtype]
    W = dev.row_subgroup_size
    K = {}

    def add(name, fn):
        K[name] = RowKernel(dev, name, fn)

    def rows_of(n):
        if n % W:
            raise VkError(f"row kernels are dispatched with n = rows * {W} (dev.row_subgroup_size); got {n}")
        return n // W

    # buffers: x, gamma, beta, y16, mu, rstd ; n = rows * W ; args: D
    add("layernorm", lambda lib, ctx, p, n, D:
        lib.mg_tk_layernorm(ctx, p[0], p[1], p[2], p[3], p[4], p[5], rows_of(n), int(D), dt))
    # buffers: dy, x, gamma, mu, rstd, dx, dyxh16, dy16
    add("layernorm_bwd", lambda lib, ctx, p, n, D:
        lib.mg_tk_layernorm_bwd(ctx, p[0], p[1], p[2], p[3], p[4], p[5], p[6], p[7], rows_of(n), int(D), dt))
    # buffers: s, p16 ; args: T, scale
    add("attn_softmax", lambda lib, ctx, p, n, T, scale:
        lib.mg_tk_attn_softmax(ctx, p[0], None, p[1], rows_of(n), int(T), 1, float(scale), dt))
    # buffers: s, seg, p16 ; args: T, H, scale
    add("attn_softmax_doc", lambda lib, ctx, p, n, T, H, scale:
        lib.mg_tk_attn_softmax(ctx, p[0], p[1], p[2], rows_of(n), int(T), int(H), float(scale), dt))
    # buffers: dp, p16, ds16 ; args: T, scale
    add("attn_softmax_bwd", lambda lib, ctx, p, n, T, scale:
        lib.mg_tk_attn_softmax_bwd(ctx, p[0], p[1], p[2], rows_of(n), int(T), float(scale), dt))
    # buffers: a16, b32, out ; n = rows * W ; args: D  (out[r] = sum_d a16[r][d] * b32[r][d])
    add("attn_rowdot", lambda lib, ctx, p, n, D:
        lib.mg_tk_attn_rowdot(ctx, p[0], p[1], p[2], rows_of(n), int(D), dt))
    # buffers: q16, k16, seg (or None), p16 ; n = heads ; args: T, H, hd, scale, causal
    add("attn_p", lambda lib, ctx, p, n, T, H, hd, scale, causal:
        lib.mg_tk_attn_p(ctx, p[0], p[1], p[2], p[3], int(n), int(T), int(H), int(hd), float(scale), int(bool(causal)), dt))
    # buffers: q16, k16, v16, seg (or None), p16, out32, out16 merged (or None) ; n = heads ; args: T, H, hd, scale, causal
    add("attn_fwd", lambda lib, ctx, p, n, T, H, hd, scale, causal:
        lib.mg_tk_attn_fwd(ctx, p[0], p[1], p[2], p[3], p[4], p[5], p[6], int(n), int(T), int(H), int(hd), float(scale),
                           int(bool(causal)), dt))
    # buffers: dout16, v16, p16, rowsub, ds16 ; n = heads ; args: T, hd, scale, causal
    add("attn_ds", lambda lib, ctx, p, n, T, hd, scale, causal:
        lib.mg_tk_attn_ds(ctx, p[0], p[1], p[2], p[3], p[4], int(n), int(T), int(hd), float(scale), int(bool(causal)), dt))
    # buffers: qkv, bias, q16, k16, v16 ; n = rows * D ; args: D, T, H, hd
    add("split_qkv", lambda lib, ctx, p, n, D, T, H, hd:
        lib.mg_tk_split_qkv(ctx, p[0], p[1], p[2], p[3], p[4], n, int(D), int(T), int(H), int(hd), dt))
    # buffers: dq, dk, dv, dqkv16
    add("merge_qkv_grad", lambda lib, ctx, p, n, D, T, H, hd:
        lib.mg_tk_merge_qkv_grad(ctx, p[0], p[1], p[2], p[3], n, int(D), int(T), int(H), int(hd), dt))
    # buffers: src, y16 / src, dst16
    add("merge_heads", lambda lib, ctx, p, n, D, T, H, hd:
        lib.mg_tk_merge_heads(ctx, p[0], p[1], n, int(D), int(T), int(H), int(hd), dt))
    add("split_heads", lambda lib, ctx, p, n, D, T, H, hd:
        lib.mg_tk_split_heads(ctx, p[0], p[1], n, int(D), int(T), int(H), int(hd), dt))
    # column sums: zero, then chunks add into sums (transformer.py:30-37)
    add("col_sum_zero", lambda lib, ctx, p, n: lib.mg_ew_zero(ctx, p[0], n))
    add("col_sum_chunk", lambda lib, ctx, p, n, ncol, nrow, nchunk:
        lib.mg_ew_col_sum(ctx, p[0], p[1], int(ncol), int(nrow), 1))
    add("col_sum_chunk16", lambda lib, ctx, p, n, ncol, nrow, nchunk:
        lib.mg_tk_col_sum16(ctx, p[0], p[1], int(ncol), int(nrow), 1, dt))
    # one-launch forms (no clear needed): buffers: g16 (or g32), sums ; n = ncol ; args: nrow
    add("col_sum16", lambda lib, ctx, p, n, nrow: lib.mg_tk_col_sum16(ctx, p[0], p[1], n, int(nrow), 0, dt))
    add("col_sum", lambda lib, ctx, p, n, nrow: lib.mg_ew_col_sum(ctx, p[0], p[1], n, int(nrow), 0))
    # buffers: tok, pos, ids, x / tok, pos, ids, seg, x ; n = rows * D ; args: D, T
    add("embed", lambda lib, ctx, p, n, D, T: lib.mg_tk_embed(ctx, p[0], p[1], p[2], None, p[3], n, int(D), int(T)))
    add("embed_doc", lambda lib, ctx, p, n, D, T: lib.mg_tk_embed(ctx, p[0], p[1], p[2], p[3], p[4], n, int(D), int(T)))
    # buffers: dx, ids, dtok, dpos / dx, ids, seg, dtok, dpos
    add("embed_bwd", lambda lib, ctx, p, n, D, T:
        lib.mg_tk_embed_bwd(ctx, p[0], p[1], None, p[2], p[3], n, int(D), int(T)))
    add("embed_doc_bwd", lambda lib, ctx, p, n, D, T:
        lib.mg_tk_embed_bwd(ctx, p[0], p[1], p[2], p[3], p[4], n, int(D), int(T)))
    # buffers: acc, bias, res, out ; args: D
    add("residual", lambda lib, ctx, p, n, D: lib.mg_tk_residual(ctx, p[0], p[1], p[2], p[3], n, int(D)))
    add("add", lambda lib, ctx, p, n: lib.mg_tk_add(ctx, p[0], p[1], p[2], n))
    # buffers: a, b, out, out16 ; out = a + b and its 16-bit copy
    add("add16", lambda lib, ctx, p, n: lib.mg_tk_add16(ctx, p[0], p[1], p[2], p[3], n, dt))
    add("add_bias", lambda lib, ctx, p, n, ncol: lib.mg_tk_add_bias(ctx, p[0], p[1], n, int(ncol)))
    add("to16", lambda lib, ctx, p, n: lib.mg_ew_cast16(ctx, p[0], p[1], n, dt))
    # softmax + cross-entropy over wide rows (the LM head; kernels.py:766-823) — same buffers and
    # arguments as the MLP's kernels: logits, labels, dl16, dl32, loss / logits, labels, w, dl16, loss
    add("softmax_ce", lambda lib, ctx, p, n, stride, ncls:
        lib.mg_tk_softmax_ce(ctx, p[0], p[1], None, p[2], p[3], p[4], n, int(stride), int(ncls), dt))
    add("softmax_ce_w", lambda lib, ctx, p, n, stride, ncls:
        lib.mg_tk_softmax_ce(ctx, p[0], p[1], p[2], p[3], None, p[4], n, int(stride), int(ncls), dt))
    return K
