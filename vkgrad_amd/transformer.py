"""Decoder-only transformer built from the GEMM library and the row kernels.

Public surface = the reference's (/root/reference/transformer.py): `TCtx`,
`LayerNorm`, `Dense`, `Attention`, `Block`, `GPT` with the same constructor
arguments, `forward` / `backward` / `record` / `params` / `read_loss`, the
same parameter attributes (`blk.attn.qkv.W`, `blk.fc1.b`, `model.tok`, ...)
and the same stage numbering for multi-graph recording (transformer.py:326-334),
so scripts and checks written against it run unchanged.  The tensor
conventions are its too (transformer.py:3-13): an f32 residual stream of shape
(B*T, D), 16-bit GEMM operands, f32 GEMM results, heads as (B*H, T, hd).

Inside, each module is a short program over two primitives - `Dense.matmul`
style GEMM calls with epilogue options, and row kernels - and comes in two
flavours chosen by `TCtx(fuse=...)`:

  fuse=False  one kernel per pass, the reference's schedule: GEMM, then bias /
              GELU / residual passes, GELU' as its own pass in backward;
  fuse=True   those passes ride in GEMM epilogues: QKV bias, proj and fc2
              bias + residual (`res=`), fc1 bias + GELU + 16-bit copy (`act=`,
              `y16=`), GELU' inside fc2's dX GEMM (`act='gelu_grad'`, `z=`), the
              softmax backward inside attention's dP GEMM (`act='softmax_grad'`).

Shapes are free (tiles mask their edges); only the vocabulary is padded, to a
multiple of 64 so that rows of the logits stay 16-byte aligned.
"""

import ctypes as C

import numpy as np

from . import _lib as _L
from .autograd import Ctx, Param, _seed
from .kernels import Elementwise
from .tkernels import make_transformer_kernels

NCHUNK = 32   # part of the reference's column-sum call shape; the library picks its own chunks


def _f32(ctx, *dims):
    return ctx.buf(int(np.prod(dims)) * 4)


def _h16(ctx, *dims):
    return ctx.buf(int(np.prod(dims)) * 2)


class TCtx(Ctx):
    """`Ctx` + the transformer's row kernels under `.TK` (transformer.py:22-42)."""

    def __init__(self, dev, tune=False, scalar_only=None, *, dtype="f16", fuse=False, causal_gemms=True):
        super().__init__(dev, tune, scalar_only, dtype=dtype, fuse_bias=fuse)
        self.fuse = bool(fuse)
        self.causal_gemms = bool(causal_gemms)   # attention GEMMs skip what the causal mask zeroes
        self.TK = make_transformer_kernels(dev, dtype)
        self.wave = dev.row_subgroup_size
        self._cleared = set()   # gradient buffers that clear_grads zeroes at the start of a backward pass

    def rowwise(self, name, buffers, rows, *args, graph=None):
        """A row kernel over `rows` rows (dispatch size rows * wavefront width)."""
        self.TK[name](buffers, rows * self.wave, *args, graph=graph)

    def col_sum(self, src, dst, ncol, nrow, graph=None, f16=True):
        """dst[c] = sum over rows of src[r, c]; reads the 16-bit copy unless f16=False.  The
        library clears dst itself when the rows span several chunks (the reference's
        `col_sum_zero` + `col_sum_chunk16` pair, transformer.py:30-37, in one call) - unless
        `clear_grads` has cleared it at the start of this backward pass already."""
        if dst.ptr in self._cleared:
            self.TK["col_sum_chunk16" if f16 else "col_sum_chunk"]([src, dst], NCHUNK * ncol, ncol, nrow, NCHUNK,
                                                                    graph=graph)
        else:
            self.TK["col_sum16" if f16 else "col_sum"]([src, dst], ncol, nrow, graph=graph)

    def clear_grads(self, params, graph=None):
        """One launch that zeroes the gradients of `params` (the step's bias and LayerNorm
        parameters); `col_sum` into them then only adds.  The reference clears in front of every
        sum (transformer.py:30-37): a hundred 4 us launches in a GPT-2-small step."""
        params = list(params)
        if not params:
            return
        entries = (_L.AdamWEntry * len(params))()
        blocks = 0
        for e, p in zip(entries, params):
            e.g, e.n, e.first_block = p.g32.ptr, p.n, blocks
            blocks += -(-p.n // 1024)
        table = self.buf(C.sizeof(entries), "device")
        table.upload(np.frombuffer(entries, dtype=np.uint8))
        n = len(params)
        Elementwise(self.dev, "zero_multi", lambda lib, mg, ptrs, _n: lib.mg_ew_zero_multi(mg, ptrs[0], n, blocks))(
            [table], n, graph=graph)
        self._cleared.update(p.g32.ptr for p in params)

    def destroy(self):
        for kern in self.TK.values():
            kern.destroy()
        super().destroy()


class LayerNorm:
    """Row normalisation with learned gain `g` and shift `b`; emits the 16-bit operand
    of the next GEMM and keeps the row statistics for backward."""

    def __init__(self, ctx, rows, D, name=""):
        self.ctx, self.rows, self.D = ctx, rows, D
        self.g = Param(ctx, (D,), np.ones(D, np.float32), name + ".g", no_decay=True)
        self.b = Param(ctx, (D,), np.zeros(D, np.float32), name + ".b", no_decay=True)
        self.y16 = _h16(ctx, rows, D)
        self.mu, self.rstd = _f32(ctx, rows), _f32(ctx, rows)
        self.dx = _f32(ctx, rows, D)
        self.dyxh, self.dy16 = _h16(ctx, rows, D), _h16(ctx, rows, D)
        self.x32 = None

    def forward(self, x32, graph=None):
        self.x32 = x32
        self.ctx.rowwise("layernorm", [x32, self.g.w32, self.b.w32, self.y16, self.mu, self.rstd],
                         self.rows, self.D, graph=graph)
        return self.y16

    def backward(self, dy32, graph=None):
        ctx = self.ctx
        ctx.rowwise("layernorm_bwd", [dy32, self.x32, self.g.w32, self.mu, self.rstd, self.dx, self.dyxh, self.dy16],
                    self.rows, self.D, graph=graph)
        for src, param in ((self.dyxh, self.g), (self.dy16, self.b)):   # dgain, dshift
            ctx.col_sum(src, param.g32, self.D, self.rows, graph=graph)
        return self.dx


class Dense:
    """Weights (in_f, out_f) + bias.  `forward(x16)` alone is the reference's contract
    (transformer.py:90-95): the bare product lands in `.acc`, the bias is the caller's
    next pass.  Keyword options select GEMM epilogues instead."""

    def __init__(self, ctx, rows, in_f, out_f, name="", scale=None):
        self.ctx, self.rows, self.in_f, self.out_f = ctx, rows, in_f, out_f
        std = np.sqrt(2.0 / in_f) if scale is None else scale
        init = np.random.default_rng(_seed(name)).standard_normal((in_f, out_f)) * std
        self.W = Param(ctx, (in_f, out_f), init.astype(np.float32), name + ".W")
        self.b = Param(ctx, (out_f,), np.zeros(out_f, np.float32), name + ".b", no_decay=True)
        self.acc = _f32(ctx, rows, out_f)
        self.dx32 = _f32(ctx, rows, in_f)
        self.x16 = None

    def forward(self, x16, graph=None, *, bias=False, act=None, y16=None, res=None, out=None):
        """out (default .acc) = x16 @ W [+ b] [+ res]; y16 = narrow(act(out)) when given."""
        self.x16 = x16
        dst = out if out is not None else self.acc
        R, N, K = self.rows, self.out_f, self.in_f
        self.ctx.matmul(R, N, K)(x16, self.W.w16, dst, R, N, K, graph=graph,
                                 bias=self.b.w32 if bias else None, act=act, y16=y16, res=res)
        return dst

    def backward(self, dy16, need_dx=True, graph=None, *, act_grad=None, z=None, dz16=None):
        """Writes W.g32 and b.g32; returns dx32 - or, with act_grad / z / dz16, the 16-bit
        dz16 = narrow(dX * act'(z)) straight from the dX GEMM."""
        ctx, R, N, K = self.ctx, self.rows, self.out_f, self.in_f
        ctx.matmul(K, N, R, trans_a=True)(self.x16, dy16, self.W.g32, K, N, R, graph=graph)      # dW = x^T dy
        ctx.col_sum(dy16, self.b.g32, N, R, graph=graph)
        if not need_dx:
            return None
        dx_gemm = ctx.matmul(R, K, N, trans_b=True)                                               # dX = dy W^T
        if act_grad is None:
            dx_gemm(dy16, self.W.w16, self.dx32, R, K, N, graph=graph)
            return self.dx32
        dx_gemm(dy16, self.W.w16, None, R, K, N, graph=graph, act=act_grad, z=z, y16=dz16)
        return dz16


class Attention:
    """Causal multi-head self-attention: fused QKV projection, six strided-batched GEMMs
    over the B*H heads, the softmax row kernels, and the output projection."""

    def __init__(self, ctx, B, T, D, H, name=""):
        if D % H:
            raise ValueError(f"d_model {D} is not a multiple of the head count {H}")
        self.ctx, self.B, self.T, self.D, self.H = ctx, B, T, D, H
        self.hd, self.rows, self.nbh = D // H, B * T, B * H
        self.scale = 1.0 / np.sqrt(self.hd)
        self.qkv = Dense(ctx, self.rows, D, 3 * D, name + ".qkv")
        self.proj = Dense(ctx, self.rows, D, D, name + ".proj", scale=np.sqrt(2.0 / D) * 0.5)
        nbh, T_, hd = self.nbh, T, self.hd
        self.q16, self.k16, self.v16 = (_h16(ctx, nbh, T_, hd) for _ in range(3))
        lib = ctx.dev._lib
        self._one_kernel_p = bool(ctx.fuse and lib.mg_tk_attn_p_supported(self.hd, T))
        # P, Out = P V and the merged 16-bit copy of Out from one kernel (P is written, not read back).
        # For heads up to 64 wide: 96 heads x 1024 x 64 take 115 us against 77 + 39 + 8 for P, the
        # P V GEMM and merge_heads, 32 wide 62 against 103; 128 wide the kernel needs the registers
        # of a whole SIMD lane and loses (167 against 133 us).
        self._one_kernel_fwd = bool(ctx.fuse and self.hd <= 64 and lib.mg_tk_attn_fwd_supported(self.hd, T))
        self._one_kernel_ds = bool(ctx.fuse and lib.mg_tk_attn_ds_supported(self.hd, T))
        if self._one_kernel_p:
            # P comes out of one kernel (scores + softmax): no f32 scores.  Wavefronts whose keys all
            # lie beyond their queries write nothing, so P is cleared once, here.
            self.scores = None
            self.p16 = ctx.zeros(nbh * T_ * T_ // 2 + 1)
        else:
            self.scores, self.p16 = _f32(ctx, nbh, T_, T_), _h16(ctx, nbh, T_, T_)
        self.ao32, self.ao16 = _f32(ctx, nbh, T_, hd), _h16(ctx, self.rows, D)
        self.dao16 = _h16(ctx, nbh, T_, hd)
        if ctx.fuse:
            # dS comes straight out of the dP GEMM (act='softmax_grad'): no f32 dP.  Tiles wholly
            # above the diagonal are never written, and the dQ / dK GEMMs may read into them
            # (their row blocks can be taller than the dP GEMM's tiles): they stay zero from here.
            self.dp32 = None
            self.ds16 = ctx.zeros(nbh * T_ * T_ // 2 + 1)
            self.dsum = _f32(ctx, nbh, T_)
        else:
            self.dp32, self.ds16 = _f32(ctx, nbh, T_, T_), _h16(ctx, nbh, T_, T_)
        self.dq32, self.dk32, self.dv32 = (_f32(ctx, nbh, T_, hd) for _ in range(3))
        self.dqkv16 = _h16(ctx, self.rows, 3 * D)
        # per-head GEMMs as (M, N, K, trans_a, trans_b); a (T, hd) tensor advances `vec`
        # elements per head, a (T, T) tensor `sq`
        vec, sq = T * self.hd, T * T
        # The last entry is the causal structure: scores and dP are only read at keys <= query;
        # P and dS are zero beyond the query, so products with them stop (or start) there.
        self._head_gemms = {
            "scores": (T, T, self.hd, False, True, (vec, vec, sq), "c_lower"),    # Q K^T
            "mix":    (T, self.hd, T, False, False, (sq, vec, vec), "a_lower"),   # P V
            "dV":     (T, self.hd, T, True, False, (sq, vec, vec), "a_upper"),    # P^T dOut
            "dP":     (T, T, self.hd, False, True, (vec, vec, sq), "c_lower"),    # dOut V^T
            "dQ":     (T, self.hd, T, False, False, (sq, vec, vec), "a_lower"),   # dS K
            "dK":     (T, self.hd, T, True, False, (sq, vec, vec), "a_upper"),    # dS^T Q
        }

    def _heads(self, which, a, b, c, graph, **epilogue):
        m, n, k, ta, tb, strides, tri = self._head_gemms[which]
        mm = self.ctx.matmul(m, n, k, trans_a=ta, trans_b=tb, batched=True, nbatch=self.nbh)
        mm(a, b, c, m, n, k, graph=graph, nbatch=self.nbh, strides=strides,
           tri=tri if self.ctx.causal_gemms else None, **epilogue)

    def _permute(self, name, buffers, graph):
        self.ctx.TK[name](buffers, self.rows * self.D, self.D, self.T, self.H, self.hd, graph=graph)

    def forward(self, x16, graph=None, seg=None, *, res=None, out=None):
        """Returns the projection's bare accumulator; in a fused context with `res` and `out`
        the projection writes out = res + proj + bias instead and returns `out`."""
        ctx = self.ctx
        fused = ctx.fuse
        qkv = self.qkv.forward(x16, graph=graph, bias=fused)
        self._permute("split_qkv", [qkv, None if fused else self.qkv.b.w32, self.q16, self.k16, self.v16], graph)
        if self._one_kernel_fwd:
            ctx.TK["attn_fwd"]([self.q16, self.k16, self.v16, seg, self.p16, self.ao32, self.ao16], self.nbh, self.T,
                               self.H, self.hd, self.scale, ctx.causal_gemms, graph=graph)
            if fused and res is not None:
                return self.proj.forward(self.ao16, graph=graph, bias=True, res=res, out=out)
            return self.proj.forward(self.ao16, graph=graph)
        if self._one_kernel_p:
            ctx.TK["attn_p"]([self.q16, self.k16, seg, self.p16], self.nbh, self.T, self.H, self.hd, self.scale,
                             ctx.causal_gemms, graph=graph)
        else:
            self._heads("scores", self.q16, self.k16, self.scores, graph)
            if seg is None:
                ctx.rowwise("attn_softmax", [self.scores, self.p16], self.nbh * self.T, self.T, self.scale, graph=graph)
            else:
                ctx.rowwise("attn_softmax_doc", [self.scores, seg, self.p16], self.nbh * self.T, self.T, self.H,
                            self.scale, graph=graph)
        self._heads("mix", self.p16, self.v16, self.ao32, graph)
        self._permute("merge_heads", [self.ao32, self.ao16], graph)
        if fused and res is not None:
            return self.proj.forward(self.ao16, graph=graph, bias=True, res=res, out=out)
        return self.proj.forward(self.ao16, graph=graph)

    def backward(self, dy16, graph=None):
        ctx = self.ctx
        dao32 = self.proj.backward(dy16, need_dx=True, graph=graph)
        self._permute("split_heads", [dao32, self.dao16], graph)
        self._heads("dV", self.p16, self.dao16, self.dv32, graph)
        if ctx.fuse:
            # sum_j P_j dP_j = sum_d dOut_d Out_d (dP = dOut V^T, Out = P V), so the row term of the
            # softmax backward is known before dP, and dS leaves the dP GEMM's epilogue directly
            ctx.rowwise("attn_rowdot", [self.dao16, self.ao32, self.dsum], self.nbh * self.T, self.hd, graph=graph)
            if self._one_kernel_ds:
                # common head widths: product, P and the row term meet in one kernel without LDS
                ctx.TK["attn_ds"]([self.dao16, self.v16, self.p16, self.dsum, self.ds16], self.nbh, self.T, self.hd,
                                  self.scale, ctx.causal_gemms, graph=graph)
            else:
                self._heads("dP", self.dao16, self.v16, None, graph, act="softmax_grad", y16=self.ds16,
                            p16=self.p16, rowsub=self.dsum, scale=self.scale)
        else:
            self._heads("dP", self.dao16, self.v16, self.dp32, graph)
            ctx.rowwise("attn_softmax_bwd", [self.dp32, self.p16, self.ds16], self.nbh * self.T, self.T, self.scale,
                        graph=graph)
        self._heads("dQ", self.ds16, self.k16, self.dq32, graph)
        self._heads("dK", self.ds16, self.q16, self.dk32, graph)
        self._permute("merge_qkv_grad", [self.dq32, self.dk32, self.dv32, self.dqkv16], graph)
        return self.qkv.backward(self.dqkv16, need_dx=True, graph=graph)


class Block:
    """Pre-norm block: x -> res1 = x + attn(ln1(x)) -> res2 = res1 + mlp(ln2(res1))."""

    def __init__(self, ctx, B, T, D, H, name=""):
        self.ctx, self.rows, self.D = ctx, B * T, D
        R = self.rows
        self.ln1 = LayerNorm(ctx, R, D, name + ".ln1")
        self.attn = Attention(ctx, B, T, D, H, name + ".attn")
        self.ln2 = LayerNorm(ctx, R, D, name + ".ln2")
        self.fc1 = Dense(ctx, R, D, 4 * D, name + ".fc1")
        self.fc2 = Dense(ctx, R, 4 * D, D, name + ".fc2", scale=np.sqrt(2.0 / (4 * D)) * 0.5)
        self.res1, self.res2 = _f32(ctx, R, D), _f32(ctx, R, D)
        self.z1, self.h16, self.dh16 = _f32(ctx, R, 4 * D), _h16(ctx, R, 4 * D), _h16(ctx, R, 4 * D)
        self.dres1, self.dx = _f32(ctx, R, D), _f32(ctx, R, D)
        self.attn16, self.mlp16 = _h16(ctx, R, D), _h16(ctx, R, D)
        self.dx16 = _h16(ctx, R, D) if ctx.fuse else None
        self.x32 = None

    # -- forward -----------------------------------------------------------
    def _attn_sublayer(self, x32, graph, seg):
        normed = self.ln1.forward(x32, graph=graph)
        if self.ctx.fuse:
            self.attn.forward(normed, graph=graph, seg=seg, res=x32, out=self.res1)
        else:
            proj = self.attn.forward(normed, graph=graph, seg=seg)
            self.ctx.TK["residual"]([proj, self.attn.proj.b.w32, x32, self.res1], self.rows * self.D, self.D,
                                    graph=graph)

    def _mlp_sublayer(self, graph):
        ctx, wide = self.ctx, 4 * self.D
        normed = self.ln2.forward(self.res1, graph=graph)
        if ctx.fuse:
            self.fc1.forward(normed, graph=graph, bias=True, act="gelu", y16=self.h16, out=self.z1)
            self.fc2.forward(self.h16, graph=graph, bias=True, res=self.res1, out=self.res2)
            return
        pre = self.fc1.forward(normed, graph=graph)
        ctx.K["bias_gelu"]([pre, self.fc1.b.w32, self.z1, self.h16], self.rows * wide, wide, graph=graph)
        down = self.fc2.forward(self.h16, graph=graph)
        ctx.TK["residual"]([down, self.fc2.b.w32, self.res1, self.res2], self.rows * self.D, self.D, graph=graph)

    def forward(self, x32, graph=None, seg=None):
        self.x32 = x32
        self._attn_sublayer(x32, graph, seg)
        self._mlp_sublayer(graph)
        return self.res2

    # -- backward ----------------------------------------------------------
    def backward(self, d32, graph=None, d16=None):
        """d32 = dLoss/d res2 (d16: its 16-bit copy, if the caller has one).  A residual passes
        its gradient to both of its inputs, so each sublayer's input gradient is the incoming one
        plus what comes back through the branch.  In a fused context the sums leave their `add`
        together with the 16-bit copy the next GEMMs read (`self.dx16` for the block below)."""
        ctx, TK, n = self.ctx, self.ctx.TK, self.rows * self.D
        if d16 is None:
            d16 = self.mlp16
            TK["to16"]([d32, d16], n, graph=graph)
        if ctx.fuse:
            self.fc2.backward(d16, graph=graph, act_grad="gelu_grad", z=self.z1, dz16=self.dh16)
        else:
            dh32 = self.fc2.backward(d16, graph=graph)
            ctx.K["bias_gelu_bwd16"]([dh32, self.z1, self.dh16], self.rows * 4 * self.D, graph=graph)
        through_mlp = self.ln2.backward(self.fc1.backward(self.dh16, graph=graph), graph=graph)
        if ctx.fuse:
            TK["add16"]([d32, through_mlp, self.dres1, self.attn16], n, graph=graph)
        else:
            TK["add"]([d32, through_mlp, self.dres1], n, graph=graph)
            TK["to16"]([self.dres1, self.attn16], n, graph=graph)
        through_attn = self.ln1.backward(self.attn.backward(self.attn16, graph=graph), graph=graph)
        if ctx.fuse:
            TK["add16"]([self.dres1, through_attn, self.dx, self.dx16], n, graph=graph)
        else:
            TK["add"]([self.dres1, through_attn, self.dx], n, graph=graph)
        return self.dx

    def params(self):
        a = self.attn
        yield from (self.ln1.g, self.ln1.b, self.ln2.g, self.ln2.b, a.qkv.W, a.qkv.b, a.proj.W, a.proj.b,
                    self.fc1.W, self.fc1.b, self.fc2.W, self.fc2.b)


class GPT:
    """Token + position embeddings, n_layer blocks, final LayerNorm, LM head (its own Dense,
    or with tie=True the token table transposed), mean or weighted cross-entropy."""

    def __init__(self, ctx, B, T, D, H, n_layer, vocab, pad_vocab=None, tie=False):
        self.ctx, self.B, self.T, self.D, self.tie = ctx, B, T, D, tie
        self.rows, self.vocab = B * T, vocab
        self.pad_vocab = pad_vocab or -(-vocab // 64) * 64
        if self.pad_vocab < vocab:
            raise ValueError(f"pad_vocab {self.pad_vocab} < vocab {vocab}")
        V, R = self.pad_vocab, self.rows
        rng = np.random.default_rng(1234)
        self.tok = Param(ctx, (V, D), (rng.standard_normal((V, D)) * 0.02).astype(np.float32), "tok")
        self.pos = Param(ctx, (T, D), (rng.standard_normal((T, D)) * 0.02).astype(np.float32), "pos")
        self.x0 = _f32(ctx, R, D)
        self.blocks = [Block(ctx, B, T, D, H, f"b{i}") for i in range(n_layer)]
        self.lnf = LayerNorm(ctx, R, D, "lnf")
        if tie:
            self.logits, self.dh32 = _f32(ctx, R, V), _f32(ctx, R, D)
        else:
            self.head = Dense(ctx, R, D, V, "head", scale=0.02)
        self.dlog16, self.dlog32 = _h16(ctx, R, V), None   # nothing downstream reads an f32 copy of dlogits
        self.loss = ctx.buf(R * 4, "cached")
        self.h16 = None

    def params(self):
        yield from (self.tok, self.pos)
        for blk in self.blocks:
            yield from blk.params()
        yield from (self.lnf.g, self.lnf.b)
        if not self.tie:
            yield from (self.head.W, self.head.b)

    def n_params(self):
        return sum(p.n for p in self.params())

    def n_stages(self):
        return 2 * len(self.blocks) + 3

    @staticmethod
    def _stages(graph):
        return graph if callable(graph) else (lambda stage: graph)

    def _embedding(self, name, lead, ids_buf, seg, tail, graph):
        """embed / embed_bwd, or their _doc forms when the rows hold packed samples."""
        if seg is None:
            bufs = lead + [ids_buf] + tail
        else:
            name = name.replace("embed", "embed_doc")
            bufs = lead + [ids_buf, seg] + tail
        self.ctx.TK[name](bufs, self.rows * self.D, self.D, self.T, graph=graph)

    def forward(self, ids_buf, graph=None, seg=None):
        """-> logits buffer (rows, pad_vocab).  seg, optional (B*T,) u32: start of each token's
        sample inside its row - attention and positions then restart per sample."""
        ctx, stage, L = self.ctx, self._stages(graph), len(self.blocks)
        self._embedding("embed", [self.tok.w32, self.pos.w32], ids_buf, seg, [self.x0], stage(0))
        x = self.x0
        for i, blk in enumerate(self.blocks):
            x = blk.forward(x, graph=stage(i), seg=seg)
        h16 = self.lnf.forward(x, graph=stage(L))
        R, V, D = self.rows, self.pad_vocab, self.D
        if self.tie:
            self.h16 = h16
            ctx.matmul(R, V, D, trans_b=True)(h16, self.tok.w16, self.logits, R, V, D, graph=stage(L))   # h tok^T
            return self.logits
        if ctx.fuse:
            return self.head.forward(h16, graph=stage(L), bias=True)
        logits = self.head.forward(h16, graph=stage(L))
        ctx.TK["add_bias"]([logits, self.head.b.w32], R * V, V, graph=stage(L))
        return logits

    def _head_backward(self, graph):
        """-> dLoss/d(final LayerNorm output), f32; also the head's parameter gradients."""
        ctx, R, V, D = self.ctx, self.rows, self.pad_vocab, self.D
        if not self.tie:
            d = self.head.backward(self.dlog16, need_dx=True, graph=graph)
            ctx.TK["col_sum_zero"]([self.tok.g32], self.tok.n, graph=graph)     # the scatter-add starts from zero
            return d
        ctx.matmul(R, D, V)(self.dlog16, self.tok.w16, self.dh32, R, D, V, graph=graph)                  # dlogits tok
        # the head's share of dtok; a GEMM overwrites, which doubles as the clear before the scatter-add
        ctx.matmul(V, D, R, trans_a=True)(self.dlog16, self.h16, self.tok.g32, V, D, R, graph=graph)     # dlogits^T h
        return self.dh32

    def record(self, ids_buf, targets_buf, graph, backward=True, seg=None, weights=None):
        """Record loss and (unless backward=False) all gradients into `graph`, a Graph or a
        callable stage -> Graph.  Stage order: 0..L-1 embedding (in 0) and block i forward;
        L head + loss; L+1 head and final-norm backward; L+2+k block L-1-k backward; 2L+2
        embedding backward.  weights, optional (B*T,) f32, replace the 1/rows mean by per-row
        factors; `loss` then holds unweighted per-row cross-entropy, 0 where the weight is 0."""
        TK, stage, L = self.ctx.TK, self._stages(graph), len(self.blocks)
        logits = self.forward(ids_buf, graph=stage, seg=seg)
        shape = (self.rows, self.pad_vocab, self.vocab)
        if weights is None:
            TK["softmax_ce"]([logits, targets_buf, self.dlog16, self.dlog32, self.loss], *shape, graph=stage(L))
        else:
            TK["softmax_ce_w"]([logits, targets_buf, weights, self.dlog16, self.loss], *shape, graph=stage(L))
        if not backward:
            return
        if self.ctx.fuse:
            # every bias and LayerNorm gradient is a column sum: clear them all in one launch here
            # instead of one small launch in front of each sum
            self.ctx.clear_grads([p for p in self.params() if len(p.shape) == 1], graph=stage(L + 1))
        d = self.lnf.backward(self._head_backward(stage(L + 1)), graph=stage(L + 1))
        d16 = None
        for k, blk in enumerate(reversed(self.blocks)):
            d = blk.backward(d, graph=stage(L + 2 + k), d16=d16)
            d16 = blk.dx16
        self.ctx._cleared.clear()   # later recordings clear for themselves again
        last = stage(2 * L + 2)
        TK["col_sum_zero"]([self.pos.g32], self.pos.n, graph=last)
        self._embedding("embed_bwd", [d], ids_buf, seg, [self.tok.g32, self.pos.g32], last)

    def read_loss(self):
        self.loss.invalidate()
        return float(self.loss.array(np.float32, (self.rows,)).mean())
