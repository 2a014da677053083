"""GPU parity of the decoder-block row kernels and of a whole GPT step.

Kernels are called by the reference's names and call shapes through
vkgrad_amd.tkernels (the C entry points mg_tk_*) and compared with
oracle/ref_transformer.py; the whole model follows the protocol of
/root/reference/test_transformer.py (loss within 5e-3, every gradient tensor
within 3e-2 of its largest entry, against an independent numpy model; tied and
untied head; packed samples with loss weights and one graph per stage)."""

import numpy as np
import pytest

from oracle import ref_gemm as O
from oracle import ref_transformer as RT

pytestmark = pytest.mark.gpu

ULP = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7}


def close16(got_stored, want_stored, dtype, slack=0.0):
    """16-bit results may differ by one rounding step where the f32 values before rounding
    differ in their last bits."""
    g, w = O.widen(got_stored, dtype), O.widen(want_stored, dtype)
    return bool(np.all(np.abs(g - w) <= ULP[dtype] * np.maximum(np.abs(w), 2.0 ** -14) + slack))


def up(dev, arr):
    b = dev.buffer(max(arr.nbytes, 4), "device")
    b.upload(np.ascontiguousarray(arr))
    return b


def stored(buf, dtype, shape):
    raw = buf.download(np.uint16, shape)
    return raw.view(np.float16) if dtype == "f16" else raw


@pytest.fixture(scope="module", params=["f16", "bf16"])
def tk(request, dev):
    from vkgrad_amd.tkernels import make_transformer_kernels
    return request.param, make_transformer_kernels(dev, request.param)


def test_layernorm_forward_backward(dev, tk):
    dtype, TK = tk
    W = dev.row_subgroup_size
    rng = np.random.default_rng(0)
    for rows, D in ((5, 48), (64, 768), (33, 100), (2, 1), (9, 300), (7, 1024), (3, 1028), (6, 77)):
        x = (rng.standard_normal((rows, D)) * 2 + 1).astype(np.float32)
        g = rng.uniform(0.5, 1.5, D).astype(np.float32)
        b = rng.standard_normal(D).astype(np.float32)
        dy = rng.standard_normal((rows, D)).astype(np.float32)
        bx, bg, bb, bdy = up(dev, x), up(dev, g), up(dev, b), up(dev, dy)
        by, bmu, brs = dev.buffer(rows * D * 2, "device"), dev.buffer(rows * 4, "device"), dev.buffer(rows * 4, "device")
        bdx, bxh, bd16 = dev.buffer(rows * D * 4, "device"), dev.buffer(rows * D * 2, "device"), dev.buffer(rows * D * 2, "device")
        bufs = [bx, bg, bb, bdy, by, bmu, brs, bdx, bxh, bd16]
        try:
            TK["layernorm"]([bx, bg, bb, by, bmu, brs], rows * W, D)
            y16, mu, rstd = RT.layernorm(x, g, b, dtype)
            gmu, grs = bmu.download(np.float32, (rows,)), brs.download(np.float32, (rows,))
            assert np.allclose(gmu, mu, atol=1e-5) and np.allclose(grs, rstd, rtol=2e-5)
            assert close16(stored(by, dtype, (rows, D)), y16, dtype, slack=2e-5)
            TK["layernorm_bwd"]([bdy, bx, bg, bmu, brs, bdx, bxh, bd16], rows * W, D)
            dx, dyxh16, dy16 = RT.layernorm_bwd(dy, x, g, gmu, grs, dtype)
            assert np.abs(bdx.download(np.float32, (rows, D)) - dx).max() <= 1e-4 * max(1.0, np.abs(dx).max())
            assert close16(stored(bxh, dtype, (rows, D)), dyxh16, dtype, slack=1e-5)
            assert np.array_equal(stored(bd16, dtype, (rows, D)).view(np.uint16), dy16.view(np.uint16))
        finally:
            for t in bufs:
                t.destroy()


def test_attention_softmax_forward_backward(dev, tk):
    dtype, TK = tk
    W = dev.row_subgroup_size
    rng = np.random.default_rng(1)
    for B, H, T in ((1, 2, 16), (2, 3, 70), (1, 1, 200), (1, 1, 512), (1, 2, 1024), (1, 1, 1100)):
        rows = B * H * T
        s = (rng.standard_normal((rows, T)) * 3).astype(np.float32)
        s[:, T // 2:] += np.where(rng.random((rows, T - T // 2)) < 0.1, 1e4, 0).astype(np.float32)   # masked junk must not leak
        seg = np.zeros(B * T, np.uint32)
        for b in range(B):
            cut = 1 + (7 * b + T // 3) % (T - 1)
            seg[b * T + cut:(b + 1) * T] = cut
        dp = rng.standard_normal((rows, T)).astype(np.float32)
        scale = 1.0 / np.sqrt(8.0)
        bs, bseg, bdp = up(dev, s), up(dev, seg), up(dev, dp)
        bp, bds = dev.buffer(rows * T * 2, "device"), dev.buffer(rows * T * 2, "device")
        try:
            # junk beyond the diagonal only: keep the visible scores tame
            tri = np.arange(T)[None, :] <= (np.arange(rows) % T)[:, None]
            s_vis = np.where(tri, np.minimum(s, 50.0), s).astype(np.float32)
            bs.upload(s_vis)
            TK["attn_softmax"]([bs, bp], rows * W, T, scale)
            want = RT.attn_softmax(s_vis, T, scale, dtype)
            got = stored(bp, dtype, (rows, T))
            assert close16(got, want, dtype, slack=2e-6)
            assert not O.widen(got, dtype)[~tri].any()
            TK["attn_softmax_bwd"]([bdp, bp, bds], rows * W, T, scale)
            want_ds = RT.attn_softmax_bwd(dp, got, T, scale, dtype)
            assert close16(stored(bds, dtype, (rows, T)), want_ds, dtype, slack=2e-5)
            TK["attn_softmax_doc"]([bs, bseg, bp], rows * W, T, H, scale)
            want = RT.attn_softmax(s_vis, T, scale, dtype, seg=seg, H=H)
            assert close16(stored(bp, dtype, (rows, T)), want, dtype, slack=2e-6)
        finally:
            for t in (bs, bseg, bdp, bp, bds):
                t.destroy()


def test_softmax_backward_in_the_dp_gemm(dev, tk):
    """act='softmax_grad': dS leaves the epilogue of dP = dOut V^T (batched over the heads),
    with the row term sum_j P_j dP_j taken from attn_rowdot(dOut, Out).  Checked against the
    separate-pass oracle (attn_softmax_bwd on the f32 dP), for every tile that carries the
    epilogue, with and without the causal tile skipping, ragged sizes included."""
    from vkgrad_amd.kernels import Matmul
    dtype, TK = tk
    W = dev.row_subgroup_size
    rng = np.random.default_rng(11)
    for nbh, T, hd in ((3, 200, 40), (2, 64, 64), (1, 1024, 64), (2, 330, 24), (2, 80, 32), (1, 200, 128), (3, 129, 64), (3, 136, 64), (2, 520, 64), (2, 64, 20)):
        rows = nbh * T
        scale = 1.0 / np.sqrt(hd)
        s = (rng.standard_normal((rows, T)) * 2).astype(np.float32)
        p16 = RT.attn_softmax(s, T, 1.0, dtype)
        p = O.widen(p16, dtype).reshape(nbh, T, T)
        v16 = O.round_to(rng.standard_normal((nbh, T, hd)).astype(np.float32), dtype)
        do16 = O.round_to(rng.standard_normal((nbh, T, hd)).astype(np.float32), dtype)
        v, do = O.widen(v16, dtype), O.widen(do16, dtype)
        out32 = np.einsum("bij,bjd->bid", p, v).astype(np.float32)
        dp = np.einsum("bid,bjd->bij", do, v).astype(np.float32)
        want = RT.attn_softmax_bwd(dp.reshape(rows, T), p16, T, scale, dtype)
        bp, bv, bdo, bout = up(dev, p16), up(dev, v16), up(dev, do16), up(dev, out32)
        bsum, bds, bc = dev.buffer(rows * 4, "device"), dev.buffer(rows * T * 2, "device"), dev.buffer(rows * T * 4, "device")
        try:
            TK["attn_rowdot"]([bdo, bout, bsum], rows * W, hd)
            dot = bsum.download(np.float32, (rows,))
            ref_dot = (dp * p).sum(2, dtype=np.float64).reshape(rows)
            assert np.abs(dot - ref_dot).max() <= 1e-5 * max(1.0, np.abs(ref_dot).max())
            for tile in (None, 3, 4, 10, 11):
                for tri in (None, "c_lower"):
                    bds.upload(np.zeros(rows * T, np.uint16))
                    mm = Matmul(dev, trans_b=True, batched=True, dtype=dtype, tile=tile)
                    mm(bdo, bv, None, T, T, hd, nbatch=nbh, strides=(T * hd, T * hd, T * T), tri=tri,
                       act="softmax_grad", y16=bds, p16=bp, rowsub=bsum, scale=scale)
                    got = stored(bds, dtype, (rows, T))
                    assert close16(got, want, dtype, slack=5e-5), (nbh, T, hd, tile, tri)
            # the one-kernel form for common head widths (same formula, operands straight from memory)
            if dev._lib.mg_tk_attn_ds_supported(hd, T):
                for causal in (False, True):
                    bds.upload(np.zeros(rows * T, np.uint16))
                    TK["attn_ds"]([bdo, bv, bp, bsum, bds], nbh, T, hd, scale, causal)
                    assert close16(stored(bds, dtype, (rows, T)), want, dtype, slack=5e-5), (nbh, T, hd, causal)
            else:
                with pytest.raises(Exception):
                    TK["attn_ds"]([bdo, bv, bp, bsum, bds], nbh, T, hd, scale, False)
            # the f32 copy of the same values, one head
            mm = Matmul(dev, trans_b=True, dtype=dtype)
            mm(bdo, bv, bc, T, T, hd, act="softmax_grad", y16=bds, p16=bp, rowsub=bsum, scale=scale)
            c = bc.download(np.float32, (rows, T))[:T]
            exact = (p[0] * (dp[0] - ref_dot[:T, None]) * scale).astype(np.float32)
            assert np.abs(c - exact).max() <= 5e-5
            assert np.array_equal(stored(bds, dtype, (rows, T))[:T], O.round_to(c, dtype))
        finally:
            for t in (bp, bv, bdo, bout, bsum, bds, bc):
                t.destroy()


def test_scores_and_softmax_in_one_kernel(dev, tk):
    """attn_p: P straight from Q and K (no f32 scores), against the oracle's softmax of the
    numpy scores; plain causal and packed samples (seg), with and without the causal skipping."""
    dtype, TK = tk
    rng = np.random.default_rng(12)
    for B, H, T, hd in ((1, 2, 64, 64), (2, 3, 200, 32), (1, 1, 1024, 64), (1, 2, 520, 128), (2, 1, 136, 64),
                        (1, 1, 1288, 64), (1, 2, 8, 32)):
        nbh, rows = B * H, B * H * T
        scale = 1.0 / np.sqrt(hd)
        assert dev._lib.mg_tk_attn_p_supported(hd, T)
        q16 = O.round_to((rng.standard_normal((nbh, T, hd)) * 1.5).astype(np.float32), dtype)
        k16 = O.round_to((rng.standard_normal((nbh, T, hd)) * 1.5).astype(np.float32), dtype)
        sc = np.einsum("bid,bjd->bij", O.widen(q16, dtype), O.widen(k16, dtype)).astype(np.float32).reshape(rows, T)
        seg = np.zeros(B * T, np.uint32)
        for b in range(B):
            cut = 1 + (7 * b + T // 3) % (T - 1)
            seg[b * T + cut:(b + 1) * T] = cut
        bq, bk, bseg = up(dev, q16), up(dev, k16), up(dev, seg)
        bp = dev.buffer(rows * T * 2, "device")
        try:
            for use_seg in (False, True):
                want = RT.attn_softmax(sc, T, scale, dtype, seg=seg if use_seg else None, H=H)
                for causal in (False, True):
                    bp.upload(np.zeros(rows * T, np.uint16))
                    TK["attn_p"]([bq, bk, bseg if use_seg else None, bp], nbh, T, H, hd, scale, causal)
                    got = stored(bp, dtype, (rows, T))
                    assert close16(got, want, dtype, slack=2e-5), (B, H, T, hd, use_seg, causal)
                    tri = np.arange(T)[None, :] <= (np.arange(rows) % T)[:, None]
                    assert not O.widen(got, dtype)[~tri].any()
        finally:
            for t in (bq, bk, bseg, bp):
                t.destroy()
    assert not dev._lib.mg_tk_attn_p_supported(128, 2048) and not dev._lib.mg_tk_attn_p_supported(40, 64)
    assert not dev._lib.mg_tk_attn_p_supported(64, 100)


def test_attention_forward_in_one_kernel(dev, tk):
    """attn_fwd: P as attn_p writes it (bit for bit: the same arithmetic) and Out = P V behind
    it in the same kernel.  Out is checked against the product of the 16-bit P the kernel stored
    with V, summed in float64 (tolerance: f32 sums of up to 1024 terms, 2e-5 of the largest
    entry plus 1e-5 relative), and P against the oracle's softmax as in the test above; the
    optional 16-bit output must be Out narrowed, in the merged (B*T, H*hd) layout.  Head widths
    32 / 64 / 128; T of one block of queries, of a ragged last block, beyond one wavefront's 256
    keys and of all four; plain causal and packed samples (seg), with and without the causal
    skipping; what the kernel does not take is refused."""
    dtype, TK = tk
    rng = np.random.default_rng(21)
    lib = dev._lib
    for B, H, T, hd in ((1, 2, 72, 64), (2, 3, 264, 32), (1, 1, 1024, 64), (1, 2, 520, 128), (2, 1, 136, 64),
                        (1, 2, 8, 32), (1, 1, 1024, 128), (2, 2, 1024, 32), (1, 3, 264, 128), (1, 1, 776, 64)):
        nbh, rows, D = B * H, B * H * T, H * hd
        scale = 1.0 / np.sqrt(hd)
        assert lib.mg_tk_attn_fwd_supported(hd, T)
        q16 = O.round_to((rng.standard_normal((nbh, T, hd)) * 1.5).astype(np.float32), dtype)
        k16 = O.round_to((rng.standard_normal((nbh, T, hd)) * 1.5).astype(np.float32), dtype)
        v16 = O.round_to((rng.standard_normal((nbh, T, hd)) * 2.0 + 0.25).astype(np.float32), dtype)
        sc = np.einsum("bid,bjd->bij", O.widen(q16, dtype), O.widen(k16, dtype)).astype(np.float32).reshape(rows, T)
        seg = np.zeros(B * T, np.uint32)
        for b in range(B):
            cut = 1 + (7 * b + T // 3) % (T - 1)
            seg[b * T + cut:(b + 1) * T] = cut
        bq, bk, bv, bseg = up(dev, q16), up(dev, k16), up(dev, v16), up(dev, seg)
        bp, bp2 = dev.buffer(rows * T * 2, "device"), dev.buffer(rows * T * 2, "device")
        bo, bo16 = dev.buffer(rows * hd * 4, "device"), dev.buffer(rows * hd * 2, "device")
        try:
            for use_seg in (False, True):
                want = RT.attn_softmax(sc, T, scale, dtype, seg=seg if use_seg else None, H=H)
                for causal in (False, True):
                    for with16 in (False, True):
                        for x in (bp, bp2):
                            x.upload(np.zeros(rows * T, np.uint16))
                        bo.upload(np.full(rows * hd, np.nan, np.float32))
                        bo16.upload(np.full(rows * hd, 0x7FFF, np.uint16))
                        sg = bseg if use_seg else None
                        TK["attn_p"]([bq, bk, sg, bp2], nbh, T, H, hd, scale, causal)
                        TK["attn_fwd"]([bq, bk, bv, sg, bp, bo, bo16 if with16 else None], nbh, T, H, hd, scale, causal)
                        got = stored(bp, dtype, (rows, T))
                        case = (B, H, T, hd, use_seg, causal, with16)
                        assert np.array_equal(np.asarray(got).view(np.uint16), np.asarray(stored(bp2, dtype, (rows, T))).view(np.uint16)), case
                        assert close16(got, want, dtype, slack=2e-5), case
                        out = bo.download(np.float32, (nbh, T, hd))
                        ref = np.einsum("bij,bjd->bid", O.widen(got, dtype).reshape(nbh, T, T).astype(np.float64),
                                        O.widen(v16, dtype).astype(np.float64))
                        assert np.isfinite(out).all(), case
                        tol = 2e-5 * np.abs(ref).max() + 1e-5 * np.abs(ref)
                        assert np.all(np.abs(out - ref) <= tol), (case, float(np.abs(out - ref).max()))
                        raw16 = bo16.download(np.uint16, (B, T, H, hd))
                        if with16:
                            merged = out.reshape(B, H, T, hd).transpose(0, 2, 1, 3)
                            assert np.array_equal(raw16, np.asarray(O.round_to(np.ascontiguousarray(merged), dtype)).view(np.uint16)), case
                        else:
                            assert np.all(raw16 == 0x7FFF), case
        finally:
            for t in (bq, bk, bv, bseg, bp, bp2, bo, bo16):
                t.destroy()
    assert not lib.mg_tk_attn_fwd_supported(64, 1032) and not lib.mg_tk_attn_fwd_supported(40, 64)
    assert not lib.mg_tk_attn_fwd_supported(64, 100) and lib.mg_tk_attn_fwd_supported(128, 1024)


def test_head_permutes(dev, tk):
    dtype, TK = tk
    rng = np.random.default_rng(2)
    for B, T, H, hd in ((2, 5, 3, 4), (1, 64, 12, 64), (2, 7, 3, 5)):      # the last: no groups of four
        D, rows = H * hd, B * T
        qkv = rng.standard_normal((rows, 3 * D)).astype(np.float32)
        bias = rng.standard_normal(3 * D).astype(np.float32)
        bq, bb = up(dev, qkv), up(dev, bias)
        outs = [dev.buffer(rows * D * 2, "device") for _ in range(3)]
        heads32 = [rng.standard_normal((B * H, T, hd)).astype(np.float32) for _ in range(3)]
        hb = [up(dev, h) for h in heads32]
        bm, bx = dev.buffer(rows * 3 * D * 2, "device"), up(dev, qkv[:, :D].copy())
        b16 = dev.buffer(rows * D * 2, "device")
        try:
            TK["split_qkv"]([bq, bb] + outs, rows * D, D, T, H, hd)
            for o, w in zip(outs, RT.split_qkv(qkv, bias, B, T, H, hd, dtype)):
                assert np.array_equal(stored(o, dtype, (B * H, T, hd)).view(np.uint16), w.view(np.uint16))
            TK["merge_qkv_grad"](hb + [bm], rows * D, D, T, H, hd)
            assert np.array_equal(stored(bm, dtype, (rows, 3 * D)).view(np.uint16),
                                  RT.merge_qkv_grad(*heads32, B, T, H, hd, dtype).view(np.uint16))
            TK["merge_heads"]([hb[0], b16], rows * D, D, T, H, hd)
            assert np.array_equal(stored(b16, dtype, (rows, D)).view(np.uint16),
                                  RT.merge_heads(heads32[0], B, T, H, hd, dtype).view(np.uint16))
            TK["split_heads"]([bx, b16], rows * D, D, T, H, hd)
            assert np.array_equal(stored(b16, dtype, (B * H, T, hd)).view(np.uint16),
                                  RT.split_heads(qkv[:, :D].copy(), B, T, H, hd, dtype).view(np.uint16))
        finally:
            for t in [bq, bb, bm, bx, b16] + outs + hb:
                t.destroy()


def test_embeddings_residual_and_column_sums(dev, tk):
    dtype, TK = tk
    rng = np.random.default_rng(3)
    B, T, D, V = 3, 17, 24, 29
    rows = B * T
    tok = rng.standard_normal((V, D)).astype(np.float32)
    pos = rng.standard_normal((T, D)).astype(np.float32)
    ids = rng.integers(0, V, rows).astype(np.uint32)
    seg = np.zeros(rows, np.uint32)
    seg[5:T] = 5
    seg[T + 9:2 * T] = 9
    dx = rng.integers(-8, 8, (rows, D)).astype(np.float32)          # integers: the scatter-add is exact in any order
    btok, bpos, bids, bseg, bdx = up(dev, tok), up(dev, pos), up(dev, ids), up(dev, seg), up(dev, dx)
    bx, bdt, bdp = dev.buffer(rows * D * 4, "device"), dev.buffer(V * D * 4, "device"), dev.buffer(T * D * 4, "device")
    try:
        for sg, bsg in ((None, None), (seg, bseg)):
            if sg is None:
                TK["embed"]([btok, bpos, bids, bx], rows * D, D, T)
            else:
                TK["embed_doc"]([btok, bpos, bids, bsg, bx], rows * D, D, T)
            assert np.array_equal(bx.download(np.float32, (rows, D)), RT.embed(tok, pos, ids, T, sg))
            TK["col_sum_zero"]([bdt], V * D)
            TK["col_sum_zero"]([bdp], T * D)
            if sg is None:
                TK["embed_bwd"]([bdx, bids, bdt, bdp], rows * D, D, T)
            else:
                TK["embed_doc_bwd"]([bdx, bids, bsg, bdt, bdp], rows * D, D, T)
            wt, wp = RT.embed_bwd(dx, ids, T, V, sg)
            assert np.array_equal(bdt.download(np.float32, (V, D)), wt)
            assert np.array_equal(bdp.download(np.float32, (T, D)), wp)
        # residual, add, add_bias, to16
        acc, res = rng.standard_normal((rows, D)).astype(np.float32), rng.standard_normal((rows, D)).astype(np.float32)
        bias = rng.standard_normal(D).astype(np.float32)
        ba, br, bb, bo = up(dev, acc), up(dev, res), up(dev, bias), dev.buffer(rows * D * 4, "device")
        b16 = dev.buffer(rows * D * 2, "device")
        bsum = dev.buffer(D * 4, "device")
        try:
            TK["residual"]([ba, bb, br, bo], rows * D, D)
            assert np.array_equal(bo.download(np.float32, (rows, D)), (res + acc) + bias[None, :]) or \
                np.allclose(bo.download(np.float32, (rows, D)), RT.residual(acc, bias, res), atol=1e-6)
            TK["add"]([ba, br, bo], rows * D)
            assert np.array_equal(bo.download(np.float32, (rows, D)), acc + res)
            TK["add16"]([ba, br, bo, b16], rows * D)        # the sum and its 16-bit copy in one pass
            assert np.array_equal(bo.download(np.float32, (rows, D)), acc + res)
            assert np.array_equal(stored(b16, dtype, (rows, D)).view(np.uint16), O.round_to(acc + res, dtype).view(np.uint16))
            TK["add_bias"]([bo, bb], rows * D, D)
            assert np.array_equal(bo.download(np.float32, (rows, D)), (acc + res) + bias[None, :])
            TK["to16"]([ba, b16], rows * D)
            got16 = stored(b16, dtype, (rows, D))
            assert np.array_equal(got16.view(np.uint16), O.round_to(acc, dtype).view(np.uint16))
            # column sums of the 16-bit matrix, few rows (one chunk) and many (atomics between chunks)
            TK["col_sum_zero"]([bsum], D)
            TK["col_sum_chunk16"]([b16, bsum], 32 * D, D, rows, 32)
            assert np.allclose(bsum.download(np.float32, (D,)), RT.col_sum16(got16, dtype), rtol=1e-6, atol=1e-5)
            TK["col_sum_chunk16"]([b16, bsum], 32 * D, D, rows, 32)       # adds: twice the sums now
            assert np.allclose(bsum.download(np.float32, (D,)), 2 * RT.col_sum16(got16, dtype), rtol=1e-6, atol=1e-5)
        finally:
            for t in (ba, br, bb, bo, b16, bsum):
                t.destroy()
        # sizes that are not multiples of four take the element-wise forms of the same kernels
        r2, d2 = 3, 25
        acc2, res2 = rng.standard_normal((r2, d2)).astype(np.float32), rng.standard_normal((r2, d2)).astype(np.float32)
        bias2 = rng.standard_normal(d2).astype(np.float32)
        ba, br, bb, bo, b16 = up(dev, acc2), up(dev, res2), up(dev, bias2), dev.buffer(r2 * d2 * 4, "device"), dev.buffer(r2 * d2 * 2, "device")
        try:
            TK["residual"]([ba, bb, br, bo], r2 * d2, d2)
            assert np.array_equal(bo.download(np.float32, (r2, d2)), (res2 + acc2) + bias2[None, :])
            TK["add"]([ba, br, bo], r2 * d2)
            assert np.array_equal(bo.download(np.float32, (r2, d2)), acc2 + res2)
            TK["add16"]([ba, br, bo, b16], r2 * d2)
            assert np.array_equal(bo.download(np.float32, (r2, d2)), acc2 + res2)
            assert np.array_equal(stored(b16, dtype, (r2, d2)).view(np.uint16), O.round_to(acc2 + res2, dtype).view(np.uint16))
            TK["to16"]([ba, b16], r2 * d2)
            assert np.array_equal(stored(b16, dtype, (r2, d2)).view(np.uint16), O.round_to(acc2, dtype).view(np.uint16))
        finally:
            for t in (ba, br, bb, bo, b16):
                t.destroy()
        big = O.round_to(rng.integers(-4, 4, (1500, 70)).astype(np.float32), dtype)
        bbig, bs2 = up(dev, big.view(np.uint16)), dev.buffer(70 * 4, "device")
        try:
            TK["col_sum_zero"]([bs2], 70)
            TK["col_sum_chunk16"]([bbig, bs2], 32 * 70, 70, 1500, 32)
            assert np.array_equal(bs2.download(np.float32, (70,)), RT.col_sum16(big, dtype))
            # the one-launch form overwrites whatever sums held, call after call (the chunks'
            # arrival counters are back at zero after each launch)
            for _ in range(3):
                bs2.upload(np.full(70, np.nan, np.float32))
                TK["col_sum16"]([bbig, bs2], 70, 1500)
                assert np.array_equal(bs2.download(np.float32, (70,)), RT.col_sum16(big, dtype))
            TK["col_sum_chunk16"]([bbig, bs2], 32 * 70, 70, 1500, 32)
            assert np.array_equal(bs2.download(np.float32, (70,)), 2 * RT.col_sum16(big, dtype))
            b32 = up(dev, O.widen(big, dtype))
            bs2.upload(np.full(70, np.nan, np.float32))
            TK["col_sum"]([b32, bs2], 70, 1500)
            assert np.array_equal(bs2.download(np.float32, (70,)), RT.col_sum16(big, dtype))
            b32.destroy()
        finally:
            bbig.destroy()
            bs2.destroy()
    finally:
        for t in (btok, bpos, bids, bseg, bdx, bx, bdt, bdp):
            t.destroy()


def test_wide_softmax_cross_entropy(dev, tk):
    dtype, TK = tk
    rng = np.random.default_rng(4)
    for rows, stride, ncls in ((6, 16, 10), (5, 1040, 1000), (3, 50304, 50257), (3, 4100, 4099), (2, 20480, 20000),
                               (2, 60000, 59999), (2, 3001, 3000)):
        logits = (rng.standard_normal((rows, stride)) * 2).astype(np.float32)
        logits[:, ncls:] = 1e4                                      # padding must be masked
        labels = rng.integers(0, ncls, rows).astype(np.uint32)
        w = rng.uniform(0.5, 2.0, rows).astype(np.float32)
        w[1] = 0
        bl, by, bw = up(dev, logits), up(dev, labels), up(dev, w)
        b16, b32, bloss = dev.buffer(rows * stride * 2, "device"), dev.buffer(rows * stride * 4, "device"), dev.buffer(rows * 4, "device")
        try:
            TK["softmax_ce"]([bl, by, b16, b32, bloss], rows, stride, ncls)
            loss, dl16, dl32 = RT.softmax_ce_rows(logits, labels, ncls, None, dtype)
            assert np.allclose(bloss.download(np.float32, (rows,)), loss, rtol=1e-5, atol=1e-5)
            g32 = b32.download(np.float32, (rows, stride))
            assert np.abs(g32 - dl32).max() <= 1e-6 and not g32[:, ncls:].any()
            assert close16(stored(b16, dtype, (rows, stride)), dl16, dtype, slack=1e-7)
            TK["softmax_ce_w"]([bl, by, bw, b16, bloss], rows, stride, ncls)
            loss, dl16, dl32 = RT.softmax_ce_rows(logits, labels, ncls, w, dtype)
            assert np.allclose(bloss.download(np.float32, (rows,)), loss, rtol=1e-5, atol=1e-5)
            got = stored(b16, dtype, (rows, stride))
            assert close16(got, dl16, dtype, slack=1e-6) and not O.widen(got, dtype)[1].any()
        finally:
            for t in (bl, by, bw, b16, b32, bloss):
                t.destroy()


# --------------------------------------------------------------------------
# whole model
# --------------------------------------------------------------------------

def _oracle_name(param_name):
    """'b0.attn.qkv.W' -> 'b0.qkv.W' (the oracle's flat names)."""
    return param_name.replace(".attn.", ".")


def _shared(ctx, arr):
    buf = ctx.buf(arr.nbytes, "shared")
    buf.array(arr.dtype, arr.shape)[:] = arr
    buf.flush()
    return buf


def _relerr(got, want):
    return float(np.abs(got - want).max() / max(np.abs(want).max(), 1e-8))


def _check_model(dev, B, T, D, H, L, vocab, tie, fuse, dtype, packed=False, staged=False, one_kernel=None,
                 replay_other_first=False):
    """one_kernel: assert that Attention took (True) or did not take (False) its one-kernel
    P and dS paths.  replay_other_first: the recorded graphs are first replayed on another
    batch (other tokens, another packing), then on the batch that is checked - what the
    first replay left in P, dS and the gradient buffers must not show."""
    from vkgrad_amd.transformer import GPT, TCtx
    rows = B * T
    ctx = TCtx(dev, dtype=dtype, fuse=fuse)
    try:
        model = GPT(ctx, B, T, D, H, L, vocab, tie=tie)
        if one_kernel is not None:
            for blk in model.blocks:
                assert blk.attn._one_kernel_p == one_kernel and blk.attn._one_kernel_ds == one_kernel
        rng = np.random.default_rng(0)
        ids = rng.integers(0, vocab, rows).astype(np.uint32)
        tgt = rng.integers(0, vocab, rows).astype(np.uint32)
        # non-zero biases (head.b large), or a forward pass that drops one goes unnoticed
        # (test_transformer.py:243-254)
        rb = np.random.default_rng(1)
        for p in model.params():
            if p.name.endswith(".b"):
                p.set((rb.standard_normal(p.shape) * (1.0 if p.name == "head.b" else 0.1)).astype(np.float32))
        seg = weights = segb = wb = None
        if packed:
            seg = np.zeros(rows, np.uint32)
            for b, starts in enumerate(((0, 23, 40, 57), (0, 5, 33))):
                for s, e in zip(starts, starts[1:] + (T,)):
                    seg[b * T + s:b * T + e] = s
            weights = rng.uniform(0.5, 2.0, rows).astype(np.float32)
            weights[rng.random(rows) < 0.3] = 0.0
            segb, wb = _shared(ctx, seg), _shared(ctx, weights)
        idb, tgb = _shared(ctx, ids), _shared(ctx, tgt)
        P = {_oracle_name(p.name): p.numpy() for p in model.params()}
        graphs = {}

        def stage(s):
            if s not in graphs:
                graphs[s] = dev.graph(f"stage{s}")
            return graphs[s]

        model.record(idb, tgb, stage if staged else stage(0), seg=segb, weights=wb)
        if staged:
            assert sorted(graphs) == list(range(model.n_stages()))
        for s in sorted(graphs):
            graphs[s].finish()
        if replay_other_first:
            ro = np.random.default_rng(7)
            idb.array(np.uint32, (rows,))[:] = ro.integers(0, vocab, rows)
            tgb.array(np.uint32, (rows,))[:] = ro.integers(0, vocab, rows)
            if packed:
                other = np.zeros(rows, np.uint32)
                for b in range(B):
                    cut = int(ro.integers(T // 4, 3 * T // 4))
                    other[b * T + cut:(b + 1) * T] = cut
                segb.array(np.uint32, (rows,))[:] = other
                wb.array(np.float32, (rows,))[:] = ro.uniform(0.5, 2.0, rows)
            for s in sorted(graphs):
                graphs[s].submit()
            dev.sync()
            idb.array(np.uint32, (rows,))[:] = ids
            tgb.array(np.uint32, (rows,))[:] = tgt
            if packed:
                segb.array(np.uint32, (rows,))[:] = seg
                wb.array(np.float32, (rows,))[:] = weights
        for s in sorted(graphs):
            graphs[s].submit()
        dev.sync()
        model.loss.invalidate()
        per_row = model.loss.array(np.float32, (rows,)).copy()
        ref = RT.GPTModel(P, B, T, D, H, L, vocab, model.pad_vocab, tie=tie)
        want_loss, G, ce = ref.loss_and_grads(ids, tgt, seg=seg, weights=weights)
        if packed:
            assert not per_row[weights == 0].any(), "rows of weight 0 must report loss 0"
            loss = float((per_row * weights).sum())
        else:
            loss = model.read_loss()
        tol_loss, tol_grad = (5e-3, 3e-2) if dtype == "f16" else (2e-2, 1e-1)
        assert abs(loss - want_loss) / abs(want_loss) < tol_loss, (loss, want_loss)
        worst = {}
        for p in model.params():
            e = _relerr(p.grad_numpy(), G[_oracle_name(p.name)].reshape(p.shape))
            if e >= tol_grad:
                worst[p.name] = e
        assert not worst, f"gradients off: {worst}"
        for g in graphs.values():
            g.destroy()
        return model, G, ref
    finally:
        ctx.destroy()


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("tie", [False, True])
def test_gpt_loss_and_gradients(dev, tie, fuse):
    _check_model(dev, 2, 16, 32, 2, 2, 16, tie, fuse, "f16")


def test_gpt_bf16_ragged_dimensions(dev):
    """bf16 operands, and sizes that are multiples of nothing (T = 19, hd = 9 -> D = 27,
    vocabulary 21): no padding is needed anywhere but the logits' pitch."""
    _check_model(dev, 2, 19, 27, 3, 1, 21, True, True, "bf16")


def test_gpt_one_kernel_attention_paths(dev):
    """Head width 32: Attention takes mg_tk_attn_p and mg_tk_attn_ds (one kernel each for
    P and dS, half-size P / dS buffers cleared once at construction, the row term from
    attn_rowdot, and dQ / dK / dV GEMMs that read the never-written zero region above the
    diagonal) - the path a GPT-2-small step runs."""
    _check_model(dev, 2, 72, 64, 2, 2, 16, True, True, "f16", one_kernel=True)


def test_gpt_one_kernel_attention_long_rows(dev):
    """Head width 64, T = 264 > 256: wavefronts of attn_p with no key to see and key blocks
    that attn_ds skips occur; bf16."""
    _check_model(dev, 1, 264, 128, 2, 1, 32, True, True, "bf16", one_kernel=True)


def test_gpt_one_kernel_attention_packed_replayed_twice(dev):
    """Packed samples, loss weights and one graph per stage through the one-kernel paths;
    every graph is first replayed on another batch with another packing, then on the one
    that is checked: entries of P and dS that the first packing filled and the second masks
    must come back as zeros, and no gradient may carry over."""
    _check_model(dev, 2, 72, 64, 2, 2, 16, True, True, "f16", packed=True, staged=True, one_kernel=True,
                 replay_other_first=True)


def test_gpt_small_heads_do_not_take_the_one_kernel_paths(dev):
    _check_model(dev, 2, 16, 32, 2, 1, 16, True, True, "f16", one_kernel=False)


@pytest.mark.parametrize("fuse", [False, True])
def test_gpt_packed_samples_weights_and_stages(dev, fuse):
    """Samples packed into rows (seg), per-row loss weights and one graph per stage, at once
    (test_transformer.py:279-339): T is past one wavefront's 64 lanes and samples start
    mid-wavefront.  The same device gradients are also compared with a model that ignores
    seg, to show that the check can fail."""
    from vkgrad_amd.transformer import GPT, TCtx
    B, T, D, H, L, vocab = 2, 80, 32, 2, 2, 16
    _check_model(dev, B, T, D, H, L, vocab, True, fuse, "f16", packed=True, staged=True)
    # negative control on the oracle side: without seg the position gradient differs grossly
    rng = np.random.default_rng(0)
    rows = B * T
    ids = rng.integers(0, vocab, rows).astype(np.uint32)
    tgt = rng.integers(0, vocab, rows).astype(np.uint32)
    seg = np.zeros(rows, np.uint32)
    seg[23:T] = 23
    Pr = {"tok": rng.standard_normal((64, D)) * 0.02, "pos": rng.standard_normal((T, D)) * 0.02,
          "lnf.g": np.ones(D), "lnf.b": np.zeros(D)}
    for l in range(L):
        for n, shp in (("ln1.g", (D,)), ("ln1.b", (D,)), ("qkv.W", (D, 3 * D)), ("qkv.b", (3 * D,)),
                       ("proj.W", (D, D)), ("proj.b", (D,)), ("ln2.g", (D,)), ("ln2.b", (D,)),
                       ("fc1.W", (D, 4 * D)), ("fc1.b", (4 * D,)), ("fc2.W", (4 * D, D)), ("fc2.b", (D,))):
            Pr[f"b{l}.{n}"] = np.ones(shp) if n.endswith(".g") else rng.standard_normal(shp) * 0.2
    m = RT.GPTModel(Pr, B, T, D, H, L, vocab, 64, tie=True)
    _, Ga, _ = m.loss_and_grads(ids, tgt, seg=seg)
    _, Gb, _ = m.loss_and_grads(ids, tgt)
    assert _relerr(Ga["pos"], Gb["pos"]) > 0.3
