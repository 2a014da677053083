"""Pins oracle/ref_transformer.py (CPU only): closed forms, inverse pairs, explicit index
loops and finite differences - nothing here retypes the formula it checks."""

import numpy as np
import pytest

from oracle import ref_gemm as O
from oracle import ref_transformer as RT


def test_layernorm_rows_are_standardised():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((7, 96)) * 3 + 5).astype(np.float32)
    g = rng.uniform(0.5, 2.0, 96).astype(np.float32)
    b = rng.standard_normal(96).astype(np.float32)
    y16, mu, rstd = RT.layernorm(x, g, b, "f16")
    y = O.widen(y16, "f16")
    xh = (y - b) / g                                   # undo the affine part
    assert np.abs(xh.mean(1)).max() < 2e-3 and np.abs(xh.std(1) - 1).max() < 2e-3
    assert np.allclose(mu, x.astype(np.float64).mean(1), atol=1e-5)
    assert np.allclose(rstd, 1 / np.sqrt(x.astype(np.float64).var(1) + 1e-5), rtol=1e-5)
    # a constant row has no spread: the output is beta and rstd = 1 / sqrt(eps)
    y16, mu, rstd = RT.layernorm(np.full((1, 96), 3.0, np.float32), g, b, "f16")
    assert np.array_equal(y16, O.round_to(b[None, :], "f16")) and abs(rstd[0] - 1 / np.sqrt(1e-5)) < 1


def test_layernorm_backward_matches_finite_differences():
    rng = np.random.default_rng(1)
    rows, D = 3, 16
    x = rng.standard_normal((rows, D))
    g = rng.uniform(0.5, 2.0, D)
    dy = rng.standard_normal((rows, D))

    def f(xv):                                         # scalar whose gradient wrt x is what backward returns
        mu = xv.mean(1, keepdims=True)
        y = (xv - mu) / np.sqrt(((xv - mu) ** 2).mean(1, keepdims=True) + 1e-5) * g
        return float((y * dy).sum())

    num = np.zeros_like(x)
    for i in range(rows):
        for j in range(D):
            e = np.zeros_like(x)
            e[i, j] = 1e-6
            num[i, j] = (f(x + e) - f(x - e)) / 2e-6
    _, mu, rstd = RT.layernorm(x.astype(np.float32), g.astype(np.float32), np.zeros(D, np.float32), "f16")
    dx, dyxh16, dy16 = RT.layernorm_bwd(dy.astype(np.float32), x.astype(np.float32), g.astype(np.float32), mu, rstd, "f16")
    assert np.abs(dx - num).max() < 2e-4
    xh = (x - x.mean(1, keepdims=True)) / np.sqrt(x.var(1, keepdims=True) + 1e-5)
    assert np.abs(O.widen(dyxh16, "f16") - dy * xh).max() < 4e-3
    assert np.array_equal(dy16, O.round_to(dy.astype(np.float32), "f16"))


@pytest.mark.parametrize("packed", [False, True])
def test_attention_softmax_rows(packed):
    rng = np.random.default_rng(2)
    B, H, T = 2, 3, 10
    rows = B * H * T
    s = rng.standard_normal((rows, T)).astype(np.float32) * 4
    seg = None
    if packed:
        seg = np.zeros(B * T, np.uint32)
        seg[4:T] = 4                                   # batch 0: samples start at 0 and 4
        seg[T + 7:2 * T] = 7                           # batch 1: at 0 and 7
    p = O.widen(RT.attn_softmax(s, T, 0.5, "f16", seg=seg, H=H), "f16")
    assert np.abs(p.sum(1) - 1).max() < 2e-3
    for r in range(rows):
        q, b = r % T, r // T // H
        first = int(seg[b * T + q]) if packed else 0
        assert not p[r, q + 1:].any() and not p[r, :first].any()
        vis = s[r, first:q + 1].astype(np.float64) * 0.5
        want = np.exp(vis - vis.max()) / np.exp(vis - vis.max()).sum()
        assert np.abs(p[r, first:q + 1] - want).max() < 1e-3


def test_attention_softmax_backward_matches_finite_differences():
    rng = np.random.default_rng(3)
    T, scale = 6, 0.7
    s = rng.standard_normal((T, T))
    dp = rng.standard_normal((T, T))
    mask = np.tril(np.ones((T, T), bool))

    def f(sv):
        z = np.where(mask, sv * scale, -np.inf)
        p = np.exp(z - z.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        return float((p * dp).sum())

    num = np.zeros_like(s)
    for i in range(T):
        for j in range(i + 1):
            e = np.zeros_like(s)
            e[i, j] = 1e-6
            num[i, j] = (f(s + e) - f(s - e)) / 2e-6
    p16 = RT.attn_softmax(s.astype(np.float32), T, scale, "f16")
    ds = O.widen(RT.attn_softmax_bwd(dp.astype(np.float32), p16, T, scale, "f16"), "f16")
    assert np.abs(ds - num).max() < 3e-3
    assert not ds[~mask].any()


def test_head_permutes_against_index_loops():
    rng = np.random.default_rng(4)
    B, T, H, hd = 2, 3, 2, 4
    D = H * hd
    qkv = rng.standard_normal((B * T, 3 * D)).astype(np.float32)
    bias = rng.standard_normal(3 * D).astype(np.float32)
    q16, k16, v16 = RT.split_qkv(qkv, bias, B, T, H, hd, "f16")
    for which, got in enumerate((q16, k16, v16)):
        got = O.widen(got, "f16")
        for b in range(B):
            for t in range(T):
                for h in range(H):
                    for j in range(hd):
                        col = which * D + h * hd + j
                        want = np.float16(qkv[b * T + t, col] + bias[col])
                        assert got[b * H + h, t, j] == want
    # inverse pairs
    x = rng.standard_normal((B * T, D)).astype(np.float32)
    heads = O.widen(RT.split_heads(x, B, T, H, hd, "f16"), "f16")
    assert np.array_equal(O.widen(RT.merge_heads(heads, B, T, H, hd, "f16"), "f16"), O.widen(O.round_to(x, "f16"), "f16"))
    dq, dk, dv = (rng.standard_normal((B * H, T, hd)).astype(np.float32) for _ in range(3))
    merged = O.widen(RT.merge_qkv_grad(dq, dk, dv, B, T, H, hd, "f16"), "f16")
    back = RT.split_qkv(merged, None, B, T, H, hd, "f16")
    for a, b_ in zip((dq, dk, dv), back):
        assert np.array_equal(O.widen(b_, "f16"), O.widen(O.round_to(a, "f16"), "f16"))


def test_embeddings_against_loops():
    rng = np.random.default_rng(5)
    B, T, D, V = 2, 5, 4, 7
    tok = rng.standard_normal((V, D)).astype(np.float32)
    pos = rng.standard_normal((T, D)).astype(np.float32)
    ids = rng.integers(0, V, B * T).astype(np.uint32)
    seg = np.array([0, 0, 2, 2, 2, 0, 1, 1, 1, 4], np.uint32)
    for sg in (None, seg):
        x = RT.embed(tok, pos, ids, T, sg)
        dx = rng.standard_normal((B * T, D)).astype(np.float32)
        dtok, dpos = RT.embed_bwd(dx, ids, T, V, sg)
        wt, wp = np.zeros((V, D)), np.zeros((T, D))
        for bt in range(B * T):
            t = bt % T - (int(sg[bt]) if sg is not None else 0)
            assert np.array_equal(x[bt], tok[ids[bt]] + pos[t])
            wt[ids[bt]] += dx[bt]
            wp[t] += dx[bt]
        assert np.allclose(dtok, wt, atol=1e-6) and np.allclose(dpos, wp, atol=1e-6)


def test_softmax_ce_rows():
    rng = np.random.default_rng(6)
    rows, stride, ncls = 5, 12, 9
    logits = rng.standard_normal((rows, stride)).astype(np.float32) * 3
    labels = rng.integers(0, ncls, rows).astype(np.uint32)
    loss, dl16, dl32 = RT.softmax_ce_rows(logits, labels, ncls)
    assert np.abs(dl32.sum(1)).max() < 1e-7 and not dl32[:, ncls:].any()       # probabilities minus one-hot
    # uniform logits: loss = log(ncls)
    l2, _, _ = RT.softmax_ce_rows(np.zeros((2, stride), np.float32), np.array([0, 3], np.uint32), ncls)
    assert np.allclose(l2, np.log(ncls), atol=1e-6)
    # the gradient is the derivative of the mean loss
    num = np.zeros((rows, ncls))
    for i in range(rows):
        for c in range(ncls):
            e = np.zeros_like(logits, dtype=np.float64)
            e[i, c] = 1e-4
            lp, _, _ = RT.softmax_ce_rows((logits + e).astype(np.float32), labels, ncls)
            lm, _, _ = RT.softmax_ce_rows((logits - e).astype(np.float32), labels, ncls)
            num[i, c] = (lp.astype(np.float64).mean() - lm.astype(np.float64).mean()) / 2e-4
    assert np.abs(dl32[:, :ncls] - num).max() < 2e-3
    w = np.array([0.5, 0, 2, 1, 0], np.float32)
    lw, d16, dw = RT.softmax_ce_rows(logits, labels, ncls, weights=w)
    assert not lw[w == 0].any() and not dw[w == 0].any()
    assert np.allclose(dw[w > 0], dl32[w > 0] * rows * w[w > 0, None], rtol=1e-5, atol=1e-7)


def _random_params(rng, T, D, n_layer, pad_vocab, tie):
    P = {"tok": rng.standard_normal((pad_vocab, D)) * 0.3, "pos": rng.standard_normal((T, D)) * 0.3,
         "lnf.g": rng.uniform(0.5, 1.5, D), "lnf.b": rng.standard_normal(D) * 0.1}
    if not tie:
        P["head.W"] = rng.standard_normal((D, pad_vocab)) * 0.3
        P["head.b"] = rng.standard_normal(pad_vocab) * 0.3
    shapes = {"ln1.g": (D,), "ln1.b": (D,), "qkv.W": (D, 3 * D), "qkv.b": (3 * D,), "proj.W": (D, D), "proj.b": (D,),
              "ln2.g": (D,), "ln2.b": (D,), "fc1.W": (D, 4 * D), "fc1.b": (4 * D,), "fc2.W": (4 * D, D), "fc2.b": (D,)}
    for l in range(n_layer):
        for n, shp in shapes.items():
            P[f"b{l}.{n}"] = rng.uniform(0.5, 1.5, shp) if n.endswith(".g") else rng.standard_normal(shp) * 0.3
    return P


@pytest.mark.parametrize("tie,packed", [(False, False), (True, False), (True, True)])
def test_whole_model_gradients_match_finite_differences(tie, packed):
    rng = np.random.default_rng(7)
    B, T, D, H, L, vocab, pad = 2, 6, 8, 2, 2, 11, 16
    P = _random_params(rng, T, D, L, pad, tie)
    ids = rng.integers(0, vocab, B * T).astype(np.uint32)
    tgt = rng.integers(0, vocab, B * T).astype(np.uint32)
    seg = weights = None
    if packed:
        seg = np.array([0, 0, 0, 3, 3, 3, 0, 0, 2, 2, 2, 5], np.uint32)
        weights = rng.uniform(0.5, 2.0, B * T)
        weights[[1, 7]] = 0
    model = RT.GPTModel(P, B, T, D, H, L, vocab, pad, tie=tie)
    loss, G, _ = model.loss_and_grads(ids, tgt, seg=seg, weights=weights)
    assert np.isfinite(loss)
    for name in sorted(G):
        flat = model.P[name].reshape(-1)
        picks = rng.choice(flat.size, size=min(4, flat.size), replace=False)
        for i in picks:
            old = flat[i]
            flat[i] = old + 1e-5
            lp, _, _ = model.loss_and_grads(ids, tgt, seg=seg, weights=weights, need_grads=False)
            flat[i] = old - 1e-5
            lm, _, _ = model.loss_and_grads(ids, tgt, seg=seg, weights=weights, need_grads=False)
            flat[i] = old
            num = (lp - lm) / 2e-5
            got = G[name].reshape(-1)[i]
            assert abs(got - num) < 1e-6 + 1e-5 * abs(num), (name, int(i), got, num)
    # padded vocabulary rows take no gradient from the loss
    if not tie:
        assert not G["head.W"][:, vocab:].any() and not G["head.b"][vocab:].any()


def test_packed_samples_equal_separate_sequences():
    """Two samples packed into one row give each sample the loss it has alone."""
    rng = np.random.default_rng(8)
    T, D, H, L, vocab, pad = 8, 8, 2, 1, 11, 16
    P = _random_params(rng, T, D, L, pad, True)
    ids = rng.integers(0, vocab, T).astype(np.uint32)
    tgt = rng.integers(0, vocab, T).astype(np.uint32)
    seg = np.array([0, 0, 0, 3, 3, 3, 3, 3], np.uint32)
    _, _, ce = RT.GPTModel(P, 1, T, D, H, L, vocab, pad, tie=True).loss_and_grads(ids, tgt, seg=seg, need_grads=False)
    Pa = dict(P, pos=P["pos"][:3])
    _, _, ce_a = RT.GPTModel(Pa, 1, 3, D, H, L, vocab, pad, tie=True).loss_and_grads(ids[:3], tgt[:3], need_grads=False)
    Pb = dict(P, pos=P["pos"][:5])
    _, _, ce_b = RT.GPTModel(Pb, 1, 5, D, H, L, vocab, pad, tie=True).loss_and_grads(ids[3:], tgt[3:], need_grads=False)
    assert np.allclose(ce, np.concatenate([ce_a, ce_b]), atol=1e-10)
