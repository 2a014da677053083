"""numpy restatement of the decoder-block row kernels and of a whole GPT step.
TEST INFRASTRUCTURE ONLY: nothing outside tests/, the smoke check and the CPU
baseline may import this module.

Part 1 - the row kernels, one function per kernel of /root/reference/tkernels.py,
float32 arithmetic, 16-bit outputs rounded (round to nearest even) where the
device rounds:

  layernorm / layernorm_bwd              tkernels.py:32-56, 58-92
  attn_softmax(_doc) / attn_softmax_bwd  tkernels.py:105-133, 135-165, 167-187
  split_qkv / merge_qkv_grad             tkernels.py:195-213, 215-231
  merge_heads / split_heads              tkernels.py:274-286, 288-300
  embed(_doc) / embed(_doc)_bwd          tkernels.py:303-315, 334-345, 317-332, 347-360
  residual / add / add_bias              tkernels.py:362-382
  col_sum16                              tkernels.py:238-270 (zero, then chunked sums)
  softmax_ce_rows                        kernels.py:766-823 (mean or per-row weights)

Part 2 - `GPTModel`: forward and backward of the architecture the reference's
transformer.py builds (pre-norm blocks, fused QKV projection, causal attention
optionally restricted to packed samples, GELU MLP, final LayerNorm, tied or
untied head, mean or weighted cross-entropy), in one float type with no
16-bit rounding: the independent model of the reference's own whole-model check
(test_transformer.py:39-152, tolerances :152-230: loss 5e-3, gradients 3e-2 of
the largest entry).

Pinned by tests/test_oracle_transformer.py: LayerNorm rows have mean beta and
spread gamma, its backward and the softmax backward match finite differences in
float64, softmax rows sum to one with zeros beyond the mask, permutes are
inverse pairs that match an explicit index loop, the scatter-add matches a
loop, and every gradient tensor of GPTModel matches central differences of its
loss in float64 (tied and untied, packed samples with weights).
"""

import numpy as np

from .ref_gemm import round_to, widen
from .ref_mlp import dgelu, gelu

LN_EPS = np.float32(1e-5)


# --------------------------------------------------------------------------
# Part 1: kernels
# --------------------------------------------------------------------------

def layernorm(x, gamma, beta, dtype="f16"):
    """-> (y16 stored, mu, rstd); x is (rows, D) float32."""
    D = x.shape[1]
    mu = (x.sum(1, dtype=np.float32) / np.float32(D)).astype(np.float32)
    cen = x - mu[:, None]
    var = (cen * cen).sum(1, dtype=np.float32) / np.float32(D)
    rstd = (np.float32(1.0) / np.sqrt(var + LN_EPS)).astype(np.float32)
    y = cen * rstd[:, None] * gamma[None, :] + beta[None, :]
    return round_to(y.astype(np.float32), dtype), mu, rstd


def layernorm_bwd(dy, x, gamma, mu, rstd, dtype="f16"):
    """-> (dx float32, (dy * xhat) stored 16-bit, dy stored 16-bit)."""
    D = np.float32(x.shape[1])
    xh = (x - mu[:, None]) * rstd[:, None]
    dxh = dy * gamma[None, :]
    s1 = dxh.sum(1, dtype=np.float32)[:, None] / D
    s2 = (dxh * xh).sum(1, dtype=np.float32)[:, None] / D
    dx = rstd[:, None] * (dxh - s1 - xh * s2)
    return dx.astype(np.float32), round_to((dy * xh).astype(np.float32), dtype), round_to(dy, dtype)


def _key_mask(rows, T, H, seg):
    """mask[r, j]: key j is visible to the query of row r (rows = B*H*T)."""
    q = np.arange(rows) % T
    j = np.arange(T)[None, :]
    mask = j <= q[:, None]
    if seg is not None:
        first = seg.astype(np.int64)[(np.arange(rows) // T // H) * T + q]
        mask &= j >= first[:, None]
    return mask


def attn_softmax(s, T, scale, dtype="f16", seg=None, H=1):
    """s: (rows, T) float32 scores -> probabilities stored 16-bit, zeros where masked."""
    rows = s.shape[0]
    mask = _key_mask(rows, T, H, seg)
    z = np.where(mask, s * np.float32(scale), np.float32(-1e30)).astype(np.float32)
    z = z - z.max(1, keepdims=True)
    e = np.where(mask, np.exp(z), np.float32(0)).astype(np.float32)
    p = e / e.sum(1, keepdims=True, dtype=np.float32)
    return round_to(p.astype(np.float32), dtype)


def attn_softmax_bwd(dp, p16, T, scale, dtype="f16"):
    """dS = P (dP - sum_j dP_j P_j) scale with the 16-bit P; masked entries have P = 0."""
    rows = dp.shape[0]
    mask = _key_mask(rows, T, 1, None)
    p = np.where(mask, widen(p16, dtype), np.float32(0))
    dot = (np.where(mask, dp, np.float32(0)) * p).sum(1, keepdims=True, dtype=np.float32)
    ds = np.where(mask, p * (dp - dot) * np.float32(scale), np.float32(0))
    return round_to(ds.astype(np.float32), dtype)


def to_heads(x, B, T, H, hd):
    """(B*T, H*hd) -> (B*H, T, hd)"""
    return np.ascontiguousarray(x.reshape(B, T, H, hd).transpose(0, 2, 1, 3)).reshape(B * H, T, hd)


def from_heads(x, B, T, H, hd):
    """(B*H, T, hd) -> (B*T, H*hd)"""
    return np.ascontiguousarray(x.reshape(B, H, T, hd).transpose(0, 2, 1, 3)).reshape(B * T, H * hd)


def split_qkv(qkv, bias, B, T, H, hd, dtype="f16"):
    D = H * hd
    full = qkv + (bias[None, :] if bias is not None else np.float32(0))
    return tuple(round_to(to_heads(full[:, i * D:(i + 1) * D], B, T, H, hd).astype(np.float32), dtype)
                 for i in range(3))


def merge_qkv_grad(dq, dk, dv, B, T, H, hd, dtype="f16"):
    parts = [from_heads(t, B, T, H, hd) for t in (dq, dk, dv)]
    return round_to(np.concatenate(parts, axis=1).astype(np.float32), dtype)


def merge_heads(src, B, T, H, hd, dtype="f16"):
    return round_to(from_heads(src, B, T, H, hd).astype(np.float32), dtype)


def split_heads(src, B, T, H, hd, dtype="f16"):
    return round_to(to_heads(src, B, T, H, hd).astype(np.float32), dtype)


def positions(rows, T, seg=None):
    t = np.arange(rows) % T
    return t if seg is None else t - seg.astype(np.int64)


def embed(tok, pos, ids, T, seg=None):
    return (tok[ids.astype(np.int64)] + pos[positions(len(ids), T, seg)]).astype(np.float32)


def embed_bwd(dx, ids, T, tok_rows, seg=None):
    """-> (dtok, dpos): scatter-add of dx rows by token id and by position."""
    D = dx.shape[1]
    dtok = np.zeros((tok_rows, D), np.float64)
    dpos = np.zeros((T, D), np.float64)
    np.add.at(dtok, ids.astype(np.int64), dx)
    np.add.at(dpos, positions(len(ids), T, seg), dx)
    return dtok.astype(np.float32), dpos.astype(np.float32)


def residual(acc, bias, res):
    return (res + acc + bias[None, :]).astype(np.float32)


def col_sum16(g16, dtype="f16"):
    return widen(g16, dtype).sum(0, dtype=np.float64).astype(np.float32)


def softmax_ce_rows(logits, labels, ncls, weights=None, dtype="f16"):
    """logits (rows, stride) -> (loss per row, dl16 stored, dl32); classes >= ncls are padding."""
    rows, stride = logits.shape
    v = logits[:, :ncls].astype(np.float32)
    mx = v.max(1, keepdims=True)
    logz = mx + np.log(np.exp(v - mx).sum(1, keepdims=True, dtype=np.float32))
    lab = labels.astype(np.int64)
    loss = (logz[:, 0] - v[np.arange(rows), lab]).astype(np.float32)
    g = np.exp(v - logz)
    g[np.arange(rows), lab] -= np.float32(1)
    w = np.full(rows, np.float32(1.0) / np.float32(rows)) if weights is None else weights.astype(np.float32)
    dl = np.zeros((rows, stride), np.float32)
    dl[:, :ncls] = g * w[:, None]
    if weights is not None:
        dead = w == 0
        dl[dead] = 0
        loss[dead] = 0
    return loss, round_to(dl, dtype), dl


# --------------------------------------------------------------------------
# Part 2: the whole model
# --------------------------------------------------------------------------

BLOCK_TENSORS = ("ln1.g", "ln1.b", "qkv.W", "qkv.b", "proj.W", "proj.b",
                 "ln2.g", "ln2.b", "fc1.W", "fc1.b", "fc2.W", "fc2.b")


def _ln_fwd(x, g, b):
    mu = x.mean(1, keepdims=True)
    cen = x - mu
    rstd = 1.0 / np.sqrt((cen * cen).mean(1, keepdims=True) + x.dtype.type(1e-5))
    xh = cen * rstd
    return xh * g + b, (xh, rstd)


def _ln_bwd(dy, saved, g):
    xh, rstd = saved
    dxh = dy * g
    dx = rstd * (dxh - dxh.mean(1, keepdims=True) - xh * (dxh * xh).mean(1, keepdims=True))
    return dx, (dy * xh).sum(0), dy.sum(0)


class GPTModel:
    """params: dict with 'tok' (V, D), 'pos' (T, D), 'lnf.g', 'lnf.b', 'head.W' (D, V),
    'head.b' (V,) unless tied, and 'b<i>.<name>' for every name in BLOCK_TENSORS
    (weights stored (in, out) as the reference stores them)."""

    def __init__(self, params, B, T, D, H, n_layer, vocab, pad_vocab, tie=False, ftype=np.float64):
        self.P = {k: np.asarray(v, ftype) for k, v in params.items()}
        self.B, self.T, self.D, self.H, self.L = B, T, D, H, n_layer
        self.vocab, self.pad_vocab, self.tie, self.ft = vocab, pad_vocab, tie, ftype

    def loss_and_grads(self, ids, targets, seg=None, weights=None, need_grads=True):
        P, B, T, D, H = self.P, self.B, self.T, self.D, self.H
        hd, rows, ft = D // H, B * T, self.ft
        scale = ft(1.0 / np.sqrt(hd))
        ids = ids.astype(np.int64)
        pos_idx = positions(rows, T, seg)
        # visible[b, q, j]
        visible = np.tril(np.ones((T, T), bool))[None].repeat(B, 0)
        if seg is not None:
            visible &= np.arange(T)[None, None, :] >= seg.astype(np.int64).reshape(B, T, 1)
        visible = visible[:, None]          # broadcast over heads

        def heads(t):
            return t.reshape(B, T, H, hd).transpose(0, 2, 1, 3)

        def unheads(t):
            return t.transpose(0, 2, 1, 3).reshape(rows, D)

        x = P["tok"][ids] + P["pos"][pos_idx]
        tape = []
        for l in range(self.L):
            w = {n: P[f"b{l}.{n}"] for n in BLOCK_TENSORS}
            h1, ln1 = _ln_fwd(x, w["ln1.g"], w["ln1.b"])
            qkv = h1 @ w["qkv.W"] + w["qkv.b"]
            q, k, v = (heads(qkv[:, i * D:(i + 1) * D]) for i in range(3))
            s = np.where(visible, (q @ k.transpose(0, 1, 3, 2)) * scale, -np.inf)
            e = np.exp(s - s.max(-1, keepdims=True))
            p = e / e.sum(-1, keepdims=True)
            ao = unheads(p @ v)
            r1 = x + ao @ w["proj.W"] + w["proj.b"]
            h2, ln2 = _ln_fwd(r1, w["ln2.g"], w["ln2.b"])
            z = h2 @ w["fc1.W"] + w["fc1.b"]
            a = gelu(z)
            x_out = r1 + a @ w["fc2.W"] + w["fc2.b"]
            tape.append(dict(w=w, h1=h1, ln1=ln1, q=q, k=k, v=v, p=p, ao=ao, h2=h2, ln2=ln2, z=z, a=a))
            x = x_out
        hf, lnf = _ln_fwd(x, P["lnf.g"], P["lnf.b"])
        head_w = P["tok"].T if self.tie else P["head.W"]
        logits = hf @ head_w
        if not self.tie:
            logits = logits + P["head.b"]
        v_ = logits[:, :self.vocab]
        mx = v_.max(1, keepdims=True)
        logz = mx + np.log(np.exp(v_ - mx).sum(1, keepdims=True))
        ce = logz[:, 0] - v_[np.arange(rows), targets.astype(np.int64)]
        wrow = np.full(rows, ft(1.0) / rows) if weights is None else weights.astype(ft)
        loss = float((ce * wrow).sum())
        if not need_grads:
            return loss, None, ce

        dlogits = np.zeros_like(logits)
        g = np.exp(v_ - logz)
        g[np.arange(rows), targets.astype(np.int64)] -= 1
        dlogits[:, :self.vocab] = g * wrow[:, None]
        G = {}
        head_grad = hf.T @ dlogits            # (D, V)
        if not self.tie:
            G["head.W"], G["head.b"] = head_grad, dlogits.sum(0)
        d, G["lnf.g"], G["lnf.b"] = _ln_bwd(dlogits @ head_w.T, lnf, P["lnf.g"])
        for l in reversed(range(self.L)):
            c = tape[l]
            w = c["w"]
            gl = {}
            gl["fc2.W"], gl["fc2.b"] = c["a"].T @ d, d.sum(0)
            dz = (d @ w["fc2.W"].T) * dgelu(c["z"])
            gl["fc1.W"], gl["fc1.b"] = c["h2"].T @ dz, dz.sum(0)
            dr1_mlp, gl["ln2.g"], gl["ln2.b"] = _ln_bwd(dz @ w["fc1.W"].T, c["ln2"], w["ln2.g"])
            dr1 = d + dr1_mlp
            gl["proj.W"], gl["proj.b"] = c["ao"].T @ dr1, dr1.sum(0)
            dao = heads(dr1 @ w["proj.W"].T)
            dv = c["p"].transpose(0, 1, 3, 2) @ dao
            dp = dao @ c["v"].transpose(0, 1, 3, 2)
            ds = c["p"] * (dp - (dp * c["p"]).sum(-1, keepdims=True)) * scale
            dq, dk = ds @ c["k"], ds.transpose(0, 1, 3, 2) @ c["q"]
            dqkv = np.concatenate([unheads(dq), unheads(dk), unheads(dv)], axis=1)
            gl["qkv.W"], gl["qkv.b"] = c["h1"].T @ dqkv, dqkv.sum(0)
            dx_attn, gl["ln1.g"], gl["ln1.b"] = _ln_bwd(dqkv @ w["qkv.W"].T, c["ln1"], w["ln1.g"])
            d = dr1 + dx_attn
            for n, val in gl.items():
                G[f"b{l}.{n}"] = val
        G["tok"] = np.zeros_like(P["tok"])
        G["pos"] = np.zeros_like(P["pos"])
        np.add.at(G["tok"], ids, d)
        np.add.at(G["pos"], pos_idx, d)
        if self.tie:
            G["tok"] = G["tok"] + head_grad.T
        return loss, G, ce
