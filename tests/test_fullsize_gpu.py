"""Parity at the full sizes of the workload configurations, through size-independent properties.

The numpy oracle needs seconds to minutes at these sizes, so the full result is
checked by (a) a random sample of output entries recomputed exactly in float64
from the same rounded operands, (b) linearity / checksum identities that any
indexing mistake breaks: sum over rows of C equals (colsum of op(A)) . op(B),
computed by the oracle on a (1 x K) @ (K x N) problem, and (c) the exactness
class (integer inputs) on a full-size shape.  Tolerances: rel Frobenius <= 1e-3
over the sample, elementwise rtol 1e-2 with the documented absolute floor.
"""

import numpy as np
import pytest

from oracle import ref_gemm as O

pytestmark = pytest.mark.gpu

LAY = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}


def _run(dev, a, b, m, n, k, ta, tb, dtype, **kw):
    from tests.util import run_gemm
    return run_gemm(dev, a, b, m, n, k, ta, tb, dtype, poison=False, **kw)


def _sample_check(got, a, b, m, n, k, ta, tb, dtype, nsample=4000, seed=0):
    rng = np.random.default_rng(seed)
    ii = rng.integers(0, m, nsample)
    jj = rng.integers(0, n, nsample)
    a32 = O.widen(a, dtype)
    b32 = O.widen(b, dtype)
    rows = (a32[:, ii].T if ta else a32[ii, :]).astype(np.float64)       # (s, k)
    cols = (b32[jj, :] if tb else b32[:, jj].T).astype(np.float64)       # (s, k)
    ref = np.einsum("sk,sk->s", rows, cols)
    g = got[ii, jj].astype(np.float64)
    fro = np.linalg.norm(g - ref) / np.linalg.norm(ref)
    atol = 1e-2 * np.sqrt(k) * np.sqrt(np.mean(rows ** 2)) * np.sqrt(np.mean(cols ** 2))
    assert fro <= 1e-3, fro
    assert np.all(np.abs(g - ref) <= atol + 1e-2 * np.abs(ref))
    return fro


def _checksum_check(got, a, b, ta, tb, dtype):
    """1^T C == (1^T op(A)) op(B): column sums of C from a skinny oracle GEMM."""
    a32 = O.widen(a, dtype).astype(np.float64)
    b32 = O.widen(b, dtype).astype(np.float64)
    va = a32.sum(1) if ta else a32.sum(0)                 # (k,)
    ref = (b32 @ va) if tb else (va @ b32)                # (n,)
    g = got.astype(np.float64).sum(0)
    scale = np.abs(ref).max() + 1e-30
    assert np.abs(g - ref).max() / scale < 2e-4


@pytest.mark.parametrize("layout", list(LAY))
@pytest.mark.parametrize("n", [1024, 4096])
def test_square_sweep_sizes(dev, layout, n):
    """The square configuration (seed 7, f16, ~N(0,1)); 8192^3 runs in the benchmark."""
    ta, tb = LAY[layout]
    a, b = O.make_operands(n, n, n, ta, tb, "f16", seed=7)
    got = _run(dev, a, b, n, n, n, ta, tb, "f16")
    _sample_check(got, a, b, n, n, n, ta, tb, "f16")
    _checksum_check(got, a, b, ta, tb, "f16")
    if n == 1024:
        ref = O.ref_gemm(a, b, ta, tb, "f16")
        assert O.err_fro(got, ref) <= 1e-3 and O.elementwise_ok(got, ref, n)


GPT2 = [("qkv", 768, 2304), ("proj", 768, 768), ("fc1", 768, 3072), ("fc2", 3072, 768)]


@pytest.mark.parametrize("name,fin,fout", GPT2)
def test_gpt2_small_linears(dev, name, fin, fout):
    """The GPT-2-small configuration: R=8192, bf16, X~N(0,1), W~N(0,0.02), dY~N(0,1); the
    three GEMMs of each linear with W stored out x in (NT fwd, NN dX, TN dW)."""
    R = 8192
    rng = np.random.default_rng(1)
    x = O.round_to(rng.standard_normal((R, fin), dtype=np.float32), "bf16")
    w = O.round_to(rng.standard_normal((fout, fin), dtype=np.float32) * 0.02, "bf16")
    dy = O.round_to(rng.standard_normal((R, fout), dtype=np.float32), "bf16")
    y = _run(dev, x, w, R, fout, fin, False, True, "bf16")
    _sample_check(y, x, w, R, fout, fin, False, True, "bf16")
    _checksum_check(y, x, w, False, True, "bf16")
    dx = _run(dev, dy, w, R, fin, fout, False, False, "bf16")
    _sample_check(dx, dy, w, R, fin, fout, False, False, "bf16")
    _checksum_check(dx, dy, w, False, False, "bf16")
    dw = _run(dev, dy, x, fout, fin, R, True, False, "bf16")
    _sample_check(dw, dy, x, fout, fin, R, True, False, "bf16")
    _checksum_check(dw, dy, x, True, False, "bf16")
    # full comparison on the smallest output
    if name == "proj":
        ref = O.ref_gemm(dy, x, True, False, "bf16")
        assert O.err_fro(dw, ref) <= 1e-3 and O.elementwise_ok(dw, ref, R)


def test_lm_head_unpadded_vocab(dev):
    """Tied head 768 -> 50257 at 2048 rows (a quarter of the benchmark's rows keeps
    host memory and time small; the vocabulary, the odd leading dimension and the
    unaligned rows of dlogits are the real ones)."""
    R, D, V = 2048, 768, 50257
    rng = np.random.default_rng(1)
    h = O.round_to(rng.standard_normal((R, D), dtype=np.float32), "bf16")
    tok = O.round_to(rng.standard_normal((V, D), dtype=np.float32) * 0.02, "bf16")
    dlog = O.round_to(rng.standard_normal((R, V), dtype=np.float32), "bf16")
    logits = _run(dev, h, tok, R, V, D, False, True, "bf16")
    _sample_check(logits, h, tok, R, V, D, False, True, "bf16")
    _checksum_check(logits, h, tok, False, True, "bf16")
    dh = _run(dev, dlog, tok, R, D, V, False, False, "bf16")
    _sample_check(dh, dlog, tok, R, D, V, False, False, "bf16")
    dtok = _run(dev, dlog, h, V, D, R, True, False, "bf16")
    _sample_check(dtok, dlog, h, V, D, R, True, False, "bf16")
    _checksum_check(dtok, dlog, h, True, False, "bf16")


@pytest.mark.parametrize("m", [1, 7, 63, 129, 4097])
@pytest.mark.parametrize("n", [96, 2304, 50257])
def test_skinny_and_ragged_with_bias(dev, m, n):
    """The skinny configuration: M x 768 x N, NT, f16, fused bias, non-tile-multiples."""
    k = 768
    a, b = O.make_operands(m, n, k, False, True, "f16", seed=3)
    bias = (np.random.default_rng(3).standard_normal(n) * 2 + 1).astype(np.float32)
    got = _run(dev, a, b, m, n, k, False, True, "f16", bias=bias)
    ref = O.ref_gemm(a, b, False, True, "f16", bias)
    assert O.err_fro(got, ref) <= 1e-3
    assert O.elementwise_ok(got, ref, k)


def test_charlm_shapes(dev):
    """The char-LM configuration: d_model 256, vocab 96, 64 x 256 rows."""
    R = 16384
    for fin, fout in [(256, 768), (256, 256), (256, 1024), (1024, 256), (256, 96)]:
        rng = np.random.default_rng(3)
        x = O.round_to(rng.standard_normal((R, fin), dtype=np.float32), "f16")
        w = O.round_to(rng.standard_normal((fin, fout), dtype=np.float32) * 0.05, "f16")   # reference layout in x out
        dy = O.round_to(rng.standard_normal((R, fout), dtype=np.float32), "f16")
        y = _run(dev, x, w, R, fout, fin, False, False, "f16")                  # fwd  (F,F)
        assert O.err_fro(y, O.ref_gemm(x, w)) <= 1e-3
        dw = _run(dev, x, dy, fin, fout, R, True, False, "f16")                 # dW   (T,F)
        assert O.err_fro(dw, O.ref_gemm(x, dy, True, False)) <= 1e-3
        dx = _run(dev, dy, w, R, fin, fout, False, True, "f16")                 # dX   (F,T)
        assert O.err_fro(dx, O.ref_gemm(dy, w, False, True)) <= 1e-3
