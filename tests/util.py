"""Shared helpers for the parity tests: run one GEMM through the library's
Python surface (which goes through the C ABI) and build the oracle's answer."""

import numpy as np

from oracle import ref_gemm as O


def stored_shapes(m, n, k, trans_a, trans_b):
    return ((k, m) if trans_a else (m, k)), ((n, k) if trans_b else (k, n))


def np16(dtype):
    return np.float16 if dtype == "f16" else np.uint16


def pad_pitch(x, ld, fill):
    """Copy of 2-D x with its rows spread to a pitch of ld elements (padding = fill)."""
    out = np.full((x.shape[0], ld), fill, dtype=x.dtype)
    out[:, :x.shape[1]] = x
    return out


def run_gemm(dev, a, b, m, n, k, trans_a=False, trans_b=False, dtype="f16", bias=None,
             c_in=None, tile=None, split_k=0, group_m=0, kind="device", poison=True,
             lda=None, ldb=None, ldc=None, xcd_rotate=None):
    """a, b: stored operands (f16 arrays or bf16 bit patterns).  Returns C (m,n) f32.
    lda/ldb: upload the operand with that row pitch; the padding holds NaN so that
    anything read from it and used shows.  ldc: C has that row pitch; its padding
    holds a sentinel that must come back untouched."""
    from vkgrad_amd.kernels import Matmul
    nan16 = np.float16(np.nan) if dtype == "f16" else np.uint16(0x7FC0)
    if lda is not None:
        a = pad_pitch(a, lda, nan16)
    if ldb is not None:
        b = pad_pitch(b, ldb, nan16)
    ba = dev.buffer(max(a.nbytes, 2), kind)
    bb = dev.buffer(max(b.nbytes, 2), kind)
    pc = n if ldc is None else ldc
    bc = dev.buffer(m * pc * 4, kind)
    bbias = None
    SENT = np.float32(-12345.5)
    mm = Matmul(dev, trans_a=trans_a, trans_b=trans_b, tile=tile, dtype=dtype, split_k=split_k,
                group_m=group_m, xcd_rotate=xcd_rotate)
    try:
        ba.upload(a)
        bb.upload(b)
        if c_in is not None:
            bc.upload(pad_pitch(np.ascontiguousarray(c_in, np.float32), pc, SENT))
        elif poison:
            bc.upload(pad_pitch(np.full((m, n), np.nan, np.float32), pc, SENT))   # beta=0 must overwrite
        if bias is not None:
            bbias = dev.buffer(n * 4, kind)
            bbias.upload(np.ascontiguousarray(bias, np.float32))
        mm(ba, bb, bc, m, n, k, bias=bbias, accumulate=c_in is not None, lda=lda, ldb=ldb, ldc=ldc)
        full = bc.download(np.float32, (m, pc))
        if pc != n and (c_in is not None or poison):
            assert np.all(full[:, n:] == SENT), "the padding between rows of C was written"
        return np.ascontiguousarray(full[:, :n])
    finally:
        mm.destroy()
        for x in (ba, bb, bc, bbias):
            if x is not None:
                x.destroy()


def check_case(dev, m, n, k, trans_a=False, trans_b=False, dtype="f16", seed=0, bias=False,
               accumulate=False, tile=None, split_k=0, integer=False, group_m=0, lda=None, ldb=None, ldc=None,
               xcd_rotate=None):
    """Run one seeded case and compare with the oracle.  Returns metrics dict."""
    a, b = O.make_operands(m, n, k, trans_a, trans_b, dtype, seed, integer=integer)
    rng = np.random.default_rng(seed + 1000)
    if integer:
        bias_v = rng.integers(-8, 9, n).astype(np.float32) if bias else None
        c_in = rng.integers(-8, 9, (m, n)).astype(np.float32) if accumulate else None
    else:
        # per-column-distinct, non-zero biases: a skipped bias add must show
        bias_v = (rng.standard_normal(n) * 3 + np.arange(n) % 7 + 1).astype(np.float32) if bias else None
        c_in = rng.standard_normal((m, n)).astype(np.float32) * 5 if accumulate else None
    got = run_gemm(dev, a, b, m, n, k, trans_a, trans_b, dtype, bias_v, c_in, tile, split_k, group_m,
                   lda=lda, ldb=ldb, ldc=ldc, xcd_rotate=xcd_rotate)
    ref = O.ref_gemm(a, b, trans_a, trans_b, dtype, bias_v, c_in)
    out = dict(maxrel=O.err_maxrel(got, ref), fro=O.err_fro(got, ref),
               exact=bool(np.array_equal(got, ref)), finite=bool(np.isfinite(got).all()),
               elem_ok=O.elementwise_ok(got, ref, k))
    return out, got, ref
