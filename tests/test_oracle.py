"""Pins the oracle without a GPU.

The reference holds no golden data files (its tests regenerate inputs from
seeds), so the oracle is pinned by: the reference's own known-answer case
(test_kernels.py:69-95), an independent C triple loop with float64 accumulation
(oracle/ref_gemm.c), integer inputs where any summation order is exact, algebraic
identities a wrong index or transposed operand would break, the committed golden
vectors under tests/golden/, and for the MLP step finite differences and closed
forms of AdamW and softmax-CE.
"""

import ctypes as C
import os
import subprocess

import numpy as np
import pytest

from oracle import ref_gemm as O
from oracle import ref_mlp as RM

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LAYOUTS = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}


@pytest.fixture(scope="module")
def cref():
    so = os.path.join(ROOT, "oracle", "libref_gemm.so")
    src = os.path.join(ROOT, "oracle", "ref_gemm.c")
    if not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.run(["gcc", "-O2", "-shared", "-fPIC", "-o", so, src], check=True)
    lib = C.CDLL(so)
    lib.ref_gemm_scalar.restype = C.c_int
    lib.ref_gemm_scalar.argtypes = [C.c_int] * 4 + [C.c_int64] * 3 + [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64,
                                                                   C.c_void_p, C.c_int64, C.c_void_p, C.c_int]
    lib.ref_half_to_float.restype = C.c_float
    lib.ref_half_to_float.argtypes = [C.c_uint16]
    lib.ref_bf16_to_float.restype = C.c_float
    lib.ref_bf16_to_float.argtypes = [C.c_uint16]
    return lib


def c_gemm(lib, a, b, m, n, k, ta, tb, dtype, acc64=1, bias=None, c_in=None):
    a16 = np.ascontiguousarray(a).view(np.uint16)
    b16 = np.ascontiguousarray(b).view(np.uint16)
    c = np.zeros((m, n), np.float32) if c_in is None else np.array(c_in, np.float32)
    bias_p = None if bias is None else np.ascontiguousarray(bias, np.float32).ctypes.data
    rc = lib.ref_gemm_scalar(0 if dtype == "f16" else 1, int(ta), int(tb), acc64, m, n, k,
                             a16.ctypes.data, a16.shape[1], b16.ctypes.data, b16.shape[1],
                             c.ctypes.data, n, bias_p, 0 if c_in is None else 1)
    assert rc == 0
    return c


def test_widening_is_exact_for_every_bit_pattern(cref):
    bits = np.arange(65536, dtype=np.uint16)
    f16 = bits.view(np.float16).astype(np.float32)
    bf = O.bf16_bits_to_f32(bits)
    for i in range(0, 65536, 97):
        h = cref.ref_half_to_float(int(bits[i]))
        b = cref.ref_bf16_to_float(int(bits[i]))
        assert (np.isnan(h) and np.isnan(f16[i])) or h == f16[i]
        assert (np.isnan(b) and np.isnan(bf[i])) or b == bf[i]


def test_bf16_rounding_is_nearest_even():
    # halfway cases: 1 + 2^-8 rounds down to even (1.0), 1 + 3*2^-8 rounds up to 1 + 2^-6
    x = np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, -1.0 - 2.0 ** -8], np.float32)
    got = O.bf16_bits_to_f32(O.f32_to_bf16_bits(x))
    assert got.tolist() == [1.0, 1.0 + 2.0 ** -6, 1.0 + 2.0 ** -7, -1.0]
    # every bf16 value survives a round trip; nearest: error never exceeds half an ulp
    bits = np.arange(0, 0x7F80, dtype=np.uint16)
    assert np.array_equal(O.f32_to_bf16_bits(O.bf16_bits_to_f32(bits)), bits)
    r = np.random.default_rng(0).standard_normal(10000).astype(np.float32)
    back = O.bf16_bits_to_f32(O.f32_to_bf16_bits(r))
    assert np.all(np.abs(back - r) <= np.abs(r) * 2.0 ** -8)
    assert O.f32_to_bf16_bits(np.array([np.nan], np.float32))[0] == 0x7FC0


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_ones_exact_closed_form(layout, dtype):
    """test_kernels.py:69-95: K ones sum to exactly K in float32."""
    ta, tb = LAYOUTS[layout]
    m = n = 8
    for k in (1024, 4096):
        a = O.round_to(np.ones((k, m) if ta else (m, k), np.float32), dtype)
        b = O.round_to(np.ones((n, k) if tb else (k, n), np.float32), dtype)
        assert np.all(O.ref_gemm(a, b, ta, tb, dtype) == float(k))


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_integer_inputs_match_c_triple_loop_bit_for_bit(cref, layout, dtype):
    ta, tb = LAYOUTS[layout]
    for (m, n, k) in [(1, 1, 1), (7, 5, 3), (33, 17, 65), (64, 48, 200)]:
        a, b = O.make_operands(m, n, k, ta, tb, dtype, seed=m + k, integer=True)
        rng = np.random.default_rng(9)
        bias = rng.integers(-5, 6, n).astype(np.float32)
        c0 = rng.integers(-5, 6, (m, n)).astype(np.float32)
        got = O.ref_gemm(a, b, ta, tb, dtype, bias, c0)
        for acc64 in (0, 1):
            ref = c_gemm(cref, a, b, m, n, k, ta, tb, dtype, acc64, bias, c0)
            assert np.array_equal(got, ref), (layout, dtype, m, n, k, acc64)


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_random_inputs_match_float64_accumulation(cref, layout, dtype):
    """numpy's float32 sgemm against a correctly rounded float64 sum: the
    difference is float32 accumulation noise, ~sqrt(K) ulp."""
    ta, tb = LAYOUTS[layout]
    m, n, k = 48, 40, 512
    a, b = O.make_operands(m, n, k, ta, tb, dtype, seed=1)
    got = O.ref_gemm(a, b, ta, tb, dtype)
    ref = c_gemm(cref, a, b, m, n, k, ta, tb, dtype, 1)
    assert O.err_fro(got, ref) < 1e-6
    assert O.err_maxrel(got, ref) < 1e-5


def test_layout_identities_and_negative_control():
    """(A B)^T = B^T A^T ties the three layouts together; reading a square
    operand with the wrong layout must not pass."""
    m, n, k = 24, 40, 56
    rng = np.random.default_rng(3)
    a = rng.integers(-3, 4, (m, k)).astype(np.float16)
    b = rng.integers(-3, 4, (k, n)).astype(np.float16)
    nn = O.ref_gemm(a, b, False, False)
    nt = O.ref_gemm(a, np.ascontiguousarray(b.T), False, True)
    tn = O.ref_gemm(np.ascontiguousarray(a.T), b, True, False)
    assert np.array_equal(nn, nt) and np.array_equal(nn, tn)
    # transpose identity: C^T computed as B^T A^T in NN form
    assert np.array_equal(nn.T, O.ref_gemm(np.ascontiguousarray(b.T), np.ascontiguousarray(a.T)))
    sq_a = rng.standard_normal((32, 32)).astype(np.float16)
    sq_b = rng.standard_normal((32, 32)).astype(np.float16)
    assert O.err_fro(O.ref_gemm(sq_a, sq_b, False, False), O.ref_gemm(sq_a, sq_b, False, True)) > 0.5
    with pytest.raises(ValueError):
        O.layout_name(True, True)


def test_linearity_bias_and_accumulate_clauses():
    m, n, k = 16, 24, 32
    a, b = O.make_operands(m, n, k, seed=2, integer=True)
    a2, _ = O.make_operands(m, n, k, seed=5, integer=True)
    base = O.ref_gemm(a, b)
    # linear in A (integers: exact)
    s = (a.astype(np.float32) + a2.astype(np.float32)).astype(np.float16)
    assert np.array_equal(O.ref_gemm(s, b), base + O.ref_gemm(a2, b))
    bias = np.arange(n, dtype=np.float32) - 7
    assert np.array_equal(O.ref_gemm(a, b, bias=bias), base + bias[None, :])
    c0 = np.full((m, n), 3.0, np.float32)
    assert np.array_equal(O.ref_gemm(a, b, c_in=c0), base + 3.0)
    # micro-batch accumulation == one GEMM over the concatenated K (test_accum.py:149-166)
    parts = [O.make_operands(m, n, k, True, False, "bf16", seed=10 + i, integer=True) for i in range(4)]
    acc = O.ref_gemm_accumulate(parts, True, False, "bf16", np.zeros((m, n), np.float32))
    big_a = np.concatenate([p[0] for p in parts], 0)
    big_b = np.concatenate([p[1] for p in parts], 0)
    assert np.array_equal(acc, O.ref_gemm(big_a, big_b, True, False, "bf16"))
    # dirty accumulator stays in the sum
    dirty = np.full((m, n), 5.0, np.float32)
    assert np.array_equal(O.ref_gemm_accumulate(parts, True, False, "bf16", dirty), acc + 5.0)


def test_batched_is_a_loop_over_strides():
    m, n, k, nb = 8, 12, 16, 3
    rng = np.random.default_rng(4)
    a = rng.integers(-3, 4, nb * m * k).astype(np.float16)
    b = rng.integers(-3, 4, nb * k * n).astype(np.float16)
    out = O.ref_gemm_batched(a, b, m, n, k, nb, (m * k, k * n, m * n))
    for z in range(nb):
        ref = a[z * m * k:(z + 1) * m * k].reshape(m, k).astype(np.float32) @ \
            b[z * k * n:(z + 1) * k * n].reshape(k, n).astype(np.float32)
        assert np.array_equal(out[z * m * n:(z + 1) * m * n].reshape(m, n), ref)


def test_golden_vectors():
    """Committed fixtures (tests/golden/make_golden.py wrote them from the
    oracle, then checked them against the C triple loop)."""
    z = np.load(os.path.join(ROOT, "tests", "golden", "gemm_golden.npz"))
    names = sorted({k.rsplit("_", 1)[0] for k in z.files})
    assert len(names) >= 12
    for name in names:
        layout, dtype = name.split("-")[1:3]
        ta, tb = LAYOUTS[layout]
        a, b, c = z[name + "_a"], z[name + "_b"], z[name + "_c"]
        bias = z[name + "_bias"] if name + "_bias" in z.files else None
        c0 = z[name + "_c0"] if name + "_c0" in z.files else None
        if dtype == "f16":
            a, b = a.view(np.float16), b.view(np.float16)
        got = O.ref_gemm(a, b, ta, tb, dtype, bias, c0)
        assert O.err_fro(got, c) < 1e-6, name


# ---------------------------------------------------------------------------
# MLP step
# ---------------------------------------------------------------------------

def _f64_model(sizes, n_cls, pad, act, seed):
    Ws, bs = RM.he_init(list(sizes) + [pad], seed)
    rng = np.random.default_rng(seed + 1)
    bs = [rng.standard_normal(b.shape) * 0.3 for b in bs]
    m = RM.RefMLP(sizes, n_cls, pad, act=act, pure_f32=True, ftype=np.float64)
    m.set_params(Ws, bs)
    return m


@pytest.mark.parametrize("act", ["gelu", "relu"])
def test_mlp_gradients_match_finite_differences(act):
    """Central differences in float64 on every parameter tensor's largest entries."""
    sizes, n_cls, pad, batch = (12, 9, 7), 4, 6, 5
    m = _f64_model(sizes, n_cls, pad, act, seed=3)
    rng = np.random.default_rng(0)
    x = rng.standard_normal((batch, sizes[0]))
    y = rng.integers(0, n_cls, batch)
    _, dW, db = m.loss_and_grads(x, y)
    eps = 1e-6
    for params, grads in ((m.W, dW), (m.b, db)):
        for p, g in zip(params, grads):
            for flat in np.argsort(-np.abs(g).ravel())[:3]:
                i = np.unravel_index(flat, g.shape)
                old = p[i]
                p[i] = old + eps
                lp = m.loss_and_grads(x, y)[0]
                p[i] = old - eps
                lm = m.loss_and_grads(x, y)[0]
                p[i] = old
                fd = (lp - lm) / (2 * eps)
                assert abs(fd - g[i]) < 1e-6 * max(1.0, abs(g[i])), (act, i, fd, g[i])


def test_padded_classes_get_no_gradient_and_rows_sum_to_zero():
    m = _f64_model((6, 5), 3, 8, "gelu", seed=1)
    rng = np.random.default_rng(2)
    x, y = rng.standard_normal((4, 6)), rng.integers(0, 3, 4)
    _, dW, db = m.loss_and_grads(x, y)
    assert np.all(dW[-1][:, 3:] == 0) and np.all(db[-1][3:] == 0)
    assert abs(db[-1][:3].sum()) < 1e-12          # sum over classes of (p - onehot) is 0 per row
    # uniform logits: loss = log(n_classes)
    m0 = RM.RefMLP((6,), 3, 8, pure_f32=True, ftype=np.float64)
    m0.set_params([np.zeros((6, 8))], [np.zeros(8)])
    assert abs(m0.loss_and_grads(x, y)[0] - np.log(3)) < 1e-12


def test_first_adamw_step_closed_form():
    """t=1: m_hat = g, v_hat = g^2, so dw = -lr * (g/(|g|+eps) + wd*w)
    (autograd.py:319-329, kernels.py:832-851); biases get no decay."""
    m = _f64_model((5, 4), 3, 3, "relu", seed=5)
    w0 = [w.copy() for w in m.W]
    b0 = [b.copy() for b in m.b]
    rng = np.random.default_rng(1)
    dW = [rng.standard_normal(w.shape) for w in m.W]
    db = [rng.standard_normal(b.shape) for b in m.b]
    lr, wd, eps = 1e-3, 0.01, 1e-8
    m.adamw_step(dW, db, lr=lr, wd=wd, eps=eps)
    for w, w_old, g in zip(m.W, w0, dW):
        want = w_old - np.float32(lr) * (g / (np.abs(g) + np.float32(eps)) + np.float32(wd) * w_old)
        # float32-rounded beta/bias-correction constants leave ~1e-5 relative slack on a
        # step of size lr; a dropped decay term (~5e-6) or a wrong sign (~2e-3) still fails
        assert np.allclose(w, want, rtol=0, atol=2e-8)
    for b, b_old, g in zip(m.b, b0, db):
        want = b_old - np.float32(lr) * (g / (np.abs(g) + np.float32(eps)))
        assert np.allclose(b, want, rtol=0, atol=2e-8)
    assert m.t == 1


def test_numpy_mlp_learns():
    xs, xf, y = RM.synthetic_batch(32, 64, 8, seed=0)
    Ws, bs = RM.he_init([64, 32, 16], 5)
    m = RM.RefMLP((64, 32), 8, 16, act="gelu")
    m.set_params(Ws, bs)
    losses = [m.train_step(xf, y, lr=3e-3) for _ in range(200)]
    assert losses[-1] < 0.2 * losses[0]
