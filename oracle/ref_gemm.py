"""numpy restatement of the reference's GEMM oracle.  TEST INFRASTRUCTURE ONLY.

Follows /root/reference/kernels.py:606-610 (``matmul_reference``: operands are
widened to float32 *after* rounding to the storage type, then multiplied in
float32) and the operand conventions of kernels.py:42-43 / test_kernels.py:12-14:

    A is stored (M, K), or (K, M) when trans_a
    B is stored (K, N), or (N, K) when trans_b
    C is (M, N) float32, row-major

Extensions the reference expresses as separate passes, restated here as
epilogue clauses:
    bias   z = acc + bias[col]             kernels.py:742-749 (``bias`` kernel)
    beta=1 c = c_in + acc                  dataparallel.py:54-58 (``grad_add``)
    batch  per-batch loop with element strides  kernels.py:58-62, 98-101, 135

Pinned by (tests/test_oracle.py): the ones-exact closed form of
test_kernels.py:69-95, an independent C triple loop (oracle/ref_gemm.c) that
accumulates in float64, integer-valued inputs where every summation order is
exact, linearity/transposition identities, and a wrong-layout negative control.

bf16 has no numpy dtype; bf16 tensors are uint16 bit patterns throughout.
"""

import numpy as np

LAYOUTS = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}


def layout_name(trans_a, trans_b):
    if trans_a and trans_b:
        raise ValueError("the (T,T) layout is not part of the path")
    return "TN" if trans_a else ("NT" if trans_b else "NN")


# --------------------------------------------------------------------------
# storage-type rounding
# --------------------------------------------------------------------------

def f32_to_bf16_bits(x):
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (uint16)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        rounded = np.where(nan, np.uint16(0x7FC0), rounded)
    return rounded


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_to(x, dtype):
    """Round float32 data to the storage type; returns the stored array
    (float16 array, or uint16 bf16 bit patterns)."""
    if dtype == "f16":
        return np.asarray(x, dtype=np.float32).astype(np.float16)
    if dtype == "bf16":
        return f32_to_bf16_bits(x)
    raise ValueError(f"unknown dtype {dtype!r}")


def widen(stored, dtype):
    """Stored operand -> float32, exactly."""
    if dtype == "f16":
        return np.asarray(stored, dtype=np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_bits_to_f32(stored)
    raise ValueError(f"unknown dtype {dtype!r}")


# --------------------------------------------------------------------------
# the oracle
# --------------------------------------------------------------------------

def matmul_reference(a, b, trans_a=False, trans_b=False):
    """kernels.py:606-610 verbatim in meaning: f16 in, f32 out."""
    a32 = (a.T if trans_a else a).astype(np.float32)
    b32 = (b.T if trans_b else b).astype(np.float32)
    return a32 @ b32


def ref_gemm(a, b, trans_a=False, trans_b=False, dtype="f16", bias=None,
             c_in=None):
    """C = op(A) op(B) [+ bias[col]] [+ c_in], float32.

    a, b are *stored* operands (float16 arrays or uint16 bf16 bits) in the
    reference's storage convention.  The order of the epilogue matches the
    fused kernel: acc, then + bias, then + c_in, each one float32 add.
    """
    a32 = widen(a, dtype)
    b32 = widen(b, dtype)
    a32 = a32.T if trans_a else a32
    b32 = b32.T if trans_b else b32
    c = a32 @ b32
    if bias is not None:
        c = c + np.asarray(bias, np.float32)[None, :]
    if c_in is not None:
        c = np.asarray(c_in, np.float32) + c
    return c.astype(np.float32, copy=False)


def ref_gemm_batched(a_flat, b_flat, m, n, k, nbatch, strides, trans_a=False,
                     trans_b=False, dtype="f16"):
    """Strided-batched form (kernels.py:98-101): batch z reads A at element
    offset z*sa, B at z*sb and writes C at z*sc.  Returns the flat C array of
    (nbatch-1)*sc + m*n floats (unwritten gaps stay zero)."""
    sa, sb, sc = strides
    a_shape = (k, m) if trans_a else (m, k)
    b_shape = (n, k) if trans_b else (k, n)
    out = np.zeros((nbatch - 1) * sc + m * n, np.float32)
    for z in range(nbatch):
        az = a_flat[z * sa: z * sa + m * k].reshape(a_shape)
        bz = b_flat[z * sb: z * sb + k * n].reshape(b_shape)
        out[z * sc: z * sc + m * n] = ref_gemm(az, bz, trans_a, trans_b, dtype).ravel()
    return out


def ref_gemm_accumulate(pairs, trans_a, trans_b, dtype, c0):
    """dW over micro-batches: c = c0; c = c + gemm_i, one float32 add per
    micro-batch (dataparallel.py:54-58 applied after each overwriting GEMM)."""
    c = np.asarray(c0, np.float32).copy()
    for a, b in pairs:
        c = c + ref_gemm(a, b, trans_a, trans_b, dtype)
    return c


# --------------------------------------------------------------------------
# error metrics
# --------------------------------------------------------------------------

def err_maxrel(got, ref):
    """test_kernels.py:35 — max abs error over max abs reference."""
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-6))


def err_fro(got, ref):
    """Relative Frobenius error, in float64."""
    g = np.asarray(got, np.float64)
    r = np.asarray(ref, np.float64)
    return float(np.linalg.norm(g - r) / max(np.linalg.norm(r), 1e-30))


def elementwise_ok(got, ref, k, rtol=1e-2, scale=None):
    """Elementwise |got-ref| <= atol + rtol*|ref|.

    A pure rtol cannot hold for entries that cancel to ~0, so there is an
    absolute floor of rtol * sqrt(K) * rms(a)*rms(b); callers pass that product
    as `scale` (default: the rms of ref / sqrt(K) gives the same thing)."""
    ref = np.asarray(ref, np.float32)
    if scale is None:
        scale = float(np.sqrt(np.mean(np.square(ref, dtype=np.float64)))) / max(np.sqrt(k), 1.0)
    atol = rtol * np.sqrt(max(k, 1)) * scale
    return bool(np.all(np.abs(got - ref) <= atol + rtol * np.abs(ref)))


# --------------------------------------------------------------------------
# synthetic inputs
# --------------------------------------------------------------------------

def make_operands(m, n, k, trans_a=False, trans_b=False, dtype="f16", seed=0,
                  scale_a=1.0, scale_b=1.0, integer=False):
    """Operands drawn the way test_kernels.py:10-16 draws them
    (default_rng(seed), standard_normal, A first then B), rounded to dtype.
    integer=True draws small integers instead so that every accumulation order
    is exact in float32."""
    rng = np.random.default_rng(seed)
    a_shape = (k, m) if trans_a else (m, k)
    b_shape = (n, k) if trans_b else (k, n)
    if integer:
        a = rng.integers(-4, 5, a_shape).astype(np.float32)
        b = rng.integers(-4, 5, b_shape).astype(np.float32)
    else:
        a = (rng.standard_normal(a_shape) * scale_a).astype(np.float32)
        b = (rng.standard_normal(b_shape) * scale_b).astype(np.float32)
    return round_to(a, dtype), round_to(b, dtype)
