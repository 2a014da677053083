"""Parity of the plans that are timed, at the shapes they are timed on.

The benchmark and the sweeps do not run the library's picker: they take (tile, K split,
rasterisation band, split mode) from the shipped tuned table.  These tests build every GEMM
through the same functions (bench.plan_for, kernels.tuned_matmul) and check it against the
oracle at full size:

  * every GEMM of the benchmark step (the GPT-2-small configuration) with the benchmark's operand
    statistics and the LM head's padded logits pitch: sampled exact recomputation in float64
    plus the column-checksum identity (tests/test_fullsize_gpu.py explains both);
  * every entry of the tuned table at the shape, layout, dtype, pitches and batch count it is
    keyed on, with small-integer operands, where the float32 result is exact in any summation
    order, compared bit for bit with the oracle over the whole output;
  * the d_model-1024 decoder of configs[3]: forward and dX of all five linears at 16384 rows,
    and dW accumulated with beta = 1 over 4 micro-batches;
  * the square sizes of configs[1] the other tests leave out (2048, 8192);
  * the tuner itself on the device (reference: test_kernels.py:103-118 - tune, then check the
    winner is correct).
"""

import json
import os
import re
import zlib

import numpy as np
import pytest

from oracle import ref_gemm as O
from tests.test_fullsize_gpu import _checksum_check, _sample_check

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LAY = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}
VOCAB = 50257


def _int16bits(rng, shape, dtype, lo=-2, hi=3):
    """Small integers as 16-bit operands (exact in f16 and bf16), drawn as int8 to keep the
    host cost of multi-gigabyte operands low."""
    v = rng.integers(lo, hi, shape, dtype=np.int8)
    table = O.round_to(np.arange(lo, hi, dtype=np.float32), dtype)
    return table[v - lo]


def _normal16(rng, shape, dtype, scale=1.0):
    return O.round_to(rng.standard_normal(shape, dtype=np.float32) * np.float32(scale), dtype)


def _stored(m, n, k, ta, tb):
    return ((k, m) if ta else (m, k)), ((n, k) if tb else (k, n))


def _run_mm(dev, mm, a, b, m, n, k, lda=None, ldb=None, ldc=None, c_in=None, nbatch=1, sentinel=True):
    """One call of a prepared Matmul on host operands; returns C (nbatch, m, n) f32 (batch axis
    dropped for nbatch == 1).  Operands are uploaded with the requested pitches, padding filled
    with NaN so that anything read from it and used shows; C's padding must come back untouched."""
    from tests.util import pad_pitch
    nan16 = np.float16(np.nan) if mm.dtype == "f16" else np.uint16(0x7FC0)
    pa = a.shape[-1] if lda is None else lda
    pb = b.shape[-1] if ldb is None else ldb
    pc = n if ldc is None else ldc
    if nbatch == 1:
        a, b = a[None], b[None]
    au = np.stack([pad_pitch(x, pa, nan16) for x in a]) if pa != a.shape[-1] else a
    bu = np.stack([pad_pitch(x, pb, nan16) for x in b]) if pb != b.shape[-1] else b
    SENT = np.float32(-12345.5)
    ba, bb = dev.buffer(au.nbytes, "device"), dev.buffer(bu.nbytes, "device")
    bc = dev.buffer(nbatch * m * pc * 4, "device")
    try:
        ba.upload(au)
        bb.upload(bu)
        if c_in is not None:
            cin = np.ascontiguousarray(c_in, np.float32).reshape(nbatch, m, n)
            bc.upload(np.stack([pad_pitch(x, pc, SENT) for x in cin]))
        elif sentinel and pc != n:
            bc.upload(np.full((nbatch, m, pc), SENT, np.float32))
        strides = (au.shape[1] * pa, bu.shape[1] * pb, m * pc)
        kw = dict(nbatch=nbatch, strides=strides) if mm.batched else {}
        mm(ba, bb, bc, m, n, k, accumulate=c_in is not None, lda=lda, ldb=ldb, ldc=ldc, **kw)
        full = bc.download(np.float32, (nbatch, m, pc))
        if pc != n and (sentinel or c_in is not None):
            assert np.all(full[:, :, n:] == SENT), "the padding between rows of C was written"
        got = np.ascontiguousarray(full[:, :, :n])
        return got[0] if nbatch == 1 else got
    finally:
        for x in (ba, bb, bc):
            x.destroy()


# ---------------------------------------------------------------------------
# the benchmark step, plan for plan
# ---------------------------------------------------------------------------

def _bench_cases():
    """Every GEMM of the benchmark step with the plan chosen alone (the in-order schedule and
    the fallback of every other) and with the plan chosen inside the step of the default
    schedule, and the three LM-head GEMMs once more with logits rows exactly 50257 elements
    apart (the step bench.py reports as `dense_head`)."""
    import bench
    cases = [(name, layout, m, n, k, False, None) for name, layout, m, n, k, _ in bench.gemm_list()]
    ctx = bench.context_of("dw-stream")
    return (cases + [c[:6] + (ctx,) for c in cases] +
            [c[:5] + (True, x) for c in cases if c[0].startswith("head") for x in (None, ctx)])


@pytest.mark.parametrize("name,layout,m,n,k,dense,context", _bench_cases(),
                         ids=[c[0] + (".dense" if c[5] else "") + ("@" + c[6] if c[6] else "") for c in _bench_cases()])
def test_benchmark_plan_at_full_size(dev, name, layout, m, n, k, dense, context):
    import bench
    vpitch = bench.head_pitch(dense)
    mm, kw = bench.plan_for(dev, name, layout, m, n, k, vpitch, context)
    assert (kw == {}) == (dense or not name.startswith("head"))
    if os.path.exists(os.path.join(ROOT, "vkgrad_amd", "tuned_mi355x.json")) and dev.name.startswith("gfx950"):
        assert mm.tile >= 0, f"{name}: the tuned table has no plan for this shape (the benchmark would run the picker)"
    ta, tb = LAY[layout]
    rng = np.random.default_rng(zlib.crc32(name.encode()) % 1000 + 1)
    sa, sb = _stored(m, n, k, ta, tb)
    # operand statistics of bench.py: activations and upstream gradients ~N(0,1), weights ~N(0,0.02)
    role = name.split(".")[1]
    a = _normal16(rng, sa, "bf16", 1.0)
    b = _normal16(rng, sb, "bf16", 0.02 if role in ("fwd", "dX") else 1.0)
    got = _run_mm(dev, mm, a, b, m, n, k, **kw)
    assert np.isfinite(got).all()
    _sample_check(got, a, b, m, n, k, ta, tb, "bf16")
    _checksum_check(got, a, b, ta, tb, "bf16")
    mm.destroy()


# ---------------------------------------------------------------------------
# every entry of the shipped table, exact on integer operands
# ---------------------------------------------------------------------------

_KEY = re.compile(r"^(?P<dev>.*)\|(?P<m>\d+)x(?P<n>\d+)x(?P<k>\d+)\|ta(?P<ta>[01])tb(?P<tb>[01])\|(?P<dt>f16|bf16)"
                  r"(?P<acc>\|acc)?(?:\|bat(?P<bat>\d+))?(?:\|ld(?P<lda>\d+),(?P<ldb>\d+),(?P<ldc>\d+))?"
                  r"(?:\|in:(?P<ctx>[\w-]+))?$")


def _table():
    with open(os.path.join(ROOT, "vkgrad_amd", "tuned_mi355x.json")) as f:
        return json.load(f)


def _table_ids():
    return [k.split("|", 1)[1] for k in _table()]


@pytest.mark.parametrize("key", list(_table()), ids=_table_ids())
def test_tuned_table_entry_is_exact_at_its_shape(dev, key):
    from vkgrad_amd.kernels import matmul_from_entry
    e = _table()[key]
    g = _KEY.match(key)
    assert g, f"unparsable tuned-table key {key!r}"
    m, n, k = int(g["m"]), int(g["n"]), int(g["k"])
    ta, tb, dtype = g["ta"] == "1", g["tb"] == "1", g["dt"]
    nbatch = int(g["bat"]) if g["bat"] else 1
    pitch = {x: int(g[x]) for x in ("lda", "ldb", "ldc")} if g["lda"] else {}
    # a pitch equal to the default says nothing
    dflt = dict(lda=m if ta else k, ldb=k if tb else n, ldc=n)
    pitch = {x: v for x, v in pitch.items() if v != dflt[x]}
    mm = matmul_from_entry(dev, e, ta, tb, dtype, nbatch > 1)
    rng = np.random.default_rng(len(key) * 7919 + m + 3 * n + 5 * k)
    sa, sb = _stored(m, n, k, ta, tb)
    if nbatch > 1:
        sa, sb = (nbatch,) + sa, (nbatch,) + sb
    a = _int16bits(rng, sa, dtype)
    b = _int16bits(rng, sb, dtype)
    c_in = rng.integers(-8, 9, (nbatch, m, n)).astype(np.float32) if g["acc"] else None
    got = _run_mm(dev, mm, a, b, m, n, k, c_in=c_in, nbatch=nbatch, **pitch)
    if nbatch > 1:
        ref = np.stack([O.ref_gemm(a[i], b[i], ta, tb, dtype, None, None if c_in is None else c_in[i])
                        for i in range(nbatch)])
    else:
        ref = O.ref_gemm(a, b, ta, tb, dtype, None, None if c_in is None else c_in[0])
    assert got.shape == ref.shape
    if not np.array_equal(got, ref):
        bad = np.argwhere(got != ref)
        raise AssertionError(f"{key}: {len(bad)} of {got.size} entries differ, first at {bad[0].tolist()}: "
                             f"{got[tuple(bad[0])]} != {ref[tuple(bad[0])]}")
    mm.destroy()


# ---------------------------------------------------------------------------
# configs[3]: d_model 1024, 16384 rows, dW accumulated over 4 micro-batches
# ---------------------------------------------------------------------------

DECODER = [("qkv", 1024, 3072), ("proj", 1024, 1024), ("fc1", 1024, 4096), ("fc2", 4096, 1024), ("head", 1024, VOCAB)]


@pytest.mark.parametrize("name,fin,fout", DECODER, ids=[d[0] for d in DECODER])
def test_decoder_1024_forward_and_dx(dev, name, fin, fout):
    """Forward (NT) and dX (NN) of one linear at 16384 rows, bf16, random operands (seed 2),
    built like the decoder sweep builds them (tuned plan, padded logits pitch for the head)."""
    from vkgrad_amd.kernels import tuned_matmul
    R = 16384
    vp = (VOCAB + 63) // 64 * 64 if name == "head" else None
    rng = np.random.default_rng(2)
    x = _normal16(rng, (R, fin), "bf16")
    w = _normal16(rng, (fout, fin), "bf16", 0.02)
    yp = {} if vp is None else {"ldc": vp}
    mm, how = tuned_matmul(dev, R, fout, fin, False, True, "bf16", **yp)
    assert how == "tuned table", f"{name}.fwd is not in the tuned table"
    y = _run_mm(dev, mm, x, w, R, fout, fin, **yp)
    _sample_check(y, x, w, R, fout, fin, False, True, "bf16")
    _checksum_check(y, x, w, False, True, "bf16")
    del y
    dy = _normal16(rng, (R, fout), "bf16")
    dp = {} if vp is None else {"lda": vp}
    mm2, how = tuned_matmul(dev, R, fin, fout, False, False, "bf16", **dp)
    assert how == "tuned table", f"{name}.dX is not in the tuned table"
    dx = _run_mm(dev, mm2, dy, w, R, fin, fout, **dp)
    _sample_check(dx, dy, w, R, fin, fout, False, False, "bf16")
    _checksum_check(dx, dy, w, False, False, "bf16")
    mm.destroy()
    mm2.destroy()


@pytest.mark.parametrize("name,fin,fout", DECODER, ids=[d[0] for d in DECODER])
def test_decoder_1024_dw_over_four_micro_batches(dev, name, fin, fout):
    """dW = dY^T X (TN) at 16384 rows: the first micro-batch overwrites a poisoned gradient with
    the beta = 0 plan, the other three add with the beta = 1 plan (the two have different table
    entries); integer operands, so the f32 sum is exact whatever the order."""
    from tests.util import pad_pitch
    from vkgrad_amd.kernels import tuned_matmul
    R = 16384
    vp = (VOCAB + 63) // 64 * 64 if name == "head" else None
    dp = {} if vp is None else {"lda": vp}
    mm0, how0 = tuned_matmul(dev, fout, fin, R, True, False, "bf16", accumulate=False, **dp)
    mm1, how1 = tuned_matmul(dev, fout, fin, R, True, False, "bf16", accumulate=True, **dp)
    assert how0 == how1 == "tuned table", f"{name}.dW is not in the tuned table"
    rng = np.random.default_rng(2)
    nan16 = np.uint16(0x7FC0)
    bg = dev.buffer(fout * fin * 4, "device")
    bg.upload(np.full((fout, fin), np.nan, np.float32))
    ref = np.zeros((fout, fin), np.float32)
    bx, bdy = dev.buffer(R * fin * 2, "device"), dev.buffer(R * (vp or fout) * 2, "device")
    for i in range(4):
        dy = _int16bits(rng, (R, fout), "bf16")
        x = _int16bits(rng, (R, fin), "bf16")
        bdy.upload(dy if vp is None else pad_pitch(dy, vp, nan16))
        bx.upload(x)
        (mm0 if i == 0 else mm1)(bdy, bx, bg, fout, fin, R, accumulate=(i > 0), **dp)
        ref += O.ref_gemm(dy, x, True, False, "bf16")
        del dy, x
    got = bg.download(np.float32, (fout, fin))
    assert np.array_equal(got, ref)
    for x in (bg, bx, bdy):
        x.destroy()
    mm0.destroy()
    mm1.destroy()


# ---------------------------------------------------------------------------
# configs[1]: the square sizes the other tests leave out
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("layout", list(LAY))
@pytest.mark.parametrize("n", [2048, 8192])
def test_square_sweep_with_tuned_plans(dev, layout, n):
    """Seed 7, f16, ~N(0,1) as bench/matmul_sweep.py:36-53; the plan is the table's."""
    from vkgrad_amd.kernels import tuned_matmul
    ta, tb = LAY[layout]
    mm, how = tuned_matmul(dev, n, n, n, ta, tb, "f16")
    assert how == "tuned table"
    a, b = O.make_operands(n, n, n, ta, tb, "f16", seed=7)
    got = _run_mm(dev, mm, a, b, n, n, n)
    _sample_check(got, a, b, n, n, n, ta, tb, "f16")
    _checksum_check(got, a, b, ta, tb, "f16")
    mm.destroy()


# ---------------------------------------------------------------------------
# the tuner on the device
# ---------------------------------------------------------------------------

def _check_tuned(dev, mm, best, m, n, k, ta, tb, dtype, nbatch=1):
    assert best["tflops"] > 0 and best["ms"] > 0
    assert best["evaluated"] >= 2, "the tuner timed fewer than two candidates"
    assert len(best["tile"]) == 2 and len(best["config"]) == 3
    assert mm.tile == best["tile_id"] and mm.split_k == best["split_k"] and mm.group_m == best["group_m"]
    sa, sb = _stored(m, n, k, ta, tb)
    if nbatch > 1:
        sa, sb = (nbatch,) + sa, (nbatch,) + sb
    rng = np.random.default_rng(0)
    a = _normal16(rng, sa, dtype)
    b = _normal16(rng, sb, dtype)
    got = _run_mm(dev, mm, a, b, m, n, k, nbatch=nbatch)
    if nbatch == 1:
        ref = O.ref_gemm(a, b, ta, tb, dtype)
    else:
        ref = np.stack([O.ref_gemm(a[i], b[i], ta, tb, dtype) for i in range(nbatch)])
    # the reference's bound for a tuned winner (test_kernels.py:113-116) and this build's own
    assert O.err_maxrel(got, ref) < 2e-3
    assert O.err_fro(got, ref) <= 1e-3
    assert O.elementwise_ok(got, ref, k)


def test_autotune_on_device_then_check_the_winner(dev):
    """reference test_kernels.py:103-118: tune 512^3 without the cache, then run the winner
    against the oracle ("a tuned config that is fast and wrong is worse than useless",
    bench/matmul_sweep.py:36-57)."""
    from vkgrad_amd.kernels import autotune_matmul
    mm, best = autotune_matmul(dev, 512, 512, 512, use_cache=False, reps=2)
    try:
        _check_tuned(dev, mm, best, 512, 512, 512, False, False, "f16")
    finally:
        mm.destroy()


def test_autotune_ragged_split_k_shape(dev):
    """A short, fat dW-like shape (TN, bf16, ragged M and N): the candidate list holds K splits
    in both modes (workspace and atomic), which the real timer path has to run."""
    from vkgrad_amd.kernels import autotune_matmul
    m, n, k = 200, 328, 4104
    mm, best = autotune_matmul(dev, m, n, k, trans_a=True, use_cache=False, reps=2, dtype="bf16")
    try:
        _check_tuned(dev, mm, best, m, n, k, True, False, "bf16")
    finally:
        mm.destroy()


def test_autotune_batched_shape_and_cache_roundtrip(dev, tmp_path, monkeypatch):
    """A strided-batched attention-like shape, with the cache: the second call must come back
    from the file without timing anything (kernels.py:462-466), with the same plan."""
    from vkgrad_amd import kernels as K
    monkeypatch.setattr(K, "_TUNE_CACHE", str(tmp_path / "tune.json"))
    m, n, k, nb = 256, 256, 64, 12
    mm, best = K.autotune_matmul(dev, m, n, k, trans_b=True, batched=True, nbatch=nb, reps=2, dtype="bf16")
    try:
        _check_tuned(dev, mm, best, m, n, k, False, True, "bf16", nbatch=nb)
        assert os.path.exists(K._TUNE_CACHE)
        calls = []
        mm2, best2 = K.autotune_matmul(dev, m, n, k, trans_b=True, batched=True, nbatch=nb, dtype="bf16",
                                       timer=lambda *a: calls.append(1) or 1.0)
        assert not calls, "a cached shape was timed again"
        assert (mm2.tile, mm2.split_k, mm2.group_m) == (mm.tile, mm.split_k, mm.group_m)
        mm2.destroy()
    finally:
        mm.destroy()


# ---------------------------------------------------------------------------
# Kernel resource statistics (Kernel.statistics, /root/reference/vk.py:690-736; occupancy,
# /root/reference/kernels.py:384-411): no instantiation spills, and each tile holds the
# workgroups per CU its design and the picker's cost model assume.
# ---------------------------------------------------------------------------

# workgroups per CU by tile name: two for the four-wave tiles whose ring takes at most half the
# LDS, one for the 256 x 256 tiles and the register-staged tiles with more than half the LDS
_WGS_PER_CU = {
    "mm_256x256x32_w2x4": 1, "mm_256x128x64_w2x2": 1, "mm_128x256x64_w2x2": 1, "mm_128x128x64_w2x2": 2,
    "mm_64x256x64_w1x4": 1, "mm_32x256x64_w1x4": 1, "mm_256x64x64_w4x1": 1, "mm_256x32x64_w4x1": 1,
    "mmd_256x256x32_w2x4_s4": 1, "mmd_256x256x64_w2x4_s2": 1, "mmd_128x128x64_w2x2_s2": 2,
    "mmd_128x256x32_w2x2_s3": 2, "mmd_256x128x32_w2x2_s3": 2, "mmd_128x128x32_w2x2_s3": 2,
    "mmp_256x256x64_w2x4_s2": 1, "mmp_256x256x32_w2x4_s4": 1, "mmp_128x128x64_w2x2_s2": 2,
    "mmk_256x256x64_w2x4_s2": 1, "mmk_128x128x64_w2x2_s2": 2, "mmq_256x256x64_w2x4_s2": 1,
}


def test_no_instantiation_spills_and_occupancy_is_as_designed(dev):
    from vkgrad_amd import kernels as K
    seen = 0
    for t in K.CONFIGS:
        skinny = t["name"].startswith(("mv_", "ms_"))
        for layout in (K.L.MG_NN, K.L.MG_NT, K.L.MG_TN):
            for dtype in ("f16", "bf16"):
                for variant in (range(16) if skinny else range(3)):
                    st = K.tile_statistics(dev, t["id"], layout, dtype, variant)
                    if st is None:
                        continue
                    seen += 1
                    what = (t["name"], layout, dtype, variant, st)
                    assert st["scratchMemUsageInBytes"] == 0, what
                    assert 0 < st["numUsedVgprs"] <= 512, what
                    assert st["workgroupsPerCU"] >= 1, what
                    if skinny:
                        continue
                    assert st["workgroupThreads"] == t["threads"], what
                    assert st["ldsUsageSizeInBytes"] <= 160 * 1024, what
                    if t["name"] in _WGS_PER_CU:
                        assert st["workgroupsPerCU"] == _WGS_PER_CU[t["name"]], what
                    else:
                        assert t["name"] == "mm_64x64x64_w2x2" and st["workgroupsPerCU"] >= 3, what
                    occ, reason = K.occupancy(dev, st)
                    assert reason is None and occ == st["wavesPerSimd"], what
    # 23 tiles x 3 layouts x 2 dtypes, most with two or three variants
    assert seen > 250


def test_statistics_of_a_planned_gemm_and_tuner_fields(dev):
    """Matmul.statistics names the kernel the call would launch; the tuner records vgpr and
    occupancy with its pick as the reference does (kernels.py:527-529)."""
    from vkgrad_amd.kernels import Matmul, autotune_matmul, CONFIGS
    mm = Matmul(dev, trans_b=True, dtype="bf16", tile=21)
    st = mm.statistics(8192, 3072, 768)
    assert CONFIGS[st["tile_id"]]["name"] == "mmq_256x256x64_w2x4_s2"
    assert st["workgroupThreads"] == 512 and st["ldsUsageSizeInBytes"] == 131072 and st["workgroupsPerCU"] == 1
    # unaligned operands: the plan falls back to the register-staged 256 x 256 tile
    st = mm.statistics(8192, 3072, 770, lda=771, ldb=771)
    assert CONFIGS[st["tile_id"]]["name"] == "mm_256x256x32_w2x4" and st["scratchMemUsageInBytes"] == 0
    mm.destroy()
    mm, best = autotune_matmul(dev, 512, 512, 512, reps=1, use_cache=False, dtype="bf16")
    assert best["vgpr"] and best["vgpr"] <= 512 and best["occupancy"] >= 1 and best["spilling"] == []
    mm.destroy()
