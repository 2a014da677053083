"""CPU-only checks of the C ABI and the host logic: the library loads, exports
every symbol include/mi_gemm.h declares, validates arguments before touching HIP,
and the picker / tuner logic behaves.  No compute runs here.

Error cases mirror the ones the reference can raise from the host
(kernels.py:274-276, 247-248; vk.py:843-844, 878-879, 1184-1185, 586-587;
autograd.py:39-40)."""

import ctypes as C
import os
import re

import pytest

from vkgrad_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return L.load()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mi_gemm.h")).read()
    return sorted(set(re.findall(r"\b(mg_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(lib):
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"libmigemm.so does not export {n}"
        assert n in L.SIGNATURES, f"{n} is declared in the header but not bound"
    assert set(L.SIGNATURES) == set(names)


def test_struct_layouts_match(lib):
    # the library checks struct_size; a mismatch would make every call fail
    ga = L.GemmArgs()
    ga.struct_size = C.sizeof(L.GemmArgs) - 8
    assert lib.mg_gemm_check(C.byref(ga)) == L.MG_ERR_ARG
    assert "struct_size" in L.last_error()
    t = L.Tile()
    assert lib.mg_tile_info(0, C.byref(t)) == L.MG_OK and t.bm > 0 and t.name


def good_args(**kw):
    ga = L.GemmArgs()
    ga.struct_size = C.sizeof(L.GemmArgs)
    ga.layout, ga.dtype, ga.beta = L.MG_NN, L.MG_F16, 0
    ga.m, ga.n, ga.k = 128, 96, 64
    ga.a, ga.b, ga.c = 0x1000, 0x2000, 0x3000
    ga.lda, ga.ldb, ga.ldc = 64, 96, 96
    ga.nbatch, ga.tile = 1, -1
    for k, v in kw.items():
        setattr(ga, k, v)
    return ga


def test_validation_accepts_ragged_shapes(lib):
    assert lib.mg_gemm_check(C.byref(good_args())) == L.MG_OK
    # any positive shape is legal (the reference refuses non-tile-multiples)
    assert lib.mg_gemm_check(C.byref(good_args(m=1, n=7, k=3, lda=3, ldb=7, ldc=7))) == L.MG_OK
    assert lib.mg_gemm_check(C.byref(good_args(m=4097, n=50257, k=768, lda=768, ldb=50257, ldc=50257))) == L.MG_OK


@pytest.mark.parametrize("kw,needle", [
    (dict(layout=3), "layout"), (dict(dtype=2), "dtype"), (dict(beta=2), "beta"),
    (dict(m=0), "positive"), (dict(k=-5), "positive"), (dict(a=None), "NULL"), (dict(c=None), "NULL"),
    (dict(a=0x1001), "2-byte"), (dict(c=0x3002), "4-byte"), (dict(bias=0x4002), "bias"),
    (dict(lda=63), "lda"), (dict(ldb=95), "ldb"), (dict(ldc=95), "ldc"),
    (dict(nbatch=0), "nbatch"), (dict(nbatch=2, sc=0), "overwrite"), (dict(nbatch=2, sc=10), "overlap"),
    (dict(tile=999), "tile"), (dict(split_k=-1), "split_k"), (dict(group_m=-2), "group_m"),
    (dict(m=2 ** 31), "32-bit"), (dict(flags=32), "unknown flags"), (dict(flags=8 | 16), "exclude each other"),
])
def test_validation_rejects(lib, kw, needle):
    assert lib.mg_gemm_check(C.byref(good_args(**kw))) == L.MG_ERR_ARG
    assert needle in L.last_error(), L.last_error()


def test_softmax_grad_epilogue_validation(lib):
    """act = MG_ACT_SOFTMAX_GRAD: needs y16, p16 and rowsub, beta 0, no bias; batches allowed
    (the other fused outputs are not), their stride must keep the batches of y16 and p16 apart."""
    sg = dict(act=L.MG_ACT_SOFTMAX_GRAD, y16=0x5000, ldy=96, p16=0x6000, ldp=96, rowsub=0x7000, scale=0.125)
    assert lib.mg_gemm_check(C.byref(good_args(**sg))) == L.MG_OK
    assert lib.mg_gemm_check(C.byref(good_args(c=None, **sg))) == L.MG_OK          # C is optional
    assert lib.mg_gemm_check(C.byref(good_args(nbatch=3, sa=128 * 64, sb=64 * 96, sc=128 * 96, **sg))) == L.MG_OK
    for bad, needle in ((dict(p16=None), "p16"), (dict(rowsub=None), "rowsub"), (dict(ldp=95), "ldp"),
                        (dict(beta=1), "beta"), (dict(bias=0x4000), "bias"), (dict(z=0x8000, ldz=96), "z and colsum"),
                        (dict(scale=float("nan")), "NaN"), (dict(y16=None), "y16"), (dict(layout=L.MG_TN, lda=128), "NN and NT"),
                        (dict(nbatch=3, sa=128 * 64, sb=64 * 96, sc=128 * 96 - 8, ldc=90, n=90, ldb=90, ldy=96, ldp=96), "overlaps")):
        assert lib.mg_gemm_check(C.byref(good_args(**{**sg, **bad}))) == L.MG_ERR_ARG, bad
        assert needle in L.last_error(), (bad, L.last_error())
    # p16 / rowsub without the activation, and batches with another fused output
    assert lib.mg_gemm_check(C.byref(good_args(p16=0x6000, ldp=96))) == L.MG_ERR_ARG
    assert lib.mg_gemm_check(C.byref(good_args(nbatch=2, sa=128 * 64, sb=64 * 96, sc=128 * 96, y16=0x5000, ldy=96))) == L.MG_ERR_ARG


def test_layout_dependent_leading_dimensions(lib):
    # TN: A is (K, M), so lda >= M; NT: B is (N, K), so ldb >= K
    assert lib.mg_gemm_check(C.byref(good_args(layout=L.MG_TN, lda=128))) == L.MG_OK
    assert lib.mg_gemm_check(C.byref(good_args(layout=L.MG_TN, lda=64))) == L.MG_ERR_ARG
    assert lib.mg_gemm_check(C.byref(good_args(layout=L.MG_NT, ldb=64))) == L.MG_OK
    assert lib.mg_gemm_check(C.byref(good_args(layout=L.MG_NT, ldb=63))) == L.MG_ERR_ARG


def test_null_context_is_an_error_not_a_crash(lib):
    assert lib.mg_gemm(None, C.byref(good_args())) == L.MG_ERR_ARG
    assert lib.mg_sync(None) == L.MG_ERR_ARG
    assert lib.mg_ew_zero(None, 0x1000, 4) == L.MG_ERR_ARG
    assert lib.mg_destroy(None) == L.MG_OK


def test_init_without_gpu_reports_nodevice(lib):
    import subprocess, sys
    # in a subprocess: on a GPU box this would create a context we do not want here
    code = ("import ctypes as C, sys; sys.path.insert(0, %r); from vkgrad_amd import _lib as L; l = L.load(); "
            "c = C.c_void_p(); rc = l.mg_init(0, C.byref(c)); print(rc, L.last_error()); "
            "l.mg_destroy(c) if rc == 0 else None" % ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120).stdout
    rc = int(out.split()[0])
    assert rc in (L.MG_OK, L.MG_ERR_NODEVICE), out
    if rc == L.MG_ERR_NODEVICE:
        assert "no HIP device" in out


def test_tile_table(lib):
    n = lib.mg_tile_count()
    assert n >= 9
    seen = set()
    for i in range(n):
        t = L.Tile()
        assert lib.mg_tile_info(i, C.byref(t)) == L.MG_OK
        assert t.id == i and t.threads == t.waves_m * t.waves_n * 64
        assert t.lds_bytes <= 160 * 1024
        assert 0 <= t.fallback < n
        seen.add(t.name)
        if t.name.startswith((b"mv_", b"ms_")):
            # the skinny-M streaming tiles (mv_: no matrix cores, no LDS; ms_: matrix cores, A in
            # LDS); what they cannot run goes to a register-staged tile
            fb = L.Tile()
            lib.mg_tile_info(t.fallback, C.byref(fb))
            assert (t.lds_bytes == 0) == t.name.startswith(b"mv_") and fb.stages == 0 and fb.fallback == fb.id
            continue
        assert t.bm % (32 * t.waves_m) == 0 and t.bn % (32 * t.waves_n) == 0
        # the fallback chain ends at a register-staged tile of the same BM x BN
        fb, hops = t, 0
        while fb.stages:
            nxt = L.Tile()
            lib.mg_tile_info(fb.fallback, C.byref(nxt))
            assert (nxt.bm, nxt.bn) == (t.bm, t.bn) and nxt.id != fb.id
            fb, hops = nxt, hops + 1
            assert hops <= 3
        assert fb.fallback == fb.id and not fb.persistent
    assert len(seen) == n
    assert lib.mg_tile_info(n, C.byref(L.Tile())) == L.MG_ERR_ARG
    assert lib.mg_tile_fits(0, C.byref(good_args())) == 1
    assert lib.mg_tile_fits(n, C.byref(good_args())) == 0


def tile_name(lib, i):
    t = L.Tile()
    lib.mg_tile_info(i, C.byref(t))
    return t.name.decode()


def pick(lib, cus=256, **kw):
    t, s, g = C.c_int(), C.c_int(), C.c_int()
    assert lib.mg_pick(C.byref(good_args(**kw)), cus, C.byref(t), C.byref(s), C.byref(g)) == L.MG_OK
    info = L.Tile()
    lib.mg_tile_info(t.value, C.byref(info))
    return info, s.value, g.value


def test_picker_properties(lib):
    # a big aligned square problem gets a big tile and no K split
    info, split, gm = pick(lib, m=8192, n=8192, k=8192, lda=8192, ldb=8192, ldc=8192)
    assert info.bm * info.bn >= 128 * 128 and split == 1 and gm >= 1
    # deep-K, small-MN (a dW shape) is cut along K to fill the chip: an explicit split, or a stream-K tile
    info, split, _ = pick(lib, layout=L.MG_TN, m=768, n=768, k=8192, lda=768, ldb=768, ldc=768)
    assert split > 1 or info.persistent == 2
    assert info.persistent == 2 or -(-768 // info.bm) * -(-768 // info.bn) * split >= 64
    # unaligned operands never get a direct-to-LDS tile
    info, _, _ = pick(lib, m=8192, n=768, k=50257, lda=50257, ldb=768, ldc=768)
    assert info.stages == 0
    # an explicit split is honoured, an explicit tile too
    info, split, _ = pick(lib, m=1024, n=1024, k=4096, lda=4096, ldb=1024, ldc=1024, tile=3, split_k=4)
    assert info.id == 3 and split == 4
    # a split never exceeds the number of K blocks
    _, split, _ = pick(lib, m=128, n=96, k=64, tile=3, split_k=50)
    assert split == 1
    # tiny problems still get a plan
    info, split, _ = pick(lib, m=1, n=1, k=1, lda=1, ldb=1, ldc=1)
    assert split == 1
    # many batches of a narrow problem: the batches fill the chip, so no tile is cut along K and
    # a tile four times wider than N is not worth its padding
    info, split, _ = pick(lib, m=1024, n=64, k=1024, lda=1024, ldb=64, ldc=64, nbatch=96,
                          sa=1024 * 1024, sb=1024 * 64, sc=1024 * 64)
    assert split == 1 and info.bn <= 128
    # the skinny-M streaming tile runs NT with at most 8 rows over K <= 2048 and hands
    # everything else to its fallback
    mv = next(i for i in range(lib.mg_tile_count()) if tile_name(lib, i).startswith("mv_"))
    info, split, _ = pick(lib, layout=L.MG_NT, m=3, n=50257, k=768, lda=768, ldb=768, ldc=50257, tile=mv)
    assert info.id == mv and split == 1
    for kw in (dict(layout=L.MG_NT, m=9, n=4096, k=768, lda=768, ldb=768, ldc=4096),
               dict(layout=L.MG_NT, m=1, n=4096, k=4096, lda=4096, ldb=4096, ldc=4096),
               dict(layout=L.MG_NT, m=4, n=4096, k=772, lda=772, ldb=772, ldc=4096),
               dict(layout=L.MG_NN, m=4, n=4096, k=768, lda=768, ldb=4096, ldc=4096)):
        info, _, _ = pick(lib, tile=mv, **kw)
        assert not info.name.startswith(b"mv_"), kw


# ---------------------------------------------------------------------------
# Python surface
# ---------------------------------------------------------------------------

class FakeDev:
    name = "fake-mi355x"
    compute_units = 256


def test_matmul_object_surface():
    from vkgrad_amd.kernels import CONFIGS, Matmul
    from vkgrad_amd.vk import VkError
    mm = Matmul(FakeDev(), 8, 2, 8, trans_b=True)       # reference-style (sg, wm, wn): 256 x 128
    assert (mm.bm, mm.bn) == (256, 128) and mm.trans_b and not mm.trans_a
    assert mm.fits(1, 7, 3) and not mm.fits(0, 1, 1)
    assert mm.flops(2, 3, 4) == 48
    assert mm.traffic_bytes(4, 8, 16) == 2 * (4 * 16 + 16 * 8) + 4 * 4 * 8
    assert "tb" in mm.name
    with pytest.raises(VkError):
        Matmul(FakeDev(), trans_a=True, trans_b=True)
    with pytest.raises(VkError):
        Matmul(FakeDev(), acc16=True)
    with pytest.raises(VkError):
        Matmul(FakeDev(), dtype="f32")
    with pytest.raises(VkError):
        Matmul(FakeDev(), tile=len(CONFIGS))


def test_pick_config_restatement():
    from vkgrad_amd.autograd import pick_config
    from vkgrad_amd.kernels import CONFIGS
    t = CONFIGS[pick_config(8192, 8192, 8192)]
    assert t["bm"] * t["bn"] == max(c["bm"] * c["bn"] for c in CONFIGS)
    small = CONFIGS[pick_config(64, 64, 64)]
    assert small["bm"] * small["bn"] <= 64 * 64      # most workgroups wins when nothing fills the chip


def test_autotuner_logic_with_fake_timer(tmp_path, monkeypatch):
    """Round-robin order, equal-time repeats, best-of-reps, cache reuse
    (kernels.py:433-447, 462-466, 513-521) — against a deterministic fake clock."""
    import vkgrad_amd.kernels as K
    monkeypatch.setattr(K, "_TUNE_CACHE", str(tmp_path / "tune.json"))
    monkeypatch.setattr(K, "_SHIPPED_CACHE", str(tmp_path / "none.json"))
    calls = []
    fast_tile = K.CONFIGS[3]["id"]

    def timer(mm, repeat):
        calls.append((mm.tile, mm.split_k, mm.group_m, repeat, mm.atomic_split))
        per = 1e-4 if mm.tile == fast_tile else 5e-4
        if mm.group_m == 4:
            per *= 0.9
        return per * repeat

    mm, best = K.autotune_matmul(FakeDev(), 1024, 1024, 1024, reps=3, timer=timer)
    assert best["tile_id"] == fast_tile and best["group_m"] == 4 and mm.tile == fast_tile
    assert best["tflops"] > 0 and best["evaluated"] >= 2 and "pruned" in best and best["lds"] is True
    # equal GPU time per candidate: slow candidates get proportionally fewer repeats
    first_stage2 = next(i for i, c in enumerate(calls) if c[2] != 0)
    stage1 = [c for c in calls[:first_stage2 - 1] if c[3] > 1]
    reps_fast = {c[3] for c in stage1 if c[0] == fast_tile}
    reps_slow = {c[3] for c in stage1 if c[0] != fast_tile}
    assert reps_fast and reps_slow and min(reps_fast) == 5 * max(reps_slow)
    # round-robin: no candidate is measured twice in a row within stage one
    timed = [(c[0], c[1], c[4]) for c in stage1]   # a K split is a candidate twice: workspace and atomic
    ncand = len(set(timed))
    assert ncand > 1 and len(timed) == 3 * ncand
    assert timed[:ncand] == timed[ncand:2 * ncand] == timed[2 * ncand:]
    # cached pick is reused without timing anything
    n = len(calls)
    mm2, e = K.autotune_matmul(FakeDev(), 1024, 1024, 1024, timer=timer)
    assert len(calls) == n and mm2.tile == fast_tile and e["tile_id"] == fast_tile
    # a different dtype or layout is a different key
    assert K.tune_key("d", 1, 2, 3, False, True, "bf16") != K.tune_key("d", 1, 2, 3, False, True, "f16")
    assert K.tune_key("d", 1, 2, 3, False, True) != K.tune_key("d", 1, 2, 3, True, False)


def test_plans_tuned_in_context(tmp_path, monkeypatch):
    """kernels.tune_in_context against a deterministic cost: coordinate descent finds plans whose
    merit only shows in the sum (a GEMM that is slower alone but leaves room for its neighbour),
    differences below the noise threshold change nothing, the refinement sweep picks band and
    walk, every kept change is confirmed by a second measurement; a plan tuned in a context is
    found under that context only, and a context without its own plan falls back to the one
    tuned alone."""
    import vkgrad_amd.kernels as K
    monkeypatch.setattr(K, "_TUNE_CACHE", str(tmp_path / "tune.json"))
    monkeypatch.setattr(K, "_SHIPPED_CACHE", str(tmp_path / "none.json"))
    # operand sets of a timing loop: sized by what a launch reads, so that a rotation's reads are twice the cache
    mb = 1 << 20
    assert K.buffer_sets_for(600 * mb) == 1 and K.buffer_sets_for(512 * mb) == 1
    assert K.buffer_sets_for(17 * mb) == 32 and K.buffer_sets_for(1) == 32
    assert K.buffer_sets_for(90 * mb) == 7 and K.buffer_sets_for(268 * mb) == 3 and K.buffer_sets_for(300 * mb) == 3
    assert all(K.buffer_sets_for(r * mb) * r >= 512 for r in (20, 50, 64, 100, 128, 200, 255))
    cands = K.plan_candidates(3072, 768, 8192, K.L.MG_TN)
    assert len(cands) > 20 and cands[0]["split_k"] == 1
    names = {K.CONFIGS[c["tile_id"]]["name"] for c in cands}
    assert "mmq_256x256x64_w2x4_s2" in names and "mmd_128x128x64_w2x2_s2" in names and "mm_64x64x64_w2x2" in names
    assert all(c["split_k"] == 1 or 8192 // (4 * c["config"][2]) >= c["split_k"] for c in cands)
    assert {c["atomic_split"] for c in cands if c["split_k"] > 1} == {False, True}
    assert not any(c["atomic_split"] for c in cands if c["split_k"] == 1)
    big = K.plan_candidates(8192, 50257, 768, K.L.MG_NT)
    assert all(c["split_k"] == 1 for c in big)          # 12 K-blocks: nothing to split
    pp = next(t["id"] for t in K.CONFIGS if t["name"].startswith("mmq_"))
    calls = []

    def measure(assign):
        calls.append({k: dict(v) for k, v in assign.items()})
        t = 10.0
        # the ping-pong tile for "dw" is worth 1.0, but only while "fwd" keeps its first plan
        if assign["dw"]["tile_id"] == pp and assign["dw"]["split_k"] == 2 and assign["fwd"] == slots["fwd"][0]:
            t -= 1.0
        if assign["fwd"]["tile_id"] == pp:
            t -= 0.01                                   # below min_gain: noise
        if assign["dw"]["group_m"] == 4 and assign["dw"]["xcd_rotate"] is True:
            t -= 0.2
        return t

    slots = {"fwd": K.plan_candidates(8192, 3072, 768, K.L.MG_NT), "dw": cands}
    assign, best, log = K.tune_in_context(slots, measure, passes=3, min_gain=0.003)
    assert assign["dw"]["tile_id"] == pp and assign["dw"]["split_k"] == 2
    assert assign["dw"]["group_m"] == 4 and assign["dw"]["xcd_rotate"] is True
    assert assign["fwd"] == slots["fwd"][0] and abs(best - 8.8) < 1e-9
    assert [x[0] for x in log] == ["start", "dw", "dw"]
    # a kept change was measured twice in a row with the same assignment
    i = next(i for i, c in enumerate(calls) if c["dw"]["tile_id"] == pp and c["dw"]["split_k"] == 2)
    assert calls[i] == calls[i + 1]
    # keys: the context is part of the key, and lookup falls back to the plan tuned alone
    k0 = K.tune_key("d", 8, 9, 10, True, False, "bf16")
    k1 = K.tune_key("d", 8, 9, 10, True, False, "bf16", context="gpt2s-dw-stream")
    assert k1 == k0 + "|in:gpt2s-dw-stream"
    K._save_cache({k0: dict(cands[0], tile_id=3), k1: dict(cands[0], tile_id=pp)})
    assert K.lookup_tuned("d", 8, 9, 10, True, False, "bf16")["tile_id"] == 3
    assert K.lookup_tuned("d", 8, 9, 10, True, False, "bf16", context="gpt2s-dw-stream")["tile_id"] == pp
    assert K.lookup_tuned("d", 8, 9, 10, True, False, "bf16", context="another")["tile_id"] == 3
    assert K.lookup_tuned("d", 8, 9, 11, True, False, "bf16", context="gpt2s-dw-stream") is None


def test_graph_state_errors():
    from vkgrad_amd.vk import Graph, VkError
    g = Graph(FakeDev(), "g")
    with pytest.raises(VkError):
        g.submit()                      # submit before finish (vk.py:878-879)
    with pytest.raises(VkError):
        g.finish()                      # nothing recorded
    with pytest.raises(VkError):
        g.record("not callable")
    g._finished = True
    with pytest.raises(VkError):
        g.record(lambda: None)          # record after finish (vk.py:843-844)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(L, "_lib", None)
    monkeypatch.setattr(L, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(OSError, match="build it"):
        L.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "vkgrad_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, f"{f} mentions the oracle"
                assert "_work" not in text


def test_sweep_workloads_match_the_stated_configurations():
    """vkgrad_amd.sweep lists the GEMMs of the other workloads: the d_model-1024 decoder
    has 1164 GEMMs and 139 TFLOP per optimiser step (4 micro-batches, dW with beta = 1 on
    three of them), the square sweep 4 sizes x 3 layouts, the skinny sweep 5 x 3 NT cases
    with bias, the char-LM 5 linears x 3 products."""
    from vkgrad_amd.sweep import algorithmic_bytes, cases_for
    dec = cases_for("decoder")
    assert sum(c["count"] for c in dec) == 1164
    assert abs(sum(2.0 * c["m"] * c["n"] * c["k"] * c["count"] for c in dec) / 1e12 - 138.98) < 0.01
    acc = [c for c in dec if c["accumulate"]]
    assert acc and all(c["layout"] == "TN" for c in acc) and sum(c["count"] for c in acc) == 3 * (24 * 4 + 1)
    head = [c for c in dec if c["name"].startswith("head")]
    assert {tuple(c["pitch"].items()) for c in head} == {(("ldc", 50304),), (("lda", 50304),)}
    sq = cases_for("square")
    assert len(sq) == 12 and {c["layout"] for c in sq} == {"NN", "NT", "TN"} and all(c["dtype"] == "f16" for c in sq)
    sk = cases_for("skinny")
    assert len(sk) == 15 and all(c["bias"] and c["layout"] == "NT" and c["k"] == 768 for c in sk)
    one = next(c for c in sk if (c["m"], c["n"]) == (1, 50257))
    assert algorithmic_bytes(one) == 2 * (768 + 768 * 50257) + 4 * 50257 + 4 * 50257
    assert len(cases_for("charlm")) == 15


def test_documented_ctypes_stub_matches_the_binding():
    """INTEGRATION.md shows a maintainer the ctypes struct to bind mg_gemm_args with; the library
    rejects any other struct_size, so the documented definition must stay the real one."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    start = text.index("class GemmArgs(C.Structure):")
    end = text.index("\n\n", start)
    ns = {"C": C}
    exec(text[start:end], ns)   # the class statement only
    doc = ns["GemmArgs"]
    assert C.sizeof(doc) == C.sizeof(L.GemmArgs)
    assert [f[0] for f in doc._fields_] == [f[0] for f in L.GemmArgs._fields_]
    for name, ctype in L.GemmArgs._fields_:
        assert getattr(doc, name).offset == getattr(L.GemmArgs, name).offset, name
        assert getattr(doc, name).size == getattr(L.GemmArgs, name).size, name
    # and the call the document shows passes validation
    m, n, k = 96, 64, 128
    args = doc(struct_size=C.sizeof(doc), layout=2, dtype=1, beta=1, m=m, n=n, k=k, a=0x1000, lda=m, b=0x2000, ldb=n,
               c=0x3000, ldc=n, nbatch=1, tile=-1)
    lib = L.load()
    assert lib.mg_gemm_check(C.cast(C.byref(args), C.POINTER(L.GemmArgs))) == L.MG_OK, L.last_error()


def test_static_entry_point_validates_before_touching_a_device(lib):
    """mg_gemm_static runs the same argument checks first, so its refusals are testable here."""
    assert lib.mg_gemm_static(0, None, None) == L.MG_ERR_ARG
    ga = good_args(k=-1)
    assert lib.mg_gemm_static(0, None, C.byref(ga)) == L.MG_ERR_ARG and "positive" in L.last_error()
    ga = good_args(flags=L.MG_FLAG_SIDE_STREAM)
    assert lib.mg_gemm_static(0, None, C.byref(ga)) == L.MG_ERR_ARG and "SIDE_STREAM" in L.last_error()


def test_graph_refuses_replay_after_a_buffer_was_destroyed():
    """A finished graph has device addresses baked in; replaying it on freed memory must
    be refused on the host (no device needed: the check precedes the library call)."""
    from vkgrad_amd.vk import Graph, VkError

    class FakeBuf:
        def __init__(self):
            self.ptr, self.size = 0x1000, 64

    class FakeDev:
        _graphs = set()
    g = Graph(FakeDev(), "g")
    b = FakeBuf()
    g.record(lambda: None, [b], name="k")
    g._finished, g._handle = True, object()
    b.ptr = None
    with pytest.raises(VkError, match="destroyed"):
        g.submit()
    with pytest.raises(VkError, match="destroyed"):
        g.enqueue()
    dead = FakeBuf()
    dead.ptr = None
    g2 = Graph(FakeDev(), "g2")
    with pytest.raises(VkError, match="destroyed"):
        g2.record(lambda: None, [dead], name="k")


def _tiles(lib):
    out = []
    for i in range(lib.mg_tile_count()):
        t = L.Tile()
        assert lib.mg_tile_info(i, C.byref(t)) == L.MG_OK
        out.append(dict(id=t.id, name=t.name.decode(), fallback=t.fallback))
    return out


def _count(lib, ga, ws_mb, counters=1 << 18, clear=0, cus=256):
    n = C.c_int(-1)
    assert lib.mg_launch_count(C.byref(ga), cus, int(ws_mb) << 20, counters, clear, C.byref(n)) == L.MG_OK, L.last_error()
    return n.value


def test_atomic_flag_keeps_a_call_off_the_workspace(lib):
    """What include/mi_gemm.h promises concurrent callers: with MG_FLAG_SPLITK_ATOMIC a call
    touches neither partial tiles nor counters.  Counted without a device (mg_launch_count):
    the ping-pong tile with a partial last round records two GEMM launches when it may use the
    workspace (whole rounds unsplit, the rest cut into K slices) and one with the flag; a
    stream-K tile and an explicit split record no counter clear with the flag."""
    pp = next(t["id"] for t in _tiles(lib) if t["name"].startswith("mmq_"))
    sk = next(t["id"] for t in _tiles(lib) if t["name"].startswith("mmk_128"))
    # 50257 x 768 x 8192 TN: 591 tiles of 256 x 256 on 256 CUs, the LM-head dW of the benchmark
    ga = good_args(layout=L.MG_TN, dtype=L.MG_BF16, m=50257, n=768, k=8192, lda=50304, ldb=768, ldc=768, tile=pp, split_k=1)
    assert _count(lib, ga, 256) == 2
    assert _count(lib, ga, 256, clear=1) == 3          # + the clear of the tail's counters
    assert _count(lib, ga, 32, clear=1) == 1           # 81 tiles x 3 slices x 256 KiB do not fit 32 MiB: no cut
    assert _count(lib, ga, 0) == 1
    ga.flags = L.MG_FLAG_SPLITK_ATOMIC
    assert _count(lib, ga, 256, clear=1) == 1
    # explicit split: slices meet in the workspace (clear + GEMM), or add atomically (clear of C + GEMM)
    ga = good_args(layout=L.MG_TN, dtype=L.MG_BF16, m=768, n=768, k=8192, lda=768, ldb=768, ldc=768, tile=pp, split_k=4)
    assert _count(lib, ga, 256, clear=1) == 2 and _count(lib, ga, 256, clear=0) == 1
    ga.flags = L.MG_FLAG_SPLITK_ATOMIC
    assert _count(lib, ga, 256, clear=1) == 2          # zero_c + GEMM, no counter clear
    ga.beta = 1
    assert _count(lib, ga, 256, clear=1) == 1
    # stream-K tile: pieces meet in the workspace unless the flag forbids it
    ga = good_args(layout=L.MG_NN, dtype=L.MG_BF16, m=8192, n=1152, k=2304, lda=2304, ldb=1152, ldc=1152, tile=sk, split_k=1)
    assert _count(lib, ga, 256, clear=1) == 2
    ga.flags = L.MG_FLAG_SPLITK_ATOMIC
    assert _count(lib, ga, 256, clear=1) == 1


def test_ping_pong_tile_is_refused_where_its_lane_offsets_would_overflow(lib):
    """The ping-pong kernel addresses a lane's load as scalar base + 32-bit offset; a row pitch
    that pushes 7 rows (K-contiguous) or 1 row (M/N-contiguous) past 2^32 bytes must fall back."""
    tiles = _tiles(lib)
    pp = next(t for t in tiles if t["name"].startswith("mmq_"))
    def picked(**kw):
        ga = good_args(dtype=L.MG_BF16, tile=pp["id"], split_k=1, **kw)
        t, s, g = C.c_int(), C.c_int(), C.c_int()
        assert lib.mg_pick(C.byref(ga), 256, C.byref(t), C.byref(s), C.byref(g)) == L.MG_OK, L.last_error()
        return t.value
    ok_ld = 300_000_000         # 7 * ld * 2 + 128 < 2^32
    bad_ld = 310_000_000        # >= 2^32
    assert picked(layout=L.MG_NT, m=512, n=512, k=512, lda=ok_ld, ldb=512, ldc=512) == pp["id"]
    assert picked(layout=L.MG_NT, m=512, n=512, k=512, lda=bad_ld, ldb=512, ldc=512) == pp["fallback"]
    assert picked(layout=L.MG_NT, m=512, n=512, k=512, lda=512, ldb=bad_ld, ldc=512) == pp["fallback"]
    # M/N-contiguous operand: one row of pitch
    assert picked(layout=L.MG_TN, m=512, n=512, k=512, lda=2_000_000_000, ldb=512, ldc=512) == pp["id"]
    assert picked(layout=L.MG_TN, m=512, n=512, k=512, lda=2_147_483_400, ldb=512, ldc=512) == pp["fallback"]
