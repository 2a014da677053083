"""GPU parity: the HIP GEMM path against the oracle, through the C ABI.

Cases and tolerances follow the reference's own kernel tests
(/root/reference/test_kernels.py:10-95: five NN shapes and the two transposes at
256^3 with max-abs/max-abs < 2e-3, and the ones-exact K=1024 case), tightened to
the bar of this build: relative Frobenius error <= 1e-3 and elementwise
rtol 1e-2 (with the absolute floor oracle.ref_gemm.elementwise_ok documents).
Integer-valued inputs must match bit for bit in every accumulation order.
"""

import numpy as np
import pytest

from oracle import ref_gemm as O
from tests.util import check_case, run_gemm

pytestmark = pytest.mark.gpu

LAYOUTS = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}
FRO_TOL = 1e-3
MAXREL_TOL = 2e-3   # test_kernels.py:36


def _assert_close(r, label):
    assert r["finite"], f"{label}: non-finite output"
    assert r["fro"] <= FRO_TOL, f"{label}: rel Frobenius {r['fro']:.3e}"
    assert r["maxrel"] < MAXREL_TOL, f"{label}: max rel {r['maxrel']:.3e}"
    assert r["elem_ok"], f"{label}: elementwise rtol 1e-2 violated"


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (128, 128, 128), (512, 256, 128),
                                    (256, 512, 256), (64, 64, 512)])
def test_reference_shapes_nn(dev, m, n, k):
    """test_kernels.py:48-59."""
    r, _, _ = check_case(dev, m, n, k, seed=0)
    _assert_close(r, f"NN {m}x{n}x{k}")


@pytest.mark.parametrize("layout", ["TN", "NT"])
def test_reference_transposes(dev, layout):
    """test_kernels.py:62-66."""
    ta, tb = LAYOUTS[layout]
    r, _, _ = check_case(dev, 256, 256, 256, ta, tb, seed=0)
    _assert_close(r, f"{layout} 256^3")


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_ones_exact(dev, layout, dtype):
    """test_kernels.py:69-95: K=1024 products of 1.0 sum to exactly 1024.0 only
    with float32 accumulation."""
    ta, tb = LAYOUTS[layout]
    m = n = 64
    k = 1024
    one = np.float16(1.0) if dtype == "f16" else np.uint16(0x3F80)
    a = np.full((k, m) if ta else (m, k), one)
    b = np.full((n, k) if tb else (k, n), one)
    got = run_gemm(dev, a, b, m, n, k, ta, tb, dtype)
    assert np.all(got == float(k)), f"min {got.min()} max {got.max()}"


def test_every_tile_every_layout_exact(dev):
    """Integer inputs: exact in any summation order, so every tile, layout and
    dtype must reproduce the oracle bit for bit on a ragged shape."""
    from vkgrad_amd.kernels import CONFIGS
    m, n, k = 300, 520, 200
    for layout, (ta, tb) in LAYOUTS.items():
        for dtype in ("f16", "bf16"):
            for t in CONFIGS:
                r, got, ref = check_case(dev, m, n, k, ta, tb, dtype, seed=3, tile=t["id"], integer=True,
                                         bias=True, accumulate=True)
                assert r["exact"], f"{layout} {dtype} tile {t['name']}: max diff {np.abs(got - ref).max()}"


def test_direct_to_lds_tiles_exact(dev):
    """Aligned shapes that keep the direct-to-LDS kernels eligible (K a multiple
    of every BK, extents multiples of 8 but not of the tile, so edge clamping
    runs), every tile x layout x dtype, with bias, beta=1 and a K split."""
    from vkgrad_amd.kernels import CONFIGS
    m, n, k = 392, 648, 512
    for layout, (ta, tb) in LAYOUTS.items():
        for dtype in ("f16", "bf16"):
            for t in CONFIGS:
                if not t["stages"]:
                    continue
                for split in (1, 2):
                    r, got, ref = check_case(dev, m, n, k, ta, tb, dtype, seed=13, tile=t["id"], integer=True,
                                             bias=True, accumulate=True, split_k=split)
                    assert r["exact"], (f"{layout} {dtype} tile {t['name']} split {split}: "
                                        f"max diff {np.abs(got - ref).max()}")


def test_direct_to_lds_ragged_k_and_edges_with_padded_pitch(dev):
    """K not a multiple of BK (nor of 8) and ragged M/N, with row pitches padded to
    a multiple of 8: the direct-to-LDS kernels stay eligible, multiply the K
    remainder first through registers, and must never use what they read from
    the padding (it holds NaN)."""
    from vkgrad_amd.kernels import CONFIGS, Matmul
    for m, n, k in [(264, 392, 150), (200, 136, 1001), (129, 257, 77)]:
        for layout, (ta, tb) in LAYOUTS.items():
            a_cols = m if ta else k
            b_cols = k if tb else n
            lda, ldb = (a_cols + 7) // 8 * 8 + 8, (b_cols + 7) // 8 * 8
            for t in CONFIGS:
                if not t["stages"]:
                    continue
                mm = Matmul(dev, trans_a=ta, trans_b=tb, tile=t["id"])
                for split in (1, 2):
                    r, got, ref = check_case(dev, m, n, k, ta, tb, "bf16", seed=21, tile=t["id"], integer=True,
                                             bias=True, split_k=split, lda=lda, ldb=ldb)
                    assert r["exact"], (f"{layout} {m}x{n}x{k} tile {t['name']} split {split}: "
                                        f"max diff {np.abs(got - ref).max()}")


def test_tight_buffers_fall_back(dev):
    """Unpadded buffers whose extents are not multiples of 8 must not be served by
    a kernel that reads row padding: same answer through the any-alignment path."""
    from vkgrad_amd.kernels import CONFIGS
    dma = next(t for t in CONFIGS if t["stages"] and not t["persistent"])
    r, got, ref = check_case(dev, 264, 392, 1001, False, True, "f16", seed=5, tile=dma["id"], integer=True)
    assert r["exact"]


def test_direct_to_lds_plan_is_used(dev):
    """The picker must keep a direct-to-LDS tile when its preconditions hold and
    fall back to the register-staged sibling when they do not."""
    from vkgrad_amd.kernels import CONFIGS, Matmul
    dma = next(t for t in CONFIGS if t["stages"] and not t["persistent"])
    mm = Matmul(dev, trans_b=True, tile=dma["id"])
    assert mm.plan(512, 512, 512)[0] == dma["id"]
    assert mm.plan(512, 512, 504)[0] == dma["id"]            # ragged K, pitch still a multiple of 8
    assert mm.plan(512, 512, 500)[0] == dma["fallback"]      # pitch 500 breaks 16-byte row alignment
    per = next(t for t in CONFIGS if t["persistent"])
    mp = Matmul(dev, trans_b=True, tile=per["id"])
    assert mp.plan(512, 512, 512)[0] == per["id"]
    assert mp.plan(512, 512, 504)[0] == per["fallback"]      # persistent tiles need whole K blocks


@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_ragged_small_exact(dev, layout):
    """Odd shapes (unaligned rows, K tails of every residue) through the
    general-alignment kernels, bit exact on integer data."""
    ta, tb = LAYOUTS[layout]
    for m, n, k in [(1, 1, 1), (7, 5, 3), (33, 31, 17), (63, 96, 129), (129, 65, 67), (100, 257, 250),
                    (31, 33, 1025)]:
        r, got, ref = check_case(dev, m, n, k, ta, tb, "f16", seed=m + n + k, integer=True, bias=True)
        assert r["exact"], f"{layout} {m}x{n}x{k}: max diff {np.abs(got - ref).max()}"


@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_split_k_exact_and_close(dev, layout):
    ta, tb = LAYOUTS[layout]
    for split in (2, 3, 8):
        r, got, ref = check_case(dev, 192, 320, 2048, ta, tb, "bf16", seed=5, integer=True, split_k=split,
                                 bias=True, accumulate=True, tile=3)
        assert r["exact"], f"{layout} split {split}: max diff {np.abs(got - ref).max()}"
        r, _, _ = check_case(dev, 192, 320, 2048, ta, tb, "bf16", seed=6, split_k=split, tile=3)
        _assert_close(r, f"{layout} split {split}")


def test_beta0_overwrites_nan(dev):
    """dW with beta=0 doubles as the zeroing of a stale gradient
    (transformer.py:367-370): a NaN-poisoned C must come back clean."""
    for split in (1, 4):
        r, _, _ = check_case(dev, 256, 256, 1024, True, False, "f16", seed=2, split_k=split)
        _assert_close(r, f"TN poisoned split {split}")


@pytest.mark.parametrize("tile", [3, 11, 17])
def test_split_k_clear_respects_pitch_and_tails(dev, tile):
    """beta=0 with a K split clears C first: with a padded row pitch (aligned and
    not), an odd width, and a poisoned C, the result is exact and the padding
    between rows keeps its contents."""
    for n, ldc in [(320, 320), (317, 328), (317, 321), (5, 5), (1027, 1032)]:
        r, got, ref = check_case(dev, 200, n, 1024, True, False, "f16", seed=n, integer=True, split_k=4,
                                 tile=tile, ldc=ldc)
        assert r["exact"], f"tile {tile} n {n} ldc {ldc}: max diff {np.abs(got - ref).max()}"


@pytest.mark.parametrize("tile", [0, 10, 15, 17, 21])
def test_split_k_is_bit_reproducible(dev, tile):
    """The K slices meet in a workspace and are summed in slice order by whichever
    slice arrives last, so random data gives the same bits on every run."""
    outs = []
    for _ in range(3):
        r, got, _ = check_case(dev, 512, 512, 4096, True, False, "bf16", seed=77, split_k=8, tile=tile, bias=True,
                               accumulate=True)
        _assert_close(r, f"tile {tile}")
        outs.append(got)
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_split_k_without_workspace_adds_atomically(monkeypatch):
    """With the workspace switched off the slices add into C with atomics (after a
    clear when beta = 0): exact on integers, within tolerance on random data."""
    from vkgrad_amd.vk import Device
    monkeypatch.setenv("MIGEMM_SPLITK_WORKSPACE_MB", "0")
    d = Device()
    try:
        for tile in (3, 11, 17):
            r, got, ref = check_case(d, 200, 317, 1024, True, False, "f16", seed=3, integer=True, split_k=4,
                                     tile=tile, ldc=328)
            assert r["exact"], f"tile {tile}: max diff {np.abs(got - ref).max()}"
            r, _, _ = check_case(d, 192, 320, 2048, False, True, "bf16", seed=6, split_k=3, tile=tile, bias=True,
                                 accumulate=True)
            _assert_close(r, f"tile {tile}")
    finally:
        d.destroy()


@pytest.mark.parametrize("layout", list(LAYOUTS))
def test_stream_k_tiles_exact(dev, layout):
    """Stream-K tiles: the tiles beyond the last whole round of the resident grid are cut
    along K into one run per workgroup and the pieces meet in the workspace.  Shapes with
    more tiles than slots (a remainder after whole rounds), fewer tiles than slots (all
    pieces), ragged edges, bias and beta = 1; bit exact on integer data and bit identical
    from run to run on random data."""
    from vkgrad_amd.kernels import CONFIGS
    ta, tb = LAYOUTS[layout]
    sk = [t for t in CONFIGS if t["persistent"] == 2]
    assert len(sk) >= 2
    for t in sk:
        big = 3000 if t["bm"] == 128 else 4400          # 576 tiles on 512 slots / 324 on 256
        for m, n, k in [(big, big, 512), (1000, 1016, 1024), (392, 648, 2048), (128, 128, 4096)]:
            r, got, ref = check_case(dev, m, n, k, ta, tb, "bf16", seed=m + k, integer=True, tile=t["id"], bias=True,
                                     accumulate=True)
            assert r["exact"], f"{t['name']} {layout} {m}x{n}x{k}: max diff {np.abs(got - ref).max()}"
        r, got, ref = check_case(dev, 1000, 1016, 1024, ta, tb, "f16", seed=9, tile=t["id"])
        _assert_close(r, f"{t['name']} {layout}")
        r2, got2, _ = check_case(dev, 1000, 1016, 1024, ta, tb, "f16", seed=9, tile=t["id"])
        assert np.array_equal(got, got2)


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_skinny_stream_tile_exact(dev, dtype):
    """The skinny-M streaming tile (NT, M <= 8, K <= 2048, no matrix cores): every row
    count 1..8, K of one to four 512-element chunks with ragged ends (and the 513..768 class,
    whose last chunk pairs of rows share), N from one row to more than the resident wavefronts
    take at once, bias, beta = 1, a padded pitch of C; bit exact on integer data,
    within tolerance on random data; and the plan must really be that tile."""
    from vkgrad_amd.kernels import CONFIGS, Matmul
    mv = next(t for t in CONFIGS if t["name"].startswith("mv_"))
    mp = Matmul(dev, trans_b=True, dtype=dtype, tile=mv["id"])
    cases = [(1, 50257, 768), (4, 2304, 768), (3, 1000, 1024), (3, 96, 768), (2, 777, 2048), (4, 129, 8),
             (1, 1, 8), (4, 4097, 520), (4, 63, 1536), (1, 17, 2048), (2, 64, 512), (2, 65, 1032), (4, 300, 2048),
             (7, 50257, 768), (8, 2304, 768), (5, 96, 768), (6, 100003, 264), (8, 33000, 2048), (7, 31, 1024),
             (3, 45, 648), (8, 77, 760), (1, 130, 768), (2, 5, 528)]
    for i, (m, n, k) in enumerate(cases):
        assert mp.plan(m, n, k)[0] == mv["id"], (m, n, k)
        r, got, ref = check_case(dev, m, n, k, False, True, dtype, seed=m + n + k, integer=True, tile=mv["id"],
                                 bias=bool(i & 1), accumulate=bool(i & 2), ldc=(n + 5 if i % 3 == 0 else None))
        assert r["exact"], f"{m}x{n}x{k}: max diff {np.abs(got - ref).max()}"
    for m, n, k in [(1, 50257, 768), (4, 3000, 1024)]:
        r, got, ref = check_case(dev, m, n, k, False, True, dtype, seed=3, tile=mv["id"], bias=True)
        _assert_close(r, f"mv {m}x{n}x{k}")
    # what it cannot run goes to its fallback and is still right
    r, got, ref = check_case(dev, 9, 300, 768, False, True, dtype, seed=1, integer=True, tile=mv["id"])
    assert r["exact"]
    r, got, ref = check_case(dev, 4, 300, 768, False, False, dtype, seed=1, integer=True, tile=mv["id"])
    assert r["exact"]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_skinny_matrix_core_tile_exact(dev, dtype):
    """The skinny-M tile on the matrix cores (NT, M <= 64, A whole in LDS, every wavefront
    streaming 32 rows of B through its own LDS buffer): row counts around the 32-row blocks,
    K of one 8-element piece up to what fits LDS with ragged ends (K not a multiple of the
    64-element phase, nor of 16), N from one column to more than a round of workgroups,
    padded pitches of A, B and C with NaN / sentinel padding, bias, beta = 1; bit exact on
    integer data, within tolerance on random data; the plan must really be that tile, and
    what it cannot run goes to its fallback."""
    from vkgrad_amd.kernels import CONFIGS, Matmul
    ms = next(t for t in CONFIGS if t["name"].startswith("ms_"))
    mp = Matmul(dev, trans_b=True, dtype=dtype, tile=ms["id"])
    cases = [(5, 50257, 768), (7, 50257, 768), (8, 2304, 768), (9, 96, 768), (31, 4097, 768), (32, 1000, 1024),
             (33, 777, 520), (63, 50257, 768), (64, 2304, 768), (64, 300, 960), (1, 1, 8), (17, 129, 8), (20, 127, 24),
             (32, 128, 2176), (12, 257, 2048), (40, 255, 72), (64, 33, 136), (6, 100003, 264), (48, 513, 648)]
    for i, (m, n, k) in enumerate(cases):
        assert mp.plan(m, n, k)[0] == ms["id"], (m, n, k)
        r, got, ref = check_case(dev, m, n, k, False, True, dtype, seed=m + n + k, integer=True, tile=ms["id"],
                                 bias=bool(i & 1), accumulate=bool(i & 2), ldc=(n + 5 if i % 3 == 0 else None),
                                 lda=(k + 8 if i % 4 == 1 else None), ldb=(k + 16 if i % 5 == 2 else None))
        assert r["exact"], f"{m}x{n}x{k}: max diff {np.abs(got - ref).max()}"
    for m, n, k in [(7, 50257, 768), (63, 3000, 768), (24, 2000, 1536)]:
        r, got, ref = check_case(dev, m, n, k, False, True, dtype, seed=3, tile=ms["id"], bias=True)
        _assert_close(r, f"ms {m}x{n}x{k}")
    # what it cannot run goes to its fallback and is still right: too many rows, A too large for
    # LDS, K not in whole 8-element pieces, another layout
    for m, n, k, ta, tb in [(65, 300, 768, False, True), (64, 300, 1024, False, True), (33, 200, 2048, False, True),
                            (16, 300, 516, False, True), (16, 304, 768, False, False)]:
        assert mp.plan(m, n, k)[0] != ms["id"] or (ta, tb) != (False, True), (m, n, k)
        r, got, ref = check_case(dev, m, n, k, ta, tb, dtype, seed=1, integer=True, tile=ms["id"])
        assert r["exact"], (m, n, k)
    mp.destroy()


@pytest.mark.parametrize("tile", [3, 4, 11, 13, 21])
def test_xcd_major_order_and_rotated_walk_cover_every_tile(dev, tile):
    """The tiled kernels renumber workgroups XCD-major - XCD x takes the x-th eighth of the
    tile order, the first (tiles % 8) XCDs one tile more - and with MG_FLAG_XCD_ROTATE each XCD
    starts elsewhere in its share.  Either way every output tile must be computed exactly once:
    tile counts with every remainder modulo 8, fewer tiles than XCDs, bands that do not divide
    the rows, with and without a K split (which keeps the renumbering only for whole eights),
    on integer data where a tile computed twice or not at all cannot hide (beta = 1 doubles the
    first, NaN poison shows the second)."""
    from vkgrad_amd.kernels import CONFIGS
    t = CONFIGS[tile]
    bm, bn = t["bm"], t["bn"]
    grids = [(1, 1), (3, 1), (2, 4), (3, 3), (5, 2), (11, 1), (3, 4), (13, 1), (7, 2), (5, 3), (4, 4), (17, 1),
             (3, 6), (19, 1), (5, 4), (7, 3), (11, 2), (23, 1), (6, 4), (9, 5), (8, 8)]
    for i, (gm, gn) in enumerate(grids):
        m, n = gm * bm - (i % 3) * 8, gn * bn - (i % 2) * 8
        for rot in (False, True):
            for split, acc in ((0, False), (1, True), (2, False)):
                k = 256 if split != 2 else 512
                r, got, ref = check_case(dev, m, n, k, i % 3 == 2, i % 3 == 1, "bf16", seed=i, integer=True,
                                         tile=tile, split_k=split, group_m=(0, 1, 3, 4)[i % 4], accumulate=acc,
                                         xcd_rotate=rot)
                assert r["exact"], (tile, gm, gn, rot, split, float(np.abs(got - ref).max()))


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("layout", ["NN", "NT"])
def test_fused_activation_output(dev, layout, dtype):
    """Forward epilogue with the activated 16-bit output (the reference's separate
    bias_gelu / bias pass, kernels.py:709-718, 742-749, folded into the GEMM):
    C holds z = A.B + bias exactly (integer data), y16 = narrow(act(z)) - bit exact for
    none and ReLU, within two 16-bit ulps of the numpy GELU (the device tanh differs in the
    last bits); tiles with and without a fused variant, a K split through the workspace,
    ragged and padded shapes, C omitted, and the misuse cases."""
    from oracle import ref_mlp as R
    from vkgrad_amd.kernels import CONFIGS, Matmul
    from vkgrad_amd.vk import VkError
    ta, tb = LAYOUTS[layout]
    np16 = np.float16 if dtype == "f16" else np.uint16
    cases = [(200, 136, 320, None, 0, "gelu"), (512, 384, 256, 11, 0, "relu"), (1000, 1016, 1024, 10, 0, "gelu"),
             (392, 648, 2048, 11, 4, None), (129, 96, 768, 4, 3, "relu"), (300, 200, 264, 15, 0, "gelu"),
             (64, 50, 72, 20, 0, "relu"), (520, 776, 1024, 21, 0, "gelu"), (512, 264, 2048, 21, 3, "relu")]
    for m, n, k, tile, split, act in cases:
        a, b = O.make_operands(m, n, k, ta, tb, dtype, seed=m + k, integer=True)
        bias = (np.arange(n) % 9 - 4).astype(np.float32) * 0.5
        z_ref = O.ref_gemm(a, b, ta, tb, dtype, bias, None)
        y_ref = O.round_to(R.act_fn(z_ref, act) if act else z_ref, dtype)
        ldy = n + 6
        ba, bb, bz = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(n * 4, "device")
        bc, by = dev.buffer(m * n * 4, "device"), dev.buffer(m * ldy * 2, "device")
        ba.upload(a); bb.upload(b); bz.upload(bias)
        mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype, tile=tile, split_k=split)
        try:
            for with_c in (True, False):
                bc.upload(np.full((m, n), np.nan, np.float32))
                by.upload(np.full((m, ldy), 0x7e01, np.uint16))
                mm(ba, bb, bc if with_c else None, m, n, k, bias=bz, act=act, y16=by, ldy=ldy)
                if with_c:
                    assert np.array_equal(bc.download(np.float32, (m, n)), z_ref), (m, n, k, tile, "z")
                yfull = by.download(np.uint16, (m, ldy))
                assert np.all(yfull[:, n:] == 0x7e01), "the padding between rows of y16 was written"
                got = np.ascontiguousarray(yfull[:, :n]).view(np16) if dtype == "f16" else np.ascontiguousarray(yfull[:, :n])
                if act == "gelu":
                    g32, w32 = O.widen(got, dtype), O.widen(y_ref, dtype)
                    assert np.all(np.abs(g32 - w32) <= 2 * np.maximum(np.abs(w32), 2.0 ** -14) * 2.0 ** (-10 if dtype == "f16" else -7)), \
                        (m, n, k, tile, np.abs(g32 - w32).max())
                else:
                    assert np.array_equal(got.view(np.uint16), y_ref.view(np.uint16)), (m, n, k, tile, act)
        finally:
            mm.destroy()
            for x in (ba, bb, bz, bc, by):
                x.destroy()
    # misuse
    mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype)
    buf = dev.buffer(64 * 64 * 4, "device")
    try:
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, act="gelu")                  # activation without y16
        with pytest.raises(VkError):
            mm(buf, buf, None, 64, 64, 64)                             # nothing to write
        with pytest.raises(VkError):
            mm(buf, buf, None, 64, 64, 64, y16=buf, accumulate=True)   # beta = 1 needs C
    finally:
        mm.destroy()
        buf.destroy()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("layout", ["NN", "NT"])
def test_fused_activation_gradient_output(dev, layout, dtype):
    """Backward epilogue (the reference's separate bias_gelu_bwd pass, kernels.py:720-739,
    folded into the dX GEMM that feeds it, autograd.py:204-207, 224-227): with integer
    operands the product is exact, so C and y16 must equal product * act'(z) - bit exact for
    ReLU (the factor is 0 or 1), within 1e-5 of the product's magnitude (f32) and two 16-bit
    ulps for GELU, whose derivative the device forms from one exponential; z has its own
    pitch, padding of y16 stays untouched, C may be omitted, tiles with and without a fused
    variant and a K split through the workspace.  colsum (the reference's col_sum pass,
    kernels.py:753-761, in the same epilogue) receives the column sums of that result on top
    of what it held: exact for ReLU, where every term is an integer."""
    from oracle import ref_mlp as R
    from vkgrad_amd.kernels import Matmul
    from vkgrad_amd.vk import VkError
    ta, tb = LAYOUTS[layout]
    np16 = np.float16 if dtype == "f16" else np.uint16
    cases = [(200, 136, 320, None, 0, "gelu"), (512, 384, 256, 11, 0, "relu"), (1000, 1016, 1024, 10, 0, "gelu"),
             (392, 648, 2048, 11, 4, "relu"), (129, 96, 768, 4, 3, "gelu"), (300, 200, 264, 15, 0, "relu"),
             (64, 50, 72, 3, 0, "gelu")]
    for m, n, k, tile, split, act in cases:
        a, b = O.make_operands(m, n, k, ta, tb, dtype, seed=m + k, integer=True)
        prod = O.ref_gemm(a, b, ta, tb, dtype, None, None)
        ldz, ldy = n + 3, n + 6
        rng = np.random.default_rng(m * 7 + n)
        z = np.zeros((m, ldz), np.float32)
        z[:, :n] = rng.standard_normal((m, n)).astype(np.float32) * 2.0
        z[:, n:] = np.nan
        g_ref = (prod.astype(np.float64) * R.dact_fn(z[:, :n].astype(np.float64), act)).astype(np.float32)
        ba, bb, bz = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(z.nbytes, "device")
        bc, by = dev.buffer(m * n * 4, "device"), dev.buffer(m * ldy * 2, "device")
        bs = dev.buffer(n * 4 + 8, "device")
        ba.upload(a); bb.upload(b); bz.upload(z)
        s0 = np.concatenate([(np.arange(n) % 5 - 2).astype(np.float32), [np.float32(77.0), np.float32(78.0)]])
        mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype, tile=tile, split_k=split)
        try:
            for with_c in (True, False):
                bc.upload(np.full((m, n), np.nan, np.float32))
                by.upload(np.full((m, ldy), 0x7e01, np.uint16))
                bs.upload(s0)
                mm(ba, bb, bc if with_c else None, m, n, k, act=act + "_grad", y16=by, ldy=ldy, z=bz, ldz=ldz,
                   colsum=bs if with_c else None)
                sums = bs.download(np.float32, (n + 2,))
                assert sums[n] == 77.0 and sums[n + 1] == 78.0, "wrote beyond N column sums"
                if not with_c:
                    assert np.array_equal(sums, s0), "column sums written although none were asked for"
                elif act == "relu":
                    # integers: exact in any order of addition
                    assert np.array_equal(sums[:n], s0[:n] + g_ref.astype(np.float64).sum(0)), (m, n, k, tile, "colsum")
                else:
                    want = s0[:n] + g_ref.astype(np.float64).sum(0)
                    bound = 1e-5 * np.maximum(np.abs(prod), 1.0).sum(0) + 1e-6 * np.abs(g_ref).sum(0)
                    assert np.all(np.abs(sums[:n] - want) <= bound), (m, n, k, tile, np.abs(sums[:n] - want).max())
                yfull = by.download(np.uint16, (m, ldy))
                assert np.all(yfull[:, n:] == 0x7e01), "the padding between rows of y16 was written"
                got16 = np.ascontiguousarray(yfull[:, :n])
                if dtype == "f16":
                    got16 = got16.view(np16)
                if act == "relu":
                    if with_c:
                        assert np.array_equal(bc.download(np.float32, (m, n)), g_ref), (m, n, k, tile, "dz32")
                    assert np.array_equal(got16.view(np.uint16), O.round_to(g_ref, dtype).view(np.uint16)), (m, n, k, tile)
                else:
                    tol = 1e-5 * np.maximum(np.abs(prod), 1.0)
                    if with_c:
                        got = bc.download(np.float32, (m, n))
                        assert np.all(np.abs(got - g_ref) <= tol), (m, n, k, tile, np.abs(got - g_ref).max())
                    g32 = O.widen(got16, dtype)
                    ulp = np.maximum(np.abs(g_ref), 2.0 ** -14) * 2.0 ** (-10 if dtype == "f16" else -7)
                    assert np.all(np.abs(g32 - g_ref) <= 2 * ulp + tol), (m, n, k, tile, np.abs(g32 - g_ref).max())
        finally:
            mm.destroy()
            for x in (ba, bb, bz, bc, by, bs):
                x.destroy()
    # misuse
    mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype)
    buf = dev.buffer(64 * 64 * 4, "device")
    try:
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, act="gelu_grad", y16=buf)                          # no z
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, act="relu", y16=buf, colsum=buf)                   # column sums of a forward GEMM
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, act="gelu", y16=buf, z=buf)                        # z without a _grad activation
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, act="relu_grad", y16=buf, z=buf, bias=buf)         # bias
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, act="relu_grad", y16=buf, z=buf, accumulate=True)  # beta = 1
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, act="relu_grad", y16=buf, z=buf, ldz=60)           # pitch below N
    finally:
        mm.destroy()
        buf.destroy()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
def test_residual_epilogue(dev, layout, dtype):
    """C = res + A.B + bias with res another matrix than C (the reference's `residual` pass,
    tkernels.py:362-371, after the projection GEMMs, transformer.py:216, 223): exact on
    integer data for register-staged, direct-to-LDS, persistent (which hand over: their
    beta = 1 is an atomic add into C), stream-K and skinny tiles, with a K split through the
    workspace, ragged shapes and a padded res pitch; res itself stays untouched, and
    res == C is the plain in-place accumulation."""
    from vkgrad_amd.kernels import Matmul
    from vkgrad_amd.vk import VkError
    ta, tb = LAYOUTS[layout]
    cases = [(200, 136, 320, None, 0), (512, 384, 256, 11, 0), (1000, 1016, 1024, 10, 0), (392, 648, 2048, 11, 4),
             (129, 96, 768, 4, 3), (512, 768, 512, 15, 0), (640, 384, 1024, 18, 0), (4, 300, 768, 20, 0),
             (77, 50, 72, 0, 0), (512, 512, 4096, 17, 4)]
    for m, n, k, tile, split in cases:
        a, b = O.make_operands(m, n, k, ta, tb, dtype, seed=m + k, integer=True)
        bias = (np.arange(n) % 7 - 3).astype(np.float32)
        ldr = n + 5
        rng = np.random.default_rng(n)
        res = np.full((m, ldr), np.nan, np.float32)
        res[:, :n] = rng.integers(-50, 50, (m, n)).astype(np.float32)
        want = O.ref_gemm(a, b, ta, tb, dtype, bias, np.ascontiguousarray(res[:, :n]))
        ba, bb, bz = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(n * 4, "device")
        bc, br = dev.buffer(m * n * 4, "device"), dev.buffer(res.nbytes, "device")
        ba.upload(a); bb.upload(b); bz.upload(bias); br.upload(res)
        bc.upload(np.full((m, n), np.nan, np.float32))
        mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype, tile=tile, split_k=split)
        try:
            mm(ba, bb, bc, m, n, k, bias=bz, res=br, ldr=ldr)
            assert np.array_equal(bc.download(np.float32, (m, n)), want), (layout, m, n, k, tile, split)
            back = br.download(np.float32, (m, ldr))
            assert np.array_equal(back[:, :n], res[:, :n]) and np.isnan(back[:, n:]).all(), "res was written"
            # res == C: in place, the same as accumulate=True
            bc.upload(np.ascontiguousarray(res[:, :n]))
            mm(ba, bb, bc, m, n, k, bias=bz, res=bc)
            assert np.array_equal(bc.download(np.float32, (m, n)), want), (layout, m, n, k, tile, "in place")
        finally:
            mm.destroy()
            for x in (ba, bb, bz, bc, br):
                x.destroy()
    buf = dev.buffer(64 * 64 * 4, "device")
    mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype, split_k=2, atomic_split=True)
    try:
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, res=buf)              # atomic slices have nothing to add res once
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, res=buf, ldr=60)      # pitch below N
    finally:
        mm.destroy()
        buf.destroy()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_triangular_structure_of_causal_attention(dev, dtype):
    """tri= skips work that only meets masked entries of causal attention (the per-head
    GEMMs of transformer.py:144-182).  'c_lower': every C[i, j <= i] equals the full product
    (integer data: bit exact) whatever the tile, and whole tiles above the diagonal keep
    their poison; 'a_lower' / 'a_upper': with op(A) triangular the full product comes out,
    exactly, although part of the K range is never visited.  Batched, ragged, tiles that
    hand over (persistent, skinny), and the misuse cases."""
    from vkgrad_amd.kernels import Matmul
    from vkgrad_amd.vk import VkError
    rng = np.random.default_rng(5)

    def run(layout, m, n, k, tile, tri, nb, a, b, split_k=0, atomic=False):
        ta, tb = LAYOUTS[layout]
        ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(nb * m * n * 4, "device")
        ba.upload(a); bb.upload(b)
        bc.upload(np.full((nb, m, n), np.nan, np.float32))
        mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype, tile=tile, batched=nb > 1, split_k=split_k,
                    atomic_split=atomic)
        try:
            mm(ba, bb, bc, m, n, k, nbatch=nb, strides=(a[0].size, b[0].size, m * n), tri=tri)
            return bc.download(np.float32, (nb, m, n))
        finally:
            mm.destroy()
            for x in (ba, bb, bc):
                x.destroy()

    def operands(layout, m, n, k, nb, seed):
        ta, tb = LAYOUTS[layout]
        pairs = [O.make_operands(m, n, k, ta, tb, dtype, seed=seed + i, integer=True) for i in range(nb)]
        return np.stack([p[0] for p in pairs]), np.stack([p[1] for p in pairs])

    def product(layout, a, b):
        ta, tb = LAYOUTS[layout]
        return np.stack([O.ref_gemm(a[i], b[i], ta, tb, dtype) for i in range(a.shape[0])])

    # scores-like: C = A . B^T, lower triangle needed
    for m, n, k, tile, nb in ((200, 200, 64, None, 3), (1024, 1024, 64, None, 2), (512, 512, 64, 11, 1),
                              (512, 512, 128, 10, 2), (300, 300, 40, 4, 1), (512, 512, 64, 15, 1), (640, 640, 64, 3, 2)):
        a, b = operands("NT", m, n, k, nb, m + k)
        got = run("NT", m, n, k, tile, "c_lower", nb, a, b)
        want = product("NT", a, b)
        low = np.tril(np.ones((m, n), bool))
        assert np.array_equal(got[:, low], want[:, low]), (m, n, k, tile)
        if m >= 512:
            assert np.isnan(got[:, :256, m - 256:]).all(), "a tile wholly above the diagonal was written"
    # P V-like (NN) and dS K: op(A) lower triangular
    for m, n, k, tile, nb in ((256, 64, 256, None, 3), (1000, 72, 1000, None, 1), (512, 64, 512, 11, 2),
                              (512, 128, 512, 10, 1), (1024, 64, 1024, 14, 2), (300, 64, 300, 4, 1)):
        a, b = operands("NN", m, n, k, nb, m + n)
        a_tri = a.copy()
        a_tri[:, ~np.tril(np.ones((m, k), bool))] = 0
        got = run("NN", m, n, k, tile, "a_lower", nb, a_tri, b)
        assert np.array_equal(got, product("NN", a_tri, b)), (m, n, k, tile, "a_lower")
        # P^T dOut-like (TN): A stored (k, m); op(A)[i, kk] = A[kk, i] is zero for kk < i
        at, bt = operands("TN", m, n, k, nb, m + n + 1)
        at_tri = at.copy()
        at_tri[:, ~np.tril(np.ones((k, m), bool))] = 0          # stored A lower triangular = op(A) upper
        got = run("TN", m, n, k, tile, "a_upper", nb, at_tri, bt)
        assert np.array_equal(got, product("TN", at_tri, bt)), (m, n, k, tile, "a_upper")
        # with a K split (on request only): slices wholly outside a row block's K range are empty;
        # they meet in the workspace, or add into C with atomics (integer data: exact either way)
        if tile in (None, 14, 4, 11):
            for split, atomic in ((4, False), (3, True), (4, True)):
                got = run("NN", m, n, k, tile, "a_lower", nb, a_tri, b, split, atomic)
                assert np.array_equal(got, product("NN", a_tri, b)), (m, n, k, tile, "a_lower", split, atomic)
                got = run("TN", m, n, k, tile, "a_upper", nb, at_tri, bt, split, atomic)
                assert np.array_equal(got, product("TN", at_tri, bt)), (m, n, k, tile, "a_upper", split, atomic)
    buf = dev.buffer(64 * 64 * 4, "device")
    mm = Matmul(dev, dtype=dtype)
    mm2 = Matmul(dev, dtype=dtype, split_k=2)
    try:
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 32, 48, tri="a_lower")        # op(A) must be square
        with pytest.raises(VkError):
            mm2(buf, buf, buf, 64, 64, 64, tri="c_lower")       # runs unsplit
        with pytest.raises(VkError):
            mm(buf, buf, buf, 64, 64, 64, tri="upper")
    finally:
        mm.destroy()
        mm2.destroy()
        buf.destroy()


@pytest.mark.parametrize("tile", [None, 4, 11, 14])
def test_triangular_a_with_bias_and_atomic_k_split(dev, tile):
    """op(A) upper triangular (TN, A stored lower triangular), a bias, and K slices that add
    into C atomically: for the lower row blocks slice 0 - the one that carries the bias - has
    an empty K range, and must still add the bias."""
    from vkgrad_amd.kernels import Matmul
    m, n, k = 512, 64, 512
    a, b = O.make_operands(m, n, k, True, False, "bf16", seed=21, integer=True)
    a[~np.tril(np.ones((k, m), bool))] = 0
    bias = (np.arange(n, dtype=np.float32) % 9) - 4
    ref = O.ref_gemm(a, b, True, False, "bf16", bias, None)
    for split, atomic in ((4, True), (4, False), (3, True)):
        ba, bb, bc, bz = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), \
            dev.buffer(m * n * 4, "device"), dev.buffer(n * 4, "device")
        ba.upload(a); bb.upload(b); bz.upload(bias)
        bc.upload(np.full((m, n), np.nan, np.float32))
        mm = Matmul(dev, trans_a=True, dtype="bf16", tile=tile, split_k=split, atomic_split=atomic)
        try:
            mm(ba, bb, bc, m, n, k, bias=bz, tri="a_upper")
            got = bc.download(np.float32, (m, n))
            assert np.array_equal(got, ref), (tile, split, atomic, int((got != ref).sum()))
        finally:
            mm.destroy()
            for x in (ba, bb, bc, bz):
                x.destroy()


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_ping_pong_tile(dev, layout, dtype):
    """The ping-pong tile (two wavefront groups half a K-block apart, three operand tiles per
    ring stage, loads addressed by a scalar base): integer data, so every case is exact.
    Shapes where a half tile of A lies wholly or partly beyond M, ragged N and K (the K
    remainder goes through registers), one to five K-blocks (prologue and tail branches of
    the load schedule), padded pitches, bias, beta = 1, K splits both ways, batches, and
    the causal forms."""
    from vkgrad_amd.kernels import CONFIGS, Matmul
    pp = next(t["id"] for t in CONFIGS if t["name"].startswith("mmq_"))
    ta, tb = LAYOUTS[layout]
    shapes = [(256, 256, 64), (256, 256, 128), (256, 256, 192), (512, 512, 320), (100, 256, 256), (130, 300, 264),
              (257, 8, 72), (384, 520, 200), (1000, 264, 1032), (777, 1031, 136), (640, 768, 4096)]
    for m, n, k in shapes:
        if layout == "TN":
            m = max(8, m)
        r, got, ref = check_case(dev, m, n, k, ta, tb, dtype, seed=m + n + k, integer=True, tile=pp, bias=(k % 128 == 0),
                                 accumulate=(m % 2 == 1))
        assert r["exact"], f"{layout} {dtype} {m}x{n}x{k}: {int((got != ref).sum())} entries differ"
    # more workgroups than CUs with a short K loop: the first round starts staggered (ragged
    # edges; unsplit, and with a K split whose slices make up the surplus)
    if dtype == "bf16":
        r, got, ref = check_case(dev, 4344, 4104, 200, ta, tb, dtype, seed=9, integer=True, tile=pp, bias=True)
        assert r["exact"], f"{layout} staggered: {int((got != ref).sum())} entries differ"
        r, got, ref = check_case(dev, 2300, 2304, 2048, ta, tb, dtype, seed=10, integer=True, tile=pp, split_k=4, accumulate=True)
        assert r["exact"], f"{layout} staggered, split: {int((got != ref).sum())} entries differ"
    # padded pitches (the padding holds NaN) and K splits through the workspace and with atomics
    r, got, ref = check_case(dev, 300, 520, 1024, ta, tb, dtype, seed=5, integer=True, tile=pp, split_k=4, bias=True,
                             lda=(304 if ta else 1032), ldb=(1032 if tb else 528), ldc=536)
    assert r["exact"]
    mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype, tile=pp, split_k=3, atomic_split=True)
    a, b = O.make_operands(264, 392, 1536, ta, tb, dtype, seed=6, integer=True)
    ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(264 * 392 * 4, "device")
    try:
        ba.upload(a); bb.upload(b)
        bc.upload(np.full((264, 392), np.nan, np.float32))
        mm(ba, bb, bc, 264, 392, 1536)
        assert np.array_equal(bc.download(np.float32, (264, 392)), O.ref_gemm(a, b, ta, tb, dtype))
        assert mm.plan(264, 392, 1536)[0] == pp
    finally:
        mm.destroy()
        for x in (ba, bb, bc):
            x.destroy()
    # random data within the tolerances
    r, _, _ = check_case(dev, 1024, 768, 1536, ta, tb, dtype, seed=12, bias=True, tile=pp)
    _assert_close(r, f"ping-pong {layout} {dtype}")


def test_ping_pong_tile_batched_and_causal(dev):
    """Strided batches and the causal forms on the ping-pong tile (integer data, exact)."""
    from vkgrad_amd.kernels import CONFIGS, Matmul
    pp = next(t["id"] for t in CONFIGS if t["name"].startswith("mmq_"))

    def run(layout, m, n, k, nb, a, b, tri=None):
        ta, tb = LAYOUTS[layout]
        ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(nb * m * n * 4, "device")
        ba.upload(a); bb.upload(b)
        bc.upload(np.full((nb, m, n), np.nan, np.float32))
        mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype="bf16", tile=pp, batched=True)
        try:
            mm(ba, bb, bc, m, n, k, nbatch=nb, strides=(a[0].size, b[0].size, m * n), tri=tri)
            assert mm.plan(m, n, k, nbatch=nb)[0] == pp
            return bc.download(np.float32, (nb, m, n))
        finally:
            mm.destroy()
            for x in (ba, bb, bc):
                x.destroy()

    def operands(layout, m, n, k, nb, seed):
        ta, tb = LAYOUTS[layout]
        pairs = [O.make_operands(m, n, k, ta, tb, "bf16", seed=seed + i, integer=True) for i in range(nb)]
        return np.stack([p[0] for p in pairs]), np.stack([p[1] for p in pairs])

    def product(layout, a, b):
        ta, tb = LAYOUTS[layout]
        return np.stack([O.ref_gemm(a[i], b[i], ta, tb, "bf16") for i in range(a.shape[0])])

    a, b = operands("NT", 520, 520, 128, 3, 1)
    got = run("NT", 520, 520, 128, 3, a, b, tri="c_lower")
    low = np.tril(np.ones((520, 520), bool))
    assert np.array_equal(got[:, low], product("NT", a, b)[:, low])
    assert np.isnan(got[:, :256, 256:512]).all(), "a tile wholly above the diagonal was written"
    a, b = operands("NN", 768, 64, 768, 2, 2)
    a[:, ~np.tril(np.ones((768, 768), bool))] = 0
    assert np.array_equal(run("NN", 768, 64, 768, 2, a, b, tri="a_lower"), product("NN", a, b))
    a, b = operands("TN", 768, 72, 768, 2, 3)
    a[:, ~np.tril(np.ones((768, 768), bool))] = 0
    assert np.array_equal(run("TN", 768, 72, 768, 2, a, b, tri="a_upper"), product("TN", a, b))
    a, b = operands("NN", 300, 264, 200, 4, 4)
    assert np.array_equal(run("NN", 300, 264, 200, 4, a, b), product("NN", a, b))


def test_timing_over_rotating_operand_sets(dev):
    """The rotating timer launches argument set i % nsets on launch i: after seven
    launches over three sets with different integer operands, every set's C holds
    its own exact product (beta = 0 overwrites the poison), and the time is positive."""
    from vkgrad_amd.kernels import Matmul
    from vkgrad_amd.vk import VkError
    m, n, k = 200, 136, 320
    mm = Matmul(dev, trans_b=True, dtype="f16")
    sets, refs = [], []
    try:
        for s in range(3):
            a, b = O.make_operands(m, n, k, False, True, "f16", 40 + s, integer=True)
            bias = np.arange(n, dtype=np.float32) - s
            ba, bb, bc, bz = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), \
                dev.buffer(m * n * 4, "device"), dev.buffer(n * 4, "device")
            ba.upload(a); bb.upload(b); bz.upload(bias)
            bc.upload(np.full((m, n), np.nan, np.float32))
            sets.append((ba, bb, bc, bz))
            refs.append(O.ref_gemm(a, b, False, True, "f16", bias, None))
        sec = mm.time_rotating(sets, m, n, k, repeat=7)
        assert sec > 0
        for s in range(3):
            assert np.array_equal(sets[s][2].download(np.float32, (m, n)), refs[s]), f"set {s}"
        with pytest.raises(VkError):
            mm.time_rotating([], m, n, k, repeat=1)
        with pytest.raises(VkError):
            mm.time_rotating(sets, m, n, k, repeat=0)
    finally:
        mm.destroy()
        for st in sets:
            for x in st:
                x.destroy()


def test_wrong_layout_fails(dev):
    """Negative control (idea: test_hf_gpt2.py:129-136): a square operand read
    with the wrong layout passes every shape check and must fail on values."""
    m = n = k = 256
    a, b = O.make_operands(m, n, k, False, True, "f16", seed=9)       # B stored (n, k)
    got_wrong = run_gemm(dev, a, b, m, n, k, False, False, "f16")      # read as (k, n)
    ref = O.ref_gemm(a, b, False, True, "f16")
    assert O.err_fro(got_wrong, ref) > 0.5


@pytest.mark.parametrize("layout", list(LAYOUTS))
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_medium_random(dev, layout, dtype):
    ta, tb = LAYOUTS[layout]
    r, _, _ = check_case(dev, 1024, 768, 1536, ta, tb, dtype, seed=11, bias=True)
    _assert_close(r, f"{layout} {dtype} 1024x768x1536")


def test_ping_pong_partial_round_split(dev):
    """An unsplit ping-pong GEMM with a long K loop whose tiles leave a partial last round runs
    as two launches - whole rounds of tile rows unsplit, the remaining tile rows with a K split
    that fills the chip - and the result is what the oracle says (integer data: exact), with
    ragged edges, a K remainder, bias and beta = 1.  A shape without a partial round, and one
    whose K loop is too short to pay for the second launch, stay one launch."""
    from vkgrad_amd.kernels import CONFIGS, Matmul
    pp = next(t["id"] for t in CONFIGS if t["name"].startswith("mmq_"))
    cus = dev.compute_units
    if cus != 256:
        pytest.skip("shapes below are laid out for 256 CUs")

    def launches(layout, m, n, k):
        ta, tb = LAYOUTS[layout]
        a, b = O.make_operands(m, n, k, ta, tb, "bf16", seed=1, integer=True)
        ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(m * n * 4, "device")
        mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype="bf16", tile=pp, split_k=1)
        g = dev.graph("count")
        try:
            ba.upload(a); bb.upload(b)
            mm(ba, bb, bc, m, n, k, graph=g)
            g.finish()
            return g.kernel_count()
        finally:
            g.destroy(); mm.destroy()
            for x in (ba, bb, bc):
                x.destroy()

    # 17 x 16 = 272 tiles: 16 whole tile rows, then 16 tiles cut 8 ways along K = 4096 (+ 8)
    assert launches("NT", 4352, 4096, 4096) == 2
    assert launches("NT", 4096, 4096, 4096) == 1          # 256 tiles: whole rounds
    assert launches("NT", 4352, 4096, 512) == 1           # 8 K-blocks: not worth a second launch
    for layout in ("NT", "NN", "TN"):
        ta, tb = LAYOUTS[layout]
        r, got, ref = check_case(dev, 4352 - 8, 4096 - 24, 4096 + 8, ta, tb, "bf16", seed=21, integer=True, tile=pp, split_k=1,
                                 bias=True, accumulate=True)
        assert r["exact"], f"{layout}: {int((got != ref).sum())} entries differ"
