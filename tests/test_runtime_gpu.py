"""GPU checks of the runtime surface (Device, Buffer, Graph) and the elementwise
companions, following /root/reference/test_runtime.py (memory kinds :139-149,
zero-copy round trip :57-75, one MFMA-sized tile :103-136) and test_accum.py
(accumulation over micro-batches :139-168)."""

import numpy as np
import pytest

from oracle import ref_gemm as O
from tests.util import run_gemm

pytestmark = pytest.mark.gpu


def test_memory_kinds_round_trip(dev):
    from vkgrad_amd.vk import VkError
    for kind in ("device", "shared", "cached", "bar"):
        b = dev.buffer(1 << 16, kind)
        try:
            if b.host_visible:
                b.array(np.uint32)[:16] = np.arange(16, dtype=np.uint32)
                assert np.array_equal(b.array(np.uint32)[:16], np.arange(16))
            else:
                with pytest.raises(VkError):
                    b.array(np.uint32)
                b.upload(np.arange(16, dtype=np.uint32))
                assert np.array_equal(b.download(np.uint32, (16,)), np.arange(16))
        finally:
            b.destroy()
    with pytest.raises(VkError):
        dev.buffer(64, "texture")
    with pytest.raises(VkError):
        dev.buffer(0, "device")


def test_zero_copy_round_trip(dev):
    """A host-visible tensor is a numpy array and a GPU buffer at once."""
    from vkgrad_amd.kernels import make_kernels
    K = make_kernels(dev)
    n = 4096
    src = dev.buffer(n * 4, "shared")
    dst = dev.buffer(n * 4, "shared")
    x = src.array(np.float32, (n,))
    x[:] = np.arange(n, dtype=np.float32)
    d = dst.array(np.float32, (n,))
    d[:] = 1.0
    src.flush()
    K["grad_add"]([dst, src], n)          # dst += src on the device, visible through the view
    dst.invalidate()
    assert np.array_equal(d, np.arange(n, dtype=np.float32) + 1.0)
    src.destroy()
    dst.destroy()


def test_device_copy(dev):
    a = dev.buffer(1024, "shared")
    b = dev.buffer(1024, "device")
    c = dev.buffer(1024, "cached")
    a.array(np.uint8)[:] = np.arange(1024) % 251
    dev.copy(a, b)
    dev.copy(b, c, 512)
    assert np.array_equal(c.array(np.uint8)[:512], a.array(np.uint8)[:512])
    for x in (a, b, c):
        x.destroy()


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_single_mfma_tile(dev, dtype):
    """32x32x16: one accumulator tile, one K step (test_runtime.py:103-136 does 16^3)."""
    a, b = O.make_operands(32, 32, 16, False, True, dtype, seed=0)
    got = run_gemm(dev, a, b, 32, 32, 16, False, True, dtype)
    ref = O.ref_gemm(a, b, False, True, dtype)
    assert np.abs(got - ref).max() < 1e-4


def test_golden_vectors_through_hip(dev):
    import os
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "gemm_golden.npz"))
    LAY = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}
    names = sorted({k.rsplit("_", 1)[0] for k in z.files})
    for name in names:
        layout, dtype = name.split("-")[1:3]
        ta, tb = LAY[layout]
        a, b, c = z[name + "_a"], z[name + "_b"], z[name + "_c"]
        if dtype == "f16":
            a, b = a.view(np.float16), b.view(np.float16)
        m, n = c.shape
        k = a.shape[0] if ta else a.shape[1]
        bias = z[name + "_bias"] if name + "_bias" in z.files else None
        c0 = z[name + "_c0"] if name + "_c0" in z.files else None
        got = run_gemm(dev, a, b, m, n, k, ta, tb, dtype, bias, c0)
        assert O.err_fro(got, c) <= 1e-5, name
        assert np.abs(got - c).max() <= 1e-4 * max(1.0, np.abs(c).max()), name


@pytest.mark.parametrize("layout", ["NN", "NT", "TN"])
def test_strided_batched(dev, layout):
    """z-batched GEMM with element strides (kernels.py:58-62, 98-101), at the
    attention shapes' pattern: several small matrices per launch."""
    from vkgrad_amd.kernels import Matmul
    ta, tb = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}[layout]
    m, n, k, nb = 96, 64, 40, 5
    rng = np.random.default_rng(1)
    a = rng.integers(-3, 4, nb * m * k).astype(np.float16)
    b = rng.integers(-3, 4, nb * k * n).astype(np.float16)
    strides = (m * k, k * n, m * n)
    ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(nb * m * n * 4, "device")
    ba.upload(a)
    bb.upload(b)
    mm = Matmul(dev, trans_a=ta, trans_b=tb, batched=True)
    mm(ba, bb, bc, m, n, k, nbatch=nb, strides=strides)
    got = bc.download(np.float32, (nb * m * n,))
    ref = O.ref_gemm_batched(a, b, m, n, k, nb, strides, ta, tb)
    assert np.array_equal(got, ref)
    for x in (ba, bb, bc):
        x.destroy()


def test_dw_accumulation_over_micro_batches(dev):
    """beta=1 over 4 micro-batches == one GEMM over the concatenated rows, also
    into a dirty accumulator (test_accum.py:51-58, 149-166)."""
    from vkgrad_amd.kernels import Matmul
    m, n, rows, micro = 192, 160, 256, 4
    parts = [O.make_operands(m, n, rows, True, False, "bf16", seed=20 + i) for i in range(micro)]
    for start in (0.0, 5.0):
        bc = dev.buffer(m * n * 4, "device")
        bc.upload(np.full((m, n), start, np.float32))
        mm = Matmul(dev, trans_a=True, dtype="bf16")
        for a, b in parts:
            ba, bb = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device")
            ba.upload(a)
            bb.upload(b)
            mm(ba, bb, bc, m, n, rows, accumulate=True)
            ba.destroy()
            bb.destroy()
        got = bc.download(np.float32, (m, n))
        ref = O.ref_gemm_accumulate(parts, True, False, "bf16", np.full((m, n), start, np.float32))
        big = O.ref_gemm(np.concatenate([p[0] for p in parts]), np.concatenate([p[1] for p in parts]),
                         True, False, "bf16") + start
        assert O.err_fro(got, ref) <= 1e-5
        assert O.err_fro(got, big) <= 2e-5        # measured 8.8e-06 in the reference
        bc.destroy()


def test_graph_records_and_replays_gemm_with_split_k(dev):
    """A recorded split-K GEMM (fill kernel + atomics) must give the same answer
    on every replay, with eager work and syncs between replays."""
    from vkgrad_amd.kernels import Matmul
    m, n, k = 256, 192, 4096
    a, b = O.make_operands(m, n, k, True, False, "f16", seed=8, integer=True)
    ref = O.ref_gemm(a, b, True, False, "f16")
    ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(m * n * 4, "device")
    ba.upload(a)
    bb.upload(b)
    mm = Matmul(dev, trans_a=True, tile=3, split_k=8)
    g = dev.graph("splitk")
    mm(ba, bb, bc, m, n, k, graph=g)
    g.finish()
    for i in range(4):
        bc.upload(np.full((m, n), np.nan, np.float32))
        g.submit()
        assert np.array_equal(bc.download(np.float32, (m, n)), ref), f"replay {i}"
        mm(ba, bb, bc, m, n, k)                      # eager work between replays
        dev.sync()
    g.destroy()
    for x in (ba, bb, bc):
        x.destroy()


def _linear_backward_case(dev, rows, fin, fout, seed):
    """Operands of one linear layer's backward pass on integer data: dY (rows, fout),
    W (fout, fin), X (rows, fin) and the two exact products dX = dY W, dW = dY^T X."""
    dy, w = O.make_operands(rows, fin, fout, False, False, "bf16", seed, integer=True)        # NN: (M,K), (K,N)
    dy2, x = O.make_operands(fout, fin, rows, True, False, "bf16", seed + 1, integer=True)     # TN: (K,M), (K,N)
    ref_dx = O.ref_gemm(dy, w, False, False, "bf16")
    ref_dw = O.ref_gemm(dy2, x, True, False, "bf16")
    bufs = {}
    for name, arr in (("dy", dy), ("w", w), ("dy2", dy2), ("x", x)):
        bufs[name] = dev.buffer(arr.nbytes, "device")
        bufs[name].upload(arr)
    bufs["dx"] = dev.buffer(rows * fin * 4, "device")
    bufs["dw"] = dev.buffer(fout * fin * 4, "device")
    return bufs, ref_dx, ref_dw


def test_side_stream_runs_independent_gemms_concurrently(dev):
    """dX on the main stream and dW on the side stream between fork and join, both with a
    K split through the workspace (each stream owns its half, so the same tile numbers do
    not collide): exact on integer data, several rounds back to back; misuse is refused."""
    from vkgrad_amd.kernels import Matmul
    from vkgrad_amd.vk import VkError
    rows, fin, fout = 1024, 256, 384
    bufs, ref_dx, ref_dw = _linear_backward_case(dev, rows, fin, fout, 21)
    mm_dx = Matmul(dev, dtype="bf16", tile=3, split_k=3)
    mm_dw = Matmul(dev, trans_a=True, dtype="bf16", tile=3, split_k=4)
    try:
        with pytest.raises(VkError):          # no fork yet
            mm_dw.enqueue(bufs["dy2"], bufs["x"], bufs["dw"], fout, fin, rows, side=True)
        with pytest.raises(VkError):          # an eager call waits for its result
            mm_dw(bufs["dy2"], bufs["x"], bufs["dw"], fout, fin, rows, side=True)
        for it in range(5):
            bufs["dx"].upload(np.full((rows, fin), np.nan, np.float32))
            bufs["dw"].upload(np.full((fout, fin), np.nan, np.float32))
            dev.side_fork()
            mm_dw.enqueue(bufs["dy2"], bufs["x"], bufs["dw"], fout, fin, rows, side=True)
            mm_dx.enqueue(bufs["dy"], bufs["w"], bufs["dx"], rows, fin, fout)
            dev.side_join()
            dev.sync()
            assert np.array_equal(bufs["dx"].download(np.float32, (rows, fin)), ref_dx), f"dX round {it}"
            assert np.array_equal(bufs["dw"].download(np.float32, (fout, fin)), ref_dw), f"dW round {it}"
    finally:
        dev.side_join()
        mm_dx.destroy()
        mm_dw.destroy()
        for b in bufs.values():
            b.destroy()


def test_graph_with_parallel_branches_replays(dev):
    """A recorded step whose dW GEMMs sit on the side stream (fork before each, one join
    at the end by finish()): every replay gives the exact products, with eager work and
    synchronisations between the replays."""
    from vkgrad_amd.kernels import Matmul
    rows, fin, fout = 768, 512, 256
    cases = [_linear_backward_case(dev, rows, fin, fout, 31 + 2 * i) for i in range(3)]
    mm_dx = Matmul(dev, dtype="bf16")
    mm_dw = Matmul(dev, trans_a=True, dtype="bf16", tile=11, split_k=3)
    g = dev.graph("backward")
    for bufs, _, _ in cases:
        g.fork()
        mm_dw(bufs["dy2"], bufs["x"], bufs["dw"], fout, fin, rows, graph=g, side=True)
        mm_dx(bufs["dy"], bufs["w"], bufs["dx"], rows, fin, fout, graph=g)
    g.finish()
    try:
        for it in range(4):
            for bufs, _, _ in cases:
                bufs["dx"].upload(np.full((rows, fin), np.nan, np.float32))
                bufs["dw"].upload(np.full((fout, fin), np.nan, np.float32))
            g.submit()
            for j, (bufs, ref_dx, ref_dw) in enumerate(cases):
                assert np.array_equal(bufs["dx"].download(np.float32, (rows, fin)), ref_dx), f"replay {it} dX {j}"
                assert np.array_equal(bufs["dw"].download(np.float32, (fout, fin)), ref_dw), f"replay {it} dW {j}"
            b0 = cases[0][0]
            mm_dx(b0["dy"], b0["w"], b0["dx"], rows, fin, fout)      # eager work between replays
            dev.sync()
    finally:
        g.destroy()
        mm_dx.destroy()
        mm_dw.destroy()
        for bufs, _, _ in cases:
            for b in bufs.values():
                b.destroy()


def test_graph_with_a_free_running_side_chain_replays_back_to_back(dev):
    """The benchmark's default schedule in small: one fork at the start of the recorded step,
    the dW GEMMs of several linears queued behind each other on the side stream - an unsplit
    ping-pong tile, a K split through the side stream's half of the workspace, a persistent
    tile with a split, an atomic split - beside the dX chain on the main stream (one of them
    split through the main half), one join at the end.  Replays are enqueued back to back
    without a synchronisation in between, as the benchmark times them; afterwards every
    product must be exact (integer data), and again after a second burst."""
    from vkgrad_amd.kernels import Matmul
    rows = 2048
    dims = [(512, 768), (768, 256), (256, 1024), (1024, 512)]
    cases = [_linear_backward_case(dev, rows, fin, fout, 51 + 2 * i) for i, (fin, fout) in enumerate(dims)]
    dw_plans = [dict(tile=21), dict(tile=11, split_k=2), dict(tile=17, split_k=4), dict(tile=14, split_k=3, atomic_split=True)]
    dx_plans = [dict(tile=11), dict(tile=21), dict(tile=11, split_k=2), dict(tile=14)]
    mm_dw = [Matmul(dev, trans_a=True, dtype="bf16", **kw) for kw in dw_plans]
    mm_dx = [Matmul(dev, dtype="bf16", **kw) for kw in dx_plans]
    g = dev.graph("free_side_chain")
    g.fork()
    for (bufs, _, _), (fin, fout), dx, dw in zip(cases, dims, mm_dx, mm_dw):
        dx(bufs["dy"], bufs["w"], bufs["dx"], rows, fin, fout, graph=g)
        dw(bufs["dy2"], bufs["x"], bufs["dw"], fout, fin, rows, graph=g, side=True)
    g.finish()
    try:
        for burst in range(2):
            for (bufs, _, _), (fin, fout) in zip(cases, dims):
                bufs["dx"].upload(np.full((rows, fin), np.nan, np.float32))
                bufs["dw"].upload(np.full((fout, fin), np.nan, np.float32))
            for _ in range(6):
                g.enqueue()
            dev.sync()
            for j, ((bufs, ref_dx, ref_dw), (fin, fout)) in enumerate(zip(cases, dims)):
                assert np.array_equal(bufs["dx"].download(np.float32, (rows, fin)), ref_dx), f"burst {burst} dX {j}"
                assert np.array_equal(bufs["dw"].download(np.float32, (fout, fin)), ref_dw), f"burst {burst} dW {j}"
    finally:
        g.destroy()
        for m in mm_dw + mm_dx:
            m.destroy()
        for bufs, _, _ in cases:
            for b in bufs.values():
                b.destroy()


def test_elementwise_kernels(dev):
    from vkgrad_amd.kernels import make_kernels
    from oracle import ref_mlp as RM
    K = make_kernels(dev, "f16")
    rng = np.random.default_rng(0)
    rows, ncol = 37, 50
    n = rows * ncol
    acc = rng.standard_normal((rows, ncol)).astype(np.float32)
    bias = rng.standard_normal(ncol).astype(np.float32)

    def up(x):
        b = dev.buffer(max(x.nbytes, 4), "device")
        b.upload(x)
        return b

    bacc, bbias = up(acc), up(bias)
    bz, by = dev.buffer(n * 4, "device"), dev.buffer(n * 2, "device")
    for name, act in (("bias_gelu", "gelu"), ("bias_relu", "relu")):
        K[name]([bacc, bbias, bz, by], n, ncol)
        z = bz.download(np.float32, (rows, ncol))
        y = by.download(np.float16, (rows, ncol))
        assert np.array_equal(z, acc + bias[None, :])
        want = RM.act_fn(z, act).astype(np.float16)
        assert np.abs(y.astype(np.float32) - want.astype(np.float32)).max() <= 2e-3
    # col_sum and its accumulating form
    bs = dev.buffer(ncol * 4, "device")
    K["col_sum"]([bz, bs], ncol, rows)
    s1 = bs.download(np.float32, (ncol,))
    assert np.allclose(s1, z.sum(0), rtol=1e-5, atol=1e-5)
    K["col_sum_acc"]([bz, bs], ncol, rows)
    assert np.allclose(bs.download(np.float32, (ncol,)), 2 * s1, rtol=1e-6, atol=1e-6)
    # cast16 in both types is round-to-nearest-even
    x = rng.standard_normal(1000).astype(np.float32)
    bx, b16 = up(x), dev.buffer(2000, "device")
    K["cast16"]([bx, b16], 1000)
    assert np.array_equal(b16.download(np.float16, (1000,)), x.astype(np.float16))
    Kb = make_kernels(dev, "bf16")
    Kb["cast16"]([bx, b16], 1000)
    assert np.array_equal(b16.download(np.uint16, (1000,)), O.f32_to_bf16_bits(x))
    # zero
    K["zero"]([bx], 1000)
    assert not bx.download(np.float32, (1000,)).any()


def test_column_sums_and_recordable_copy(dev):
    """col_sum over one chunk of rows (fixed order) and over several (chunks meet through
    atomics after a clear), overwriting and accumulating; the recordable copy kernel for
    16-byte-aligned and merely 4-byte-aligned ends, with a tail."""
    from vkgrad_amd.kernels import make_kernels
    K = make_kernels(dev, "f16")
    rng = np.random.default_rng(5)
    for nrow, ncol in [(128, 512), (1, 10), (513, 70), (2000, 300), (5000, 64)]:
        g = rng.standard_normal((nrow, ncol)).astype(np.float32)
        bg, bs = dev.buffer(g.nbytes, "device"), dev.buffer(ncol * 4, "device")
        bg.upload(g)
        bs.upload(np.full(ncol, 7.0, np.float32))
        want = g.astype(np.float64).sum(0)
        K["col_sum"]([bg, bs], ncol, nrow)
        got = bs.download(np.float32, (ncol,))
        assert np.allclose(got, want, rtol=1e-5, atol=1e-4 * np.sqrt(nrow)), (nrow, ncol)
        K["col_sum_acc"]([bg, bs], ncol, nrow)
        got2 = bs.download(np.float32, (ncol,))
        assert np.allclose(got2, 2 * want, rtol=1e-5, atol=2e-4 * np.sqrt(nrow)), (nrow, ncol)
        bg.destroy()
        bs.destroy()
    src = dev.buffer(4096, "shared")
    dst = dev.buffer(4096, "device")
    data = rng.integers(0, 2 ** 32, 1024, dtype=np.uint64).astype(np.uint32)
    src.array(np.uint32, (1024,))[:] = data
    for nbytes in (32, 1000, 4096):
        dst.upload(np.zeros(1024, np.uint32))
        K["copy"]([src, dst], nbytes)
        out = dst.download(np.uint32, (1024,))
        assert np.array_equal(out[:nbytes // 4], data[:nbytes // 4]) and not out[nbytes // 4:].any()
    # ends that are only 4-byte aligned: through the C ABI with offset pointers
    dst.upload(np.zeros(1024, np.uint32))
    assert dev._lib.mg_ew_copy(dev._ctx, dst.ptr + 4, src.ptr + 8, 400) == 0
    out = dst.download(np.uint32, (1024,))
    assert np.array_equal(out[1:101], data[2:102]) and out[0] == 0 and not out[101:].any()
    assert dev._lib.mg_ew_copy(dev._ctx, dst.ptr, src.ptr, 6) != 0     # not a multiple of 4
    src.destroy()
    dst.destroy()


def test_mfma_ceiling_probe(dev):
    """mg_probe_mfma: the register-only MFMA rate, on zero and on random operands.  The rate
    equals 2 wavefronts x 4 SIMDs x CUs x 1024 FLOP per clock at the clock it reports (the loop
    has no other instruction), and random operands never run faster than zeros."""
    from vkgrad_amd.probe import mfma_ceiling
    z_tf, z_ghz = mfma_ceiling(dev, "bf16", False, seconds=0.05)
    r_tf, r_ghz = mfma_ceiling(dev, "bf16", True, seconds=0.05)
    for tf, ghz in ((z_tf, z_ghz), (r_tf, r_ghz)):
        assert 0.5 < ghz < 3.5 and tf > 100.0
        per_clock = tf * 1e12 / (ghz * 1e9) / (dev.compute_units * 4)
        assert 0.85 * 1024 <= per_clock <= 1.02 * 1024, per_clock
    assert r_tf <= z_tf * 1.03
    f_tf, _ = mfma_ceiling(dev, "f16", True, seconds=0.05)
    assert f_tf > 100.0
    # a quarter of the CUs busy: a quarter of the work per clock, at a clock that is no lower
    q = dev.compute_units // 4
    q_tf, q_ghz = mfma_ceiling(dev, "bf16", True, seconds=0.05, busy_cus=q)
    per_clock = q_tf * 1e12 / (q_ghz * 1e9) / (q * 4)
    assert 0.85 * 1024 <= per_clock <= 1.02 * 1024, per_clock
    assert q_ghz >= r_ghz * 0.97


def test_stream_floor_probe(dev):
    """mg_probe_stream: a read-only and a fill-only launch over the bytes of the 50257 x 768 f16
    weight matrix, shaped like the skinny-M stream.  Between a tenth of the HBM peak and the
    peak; a buffer 16 bytes long still runs (one partly filled wavefront)."""
    from vkgrad_amd.probe import stream_floor
    nbytes = 50257 * 768 * 2
    r, f = stream_floor(dev, nbytes, nsets=8, repeat=50)
    for us in (r, f):
        assert 0.8e12 <= nbytes / (us * 1e-6) <= 8.0e12, us
    r, f = stream_floor(dev, 16, nsets=1, repeat=3)
    assert r > 0 and f > 0
