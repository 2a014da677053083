"""mg_gemm_static: the GEMM entry point that allocates nothing (no context, the caller's
stream, K slices meeting in a workspace that is part of the library's image).

It must give what mg_gemm gives, bit for bit where both take the same plan (same kernels, and
the workspace split sums its slices in slice order), on two calls in a row - the second on a
smaller problem, so that whatever the first left in the shared workspace and its counters
shows if it is not cleared - must refuse a K split that needs more than the static workspace,
must clear the counters of the launches the library splits by itself, and must work when
captured into a graph on a stream the caller owns.
Collected last (by its file name), so a failure here hides no other test.
"""

import ctypes as C

import numpy as np
import pytest

from oracle import ref_gemm as O

pytestmark = pytest.mark.gpu


def _hip():
    return C.CDLL("libamdhip64.so")


def _both(dev, m, n, k, ta, tb, dtype, tile, split, seed, bias=False, accumulate=False, integer=False):
    """The same GEMM through mg_gemm (context) and mg_gemm_static (no context, default
    stream); returns (C from mg_gemm, C from mg_gemm_static, oracle)."""
    from vkgrad_amd import _lib as L
    from vkgrad_amd.kernels import Matmul
    lib = dev._lib
    a, b = O.make_operands(m, n, k, ta, tb, dtype, seed, integer=integer)
    rng = np.random.default_rng(seed + 1)
    bias_v = rng.standard_normal(n).astype(np.float32) if bias else None
    c_in = rng.standard_normal((m, n)).astype(np.float32) if accumulate else None
    if integer:
        bias_v = None if bias_v is None else np.round(bias_v * 4)
        c_in = None if c_in is None else np.round(c_in * 4)
    ba, bb = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device")
    bc1, bc2 = dev.buffer(m * n * 4, "device"), dev.buffer(m * n * 4, "device")
    bz = dev.buffer(n * 4, "device") if bias else None
    mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype=dtype, tile=tile, split_k=split)
    try:
        ba.upload(a)
        bb.upload(b)
        if bias:
            bz.upload(bias_v)
        start = c_in if accumulate else np.full((m, n), np.nan, np.float32)
        bc1.upload(start)
        bc2.upload(start)
        mm(ba, bb, bc1, m, n, k, bias=bz, accumulate=accumulate)
        ga = mm._args(ba, bb, bc2, m, n, k, 1, (0, 0, 0), bz, accumulate, None, None, None)
        rc = lib.mg_gemm_static(0, None, C.byref(ga))
        assert rc == L.MG_OK, L.last_error()
        assert _hip().hipDeviceSynchronize() == 0
        plan = mm.plan(m, n, k)
        return (bc1.download(np.float32, (m, n)), bc2.download(np.float32, (m, n)),
                O.ref_gemm(a, b, ta, tb, dtype, bias_v, c_in), plan)
    finally:
        mm.destroy()
        for x in (ba, bb, bc1, bc2, bz):
            if x is not None:
                x.destroy()


def test_static_entry_point_matches_mg_gemm_twice(dev):
    # first call: a dW-like product whose K slices meet in the workspace (TN, bf16, split 4)
    g1, s1, ref, plan = _both(dev, 768, 512, 4096, True, False, "bf16", 11, 4, seed=31, accumulate=True)
    assert plan[1] == 4, plan
    assert np.array_equal(g1, s1), int((g1 != s1).sum())
    assert O.err_fro(s1, ref) <= 1e-3 and O.elementwise_ok(s1, ref, 4096)
    # second call, smaller, other layout and tile, ragged, with a bias: finds the first call's
    # partial tiles and counters in the shared workspace
    g2, s2, ref, plan = _both(dev, 200, 136, 1032, False, True, "f16", 4, 3, seed=32, bias=True)
    assert plan[1] == 3, plan
    assert np.array_equal(g2, s2), int((g2 != s2).sum())
    assert O.err_fro(s2, ref) <= 1e-3 and O.elementwise_ok(s2, ref, 1032)
    # third: integer data, stream-K tile (pieces meet in the same workspace), exact against the oracle
    g3, s3, ref, plan = _both(dev, 640, 384, 2048, False, False, "bf16", 19, 0, seed=33, integer=True)
    assert np.array_equal(g3, s3) and np.array_equal(s3, ref)
    # and an unsplit product, which uses no workspace at all
    g4, s4, ref, plan = _both(dev, 333, 96, 72, False, True, "f16", None, 1, seed=34, bias=True)
    assert np.array_equal(g4, s4)
    assert O.err_fro(s4, ref) <= 1e-3


def test_static_entry_point_refuses_what_does_not_fit(dev):
    """A K split whose partial tiles exceed the static workspace is refused before anything is
    launched, with a message that names both sizes."""
    from vkgrad_amd import _lib as L
    from vkgrad_amd.kernels import Matmul
    m, n, k = 4096, 4096, 4096                      # 64 MiB of f32 per slice
    ba, bb, bc = dev.buffer(m * k * 2, "device"), dev.buffer(k * n * 2, "device"), dev.buffer(m * n * 4, "device")
    mm = Matmul(dev, dtype="bf16", tile=11, split_k=2)
    try:
        bc.upload(np.full((m, n), 7.0, np.float32))
        ga = mm._args(ba, bb, bc, m, n, k, 1, (0, 0, 0), None, False, None, None, None)
        assert dev._lib.mg_gemm_static(0, None, C.byref(ga)) == L.MG_ERR_ARG
        msg = L.last_error()
        assert "static workspace" in msg and str(L.MG_STATIC_WS_BYTES) in msg, msg
        assert _hip().hipDeviceSynchronize() == 0
        assert np.all(bc.download(np.float32, (m, n)) == 7.0), "a refused call wrote C"
        # the same split with atomic adds needs no workspace and is accepted
        ga.flags |= L.MG_FLAG_SPLITK_ATOMIC
        assert dev._lib.mg_gemm_static(0, None, C.byref(ga)) == L.MG_OK, L.last_error()
        assert _hip().hipDeviceSynchronize() == 0
    finally:
        mm.destroy()
        for x in (ba, bb, bc):
            x.destroy()


def test_static_ping_pong_partial_round_and_dirty_counters(dev):
    """The ping-pong tile with a partial last round: the library cuts the remaining tile rows
    into K slices that meet in the workspace, and that second launch is planned unsplit at the
    top level - its counters must be cleared all the same.  Integer data, exact against the
    oracle, after another split call has used the workspace and twice in a row."""
    from vkgrad_amd import _lib as L
    from vkgrad_amd.kernels import Matmul
    lib = dev._lib
    # 67 x 4 = 268 tiles of 256 x 256 on 256 CUs: one whole round and 12 tiles more, cut into 8
    # K slices of 8 K-blocks each (24 MiB of partial tiles: fits the static workspace)
    m, n, k = 67 * 256, 1024, 4096
    a, b = O.make_operands(m, n, k, True, False, "bf16", 41, integer=True)
    ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(m * n * 4, "device")
    mm = Matmul(dev, trans_a=True, dtype="bf16", tile=21, split_k=1)
    try:
        ba.upload(a)
        bb.upload(b)
        ga = mm._args(ba, bb, bc, m, n, k, 1, (0, 0, 0), None, False, None, None, None)
        nk = C.c_int()
        assert lib.mg_gemm_static_launches(0, C.byref(ga), C.byref(nk)) == L.MG_OK, L.last_error()
        if dev.compute_units == 256:
            assert nk.value == 3, nk.value      # whole rounds, clear of the tail's counters, the tail's slices
        # a split call on a small problem first: it leaves its partial tiles in the workspace
        small = Matmul(dev, trans_a=True, dtype="bf16", tile=11, split_k=2)
        sa, sb = O.make_operands(128, 128, 256, True, False, "bf16", 42, integer=True)
        bsa, bsb, bsc = dev.buffer(sa.nbytes, "device"), dev.buffer(sb.nbytes, "device"), dev.buffer(128 * 128 * 4, "device")
        bsa.upload(sa)
        bsb.upload(sb)
        gs = small._args(bsa, bsb, bsc, 128, 128, 256, 1, (0, 0, 0), None, False, None, None, None)
        assert lib.mg_gemm_static(0, None, C.byref(gs)) == L.MG_OK, L.last_error()
        for _ in range(2):                      # twice: the second finds what the first left
            bc.upload(np.full((m, n), np.nan, np.float32))
            assert lib.mg_gemm_static(0, None, C.byref(ga)) == L.MG_OK, L.last_error()
            assert _hip().hipDeviceSynchronize() == 0
            got = bc.download(np.float32, (m, n))
            assert np.array_equal(got, O.ref_gemm(a, b, True, False, "bf16"))
        # with the atomic flag the same call is one launch and touches no workspace
        ga.flags |= L.MG_FLAG_SPLITK_ATOMIC
        assert lib.mg_gemm_static_launches(0, C.byref(ga), C.byref(nk)) == L.MG_OK and nk.value == 1
        bc.upload(np.full((m, n), np.nan, np.float32))
        assert lib.mg_gemm_static(0, None, C.byref(ga)) == L.MG_OK, L.last_error()
        assert _hip().hipDeviceSynchronize() == 0
        assert np.array_equal(bc.download(np.float32, (m, n)), O.ref_gemm(a, b, True, False, "bf16"))
        small.destroy()
        for x in (bsa, bsb, bsc):
            x.destroy()
    finally:
        mm.destroy()
        for x in (ba, bb, bc):
            x.destroy()


def test_static_entry_point_under_stream_capture(dev):
    """What the entry point is for: after one priming call outside the capture, a split and an
    unsplit GEMM are captured on a stream the caller owns, instantiated as a graph and replayed
    twice, with eager work and synchronisations between the replays; every replay is exact
    against the oracle, and the caller's current device is left alone."""
    from vkgrad_amd import _lib as L
    from vkgrad_amd.kernels import Matmul
    lib, hip = dev._lib, _hip()
    hip.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipStreamSynchronize.argtypes = [C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    hip.hipStreamDestroy.argtypes = [C.c_void_p]
    hip.hipGetDevice.argtypes = [C.POINTER(C.c_int)]
    cases = [(768, 512, 4096, True, False, 11, 4), (300, 264, 520, False, True, 11, 1)]   # split, unsplit
    bufs, mms, gas, refs = [], [], [], []
    for i, (m, n, k, ta, tb, tile, split) in enumerate(cases):
        a, b = O.make_operands(m, n, k, ta, tb, "bf16", 50 + i, integer=True)
        ba, bb, bc = dev.buffer(a.nbytes, "device"), dev.buffer(b.nbytes, "device"), dev.buffer(m * n * 4, "device")
        ba.upload(a)
        bb.upload(b)
        mm = Matmul(dev, trans_a=ta, trans_b=tb, dtype="bf16", tile=tile, split_k=split)
        gas.append(mm._args(ba, bb, bc, m, n, k, 1, (0, 0, 0), None, False, None, None, None))
        bufs.append((ba, bb, bc, m, n))
        mms.append(mm)
        refs.append(O.ref_gemm(a, b, ta, tb, "bf16"))
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    try:
        before = C.c_int(-1)
        assert hip.hipGetDevice(C.byref(before)) == 0
        for ga in gas:                                       # priming calls, outside the capture
            assert lib.mg_gemm_static(0, None, C.byref(ga)) == L.MG_OK, L.last_error()
        assert hip.hipDeviceSynchronize() == 0
        assert hip.hipStreamCreate(C.byref(stream)) == 0
        assert hip.hipStreamBeginCapture(stream, 2) == 0     # hipStreamCaptureModeRelaxed
        for ga in gas:
            assert lib.mg_gemm_static(0, stream, C.byref(ga)) == L.MG_OK, L.last_error()
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        after = C.c_int(-2)
        assert hip.hipGetDevice(C.byref(after)) == 0 and after.value == before.value
        for replay in range(3):
            for ba, bb, bc, m, n in bufs:
                bc.upload(np.full((m, n), np.nan, np.float32))      # eager work between the replays
            assert hip.hipGraphLaunch(gexec, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            for (ba, bb, bc, m, n), ref in zip(bufs, refs):
                assert np.array_equal(bc.download(np.float32, (m, n)), ref), f"replay {replay}"
    finally:
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        if stream:
            hip.hipStreamDestroy(stream)
        for mm in mms:
            mm.destroy()
        for ba, bb, bc, m, n in bufs:
            for x in (ba, bb, bc):
                x.destroy()
