#!/usr/bin/env python3
"""Benchmark of the training-GEMM path on one MI355X.

One step = every GEMM of one GPT-2-small training step (the GPT-2-small configuration of the workload list):
d_model 768, 12 layers, 8 x 1024 = 8192 token rows, per layer QKV 768->2304,
proj 768->768, MLP 768->3072->768, plus the tied LM head 768->50257; for every
linear the forward, dX and dW products (147 GEMMs, 6.07 TFLOP), bf16 inputs,
fp32 accumulate and fp32 outputs, synthetic operands already resident in HBM.
Weights are stored out x in (the tied-head convention), so the kernel layouts
are NT forward, NN dX, TN dW.  The step is given to the device as forward, dX,
dW of each linear in turn; the dW GEMMs go to the library's second stream, which
is forked once at the start of the step and joined once at its end (a weight
gradient is needed by nothing before the optimiser), so they fill the compute
units the forward / dX chain leaves idle in its partial rounds.  `in_order` in
the line is the same step with every GEMM behind the previous one on one stream;
--schedule names the other orders that were measured.

Prints ONE JSON line: whole-step TFLOP/s, the MFMA roofline of the dominant
GEMM measured with HIP events on the library's stream, and the numpy oracle
timed on this machine's host cores over whole steps of the same workload (about 10 s).
"""

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = 2500.0     # MI355X dense bf16/fp16 MFMA peak
ROWS, D, LAYERS, VOCAB = 8192, 768, 12, 50257
LINEARS = [("qkv", 768, 2304), ("proj", 768, 768), ("fc1", 768, 3072), ("fc2", 3072, 768)]
DTYPE = "bf16"


def gemm_list():
    """(name, layout, M, N, K, count) for one step.  W is (out, in)."""
    out = []
    for name, fin, fout in LINEARS:
        out.append((name + ".fwd", "NT", ROWS, fout, fin, LAYERS))   # Y  = X  W^T
        out.append((name + ".dX", "NN", ROWS, fin, fout, LAYERS))    # dX = dY W
        out.append((name + ".dW", "TN", fout, fin, ROWS, LAYERS))    # dW = dY^T X
    out.append(("head.fwd", "NT", ROWS, VOCAB, D, 1))
    out.append(("head.dX", "NN", ROWS, D, VOCAB, 1))
    out.append(("head.dW", "TN", VOCAB, D, ROWS, 1))
    return out


SCHEDULES = {
    "dw-stream": "forward, dX, dW per linear; the dW GEMMs on a second stream, forked once at the start of the "
                 "step and joined once at its end",
    "in-order": "forward, dX, dW per linear, every GEMM behind the previous one on one stream",
    "dw-stream-waits": "forward, dX, dW per linear; the dW GEMMs on a second stream that waits before each for what "
                       "the main stream has been given so far, joined at the end of the step",
    "pairs": "forward, then dX and dW of the linear side by side on two streams, forked and joined per pair",
    "passes": "forward pass, then backward pass with a layer's dW GEMMs on a second stream beside the next "
              "layer's dX chain, joined at the end of the step",
}

LAYOUT_FLAGS = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}


def head_pitch(dense_head=False):
    """Row pitch of logits / dlogits: the next multiple of 64 elements, as any allocator of a
    (rows x vocab) tensor would give it (the reference pads the vocabulary itself,
    transformer.py:258), or exactly VOCAB with dense_head (rows then start at odd addresses)."""
    return VOCAB if dense_head else (VOCAB + 63) // 64 * 64


def pitches_for(name, vpitch):
    """Non-default row pitches of one GEMM of gemm_list(): the LM head's logits (C of the
    forward product) and dlogits (A of dX and dW) have pitch vpitch."""
    if not name.startswith("head") or vpitch == VOCAB:
        return {}
    return {"ldc": vpitch} if name.endswith(".fwd") else {"lda": vpitch}


def plan_for(dev, name, layout, m, n, k, vpitch, context=None):
    """(Matmul, pitches) exactly as the timed step builds them: the tuned table's plan for
    the shape (tile, K split, band, split mode, walk) - the one chosen inside the step of the
    named schedule when the table holds one (kernels.tune_in_context), else the one chosen
    alone - and the library's picker where the table has none."""
    from vkgrad_amd.kernels import tuned_matmul
    ta, tb = LAYOUT_FLAGS[layout]
    kw = pitches_for(name, vpitch)
    return tuned_matmul(dev, m, n, k, ta, tb, DTYPE, context=context, **kw)[0], kw


def context_of(schedule):
    """Name under which plans tuned inside a step of this schedule are kept (where the table has
    none for it, the plans tuned alone apply)."""
    return "gpt2s-" + schedule

# HBM-side bytes per launch (L2 fetches + L2 write-backs) of each GEMM of the step,
# measured on MI355X with `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` over
# `bench.py --pmc-pass`, each counter scaled by what it reads for the cast kernel of
# known size in the same pass (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000).  A figure is
# only valid for the (tile, split_k) it was measured with; for another plan the
# bench line reports null.  gemm -> (tile, split_k, fetch bytes, write bytes)
MEASURED_TRAFFIC = {
    "qkv.fwd": (21, 1, 52.1e6, 75.5e6), "qkv.dX": (11, 1, 66.2e6, 25.2e6), "qkv.dW": (21, 1, 151.2e6, 7.1e6),
    "proj.fwd": (11, 1, 22.2e6, 25.2e6), "proj.dX": (14, 1, 22.2e6, 25.2e6),
    "proj.dW": (17, 4, 47.4e6, 11.8e6), "fc1.fwd": (21, 1, 76.9e6, 100.7e6),
    "fc1.dX": (21, 1, 126.1e6, 25.2e6), "fc1.dW": (11, 2, 260.1e6, 28.3e6), "fc2.fwd": (11, 1, 90.8e6, 25.2e6),
    "fc2.dX": (21, 1, 77.8e6, 100.7e6), "fc2.dW": (11, 3, 192.0e6, 37.8e6),
    "head.fwd": (21, 1, 733.4e6, 1647.6e6), "head.dX": (21, 8, 1662.6e6, 226.5e6),
    "head.dW": (21, 1, 1464.0e6, 218.1e6),
}


def fill_bf16(dev, buf, n, rng, scale):
    """Upload n bf16 values ~N(0, scale) in slabs (keeps host memory small)."""
    from vkgrad_amd.dtypes import f32_to_bf16_bits
    slab = 1 << 24
    tmp = dev.buffer(min(n, slab) * 2, "device")
    done = 0
    lib, ctx = dev._lib, dev._ctx
    while done < n:
        m = min(slab, n - done)
        bits = f32_to_bf16_bits((rng.standard_normal(m, dtype=np.float32) * scale))
        tmp.upload(bits)
        rc = lib.mg_copy(ctx, buf.ptr + done * 2, tmp.ptr, m * 2)
        assert rc == 0
        done += m
    tmp.destroy()


def cpu_baseline(min_seconds=10.0):
    """The oracle (numpy float32 matmul of the rounded operands, reference
    kernels.py:606-610) on this host: whole steps of the same workload (every GEMM
    of the 12 layers and the LM head, fwd + dX + dW) until min_seconds of matmul
    time have passed."""
    from oracle.ref_gemm import f32_to_bf16_bits, bf16_bits_to_f32
    rng = np.random.default_rng(1)

    def rounded(shape, scale):
        return bf16_bits_to_f32(f32_to_bf16_bits(rng.standard_normal(shape, dtype=np.float32) * scale))

    ops = []
    for name, fin, fout in LINEARS + [("head", D, VOCAB)]:
        ops.append((LAYERS if name != "head" else 1, rounded((ROWS, fin), 1.0), rounded((fout, fin), 0.02),
                    rounded((ROWS, fout), 1.0)))
    w = rng.standard_normal((512, 512), dtype=np.float32)
    (w @ w).sum()   # warm the BLAS thread pool
    flops = secs = 0.0
    steps = 0
    while secs < min_seconds:
        for count, x, wt, dy in ops:
            for _ in range(count):
                t0 = time.perf_counter()
                y = x @ wt.T
                dx = dy @ wt
                dw = dy.T @ x
                secs += time.perf_counter() - t0
                flops += 3 * 2.0 * x.shape[0] * x.shape[1] * wt.shape[0]
                del y, dx, dw
        steps += 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    threads = int(os.environ.get("OPENBLAS_NUM_THREADS") or os.environ.get("OMP_NUM_THREADS") or cores)
    mlp = cpu_mlp_step()
    return {"value": round(flops / secs / 1e12, 4), "unit": "TFLOP/s", "cores": min(threads, cores),
            "kind": "port", "mnist_mlp_step_ms": mlp,
            "sample": f"{steps} whole steps of the benchmark workload (147 GEMMs, 6.07 TFLOP each), numpy float32 matmul "
                      f"of bf16-rounded operands, {secs:.1f} s of matmul time"}


MLP_SIZES, MLP_BATCH, MLP_CLASSES = (784, 512, 512), 128, 10


def mlp_step_device(dev, steps=300):
    """The MLP configuration on the device: the synthetic-MNIST MLP train step (batch 128, 784 ->
    512 -> 512 -> 10, ReLU, He-normal weights, f16, fwd + dX + dW + bias gradients + AdamW)
    recorded once and replayed as one HIP graph; microseconds per step including the read-back
    of the loss, as the reference's TrainStep measures it (bench/mnist-repro.json:5-24)."""
    from vkgrad_amd.autograd import AdamW, Ctx, MLP, TrainStep
    rng = np.random.default_rng(0)
    ctx = Ctx(dev, dtype="f16", fuse_bias=True)
    try:
        model = MLP(ctx, MLP_BATCH, list(MLP_SIZES), MLP_CLASSES, pad_classes=MLP_CLASSES, activation="relu")
        widths = list(MLP_SIZES) + [MLP_CLASSES]
        for layer, fin, fout in zip(model.layers, widths[:-1], widths[1:]):
            layer.W.set((rng.standard_normal((fin, fout)) * np.sqrt(2.0 / fin)).astype(np.float32))
            layer.b.set(np.zeros(fout, np.float32))
        xb = ctx.buf(MLP_BATCH * MLP_SIZES[0] * 2, "shared")
        xb.array(np.float16, (MLP_BATCH, MLP_SIZES[0]))[:] = rng.random((MLP_BATCH, MLP_SIZES[0]),
                                                                        dtype=np.float32).astype(np.float16)
        yb = ctx.buf(MLP_BATCH * 4, "shared")
        yb.array(np.uint32, (MLP_BATCH,))[:] = rng.integers(0, MLP_CLASSES, MLP_BATCH)
        step = TrainStep(model, AdamW(ctx, model.params(), lr=1e-3), xb, yb)
        first = step()[0]
        for _ in range(20):
            step()
        t0 = time.perf_counter()
        for _ in range(steps):
            loss, _ = step()
        dt = (time.perf_counter() - t0) / steps
        return {"us_per_step": round(dt * 1e6, 1), "kernels_per_step": step.n_dispatch, "steps": steps,
                "loss_first": round(float(first), 4), "loss_last": round(float(loss), 4),
                "what": "graph replay + loss read-back, batch 128, 784-512-512-10, ReLU, f16, AdamW"}
    finally:
        ctx.destroy()


def cpu_mlp_step(steps=30):
    """The numpy model of the configs[0] train step (oracle/ref_mlp.py, the restatement of the
    reference's numpy path) on this host: milliseconds per step."""
    from oracle import ref_mlp
    Ws, bs = ref_mlp.he_init(list(MLP_SIZES) + [MLP_CLASSES], 0)
    ref = ref_mlp.RefMLP(MLP_SIZES, MLP_CLASSES, MLP_CLASSES, act="relu", dtype="f16")
    ref.set_params(Ws, bs)
    _, xf, y = ref_mlp.synthetic_batch(MLP_BATCH, MLP_SIZES[0], MLP_CLASSES, 0, "f16")
    for _ in range(3):
        ref.train_step(xf, y, lr=1e-3)
    t0 = time.perf_counter()
    for _ in range(steps):
        ref.train_step(xf, y, lr=1e-3)
    return round((time.perf_counter() - t0) / steps * 1e3, 3)


def other_workloads(dev):
    """Compact figures for the workloads the headline does not cover (the reference's
    bench/matmul_sweep.py:60-107 writes one record with every size): the MLP train step of
    configs[0], the squares of configs[1] in the three layouts (8192^3 timed over batches of
    >= 0.1 s so that it runs at the sustained clock), one optimiser step of the d_model-1024
    decoder of configs[3] (every distinct GEMM timed, weighted by its count), the char-LM
    GEMMs of configs[4] and its N = 50257 skinny rows.  Median of the batches per GEMM."""
    from vkgrad_amd import sweep
    r = sweep.Runner(dev=dev, warm=False)
    out = {"mnist_mlp_step_f16": mlp_step_device(dev)}
    sq = {}
    for c in sweep.cases_for("square"):
        big = c["m"] == 8192
        row = r.time_case(c, samples=4 if big else 3, min_seconds=0.1 if big else 0.01)
        sq.setdefault(str(c["m"]), {})[c["layout"]] = {"tflops": row["tflops"], "frac_mfma": row["frac_mfma"],
                                                       "us": row["us"], "tile": row["tile"]}
    out["square_f16"] = sq
    rows = [r.time_case(c, samples=3, min_seconds=0.01) for c in sweep.cases_for("decoder")]
    us = sum(x["us"] * x["count"] for x in rows)
    fl = sum(2.0 * x["m"] * x["n"] * x["k"] * x["count"] for x in rows)
    out["decoder_1024_optimiser_step_bf16"] = {
        "gemms": sum(x["count"] for x in rows), "tflop": round(fl / 1e12, 2), "gemm_ms": round(us / 1e3, 2),
        "tflops": round(fl / us / 1e6, 1), "frac_mfma": round(fl / us / 1e6 / PEAK_TFLOPS, 4),
        "dw": "beta = 1 over 4 micro-batches (the first overwrites)"}
    rows = [r.time_case(c, samples=3, min_seconds=0.005) for c in sweep.cases_for("charlm")]
    us = sum(x["us"] for x in rows)
    fl = sum(2.0 * x["m"] * x["n"] * x["k"] for x in rows)
    out["charlm_gemms_f16"] = {"gemms": len(rows), "total_us": round(us, 1), "tflops": round(fl / us / 1e6, 1),
                               "what": "d_model 256, vocabulary 96, 16384 rows: fwd + dX + dW of 5 linears"}
    sk = {}
    for c in sweep.cases_for("skinny"):
        if c["n"] == VOCAB:
            row = r.time_case(c, samples=3, min_seconds=0.01)
            sk[f"{c['m']}x{c['n']}x{c['k']}"] = {"us": row["us"], "gbps": row["gbps"], "frac_hbm": row["frac_hbm"],
                                                 "tile": row["tile"]}
    out["skinny_nt_bias_f16"] = sk
    return out


def tune_step(dev, args, vpitch, context, step_calls, record):
    """Plans for the step's GEMMs as they run under args.schedule, by coordinate descent on the
    time of the whole replayed step; the picks go to the tuner's cache under `context`."""
    import statistics
    from vkgrad_amd import kernels as K
    fields = ("tile_id", "split_k", "atomic_split", "group_m", "xcd_rotate")
    slots, meta = {}, {}
    for name, layout, m, n, k, _ in gemm_list():
        ta, tb = LAYOUT_FLAGS[layout]
        kw = pitches_for(name, vpitch)
        cur = K.lookup_tuned(dev.name, m, n, k, ta, tb, DTYPE, context=context, **kw)
        cands = []
        for c in K.plan_candidates(m, n, k, K.layout_of(ta, tb), dev.compute_units):
            mm = K.matmul_from_entry(dev, c, ta, tb, DTYPE)
            tile, split, _ = mm.plan(m, n, k, **kw)          # what the library would really run
            mm.destroy()
            if (tile, split) == (c["tile_id"], c["split_k"]):
                cands.append(c)
        first = dict(cands[0]) if cur is None else dict(cands[0], **{f: cur.get(f, cands[0][f]) for f in fields},
                                                       tile=cur["tile"], config=cur["config"])
        slots[name] = [first] + [c for c in cands if any(c[f] != first[f] for f in fields)]
        meta[name] = (m, n, k, ta, tb, kw)
        print(f"{name}: {len(slots[name])} candidates, held tile {first['tile_id']} split {first['split_k']}", flush=True)

    def measure(assign):
        graph = record(step_calls(vpitch, context, assign), "tune_step", args.schedule)
        for _ in range(2):
            graph.enqueue()
        dev.sync()
        each = graph.time(6)
        graph.destroy()
        return statistics.median(each)

    assign, best, log = K.tune_in_context(slots, measure, verbose=True)
    for what, plan, t in log:
        print(f"  {what}: {plan} -> {t * 1e3:.4f} ms", flush=True)
    cache = K._load_cache()
    for name, e in assign.items():
        m, n, k, ta, tb, kw = meta[name]
        cache[K.tune_key(dev.name, m, n, k, ta, tb, DTYPE, context=context, **kw)] = dict(
            e, context=context, step_ms=round(best * 1e3, 4))
    K._save_cache(cache)
    print(json.dumps({"context": context, "ms_per_step": round(best * 1e3, 4),
                      "plans": {nm: [e[f] for f in fields] for nm, e in assign.items()}}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the dense-head step and the other workloads (square, decoder, skinny)")
    ap.add_argument("--warm-seconds", type=float, default=2.0,
                    help="sustained GEMM load before anything is timed (kernels.py:353-381)")
    ap.add_argument("--eager", action="store_true", help="enqueue GEMMs one by one instead of replaying a graph")
    ap.add_argument("--schedule", default="dw-stream",
                    choices=("dw-stream", "in-order", "dw-stream-waits", "pairs", "passes"),
                    help="how the step's GEMMs are given to the device.  dw-stream (default): forward, dX, dW "
                         "of each linear in turn, every dW GEMM on the library's second stream, which is forked "
                         "once at the start of the step and joined once at its end - a weight gradient is "
                         "needed by nothing before the optimiser (autograd.py:218-227).  in-order: every GEMM "
                         "behind the previous one on one stream.  dw-stream-waits: like dw-stream, but the second "
                         "stream waits, before every dW GEMM, for what the main stream has been given up to "
                         "there.  pairs: dX and dW of a linear side by side, forked and joined per pair.  passes: "
                         "the forward pass, then the backward pass with a layer's dW GEMMs on the second stream "
                         "beside the next layer's dX chain")
    ap.add_argument("--tune-step", action="store_true",
                    help="no benchmark line: choose the plan of every GEMM of the step by what the whole step "
                         "takes under --schedule (kernels.tune_in_context) and write the picks to the tuner's "
                         "cache (VKGRAD_AMD_TUNE_CACHE) under the schedule's context")
    ap.add_argument("--dense-head", action="store_true",
                    help="row pitch of logits/dlogits = 50257 exactly (rows then start at odd addresses) instead of "
                         "the next multiple of 64")
    ap.add_argument("--pmc-pass", action="store_true",
                    help="for a counter run under rocprofv3 --pmc: 3 launches of a cast kernel of known size "
                         "(calibration), then every distinct GEMM of the step twice, eagerly; prints the dispatch "
                         "order instead of the benchmark line")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the path has no multi-GPU part); run with --gpus 1")

    from vkgrad_amd.vk import Device
    from vkgrad_amd.kernels import warmup

    dev = Device()
    rng = np.random.default_rng(1)

    # Operands: per linear one activation X, one weight W (out x in) and one
    # upstream gradient dY; three rotating sets so that consecutive layers never
    # reuse a buffer that may still sit in the 256 MB last-level cache.
    NSET = 3
    sets = []
    for s in range(NSET):
        bufs = {}
        for name, fin, fout in LINEARS:
            x = dev.buffer(ROWS * fin * 2, "device")
            w = dev.buffer(fout * fin * 2, "device")
            dy = dev.buffer(ROWS * fout * 2, "device")
            fill_bf16(dev, x, ROWS * fin, rng, 1.0)
            fill_bf16(dev, w, fout * fin, rng, 0.02)
            fill_bf16(dev, dy, ROWS * fout, rng, 1.0)
            bufs[name] = dict(x=x, w=w, dy=dy, y=dev.buffer(ROWS * fout * 4, "device"),
                              dx=dev.buffer(ROWS * fin * 4, "device"), dw=dev.buffer(fout * fin * 4, "device"))
        sets.append(bufs)
    # logits / dlogits: N = 50257 columns are computed and counted; see head_pitch()
    vpitch = head_pitch(args.dense_head)
    vmax = head_pitch(False)
    head = dict(x=dev.buffer(ROWS * D * 2, "device"), w=dev.buffer(VOCAB * D * 2, "device"),
                dy=dev.buffer(ROWS * vmax * 2, "device"), y=dev.buffer(ROWS * vmax * 4, "device"),
                dx=dev.buffer(ROWS * D * 4, "device"), dw=dev.buffer(VOCAB * D * 4, "device"))
    fill_bf16(dev, head["x"], ROWS * D, rng, 1.0)
    fill_bf16(dev, head["w"], VOCAB * D, rng, 0.02)
    fill_bf16(dev, head["dy"], ROWS * vmax, rng, 1.0)

    mms = {}

    def mm_for(name, layout, m, n, k, vp, context, entry=None):
        """The step's Matmul for one GEMM: the table's plan for the context, or the plan `entry`
        names (the step tuner's candidates)."""
        kw = pitches_for(name, vp)
        tag = None if entry is None else (entry["tile_id"], entry["split_k"], entry["atomic_split"],
                                          entry["group_m"], entry["xcd_rotate"])
        key = (layout, m, n, k, tuple(sorted(kw.items())), context, tag)
        if key not in mms:
            if entry is None:
                mms[key] = plan_for(dev, name, layout, m, n, k, vp, context)[0]
            else:
                from vkgrad_amd.kernels import matmul_from_entry
                mms[key] = matmul_from_entry(dev, entry, *LAYOUT_FLAGS[layout], DTYPE)
        return mms[key], kw

    role_bufs = {"fwd": ("x", "w", "y"), "dX": ("dy", "w", "dx"), "dW": ("dy", "x", "dw")}

    def step_calls(vp, context, plans=None):
        """Every GEMM of one step in order: (mm, a, b, c, m, n, k, pitches); plans: {GEMM name:
        table entry} overrides the table."""
        shapes = {nm: (lay, m, n, k) for nm, lay, m, n, k, _ in gemm_list()}
        plans = plans or {}
        calls = []
        for layer in range(LAYERS):
            b = sets[layer % NSET]
            for name, _, _ in LINEARS:
                for role in ("fwd", "dX", "dW"):
                    lay, m, n, k = shapes[f"{name}.{role}"]
                    mm, kw = mm_for(f"{name}.{role}", lay, m, n, k, vp, context, plans.get(f"{name}.{role}"))
                    calls.append((mm,) + tuple(b[name][x] for x in role_bufs[role]) + (m, n, k, kw))
        for role in ("fwd", "dX", "dW"):
            lay, m, n, k = shapes[f"head.{role}"]
            mm, kw = mm_for(f"head.{role}", lay, m, n, k, vp, context, plans.get(f"head.{role}"))
            calls.append((mm,) + tuple(head[x] for x in role_bufs[role]) + (m, n, k, kw))
        return calls

    context = context_of(args.schedule)
    calls = step_calls(vpitch, context)
    step_flops = sum(2.0 * c[4] * c[5] * c[6] for c in calls)

    if args.pmc_pass:
        from vkgrad_amd.kernels import make_kernels
        K = make_kernels(dev, DTYPE)
        ncal = 1 << 26
        src, dst = dev.buffer(ncal * 4, "device"), dev.buffer(ncal * 2, "device")
        K["zero"]([src], ncal)
        order = []
        for _ in range(3):
            K["cast16"]([src, dst], ncal)
            order.append({"kernel": "k_cast16", "fetch_bytes": ncal * 4, "write_bytes": ncal * 2})
        seen = set()
        for mm, a, b, c, m, n, k, kw in calls:
            key = (id(mm), m, n, k)
            if key in seen:
                continue
            seen.add(key)
            tile, split, gm = mm.plan(m, n, k, **kw)
            probe = dev.graph("count")          # kernel launches this call stands for
            mm(a, b, c, m, n, k, graph=probe, **kw)
            probe.finish()
            launches = probe.kernel_count()
            probe.destroy()
            for _ in range(2):
                mm(a, b, c, m, n, k, **kw)
                order.append({"gemm": f"{'NT' if mm.trans_b else ('TN' if mm.trans_a else 'NN')} {m}x{n}x{k}",
                              "tile": tile, "split_k": split, "kernel_launches": launches,
                              "algorithmic_bytes": 2 * (m * k + k * n) + 4 * m * n})
        dev.sync()
        print(json.dumps({"dispatch_order": order}))
        dev.destroy()
        return

    def schedule_of(calls, schedule):
        """One step as a list of ("gemm", call, on_side_stream) | ("fork",) | ("join",): fork lets
        the library's second stream wait for what the main stream has been given so far, join
        lets the main stream wait for the second.  calls holds (fwd, dX, dW) per linear, the LM
        head last."""
        triples = [calls[i:i + 3] for i in range(0, len(calls), 3)]
        if schedule == "in-order":
            return [("gemm", c, False) for c in calls]
        if schedule in ("dw-stream", "dw-stream-waits"):
            out = [("fork",)] if schedule == "dw-stream" else []
            for fwd, dx, dw in triples:
                out += [("gemm", fwd, False), ("gemm", dx, False)]
                if schedule == "dw-stream-waits":
                    out.append(("fork",))
                out.append(("gemm", dw, True))
            return out + [("join",)]
        if schedule == "pairs":
            out = []
            for fwd, dx, dw in triples:
                out += [("gemm", fwd, False), ("fork",), ("gemm", dx, False), ("gemm", dw, True), ("join",)]
            return out
        # passes: forward of layer 0 .. 11 and the head, then backward from the head down; the dW
        # GEMMs of a layer go to the second stream once that layer's dX chain has been given to
        # the main stream.  (The head's two backward products stay on the main stream: each fills
        # the chip with resident workgroups and two such kernels only take CUs from each other.)
        out = [("gemm", fwd, False) for fwd, _, _ in triples]
        out += [("gemm", triples[-1][1], False), ("gemm", triples[-1][2], False)]
        for l in reversed(range(LAYERS)):
            g = triples[l * len(LINEARS):(l + 1) * len(LINEARS)][::-1]
            out += [("gemm", dx, False) for _, dx, _ in g]
            out.append(("fork",))
            out += [("gemm", dw, True) for _, _, dw in g]
        return out + [("join",)]

    def record(calls, name, schedule):
        graph = dev.graph(name)
        for item in schedule_of(calls, schedule):
            if item[0] == "fork":
                graph.fork()
            elif item[0] == "join":
                graph.join()
            else:
                mm, a, b, c, m, n, k, kw = item[1]
                mm(a, b, c, m, n, k, graph=graph, side=item[2], **kw)
        return graph.finish()

    def run_eager(calls, schedule):
        for item in schedule_of(calls, schedule):
            if item[0] == "fork":
                dev.side_fork()
            elif item[0] == "join":
                dev.side_join()
            else:
                mm, a, b, c, m, n, k, kw = item[1]
                mm.enqueue(a, b, c, m, n, k, side=item[2], **kw)

    def time_steps(calls, name, steps, nwarm, schedule):
        """nwarm untimed steps, then `steps` timed ones: host wall clock around all of them
        (synchronised on both sides) and, for a graph, device time of each replay."""
        if args.eager:
            for _ in range(nwarm):
                run_eager(calls, schedule)
            dev.sync()
            t0 = time.perf_counter()
            for _ in range(steps):
                run_eager(calls, schedule)
            dev.sync()
            return time.perf_counter() - t0, None
        graph = record(calls, name, schedule)
        for _ in range(nwarm):
            graph.enqueue()
        dev.sync()
        t0 = time.perf_counter()
        each = graph.time(steps)
        dev.sync()
        wall = time.perf_counter() - t0
        graph.destroy()
        return wall, each

    # Sustained load first: the chip's clock under matrix load settles over milliseconds, and the
    # first kernels after an idle period run at a different clock than a training loop sees.
    warm_s = warmup(dev, args.warm_seconds, force=True) if args.warm_seconds > 0 else 0.0
    if args.tune_step:
        tune_step(dev, args, vpitch, context, step_calls, record)
        dev.destroy()
        return
    dt, each = time_steps(calls, "gpt2_small_gemms", args.steps, args.warmup, args.schedule)
    ms_per_step = dt / args.steps * 1e3
    tflops = step_flops / (dt / args.steps) / 1e12

    # Per-shape launch durations with HIP events on the library's stream
    # (mg_gemm_time_rotating): median of 5 batches of back-to-back launches that rotate
    # through the step's buffer sets, so a layer GEMM reads its operands from HBM as
    # it does inside the step.
    per_shape = []
    for name, layout, m, n, k, count in gemm_list():
        mm, kw = mm_for(name, layout, m, n, k, vpitch, context)
        is_head = name.startswith("head")
        lin, role = name.split(".")
        groups = [head] if is_head else [s[lin] for s in sets]
        rot = [tuple(g[x] for x in role_bufs[role]) for g in groups]
        t1 = mm.time_rotating(rot, m, n, k, repeat=len(rot), **kw) / len(rot)
        rep = max(1, int(0.02 / max(t1, 1e-6)) // len(rot)) * len(rot)
        secs = sorted(mm.time_rotating(rot, m, n, k, repeat=rep, **kw) / rep for _ in range(5))
        sec = secs[2]
        fl = 2.0 * m * n * k
        by = 2.0 * (m * k + k * n) + 4.0 * m * n
        tile, split, gm = mm.plan(m, n, k, **kw)
        per_shape.append({"gemm": name, "layout": layout, "m": m, "n": n, "k": k, "count": count,
                          "us": round(sec * 1e6, 2), "us_min": round(secs[0] * 1e6, 2), "us_max": round(secs[-1] * 1e6, 2),
                          "tflops": round(fl / sec / 1e12, 1),
                          "frac_mfma": round(fl / sec / 1e12 / PEAK_TFLOPS, 4),
                          "gbps": round(by / sec / 1e9, 1), "tile": tile, "split_k": split})
    # The same GEMMs timed inside the step: the step's calls in order, eagerly, a HIP event behind
    # each (mg_gemm_time_each); per GEMM the median over its occurrences in 5 passes.
    from vkgrad_amd.kernels import time_sequence
    order = [f"{nm}.{role}" for _ in range(LAYERS) for nm, _, _ in LINEARS for role in ("fwd", "dX", "dW")]
    order += ["head.fwd", "head.dX", "head.dW"]
    time_sequence(dev, calls)
    seen, passes = {}, []
    for _ in range(5):
        one_pass = time_sequence(dev, calls)
        passes.append(sum(one_pass))
        for nm, t in zip(order, one_pass):
            seen.setdefault(nm, []).append(t)
    for r in per_shape:
        ts = sorted(seen[r["gemm"]])
        r["us_in_step"] = round(ts[len(ts) // 2] * 1e6, 2)
    in_step_ms = sorted(passes)[2] * 1e3
    # the dominant kernel: the GEMM with the largest share of the step's arithmetic (the LM-head
    # forward; under the two-stream schedule the time of a GEMM alone says nothing about its share)
    dom = max(per_shape, key=lambda r: 2.0 * r["m"] * r["n"] * r["k"] * r["count"])
    mt = MEASURED_TRAFFIC.get(dom["gemm"])
    traffic = None
    if mt and (mt[0], mt[1]) == (dom["tile"], dom["split_k"]) and not args.dense_head:
        traffic = mt[2] + mt[3]
    roofline = {"bound": "mfma", "kernel": f"gemm {dom['gemm']} {dom['layout']} {dom['m']}x{dom['n']}x{dom['k']}",
                "achieved": dom["tflops"], "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(dom["tflops"] / PEAK_TFLOPS, 4), "traffic": traffic,
                "traffic_unit": "bytes per launch (HBM side of L2: fetch + write-back)",
                "algorithmic_bytes": int(2 * (dom["m"] * dom["k"] + dom["k"] * dom["n"]) + 4 * dom["m"] * dom["n"]),
                "flops_per_launch": 2.0 * dom["m"] * dom["n"] * dom["k"]}
    events_ms = sum(r["us"] * r["count"] for r in per_shape) / 1e3

    out = {
        "metric": "GEMM TFLOP/s (fwd+dX+dW) at GPT-2-small shapes, % of fp16 MFMA peak, 1 GPU",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": DTYPE, "data": "synthetic",
        "config": {"workload": "GPT-2-small training GEMMs: d_model 768, 12 layers, 8192 token rows, "
                               "QKV/proj/MLP + tied head 50257, fwd+dX+dW, 147 GEMMs, 6.07 TFLOP per step",
                   "rows": ROWS, "d_model": D, "layers": LAYERS, "vocab": VOCAB, "logits_row_pitch": vpitch,
                   "launch": "eager" if args.eager else "hip-graph replay",
                   "schedule": SCHEDULES[args.schedule]},
        "frac_of_mfma_peak": round(tflops / PEAK_TFLOPS, 4),
        "sustained_warmup_s": round(warm_s, 2),
        "sum_of_event_timed_gemms_ms": round(events_ms, 4),
        "step_with_an_event_after_every_gemm_ms": round(in_step_ms, 4),
        "roofline": roofline,
        "device": {"name": dev.name, "compute_units": dev.compute_units, "clock_khz": dev.clock_khz,
                   "derived_peak_tflops": round(dev.compute_units * 4 * 1024 * dev.clock_khz * 1e3 / 1e12, 1)},
        "per_shape": per_shape,
    }
    if args.schedule != "in-order":
        # the same step with every GEMM behind the previous one on one stream
        idt, _ = time_steps(step_calls(vpitch, context_of("in-order")), "gpt2_small_gemms_in_order", args.steps, args.warmup,
                            "in-order")
        out["in_order"] = {"schedule": SCHEDULES["in-order"], "value": round(step_flops / (idt / args.steps) / 1e12, 2),
                           "unit": "TFLOP/s", "ms_per_step": round(idt / args.steps * 1e3, 4)}
    if each is not None:
        ev = sorted(x * 1e3 for x in each)
        out["ms_per_step_events"] = {"median": round(ev[len(ev) // 2], 4), "min": round(ev[0], 4), "max": round(ev[-1], 4),
                                     "what": "device time of each timed replay, HIP events on the library's stream"}
    if not args.no_extra:
        if not args.dense_head and not args.eager:
            # the same step with logits / dlogits rows exactly 50257 elements apart
            dcalls = step_calls(VOCAB, context)
            ddt, deach = time_steps(dcalls, "gpt2_small_gemms_dense_head", args.steps, args.warmup, args.schedule)
            out["dense_head"] = {"logits_row_pitch": VOCAB, "value": round(step_flops / (ddt / args.steps) / 1e12, 2),
                                 "unit": "TFLOP/s", "ms_per_step": round(ddt / args.steps * 1e3, 4)}
        out["other_workloads"] = other_workloads(dev)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))
    dev.destroy()


if __name__ == "__main__":
    main()
