"""Timing sweeps over the GEMM shapes of the training path.

The counterpart of the reference's bench/matmul_sweep.py (shape list and
per-shape timing: bench/matmul_sweep.py:22-53, tuned pick per shape: 81-92),
for the workloads this library is sized for:

    square   M = N = K in {1024, 2048, 4096, 8192}, f16, layouts NT / NN / TN
    decoder  d_model 1024, 24 layers, 16384 token rows, LM head 50257, bf16;
             forward, dX and dW of every linear, dW accumulated (beta = 1) over
             4 micro-batches (the first one overwrites)
    charlm   d_model 256, vocabulary 96, 16384 token rows, f16
    skinny   M in {1, 7, 63, 129, 4097} x K = 768 x N in {96, 2304, 50257},
             f16, NT with the fused bias epilogue (memory-bound: GB/s)

    python -m vkgrad_amd.sweep --config square [--tune] [--json FILE]

Per case: operands are pseudo-random (zeros run at a higher clock and
overstate), several buffer sets are rotated when one set would fit the 256 MB
last-level cache, and the median of 7 batches of back-to-back launches, each
lasting >= 20 ms between two HIP events, is taken.  FLOP are algorithmic (2 M N K), bytes
are each operand once (2 (MK + KN) + 4 MN, + 4 MN when C is read, + 4 N bias).
Results are not checked here; parity is the test suite's job.
"""

import argparse
import json
import math
import statistics
import sys

LAYOUT_FLAGS = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}
VOCAB = 50257


def linear_gemms(name, rows, fin, fout, dtype, count, accumulate_dw=False, ypitch=None):
    """The three GEMMs of one linear layer in (M, N, K) form (autograd.py:186-228):
    forward Y = X W^T (NT), dX = dY W (NN), dW = dY^T X (TN)."""
    yp = {} if ypitch is None else {"ldc": ypitch}
    dp = {} if ypitch is None else {"lda": ypitch}
    base = dict(dtype=dtype, bias=False, accumulate=False, count=count)
    return [
        dict(base, name=name + ".fwd", layout="NT", m=rows, n=fout, k=fin, pitch=yp),
        dict(base, name=name + ".dX", layout="NN", m=rows, n=fin, k=fout, pitch=dp),
        dict(base, name=name + ".dW", layout="TN", m=fout, n=fin, k=rows, pitch=dp,
             accumulate=accumulate_dw),
    ]


def cases_for(config):
    out = []
    if config == "square":
        for n in (1024, 2048, 4096, 8192):
            for lay in ("NT", "NN", "TN"):
                out.append(dict(name=f"{lay} {n}^3", layout=lay, m=n, n=n, k=n, dtype="f16", bias=False,
                                accumulate=False, count=1, pitch={}))
    elif config == "decoder":
        rows, d, layers = 16384, 1024, 24
        vpitch = (VOCAB + 63) // 64 * 64
        micro = 4
        linears = [(nm, fin, fout, layers, None) for nm, fin, fout in
                   (("qkv", d, 3 * d), ("proj", d, d), ("fc1", d, 4 * d), ("fc2", 4 * d, d))]
        linears.append(("head", d, VOCAB, 1, vpitch))
        for nm, fin, fout, mult, yp in linears:
            fwd, dx, dw = linear_gemms(nm, rows, fin, fout, "bf16", mult * micro, ypitch=yp)
            # dW overwrites on the first micro-batch and adds (beta = 1) on the other three
            dw_first = dict(dw, name=nm + ".dW first", count=mult)
            dw_acc = dict(dw, name=nm + ".dW", accumulate=True, count=mult * (micro - 1))
            out += [fwd, dx, dw_first, dw_acc]
    elif config == "charlm":
        rows, d = 16384, 256
        for nm, fin, fout in (("qkv", d, 3 * d), ("proj", d, d), ("fc1", d, 4 * d), ("fc2", 4 * d, d),
                              ("head", d, 96)):
            out += linear_gemms(nm, rows, fin, fout, "f16", 1)
    elif config == "skinny":
        for n in (96, 2304, VOCAB):
            for m in (1, 7, 63, 129, 4097):
                out.append(dict(name=f"NT+bias {m}x{n}x768", layout="NT", m=m, n=n, k=768, dtype="f16", bias=True,
                                accumulate=False, count=1, pitch={}))
    else:
        raise SystemExit(f"unknown config {config!r}")
    return out


def algorithmic_bytes(c):
    m, n, k = c["m"], c["n"], c["k"]
    return 2 * (m * k + k * n) + 4 * m * n * (2 if c["accumulate"] else 1) + (4 * n if c["bias"] else 0)


def read_bytes(c):
    """What one launch reads: the operands, and C with beta = 1."""
    m, n, k = c["m"], c["n"], c["k"]
    return 2 * (m * k + k * n) + (4 * m * n if c["accumulate"] else 0)


class Runner:
    def __init__(self, tune=False, warm=True, dev=None):
        from . import kernels
        from .vk import Device
        self.K = kernels
        self.dev = dev if dev is not None else Device()
        self.tune = tune
        self.fill = {}
        if warm:
            kernels.warmup(self.dev, 2.0)

    def _fill(self, dtype, buf, n, seed):
        if dtype not in self.fill:
            self.fill[dtype] = self.K.make_kernels(self.dev, dtype)["fill_uniform16"]
        self.fill[dtype]([buf], n, seed)

    def matmul_for(self, c):
        K, dev = self.K, self.dev
        ta, tb = LAYOUT_FLAGS[c["layout"]]
        if self.tune and K.lookup_tuned(dev.name, c["m"], c["n"], c["k"], ta, tb, c["dtype"],
                                        accumulate=c["accumulate"], **c["pitch"]) is None:
            mm, e = K.autotune_matmul(dev, c["m"], c["n"], c["k"], ta, tb, dtype=c["dtype"],
                                      accumulate=c["accumulate"], **c["pitch"])
            return mm, "tuned now"
        return K.tuned_matmul(dev, c["m"], c["n"], c["k"], ta, tb, c["dtype"], accumulate=c["accumulate"],
                              **c["pitch"])

    def allocate(self, c, nsets):
        dev = self.dev
        m, n, k = c["m"], c["n"], c["k"]
        ta, tb = LAYOUT_FLAGS[c["layout"]]
        pa = c["pitch"].get("lda", m if ta else k)
        pb = c["pitch"].get("ldb", k if tb else n)
        pc = c["pitch"].get("ldc", n)
        ea, eb = (k if ta else m) * pa, (n if tb else k) * pb
        sets, outs = [], []
        for s in range(nsets):
            a = dev.buffer(ea * 2 + 64, "device")
            b = dev.buffer(eb * 2 + 64, "device")
            # results that are only written share three buffers (they do not displace operands
            # in the last-level cache); with beta = 1 they are operands too
            if c["accumulate"] or s < 3:
                outs.append(dev.buffer(m * pc * 4, "device"))
            cc = outs[s % len(outs)]
            self._fill(c["dtype"], a, ea, 11 + 2 * s)
            self._fill(c["dtype"], b, eb, 12 + 2 * s)
            bias = None
            if c["bias"]:
                import numpy as np
                bias = dev.buffer(n * 4, "device")
                bias.upload(np.linspace(-1.0, 1.0, n, dtype=np.float32))
            sets.append((a, b, cc, bias))
        return sets

    def time_case(self, c, samples=7, min_seconds=0.02, trace_launches=0):
        mm, how = self.matmul_for(c)
        nsets = self.K.buffer_sets_for(read_bytes(c))
        sets = self.allocate(c, nsets)
        m, n, k = c["m"], c["n"], c["k"]
        kw = dict(c["pitch"])

        try:
            tile, split, gm = mm.plan(m, n, k, **kw)
            if trace_launches:
                mm.time_rotating(sets, m, n, k, repeat=trace_launches, accumulate=c["accumulate"], **kw)
                return dict(c, tile=self.K.CONFIGS[tile]["name"], split_k=split, sets=nsets, plan=how)
            t1 = mm.time_rotating(sets, m, n, k, repeat=nsets, accumulate=c["accumulate"], **kw) / nsets
            reps = int(min(4000, max(nsets, math.ceil(min_seconds / max(t1, 1e-7)))))
            reps = (reps + nsets - 1) // nsets * nsets
            ts = [mm.time_rotating(sets, m, n, k, repeat=reps, accumulate=c["accumulate"], **kw) / reps
                  for _ in range(samples)]
        finally:
            mm.destroy()
            for x in {id(b): b for st in sets for b in st if b is not None}.values():
                x.destroy()
        t = statistics.median(ts)
        fl = 2.0 * m * n * k
        by = algorithmic_bytes(c)
        return dict(c, us=round(t * 1e6, 2), us_min=round(min(ts) * 1e6, 2), tflops=round(fl / t / 1e12, 2),
                    frac_mfma=round(fl / t / 2.5e15, 4), gbps=round(by / t / 1e9, 1), frac_hbm=round(by / t / 8e12, 4),
                    tile=self.K.CONFIGS[tile]["name"], split_k=split, group_m=gm, sets=nsets, launches=reps, plan=how)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--config", required=True, choices=("square", "decoder", "charlm", "skinny"))
    ap.add_argument("--tune", action="store_true", help="autotune shapes the tuned table does not hold")
    ap.add_argument("--json", help="also write the rows to this file")
    ap.add_argument("--trace-pass", type=int, default=0, metavar="N",
                    help="no timing: launch every case N times in listed order (for a kernel trace)")
    args = ap.parse_args(argv)
    r = Runner(tune=args.tune, warm=not args.trace_pass)
    rows = []
    print(f"# {args.config} on {r.dev.name}", flush=True)
    if args.trace_pass:
        for i, c in enumerate(cases_for(args.config)):
            row = r.time_case(c, trace_launches=args.trace_pass)
            print(f"trace {i} {c['name']} | {row['tile']} split {row['split_k']} | {args.trace_pass} launches", flush=True)
        r.dev.sync()
        r.dev.destroy()
        return 0
    print("| case | dtype | tile | split_k | plan | sets | us | TFLOP/s | of 2.5 PFLOP/s | GB/s | of 8 TB/s | count |")
    print("|---|---|---|---|---|---|---|---|---|---|---|---|", flush=True)
    for c in cases_for(args.config):
        row = r.time_case(c)
        rows.append(row)
        print(f"| {row['name']}{' b1' if row['accumulate'] else ''} {row['layout']} {row['m']}x{row['n']}x{row['k']} "
              f"| {row['dtype']} | {row['tile']} | {row['split_k']} | {row['plan']} | {row['sets']} | {row['us']} "
              f"| {row['tflops']} | {row['frac_mfma']:.3f} | {row['gbps']} | {row['frac_hbm']:.3f} | {row['count']} |", flush=True)
    tot_us = sum(x["us"] * x["count"] for x in rows)
    tot_fl = sum(2.0 * x["m"] * x["n"] * x["k"] * x["count"] for x in rows)
    summary = dict(config=args.config, device=r.dev.name, gemms=sum(x["count"] for x in rows),
                   total_ms=round(tot_us / 1e3, 3), tflop=round(tot_fl / 1e12, 3),
                   tflops=round(tot_fl / tot_us / 1e6, 1), frac_mfma=round(tot_fl / tot_us / 1e6 / 2500.0, 4))
    print(json.dumps(summary), flush=True)
    if args.json:
        with open(args.json, "w") as f:
            json.dump(dict(summary=summary, rows=rows), f, indent=1)
    r.dev.destroy()
    return 0


if __name__ == "__main__":
    sys.exit(main())
