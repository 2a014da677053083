"""Achieved HBM bandwidth of the decoder-block row kernels at GPT-2-small shapes
(8 sequences x 1024 tokens, d_model 768, 12 heads, vocabulary 50257, bf16).

    python -m vkgrad_amd.rowbench [--json FILE]

Every kernel is HBM-bound; its algorithmic bytes are each tensor it must read or
write once (masked halves of the attention matrices are not counted as reads:
the kernels never fetch them).  Buffers are rotated over enough sets to overflow
the 256 MB last-level cache, launches are back to back, the median of 5 batches
is reported against the 8 TB/s peak.
"""

import argparse
import json
import statistics
import sys
import time

import numpy as np

B, T, D, H, V = 8, 1024, 768, 12, 50257
VP = (V + 63) // 64 * 64
R, HD, NBH = B * T, D // H, B * H


def cases(W):
    """name -> (kernel, [(buffer bytes, kind)], n, args, algorithmic bytes)"""
    att = NBH * T * T
    tri = att // 2 + NBH * T // 2            # keys <= query
    return [
        ("layernorm", ["f:R*D", "f:D", "f:D", "h:R*D", "f:R", "f:R"], R * W, (D,), R * D * 6 + R * 8),
        ("layernorm_bwd", ["f:R*D", "f:R*D", "f:D", "f:R", "f:R", "f:R*D", "h:R*D", "h:R*D"], R * W, (D,), R * D * 16),
        ("attn_softmax", ["f:att", "h:att"], NBH * T * W, (T, 0.125), tri * 4 + att * 2),
        ("attn_softmax_bwd", ["f:att", "h:att", "h:att"], NBH * T * W, (T, 0.125), tri * 6 + att * 2),
        ("split_qkv", ["f:R*3*D", "f:3*D", "h:R*D", "h:R*D", "h:R*D"], R * D, (D, T, H, HD), R * D * 18),
        ("merge_qkv_grad", ["f:R*D", "f:R*D", "f:R*D", "h:R*3*D"], R * D, (D, T, H, HD), R * D * 18),
        ("merge_heads", ["f:R*D", "h:R*D"], R * D, (D, T, H, HD), R * D * 6),
        ("split_heads", ["f:R*D", "h:R*D"], R * D, (D, T, H, HD), R * D * 6),
        ("residual", ["f:R*D", "f:D", "f:R*D", "f:R*D"], R * D, (D,), R * D * 12),
        ("add", ["f:R*D", "f:R*D", "f:R*D"], R * D, (), R * D * 12),
        ("to16", ["f:R*D", "h:R*D"], R * D, (), R * D * 6),
        ("col_sum_chunk16", ["h:R*4*D", "f:4*D"], 32 * 4 * D, (4 * D, R, 32), R * 4 * D * 2),
        ("softmax_ce", ["f:R*VP", "u:R", "h:R*VP", None, "f:R"], R, (VP, V), R * VP * 6),
    ]


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--json")
    args = ap.parse_args(argv)
    from .tkernels import make_transformer_kernels
    from .vk import Device
    dev = Device()
    TK = make_transformer_kernels(dev, "bf16")
    W = dev.row_subgroup_size
    env = dict(R=R, D=D, att=NBH * T * T, VP=VP)
    rng = np.random.default_rng(0)
    rows = []
    print(f"# row kernels at GPT-2-small shapes on {dev.name}")
    print("| kernel | algorithmic MB | us | GB/s | of 8 TB/s |")
    print("|---|---|---|---|---|", flush=True)
    for name, specs, n, kargs, nbytes in cases(W):
        total = 0
        for sp in specs:
            if sp is not None:
                total += eval(sp[2:], {}, env) * (2 if sp[0] == "h" else 4)
        nsets = max(2, min(6, -(-(600 << 20) // total)))
        sets = []
        for s in range(nsets):
            bufs = []
            for sp in specs:
                if sp is None:
                    bufs.append(None)
                    continue
                count = eval(sp[2:], {}, env)
                b = dev.buffer(count * (2 if sp[0] == "h" else 4), "device")
                if sp[0] == "u":
                    b.upload(rng.integers(0, V, count).astype(np.uint32))
                elif sp[0] == "f" and count <= 4 * D:
                    b.upload(rng.uniform(0.5, 1.5, count).astype(np.float32))
                elif sp[0] == "f":
                    chunk = rng.standard_normal(min(count, 1 << 22)).astype(np.float32)
                    b.upload(np.resize(chunk, count))
                else:
                    b.upload(np.resize(rng.integers(0, 0x3c00, min(count, 1 << 22)).astype(np.uint16), count))
                bufs.append(b)
            sets.append(bufs)
        kern = TK[name]
        lib, ctx = dev._lib, dev._ctx

        def batch(reps):
            t0 = time.perf_counter()
            for i in range(reps):
                bufs = sets[i % nsets]
                ptrs = [None if b is None else b.ptr for b in bufs]
                kern._launch(lib, ctx, ptrs, n, *kargs)
            dev.sync()
            return (time.perf_counter() - t0) / reps

        batch(nsets)
        reps = max(nsets, int(0.02 / max(batch(nsets), 1e-6)) // nsets * nsets)
        t = statistics.median(batch(reps) for _ in range(5))
        gbps = nbytes / t / 1e9
        rows.append(dict(kernel=name, algorithmic_bytes=nbytes, us=round(t * 1e6, 1), gbps=round(gbps, 1),
                         frac_hbm=round(gbps / 8000.0, 4)))
        print(f"| {name} | {nbytes / 1e6:.1f} | {t * 1e6:.1f} | {gbps:.0f} | {gbps / 8000.0:.3f} |", flush=True)
        for bufs in sets:
            for b in bufs:
                if b is not None:
                    b.destroy()
    if args.json:
        with open(args.json, "w") as f:
            json.dump(dict(device=dev.name, rows=rows), f, indent=1)
    dev.destroy()
    return 0


if __name__ == "__main__":
    sys.exit(main())
