"""Times one whole training step of the decoder (forward, loss, backward, AdamW)
recorded as a single HIP graph and replayed - the GEMM numbers restated as
tokens per second.

    python -m vkgrad_amd.gpt_step [--config gpt2-small] [--no-fuse] [--steps 10]

gpt2-small: 12 layers, d_model 768, 12 heads, context 1024, vocabulary 50257
(tied head), 8 sequences per step = 8192 token rows, bf16 operands - the
shapes of the GEMM benchmark.  Token ids and targets are pseudo-random; the
loss of the first replays is printed so a broken step shows (it starts near
ln(vocab) and falls).
"""

import argparse
import json
import statistics
import sys

import numpy as np

CONFIGS = {
    "gpt2-small": dict(B=8, T=1024, D=768, H=12, L=12, vocab=50257, dtype="bf16"),
    "gpt2-small-b4": dict(B=4, T=1024, D=768, H=12, L=12, vocab=50257, dtype="bf16"),
    "tiny": dict(B=2, T=64, D=64, H=4, L=2, vocab=96, dtype="f16"),
}


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--config", default="gpt2-small", choices=sorted(CONFIGS))
    ap.add_argument("--no-fuse", action="store_true", help="one kernel per pass, as the reference schedules it")
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--lr", type=float, default=3e-4)
    args = ap.parse_args(argv)

    from .autograd import AdamW
    from .transformer import GPT, TCtx
    from .vk import Device

    cfg = CONFIGS[args.config]
    dev = Device()
    ctx = TCtx(dev, dtype=cfg["dtype"], fuse=not args.no_fuse)
    try:
        model = GPT(ctx, cfg["B"], cfg["T"], cfg["D"], cfg["H"], cfg["L"], cfg["vocab"], tie=True)
        rows = cfg["B"] * cfg["T"]
        rng = np.random.default_rng(0)
        ids = ctx.buf(rows * 4, "shared")
        tgt = ctx.buf(rows * 4, "shared")
        ids.array(np.uint32, (rows,))[:] = rng.integers(0, cfg["vocab"], rows)
        tgt.array(np.uint32, (rows,))[:] = rng.integers(0, cfg["vocab"], rows)
        ids.flush()
        tgt.flush()
        opt = AdamW(ctx, model.params(), lr=args.lr)
        graph = dev.graph("gpt_step")
        model.record(ids, tgt, graph)
        opt.record(graph)
        graph.finish()
        losses, times = [], []
        for i in range(args.warmup + args.steps):
            opt.advance()
            dt = graph.submit()
            if i < 3 or i == args.warmup + args.steps - 1:
                losses.append(round(model.read_loss(), 4))
            if i >= args.warmup:
                times.append(dt)
        ms = statistics.median(times) * 1e3
        out = dict(config=args.config, fused=not args.no_fuse, dtype=cfg["dtype"], device=dev.name,
                   params=model.n_params(), kernels_per_step=graph.n_dispatch, tokens_per_step=rows,
                   ms_per_step=round(ms, 3), ms_min=round(min(times) * 1e3, 3),
                   tokens_per_s=round(rows / (ms / 1e3), 1), losses=losses)
        print(json.dumps(out), flush=True)
    finally:
        ctx.destroy()
        dev.destroy()
    return 0


if __name__ == "__main__":
    sys.exit(main())
