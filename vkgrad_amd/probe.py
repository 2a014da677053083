"""MFMA ceiling of the device on zero and on random operands.

    python -m vkgrad_amd.probe [--dtype bf16] [--seconds 0.5] [--busy-cus 256 192 128 64] [--stream-bytes B]

Prints the rate a register-only MFMA loop sustains on every SIMD of the chip and the shader
clock it ran at, for all-zero operands (the chip holds its boost clock) and for random ones
(the power-managed clock drops).  GEMM throughput on real data is bounded by the second
figure, not by the datasheet peak, which assumes the boost clock.  --busy-cus repeats the
random-operand loop with only that many CUs multiplying (the others idle): the clock each count
allows shows whether the chip is bound by its power budget.
"""

import argparse
import ctypes as C
import json

from . import _lib as L
from .vk import Device, _check


def mfma_ceiling(dev, dtype="bf16", random_operands=True, seconds=0.5, busy_cus=0):
    """(TFLOP/s, GHz) of the register-only MFMA loop on busy_cus CUs (0: all); the iteration
    count is scaled from a short launch so that the timed one lasts about `seconds`."""
    lib, ctx = dev._lib, dev._ctx
    tf, ghz = C.c_double(), C.c_double()
    iters = 20000
    busy = int(busy_cus) if 0 < int(busy_cus) < dev.compute_units else 0
    _check(lib.mg_probe_mfma(ctx, L.DTYPES[dtype], int(bool(random_operands)), iters, busy, C.byref(tf), C.byref(ghz)), "probe")
    per_iter = (busy or dev.compute_units) * 8 * 8 * 32768.0 / (tf.value * 1e12)
    iters = int(max(iters, min(1 << 24, seconds / per_iter)))
    _check(lib.mg_probe_mfma(ctx, L.DTYPES[dtype], int(bool(random_operands)), iters, busy, C.byref(tf), C.byref(ghz)), "probe")
    return tf.value, ghz.value


def stream_floor(dev, nbytes, nsets=8, repeat=400):
    """(read us, fill us) per launch of a kernel that only reads / only writes `nbytes`, shaped
    like the skinny-M stream (24 KB per wavefront, everything in flight), over rotating buffers."""
    r, f = C.c_double(), C.c_double()
    _check(dev._lib.mg_probe_stream(dev._ctx, int(nbytes), int(nsets), int(repeat), C.byref(r), C.byref(f)), "probe")
    return r.value, f.value


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--dtype", default="bf16", choices=("f16", "bf16"))
    ap.add_argument("--seconds", type=float, default=0.5)
    ap.add_argument("--busy-cus", type=int, nargs="*", default=[], metavar="N",
                    help="also run the random-operand loop with only N CUs multiplying")
    ap.add_argument("--stream-bytes", type=int, default=0, metavar="B",
                    help="also time a read-only and a fill-only kernel over B bytes, shaped like the skinny-M "
                         "stream (e.g. 77194752 = the 50257 x 768 f16 weights)")
    args = ap.parse_args(argv)
    dev = Device()
    out = {"device": dev.name, "compute_units": dev.compute_units, "dtype": args.dtype}
    for name, rnd in (("zeros", False), ("random", True), ("zeros_again", False), ("random_again", True)):
        tf, ghz = mfma_ceiling(dev, args.dtype, rnd, args.seconds)
        out[name] = {"tflops": round(tf, 1), "ghz": round(ghz, 3), "of_2500": round(tf / 2500.0, 4)}
        print(f"{name:13s} {tf:8.1f} TFLOP/s at {ghz:.3f} GHz  ({tf / 25.0:.1f} % of 2.5 PFLOP/s)", flush=True)
    for n in args.busy_cus:
        tf, ghz = mfma_ceiling(dev, args.dtype, True, args.seconds, busy_cus=n)
        out[f"random_{n}_cus"] = {"tflops": round(tf, 1), "ghz": round(ghz, 3)}
        print(f"random, {n:3d} CUs busy {tf:8.1f} TFLOP/s at {ghz:.3f} GHz", flush=True)
    if args.stream_bytes:
        r, f = stream_floor(dev, args.stream_bytes)
        out["stream"] = {"bytes": args.stream_bytes, "read_us": round(r, 2), "read_gbps": round(args.stream_bytes / r / 1e3, 1),
                         "fill_us": round(f, 2), "fill_gbps": round(args.stream_bytes / f / 1e3, 1)}
        print(f"stream of {args.stream_bytes} bytes: read-only {r:.2f} us ({args.stream_bytes / r / 1e3:.0f} GB/s), "
              f"fill-only {f:.2f} us ({args.stream_bytes / f / 1e3:.0f} GB/s)", flush=True)
    print(json.dumps(out))
    dev.destroy()


if __name__ == "__main__":
    main()
