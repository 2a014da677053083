"""Writes tests/golden/gemm_golden.npz: small GEMM cases with the oracle's answer.

The reference ships no data fixtures for this path (its tests regenerate inputs
from numpy seeds), so these vectors restate the reference's own recipe
(test_kernels.py:10-16: default_rng(seed), standard_normal, A then B) at cropped
sizes, in all three layouts and both input types, with and without the bias and
beta=1 clauses.  Each expected C is the numpy oracle's, cross-checked here
against the independent C triple loop with float64 accumulation before it is
written.  Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import ref_gemm as O          # noqa: E402
from tests.test_oracle import c_gemm      # noqa: E402

LAYOUTS = {"NN": (False, False), "NT": (False, True), "TN": (True, False)}


def main():
    import ctypes as C
    import subprocess
    so = os.path.join(ROOT, "oracle", "libref_gemm.so")
    subprocess.run(["gcc", "-O2", "-shared", "-fPIC", "-o", so, os.path.join(ROOT, "oracle", "ref_gemm.c")], check=True)
    lib = C.CDLL(so)
    lib.ref_gemm_scalar.restype = C.c_int
    lib.ref_gemm_scalar.argtypes = [C.c_int] * 4 + [C.c_int64] * 3 + [C.c_void_p, C.c_int64, C.c_void_p, C.c_int64,
                                                                   C.c_void_p, C.c_int64, C.c_void_p, C.c_int]
    out = {}
    shapes = [(32, 32, 32), (24, 40, 48), (33, 17, 65)]
    for si, (m, n, k) in enumerate(shapes):
        for layout, (ta, tb) in LAYOUTS.items():
            for dtype in ("f16", "bf16"):
                for extra in (False, True):
                    name = f"s{si}-{layout}-{dtype}-{'be' if extra else 'plain'}"
                    a, b = O.make_operands(m, n, k, ta, tb, dtype, seed=si)
                    rng = np.random.default_rng(100 + si)
                    bias = (rng.standard_normal(n) * 2 + 1).astype(np.float32) if extra else None
                    c0 = rng.standard_normal((m, n)).astype(np.float32) if extra else None
                    c = O.ref_gemm(a, b, ta, tb, dtype, bias, c0)
                    ref = c_gemm(lib, a, b, m, n, k, ta, tb, dtype, 1, bias, c0)
                    assert O.err_fro(c, ref) < 1e-6, name
                    out[name + "_a"] = np.ascontiguousarray(a).view(np.uint16)
                    out[name + "_b"] = np.ascontiguousarray(b).view(np.uint16)
                    out[name + "_c"] = c
                    if extra:
                        out[name + "_bias"] = bias
                        out[name + "_c0"] = c0
    path = os.path.join(ROOT, "tests", "golden", "gemm_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
