#!/usr/bin/env python3
"""Writes tests/golden/tq8_cases.npz from the CPU oracle (oracle/tq_oracle.c).

The reference ships no tensor fixtures or expected outputs for this path (its tests build
inputs with an LCG and compare GPU against CPU), so the vectors come from the restated
reference algorithm, which tests/test_oracle_pins.py pins independently.  Inputs use the
reference tests' LCG (tests/integration/test_linear.cpp:26-34).  Run from the repo root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as o  # noqa: E402

CASES = [
    # name, out, in, block, primary_bits, residual_bits, shared_rotation, batch
    ("shared_8x128_b128", 8, 128, 128, 4, 4, True, 2),
    ("dual_8x128_b128", 8, 128, 128, 4, 4, False, 2),
    ("primary_16x512_b256", 16, 512, 256, 4, 0, False, 1),
    ("shared_16x512_b512", 16, 512, 512, 4, 4, True, 3),
    ("dual_16x512_b256", 16, 512, 256, 4, 4, False, 1),
    ("shared_24x384_b128", 24, 384, 128, 4, 4, True, 1),
    ("shared53_8x128_b128", 8, 128, 128, 5, 3, True, 1),
    ("dual53_8x128_b128", 8, 128, 128, 5, 3, False, 1),
]


def main():
    out = {}
    for name, rows, cols, bs, pb, rb, shared, batch in CASES:
        w = o.lcg_matrix(rows, cols, 42)
        x = o.lcg_matrix(batch, cols, 99)
        cbp = o.generate_codebook(pb)
        cbr = o.generate_codebook(rb if rb else 4)
        qw = o.quantize_weight(w, cbp, cbr, pb, rb, bs, shared)
        W = o.dequantize_weight_cpu(qw, cbp, cbr, bs)
        y = o.matmul_xwT(x, W, acc_double=True)
        for key, val in dict(pp=qw.packed_primary, pr=qw.packed_residual, norms=qw.norms, seeds=qw.seeds,
                             cbp=cbp.centroids, cbr=cbr.centroids, x=x, W=W, y=y,
                             bs=np.array([bs], np.uint32)).items():
            out[f"{name}/{key}"] = val
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tq8_cases.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(CASES)} cases, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
