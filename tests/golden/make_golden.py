"""Writes tests/golden/ref_cpu_vectors.npz from the reference's own C++ CPU scan.

Run in the development container, where the reference checkout exists:

    make -C oracle ref && python tests/golden/make_golden.py

The vectors are produced by csrc/include/sequential_scan_cpu.hpp of the
reference, compiled unchanged through oracle/ref_driver.cpp (no OpenMP).  Inputs
come from a fixed NumPy seed.  Only data is stored: inputs and the reference's
outputs, fp32.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402

SMALL = [(1, 2, 3), (2, 4, 8), (3, 7, 5), (2, 33, 24)]


def main() -> None:
    rng = np.random.default_rng(20240917)
    out = {}
    for bs, seq, d in SMALL:
        key = f"{bs}x{seq}x{d}"
        alpha = rng.standard_normal((bs, seq, d)).astype(np.float32)
        beta = rng.standard_normal((bs, seq, d)).astype(np.float32)
        dout = rng.standard_normal((bs, seq, d)).astype(np.float32)
        h = oracle.ref_scan_fwd(alpha, beta)
        galpha, gbeta = oracle.ref_scan_bwd(alpha, h, dout)
        for name, arr in dict(alpha=alpha, beta=beta, dout=dout, h=h, galpha=galpha, gbeta=gbeta).items():
            out[f"{key}/{name}"] = arr
    # closed-form case of the survey: alpha=0.5, beta=1, dout=1, T=4
    alpha = np.full((2, 4, 8), 0.5, np.float32)
    beta = np.ones((2, 4, 8), np.float32)
    dout = np.ones((2, 4, 8), np.float32)
    h = oracle.ref_scan_fwd(alpha, beta)
    galpha, gbeta = oracle.ref_scan_bwd(alpha, h, dout)
    for name, arr in dict(alpha=alpha, beta=beta, dout=dout, h=h, galpha=galpha, gbeta=gbeta).items():
        out[f"const/{name}"] = arr
    path = os.path.join(HERE, "ref_cpu_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
