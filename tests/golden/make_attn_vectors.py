"""Writes tests/golden/attn_vectors.npz: known-answer vectors for the attention path.

The reference repository ships no fixtures for this path (its only test draws unseeded
random inputs), so these vectors are produced here, once, from the numpy fp64 closed
forms in oracle/attn_oracle.py::closed_form_fp64 (the textbook formulas, themselves
pinned by finite differences in tests/test_oracle.py) on seeded inputs.  They freeze the
expected numbers: a later change to the oracle or to the kernels that moves any of them
is caught by tests/test_oracle.py::test_golden_vectors and
tests/test_attn_gpu.py::test_golden_vectors.

Run from the repository root:  python tests/golden/make_attn_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attn_oracle as ao  # noqa: E402

CASES = {"d64": (1, 8, 2, 64, 101), "d72_cross": (1, 8, 2, 72, 102)}   # name: (B, L, H, D, seed); d72_cross uses Lkv = 12


def main():
    out = {}
    for name, (B, L, H, D, seed) in CASES.items():
        Lkv = 12 if name.endswith("cross") else None
        q, k, v, tq, tk, tv, do = ao.make_inputs(B, L, H, D, seed, Lkv=Lkv)
        cf = ao.closed_form_fp64(q, k, v, tq, tk, tv, do)
        for key, t in zip(("q", "k", "v", "tq", "tk", "tv", "dout"), (q, k, v, tq, tk, tv, do)):
            out[f"{name}.{key}"] = t.numpy().astype(np.float32)
        for key in ("o", "to", "lse", "mu", "dq", "dk", "dv"):
            out[f"{name}.{key}"] = np.asarray(cf[key], dtype=np.float64)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attn_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
