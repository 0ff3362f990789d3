"""Writes tests/golden/block_vectors.npz: known-answer vectors for the block-glue kernels
(LayerNorm + modulate, gated residual, tanh-GELU, SiLU, per-head RMS norm), each with its
tangent and gradients, from the numpy fp64 closed forms in oracle/block_oracle.py on seeded
inputs.  The reference ships no fixtures for these expressions; the vectors freeze the
expected numbers for tests/test_block_oracle.py::test_golden_vectors (CPU) and
tests/test_block_gpu.py::test_golden_vectors (GPU).

Run from the repository root:  python tests/golden/make_block_vectors.py
"""
import math
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import block_oracle as bo  # noqa: E402


def main():
    B, L, C = 2, 5, 32
    d = {k: v.numpy().astype(np.float32) for k, v in bo.make_block_inputs(B, L, C, seed=201).items()}
    out = dict(d)
    f64 = {k: v.astype(np.float64) for k, v in d.items()}
    ln = bo.ln_modulate_closed_fp64(f64["x"], f64["shift"], f64["scale"], f64["tx"], f64["tshift"], f64["tscale"], gy=f64["gy"])
    for k, v in ln.items():
        out["ln_modulate." + k] = v
    out["gate_residual.y"] = f64["x"] + f64["gate"] * f64["h"]
    out["gate_residual.ty"] = f64["tx"] + f64["tgate"] * f64["h"] + f64["gate"] * f64["th"]
    out["gate_residual.gh"] = f64["gate"] * f64["gy"]
    out["gate_residual.ggate"] = (f64["gy"] * f64["h"]).sum(1, keepdims=True)
    u = 2.0 * f64["h"]
    a, b = math.sqrt(2.0 / math.pi), 0.044715
    out["gelu.x"] = u.astype(np.float32)
    u = out["gelu.x"].astype(np.float64)
    out["gelu.y"] = 0.5 * u * (1 + np.tanh(a * (u + b * u ** 3)))
    out["gelu.dy"] = bo.gelu_tanh_grad_fp64(u)
    sg = 1 / (1 + np.exp(-u))
    out["silu.y"] = u * sg
    out["silu.dy"] = sg * (1 + u * (1 - sg))
    rng = np.random.default_rng(202)
    xq = rng.standard_normal((2, 3, 2, 24)).astype(np.float32)
    txq = rng.standard_normal((2, 3, 2, 24)).astype(np.float32)
    gyq = rng.standard_normal((2, 3, 2, 24)).astype(np.float32)
    gain = (1 + 0.2 * rng.standard_normal(24)).astype(np.float32)
    out.update({"rms.x": xq, "rms.tx": txq, "rms.gy": gyq, "rms.gain": gain})
    for k, v in bo.rms_norm_closed_fp64(xq, gain, txq, gyq).items():
        out["rms." + k] = v
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "block_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
