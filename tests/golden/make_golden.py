"""Writes tests/golden/inputs_sha256.json: SHA-256 of the seeded synthetic inputs of each
benchmark configuration (first rows only, so the check stays fast), so that every machine
can prove it generated the same bytes.  The reference holds no fixtures for this path;
these pin the build's own generator and quantizers against silent drift.

    python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from tattletale_amd import configs as CFG  # noqa: E402

ROWS = 256  # rows of each weight matrix that are hashed


def digest(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def compute() -> dict:
    out = {}
    for name in ("q8_0_gemv", "q4_k_gemv", "q6_k_gemv", "q4_k_gemm_m512", "exl3_gemv"):
        cfg = CFG.CONFIGS[name]
        entry = {"rows": ROWS, "n_in": cfg.n_in, "seed": cfg.seed}
        entry["w_f32"] = digest(CFG.weights_f32(cfg, ROWS))
        entry["x"] = digest(CFG.activations(cfg, min(cfg.m, 4)))
        pk = CFG.packed_weights(cfg, ROWS)
        if isinstance(pk, tuple):
            entry["trellis"], entry["suh"], entry["svh"] = (digest(p) for p in pk)
        else:
            entry["packed"] = digest(pk)
        out[name] = entry
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "inputs_sha256.json")
    with open(path, "w") as f:
        json.dump(compute(), f, indent=1, sort_keys=True)
    print("wrote", path)
