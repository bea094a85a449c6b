"""Writes tests/golden/golden.json: SHA-256 of what the seeded synthetic generator
(oxillama_amd/synth) produces and of what the CPU oracle computes from it, for small
shapes of every format.  The checksums pin the benchmark's inputs (same bytes on every
box) and catch accidental changes of the oracle; they are data, regenerated only when
the generator or the oracle is changed on purpose:  python tests/golden/make_golden.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle as O  # noqa: E402
from oxillama_amd import synth  # noqa: E402

CASES = [(t, 24, 1024) for t in O.ALL_TYPES] + [(O.Q4_K, 7, 4096), (O.Q6_K, 5, 14336)]


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def build():
    O.load()
    out = {"activations": {}, "cases": []}
    for n in (1024, 4096, 14336):
        x = synth.normal_f32(1, n)
        out["activations"][str(n)] = {"x_f32": sha(x), "q8_0": sha(O.quantize_q8_0(x))}
    for t, n_rows, n_cols in CASES:
        w = synth.weights(t, 100 + t, n_rows, n_cols)
        a = O.quantize_q8_0(synth.normal_f32(1, n_cols))
        y = O.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=O.TIER_AVX2)
        sums = O.block_sums(t, w, a, n_rows, n_cols)
        out["cases"].append({"type": O.NAMES[t], "type_id": int(t), "n_rows": n_rows, "n_cols": n_cols,
                             "weights": sha(w), "fused_avx2_tier_f32": sha(y), "block_sums_i32": sha(sums),
                             "y0": float(y[0]), "sum0": int(sums.reshape(-1)[0])})
    return out


if __name__ == "__main__":
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(build(), f, indent=1)
    print("wrote golden.json")
