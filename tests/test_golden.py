"""The committed checksums of the seeded synthetic inputs and of the oracle's outputs on them
(tests/golden/golden.json) still hold: the benchmark's inputs are the same bytes everywhere, and
the oracle has not drifted.  On the GPU the same inputs must give the checksummed integer sums."""
import json
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_golden as G  # noqa: E402

import oracle as O  # noqa: E402
from oxillama_amd import synth  # noqa: E402

GOLD = json.load(open(os.path.join(HERE, "golden", "golden.json")))


def test_generator_and_oracle_match_committed_checksums(ref):
    assert G.build() == GOLD


@pytest.mark.gpu
@pytest.mark.parametrize("case", GOLD["cases"], ids=lambda c: f"{c['type']}_{c['n_rows']}x{c['n_cols']}")
def test_gpu_integer_sums_match_committed_checksums(hip, ref, case):
    t, n_rows, n_cols = case["type_id"], case["n_rows"], case["n_cols"]
    w = synth.weights(t, 100 + t, n_rows, n_cols)
    a = hip.quantize_f32_to_q8_0(synth.normal_f32(1, n_cols))
    assert G.sha(a) == GOLD["activations"][str(n_cols)]["q8_0"]
    sums = hip.HipKernel(t).block_sums(w, a, n_rows, n_cols)
    assert G.sha(sums) == case["block_sums_i32"]
