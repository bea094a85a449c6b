"""Host-side mixture-of-experts routing (oxillama_amd/moe.py) against the semantics of
MoeFfn::forward, crates/oxillama-arch/src/common/moe.rs:197-248, restated here with plain
Python loops (softmax -> sort descending -> top-k -> renormalise)."""
import math

import numpy as np
import pytest

from oxillama_amd import moe


def loop_route(logits_row, top_k):
    mx = max(logits_row)
    ev = [np.float32(math.exp(np.float32(l) - np.float32(mx))) for l in logits_row]
    tot = np.float32(sum(ev))
    probs = [np.float32(v / tot) for v in ev]
    idx = sorted(range(len(probs)), key=lambda i: -probs[i])[:min(top_k, len(probs))]
    ssum = np.float32(sum(probs[i] for i in idx))
    return idx, [np.float32(probs[i] / ssum) for i in idx]


@pytest.mark.parametrize("n_exp,top_k", [(8, 2), (8, 1), (4, 4), (3, 5), (16, 2)])
def test_route_top_k_matches_loop_restatement(n_exp, top_k):
    rng = np.random.default_rng(n_exp * 10 + top_k)
    logits = rng.random((64, n_exp), dtype=np.float32)
    experts, weights = moe.route_top_k(logits, top_k)
    assert experts.shape == (64, min(top_k, n_exp))
    for t in range(64):
        idx, w = loop_route(list(logits[t]), top_k)
        assert list(experts[t]) == idx
        np.testing.assert_allclose(weights[t], np.array(w, dtype=np.float32), rtol=1e-6)
    np.testing.assert_allclose(weights.sum(axis=1), 1.0, rtol=1e-6)
    assert np.all(np.diff(weights, axis=1) <= 0)  # descending softmax weight (moe.rs:219-225)


def test_single_expert_gets_weight_one():
    # moe.rs tests: one expert, top_k = 1 -> weight 1.0
    experts, weights = moe.route_top_k(np.zeros((3, 1), dtype=np.float32), 1)
    assert np.all(experts == 0) and np.all(weights == 1.0)


def test_top_k_zero_is_rejected():
    with pytest.raises(ValueError):  # moe.rs:167-171
        moe.route_top_k(np.zeros((1, 4), dtype=np.float32), 0)


def test_group_by_expert_is_a_stable_partition():
    rng = np.random.default_rng(3)
    logits = rng.random((64, 8), dtype=np.float32)
    experts, _ = moe.route_top_k(logits, 2)
    offsets, tok, slot = moe.group_by_expert(experts, 8)
    assert offsets[0] == 0 and offsets[-1] == 128 and np.all(np.diff(offsets) >= 0)
    for e in range(8):
        rows = range(offsets[e], offsets[e + 1])
        assert all(experts[tok[r], slot[r]] == e for r in rows)
        assert list(tok[offsets[e]:offsets[e + 1]]) == sorted(tok[offsets[e]:offsets[e + 1]])
    assert sorted(zip(tok.tolist(), slot.tolist())) == [(t, s) for t in range(64) for s in range(2)]
