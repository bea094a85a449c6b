"""The oracle's restatement of the sampler after its candidate list (sample_with_rng from the greedy shortcut on,
crates/oxillama-runtime/src/sampling/mod.rs:487-564, softmax_candidates :617-638, Xorshift64 :669-690), pinned by the
reference's own tests (mod.rs:707-955: they hold properties, not sequences), by an independent big-integer generator,
and by an independent float64 recomputation of the probabilities and of the draw."""
import math

import numpy as np
import pytest

import oracle as O

MASK = (1 << 64) - 1


def py_xorshift(state):
    x = state
    x ^= (x << 13) & MASK
    x ^= x >> 7
    x ^= (x << 17) & MASK
    return x


def test_xorshift64_against_big_integers():
    assert O.xorshift64_seed(0) == 0x517CC1B727220A95  # Xorshift64::new, mod.rs:670-675
    assert O.xorshift64_seed(42) == 42
    for seed in (1, 42, 12345, 0xDEADBEEFCAFEBABE, 0x517CC1B727220A95, MASK):
        st = seed
        for _ in range(200):
            want = py_xorshift(st)
            v, st2 = O.xorshift64_next_f32(st)
            assert st2 == want
            assert v == (want >> 40) / float(1 << 24)  # exact: 24 bits over 2^24
            st = st2


def test_xorshift_range_as_the_reference_tests_it():  # mod.rs:859-865
    st = O.xorshift64_seed(12345)
    for _ in range(10000):
        v, st = O.xorshift64_next_f32(st)
        assert 0.0 <= v < 1.0


def sample_full(logits, temperature=1.0, top_k=0, top_p=1.0, min_p=0.0, state=None, seed=None):
    """sample() of the reference over a whole logit vector: candidates by the oracle's top-k (all of them for top_k = 0)."""
    logits = np.asarray(logits, dtype=np.float32)
    if logits.size == 0:
        return 0, state
    if state is None:
        state = O.xorshift64_seed(0xDEADBEEFCAFEBABE if seed is None else seed)
    k = logits.size if top_k == 0 or top_k >= logits.size else top_k
    vals, idx = O.topk(logits, k)
    tok, state, _, _ = O.sample_candidates(vals, idx, temperature, min_p, top_p, state)
    return tok, state


def test_reference_sampler_cases():
    # test_greedy_sampling, test_temperature_zero_is_greedy, test_top_k_1_is_greedy (mod.rs:709-745)
    assert sample_full([0.1, 0.5, 0.3, 0.8, 0.2], temperature=0.0)[0] == 3
    assert sample_full([1.0, 5.0, 3.0, 2.0], temperature=0.0)[0] == 1
    assert sample_full([1.0, 5.0, 3.0, 2.0], temperature=1.0, top_k=1)[0] == 1
    assert sample_full([], temperature=0.0)[0] == 0  # test_empty_logits
    # test_top_p_filters_low_prob (mod.rs:771-786)
    assert sample_full([100.0, 0.0, 0.0, 0.0, 0.0], top_p=0.5, seed=123)[0] == 0
    # test_min_p_filtering (mod.rs:839-856): 100 draws of one sampler
    st = O.xorshift64_seed(42)
    for _ in range(100):
        tok, st = sample_full([10.0, -10.0, -10.0, -10.0], min_p=0.1, state=st)
        assert tok == 0
    # test_seeded_determinism (mod.rs:748-768)
    a = b = O.xorshift64_seed(42)
    for _ in range(10):
        ta, a = sample_full([1.0, 2.0, 3.0, 2.0, 1.0], state=a)
        tb, b = sample_full([1.0, 2.0, 3.0, 2.0, 1.0], state=b)
        assert ta == tb and a == b
    # test_sampling_distribution (mod.rs:809-836)
    st, counts = O.xorshift64_seed(999), [0] * 4
    for _ in range(1000):
        tok, st = sample_full([2.0, 2.0, 2.0, 2.0], state=st)
        counts[tok] += 1
    assert all(100 < c < 400 for c in counts), counts
    # test_softmax_candidates_basic (mod.rs:945-953)
    _, _, probs, n = O.sample_candidates([0.0, 0.0, 0.0], [0, 1, 2], 1.0, 0.0, 1.0, 1)
    assert n == 3 and np.all(np.abs(probs - 1.0 / 3.0) < 0.01)


def reference_in_float64(vals, temperature, min_p, top_p):
    """The same steps in float64 (no shared code with the oracle): final probabilities and their count."""
    v = np.asarray(vals, dtype=np.float64) * (1.0 / temperature if temperature != 1.0 else 1.0)
    e = np.exp(v - v.max())
    p = e / e.sum()
    if min_p > 0.0:
        p = p[p >= min_p * p[0]]
    if top_p < 1.0:
        c = np.cumsum(p)
        p = p[:int(np.argmax(c >= top_p)) + 1] if np.any(c >= top_p) else p
    return p / p.sum()


@pytest.mark.parametrize("k", [2, 5, 40, 256])
@pytest.mark.parametrize("cfg", [(1.0, 0.0, 1.0), (0.7, 0.0, 0.9), (1.5, 0.05, 1.0), (0.9, 0.02, 0.5), (2.0, 0.0, 0.95)],
                         ids=lambda c: "T%g_minp%g_topp%g" % c)
def test_probabilities_and_draw_against_float64(k, cfg):
    temperature, min_p, top_p = cfg
    rng = np.random.default_rng(1000 + k)
    state = O.xorshift64_seed(77 + k)
    checked = 0
    for trial in range(40):
        vals = np.sort((rng.standard_normal(k) * 3.0).astype(np.float32))[::-1].copy()
        idx = rng.permutation(100000)[:k].astype(np.uint32)
        before = state
        tok, state, probs, n = O.sample_candidates(vals, idx, temperature, min_p, top_p, state)
        want = reference_in_float64(vals, temperature, min_p, top_p)
        # a survivor count can differ only where float32 and float64 fall on different sides of a threshold
        if n != want.size:
            continue
        assert np.allclose(probs[:n], want, rtol=2e-6, atol=1e-9)
        assert np.all(probs[n:] == 0.0)
        if n == 1:
            assert tok == idx[0] and state == before  # no draw, the generator stands still
            checked += 1
            continue
        assert state == py_xorshift(before)
        r = (state >> 40) / float(1 << 24)
        c = np.cumsum(want)
        pick = int(np.argmax(r < c)) if np.any(r < c) else n - 1
        if min(abs(r - x) for x in c) < 1e-5:  # r on a boundary of the float64 partition: either side is right
            continue
        assert tok == idx[pick]
        checked += 1
    assert checked >= 10


def test_edges():
    # all but one candidate at -inf: probability one, no draw
    tok, st, probs, n = O.sample_candidates([3.0, -math.inf, -math.inf], [7, 8, 9], 0.8, 0.0, 0.99, 5)
    assert (tok, st, n) == (7, 5, 1) and probs[0] == 1.0
    # temperature below zero is greedy as well (mod.rs:488)
    assert O.sample_candidates([1.0, 0.5], [4, 2], -1.0, 0.0, 1.0, 9)[:2] == (4, 9)
    # the last candidate is the fallback when rounding leaves r above the last cumulative sum: cannot be forced from
    # outside; the partition is checked instead: cumulative sums of the final probabilities end within 1e-6 of one
    _, _, probs, n = O.sample_candidates(np.linspace(5, -5, 200), np.arange(200), 1.3, 0.0, 1.0, 3)
    assert n == 200 and abs(float(np.cumsum(probs.astype(np.float64))[-1]) - 1.0) < 1e-6


def py_logits_edit(logits, banned, bias, recent, window, penalty):
    """The reference's two functions (mod.rs:573-613) as plain Python over numpy float32 scalars."""
    out = [np.float32(v) for v in logits]
    for tkn in banned:
        if tkn < len(out):
            out[tkn] = np.float32(-np.inf)
    for tkn, b in bias.items():
        if tkn < len(out) and np.isfinite(out[tkn]):
            out[tkn] = np.float32(out[tkn] + np.float32(b))
    if penalty != 1.0 and len(recent):
        for tkn in recent[max(0, len(recent) - window):]:
            if tkn < len(out):
                out[tkn] = np.float32(out[tkn] / np.float32(penalty)) if out[tkn] > 0 else np.float32(out[tkn] * np.float32(penalty))
    return np.array(out, dtype=np.float32)


def test_logits_edit_reference_cases():
    # test_repetition_penalty (mod.rs:789-806): token 1 penalised, token 2 wins
    out = O.logits_edit([1.0, 5.0, 4.9, 1.0], recent=[1], window=64, repetition_penalty=100.0)
    assert int(np.argmax(out)) == 2 and out[1] == np.float32(5.0) / np.float32(100.0)
    # banned_tokens_never_sampled (mod.rs:956-983): everything but token 3 at -inf
    out = O.logits_edit(np.arange(5, dtype=np.float32), banned=[0, 1, 2, 4])
    assert np.all(np.isneginf(out[[0, 1, 2, 4]])) and out[3] == 3.0
    # positive_bias / negative_bias (mod.rs:986-1028)
    assert int(np.argmax(O.logits_edit([10.0, -20.0, -20.0, -20.0], bias={1: 100.0}))) == 1
    assert int(np.argmax(O.logits_edit([100.0, 1.0, 0.5, 0.1], bias={0: -200.0}))) == 1
    # logit_bias_empty_config_no_op (mod.rs:1031-1044)
    assert np.array_equal(O.logits_edit([1.0, 2.0, 3.0, 0.5]), np.float32([1.0, 2.0, 3.0, 0.5]))
    # a banned token stays banned whatever its bias (mod.rs:586-590)
    assert np.isneginf(O.logits_edit([1.0, 2.0], banned=[1], bias={1: 50.0})[1])


def test_logits_edit_against_plain_python():
    rng = np.random.default_rng(5)
    for trial in range(30):
        n = int(rng.integers(5, 300))
        logits = (rng.standard_normal(n) * 4).astype(np.float32)
        banned = rng.integers(0, n + 3, size=int(rng.integers(0, 6))).tolist()  # some ids past the vocabulary
        bias = {int(t): float(rng.standard_normal() * 10) for t in rng.choice(n + 2, size=int(rng.integers(0, 6)), replace=False)}
        recent = rng.integers(0, min(n + 2, 12), size=int(rng.integers(0, 90))).tolist()  # few distinct ids: repeats
        window = int(rng.integers(0, 100))
        penalty = float(rng.choice([1.0, 1.1, 1.3, 0.8]))
        got = O.logits_edit(logits, banned, bias, recent, window, penalty)
        want = py_logits_edit(logits, banned, bias, recent, window, penalty)
        assert np.array_equal(got, want, equal_nan=True), trial
