"""Logits -> token on the device: oxq_topk_dev's candidates through oxq_sample_candidates_dev (temperature, softmax over
the candidates, min-p, top-p, renormalisation, the draw against the reference's Xorshift64) against the oracle's
restatement of sample_with_rng (crates/oxillama-runtime/src/sampling/mod.rs:487-564).  Index work and a chain of fp32
operations in a fixed order: token ids and generator states `==`, probabilities bit for bit."""
import numpy as np
import pytest

import oracle as O
from oxillama_amd import linear, synth

pytestmark = pytest.mark.gpu


def say(*a):
    print("[sampler]", *a, flush=True)


def _device_sampler(logits, k):
    import torch
    d_logits = torch.from_numpy(logits).cuda()
    ws = torch.empty(max(linear.topk_workspace_bytes(logits.size, k), 8) // 8 + 1, dtype=torch.int64, device="cuda")
    d_vals = torch.empty(k, dtype=torch.float32, device="cuda")
    d_idx = torch.empty(k, dtype=torch.int32, device="cuda")
    linear.topk_dev(d_logits, k, d_vals, d_idx, ws)
    return d_vals, d_idx


@pytest.mark.parametrize("k", [1, 2, 8, 40, 256])
@pytest.mark.parametrize("cfg", [(1.0, 0.0, 1.0), (0.7, 0.0, 0.9), (1.5, 0.05, 1.0), (0.9, 0.02, 0.5), (0.0, 0.0, 1.0)],
                         ids=lambda c: "T%g_minp%g_topp%g" % c)
def test_draws_follow_the_oracle(hip, ref, k, cfg):
    import torch
    temperature, min_p, top_p = cfg
    n = 128256
    logits = (synth.normal_f32(7000 + k, n) * 2.5).astype(np.float32)
    say("k", k, "cfg", cfg)
    d_vals, d_idx = _device_sampler(logits, k)
    vals, idx = ref.topk(logits, k)
    assert np.array_equal(d_vals.cpu().numpy(), vals) and np.array_equal(d_idx.cpu().numpy().view(np.uint32), idx)
    state = O.xorshift64_seed(4242 + k)
    d_state = torch.tensor([state], dtype=torch.int64, device="cuda")
    d_tok = torch.full((1,), -1, dtype=torch.int32, device="cuda")
    d_probs = torch.full((k,), 9.0, dtype=torch.float32, device="cuda")
    for draw in range(60):  # one sampler, sixty tokens: the generator state threads through
        tok, state, probs, n_left = ref.sample_candidates(vals, idx, temperature, min_p, top_p, state)
        linear.sample_candidates_dev(d_vals, d_idx, k, temperature, min_p, top_p, d_state, d_tok, d_probs)
        torch.cuda.synchronize()
        assert int(d_tok.item()) == tok, (draw, tok)
        assert int(d_state.item()) & ((1 << 64) - 1) == state, draw
        assert np.array_equal(d_probs.cpu().numpy(), probs), draw


def test_reference_cases_on_the_device(hip, ref):
    """The reference's own sampler tests (mod.rs:707-856) with the candidate list and the draw on the device."""
    import torch

    def run(logits, k, temperature=1.0, top_p=1.0, min_p=0.0, seed=0xDEADBEEFCAFEBABE, draws=1):
        logits = np.asarray(logits, dtype=np.float32)
        d_vals, d_idx = _device_sampler(logits, k)
        d_state = torch.tensor([np.int64(np.uint64(O.xorshift64_seed(seed)))], dtype=torch.int64, device="cuda")
        d_tok = torch.zeros(1, dtype=torch.int32, device="cuda")
        out = []
        for _ in range(draws):
            linear.sample_candidates_dev(d_vals, d_idx, k, temperature, min_p, top_p, d_state, d_tok)
            out.append(int(d_tok.item()))
        return out

    assert run([0.1, 0.5, 0.3, 0.8, 0.2], 5, temperature=0.0) == [3]
    assert run([1.0, 5.0, 3.0, 2.0], 4, temperature=0.0) == [1]
    assert run([1.0, 5.0, 3.0, 2.0], 1, temperature=1.0) == [1]
    assert run([100.0, 0.0, 0.0, 0.0, 0.0], 5, top_p=0.5, seed=123) == [0]
    assert run([10.0, -10.0, -10.0, -10.0], 4, min_p=0.1, seed=42, draws=100) == [0] * 100
    counts = np.bincount(run([2.0, 2.0, 2.0, 2.0], 4, seed=999, draws=1000), minlength=4)
    assert all(100 < c < 400 for c in counts), counts


def test_edges_and_errors(hip, ref):
    import torch
    from oxillama_amd import capi, quant
    lib = capi.load()
    # one finite candidate: probability one, the generator stands still
    vals = torch.tensor([3.0, -np.inf, -np.inf], dtype=torch.float32, device="cuda")
    idx = torch.tensor([7, 8, 9], dtype=torch.int32, device="cuda")
    st = torch.tensor([5], dtype=torch.int64, device="cuda")
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    probs = torch.zeros(3, dtype=torch.float32, device="cuda")
    linear.sample_candidates_dev(vals, idx, 3, 0.8, 0.0, 0.99, st, tok, probs)
    assert (int(tok.item()), int(st.item())) == (7, 5) and probs.cpu().tolist() == [1.0, 0.0, 0.0]
    # k outside 1..256
    for k in (0, 257):
        assert lib.oxq_sample_candidates_dev(vals.data_ptr(), idx.data_ptr(), k, 1.0, 0.0, 1.0, st.data_ptr(), tok.data_ptr(),
                                             None, None) == capi.ERR_UNSUPPORTED_SHAPE


def test_sampler_in_a_graph_continues_the_sequence(hip, ref):
    """top-k + sampler recorded once, replayed: every replay draws the next value of the generator, as sixty eager calls
    of the oracle do."""
    import torch
    n, k, cfg = 32000, 40, (0.8, 0.0, 0.95)
    logits = (synth.normal_f32(7100, n) * 2.0).astype(np.float32)
    d_logits = torch.from_numpy(logits).cuda()
    ws = torch.empty(linear.topk_workspace_bytes(n, k) // 8 + 1, dtype=torch.int64, device="cuda")
    d_vals = torch.empty(k, dtype=torch.float32, device="cuda")
    d_idx = torch.empty(k, dtype=torch.int32, device="cuda")
    state = O.xorshift64_seed(31337)
    d_state = torch.tensor([state], dtype=torch.int64, device="cuda")
    d_tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        linear.topk_dev(d_logits, k, d_vals, d_idx, ws)
        stream.synchronize()
        with torch.cuda.graph(g, stream=stream):
            linear.topk_dev(d_logits, k, d_vals, d_idx, ws)
            linear.sample_candidates_dev(d_vals, d_idx, k, *cfg, d_state, d_tok)
        vals, idx = ref.topk(logits, k)
        for i in range(20):
            g.replay()
            stream.synchronize()
            tok, state, _, _ = ref.sample_candidates(vals, idx, *cfg, state)
            assert int(d_tok.item()) == tok and int(d_state.item()) & ((1 << 64) - 1) == state, i


def _edit_on_device(logits, banned, bias, recent, window, penalty):
    import torch

    def u32(v):
        return torch.from_numpy(np.ascontiguousarray(v, dtype=np.uint32).view(np.int32)).cuda() if len(v) else None
    d = torch.from_numpy(np.ascontiguousarray(logits, dtype=np.float32)).cuda()
    bt, bv = list(bias.keys()), list(bias.values())
    linear.logits_edit_dev(d, u32(banned), u32(bt), torch.tensor(bv, dtype=torch.float32, device="cuda") if bv else None,
                           u32(recent), window, penalty)
    torch.cuda.synchronize()
    return d.cpu().numpy()


def test_logits_edit_follows_the_oracle(hip, ref):
    """Banned tokens, logit bias and the repetition penalty (a token that occurs several times in the window is
    penalised that many times) on the device: every logit bit for bit the oracle's."""
    rng = np.random.default_rng(11)
    for trial in range(25):
        n = int(rng.choice([7, 300, 32000, 128256]))
        logits = (rng.standard_normal(n) * 4).astype(np.float32)
        logits[rng.integers(0, n, size=3)] = -np.inf
        banned = rng.integers(0, n + 3, size=int(rng.integers(0, 40))).tolist()
        bias = {int(t): float(rng.standard_normal() * 10) for t in rng.choice(n + 2, size=int(rng.integers(0, min(30, n))), replace=False)}
        recent = rng.integers(0, min(n + 2, 40), size=int(rng.integers(0, 600))).tolist()
        window = int(rng.choice([0, 1, 64, 300, 5000]))
        if min(window, len(recent)) > 4096:
            window = 64
        penalty = float(rng.choice([1.0, 1.1, 1.3, 0.8]))
        got = _edit_on_device(logits, banned, bias, recent, window, penalty)
        want = ref.logits_edit(logits, banned, bias, recent, window, penalty)
        assert np.array_equal(got, want), (trial, n, window, penalty)


def test_default_sampler_config_end_to_end(hip, ref):
    """The reference's default configuration (repetition penalty 1.1 over 64 tokens, temperature 0.7, top-k 40, top-p
    0.9: SamplerConfig::default, mod.rs:140-160) as three launches -- logit edits, candidate list, draw -- against the
    oracle's three functions, thirty tokens in a row with the sampled token joining the recent ones."""
    import torch
    n, k = 32000, 40
    state = O.xorshift64_seed(2024)
    d_state = torch.tensor([state], dtype=torch.int64, device="cuda")
    d_tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    d_vals = torch.empty(k, dtype=torch.float32, device="cuda")
    d_idx = torch.empty(k, dtype=torch.int32, device="cuda")
    ws = torch.empty(linear.topk_workspace_bytes(n, k) // 8 + 1, dtype=torch.int64, device="cuda")
    recent = []
    for step in range(30):
        logits = (synth.normal_f32(9000 + step, n) * 3.0).astype(np.float32)
        want_logits = ref.logits_edit(logits, recent=recent, window=64, repetition_penalty=1.1)
        vals, idx = ref.topk(want_logits, k)
        tok, state, _, _ = ref.sample_candidates(vals, idx, 0.7, 0.0, 0.9, state)
        d_logits = torch.from_numpy(logits).cuda()
        d_recent = torch.tensor(recent, dtype=torch.int32, device="cuda") if recent else None
        linear.logits_edit_dev(d_logits, d_recent=d_recent, window=64, repetition_penalty=1.1)
        linear.topk_dev(d_logits, k, d_vals, d_idx, ws)
        linear.sample_candidates_dev(d_vals, d_idx, k, 0.7, 0.0, 0.9, d_state, d_tok)
        torch.cuda.synchronize()
        assert int(d_tok.item()) == tok and int(d_state.item()) & ((1 << 64) - 1) == state, step
        recent.append(tok)
        if step % 3 == 0:
            recent.append(tok)  # repeats in the window


def test_reference_bias_and_ban_cases_on_the_device(hip, ref):
    out = _edit_on_device([1.0, 5.0, 4.9, 1.0], [], {}, [1], 64, 100.0)
    assert int(np.argmax(out)) == 2
    out = _edit_on_device(np.arange(5, dtype=np.float32), [0, 1, 2, 4], {}, [], 0, 1.0)
    assert np.all(np.isneginf(out[[0, 1, 2, 4]])) and out[3] == 3.0
    assert int(np.argmax(_edit_on_device([10.0, -20.0, -20.0, -20.0], [], {1: 100.0}, [], 0, 1.0))) == 1
    assert int(np.argmax(_edit_on_device([100.0, 1.0, 0.5, 0.1], [], {0: -200.0}, [], 0, 1.0))) == 1
    assert np.isneginf(_edit_on_device([1.0, 2.0], [1], {1: 50.0}, [], 0, 1.0)[1])
