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
