"""The device-pointer entry points under HIP graph capture: a decode-layer step (quantize, q_proj,
the fused dense feed-forward block), a prefill matmul on a caller workspace and the whole
mixture-of-experts layer are each recorded once and replayed several times, with eager work of the
same library and synchronisations between the replays.  Every replay has to reproduce the eager
result bit for bit: the calls allocate nothing, synchronise nothing and read no host state that a
replay would miss."""
import sys

import numpy as np
import pytest
import torch

import oracle as O
from oxillama_amd import linear as L
from oxillama_amd import moe, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def replay_and_compare(hip, record, outputs, poison, between):
    """record(): the launches (on the current stream).  outputs: tensors they write.  Eager first,
    then capture, then three replays with `between` run eagerly in front of each."""
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        record()
        stream.synchronize()
        want = [o.clone() for o in outputs]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            record()
        for rep in range(3):
            for o in outputs:
                o.copy_(poison(o))
            between(rep)
            stream.synchronize()
            graph.replay()
            stream.synchronize()
            for o, w in zip(outputs, want):
                assert torch.equal(o.view(torch.uint8), w.view(torch.uint8)), f"replay {rep} differs from the eager run"


def test_decode_layer_step_replays(hip, ref):
    hidden, inter = 4096, 14336
    wq = dev(synth.weights(O.Q8_0, 11, hidden, hidden))
    wg, wu = dev(synth.weights(O.Q4_K, 12, inter, hidden)), dev(synth.weights(O.Q4_K, 13, inter, hidden))
    wd = dev(synth.weights(O.Q6_K, 14, hidden, inter))
    x = dev(synth.normal_f32(15, hidden))
    acts = torch.empty(hidden // 32 * 34, dtype=torch.uint8, device=DEV)
    q = torch.empty(hidden, dtype=torch.float32, device=DEV)
    y = torch.empty(hidden, dtype=torch.float32, device=DEV)
    ws = torch.empty(L.ffn_workspace_bytes(hidden, inter), dtype=torch.uint8, device=DEV)
    kq = hip.HipKernel(O.Q8_0)

    def record():
        hip.quantize_q8_0_dev(x, acts)
        kq.matvec_q8_fused_dev(wq, acts, q, hidden, hidden, accumulate=False)
        L.ffn_swiglu_dev((O.Q4_K, wg), (O.Q4_K, wu), (O.Q6_K, wd), acts, y, hidden, inter, ws)

    other = dev(synth.weights(O.Q6_K, 16, 64, hidden))
    scratch = torch.empty(64, dtype=torch.float32, device=DEV)

    def between(rep):  # eager launches of the same kernels on other data, and a changed activation buffer
        hip.HipKernel(O.Q6_K).matvec_q8_fused_dev(other, acts, scratch, 64, hidden, accumulate=False)
        acts.fill_(rep + 1)

    say("decode step under graph replay")
    replay_and_compare(hip, record, [acts, q, y], lambda o: torch.full_like(o, 3), between)


@pytest.mark.parametrize("t", [O.Q4_K, O.Q6_K, O.IQ4_XS], ids=lambda t: O.NAMES[t])
def test_prefill_matmul_replays(hip, ref, t):
    m, n, k_ = 200, 512, 2048
    w = dev(synth.weights(t, 21, n, k_))
    acts = dev(ref.quantize_q8_0(synth.normal_f32(22, m * k_)))
    kern = hip.HipKernel(t)
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device=DEV)
    out = torch.empty(m * n, dtype=torch.float32, device=DEV)

    def record():
        kern.gemm_q8_dev(w, acts, out, m, n, k_, accumulate=False, workspace=ws)

    def between(rep):
        ws.fill_(0xA5)  # the workspace is rebuilt by every replay

    say("prefill matmul under graph replay", O.NAMES[t])
    replay_and_compare(hip, record, [out], lambda o: torch.full_like(o, -1.0), between)


def test_moe_layer_replays(hip, ref):
    n_exp, top_k, n_tok, hidden, inter = 8, 2, 24, 512, 1024
    t = O.IQ4_XS
    wg, wu, wd = (np.concatenate([synth.weights(t, s + e, inter if s < 300 else hidden, hidden if s < 300 else inter)
                                  for e in range(n_exp)]) for s in (100, 200, 300))
    stride_gu, stride_d = wg.size // n_exp, wd.size // n_exp
    logits = synth.normal_f32(31, n_tok * n_exp).reshape(n_tok, n_exp)
    experts, weights = moe.route_top_k(logits, top_k)
    offsets, tok, slot = moe.group_by_expert(experts, n_exp)
    rows = moe.token_rows(offsets, tok, slot, n_tok, top_k)
    x = dev(synth.normal_f32(32, n_tok * hidden))
    ws = torch.empty(moe.moe_ffn_workspace_bytes((t, t, t), n_tok * top_k, hidden, inter), dtype=torch.uint8, device=DEV)
    out = torch.empty(n_tok * hidden, dtype=torch.float32, device=DEV)
    args = ((t, dev(wg), stride_gu), (t, dev(wu), stride_gu), (t, dev(wd), stride_d), n_exp, x, n_tok, top_k, dev(offsets),
            dev(tok), dev(rows), dev(weights), 0, out, hidden, inter)

    def record():
        moe.moe_ffn_dev(*args, ws)

    def between(rep):
        ws.fill_(rep)

    say("mixture-of-experts layer under graph replay")
    replay_and_compare(hip, record, [out], lambda o: torch.full_like(o, 9.0), between)


@pytest.mark.parametrize("n_tok", [1, 24], ids=["one_token", "24_tokens"])
def test_moe_forward_on_device_pointers_replays(hip, ref, n_tok):
    """oxq_moe_forward_dev (routing tables in the workspace; for one token the router's launch writes the activation
    rows too) captured once and replayed over a workspace that eager work overwrites in between."""
    n_exp, top_k, hidden, inter = 8, 2, 512, 1024
    t = O.IQ4_XS
    wg, wu, wd = (np.concatenate([synth.weights(t, s + e, inter if s < 300 else hidden, hidden if s < 300 else inter)
                                  for e in range(n_exp)]) for s in (100, 200, 300))
    stride_gu, stride_d = wg.size // n_exp, wd.size // n_exp
    router = dev(synth.normal_f32(41, n_exp * hidden, 0.05))
    x = dev(synth.normal_f32(42, n_tok * hidden))
    ws = torch.empty(moe.moe_forward_workspace_bytes((t, t, t), n_tok, top_k, n_exp, hidden, inter), dtype=torch.uint8,
                     device=DEV)
    out = torch.empty(n_tok * hidden, dtype=torch.float32, device=DEV)
    args = ((t, dev(wg), stride_gu), (t, dev(wu), stride_gu), (t, dev(wd), stride_d), n_exp, router, x, n_tok, top_k, out,
            hidden, inter)

    def record():
        moe.moe_forward_dev(*args, ws)

    def between(rep):
        ws.fill_(rep + 1)

    say("MoeFfn::forward on device pointers under graph replay,", n_tok, "token(s)")
    replay_and_compare(hip, record, [out], lambda o: torch.full_like(o, 9.0), between)
