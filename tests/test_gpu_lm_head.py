"""The vocabulary projection with a short candidate list (k <= 8: greedy decoding, small top_k) in one launch (oxq_lm_head_topk_dev) through the C ABI: logits
bit-identical to oxq_matvec_q8_fused_dev's (which test_gpu_parity holds against the CPU oracle, the C3 matrix at full
size included), candidates those of a stable descending sort of these logits (lower index first among equal
values: the order oxq_topk_dev gives, held against the oracle's top-k in test_gpu_linear).  Every case asserts which
launch the library took."""
import ctypes as C
import sys

import numpy as np
import pytest
import torch

import oracle as O
from oxillama_amd import linear as L
from oxillama_amd import synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(*a):
    print("[lm_head]", *a, flush=True)
    sys.stdout.flush()


def last_launch():
    from oxillama_amd import capi
    buf = C.create_string_buffer(256)
    capi.load().oxq_last_launch(buf, 256)
    return buf.value.decode()


def weights(t, seed, n, k_):
    if t in synth.BLOCK:
        return synth.weights(t, seed, n, k_)
    return O.random_blocks(t, seed, n, k_)


def expected(logits, k):
    key = np.where(np.isnan(logits), -np.inf, logits.astype(np.float64))
    order = np.argsort(-key, kind="stable")[:k]
    return logits[order], order.astype(np.uint32)


def run_case(hip, ref, t, n, k_, k, fused, seed=7, ties=True):
    say(O.NAMES[t], n, k_, "k", k)
    w = weights(t, seed, n, k_).reshape(n, -1).copy()
    if ties and n > 200:
        w[100:110] = w[17]   # equal logits: the lower index first
        w[n - 1] = w[17]
    acts = ref.quantize_q8_0(synth.normal_f32(seed + 1, k_))
    kern = hip.HipKernel(t)
    dw, da = torch.from_numpy(w.reshape(-1)).to(DEV), torch.from_numpy(acts).to(DEV)
    plain = torch.zeros(n, dtype=torch.float32, device=DEV)
    kern.matvec_q8_fused_dev(dw, da, plain, n, k_, accumulate=False)
    need = L.lm_head_topk_workspace_bytes(t, n, k_, k)
    assert need > 0
    ws = torch.full((need // 8 + 1,), -1, dtype=torch.int64, device=DEV)  # the lists may hold anything before the call
    logits = torch.full((n + 1,), 7.0, dtype=torch.float32, device=DEV)
    vals = torch.full((k + 1,), 7.0, dtype=torch.float32, device=DEV)
    idx = torch.full((k + 1,), -7, dtype=torch.int32, device=DEV)
    for rep in range(3):  # the ticket goes back to zero: the same answer every time
        L.lm_head_topk_dev(t, dw, da, logits, n, k_, k, vals, idx, ws)
        torch.cuda.synchronize()
        took = last_launch()
        assert took.startswith("gemv_q8_topk") == fused, took
        assert torch.equal(logits[:n], plain) and float(logits[n]) == 7.0
        want_v, want_i = expected(plain.cpu().numpy(), k)
        got_i = idx.cpu().numpy().view(np.uint32)
        assert np.array_equal(got_i[:k], want_i), f"rep {rep}: indices differ at {np.nonzero(got_i[:k] != want_i)[0][:5]}"
        assert np.array_equal(vals.cpu().numpy()[:k].view(np.uint32), want_v.view(np.uint32))
        assert float(vals[k]) == 7.0 and int(idx[k]) == -7
        vals[:k] = 0
        idx[:k] = 0
    return took


@pytest.mark.parametrize("case", [(O.Q6_K, 32000, 4096, 8), (O.Q6_K, 32000, 4096, 1), (O.Q4_K, 32003, 4096, 8),
                                  (O.Q8_0, 5000, 2048, 5), (O.Q5_K, 9000, 8192, 3), (O.Q4_0, 50000, 1024, 8),
                                  (O.Q6_K, 300, 256, 8), (O.Q8_0, 8, 4096, 8), (O.Q4_K, 3, 512, 2), (O.Q4_K, 151936, 1024, 4)],
                         ids=lambda c: "%s_%dx%d_k%d" % (O.NAMES[c[0]], c[1], c[2], c[3]))
def test_lm_head_topk_one_launch(hip, ref, case):
    t, n, k_, k = case
    run_case(hip, ref, t, n, k_, k, fused=True)


@pytest.mark.parametrize("k", [1, 8])
def test_lm_head_topk_full_vocabulary(hip, ref, k):
    """C3's matrix (128256 x 4096 Q6_K): the argmax of greedy decoding, and a list of eight."""
    took = run_case(hip, ref, O.Q6_K, 128256, 4096, k, fused=True, seed=3)
    say(took)


@pytest.mark.parametrize("case", [(O.Q6_K, 128256 // 4, 4096, 40), (O.Q3_K, 4000, 4096, 8), (O.Q4_K, 3000, 16384, 8),
                                  (O.Q6_K, 9000, 2048, 256)],
                         ids=["k_40", "format_without_the_kernel", "rows_of_four_steps", "k_256"])
def test_lm_head_topk_other_shapes_take_the_separate_launches(hip, ref, case):
    t, n, k_, k = case
    run_case(hip, ref, t, n, k_, k, fused=False)


def test_lm_head_topk_in_a_graph_and_over_many_calls(hip, ref):
    """Replays of a recorded launch (the ticket's address is part of it) with eager calls between them, and more calls
    than the library has tickets."""
    t, n, k_, k = O.Q6_K, 20000, 2048, 4
    w = weights(t, 11, n, k_)
    kern = hip.HipKernel(t)
    dw = torch.from_numpy(w).to(DEV)
    acts = [torch.from_numpy(ref.quantize_q8_0(synth.normal_f32(20 + i, k_))).to(DEV) for i in range(3)]
    ws = torch.zeros(L.lm_head_topk_workspace_bytes(t, n, k_, k) // 8 + 1, dtype=torch.int64, device=DEV)
    logits = torch.zeros(n, dtype=torch.float32, device=DEV)
    vals, idx = torch.zeros(k, dtype=torch.float32, device=DEV), torch.zeros(k, dtype=torch.int32, device=DEV)
    da = acts[0].clone()
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        L.lm_head_topk_dev(t, dw, da, logits, n, k_, k, vals, idx, ws)
        stream.synchronize()
        with torch.cuda.graph(g, stream=stream):
            L.lm_head_topk_dev(t, dw, da, logits, n, k_, k, vals, idx, ws)
    assert last_launch().startswith("gemv_q8_topk"), last_launch()

    def check(a):
        plain = torch.zeros(n, dtype=torch.float32, device=DEV)
        kern.matvec_q8_fused_dev(dw, a, plain, n, k_, accumulate=False)
        torch.cuda.synchronize()
        want_v, want_i = expected(plain.cpu().numpy(), k)
        assert np.array_equal(idx.cpu().numpy().view(np.uint32), want_i)
        assert np.array_equal(vals.cpu().numpy().view(np.uint32), want_v.view(np.uint32))

    for i in range(3):
        da.copy_(acts[i])
        torch.cuda.synchronize()
        with torch.cuda.stream(stream):
            g.replay()
            stream.synchronize()
        check(acts[i])
        L.lm_head_topk_dev(t, dw, acts[(i + 1) % 3], logits, n, k_, k, vals, idx, ws)  # eager, between the replays
        torch.cuda.synchronize()
        check(acts[(i + 1) % 3])
    for i in range(1100):
        L.lm_head_topk_dev(t, dw, acts[i % 3], logits, n, k_, k, vals, idx, ws)
    torch.cuda.synchronize()
    check(acts[1099 % 3])


def test_lm_head_topk_argument_errors(hip):
    z = torch.zeros(1 << 16, dtype=torch.uint8, device=DEV)
    f = torch.zeros(512, dtype=torch.float32, device=DEV)
    i32 = torch.zeros(512, dtype=torch.int32, device=DEV)
    ws = torch.zeros(1 << 14, dtype=torch.int64, device=DEV)
    with pytest.raises(hip.DimensionMismatch):
        L.lm_head_topk_dev(O.Q6_K, z, z, f, 64, 256, 0, f, i32, ws)
    with pytest.raises(hip.DimensionMismatch):
        L.lm_head_topk_dev(O.Q6_K, z, z, f, 64, 256, 65, f, i32, ws)
    with pytest.raises(hip.BufferTooSmall):
        L.lm_head_topk_dev(O.Q6_K, z, z, f, 64, 256, 8, f, i32, ws[:1])
    assert L.lm_head_topk_workspace_bytes(O.Q6_K, 64, 256, 65) == 0
    assert L.lm_head_topk_workspace_bytes(O.Q6_K, 128256, 4096, 8) == 255 * 8 * 8
    assert L.lm_head_topk_workspace_bytes(O.Q6_K, 128256, 4096, 40) == L.topk_workspace_bytes(128256, 40)
