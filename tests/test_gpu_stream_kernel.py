"""The streamed form of the int8-MFMA tile kernel (weights through LDS by direct-to-LDS loads; opt-in through
oxq_set_gemm_variant): integer sub-block sums bit-exact, fp32 within 1e-5 * |y|_inf of the oracle, every launch
shape it has, plain and grouped (mixture-of-experts) form, ragged edges, accumulate."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O
from oxillama_amd import capi, synth

pytestmark = pytest.mark.gpu
TOL = 1e-5


def say(*a):
    print("[stream]", *a, flush=True)


def _launch_name():
    buf = C.create_string_buffer(256)
    capi.load().oxq_last_launch(buf, 256)
    return buf.value.decode()


# (variant, tokens): many-token shapes need an even number of stages per tile, few-token shapes whole stages per
# quarter of k -- the shapes below satisfy both for Q4_K (one super-block per stage) and IQ4_XS (two)
CASES = [(101, 200), (102, 130), (103, 512), (111, 16), (112, 32), (116, 7), (100, 20), (100, 300)]


@pytest.mark.parametrize("variant,m", CASES, ids=lambda v: str(v))
@pytest.mark.parametrize("t", [O.Q4_K, O.IQ4_XS], ids=lambda t: O.NAMES[t])
def test_streamed_kernel_against_oracle(hip, ref, tuning, t, variant, m):
    n, k_ = 257, 4096
    say(O.NAMES[t], variant, m, n, k_)
    tuning("gemm_tile_min_rows", 1)
    w = synth.weights(t, 1200 + m, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(1300 + m, m * k_))
    kern = hip.HipKernel(t)
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device="cuda")
    base = torch.full((m, n), 2.5, dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(dw, da, base, m, n, k_, accumulate=False, workspace=ws)  # the default (tile) kernel
    torch.cuda.synchronize()
    tuning("gemm_variant", variant)
    dy = torch.full((m, n), 2.5, dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(dw, da, dy, m, n, k_, accumulate=False, workspace=ws)
    torch.cuda.synchronize()
    streamed = "gemm_stream_kernel" in _launch_name()
    if t == O.IQ4_XS and m > 64:
        assert not streamed  # many-token shapes of this format stay on the tile kernel
    else:
        assert streamed, _launch_name()
    arb = k_ // 32 * 34
    y = dy.cpu().numpy()
    for r in sorted(set(range(0, m, max(1, m // 9))) | {m - 1}):
        y_ref = ref.matvec_q8_fused(t, w, acts[r * arb:(r + 1) * arb], n, k_, tier=O.TIER_AVX2)
        assert np.abs(y[r] - y_ref).max() <= TOL * np.abs(y_ref).max(), (O.NAMES[t], variant, r)
    # the two kernels order the fp32 sums differently (zero-point term), never by more than the tolerance
    assert (dy - base).abs().max().item() <= TOL * base.abs().max().item()
    # accumulate adds the same bits to what is there
    dy2 = dy.clone()
    kern.gemm_q8_dev(dw, da, dy2, m, n, k_, accumulate=True, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(dy2, dy + dy)
    # exact integer sums from this kernel's own dump instantiation
    dsum = torch.empty((m, n, k_ // 32), dtype=torch.int32, device="cuda")
    dy3 = torch.empty_like(dy)
    kern.gemm_block_sums_dev(dw, da, dy3, dsum, m, n, k_, workspace=ws)
    torch.cuda.synchronize()
    rows = sorted(set(range(0, m, max(1, m // 5))) | {m - 1})
    want = np.stack([ref.block_sums(t, w, acts[r * arb:(r + 1) * arb], n, k_) for r in rows])
    assert np.array_equal(dsum.cpu().numpy()[rows], want)
    if streamed and (m > 64 or m <= 32):
        assert "gemm_stream_kernel" in _launch_name() and torch.equal(dy3, dy)


@pytest.mark.parametrize("t", [O.Q4_K, O.IQ4_XS], ids=lambda t: O.NAMES[t])
def test_streamed_kernel_grouped_form(hip, ref, tuning, t):
    """Expert groups of uneven size (one empty) on the few-token streamed kernel: each expert's rows against its
    own weights, bit-equal to one plain streamed call per expert."""
    n, k_, n_exp = 160, 2048, 5
    counts = [9, 0, 31, 1, 17]
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    rows = int(offsets[-1])
    w = np.stack([synth.weights(t, 1400 + e, n, k_) for e in range(n_exp)])
    acts = ref.quantize_q8_0(synth.normal_f32(1500, rows * k_))
    kern = hip.HipKernel(t)
    dw, da, doff = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), torch.from_numpy(offsets).cuda()
    ws = torch.empty(kern.moe_gemm_workspace_bytes(rows, n, k_), dtype=torch.uint8, device="cuda")
    tuning("gemm_tile_min_rows", 1)
    tuning("gemm_variant", 111)
    dy = torch.zeros((rows, n), dtype=torch.float32, device="cuda")
    kern.moe_gemm_q8_dev(dw, w[0].nbytes, n_exp, da, doff, rows, max(counts), dy, n, k_, ws)
    torch.cuda.synchronize()
    assert "gemm_stream_kernel" in _launch_name()
    arb = k_ // 32 * 34
    for e in range(n_exp):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi == lo:
            continue
        one = torch.zeros((hi - lo, n), dtype=torch.float32, device="cuda")
        ws1 = torch.empty(kern.gemm_workspace_bytes(hi - lo, n, k_), dtype=torch.uint8, device="cuda")
        kern.gemm_q8_dev(dw[e], da[lo * arb:hi * arb], one, hi - lo, n, k_, accumulate=False, workspace=ws1)
        torch.cuda.synchronize()
        assert torch.equal(dy[lo:hi], one), (O.NAMES[t], e)
        y_ref = ref.matvec_q8_fused(t, w[e], acts[lo * arb:(lo + 1) * arb], n, k_, tier=O.TIER_AVX2)
        assert np.abs(dy[lo].cpu().numpy() - y_ref).max() <= TOL * np.abs(y_ref).max()
