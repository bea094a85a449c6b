"""The allocation-free form of the batched matmul (oxq_gemm_q8_static_dev): its workspace is a static array in
device memory, so the call may not touch the allocator; its results are those of oxq_gemm_q8_dev with a caller
workspace, bit for bit, also when a smaller call follows a larger one on the same array."""
import numpy as np
import pytest

import oracle as O
from oxillama_amd import capi, quant, synth

pytestmark = pytest.mark.gpu


def say(*a):
    print("[no-alloc]", *a, flush=True)


def _case(hip, ref, t, m, n, k_, seed):
    import torch
    w = synth.weights(t, seed, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(seed + 1, m * k_))
    kern = hip.HipKernel(t)
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    ws = torch.empty(max(kern.gemm_workspace_bytes(m, n, k_), 256), dtype=torch.uint8, device="cuda")
    want = torch.full((m, n), 3.0, dtype=torch.float32, device="cuda")
    got = torch.full((m, n), 3.0, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    for acc in (False, True):
        kern.gemm_q8_dev(dw, da, want, m, n, k_, accumulate=acc, workspace=ws)
        torch.cuda.synchronize()
        # neither torch's allocator nor the device's own (free bytes as the driver reports them: a hipMalloc inside
        # the library would lower them) moves across the call
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]
        kern.gemm_q8_static_dev(dw, da, got, m, n, k_, accumulate=acc)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
        assert torch.equal(got, want), (O.NAMES[t], m, n, k_, acc)
    # and against the oracle, so that "equal" cannot mean "equally wrong"
    arb = k_ // 32 * 34
    rows = range(0, m, max(1, m // 7))
    y = got.cpu().numpy()
    for r in rows:
        y1 = ref.matvec_q8_fused(t, w, acts[r * arb:(r + 1) * arb], n, k_, tier=O.TIER_AVX2)
        y_ref = y1 + y1  # overwrite, then accumulate: the buffer holds y + y after both passes
        assert np.abs(y[r] - y_ref).max() <= 1e-5 * np.abs(y_ref).max(), (O.NAMES[t], r)


def test_static_scratch_matmul_equals_workspace_matmul_twice_in_a_row(hip, ref):
    lib = capi.load()
    assert lib.oxq_gemm_q8_static_max_workspace_bytes() == 16 << 20
    # a larger call first, then smaller ones on the same array (stale bytes of the first call lie behind them),
    # then one below the tile kernel's row threshold (GEMV launches, no workspace at all), then a few-token
    # shape whose k is split over work groups (per-split sums in the array too) and a small one after it
    for t, m, n, k_, seed in ((O.Q4_K, 200, 257, 2048, 31), (O.Q4_K, 40, 100, 512, 33), (O.IQ4_XS, 130, 129, 1024, 35),
                              (O.Q6_K, 33, 64, 768, 37), (O.Q8_0, 16, 96, 256, 39), (O.Q4_K, 3, 64, 512, 41),
                              (O.Q4_K, 12, 4096, 8192, 43), (O.IQ4_XS, 16, 200, 1024, 45)):
        say(O.NAMES[t], m, n, k_)
        _case(hip, ref, t, m, n, k_, seed)


def test_static_scratch_matmul_under_stream_capture(hip, ref):
    """Recorded into a HIP graph (where an allocation or a synchronisation inside the call would end the capture with an
    error) and replayed three times with eager work between the replays: every replay gives the eager call's bits."""
    import torch
    t, m, n, k_ = O.Q4_K, 24, 512, 1024
    w = synth.weights(t, 51, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(52, m * k_))
    kern = hip.HipKernel(t)
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    want = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    got = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    other = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    kern.gemm_q8_static_dev(dw, da, want, m, n, k_)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(g, stream=stream):
            kern.gemm_q8_static_dev(dw, da, got, m, n, k_)
        for i in range(3):
            got.zero_()
            # eager work on the same array between the replays: another shape's bytes lie in it when the graph runs
            kern.gemm_q8_static_dev(dw, da[:8 * (k_ // 32 * 34)], other[:8], 8, n, k_)
            stream.synchronize()
            g.replay()
            stream.synchronize()
            assert torch.equal(got, want), i


def test_static_scratch_limits(hip, ref):
    import torch
    lib = capi.load()
    t = O.Q4_K
    # 4096 tokens of 4096 columns need 25 MB of workspace: refused, with the sizes, before anything is launched
    m, n, k_ = 4096, 64, 4096
    need = hip.HipKernel(t).gemm_workspace_bytes(m, n, k_)
    assert need > 16 << 20
    d = torch.zeros(16, dtype=torch.uint8, device="cuda")
    with pytest.raises(quant.BufferTooSmall) as e:
        hip.HipKernel(t).gemm_q8_static_dev(d, d, d, m, n, k_)
    assert (e.value.needed, e.value.available) == (need, 16 << 20)
    # the shape checks of oxq_gemm_q8_dev come first
    assert lib.oxq_gemm_q8_static_dev(15, d.data_ptr(), d.data_ptr(), d.data_ptr(), 8, 64, 256, 0, None) == \
        capi.ERR_UNSUPPORTED_TYPE
