"""The prefill kernel of the formats whose scaled weights are exact in f16 (Q4_K; oxq_gemm_prefill.hip): many token
rows x Q4_K weights on the f16 matrix cores with the 6-bit sub-block scale inside the weight operand
(reference: gemm = m fused matvecs, crates/oxillama-quant/src/reference/q4_k.rs:186-201, 218-333).

Bars: the matrix core's result per (token, row, 32-weight sub-block) is sc * I exactly, compared == with the
scale decoded here from the raw block bytes (decode_scales_mins, q4_k.rs:27-49) times the oracle's integer group
sum; fp32 within 1e-5 * |y|_inf of the oracle's fused matvec per token row (tolerance of the path; the kernel
applies d and dmin once per super-block, the reference once per sub-block)."""
import sys

import numpy as np
import pytest
import torch

import oracle as O
from oxillama_amd import capi, synth

pytestmark = pytest.mark.gpu
FP32_REL_TOL = 1e-5


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def q4k_sub_block_scales(w, n, k):
    """sc[row][sub-block] of Q4_K rows (decode_scales_mins, reference/q4_k.rs:27-49), from the raw bytes."""
    blocks = w.reshape(n, k // 256, 144)
    s = blocks[:, :, 4:16].astype(np.int32)
    sc = np.empty((n, k // 256, 8), np.int32)
    for j in range(4):
        sc[:, :, j] = s[:, :, j] & 63
        sc[:, :, j + 4] = (s[:, :, j + 8] & 15) | ((s[:, :, j] >> 6) << 4)
    return sc.reshape(n, k // 32)


def last_launch():
    import ctypes
    buf = ctypes.create_string_buffer(256)
    capi.load().oxq_last_launch(buf, 256)
    return buf.value.decode()


def oracle_rows(ref, t, w, acts, n, k, rows):
    arb = k // 32 * 34
    return np.stack([ref.matvec_q8_fused_mt(t, w, acts[r * arb:(r + 1) * arb], n, k, 16) for r in rows])


@pytest.mark.parametrize("shape", [(1, 32, 256), (33, 100, 1024), (96, 128, 256), (128, 160, 512), (200, 257, 1024),
                                   (130, 129, 2048), (384, 520, 4096)], ids=lambda s: "x".join(map(str, s)))
def test_prefill_f16_kernel(hip, ref, tuning, shape):
    m, n, k = shape
    t = O.Q4_K
    say("prefill f16", shape)
    tuning("gemm_variant", 300)  # this kernel for any number of token rows
    tuning("gemm_tile_min_rows", 1)  # (a handful of rows would otherwise go to the GEMV launches)
    w = synth.weights(t, 900 + m, n, k)
    x = synth.normal_f32(901 + n, m * k)
    x[:k] *= 300.0  # a token with large activations: its block sums' products need all three bf16 pieces
    acts = ref.quantize_q8_0(x)
    kern = hip.HipKernel(t)
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    dy = torch.full((m, n), 7.0, dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(dw, da, dy, m, n, k, accumulate=False, workspace=ws)
    torch.cuda.synchronize()
    assert "gemm_prefill_q4k" in last_launch(), last_launch()
    y = dy.cpu().numpy()
    y_ref = oracle_rows(ref, t, w, acts, n, k, range(m))
    for r in range(m):  # per token row: the bar of the batch-1 matvec
        err, scale = np.abs(y[r] - y_ref[r]).max(), np.abs(y_ref[r]).max()
        assert err <= FP32_REL_TOL * scale, f"token {r}: max err {err:.3e} vs |y|inf {scale:.3e}"
    # accumulate adds the same values to what is there
    dy2 = dy.clone()
    kern.gemm_q8_dev(dw, da, dy2, m, n, k, accumulate=True, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(dy2, dy + dy)
    # the matrix core's results: sc * I exactly, and the dump launch gives the product launch's bits
    dsum = torch.empty((m, n, k // 32), dtype=torch.int32, device="cuda")
    dy3 = torch.empty_like(dy)
    kern.gemm_scaled_sums_dev(dw, da, dy3, dsum, m, n, k, ws)
    torch.cuda.synchronize()
    sc = q4k_sub_block_scales(w, n, k)
    arb = k // 32 * 34
    got = dsum.cpu().numpy()
    for r in range(m):
        want = sc * ref.block_sums(t, w, acts[r * arb:(r + 1) * arb], n, k)
        assert np.array_equal(got[r], want), f"token {r}"
    assert torch.equal(dy3, dy)


def test_prefill_f16_kernel_is_the_default_where_it_fills_the_chip(hip, ref):
    """Without any knob: a Q4_K matmul whose 128-token x 256-row work groups fill 7/8 of the compute units takes this
    kernel (also with 96 of a tile's 128 token rows in use); one that fills 40 % of them, one with 64 token rows (half
    of every work group's token tile empty), and any Q6_K matmul, stay on the int8 tile kernel."""
    cus = hip.device_info()["compute_units"]
    k = 256
    for t, m, n, expect in ((O.Q4_K, 128, 256 * (cus * 7 // 8), True), (O.Q4_K, 128, 256 * (cus * 2 // 5), False),
                            (O.Q4_K, 96, 256 * (cus * 7 // 8), True), (O.Q4_K, 64, 256 * (cus * 7 // 8), False),
                            (O.Q6_K, 128, 256 * (cus * 7 // 8), False)):
        say("default kernel", O.NAMES[t], m, n, k)
        w = synth.weights(t, 5, n, k)
        acts = ref.quantize_q8_0(synth.normal_f32(6, m * k))
        kern = hip.HipKernel(t)
        ws = torch.empty(kern.gemm_workspace_bytes(m, n, k), dtype=torch.uint8, device="cuda")
        dy = torch.empty((m, n), dtype=torch.float32, device="cuda")
        kern.gemm_q8_dev(torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), dy, m, n, k, accumulate=False,
                         workspace=ws)
        torch.cuda.synchronize()
        assert ("gemm_prefill_q4k" in last_launch()) == expect, (O.NAMES[t], m, n, last_launch())
        rows = [0, 1, 63, m - 1]
        y_ref = oracle_rows(ref, t, w, acts, n, k, rows)
        assert np.abs(dy.cpu().numpy()[rows] - y_ref).max() <= FP32_REL_TOL * np.abs(y_ref).max()


def test_scaled_sums_errors(hip):
    kern = hip.HipKernel(O.Q6_K)
    z = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    with pytest.raises(hip.UnsupportedShape):
        kern.gemm_scaled_sums_dev(z, z, z, z, 4, 32, 256, z)
    kern = hip.HipKernel(O.Q4_K)
    with pytest.raises(hip.BufferTooSmall):
        kern.gemm_scaled_sums_dev(z, z, z, z, 4, 32, 256, z[:256])
