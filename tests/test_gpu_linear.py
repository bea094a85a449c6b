"""Parity of the callers' side of the HIP library (QuantLinear::forward / forward_batch, LoRA,
SwiGLU + quantize, RMSNorm + quantize, the dense feed-forward block, several projections of
different heights in one launch) against the CPU oracle, through the C ABI.

Bars: Q8_0 bytes bit-exact given the same fp32 values; matvec results bit-identical between the
fused entry points and the plain ones; fp32 within 1e-5 * |y_ref|_inf of the oracle (SwiGLU's
exp and RMSNorm's tree sum differ from libm / index order in the last place)."""
import sys

import numpy as np
import pytest
import torch

import oracle as O
from oxillama_amd import linear as L
from oxillama_amd import synth

pytestmark = pytest.mark.gpu

FP32_REL_TOL = 1e-5
DEV = "cuda:0"


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def assert_close(y, y_ref, what, tol=FP32_REL_TOL):
    scale = float(np.abs(y_ref).max())
    err = float(np.abs(y.astype(np.float64) - y_ref.astype(np.float64)).max())
    assert err <= tol * scale + 1e-30, f"{what}: max err {err:.3e} > {tol} * {scale:.3e}"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def q8_identity(n, scale=1.0):
    rows = []
    for r in range(n):
        for b in range(n // 32):
            qs = [0] * 32
            if r // 32 == b:
                qs[r % 32] = 1
            rows.append(O.make_q8_0_block(scale, qs))
    return np.frombuffer(b"".join(rows), dtype=np.uint8)


# ---- SwiGLU + quantize -----------------------------------------------------------------------

def test_swiglu_quantize(hip, ref):
    for seed, n in ((1, 14336), (2, 32), (3, 64 * 14336)):
        say("swiglu seed", seed, "n", n)
        g = synth.normal_f32(seed, n, 3.0)
        u = synth.normal_f32(seed + 100, n, 1.0)
        g[:6] = [0.0, -0.0, 88.0, -88.0, -100.0, -1000.0]
        d_h = torch.empty(n, dtype=torch.float32, device=DEV)
        d_q = torch.empty(n // 32 * 34, dtype=torch.uint8, device=DEV)
        L.swiglu_quantize_dev(dev(g), dev(u), d_h, d_q)
        h, q = host(d_h), host(d_q)
        want = ref.swiglu(g, u)
        assert np.all(np.isfinite(h))
        # elementwise: the device evaluates exp as the C library does, so h is the oracle's value bit for bit (but
        # for a handful of arguments in 10^8 on which the library's own last place differs)
        assert np.all(np.abs(h - want) <= 4e-7 * np.abs(want) + 1e-37), "swiglu fp32"
        assert np.count_nonzero(h.view(np.uint32) != want.view(np.uint32)) <= 2, "swiglu fp32, bit for bit"
        # the bytes are the quantizer's bytes for the values the kernel itself produced
        assert np.array_equal(q, ref.quantize_q8_0(h))
        # each output alone gives the same result
        d_q2 = torch.empty_like(d_q)
        L.swiglu_quantize_dev(dev(g), dev(u), None, d_q2)
        assert np.array_equal(host(d_q2), q)


def test_swiglu_reference_values(hip):
    # crates/oxillama-arch/src/common/swiglu.rs:62-77, padded to one block
    g = np.zeros(32, dtype=np.float32); g[:3] = [1.0, -1.0, 0.0]
    u = np.zeros(32, dtype=np.float32); u[:3] = [2.0, 3.0, 4.0]
    d_h = torch.empty(32, dtype=torch.float32, device=DEV)
    L.swiglu_quantize_dev(dev(g), dev(u), d_h, None)
    h = host(d_h)
    assert abs(h[0] - 1.4621) < 0.01 and abs(h[2]) < 1e-6


def test_swiglu_rejects_ragged_length(hip):
    g = torch.zeros(33, dtype=torch.float32, device=DEV)
    with pytest.raises(hip.DimensionMismatch) as e:
        L.swiglu_quantize_dev(g, g, g, None)
    assert (e.value.expected, e.value.got) == (64, 33)


# ---- RMSNorm + quantize ----------------------------------------------------------------------

def test_rmsnorm_quantize(hip, ref):
    for seed, rows, n in ((1, 1, 4096), (2, 5, 4096), (3, 3, 14336), (4, 2, 32), (5, 512, 4096)):
        say("rmsnorm seed", seed, rows, "x", n)
        x = synth.normal_f32(seed, rows * n, 2.0)
        w = (1.0 + 0.1 * synth.normal_f32(seed + 50, n, 1.0)).astype(np.float32)
        d_y = torch.empty(rows * n, dtype=torch.float32, device=DEV)
        d_q = torch.empty(rows * n // 32 * 34, dtype=torch.uint8, device=DEV)
        L.rmsnorm_quantize_dev(dev(x), dev(w), 1e-5, rows, n, d_y, d_q)
        y, q = host(d_y), host(d_q)
        want = np.concatenate([ref.rmsnorm(x[r * n:(r + 1) * n], w, 1e-5) for r in range(rows)])
        assert_close(y, want, f"rmsnorm {rows}x{n}", tol=2e-6)
        assert np.array_equal(q, ref.quantize_q8_0(y))
        d_q2 = torch.empty_like(d_q)
        L.rmsnorm_quantize_dev(dev(x), dev(w), 1e-5, rows, n, None, d_q2)
        assert np.array_equal(host(d_q2), q)


def test_rmsnorm_reference_values(hip):
    # crates/oxillama-arch/src/common/rms_norm.rs:72-88, padded with zeros to 32 (same sum of squares,
    # mean over 32 instead of 4)
    x = np.zeros(32, dtype=np.float32); x[:4] = [1, 2, 3, 4]
    d_y = torch.empty(32, dtype=torch.float32, device=DEV)
    L.rmsnorm_quantize_dev(dev(x), dev(np.ones(32, dtype=np.float32)), 1e-5, 1, 32, d_y, None)
    y = host(d_y)
    rms = np.sqrt(np.float32(30.0) / np.float32(32.0) + np.float32(1e-5))
    assert np.all(np.abs(y[:4] - x[:4] / rms) < 1e-5) and np.all(y[4:] == 0)
    # all-zero row: zeros, not NaN
    L.rmsnorm_quantize_dev(dev(np.zeros(32, dtype=np.float32)), dev(np.ones(32, dtype=np.float32)), 1e-5, 1, 32, d_y,
                           None)
    assert np.all(host(d_y) == 0.0)


# ---- LoRA ------------------------------------------------------------------------------------

def test_lora_apply(hip, ref):
    for seed, rank, n_in, n_out in ((1, 16, 4096, 4096), (2, 4, 4096, 14336), (3, 64, 14336, 4096), (4, 1, 32, 8)):
        say("lora seed", seed, rank, n_in, n_out)
        a = synth.normal_f32(seed, rank * n_in, 0.05)
        b = synth.normal_f32(seed + 10, n_out * rank, 0.05)
        x = synth.normal_f32(seed + 20, n_in, 1.0)
        base = synth.normal_f32(seed + 30, n_out, 1.0)
        d_out = dev(base)
        d_r = torch.empty(rank, dtype=torch.float32, device=DEV)
        d_a, d_b = dev(a), dev(b)
        lora = L.lora_struct(d_a, d_b, d_r, rank, 0.25)
        L.lora_apply_dev(lora, dev(x), d_out, n_out, n_in)
        want = base.copy()
        ref.lora_apply(a, b, rank, 0.25, n_in, n_out, x, want)
        assert_close(host(d_out), want, "lora")
        # the up-projection is in the reference's order: exact given the kernel's own r
        r = host(d_r)
        exact = base.copy()
        s = np.zeros(n_out, dtype=np.float32)
        bm = b.reshape(n_out, rank)
        for j in range(rank):
            s = (s + (bm[:, j] * r[j]).astype(np.float32)).astype(np.float32)
        exact = (exact + (s * np.float32(0.25)).astype(np.float32)).astype(np.float32)
        assert np.array_equal(host(d_out), exact)


# ---- QuantLinear::forward --------------------------------------------------------------------

@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_linear_forward_dev(hip, ref, t):
    for seed, n_rows, n_cols in ((1, 96, 512), (2, 4096, 4096), (3, 1024, 14336)):
        say("linear", O.NAMES[t], n_rows, n_cols)
        w = synth.weights(t, seed, n_rows, n_cols)
        x = synth.normal_f32(seed + 1, n_cols)
        bias = synth.normal_f32(seed + 2, n_rows)
        rank = 8
        a = synth.normal_f32(seed + 3, rank * n_cols, 0.05)
        b = synth.normal_f32(seed + 4, n_rows * rank, 0.05)
        d_w, d_x, d_bias = dev(w), dev(x), dev(bias)
        d_acts = torch.empty(n_cols // 32 * 34, dtype=torch.uint8, device=DEV)
        hip.quantize_q8_0_dev(d_x, d_acts)
        k = hip.HipKernel(t)
        plain = torch.zeros(n_rows, dtype=torch.float32, device=DEV)
        k.matvec_q8_fused_dev(d_w, d_acts, plain, n_rows, n_cols, accumulate=False)
        y0 = host(plain)
        # no bias, no LoRA: the plain matvec, bit for bit (linear.rs:161-177)
        d_out = torch.full((n_rows,), 7.0, dtype=torch.float32, device=DEV)
        L.linear_forward_dev(t, d_w, d_out, n_rows, n_cols, d_acts=d_acts)
        assert np.array_equal(host(d_out), y0)
        # bias in the epilogue == matvec, then + bias
        L.linear_forward_dev(t, d_w, d_out, n_rows, n_cols, d_acts=d_acts, d_bias=d_bias)
        assert np.array_equal(host(d_out), (y0 + bias).astype(np.float32))
        # in-kernel quantization of x gives the same
        if n_cols <= 46080:  # the quantized vector is staged in LDS
            L.linear_forward_dev(t, d_w, d_out, n_rows, n_cols, d_x=d_x, d_bias=d_bias)
            assert np.array_equal(host(d_out), (y0 + bias).astype(np.float32))
        # bias, then LoRA, against the oracle (linear.rs:236-262)
        d_r = torch.empty(rank, dtype=torch.float32, device=DEV)
        d_a, d_b = dev(a), dev(b)
        lora = L.lora_struct(d_a, d_b, d_r, rank, 0.5)
        L.linear_forward_dev(t, d_w, d_out, n_rows, n_cols, d_x=d_x, d_acts=d_acts, d_bias=d_bias, lora=lora)
        want = ref.linear_forward(t, w, n_rows, n_cols, x, bias=bias, lora=(a, b, rank, 0.5))
        assert_close(host(d_out), want, "linear forward")


def test_linear_forward_host_reference_cases(hip, ref):
    """The QuantLinear tests of linear.rs:161-270 on a Q8_0 identity, through the host-slice route."""
    n = 32
    w = q8_identity(n)
    lin = L.QuantLinear(hip.QuantTensor(w, [n, n], O.Q8_0))
    assert lin.lora is None and (lin.out_features, lin.in_features) == (n, n)  # linear.rs:265-270
    k = hip.HipKernel(O.Q8_0)
    x = np.zeros(n, dtype=np.float32); x[3], x[7] = 2.0, -2.0
    out = np.zeros(n, dtype=np.float32)
    lin.forward(k, x, out)
    assert np.array_equal(out, ref.linear_forward(O.Q8_0, w, n, n, x))
    assert abs(out[3] - 2.0) < 2e-3 and abs(out[7] + 2.0) < 2e-3
    eye = np.eye(n, dtype=np.float32)
    lin.set_lora(L.LoraAdapter(eye, eye, n, 1.0, n, n))
    lin.bias = np.full(n, 10.0, dtype=np.float32)
    lin.forward(k, x, out)  # linear.rs:236-262: W x + bias + delta
    assert abs(out[3] - 14.0) < 2e-3 and abs(out[7] - 6.0) < 2e-3 and out[0] == 10.0
    assert_close(out, ref.linear_forward(O.Q8_0, w, n, n, x, bias=lin.bias, lora=(eye, eye, n, 1.0)), "host lora")
    lin.clear_lora()  # linear.rs:207-233
    lin.bias = None
    lin.forward(k, x, out)
    assert np.array_equal(out, ref.linear_forward(O.Q8_0, w, n, n, x))
    # a short bias covers its own length (zip semantics)
    lin.bias = np.full(4, 10.0, dtype=np.float32)
    lin.forward(k, x, out)
    assert np.array_equal(out, ref.linear_forward(O.Q8_0, w, n, n, x, bias=lin.bias))
    # errors: gemv's checks, then the adapter's
    with pytest.raises(hip.DimensionMismatch) as e:
        lin.forward(k, x[:31], out)
    assert (e.value.expected, e.value.got) == (32, 31)
    with pytest.raises(hip.DimensionMismatch) as e:
        lin.forward(k, x, out[:31])
    assert (e.value.expected, e.value.got) == (32, 31)
    with pytest.raises(hip.DimensionMismatch):
        L.LoraAdapter([1.0], [1, 0, 0, 1], 2, 1.0, 1, 2)  # lora.rs:203-214


@pytest.mark.parametrize("t", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K], ids=lambda t: O.NAMES[t])
def test_linear_forward_host_rows_that_end_inside_a_block(hip, ref, t):
    """in_features that is not a whole number of blocks: QuantLinear::forward goes through gemv, which skips the
    columns past n_cols (Q/reference/q4_k.rs:161,168); bias and LoRA see the n_cols inputs as they are."""
    bs = O.BLOCK[t][0]
    for n_rows, n_cols in ((33, bs + 20), (40, 5 * bs - 7)):
        full = -(-n_cols // bs) * bs
        w = synth.weights(t, 1200 + n_cols, n_rows, full)
        x = synth.normal_f32(1201, n_cols)
        bias = synth.normal_f32(1202, n_rows)
        rank = 3
        a = synth.normal_f32(1203, rank * n_cols) * np.float32(0.1)
        b = synth.normal_f32(1204, n_rows * rank) * np.float32(0.1)
        lin = L.QuantLinear(hip.QuantTensor(w, [n_rows, n_cols], t), bias=bias)
        lin.set_lora(L.LoraAdapter(a, b, rank, 0.5, n_cols, n_rows))
        out = np.zeros(n_rows, dtype=np.float32)
        lin.forward(hip.HipKernel(t), x, out)
        want = ref.linear_forward(t, w, n_rows, n_cols, x, bias=bias, lora=(a, b, rank, 0.5))
        assert_close(out, want, f"ragged linear {O.NAMES[t]} {n_rows}x{n_cols}")


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_linear_forward_batch(hip, ref, t):
    n, kk = 512, 1024
    w = synth.weights(t, 9, n, kk)
    bias = synth.normal_f32(10, n)
    k = hip.HipKernel(t)
    lin = L.QuantLinear(hip.QuantTensor(w, [n, kk], t), bias)
    for m in (1, 3, 40):  # single GEMV, several vectors per pass, tile kernel
        say("forward_batch", O.NAMES[t], m)
        x = synth.normal_f32(11 + m, m * kk)
        out = np.zeros(m * n, dtype=np.float32)
        lin.forward_batch(k, x, out, m)
        plain = np.zeros(m * n, dtype=np.float32)
        k.gemm(lin.weight, x, plain, m, n, kk)
        assert np.array_equal(out, (plain.reshape(m, n) + bias[None, :]).astype(np.float32).ravel())
        want = ref.gemm_q8(t, w, x, m, n, kk).reshape(m, n) + bias[None, :]
        assert_close(out, want.astype(np.float32).ravel(), "forward_batch")
        # device route with a caller workspace
        d_x = dev(x)
        d_acts = torch.empty(m * (kk // 32 * 34), dtype=torch.uint8, device=DEV)
        hip.quantize_q8_0_dev(d_x, d_acts)
        ws_bytes = k.gemm_workspace_bytes(m, n, kk)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=DEV)
        d_out = torch.empty(m * n, dtype=torch.float32, device=DEV)
        L.linear_forward_batch_dev(t, dev(w), d_acts, d_out, m, n, kk, d_bias=dev(bias),
                                   workspace=ws if ws_bytes else None)
        assert np.array_equal(host(d_out), out)


# ---- several projections of different heights in one launch ------------------------------------

@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_linear_forward_multi_unequal_rows(hip, ref, t):
    for n_cols, heights in ((4096, (4096, 1024, 1024)), (512, (96, 8, 40, 2)), (14336, (256, 4096))):
        say("multi", O.NAMES[t], n_cols, heights)
        x = synth.normal_f32(3, n_cols)
        d_x = dev(x)
        d_acts = torch.empty(n_cols // 32 * 34, dtype=torch.uint8, device=DEV)
        hip.quantize_q8_0_dev(d_x, d_acts)
        ws_, bs_, outs, singles = [], [], [], []
        k = hip.HipKernel(t)
        for i, h in enumerate(heights):
            w = dev(synth.weights(t, 20 + i, h, n_cols))
            b = dev(synth.normal_f32(30 + i, h)) if i != 1 else None
            ws_.append(w); bs_.append(b)
            outs.append(torch.full((h + 3,), -5.0, dtype=torch.float32, device=DEV))  # 3 guard floats
            one = torch.empty(h, dtype=torch.float32, device=DEV)
            L.linear_forward_dev(t, w, one, h, n_cols, d_acts=d_acts, d_bias=b)
            singles.append(host(one))
        L.linear_forward_multi_dev(t, ws_, d_acts, outs, heights, n_cols, d_biases=bs_)
        for i, h in enumerate(heights):
            got = host(outs[i])
            assert np.array_equal(got[:h], singles[i]), f"matrix {i}"
            assert np.all(got[h:] == -5.0), "wrote past the matrix's rows"
        # and against the oracle
        w0 = host(ws_[0])
        want = ref.linear_forward(t, w0, heights[0], n_cols, x, bias=host(bs_[0]))
        assert_close(host(outs[0])[:heights[0]], want, "multi vs oracle")


# ---- the dense feed-forward block ---------------------------------------------------------------

@pytest.mark.parametrize("types", [(O.Q4_K, O.Q4_K, O.Q6_K), (O.Q4_0, O.Q4_0, O.Q4_0), (O.Q8_0, O.Q4_K, O.IQ4_XS)],
                         ids=["q4k_q4k_q6k", "q4_0", "mixed"])
def test_ffn_swiglu(hip, ref, tuning, types):
    for hidden, inter in ((512, 1024), (4096, 14336)):
        say("ffn", types, hidden, inter)
        tg, tu, td = types
        wg, wu = synth.weights(tg, 1, inter, hidden), synth.weights(tu, 2, inter, hidden)
        wd = synth.weights(td, 3, hidden, inter)
        x = synth.normal_f32(4, hidden)
        d_acts = torch.empty(hidden // 32 * 34, dtype=torch.uint8, device=DEV)
        hip.quantize_q8_0_dev(dev(x), d_acts)
        ws = torch.empty(L.ffn_workspace_bytes(hidden, inter), dtype=torch.uint8, device=DEV)
        d_out = torch.empty(hidden, dtype=torch.float32, device=DEV)
        d_wg, d_wu, d_wd = dev(wg), dev(wu), dev(wd)
        L.ffn_swiglu_dev((tg, d_wg), (tu, d_wu), (td, d_wd), d_acts, d_out, hidden, inter, ws)
        got = host(d_out)
        tuning("ffn_fusion", 0)  # gate + up, SwiGLU, down as three launches: the same bits
        d_out3 = torch.empty_like(d_out)
        L.ffn_swiglu_dev((tg, d_wg), (tu, d_wu), (td, d_wd), d_acts, d_out3, hidden, inter, ws)
        assert np.array_equal(got.view(np.uint32), host(d_out3).view(np.uint32))
        tuning("ffn_fusion", 1)
        # step by step with the plain entry points: bit-identical
        g = torch.empty(inter, dtype=torch.float32, device=DEV)
        u = torch.empty(inter, dtype=torch.float32, device=DEV)
        hip.HipKernel(tg).matvec_q8_fused_dev(d_wg, d_acts, g, inter, hidden, accumulate=False)
        hip.HipKernel(tu).matvec_q8_fused_dev(d_wu, d_acts, u, inter, hidden, accumulate=False)
        hq = torch.empty(inter // 32 * 34, dtype=torch.uint8, device=DEV)
        L.swiglu_quantize_dev(g, u, None, hq)
        step = torch.empty(hidden, dtype=torch.float32, device=DEV)
        hip.HipKernel(td).matvec_q8_fused_dev(d_wd, hq, step, hidden, inter, accumulate=False)
        assert np.array_equal(got, host(step))
        # against the oracle end to end: gate/up within 1e-5, then the oracle's SwiGLU and down on
        # the oracle's own h; Q8_0 re-quantization of h amplifies last-place differences of gate/up,
        # so the end-to-end bar is the quantization step of h (1/127 of a block's range) carried
        # through down -- checked instead on the GPU's own h, which isolates each stage exactly.
        acts = host(d_acts)
        g_ref = ref.matvec_q8_fused_mt(tg, wg, acts, inter, hidden, 8)
        u_ref = ref.matvec_q8_fused_mt(tu, wu, acts, inter, hidden, 8)
        assert_close(host(g), g_ref, "gate")
        assert_close(host(u), u_ref, "up")
        h_gpu = ref.swiglu(host(g), host(u))
        hq_ref = ref.quantize_q8_0(h_gpu)
        same = np.mean(host(hq) == hq_ref)
        assert same > 0.999, f"only {same:.5f} of the h bytes match the oracle's SwiGLU of the same gate/up"
        down_ref = ref.matvec_q8_fused_mt(td, wd, host(hq), hidden, inter, 8)
        assert_close(got, down_ref, "down")


@pytest.mark.parametrize("t", [O.Q4_K, O.Q6_K, O.Q8_0, O.Q4_0, O.IQ4_XS, O.Q5_K, O.Q4_1, O.Q5_0, O.Q5_1], ids=lambda t: O.NAMES[t])
def test_gate_up_swiglu_one_launch(hip, ref, t):
    """gate + up + SwiGLU + quantize in one launch: the bytes (and h) of the separate calls, bit for bit."""
    for hidden, inter in ((256, 64), (4096, 14336), (2048, 5632), (5120, 96)):  # (5120: two steps per row for the K-quants too)
        if hidden > 4096 and t not in (O.Q4_K, O.Q6_K, O.Q5_K):
            continue  # (more than two steps of 64 lanes for the formats whose lanes take 32 weights: separate launches)
        say("gate_up_swiglu", O.NAMES[t], hidden, inter)
        if t in (O.Q4_K, O.Q6_K, O.Q8_0, O.Q4_0, O.IQ4_XS):
            wg, wu = synth.weights(t, 21, inter, hidden), synth.weights(t, 22, inter, hidden)
        else:
            wg, wu = O.random_blocks(t, 21, inter, hidden), O.random_blocks(t, 22, inter, hidden)
        x = synth.normal_f32(23, hidden)
        d_acts = torch.empty(hidden // 32 * 34, dtype=torch.uint8, device=DEV)
        hip.quantize_q8_0_dev(dev(x), d_acts)
        d_wg, d_wu = dev(wg), dev(wu)
        hq = torch.zeros(inter // 32 * 34, dtype=torch.uint8, device=DEV)
        h = torch.zeros(inter, dtype=torch.float32, device=DEV)
        L.gate_up_swiglu_dev(t, d_wg, d_wu, d_acts, h, hq, inter, hidden)
        g = torch.empty(inter, dtype=torch.float32, device=DEV)
        u = torch.empty(inter, dtype=torch.float32, device=DEV)
        hip.HipKernel(t).matvec_q8_fused_dev(d_wg, d_acts, g, inter, hidden, accumulate=False)
        hip.HipKernel(t).matvec_q8_fused_dev(d_wu, d_acts, u, inter, hidden, accumulate=False)
        hq2 = torch.zeros_like(hq)
        h2 = torch.zeros_like(h)
        L.swiglu_quantize_dev(g, u, h2, hq2)
        assert np.array_equal(host(hq), host(hq2))
        assert np.array_equal(host(h).view(np.uint32), host(h2).view(np.uint32))
        # and against the oracle: the SwiGLU of the oracle's own gate / up sums, within the fp32 bar
        acts = host(d_acts)
        h_ref = ref.swiglu(ref.matvec_q8_fused_mt(t, wg, acts, inter, hidden, 8),
                           ref.matvec_q8_fused_mt(t, wu, acts, inter, hidden, 8))
        assert_close(host(h), h_ref, "h")
        hq3 = torch.zeros_like(hq)  # without the fp32 copy of h
        L.gate_up_swiglu_dev(t, d_wg, d_wu, d_acts, None, hq3, inter, hidden)
        assert np.array_equal(host(hq3), host(hq2))


def test_gate_up_swiglu_unsupported(hip):
    z = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    with pytest.raises(hip.UnsupportedShape):  # rows of 16384 columns take four waves per row
        L.gate_up_swiglu_dev(O.Q4_K, z, z, z, None, z, 32, 16384)
    with pytest.raises(hip.UnsupportedShape):  # a format without the fused kernel
        L.gate_up_swiglu_dev(O.Q2_K, z, z, z, None, z, 32, 256)
    with pytest.raises(hip.UnsupportedShape):  # not whole Q8_0 blocks of h
        L.gate_up_swiglu_dev(O.Q4_K, z, z, z, None, z, 48, 256)


def test_ffn_swiglu_errors(hip):
    z = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    with pytest.raises(hip.BufferTooSmall) as e:
        L.ffn_swiglu_dev((O.Q4_K, z), (O.Q4_K, z), (O.Q6_K, z), z, z, 256, 512, z[:64])
    assert e.value.needed == L.ffn_workspace_bytes(256, 512)
    with pytest.raises(hip.UnsupportedShape):
        L.ffn_swiglu_dev((O.Q4_K, z), (O.Q4_K, z), (O.Q6_K, z), z, z, 100, 512, z)


# ---- top-k / argmax of the logits ------------------------------------------------------------------

def test_topk_matches_oracle(hip, ref):
    rng = np.random.default_rng(21)
    for n, ks in ((128256, (1, 40, 256)), (1000, (1, 7, 256)), (5, (1, 5)), (300000, (2, 50)), (1 << 20, (1, 64)),
                  (151936, (1, 40, 64)), (262144, (40,)), (4097, (3, 64))):
        v = (rng.standard_normal(n) * 3).astype(np.float32)
        if n > 2000:
            v[1000:1010] = v[17]          # exact ties across and inside slices
            v[5] = v.max()                # two equal maxima: the lower index wins
            v[n - 1] = np.float32(np.inf)
            v[n // 2] = np.float32(-np.inf)
            v[123] = np.float32(np.nan)   # NaN ranks last
        d_v = dev(v)
        for k in ks:
            say("topk n", n, "k", k)
            ws = torch.empty(L.topk_workspace_bytes(n, k) // 8, dtype=torch.int64, device=DEV)
            d_vals = torch.empty(k, dtype=torch.float32, device=DEV)
            d_idx = torch.empty(k, dtype=torch.int32, device=DEV)
            L.topk_dev(d_v, k, d_vals, d_idx, ws)
            vals, idx = host(d_vals), host(d_idx).view(np.uint32)
            if n <= 130000:  # the oracle's selection is O(n k)
                want_vals, want_idx = ref.topk(v, k)
            else:
                key = np.where(np.isnan(v), -np.inf, v.astype(np.float64))
                order = np.argsort(-key, kind="stable")[:k]
                want_vals, want_idx = v[order], order.astype(np.uint32)
            assert np.array_equal(idx, want_idx), f"indices differ at {np.nonzero(idx != want_idx)[0][:5]}"
            assert np.array_equal(vals.view(np.uint32), want_vals.view(np.uint32))
        v2 = np.where(np.isnan(v), np.float32(-np.inf), v)
        ws = torch.empty(L.topk_workspace_bytes(n, 1) // 8, dtype=torch.int64, device=DEV)
        d_vals, d_idx = torch.empty(1, dtype=torch.float32, device=DEV), torch.empty(1, dtype=torch.int32, device=DEV)
        L.topk_dev(dev(v2), 1, d_vals, d_idx, ws)
        assert int(host(d_idx)[0]) == ref.argmax(v2)  # k = 1 is the reference's argmax


def _topk_check(v, k, offset=0):
    """offset: the vector starts that many floats into its allocation (not on a 16-byte boundary)."""
    d_all = dev(v)
    v = v[offset:]
    n = v.size
    ws = torch.empty(max(L.topk_workspace_bytes(n, k) // 8, 1), dtype=torch.int64, device=DEV)
    d_vals = torch.empty(k, dtype=torch.float32, device=DEV)
    d_idx = torch.empty(k, dtype=torch.int32, device=DEV)
    L.topk_dev(d_all[offset:], k, d_vals, d_idx, ws)
    vals, idx = host(d_vals), host(d_idx).view(np.uint32)
    key = np.where(np.isnan(v), -np.inf, v.astype(np.float64))
    order = np.argsort(-key, kind="stable")[:k]  # value descending, lower index first among equals
    assert np.array_equal(idx, order.astype(np.uint32)), f"indices differ at {np.nonzero(idx != order)[0][:5]}"
    assert np.array_equal(vals.view(np.uint32), v[order].view(np.uint32))


@pytest.mark.parametrize("k", [8, 39, 40, 64, 65, 100, 200, 256])
def test_topk_radix_select_cases(hip, k):
    """The one-work-group radix select (k >= 8): distributions that stress each of its stages."""
    rng = np.random.default_rng(100 + k)
    n = 128256
    say("topk select k", k)
    _topk_check((rng.standard_normal(n) * 3).astype(np.float32), k)               # logits-like
    _topk_check(np.full(n, 1.25, dtype=np.float32), k)                               # all equal: decided by index alone
    masked = (rng.standard_normal(n) * 3).astype(np.float32)
    masked[rng.random(n) < 0.9] = -np.inf                                            # 90 % masked out
    _topk_check(masked, k)
    few = np.full(n, -np.inf, dtype=np.float32)                                      # fewer finite values than k
    few[rng.choice(n, k // 2, replace=False)] = rng.standard_normal(k // 2).astype(np.float32)
    _topk_check(few, k)
    close = (1.0 + rng.integers(0, 3, n) * np.float32(2.0 ** -23)).astype(np.float32)  # three adjacent floats, many ties
    _topk_check(close, k)
    _topk_check(rng.integers(-3, 4, n).astype(np.float32), k)                        # seven distinct values incl. +-0
    wide = (rng.standard_normal(n) * np.exp(rng.uniform(-30, 30, n))).astype(np.float32)
    _topk_check(wide, k)
    _topk_check(rng.standard_normal(k).astype(np.float32), k)                        # n == k
    _topk_check(rng.standard_normal(20000).astype(np.float32), k)
    _topk_check(np.sort(rng.standard_normal(300000).astype(np.float32)), k)         # ascending: winners at the end
    # the layout that defeats the filter by thread maxima: all large values in the shares of 200 of the 1024 threads
    # (thread of index i: (i % 16384) // 4 % 1024), so that more keys pass the filter than LDS holds
    adv = (rng.standard_normal(n) * 0.01).astype(np.float32)
    owner = (np.arange(n) % 16384) // 4 % 1024
    adv[owner < 200] += 100.0
    _topk_check(adv, k)
    for off, n2 in ((1, 128255), (3, 70001), (0, 70002), (0, 70003)):                 # unaligned start; n % 4 = 1, 2, 3
        _topk_check((rng.standard_normal(n2 + off) * 3).astype(np.float32), k, offset=off)


def test_topk_argument_errors(hip):
    v = torch.zeros(64, dtype=torch.float32, device=DEV)
    ws = torch.empty(4096, dtype=torch.int64, device=DEV)
    out_v, out_i = torch.empty(300, dtype=torch.float32, device=DEV), torch.empty(300, dtype=torch.int32, device=DEV)
    with pytest.raises(hip.DimensionMismatch):
        L.topk_dev(v, 0, out_v, out_i, ws)
    with pytest.raises(hip.DimensionMismatch):
        L.topk_dev(v, 65, out_v, out_i, ws)
    big = torch.zeros(1024, dtype=torch.float32, device=DEV)
    with pytest.raises(hip.UnsupportedShape):
        L.topk_dev(big, 257, out_v, out_i, ws)
    with pytest.raises(hip.BufferTooSmall):
        L.topk_dev(big, 16, out_v, out_i, ws[:1])
    assert L.topk_workspace_bytes((1 << 20) + 1, 4) == 0
