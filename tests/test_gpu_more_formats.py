"""Parity of the HIP path for the formats beyond the first five (Q4_1, Q5_0, Q5_1, Q8_1, IQ4_NL,
Q2_K, Q3_K, Q5_K) against the CPU oracle, through the C ABI: dequant_block and integer group
sums bit-exact, fp32 within 1e-5 * |y_ref|_inf of the reference's *Ref kernels
(crates/oxillama-quant/src/reference/*.rs).  Weights are random bytes with finite f16 scale
fields, so every bit pattern of the payload is exercised."""
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
TYPES = O.MORE_TYPES
TILE_TYPES = [O.Q5_K, O.Q4_1, O.Q5_0, O.Q5_1, O.Q8_1, O.IQ4_NL, O.Q3_K, O.Q2_K]
ids = lambda t: O.NAMES[t]


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


KAT_BLOCKS = {
    O.Q4_1: [O.make_q4_1_block(1.0, 2.0, [0x88] * 16), O.make_q4_1_block(0.0, 5.0, [0] * 16)],
    O.Q5_0: [O.make_q5_0_block(1.0, 0xFFFFFFFF, [0xFF] * 16), O.make_q5_0_block(2.0, 0, [0] * 16),
             O.make_q5_0_block(0.5, 0xA5A5A5A5, [(i * 11 + 5) & 0xFF for i in range(16)])],
    O.Q5_1: [O.make_q5_1_block(1.0, 0.0, 0xFFFFFFFF, [0xFF] * 16), O.make_q5_1_block(0.0, 3.0, 0, [0] * 16)],
    O.Q8_1: [O.make_q8_1_block(0.5, [10] * 32), O.make_q8_1_block(2.0, [-5] * 32)],
    O.IQ4_NL: [O.make_iq4_nl_block(1.0, [0x50] + [0] * 15), O.make_iq4_nl_block(1.0, [0xFF] * 16)],
    O.Q2_K: [O.make_q2_k_block(1.0, 0.0, [0x01] * 16, [0xFF] * 64), O.make_q2_k_block(2.0, 1.0, [0x11] * 16, [0] * 64)],
    O.Q3_K: [O.make_q3_k_block(1.0, [0xA1] * 8 + [0x11] * 4, [0] * 32, [0] * 64),
             O.make_q3_k_block(1.0, [0xA1] * 8 + [0x11] * 4, [0xFF] * 32, [0xFF] * 64)],
    O.Q5_K: [O.make_q5_k_block(1.0, 0.0, [1] * 4 + [0] * 4 + [1] * 4, [0] * 32, [0x88] * 128),
             O.make_q5_k_block(1.0, 0.0, [1] * 4 + [0] * 4 + [1] * 4, [0xFF] * 32, [0] * 128)],
}
KAT_VALUES = {O.Q4_1: [10.0, 5.0], O.Q5_0: [15.0, -32.0, None], O.Q5_1: [31.0, 3.0], O.Q8_1: [5.0, -10.0],
              O.IQ4_NL: [None, 113.0], O.Q2_K: [3.0, -1.0], O.Q3_K: [-4.0, 3.0], O.Q5_K: [8.0, 16.0]}


@pytest.mark.parametrize("t", TYPES, ids=ids)
def test_metadata_and_dispatch(hip, t):
    k = hip.KernelDispatcher().get_kernel(t)
    assert (k.block_size(), k.block_bytes(), k.name()) == (*O.BLOCK[t], O.NAMES[t])
    # the int8-MFMA tile kernel takes all of them
    assert (k.gemm_workspace_bytes(64, 4096, 4096) > 0) == (t in TILE_TYPES)


def test_unknown_types_still_rejected(hip):
    for t in (0, 1, 15, 16, 24, 30, 99):  # F32, F16, Q8_K, IQ2_XXS, I8, BF16, nonsense
        with pytest.raises(hip.UnsupportedType):
            hip.HipKernel(t)


@pytest.mark.parametrize("t", TYPES, ids=ids)
def test_dequant_block(hip, ref, t):
    bs, bb = O.BLOCK[t]
    k = hip.HipKernel(t)
    for blk, val in zip(KAT_BLOCKS[t], KAT_VALUES[t]):  # the reference's hand-built blocks
        out = np.zeros(bs, dtype=np.float32)
        k.dequant_block(np.frombuffer(blk, dtype=np.uint8), out)
        if val is not None:
            assert np.all(out == val)
        assert np.array_equal(out, ref.dequant_block(t, np.frombuffer(blk, dtype=np.uint8)))
    w = O.random_blocks(t, 200 + t, 12, bs)
    for i in range(12):
        out = np.zeros(bs, dtype=np.float32)
        k.dequant_block(w[i * bb:(i + 1) * bb], out)
        assert np.array_equal(out, ref.dequant_block(t, w[i * bb:(i + 1) * bb])), f"block {i}"
    with pytest.raises(hip.BufferTooSmall) as e:
        k.dequant_block(w[:bb - 1], np.zeros(bs, dtype=np.float32))
    assert (e.value.needed, e.value.available) == (bb, bb - 1)


SHAPES = ((5, 256), (96, 512), (64, 4096), (33, 14336), (9, 2 * 32768 + 256))


@pytest.mark.parametrize("t", TYPES, ids=ids)
def test_fused_matvec_sums_and_fp32(hip, ref, t):
    k = hip.HipKernel(t)
    for seed, (n_rows, n_cols) in enumerate(SHAPES):
        say("fused", O.NAMES[t], n_rows, n_cols)
        w = O.random_blocks(t, 300 + 10 * t + seed, n_rows, n_cols)
        x = synth.normal_f32(400 + seed, n_cols)
        a = ref.quantize_q8_0(x)
        sums = k.block_sums(w, a, n_rows, n_cols)
        assert np.array_equal(sums, ref.block_sums(t, w, a, n_rows, n_cols)), "integer group sums"
        out = np.full(n_rows, 42.0, dtype=np.float32)  # accumulate semantics (traits.rs:169)
        k.matvec_q8_fused(w, a, out, n_rows, n_cols)
        want = ref.matvec_q8_fused(t, w, a, n_rows, n_cols, out=np.full(n_rows, 42.0, dtype=np.float32))
        # Rows of 65 792 columns (the kernel without cached activations): the reference adds every element
        # into one fp32 accumulator, whose own rounding noise there is about sqrt(n) * 2^-24 * |partial sums|,
        # i.e. 1e-5 of |y|; the bar is widened for that shape only.
        assert_close(out - 42.0, want - 42.0, f"fused {O.NAMES[t]} {n_rows}x{n_cols}",
                     tol=FP32_REL_TOL if n_cols <= 32768 else 5e-5)
        # zero activations contribute nothing (q4_0.rs:382-392 applied to every format)
        zero = ref.quantize_q8_0(np.zeros(n_cols, dtype=np.float32))
        out = np.full(n_rows, 77.0, dtype=np.float32)
        k.matvec_q8_fused(w, zero, out, n_rows, n_cols)
        assert np.all(out == 77.0)


@pytest.mark.parametrize("t", TYPES, ids=ids)
def test_rows_that_end_inside_a_block(hip, ref, t):
    """n_cols that is not a whole number of blocks: the reference's fused rows skip the columns past it
    (traits.rs:150-166 for the 32-weight formats; q2_k.rs:224-292, q3_k.rs:258-322, q5_k.rs:270-345).  The
    activation blocks past n_cols hold non-zero bytes, so a kernel that did not skip them fails."""
    k = hip.HipKernel(t)
    bs = O.BLOCK[t][0]
    for i, n_cols in enumerate((20, 45, 1000, 4101) if bs == 32 else (200, 300, 1000, 4097, 14336 - 100)):
        n_rows = (33, 64, 40, 35, 48)[i]
        full = -(-n_cols // bs) * bs
        say("ragged", O.NAMES[t], n_rows, n_cols, "of", full)
        w = O.random_blocks(t, 900 + 10 * t + i, n_rows, full)
        x = synth.normal_f32(950 + i, full)
        a = ref.quantize_q8_0(x)
        want = ref.matvec_q8_fused(t, w, a, n_rows, n_cols)
        out = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(w, a, out, n_rows, n_cols)
        assert_close(out, want, f"fused {O.NAMES[t]} {n_rows}x{n_cols}")
        y = torch.full((n_rows,), 2.0, dtype=torch.float32, device=DEV)
        k.matvec_q8_fused_dev(dev(w), dev(a), y, n_rows, n_cols, accumulate=True)
        assert np.array_equal(host(y), np.float32(2.0) + out)
        # fp32 activations, exactly n_cols of them: quantize (zero-padded) + fused
        xz = x.copy()
        xz[n_cols:] = 0.0
        want_q = ref.matvec_q8_fused(t, w, ref.quantize_q8_0(xz), n_rows, n_cols)
        yg = torch.zeros(n_rows, dtype=torch.float32, device=DEV)
        k.gemv_dev(dev(w), dev(x[:n_cols].copy()), yg, n_rows, n_cols)
        assert_close(host(yg), want_q, "gemv_dev ragged")
        yh = np.full(n_rows, 7.0, dtype=np.float32)
        k.gemv(hip.QuantTensor(w, [n_rows, n_cols], t), x[:n_cols], yh)
        assert_close(yh, want_q, "gemv ragged")
        xs = synth.normal_f32(970 + i, 7 * n_cols).reshape(7, n_cols)
        ym = np.zeros((7, n_rows), dtype=np.float32)
        k.gemm(hip.QuantTensor(w, [n_rows, n_cols], t), xs, ym, 7, n_rows, n_cols)
        for r in range(7):
            xr = np.zeros(full, dtype=np.float32)
            xr[:n_cols] = xs[r]
            assert_close(ym[r], ref.matvec_q8_fused(t, w, ref.quantize_q8_0(xr), n_rows, n_cols), f"gemm ragged row {r}")


@pytest.mark.parametrize("t", [O.IQ4_NL, O.Q5_0], ids=ids)
def test_weights_two_bytes_off_a_dword_boundary(hip, ref, t):
    """The 18- and 22-byte formats pick one of two load forms per block from the block's address; a matrix
    that starts two bytes off a dword boundary swaps the forms of all its blocks and must give the same bits."""
    for n_rows, n_cols in ((40, 4096), (16, 14336)):
        w = O.random_blocks(t, 990 + t, n_rows, n_cols)
        da = dev(ref.quantize_q8_0(synth.normal_f32(991, n_cols)))
        aligned = dev(w)
        buf = torch.zeros(w.size + 8, dtype=torch.uint8, device=DEV)
        buf[2:2 + w.size] = aligned
        y0 = torch.zeros(n_rows, dtype=torch.float32, device=DEV)
        y2 = torch.zeros(n_rows, dtype=torch.float32, device=DEV)
        k = hip.HipKernel(t)
        k.matvec_q8_fused_dev(aligned, da, y0, n_rows, n_cols, accumulate=False)
        k.matvec_q8_fused_dev(buf[2:], da, y2, n_rows, n_cols, accumulate=False)
        assert np.array_equal(host(y0), host(y2)), (O.NAMES[t], n_rows, n_cols)


@pytest.mark.parametrize("t", TYPES, ids=ids)
def test_gemv_gemm_host_route(hip, ref, t):
    n, kk = 160, 1024
    w = O.random_blocks(t, 500 + t, n, kk)
    k = hip.HipKernel(t)
    qt = hip.QuantTensor(w, [n, kk], t)
    x = synth.normal_f32(3, kk)
    y = np.full(n, -1.0, dtype=np.float32)
    k.gemv(qt, x, y)
    z = np.zeros(n, dtype=np.float32)
    k.matvec_q8_fused(w, ref.quantize_q8_0(x), z, n, kk)
    assert np.array_equal(y, z)  # gemv = quantize + fused into zeros
    # against the reference's fp32-activation gemv: equal up to the Q8_0 rounding of x (about 1/127 per element)
    y_f32 = ref.gemv(t, w, n, kk, x)
    assert np.abs(y - y_f32).max() <= 0.02 * np.abs(y_f32).max()
    for m in (2, 5, 13):  # several vectors per pass, chunks of four, more rows than the tile threshold
        xs = synth.normal_f32(10 + m, m * kk)
        ys = np.zeros(m * n, dtype=np.float32)
        k.gemm(qt, xs, ys, m, n, kk)
        for r in range(m):
            yr = np.zeros(n, dtype=np.float32)
            k.gemv(qt, xs[r * kk:(r + 1) * kk], yr)
            if m >= 9 and t in TILE_TYPES:  # the tile kernel adds the groups in another order
                assert_close(ys[r * n:(r + 1) * n], yr, f"gemm row {r} of {m}")
            else:
                assert np.array_equal(ys[r * n:(r + 1) * n], yr), f"gemm row {r} of {m}"
        assert_close(ys, ref.gemm_q8(t, w, xs, m, n, kk).ravel(), f"gemm {m}")
    with pytest.raises(hip.DimensionMismatch) as e:
        k.gemv(qt, x[:-1], y)
    assert (e.value.expected, e.value.got) == (kk, kk - 1)


@pytest.mark.parametrize("t", TYPES, ids=ids)
def test_device_route_forms(hip, ref, t):
    """fp32 activations quantized in the kernel, bias epilogue, several matrices of different heights in one
    launch, several vectors per pass: each bit-identical to the plain fused launch."""
    k = hip.HipKernel(t)
    for n_cols, heights in ((4096, (1024, 256, 512)), (14336, (96, 200))):
        say("device forms", O.NAMES[t], n_cols, heights)
        x = synth.normal_f32(5, n_cols)
        d_x = dev(x)
        d_acts = torch.empty(n_cols // 32 * 34, dtype=torch.uint8, device=DEV)
        hip.quantize_q8_0_dev(d_x, d_acts)
        ws, bs_, singles = [], [], []
        for i, h in enumerate(heights):
            w = dev(O.random_blocks(t, 600 + 10 * t + i, h, n_cols))
            b = dev(synth.normal_f32(40 + i, h))
            one = torch.zeros(h, dtype=torch.float32, device=DEV)
            k.matvec_q8_fused_dev(w, d_acts, one, h, n_cols, accumulate=False)
            ws.append(w); bs_.append(b); singles.append(host(one))
            f32 = torch.empty(h, dtype=torch.float32, device=DEV)
            k.gemv_dev(w, d_x, f32, h, n_cols)
            assert np.array_equal(host(f32), singles[i]), "in-kernel quantization"
        outs = [torch.empty(h, dtype=torch.float32, device=DEV) for h in heights]
        L.linear_forward_multi_dev(t, ws, d_acts, outs, heights, n_cols, d_biases=bs_)
        for i, h in enumerate(heights):
            assert np.array_equal(host(outs[i]), (singles[i] + host(bs_[i])).astype(np.float32)), f"matrix {i}"
        # against the oracle
        want = ref.matvec_q8_fused_mt(t, host(ws[0]), host(d_acts), heights[0], n_cols, 8)
        assert_close(singles[0], want, "device fused")
        # a small batch through the batched entry point (GEMV launches of up to four vectors)
        m = 4
        xs = synth.normal_f32(77, m * n_cols)
        d_as = torch.empty(m * (n_cols // 32 * 34), dtype=torch.uint8, device=DEV)
        hip.quantize_q8_0_dev(dev(xs), d_as)
        d_y = torch.empty(m * heights[0], dtype=torch.float32, device=DEV)
        k.gemm_q8_dev(ws[0], d_as, d_y, m, heights[0], n_cols)
        ys = host(d_y).reshape(m, heights[0])
        for r in range(m):
            one = torch.zeros(heights[0], dtype=torch.float32, device=DEV)
            k.matvec_q8_fused_dev(ws[0], d_as[r * (n_cols // 32 * 34):], one, heights[0], n_cols, accumulate=False)
            assert np.array_equal(ys[r], host(one)), f"batch row {r}"


def test_grouped_form_reports_unsupported(hip):
    z = torch.zeros(4096, dtype=torch.uint8, device=DEV)
    k = hip.HipKernel(O.Q5_0)  # the tile kernel walks 256 columns at a time: rows of at least eight blocks
    assert k.moe_gemm_workspace_bytes(64, 256, 288) > 0
    assert k.moe_gemm_workspace_bytes(64, 256, 224) == 0
    with pytest.raises(hip.UnsupportedShape):
        k.moe_gemm_q8_dev(z, 256 * 7 * 22, 1, z, z, 4, 4, z, 256, 224, z)
    k = hip.HipKernel(O.Q5_K)  # ... and the 256-weight formats whole super-blocks, which the shape check says first
    assert k.moe_gemm_workspace_bytes(64, 256, 288) == 0


def _tile_zero_point(t, acts, rows, k_):
    """Q5_0's tile policy multiplies the unsigned 5-bit values and applies the "- 16" in fp32 through the
    zero-point term, so its integer sums are sum q5*a = sum (q5 - 16)*a + 16 * sum a."""
    if t != O.Q5_0:
        return 0
    a = acts.reshape(rows, k_ // 32, 34)[:, :, 2:].view(np.int8).astype(np.int32).sum(axis=2)
    return (16 * a)[:, None, :]


@pytest.mark.parametrize("shape", [(8, 32, 256), (40, 100, 1024), (130, 129, 2048), (200, 257, 1024), (512, 160, 512)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("t", TILE_TYPES, ids=ids)
def test_prefill_tile_kernel(hip, ref, tuning, shape, t):
    """The int8-MFMA tile kernel on the added formats: integer sub-block sums bit-exact, fp32 within 1e-5 of
    the reference's fused kernel, every tile shape (split k, 64 x 128, 128 x 64), ragged edges, accumulate."""
    say("prefill", O.NAMES[t], shape)
    tuning("gemm_tile_min_rows", 1)
    _prefill_tile_case(hip, ref, shape, t)


@pytest.mark.parametrize("shape", [(8, 32, 288), (33, 100, 416), (130, 129, 352), (40, 64, 1408), (450, 140, 480)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("t", [t for t in TILE_TYPES if O.BLOCK[t][0] == 32], ids=ids)
def test_prefill_tile_kernel_rows_of_whole_32_blocks(hip, ref, tuning, shape, t):
    """Rows of whole 32-weight blocks that are not whole 256-weight steps, on the added formats of independent
    blocks: the same bars."""
    say("prefill, ragged k", O.NAMES[t], shape)
    tuning("gemm_tile_min_rows", 1)
    _prefill_tile_case(hip, ref, shape, t)


@pytest.mark.parametrize("t", TILE_TYPES, ids=ids)
def test_prefill_many_tokens_takes_the_wide_tile_shape(hip, ref, t):
    """More than 384 tokens on a matrix whose 128 x 128 work-group tiles give every compute unit one and a half: the
    library's own choice is the shape with four token tiles against one weight-row tile per wave.  Sampled tokens
    against the oracle on all outputs (ragged n); the debug dump's launch (another shape) gives the same bits."""
    from oxillama_amd import capi
    import ctypes as C
    cus = hip.device_info()["compute_units"]
    m, k_ = 400, 256
    n = 128 * ((3 * cus + 7) // 8) - 5
    say("prefill, wide tiles", O.NAMES[t], (m, n, k_))
    w = O.random_blocks(t, 990, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(991, m * k_))
    kern = hip.HipKernel(t)
    dw, da = dev(w), dev(acts)
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device=DEV)
    dy = torch.full((m + 1, n), 7.0, dtype=torch.float32, device=DEV)
    kern.gemm_q8_dev(dw, da, dy, m, n, k_, accumulate=False, workspace=ws)
    torch.cuda.synchronize()
    buf = C.create_string_buffer(256)
    capi.load().oxq_last_launch(buf, 256)
    took = buf.value.decode()
    assert took.startswith("gemm_tile_kernel") and ",4,1,1,1>" in took, took
    rows = sorted(set(list(range(0, m, 37)) + [127, 128, 383, 384, m - 1]))
    arb = k_ // 32 * 34
    y = host(dy)
    assert np.all(y[m] == 7.0)
    y_ref = np.stack([ref.matvec_q8_fused_mt(t, w, acts[r * arb:(r + 1) * arb], n, k_, 16) for r in rows])
    assert_close(y[rows], y_ref, f"wide tiles {O.NAMES[t]}")
    dsum = torch.empty((m, n, k_ // O.GROUP_COLS[t]), dtype=torch.int32, device=DEV)
    dy2 = torch.empty((m, n), dtype=torch.float32, device=DEV)
    kern.gemm_block_sums_dev(dw, da, dy2, dsum, m, n, k_, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(dy2, dy[:m])


def _prefill_tile_case(hip, ref, shape, t):
    m, n, k_ = shape
    if True:
        w = O.random_blocks(t, 900 + m, n, k_)
        x = synth.normal_f32(950 + n, m * k_)
        acts = ref.quantize_q8_0(x)
        kern = hip.HipKernel(t)
        ws_bytes = kern.gemm_workspace_bytes(m, n, k_)
        assert ws_bytes > 0
        dw, da = dev(w), dev(acts)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
        dy = torch.full((m, n), 7.0, dtype=torch.float32, device=DEV)
        kern.gemm_q8_dev(dw, da, dy, m, n, k_, accumulate=False, workspace=ws)
        arb = k_ // 32 * 34
        y_ref = np.stack([ref.matvec_q8_fused_mt(t, w, acts[r * arb:(r + 1) * arb], n, k_, 16) for r in range(m)])
        assert_close(host(dy), y_ref, f"prefill {O.NAMES[t]} {shape}")
        dy2 = dy.clone()
        kern.gemm_q8_dev(dw, da, dy2, m, n, k_, accumulate=True, workspace=None)
        torch.cuda.synchronize()
        assert torch.equal(dy2, dy + dy)
        dsum = torch.empty((m, n, k_ // O.GROUP_COLS[t]), dtype=torch.int32, device=DEV)  # Q2_K, Q3_K: 16-weight groups
        dy3 = torch.empty_like(dy)
        kern.gemm_block_sums_dev(dw, da, dy3, dsum, m, n, k_, workspace=ws)
        want = np.stack([ref.block_sums(t, w, acts[r * arb:(r + 1) * arb], n, k_) for r in range(m)])
        assert np.array_equal(host(dsum) - _tile_zero_point(t, acts, m, k_), want), "integer sub-block sums"
        assert torch.equal(dy3, dy)


@pytest.mark.parametrize("t", [O.Q5_K, O.Q5_0, O.IQ4_NL, O.Q3_K, O.Q2_K], ids=ids)
def test_grouped_expert_matmul(hip, ref, t):
    """Grouped (mixture-of-experts) form on added formats: each expert's rows against its own weights."""
    n_exp, n, k_ = 4, 96, 512
    rows = [5, 0, 33, 17]
    total = sum(rows)
    offsets = np.concatenate([[0], np.cumsum(rows)]).astype(np.int32)
    bs, bb = O.BLOCK[t]
    stride = n * (k_ // bs) * bb
    w = O.random_blocks(t, 77, n_exp * n, k_)
    x = synth.normal_f32(78, total * k_)
    acts = ref.quantize_q8_0(x)
    kern = hip.HipKernel(t)
    ws = torch.empty(kern.moe_gemm_workspace_bytes(total, n, k_), dtype=torch.uint8, device=DEV)
    dy = torch.zeros((total, n), dtype=torch.float32, device=DEV)
    kern.moe_gemm_q8_dev(dev(w), stride, n_exp, dev(acts), dev(offsets), total, max(rows), dy, n, k_, ws)
    got = host(dy)
    arb = k_ // 32 * 34
    for e in range(n_exp):
        for r in range(offsets[e], offsets[e + 1]):
            want = ref.matvec_q8_fused(t, w[e * stride:(e + 1) * stride], acts[r * arb:(r + 1) * arb], n, k_)
            assert_close(got[r], want, f"expert {e} row {r}")
