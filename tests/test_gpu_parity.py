"""Parity of the HIP path (through the C ABI) against the CPU oracle on identical
seeded inputs.  Bars: Q8_0 activation bytes and integer group sums bit-exact; fp32
outputs within 1e-5 * |y_ref|_inf (block-accumulation order differs)."""
import sys

import numpy as np
import pytest

import fixtures as FX
import oracle as O
from oxillama_amd import synth

pytestmark = pytest.mark.gpu

FP32_REL_TOL = 1e-5  # max|y - y_ref| <= 1e-5 * max|y_ref|


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def assert_close(y, y_ref, what):
    scale = float(np.abs(y_ref).max())
    err = float(np.abs(y.astype(np.float64) - y_ref.astype(np.float64)).max())
    assert err <= FP32_REL_TOL * scale + 1e-30, f"{what}: max err {err:.3e} > 1e-5 * {scale:.3e}"


def canonical_ref(ref, t, w, a, n_rows, n_cols, threads=8):
    """Reference-order result the GPU is held to: the AVX2 tier for Q4_0/Q8_0/Q4_K, the
    (scalar-bodied) fused kernel for Q6_K, the integer form for IQ4_XS."""
    return ref.matvec_q8_fused_mt(t, w, a, n_rows, n_cols, threads, tier=O.TIER_AVX2)


# ---- (1) Q8_0 activation quantizer -----------------------------------------------------

def test_quantize_q8_0_bit_exact_random(hip, ref):
    for seed, n, sigma in ((1, 4096, 1.0), (2, 14336, 1.0), (3, 32, 1.0), (4, 64 * 4096, 3.0), (5, 4096, 1e-4)):
        x = synth.normal_f32(seed, n, sigma)
        say("quantize seed", seed, "n", n)
        assert np.array_equal(hip.quantize_f32_to_q8_0(x), ref.quantize_q8_0(x))


def test_quantize_q8_0_bit_exact_edge_cases(hip, ref):
    rng = np.random.default_rng(7)
    blocks = []
    blocks.append(np.zeros(32, dtype=np.float32))                                   # d = 0
    b = np.zeros(32, dtype=np.float32); b[:8] = [127, .5, 1.5, 2.5, -.5, -1.5, -2.5, 3.49]; blocks.append(b)
    b = np.zeros(32, dtype=np.float32); b[0] = 1000; b[1] = -1000; b[31] = 500; blocks.append(b)  # quantize.rs:425
    blocks.append(np.full(32, -0.0, dtype=np.float32))
    blocks.append((np.arange(32, dtype=np.float32) / np.float32(15.5)) - 1)        # quantize.rs:263
    blocks.append(np.full(32, 1e-30, dtype=np.float32))                            # d underflows f16
    blocks.append(np.full(32, 6e-6, dtype=np.float32))                             # d subnormal in f16
    blocks.append((rng.standard_normal(32) * 1e4).astype(np.float32))
    blocks.append((rng.standard_normal(32) * 6e6).astype(np.float32))              # d overflows f16 -> inf
    b = rng.standard_normal(32).astype(np.float32); b[5] = np.float32(3.0e38); blocks.append(b)
    for k in range(40):                                                            # exact .5 ties after scaling
        b = (rng.integers(-254, 255, size=32) * 0.5).astype(np.float32); b[0] = 127.0; blocks.append(b)
    x = np.concatenate(blocks)
    got, want = hip.quantize_f32_to_q8_0(x), ref.quantize_q8_0(x)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, f"first mismatch at byte {bad[:5]} (block {bad[:5] // 34})"
    assert hip.quantize_f32_to_q8_0(np.zeros(0, dtype=np.float32)).size == 0       # quantize.rs:432


# ---- (2) dequant_block -------------------------------------------------------------------

@pytest.mark.parametrize("case", FX.dequant_cases(), ids=lambda c: c[0])
def test_dequant_block_known_answers(hip, ref, case):
    _, t, block, expected, tol = case
    out = np.zeros(O.BLOCK[t][0], dtype=np.float32)
    hip.HipKernel(t).dequant_block(block, out)
    for i, v in expected.items():
        assert abs(out[i] - v) <= tol
    assert np.array_equal(out, ref.dequant_block(t, block))


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_dequant_block_bit_exact_random(hip, ref, t):
    bs, bb = O.BLOCK[t]
    w = synth.weights(t, 100 + t, 8, bs)
    k = hip.HipKernel(t)
    for i in range(8):
        out = np.zeros(bs, dtype=np.float32)
        k.dequant_block(w[i * bb:(i + 1) * bb], out)
        assert np.array_equal(out, ref.dequant_block(t, w[i * bb:(i + 1) * bb]))


# ---- (3) fused matvec: the reference's own fixtures ------------------------------------------

@pytest.mark.parametrize("case", FX.fused_cases(), ids=lambda c: c[0])
def test_fused_reference_fixtures(hip, ref, case):
    name, t, w, a, n_rows, n_cols, tol = case
    say("fixture", name)
    out = np.zeros(n_rows, dtype=np.float32)
    hip.HipKernel(t).matvec_q8_fused(w, a, out, n_rows, n_cols)
    for tier in (O.TIER_SCALAR, O.TIER_AVX2):
        assert np.abs(out - ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=tier)).max() < tol
    assert np.array_equal(hip.HipKernel(t).block_sums(w, a, n_rows, n_cols), ref.block_sums(t, w, a, n_rows, n_cols))


@pytest.mark.parametrize("case", FX.accumulate_cases(), ids=lambda c: c[0])
def test_fused_accumulate_semantics(hip, case):
    _, t, w, a, n_cols, preset = case
    out = np.full(1, preset, dtype=np.float32)
    hip.HipKernel(t).matvec_q8_fused(w, a, out, 1, n_cols)
    assert out[0] == preset


def test_fused_zero_activations(hip):
    w = np.frombuffer(O.make_q4_k_block(1.0, 0.0, FX.Q4K_SCALES_ONES, [0x88] * 128), dtype=np.uint8)
    a = np.frombuffer(O.make_q8_0_block(1.0, [0] * 32) * 8, dtype=np.uint8)
    out = np.zeros(1, dtype=np.float32)
    hip.HipKernel(O.Q4_K).matvec_q8_fused(w, a, out, 1, 256)
    assert out[0] == 0.0


# ---- (4) seeded random shapes: every launch variant -------------------------------------------

def _shapes(t):
    """n_cols covering 1..8 cached steps, ragged last steps and the uncached path."""
    unit = 64 if t == O.Q6_K else 32
    bs = O.BLOCK[t][0]
    cols = set()
    for units in (1, 8, 63, 64, 65, 128, 130, 192, 250, 256, 300, 448, 512, 520, 1100):
        c = units * unit
        c = -(-c // bs) * bs
        cols.add(c)
    return sorted(cols)


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_fused_random_shapes(hip, ref, t):
    """Row counts stay >= 32 so that |y_ref|_inf is the magnitude of a typical large output, as
    in the benchmark configurations (with one or two rows it can be near zero by chance).
    Single-row behaviour is covered by the reference's own fixtures above."""
    k = hip.HipKernel(t)
    for i, n_cols in enumerate(_shapes(t)):
        n_rows = (32, 33, 64, 35, 257, 48, 37)[i % 7]
        say(O.NAMES[t], "n_rows", n_rows, "n_cols", n_cols)
        w = synth.weights(t, 1000 + i, n_rows, n_cols)
        a = ref.quantize_q8_0(synth.normal_f32(2000 + i, n_cols))
        out = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(w, a, out, n_rows, n_cols)
        y_ref = canonical_ref(ref, t, w, a, n_rows, n_cols)
        assert_close(out, y_ref, f"{O.NAMES[t]} {n_rows}x{n_cols}")
        assert np.array_equal(k.block_sums(w, a, n_rows, n_cols), ref.block_sums(t, w, a, n_rows, n_cols))
        # ACCUMULATE: a second call adds the same fp32 vector to what is there
        preset = synth.normal_f32(3000 + i, n_rows)
        acc = preset.copy()
        k.matvec_q8_fused(w, a, acc, n_rows, n_cols)
        assert np.array_equal(acc, preset + out)


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_fused_few_rows(hip, ref, t):
    """1..5 rows (ragged row batches): integer sums exact; fp32 against the exact value computed
    in float64 from the same integer sums, to the accuracy of one fp32 accumulation."""
    k = hip.HipKernel(t)
    n_cols = 2048
    for n_rows in (1, 2, 3, 5):
        w = synth.weights(t, 1500 + n_rows, n_rows, n_cols)
        a = ref.quantize_q8_0(synth.normal_f32(1600 + n_rows, n_cols))
        out = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(w, a, out, n_rows, n_cols)
        assert np.array_equal(k.block_sums(w, a, n_rows, n_cols), ref.block_sums(t, w, a, n_rows, n_cols))
        xhat = np.concatenate([ref.dequant_block(O.Q8_0, a[j:j + 34]) for j in range(0, a.size, 34)])
        wd = ref.dequant_rows(t, w, n_rows, n_cols).astype(np.float64)
        exact = wd @ xhat.astype(np.float64)
        bound = 2e-6 * (np.abs(wd) @ np.abs(xhat.astype(np.float64)))  # ~ eps * sum |terms|
        assert (np.abs(out - exact) <= bound).all()


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_fused_extreme_bytes(hip, ref, t):
    """Uniformly random block payloads (all nibble / 6-bit / int8 codes, extreme scales kept finite)
    against saturated activations: integer sums must still be exact."""
    rng = np.random.default_rng(900 + t)
    bs, bb = O.BLOCK[t]
    n_rows, n_cols = 9, 8 * 256
    w = rng.integers(0, 256, size=n_rows * (n_cols // bs) * bb, dtype=np.uint8).reshape(-1, bb)
    one = np.frombuffer(O.f16_bytes(0.0078125), dtype=np.uint8)
    if t == O.Q6_K:
        w[:, 208:210] = one
    else:
        w[:, 0:2] = one
    if t == O.Q4_K:
        w[:, 2:4] = one
    w = w.ravel()
    q = rng.choice(np.array([-128, -127, 127, 0, 1, -1], dtype=np.int8), size=n_cols)
    a = np.concatenate([np.frombuffer(O.make_q8_0_block(0.5, [int(v) for v in q[i:i + 32]]), dtype=np.uint8)
                        for i in range(0, n_cols, 32)])
    k = hip.HipKernel(t)
    assert np.array_equal(k.block_sums(w, a, n_rows, n_cols), ref.block_sums(t, w, a, n_rows, n_cols))
    out = np.zeros(n_rows, dtype=np.float32)
    k.matvec_q8_fused(w, a, out, n_rows, n_cols)
    assert_close(out, canonical_ref(ref, t, w, a, n_rows, n_cols), O.NAMES[t])


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
@pytest.mark.parametrize("n_mats", [2, 3, 4])
def test_fused_multi_matrix_launch_is_bit_identical(hip, ref, t, n_mats):
    """wq/wk/wv- or gate/up-style launch of several matrices sharing one activation vector:
    the same bits as one call per matrix, overwrite and accumulate, for row counts that are
    and are not a multiple of the kernel's batch (the latter falls back to separate launches)."""
    import torch
    for n_rows, n_cols in ((64, 4096), (36, 1024), (30, 512), (8, 14336)):
        ws = [torch.from_numpy(synth.weights(t, 800 + i, n_rows, n_cols)).cuda() for i in range(n_mats)]
        a = torch.from_numpy(ref.quantize_q8_0(synth.normal_f32(810, n_cols))).cuda()
        kern = hip.HipKernel(t)
        single = [torch.full((n_rows,), 3.0, dtype=torch.float32, device="cuda") for _ in range(n_mats)]
        multi = [torch.full((n_rows,), 3.0, dtype=torch.float32, device="cuda") for _ in range(n_mats)]
        for acc in (False, True):
            for w, y in zip(ws, single):
                kern.matvec_q8_fused_dev(w, a, y, n_rows, n_cols, accumulate=acc)
            kern.matvec_q8_fused_multi_dev(ws, a, multi, n_rows, n_cols, accumulate=acc)
            torch.cuda.synchronize()
            for y1, y2 in zip(single, multi):
                assert torch.equal(y1, y2), (O.NAMES[t], n_mats, n_rows, n_cols, acc)


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_gemv_dev_quantizes_in_kernel_bit_identically(hip, ref, t):
    """fp32 activations quantized inside the GEMV: the same bits as quantize + fused, for one and
    for several matrices, short and long rows (1, 2, 4 steps and rows split over four waves)."""
    import torch
    for n_rows, n_cols in ((48, 512), (64, 4096), (33, 8192), (20, 14336)):
        x = synth.normal_f32(820 + n_cols, n_cols)
        x[32:64] = 0.0                      # an all-zero block (d = 0)
        x[64:96] *= 1.0e-30                 # a block of tiny values
        dx = torch.from_numpy(x).cuda()
        da = torch.from_numpy(ref.quantize_q8_0(x)).cuda()
        ws = [torch.from_numpy(synth.weights(t, 830 + i, n_rows, n_cols)).cuda() for i in range(2)]
        kern = hip.HipKernel(t)
        want = [torch.full((n_rows,), 2.0, dtype=torch.float32, device="cuda") for _ in range(2)]
        got = [torch.full((n_rows,), 2.0, dtype=torch.float32, device="cuda") for _ in range(2)]
        for acc in (False, True):
            for w, y in zip(ws, want):
                kern.matvec_q8_fused_dev(w, da, y, n_rows, n_cols, accumulate=acc)
            kern.gemv_dev(ws[0], dx, got[0], n_rows, n_cols, accumulate=acc)
            kern.gemv_dev(ws[1], dx, got[1], n_rows, n_cols, accumulate=acc)
            torch.cuda.synchronize()
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1]), (O.NAMES[t], n_rows, n_cols, acc)
        multi = [torch.zeros(n_rows, dtype=torch.float32, device="cuda") for _ in range(2)]
        single = [torch.zeros(n_rows, dtype=torch.float32, device="cuda") for _ in range(2)]
        kern.gemv_multi_dev(ws, dx, multi, n_rows, n_cols)
        for w, y in zip(ws, single):
            kern.matvec_q8_fused_dev(w, da, y, n_rows, n_cols, accumulate=False)
        torch.cuda.synchronize()
        assert torch.equal(multi[0], single[0]) and torch.equal(multi[1], single[1])


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_gemm_few_rows_share_one_weight_pass(hip, ref, tuning, t):
    """2..7 activation rows without the tile kernel: GEMV launches that take up to four rows per
    pass over the weights give the same bits as one fused matvec per row (short rows, rows split
    over four waves, and rows too long for the shared pass)."""
    import torch
    tuning("gemm_tile_min_rows", 1000)
    if True:
        for n, k_ in ((40, 768), (24, 4096), (12, 14336), (6, 32768)):
            w = synth.weights(t, 840 + n, n, k_)
            dw = torch.from_numpy(w).cuda()
            kern = hip.HipKernel(t)
            for m in (2, 3, 4, 5, 7):
                acts = ref.quantize_q8_0(synth.normal_f32(850 + m, m * k_))
                da = torch.from_numpy(acts).cuda()
                arb = k_ // 32 * 34
                want = torch.full((m, n), 1.5, dtype=torch.float32, device="cuda")
                got = torch.full((m, n), 1.5, dtype=torch.float32, device="cuda")
                for acc in (False, True):
                    for r in range(m):
                        kern.matvec_q8_fused_dev(dw, da[r * arb:(r + 1) * arb], want[r], n, k_, accumulate=acc)
                    kern.gemm_q8_dev(dw, da, got, m, n, k_, accumulate=acc)
                    torch.cuda.synchronize()
                    assert torch.equal(got, want), (O.NAMES[t], n, k_, m, acc)


def _ragged_cols(t):
    bs = O.BLOCK[t][0]
    return (20, 33, 1000, 4097, 8200 - 13) if bs == 32 else (200, 300, 1000, 4097, 14336 - 100, 17000)


def _ragged_ref(ref, t, w, a, n_rows, n_cols):
    """Rows that end inside a block: the reference skips the columns past n_cols
    (Q/reference/q4_k.rs:307-321, Q/simd/avx2/q4_0.rs:266-287, q8_0.rs:244-252, Q/reference/q6_k.rs:327).
    IQ4_XS has no working fused kernel in the reference; its integer form is defined by this library and takes whole
    blocks, so the columns past n_cols are given zero activation bytes, which is what skipping them means."""
    bs = O.BLOCK[t][0]
    if t != O.IQ4_XS:
        return ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=O.TIER_AVX2)
    full = -(-n_cols // bs) * bs
    am = a.copy().reshape(-1, 34)
    for b in range(am.shape[0]):
        keep = min(max(n_cols - 32 * b, 0), 32)
        am[b, 2 + keep:] = 0
    return ref.matvec_q8_fused(t, w, am.ravel(), n_rows, full, tier=O.TIER_AVX2)


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_rows_that_end_inside_a_block(hip, ref, t):
    """n_cols that is not a whole number of blocks (the reference's partial-block cases,
    Q/simd/avx2/q4_0.rs:557-580 with 20 columns, Q/simd/avx2/q4_k.rs:837-864 with 200): host slices,
    device pointers, several matrices per launch, fp32 activations quantized in the kernel, and gemm.
    The activation blocks past n_cols hold non-zero bytes, so a kernel that did not skip them fails."""
    import torch
    k = hip.HipKernel(t)
    bs = O.BLOCK[t][0]
    for i, n_cols in enumerate(_ragged_cols(t)):
        n_rows = (33, 64, 40, 35, 48, 37)[i]
        full = -(-n_cols // bs) * bs
        say(O.NAMES[t], "n_rows", n_rows, "n_cols", n_cols, "of", full)
        w = synth.weights(t, 1700 + i, n_rows, full)
        x = synth.normal_f32(1800 + i, full)
        a = ref.quantize_q8_0(x)
        y_ref = _ragged_ref(ref, t, w, a, n_rows, n_cols)
        out = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(w, a, out, n_rows, n_cols)
        assert_close(out, y_ref, f"{O.NAMES[t]} fused {n_rows}x{n_cols}")
        # the same as whole blocks with the activations past n_cols set to zero
        xz = x.copy()
        xz[n_cols:] = 0.0
        az = a.copy().reshape(-1, 34)
        for b in range(az.shape[0]):
            az[b, 2 + min(max(n_cols - 32 * b, 0), 32):] = 0
        outz = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(w, az.ravel(), outz, n_rows, full)
        assert_close(out, outz, "ragged against zeroed activations")
        # device pointers: accumulate, two matrices per launch
        dw = torch.from_numpy(w).cuda()
        dw2 = torch.from_numpy(synth.weights(t, 1750 + i, n_rows, full)).cuda()
        da = torch.from_numpy(a).cuda()
        y1 = torch.full((n_rows,), 3.0, dtype=torch.float32, device="cuda")
        k.matvec_q8_fused_dev(dw, da, y1, n_rows, n_cols, accumulate=True)
        torch.cuda.synchronize()
        assert np.array_equal(y1.cpu().numpy(), np.float32(3.0) + out)
        m1 = [torch.zeros(n_rows, dtype=torch.float32, device="cuda") for _ in range(2)]
        s2 = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
        k.matvec_q8_fused_multi_dev([dw, dw2], da, m1, n_rows, n_cols, accumulate=False)
        k.matvec_q8_fused_dev(dw2, da, s2, n_rows, n_cols, accumulate=False)
        torch.cuda.synchronize()
        assert np.array_equal(m1[0].cpu().numpy(), out) and torch.equal(m1[1], s2)
        # fp32 activations, exactly n_cols of them: quantize (zero-padded) + fused
        xq = ref.quantize_q8_0(xz)
        y_q = _ragged_ref(ref, t, w, xq, n_rows, n_cols)
        dx = torch.from_numpy(x[:n_cols].copy()).cuda()
        yg = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
        k.gemv_dev(dw, dx, yg, n_rows, n_cols)
        torch.cuda.synchronize()
        assert_close(yg.cpu().numpy(), y_q, "gemv_dev ragged")
        yh = np.full(n_rows, 7.0, dtype=np.float32)
        k.gemv(hip.QuantTensor(w, [n_rows, n_cols], t), x[:n_cols], yh)
        assert_close(yh, y_q, "gemv ragged")
        # gemm on host slices: rows of n_cols floats, few rows and more rows than the tile threshold
        for m in (3, 11):
            xs = synth.normal_f32(1900 + i + m, m * n_cols).reshape(m, n_cols)
            ym = np.zeros((m, n_rows), dtype=np.float32)
            k.gemm(hip.QuantTensor(w, [n_rows, n_cols], t), xs, ym, m, n_rows, n_cols)
            for r in range(m):
                xr = np.zeros(full, dtype=np.float32)
                xr[:n_cols] = xs[r]
                assert_close(ym[r], _ragged_ref(ref, t, w, ref.quantize_q8_0(xr), n_rows, n_cols), f"gemm ragged row {r}")
    # the debug dump of the group sums wants whole blocks
    with pytest.raises(hip.UnsupportedShape):
        k.block_sums(synth.weights(t, 1, 2, bs), ref.quantize_q8_0(synth.normal_f32(2, bs)), 2, bs - 3)


@pytest.mark.parametrize("t", [O.Q8_0, O.Q4_0], ids=lambda t: O.NAMES[t])
def test_weights_two_bytes_off_a_dword_boundary(hip, ref, t):
    """The 34- and 18-byte formats pick one of two load forms per block from the block's address; a matrix
    that starts two bytes off a dword boundary swaps the forms of all its blocks and must give the same bits."""
    import torch
    for n_rows, n_cols in ((40, 4096), (33, 8192), (16, 14336)):
        w = synth.weights(t, 91, n_rows, n_cols)
        da = torch.from_numpy(ref.quantize_q8_0(synth.normal_f32(92, n_cols))).cuda()
        aligned = torch.from_numpy(w).cuda()
        buf = torch.zeros(w.size + 8, dtype=torch.uint8, device="cuda")
        buf[2:2 + w.size] = aligned
        y0 = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
        y2 = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
        k = hip.HipKernel(t)
        k.matvec_q8_fused_dev(aligned, da, y0, n_rows, n_cols, accumulate=False)
        k.matvec_q8_fused_dev(buf[2:], da, y2, n_rows, n_cols, accumulate=False)
        torch.cuda.synchronize()
        assert torch.equal(y0, y2), (O.NAMES[t], n_rows, n_cols)


def test_q6_k_weights_off_a_dword_boundary_are_refused(hip, ref):
    """The Q6_K kernel reads from the dword-aligned address at or below a block, so the matrix has to start
    on one (device allocations and GGUF tensor data do); two bytes off, the call fails and launches nothing."""
    import torch
    n_rows, n_cols = 8, 512
    w = synth.weights(O.Q6_K, 77, n_rows, n_cols)
    buf = torch.zeros(w.size + 4, dtype=torch.uint8, device="cuda")
    buf[2:2 + w.size] = torch.from_numpy(w).cuda()
    da = torch.from_numpy(ref.quantize_q8_0(synth.normal_f32(78, n_cols))).cuda()
    y = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
    with pytest.raises(hip.KernelError):
        hip.HipKernel(O.Q6_K).matvec_q8_fused_dev(buf[2:], da, y, n_rows, n_cols)
    # four bytes off is fine
    buf2 = torch.zeros(w.size + 4, dtype=torch.uint8, device="cuda")
    buf2[4:] = torch.from_numpy(w).cuda()
    hip.HipKernel(O.Q6_K).matvec_q8_fused_dev(buf2[4:], da, y, n_rows, n_cols, accumulate=False)
    torch.cuda.synchronize()
    want = np.zeros(n_rows, dtype=np.float32)
    hip.HipKernel(O.Q6_K).matvec_q8_fused(w, da.cpu().numpy(), want, n_rows, n_cols)
    assert np.array_equal(y.cpu().numpy(), want)


def test_empty_inputs(hip):
    for t in O.ALL_TYPES:
        k = hip.HipKernel(t)
        out = np.full(2, 3.0, dtype=np.float32)
        k.matvec_q8_fused(np.zeros(0, dtype=np.uint8), np.zeros(0, dtype=np.uint8), out, 0, 0)
        assert (out == 3.0).all()


# ---- (5) the benchmark configurations at full size ---------------------------------------------

CONFIGS = [
    ("C1 Q4_0 4096x4096", O.Q4_0, 4096, 4096),
    ("C2 q_proj Q8_0 4096x4096", O.Q8_0, 4096, 4096),
    ("C2 ffn_gate Q4_K 14336x4096", O.Q4_K, 14336, 4096),
    ("C2 ffn_down Q6_K 4096x14336", O.Q6_K, 4096, 14336),
    ("C5 expert gate IQ4_XS 14336x4096", O.IQ4_XS, 14336, 4096),
    ("C5 expert down IQ4_XS 4096x14336", O.IQ4_XS, 4096, 14336),
]


@pytest.mark.parametrize("cfg", CONFIGS, ids=lambda c: c[0])
def test_full_size_configs(hip, ref, cfg):
    import torch
    name, t, n_rows, n_cols = cfg
    say(name)
    w = synth.weights(t, 11, n_rows, n_cols)
    x = synth.normal_f32(12, n_cols)
    a_ref = ref.quantize_q8_0(x)
    dw = torch.from_numpy(w).cuda()
    dx = torch.from_numpy(x).cuda()
    da = torch.empty(a_ref.size, dtype=torch.uint8, device="cuda")
    hip.quantize_q8_0_dev(dx, da)
    assert np.array_equal(da.cpu().numpy(), a_ref)                      # activation bytes bit-exact
    k = hip.HipKernel(t)
    dy = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
    k.matvec_q8_fused_dev(dw, da, dy, n_rows, n_cols, accumulate=True)
    sums = torch.empty((n_rows, O.groups_per_row(t, n_cols)), dtype=torch.int32, device="cuda")
    k.block_sums_dev(dw, da, sums, n_rows, n_cols)
    torch.cuda.synchronize()
    y_ref = canonical_ref(ref, t, w, a_ref, n_rows, n_cols)
    assert_close(dy.cpu().numpy(), y_ref, name)
    assert np.array_equal(sums.cpu().numpy(), ref.block_sums(t, w, a_ref, n_rows, n_cols))
    # linearity in the accumulator: a second call adds the same vector again
    k.matvec_q8_fused_dev(dw, da, dy, n_rows, n_cols, accumulate=True)
    torch.cuda.synchronize()
    assert_close(dy.cpu().numpy(), 2 * y_ref, name + " (accumulated twice)")


def test_lm_head_full_size(hip, ref):
    """C3: 128256 x 4096 Q6_K, the largest matrix.  Oracle on every row (threaded row split)."""
    import torch
    n_rows, n_cols, t = 128256, 4096, O.Q6_K
    say("C3 lm_head: generating")
    w = synth.weights(t, 21, n_rows, n_cols)
    a = ref.quantize_q8_0(synth.normal_f32(22, n_cols))
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(a).cuda()
    dy = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
    hip.HipKernel(t).matvec_q8_fused_dev(dw, da, dy, n_rows, n_cols, accumulate=False)
    torch.cuda.synchronize()
    say("C3 lm_head: oracle")
    y_ref = canonical_ref(ref, t, w, a, n_rows, n_cols, threads=16)
    assert_close(dy.cpu().numpy(), y_ref, "lm_head")
    # row-permutation equivariance on the device copy: rows are independent
    perm = torch.randperm(n_rows, generator=torch.Generator().manual_seed(5))
    rb = O.row_bytes(t, n_cols)
    dwp = dw.view(n_rows, rb)[perm.cuda()].contiguous()
    dyp = torch.zeros_like(dy)
    hip.HipKernel(t).matvec_q8_fused_dev(dwp, da, dyp, n_rows, n_cols, accumulate=False)
    torch.cuda.synchronize()
    assert torch.equal(dyp, dy[perm.cuda()])


# ---- (6) gemv / gemm on host slices ---------------------------------------------------------

@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_gemv_is_quantize_plus_fused(hip, ref, t):
    n_rows, n_cols = 33, 1024
    w = synth.weights(t, 301, n_rows, n_cols)
    x = synth.normal_f32(302, n_cols)
    k = hip.HipKernel(t)
    y = np.full(n_rows, 9.0, dtype=np.float32)  # overwritten, not accumulated (Q/traits.rs:39)
    k.gemv(hip.QuantTensor(w, [n_rows, n_cols], t), x, y)
    y_ref = canonical_ref(ref, t, w, ref.quantize_q8_0(x), n_rows, n_cols)
    assert_close(y, y_ref, "gemv")
    # and close to the reference's f32-activation gemv up to the Q8_0 rounding of x
    y_f32 = ref.gemv(t, w, n_rows, n_cols, x)
    assert np.abs(y - y_f32).max() < 0.02 * np.abs(y_f32).max()


def test_gemv_known_answers(hip):
    # Q/reference/q4_k.rs:411-436 (256) and Q/reference/q8_0.rs:175-190 (6.0): exact even after Q8_0
    w = np.frombuffer(O.make_q4_k_block(1.0, 0.0, FX.Q4K_SCALES_ONES, [0x11] * 128), dtype=np.uint8)
    y = np.zeros(1, dtype=np.float32)
    hip.HipKernel(O.Q4_K).gemv(hip.QuantTensor(w, [1, 256], O.Q4_K), np.ones(256, dtype=np.float32), y)
    assert abs(y[0] - 256.0) < 1.0
    q = [0] * 32
    q[0] = 1
    x = np.zeros(32, dtype=np.float32)
    x[0] = 3.0
    w = np.frombuffer(O.make_q8_0_block(2.0, q), dtype=np.uint8)
    hip.HipKernel(O.Q8_0).gemv(hip.QuantTensor(w, [1, 32], O.Q8_0), x, y)
    assert abs(y[0] - 6.0) < 0.1
    # partial blocks, Q/simd/avx2/q4_k.rs:837-864 (200 of 256 columns, all weights 1 -> 200) and
    # Q/simd/avx2/q4_0.rs:557-580 (20 of 32 columns, all weights 0 -> 0), at the reference's tolerances
    # (plus the Q8_0 rounding of the all-ones input, 127 * f16(1/127) = 0.99994)
    w = np.frombuffer(O.make_q4_k_block(1.0, 0.0, FX.Q4K_SCALES_ONES, [0x11] * 128), dtype=np.uint8)
    hip.HipKernel(O.Q4_K).gemv(hip.QuantTensor(w, [1, 200], O.Q4_K), np.ones(200, dtype=np.float32), y)
    assert abs(y[0] - 200.0) < 0.1
    w = np.frombuffer(O.make_q4_0_block(1.0, [0x88] * 16), dtype=np.uint8)
    y[0] = 5.0
    hip.HipKernel(O.Q4_0).gemv(hip.QuantTensor(w, [1, 20], O.Q4_0), np.ones(20, dtype=np.float32), y)
    assert abs(y[0]) < 1e-4


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_gemm_matches_oracle(hip, ref, t):
    m, n, k_ = 5, 40, 768
    w = synth.weights(t, 401, n, k_)
    x = synth.normal_f32(402, m * k_).reshape(m, k_)
    y = np.zeros((m, n), dtype=np.float32)
    hip.HipKernel(t).gemm(hip.QuantTensor(w, [n, k_], t), x, y, m, n, k_)
    assert_close(y, ref.gemm_q8(t, w, x, m, n, k_), "gemm")


def _tile_zero_point(t, acts, rows, k_):
    """The tile kernel multiplies Q4_0's unsigned nibbles and applies the "- 8" of (q - 8) in fp32
    through the zero-point term, so its integer sums are sum q*a = sum (q-8)*a + 8 * sum a."""
    if t != O.Q4_0:
        return 0
    a = acts.reshape(rows, k_ // 32, 34)[:, :, 2:].view(np.int8).astype(np.int32).sum(axis=2)
    return (8 * a)[:, None, :]


def _oracle_prefill(ref, t, w, acts, m, n, k_, rows=None):
    """m fused matvecs (threaded row split) on already-quantized activation rows."""
    arb = k_ // 32 * 34
    rows = range(m) if rows is None else rows
    return np.stack([canonical_ref(ref, t, w, acts[r * arb:(r + 1) * arb], n, k_, threads=16) for r in rows])


@pytest.mark.parametrize("shape", [(8, 32, 256), (33, 100, 1024), (128, 160, 512), (200, 257, 1024), (64, 64, 4096),
                                   (130, 129, 2048)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_prefill_tile_kernel(hip, ref, tuning, shape, t):
    """Weights of every format x Q8_0 activations on the int8-MFMA tile kernel: integer sub-block sums bit-exact, fp32 within
    1e-5, ragged tile edges in both directions, overwrite and accumulate."""
    import torch
    from oxillama_amd import capi
    m, n, k_ = shape
    say("prefill", O.NAMES[t], shape)
    tuning("gemm_tile_min_rows", 1)  # small shapes would otherwise take the GEMV route
    _prefill_tile_case(hip, ref, shape, t)


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_prefill_many_tokens_takes_the_wide_tile_shape(hip, ref, t):
    """More than 384 tokens on a matrix whose 128 x 128 work-group tiles give every compute unit one and a half: the tile
    kernel with four token tiles against one weight-row tile per wave (every format but Q4_K).  The library's own choice, no knob; sampled tokens against the oracle on all outputs, ragged n."""
    import torch
    from test_gpu_prefill_f16 import last_launch
    cus = hip.device_info()["compute_units"]
    m, k_ = 400, 256
    n = 128 * ((3 * cus + 7) // 8) - 5
    say("prefill, wide tiles", O.NAMES[t], (m, n, k_))
    w = synth.weights(t, 650, n, k_)
    acts = ref.quantize_q8_0(synth.normal_f32(651, m * k_))
    kern = hip.HipKernel(t)
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device="cuda")
    dy = torch.full((m + 1, n), 7.0, dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(dw, da, dy, m, n, k_, accumulate=False, workspace=ws)
    torch.cuda.synchronize()
    took = last_launch()
    if t == O.Q4_K:  # its f16 kernel where that fills the chip, else the tile kernel's 64 x 64 waves
        assert "gemm_prefill_q4k" in took or took.startswith("gemm_tile_kernel<Q4_K,2,2,2,2>"), took
    else:
        assert took.startswith("gemm_tile_kernel") and ",4,1,1,1>" in took, took
    rows = sorted(set(list(range(0, m, 37)) + [127, 128, 383, 384, m - 1]))
    y = dy.cpu().numpy()
    assert np.all(y[m] == 7.0)
    assert_close(y[rows], _oracle_prefill(ref, t, w, acts, m, n, k_, rows=rows), f"wide tiles {O.NAMES[t]}")
    # the debug dump's launch (another tile shape) gives the same bits and the oracle's integer sums
    if t != O.Q4_K:
        dsum = torch.empty((m, n, k_ // (16 if t in (O.Q6_K, O.Q2_K, O.Q3_K) else 32)), dtype=torch.int32, device="cuda")
        dy2 = torch.empty((m, n), dtype=torch.float32, device="cuda")
        kern.gemm_block_sums_dev(dw, da, dy2, dsum, m, n, k_, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(dy2, dy[:m])


@pytest.mark.parametrize("shape", [(40, 40, 28672), (100, 72, 17408), (400, 40, 28672), (70, 33, 36864), (400, 36, 36864),
                                   (9, 48, 65536)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_prefill_tile_kernel_long_rows(hip, ref, tuning, shape, t):
    """Rows of more than 16384 columns (the down projections of the large models: 17408, 28672, ...): the token scales of
    a 128-token tile for the whole row no longer fit LDS, and the library takes 64-token tiles (up to 32768 columns) or
    32-token tiles (up to 65536) instead of falling back to one GEMV launch per four rows.  Same checks as above."""
    from test_gpu_prefill_f16 import last_launch
    say("prefill, long rows", O.NAMES[t], shape)
    tuning("gemm_tile_min_rows", 1)
    _prefill_tile_case(hip, ref, shape, t)
    assert last_launch().startswith("gemm_tile_kernel"), last_launch()  # (the last call there is the sums' dump)


BLOCKS32 = [t for t in O.ALL_TYPES if O.BLOCK[t][0] == 32]


@pytest.mark.parametrize("shape", [(8, 32, 288), (33, 100, 416), (130, 129, 352), (40, 64, 1408), (200, 130, 480),
                                   (450, 140, 288)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("t", BLOCKS32, ids=lambda t: O.NAMES[t])
def test_prefill_tile_kernel_rows_of_whole_32_blocks(hip, ref, tuning, shape, t):
    """Rows that are whole 32-weight blocks but not whole 256-weight steps (the formats of independent blocks):
    the last step reads the row's last eight blocks and counts only those the step before has not covered.
    Integer sums bit-exact, fp32 within 1e-5, every tile shape's row count."""
    say("prefill, ragged k", O.NAMES[t], shape)
    tuning("gemm_tile_min_rows", 1)
    _prefill_tile_case(hip, ref, shape, t)


def _prefill_tile_case(hip, ref, shape, t):
    import torch
    m, n, k_ = shape
    w = synth.weights(t, 600 + m, n, k_)
    x = synth.normal_f32(700 + n, m * k_)
    acts = ref.quantize_q8_0(x)
    kern = hip.HipKernel(t)
    ws_bytes = kern.gemm_workspace_bytes(m, n, k_)
    assert ws_bytes > 0
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    dy = torch.full((m, n), 7.0, dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(dw, da, dy, m, n, k_, accumulate=False, workspace=ws)
    torch.cuda.synchronize()
    y_ref = _oracle_prefill(ref, t, w, acts, m, n, k_)
    assert_close(dy.cpu().numpy(), y_ref, f"prefill {shape}")
    # accumulate adds the same values to what is there; library-owned scratch gives the same bits
    dy2 = dy.clone()
    kern.gemm_q8_dev(dw, da, dy2, m, n, k_, accumulate=True, workspace=None)
    torch.cuda.synchronize()
    assert torch.equal(dy2, dy + dy)
    # exact integer sums of every (token, weight row, sub-block)
    dsum = torch.empty((m, n, k_ // (16 if t == O.Q6_K else 32)), dtype=torch.int32, device="cuda")
    dy3 = torch.empty_like(dy)
    kern.gemm_block_sums_dev(dw, da, dy3, dsum, m, n, k_, workspace=ws)
    torch.cuda.synchronize()
    arb = k_ // 32 * 34
    want = np.stack([ref.block_sums(t, w, acts[r * arb:(r + 1) * arb], n, k_) for r in range(m)])
    assert np.array_equal(dsum.cpu().numpy() - _tile_zero_point(t, acts, m, k_), want)
    assert torch.equal(dy3, dy)


def test_prefill_full_size_c4(hip, ref):
    """C4: 512 tokens x Q4_K 14336 x 4096.  Oracle on every token and every output, and bit-exact integer sums (the tile
    kernel's, and the prefill kernel's scaled ones) on two 512-row slabs of W."""
    import torch
    m, n, k_, t = 512, 14336, 4096, O.Q4_K
    w = synth.weights(t, 31, n, k_)
    x = synth.normal_f32(32, m * k_)
    kern = hip.HipKernel(t)
    dw, dx = torch.from_numpy(w).cuda(), torch.from_numpy(x).cuda()
    da = torch.empty(m * (k_ // 32 * 34), dtype=torch.uint8, device="cuda")
    hip.quantize_q8_0_dev(dx, da)
    acts = ref.quantize_q8_0(x)
    assert np.array_equal(da.cpu().numpy(), acts)  # row-wise Q8_0 bytes bit-exact
    ws = torch.empty(kern.gemm_workspace_bytes(m, n, k_), dtype=torch.uint8, device="cuda")
    dy = torch.zeros((m, n), dtype=torch.float32, device="cuda")
    kern.gemm_q8_dev(dw, da, dy, m, n, k_, accumulate=False, workspace=ws)
    torch.cuda.synchronize()
    from test_gpu_prefill_f16 import last_launch, q4k_sub_block_scales
    assert "gemm_prefill_q4k" in last_launch(), last_launch()  # C4 is the shape the f16 prefill kernel is for
    rows = list(range(m))  # every token, every output: 512 oracle matvecs of 14336 x 4096 on the host's threads
    y_ref = _oracle_prefill(ref, t, w, acts, m, n, k_, rows=rows)
    assert_close(dy.cpu().numpy()[rows], y_ref, "C4 prefill")
    # two 512-row slabs of W (one that straddles tile boundaries in the middle, and the last rows): the oracle
    # on ALL 512 tokens, and the exact integer sums of every (token, weight row, 32-weight group) of the slab
    arb, rb = k_ // 32 * 34, O.row_bytes(t, k_)
    for r0 in (4000, n - 512):
        w_slab = w[r0 * rb:(r0 + 512) * rb]
        y_slab = _oracle_prefill(ref, t, w_slab, acts, m, 512, k_)
        assert_close(dy[:, r0:r0 + 512].cpu().numpy(), y_slab, f"C4 prefill, rows {r0}..{r0 + 511}, all tokens")
        dw_slab = dw[r0 * rb:(r0 + 512) * rb]
        dsum = torch.empty((m, 512, k_ // 32), dtype=torch.int32, device="cuda")
        dy_slab = torch.empty((m, 512), dtype=torch.float32, device="cuda")
        ws_slab = torch.empty(kern.gemm_workspace_bytes(m, 512, k_), dtype=torch.uint8, device="cuda")
        kern.gemm_block_sums_dev(dw_slab, da, dy_slab, dsum, m, 512, k_, workspace=ws_slab)
        torch.cuda.synchronize()
        got = dsum.cpu().numpy()
        for r in range(m):
            assert np.array_equal(got[r], ref.block_sums(t, w_slab, acts[r * arb:(r + 1) * arb], 512, k_)), (r0, r)
        # the slab on its own (the int8 tile kernel at this size) meets the same bar
        assert_close(dy_slab.cpu().numpy(), y_slab, f"C4 slab launch, rows {r0}")
        # and the prefill kernel's own matrix-core results on the slab: sub-block scale x integer sum, exactly
        kern.gemm_scaled_sums_dev(dw_slab, da, dy_slab, dsum, m, 512, k_, ws)
        torch.cuda.synchronize()
        got = dsum.cpu().numpy()
        sc = q4k_sub_block_scales(w_slab, 512, k_)
        for r in range(0, m, 7):
            assert np.array_equal(got[r], sc * ref.block_sums(t, w_slab, acts[r * arb:(r + 1) * arb], 512, k_)), (r0, r)
        assert_close(dy_slab.cpu().numpy(), y_slab, f"C4 slab on the prefill kernel, rows {r0}")
        del dsum, got
    # every token row also equals the batch-1 fused matvec of the same activations, to fp32 order
    yv = torch.zeros(n, dtype=torch.float32, device="cuda")
    for r in (1, 255, 510):
        yv.zero_()
        kern.matvec_q8_fused_dev(dw, da[r * arb:(r + 1) * arb], yv, n, k_, accumulate=False)
        torch.cuda.synchronize()
        assert_close(dy[r].cpu().numpy(), yv.cpu().numpy(), f"row {r} vs matvec")


# ---- (7) residency helpers -----------------------------------------------------------------

def _moe_case(ref, t, n_experts, n_tok, top_k, n, k_, seed):
    """Seeded uniform router logits -> top-k routing -> pairs grouped by expert."""
    from oxillama_amd import moe
    rng = np.random.default_rng(seed)
    logits = rng.random((n_tok, n_experts), dtype=np.float32)
    experts, weights = moe.route_top_k(logits, top_k)
    offsets, tok, slot = moe.group_by_expert(experts, n_experts)
    x = synth.normal_f32(seed + 1, n_tok * k_).reshape(n_tok, k_)
    acts_tok = ref.quantize_q8_0(x.reshape(-1)).reshape(n_tok, k_ // 32 * 34)
    acts = np.ascontiguousarray(acts_tok[tok])  # one activation row per (token, expert) pair
    w = np.stack([synth.weights(t, seed + 10 + e, n, k_) for e in range(n_experts)])
    return offsets, tok, slot, weights, acts, w


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
@pytest.mark.parametrize("cfg", [(8, 64, 2, 96, 1024), (4, 7, 2, 300, 512), (8, 200, 2, 64, 256), (3, 5, 1, 33, 2048)],
                         ids=lambda c: "e%d_t%d_k%d_n%d_k%d" % c)
def test_moe_grouped_matmul(hip, ref, t, cfg):
    """Grouped expert matmul: every (token, expert) pair equals the fused matvec of that expert's
    weights with the token's Q8_0 row (fp32 within 1e-5, integer sums bit-exact); rows of experts
    with no tokens and tile padding are never written."""
    import torch
    n_experts, n_tok, top_k, n, k_ = cfg
    say("moe", O.NAMES[t], cfg)
    offsets, tok, slot, weights, acts, w = _moe_case(ref, t, n_experts, n_tok, top_k, n, k_, 900 + n_tok)
    rows = int(offsets[-1])
    assert rows == n_tok * top_k
    kern = hip.HipKernel(t)
    ws = torch.empty(kern.moe_gemm_workspace_bytes(rows, n, k_), dtype=torch.uint8, device="cuda")
    dw, da = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda()
    doff = torch.from_numpy(offsets).cuda()
    dy = torch.full((rows + 3, n), 7.0, dtype=torch.float32, device="cuda")  # 3 guard rows
    groups = k_ // (16 if t == O.Q6_K else 32)
    dsum = torch.full((rows, n, groups), -1, dtype=torch.int32, device="cuda")
    max_rows = int(np.diff(offsets).max())
    kern.moe_gemm_q8_dev(dw, w[0].nbytes, n_experts, da, doff, rows, max_rows, dy, n, k_, ws, d_sums=dsum)
    torch.cuda.synchronize()
    y = dy.cpu().numpy()
    assert np.all(y[rows:] == 7.0)
    y_ref = np.empty((rows, n), dtype=np.float32)
    s_ref = np.empty((rows, n, groups), dtype=np.int32)
    for e in range(n_experts):
        for r in range(offsets[e], offsets[e + 1]):
            y_ref[r] = canonical_ref(ref, t, w[e], acts[r], n, k_)
            s_ref[r] = ref.block_sums(t, w[e], acts[r], n, k_)
    assert_close(y[:rows], y_ref, f"moe {cfg}")
    assert np.array_equal(dsum.cpu().numpy() - _tile_zero_point(t, acts.reshape(-1), rows, k_), s_ref)
    # production launch (no sums): the same bits as the dump launch -- except for a handful of rows in all, which one
    # GEMV launch serves (a matvec per row; the dump is the matmul kernels'): the same values within the bar.
    # Overwrite then accumulate: twice the production launch's bits.
    dy1 = torch.zeros((rows, n), dtype=torch.float32, device="cuda")
    kern.moe_gemm_q8_dev(dw, w[0].nbytes, n_experts, da, doff, rows, max_rows, dy1, n, k_, ws)
    torch.cuda.synchronize()
    if rows > 8:
        assert torch.equal(dy1, dy[:rows])
    else:
        assert_close(dy1.cpu().numpy(), y_ref, f"moe {cfg} production launch")
    dy2 = dy1.clone()
    kern.moe_gemm_q8_dev(dw, w[0].nbytes, n_experts, da, doff, rows, max_rows, dy2, n, k_, ws, accumulate=True)
    torch.cuda.synchronize()
    assert torch.equal(dy2, dy1 + dy1)
    # max_rows = 0 (unknown) sizes the launch for the worst case: another tile shape and fp32
    # summation order, the same values within the bar
    dy3 = torch.zeros((rows, n), dtype=torch.float32, device="cuda")
    kern.moe_gemm_q8_dev(dw, w[0].nbytes, n_experts, da, doff, rows, 0, dy3, n, k_, ws)
    torch.cuda.synchronize()
    assert_close(dy3.cpu().numpy(), y_ref, f"moe {cfg} max_rows=0")


def test_moe_full_size_c5_one_projection(hip, ref):
    """C5 shapes: 8 experts of IQ4_XS 14336 x 4096 (gate) and 4096 x 14336 (down), 64 tokens top-2.
    Oracle on every pair row, every output."""
    import torch
    t, n_experts, n_tok, top_k = O.IQ4_XS, 8, 64, 2
    kern = hip.HipKernel(t)
    for n, k_ in ((14336, 4096), (4096, 14336)):
        offsets, tok, slot, weights, acts, w = _moe_case(ref, t, n_experts, n_tok, top_k, n, k_, 5000 + n)
        rows = int(offsets[-1])
        ws = torch.empty(kern.moe_gemm_workspace_bytes(rows, n, k_), dtype=torch.uint8, device="cuda")
        dw, da, doff = torch.from_numpy(w).cuda(), torch.from_numpy(acts).cuda(), torch.from_numpy(offsets).cuda()
        dy = torch.zeros((rows, n), dtype=torch.float32, device="cuda")
        kern.moe_gemm_q8_dev(dw, w[0].nbytes, n_experts, da, doff, rows, int(np.diff(offsets).max()), dy, n, k_, ws)
        torch.cuda.synchronize()
        y = dy.cpu().numpy()
        for r in range(rows):
            e = int(np.searchsorted(offsets, r, side="right") - 1)
            y_ref = canonical_ref(ref, t, w[e], acts[r], n, k_, threads=16)
            assert_close(y[r], y_ref, f"c5 {n}x{k_} pair row {r} expert {e}")
        del dw, da, dy, ws




def test_registered_weights_and_cache(hip, ref):
    import ctypes as C
    from oxillama_amd import capi
    lib = capi.load()
    t, n_rows, n_cols = O.Q4_K, 64, 1024
    w = synth.weights(t, 501, n_rows, n_cols)
    a = ref.quantize_q8_0(synth.normal_f32(502, n_cols))
    h = C.c_void_p()
    assert lib.oxq_weights_register(t, n_rows, n_cols, w.ctypes.data, w.size, C.byref(h)) == capi.OK
    assert lib.oxq_weights_nbytes(h) == w.size
    import torch
    da = torch.from_numpy(a).cuda()
    dy = torch.zeros(n_rows, dtype=torch.float32, device="cuda")
    st = lib.oxq_matvec_q8_fused_dev(t, lib.oxq_weights_device_ptr(h), da.data_ptr(), dy.data_ptr(), n_rows, n_cols,
                                     0, None)
    assert st == capi.OK
    torch.cuda.synchronize()
    y_ref = canonical_ref(ref, t, w, a, n_rows, n_cols)
    assert_close(dy.cpu().numpy(), y_ref, "registered")
    assert lib.oxq_weights_release(h) == capi.OK
    # host-slice route with the cache on: same answer, and a changed buffer is noticed
    import ctypes as C

    def stats():
        e, b, h, u = C.c_size_t(), C.c_size_t(), C.c_uint64(), C.c_uint64()
        assert lib.oxq_weight_cache_stats(C.byref(e), C.byref(b), C.byref(h), C.byref(u)) == capi.OK
        return e.value, b.value, h.value, u.value

    lib.oxq_weight_cache_enable(1)
    try:
        k = hip.HipKernel(t)
        _, _, hits0, ups0 = stats()
        for _ in range(2):
            out = np.zeros(n_rows, dtype=np.float32)
            k.matvec_q8_fused(w, a, out, n_rows, n_cols)
            assert_close(out, y_ref, "cached")
        assert stats() == (1, w.nbytes, hits0 + 1, ups0 + 1)
        w2 = synth.weights(t, 503, n_rows, n_cols)
        w[:] = w2
        out = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(w, a, out, n_rows, n_cols)
        assert_close(out, canonical_ref(ref, t, w2, a, n_rows, n_cols), "cache refreshed")
        # the contract of mode 1: a caller that changes bytes in place says so
        w[5] ^= 0xFF
        assert lib.oxq_weight_cache_invalidate(w.ctypes.data) == capi.OK
        assert stats()[0] == 0
        out = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(w, a, out, n_rows, n_cols)
        assert_close(out, canonical_ref(ref, t, w, a, n_rows, n_cols), "invalidated")
        # mode 2 hashes every byte: a change between the sampled pieces is seen without being told
        lib.oxq_weight_cache_enable(2)
        big_rows = 256
        wb = synth.weights(t, 504, big_rows, n_cols)  # larger than the 4096 sampled bytes
        assert wb.nbytes > 64 * 64 * 2
        for flip in (None, 64 + 3, wb.nbytes // 2 + 1):
            if flip is not None:
                wb[flip] ^= 0x10
            before = stats()[3]
            out = np.zeros(big_rows, dtype=np.float32)
            k.matvec_q8_fused(wb, a, out, big_rows, n_cols)
            assert stats()[3] == before + 1, "a changed byte must cause a new upload"
            assert_close(out, canonical_ref(ref, t, wb, a, big_rows, n_cols), f"verified cache, flip {flip}")
        # byte cap: the least recently used copy goes first
        lib.oxq_weight_cache_enable(1)
        lib.oxq_weight_cache_clear()
        bufs = [synth.weights(t, 510 + i, n_rows, n_cols) for i in range(3)]
        lib.oxq_weight_cache_set_limit(2 * bufs[0].nbytes)
        for wi in bufs:
            k.matvec_q8_fused(wi, a, np.zeros(n_rows, dtype=np.float32), n_rows, n_cols)
        assert stats()[:2] == (2, 2 * bufs[0].nbytes)
        hits = stats()[2]
        k.matvec_q8_fused(bufs[2], a, np.zeros(n_rows, dtype=np.float32), n_rows, n_cols)
        k.matvec_q8_fused(bufs[1], a, np.zeros(n_rows, dtype=np.float32), n_rows, n_cols)
        assert stats()[2] == hits + 2
        ups = stats()[3]
        out = np.zeros(n_rows, dtype=np.float32)
        k.matvec_q8_fused(bufs[0], a, out, n_rows, n_cols)  # evicted earlier: uploaded again
        assert stats()[3] == ups + 1
        assert_close(out, canonical_ref(ref, t, bufs[0], a, n_rows, n_cols), "after eviction")
    finally:
        lib.oxq_weight_cache_enable(0)
        lib.oxq_weight_cache_clear()
        lib.oxq_weight_cache_set_limit(16 << 30)


# ---- concurrency and lifecycle ------------------------------------------------------------------

def test_concurrent_host_calls_from_threads(hip, ref):
    """The header promises thread safety: host-slice calls from several threads serialise on the library's
    lock (they share its staging buffers) and each gets its own result."""
    import threading
    jobs = []
    for i, t in enumerate((O.Q4_K, O.Q6_K, O.Q8_0, O.Q4_0, O.IQ4_XS, O.Q4_K)):
        n_rows, n_cols = 64 + 32 * i, 1024
        w = synth.weights(t, 700 + i, n_rows, n_cols)
        x = synth.normal_f32(800 + i, n_cols)
        jobs.append((t, w, x, n_rows, n_cols, ref.matvec_q8_fused(t, w, ref.quantize_q8_0(x), n_rows, n_cols)))
    errors = []

    def work(job):
        t, w, x, n_rows, n_cols, want = job
        try:
            k = hip.HipKernel(t)
            for _ in range(20):
                y = np.zeros(n_rows, dtype=np.float32)
                k.gemv(hip.QuantTensor(w, [n_rows, n_cols], t), x, y)
                if np.abs(y - want).max() > FP32_REL_TOL * np.abs(want).max():
                    errors.append((O.NAMES[t], float(np.abs(y - want).max())))
                    return
        except Exception as e:  # noqa: BLE001 - report any failure of a worker
            errors.append((O.NAMES[t], repr(e)))

    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_shutdown_and_reinitialise(hip, ref):
    lib = hip.capi.load()
    w = synth.weights(O.Q4_K, 1, 32, 512)
    x = synth.normal_f32(2, 512)
    want = ref.matvec_q8_fused(O.Q4_K, w, ref.quantize_q8_0(x), 32, 512)
    k = hip.HipKernel(O.Q4_K)
    y = np.zeros(32, dtype=np.float32)
    k.gemv(hip.QuantTensor(w, [32, 512], O.Q4_K), x, y)
    assert lib.oxq_shutdown() == 0 and lib.oxq_shutdown() == 0  # idempotent; scratch and caches are released
    y2 = np.zeros(32, dtype=np.float32)
    k.gemv(hip.QuantTensor(w, [32, 512], O.Q4_K), x, y2)  # the next call initialises the device again
    assert np.array_equal(y, y2) and np.abs(y - want).max() <= FP32_REL_TOL * np.abs(want).max()
    hip.init(0)
