"""Pins the CPU oracle (oracle/oxq_oracle.c) without running the reference:
hardware F16C, the reference's own unit-test vectors (tests/fixtures.py),
closed-form cases and brute force.  CPU only."""
import ctypes as C
import os

import numpy as np
import pytest

import fixtures as FX
import oracle as O


def _has_f16c():
    try:
        with open("/proc/cpuinfo") as f:
            return " f16c" in f.read()
    except OSError:
        return False


@pytest.fixture(scope="module")
def f16c():
    if not _has_f16c():
        pytest.skip("host CPU has no F16C")
    O.load()
    if not os.path.exists(O.F16C_PATH):
        O.build()
    lib = C.CDLL(O.F16C_PATH)
    lib.oxq_f16c_to_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    lib.oxq_f16c_from_f32.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
    return lib


# ---- half floats -------------------------------------------------------------

def test_f16_to_f32_all_values_match_hardware(ref, f16c):
    h = np.arange(65536, dtype=np.uint16)
    hw = np.zeros(65536, dtype=np.float32)
    f16c.oxq_f16c_to_f32(h.ctypes.data, hw.ctypes.data, h.size)
    sw = np.array([ref.f16_to_f32(int(v)) for v in h], dtype=np.float32)
    same = (hw.view(np.uint32) == sw.view(np.uint32)) | (np.isnan(hw) & np.isnan(sw))
    assert same.all()
    # and numpy's own binary16 agrees (third opinion)
    assert np.array_equal(h.view(np.float16).astype(np.float32)[~np.isnan(hw)], sw[~np.isnan(hw)])


def test_f32_to_f16_matches_hardware(ref, f16c):
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2**32, size=200_000, dtype=np.uint64).astype(np.uint32)
    # dense coverage of the half range incl. subnormals, ties and overflow
    grid = np.concatenate([
        np.linspace(-70000, 70000, 50_001, dtype=np.float32),
        (np.arange(0, 4096, dtype=np.float32) * np.float32(2.0**-26)),      # subnormal halves and ties
        np.float32(2.0**-14) + np.arange(0, 4096, dtype=np.float32) * np.float32(2.0**-27),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e-8, 2.98e-8, 2.9802322e-8, 5.96e-8,
                  np.inf, -np.inf, 0.1, 0.01, 1.0 / 3.0], dtype=np.float32),
    ])
    x = np.concatenate([bits.view(np.float32), grid])
    hw = np.zeros(x.size, dtype=np.uint16)
    f16c.oxq_f16c_from_f32(x.ctypes.data, hw.ctypes.data, x.size)
    sw = np.array([ref.f32_to_f16(v) for v in x], dtype=np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(hw[~nan], sw[~nan])
    assert ((sw[nan] & 0x7C00) == 0x7C00).all() and ((sw[nan] & 0x03FF) != 0).all()


def test_f16_known_roundings(ref):
    # the only inexact scales the reference tests use: 0.1 and 0.01
    assert ref.f16_to_f32(ref.f32_to_f16(0.1)) == 0.0999755859375
    assert abs(ref.f16_to_f32(ref.f32_to_f16(0.01)) - 0.010002136) < 1e-9
    for v in (0.5, 0.25, 1.0, 0.125, 2.0):
        assert ref.f16_to_f32(ref.f32_to_f16(v)) == v


# ---- quantizers ----------------------------------------------------------------

def test_q8_0_round_half_away_from_zero(ref):
    x = np.zeros(32, dtype=np.float32)
    x[:8] = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49]
    q = ref.quantize_q8_0(x)
    assert q[0:2].tobytes() == O.f16_bytes(1.0)  # d = 127/127
    assert list(q[2:10].view(np.int8)) == [127, 1, 2, 3, -1, -2, -3, 3]  # rint would give 0,2,2


def test_q8_0_invariants(ref):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(32 * 500) * rng.choice([1e-3, 1.0, 50.0], size=32 * 500)).astype(np.float32)
    x[:32] = 0.0
    q = ref.quantize_q8_0(x).reshape(-1, 34)
    vals = q[:, 2:].view(np.int8).astype(np.int32)
    d = np.array([ref.f16_to_f32(int(b[0]) | int(b[1]) << 8) for b in q], dtype=np.float32)
    xb = x.reshape(-1, 32)
    assert (np.abs(vals) <= 127).all()
    assert d[0] == 0.0 and (vals[0] == 0).all()  # Q/quantize.rs:371-379
    amax_idx = np.abs(xb).argmax(axis=1)
    rows = np.arange(1, xb.shape[0])
    assert (np.abs(vals[rows, amax_idx[rows]]) == 127).all()
    assert (np.sign(vals[rows, amax_idx[rows]]) == np.sign(xb[rows, amax_idx[rows]])).all()
    # reconstruction within half a step of the unrounded scale (+ f16 rounding of d)
    d_exact = np.abs(xb).max(axis=1) / np.float32(127.0)
    err = np.abs(vals * d_exact[:, None] - xb)
    assert (err <= 0.5 * d_exact[:, None] * (1 + 1e-5) + 1e-30).all()
    assert np.allclose(d, d_exact, rtol=2.0**-11, atol=1e-8)


def test_q8_0_reference_round_trips(ref):
    # Q/quantize.rs:262-291
    for data, tol in (((np.arange(32, dtype=np.float32) / np.float32(15.5)) - 1, 0.02),
                      ((np.arange(128, dtype=np.float32) - 64) * np.float32(0.01), 0.01)):
        q = ref.quantize_q8_0(data)
        assert q.size == data.size // 32 * 34
        back = np.concatenate([ref.dequant_block(O.Q8_0, q[i:i + 34]) for i in range(0, q.size, 34)])
        assert np.abs(back - data).max() < tol


def test_q4_0_encoder_closed_form(ref):
    # extreme element -> nibble 0 (Q/quantize.rs:163); truncation of x*id + 8.5 (:176)
    x = np.zeros(32, dtype=np.float32)
    x[:6] = [-8.0, 0.4, 0.5, -0.6, 7.0, 7.6]
    q = ref.quantize_q4_0(x)
    assert q[0:2].tobytes() == O.f16_bytes(1.0)
    nibs = [(int(q[2 + i // 2]) >> (4 * (i % 2))) & 15 for i in range(32)]
    assert nibs[:6] == [0, 8, 9, 7, 15, 15]
    assert all(n == 8 for n in nibs[6:])
    # ties on |x|: the first element wins (strict >, :161)
    a = np.zeros(32, dtype=np.float32)
    a[0], a[1] = -8.0, 8.0
    b = np.zeros(32, dtype=np.float32)
    b[0], b[1] = 8.0, -8.0
    qa, qb = ref.quantize_q4_0(a), ref.quantize_q4_0(b)
    assert qa[0:2].tobytes() == O.f16_bytes(1.0) and qb[0:2].tobytes() == O.f16_bytes(-1.0)
    assert qa[2] == 0xF0 and qb[2] == 0xF0
    # zero block -> d = 0.0 / -8.0 = -0.0, nibbles 8 (Q/quantize.rs:360-368)
    z = ref.quantize_q4_0(np.zeros(32, dtype=np.float32))
    assert z[0] == 0 and z[1] == 0x80 and (z[2:] == 0x88).all()


def test_q4_0_reference_round_trips(ref):
    # Q/quantize.rs:228-257 and :399-423
    for data, tol in (((np.arange(32, dtype=np.float32) / np.float32(15.5)) - 1, 0.15),
                      ((np.arange(128, dtype=np.float32) - 64) * np.float32(0.01), 0.15)):
        q = ref.quantize_q4_0(data)
        back = np.concatenate([ref.dequant_block(O.Q4_0, q[i:i + 18]) for i in range(0, q.size, 18)])
        assert np.abs(back - data).max() < tol
    big = np.zeros(32, dtype=np.float32)
    big[0], big[1], big[31] = 1000.0, -1000.0, 500.0
    back = ref.dequant_block(O.Q4_0, ref.quantize_q4_0(big))
    assert back[0] > 0 and back[1] < 0 and back[31] > 0 and abs(back[0] - 1000) / 1000 < 0.15


def test_quantizers_reject_unaligned_and_accept_empty(ref):
    # Q/quantize.rs:333-353, :445
    with pytest.raises(O.OracleError) as e:
        ref.quantize_q8_0(np.zeros(31, dtype=np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 32, 31)
    with pytest.raises(O.OracleError) as e:
        ref.quantize_q4_0(np.zeros(33, dtype=np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 64, 33)
    assert ref.quantize_q8_0(np.zeros(0, dtype=np.float32)).size == 0
    assert ref.quantize_q4_0(np.zeros(0, dtype=np.float32)).size == 0


def test_synth_encoders_match_oracle_quantizers(ref):
    """The benchmark generator's Q4_0/Q8_0 encoders are an independent restatement of
    Q/quantize.rs:154-210; the two must agree byte for byte."""
    from oxillama_amd import synth
    x = synth.normal_f32(7, 32 * 4096, 0.02).reshape(64, -1)
    x[0, :32] = 0.0
    assert np.array_equal(synth.encode(O.Q8_0, x), ref.quantize_q8_0(x))
    assert np.array_equal(synth.encode(O.Q4_0, x), ref.quantize_q4_0(x))


# ---- block decoders ------------------------------------------------------------

@pytest.mark.parametrize("case", FX.dequant_cases(), ids=lambda c: c[0])
def test_dequant_block_known_answers(ref, case):
    _, t, block, expected, tol = case
    out = ref.dequant_block(t, block)
    for i, v in expected.items():
        assert abs(out[i] - v) <= tol, (i, out[i], v)


def test_q4_k_scale_unpack_known_answer(ref):
    # scales of Q/reference/q4_k.rs:499-511 -> sc=[5,3,7,2,9,11,13,15], mn=[4,6,1,3,0,0,0,0]
    block = np.frombuffer(O.make_q4_k_block(1.0, 1.0, FX.Q4K_SCALES_MIXED, [0x11] * 128), dtype=np.uint8)
    out = ref.dequant_block(O.Q4_K, block).reshape(8, 32)
    assert [float(r[0]) for r in out] == [1.0, -3.0, 6.0, -1.0, 9.0, 11.0, 13.0, 15.0]
    assert (out == out[:, :1]).all()


def test_q4_k_scale_unpack_high_bits(ref):
    # 6-bit values with bits 4-5 set in sub-blocks 4..7, packed by hand per decode_scales_mins
    sc = [63, 1, 32, 17, 48, 33, 63, 16]
    mn = [2, 62, 31, 5, 47, 18, 0, 63]
    s = [0] * 12
    for j in range(4):
        s[j] = sc[j] | ((sc[j + 4] >> 4) << 6)
        s[j + 4] = mn[j] | ((mn[j + 4] >> 4) << 6)
        s[j + 8] = (sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4)
    block = np.frombuffer(O.make_q4_k_block(1.0, 1.0, s, [0x11] * 128), dtype=np.uint8)
    out = ref.dequant_block(O.Q4_K, block).reshape(8, 32)
    assert [float(r[0]) for r in out] == [float(a - b) for a, b in zip(sc, mn)]


def test_q4_k_nibble_order(ref):
    # low nibbles are the first 32 weights of a 64-group, high nibbles the next 32
    qs = [(l % 16) | (((l + 5) % 16) << 4) for l in range(32)] * 4
    block = np.frombuffer(O.make_q4_k_block(1.0, 0.0, FX.Q4K_SCALES_ONES, qs), dtype=np.uint8)
    out = ref.dequant_block(O.Q4_K, block)
    for g in range(4):
        assert list(out[64 * g:64 * g + 32]) == [float(l % 16) for l in range(32)]
        assert list(out[64 * g + 32:64 * g + 64]) == [float((l + 5) % 16) for l in range(32)]


def test_iq4_xs_sub_scale_round_trip(ref):
    # Q/reference/iq4_xs.rs:364-380: [32,0,63,1,31,33,16,48] -> [0,-32,31,-31,-1,1,-16,16]
    block = np.frombuffer(O.make_iq4_xs_block(1.0, [32, 0, 63, 1, 31, 33, 16, 48], [0x88] * 128), dtype=np.uint8)
    out = ref.dequant_block(O.IQ4_XS, block).reshape(8, 32)
    assert [float(r[0]) for r in out] == [0.0, -32.0, 31.0, -31.0, -1.0, 1.0, -16.0, 16.0]


def test_iq4_xs_codebook_and_nibble_order(ref):
    kv = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]
    nib = [((2 * i) % 16) | (((2 * i + 1) % 16) << 4) for i in range(128)]
    block = np.frombuffer(O.make_iq4_xs_block(1.0, [33] * 8, nib), dtype=np.uint8)
    out = ref.dequant_block(O.IQ4_XS, block)
    assert list(out) == [float(kv[i % 16]) for i in range(256)]  # byte j -> weights 2j (lo), 2j+1 (hi)


def test_q4_0_nibble_order(ref):
    nib = [(2 * i) % 16 | (((2 * i + 1) % 16) << 4) for i in range(16)]
    out = ref.dequant_block(O.Q4_0, np.frombuffer(O.make_q4_0_block(1.0, nib), dtype=np.uint8))
    assert list(out) == [float(i % 16 - 8) for i in range(32)]


def test_q6_k_bit_layout_brute_force(ref):
    """Build a block from 256 known 6-bit values with the published layout (weight
    128h + 32j + l: low nibble in ql[64h + 32(j&1) + l] (upper half for j>=2), two
    high bits in qh[32h + l] at bit 2j) and check every decoded weight."""
    rng = np.random.default_rng(3)
    q = rng.integers(0, 64, size=256)
    sc = rng.integers(-128, 128, size=16)
    b = bytearray(210)
    for h in range(2):
        for j in range(4):
            for l in range(32):
                v = int(q[128 * h + 32 * j + l])
                b[64 * h + 32 * (j & 1) + l] |= (v & 15) << (4 if j >= 2 else 0)
                b[128 + 32 * h + l] |= (v >> 4) << (2 * j)
    for i in range(16):
        b[192 + i] = int(sc[i]) & 0xFF
    b[208:210] = O.f16_bytes(0.5)
    out = ref.dequant_block(O.Q6_K, np.frombuffer(bytes(b), dtype=np.uint8))
    expect = np.float32(0.5) * sc[np.arange(256) // 16].astype(np.float32) * (q - 32).astype(np.float32)
    assert np.array_equal(out, expect.astype(np.float32))


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_dequant_block_buffer_checks(ref, t):
    bs, bb = O.BLOCK[t]
    with pytest.raises(O.OracleError) as e:
        ref.dequant_block(t, np.zeros(4, dtype=np.uint8))
    assert (e.value.code, e.value.a, e.value.b) == (O.BUFFER_TOO_SMALL, bb, 4)
    with pytest.raises(O.OracleError) as e:
        ref.dequant_block(t, np.zeros(bb, dtype=np.uint8), out_len=1)
    assert (e.value.code, e.value.a, e.value.b) == (O.BUFFER_TOO_SMALL, bs, 1)


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_encode_decode_round_trip(ref, t):
    """dequant(encode(x)) stays within the format's quantisation step: a transposed
    index or swapped nibble order in either side shows up as O(sigma) error."""
    from oxillama_amd import synth
    x = synth.normal_f32(11, 8 * 1024, 0.02).reshape(8, 1024)
    w = synth.encode(t, x)
    back = ref.dequant_rows(t, w, 8, 1024)
    step = {O.Q4_0: 0.1, O.Q8_0: 0.006, O.Q4_K: 0.08, O.Q6_K: 0.03, O.IQ4_XS: 0.12}[t]
    assert np.abs(back - x).max() < step * np.abs(x).max()
    assert np.corrcoef(back.ravel(), x.ravel())[0, 1] > 0.99


# ---- gemv / gemm (f32 activations) -----------------------------------------------

def test_gemv_known_answers(ref):
    # Q/reference/q8_0.rs:175-190: 1 * 2.0 * 3.0 = 6.0
    q = [0] * 32
    q[0] = 1
    x = np.zeros(32, dtype=np.float32)
    x[0] = 3.0
    w = np.frombuffer(O.make_q8_0_block(2.0, q), dtype=np.uint8)
    assert ref.gemv(O.Q8_0, w, 1, 32, x)[0] == 6.0
    # Q/reference/q8_0.rs:216-232: gemm 4 * 0.5 * 3 = 6.0
    q[0] = 4
    w = np.frombuffer(O.make_q8_0_block(0.5, q), dtype=np.uint8)
    assert ref.gemm(O.Q8_0, w, x, 1, 1, 32)[0, 0] == 6.0
    # Q/reference/q4_k.rs:411-436: all weights 1.0, ones input -> 256
    w = np.frombuffer(O.make_q4_k_block(1.0, 0.0, FX.Q4K_SCALES_ONES, [0x11] * 128), dtype=np.uint8)
    assert ref.gemv(O.Q4_K, w, 1, 256, np.ones(256, dtype=np.float32))[0] == 256.0
    # Q/reference/iq4_xs.rs:304-353
    b0 = O.make_iq4_xs_block(1.0, [32] * 8, [0x88] * 128)
    b1 = O.make_iq4_xs_block(1.0, [33] * 8, [0x88] * 128)
    y = ref.gemv(O.IQ4_XS, np.frombuffer(b0 + b1, dtype=np.uint8), 2, 256, np.ones(256, dtype=np.float32))
    assert y[0] == 0.0 and y[1] == 256.0
    # Q/reference/q4_0.rs:273-308: zero weights
    w = np.frombuffer(O.make_q4_0_block(1.0, [0x88] * 16) * 2, dtype=np.uint8)
    assert (ref.gemm(O.Q4_0, w, np.ones(64, dtype=np.float32), 2, 2, 32) == 0).all()


def test_q6_k_gemv_equals_dequant_dot(ref):
    # Q/reference/q6_k.rs:417-460 (tolerance 0.1 there; fp32 order differs only slightly)
    block, x = FX.q6k_pattern_block()
    deq = ref.dequant_block(O.Q6_K, block)
    y = ref.gemv(O.Q6_K, block, 1, 256, x)[0]
    assert abs(y - float(np.dot(deq.astype(np.float64), x.astype(np.float64)))) < 1e-3


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_gemv_equals_dequant_matmul(ref, t):
    from oxillama_amd import synth
    n_rows, n_cols = 5, 768
    w = synth.weights(t, 21, n_rows, n_cols)
    x = synth.normal_f32(22, n_cols)
    y = ref.gemv(t, w, n_rows, n_cols, x)
    y64 = ref.dequant_rows(t, w, n_rows, n_cols).astype(np.float64) @ x.astype(np.float64)
    assert np.abs(y - y64).max() <= 1e-5 * np.abs(y64).max() + 1e-7


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_gemv_dimension_errors(ref, t):
    # Q/reference/q4_0.rs:311-337 and the same tests per format
    bs, bb = O.BLOCK[t]
    w = np.zeros(2 * bb, dtype=np.uint8)
    with pytest.raises(O.OracleError) as e:
        ref.gemv(t, w, 1, bs, np.zeros(4, dtype=np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, bs, 4)
    with pytest.raises(O.OracleError) as e:
        ref.gemv(t, w, 2, bs, np.zeros(bs, dtype=np.float32), y_len=1)
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 2, 1)


def test_gemv_partial_block_skips_out_of_range_columns(ref):
    # Q/simd/avx2/q4_0.rs:557-580 (20 of 32 columns), Q/simd/avx2/q4_k.rs:837-864 (200 of 256)
    from oxillama_amd import synth
    for t, n_cols, full in ((O.Q4_0, 20, 32), (O.Q8_0, 20, 32), (O.Q4_K, 200, 256), (O.Q6_K, 200, 256),
                            (O.IQ4_XS, 200, 256)):
        w = synth.weights(t, 5, 2, full)
        x = synth.normal_f32(6, full)
        xz = x.copy()
        xz[n_cols:] = 0.0
        assert np.allclose(ref.gemv(t, w, 2, n_cols, x[:n_cols]), ref.gemv(t, w, 2, full, xz), rtol=0, atol=1e-6)


# ---- matvec_q8_fused -----------------------------------------------------------------

@pytest.mark.parametrize("case", FX.fused_cases(), ids=lambda c: c[0])
def test_fused_fixture_tiers_agree(ref, case):
    """Replays the reference's SIMD-vs-scalar and fused-vs-unfused fixtures at its tolerance."""
    _, t, w, a, n_rows, n_cols, tol = case
    tiers = [O.TIER_SCALAR, O.TIER_AVX2] + ([O.TIER_Q4_0_STANDALONE] if t == O.Q4_0 else [])
    ys = [ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=tier) for tier in tiers]
    ys.append(ref.matvec_q8_intdot(t, w, a, n_rows, n_cols))
    # unfused: gemv on the dequantized activations
    xhat = np.concatenate([ref.dequant_block(O.Q8_0, a[i:i + 34]) for i in range(0, a.size, 34)])
    ys.append(ref.gemv(t, w, n_rows, n_cols, xhat))
    for y in ys[1:]:
        assert np.abs(y - ys[0]).max() < tol
    # exact value in integer arithmetic (all fixture scales are dyadic or shared)
    exact = ref.dequant_rows(t, w, n_rows, n_cols).astype(np.float64) @ xhat.astype(np.float64)
    assert np.abs(ys[1] - exact).max() < tol


@pytest.mark.parametrize("case", FX.accumulate_cases(), ids=lambda c: c[0])
def test_fused_accumulates(ref, case):
    _, t, w, a, n_cols, preset = case
    for tier in (O.TIER_SCALAR, O.TIER_AVX2):
        out = np.full(1, preset, dtype=np.float32)
        ref.matvec_q8_fused(t, w, a, 1, n_cols, tier=tier, out=out)
        assert out[0] == preset


def test_fused_adds_to_existing_output(ref):
    from oxillama_amd import synth
    for t in O.ALL_TYPES:
        w = synth.weights(t, 31, 3, 512)
        a = ref.quantize_q8_0(synth.normal_f32(32, 512))
        base = ref.matvec_q8_fused(t, w, a, 3, 512)
        out = np.array([1.5, -2.0, 100.0], dtype=np.float32)
        ref.matvec_q8_fused(t, w, a, 3, 512, out=out)
        assert np.array_equal(out, np.array([1.5, -2.0, 100.0], dtype=np.float32) + base)


def test_fused_zero_activations(ref):
    # Q/reference/q4_0.rs:382-392, q4_k.rs:451-471
    w = np.frombuffer(O.make_q4_0_block(1.0, [0x5A] * 16), dtype=np.uint8)
    a = np.frombuffer(O.make_q8_0_block(1.0, [0] * 32), dtype=np.uint8)
    assert ref.matvec_q8_fused(O.Q4_0, w, a, 1, 32, tier=O.TIER_Q4_0_STANDALONE)[0] == 0.0
    w = np.frombuffer(O.make_q4_k_block(1.0, 0.0, FX.Q4K_SCALES_ONES, [0x88] * 128), dtype=np.uint8)
    a = np.frombuffer(O.make_q8_0_block(1.0, [0] * 32) * 8, dtype=np.uint8)
    assert ref.matvec_q8_fused(O.Q4_K, w, a, 1, 256, tier=O.TIER_SCALAR)[0] == 0.0


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_fused_validation_order(ref, t):
    """out length, then weights, then activations (Q/reference/q4_k.rs:226-250)."""
    bs, bb = O.BLOCK[t]
    n_rows, n_cols = 3, 2 * bs
    rb = 2 * bb
    acts_needed = 2 * (bs // 32) * 34
    w = np.zeros(n_rows * rb, dtype=np.uint8)
    a = np.zeros(acts_needed, dtype=np.uint8)
    with pytest.raises(O.OracleError) as e:  # everything too small: out is reported first
        ref.matvec_q8_fused(t, w[:-1], a[:-1], n_rows, n_cols, out=np.zeros(2, dtype=np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 3, 2)
    with pytest.raises(O.OracleError) as e:
        ref.matvec_q8_fused(t, w[:-1], a[:-1], n_rows, n_cols)
    assert (e.value.code, e.value.a, e.value.b) == (O.BUFFER_TOO_SMALL, n_rows * rb, n_rows * rb - 1)
    with pytest.raises(O.OracleError) as e:
        ref.matvec_q8_fused(t, w, a[:-1], n_rows, n_cols)
    assert (e.value.code, e.value.a, e.value.b) == (O.BUFFER_TOO_SMALL, acts_needed, acts_needed - 1)


def _integer_weights(ref, t, w, n_rows, n_cols):
    """Integer weight values via dequant_block on a copy whose scales are forced to 1."""
    bs, bb = O.BLOCK[t]
    w = w.copy().reshape(-1, bb)
    one = np.frombuffer(O.f16_bytes(1.0), dtype=np.uint8)
    if t in (O.Q4_0, O.Q8_0):
        w[:, 0:2] = one
    elif t == O.Q4_K:
        w[:, 0:2] = one
        w[:, 2:4] = 0
        w[:, 4:16] = np.array(FX.Q4K_SCALES_ONES, dtype=np.uint8)
    elif t == O.Q6_K:
        w[:, 192:208] = 1
        w[:, 208:210] = one
    else:
        w[:, 0:2] = one
        w[:, 2:8] = np.frombuffer(O.make_iq4_xs_block(1.0, [33] * 8, [0] * 128)[2:8], dtype=np.uint8)
    return ref.dequant_rows(t, w.ravel(), n_rows, n_cols).astype(np.int64)


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_block_sums_brute_force(ref, t):
    from oxillama_amd import synth
    n_rows, n_cols = 4, 1024
    w = synth.weights(t, 41, n_rows, n_cols)
    a = ref.quantize_q8_0(synth.normal_f32(42, n_cols))
    qa = a.reshape(-1, 34)[:, 2:].view(np.int8).astype(np.int64).ravel()
    wi = _integer_weights(ref, t, w, n_rows, n_cols)
    if t == O.Q4_K:
        pass  # dequant with sc=1, dmin=0 gives the unsigned nibble: sum q*a as defined
    g = 16 if t == O.Q6_K else 32
    expect = (wi * qa[None, :]).reshape(n_rows, n_cols // g, g).sum(axis=2)
    assert np.array_equal(ref.block_sums(t, w, a, n_rows, n_cols), expect.astype(np.int32))


@pytest.mark.parametrize("t", O.ALL_TYPES, ids=lambda t: O.NAMES[t])
def test_intdot_form_from_block_sums(ref, t):
    """The integer-dot row equals scales x block sums recombined in float64 to fp32 accuracy,
    and agrees with the reference-order fused kernel within the parity tolerance."""
    from oxillama_amd import synth
    n_rows, n_cols = 6, 2048
    w = synth.weights(t, 51, n_rows, n_cols)
    a = ref.quantize_q8_0(synth.normal_f32(52, n_cols))
    xhat = np.concatenate([ref.dequant_block(O.Q8_0, a[i:i + 34]) for i in range(0, a.size, 34)])
    exact = ref.dequant_rows(t, w, n_rows, n_cols).astype(np.float64) @ xhat.astype(np.float64)
    tol = 1e-5 * np.abs(exact).max()
    y_int = ref.matvec_q8_intdot(t, w, a, n_rows, n_cols)
    assert np.abs(y_int - exact).max() <= tol
    for tier in (O.TIER_SCALAR, O.TIER_AVX2):
        assert np.abs(ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=tier) - y_int).max() <= tol
    if t != O.Q6_K and t != O.IQ4_XS:
        # Q4_0 / Q8_0 / Q4_K: the integer-dot form *is* the AVX2 tier, bit for bit
        assert np.array_equal(y_int, ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=O.TIER_AVX2))


def test_iq4_xs_fused_matches_reference_gemv_on_dequantized_activations(ref):
    """IQ4_XS has no working fused kernel in the reference; the integer form defined by this
    build is pinned against the reference's gemv applied to x_hat = d_a * q_a."""
    from oxillama_amd import synth
    n_rows, n_cols = 8, 4096
    w = synth.weights(O.IQ4_XS, 61, n_rows, n_cols)
    a = ref.quantize_q8_0(synth.normal_f32(62, n_cols))
    xhat = np.concatenate([ref.dequant_block(O.Q8_0, a[i:i + 34]) for i in range(0, a.size, 34)])
    y_gemv = ref.gemv(O.IQ4_XS, w, n_rows, n_cols, xhat)
    y = ref.matvec_q8_fused(O.IQ4_XS, w, a, n_rows, n_cols)
    assert np.abs(y - y_gemv).max() <= 1e-5 * np.abs(y_gemv).max()


@pytest.mark.parametrize("t,n_cols", [(O.Q4_K, 4096), (O.Q6_K, 14336), (O.Q8_0, 4096), (O.Q4_0, 4096)],
                         ids=["Q4_K-4096", "Q6_K-14336", "Q8_0-4096", "Q4_0-4096"])
def test_tolerance_budget_at_model_shapes(ref, t, n_cols):
    """At the Llama-3-8B inner dimensions, every fp32 ordering used (scalar tier, AVX2 tier,
    integer-dot) sits well inside 1e-5 * |y|_inf of the exact value, so the bound is a
    meaningful gate for a kernel that only reorders the block accumulation."""
    from oxillama_amd import synth
    n_rows = 16
    w = synth.weights(t, 71, n_rows, n_cols)
    a = ref.quantize_q8_0(synth.normal_f32(72, n_cols))
    xhat = np.concatenate([ref.dequant_block(O.Q8_0, a[i:i + 34]) for i in range(0, a.size, 34)])
    exact = ref.dequant_rows(t, w, n_rows, n_cols).astype(np.float64) @ xhat.astype(np.float64)
    tol = 1e-5 * np.abs(exact).max()
    for y in (ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=O.TIER_SCALAR),
              ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=O.TIER_AVX2),
              ref.matvec_q8_intdot(t, w, a, n_rows, n_cols)):
        assert np.abs(y - exact).max() <= 0.5 * tol


def test_gemm_q8_is_row_wise_quantize_plus_fused(ref):
    from oxillama_amd import synth
    m, n, k = 3, 4, 512
    w = synth.weights(O.Q4_K, 81, n, k)
    x = synth.normal_f32(82, m * k).reshape(m, k)
    y = ref.gemm_q8(O.Q4_K, w, x, m, n, k)
    for r in range(m):
        assert np.array_equal(y[r], ref.matvec_q8_fused(O.Q4_K, w, ref.quantize_q8_0(x[r]), n, k))


def test_threaded_row_split_is_bit_identical(ref):
    from oxillama_amd import synth
    w = synth.weights(O.Q4_K, 91, 37, 512)
    a = ref.quantize_q8_0(synth.normal_f32(92, 512))
    assert np.array_equal(ref.matvec_q8_fused_mt(O.Q4_K, w, a, 37, 512, 4), ref.matvec_q8_fused(O.Q4_K, w, a, 37, 512))


@pytest.mark.parametrize("t", [O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K], ids=lambda t: O.NAMES[t])
def test_avx2_twin_is_bit_identical_to_the_avx2_tier_restatement(ref, t):
    """The intrinsics twin timed as the CPU baseline computes exactly what the oracle's
    AVX2-order rows compute (integer sums are exact; the fp32 order is the same)."""
    from oxillama_amd import synth
    if ref.load_avx2() is None:
        pytest.skip("host CPU lacks AVX2/FMA/F16C")
    n_rows, n_cols = 19, 2048
    w = synth.weights(t, 95, n_rows, n_cols)
    a = ref.quantize_q8_0(synth.normal_f32(96, n_cols))
    want = ref.matvec_q8_fused(t, w, a, n_rows, n_cols, tier=O.TIER_AVX2)
    assert np.array_equal(ref.avx2_matvec_q8_fused(t, w, a, n_rows, n_cols, threads=1), want)
    assert np.array_equal(ref.avx2_matvec_q8_fused(t, w, a, n_rows, n_cols, threads=3), want)


def test_avx512_twin_of_the_f32_gemv_matches_the_scalar_restatement(ref):
    """The AVX-512 twin timed as the CPU figure of the fp32-activation route (Q/simd/avx512/q4_k.rs:279-415) against the
    scalar gemv (Q/reference/q4_k.rs:135-178): sixteen partial sums and a fused multiply-subtract instead of one chain,
    so within 1e-5 of the largest |y|, not bit for bit; threads split rows and change nothing.  A dequantized dot
    product in float64 bounds both from the other side (a wrong nibble order or scale index would be off by far more)."""
    from oxillama_amd import synth
    if ref.load_avx512() is None:
        pytest.skip("host CPU lacks AVX-512F")
    n_rows, n_cols = 23, 2048
    w = synth.weights(O.Q4_K, 97, n_rows, n_cols)
    x = synth.normal_f32(98, n_cols)
    want = ref.gemv(O.Q4_K, w, n_rows, n_cols, x)
    got = ref.avx512_gemv_q4_k(w, x, n_rows, n_cols, threads=1)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
    assert np.array_equal(ref.avx512_gemv_q4_k(w, x, n_rows, n_cols, threads=3), got)
    deq = ref.dequant_rows(O.Q4_K, w, n_rows, n_cols).astype(np.float64)
    exact = deq @ x.astype(np.float64)
    assert np.abs(got - exact).max() <= 1e-5 * np.abs(exact).max()
    with pytest.raises(ValueError):
        ref.avx512_gemv_q4_k(w, x, n_rows, 2000)
