"""Pins the oracle's restatement of the formats beyond the first five (oracle/oxq_oracle_more.c)
against the known answers the reference's own tests hold (Q/reference/{q4_1,q5_0,q5_1,q8_1,
iq4_nl,q2_k,q3_k,q5_k}.rs, Q/ = crates/oxillama-quant/src), against numpy decoders written
independently from the format definitions, and against identities that a wrong index, sign or
bit position breaks.  CPU only."""
import numpy as np
import pytest

import oracle as O

KV = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.int32)


def f16(b, off):
    return np.frombuffer(bytes(b[off:off + 2]), dtype=np.float16)[0].astype(np.float32)


def decode(t, blk):
    """Independent decoder: (integer weights [n], fp32 multiplier per weight, fp32 offset per weight)."""
    b = np.frombuffer(bytes(blk), dtype=np.uint8).astype(np.int32)
    if t == O.Q4_1:
        q = np.stack([b[4:20] & 15, b[4:20] >> 4], axis=1).ravel()
        return q, np.full(32, f16(blk, 0)), np.full(32, f16(blk, 2))
    if t in (O.Q5_0, O.Q5_1):
        base = 2 if t == O.Q5_0 else 4
        qh = int.from_bytes(bytes(blk[base:base + 4]), "little")
        qs = b[base + 4:base + 20]
        bits = np.array([(qh >> i) & 1 for i in range(32)], dtype=np.int32)
        q = np.concatenate([(qs & 15) | (bits[:16] << 4), (qs >> 4) | (bits[16:] << 4)])
        if t == O.Q5_0:
            return q - 16, np.full(32, f16(blk, 0)), np.zeros(32, dtype=np.float32)
        return q, np.full(32, f16(blk, 0)), np.full(32, f16(blk, 2))
    if t == O.Q8_1:
        return b[4:36].astype(np.int8).astype(np.int32), np.full(32, f16(blk, 0)), np.zeros(32, dtype=np.float32)
    if t == O.IQ4_NL:
        q = np.stack([KV[b[2:18] & 15], KV[b[2:18] >> 4]], axis=1).ravel()
        return q, np.full(32, f16(blk, 0)), np.zeros(32, dtype=np.float32)
    if t == O.Q2_K:
        qs = b[16:80]
        q = np.zeros(256, dtype=np.int32)
        for col in range(256):
            n, r = divmod(col, 128)
            j, l = divmod(r, 32)
            q[col] = (qs[32 * n + l] >> (2 * j)) & 3
        sc = np.repeat(b[:16] & 15, 16).astype(np.float32)
        mn = np.repeat(b[:16] >> 4, 16).astype(np.float32)
        return q, f16(blk, 80) * sc, -(f16(blk, 82) * mn)
    if t == O.Q3_K:
        hm, qs, s = b[:32], b[32:96], b[96:108]
        q = np.zeros(256, dtype=np.int32)
        for col in range(256):
            n, r = divmod(col, 128)
            j, l = divmod(r, 32)
            lo = (qs[32 * n + l] >> (2 * j)) & 3
            q[col] = lo - (0 if (hm[l] >> (4 * n + j)) & 1 else 4)
        sc = np.zeros(16, dtype=np.int32)
        for j in range(4):
            sc[j] = s[j] & 63
            sc[4 + j] = s[4 + j] & 63
            sc[8 + j] = (s[8 + j] & 15) | ((s[j] >> 6) << 4)
            sc[12 + j] = (s[8 + j] >> 4) | ((s[4 + j] >> 6) << 4)
        return q, f16(blk, 108) * np.repeat(sc - 32, 16).astype(np.float32), np.zeros(256, dtype=np.float32)
    if t == O.Q5_K:
        s, qh, qs = b[4:16], b[16:48], b[48:176]
        q = np.zeros(256, dtype=np.int32)
        for col in range(256):
            g, r = divmod(col, 64)
            hi, l = divmod(r, 32)
            nib = (qs[32 * g + l] >> (4 * hi)) & 15
            q[col] = nib | (((qh[l] >> (g + 4 * hi)) & 1) << 4)
        sc = np.zeros(8, dtype=np.int32)
        mn = np.zeros(8, dtype=np.int32)
        for j in range(4):
            sc[j], mn[j] = s[j] & 63, s[j + 4] & 63
            sc[4 + j] = (s[8 + j] & 15) | ((s[j] >> 6) << 4)
            mn[4 + j] = (s[8 + j] >> 4) | ((s[4 + j] >> 6) << 4)
        return q, f16(blk, 0) * np.repeat(sc, 32).astype(np.float32), -(f16(blk, 2) * np.repeat(mn, 32).astype(np.float32))
    raise AssertionError(t)


def dequant_np(t, blk):
    q, mul, off = decode(t, blk)
    return (mul.astype(np.float32) * q.astype(np.float32) + off.astype(np.float32)).astype(np.float32)


# ---- known answers held by the reference's tests --------------------------------------------------

def test_reference_known_answers(ref):
    dq = ref.dequant_block
    # q4_1.rs tests: zeros; min only -> 5.0; d=1, m=2, nibbles 8 -> 10.0
    assert np.all(dq(O.Q4_1, O.make_q4_1_block(0.0, 0.0, [0] * 16)) == 0)
    assert np.all(dq(O.Q4_1, O.make_q4_1_block(0.0, 5.0, [0] * 16)) == 5.0)
    assert np.all(dq(O.Q4_1, O.make_q4_1_block(1.0, 2.0, [0x88] * 16)) == 10.0)
    # q5_0.rs:257-317: zeros; all q = 16 -> 0; all q = 31 -> 15; all q = 0, d = 2 -> -32
    assert np.all(dq(O.Q5_0, O.make_q5_0_block(0.0, 0, [0] * 16)) == 0)
    assert np.all(dq(O.Q5_0, O.make_q5_0_block(1.0, 0xFFFFFFFF, [0] * 16)) == 0)
    assert np.all(dq(O.Q5_0, O.make_q5_0_block(1.0, 0xFFFFFFFF, [0xFF] * 16)) == 15.0)
    assert np.all(dq(O.Q5_0, O.make_q5_0_block(2.0, 0, [0] * 16)) == -32.0)
    # q5_1.rs tests: zeros; min only -> 3; high bit only -> 16; max -> 31
    assert np.all(dq(O.Q5_1, O.make_q5_1_block(0.0, 0.0, 0, [0] * 16)) == 0)
    assert np.all(dq(O.Q5_1, O.make_q5_1_block(0.0, 3.0, 0, [0] * 16)) == 3.0)
    assert np.all(dq(O.Q5_1, O.make_q5_1_block(1.0, 0.0, 0xFFFFFFFF, [0] * 16)) == 16.0)
    assert np.all(dq(O.Q5_1, O.make_q5_1_block(1.0, 0.0, 0xFFFFFFFF, [0xFF] * 16)) == 31.0)
    # q8_1.rs tests: zeros; d = 0.5, q = 10 -> 5; d = 2, q = -5 -> -10
    assert np.all(dq(O.Q8_1, O.make_q8_1_block(0.0, [0] * 32)) == 0)
    assert np.all(dq(O.Q8_1, O.make_q8_1_block(0.5, [10] * 32)) == 5.0)
    assert np.all(dq(O.Q8_1, O.make_q8_1_block(2.0, [-5] * 32)) == -10.0)
    # iq4_nl.rs:159-201: byte 0x50 -> -127, -35; index 0 at d = 2 -> -254; index 15 -> 113
    out = dq(O.IQ4_NL, O.make_iq4_nl_block(1.0, [0x50] + [0] * 15))
    assert out[0] == -127.0 and out[1] == -35.0
    assert np.all(dq(O.IQ4_NL, O.make_iq4_nl_block(2.0, [0] * 16)) == -254.0)
    assert np.all(dq(O.IQ4_NL, O.make_iq4_nl_block(1.0, [0xFF] * 16)) == 113.0)
    # q2_k.rs tests: zeros; scales 0x01, qs 0xFF -> 3; d=2, dmin=1, scales 0x11, qs 0 -> -1
    assert np.all(dq(O.Q2_K, O.make_q2_k_block(0.0, 0.0, [0] * 16, [0] * 64)) == 0)
    assert np.all(dq(O.Q2_K, O.make_q2_k_block(1.0, 0.0, [0x01] * 16, [0xFF] * 64)) == 3.0)
    assert np.all(dq(O.Q2_K, O.make_q2_k_block(2.0, 1.0, [0x11] * 16, [0] * 64)) == -1.0)
    # q3_k.rs tests: zeros; hmask set, qs 0 -> 0; hmask clear, all scales +1 -> -4; hmask set, qs 0xFF -> 3
    sc1 = [0xA1] * 8 + [0x11] * 4
    assert np.all(dq(O.Q3_K, O.make_q3_k_block(0.0, [0] * 12, [0] * 32, [0] * 64)) == 0)
    assert np.all(dq(O.Q3_K, O.make_q3_k_block(1.0, [0x21] * 8 + [0] * 4, [0xFF] * 32, [0] * 64)) == 0)
    assert np.all(dq(O.Q3_K, O.make_q3_k_block(1.0, sc1, [0] * 32, [0] * 64)) == -4.0)
    assert np.all(dq(O.Q3_K, O.make_q3_k_block(1.0, sc1, [0xFF] * 32, [0xFF] * 64)) == 3.0)
    # q5_k.rs:380-438: zeros; scales 1, qh 0, nibbles 8 -> 8; qh 0xFF, nibbles 0 -> 16
    sc5 = [1] * 4 + [0] * 4 + [1] * 4
    assert np.all(dq(O.Q5_K, O.make_q5_k_block(0.0, 0.0, [0] * 12, [0] * 32, [0] * 128)) == 0)
    assert np.all(dq(O.Q5_K, O.make_q5_k_block(1.0, 0.0, sc5, [0] * 32, [0x88] * 128)) == 8.0)
    assert np.all(dq(O.Q5_K, O.make_q5_k_block(1.0, 0.0, sc5, [0xFF] * 32, [0] * 128)) == 16.0)


def test_iq4_nl_gemv_reference_rows(ref):
    # iq4_nl.rs:220-271: nibbles 0x88 (kv = 1) against ones -> 32; 0xFF (kv = 113) -> 3616
    w = O.make_iq4_nl_block(1.0, [0x88] * 16) + O.make_iq4_nl_block(1.0, [0xFF] * 16)
    y = ref.gemv(O.IQ4_NL, np.frombuffer(w, dtype=np.uint8), 2, 32, np.ones(32, dtype=np.float32))
    assert y[0] == 32.0 and y[1] == 3616.0


def test_reference_gemv_pattern_blocks(ref):
    """The `test_gemv_*` cases of the reference: gemv == sum dequant * x (their tolerance 0.1; here 1e-4)."""
    cases = [
        (O.Q5_0, O.make_q5_0_block(0.5, 0xA5A5A5A5, [(i * 11 + 5) & 0xFF for i in range(16)]),
         [(i * 0.1) - 1.6 for i in range(32)]),  # q5_0.rs:320-345
        (O.Q5_K, O.make_q5_k_block(0.5, 0.25, [(i * 17 + 3) & 0xFF for i in range(12)],
                                   [(i * 13 + 7) & 0xFF for i in range(32)], [(i * 5 + 11) & 0xFF for i in range(128)]),
         [(i * 0.01) - 1.28 for i in range(256)]),  # q5_k.rs:441-475
    ]
    for t, blk, x in cases:
        x = np.array(x, dtype=np.float32)
        w = np.frombuffer(blk, dtype=np.uint8)
        y = ref.gemv(t, w, 1, x.size, x)
        want = float(ref.dequant_block(t, w).astype(np.float64) @ x.astype(np.float64))
        assert abs(y[0] - want) < 1e-4 * max(1.0, abs(want))


# ---- independent decoders on random bytes -------------------------------------------------------------

@pytest.mark.parametrize("t", O.MORE_TYPES, ids=lambda t: O.NAMES[t])
def test_dequant_matches_independent_decoder(ref, t):
    bs, bb = O.BLOCK[t]
    w = O.random_blocks(t, 40 + t, 16, bs)
    for i in range(16):
        blk = w[i * bb:(i + 1) * bb]
        got, want = ref.dequant_block(t, blk), dequant_np(t, blk)
        assert np.array_equal(got, want), f"block {i}: first diff at {np.nonzero(got != want)[0][:4]}"


@pytest.mark.parametrize("t", O.MORE_TYPES, ids=lambda t: O.NAMES[t])
def test_block_sizes(ref, t):
    lib = O.load()
    assert (lib.oxq_ref_block_size(t), lib.oxq_ref_block_bytes(t)) == O.BLOCK[t]


@pytest.mark.parametrize("t", O.MORE_TYPES, ids=lambda t: O.NAMES[t])
def test_gemv_and_fused_against_float64(ref, t):
    bs, bb = O.BLOCK[t]
    n_rows, n_cols = 7, 2 * 256
    w = O.random_blocks(t, 60 + t, n_rows, n_cols)
    x = np.random.default_rng(t).standard_normal(n_cols).astype(np.float32)
    W = np.stack([np.concatenate([dequant_np(t, w[(r * (n_cols // bs) + b) * bb:][:bb]) for b in range(n_cols // bs)])
                  for r in range(n_rows)]).astype(np.float64)
    y = ref.gemv(t, w, n_rows, n_cols, x)
    want = W @ x.astype(np.float64)
    assert np.max(np.abs(y - want)) <= 2e-5 * np.max(np.abs(want))
    # fused: the same product with x replaced by the dequantized Q8_0 activations, accumulated onto out
    acts = ref.quantize_q8_0(x)
    a = np.frombuffer(acts.tobytes(), dtype=np.uint8).reshape(-1, 34)
    xhat = (a[:, 2:].view(np.int8).astype(np.float64) * a[:, :2].copy().view(np.float16).astype(np.float64)).ravel()
    out = np.full(n_rows, 42.0, dtype=np.float32)  # accumulate semantics
    ref.matvec_q8_fused(t, w, acts, n_rows, n_cols, out=out)
    want = 42.0 + W @ xhat
    assert np.max(np.abs(out - want)) <= 2e-5 * np.max(np.abs(want))
    # the integer-dot form agrees too
    y2 = ref.matvec_q8_intdot(t, w, acts, n_rows, n_cols)
    assert np.max(np.abs(y2 - W @ xhat)) <= 2e-5 * np.max(np.abs(want))


@pytest.mark.parametrize("t", O.MORE_TYPES, ids=lambda t: O.NAMES[t])
def test_block_sums_brute_force(ref, t):
    bs, bb = O.BLOCK[t]
    n_rows, n_cols = 3, 512
    w = O.random_blocks(t, 80 + t, n_rows, n_cols)
    x = np.random.default_rng(100 + t).standard_normal(n_cols).astype(np.float32)
    acts = ref.quantize_q8_0(x)
    qa = np.frombuffer(acts.tobytes(), dtype=np.uint8).reshape(-1, 34)[:, 2:].view(np.int8).astype(np.int64).ravel()
    got = ref.block_sums(t, w, acts, n_rows, n_cols)
    g = O.GROUP_COLS[t]
    for r in range(n_rows):
        q = np.concatenate([decode(t, w[(r * (n_cols // bs) + b) * bb:][:bb])[0] for b in range(n_cols // bs)])
        want = (q.astype(np.int64) * qa).reshape(-1, g).sum(axis=1)
        assert np.array_equal(got[r], want)


@pytest.mark.parametrize("t", O.MORE_TYPES, ids=lambda t: O.NAMES[t])
def test_fused_tail_columns_and_errors(ref, t):
    bs, bb = O.BLOCK[t]
    if t in (O.Q5_0, O.Q8_1):
        n_cols = 2 * bs  # the reference's Q5_0 and Q8_1 gemv loops have no tail handling
    else:
        n_cols = 2 * bs - 12  # ragged: the last 12 columns of the second block do not exist
    w = O.random_blocks(t, 120 + t, 2, 2 * bs)
    x = np.random.default_rng(7).standard_normal(2 * bs).astype(np.float32)
    y = ref.gemv(t, w, 2, n_cols, x[:n_cols])
    W = np.stack([np.concatenate([dequant_np(t, w[(r * 2 + b) * bb:][:bb]) for b in range(2)]) for r in range(2)])
    want = W[:, :n_cols].astype(np.float64) @ x[:n_cols].astype(np.float64)
    assert np.max(np.abs(y - want)) <= 2e-5 * np.max(np.abs(want))
    with pytest.raises(O.OracleError) as e:
        ref.gemv(t, w, 2, 2 * bs, x[:5])
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 2 * bs, 5)
    with pytest.raises(O.OracleError) as e:
        ref.matvec_q8_fused(t, w[:-1], ref.quantize_q8_0(x), 2, 2 * bs)
    assert (e.value.code, e.value.a, e.value.b) == (O.BUFFER_TOO_SMALL, 4 * bb, 4 * bb - 1)
