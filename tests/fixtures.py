"""Input vectors held by the reference's own unit tests for this path, as data.

Each entry names the test it comes from (Q/ = crates/oxillama-quant/src in the
reference tree).  The expected values are the closed-form answers those tests
state; tolerances are the reference's.
"""
import numpy as np

import oracle as O

Q8_ALT16 = [1, -2, 3, -4, 5, -6, 7, -8, 9, -10, 11, -12, 13, -14, 15, -16,
            -1, 2, -3, 4, -5, 6, -7, 8, -9, 10, -11, 12, -13, 14, -15, 16]
Q8_MULTI = [2, 4, -6, 8, -10, 12, -14, 16, 1, -3, 5, -7, 9, -11, 13, -15,
            0, 1, -2, 3, -4, 5, -6, 7, -8, 9, -10, 11, -12, 13, -14, 15]
Q8_Q4K_MULTI = [2, -1, 4, -3, 6, -5, 8, -7, 1, -2, 3, -4, 5, -6, 7, -8,
                -2, 1, -4, 3, -6, 5, -8, 7, -1, 2, -3, 4, -5, 6, -7, 8]
Q8_Q6K_SINGLE = [1, -2, 3, -4, 5, -6, 7, -8, 9, -10, 11, -12, 13, -14, 15, -16,
                 0, 1, -1, 2, -2, 3, -3, 4, -4, 5, -5, 6, -6, 7, -7, 8]
Q8_Q6K_MULTI = [2, -3, 5, -7, 1, -1, 4, -4, 6, -6, 3, -3, 2, -2, 1, -1,
                8, -8, 7, -7, 6, -6, 5, -5, 4, -4, 3, -3, 2, -2, 1, -1]
NIB_A = [0x5A, 0xF0, 0x13, 0x7E, 0xC2, 0x48, 0x9D, 0x6B, 0xA3, 0x2F, 0x71, 0xE4, 0x0C, 0x58, 0xB6, 0xD9]
NIB_B = [0x13, 0x57, 0x9B, 0xDF, 0x24, 0x68, 0xAC, 0xE0, 0x5F, 0x3A, 0x72, 0x8D, 0xC6, 0x4E, 0x91, 0xB7]
Q4K_SCALES_MIXED = [5, 3, 7, 2, 4, 6, 1, 3, 9, 11, 13, 15]
Q4K_SCALES_ONES = [1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1]
Q8W_SINGLE = [10, -20, 30, -40, 50, -60, 70, -80, 90, -100, 110, -120, 100, -90, 80, -70,
              60, -50, 40, -30, 20, -10, 5, -15, 25, -35, 45, -55, 65, -75, 85, -95]
Q8W_B = [20, -30, 40, -50, 60, -70, 80, -90, 100, -110, 120, -127, 100, -90, 80, -70,
         50, -40, 30, -20, 10, -5, 15, -25, 35, -45, 55, -65, 75, -85, 95, -100]


def _cat(*parts):
    return np.frombuffer(b"".join(parts), dtype=np.uint8).copy()


def fused_cases():
    """(name, type, weights, acts, n_rows, n_cols, tol) -- fused-kernel fixtures whose
    reference tests compare two tiers (or fused vs unfused) at `tol` absolute."""
    cases = []
    # Q/reference/q4_0.rs:423-464 and Q/simd/avx2/q4_0.rs:637-671
    cases.append(("q4_0_single", O.Q4_0, _cat(O.make_q4_0_block(0.25, NIB_A)),
                  _cat(O.make_q8_0_block(0.5, Q8_ALT16)), 1, 32, 1e-3))
    # Q/reference/q4_0.rs:467-537 (d_a = 0.125) and Q/simd/avx2/q4_0.rs:673-727 (d_a = 0.5)
    for d_a in (0.125, 0.5):
        w = _cat(*[O.make_q4_0_block(s, NIB_B) for s in (0.1, 0.25, 0.5, 1.0) for _ in range(2)])
        a = _cat(*[O.make_q8_0_block(d_a, Q8_MULTI) for _ in range(2)])
        cases.append((f"q4_0_multi_row_da{d_a}", O.Q4_0, w, a, 4, 64, 1e-3))
    # Q/simd/avx2/q8_0.rs:546-580
    cases.append(("q8_0_single", O.Q8_0, _cat(O.make_q8_0_block(0.5, Q8W_SINGLE)),
                  _cat(O.make_q8_0_block(0.1, Q8_Q6K_SINGLE)), 1, 32, 1e-3))
    # Q/simd/avx2/q8_0.rs:582-636
    w = _cat(*[blk for s in (0.25, 0.5, 1.0)
               for blk in (O.make_q8_0_block(s, Q8_ALT16), O.make_q8_0_block(s * 0.5, Q8W_B))])
    a = _cat(*[O.make_q8_0_block(0.05, Q8_Q6K_MULTI) for _ in range(2)])
    cases.append(("q8_0_multi_row", O.Q8_0, w, a, 3, 64, 1e-3))
    # Q/reference/q4_k.rs:496-559 and Q/simd/avx2/q4_k.rs:903-955
    cases.append(("q4_k_mixed_scales", O.Q4_K,
                  _cat(O.make_q4_k_block(0.5, 0.1, Q4K_SCALES_MIXED, [0xA5] * 128)),
                  _cat(*[O.make_q8_0_block(0.25, Q8_ALT16) for _ in range(8)]), 1, 256, 1e-3))
    # Q/reference/q4_k.rs:562-625 and Q/simd/avx2/q4_k.rs:978-1028
    w = _cat(*[O.make_q4_k_block(s, 0.0, Q4K_SCALES_ONES, [0x55] * 128) for s in (0.5, 1.0, 0.25, 0.1)])
    a = _cat(*[O.make_q8_0_block(0.5, Q8_Q4K_MULTI) for _ in range(8)])
    cases.append(("q4_k_multi_row", O.Q4_K, w, a, 4, 256, 1e-3))
    # Q/simd/avx2/q6_k.rs:939-980
    ql = [(i * 5 + 11) & 0xFF for i in range(128)]
    qh = [(i * 13 + 7) & 0xFF for i in range(64)]
    cases.append(("q6_k_single", O.Q6_K, _cat(O.make_q6k_block(0.01, ql, qh, list(range(1, 17)))),
                  _cat(*[O.make_q8_0_block(0.1, Q8_Q6K_SINGLE) for _ in range(8)]), 1, 256, 1e-3))
    # Q/simd/avx2/q6_k.rs:983-1036
    blocks = []
    for r in range(3):
        for b in range(2):
            ql = [(r * 17 + b * 11 + i * 5) & 0xFF for i in range(128)]
            qh = [(r * 13 + b * 19 + i * 3) & 0xFF for i in range(64)]
            sc = [(r * 7 + b * 11 + i * 13 + 5) & 0xFF for i in range(16)]
            blocks.append(O.make_q6k_block(0.01 + np.float32(r) * np.float32(0.005), ql, qh, sc))
    cases.append(("q6_k_multi_row", O.Q6_K, _cat(*blocks),
                  _cat(*[O.make_q8_0_block(0.05, Q8_Q6K_MULTI) for _ in range(16)]), 3, 512, 1e-3))
    return cases


def accumulate_cases():
    """(name, type, weights, acts, n_cols, preset) -- zero contribution must leave `preset`."""
    z8 = [0] * 32
    return [
        # Q/reference/q4_0.rs:407-420, Q/simd/avx2/q4_0.rs:729-745
        ("q4_0", O.Q4_0, _cat(O.make_q4_0_block(1.0, [0x88] * 16)), _cat(O.make_q8_0_block(1.0, z8)), 32, 42.0),
        # Q/simd/avx2/q8_0.rs:638-655
        ("q8_0", O.Q8_0, _cat(O.make_q8_0_block(1.0, z8)), _cat(O.make_q8_0_block(1.0, z8)), 32, 55.0),
        # Q/reference/q4_k.rs:474-493, Q/simd/avx2/q4_k.rs:957-975
        ("q4_k", O.Q4_K, _cat(O.make_q4_k_block(0.0, 0.0, [0] * 12, [0] * 128)),
         _cat(*[O.make_q8_0_block(1.0, z8) for _ in range(8)]), 256, 42.0),
        # Q/simd/avx2/q6_k.rs:1039-1057
        ("q6_k", O.Q6_K, _cat(O.make_q6k_block(0.0, [0] * 128, [0] * 64, [0] * 16)),
         _cat(*[O.make_q8_0_block(0.0, z8) for _ in range(8)]), 256, 77.0),
    ]


def dequant_cases():
    """(name, type, block bytes, {index: expected}, tol) -- known answers of dequant_block."""
    nib = [0x88] * 16
    nib2 = list(nib)
    nib2[0] = 0xF0
    q8 = [0] * 32
    q8[0], q8[1], q8[31] = 10, -5, 127
    sub = [32] * 8
    sub[0] = 33
    q6 = bytearray(210)
    for i in range(64):
        q6[128 + i] = 0xAA
    for i in range(16):
        q6[192 + i] = 1
    q6[208:210] = O.f16_bytes(1.0)
    return [
        # Q/reference/q4_0.rs:247-256
        ("q4_0_zeros", O.Q4_0, _cat(O.make_q4_0_block(1.0, nib)), {i: 0.0 for i in range(32)}, 1e-5),
        # Q/reference/q4_0.rs:259-270
        ("q4_0_simple", O.Q4_0, _cat(O.make_q4_0_block(0.5, nib2)), {0: -4.0, 1: 3.5}, 0.0),
        # Q/reference/q8_0.rs:159-172
        ("q8_0_simple", O.Q8_0, _cat(O.make_q8_0_block(0.5, q8)), {0: 5.0, 1: -2.5, 31: 63.5}, 0.0),
        # Q/reference/q4_k.rs:369-378
        ("q4_k_zero_scale", O.Q4_K, _cat(O.make_q4_k_block(0.0, 0.0, [0] * 12, [0] * 128)),
         {i: 0.0 for i in range(256)}, 1e-5),
        # Q/reference/q4_k.rs:381-408
        ("q4_k_uniform", O.Q4_K, _cat(O.make_q4_k_block(1.0, 0.0, Q4K_SCALES_ONES, [0x88] * 128)),
         {i: 8.0 for i in range(256)}, 0.0),
        # Q/reference/q6_k.rs:369-379
        ("q6_k_zero", O.Q6_K, np.zeros(210, dtype=np.uint8), {i: 0.0 for i in range(256)}, 1e-5),
        # Q/reference/q6_k.rs:382-414
        ("q6_k_centre", O.Q6_K, np.frombuffer(bytes(q6), dtype=np.uint8).copy(), {i: 0.0 for i in range(256)}, 0.0),
        # Q/reference/iq4_xs.rs:252-263
        ("iq4_xs_zero_sub_scale", O.IQ4_XS, _cat(O.make_iq4_xs_block(1.0, [32] * 8, [0xAA] * 128)),
         {i: 0.0 for i in range(256)}, 1e-6),
        # Q/reference/iq4_xs.rs:266-285
        ("iq4_xs_unit_sub_scale", O.IQ4_XS, _cat(O.make_iq4_xs_block(1.0, sub, [0x88] * 128)),
         {**{i: 1.0 for i in range(32)}, **{i: 0.0 for i in range(32, 256)}}, 0.0),
    ]


def q6k_pattern_block():
    """The block of Q/reference/q6_k.rs:417-436 and its input vector (:444)."""
    b = bytearray(210)
    for i in range(128):
        b[i] = (i * 7 + 3) & 0xFF
    for i in range(64):
        b[128 + i] = (i * 13 + 5) & 0xFF
    for i in range(16):
        b[192 + i] = (i * 3 - 8) & 0xFF
    b[208:210] = O.f16_bytes(0.5)
    x = (np.arange(256, dtype=np.float32) * np.float32(0.01)) - np.float32(1.28)
    return np.frombuffer(bytes(b), dtype=np.uint8).copy(), x
