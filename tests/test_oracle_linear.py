"""Pins the oracle's restatement of the callers' glue (oracle/oxq_oracle_linear.c): SwiGLU,
RMSNorm, LoRA and QuantLinear::forward, against the values the reference's own tests hold and
against float64 closed forms.  CPU only."""
import numpy as np
import pytest

import oracle as O


def test_swiglu_reference_values(ref):
    # crates/oxillama-arch/src/common/swiglu.rs:62-77
    h = ref.swiglu([1.0, -1.0, 0.0], [2.0, 3.0, 4.0])
    assert abs(h[0] - 1.4621) < 0.01
    assert abs(h[2]) < 1e-6
    # silu(-1) * 3 = -0.26894 * 3
    assert abs(h[1] - (-0.8068)) < 1e-3


def test_swiglu_closed_form(ref):
    rng = np.random.default_rng(5)
    g = (rng.standard_normal(4096) * 4).astype(np.float32)
    u = rng.standard_normal(4096).astype(np.float32)
    g[:4] = [0.0, -0.0, 88.0, -88.0]  # exp(-g) tiny / huge but finite
    h = ref.swiglu(g, u)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * u64
    assert np.all(np.abs(h - want) <= 4e-7 * np.abs(want) + 1e-30)
    # operation order: (g * sigmoid) * u with every step rounded to fp32
    sig = (np.float32(1.0) / (np.float32(1.0) + np.exp(-g).astype(np.float32))).astype(np.float32)
    step = ((g * sig).astype(np.float32) * u).astype(np.float32)
    # numpy's float32 exp may differ from libm's by an ulp; allow that much and no more
    assert np.all(np.abs(h - step) <= 3e-7 * np.abs(step) + 1e-30)
    assert h[0] == 0.0 and h[1] == 0.0


def test_swiglu_overflowing_exp(ref):
    # exp(-g) = inf for g < -88.7: sigmoid = 1/inf = 0, h = g * 0 * u = -0 or 0, never NaN
    h = ref.swiglu([-100.0, -1000.0, 100.0], [2.0, -3.0, 5.0])
    assert h[0] == 0.0 and h[1] == 0.0 and h[2] == 500.0


def test_rmsnorm_reference_values(ref):
    # crates/oxillama-arch/src/common/rms_norm.rs:72-88
    y = ref.rmsnorm([1.0, 2.0, 3.0, 4.0], [1.0] * 4, 1e-5)
    rms = np.sqrt(np.float32(7.5) + np.float32(1e-5))
    assert np.all(np.abs(y - np.array([1, 2, 3, 4], dtype=np.float32) / rms) < 1e-5)
    # doubling the weight doubles the output (rms_norm.rs:111-127)
    y1 = ref.rmsnorm([1.0, 2.0, 3.0], [1.0] * 3, 1e-5)
    y2 = ref.rmsnorm([1.0, 2.0, 3.0], [2.0] * 3, 1e-5)
    assert np.all(np.abs(y2 - 2 * y1) < 1e-6)
    assert ref.rmsnorm([], [], 1e-5).size == 0  # empty input: no work, no crash (rms_norm.rs:130-134)


def test_rmsnorm_closed_form(ref):
    rng = np.random.default_rng(6)
    for n in (32, 4096, 14336):
        x = (rng.standard_normal(n) * 3).astype(np.float32)
        w = (1 + 0.1 * rng.standard_normal(n)).astype(np.float32)
        y = ref.rmsnorm(x, w, 1e-5)
        x64 = x.astype(np.float64)
        want = x64 / np.sqrt(np.mean(x64 * x64) + 1e-5) * w
        assert np.max(np.abs(y - want)) <= 2e-6 * np.max(np.abs(want))
    # a sign error or a dropped eps would show here: all-zero input must give zeros, not NaN
    assert np.all(ref.rmsnorm(np.zeros(64), np.ones(64), 1e-5) == 0.0)


def test_lora_reference_values(ref):
    # crates/oxillama-quant/src/lora.rs:141-200
    out = np.zeros(2, dtype=np.float32)
    ref.lora_apply([1, 0, 0, 1], [2, 0, 0, 2], 2, 1.0, 2, 2, [3.0, 4.0], out)
    assert np.all(np.abs(out - [6.0, 8.0]) < 1e-6)
    out = np.array([10.0], dtype=np.float32)
    ref.lora_apply([1.0], [1.0], 1, 0.5, 1, 1, [4.0], out)
    assert abs(out[0] - 12.0) < 1e-6
    out = np.array([5.0], dtype=np.float32)
    ref.lora_apply([1.0], [1.0], 1, 1.0, 1, 1, [1.0], out)
    assert abs(out[0] - 6.0) < 1e-6


def test_lora_errors(ref):
    # lora.rs:203-259: construction and apply report DimensionMismatch{expected, got}
    with pytest.raises(O.OracleError) as e:
        ref.lora_new(1, 4, 2, 1, 2)
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 2, 1)
    with pytest.raises(O.OracleError) as e:
        ref.lora_new(2, 1, 1, 2, 2)
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 2, 1)
    ref.lora_new(4, 4, 2, 2, 2)
    with pytest.raises(O.OracleError) as e:
        ref.lora_apply([1, 0, 0, 1], [1, 0, 0, 1], 2, 1.0, 2, 2, [1.0], np.zeros(2, dtype=np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 2, 1)
    with pytest.raises(O.OracleError) as e:
        ref.lora_apply([1, 0, 0, 1], [1, 0, 0, 1], 2, 1.0, 2, 2, [1.0, 2.0], np.zeros(1, dtype=np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 2, 1)


def test_lora_float64(ref):
    rng = np.random.default_rng(7)
    rank, n_in, n_out = 16, 512, 384
    a = (rng.standard_normal((rank, n_in)) * 0.05).astype(np.float32)
    b = (rng.standard_normal((n_out, rank)) * 0.05).astype(np.float32)
    x = rng.standard_normal(n_in).astype(np.float32)
    base = rng.standard_normal(n_out).astype(np.float32)
    out = base.copy()
    ref.lora_apply(a, b, rank, 0.25, n_in, n_out, x, out)
    want = base + (b.astype(np.float64) @ (a.astype(np.float64) @ x)) * 0.25
    assert np.max(np.abs(out - want)) <= 1e-6 * max(1.0, np.max(np.abs(want)))
    # a transposed B or A would not even have the right shape semantics: check one element by hand
    r = a.astype(np.float64) @ x
    assert abs(out[5] - (base[5] + float(b[5].astype(np.float64) @ r) * 0.25)) < 1e-6


def _q8_identity(n, scale=1.0):
    """n x n identity as Q8_0 blocks: weight (r, r) = 1 * scale, everything else 0."""
    assert n % 32 == 0
    rows = []
    for r in range(n):
        for b in range(n // 32):
            qs = [0] * 32
            if r // 32 == b:
                qs[r % 32] = 1
            rows.append(O.make_q8_0_block(scale, qs))
    return b"".join(rows)


def test_linear_forward_reference_cases(ref):
    """QuantLinear tests of linear.rs:161-270 replayed on a Q8_0 identity (the reference uses an
    F32 tensor; the quantized-activation path adds the Q8_0 rounding of the input, so inputs are
    chosen to quantize exactly: one nonzero magnitude per 32-block)."""
    n = 32
    w = np.frombuffer(_q8_identity(n), dtype=np.uint8)
    x = np.zeros(n, dtype=np.float32)
    x[3], x[7] = 2.0, -2.0  # amax = 2: q = +-127, d = 2/127 in f16
    d = ref.f16_to_f32(ref.f32_to_f16(np.float32(2.0) / np.float32(127.0)))
    y = ref.linear_forward(O.Q8_0, w, n, n, x)
    assert y[3] == np.float32(d) * 127 and y[7] == -np.float32(d) * 127 and y[0] == 0.0
    assert abs(y[3] - 2.0) < 2e-3  # f16 rounding of the activation scale
    # bias, then LoRA (A = B = I, scale 1: delta = x), linear.rs:236-262: 2 + 10 + 2
    eye = np.eye(n, dtype=np.float32)
    y = ref.linear_forward(O.Q8_0, w, n, n, x, bias=np.full(n, 10.0, dtype=np.float32), lora=(eye, eye, n, 1.0))
    assert abs(y[3] - 14.0) < 2e-3 and abs(y[7] - 6.0) < 2e-3 and y[0] == 10.0
    # a short bias covers its own length only (zip semantics, linear.rs:87-89)
    y = ref.linear_forward(O.Q8_0, w, n, n, x, bias=np.full(4, 10.0, dtype=np.float32))
    assert abs(y[3] - 12.0) < 2e-3 and abs(y[7] + 2.0) < 2e-3 and y[1] == 10.0 and y[5] == 0.0
    # no LoRA = plain gemv (linear.rs:161-177, 207-233)
    y0 = ref.linear_forward(O.Q8_0, w, n, n, x)
    acts = ref.quantize_q8_0(x)
    assert np.array_equal(y0, ref.matvec_q8_fused(O.Q8_0, w, acts, n, n))


def test_linear_forward_errors(ref):
    w = np.frombuffer(_q8_identity(32), dtype=np.uint8)
    with pytest.raises(O.OracleError) as e:
        ref.linear_forward(O.Q8_0, w, 32, 32, np.zeros(31, dtype=np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 32, 31)
    with pytest.raises(O.OracleError) as e:
        ref.linear_forward(O.Q8_0, w, 32, 32, np.zeros(32, dtype=np.float32), out_len=31)
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 32, 31)


def test_argmax_and_topk(ref):
    # crates/oxillama-runtime/src/sampling/mod.rs:652-662: first of equal maxima; nothing above -inf -> 0
    assert ref.argmax([1.0, 5.0, 5.0, 2.0]) == 1
    assert ref.argmax([-np.inf, -np.inf]) == 0 and ref.argmax([]) == 0
    assert ref.argmax([np.nan, 3.0, np.nan]) == 1  # comparisons with NaN are false
    rng = np.random.default_rng(3)
    v = rng.standard_normal(5000).astype(np.float32)
    v[100:110] = v[7]  # exact ties
    for k in (1, 2, 40, 256):
        vals, idx = ref.topk(v, k)
        order = np.argsort(-v.astype(np.float64), kind="stable")[:k]  # stable: lower index first among equals
        assert np.array_equal(idx, order.astype(np.uint32)) and np.array_equal(vals, v[order])
        assert np.all(vals[:-1] >= vals[1:])
    assert ref.topk(v, 1)[1][0] == ref.argmax(v)
    # mod.rs:500-509 on a hand-made list: sorted by value, truncated
    vals, idx = ref.topk([0.1, 0.7, 0.05, 0.15], 2)
    assert list(idx) == [1, 3] and list(vals) == [np.float32(0.7), np.float32(0.15)]
