"""ctypes binding of oracle/liboxq_oracle.so -- the CPU oracle (test infrastructure)."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB_PATH = os.path.join(ORACLE_DIR, "liboxq_oracle.so")
F16C_PATH = os.path.join(ORACLE_DIR, "liboxq_f16c_check.so")
AVX2_PATH = os.path.join(ORACLE_DIR, "liboxq_cpu_avx2.so")

Q4_0, Q8_0, Q4_K, Q6_K, IQ4_XS = 2, 8, 12, 14, 23
ALL_TYPES = [Q4_0, Q8_0, Q4_K, Q6_K, IQ4_XS]
BLOCK = {Q4_0: (32, 18), Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210), IQ4_XS: (256, 136)}
NAMES = {Q4_0: "Q4_0", Q8_0: "Q8_0", Q4_K: "Q4_K", Q6_K: "Q6_K", IQ4_XS: "IQ4_XS"}

# formats beyond the first five (oracle/oxq_oracle_more.c); integer groups of 16 for Q2_K / Q3_K
Q4_1, Q5_0, Q5_1, Q8_1, Q2_K, Q3_K, Q5_K, IQ4_NL = 3, 6, 7, 9, 10, 11, 13, 20
MORE_TYPES = [Q4_1, Q5_0, Q5_1, Q8_1, Q2_K, Q3_K, Q5_K, IQ4_NL]
BLOCK.update({Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_1: (32, 36), Q2_K: (256, 84), Q3_K: (256, 110),
              Q5_K: (256, 176), IQ4_NL: (32, 18)})
NAMES.update({Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q8_1: "Q8_1", Q2_K: "Q2_K", Q3_K: "Q3_K", Q5_K: "Q5_K",
              IQ4_NL: "IQ4_NL"})
GROUP_COLS = {t: 32 for t in BLOCK}
GROUP_COLS.update({Q6_K: 16, Q2_K: 16, Q3_K: 16})

TIER_SCALAR, TIER_AVX2, TIER_Q4_0_STANDALONE = 0, 1, 2
OK, UNSUPPORTED_TYPE, DIMENSION_MISMATCH, KERNEL_ERROR, BUFFER_TOO_SMALL = 0, 1, 3, 4, 6


class Status(C.Structure):
    _fields_ = [("code", C.c_int), ("a", C.c_size_t), ("b", C.c_size_t)]


class OracleError(Exception):
    def __init__(self, st):
        super().__init__(f"oracle status {st.code} ({st.a}, {st.b})")
        self.code, self.a, self.b = st.code, st.a, st.b


_lib = None


def build():
    subprocess.run(["make", "-C", ORACLE_DIR, "-s", "liboxq_oracle.so", "liboxq_f16c_check.so"], check=True)


def host_has(flag):
    try:
        with open("/proc/cpuinfo") as f:
            return f" {flag}" in f.read()
    except OSError:
        return False


_avx2 = None


def load_avx2():
    """AVX2 intrinsics twin of the reference's SIMD fused rows (CPU baseline); None when the
    host CPU lacks AVX2/FMA/F16C."""
    global _avx2
    if _avx2 is not None:
        return _avx2
    if not (host_has("avx2") and host_has("fma") and host_has("f16c")):
        return None
    if not os.path.exists(AVX2_PATH):
        subprocess.run(["make", "-C", ORACLE_DIR, "-s", "liboxq_cpu_avx2.so"], check=True)
    lib = C.CDLL(AVX2_PATH)
    lib.oxq_avx2_matvec_q8_fused.restype = C.c_int
    lib.oxq_avx2_matvec_q8_fused.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                             C.c_size_t, C.c_int]
    _avx2 = lib
    return lib


def avx2_matvec_q8_fused(t, w, acts, n_rows, n_cols, threads=1, out=None):
    lib = load_avx2()
    w, acts = _u8(w), _u8(acts)
    if out is None:
        out = np.zeros(max(n_rows, 1), dtype=np.float32)
    rc = lib.oxq_avx2_matvec_q8_fused(t, _p(w), _p(acts), _p(out), n_rows, n_cols, threads)
    if rc != 0:
        raise ValueError("unsupported type or partial block")
    return out[:n_rows]


_avx512 = None
AVX512_PATH = os.path.join(ORACLE_DIR, "liboxq_cpu_avx512.so")


def load_avx512():
    """AVX-512 intrinsics twin of the reference's fp32-activation gemv for Q4_K (CPU baseline of that route);
    None when the host CPU lacks AVX-512F."""
    global _avx512
    if _avx512 is not None:
        return _avx512
    if not (host_has("avx512f") and host_has("fma") and host_has("f16c")):
        return None
    if not os.path.exists(AVX512_PATH):
        subprocess.run(["make", "-C", ORACLE_DIR, "-s", "liboxq_cpu_avx512.so"], check=True)
    lib = C.CDLL(AVX512_PATH)
    lib.oxq_avx512_gemv_q4_k.restype = C.c_int
    lib.oxq_avx512_gemv_q4_k.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int]
    _avx512 = lib
    return lib


def avx512_gemv_q4_k(w, x, n_rows, n_cols, threads=1):
    lib = load_avx512()
    w = _u8(w)
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(max(n_rows, 1), dtype=np.float32)
    if lib.oxq_avx512_gemv_q4_k(_p(w), _p(x), _p(out), n_rows, n_cols, threads) != 0:
        raise ValueError("partial block")
    return out[:n_rows]


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        build()
    lib = C.CDLL(LIB_PATH)
    vp, sz, u32 = C.c_void_p, C.c_size_t, C.c_uint32
    lib.oxq_ref_block_size.restype = sz
    lib.oxq_ref_block_size.argtypes = [u32]
    lib.oxq_ref_block_bytes.restype = sz
    lib.oxq_ref_block_bytes.argtypes = [u32]
    lib.oxq_ref_f32_to_f16.restype = C.c_uint16
    lib.oxq_ref_f32_to_f16.argtypes = [C.c_float]
    lib.oxq_ref_f16_to_f32.restype = C.c_float
    lib.oxq_ref_f16_to_f32.argtypes = [C.c_uint16]
    for name, args in {
        "oxq_ref_quantize_f32_to_q8_0": [vp, sz, vp],
        "oxq_ref_quantize_f32_to_q4_0": [vp, sz, vp],
        "oxq_ref_dequant_block": [u32, vp, sz, vp, sz],
        "oxq_ref_gemv": [u32, vp, sz, sz, sz, vp, sz, vp, sz],
        "oxq_ref_gemm": [u32, vp, sz, vp, vp, sz, sz, sz],
        "oxq_ref_matvec_q8_fused": [u32, C.c_int, vp, sz, vp, sz, vp, sz, sz, sz],
        "oxq_ref_matvec_q8_intdot": [u32, vp, sz, vp, sz, vp, sz, sz, sz],
        "oxq_ref_block_sums": [u32, vp, sz, vp, sz, vp, sz, sz],
        "oxq_ref_gemm_q8": [u32, C.c_int, vp, sz, vp, vp, sz, sz, sz],
        "oxq_ref_matvec_q8_fused_mt": [u32, C.c_int, vp, sz, vp, sz, vp, sz, sz, sz, C.c_int],
        "oxq_ref_lora_new": [sz, sz, sz, sz, sz],
        "oxq_ref_lora_apply": [vp, vp, sz, C.c_float, sz, sz, vp, sz, vp, sz],
        "oxq_ref_linear_forward": [u32, C.c_int, vp, sz, sz, sz, vp, sz, vp, vp, sz, C.c_float, vp, sz, vp, sz],
        "oxq_ref_expert_forward": [vp, sz, vp, sz, vp, sz, sz, sz, vp, vp],
        "oxq_ref_moe_route": [vp, sz, sz, sz, sz, vp, vp, vp, vp],
        "oxq_ref_moe_forward": [vp, sz, vp, vp, vp, sz, sz, sz, sz, vp, vp],
        "oxq_ref_expert_forward_q": [u32, C.c_int, vp, vp, vp, sz, sz, vp, vp],
        "oxq_ref_moe_forward_q": [u32, C.c_int, vp, sz, vp, vp, vp, sz, sz, sz, sz, vp, vp, vp, vp],
    }.items():
        fn = getattr(lib, name)
        fn.restype = Status
        fn.argtypes = args
    lib.oxq_ref_swiglu_inplace.restype = None
    lib.oxq_ref_swiglu_inplace.argtypes = [vp, vp, sz]
    lib.oxq_ref_moe_accumulate.restype = None
    lib.oxq_ref_moe_accumulate.argtypes = [vp, vp, C.c_float, sz]
    lib.oxq_ref_argmax.restype = C.c_uint32
    lib.oxq_ref_argmax.argtypes = [vp, sz]
    lib.oxq_ref_topk.restype = None
    lib.oxq_ref_topk.argtypes = [vp, sz, sz, vp, vp]
    lib.oxq_ref_logits_edit.restype = None
    lib.oxq_ref_logits_edit.argtypes = [vp, sz, vp, sz, vp, vp, sz, vp, sz, sz, C.c_float]
    lib.oxq_ref_xorshift64_seed.restype = C.c_uint64
    lib.oxq_ref_xorshift64_seed.argtypes = [C.c_uint64]
    lib.oxq_ref_xorshift64_next_f32.restype = C.c_float
    lib.oxq_ref_xorshift64_next_f32.argtypes = [vp]
    lib.oxq_ref_sample_candidates.restype = C.c_uint32
    lib.oxq_ref_sample_candidates.argtypes = [vp, vp, sz, C.c_float, C.c_float, C.c_float, vp, vp, vp]
    lib.oxq_ref_rmsnorm_forward_to.restype = None
    lib.oxq_ref_rmsnorm_forward_to.argtypes = [vp, vp, C.c_float, sz, vp]
    _lib = lib
    return lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def _chk(st):
    if st.code != OK:
        raise OracleError(st)


def _u8(a):
    return np.ascontiguousarray(a).view(np.uint8).ravel()


def groups_per_row(t, n_cols):
    return n_cols // GROUP_COLS[t]


def row_bytes(t, n_cols):
    bs, bb = BLOCK[t]
    return -(-n_cols // bs) * bb


def f32_to_f16(v):
    return load().oxq_ref_f32_to_f16(float(v))


def f16_to_f32(h):
    return load().oxq_ref_f16_to_f32(int(h))


def quantize_q8_0(x):
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.zeros(x.size // 32 * 34 + 34, dtype=np.uint8)
    _chk(load().oxq_ref_quantize_f32_to_q8_0(_p(x), x.size, _p(out)))
    return out[: x.size // 32 * 34]


def quantize_q4_0(x):
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.zeros(x.size // 32 * 18 + 18, dtype=np.uint8)
    _chk(load().oxq_ref_quantize_f32_to_q4_0(_p(x), x.size, _p(out)))
    return out[: x.size // 32 * 18]


def dequant_block(t, block, out_len=None):
    block = _u8(block)
    n = BLOCK[t][0] if out_len is None else out_len
    out = np.zeros(max(n, 1), dtype=np.float32)
    _chk(load().oxq_ref_dequant_block(t, _p(block), block.size, _p(out), n))
    return out[:n]


def dequant_rows(t, w, n_rows, n_cols):
    """Dequantize a whole matrix with dequant_block, block by block."""
    w = _u8(w)
    bs, bb = BLOCK[t]
    bpr = n_cols // bs
    out = np.zeros((n_rows, n_cols), dtype=np.float32)
    for r in range(n_rows):
        for b in range(bpr):
            off = (r * bpr + b) * bb
            out[r, b * bs:(b + 1) * bs] = dequant_block(t, w[off:off + bb])
    return out


def gemv(t, w, n_rows, n_cols, x, y_len=None, x_len=None):
    w = _u8(w)
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    y = np.zeros(max(n_rows if y_len is None else y_len, 1), dtype=np.float32)
    _chk(load().oxq_ref_gemv(t, _p(w), w.size, n_rows, n_cols, _p(x), x.size if x_len is None else x_len,
                             _p(y), n_rows if y_len is None else y_len))
    return y[:n_rows]


def gemm(t, w, x, m, n, k):
    w = _u8(w)
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    y = np.zeros(m * n, dtype=np.float32)
    _chk(load().oxq_ref_gemm(t, _p(w), w.size, _p(x), _p(y), m, n, k))
    return y.reshape(m, n)


def matvec_q8_fused(t, w, acts, n_rows, n_cols, tier=TIER_AVX2, out=None, out_len=None):
    w, acts = _u8(w), _u8(acts)
    if out is None:
        out = np.zeros(max(n_rows, 1), dtype=np.float32)
    _chk(load().oxq_ref_matvec_q8_fused(t, tier, _p(w), w.size, _p(acts), acts.size, _p(out),
                                        out.size if out_len is None else out_len, n_rows, n_cols))
    return out[:n_rows]


def matvec_q8_intdot(t, w, acts, n_rows, n_cols):
    w, acts = _u8(w), _u8(acts)
    out = np.zeros(max(n_rows, 1), dtype=np.float32)
    _chk(load().oxq_ref_matvec_q8_intdot(t, _p(w), w.size, _p(acts), acts.size, _p(out), out.size,
                                         n_rows, n_cols))
    return out[:n_rows]


def matvec_q8_fused_mt(t, w, acts, n_rows, n_cols, threads, tier=TIER_AVX2):
    w, acts = _u8(w), _u8(acts)
    out = np.zeros(max(n_rows, 1), dtype=np.float32)
    _chk(load().oxq_ref_matvec_q8_fused_mt(t, tier, _p(w), w.size, _p(acts), acts.size, _p(out), out.size,
                                           n_rows, n_cols, threads))
    return out[:n_rows]


def block_sums(t, w, acts, n_rows, n_cols):
    w, acts = _u8(w), _u8(acts)
    g = groups_per_row(t, n_cols)
    sums = np.zeros(n_rows * g, dtype=np.int32)
    _chk(load().oxq_ref_block_sums(t, _p(w), w.size, _p(acts), acts.size, _p(sums), n_rows, n_cols))
    return sums.reshape(n_rows, g)


def gemm_q8(t, w, x, m, n, k, tier=TIER_AVX2):
    w = _u8(w)
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    y = np.zeros(m * n, dtype=np.float32)
    _chk(load().oxq_ref_gemm_q8(t, tier, _p(w), w.size, _p(x), _p(y), m, n, k))
    return y.reshape(m, n)


# ---- block builders mirroring the reference tests' make_*_block helpers ----

def f16_bytes(v):
    h = f32_to_f16(v)
    return bytes([h & 0xFF, h >> 8])


def make_q4_0_block(scale, nibbles):  # Q/reference/q4_0.rs:238-244
    assert len(nibbles) == 16
    return f16_bytes(scale) + bytes(nibbles)


def make_q8_0_block(scale, qs):  # Q/reference/q8_0.rs:137-145
    assert len(qs) == 32
    return f16_bytes(scale) + bytes((q & 0xFF) for q in qs)


def make_q4_k_block(d, dmin, scales, qs):  # Q/reference/q4_k.rs:359-366
    assert len(scales) == 12 and len(qs) == 128
    return f16_bytes(d) + f16_bytes(dmin) + bytes(scales) + bytes(qs)


def make_q6k_block(d, ql, qh, scales):  # Q/simd/avx2/q6_k.rs make_q6k_block
    assert len(ql) == 128 and len(qh) == 64 and len(scales) == 16
    return bytes(ql) + bytes(qh) + bytes((s & 0xFF) for s in scales) + f16_bytes(d)


def make_iq4_xs_block(scale, sub_scales, nibbles):  # Q/reference/iq4_xs.rs:211-249
    assert len(sub_scales) == 8 and len(nibbles) == 128
    scales_h, scales_l = 0, [0, 0, 0, 0]
    for i, v in enumerate(sub_scales):
        v &= 0x3F
        low, high = v & 0x0F, (v >> 4) & 0x03
        scales_l[i // 2] |= low if i % 2 == 0 else (low << 4)
        scales_h |= high << (2 * i)
    return f16_bytes(scale) + bytes([scales_h & 0xFF, scales_h >> 8]) + bytes(scales_l) + bytes(nibbles)


# ---- the callers' glue (oracle/oxq_oracle_linear.c) ----

def swiglu(gate, up):
    """silu(gate) * up as swiglu_inplace computes it; returns a new array."""
    g = np.array(gate, dtype=np.float32).ravel().copy()
    u = np.ascontiguousarray(up, dtype=np.float32).ravel()
    assert g.size == u.size
    load().oxq_ref_swiglu_inplace(_p(g), _p(u), g.size)
    return g


def rmsnorm(x, weight, eps):
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    w = np.ascontiguousarray(weight, dtype=np.float32).ravel()
    out = np.zeros(x.size, dtype=np.float32)
    load().oxq_ref_rmsnorm_forward_to(_p(x), _p(w), float(eps), x.size, _p(out))
    return out


def lora_new(a_len, b_len, rank, in_features, out_features):
    _chk(load().oxq_ref_lora_new(a_len, b_len, rank, in_features, out_features))


def lora_apply(a, b, rank, scale, in_features, out_features, x, out):
    """out += b (a x) * scale in place (LoraAdapter::apply); out is a float32 array."""
    a = np.ascontiguousarray(a, dtype=np.float32).ravel()
    b = np.ascontiguousarray(b, dtype=np.float32).ravel()
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    assert out.dtype == np.float32 and out.flags.c_contiguous
    _chk(load().oxq_ref_lora_apply(_p(a), _p(b), rank, float(scale), in_features, out_features, _p(x), x.size,
                                   _p(out), out.size))
    return out


def linear_forward(t, w, n_rows, n_cols, x, bias=None, lora=None, tier=TIER_AVX2, out_len=None):
    """QuantLinear::forward on the Q8_0-activation path; lora = (a, b, rank, scale) or None."""
    w = _u8(w)
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.full(n_rows if out_len is None else out_len, np.float32(7.0), dtype=np.float32)  # overwritten
    bp, bl = (None, 0)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32).ravel()
        bp, bl = _p(bias), bias.size
    ap = bq = None
    rank, scale = 0, 0.0
    if lora is not None:
        la = np.ascontiguousarray(lora[0], dtype=np.float32).ravel()
        lb = np.ascontiguousarray(lora[1], dtype=np.float32).ravel()
        ap, bq, rank, scale = _p(la), _p(lb), int(lora[2]), float(lora[3])
    _chk(load().oxq_ref_linear_forward(t, tier, _p(w), w.size, n_rows, n_cols, bp, bl, ap, bq, rank, scale, _p(x),
                                       x.size, _p(out), out.size))
    return out


# ---- builders for the other formats' blocks, mirroring the make_*_block helpers of the reference's tests ----

def make_q4_1_block(d, m, qs):  # Q/reference/q4_1.rs tests
    return f16_bytes(d) + f16_bytes(m) + bytes(qs)


def make_q5_0_block(d, qh, qs):  # Q/reference/q5_0.rs:248-254
    return f16_bytes(d) + int(qh).to_bytes(4, "little") + bytes(qs)


def make_q5_1_block(d, m, qh, qs):  # Q/reference/q5_1.rs tests
    return f16_bytes(d) + f16_bytes(m) + int(qh).to_bytes(4, "little") + bytes(qs)


def make_q8_1_block(d, qs):  # Q/reference/q8_1.rs tests: s = d * sum(qs) as f16
    return f16_bytes(d) + f16_bytes(float(d) * float(sum(qs))) + bytes(int(q) & 0xFF for q in qs)


def make_iq4_nl_block(scale, nibble_bytes):  # Q/reference/iq4_nl.rs tests
    return f16_bytes(scale) + bytes(nibble_bytes)


def make_q2_k_block(d, dmin, scales, qs):  # Q/reference/q2_k.rs tests
    return bytes(scales) + bytes(qs) + f16_bytes(d) + f16_bytes(dmin)


def make_q3_k_block(d, scales, hmask, qs):  # Q/reference/q3_k.rs tests
    return bytes(hmask) + bytes(qs) + bytes(scales) + f16_bytes(d)


def make_q5_k_block(d, dmin, scales, qh, qs):  # Q/reference/q5_k.rs:362-377
    return f16_bytes(d) + f16_bytes(dmin) + bytes(scales) + bytes(qh) + bytes(qs)


# byte offsets of the f16 fields of each format's block
F16_FIELDS = {Q4_0: (0,), Q8_0: (0,), Q4_K: (0, 2), Q6_K: (208,), IQ4_XS: (0,), Q4_1: (0, 2), Q5_0: (0,), Q5_1: (0, 2),
              Q8_1: (0, 2), Q2_K: (80, 82), Q3_K: (108,), Q5_K: (0, 2), IQ4_NL: (0,)}


def random_blocks(t, seed, n_rows, n_cols, scale=0.02):
    """Valid blocks with every payload bit random: uniform random bytes, f16 fields drawn from
    +-[scale/4, scale] (finite, normal).  Any bytes are a legal block of these formats."""
    rng = np.random.default_rng(seed)
    bs, bb = BLOCK[t]
    n_blocks = n_rows * (n_cols // bs)
    w = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
    for off in F16_FIELDS[t]:
        v = (rng.uniform(scale / 4, scale, n_blocks) * rng.choice([-1.0, 1.0], n_blocks)).astype(np.float16)
        if off in (2, 82) and t in (Q4_K, Q5_K, Q2_K):
            v = np.abs(v)  # dmin is a magnitude in real files
        w[:, off:off + 2] = v.view(np.uint8).reshape(n_blocks, 2)
    return w.reshape(-1)


def argmax(values):
    v = np.ascontiguousarray(values, dtype=np.float32).ravel()
    return int(load().oxq_ref_argmax(_p(v), v.size))


def topk(values, k):
    v = np.ascontiguousarray(values, dtype=np.float32).ravel()
    vals, idx = np.zeros(k, dtype=np.float32), np.zeros(k, dtype=np.uint32)
    load().oxq_ref_topk(_p(v), v.size, k, _p(vals), _p(idx))
    return vals, idx


def logits_edit(logits, banned=(), bias=None, recent=(), window=0, repetition_penalty=1.0):
    """Steps 0 and 1 of the sampler on a copy of the logits: banned tokens, logit bias (dict token -> bias), repetition
    penalty over the last `window` of `recent`."""
    out = np.array(logits, dtype=np.float32).ravel().copy()
    bn = np.ascontiguousarray(banned, dtype=np.uint32)
    bt = np.ascontiguousarray(list((bias or {}).keys()), dtype=np.uint32)
    bv = np.ascontiguousarray(list((bias or {}).values()), dtype=np.float32)
    rc = np.ascontiguousarray(recent, dtype=np.uint32)
    load().oxq_ref_logits_edit(_p(out), out.size, _p(bn), bn.size, _p(bt), _p(bv), bt.size, _p(rc), rc.size, window,
                               repetition_penalty)
    return out


def xorshift64_seed(seed):
    return int(load().oxq_ref_xorshift64_seed(seed))


def xorshift64_next_f32(state):
    """(value in [0, 1), new state)"""
    st = C.c_uint64(state)
    v = load().oxq_ref_xorshift64_next_f32(C.byref(st))
    return float(v), int(st.value)


def sample_candidates(vals, idx, temperature, min_p, top_p, rng_state):
    """The sampler after its candidate list: (token, new rng state, final probabilities, survivors)."""
    v = np.ascontiguousarray(vals, dtype=np.float32).ravel()
    i = np.ascontiguousarray(idx, dtype=np.uint32).ravel()
    probs = np.zeros(v.size, dtype=np.float32)
    st, n_left = C.c_uint64(rng_state), C.c_size_t(0)
    tok = load().oxq_ref_sample_candidates(_p(v), _p(i), v.size, temperature, min_p, top_p, C.byref(st), _p(probs),
                                           C.byref(n_left))
    return int(tok), int(st.value), probs, int(n_left.value)


# ---- mixture-of-experts feed-forward (oracle/oxq_oracle_moe.c) ----

def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32).ravel()


def expert_forward(gate, up, down, hidden, inter, x):
    gate, up, down, x = _f32(gate), _f32(up), _f32(down), _f32(x)
    out = np.zeros(hidden, dtype=np.float32)
    _chk(load().oxq_ref_expert_forward(_p(gate), gate.size, _p(up), up.size, _p(down), down.size, hidden, inter,
                                       _p(x), _p(out)))
    return out


def moe_route(router, n_exp, hidden, top_k, x):
    """-> (experts uint32 [k], weights float32 [k]) with k = min(top_k, n_exp)."""
    router, x = _f32(router), _f32(x)
    sel = np.zeros(max(n_exp, 1), dtype=np.uint32)
    wt = np.zeros(max(n_exp, 1), dtype=np.float32)
    k = C.c_size_t(0)
    _chk(load().oxq_ref_moe_route(_p(router), router.size, n_exp, hidden, top_k, _p(x), _p(sel), _p(wt),
                                  C.cast(C.byref(k), C.c_void_p)))
    return sel[:k.value].copy(), wt[:k.value].copy()


def moe_forward(router, gate_all, up_all, down_all, n_exp, hidden, inter, top_k, x):
    router, x = _f32(router), _f32(x)
    g, u, d = _f32(gate_all), _f32(up_all), _f32(down_all)
    assert g.size == u.size == d.size == n_exp * hidden * inter
    out = np.zeros(hidden, dtype=np.float32)
    _chk(load().oxq_ref_moe_forward(_p(router), router.size, _p(g), _p(u), _p(d), n_exp, hidden, inter, top_k,
                                    _p(x), _p(out)))
    return out


def expert_forward_q(t, gate, up, down, hidden, inter, x_q8, tier=TIER_AVX2):
    gate, up, down, x_q8 = _u8(gate), _u8(up), _u8(down), _u8(x_q8)
    assert gate.size == up.size == row_bytes(t, hidden) * inter and down.size == row_bytes(t, inter) * hidden
    out = np.zeros(hidden, dtype=np.float32)
    _chk(load().oxq_ref_expert_forward_q(t, tier, _p(gate), _p(up), _p(down), hidden, inter, _p(x_q8), _p(out)))
    return out


def moe_forward_q(t, router, gate_all, up_all, down_all, n_exp, hidden, inter, top_k, x, tier=TIER_AVX2):
    """-> (output float32 [hidden], experts uint32 [k], weights float32 [k])."""
    router, x = _f32(router), _f32(x)
    g, u, d = _u8(gate_all), _u8(up_all), _u8(down_all)
    assert g.size == u.size == n_exp * row_bytes(t, hidden) * inter and d.size == n_exp * row_bytes(t, inter) * hidden
    out = np.zeros(hidden, dtype=np.float32)
    k = min(top_k, n_exp)
    sel = np.zeros(max(k, 1), dtype=np.uint32)
    wt = np.zeros(max(k, 1), dtype=np.float32)
    _chk(load().oxq_ref_moe_forward_q(t, tier, _p(router), router.size, _p(g), _p(u), _p(d), n_exp, hidden, inter,
                                      top_k, _p(x), _p(out), _p(sel), _p(wt)))
    return out, sel[:k], wt[:k]
