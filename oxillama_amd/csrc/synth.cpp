// Synthetic GGUF-block weight generator for benchmarks and tests (host only).
//
// Draws fp32 weights from N(0, sigma) with a counter-seeded PRNG and encodes them
// row by row into raw GGUF blocks.  Q4_0 and Q8_0 use the reference's encoders
// (crates/oxillama-quant/src/quantize.rs:154-210).  The reference has no Q4_K,
// Q6_K or IQ4_XS encoder (crates/oxillama-cli/src/quantize.rs:12-14 returns an
// error for them), so those are simple min/max encoders of this build that emit
// valid blocks in the reference's layouts
// (crates/oxillama-quant/src/reference/{q4_k,q6_k,iq4_xs}.rs); kernel parity only
// concerns decode + dot of identical bytes.
//
// Results do not depend on the thread count: every row owns its PRNG stream.
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

namespace {

constexpr uint32_t T_Q4_0 = 2, T_Q8_0 = 8, T_Q4_K = 12, T_Q6_K = 14, T_IQ4_XS = 23;

inline uint64_t splitmix64(uint64_t &s) {
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

struct Xoshiro256 {
    uint64_t s[4];
    explicit Xoshiro256(uint64_t seed) {
        for (auto &v : s) v = splitmix64(seed);
    }
    static inline uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    inline uint64_t next() {
        uint64_t r = rotl(s[1] * 5, 7) * 9, t = s[1] << 17;
        s[2] ^= s[0];
        s[3] ^= s[1];
        s[1] ^= s[2];
        s[0] ^= s[3];
        s[2] ^= t;
        s[3] = rotl(s[3], 45);
        return r;
    }
    inline double uniform() { return (double)((next() >> 11) + 1) * (1.0 / 9007199254740993.0); }
};

// Box-Muller in double, cast to fp32.
void fill_normal(Xoshiro256 &rng, float sigma, float *out, size_t n) {
    size_t i = 0;
    for (; i + 1 < n; i += 2) {
        double u1 = rng.uniform(), u2 = rng.uniform();
        double r = std::sqrt(-2.0 * std::log(u1)), a = 6.283185307179586 * u2;
        out[i] = (float)(r * std::cos(a) * sigma);
        out[i + 1] = (float)(r * std::sin(a) * sigma);
    }
    if (i < n) {
        double u1 = rng.uniform(), u2 = rng.uniform();
        out[i] = (float)(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2) * sigma);
    }
}

// IEEE binary32 -> binary16, round to nearest even.
uint16_t f32_to_f16(float v) {
    uint32_t x;
    std::memcpy(&x, &v, 4);
    uint32_t sign = (x >> 16) & 0x8000u, exp = (x >> 23) & 0xFFu, man = x & 0x7FFFFFu;
    if (exp == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? 0x0200u : 0) | (man >> 13));
    int e = (int)exp - 112;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e), hm = man >> shift, rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13), rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            int e = -1;
            do {
                e++;
                man <<= 1;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline void put_f16(uint8_t *p, float v) {
    uint16_t h = f32_to_f16(v);
    p[0] = (uint8_t)(h & 0xFF);
    p[1] = (uint8_t)(h >> 8);
}

inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// Saturating truncation, as Rust's `f32 as i32`.
inline int trunc_sat(float f) {
    if (f != f) return 0;
    if (f >= 2147483648.0f) return INT32_MAX;
    if (f <= -2147483648.0f) return INT32_MIN;
    return (int)f;
}

// quantize.rs:154-181
void enc_q4_0(const float *x, uint8_t *out) {
    float mx = 0.0f;
    for (int i = 0; i < 32; i++)
        if (std::fabs(x[i]) > std::fabs(mx)) mx = x[i];
    float d = mx / -8.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    put_f16(out, d);
    for (int p = 0; p < 16; p++) {
        int q0 = clampi(trunc_sat(x[2 * p] * id + 8.5f), 0, 15);
        int q1 = clampi(trunc_sat(x[2 * p + 1] * id + 8.5f), 0, 15);
        out[2 + p] = (uint8_t)(q0 | (q1 << 4));
    }
}

// quantize.rs:190-210
void enc_q8_0(const float *x, uint8_t *out) {
    float amax = 0.0f;
    for (int i = 0; i < 32; i++) amax = std::fmax(amax, std::fabs(x[i]));
    float d = amax / 127.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
    put_f16(out, d);
    for (int i = 0; i < 32; i++)
        out[2 + i] = (uint8_t)(int8_t)clampi(trunc_sat(std::round(x[i] * id)), -128, 127);
}

// Min/max Q4_K encoder: w ~ d*sc*q - dmin*mn, layout of reference/q4_k.rs:27-99.
void enc_q4_k(const float *x, uint8_t *out) {
    float scale[8], mins[8], max_scale = 0.0f, max_min = 0.0f;
    for (int s = 0; s < 8; s++) {
        float lo = x[32 * s], hi = x[32 * s];
        for (int i = 1; i < 32; i++) {
            lo = std::fmin(lo, x[32 * s + i]);
            hi = std::fmax(hi, x[32 * s + i]);
        }
        if (lo > 0.0f) lo = 0.0f;
        scale[s] = (hi - lo) / 15.0f;
        mins[s] = -lo;
        max_scale = std::fmax(max_scale, scale[s]);
        max_min = std::fmax(max_min, mins[s]);
    }
    float d = f16_to_f32(f32_to_f16(max_scale / 63.0f));
    float dmin = f16_to_f32(f32_to_f16(max_min / 63.0f));
    put_f16(out, d);
    put_f16(out + 2, dmin);
    uint8_t sc[8], mn[8];
    for (int s = 0; s < 8; s++) {
        sc[s] = (uint8_t)clampi(d > 0.0f ? (int)std::lround(scale[s] / d) : 0, 0, 63);
        mn[s] = (uint8_t)clampi(dmin > 0.0f ? (int)std::lround(mins[s] / dmin) : 0, 0, 63);
    }
    uint8_t *sp = out + 4;
    for (int j = 0; j < 4; j++) {
        sp[j] = (uint8_t)((sc[j] & 0x3F) | ((sc[j + 4] >> 4) << 6));
        sp[j + 4] = (uint8_t)((mn[j] & 0x3F) | ((mn[j + 4] >> 4) << 6));
        sp[j + 8] = (uint8_t)((sc[j + 4] & 0x0F) | ((mn[j + 4] & 0x0F) << 4));
    }
    uint8_t q[256];
    for (int s = 0; s < 8; s++) {
        float ds = d * (float)sc[s], m = dmin * (float)mn[s];
        float ids = ds > 0.0f ? 1.0f / ds : 0.0f;
        for (int i = 0; i < 32; i++)
            q[32 * s + i] = (uint8_t)clampi((int)std::lround((x[32 * s + i] + m) * ids), 0, 15);
    }
    uint8_t *qs = out + 16;
    for (int g = 0; g < 4; g++)
        for (int l = 0; l < 32; l++) qs[32 * g + l] = (uint8_t)(q[64 * g + l] | (q[64 * g + 32 + l] << 4));
}

// Q6_K encoder: w ~ d*sc*(q-32), layout of reference/q6_k.rs:39-72.
void enc_q6_k(const float *x, uint8_t *out) {
    float sub[16], amax_scale = 0.0f;
    for (int s = 0; s < 16; s++) {
        float mx = 0.0f;
        for (int i = 0; i < 16; i++)
            if (std::fabs(x[16 * s + i]) > std::fabs(mx)) mx = x[16 * s + i];
        sub[s] = mx / -32.0f;
        amax_scale = std::fmax(amax_scale, std::fabs(sub[s]));
    }
    float d = f16_to_f32(f32_to_f16(amax_scale / 127.0f));
    int8_t sc[16];
    uint8_t q[256];
    for (int s = 0; s < 16; s++) {
        sc[s] = (int8_t)clampi(d > 0.0f ? (int)std::lround(sub[s] / d) : 0, -128, 127);
        float ds = d * (float)sc[s], ids = ds != 0.0f ? 1.0f / ds : 0.0f;
        for (int i = 0; i < 16; i++)
            q[16 * s + i] = (uint8_t)clampi((int)std::lround(x[16 * s + i] * ids) + 32, 0, 63);
    }
    std::memset(out, 0, 192);
    uint8_t *ql = out, *qh = out + 128;
    for (int h = 0; h < 2; h++) {
        for (int l = 0; l < 32; l++) {
            const uint8_t q1 = q[128 * h + l], q2 = q[128 * h + l + 32], q3 = q[128 * h + l + 64],
                          q4 = q[128 * h + l + 96];
            ql[64 * h + l] = (uint8_t)((q1 & 0x0F) | ((q3 & 0x0F) << 4));
            ql[64 * h + l + 32] = (uint8_t)((q2 & 0x0F) | ((q4 & 0x0F) << 4));
            qh[32 * h + l] = (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
        }
    }
    for (int s = 0; s < 16; s++) out[192 + s] = (uint8_t)sc[s];
    put_f16(out + 208, d);
}

const int8_t KV[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

// IQ4_XS encoder: w ~ d*(ls-32)*KV[idx], layout of reference/iq4_xs.rs:47-97.
void enc_iq4_xs(const float *x, uint8_t *out) {
    float sub[8], amax_scale = 0.0f;
    for (int s = 0; s < 8; s++) {
        float mx = 0.0f;
        for (int i = 0; i < 32; i++)
            if (std::fabs(x[32 * s + i]) > std::fabs(mx)) mx = x[32 * s + i];
        sub[s] = mx / -127.0f;
        amax_scale = std::fmax(amax_scale, std::fabs(sub[s]));
    }
    float d = f16_to_f32(f32_to_f16(amax_scale / 32.0f));
    put_f16(out, d);
    uint16_t scales_h = 0;
    uint8_t scales_l[4] = {0, 0, 0, 0};
    uint8_t *qs = out + 8;
    for (int s = 0; s < 8; s++) {
        int ls = clampi(d > 0.0f ? (int)std::lround(sub[s] / d) : 0, -32, 31);
        uint8_t u = (uint8_t)(ls + 32);
        scales_l[s / 2] |= (uint8_t)((u & 0x0F) << (4 * (s & 1)));
        scales_h |= (uint16_t)((u >> 4) << (2 * s));
        float ds = d * (float)ls, ids = ds != 0.0f ? 1.0f / ds : 0.0f;
        for (int i = 0; i < 16; i++) {
            int idx[2];
            for (int k = 0; k < 2; k++) {
                float t = x[32 * s + 2 * i + k] * ids;
                int best = 0;
                float bd = std::fabs(t - (float)KV[0]);
                for (int c = 1; c < 16; c++) {
                    float dd = std::fabs(t - (float)KV[c]);
                    if (dd < bd) {
                        bd = dd;
                        best = c;
                    }
                }
                idx[k] = best;
            }
            qs[16 * s + i] = (uint8_t)(idx[0] | (idx[1] << 4));
        }
    }
    out[2] = (uint8_t)(scales_h & 0xFF);
    out[3] = (uint8_t)(scales_h >> 8);
    std::memcpy(out + 4, scales_l, 4);
}

bool type_info(uint32_t type, size_t &bs, size_t &bb) {
    switch (type) {
    case T_Q4_0: bs = 32; bb = 18; return true;
    case T_Q8_0: bs = 32; bb = 34; return true;
    case T_Q4_K: bs = 256; bb = 144; return true;
    case T_Q6_K: bs = 256; bb = 210; return true;
    case T_IQ4_XS: bs = 256; bb = 136; return true;
    default: return false;
    }
}

void encode_row(uint32_t type, const float *x, size_t n_cols, uint8_t *out) {
    size_t bs = 0, bb = 0;
    type_info(type, bs, bb);
    for (size_t b = 0; b < n_cols / bs; b++) {
        const float *xb = x + b * bs;
        uint8_t *ob = out + b * bb;
        switch (type) {
        case T_Q4_0: enc_q4_0(xb, ob); break;
        case T_Q8_0: enc_q8_0(xb, ob); break;
        case T_Q4_K: enc_q4_k(xb, ob); break;
        case T_Q6_K: enc_q6_k(xb, ob); break;
        default: enc_iq4_xs(xb, ob); break;
        }
    }
}

}  // namespace

extern "C" {

// x ~ N(0, sigma), stream `seed`.
int oxq_synth_normal_f32(uint64_t seed, float sigma, float *out, size_t n) {
    Xoshiro256 rng(seed);
    fill_normal(rng, sigma, out, n);
    return 0;
}

// Encode caller-supplied fp32 rows [n_rows x n_cols] into GGUF blocks.
// Returns 0, or -1 for an unknown type / n_cols not a block multiple / short buffer.
int oxq_synth_encode(uint32_t type, const float *x, size_t n_rows, size_t n_cols, uint8_t *out,
                     size_t out_len) {
    size_t bs = 0, bb = 0;
    if (!type_info(type, bs, bb) || n_cols % bs != 0) return -1;
    size_t row_bytes = n_cols / bs * bb;
    if (out_len < n_rows * row_bytes) return -1;
    for (size_t r = 0; r < n_rows; r++) encode_row(type, x + r * n_cols, n_cols, out + r * row_bytes);
    return 0;
}

// Weights ~ N(0, sigma), row r drawn from stream (seed, r); encoded in place.
int oxq_synth_weights(uint32_t type, uint64_t seed, float sigma, size_t n_rows, size_t n_cols,
                      uint8_t *out, size_t out_len, int n_threads) {
    size_t bs = 0, bb = 0;
    if (!type_info(type, bs, bb) || n_cols % bs != 0) return -1;
    size_t row_bytes = n_cols / bs * bb;
    if (out_len < n_rows * row_bytes) return -1;
    if (n_threads < 1) n_threads = 1;
    if (n_threads > 64) n_threads = 64;
    auto work = [&](int t) {
        std::vector<float> row(n_cols);
        for (size_t r = (size_t)t; r < n_rows; r += (size_t)n_threads) {
            uint64_t s = seed * 0x9E3779B97F4A7C15ull + r;
            Xoshiro256 rng(splitmix64(s) ^ (r << 1));
            fill_normal(rng, sigma, row.data(), n_cols);
            encode_row(type, row.data(), n_cols, out + r * row_bytes);
        }
    };
    std::vector<std::thread> th;
    for (int t = 1; t < n_threads; t++) th.emplace_back(work, t);
    work(0);
    for (auto &t : th) t.join();
    return 0;
}

}  // extern "C"
