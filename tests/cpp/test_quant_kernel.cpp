// Replays the reference crate's own unit tests against the C++ mirror of its
// interface (include/oxq/quant_kernel.hpp), which calls liboxq_hip.so through the C ABI.
// Each case names the reference test it follows (Q/ = crates/oxillama-quant/src).
//
//   test_quant_kernel --host   metadata, error variants and validation order (no GPU work)
//   test_quant_kernel --gpu    the numeric cases (needs an MI355X)
//
// Exit status 0 = all passed.  `gemv`/`gemm` of this library quantize the f32 input to
// Q8_0 first, so their closed-form expectations hold to the Q8_0 rounding of the input
// (|rel err| <= 2e-3 here) instead of exactly; dequant and fused cases keep the
// reference's own tolerances.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "oxq/gguf_model.hpp"
#include "oxq/moe_ffn.hpp"
#include "oxq/quant_kernel.hpp"

using namespace oxq;

static int g_failed = 0, g_run = 0;
#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            std::printf("    CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #cond);  \
            ++g_failed;                                                              \
            return;                                                                  \
        }                                                                            \
    } while (0)
#define CHECK_NEAR(a, b, tol)                                                                        \
    do {                                                                                             \
        const double va = (a), vb = (b);                                                             \
        if (!(std::fabs(va - vb) <= (tol))) {                                                        \
            std::printf("    CHECK_NEAR failed %s:%d: %s = %.9g vs %s = %.9g (tol %g)\n", __FILE__,  \
                        __LINE__, #a, va, #b, vb, (double)(tol));                                    \
            ++g_failed;                                                                              \
            return;                                                                                  \
        }                                                                                            \
    } while (0)

static void run(const char *name, const std::function<void()> &fn) {
    const int before = g_failed;
    std::printf("test %s ... ", name);
    std::fflush(stdout);
    fn();
    ++g_run;
    std::printf("%s\n", g_failed == before ? "ok" : "FAILED");
    std::fflush(stdout);
}

// ---- block builders (little-endian f16 scale + payload) ------------------------------
static uint16_t f16_bits(float f) {  // exact for the scales used here (0.5, 0.25, 1, 2, 0.1 -> RNE)
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    int32_t e = (int32_t)((x >> 23) & 0xFF) - 127 + 15;
    uint32_t m = x & 0x7FFFFFu;
    if ((x & 0x7FFFFFFFu) == 0) return (uint16_t)sign;
    if (e <= 0 || e >= 31) return (uint16_t)(sign | 0x7C00u);  // not needed by these tests
    uint32_t h = (uint32_t)(e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
    return (uint16_t)(sign | h);
}
static float f16_value(uint16_t h) {
    const int e = (h >> 10) & 31, m = h & 1023;
    const float v = e == 0 ? std::ldexp((float)m, -24) : std::ldexp((float)(m + 1024), e - 25);
    return (h & 0x8000) ? -v : v;
}
static void put_f16(std::vector<uint8_t> &b, size_t at, float f) {
    const uint16_t h = f16_bits(f);
    b[at] = (uint8_t)(h & 0xFF);
    b[at + 1] = (uint8_t)(h >> 8);
}
static std::vector<uint8_t> q4_0_block(float d, const std::vector<uint8_t> &nib16) {
    std::vector<uint8_t> b(18, 0);
    put_f16(b, 0, d);
    for (int i = 0; i < 16; ++i) b[2 + i] = nib16[i];
    return b;
}
static std::vector<uint8_t> q8_0_block(float d, const std::vector<int> &q32) {
    std::vector<uint8_t> b(34, 0);
    put_f16(b, 0, d);
    for (int i = 0; i < 32; ++i) b[2 + i] = (uint8_t)(int8_t)q32[i];
    return b;
}
static std::vector<uint8_t> q4_k_block(float d, float dmin, const std::vector<uint8_t> &scales12, uint8_t qs_fill) {
    std::vector<uint8_t> b(144, 0);
    put_f16(b, 0, d);
    put_f16(b, 2, dmin);
    for (int i = 0; i < 12; ++i) b[4 + i] = scales12[i];
    for (int i = 0; i < 128; ++i) b[16 + i] = qs_fill;
    return b;
}
static void append(std::vector<uint8_t> &dst, const std::vector<uint8_t> &src) {
    dst.insert(dst.end(), src.begin(), src.end());
}
// Dequantized Q8_0 activations: q * d_a (the "unfused" operand of the reference's comparisons).
static std::vector<float> dequant_acts(const std::vector<uint8_t> &acts) {
    std::vector<float> x;
    for (size_t b = 0; b + 34 <= acts.size(); b += 34) {
        const float d = f16_value((uint16_t)(acts[b] | (acts[b + 1] << 8)));
        for (int i = 0; i < 32; ++i) x.push_back((float)(int8_t)acts[b + 2 + i] * d);
    }
    return x;
}
// Unfused expectation as the reference's tests build it: dequant_block each weight block, dot in f32.
static float unfused_row(const QuantKernel &k, const uint8_t *row, size_t n_cols, const std::vector<float> &x) {
    const size_t bs = k.block_size(), bb = k.block_bytes();
    std::vector<float> w(bs);
    float sum = 0.0f;
    for (size_t b = 0; b < n_cols / bs; ++b) {
        if (!k.dequant_block(Slice<const uint8_t>(row + b * bb, bb), w)) return NAN;
        for (size_t i = 0; i < bs; ++i) sum += w[i] * x[b * bs + i];
    }
    return sum;
}

static const std::vector<int> Q8_ALT16 = {1, -2, 3, -4, 5, -6, 7, -8, 9, -10, 11, -12, 13, -14, 15, -16,
                                          -1, 2, -3, 4, -5, 6, -7, 8, -9, 10, -11, 12, -13, 14, -15, 16};
static const std::vector<uint8_t> NIB_A = {0x5A, 0xF0, 0x13, 0x7E, 0xC2, 0x48, 0x9D, 0x6B,
                                           0xA3, 0x2F, 0x71, 0xE4, 0x0C, 0x58, 0xB6, 0xD9};

// All-ones experts as the reference's make_expert (moe.rs:266-274), held as Q8_0 blocks (d = 1, q = 1).
static MoeFfn ones_moe(size_t h, size_t n, size_t n_exp, size_t top_k, float router_fill = 1.0f) {
    auto ones = [](size_t rows, size_t cols) {
        std::vector<uint8_t> w;
        const std::vector<uint8_t> blk = q8_0_block(1.0f, std::vector<int>(32, 1));
        for (size_t i = 0; i < rows * cols / 32; ++i) append(w, blk);
        return QuantTensor(std::move(w), {rows, cols}, GgufTensorType::Q8_0);
    };
    MoeFfn moe;
    moe.router.assign(n_exp * h, router_fill);
    for (size_t e = 0; e < n_exp; ++e) moe.experts.push_back(QuantExpert{ones(n, h), ones(n, h), ones(h, n)});
    moe.top_k = top_k;
    moe.num_experts = n_exp;
    moe.hidden_size = h;
    moe.intermediate_size = n;
    return moe;
}

// ======================================================================================
//  host-only cases
// ======================================================================================
static void host_tests() {
    KernelDispatcher dispatcher;  // may have no device here; metadata and validation still work

    run("block_info_matches_gguf_tables (gguf/src/types.rs:199-262)", [&] {
        struct { GgufTensorType t; size_t bs, bb; } rows[] = {{GgufTensorType::Q4_0, 32, 18},
                                                              {GgufTensorType::Q8_0, 32, 34},
                                                              {GgufTensorType::Q4K, 256, 144},
                                                              {GgufTensorType::Q6K, 256, 210},
                                                              {GgufTensorType::Iq4Xs, 256, 136}};
        for (auto &r : rows) {
            HipKernel k(r.t);
            CHECK(k.block_size() == r.bs);
            CHECK(k.block_bytes() == r.bb);
            CHECK(k.name() != nullptr && std::strlen(k.name()) > 0);
        }
    });

    run("dispatcher_unknown_type_is_unsupported (Q/dispatch.rs:236-242)", [&] {
        std::unique_ptr<QuantKernel> k;
        const QuantResult r = dispatcher.get_kernel(999u, k);
        CHECK(r.is_err());
        CHECK(r.error().kind == QuantError::UnsupportedType);
        CHECK(!k);
        CHECK(dispatcher.get_kernel(GgufTensorType::Q4K, k).is_ok());
        CHECK(k && k->block_size() == 256);
    });

    run("quant_tensor_bookkeeping (Q/types.rs:30-50)", [&] {
        QuantTensor t(std::vector<uint8_t>(4 * 144), {2, 512}, GgufTensorType::Q4K);
        CHECK(t.n_elements() == 1024);
        CHECK(t.n_blocks() == 4);
        CHECK(t.expected_data_size() == 4 * 144);
        QuantTensor e({}, {}, GgufTensorType::Q8_0);
        CHECK(e.n_elements() == 0 && e.n_blocks() == 0);
    });

    run("quantize_q8_0_rejects_unaligned_length (Q/quantize.rs:59-64,307-317)", [&] {
        std::vector<float> x(33, 1.0f);
        std::vector<uint8_t> out;
        const QuantResult r = quantize_f32_to_q8_0(x, out);
        CHECK(r.is_err());
        CHECK(r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 64 && r.error().got == 33);
        CHECK(r.error().to_string() == "dimension mismatch: expected 64, got 33");
    });

    run("fused_validation_order: out, weights, acts (Q/reference/q4_k.rs:226-250)", [&] {
        HipKernel k(GgufTensorType::Q4K);
        std::vector<uint8_t> w(2 * 144), a(8 * 34);
        std::vector<float> out(2);
        // everything too small: the output check fires first
        QuantResult r = k.matvec_q8_fused(Slice<const uint8_t>(w.data(), 10), Slice<const uint8_t>(a.data(), 10),
                                          Slice<float>(out.data(), 1), 2, 256);
        CHECK(r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 2 && r.error().got == 1);
        // output fine: weights next
        r = k.matvec_q8_fused(Slice<const uint8_t>(w.data(), 287), Slice<const uint8_t>(a.data(), 10), out, 2, 256);
        CHECK(r.error().kind == QuantError::BufferTooSmall);
        CHECK(r.error().expected == 288 && r.error().got == 287);
        // then activations: 8 Q8_0 blocks per super-block
        r = k.matvec_q8_fused(w, Slice<const uint8_t>(a.data(), 271), out, 2, 256);
        CHECK(r.error().kind == QuantError::BufferTooSmall);
        CHECK(r.error().expected == 272 && r.error().got == 271);
        CHECK(r.error().to_string() == "buffer too small: need 272 bytes, have 271");
    });

    run("gemv_dimension_checks: input then output (Q/reference/q4_k.rs:117-128)", [&] {
        HipKernel k(GgufTensorType::Q8_0);
        QuantTensor t(std::vector<uint8_t>(2 * 34), {2, 32}, GgufTensorType::Q8_0);
        std::vector<float> x(31), y(1);
        QuantResult r = k.gemv(t, x, y);
        CHECK(r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 32 && r.error().got == 31);
        x.resize(32);
        r = k.gemv(t, x, y);
        CHECK(r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 2 && r.error().got == 1);
    });

    run("dequant_block_buffer_checks (Q/reference/q4_k.rs:53-64)", [&] {
        HipKernel k(GgufTensorType::Q6K);
        std::vector<uint8_t> b(209);
        std::vector<float> o(256);
        QuantResult r = k.dequant_block(b, o);
        CHECK(r.error().kind == QuantError::BufferTooSmall);
        CHECK(r.error().expected == 210 && r.error().got == 209);
        b.resize(210);
        o.resize(255);
        r = k.dequant_block(b, o);
        CHECK(r.error().kind == QuantError::BufferTooSmall);
        CHECK(r.error().expected == 256 && r.error().got == 255);
    });

    run("lora new: dimension mismatches (lora.rs:203-227)", [&] {
        std::shared_ptr<LoraAdapter> l;
        QuantResult r = LoraAdapter::create({1.0f}, {1.0f, 0.0f, 0.0f, 1.0f}, 2, 1.0f, 1, 2, l);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 2 && r.error().got == 1);
        r = LoraAdapter::create({1.0f, 0.0f}, {1.0f}, 1, 1.0f, 2, 2, l);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 2 && r.error().got == 1);
        CHECK(LoraAdapter::create({1, 0, 0, 1}, {1, 0, 0, 1}, 2, 1.0f, 2, 2, l).is_ok() && l && l->rank == 2);
    });

    run("quant linear: new has no lora; short input / output are dimension errors (linear.rs:265-270, q4_k.rs:117-128)", [&] {
        std::vector<uint8_t> w;
        for (int r = 0; r < 32; ++r) {
            std::vector<int> q(32, 0);
            q[r] = 1;
            append(w, q8_0_block(1.0f, q));
        }
        QuantLinear lin(QuantTensor(w, {32, 32}, GgufTensorType::Q8_0));
        CHECK(!lin.lora && lin.out_features == 32 && lin.in_features == 32);
        HipKernel k(GgufTensorType::Q8_0);
        std::vector<float> x(31, 0.0f), y(32, 0.0f);
        QuantResult r = lin.forward(k, x, y);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch && r.error().expected == 32 && r.error().got == 31);
        x.resize(32);
        y.resize(31);
        r = lin.forward(k, x, y);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch && r.error().expected == 32 && r.error().got == 31);
    });

    // ---- GGUF reader: the file images of crates/oxillama-gguf/src/parser.rs tests, byte for byte ----
    auto put32 = [](std::vector<uint8_t> &b, uint32_t v) { for (int i = 0; i < 4; ++i) b.push_back((uint8_t)(v >> (8 * i))); };
    auto put64 = [](std::vector<uint8_t> &b, uint64_t v) { for (int i = 0; i < 8; ++i) b.push_back((uint8_t)(v >> (8 * i))); };
    auto put_str = [&](std::vector<uint8_t> &b, const std::string &s) { put64(b, s.size()); b.insert(b.end(), s.begin(), s.end()); };
    auto build_test_gguf = [&] {  // parser.rs:232-270
        std::vector<uint8_t> d;
        put32(d, 0x46554747u); put32(d, 3); put64(d, 1); put64(d, 2);
        put_str(d, "general.architecture"); put32(d, 8); put_str(d, "llama");
        put_str(d, "llama.block_count"); put32(d, 4); put32(d, 32);
        put_str(d, "output.weight"); put32(d, 2); put64(d, 32); put64(d, 32); put32(d, 2); put64(d, 0);
        d.resize((d.size() + 31) / 32 * 32, 0);
        d.resize(d.size() + 1024, 0xAB);
        return d;
    };

    run("gguf parse_full_gguf, tensor_data_access, missing_tensor (parser.rs:277-307)", [&] {
        GgufModel m;
        CHECK(m.from_bytes(build_test_gguf()) == OXQ_OK);
        CHECK(m.header().version == 3 && m.header().tensor_count == 1 && m.header().metadata_kv_count == 2);
        std::string arch;
        uint64_t blocks = 0;
        CHECK(m.architecture(arch) == OXQ_OK && arch == "llama");
        CHECK(m.get_u64("llama.block_count", blocks) == OXQ_OK && blocks == 32);
        TensorInfo t;
        CHECK(m.tensor("output.weight", t) == OXQ_OK);
        CHECK(t.n_dims == 2 && t.dimensions == std::vector<uint64_t>({32, 32}) && t.tensor_type == 2);
        CHECK(t.n_elements() == 1024 && t.data_size() == 576);
        const uint8_t *p = nullptr;
        size_t n = 0;
        CHECK(m.tensor_data("output.weight", p, n) == OXQ_OK && n == 576 && p[0] == 0xAB && p[575] == 0xAB);
        CHECK(m.tensor_data("nonexistent", p, n) == OXQ_ERR_GGUF_TENSOR_NOT_FOUND);
    });

    run("gguf header errors: magic, version, truncation (header.rs:121-167, loader.rs tests)", [&] {
        GgufModel m;
        size_t a = 0, b = 0;
        CHECK(m.from_bytes({0, 0, 0, 0, 3, 0, 0, 0}) == OXQ_ERR_GGUF_INVALID_MAGIC);
        oxq_last_error(&a, &b, nullptr, 0);
        CHECK(a == 0);
        std::vector<uint8_t> v0;
        put32(v0, 0x46554747u); put32(v0, 0); put32(v0, 0); put32(v0, 0);
        CHECK(m.from_bytes(v0) == OXQ_ERR_GGUF_UNSUPPORTED_VERSION);
        CHECK(m.from_bytes({'G', 'G', 'U', 'F'}) == OXQ_ERR_GGUF_UNEXPECTED_EOF);
        CHECK(m.load("/nonexistent/path/does_not_exist.gguf") == OXQ_ERR_GGUF_IO);
    });

    // ---- MoeFfn (crates/oxillama-arch/src/common/moe.rs tests) -------------------------------
    run("moe top_k = 0 is an error (moe.rs:403-424); router and expert sizes are checked first (moe.rs:426-450, 307-322)", [&] {
        MoeFfn moe = ones_moe(256, 256, 2, 0);
        std::vector<float> x(256, 1.0f), y(256, 0.0f);
        QuantResult r = moe.forward(x, y);
        CHECK(!r.is_ok() && r.error().kind == QuantError::KernelError);
        moe.top_k = 1;
        moe.router.resize(5);  // wrong router size
        r = moe.forward(x, y);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 512 && r.error().got == 5);
        moe = ones_moe(256, 256, 2, 1);
        moe.experts.pop_back();  // experts.len() != num_experts
        r = moe.forward(x, y);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch && r.error().expected == 2 && r.error().got == 1);
        moe = ones_moe(256, 256, 2, 1);
        moe.experts[1].gate.data.resize(3);  // expert.gate of the wrong size
        r = moe.forward(x, y);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch);
        CHECK(r.error().expected == 2 * 256 * 8 * 34 && r.error().got == 256 * 8 * 34 + 3);
        moe = ones_moe(256, 256, 2, 1);
        std::vector<float> short_x(100, 1.0f);
        r = moe.forward(short_x, y);
        CHECK(!r.is_ok() && r.error().kind == QuantError::DimensionMismatch && r.error().expected == 256 && r.error().got == 100);
    });
}

// ======================================================================================
//  GPU cases
// ======================================================================================
static void gpu_tests() {
    KernelDispatcher dispatcher;
    if (!dispatcher.has_device()) {
        std::printf("no usable GPU: oxq_init failed\n");
        ++g_failed;
        return;
    }
    auto kernel = [&](GgufTensorType t) {
        std::unique_ptr<QuantKernel> k;
        dispatcher.get_kernel(t, k);
        return k;
    };

    run("q4_0 dequant_known_values (Q/reference/q4_0.rs:259-270)", [&] {
        auto k = kernel(GgufTensorType::Q4_0);
        std::vector<uint8_t> nib(16, 0x88);
        nib[0] = 0xF0;
        auto b = q4_0_block(0.5f, nib);
        std::vector<float> w(32, 99.0f);
        CHECK(k->dequant_block(b, w).is_ok());
        CHECK(w[0] == -4.0f);  // (0 - 8) * 0.5
        CHECK(w[1] == 3.5f);   // (15 - 8) * 0.5
        for (int i = 2; i < 32; ++i) CHECK(w[i] == 0.0f);
    });

    run("q8_0 dequant_known_values (Q/reference/q8_0.rs:159-172)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        std::vector<int> q(32, 0);
        q[0] = 10; q[1] = -5; q[31] = 127;
        auto b = q8_0_block(0.5f, q);
        std::vector<float> w(32);
        CHECK(k->dequant_block(b, w).is_ok());
        CHECK(w[0] == 5.0f && w[1] == -2.5f && w[31] == 63.5f);
    });

    run("q8_0 gemv_simple 1*2.0*3.0 (Q/reference/q8_0.rs:175-190)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        std::vector<int> q(32, 0);
        q[0] = 1;
        QuantTensor t(q8_0_block(2.0f, q), {1, 32}, GgufTensorType::Q8_0);
        std::vector<float> x(32, 0.0f), y(1, -1.0f);
        x[0] = 3.0f;
        CHECK(k->gemv(t, x, y).is_ok());
        CHECK_NEAR(y[0], 6.0, 6.0 * 2e-3);
    });

    run("q8_0 gemm two rows 4*0.5*3 (Q/reference/q8_0.rs:216-232)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        std::vector<int> q(32, 0);
        q[0] = 4;
        QuantTensor t(q8_0_block(0.5f, q), {1, 32}, GgufTensorType::Q8_0);
        std::vector<float> x(64, 0.0f), y(2, -1.0f);
        x[0] = 3.0f;
        x[32] = -3.0f;
        CHECK(k->gemm(t, x, y, 2, 1, 32).is_ok());
        CHECK_NEAR(y[0], 6.0, 6.0 * 2e-3);
        CHECK_NEAR(y[1], -6.0, 6.0 * 2e-3);
    });

    run("q4_k dequant all 8.0 (Q/reference/q4_k.rs:381-408)", [&] {
        auto k = kernel(GgufTensorType::Q4K);
        auto b = q4_k_block(1.0f, 0.0f, {1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1}, 0x88);
        std::vector<float> w(256);
        CHECK(k->dequant_block(b, w).is_ok());
        for (float v : w) CHECK(v == 8.0f);
    });

    run("q4_k gemv ones = 256 (Q/reference/q4_k.rs:411-436)", [&] {
        auto k = kernel(GgufTensorType::Q4K);
        QuantTensor t(q4_k_block(1.0f, 0.0f, {1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1}, 0x11), {1, 256},
                      GgufTensorType::Q4K);
        std::vector<float> x(256, 1.0f), y(1);
        CHECK(k->gemv(t, x, y).is_ok());
        CHECK_NEAR(y[0], 256.0, 256.0 * 2e-3);
    });

    run("q6_k zero block and qh=0xAA (Q/reference/q6_k.rs:369-414)", [&] {
        auto k = kernel(GgufTensorType::Q6K);
        std::vector<uint8_t> b(210, 0);
        std::vector<float> w(256, 1.0f);
        CHECK(k->dequant_block(b, w).is_ok());
        for (float v : w) CHECK(v == 0.0f);
        for (int i = 0; i < 64; ++i) b[128 + i] = 0xAA;  // every q6 = 32 -> q - 32 = 0
        for (int i = 0; i < 16; ++i) b[192 + i] = 1;
        put_f16(b, 208, 1.0f);
        CHECK(k->dequant_block(b, w).is_ok());
        for (float v : w) CHECK(v == 0.0f);
    });

    run("iq4_xs ls=33, qs=0x88: first 32 weights 1.0 (Q/reference/iq4_xs.rs:266-285)", [&] {
        auto k = kernel(GgufTensorType::Iq4Xs);
        std::vector<uint8_t> b(136, 0);
        put_f16(b, 0, 1.0f);
        // sub-block 0: ls = 33 -> low nibble 1 in scales_l[0], high bits 2 in scales_h bits 0..1;
        // every other sub-block: ls = 32 (low 0, high 2) -> scale 0
        uint16_t sh = 0;
        for (int i = 0; i < 8; ++i) sh |= (uint16_t)(2u << (2 * i));
        b[2] = (uint8_t)(sh & 0xFF);
        b[3] = (uint8_t)(sh >> 8);
        b[4] = 0x01;
        for (int i = 0; i < 128; ++i) b[8 + i] = 0x88;  // kvalues[8] = 1
        std::vector<float> w(256);
        CHECK(k->dequant_block(b, w).is_ok());
        for (int i = 0; i < 32; ++i) CHECK(w[i] == 1.0f);
        for (int i = 32; i < 256; ++i) CHECK(w[i] == 0.0f);
    });

    run("q4_0 fused accumulates: preset 42 survives zero acts (Q/reference/q4_0.rs:382-420)", [&] {
        auto k = kernel(GgufTensorType::Q4_0);
        auto w = q4_0_block(0.25f, NIB_A);
        auto a = q8_0_block(0.5f, std::vector<int>(32, 0));
        std::vector<float> out(1, 42.0f);
        CHECK(k->matvec_q8_fused(w, a, out, 1, 32).is_ok());
        CHECK(out[0] == 42.0f);
    });

    run("q4_k fused accumulates: preset 77 (Q/reference/q4_k.rs:474-493)", [&] {
        auto k = kernel(GgufTensorType::Q4K);
        auto w = q4_k_block(1.0f, 0.0f, {1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1}, 0x11);
        std::vector<uint8_t> a;
        for (int i = 0; i < 8; ++i) append(a, q8_0_block(0.5f, std::vector<int>(32, 0)));
        std::vector<float> out(1, 77.0f);
        CHECK(k->matvec_q8_fused(w, a, out, 1, 256).is_ok());
        CHECK(out[0] == 77.0f);
    });

    run("q4_0 fused matches unfused, single block (Q/reference/q4_0.rs:423-464)", [&] {
        auto k = kernel(GgufTensorType::Q4_0);
        auto w = q4_0_block(0.25f, NIB_A);
        auto a = q8_0_block(0.5f, Q8_ALT16);
        std::vector<float> out(1, 0.0f);
        CHECK(k->matvec_q8_fused(w, a, out, 1, 32).is_ok());
        CHECK_NEAR(out[0], unfused_row(*k, w.data(), 32, dequant_acts(a)), 1e-3);
    });

    run("q4_k fused matches unfused, mixed scales (Q/reference/q4_k.rs:496-559)", [&] {
        auto k = kernel(GgufTensorType::Q4K);
        auto w = q4_k_block(0.5f, 0.1f, {5, 3, 7, 2, 4, 6, 1, 3, 9, 11, 13, 15}, 0xA5);
        std::vector<uint8_t> a;
        for (int i = 0; i < 8; ++i) append(a, q8_0_block(0.25f, Q8_ALT16));
        std::vector<float> out(1, 0.0f);
        CHECK(k->matvec_q8_fused(w, a, out, 1, 256).is_ok());
        const float want = unfused_row(*k, w.data(), 256, dequant_acts(a));
        CHECK_NEAR(out[0], want, 1e-3 * std::fmax(1.0, std::fabs(want)));
    });

    run("q4_k fused multi-row matches unfused (Q/reference/q4_k.rs:562-625)", [&] {
        auto k = kernel(GgufTensorType::Q4K);
        std::vector<uint8_t> w, a;
        for (float s : {0.5f, 1.0f, 0.25f, 0.1f}) append(w, q4_k_block(s, 0.0f, {1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1}, 0x55));
        const std::vector<int> q = {2, -1, 4, -3, 6, -5, 8, -7, 1, -2, 3, -4, 5, -6, 7, -8,
                                    -2, 1, -4, 3, -6, 5, -8, 7, -1, 2, -3, 4, -5, 6, -7, 8};
        for (int i = 0; i < 8; ++i) append(a, q8_0_block(0.5f, q));
        std::vector<float> out(4, 0.0f);
        CHECK(k->matvec_q8_fused(w, a, out, 4, 256).is_ok());
        const auto x = dequant_acts(a);
        for (int r = 0; r < 4; ++r) CHECK_NEAR(out[r], unfused_row(*k, w.data() + r * 144, 256, x), 1e-3);
    });

    run("q6_k fused matches unfused on the pattern block (Q/simd/avx2/q6_k.rs:939-980)", [&] {
        auto k = kernel(GgufTensorType::Q6K);
        std::vector<uint8_t> w(210);
        for (int i = 0; i < 128; ++i) w[i] = (uint8_t)((i * 5 + 11) & 0xFF);
        for (int i = 0; i < 64; ++i) w[128 + i] = (uint8_t)((i * 13 + 7) & 0xFF);
        for (int i = 0; i < 16; ++i) w[192 + i] = (uint8_t)(i + 1);
        put_f16(w, 208, 0.01f);
        const std::vector<int> q = {1, -2, 3, -4, 5, -6, 7, -8, 9, -10, 11, -12, 13, -14, 15, -16,
                                    0, 1, -1, 2, -2, 3, -3, 4, -4, 5, -5, 6, -6, 7, -7, 8};
        std::vector<uint8_t> a;
        for (int i = 0; i < 8; ++i) append(a, q8_0_block(0.1f, q));
        std::vector<float> out(1, 0.0f);
        CHECK(k->matvec_q8_fused(w, a, out, 1, 256).is_ok());
        CHECK_NEAR(out[0], unfused_row(*k, w.data(), 256, dequant_acts(a)), 1e-3);
    });

    run("quantize_q8_0: max maps to +-127, zero block (Q/quantize.rs:320-379)", [&] {
        std::vector<float> x(64, 0.0f);
        for (int i = 0; i < 32; ++i) x[i] = (float)(i - 16) * 0.25f;  // extreme = -4.0 at i = 0
        std::vector<uint8_t> out;
        CHECK(quantize_f32_to_q8_0(x, out).is_ok());
        CHECK(out.size() == 68);
        CHECK((int8_t)out[2] == -127);
        for (int i = 0; i < 34; ++i) CHECK(out[34 + i] == 0);  // all-zero block: d = 0, q = 0
    });

    // The reference's own gemv / gemm known answers at the reference's own exactness: OXQ_ROUTE_F32 runs its fp32
    // arithmetic, so the closed forms hold exactly (every term is exactly representable in these cases).
    run("route F32: q8_0 gemv_simple == 6.0, gemm rows == +-6.0, q4_k ones == 256.0, exactly", [&] {
        CHECK(KernelDispatcher::select_activation_route(ActivationRoute::F32).is_ok());
        CHECK(KernelDispatcher::activation_route() == ActivationRoute::F32);
        bool ok = true;
        {
            auto k = kernel(GgufTensorType::Q8_0);
            std::vector<int> q(32, 0);
            q[0] = 1;
            QuantTensor t(q8_0_block(2.0f, q), {1, 32}, GgufTensorType::Q8_0);
            std::vector<float> x(32, 0.0f), y(1, -1.0f);
            x[0] = 3.0f;
            ok = ok && k->gemv(t, x, y).is_ok() && y[0] == 6.0f;  // Q/reference/q8_0.rs:175-190
            q[0] = 4;
            QuantTensor t2(q8_0_block(0.5f, q), {1, 32}, GgufTensorType::Q8_0);
            std::vector<float> x2(64, 0.0f), y2(2, -1.0f);
            x2[0] = 3.0f;
            x2[32] = -3.0f;
            ok = ok && k->gemm(t2, x2, y2, 2, 1, 32).is_ok() && y2[0] == 6.0f && y2[1] == -6.0f;  // q8_0.rs:216-232
        }
        {
            auto k = kernel(GgufTensorType::Q4K);
            QuantTensor t(q4_k_block(1.0f, 0.0f, {1, 1, 1, 1, 0, 0, 0, 0, 1, 1, 1, 1}, 0x11), {1, 256}, GgufTensorType::Q4K);
            std::vector<float> x(256, 1.0f), y(1);
            ok = ok && k->gemv(t, x, y).is_ok() && y[0] == 256.0f;  // Q/reference/q4_k.rs:411-436
        }
        (void)KernelDispatcher::select_activation_route(ActivationRoute::Q8);  // back before any CHECK can return
        CHECK(ok);
        CHECK(KernelDispatcher::activation_route() == ActivationRoute::Q8);
    });

    run("gemv equals quantize + fused into zeros, bit for bit", [&] {
        auto k = kernel(GgufTensorType::Q4K);
        std::vector<uint8_t> w;
        for (float s : {0.5f, 1.0f, 0.25f}) append(w, q4_k_block(s, 0.1f, {5, 3, 7, 2, 4, 6, 1, 3, 9, 11, 13, 15}, 0xA5));
        QuantTensor t(w, {3, 256}, GgufTensorType::Q4K);
        std::vector<float> x(256), y(3, -1.0f), z(3, 0.0f);
        for (int i = 0; i < 256; ++i) x[i] = std::sin(0.37f * (float)i);
        CHECK(k->gemv(t, x, y).is_ok());
        std::vector<uint8_t> a;
        CHECK(quantize_f32_to_q8_0(x, a).is_ok());
        CHECK(k->matvec_q8_fused(w, a, z, 3, 256).is_ok());
        for (int r = 0; r < 3; ++r) CHECK(y[r] == z[r]);
    });

    // QuantLinear tests of crates/oxillama-arch/src/common/linear.rs:161-270.  The reference runs them on
    // an F32 tensor; here the weight is the same matrix as Q8_0 blocks (d = 1, q in {0, 1, 2, 3}: exact) and
    // the inputs have one magnitude per block, so the activation quantization only adds the f16 rounding of
    // its scale (tolerance 2e-3 instead of 1e-5).
    auto diag_q8 = [&](const std::vector<int> &diag) {
        std::vector<uint8_t> w;
        for (size_t r = 0; r < 32; ++r) {
            std::vector<int> q(32, 0);
            if (r < diag.size()) q[r] = diag[r];
            append(w, q8_0_block(1.0f, q));
        }
        return QuantTensor(w, {32, 32}, GgufTensorType::Q8_0);
    };
    auto eye32 = [] {
        std::vector<float> m(32 * 32, 0.0f);
        for (int i = 0; i < 32; ++i) m[i * 32 + i] = 1.0f;
        return m;
    };

    run("linear forward_no_lora (linear.rs:161-177)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        QuantLinear lin(diag_q8({2, 3}));  // [[2, 0], [0, 3]]
        std::vector<float> x(32, 0.0f), y(32, -1.0f);
        x[0] = 4.0f;
        x[1] = -4.0f;  // one magnitude per block: q = +-127
        CHECK(lin.forward(*k, x, y).is_ok());
        CHECK_NEAR(y[0], 8.0, 8e-3);
        CHECK_NEAR(y[1], -12.0, 12e-3);
        CHECK(y[2] == 0.0f);
    });

    run("linear forward_with_lora_identity (linear.rs:184-204)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        QuantLinear lin(diag_q8(std::vector<int>(32, 1)));  // identity
        std::shared_ptr<LoraAdapter> l;
        CHECK(LoraAdapter::create(eye32(), eye32(), 32, 1.0f, 32, 32, l).is_ok());
        lin.set_lora(l);
        std::vector<float> x(32, 0.0f), y(32, 0.0f);
        x[0] = 2.0f;
        x[1] = -2.0f;
        CHECK(lin.forward(*k, x, y).is_ok());
        CHECK_NEAR(y[0], 4.0, 4e-3);  // W x + delta = x + x
        CHECK_NEAR(y[1], -4.0, 4e-3);
    });

    run("linear clear_lora (linear.rs:207-233)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        QuantLinear lin(diag_q8(std::vector<int>(32, 1)));
        std::shared_ptr<LoraAdapter> l;
        CHECK(LoraAdapter::create(eye32(), eye32(), 32, 1.0f, 32, 32, l).is_ok());
        lin.set_lora(l);
        lin.clear_lora();
        std::vector<float> x(32, 0.0f), y(32, 0.0f);
        x[0] = 7.0f;
        x[1] = -7.0f;
        CHECK(lin.forward(*k, x, y).is_ok());
        CHECK_NEAR(y[0], 7.0, 7e-3);
        CHECK_NEAR(y[1], -7.0, 7e-3);
    });

    run("linear lora_applied_after_bias (linear.rs:236-262)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        QuantLinear lin(diag_q8(std::vector<int>(32, 1)), std::vector<float>(32, 10.0f));
        std::shared_ptr<LoraAdapter> l;
        CHECK(LoraAdapter::create(eye32(), eye32(), 32, 1.0f, 32, 32, l).is_ok());
        lin.set_lora(l);
        std::vector<float> x(32, 0.0f), y(32, 0.0f);
        x[0] = 3.0f;
        x[1] = -3.0f;
        CHECK(lin.forward(*k, x, y).is_ok());
        CHECK_NEAR(y[0], 3.0 + 10.0 + 3.0, 6e-3);
        CHECK_NEAR(y[1], -3.0 + 10.0 - 3.0, 6e-3);
        CHECK(y[5] == 10.0f);
    });

    run("lora apply: scale and accumulation onto the base output (lora.rs:141-200)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        // base output = bias (weights all zero), delta = B (A x) * scale
        QuantLinear lin(diag_q8({}), std::vector<float>(32, 10.0f));
        std::vector<float> a(32, 0.0f), b(32, 0.0f);  // rank 1: A = e0^T, B = e0
        a[0] = 1.0f;
        b[0] = 1.0f;
        std::shared_ptr<LoraAdapter> l;
        CHECK(LoraAdapter::create(a, b, 1, 0.5f, 32, 32, l).is_ok());
        lin.set_lora(l);
        std::vector<float> x(32, 0.0f), y(32, 0.0f);
        x[0] = 4.0f;
        CHECK(lin.forward(*k, x, y).is_ok());
        CHECK_NEAR(y[0], 12.0, 1e-6);  // 10 + 1 * (1 * 4) * 0.5
        CHECK(y[1] == 10.0f);
    });

    run("linear forward_batch: gemm + bias broadcast (linear.rs:105-132)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        std::vector<float> bias(32);
        for (int i = 0; i < 32; ++i) bias[i] = (float)i;
        QuantLinear lin(diag_q8(std::vector<int>(32, 2)), bias);
        std::vector<float> x(3 * 32, 0.0f), y(3 * 32, -1.0f);
        for (int r = 0; r < 3; ++r) x[r * 32 + r] = (float)(r + 1);
        CHECK(lin.forward_batch(*k, x, y, 3).is_ok());
        for (int r = 0; r < 3; ++r) {
            CHECK_NEAR(y[r * 32 + r], 2.0 * (r + 1) + r, 8e-3);
            CHECK(y[r * 32 + 31] == 31.0f);
        }
    });

    run("gguf load_quant_linear: the tensor loads into HBM with its stored shape and size (llama/model.rs:805-822)", [&] {
        auto k = kernel(GgufTensorType::Q8_0);
        // one Q8_0 tensor [2, 32]: row 0 = d 1.0, q = 1..32; row 1 = d 0.5, q = -16..15
        std::vector<int> q0(32), q1(32);
        for (int i = 0; i < 32; ++i) { q0[i] = i + 1; q1[i] = i - 16; }
        std::vector<uint8_t> w = q8_0_block(1.0f, q0);
        append(w, q8_0_block(0.5f, q1));
        std::vector<uint8_t> d;
        auto put32 = [&](uint32_t v) { for (int i = 0; i < 4; ++i) d.push_back((uint8_t)(v >> (8 * i))); };
        auto put64 = [&](uint64_t v) { for (int i = 0; i < 8; ++i) d.push_back((uint8_t)(v >> (8 * i))); };
        auto put_str = [&](const std::string &s) { put64(s.size()); d.insert(d.end(), s.begin(), s.end()); };
        put32(0x46554747u); put32(3); put64(1); put64(0);
        put_str("blk.0.attn_q.weight"); put32(2); put64(2); put64(32); put32(8); put64(0);
        d.resize((d.size() + 31) / 32 * 32, 0);
        append(d, w);
        GgufModel m;
        CHECK(m.from_bytes(d) == OXQ_OK);
        DeviceWeights dw;
        CHECK(m.load_quant_linear("blk.0.attn_q.weight", dw) == OXQ_OK);
        CHECK(dw.shape == std::vector<size_t>({2, 32}) && dw.tensor_type == 8 && dw.nbytes() == 68);
        // the same bytes through the host-slice trait method
        std::vector<float> x(32, 1.0f), y_host(2, 0.0f);
        std::vector<uint8_t> acts;
        CHECK(quantize_f32_to_q8_0(x, acts).is_ok());
        CHECK(k->matvec_q8_fused(w, acts, y_host, 2, 32).is_ok());
        CHECK_NEAR(y_host[0], 528.0, 0.3);  // 1 + 2 + ... + 32, ones quantize to 127 * (1/127 in f16)
        CHECK_NEAR(y_host[1], -8.0, 0.01);
        DeviceWeights missing;
        CHECK(m.load_quant_linear("blk.1.attn_q.weight", missing) == OXQ_ERR_GGUF_TENSOR_NOT_FOUND);
    });

    run("moe top-1 / top-2 / clamped top-k on all-ones experts (moe.rs:324-401): the expert's own output", [&] {
        // x = 127/128 everywhere: exact under Q8_0 (d = 2^-7, q = 127).  gate = up = 256 * x = 254, silu(254) = 254
        // in fp32, h = 254^2 = 64516 (d = 508, q = 127: exact), down = 256 * 64516 = 16516096 < 2^24.
        std::vector<float> x(256, 0.9921875f), y(256, -1.0f);
        for (size_t top_k : {(size_t)1, (size_t)2, (size_t)10}) {
            MoeFfn moe = ones_moe(256, 256, 4, top_k);
            std::fill(y.begin(), y.end(), -1.0f);
            QuantResult r = moe.forward(x, y);
            CHECK(r.is_ok());
            for (float v : y) CHECK_NEAR(v, 16516096.0, 16516096.0 * 1e-6);
        }
        // one-hot router: expert 0 alone at top-1 (its down matrix doubled tells it apart)
        MoeFfn moe = ones_moe(256, 256, 4, 1, 0.0f);
        moe.router[0] = 1.0f;
        for (size_t b = 0; b < moe.experts[0].down.data.size(); b += 34) put_f16(moe.experts[0].down.data, b, 2.0f);
        CHECK(moe.forward(x, y).is_ok());
        for (float v : y) CHECK_NEAR(v, 2 * 16516096.0, 2 * 16516096.0 * 1e-6);
        // three tokens at once; a zero token gives a zero row (moe.rs:291-305)
        std::vector<float> xb(3 * 256, 0.9921875f), yb(3 * 256, -1.0f);
        std::fill(xb.begin() + 256, xb.begin() + 512, 0.0f);
        CHECK(moe.forward_batch(xb, yb, 3).is_ok());
        CHECK_NEAR(yb[0], 2 * 16516096.0, 40.0);
        CHECK(yb[256] == 0.0f && yb[511] == 0.0f);
        CHECK_NEAR(yb[767], 2 * 16516096.0, 40.0);
    });
}

int main(int argc, char **argv) {
    const std::string mode = argc > 1 ? argv[1] : "--host";
    if (mode == "--host") {
        host_tests();
    } else if (mode == "--gpu") {
        gpu_tests();
    } else {
        std::printf("usage: %s --host | --gpu\n", argv[0]);
        return 2;
    }
    std::printf("%d cases, %d failed\n", g_run, g_failed);
    return g_failed == 0 ? 0 : 1;
}
