// C ABI of liboxq_hip.so (see include/oxq.h): argument validation in the
// reference's order, HBM residency of weights, scratch buffers for the
// host-slice route, and kernel launches.  No exception or abort crosses the ABI.
#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <unordered_map>
#include <vector>

#include "oxq_internal.hpp"

namespace oxq {
hipError_t launch_dequant(uint32_t type, const uint8_t *blocks, size_t n_blocks, float *out, hipStream_t stream);
}

// Workspace of oxq_gemm_q8_static_dev: the tile kernel's re-laid-out activations (int8 payload, fp32 block sums,
// f16 scales) live here instead of in a caller's or the library's allocation.  Every GPU the library runs on holds
// its own copy at its own address until the process ends; host code reaches it only through the address that
// hipGetSymbolAddress returned for that device (static_scratch_ptr), never through this name.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)16 << 20;
static __device__ __align__(256) uint8_t scratch[STATIC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
uint8_t *static_scratch_ptr[MAX_DEVICES] = {nullptr};  // per device, filled by oxq_init with that device current

struct ErrorDetail {
    int status = OXQ_OK;
    size_t a = 0, b = 0;
    char message[256] = {0};
};
thread_local ErrorDetail g_err;

int fail(int status, size_t a, size_t b, const char *msg) {
    g_err.status = status;
    g_err.a = a;
    g_err.b = b;
    std::snprintf(g_err.message, sizeof(g_err.message), "%s", msg ? msg : "");
    return status;
}

int fail_hip(hipError_t e, const char *what) {
    char buf[256];
    std::snprintf(buf, sizeof(buf), "%s: %s", what, hipGetErrorString(e));
    return fail(OXQ_ERR_KERNEL, (size_t)e, 0, buf);
}

#define OXQ_HIP(call)                                     \
    do {                                                  \
        hipError_t e_ = (call);                           \
        if (e_ != hipSuccess) return fail_hip(e_, #call); \
    } while (0)

// A growable device buffer.
struct Scratch {
    void *ptr = nullptr;
    size_t cap = 0;
    int reserve(size_t n) {
        if (n <= cap) return OXQ_OK;
        if (ptr) (void)hipFree(ptr);
        ptr = nullptr;
        cap = 0;
        size_t want = n + n / 4 + 256;
        hipError_t e = hipMalloc(&ptr, want);
        if (e != hipSuccess) return fail_hip(e, "hipMalloc(scratch)");
        cap = want;
        return OXQ_OK;
    }
    void release() {
        if (ptr) (void)hipFree(ptr);
        ptr = nullptr;
        cap = 0;
    }
};

struct CacheKey {
    const void *ptr;
    size_t len;
    uint32_t type;
    bool operator==(const CacheKey &o) const { return ptr == o.ptr && len == o.len && type == o.type; }
};
struct CacheKeyHash {
    size_t operator()(const CacheKey &k) const {
        return std::hash<const void *>()(k.ptr) ^ (k.len * 0x9E3779B97F4A7C15ull) ^ k.type;
    }
};
struct CacheEntry {
    uint8_t *dev;
    uint64_t fingerprint;
    uint64_t last_use;  // tick of the last hit (least recently used goes first when the byte cap is reached)
};

struct State {
    std::mutex mu;
    std::atomic<bool> initialised{false};
    int device = -1;
    uint32_t cus = 0;
    // launch-shape knobs (oxq_tuning.h): written by the setters, read once per launch, no lock needed
    std::atomic<uint32_t> waves_per_cu{0};    // 0 = default
    std::atomic<uint32_t> rows_per_batch{0};  // 0 = chosen per shape
    std::atomic<uint32_t> waves_per_row{0};   // 0 = chosen per shape
    std::atomic<int> act_route{OXQ_ROUTE_Q8};  // how the fp32-input entry points treat their activations
    int cache_mode = 0;  // 0 off, 1 on (sampled fingerprint), 2 on and verified (every byte hashed on every call)
    std::unordered_map<CacheKey, CacheEntry, CacheKeyHash> cache;
    size_t cache_bytes = 0, cache_limit = (size_t)16 << 30;
    uint64_t cache_tick = 0, cache_hits = 0, cache_uploads = 0;
    uint64_t cache_pin = UINT64_MAX;  // entries used after this tick belong to the call in progress: not evicted
    Scratch s_weights, s_acts, s_x, s_out, s_sums, s_work, s_bias, s_lora_a, s_lora_b, s_lora_r;
    Scratch s_moe_up, s_moe_down, s_moe_tables;
    std::atomic<bool> fuse_swiglu{true};  // oxq_ffn_swiglu_dev: gate, up, SwiGLU and the quantizer of h in one launch where possible
};
State g;


// FNV-1a over up to 64 samples of 64 bytes spread across the buffer, plus its length; `whole`: over
// every byte, eight at a time (the verified mode: any changed byte changes the value).
uint64_t fingerprint(const uint8_t *p, size_t len, bool whole) {
    uint64_t h = 1469598103934665603ull ^ len;
    const size_t chunk = 64, samples = 64;
    if (whole) {
        uint64_t lanes[4] = {h, h ^ 0x9E3779B97F4A7C15ull, h ^ 0xC2B2AE3D27D4EB4Full, h ^ 0x165667B19E3779F9ull};
        size_t i = 0;
        for (; i + 32 <= len; i += 32) {
            uint64_t w[4];
            std::memcpy(w, p + i, 32);
            for (int l = 0; l < 4; l++) {
                lanes[l] = (lanes[l] ^ w[l]) * 0x100000001B3ull;
                lanes[l] ^= lanes[l] >> 29;
            }
        }
        for (; i < len; i++) lanes[i & 3] = (lanes[i & 3] ^ p[i]) * 0x100000001B3ull;
        for (int l = 0; l < 4; l++) h = (h ^ lanes[l]) * 1099511628211ull;
        return h;
    }
    if (len <= chunk * samples) {
        for (size_t i = 0; i < len; i++) h = (h ^ p[i]) * 1099511628211ull;
        return h;
    }
    const size_t stride = (len - chunk) / (samples - 1);
    for (size_t s = 0; s < samples; s++) {
        const uint8_t *q = p + s * stride;
        for (size_t i = 0; i < chunk; i++) h = (h ^ q[i]) * 1099511628211ull;
    }
    return h;
}

bool known_type(uint32_t type) { return oxq_block_size(type) != 0; }

int ensure_init() {
    if (g.initialised.load(std::memory_order_acquire)) return OXQ_OK;
    return oxq_init(0);
}

// Device copy of a host weight buffer: cached when the cache is on, else staged
// in scratch.  Caller holds g.mu.
int stage_weights(uint32_t type, const uint8_t *host, size_t len, const uint8_t **dev) {
    if (g.cache_mode != 0 && len <= g.cache_limit) {
        CacheKey key{host, len, type};
        const uint64_t fp = fingerprint(host, len, g.cache_mode == 2);
        auto it = g.cache.find(key);
        if (it != g.cache.end() && it->second.fingerprint == fp) {
            it->second.last_use = ++g.cache_tick;
            g.cache_hits++;
            *dev = it->second.dev;
            return OXQ_OK;
        }
        if (it != g.cache.end()) {  // same address, different content: the device copy is stale
            (void)hipFree(it->second.dev);
            g.cache_bytes -= it->first.len;
            g.cache.erase(it);
        }
        while (!g.cache.empty() && g.cache_bytes + len > g.cache_limit) {  // byte cap: least recently used first
            auto lru = g.cache.end();
            for (auto jt = g.cache.begin(); jt != g.cache.end(); ++jt)
                if (jt->second.last_use <= g.cache_pin && (lru == g.cache.end() || jt->second.last_use < lru->second.last_use))
                    lru = jt;
            if (lru == g.cache.end()) break;  // what is left was staged by this very call and is about to be read
            (void)hipFree(lru->second.dev);
            g.cache_bytes -= lru->first.len;
            g.cache.erase(lru);
        }
        uint8_t *d = nullptr;
        OXQ_HIP(hipMalloc((void **)&d, len ? len : 1));
        hipError_t e = hipMemcpy(d, host, len, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(d);
            return fail_hip(e, "hipMemcpy(weights)");
        }
        g.cache.emplace(key, CacheEntry{d, fp, ++g.cache_tick});
        g.cache_bytes += len;
        g.cache_uploads++;
        *dev = d;
        return OXQ_OK;
    }
    int st = g.s_weights.reserve(len ? len : 1);
    if (st != OXQ_OK) return st;
    OXQ_HIP(hipMemcpy(g.s_weights.ptr, host, len, hipMemcpyHostToDevice));
    *dev = (const uint8_t *)g.s_weights.ptr;
    return OXQ_OK;
}

struct FusedShape {
    size_t bpr, row_bytes, acts_needed;
};

// Validation order of the reference's matvec_q8_fused
// (crates/oxillama-quant/src/reference/q4_k.rs:226-250, traits.rs:99-130).
// whole_blocks: refuse rows that end inside a block (the debug dump of the group sums needs whole groups);
// the matvec itself takes them as the reference does, skipping the columns past n_cols.
int validate_fused(uint32_t type, size_t weights_len, size_t acts_len, size_t out_len, size_t n_rows,
                   size_t n_cols, FusedShape *fs, bool whole_blocks) {
    if (!known_type(type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "unsupported quantization type");
    if (out_len < n_rows) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_rows, out_len, "out shorter than n_rows");
    const size_t bs = oxq_block_size(type), bb = oxq_block_bytes(type);
    fs->bpr = (n_cols + bs - 1) / bs;
    fs->row_bytes = fs->bpr * bb;
    fs->acts_needed = fs->bpr * (bs / 32) * 34;
    if (weights_len < n_rows * fs->row_bytes)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, n_rows * fs->row_bytes, weights_len, "weights buffer too small");
    if (acts_len < fs->acts_needed)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, fs->acts_needed, acts_len, "activation buffer too small");
    if (whole_blocks && n_cols % bs != 0)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, bs, n_cols, "n_cols is not a multiple of the block size");
    if (n_rows > 0xFFFFFFFFull || n_cols > 0xFFFFFF00ull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFF00ull, n_rows > n_cols ? n_rows : n_cols, "dimension exceeds 2^32-257");
    return OXQ_OK;
}

oxq::GemvArgs gemv_args(const uint8_t *W, const uint8_t *A, float *out, int32_t *sums, size_t n_rows,
                        size_t n_cols, int accumulate) {
    oxq::GemvArgs a;
    a.W = W;
    a.A = A;
    a.out = out;
    a.sums = sums;
    a.n_rows = (uint32_t)n_rows;
    a.n_cols = (uint32_t)n_cols;
    a.accumulate = accumulate;
    a.waves_per_cu = g.waves_per_cu.load(std::memory_order_relaxed);
    a.rows_per_batch = g.rows_per_batch.load(std::memory_order_relaxed);
    a.waves_per_row = g.waves_per_row.load(std::memory_order_relaxed);
    return a;
}

// Resolve (n_rows, n_cols) of a QuantTensor as the reference's gemv does
// (reference/q4_k.rs:110-115).
int tensor_dims(uint32_t type, size_t data_len, const size_t *shape, size_t n_dims, size_t *n_rows,
                size_t *n_cols) {
    if (!known_type(type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "unsupported quantization type");
    if (!shape || n_dims == 0) return fail(OXQ_ERR_DIMENSION_MISMATCH, 1, 0, "tensor shape is empty");
    *n_rows = shape[0];
    if (n_dims > 1) {
        *n_cols = shape[1];
    } else {
        if (shape[0] == 0) return fail(OXQ_ERR_DIMENSION_MISMATCH, 1, 0, "tensor has zero rows");
        size_t n_elems = 1;
        for (size_t i = 0; i < n_dims; i++) n_elems *= shape[i];
        *n_cols = n_elems / shape[0];
    }
    (void)data_len;
    return OXQ_OK;
}

}  // namespace

namespace oxq {
thread_local LaunchNote g_last_launch;
std::atomic<uint64_t *> g_phase_buf{nullptr};
std::atomic<size_t> g_phase_cap{0};
uint32_t device_cus() { return g.cus ? g.cus : 256; }
int set_error(int status, size_t a, size_t b, const char *msg) { return fail(status, a, b, msg); }
int ensure_device() { return ensure_init(); }
}  // namespace oxq

extern "C" {

int oxq_init(int device) {
    std::lock_guard<std::mutex> lock(g.mu);
    if (g.initialised && g.device == device) return OXQ_OK;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(OXQ_ERR_NO_DEVICE, 0, 0, "no HIP device visible");
    }
    if (device < 0 || device >= count) return fail(OXQ_ERR_NO_DEVICE, (size_t)count, (size_t)device, "device index out of range");
    OXQ_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    OXQ_HIP(hipGetDeviceProperties(&prop, device));
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        char msg[200];
        std::snprintf(msg, sizeof(msg), "device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
        return fail(OXQ_ERR_NO_DEVICE, 0, 0, msg);
    }
    if (device < MAX_DEVICES && !static_scratch_ptr[device]) {
        uint8_t *p = nullptr;
        OXQ_HIP(hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch)));
        static_scratch_ptr[device] = p;
    }
    g.device = device;
    g.cus = (uint32_t)prop.multiProcessorCount;
    g.initialised = true;
    return OXQ_OK;
}

int oxq_shutdown(void) {
    std::lock_guard<std::mutex> lock(g.mu);
    if (!g.initialised) return OXQ_OK;
    for (auto &kv : g.cache) (void)hipFree(kv.second.dev);
    g.cache.clear();
    g.cache_bytes = 0;
    g.s_weights.release();
    g.s_acts.release();
    g.s_x.release();
    g.s_out.release();
    g.s_sums.release();
    g.s_work.release();
    g.s_bias.release();
    g.s_lora_a.release();
    g.s_lora_b.release();
    g.s_lora_r.release();
    g.s_moe_up.release();
    g.s_moe_down.release();
    g.s_moe_tables.release();
    oxq::gguf_release_staging();
    g.initialised = false;
    g.device = -1;
    return OXQ_OK;
}

int oxq_device_info(oxq_device_props *out) {
    if (!out) return fail(OXQ_ERR_INTERNAL, 0, 0, "null output");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    hipDeviceProp_t prop;
    OXQ_HIP(hipGetDeviceProperties(&prop, g.device));
    std::memset(out, 0, sizeof(*out));
    out->device = g.device;
    out->compute_units = prop.multiProcessorCount;
    out->clock_khz = prop.clockRate;
    out->memory_clock_khz = prop.memoryClockRate;
    out->memory_bus_bits = prop.memoryBusWidth;
    out->total_memory = prop.totalGlobalMem;
    std::snprintf(out->name, sizeof(out->name), "%s", prop.name);
    std::snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
    return OXQ_OK;
}

int oxq_last_error(size_t *a, size_t *b, char *message, size_t message_len) {
    if (a) *a = g_err.a;
    if (b) *b = g_err.b;
    if (message && message_len) std::snprintf(message, message_len, "%s", g_err.message);
    return g_err.status;
}

const char *oxq_status_name(int status) {
    switch (status) {
    case OXQ_OK: return "Ok";
    case OXQ_ERR_UNSUPPORTED_TYPE: return "UnsupportedType";
    case OXQ_ERR_BLOCK_SIZE_MISMATCH: return "BlockSizeMismatch";
    case OXQ_ERR_DIMENSION_MISMATCH: return "DimensionMismatch";
    case OXQ_ERR_KERNEL: return "KernelError";
    case OXQ_ERR_BLOCK_COUNT_MISMATCH: return "BlockCountMismatch";
    case OXQ_ERR_BUFFER_TOO_SMALL: return "BufferTooSmall";
    case OXQ_ERR_INTERNAL: return "Internal";
    case OXQ_ERR_UNSUPPORTED_SHAPE: return "UnsupportedShape";
    case OXQ_ERR_NO_DEVICE: return "NoDevice";
    case 10: return "GgufInvalidMagic";
    case 11: return "GgufUnsupportedVersion";
    case 12: return "GgufUnexpectedEof";
    case 13: return "GgufInvalidMetadata";
    case 14: return "GgufUnsupportedQuantType";
    case 15: return "GgufTensorNotFound";
    case 16: return "GgufInvalidString";
    case 17: return "GgufIo";
    default: return "Unknown";
    }
}

size_t oxq_block_size(uint32_t type) {
    switch (type) {
    case OXQ_TYPE_Q4_0:
    case OXQ_TYPE_Q8_0:
    case OXQ_TYPE_Q4_1:
    case OXQ_TYPE_Q5_0:
    case OXQ_TYPE_Q5_1:
    case OXQ_TYPE_Q8_1:
    case OXQ_TYPE_IQ4_NL: return 32;
    case OXQ_TYPE_Q4_K:
    case OXQ_TYPE_Q6_K:
    case OXQ_TYPE_IQ4_XS:
    case OXQ_TYPE_Q2_K:
    case OXQ_TYPE_Q3_K:
    case OXQ_TYPE_Q5_K: return 256;
    default: return 0;
    }
}

size_t oxq_block_bytes(uint32_t type) {
    switch (type) {
    case OXQ_TYPE_Q4_0: return 18;
    case OXQ_TYPE_Q8_0: return 34;
    case OXQ_TYPE_Q4_K: return 144;
    case OXQ_TYPE_Q6_K: return 210;
    case OXQ_TYPE_IQ4_XS: return 136;
    case OXQ_TYPE_Q4_1: return 20;
    case OXQ_TYPE_Q5_0: return 22;
    case OXQ_TYPE_Q5_1: return 24;
    case OXQ_TYPE_Q8_1: return 36;
    case OXQ_TYPE_IQ4_NL: return 18;
    case OXQ_TYPE_Q2_K: return 84;
    case OXQ_TYPE_Q3_K: return 110;
    case OXQ_TYPE_Q5_K: return 176;
    default: return 0;
    }
}

const char *oxq_type_name(uint32_t type) {
    switch (type) {
    case OXQ_TYPE_Q4_0: return "Q4_0";
    case OXQ_TYPE_Q8_0: return "Q8_0";
    case OXQ_TYPE_Q4_K: return "Q4_K";
    case OXQ_TYPE_Q6_K: return "Q6_K";
    case OXQ_TYPE_IQ4_XS: return "IQ4_XS";
    case OXQ_TYPE_Q4_1: return "Q4_1";
    case OXQ_TYPE_Q5_0: return "Q5_0";
    case OXQ_TYPE_Q5_1: return "Q5_1";
    case OXQ_TYPE_Q8_1: return "Q8_1";
    case OXQ_TYPE_IQ4_NL: return "IQ4_NL";
    case OXQ_TYPE_Q2_K: return "Q2_K";
    case OXQ_TYPE_Q3_K: return "Q3_K";
    case OXQ_TYPE_Q5_K: return "Q5_K";
    default: return nullptr;
    }
}

int oxq_get_kernel(uint32_t type) {
    if (!known_type(type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "unsupported quantization type");
    return OXQ_OK;
}

int oxq_set_gemv_waves_per_cu(unsigned waves) {
    g.waves_per_cu = waves > 64 ? 64 : waves;
    return OXQ_OK;
}

int oxq_set_gemv_rows_per_batch(unsigned rows) {
    g.rows_per_batch = rows > 4 ? 4 : rows;
    return OXQ_OK;
}

int oxq_set_gemv_waves_per_row(unsigned waves) {
    g.waves_per_row = waves >= 4 ? 4 : (waves ? 1 : 0);
    return OXQ_OK;
}

int oxq_last_launch(char *out, size_t out_len) {
    if (!out || out_len == 0) return fail(OXQ_ERR_INTERNAL, 0, 0, "null output");
    const oxq::LaunchNote &n = oxq::g_last_launch;
    const char *tn = oxq_type_name(n.type);
    std::snprintf(out, out_len, "%s<%s,%d,%d,%d,%d> grid %ux%u block %u", n.kernel, tn ? tn : "-", n.p[0], n.p[1], n.p[2],
                  n.p[3], n.grid_x, n.grid_y, n.block);
    return OXQ_OK;
}

int oxq_set_gemv_phase_probe(void *d_buffer, size_t bytes) {
    oxq::g_phase_cap.store(d_buffer ? bytes : 0, std::memory_order_relaxed);
    oxq::g_phase_buf.store((uint64_t *)d_buffer, std::memory_order_relaxed);
    return OXQ_OK;
}

int oxq_set_gemm_tile_min_rows(unsigned rows) {
    oxq::g_gemm_tile_min_rows.store(rows, std::memory_order_relaxed);
    return OXQ_OK;
}

int oxq_set_gemm_variant(int variant) {
    oxq::g_gemm_variant.store(variant, std::memory_order_relaxed);
    return OXQ_OK;
}

int oxq_weight_cache_enable(int mode) {
    std::lock_guard<std::mutex> lock(g.mu);
    g.cache_mode = mode == 2 ? 2 : (mode != 0 ? 1 : 0);
    return OXQ_OK;
}

int oxq_weight_cache_clear(void) {
    std::lock_guard<std::mutex> lock(g.mu);
    for (auto &kv : g.cache) (void)hipFree(kv.second.dev);
    g.cache.clear();
    g.cache_bytes = 0;
    return OXQ_OK;
}

int oxq_weight_cache_invalidate(const void *host_ptr) {
    std::lock_guard<std::mutex> lock(g.mu);
    for (auto it = g.cache.begin(); it != g.cache.end();) {
        if (it->first.ptr == host_ptr) {
            (void)hipFree(it->second.dev);
            g.cache_bytes -= it->first.len;
            it = g.cache.erase(it);
        } else {
            ++it;
        }
    }
    return OXQ_OK;
}

int oxq_weight_cache_set_limit(size_t max_bytes) {
    std::lock_guard<std::mutex> lock(g.mu);
    g.cache_limit = max_bytes;
    while (!g.cache.empty() && g.cache_bytes > g.cache_limit) {
        auto lru = g.cache.begin();
        for (auto jt = g.cache.begin(); jt != g.cache.end(); ++jt)
            if (jt->second.last_use < lru->second.last_use) lru = jt;
        (void)hipFree(lru->second.dev);
        g.cache_bytes -= lru->first.len;
        g.cache.erase(lru);
    }
    return OXQ_OK;
}

int oxq_weight_cache_stats(size_t *entries, size_t *bytes, uint64_t *hits, uint64_t *uploads) {
    std::lock_guard<std::mutex> lock(g.mu);
    if (entries) *entries = g.cache.size();
    if (bytes) *bytes = g.cache_bytes;
    if (hits) *hits = g.cache_hits;
    if (uploads) *uploads = g.cache_uploads;
    return OXQ_OK;
}

// ---- host-slice route ---------------------------------------------------

int oxq_dequant_block(uint32_t type, const uint8_t *block, size_t block_len, float *output, size_t output_len) {
    if (!known_type(type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "unsupported quantization type");
    const size_t bs = oxq_block_size(type), bb = oxq_block_bytes(type);
    if (block_len < bb) return fail(OXQ_ERR_BUFFER_TOO_SMALL, bb, block_len, "block too small");
    if (output_len < bs) return fail(OXQ_ERR_BUFFER_TOO_SMALL, bs, output_len, "output too small");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    std::lock_guard<std::mutex> lock(g.mu);
    if ((st = g.s_acts.reserve(bb)) != OXQ_OK) return st;
    if ((st = g.s_out.reserve(bs * sizeof(float))) != OXQ_OK) return st;
    OXQ_HIP(hipMemcpy(g.s_acts.ptr, block, bb, hipMemcpyHostToDevice));
    OXQ_HIP(oxq::launch_dequant(type, (const uint8_t *)g.s_acts.ptr, 1, (float *)g.s_out.ptr, nullptr));
    OXQ_HIP(hipMemcpy(output, g.s_out.ptr, bs * sizeof(float), hipMemcpyDeviceToHost));
    return OXQ_OK;
}

int oxq_quantize_f32_to_q8_0(const float *data, size_t n, uint8_t *out, size_t out_len) {
    if (n % 32 != 0) return fail(OXQ_ERR_DIMENSION_MISMATCH, (n / 32 + 1) * 32, n, "length is not a multiple of 32");
    const size_t need = n / 32 * 34;
    if (out_len < need) return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, out_len, "output too small");
    if (n == 0) return OXQ_OK;
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    std::lock_guard<std::mutex> lock(g.mu);
    if ((st = g.s_x.reserve(n * sizeof(float))) != OXQ_OK) return st;
    if ((st = g.s_acts.reserve(need)) != OXQ_OK) return st;
    OXQ_HIP(hipMemcpy(g.s_x.ptr, data, n * sizeof(float), hipMemcpyHostToDevice));
    OXQ_HIP(oxq::launch_quantize_q8_0((const float *)g.s_x.ptr, n, (uint8_t *)g.s_acts.ptr, nullptr));
    OXQ_HIP(hipMemcpy(out, g.s_acts.ptr, need, hipMemcpyDeviceToHost));
    return OXQ_OK;
}

int oxq_matvec_q8_fused(uint32_t type, const uint8_t *weights, size_t weights_len, const uint8_t *acts_q8,
                        size_t acts_len, float *out, size_t out_len, size_t n_rows, size_t n_cols) {
    FusedShape fs;
    int st = validate_fused(type, weights_len, acts_len, out_len, n_rows, n_cols, &fs, false);
    if (st != OXQ_OK) return st;
    if (n_rows == 0 || n_cols == 0) return OXQ_OK;
    if ((st = ensure_init()) != OXQ_OK) return st;
    std::lock_guard<std::mutex> lock(g.mu);
    const uint8_t *dW = nullptr;
    if ((st = stage_weights(type, weights, n_rows * fs.row_bytes, &dW)) != OXQ_OK) return st;
    if ((st = g.s_acts.reserve(fs.acts_needed)) != OXQ_OK) return st;
    if ((st = g.s_out.reserve(n_rows * sizeof(float))) != OXQ_OK) return st;
    OXQ_HIP(hipMemcpy(g.s_acts.ptr, acts_q8, fs.acts_needed, hipMemcpyHostToDevice));
    OXQ_HIP(hipMemcpy(g.s_out.ptr, out, n_rows * sizeof(float), hipMemcpyHostToDevice));
    OXQ_HIP(oxq::launch_gemv_q8(type, gemv_args(dW, (const uint8_t *)g.s_acts.ptr, (float *)g.s_out.ptr, nullptr,
                                                n_rows, n_cols, 1), nullptr));
    OXQ_HIP(hipMemcpy(out, g.s_out.ptr, n_rows * sizeof(float), hipMemcpyDeviceToHost));
    return OXQ_OK;
}

int oxq_block_sums(uint32_t type, const uint8_t *weights, size_t weights_len, const uint8_t *acts_q8,
                   size_t acts_len, int32_t *sums, size_t sums_len, size_t n_rows, size_t n_cols) {
    FusedShape fs;
    int st = validate_fused(type, weights_len, acts_len, n_rows, n_rows, n_cols, &fs, true);
    if (st != OXQ_OK) return st;
    const size_t groups = n_cols / oxq::gemv_group_cols(type);
    if (sums_len < n_rows * groups) return fail(OXQ_ERR_BUFFER_TOO_SMALL, n_rows * groups, sums_len, "sums buffer too small");
    if (n_rows == 0 || n_cols == 0) return OXQ_OK;
    if ((st = ensure_init()) != OXQ_OK) return st;
    std::lock_guard<std::mutex> lock(g.mu);
    const uint8_t *dW = nullptr;
    if ((st = stage_weights(type, weights, n_rows * fs.row_bytes, &dW)) != OXQ_OK) return st;
    if ((st = g.s_acts.reserve(fs.acts_needed)) != OXQ_OK) return st;
    if ((st = g.s_out.reserve(n_rows * sizeof(float))) != OXQ_OK) return st;
    if ((st = g.s_sums.reserve(n_rows * groups * sizeof(int32_t))) != OXQ_OK) return st;
    OXQ_HIP(hipMemcpy(g.s_acts.ptr, acts_q8, fs.acts_needed, hipMemcpyHostToDevice));
    OXQ_HIP(oxq::launch_gemv_q8(type, gemv_args(dW, (const uint8_t *)g.s_acts.ptr, (float *)g.s_out.ptr,
                                                (int32_t *)g.s_sums.ptr, n_rows, n_cols, 0), nullptr));
    OXQ_HIP(hipMemcpy(sums, g.s_sums.ptr, n_rows * groups * sizeof(int32_t), hipMemcpyDeviceToHost));
    return OXQ_OK;
}

static int gemm_host(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape, size_t n_dims,
                     const float *bias, size_t bias_len, const float *input, size_t input_len, float *output,
                     size_t output_len, size_t m, size_t n, size_t k) {
    size_t n_rows = 0, n_cols = 0;
    int st = tensor_dims(type, data_len, shape, n_dims, &n_rows, &n_cols);
    if (st != OXQ_OK) return st;
    // The reference slices input[row*k..(row+1)*k] and output[row*n..(row+1)*n] and calls gemv
    // (reference/q4_k.rs:195-199): a short slice or k < n_cols / n < n_rows is a dimension error.
    if (input_len < m * k) return fail(OXQ_ERR_DIMENSION_MISMATCH, m * k, input_len, "input shorter than m*k");
    if (output_len < m * n) return fail(OXQ_ERR_DIMENSION_MISMATCH, m * n, output_len, "output shorter than m*n");
    if (m == 0) return OXQ_OK;
    if (k < n_cols) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_cols, k, "k smaller than the tensor's columns");
    if (n < n_rows) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_rows, n, "n smaller than the tensor's rows");
    const size_t bs = oxq_block_size(type), bb = oxq_block_bytes(type);
    const size_t bpr = (n_cols + bs - 1) / bs, row_bytes = bpr * bb;
    if (data_len < n_rows * row_bytes)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, n_rows * row_bytes, data_len, "tensor data too small");
    if (n_rows == 0 || n_cols == 0) return OXQ_OK;
    if (n_rows > 0xFFFFFFFFull || n_cols > 0xFFFFFF00ull || m > 0xFFFFFFFFull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, n_rows, "dimension exceeds 2^32-1");
    if ((st = ensure_init()) != OXQ_OK) return st;
    std::lock_guard<std::mutex> lock(g.mu);
    const uint8_t *dW = nullptr;
    if ((st = stage_weights(type, data, n_rows * row_bytes, &dW)) != OXQ_OK) return st;
    // A row that ends inside a block (the reference's gemv skips the columns past n_cols,
    // reference/q4_k.rs:161,168): the input rows are staged zero-padded to whole blocks, so the padding
    // quantizes to zero bytes and the kernels mask it besides.
    const size_t k_pad = bpr * bs, act_row_bytes = k_pad / 32 * 34;
    if ((st = g.s_x.reserve(m * k_pad * sizeof(float))) != OXQ_OK) return st;
    if ((st = g.s_acts.reserve(m * act_row_bytes)) != OXQ_OK) return st;
    if ((st = g.s_out.reserve(m * n_rows * sizeof(float))) != OXQ_OK) return st;
    // Gather the first n_cols floats of each input row (k may exceed n_cols).
    if (k_pad != n_cols) OXQ_HIP(hipMemset(g.s_x.ptr, 0, m * k_pad * sizeof(float)));
    OXQ_HIP(hipMemcpy2D(g.s_x.ptr, k_pad * sizeof(float), input, k * sizeof(float), n_cols * sizeof(float), m,
                        hipMemcpyHostToDevice));
    const float *d_bias_f32 = nullptr;
    if (g.act_route.load(std::memory_order_relaxed) == OXQ_ROUTE_F32) {
        // the reference's own gemm: m gemvs on the fp32 rows (reference/q4_k.rs:186-201), bias per row (linear.rs:123-128)
        if (!oxq::gemv_f32_supported(type))
            return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "no fp32-activation kernel for this type (OXQ_ROUTE_F32)");
        if (bias && bias_len) {
            if ((st = g.s_bias.reserve(n_rows * sizeof(float))) != OXQ_OK) return st;
            const size_t nb = bias_len < n_rows ? bias_len : n_rows;
            OXQ_HIP(hipMemset(g.s_bias.ptr, 0, n_rows * sizeof(float)));
            OXQ_HIP(hipMemcpy(g.s_bias.ptr, bias, nb * sizeof(float), hipMemcpyHostToDevice));
            d_bias_f32 = (const float *)g.s_bias.ptr;
        }
        for (size_t r = 0; r < m; r++)
            OXQ_HIP(oxq::launch_gemv_f32(type, dW, (const float *)g.s_x.ptr + r * k_pad, (float *)g.s_out.ptr + r * n_rows,
                                         d_bias_f32, (uint32_t)n_rows, (uint32_t)n_cols, nullptr));
        OXQ_HIP(hipMemcpy2D(output, n * sizeof(float), g.s_out.ptr, n_rows * sizeof(float), n_rows * sizeof(float), m,
                            hipMemcpyDeviceToHost));
        return OXQ_OK;
    }
    OXQ_HIP(oxq::launch_quantize_q8_0((const float *)g.s_x.ptr, m * k_pad, (uint8_t *)g.s_acts.ptr, nullptr));
    oxq::GemmArgs ga;
    ga.W = dW;
    ga.A = (const uint8_t *)g.s_acts.ptr;
    ga.out = (float *)g.s_out.ptr;
    ga.sums = nullptr;
    ga.workspace = nullptr;
    if (oxq::gemm_uses_tiles(type, (uint32_t)m, (uint32_t)n_rows, (uint32_t)n_cols) ||
        oxq::gemm_few_rows_pay(type, (uint32_t)m, (uint32_t)n_rows, (uint32_t)n_cols)) {
        const size_t wbytes = oxq::gemm_workspace_bytes((uint32_t)m, (uint32_t)n_cols, (uint32_t)n_rows, type);
        if ((st = g.s_work.reserve(wbytes)) != OXQ_OK) return st;
        ga.workspace = (uint8_t *)g.s_work.ptr;
        ga.workspace_bytes = wbytes;
    }
    ga.m = (uint32_t)m;
    ga.n = (uint32_t)n_rows;
    ga.k = (uint32_t)n_cols;
    ga.accumulate = 0;
    if (bias && bias_len) {
        // the reference adds bias[j] for every j the bias holds (linear.rs:123-128)
        if ((st = g.s_bias.reserve(n_rows * sizeof(float))) != OXQ_OK) return st;
        const size_t nb = bias_len < n_rows ? bias_len : n_rows;
        OXQ_HIP(hipMemset(g.s_bias.ptr, 0, n_rows * sizeof(float)));
        OXQ_HIP(hipMemcpy(g.s_bias.ptr, bias, nb * sizeof(float), hipMemcpyHostToDevice));
        ga.bias = (const float *)g.s_bias.ptr;
    }
    OXQ_HIP(oxq::launch_gemm_q8(type, ga, nullptr));
    OXQ_HIP(hipMemcpy2D(output, n * sizeof(float), g.s_out.ptr, n_rows * sizeof(float), n_rows * sizeof(float), m,
                        hipMemcpyDeviceToHost));
    return OXQ_OK;
}

int oxq_gemm(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape, size_t n_dims,
             const float *input, size_t input_len, float *output, size_t output_len, size_t m, size_t n, size_t k) {
    return gemm_host(type, data, data_len, shape, n_dims, nullptr, 0, input, input_len, output, output_len, m, n, k);
}

int oxq_linear_forward_batch(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape, size_t n_dims,
                             const float *bias, size_t bias_len, const float *input, size_t input_len, float *output,
                             size_t output_len, size_t batch) {
    // QuantLinear::forward_batch: gemm with n = out_features = shape[0], k = in_features = shape[1]
    // (linear.rs:112-119), then the bias broadcast over the batch.
    const size_t out_features = (shape && n_dims > 0) ? shape[0] : 0;
    const size_t in_features = (shape && n_dims > 1) ? shape[1] : 0;
    return gemm_host(type, data, data_len, shape, n_dims, bias, bias_len, input, input_len, output, output_len, batch,
                     out_features, in_features);
}

int oxq_gemv(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape, size_t n_dims,
             const float *input, size_t input_len, float *output, size_t output_len) {
    size_t n_rows = 0, n_cols = 0;
    int st = tensor_dims(type, data_len, shape, n_dims, &n_rows, &n_cols);
    if (st != OXQ_OK) return st;
    if (input_len < n_cols) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_cols, input_len, "input shorter than n_cols");
    if (output_len < n_rows) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_rows, output_len, "output shorter than n_rows");
    const size_t shape2[2] = {n_rows, n_cols};
    return oxq_gemm(type, data, data_len, shape2, 2, input, n_cols, output, n_rows, 1, n_rows, n_cols);
}

// ---- weights resident in HBM --------------------------------------------

int oxq_weights_register(uint32_t type, size_t n_rows, size_t n_cols, const uint8_t *bytes, size_t len,
                         oxq_weights_t *handle) {
    if (!handle) return fail(OXQ_ERR_INTERNAL, 0, 0, "null handle pointer");
    *handle = nullptr;
    if (!known_type(type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "unsupported quantization type");
    const size_t bs = oxq_block_size(type), bb = oxq_block_bytes(type);
    const size_t need = n_rows * ((n_cols + bs - 1) / bs) * bb;
    if (len < need) return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, len, "weights buffer too small");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    oxq_weights *w = new (std::nothrow) oxq_weights{type, n_rows, n_cols, need, nullptr};
    if (!w) return fail(OXQ_ERR_INTERNAL, 0, 0, "out of host memory");
    hipError_t e = hipMalloc((void **)&w->dev, need ? need : 1);
    if (e == hipSuccess && need) e = hipMemcpy(w->dev, bytes, need, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        if (w->dev) (void)hipFree(w->dev);
        delete w;
        return fail_hip(e, "weights upload");
    }
    *handle = w;
    return OXQ_OK;
}

int oxq_weights_release(oxq_weights_t handle) {
    if (!handle) return OXQ_OK;
    if (handle->dev) (void)hipFree(handle->dev);
    delete handle;
    return OXQ_OK;
}

void *oxq_weights_device_ptr(oxq_weights_t handle) { return handle ? handle->dev : nullptr; }
size_t oxq_weights_nbytes(oxq_weights_t handle) { return handle ? handle->nbytes : 0; }

// ---- device-pointer route -------------------------------------------------

int oxq_quantize_q8_0_dev(const float *d_x, size_t n_total, uint8_t *d_out, void *stream) {
    if (n_total % 32 != 0)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, (n_total / 32 + 1) * 32, n_total, "length is not a multiple of 32");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_quantize_q8_0(d_x, n_total, d_out, (hipStream_t)stream));
    return OXQ_OK;
}

// ragged_ok: the entry point takes rows that end inside a block (the plain matvec / gemv / gemm, which skip the
// columns past n_cols as the reference does); the fused layers and the debug dumps want whole blocks.
static int check_dev_shape(uint32_t type, size_t n_rows, size_t n_cols, bool ragged_ok = false) {
    if (!known_type(type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "unsupported quantization type");
    const size_t bs = oxq_block_size(type);
    if (!ragged_ok && n_cols % bs != 0)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, bs, n_cols, "n_cols is not a multiple of the block size");
    if (n_rows > 0xFFFFFFFFull || n_cols > 0xFFFFFF00ull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFF00ull, n_rows, "dimension exceeds 2^32-257");
    return OXQ_OK;
}

int oxq_matvec_q8_fused_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_out,
                            size_t n_rows, size_t n_cols, int accumulate, void *stream) {
    int st = check_dev_shape(type, n_rows, n_cols, true);
    if (st != OXQ_OK) return st;
    if ((st = ensure_init()) != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_gemv_q8(type, gemv_args(d_weights, d_acts_q8, d_out, nullptr, n_rows, n_cols, accumulate ? 1 : 0),
                                (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_matvec_q8_fused_multi_dev(uint32_t type, size_t n_mats, const uint8_t *const *d_weights,
                                  const uint8_t *d_acts_q8, float *const *d_outs, size_t n_rows, size_t n_cols,
                                  int accumulate, void *stream) {
    int st = check_dev_shape(type, n_rows, n_cols, true);
    if (st != OXQ_OK) return st;
    if (n_mats == 0) return OXQ_OK;
    if (n_mats > 4) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 4, n_mats, "at most 4 matrices per call");
    if (!d_weights || !d_outs) return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer table");
    if ((st = ensure_init()) != OXQ_OK) return st;
    oxq::GemvArgs a = gemv_args(d_weights[0], d_acts_q8, d_outs[0], nullptr, n_rows, n_cols, accumulate ? 1 : 0);
    a.n_mats = (uint32_t)n_mats;
    for (size_t i = 1; i < n_mats; i++) {
        a.W_more[i - 1] = d_weights[i];
        a.out_more[i - 1] = d_outs[i];
    }
    OXQ_HIP(oxq::launch_gemv_q8(type, a, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_gemv_multi_dev(uint32_t type, size_t n_mats, const uint8_t *const *d_weights, const float *d_x,
                       float *const *d_outs, size_t n_rows, size_t n_cols, int accumulate, void *stream) {
    int st = check_dev_shape(type, n_rows, n_cols, true);
    if (st != OXQ_OK) return st;
    if (n_mats == 0) return OXQ_OK;
    if (n_mats > 4) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 4, n_mats, "at most 4 matrices per call");
    if (!d_weights || !d_outs) return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer table");
    if (!oxq::gemv_takes_f32(type, (uint32_t)n_cols))
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0, n_cols, "row too long for in-kernel activation quantization");
    if ((st = ensure_init()) != OXQ_OK) return st;
    oxq::GemvArgs a = gemv_args(d_weights[0], nullptr, d_outs[0], nullptr, n_rows, n_cols, accumulate ? 1 : 0);
    a.X = d_x;
    a.n_mats = (uint32_t)n_mats;
    for (size_t i = 1; i < n_mats; i++) {
        a.W_more[i - 1] = d_weights[i];
        a.out_more[i - 1] = d_outs[i];
    }
    OXQ_HIP(oxq::launch_gemv_q8(type, a, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_gemv_dev(uint32_t type, const uint8_t *d_weights, const float *d_x, float *d_out, size_t n_rows,
                 size_t n_cols, int accumulate, void *stream) {
    return oxq_gemv_multi_dev(type, 1, &d_weights, d_x, &d_out, n_rows, n_cols, accumulate, stream);
}

int oxq_gemv_f32_dev(uint32_t type, const uint8_t *d_weights, const float *d_x, const float *d_bias, float *d_out,
                     size_t n_rows, size_t n_cols, int accumulate, void *stream) {
    int st = check_dev_shape(type, n_rows, n_cols, true);
    if (st != OXQ_OK) return st;
    if (!oxq::gemv_f32_supported(type))
        return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "no fp32-activation kernel for this type");
    if (accumulate && d_bias) return fail(OXQ_ERR_INTERNAL, 0, 0, "accumulate and bias exclude each other");
    if ((st = ensure_init()) != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_gemv_f32(type, d_weights, d_x, d_out, accumulate ? d_out : d_bias, (uint32_t)n_rows,
                                 (uint32_t)n_cols, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_select_activation_route(int route) {
    if (route != OXQ_ROUTE_Q8 && route != OXQ_ROUTE_F32) return fail(OXQ_ERR_INTERNAL, 0, (size_t)route, "unknown route");
    g.act_route.store(route, std::memory_order_relaxed);
    return OXQ_OK;
}

int oxq_activation_route(void) { return g.act_route.load(std::memory_order_relaxed); }

int oxq_block_sums_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, int32_t *d_sums,
                       size_t n_rows, size_t n_cols, void *stream) {
    int st = check_dev_shape(type, n_rows, n_cols);
    if (st != OXQ_OK) return st;
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (n_rows == 0 || n_cols == 0) return OXQ_OK;
    std::lock_guard<std::mutex> lock(g.mu);
    if ((st = g.s_out.reserve(n_rows * sizeof(float))) != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_gemv_q8(type, gemv_args(d_weights, d_acts_q8, (float *)g.s_out.ptr, d_sums, n_rows, n_cols, 0),
                                (hipStream_t)stream));
    OXQ_HIP(hipStreamSynchronize((hipStream_t)stream));
    return OXQ_OK;
}

// The size depends on the shape alone, never on a tuning knob: a caller that sized its workspace once stays
// right whichever launch shape a later call takes.
size_t oxq_gemm_q8_workspace_bytes(uint32_t type, size_t m, size_t n, size_t k) {
    if (m > 0xFFFFFFFFull || n > 0xFFFFFFFFull || k > 0xFFFFFFFFull ||
        !oxq::gemm_tiles_supported(type, (uint32_t)m, (uint32_t)k))
        return 0;
    return oxq::gemm_workspace_bytes((uint32_t)m, (uint32_t)k, (uint32_t)n, type);
}

static int gemm_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_out, int32_t *d_sums,
                    size_t m, size_t n, size_t k, int accumulate, const float *d_bias, void *d_workspace,
                    size_t workspace_bytes, void *stream) {
    int st = check_dev_shape(type, n, k, true);
    if (st != OXQ_OK) return st;
    if (m > 0xFFFFFFFFull) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, m, "dimension exceeds 2^32-1");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (m == 0 || n == 0 || k == 0) return OXQ_OK;
    oxq::GemmArgs ga;
    ga.W = d_weights;
    ga.A = d_acts_q8;
    ga.out = d_out;
    ga.sums = d_sums;
    ga.workspace = nullptr;
    ga.m = (uint32_t)m;
    ga.n = (uint32_t)n;
    ga.k = (uint32_t)k;
    ga.accumulate = accumulate ? 1 : 0;
    ga.bias = d_bias;
    // one reading of the tuning knobs per call: tile kernel, or GEMV launches (which need no workspace)
    bool tiles = oxq::gemm_uses_tiles(type, (uint32_t)m, (uint32_t)n, (uint32_t)k);
    // a few rows fewer still pay on the few-token kernel, if the caller's workspace has the room (without one the
    // call would have to take the library's scratch and wait for the stream: the GEMV launches stay)
    if (!tiles && d_workspace && !d_sums && oxq::gemm_few_rows_pay(type, (uint32_t)m, (uint32_t)n, (uint32_t)k) &&
        workspace_bytes >= oxq::gemm_workspace_bytes((uint32_t)m, (uint32_t)k, (uint32_t)n, type) &&
        (reinterpret_cast<uintptr_t>(d_workspace) & 255) == 0)
        tiles = true;
    ga.by_rows = !tiles;
    const size_t need = tiles ? oxq::gemm_workspace_bytes((uint32_t)m, (uint32_t)k, (uint32_t)n, type) : 0;
    if (need && d_workspace) {
        if (workspace_bytes < need) return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, workspace_bytes, "workspace too small");
        if (reinterpret_cast<uintptr_t>(d_workspace) & 255)
            return fail(OXQ_ERR_KERNEL, 256, reinterpret_cast<uintptr_t>(d_workspace) & 255, "workspace must be 256-byte aligned");
        ga.workspace = (uint8_t *)d_workspace;
        ga.workspace_bytes = workspace_bytes;
        OXQ_HIP(oxq::launch_gemm_q8(type, ga, (hipStream_t)stream));
        return OXQ_OK;
    }
    if (need) {
        // Library-owned scratch: calls serialise on the lock and wait for the stream, because
        // the scratch is shared.
        std::lock_guard<std::mutex> lock(g.mu);
        if ((st = g.s_work.reserve(need)) != OXQ_OK) return st;
        ga.workspace = (uint8_t *)g.s_work.ptr;
        ga.workspace_bytes = need;
        OXQ_HIP(oxq::launch_gemm_q8(type, ga, (hipStream_t)stream));
        OXQ_HIP(hipStreamSynchronize((hipStream_t)stream));
        return OXQ_OK;
    }
    OXQ_HIP(oxq::launch_gemm_q8(type, ga, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_gemm_q8_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_out, size_t m,
                    size_t n, size_t k, int accumulate, void *d_workspace, size_t workspace_bytes, void *stream) {
    return gemm_dev(type, d_weights, d_acts_q8, d_out, nullptr, m, n, k, accumulate, nullptr, d_workspace, workspace_bytes,
                    stream);
}

size_t oxq_gemm_q8_static_max_workspace_bytes(void) { return STATIC_SCRATCH_BYTES; }

int oxq_gemm_q8_static_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_out, size_t m,
                           size_t n, size_t k, int accumulate, void *stream) {
    int st = check_dev_shape(type, n, k, true);
    if (st != OXQ_OK) return st;
    if (m > 0xFFFFFFFFull) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, m, "dimension exceeds 2^32-1");
    // no lazy initialisation here: that would be the one path of this call that allocates
    // the array of the device the calling thread has current (where the stream's work runs), not of the last one
    // oxq_init was called for: each device holds its own copy
    int device = -1;
    if (!g.initialised.load(std::memory_order_acquire) || hipGetDevice(&device) != hipSuccess || device < 0 ||
        device >= MAX_DEVICES || !static_scratch_ptr[device])
        return fail(OXQ_ERR_NO_DEVICE, 0, 0,
                    "call oxq_init for this device first: this entry point sets nothing up by itself");
    if (m == 0 || n == 0 || k == 0) return OXQ_OK;
    const bool tiles = oxq::gemm_uses_tiles(type, (uint32_t)m, (uint32_t)n, (uint32_t)k) ||
                       (oxq::gemm_few_rows_pay(type, (uint32_t)m, (uint32_t)n, (uint32_t)k) &&
                        oxq::gemm_workspace_bytes((uint32_t)m, (uint32_t)k, (uint32_t)n, type) <= STATIC_SCRATCH_BYTES);
    const size_t need = tiles ? oxq::gemm_workspace_bytes((uint32_t)m, (uint32_t)k, (uint32_t)n, type) : 0;
    if (need > STATIC_SCRATCH_BYTES)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, STATIC_SCRATCH_BYTES,
                    "shape needs more workspace than the static scratch holds: use oxq_gemm_q8_dev with a workspace");
    oxq::GemmArgs ga;
    ga.W = d_weights;
    ga.A = d_acts_q8;
    ga.out = d_out;
    ga.sums = nullptr;
    ga.workspace_bytes = tiles ? STATIC_SCRATCH_BYTES : 0;
    ga.workspace = tiles ? static_scratch_ptr[device] : nullptr;    // every byte the tile kernel reads is written
    ga.by_rows = !tiles;                                            // by the preparation kernel of this same call
    ga.m = (uint32_t)m;
    ga.n = (uint32_t)n;
    ga.k = (uint32_t)k;
    ga.accumulate = accumulate ? 1 : 0;
    OXQ_HIP(oxq::launch_gemm_q8(type, ga, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_gemm_block_sums_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_out,
                            int32_t *d_sums, size_t m, size_t n, size_t k, void *d_workspace, size_t workspace_bytes,
                            void *stream) {
    if (!d_sums) return fail(OXQ_ERR_INTERNAL, 0, 0, "null sums");
    if (m > 0xFFFFFFFFull || n > 0xFFFFFFFFull || k > 0xFFFFFFFFull ||
        !oxq::gemm_uses_tiles(type, (uint32_t)m, (uint32_t)n, (uint32_t)k))
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0, m, "no tile kernel for this type/shape");
    return gemm_dev(type, d_weights, d_acts_q8, d_out, d_sums, m, n, k, 0, nullptr, d_workspace, workspace_bytes, stream);
}

size_t oxq_moe_gemm_q8_workspace_bytes(uint32_t type, size_t total_rows, size_t n, size_t k) {
    if (total_rows > 0x7FFFFFFFull || k > 0xFFFFFFFFull || n > 0xFFFFFFFFull ||
        !oxq::gemm_tiles_supported(type, (uint32_t)total_rows, (uint32_t)k))
        return 0;
    return oxq::gemm_grouped_workspace_bytes((uint32_t)total_rows, (uint32_t)k, (uint32_t)n, type);
}

// prep_state: what an earlier call of the same sequence left in the workspace (GemmArgs::Prepared), or null.
static int moe_gemm_impl(uint32_t type, const uint8_t *d_weights, size_t expert_stride_bytes, size_t n_experts,
                         const uint8_t *d_acts_q8, const int32_t *d_row_offsets, size_t total_rows,
                         size_t max_rows_per_expert, float *d_out, int32_t *d_sums, size_t n, size_t k, int accumulate,
                         void *d_workspace, size_t workspace_bytes, void *stream,
                         oxq::GemmArgs::Prepared *prep_state, oxq::GemmArgs::SplitSums *defer_reduce = nullptr) {
    int st = check_dev_shape(type, n, k);
    if (st != OXQ_OK) return st;
    if (total_rows > 0x7FFFFFFFull || n_experts > 65535)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0x7FFFFFFFull, total_rows, "too many rows or experts");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (total_rows == 0 || n_experts == 0 || n == 0 || k == 0) return OXQ_OK;
    if (!d_row_offsets) return fail(OXQ_ERR_INTERNAL, 0, 0, "null row offsets");
    const size_t row_bytes = k / oxq_block_size(type) * oxq_block_bytes(type);
    if (expert_stride_bytes < n * row_bytes)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, n * row_bytes, expert_stride_bytes, "expert stride smaller than one expert");
    const size_t need = oxq_moe_gemm_q8_workspace_bytes(type, total_rows, n, k);
    if (need == 0) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0, k, "no grouped kernel for this type/shape");
    if (!d_workspace || workspace_bytes < need)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, d_workspace ? workspace_bytes : 0, "workspace too small");
    if (reinterpret_cast<uintptr_t>(d_workspace) & 255)
        return fail(OXQ_ERR_KERNEL, 256, reinterpret_cast<uintptr_t>(d_workspace) & 255, "workspace must be 256-byte aligned");
    oxq::GemmArgs ga;
    ga.W = d_weights;
    ga.A = d_acts_q8;
    ga.out = d_out;
    ga.sums = d_sums;
    ga.workspace = (uint8_t *)d_workspace;
    ga.workspace_bytes = workspace_bytes;
    ga.m = (uint32_t)total_rows;
    ga.n = (uint32_t)n;
    ga.k = (uint32_t)k;
    ga.accumulate = accumulate ? 1 : 0;
    ga.offsets = d_row_offsets;
    ga.n_experts = (uint32_t)n_experts;
    ga.max_rows = (uint32_t)(max_rows_per_expert ? (max_rows_per_expert < total_rows ? max_rows_per_expert : total_rows)
                                                 : total_rows);
    ga.shape_rows = ga.max_rows;
    if (!max_rows_per_expert) {
        // Row counts known only on the device: the grid covers the worst case (one expert takes every
        // row; tiles past an expert's rows exit at once), the tile shape is chosen for twice the mean.
        const size_t mean = (total_rows + n_experts - 1) / n_experts;
        ga.shape_rows = (uint32_t)(2 * mean < total_rows ? 2 * mean : total_rows);
    }
    ga.w_stride = expert_stride_bytes;
    ga.prep_state = prep_state;
    ga.defer_reduce = defer_reduce;
    OXQ_HIP(oxq::launch_gemm_q8(type, ga, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_moe_gemm_q8_dev(uint32_t type, const uint8_t *d_weights, size_t expert_stride_bytes, size_t n_experts,
                        const uint8_t *d_acts_q8, const int32_t *d_row_offsets, size_t total_rows,
                        size_t max_rows_per_expert, float *d_out, int32_t *d_sums, size_t n, size_t k, int accumulate,
                        void *d_workspace, size_t workspace_bytes, void *stream) {
    return moe_gemm_impl(type, d_weights, expert_stride_bytes, n_experts, d_acts_q8, d_row_offsets, total_rows,
                         max_rows_per_expert, d_out, d_sums, n, k, accumulate, d_workspace, workspace_bytes, stream, nullptr);
}

int oxq_gemm_scaled_sums_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_out,
                             int32_t *d_sums, size_t m, size_t n, size_t k, void *d_workspace, size_t workspace_bytes,
                             void *stream) {
    if (!d_sums) return fail(OXQ_ERR_INTERNAL, 0, 0, "null sums");
    int st = check_dev_shape(type, n, k, true);
    if (st != OXQ_OK) return st;
    if (m == 0 || m > 0xFFFFFFFFull || !oxq::gemm_prefill_supported(type, (uint32_t)m, (uint32_t)n, (uint32_t)k))
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0, m, "no prefill kernel for this type/shape");
    if ((st = ensure_init()) != OXQ_OK) return st;
    const size_t need = oxq::gemm_prefill_workspace_bytes((uint32_t)m, (uint32_t)k);
    if (!d_workspace || workspace_bytes < need)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, d_workspace ? workspace_bytes : 0, "workspace too small");
    if (reinterpret_cast<uintptr_t>(d_workspace) & 255)
        return fail(OXQ_ERR_KERNEL, 256, reinterpret_cast<uintptr_t>(d_workspace) & 255, "workspace must be 256-byte aligned");
    oxq::GemmArgs ga;
    ga.W = d_weights;
    ga.A = d_acts_q8;
    ga.out = d_out;
    ga.sums = d_sums;
    ga.scaled_sums = true;
    ga.workspace = (uint8_t *)d_workspace;
    ga.workspace_bytes = workspace_bytes;
    ga.m = (uint32_t)m;
    ga.n = (uint32_t)n;
    ga.k = (uint32_t)k;
    ga.accumulate = 0;
    OXQ_HIP(oxq::launch_gemm_q8(type, ga, (hipStream_t)stream));
    return OXQ_OK;
}

// ---- the callers' side: QuantLinear, SwiGLU feed-forward, RMSNorm ------------------------

static int check_lora(const oxq_lora *lora) {
    if (!lora || lora->rank == 0) return OXQ_OK;
    if (!lora->d_a || !lora->d_b || !lora->d_r) return fail(OXQ_ERR_INTERNAL, 0, 0, "LoRA adapter with a null pointer");
    if (lora->rank > 0xFFFFFFFFull) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, lora->rank, "rank exceeds 2^32-1");
    return OXQ_OK;
}

int oxq_lora_apply_dev(const oxq_lora *lora, const float *d_x, float *d_out, size_t out_features, size_t in_features,
                       void *stream) {
    int st = check_lora(lora);
    if (st != OXQ_OK) return st;
    if (!lora || lora->rank == 0) return OXQ_OK;
    if (out_features > 0xFFFFFFFFull || in_features > 0xFFFFFFFFull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, out_features, "dimension exceeds 2^32-1");
    if ((st = ensure_init()) != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_lora_apply(lora->d_a, lora->d_b, lora->d_r, (uint32_t)lora->rank, lora->scale, d_x, d_out,
                                   (uint32_t)out_features, (uint32_t)in_features, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_linear_forward_dev(uint32_t type, const uint8_t *d_weights, const float *d_x, const uint8_t *d_acts_q8,
                           const float *d_bias, const oxq_lora *lora, float *d_out, size_t out_features,
                           size_t in_features, void *stream) {
    int st = check_dev_shape(type, out_features, in_features);
    if (st != OXQ_OK) return st;
    if ((st = check_lora(lora)) != OXQ_OK) return st;
    const bool has_lora = lora && lora->rank;
    if (!d_acts_q8 && !d_x) return fail(OXQ_ERR_INTERNAL, 0, 0, "neither fp32 nor Q8_0 activations given");
    if (has_lora && !d_x) return fail(OXQ_ERR_INTERNAL, 0, 0, "LoRA needs the fp32 input");
    if (!d_acts_q8 && g.act_route.load(std::memory_order_relaxed) == OXQ_ROUTE_F32) {
        // QuantLinear::forward as the reference computes it: gemv on the fp32 input, then bias, then LoRA
        if (!oxq::gemv_f32_supported(type))
            return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "no fp32-activation kernel for this type (OXQ_ROUTE_F32)");
        if ((st = ensure_init()) != OXQ_OK) return st;
        OXQ_HIP(oxq::launch_gemv_f32(type, d_weights, d_x, d_out, d_bias, (uint32_t)out_features, (uint32_t)in_features,
                                     (hipStream_t)stream));
        if (has_lora) return oxq_lora_apply_dev(lora, d_x, d_out, out_features, in_features, stream);
        return OXQ_OK;
    }
    if (!d_acts_q8 && !oxq::gemv_takes_f32(type, (uint32_t)in_features))
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0, in_features, "row too long for in-kernel activation quantization");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (out_features == 0 || in_features == 0) return OXQ_OK;
    oxq::GemvArgs a = gemv_args(d_weights, d_acts_q8, d_out, nullptr, out_features, in_features, 0);
    if (!d_acts_q8) a.X = d_x;
    a.bias = d_bias;
    OXQ_HIP(oxq::launch_gemv_q8(type, a, (hipStream_t)stream));
    if (has_lora) return oxq_lora_apply_dev(lora, d_x, d_out, out_features, in_features, stream);
    return OXQ_OK;
}

int oxq_linear_forward_multi_dev(uint32_t type, size_t n_mats, const uint8_t *const *d_weights,
                                 const uint8_t *d_acts_q8, const float *const *d_biases, float *const *d_outs,
                                 const size_t *out_features, size_t in_features, void *stream) {
    if (n_mats == 0) return OXQ_OK;
    if (n_mats > 4) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 4, n_mats, "at most 4 matrices per call");
    if (!d_weights || !d_outs || !out_features) return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer table");
    int st;
    for (size_t i = 0; i < n_mats; i++) {
        if ((st = check_dev_shape(type, out_features[i], in_features)) != OXQ_OK) return st;
        if (out_features[i] == 0) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 1, 0, "a matrix of the call has no rows");
    }
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (in_features == 0) return OXQ_OK;
    oxq::GemvArgs a = gemv_args(d_weights[0], d_acts_q8, d_outs[0], nullptr, out_features[0], in_features, 0);
    a.bias = d_biases ? d_biases[0] : nullptr;
    a.n_mats = (uint32_t)n_mats;
    for (size_t i = 1; i < n_mats; i++) {
        a.W_more[i - 1] = d_weights[i];
        a.out_more[i - 1] = d_outs[i];
        a.bias_more[i - 1] = d_biases ? d_biases[i] : nullptr;
        a.n_rows_more[i - 1] = (uint32_t)out_features[i];
    }
    OXQ_HIP(oxq::launch_gemv_q8(type, a, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_linear_forward_batch_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8,
                                 const float *d_bias, float *d_out, size_t batch, size_t out_features,
                                 size_t in_features, void *d_workspace, size_t workspace_bytes, void *stream) {
    return gemm_dev(type, d_weights, d_acts_q8, d_out, nullptr, batch, out_features, in_features, 0, d_bias,
                    d_workspace, workspace_bytes, stream);
}

int oxq_swiglu_quantize_q8_0_dev(const float *d_gate, const float *d_up, size_t n_total, float *d_h,
                                 uint8_t *d_out_q8, void *stream) {
    if (n_total % 32 != 0)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, (n_total / 32 + 1) * 32, n_total, "length is not a multiple of 32");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_swiglu_quantize(d_gate, d_up, n_total, d_h, d_out_q8, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_rmsnorm_quantize_q8_0_dev(const float *d_x, const float *d_weight, float eps, size_t rows, size_t n,
                                  float *d_y, uint8_t *d_out_q8, void *stream) {
    if (n % 32 != 0) return fail(OXQ_ERR_DIMENSION_MISMATCH, (n / 32 + 1) * 32, n, "row length is not a multiple of 32");
    if (n > 0xFFFFFFFFull || rows > 0x7FFFFFFFull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, n, "dimension exceeds the launch limits");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_rmsnorm_quantize(d_x, d_weight, eps, rows, (uint32_t)n, d_y, d_out_q8, (hipStream_t)stream));
    return OXQ_OK;
}

size_t oxq_ffn_workspace_bytes(size_t hidden, size_t intermediate) {
    (void)hidden;
    // gate fp32 | up fp32 | Q8_0 blocks of silu(gate) * up, each piece 256-byte aligned
    const size_t f = (intermediate * sizeof(float) + 255) & ~(size_t)255;
    return 2 * f + ((intermediate / 32 * 34 + 255) & ~(size_t)255);
}

int oxq_ffn_gate_up_swiglu_q8_dev(uint32_t type, const uint8_t *d_gate, const uint8_t *d_up, const uint8_t *d_acts_q8,
                                  float *d_h, uint8_t *d_out_q8, size_t intermediate, size_t hidden, void *stream) {
    int st;
    if ((st = check_dev_shape(type, intermediate, hidden)) != OXQ_OK) return st;
    if (intermediate % 32 != 0)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 32, intermediate, "intermediate size is not a multiple of 32");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (hidden == 0 || intermediate == 0) return OXQ_OK;
    hipError_t e = oxq::launch_gate_up_swiglu(type, d_gate, d_up, d_acts_q8, d_out_q8, d_h, (uint32_t)intermediate,
                                              (uint32_t)hidden, (hipStream_t)stream);
    if (e == hipErrorNotSupported) {
        (void)hipGetLastError();
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0, hidden, "no fused gate/up kernel for this type and row length");
    }
    OXQ_HIP(e);
    return OXQ_OK;
}

int oxq_set_ffn_fusion(int enabled) {
    g.fuse_swiglu.store(enabled != 0, std::memory_order_relaxed);
    return OXQ_OK;
}

int oxq_ffn_swiglu_dev(uint32_t gate_type, const uint8_t *d_gate, uint32_t up_type, const uint8_t *d_up,
                       uint32_t down_type, const uint8_t *d_down, const uint8_t *d_acts_q8, float *d_out, size_t hidden,
                       size_t intermediate, void *d_workspace, size_t workspace_bytes, void *stream) {
    int st;
    if ((st = check_dev_shape(gate_type, intermediate, hidden)) != OXQ_OK) return st;
    if ((st = check_dev_shape(up_type, intermediate, hidden)) != OXQ_OK) return st;
    if ((st = check_dev_shape(down_type, hidden, intermediate)) != OXQ_OK) return st;
    if (intermediate % 32 != 0)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 32, intermediate, "intermediate size is not a multiple of 32");
    const size_t need = oxq_ffn_workspace_bytes(hidden, intermediate);
    if (!d_workspace || workspace_bytes < need)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, d_workspace ? workspace_bytes : 0, "workspace too small");
    if (reinterpret_cast<uintptr_t>(d_workspace) & 255)
        return fail(OXQ_ERR_KERNEL, 256, reinterpret_cast<uintptr_t>(d_workspace) & 255, "workspace must be 256-byte aligned");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (hidden == 0 || intermediate == 0) return OXQ_OK;
    const size_t f = (intermediate * sizeof(float) + 255) & ~(size_t)255;
    float *gate = (float *)d_workspace, *up = (float *)((uint8_t *)d_workspace + f);
    uint8_t *hq = (uint8_t *)d_workspace + 2 * f;
    hipStream_t s = (hipStream_t)stream;
    if (gate_type == up_type && g.fuse_swiglu.load(std::memory_order_relaxed)) {  // both projections, SwiGLU and the quantizer of h in one launch
        hipError_t e = oxq::launch_gate_up_swiglu(gate_type, d_gate, d_up, d_acts_q8, hq, nullptr, (uint32_t)intermediate,
                                                  (uint32_t)hidden, s);
        if (e == hipSuccess) {
            OXQ_HIP(oxq::launch_gemv_q8(down_type, gemv_args(d_down, hq, d_out, nullptr, hidden, intermediate, 0), s));
            return OXQ_OK;
        }
        if (e != hipErrorNotSupported) return fail_hip(e, "launch_gate_up_swiglu");
        (void)hipGetLastError();
    }
    if (gate_type == up_type) {  // one pass of the launch machinery over both matrices
        oxq::GemvArgs a = gemv_args(d_gate, d_acts_q8, gate, nullptr, intermediate, hidden, 0);
        a.n_mats = 2;
        a.W_more[0] = d_up;
        a.out_more[0] = up;
        OXQ_HIP(oxq::launch_gemv_q8(gate_type, a, s));
    } else {
        OXQ_HIP(oxq::launch_gemv_q8(gate_type, gemv_args(d_gate, d_acts_q8, gate, nullptr, intermediate, hidden, 0), s));
        OXQ_HIP(oxq::launch_gemv_q8(up_type, gemv_args(d_up, d_acts_q8, up, nullptr, intermediate, hidden, 0), s));
    }
    OXQ_HIP(oxq::launch_swiglu_quantize(gate, up, intermediate, nullptr, hq, s));
    OXQ_HIP(oxq::launch_gemv_q8(down_type, gemv_args(d_down, hq, d_out, nullptr, hidden, intermediate, 0), s));
    return OXQ_OK;
}

// ---- MoeFfn::forward on the device, experts in a quantized format ----

namespace {
struct MoeFfnLayout {
    size_t acts, gate, up, hq, y, gemm, total;
};
size_t align256(size_t n) { return (n + 255) & ~(size_t)255; }
bool moe_ffn_layout(uint32_t gate_type, uint32_t up_type, uint32_t down_type, size_t pairs, size_t hidden, size_t inter,
                    MoeFfnLayout *l) {
    const size_t g1 = oxq_moe_gemm_q8_workspace_bytes(gate_type, pairs, inter, hidden);
    const size_t g2 = oxq_moe_gemm_q8_workspace_bytes(up_type, pairs, inter, hidden);
    const size_t g3 = oxq_moe_gemm_q8_workspace_bytes(down_type, pairs, hidden, inter);
    if (g1 == 0 || g2 == 0 || g3 == 0 || hidden % 32 || inter % 32) return false;
    size_t off = 0;
    l->acts = off; off += align256(pairs * (hidden / 32) * 34);
    l->gate = off; off += align256(pairs * inter * sizeof(float));
    l->up = off; off += align256(pairs * inter * sizeof(float));
    l->hq = off; off += align256(pairs * (inter / 32) * 34);
    l->y = off; off += align256(pairs * hidden * sizeof(float));
    l->gemm = off; off += align256(g1 > g2 ? (g1 > g3 ? g1 : g3) : (g2 > g3 ? g2 : g3));
    l->total = off;
    return true;
}
}  // namespace

int oxq_moe_route_dev(const float *d_router, const float *d_x, size_t n_tokens, size_t n_experts, size_t hidden,
                      size_t top_k, int32_t *d_experts, float *d_weights, int32_t *d_row_offsets,
                      int32_t *d_pair_token, int32_t *d_token_rows, void *stream) {
    if (top_k == 0) return fail(OXQ_ERR_KERNEL, 1, 0, "MoeFfn top_k must be >= 1");  // moe.rs:168-172
    if (n_experts > 1024) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 1024, n_experts, "at most 1024 experts");
    const size_t k = top_k < n_experts ? top_k : n_experts;  // moe.rs:233
    if (n_tokens * k > 0x7FFFFFFFull || hidden > 0xFFFFFFFFull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0x7FFFFFFFull, n_tokens * k, "too many (token, expert) pairs");
    int st;
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (n_tokens == 0 || n_experts == 0) return OXQ_OK;
    if (!d_router || !d_x || !d_experts || !d_weights || !d_row_offsets || !d_pair_token || !d_token_rows)
        return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer");
    OXQ_HIP(oxq::launch_moe_route(d_router, d_x, d_experts, d_weights, (uint32_t)n_tokens, (uint32_t)n_experts,
                                  (uint32_t)hidden, (uint32_t)k, d_row_offsets, d_pair_token, d_token_rows,
                                  (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_moe_gather_quantize_q8_0_dev(const float *d_x, const int32_t *d_pair_token, size_t n_pairs, size_t hidden,
                                     uint8_t *d_out_q8, void *stream) {
    if (hidden % 32) return fail(OXQ_ERR_DIMENSION_MISMATCH, 32, hidden, "row length must be a multiple of 32");
    if (n_pairs > 0x7FFFFFFFull || hidden > 0xFFFFFFFFull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0x7FFFFFFFull, n_pairs, "too many rows");
    int st;
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (n_pairs == 0 || hidden == 0) return OXQ_OK;
    OXQ_HIP(oxq::launch_moe_gather_quantize(d_x, d_pair_token, d_out_q8, n_pairs, (uint32_t)hidden, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_moe_combine_dev(const float *d_y_pairs, const int32_t *d_token_rows, const float *d_weights, size_t n_tokens,
                        size_t top_k, size_t hidden, float *d_out, void *stream) {
    if (n_tokens * top_k > 0x7FFFFFFFull || hidden > 0xFFFFFFFFull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0x7FFFFFFFull, n_tokens * top_k, "too many rows");
    int st;
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (n_tokens == 0 || hidden == 0) return OXQ_OK;
    OXQ_HIP(oxq::launch_moe_combine(d_y_pairs, d_token_rows, d_weights, d_out, (uint32_t)n_tokens, (uint32_t)top_k,
                                    (uint32_t)hidden, (hipStream_t)stream));
    return OXQ_OK;
}

size_t oxq_moe_ffn_workspace_bytes(uint32_t gate_type, uint32_t up_type, uint32_t down_type, size_t n_pairs,
                                   size_t hidden, size_t intermediate) {
    MoeFfnLayout l;
    return moe_ffn_layout(gate_type, up_type, down_type, n_pairs, hidden, intermediate, &l) ? l.total : 0;
}

namespace {
// acts_ready: the grouped Q8_0 activation rows already sit at their place in the workspace (the one-token
// router launch wrote them); otherwise the gather launch comes first.
int moe_ffn_impl(uint32_t gate_type, const uint8_t *d_gate, size_t gate_stride_bytes, uint32_t up_type,
                 const uint8_t *d_up, size_t up_stride_bytes, uint32_t down_type, const uint8_t *d_down,
                 size_t down_stride_bytes, size_t n_experts, const float *d_x, size_t n_tokens, size_t top_k,
                 const int32_t *d_row_offsets, const int32_t *d_pair_token, const int32_t *d_token_rows,
                 const float *d_weights, size_t max_rows_per_expert, float *d_out, size_t hidden, size_t intermediate,
                 void *d_workspace, size_t workspace_bytes, void *stream, bool acts_ready) {
    int st;
    if ((st = check_dev_shape(gate_type, intermediate, hidden)) != OXQ_OK) return st;
    if ((st = check_dev_shape(up_type, intermediate, hidden)) != OXQ_OK) return st;
    if ((st = check_dev_shape(down_type, hidden, intermediate)) != OXQ_OK) return st;
    if (top_k == 0) return fail(OXQ_ERR_KERNEL, 1, 0, "MoeFfn top_k must be >= 1");  // moe.rs:168-172
    const size_t pairs = n_tokens * top_k;
    if (pairs > 0x7FFFFFFFull) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0x7FFFFFFFull, pairs, "too many rows");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (pairs == 0 || n_experts == 0 || hidden == 0 || intermediate == 0) return OXQ_OK;
    if (!d_row_offsets || !d_pair_token || !d_token_rows || !d_weights)
        return fail(OXQ_ERR_INTERNAL, 0, 0, "null routing table");
    MoeFfnLayout l;
    if (!moe_ffn_layout(gate_type, up_type, down_type, pairs, hidden, intermediate, &l))
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 256, hidden, "no grouped kernel for this type/shape");
    if (!d_workspace || workspace_bytes < l.total)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, l.total, d_workspace ? workspace_bytes : 0, "workspace too small");
    if (reinterpret_cast<uintptr_t>(d_workspace) & 255)
        return fail(OXQ_ERR_KERNEL, 256, reinterpret_cast<uintptr_t>(d_workspace) & 255,
                    "workspace must be 256-byte aligned");
    uint8_t *ws = (uint8_t *)d_workspace;
    uint8_t *acts = ws + l.acts, *hq = ws + l.hq;
    float *gate = (float *)(ws + l.gate), *up = (float *)(ws + l.up), *y = (float *)(ws + l.y);
    hipStream_t s = (hipStream_t)stream;
    if (!acts_ready) OXQ_HIP(oxq::launch_moe_gather_quantize(d_x, d_pair_token, acts, pairs, (uint32_t)hidden, s));
    const size_t gws = workspace_bytes - l.gemm;
    // A handful of rows (one token's top-k, a decode batch of a few): gate, up, SwiGLU and the quantizer of h in one
    // GEMV launch over the rows' experts, where the format and row length have that kernel (the bits of the
    // separate launches below).
    bool fused = false;
    if (pairs <= oxq::grouped_gemv_max_rows(n_experts) && gate_type == up_type && n_experts <= 4096 && intermediate % 32 == 0 &&
        oxq::g_gemm_variant.load(std::memory_order_relaxed) == 0 && g.fuse_swiglu.load(std::memory_order_relaxed)) {
        oxq::GateUpGroups grp;
        grp.offsets = d_row_offsets;
        grp.n_groups = (uint32_t)n_experts;
        grp.n_pairs = (uint32_t)pairs;
        grp.wg_stride = gate_stride_bytes;
        grp.wu_stride = up_stride_bytes;
        const hipError_t e = oxq::launch_gate_up_swiglu(gate_type, d_gate, d_up, acts, hq, nullptr, (uint32_t)intermediate,
                                                        (uint32_t)hidden, s, grp);
        if (e == hipSuccess) fused = true;
        else if (e != hipErrorNotSupported) return fail_hip(e, "launch_gate_up_swiglu (grouped)");
    }
    if (!fused) {
    // up reads the activations that gate re-laid out in the workspace, if gate's launch did that and in up's order
    oxq::GemmArgs::Prepared prep;
    if ((st = moe_gemm_impl(gate_type, d_gate, gate_stride_bytes, n_experts, acts, d_row_offsets, pairs,
                            max_rows_per_expert, gate, nullptr, intermediate, hidden, 0, ws + l.gemm, gws, stream,
                            &prep)) != OXQ_OK)
        return st;
    if ((st = moe_gemm_impl(up_type, d_up, up_stride_bytes, n_experts, acts, d_row_offsets, pairs, max_rows_per_expert, up,
                            nullptr, intermediate, hidden, 0, ws + l.gemm, gws, stream, &prep)) != OXQ_OK)
        return st;
    OXQ_HIP(oxq::launch_swiglu_quantize(gate, up, pairs * intermediate, nullptr, hq, s));
    }
    // where the down matmul splits k it leaves the halves' sums for the combine launch to add
    oxq::GemmArgs::SplitSums halves;
    if ((st = moe_gemm_impl(down_type, d_down, down_stride_bytes, n_experts, hq, d_row_offsets, pairs, max_rows_per_expert,
                            y, nullptr, hidden, intermediate, 0, ws + l.gemm, gws, stream, nullptr, &halves)) != OXQ_OK)
        return st;
    if (halves.splits > 1)
        OXQ_HIP(oxq::launch_moe_combine(halves.partial, d_token_rows, d_weights, d_out, (uint32_t)n_tokens, (uint32_t)top_k,
                                        (uint32_t)hidden, s, halves.splits, pairs * hidden));
    else
        OXQ_HIP(oxq::launch_moe_combine(y, d_token_rows, d_weights, d_out, (uint32_t)n_tokens, (uint32_t)top_k,
                                        (uint32_t)hidden, s));
    return OXQ_OK;
}

// Tables of the layer in front of the feed-forward workspace: experts | weights | offsets | pair_token | token_rows.
struct MoeTables {
    size_t experts, weights, offsets, pair_token, token_rows, ffn, total;
};
bool moe_forward_layout(uint32_t gate_type, uint32_t up_type, uint32_t down_type, size_t n_tokens, size_t k,
                        size_t n_experts, size_t hidden, size_t inter, MoeTables *t, MoeFfnLayout *l) {
    const size_t pairs = n_tokens * k;
    if (!moe_ffn_layout(gate_type, up_type, down_type, pairs, hidden, inter, l)) return false;
    size_t off = 0;
    t->experts = off; off += align256(pairs * 4);
    t->weights = off; off += align256(pairs * 4);
    t->offsets = off; off += align256((n_experts + 1) * 4);
    t->pair_token = off; off += align256(pairs * 4);
    t->token_rows = off; off += align256(pairs * 4);
    t->ffn = off;
    t->total = off + l->total;
    return true;
}
}  // namespace

int oxq_moe_ffn_dev(uint32_t gate_type, const uint8_t *d_gate, size_t gate_stride_bytes, uint32_t up_type,
                    const uint8_t *d_up, size_t up_stride_bytes, uint32_t down_type, const uint8_t *d_down,
                    size_t down_stride_bytes, size_t n_experts, const float *d_x, size_t n_tokens, size_t top_k,
                    const int32_t *d_row_offsets, const int32_t *d_pair_token, const int32_t *d_token_rows,
                    const float *d_weights, size_t max_rows_per_expert, float *d_out, size_t hidden,
                    size_t intermediate, void *d_workspace, size_t workspace_bytes, void *stream) {
    return moe_ffn_impl(gate_type, d_gate, gate_stride_bytes, up_type, d_up, up_stride_bytes, down_type, d_down,
                        down_stride_bytes, n_experts, d_x, n_tokens, top_k, d_row_offsets, d_pair_token, d_token_rows,
                        d_weights, max_rows_per_expert, d_out, hidden, intermediate, d_workspace, workspace_bytes, stream,
                        false);
}

size_t oxq_moe_forward_workspace_bytes(uint32_t gate_type, uint32_t up_type, uint32_t down_type, size_t n_tokens,
                                       size_t top_k, size_t n_experts, size_t hidden, size_t intermediate) {
    MoeTables t;
    MoeFfnLayout l;
    const size_t k = top_k < n_experts ? top_k : n_experts;
    return moe_forward_layout(gate_type, up_type, down_type, n_tokens, k, n_experts, hidden, intermediate, &t, &l)
               ? t.total
               : 0;
}

int oxq_moe_forward_dev(uint32_t gate_type, const uint8_t *d_gate, size_t gate_stride_bytes, uint32_t up_type,
                        const uint8_t *d_up, size_t up_stride_bytes, uint32_t down_type, const uint8_t *d_down,
                        size_t down_stride_bytes, size_t n_experts, const float *d_router, const float *d_x,
                        size_t n_tokens, size_t top_k, float *d_out, size_t hidden, size_t intermediate,
                        void *d_workspace, size_t workspace_bytes, void *stream) {
    int st;
    if ((st = check_dev_shape(gate_type, intermediate, hidden)) != OXQ_OK) return st;
    if ((st = check_dev_shape(up_type, intermediate, hidden)) != OXQ_OK) return st;
    if ((st = check_dev_shape(down_type, hidden, intermediate)) != OXQ_OK) return st;
    if (top_k == 0) return fail(OXQ_ERR_KERNEL, 1, 0, "MoeFfn top_k must be >= 1");  // moe.rs:168-172
    if (n_experts > 1024) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 1024, n_experts, "at most 1024 experts");
    const size_t k = top_k < n_experts ? top_k : n_experts;  // moe.rs:233
    if (n_tokens * k > 0x7FFFFFFFull || hidden > 0xFFFFFFFFull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0x7FFFFFFFull, n_tokens * k, "too many (token, expert) pairs");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (n_tokens == 0 || hidden == 0) return OXQ_OK;
    if (!d_x || !d_out) return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer");
    hipStream_t s = (hipStream_t)stream;
    if (n_experts == 0 || intermediate == 0) {  // no expert to add: the zeroed output (moe.rs:240-242)
        OXQ_HIP(oxq::launch_fill_zero(d_out, n_tokens * hidden, s));
        return OXQ_OK;
    }
    if (!d_router || !d_gate || !d_up || !d_down) return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer");
    MoeTables t;
    MoeFfnLayout l;
    if (!moe_forward_layout(gate_type, up_type, down_type, n_tokens, k, n_experts, hidden, intermediate, &t, &l))
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 256, hidden, "no grouped kernel for this type/shape");
    if (!d_workspace || workspace_bytes < t.total)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, t.total, d_workspace ? workspace_bytes : 0, "workspace too small");
    if (reinterpret_cast<uintptr_t>(d_workspace) & 255)
        return fail(OXQ_ERR_KERNEL, 256, reinterpret_cast<uintptr_t>(d_workspace) & 255,
                    "workspace must be 256-byte aligned");
    uint8_t *ws = (uint8_t *)d_workspace;
    int32_t *experts = (int32_t *)(ws + t.experts), *offsets = (int32_t *)(ws + t.offsets);
    int32_t *pair_token = (int32_t *)(ws + t.pair_token), *token_rows = (int32_t *)(ws + t.token_rows);
    float *weights = (float *)(ws + t.weights);
    // One token with a handful of choices: the router's launch also groups and writes the activation rows.
    const bool one = n_tokens == 1 && k <= oxq::GROUPED_GEMV_MAX_ROWS;
    // (the router's logits may lie, until the experts run, where the gate projection's outputs will)
    float *logits_scratch = n_tokens * n_experts <= n_tokens * k * intermediate ? (float *)(ws + t.ffn + l.gate) : nullptr;
    OXQ_HIP(oxq::launch_moe_route(d_router, d_x, experts, weights, (uint32_t)n_tokens, (uint32_t)n_experts,
                                  (uint32_t)hidden, (uint32_t)k, offsets, pair_token, token_rows, s,
                                  one ? ws + t.ffn + l.acts : nullptr, logits_scratch));
    return moe_ffn_impl(gate_type, d_gate, gate_stride_bytes, up_type, d_up, up_stride_bytes, down_type, d_down,
                        down_stride_bytes, n_experts, d_x, n_tokens, k, offsets, pair_token, token_rows, weights, 0, d_out,
                        hidden, intermediate, ws + t.ffn, workspace_bytes - t.ffn, stream, one);
}

// MoeFfn::forward on host slices (the drop-in route): everything is staged to the device, the layer
// runs there, the output comes back.  Validation in the reference's order (moe.rs:151-173, 33-58).
int oxq_moe_forward(uint32_t gate_type, const uint8_t *gate, size_t gate_len, uint32_t up_type, const uint8_t *up,
                    size_t up_len, uint32_t down_type, const uint8_t *down, size_t down_len, const float *router,
                    size_t router_len, size_t n_experts, size_t hidden, size_t intermediate, size_t top_k,
                    const float *input, size_t input_len, float *output, size_t output_len, size_t n_tokens) {
    if (!known_type(gate_type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, gate_type, 0, "unsupported quantization type");
    if (!known_type(up_type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, up_type, 0, "unsupported quantization type");
    if (!known_type(down_type)) return fail(OXQ_ERR_UNSUPPORTED_TYPE, down_type, 0, "unsupported quantization type");
    if (router_len != n_experts * hidden)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, n_experts * hidden, router_len, "moe.router has the wrong size");
    if (top_k == 0) return fail(OXQ_ERR_KERNEL, 1, 0, "MoeFfn top_k must be >= 1");
    auto mat_bytes = [](uint32_t t, size_t rows, size_t cols) {
        const size_t bs = oxq_block_size(t);
        return rows * ((cols + bs - 1) / bs) * oxq_block_bytes(t);
    };
    const size_t g_one = mat_bytes(gate_type, intermediate, hidden), u_one = mat_bytes(up_type, intermediate, hidden);
    const size_t d_one = mat_bytes(down_type, hidden, intermediate);
    if (gate_len != n_experts * g_one)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, n_experts * g_one, gate_len, "expert.gate has the wrong size");
    if (up_len != n_experts * u_one)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, n_experts * u_one, up_len, "expert.up has the wrong size");
    if (down_len != n_experts * d_one)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, n_experts * d_one, down_len, "expert.down has the wrong size");
    if (input_len < n_tokens * hidden)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, n_tokens * hidden, input_len, "input shorter than n_tokens * hidden");
    if (output_len < n_tokens * hidden)
        return fail(OXQ_ERR_DIMENSION_MISMATCH, n_tokens * hidden, output_len, "output shorter than n_tokens * hidden");
    if (n_tokens == 0 || hidden == 0) return OXQ_OK;
    if (n_experts == 0 || intermediate == 0) {  // no expert to add: the zeroed output (moe.rs:240-242)
        std::memset(output, 0, n_tokens * hidden * sizeof(float));
        return OXQ_OK;
    }
    const size_t ws_bytes =
        oxq_moe_forward_workspace_bytes(gate_type, up_type, down_type, n_tokens, top_k, n_experts, hidden, intermediate);
    if (ws_bytes == 0)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 256, hidden % 256 ? hidden : intermediate,
                    "no grouped kernel for this type/shape (dimensions must be multiples of 256)");
    int st;
    if ((st = ensure_init()) != OXQ_OK) return st;
    std::lock_guard<std::mutex> lock(g.mu);
    const uint8_t *dg = nullptr, *du = nullptr, *dd = nullptr;
    // The cache serves this call only if the three tensors fit under its byte cap together, and what the call has
    // staged is pinned until it returns: staging `down` must not evict (and free) the `gate` the kernels will read.
    const bool cached = g.cache_mode != 0 && gate_len + up_len + down_len <= g.cache_limit;
    struct Pin {
        uint64_t &pin;
        explicit Pin(uint64_t &p, uint64_t tick) : pin(p) { pin = tick; }
        ~Pin() { pin = UINT64_MAX; }
    } pin(g.cache_pin, g.cache_tick);
    auto stage = [&](Scratch &slot, uint32_t t, const uint8_t *host, size_t len, const uint8_t **dev) -> int {
        if (cached) return stage_weights(t, host, len, dev);
        int r = slot.reserve(len);
        if (r != OXQ_OK) return r;
        OXQ_HIP(hipMemcpy(slot.ptr, host, len, hipMemcpyHostToDevice));
        *dev = (const uint8_t *)slot.ptr;
        return OXQ_OK;
    };
    if ((st = stage(g.s_weights, gate_type, gate, gate_len, &dg)) != OXQ_OK) return st;
    if ((st = stage(g.s_moe_up, up_type, up, up_len, &du)) != OXQ_OK) return st;
    if ((st = stage(g.s_moe_down, down_type, down, down_len, &dd)) != OXQ_OK) return st;
    if ((st = g.s_moe_tables.reserve(router_len * sizeof(float))) != OXQ_OK) return st;
    if ((st = g.s_x.reserve(n_tokens * hidden * sizeof(float))) != OXQ_OK) return st;
    if ((st = g.s_out.reserve(n_tokens * hidden * sizeof(float))) != OXQ_OK) return st;
    if ((st = g.s_work.reserve(ws_bytes + 256)) != OXQ_OK) return st;
    uint8_t *ws = (uint8_t *)((reinterpret_cast<uintptr_t>(g.s_work.ptr) + 255) & ~(uintptr_t)255);
    OXQ_HIP(hipMemcpy(g.s_moe_tables.ptr, router, router_len * sizeof(float), hipMemcpyHostToDevice));
    OXQ_HIP(hipMemcpy(g.s_x.ptr, input, n_tokens * hidden * sizeof(float), hipMemcpyHostToDevice));
    if ((st = oxq_moe_forward_dev(gate_type, dg, g_one, up_type, du, u_one, down_type, dd, d_one, n_experts,
                                  (const float *)g.s_moe_tables.ptr, (const float *)g.s_x.ptr, n_tokens, top_k,
                                  (float *)g.s_out.ptr, hidden, intermediate, ws, ws_bytes, nullptr)) != OXQ_OK)
        return st;
    OXQ_HIP(hipMemcpy(output, g.s_out.ptr, n_tokens * hidden * sizeof(float), hipMemcpyDeviceToHost));
    return OXQ_OK;
}

size_t oxq_topk_workspace_bytes(size_t n, size_t k) { return oxq::topk_workspace_bytes(n, k); }

int oxq_topk_dev(const float *d_values, size_t n, size_t k, float *d_out_values, uint32_t *d_out_indices,
                 void *d_workspace, size_t workspace_bytes, void *stream) {
    if (k == 0 || k > n) return fail(OXQ_ERR_DIMENSION_MISMATCH, n, k, "k must be between 1 and the vector length");
    const size_t need = oxq::topk_workspace_bytes(n, k);
    if (need == 0) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 256, k, "k above 256 or more than 2^20 values");
    if (!d_workspace || workspace_bytes < need)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, d_workspace ? workspace_bytes : 0, "workspace too small");
    if (reinterpret_cast<uintptr_t>(d_workspace) & 7)
        return fail(OXQ_ERR_KERNEL, 8, reinterpret_cast<uintptr_t>(d_workspace) & 7, "workspace must be 8-byte aligned");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_topk(d_values, (uint32_t)n, (uint32_t)k, d_out_values, d_out_indices, d_workspace,
                             (hipStream_t)stream));
    return OXQ_OK;
}

size_t oxq_lm_head_topk_workspace_bytes(uint32_t type, size_t n_rows, size_t n_cols, size_t k) {
    if (k == 0 || k > n_rows || n_rows > 0xFFFFFFFFull || n_cols > 0xFFFFFFFFull) return 0;
    const size_t lists = oxq::lm_head_topk_lists_bytes(type, (uint32_t)n_rows, (uint32_t)n_cols, (uint32_t)k);
    const size_t topk = oxq::topk_workspace_bytes(n_rows, k);
    if (lists == 0 && topk == 0) return 0;
    return lists > topk ? lists : topk;
}

int oxq_lm_head_topk_dev(uint32_t type, const uint8_t *d_weights, const uint8_t *d_acts_q8, float *d_logits, size_t n_rows,
                         size_t n_cols, size_t k, float *d_out_values, uint32_t *d_out_indices, void *d_workspace,
                         size_t workspace_bytes, void *stream) {
    int st = check_dev_shape(type, n_rows, n_cols, true);
    if (st != OXQ_OK) return st;
    if (k == 0 || k > n_rows) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_rows, k, "k must be between 1 and the number of rows");
    const size_t need = oxq_lm_head_topk_workspace_bytes(type, n_rows, n_cols, k);
    if (need == 0) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 256, k, "k above 256 or more than 2^20 rows");
    if (!d_workspace || workspace_bytes < need)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, need, d_workspace ? workspace_bytes : 0, "workspace too small");
    if (reinterpret_cast<uintptr_t>(d_workspace) & 7)
        return fail(OXQ_ERR_KERNEL, 8, reinterpret_cast<uintptr_t>(d_workspace) & 7, "workspace must be 8-byte aligned");
    if (!d_logits || !d_out_values || !d_out_indices) return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer");
    if ((st = ensure_init()) != OXQ_OK) return st;
    if (oxq::lm_head_topk_lists_bytes(type, (uint32_t)n_rows, (uint32_t)n_cols, (uint32_t)k) != 0) {
        OXQ_HIP(oxq::launch_lm_head_topk(type, d_weights, d_acts_q8, d_logits, (uint32_t)n_rows, (uint32_t)n_cols, (uint32_t)k,
                                         d_workspace, d_out_values, d_out_indices, (hipStream_t)stream));
        return OXQ_OK;
    }
    // shapes the one-launch form does not take: the GEMV, then the top-k launches
    OXQ_HIP(oxq::launch_gemv_q8(type, gemv_args(d_weights, d_acts_q8, d_logits, nullptr, n_rows, n_cols, 0), (hipStream_t)stream));
    if (oxq::topk_workspace_bytes(n_rows, k) == 0)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 256, k, "k above 256 or more than 2^20 rows");
    OXQ_HIP(oxq::launch_topk(d_logits, (uint32_t)n_rows, (uint32_t)k, d_out_values, d_out_indices, d_workspace, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_logits_edit_dev(float *d_logits, size_t n, const uint32_t *d_banned, size_t n_banned, const uint32_t *d_bias_tokens,
                        const float *d_bias_values, size_t n_bias, const uint32_t *d_recent, size_t n_recent,
                        size_t window, float repetition_penalty, void *stream) {
    if (!d_logits || n == 0 || n > 0xFFFFFFFFull) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, n, "1 .. 2^32-1 logits");
    if ((n_banned && !d_banned) || (n_bias && (!d_bias_tokens || !d_bias_values)) || (n_recent && !d_recent))
        return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer");
    if (n_banned > 0xFFFFFFFFull || n_bias > 0xFFFFFFFFull) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFFFFull, n_banned, "list too long");
    // the window is the tail of the recent tokens (saturating_sub, sampling/mod.rs:601-603)
    const size_t n_window = n_recent < window ? n_recent : window;
    if (n_window > 4096) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 4096, n_window, "repetition window of at most 4096 tokens");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_logits_edit(d_logits, (uint32_t)n, d_banned, (uint32_t)n_banned, d_bias_tokens, d_bias_values,
                                    (uint32_t)n_bias, d_recent ? d_recent + (n_recent - n_window) : nullptr,
                                    (uint32_t)n_window, repetition_penalty, (hipStream_t)stream));
    return OXQ_OK;
}

int oxq_sample_candidates_dev(const float *d_values, const uint32_t *d_indices, size_t k, float temperature, float min_p,
                              float top_p, uint64_t *d_rng_state, uint32_t *d_token, float *d_probs, void *stream) {
    if (k == 0 || k > 256) return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 256, k, "between 1 and 256 candidates");
    if (!d_values || !d_indices || !d_rng_state || !d_token) return fail(OXQ_ERR_INTERNAL, 0, 0, "null pointer");
    int st = ensure_init();
    if (st != OXQ_OK) return st;
    OXQ_HIP(oxq::launch_sample_candidates(d_values, d_indices, (uint32_t)k, temperature, min_p, top_p, d_rng_state,
                                          d_token, d_probs, (hipStream_t)stream));
    return OXQ_OK;
}

// QuantLinear::forward on host slices (drop-in route: everything is staged per call).
int oxq_linear_forward(uint32_t type, const uint8_t *data, size_t data_len, const size_t *shape, size_t n_dims,
                       const float *bias, size_t bias_len, const float *lora_a, size_t lora_a_len, const float *lora_b,
                       size_t lora_b_len, size_t rank, float scale, const float *input, size_t input_len, float *output,
                       size_t output_len) {
    size_t n_rows = 0, n_cols = 0;
    int st = tensor_dims(type, data_len, shape, n_dims, &n_rows, &n_cols);
    if (st != OXQ_OK) return st;
    // gemv's checks first (reference/q4_k.rs:117-128), then the adapter's (lora.rs:84-95)
    if (input_len < n_cols) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_cols, input_len, "input shorter than n_cols");
    if (output_len < n_rows) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_rows, output_len, "output shorter than n_rows");
    const bool has_lora = lora_a && lora_b && rank;
    if (has_lora) {
        if (lora_a_len != rank * n_cols) return fail(OXQ_ERR_DIMENSION_MISMATCH, rank * n_cols, lora_a_len, "LoRA A has the wrong size");
        if (lora_b_len != n_rows * rank) return fail(OXQ_ERR_DIMENSION_MISMATCH, n_rows * rank, lora_b_len, "LoRA B has the wrong size");
    }
    const size_t bs = oxq_block_size(type), bb = oxq_block_bytes(type);
    const size_t row_bytes = (n_cols + bs - 1) / bs * bb;
    if (data_len < n_rows * row_bytes)
        return fail(OXQ_ERR_BUFFER_TOO_SMALL, n_rows * row_bytes, data_len, "tensor data too small");
    if (n_rows == 0 || n_cols == 0) return OXQ_OK;
    if (n_rows > 0xFFFFFFFFull || n_cols > 0xFFFFFF00ull)
        return fail(OXQ_ERR_UNSUPPORTED_SHAPE, 0xFFFFFF00ull, n_rows, "dimension exceeds 2^32-257");
    if ((st = ensure_init()) != OXQ_OK) return st;
    std::lock_guard<std::mutex> lock(g.mu);
    const uint8_t *dW = nullptr;
    if ((st = stage_weights(type, data, n_rows * row_bytes, &dW)) != OXQ_OK) return st;
    // a row that ends inside a block: the input is staged zero-padded to whole blocks (gemv skips those columns)
    const size_t k_pad = (n_cols + bs - 1) / bs * bs;
    if ((st = g.s_x.reserve(k_pad * sizeof(float))) != OXQ_OK) return st;
    if ((st = g.s_acts.reserve(k_pad / 32 * 34)) != OXQ_OK) return st;
    if ((st = g.s_out.reserve(n_rows * sizeof(float))) != OXQ_OK) return st;
    if (k_pad != n_cols) OXQ_HIP(hipMemset(g.s_x.ptr, 0, k_pad * sizeof(float)));
    OXQ_HIP(hipMemcpy(g.s_x.ptr, input, n_cols * sizeof(float), hipMemcpyHostToDevice));
    OXQ_HIP(oxq::launch_quantize_q8_0((const float *)g.s_x.ptr, k_pad, (uint8_t *)g.s_acts.ptr, nullptr));
    const float *d_bias = nullptr;
    if (bias && bias_len) {
        // the reference zips output with bias (linear.rs:87-89): a short bias covers its own length only
        if ((st = g.s_bias.reserve(n_rows * sizeof(float))) != OXQ_OK) return st;
        const size_t nb = bias_len < n_rows ? bias_len : n_rows;
        OXQ_HIP(hipMemset(g.s_bias.ptr, 0, n_rows * sizeof(float)));
        OXQ_HIP(hipMemcpy(g.s_bias.ptr, bias, nb * sizeof(float), hipMemcpyHostToDevice));
        d_bias = (const float *)g.s_bias.ptr;
    }
    if (g.act_route.load(std::memory_order_relaxed) == OXQ_ROUTE_F32) {
        if (!oxq::gemv_f32_supported(type))
            return fail(OXQ_ERR_UNSUPPORTED_TYPE, type, 0, "no fp32-activation kernel for this type (OXQ_ROUTE_F32)");
        OXQ_HIP(oxq::launch_gemv_f32(type, dW, (const float *)g.s_x.ptr, (float *)g.s_out.ptr, d_bias, (uint32_t)n_rows,
                                     (uint32_t)n_cols, nullptr));
    } else {
        oxq::GemvArgs a = gemv_args(dW, (const uint8_t *)g.s_acts.ptr, (float *)g.s_out.ptr, nullptr, n_rows, n_cols, 0);
        a.bias = d_bias;
        OXQ_HIP(oxq::launch_gemv_q8(type, a, nullptr));
    }
    if (has_lora) {
        if ((st = g.s_lora_a.reserve(lora_a_len * sizeof(float))) != OXQ_OK) return st;
        if ((st = g.s_lora_b.reserve(lora_b_len * sizeof(float))) != OXQ_OK) return st;
        if ((st = g.s_lora_r.reserve(rank * sizeof(float))) != OXQ_OK) return st;
        OXQ_HIP(hipMemcpy(g.s_lora_a.ptr, lora_a, lora_a_len * sizeof(float), hipMemcpyHostToDevice));
        OXQ_HIP(hipMemcpy(g.s_lora_b.ptr, lora_b, lora_b_len * sizeof(float), hipMemcpyHostToDevice));
        OXQ_HIP(oxq::launch_lora_apply((const float *)g.s_lora_a.ptr, (const float *)g.s_lora_b.ptr,
                                       (float *)g.s_lora_r.ptr, (uint32_t)rank, scale, (const float *)g.s_x.ptr,
                                       (float *)g.s_out.ptr, (uint32_t)n_rows, (uint32_t)n_cols, nullptr));
    }
    OXQ_HIP(hipMemcpy(output, g.s_out.ptr, n_rows * sizeof(float), hipMemcpyDeviceToHost));
    return OXQ_OK;
}

}  // extern "C"
