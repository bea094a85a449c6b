// GGUF container reader and tensor -> HBM loader (see include/oxq_gguf.h).  Host code: the
// parser follows the reference's GgufFile::parse (crates/oxillama-gguf/src/parser.rs:34-60,
// header.rs:20-96, reader.rs:47-198, tensor_info.rs:22-50) field for field; the loader copies a
// tensor's bytes from the memory-mapped file to HBM through two pinned staging buffers so that
// reading the file (page faults, memcpy) overlaps the DMA of the previous piece.
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <fcntl.h>
#include <mutex>
#include <new>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <unordered_map>
#include <vector>

#include "../../include/oxq_gguf.h"
#include "oxq_internal.hpp"

namespace {

constexpr uint32_t GGUF_MAGIC = 0x46554747u;     // types.rs:7
constexpr uint64_t GGUF_DEFAULT_ALIGNMENT = 32;  // types.rs:10

struct Value {
    uint32_t type = 0;
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0.0;
    std::string str;
    uint32_t elem_type = 0;
    uint64_t count = 0;
    uint64_t array_offset = 0, array_bytes = 0;  // arrays: where the encoded elements sit in the file image
};

struct Tensor {
    std::string name;
    uint32_t n_dims = 0;
    std::vector<uint64_t> dims;
    uint32_t type = 0;
    uint64_t offset = 0;
};

// GgufTensorType::block_size / block_bytes for every id from_u32 accepts (types.rs:152-262).
bool type_layout(uint32_t t, uint64_t *bs, uint64_t *bb) {
    static const struct { uint32_t id; uint16_t bs, bb; } T[] = {
        {0, 1, 4},      {1, 1, 2},      {2, 32, 18},    {3, 32, 20},    {6, 32, 22},    {7, 32, 24},    {8, 32, 34},
        {9, 32, 36},    {10, 256, 84},  {11, 256, 110}, {12, 256, 144}, {13, 256, 176}, {14, 256, 210}, {15, 256, 292},
        {16, 256, 66},  {17, 256, 74},  {18, 256, 98},  {19, 256, 50},  {20, 32, 18},   {21, 256, 110}, {22, 256, 82},
        {23, 256, 136}, {24, 1, 1},     {25, 1, 2},     {26, 1, 4},     {27, 1, 8},     {28, 1, 8},     {29, 256, 56},
        {30, 1, 2},     {31, 32, 18},   {32, 32, 18},   {33, 32, 18},   {34, 256, 54},  {35, 256, 66},  {36, 32, 34},
        {37, 32, 34},   {38, 32, 34},   {39, 128, 18}};
    for (const auto &e : T)
        if (e.id == t) {
            *bs = e.bs;
            *bb = e.bb;
            return true;
        }
    return false;
}

uint64_t n_elements(const Tensor &t) {  // tensor_info.rs:35-40
    if (t.dims.empty()) return 0;
    uint64_t n = 1;
    for (uint64_t d : t.dims)
        if (__builtin_mul_overflow(n, d, &n)) return UINT64_MAX;  // saturate: such a tensor can never fit a file
    return n;
}

uint64_t data_size(const Tensor &t) {  // tensor_info.rs:42-50
    uint64_t bs = 1, bb = 0;
    type_layout(t.type, &bs, &bb);
    const uint64_t n = n_elements(t);
    uint64_t bytes;
    if (__builtin_mul_overflow(n / bs + (n % bs ? 1 : 0), bb, &bytes)) return UINT64_MAX;
    return bytes;
}

bool valid_utf8(const uint8_t *s, size_t n) {
    size_t i = 0;
    while (i < n) {
        const uint8_t c = s[i];
        size_t len;
        uint32_t cp;
        if (c < 0x80) { i++; continue; }
        if ((c & 0xE0) == 0xC0) { len = 2; cp = c & 0x1F; }
        else if ((c & 0xF0) == 0xE0) { len = 3; cp = c & 0x0F; }
        else if ((c & 0xF8) == 0xF0) { len = 4; cp = c & 0x07; }
        else return false;
        if (i + len > n) return false;
        for (size_t k = 1; k < len; k++) {
            if ((s[i + k] & 0xC0) != 0x80) return false;
            cp = (cp << 6) | (s[i + k] & 0x3F);
        }
        if ((len == 2 && cp < 0x80) || (len == 3 && cp < 0x800) || (len == 4 && (cp < 0x10000 || cp > 0x10FFFF)) ||
            (cp >= 0xD800 && cp <= 0xDFFF))
            return false;
        i += len;
    }
    return true;
}

// BinaryReader (reader.rs): every read checks the bounds first and reports UnexpectedEof{pos}.
struct Reader {
    const uint8_t *data;
    size_t len, pos;
    int status = OXQ_OK;

    bool check(size_t n) {
        if (n > len - pos) {  // pos <= len always
            status = oxq::set_error(OXQ_ERR_GGUF_UNEXPECTED_EOF, pos, 0, "unexpected end of file");
            return false;
        }
        return true;
    }
    template <class T> bool rd(T *v) {
        if (!check(sizeof(T))) return false;
        std::memcpy(v, data + pos, sizeof(T));  // little-endian host
        pos += sizeof(T);
        return true;
    }
    bool rd_len(uint32_t version, uint64_t *v) {  // u64 in version 3, u32 before
        if (version >= 3) return rd(v);
        uint32_t w;
        if (!rd(&w)) return false;
        *v = w;
        return true;
    }
    bool rd_string(uint32_t version, std::string *s) {  // reader.rs:177-198
        uint64_t n;
        if (!rd_len(version, &n)) return false;
        if (n > len - pos) {
            status = oxq::set_error(OXQ_ERR_GGUF_UNEXPECTED_EOF, pos, 0, "unexpected end of file");
            return false;
        }
        if (!valid_utf8(data + pos, (size_t)n)) {
            status = oxq::set_error(OXQ_ERR_GGUF_INVALID_STRING, pos, 0, "invalid UTF-8 string");
            return false;
        }
        s->assign(reinterpret_cast<const char *>(data + pos), (size_t)n);
        pos += (size_t)n;
        return true;
    }
};

}  // namespace

struct oxq_gguf {
    const uint8_t *data = nullptr;
    size_t len = 0;
    void *map = nullptr;        // mmap'ed region, or null
    std::vector<uint8_t> owned;  // from_bytes image
    uint32_t version = 0;
    uint64_t tensor_count = 0, kv_count = 0, alignment = GGUF_DEFAULT_ALIGNMENT, data_offset = 0;
    std::vector<Tensor> tensors;                      // distinct names, first-appearance order
    std::unordered_map<std::string, size_t> by_name;  // a later entry of the same name replaces the earlier one
    std::vector<std::pair<std::string, Value>> meta;
    std::unordered_map<std::string, size_t> meta_by_key;
};

namespace {

// read_metadata_value (parser.rs:118-169).  Array elements are parsed (to find where the array ends and
// to validate them) but only their count and element type are kept.
bool read_value(Reader &r, uint32_t version, uint32_t type, Value *v, int depth) {
    v->type = type;
    switch (type) {
    case OXQ_GGUF_UINT8: { uint8_t x; if (!r.rd(&x)) return false; v->u = x; return true; }
    case OXQ_GGUF_INT8: { int8_t x; if (!r.rd(&x)) return false; v->i = x; return true; }
    case OXQ_GGUF_UINT16: { uint16_t x; if (!r.rd(&x)) return false; v->u = x; return true; }
    case OXQ_GGUF_INT16: { int16_t x; if (!r.rd(&x)) return false; v->i = x; return true; }
    case OXQ_GGUF_UINT32: { uint32_t x; if (!r.rd(&x)) return false; v->u = x; return true; }
    case OXQ_GGUF_INT32: { int32_t x; if (!r.rd(&x)) return false; v->i = x; return true; }
    case OXQ_GGUF_FLOAT32: { float x; if (!r.rd(&x)) return false; v->f = x; return true; }
    case OXQ_GGUF_FLOAT64: { double x; if (!r.rd(&x)) return false; v->f = x; return true; }
    case OXQ_GGUF_BOOL: { uint8_t x; if (!r.rd(&x)) return false; v->u = x != 0; return true; }
    case OXQ_GGUF_UINT64: { uint64_t x; if (!r.rd(&x)) return false; v->u = x; return true; }
    case OXQ_GGUF_INT64: { int64_t x; if (!r.rd(&x)) return false; v->i = x; return true; }
    case OXQ_GGUF_STRING: return r.rd_string(version, &v->str);
    case OXQ_GGUF_ARRAY: {
        uint32_t et;
        if (!r.rd(&et)) return false;
        if (et > OXQ_GGUF_FLOAT64) {
            r.status = oxq::set_error(OXQ_ERR_GGUF_INVALID_METADATA, et, 0, "<array>: unknown array element type");
            return false;
        }
        uint64_t count;
        if (!r.rd_len(version, &count)) return false;
        if (depth > 8) {
            r.status = oxq::set_error(OXQ_ERR_GGUF_INVALID_METADATA, depth, 0, "<array>: nesting too deep");
            return false;
        }
        v->elem_type = et;
        v->count = count;
        v->array_offset = r.pos;
        Value e;
        for (uint64_t k = 0; k < count; k++)
            if (!read_value(r, version, et, &e, depth + 1)) return false;
        v->array_bytes = r.pos - v->array_offset;
        return true;
    }
    default:
        r.status = oxq::set_error(OXQ_ERR_GGUF_INVALID_METADATA, type, 0, "unknown value type");
        return false;
    }
}

int parse(oxq_gguf *g) {
    Reader r{g->data, g->len, 0};
    // GgufHeader::parse, header.rs:20-66
    if (g->len < 4) return oxq::set_error(OXQ_ERR_GGUF_UNEXPECTED_EOF, 0, 0, "unexpected end of file");
    uint32_t magic = 0;
    r.rd(&magic);
    if (magic != GGUF_MAGIC) return oxq::set_error(OXQ_ERR_GGUF_INVALID_MAGIC, magic, 0, "invalid GGUF magic number");
    if (!r.rd(&g->version)) return r.status;
    if (g->version < 1 || g->version > 3)
        return oxq::set_error(OXQ_ERR_GGUF_UNSUPPORTED_VERSION, g->version, 0, "unsupported GGUF version (supported: 1, 2, 3)");
    if (!r.rd_len(g->version, &g->tensor_count)) return r.status;
    if (!r.rd_len(g->version, &g->kv_count)) return r.status;
    // parse_metadata, parser.rs:93-115
    for (uint64_t k = 0; k < g->kv_count; k++) {
        std::string key;
        if (!r.rd_string(g->version, &key)) return r.status;
        uint32_t vt;
        if (!r.rd(&vt)) return r.status;
        if (vt > OXQ_GGUF_FLOAT64) {
            char msg[200];
            std::snprintf(msg, sizeof(msg), "%.120s: unknown value type: %u", key.c_str(), vt);
            return oxq::set_error(OXQ_ERR_GGUF_INVALID_METADATA, vt, 0, msg);
        }
        Value v;
        if (!read_value(r, g->version, vt, &v, 0)) return r.status;
        auto it = g->meta_by_key.find(key);
        if (it != g->meta_by_key.end()) {
            g->meta[it->second].second = std::move(v);
        } else {
            g->meta_by_key.emplace(key, g->meta.size());
            g->meta.emplace_back(std::move(key), std::move(v));
        }
    }
    // alignment, parser.rs:41-45: general.alignment read as u64 (any unsigned width), else 32
    auto al = g->meta_by_key.find("general.alignment");
    if (al != g->meta_by_key.end()) {
        const Value &v = g->meta[al->second].second;
        if (v.type == OXQ_GGUF_UINT8 || v.type == OXQ_GGUF_UINT16 || v.type == OXQ_GGUF_UINT32 || v.type == OXQ_GGUF_UINT64)
            g->alignment = v.u;
    }
    // parse_tensor_infos, parser.rs:172-211
    for (uint64_t k = 0; k < g->tensor_count; k++) {
        Tensor t;
        if (!r.rd_string(g->version, &t.name)) return r.status;
        if (!r.rd(&t.n_dims)) return r.status;
        for (uint32_t d = 0; d < t.n_dims; d++) {
            uint64_t dim;
            if (!r.rd_len(g->version, &dim)) return r.status;
            t.dims.push_back(dim);
        }
        if (!r.rd(&t.type)) return r.status;
        uint64_t bs, bb;
        if (!type_layout(t.type, &bs, &bb))
            return oxq::set_error(OXQ_ERR_GGUF_UNSUPPORTED_QUANT_TYPE, t.type, 0, "unsupported quantization type");
        if (g->version >= 2) {
            if (!r.rd(&t.offset)) return r.status;
        } else {
            uint32_t o;
            if (!r.rd(&o)) return r.status;
            t.offset = o;
        }
        auto it = g->by_name.find(t.name);
        if (it != g->by_name.end()) {
            g->tensors[it->second] = std::move(t);
        } else {
            g->by_name.emplace(t.name, g->tensors.size());
            g->tensors.push_back(std::move(t));
        }
    }
    // data section: the position after the tensor infos, aligned up (parser.rs:50-52, align_up :214-224)
    uint64_t off = r.pos;
    if (g->alignment != 0 && off % g->alignment) off += g->alignment - off % g->alignment;
    g->data_offset = off;
    return OXQ_OK;
}

void fill(const oxq_gguf *g, const Tensor &t, oxq_gguf_tensor *out) {
    (void)g;
    out->name = t.name.c_str();
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; d++) out->dims[d] = (size_t)d < t.dims.size() ? t.dims[d] : 0;
    out->type = t.type;
    out->offset = t.offset;
    out->n_elements = n_elements(t);
    out->data_size = data_size(t);
}

void fill_value(const Value &v, oxq_gguf_value *out) {
    out->type = v.type;
    out->u = v.u;
    out->i = v.i;
    out->f = v.f;
    out->str = v.type == OXQ_GGUF_STRING ? v.str.data() : nullptr;
    out->str_len = v.type == OXQ_GGUF_STRING ? v.str.size() : 0;
    out->elem_type = v.elem_type;
    out->count = v.count;
    out->array_offset = v.array_offset;
    out->array_bytes = v.array_bytes;
}

const Tensor *find(const oxq_gguf *g, const char *name) {
    if (!g || !name) return nullptr;
    auto it = g->by_name.find(name);
    return it == g->by_name.end() ? nullptr : &g->tensors[it->second];
}

int not_found(const char *name) {
    char msg[200];
    std::snprintf(msg, sizeof(msg), "%.180s", name ? name : "");
    return oxq::set_error(OXQ_ERR_GGUF_TENSOR_NOT_FOUND, 0, 0, msg);
}

// GgufFile::tensor_data, parser.rs:66-80
int locate(const oxq_gguf *g, const Tensor &t, const uint8_t **p, size_t *n) {
    const uint64_t abs = g->data_offset + t.offset, size = data_size(t);
    if (abs < t.offset || abs > g->len || size > g->len - abs)  // the sum must not wrap either
        return oxq::set_error(OXQ_ERR_GGUF_UNEXPECTED_EOF, abs, 0, "tensor data runs past the end of the file");
    *p = g->data + abs;
    *n = (size_t)size;
    return OXQ_OK;
}

// ---- file -> HBM -----------------------------------------------------------------------------

constexpr size_t STAGE_BYTES = 8u << 20;
struct Staging {
    std::mutex mu;
    void *buf[2] = {nullptr, nullptr};
    hipStream_t stream = nullptr;
    hipEvent_t done[2] = {nullptr, nullptr};
    int device = -1;
} g_stage;

int hip_fail(hipError_t e, const char *what) {
    char msg[200];
    std::snprintf(msg, sizeof(msg), "%s: %s", what, hipGetErrorString(e));
    return oxq::set_error(OXQ_ERR_KERNEL, (size_t)e, 0, msg);
}

// Host bytes (pageable: the file mapping) -> device, in STAGE_BYTES pieces through two pinned buffers: while
// piece i is on its way, piece i+1 is read from the mapping.  Caller holds g_stage.mu.
int staged_upload(void *d_dst, const uint8_t *src, size_t n) {
    hipError_t e;
    if (!g_stage.buf[0]) {
        for (int i = 0; i < 2; i++) {
            if ((e = hipHostMalloc(&g_stage.buf[i], STAGE_BYTES, hipHostMallocDefault)) != hipSuccess) return hip_fail(e, "hipHostMalloc");
            if ((e = hipEventCreateWithFlags(&g_stage.done[i], hipEventDisableTiming)) != hipSuccess) return hip_fail(e, "hipEventCreate");
        }
        if ((e = hipStreamCreateWithFlags(&g_stage.stream, hipStreamNonBlocking)) != hipSuccess) return hip_fail(e, "hipStreamCreate");
    }
    size_t off = 0;
    int slot = 0;
    bool used[2] = {false, false};
    while (off < n) {
        const size_t piece = n - off < STAGE_BYTES ? n - off : STAGE_BYTES;
        if (used[slot] && (e = hipEventSynchronize(g_stage.done[slot])) != hipSuccess) return hip_fail(e, "hipEventSynchronize");
        std::memcpy(g_stage.buf[slot], src + off, piece);
        if ((e = hipMemcpyAsync(static_cast<uint8_t *>(d_dst) + off, g_stage.buf[slot], piece, hipMemcpyHostToDevice,
                                g_stage.stream)) != hipSuccess)
            return hip_fail(e, "hipMemcpyAsync");
        if ((e = hipEventRecord(g_stage.done[slot], g_stage.stream)) != hipSuccess) return hip_fail(e, "hipEventRecord");
        used[slot] = true;
        off += piece;
        slot ^= 1;
    }
    if ((e = hipStreamSynchronize(g_stage.stream)) != hipSuccess) return hip_fail(e, "hipStreamSynchronize");
    return OXQ_OK;
}

int open_common(oxq_gguf *g, oxq_gguf_t *out) {
    int st;
    try {  // strings, vectors and maps allocate: no exception may cross the C ABI
        st = parse(g);
    } catch (const std::bad_alloc &) {
        st = oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "out of host memory while parsing");
    } catch (...) {
        st = oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "unexpected exception while parsing");
    }
    if (st != OXQ_OK) {
        if (g->map) munmap(g->map, g->len);
        delete g;
        return st;
    }
    *out = g;
    return OXQ_OK;
}

// Runs an entry point's body; name lookups build std::string keys, which may throw.
template <class Body>
int guarded(Body body) {
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "out of host memory");
    } catch (...) {
        return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "unexpected exception");
    }
}

}  // namespace

namespace oxq {
void gguf_release_staging() {
    std::lock_guard<std::mutex> lock(g_stage.mu);
    for (int i = 0; i < 2; i++) {
        if (g_stage.buf[i]) (void)hipHostFree(g_stage.buf[i]);
        if (g_stage.done[i]) (void)hipEventDestroy(g_stage.done[i]);
        g_stage.buf[i] = nullptr;
        g_stage.done[i] = nullptr;
    }
    if (g_stage.stream) (void)hipStreamDestroy(g_stage.stream);
    g_stage.stream = nullptr;
}
}  // namespace oxq

extern "C" {

int oxq_gguf_open(const char *path, oxq_gguf_t *out) {
    if (!out) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null handle pointer");
    *out = nullptr;
    if (!path) return oxq::set_error(OXQ_ERR_GGUF_IO, EINVAL, 0, "null path");
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return oxq::set_error(OXQ_ERR_GGUF_IO, (size_t)errno, 0, std::strerror(errno));
    struct stat sb;
    if (fstat(fd, &sb) != 0) {
        const int err = errno;
        close(fd);
        return oxq::set_error(OXQ_ERR_GGUF_IO, (size_t)err, 0, std::strerror(err));
    }
    oxq_gguf *g = new (std::nothrow) oxq_gguf;
    if (!g) {
        close(fd);
        return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "out of host memory");
    }
    g->len = (size_t)sb.st_size;
    if (g->len) {
        void *m = mmap(nullptr, g->len, PROT_READ, MAP_PRIVATE, fd, 0);
        if (m == MAP_FAILED) {
            const int err = errno;
            close(fd);
            delete g;
            return oxq::set_error(OXQ_ERR_GGUF_IO, (size_t)err, 0, std::strerror(err));
        }
        g->map = m;
        g->data = static_cast<const uint8_t *>(m);
    }
    close(fd);  // the mapping keeps the file
    return open_common(g, out);
}

int oxq_gguf_open_bytes(const uint8_t *data, size_t len, oxq_gguf_t *out) {
    if (!out) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null handle pointer");
    *out = nullptr;
    oxq_gguf *g = new (std::nothrow) oxq_gguf;
    if (!g) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "out of host memory");
    try {
        if (len) g->owned.assign(data, data + len);
    } catch (...) {
        delete g;
        return oxq::set_error(OXQ_ERR_INTERNAL, len, 0, "out of host memory");
    }
    g->data = g->owned.data();
    g->len = len;
    return open_common(g, out);
}

int oxq_gguf_close(oxq_gguf_t g) {
    if (!g) return OXQ_OK;
    if (g->map) munmap(g->map, g->len);
    delete g;
    return OXQ_OK;
}

int oxq_gguf_get_summary(oxq_gguf_t g, oxq_gguf_summary *out) {
    if (!g || !out) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
    out->version = g->version;
    out->tensor_count = g->tensor_count;
    out->metadata_kv_count = g->kv_count;
    out->n_tensors = g->tensors.size();
    out->n_metadata = g->meta.size();
    out->alignment = g->alignment;
    out->data_offset = g->data_offset;
    out->file_size = g->len;
    return OXQ_OK;
}

int oxq_gguf_tensor_at(oxq_gguf_t g, uint64_t index, oxq_gguf_tensor *out) {
    if (!g || !out) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
    if (index >= g->tensors.size()) return not_found("<index past the last tensor>");
    fill(g, g->tensors[(size_t)index], out);
    return OXQ_OK;
}

int oxq_gguf_find_tensor(oxq_gguf_t g, const char *name, oxq_gguf_tensor *out) {
    return guarded([&]() -> int {
        if (!g || !out) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
        const Tensor *t = find(g, name);
        if (!t) return not_found(name);
        fill(g, *t, out);
        return OXQ_OK;
    });
}

int oxq_gguf_tensor_data(oxq_gguf_t g, const char *name, const uint8_t **data, size_t *len) {
    return guarded([&]() -> int {
        if (!g || !data || !len) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
        const Tensor *t = find(g, name);
        if (!t) return not_found(name);
        return locate(g, *t, data, len);
    });
}

int oxq_gguf_meta_find(oxq_gguf_t g, const char *key, oxq_gguf_value *out) {
    return guarded([&]() -> int {
        if (!g || !key || !out) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
        auto it = g->meta_by_key.find(key);
        if (it == g->meta_by_key.end()) {
            char msg[200];
            std::snprintf(msg, sizeof(msg), "%.150s: key not present", key);
            return oxq::set_error(OXQ_ERR_GGUF_INVALID_METADATA, 0, 0, msg);
        }
        fill_value(g->meta[it->second].second, out);
        return OXQ_OK;
    });
}

int oxq_gguf_meta_at(oxq_gguf_t g, uint64_t index, const char **key, oxq_gguf_value *out) {
    if (!g || !key || !out) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
    if (index >= g->meta.size()) return oxq::set_error(OXQ_ERR_GGUF_INVALID_METADATA, (size_t)index, 0, "index past the last key");
    *key = g->meta[(size_t)index].first.c_str();
    fill_value(g->meta[(size_t)index].second, out);
    return OXQ_OK;
}

int oxq_gguf_meta_array_data(oxq_gguf_t g, const char *key, const uint8_t **data, size_t *len) {
    return guarded([&]() -> int {
        if (!g || !key || !data || !len) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
        auto it = g->meta_by_key.find(key);
        if (it == g->meta_by_key.end() || g->meta[it->second].second.type != OXQ_GGUF_ARRAY) {
            char msg[200];
            std::snprintf(msg, sizeof(msg), "%.150s: no such array", key);
            return oxq::set_error(OXQ_ERR_GGUF_INVALID_METADATA, 0, 0, msg);
        }
        const Value &v = g->meta[it->second].second;
        *data = g->data + v.array_offset;
        *len = (size_t)v.array_bytes;
        return OXQ_OK;
    });
}

int oxq_gguf_load_weights(oxq_gguf_t g, const char *name, oxq_weights_t *handle) {
    return guarded([&]() -> int {
        if (!handle) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null handle pointer");
        *handle = nullptr;
        if (!g) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null file handle");
        const Tensor *t = find(g, name);
        if (!t) return not_found(name);
        const size_t bs = oxq_block_size(t->type);
        if (bs == 0) return oxq::set_error(OXQ_ERR_UNSUPPORTED_TYPE, t->type, 0, "no kernel for this tensor's format");
        if (t->dims.size() != 2)
            return oxq::set_error(OXQ_ERR_UNSUPPORTED_SHAPE, 2, t->dims.size(), "weight tensor is not two-dimensional");
        const uint64_t n_rows = t->dims[0], n_cols = t->dims[1];  // model.rs:816: shape = the stored dimensions
        if (n_cols % bs != 0)
            return oxq::set_error(OXQ_ERR_UNSUPPORTED_SHAPE, bs, (size_t)n_cols, "columns are not a multiple of the block size");
        const uint8_t *src = nullptr;
        size_t n = 0;
        int st = locate(g, *t, &src, &n);
        if (st != OXQ_OK) return st;
        if ((st = oxq::ensure_device()) != OXQ_OK) return st;
        oxq_weights *w = new (std::nothrow) oxq_weights{t->type, (size_t)n_rows, (size_t)n_cols, n, nullptr};
        if (!w) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "out of host memory");
        hipError_t e = hipMalloc((void **)&w->dev, n ? n : 1);
        if (e != hipSuccess) {
            delete w;
            return hip_fail(e, "hipMalloc(weights)");
        }
        {
            std::lock_guard<std::mutex> lock(g_stage.mu);
            st = staged_upload(w->dev, src, n);
        }
        if (st != OXQ_OK) {
            (void)hipFree(w->dev);
            delete w;
            return st;
        }
        *handle = w;
        return OXQ_OK;
    });
}

int oxq_gguf_upload_tensor(oxq_gguf_t g, const char *name, void *d_dst, size_t dst_len) {
    return guarded([&]() -> int {
        if (!g || !d_dst) return oxq::set_error(OXQ_ERR_INTERNAL, 0, 0, "null argument");
        const Tensor *t = find(g, name);
        if (!t) return not_found(name);
        const uint8_t *src = nullptr;
        size_t n = 0;
        int st = locate(g, *t, &src, &n);
        if (st != OXQ_OK) return st;
        if (dst_len < n) return oxq::set_error(OXQ_ERR_BUFFER_TOO_SMALL, n, dst_len, "device buffer smaller than the tensor");
        if ((st = oxq::ensure_device()) != OXQ_OK) return st;
        std::lock_guard<std::mutex> lock(g_stage.mu);
        return staged_upload(d_dst, src, n);
    });
}

}  // extern "C"
