// gguf_model.hpp -- C++ host mirror of the reference's GGUF reader over the C ABI of
// liboxq_hip.so (include/oxq_gguf.h).  Header-only; link with -loxq_hip.
//   GgufModel   crates/oxillama-gguf/src/loader.rs:21-140 (load / from_bytes / tensor_data / architecture)
//   GgufFile    crates/oxillama-gguf/src/parser.rs:17-90
//   TensorInfo  crates/oxillama-gguf/src/tensor_info.rs:22-50
//   load_quant_linear  crates/oxillama-arch/src/llama/model.rs:805-822 (the tensor lands in HBM)
// Results come back as a status (OXQ_OK or a GgufError / QuantError code); nothing throws.
#ifndef OXQ_GGUF_MODEL_HPP
#define OXQ_GGUF_MODEL_HPP

#include <cstddef>
#include <cstdint>
#include <string>
#include <utility>
#include <vector>

#include "../oxq_gguf.h"

namespace oxq {

struct TensorInfo {
    std::string name;
    uint32_t n_dims = 0;
    std::vector<uint64_t> dimensions;
    uint32_t tensor_type = 0;
    uint64_t offset = 0;
    uint64_t elements = 0, bytes = 0;
    uint64_t n_elements() const { return elements; }
    uint64_t data_size() const { return bytes; }
};

// Weights resident in HBM; released with the object.
class DeviceWeights {
  public:
    DeviceWeights() = default;
    DeviceWeights(const DeviceWeights &) = delete;
    DeviceWeights &operator=(const DeviceWeights &) = delete;
    DeviceWeights(DeviceWeights &&o) noexcept : h_(o.h_), shape(std::move(o.shape)), tensor_type(o.tensor_type) { o.h_ = nullptr; }
    ~DeviceWeights() { oxq_weights_release(h_); }
    const uint8_t *device_ptr() const { return static_cast<const uint8_t *>(oxq_weights_device_ptr(h_)); }
    size_t nbytes() const { return oxq_weights_nbytes(h_); }
    oxq_weights_t handle() const { return h_; }

  private:
    friend class GgufModel;
    oxq_weights_t h_ = nullptr;

  public:
    std::vector<size_t> shape;  // the stored dimensions: [rows, columns]
    uint32_t tensor_type = 0;
};

class GgufModel {
  public:
    GgufModel() = default;
    GgufModel(const GgufModel &) = delete;
    GgufModel &operator=(const GgufModel &) = delete;
    ~GgufModel() { oxq_gguf_close(g_); }

    int load(const std::string &path) { return reset(oxq_gguf_open(path.c_str(), &g_)); }  // load_mmap
    int from_bytes(const std::vector<uint8_t> &data) { return reset(oxq_gguf_open_bytes(data.data(), data.size(), &g_)); }

    const oxq_gguf_summary &header() const { return s_; }
    size_t file_size() const { return (size_t)s_.file_size; }

    int tensor(const std::string &name, TensorInfo &out) const {
        oxq_gguf_tensor t;
        const int st = oxq_gguf_find_tensor(g_, name.c_str(), &t);
        if (st == OXQ_OK) convert(t, out);
        return st;
    }
    int tensor_at(uint64_t index, TensorInfo &out) const {
        oxq_gguf_tensor t;
        const int st = oxq_gguf_tensor_at(g_, index, &t);
        if (st == OXQ_OK) convert(t, out);
        return st;
    }
    // &[u8] into the mapping, valid while the model is open
    int tensor_data(const std::string &name, const uint8_t *&data, size_t &len) const {
        return oxq_gguf_tensor_data(g_, name.c_str(), &data, &len);
    }
    int get_string(const std::string &key, std::string &out) const {  // MetadataStore::get_string
        oxq_gguf_value v;
        const int st = oxq_gguf_meta_find(g_, key.c_str(), &v);
        if (st != OXQ_OK) return st;
        if (v.type != OXQ_GGUF_STRING) return OXQ_ERR_GGUF_INVALID_METADATA;
        out.assign(v.str, v.str_len);
        return OXQ_OK;
    }
    int get_u64(const std::string &key, uint64_t &out) const {  // MetadataStore::get_u64: any unsigned width
        oxq_gguf_value v;
        const int st = oxq_gguf_meta_find(g_, key.c_str(), &v);
        if (st != OXQ_OK) return st;
        if (v.type != OXQ_GGUF_UINT8 && v.type != OXQ_GGUF_UINT16 && v.type != OXQ_GGUF_UINT32 && v.type != OXQ_GGUF_UINT64)
            return OXQ_ERR_GGUF_INVALID_METADATA;
        out = v.u;
        return OXQ_OK;
    }
    int architecture(std::string &out) const { return get_string("general.architecture", out); }

    // load_quant_linear with the tensor in HBM
    int load_quant_linear(const std::string &name, DeviceWeights &out) const {
        TensorInfo info;
        int st = tensor(name, info);
        if (st != OXQ_OK) return st;
        oxq_weights_t h = nullptr;
        if ((st = oxq_gguf_load_weights(g_, name.c_str(), &h)) != OXQ_OK) return st;
        oxq_weights_release(out.h_);
        out.h_ = h;
        out.shape.assign(info.dimensions.begin(), info.dimensions.end());
        out.tensor_type = info.tensor_type;
        return OXQ_OK;
    }

  private:
    int reset(int st) {
        if (st == OXQ_OK) oxq_gguf_get_summary(g_, &s_);
        return st;
    }
    static void convert(const oxq_gguf_tensor &t, TensorInfo &out) {
        out.name = t.name;
        out.n_dims = t.n_dims;
        out.dimensions.assign(t.dims, t.dims + (t.n_dims < 4 ? t.n_dims : 4));
        out.tensor_type = t.type;
        out.offset = t.offset;
        out.elements = t.n_elements;
        out.bytes = t.data_size;
    }
    oxq_gguf_t g_ = nullptr;
    oxq_gguf_summary s_{};
};

}  // namespace oxq
#endif
