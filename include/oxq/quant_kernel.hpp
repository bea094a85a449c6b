// quant_kernel.hpp -- C++ host mirror of oxillama-quant's kernel interface over the
// C ABI of liboxq_hip.so (include/oxq.h).  Header-only; link with -loxq_hip.
//
// It has the shape of the reference's Rust API so that code (and tests) written
// against the crate read the same here:
//   QuantKernel      crates/oxillama-quant/src/traits.rs:21-183
//   QuantTensor      crates/oxillama-quant/src/types.rs:11-50
//   QuantError       crates/oxillama-quant/src/error.rs:10-71
//   KernelDispatcher crates/oxillama-quant/src/dispatch.rs:141-243
//   quantize_f32_to_q8_0  crates/oxillama-quant/src/quantize.rs:58-75
//   LoraAdapter      crates/oxillama-quant/src/lora.rs:21-124
//   QuantLinear      crates/oxillama-arch/src/common/linear.rs:20-132
// Results come back as QuantResult (Ok / Err(QuantError)); nothing throws.
#ifndef OXQ_QUANT_KERNEL_HPP
#define OXQ_QUANT_KERNEL_HPP

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <utility>
#include <vector>

#include "../oxq.h"

namespace oxq {

// &[T] / &mut [T]: a borrowed pointer + length, valid for the call only.
template <class T>
struct Slice {
    T *ptr = nullptr;
    size_t len = 0;
    Slice() = default;
    Slice(T *p, size_t n) : ptr(p), len(n) {}
    template <class V, class = decltype(std::declval<V &>().data())>
    Slice(V &v) : ptr(v.data()), len(v.size()) {}
    Slice<T> first(size_t n) const { return Slice<T>(ptr, n < len ? n : len); }
};

// GgufTensorType discriminants (crates/oxillama-gguf/src/types.rs:72-150).
enum class GgufTensorType : uint32_t {
    Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9, Q2K = 10, Q3K = 11, Q4K = 12, Q5K = 13, Q6K = 14,
    Iq4Nl = 20, Iq4Xs = 23
};

struct QuantError {
    enum Kind {
        None = 0,
        UnsupportedType = OXQ_ERR_UNSUPPORTED_TYPE,
        BlockSizeMismatch = OXQ_ERR_BLOCK_SIZE_MISMATCH,
        DimensionMismatch = OXQ_ERR_DIMENSION_MISMATCH,
        KernelError = OXQ_ERR_KERNEL,
        BlockCountMismatch = OXQ_ERR_BLOCK_COUNT_MISMATCH,
        BufferTooSmall = OXQ_ERR_BUFFER_TOO_SMALL,
        Internal = OXQ_ERR_INTERNAL,
        UnsupportedShape = OXQ_ERR_UNSUPPORTED_SHAPE,  // library only: retry on the CPU tier
        NoDevice = OXQ_ERR_NO_DEVICE,                  // library only
    };
    Kind kind = None;
    size_t expected = 0;  // expected / needed
    size_t got = 0;       // got / available
    std::string message;

    // Display text of the reference's #[error(...)] attributes (error.rs:12-66).
    std::string to_string() const {
        switch (kind) {
            case UnsupportedType: return "unsupported quantization type: " + message;
            case BlockSizeMismatch:
                return "block size mismatch: expected " + std::to_string(expected) + ", got " + std::to_string(got);
            case DimensionMismatch:
                return "dimension mismatch: expected " + std::to_string(expected) + ", got " + std::to_string(got);
            case BlockCountMismatch:
                return "block count mismatch: expected " + std::to_string(expected) + " blocks, got " +
                       std::to_string(got);
            case BufferTooSmall:
                return "buffer too small: need " + std::to_string(expected) + " bytes, have " + std::to_string(got);
            case Internal: return "internal error: " + message;
            case None: return "ok";
            default: return "kernel error: " + message;
        }
    }
};

// QuantResult<()>
class QuantResult {
  public:
    QuantResult() = default;
    explicit QuantResult(QuantError e) : err_(std::move(e)) {}
    bool is_ok() const { return err_.kind == QuantError::None; }
    bool is_err() const { return !is_ok(); }
    const QuantError &error() const { return err_; }
    explicit operator bool() const { return is_ok(); }

    static QuantResult from_status(int status) {
        if (status == OXQ_OK) return QuantResult();
        QuantError e;
        e.kind = static_cast<QuantError::Kind>(status);
        char msg[256] = {0};
        oxq_last_error(&e.expected, &e.got, msg, sizeof msg);
        e.message = msg;
        return QuantResult(std::move(e));
    }

  private:
    QuantError err_;
};

struct QuantTensor {
    std::vector<uint8_t> data;  // raw GGUF blocks
    std::vector<size_t> shape;  // [out_features, in_features]
    GgufTensorType tensor_type;

    QuantTensor(std::vector<uint8_t> d, std::vector<size_t> s, GgufTensorType t)
        : data(std::move(d)), shape(std::move(s)), tensor_type(t) {}
    size_t n_elements() const {
        if (shape.empty()) return 0;
        size_t n = 1;
        for (size_t d : shape) n *= d;
        return n;
    }
    size_t n_blocks() const {
        const size_t bs = oxq_block_size(static_cast<uint32_t>(tensor_type));
        return bs ? (n_elements() + bs - 1) / bs : 0;
    }
    size_t expected_data_size() const { return n_blocks() * oxq_block_bytes(static_cast<uint32_t>(tensor_type)); }
};

// trait QuantKernel (traits.rs:21-183).
class QuantKernel {
  public:
    virtual ~QuantKernel() = default;
    virtual QuantResult dequant_block(Slice<const uint8_t> block, Slice<float> output) const = 0;
    virtual QuantResult gemv(const QuantTensor &weights, Slice<const float> input, Slice<float> output) const = 0;
    virtual QuantResult gemm(const QuantTensor &weights, Slice<const float> input, Slice<float> output, size_t m,
                             size_t n, size_t k) const = 0;
    // out[r] += ... (accumulates, traits.rs:169)
    virtual QuantResult matvec_q8_fused(Slice<const uint8_t> weights, Slice<const uint8_t> acts_q8, Slice<float> out,
                                        size_t n_rows, size_t n_cols) const = 0;
    virtual size_t block_size() const = 0;
    virtual size_t block_bytes() const = 0;
    virtual const char *name() const = 0;
};

// The GPU tier.  Stateless like the reference's kernels: all methods const, safe to
// share between threads.
class HipKernel final : public QuantKernel {
  public:
    explicit HipKernel(GgufTensorType t) : type_(static_cast<uint32_t>(t)) {}
    QuantResult dequant_block(Slice<const uint8_t> block, Slice<float> output) const override {
        return QuantResult::from_status(oxq_dequant_block(type_, block.ptr, block.len, output.ptr, output.len));
    }
    QuantResult gemv(const QuantTensor &w, Slice<const float> input, Slice<float> output) const override {
        return QuantResult::from_status(oxq_gemv(type_, w.data.data(), w.data.size(), w.shape.data(), w.shape.size(),
                                                 input.ptr, input.len, output.ptr, output.len));
    }
    QuantResult gemm(const QuantTensor &w, Slice<const float> input, Slice<float> output, size_t m, size_t n,
                     size_t k) const override {
        return QuantResult::from_status(oxq_gemm(type_, w.data.data(), w.data.size(), w.shape.data(), w.shape.size(),
                                                 input.ptr, input.len, output.ptr, output.len, m, n, k));
    }
    QuantResult matvec_q8_fused(Slice<const uint8_t> weights, Slice<const uint8_t> acts_q8, Slice<float> out,
                                size_t n_rows, size_t n_cols) const override {
        return QuantResult::from_status(oxq_matvec_q8_fused(type_, weights.ptr, weights.len, acts_q8.ptr, acts_q8.len,
                                                            out.ptr, out.len, n_rows, n_cols));
    }
    size_t block_size() const override { return oxq_block_size(type_); }
    size_t block_bytes() const override { return oxq_block_bytes(type_); }
    const char *name() const override { return oxq_type_name(type_); }

    // Debug: exact int32 group sums of the fused kernel (no reference counterpart).
    QuantResult block_sums(Slice<const uint8_t> weights, Slice<const uint8_t> acts_q8, Slice<int32_t> sums,
                           size_t n_rows, size_t n_cols) const {
        return QuantResult::from_status(oxq_block_sums(type_, weights.ptr, weights.len, acts_q8.ptr, acts_q8.len,
                                                       sums.ptr, sums.len, n_rows, n_cols));
    }

  private:
    uint32_t type_;
};

// Which arithmetic gemv / gemm / QuantLinear::forward use for their fp32 input (process-wide, oxq.h):
// Q8 = quantize to Q8_0 and run the fused kernels (the default, the reference's matvec_q8_fused arithmetic);
// F32 = the reference's own gemv arithmetic (Q/reference/q4_k.rs:135-178 and siblings), five formats.
enum class ActivationRoute : int { Q8 = OXQ_ROUTE_Q8, F32 = OXQ_ROUTE_F32 };

// KernelDispatcher (dispatch.rs:141-243) with a single tier: the GPU.
class KernelDispatcher {
  public:
    // Probes the device once (SimdCapabilities::detect, dispatch.rs:42).
    explicit KernelDispatcher(int device = 0) : init_status_(oxq_init(device)) {}
    bool has_device() const { return init_status_ == OXQ_OK; }
    static QuantResult select_activation_route(ActivationRoute r) {
        return QuantResult::from_status(oxq_select_activation_route(static_cast<int>(r)));
    }
    static ActivationRoute activation_route() { return static_cast<ActivationRoute>(oxq_activation_route()); }

    // Ok(Box<dyn QuantKernel>) or Err(UnsupportedType{quant_type}).
    QuantResult get_kernel(uint32_t tensor_type, std::unique_ptr<QuantKernel> &out) const {
        const int st = oxq_get_kernel(tensor_type);
        if (st != OXQ_OK) {
            QuantError e;
            e.kind = QuantError::UnsupportedType;
            e.message = "type id " + std::to_string(tensor_type);
            return QuantResult(std::move(e));
        }
        out.reset(new HipKernel(static_cast<GgufTensorType>(tensor_type)));
        return QuantResult();
    }
    QuantResult get_kernel(GgufTensorType t, std::unique_ptr<QuantKernel> &out) const {
        return get_kernel(static_cast<uint32_t>(t), out);
    }

  private:
    int init_status_;
};

// LoraAdapter (crates/oxillama-quant/src/lora.rs:21-124): delta = B (A input) * scale, A is
// [rank x in_features], B is [out_features x rank], both row-major.
struct LoraAdapter {
    std::vector<float> a, b;
    size_t rank = 0;
    float scale = 0.0f;
    size_t in_features = 0, out_features = 0;

    // LoraAdapter::new (lora.rs:43-73): Err(DimensionMismatch) when a matrix has the wrong size.
    static QuantResult create(std::vector<float> a, std::vector<float> b, size_t rank, float scale, size_t in_features,
                              size_t out_features, std::shared_ptr<LoraAdapter> &out) {
        auto mismatch = [](size_t expected, size_t got) {
            QuantError e;
            e.kind = QuantError::DimensionMismatch;
            e.expected = expected;
            e.got = got;
            return QuantResult(std::move(e));
        };
        if (a.size() != rank * in_features) return mismatch(rank * in_features, a.size());
        if (b.size() != out_features * rank) return mismatch(out_features * rank, b.size());
        out = std::make_shared<LoraAdapter>();
        out->a = std::move(a);
        out->b = std::move(b);
        out->rank = rank;
        out->scale = scale;
        out->in_features = in_features;
        out->out_features = out_features;
        return QuantResult();
    }
};

// QuantLinear (crates/oxillama-arch/src/common/linear.rs:20-132).
struct QuantLinear {
    QuantTensor weight;
    std::vector<float> bias;  // empty = none
    bool has_bias = false;
    size_t out_features = 0, in_features = 0;
    std::shared_ptr<LoraAdapter> lora;

    explicit QuantLinear(QuantTensor w) : weight(std::move(w)) { dims(); }
    QuantLinear(QuantTensor w, std::vector<float> b) : weight(std::move(w)), bias(std::move(b)), has_bias(true) { dims(); }
    void set_lora(std::shared_ptr<LoraAdapter> l) { lora = std::move(l); }
    void clear_lora() { lora.reset(); }

    // output = weight @ input + bias [+ lora delta] (linear.rs:77-98), one call across the ABI.
    QuantResult forward(const QuantKernel &kernel, Slice<const float> input, Slice<float> output) const {
        (void)kernel;  // the tensor's own type selects the GPU kernel, as get_kernel(weight.tensor_type) does
        const LoraAdapter *l = lora.get();
        return QuantResult::from_status(oxq_linear_forward(
            static_cast<uint32_t>(weight.tensor_type), weight.data.data(), weight.data.size(), weight.shape.data(),
            weight.shape.size(), has_bias ? bias.data() : nullptr, has_bias ? bias.size() : 0, l ? l->a.data() : nullptr,
            l ? l->a.size() : 0, l ? l->b.data() : nullptr, l ? l->b.size() : 0, l ? l->rank : 0, l ? l->scale : 0.0f,
            input.ptr, input.len, output.ptr, output.len));
    }
    // output[batch x out_features] = gemm + bias broadcast (linear.rs:105-132).
    QuantResult forward_batch(const QuantKernel &kernel, Slice<const float> input, Slice<float> output,
                              size_t batch_size) const {
        (void)kernel;
        return QuantResult::from_status(oxq_linear_forward_batch(
            static_cast<uint32_t>(weight.tensor_type), weight.data.data(), weight.data.size(), weight.shape.data(),
            weight.shape.size(), has_bias ? bias.data() : nullptr, has_bias ? bias.size() : 0, input.ptr, input.len,
            output.ptr, output.len, batch_size));
    }

  private:
    void dims() {  // linear.rs:38-48
        out_features = weight.shape.empty() ? 0 : weight.shape[0];
        in_features = weight.shape.size() < 2 ? 0 : weight.shape[1];
    }
};

// quantize_f32_to_q8_0 (quantize.rs:58-75): Ok(Vec<u8>) of data.len()/32 * 34 bytes.
inline QuantResult quantize_f32_to_q8_0(Slice<const float> data, std::vector<uint8_t> &out) {
    out.assign(data.len / 32 * 34, 0);
    return QuantResult::from_status(oxq_quantize_f32_to_q8_0(data.ptr, data.len, out.data(), out.size()));
}

}  // namespace oxq
#endif  // OXQ_QUANT_KERNEL_HPP
