// C++ mirror of the reference's mixture-of-experts feed-forward layer
// (crates/oxillama-arch/src/common/moe.rs:20-258) over the C ABI of include/oxq.h, with the
// experts' projections held as GGUF blocks (QuantTensor) instead of dense fp32 matrices.
//
//   reference                                   here
//   Expert { gate, up, down: Vec<f32>, .. }     QuantExpert { gate, up, down: QuantTensor }
//   MoeFfn { router, experts, top_k, .. }       MoeFfn { router, experts, top_k, .. }
//   MoeFfn::forward(input, output)              MoeFfn::forward(input, output)      (one token)
//                                               MoeFfn::forward_batch(input, output, n_tokens)
//
// Errors come back as QuantResult: the reference's ArchError::InvalidShape maps to
// DimensionMismatch {expected, got}, InvalidConfig (top_k = 0) to KernelError.
#ifndef OXQ_MOE_FFN_HPP
#define OXQ_MOE_FFN_HPP

#include <vector>

#include "quant_kernel.hpp"

namespace oxq {

// Expert (moe.rs:20-30): gate / up are [intermediate x hidden], down is [hidden x intermediate].
struct QuantExpert {
    QuantTensor gate, up, down;
};

struct MoeFfn {
    std::vector<float> router;  // [num_experts x hidden_size], row-major (moe.rs:139)
    std::vector<QuantExpert> experts;
    size_t top_k = 0, num_experts = 0, hidden_size = 0, intermediate_size = 0;

    // MoeFfn::forward (moe.rs:184-258): output overwritten.
    QuantResult forward(Slice<const float> input, Slice<float> output) const { return forward_batch(input, output, 1); }

    // The same for n_tokens input vectors stored back to back.
    QuantResult forward_batch(Slice<const float> input, Slice<float> output, size_t n_tokens) const {
        auto mismatch = [](size_t expected, size_t got) {
            QuantError e;
            e.kind = QuantError::DimensionMismatch;
            e.expected = expected;
            e.got = got;
            return QuantResult(std::move(e));
        };
        if (router.size() != num_experts * hidden_size) return mismatch(num_experts * hidden_size, router.size());
        if (experts.size() != num_experts) return mismatch(num_experts, experts.size());  // moe.rs:161-167
        if (num_experts == 0)
            return QuantResult::from_status(oxq_moe_forward(OXQ_TYPE_Q8_0, nullptr, 0, OXQ_TYPE_Q8_0, nullptr, 0,
                                                            OXQ_TYPE_Q8_0, nullptr, 0, router.data(), router.size(), 0,
                                                            hidden_size, intermediate_size, top_k, input.ptr,
                                                            input.len, output.ptr, output.len, n_tokens));
        // the ABI takes the experts' matrices back to back, one format per projection
        const GgufTensorType tg = experts[0].gate.tensor_type, tu = experts[0].up.tensor_type,
                             td = experts[0].down.tensor_type;
        size_t ng = 0, nu = 0, nd = 0;
        for (const QuantExpert &e : experts) {
            if (e.gate.tensor_type != tg || e.up.tensor_type != tu || e.down.tensor_type != td) {
                QuantError err;
                err.kind = QuantError::KernelError;
                err.message = "experts of one layer must share their three formats";
                return QuantResult(std::move(err));
            }
            ng += e.gate.data.size();
            nu += e.up.data.size();
            nd += e.down.data.size();
        }
        if (packed_.empty() || packed_.size() != ng + nu + nd) {  // packed once, reused by later calls
            packed_.clear();
            packed_.reserve(ng + nu + nd);
            for (const QuantExpert &e : experts) packed_.insert(packed_.end(), e.gate.data.begin(), e.gate.data.end());
            for (const QuantExpert &e : experts) packed_.insert(packed_.end(), e.up.data.begin(), e.up.data.end());
            for (const QuantExpert &e : experts) packed_.insert(packed_.end(), e.down.data.begin(), e.down.data.end());
        }
        return QuantResult::from_status(oxq_moe_forward(
            static_cast<uint32_t>(tg), packed_.data(), ng, static_cast<uint32_t>(tu), packed_.data() + ng, nu,
            static_cast<uint32_t>(td), packed_.data() + ng + nu, nd, router.data(), router.size(), num_experts,
            hidden_size, intermediate_size, top_k, input.ptr, input.len, output.ptr, output.len, n_tokens));
    }

  private:
    mutable std::vector<uint8_t> packed_;
};

}  // namespace oxq
#endif  // OXQ_MOE_FFN_HPP
