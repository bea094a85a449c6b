"""Python mirror of the callers of the kernel trait, over liboxq_hip.so.

  LoraAdapter      crates/oxillama-quant/src/lora.rs:21-124
  QuantLinear      crates/oxillama-arch/src/common/linear.rs:20-132
  swiglu / rmsnorm crates/oxillama-arch/src/common/swiglu.rs:15-21, rms_norm.rs:49-66
  dense FFN        crates/oxillama-arch/src/llama/model.rs:277-310

`QuantLinear.forward` crosses the C ABI with numpy host buffers (everything staged per call);
the `*_dev` functions take torch CUDA tensors and enqueue on torch's current stream.
"""
import ctypes as C

import numpy as np

from . import capi
from .quant import DimensionMismatch, HipKernel, QuantTensor, _check, _ptr, _u8


class LoraAdapter:
    """delta = B @ (A @ input) * scale; A is [rank x in_features], B is [out_features x rank]."""

    def __init__(self, a, b, rank, scale, in_features, out_features):
        a = np.ascontiguousarray(a, dtype=np.float32).ravel()
        b = np.ascontiguousarray(b, dtype=np.float32).ravel()
        if a.size != rank * in_features:  # lora.rs:51-57
            raise DimensionMismatch(rank * in_features, a.size)
        if b.size != out_features * rank:  # lora.rs:58-64
            raise DimensionMismatch(out_features * rank, b.size)
        self.a, self.b, self.rank, self.scale = a, b, rank, float(scale)
        self.in_features, self.out_features = in_features, out_features


class QuantLinear:
    """weight: QuantTensor [out_features, in_features]; optional fp32 bias; optional LoRA."""

    def __init__(self, weight: QuantTensor, bias=None):
        self.weight = weight
        self.bias = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32).ravel()
        self.out_features = weight.shape[0] if len(weight.shape) > 0 else 0  # linear.rs:38-48
        self.in_features = weight.shape[1] if len(weight.shape) > 1 else 0
        self.lora = None

    def set_lora(self, lora):
        self.lora = lora

    def clear_lora(self):
        self.lora = None

    def forward(self, kernel: HipKernel, input, output):
        """output = weight @ input + bias [+ lora delta] (linear.rs:77-98); output is filled in place."""
        lib = capi.load()
        w = _u8(self.weight.data)
        shape = (C.c_size_t * len(self.weight.shape))(*self.weight.shape)
        x = np.ascontiguousarray(input, dtype=np.float32).ravel()
        bias_p, bias_n = (_ptr(self.bias), self.bias.size) if self.bias is not None else (None, 0)
        if self.lora is not None:
            la, lb = self.lora.a, self.lora.b
            lora_args = (_ptr(la), la.size, _ptr(lb), lb.size, self.lora.rank, self.lora.scale)
        else:
            lora_args = (None, 0, None, 0, 0, 0.0)
        _check(lib.oxq_linear_forward(kernel.tensor_type, _ptr(w), w.size, shape, len(self.weight.shape), bias_p,
                                      bias_n, *lora_args, _ptr(x), x.size, _ptr(output), output.size))

    def forward_batch(self, kernel: HipKernel, input, output, batch_size):
        """output[batch x out] = gemm + bias broadcast (linear.rs:105-132; no LoRA in batch mode)."""
        lib = capi.load()
        w = _u8(self.weight.data)
        shape = (C.c_size_t * len(self.weight.shape))(*self.weight.shape)
        x = np.ascontiguousarray(input, dtype=np.float32).ravel()
        bias_p, bias_n = (_ptr(self.bias), self.bias.size) if self.bias is not None else (None, 0)
        _check(lib.oxq_linear_forward_batch(kernel.tensor_type, _ptr(w), w.size, shape, len(self.weight.shape),
                                            bias_p, bias_n, _ptr(x), x.size, _ptr(output), output.size, batch_size))


# ---- device route -------------------------------------------------------------------------


class LoraStruct(C.Structure):
    _fields_ = [("d_a", C.c_void_p), ("d_b", C.c_void_p), ("d_r", C.c_void_p), ("rank", C.c_size_t),
                ("scale", C.c_float)]


def _stream():
    return HipKernel._stream()


def _opt(t):
    return t.data_ptr() if t is not None else None


def lora_struct(d_a, d_b, d_r, rank, scale):
    return LoraStruct(d_a.data_ptr(), d_b.data_ptr(), d_r.data_ptr(), rank, scale)


def lora_apply_dev(lora, d_x, d_out, out_features, in_features):
    _check(capi.load().oxq_lora_apply_dev(C.byref(lora), d_x.data_ptr(), d_out.data_ptr(), out_features, in_features,
                                          _stream()))


def linear_forward_dev(tensor_type, d_weights, d_out, out_features, in_features, d_x=None, d_acts=None, d_bias=None,
                       lora=None):
    _check(capi.load().oxq_linear_forward_dev(int(tensor_type), d_weights.data_ptr(), _opt(d_x), _opt(d_acts),
                                              _opt(d_bias), C.byref(lora) if lora is not None else None,
                                              d_out.data_ptr(), out_features, in_features, _stream()))


def linear_forward_multi_dev(tensor_type, d_weights, d_acts, d_outs, out_features, in_features, d_biases=None):
    n = len(d_weights)
    wp = (C.c_void_p * n)(*[w.data_ptr() for w in d_weights])
    op = (C.c_void_p * n)(*[o.data_ptr() for o in d_outs])
    bp = (C.c_void_p * n)(*[_opt(b) for b in d_biases]) if d_biases is not None else None
    of = (C.c_size_t * n)(*out_features)
    _check(capi.load().oxq_linear_forward_multi_dev(int(tensor_type), n, wp, d_acts.data_ptr(), bp, op, of,
                                                    in_features, _stream()))


def linear_forward_batch_dev(tensor_type, d_weights, d_acts, d_out, batch, out_features, in_features, d_bias=None,
                             workspace=None):
    _check(capi.load().oxq_linear_forward_batch_dev(int(tensor_type), d_weights.data_ptr(), d_acts.data_ptr(),
                                                    _opt(d_bias), d_out.data_ptr(), batch, out_features, in_features,
                                                    _opt(workspace), workspace.numel() if workspace is not None else 0,
                                                    _stream()))


def swiglu_quantize_dev(d_gate, d_up, d_h=None, d_out_q8=None):
    _check(capi.load().oxq_swiglu_quantize_q8_0_dev(d_gate.data_ptr(), d_up.data_ptr(), d_gate.numel(), _opt(d_h),
                                                    _opt(d_out_q8), _stream()))


def rmsnorm_quantize_dev(d_x, d_weight, eps, rows, n, d_y=None, d_out_q8=None):
    _check(capi.load().oxq_rmsnorm_quantize_q8_0_dev(d_x.data_ptr(), d_weight.data_ptr(), float(eps), rows, n,
                                                     _opt(d_y), _opt(d_out_q8), _stream()))


def gate_up_swiglu_dev(tensor_type, d_gate, d_up, d_acts_q8, d_h, d_out_q8, intermediate, hidden):
    """ffn_gate + ffn_up + SwiGLU + Q8_0 quantizer of h in one launch (d_h optional)."""
    _check(capi.load().oxq_ffn_gate_up_swiglu_q8_dev(int(tensor_type), d_gate.data_ptr(), d_up.data_ptr(),
                                                     d_acts_q8.data_ptr(), d_h.data_ptr() if d_h is not None else None,
                                                     d_out_q8.data_ptr(), intermediate, hidden, HipKernel._stream()))


def ffn_workspace_bytes(hidden, intermediate):
    return capi.load().oxq_ffn_workspace_bytes(hidden, intermediate)


def ffn_swiglu_dev(gate, up, down, d_acts, d_out, hidden, intermediate, workspace):
    """gate/up/down: (tensor_type, device weights).  d_out = down(silu(gate x) * up x)."""
    _check(capi.load().oxq_ffn_swiglu_dev(int(gate[0]), gate[1].data_ptr(), int(up[0]), up[1].data_ptr(),
                                          int(down[0]), down[1].data_ptr(), d_acts.data_ptr(), d_out.data_ptr(),
                                          hidden, intermediate, workspace.data_ptr(), workspace.numel(), _stream()))


def topk_dev(d_values, k, d_out_values, d_out_indices, workspace):
    """The k largest of a float32 CUDA tensor, largest first, with their indices (uint32 viewed as int32)."""
    lib = capi.load()
    _check(lib.oxq_topk_dev(d_values.data_ptr(), d_values.numel(), k, d_out_values.data_ptr(), d_out_indices.data_ptr(),
                            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream()))


def lm_head_topk_workspace_bytes(quant_type, n_rows, n_cols, k):
    return capi.load().oxq_lm_head_topk_workspace_bytes(quant_type, n_rows, n_cols, k)


def lm_head_topk_dev(quant_type, d_weights, d_acts_q8, d_logits, n_rows, n_cols, k, d_out_values, d_out_indices, workspace):
    """The vocabulary projection (logits to d_logits) and the k largest logits with their row indices, in one launch
    where the shape allows it (oxq_lm_head_topk_dev)."""
    _check(capi.load().oxq_lm_head_topk_dev(quant_type, d_weights.data_ptr(), d_acts_q8.data_ptr(), d_logits.data_ptr(),
                                            n_rows, n_cols, k, d_out_values.data_ptr(), d_out_indices.data_ptr(),
                                            workspace.data_ptr(), workspace.numel() * workspace.element_size(), _stream()))


def logits_edit_dev(d_logits, d_banned=None, d_bias_tokens=None, d_bias_values=None, d_recent=None, window=0,
                    repetition_penalty=1.0):
    """The sampler's edits of the logits before the candidate list (sampling/mod.rs:573-613), in place: banned tokens,
    logit bias, repetition penalty over the last `window` of d_recent.  Token lists: int32 / uint32 CUDA tensors."""
    def ptr(t):
        return t.data_ptr() if t is not None and t.numel() else None

    def cnt(t):
        return t.numel() if t is not None else 0
    _check(capi.load().oxq_logits_edit_dev(d_logits.data_ptr(), d_logits.numel(), ptr(d_banned), cnt(d_banned),
                                           ptr(d_bias_tokens), ptr(d_bias_values), cnt(d_bias_tokens), ptr(d_recent),
                                           cnt(d_recent), window, repetition_penalty, _stream()))


def sample_candidates_dev(d_values, d_indices, k, temperature, min_p, top_p, d_rng_state, d_token, d_probs=None):
    """The sampler after its candidate list (sampling/mod.rs:487-564): temperature, softmax, min-p, top-p, the draw.
    d_rng_state: one uint64 (the reference's Xorshift64 state), d_token: one uint32, d_probs: optional k floats."""
    lib = capi.load()
    _check(lib.oxq_sample_candidates_dev(d_values.data_ptr(), d_indices.data_ptr(), k, temperature, min_p, top_p,
                                         d_rng_state.data_ptr(), d_token.data_ptr(),
                                         d_probs.data_ptr() if d_probs is not None else None, _stream()))


def topk_workspace_bytes(n, k):
    return capi.load().oxq_topk_workspace_bytes(n, k)
