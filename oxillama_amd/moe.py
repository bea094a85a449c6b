"""Host-side mirror of the reference's mixture-of-experts routing, and the grouping of
(token, expert) pairs that the grouped expert matmul (oxq_moe_gemm_q8_dev) consumes.

Routing follows MoeFfn::forward, crates/oxillama-arch/src/common/moe.rs:197-248: a
numerically stable softmax over the router logits, the top-k experts by descending
softmax weight, weights renormalised over the selected experts.  All arithmetic is fp32.
"""
import numpy as np


def route_top_k(logits, top_k):
    """logits: float32 [n_tokens, n_experts] -> (experts int32 [n_tokens, k], weights float32
    [n_tokens, k]), experts in descending order of softmax weight (moe.rs:201-248)."""
    logits = np.asarray(logits, dtype=np.float32)
    n_tok, n_exp = logits.shape
    if top_k < 1:
        raise ValueError("MoeFfn top_k must be >= 1")  # moe.rs:167-171
    k = min(top_k, n_exp)
    mx = logits.max(axis=1, keepdims=True)
    ev = np.exp(logits - mx, dtype=np.float32)
    tot = ev.sum(axis=1, keepdims=True, dtype=np.float32)
    probs = np.where(tot > 0, ev / np.where(tot > 0, tot, 1), np.float32(1.0 / n_exp)).astype(np.float32)
    order = np.argsort(-probs, axis=1, kind="stable")[:, :k].astype(np.int32)
    sel = np.take_along_axis(probs, order, axis=1)
    ssum = sel.sum(axis=1, keepdims=True, dtype=np.float32)
    weights = np.where(ssum > 1e-9, sel / np.where(ssum > 1e-9, ssum, 1), np.float32(1.0 / k)).astype(np.float32)
    return order, weights


def group_by_expert(experts, n_experts):
    """experts int32 [n_tokens, k] -> (offsets int32 [n_experts + 1], token int32 [pairs], slot
    int32 [pairs]): pair rows sorted by expert (tokens ascending inside an expert); row r of
    the grouped matrices belongs to token[r] and is its slot[r]-th choice."""
    n_tok, k = experts.shape
    flat = experts.reshape(-1)
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=n_experts)
    offsets = np.zeros(n_experts + 1, dtype=np.int32)
    offsets[1:] = np.cumsum(counts)
    return offsets, (order // k).astype(np.int32), (order % k).astype(np.int32)


def token_rows(offsets, token, slot, n_tokens, k):
    """Inverse of the grouping: int32 [n_tokens, k], the grouped row of each token's j-th choice."""
    rows = np.zeros((n_tokens, k), dtype=np.int32)
    rows[token, slot] = np.arange(token.size, dtype=np.int32)
    return rows


def route_dev(d_router, d_x, n_tokens, n_experts, hidden, top_k, d_experts, d_weights, d_offsets, d_pair_token,
              d_token_rows):
    """Steps 1-4 of MoeFfn::forward (moe.rs:189-250) and the grouping, on torch CUDA tensors."""
    from . import capi
    from .quant import HipKernel, _check
    _check(capi.load().oxq_moe_route_dev(d_router.data_ptr(), d_x.data_ptr(), n_tokens, n_experts, hidden, top_k,
                                         d_experts.data_ptr(), d_weights.data_ptr(), d_offsets.data_ptr(),
                                         d_pair_token.data_ptr(), d_token_rows.data_ptr(), HipKernel._stream()))


def gather_quantize_dev(d_x, d_pair_token, n_pairs, hidden, d_out_q8):
    from . import capi
    from .quant import HipKernel, _check
    _check(capi.load().oxq_moe_gather_quantize_q8_0_dev(d_x.data_ptr(), d_pair_token.data_ptr(), n_pairs, hidden,
                                                        d_out_q8.data_ptr(), HipKernel._stream()))


def combine_dev(d_y_pairs, d_token_rows, d_weights, n_tokens, top_k, hidden, d_out):
    from . import capi
    from .quant import HipKernel, _check
    _check(capi.load().oxq_moe_combine_dev(d_y_pairs.data_ptr(), d_token_rows.data_ptr(), d_weights.data_ptr(),
                                           n_tokens, top_k, hidden, d_out.data_ptr(), HipKernel._stream()))


def moe_ffn_workspace_bytes(types, n_pairs, hidden, intermediate):
    from . import capi
    tg, tu, td = (int(t) for t in types)
    return capi.load().oxq_moe_ffn_workspace_bytes(tg, tu, td, n_pairs, hidden, intermediate)


def moe_ffn_dev(gate, up, down, n_experts, d_x, n_tokens, top_k, d_offsets, d_pair_token, d_token_rows, d_weights,
                max_rows, d_out, hidden, intermediate, workspace):
    """MoeFfn::forward (moe.rs:184-258) after routing, for n_tokens tokens on torch CUDA tensors, current
    stream.  gate / up / down: (tensor_type, device tensor of all experts, bytes per expert)."""
    from . import capi
    from .quant import HipKernel, _check
    args = []
    for t, d_w, stride in (gate, up, down):
        args += [int(t), d_w.data_ptr(), stride]
    _check(capi.load().oxq_moe_ffn_dev(*args, n_experts, d_x.data_ptr(), n_tokens, top_k, d_offsets.data_ptr(),
                                       d_pair_token.data_ptr(), d_token_rows.data_ptr(), d_weights.data_ptr(),
                                       max_rows, d_out.data_ptr(), hidden, intermediate, workspace.data_ptr(),
                                       workspace.numel(), HipKernel._stream()))


def moe_forward_workspace_bytes(types, n_tokens, top_k, n_experts, hidden, intermediate):
    from . import capi
    tg, tu, td = (int(t) for t in types)
    return capi.load().oxq_moe_forward_workspace_bytes(tg, tu, td, n_tokens, top_k, n_experts, hidden, intermediate)


def moe_forward_dev(gate, up, down, n_experts, d_router, d_x, n_tokens, top_k, d_out, hidden, intermediate, workspace):
    """MoeFfn::forward (moe.rs:184-258) for n_tokens tokens on torch CUDA tensors, current stream: routing and
    the experts in one call, tables in the workspace.  gate / up / down as in moe_ffn_dev."""
    from . import capi
    from .quant import HipKernel, _check
    args = []
    for t, d_w, stride in (gate, up, down):
        args += [int(t), d_w.data_ptr(), stride]
    _check(capi.load().oxq_moe_forward_dev(*args, n_experts, d_router.data_ptr(), d_x.data_ptr(), n_tokens, top_k,
                                           d_out.data_ptr(), hidden, intermediate, workspace.data_ptr(),
                                           workspace.numel(), HipKernel._stream()))


class MoeFfn:
    """MoeFfn of the reference (moe.rs:129-258) with the experts' projections as GGUF blocks.

    gate / up / down: (tensor_type, uint8 array holding the matrices of all experts back to back).
    forward() takes one input vector like the reference's; forward_batch() takes n_tokens of them.
    Errors are the QuantError classes of oxillama_amd.quant (InvalidShape -> DimensionMismatch,
    InvalidConfig -> KernelError)."""

    def __init__(self, router, gate, up, down, top_k, num_experts, hidden_size, intermediate_size):
        self.router = np.ascontiguousarray(router, dtype=np.float32).ravel()
        self.gate, self.up, self.down = ((int(t), np.ascontiguousarray(w).view(np.uint8).ravel())
                                         for t, w in (gate, up, down))
        self.top_k, self.num_experts = top_k, num_experts
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size

    def forward(self, x, out=None):
        return self.forward_batch(x, 1, out)

    def forward_batch(self, x, n_tokens, out=None):
        import ctypes as C
        from . import capi
        from .quant import _check
        x = np.ascontiguousarray(x, dtype=np.float32).ravel()
        if out is None:
            out = np.zeros(n_tokens * self.hidden_size, dtype=np.float32)
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        (tg, g), (tu, u), (td, d) = self.gate, self.up, self.down
        _check(capi.load().oxq_moe_forward(tg, vp(g), g.size, tu, vp(u), u.size, td, vp(d), d.size, vp(self.router),
                                           self.router.size, self.num_experts, self.hidden_size,
                                           self.intermediate_size, self.top_k, vp(x), x.size, vp(out), out.size,
                                           n_tokens))
        return out
