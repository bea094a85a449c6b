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
