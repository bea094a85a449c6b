"""Pins the oracle's restatement of the reference's mixture-of-experts layer
(oracle/oxq_oracle_moe.c, following crates/oxillama-arch/src/common/moe.rs) against the
reference's own test cases (moe.rs:262-450), closed forms and float64 recomputation."""
import math

import numpy as np
import pytest

import oracle as O
from oxillama_amd import moe


def ones_expert(h, n):  # moe.rs:266-274
    return np.ones(n * h, np.float32), np.ones(n * h, np.float32), np.ones(h * n, np.float32)


def test_expert_forward_all_ones_closed_form():
    # moe.rs:277-289: gate = up = h, silu(h) * h summed over n rows of ones
    h, n = 4, 8
    out = O.expert_forward(*ones_expert(h, n), h, n, np.ones(h, np.float32))
    want = n * h * h / (1.0 + math.exp(-h))
    assert np.all(np.abs(out - want) <= 1e-5 * want) and np.all(np.abs(out) > 1e-6)


def test_expert_forward_zero_input_overwrites_output():
    # moe.rs:291-305
    out = O.expert_forward(*ones_expert(4, 8), 4, 8, np.zeros(4, np.float32))
    assert np.all(np.abs(out) < 1e-6)


def test_expert_forward_wrong_gate_size():
    # moe.rs:307-322
    g, u, d = ones_expert(4, 8)
    with pytest.raises(O.OracleError) as e:
        O.expert_forward(g[:3], u, d, 4, 8, np.ones(4, np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 32, 3)


def test_expert_forward_against_float64():
    rng = np.random.default_rng(11)
    h, n = 48, 80
    g, u, d = (rng.standard_normal(n * h).astype(np.float32) * 0.2 for _ in range(3))
    x = rng.standard_normal(h).astype(np.float32)
    out = O.expert_forward(g, u, d, h, n, x)
    g64, u64 = g.reshape(n, h).astype(np.float64), u.reshape(n, h).astype(np.float64)
    gv = g64 @ x
    hv = gv / (1 + np.exp(-gv)) * (u64 @ x)
    want = d.reshape(h, n).astype(np.float64) @ hv
    assert np.max(np.abs(out - want)) <= 1e-5 * np.max(np.abs(want))
    # a dropped sigmoid, or a down matrix read column-major, would not pass
    d64 = d.astype(np.float64)
    assert np.max(np.abs(out - d64.reshape(h, n) @ (gv * (u64 @ x)))) > 1e-2 * np.max(np.abs(want))
    assert np.max(np.abs(out - d64.reshape(n, h).T @ hv)) > 1e-2 * np.max(np.abs(want))


def test_route_one_hot_router_prefers_expert_0():
    # moe.rs:324-352
    h, n_exp = 4, 4
    router = np.zeros(n_exp * h, np.float32)
    router[0] = 1.0
    sel, wt = O.moe_route(router, n_exp, h, 1, [1, 0, 0, 0])
    assert sel.tolist() == [0] and wt.tolist() == [1.0]
    sel, wt = O.moe_route(router, n_exp, h, 2, [1, 0, 0, 0])
    e = math.e
    assert sel.tolist() == [0, 1] and abs(wt[0] - e / (e + 1)) < 1e-6 and abs(wt[1] - 1 / (e + 1)) < 1e-6


def test_route_uniform_router_gives_equal_weights():
    # moe.rs:354-379: equal logits -> equal softmax -> 1/k each
    sel, wt = O.moe_route(np.ones(16, np.float32), 4, 4, 2, np.ones(4, np.float32))
    assert sel.tolist() == [0, 1] and wt.tolist() == [0.5, 0.5]


def test_route_top_k_above_expert_count_clamps():
    # moe.rs:381-401
    sel, wt = O.moe_route(np.ones(16, np.float32), 4, 4, 10, np.ones(4, np.float32))
    assert sorted(sel.tolist()) == [0, 1, 2, 3] and wt.tolist() == [0.25] * 4


def test_route_errors():
    # moe.rs:403-424 (top_k = 0), moe.rs:426-450 (router size)
    with pytest.raises(O.OracleError) as e:
        O.moe_route(np.ones(8, np.float32), 2, 4, 0, np.ones(4, np.float32))
    assert e.value.code == O.KERNEL_ERROR
    with pytest.raises(O.OracleError) as e:
        O.moe_route(np.ones(5, np.float32), 2, 4, 1, np.ones(4, np.float32))
    assert (e.value.code, e.value.a, e.value.b) == (O.DIMENSION_MISMATCH, 8, 5)


@pytest.mark.parametrize("n_exp,k", [(8, 2), (64, 6), (5, 5)])
def test_route_against_float64_softmax(n_exp, k):
    rng = np.random.default_rng(n_exp)
    h = 96
    router = rng.standard_normal(n_exp * h).astype(np.float32) * 0.3
    x = rng.standard_normal(h).astype(np.float32)
    sel, wt = O.moe_route(router, n_exp, h, k, x)
    logits = router.reshape(n_exp, h).astype(np.float64) @ x
    p = np.exp(logits - logits.max())
    p /= p.sum()
    order = np.argsort(-p, kind="stable")[:k]
    assert sel.tolist() == order.tolist()
    assert np.max(np.abs(wt - p[order] / p[order].sum())) < 1e-6
    assert abs(float(wt.sum()) - 1) < 1e-6 and np.all(np.diff(wt) <= 0)
    # the host-side mirror used by the product's callers agrees on the same logits
    exp2, wt2 = moe.route_top_k(logits.astype(np.float32)[None, :], k)
    assert exp2[0].tolist() == sel.tolist() and np.max(np.abs(wt2[0] - wt)) < 1e-6


def test_route_degenerate_logits():
    # -inf everywhere but one expert: exp() underflows to 0 for the rest; weights stay finite
    router = np.zeros(4 * 4, np.float32)
    router[4] = 200.0
    sel, wt = O.moe_route(router, 4, 4, 2, [1, 0, 0, 0])
    assert sel.tolist() == [1, 0] and wt[0] == 1.0 and wt[1] == 0.0


def test_moe_forward_identical_experts_ignore_routing():
    # moe.rs:354-379 strengthened: equal experts and weights summing to 1 -> the expert's own output
    h, n, n_exp = 4, 4, 4
    g, u, d = ones_expert(h, n)
    one = O.expert_forward(g, u, d, h, n, np.ones(h, np.float32))
    for k in (1, 2, 10):
        out = O.moe_forward(np.ones(n_exp * h, np.float32), np.tile(g, n_exp), np.tile(u, n_exp), np.tile(d, n_exp),
                            n_exp, h, n, k, np.ones(h, np.float32))
        assert np.max(np.abs(out - one)) <= 1e-6 * np.max(np.abs(one))
    with pytest.raises(O.OracleError):  # moe.rs:403-424
        O.moe_forward(np.ones(n_exp * h, np.float32), np.tile(g, n_exp), np.tile(u, n_exp), np.tile(d, n_exp), n_exp,
                      h, n, 0, np.ones(h, np.float32))


def test_moe_forward_is_the_weighted_sum_of_the_selected_experts():
    rng = np.random.default_rng(5)
    h, n, n_exp, k = 32, 64, 6, 3
    g, u, d = (rng.standard_normal(n_exp * n * h).astype(np.float32) * 0.2 for _ in range(3))
    router = rng.standard_normal(n_exp * h).astype(np.float32)
    x = rng.standard_normal(h).astype(np.float32)
    out = O.moe_forward(router, g, u, d, n_exp, h, n, k, x)
    sel, wt = O.moe_route(router, n_exp, h, k, x)
    m = n * h
    acc = np.zeros(h, np.float32)
    want64 = np.zeros(h)
    for e, w in zip(sel, wt):
        eo = O.expert_forward(g[e * m:(e + 1) * m], u[e * m:(e + 1) * m], d[e * m:(e + 1) * m], h, n, x)
        acc = acc + np.float32(w) * eo  # numpy rounds the product and the sum separately, as moe.rs:254-256 does
        want64 += float(w) * eo.astype(np.float64)
    assert np.array_equal(out, acc)
    assert np.max(np.abs(out - want64)) <= 1e-6 * np.max(np.abs(want64))
    # an unweighted sum, or the first expert alone, would not pass
    assert np.max(np.abs(out - want64 / wt[0])) > 1e-3 * np.max(np.abs(want64))


def test_moe_forward_q_equals_dense_on_exactly_representable_q8_0_experts():
    # Q8_0 blocks with scale 1 and integer weights; integer inputs with one 127 per block, so the
    # activation quantizer is exact too (scale 1).  The intermediate vector is not integer, so its
    # Q8_0 re-quantization is applied to the dense path by hand before the down projection.
    rng = np.random.default_rng(9)
    h, n, n_exp, k = 64, 32, 4, 2
    t = O.Q8_0

    def q8_rows(rows, cols):
        q = rng.integers(-3, 4, size=(rows, cols)).astype(np.int8)
        blocks = [O.make_q8_0_block(1.0, [int(v) for v in q[r, c:c + 32]])
                  for r in range(rows) for c in range(0, cols, 32)]
        return q.astype(np.float32), np.frombuffer(b"".join(blocks), dtype=np.uint8)

    gf, gq = zip(*[q8_rows(n, h) for _ in range(n_exp)])
    uf, uq = zip(*[q8_rows(n, h) for _ in range(n_exp)])
    df, dq = zip(*[q8_rows(h, n) for _ in range(n_exp)])
    router = rng.standard_normal(n_exp * h).astype(np.float32) * 0.05
    x = rng.integers(-2, 3, size=h).astype(np.float32)
    x[::32] = 127.0
    x *= 0.0078125  # 2^-7: still exact under a power-of-two block scale
    out_q, sel, wt = O.moe_forward_q(t, router, np.concatenate(gq), np.concatenate(uq), np.concatenate(dq), n_exp, h, n,
                                     k, x)
    sel2, wt2 = O.moe_route(router, n_exp, h, k, x)
    assert sel.tolist() == sel2.tolist() and np.array_equal(wt, wt2)
    want = np.zeros(h, np.float32)
    for e, w in zip(sel, wt):
        hv = O.swiglu(gf[e] @ x, uf[e] @ x)  # small integers times 2^-7: exact in fp32 in any order
        hq = O.quantize_q8_0(hv)
        hdq = O.dequant_rows(O.Q8_0, hq, 1, n).ravel()
        eo = (df[e].astype(np.float64) @ hdq.astype(np.float64))
        want = want + np.float32(w) * eo.astype(np.float32)
    assert np.max(np.abs(out_q - want)) <= 1e-5 * np.max(np.abs(want))
