"""Parity of the mixture-of-experts layer on the device (router, grouping, gather + quantize,
grouped expert matmuls, SwiGLU + quantize, weighted combine) against the CPU oracle's restatement
of MoeFfn::forward (crates/oxillama-arch/src/common/moe.rs:184-258), through the C ABI.

Bars: the routing tables (experts, offsets, rows) exact; weights within 1e-5 (the router's fp32 dot
products are summed lane-strided, the reference's in index order); grouped Q8_0
activation bytes bit-exact; the combine bit-exact given the experts' outputs; the composed layer
bit-identical to the same steps through the plain entry points; fp32 against the oracle within
1e-5 * |y_ref|_inf per stage; on identical gate / up values the Q8_0 bytes of h equal the oracle's.
End to end a token is held to 2e-5 * |y_ref|_inf where its h bytes equal those of the oracle's own chain;
where the last-place difference between the device's and the oracle's gate / up (another summation
order) moved a byte of h across a rounding boundary, that is a whole quantization step and the bar is
2e-3 * |y_ref|_inf."""
import sys

import numpy as np
import pytest
import torch

import oracle as O
from oxillama_amd import linear as L
from oxillama_amd import moe, synth

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_close(y, y_ref, what, tol=1e-5):
    scale = float(np.abs(y_ref).max())
    err = float(np.abs(y.astype(np.float64) - y_ref.astype(np.float64)).max())
    assert err <= tol * scale + 1e-30, f"{what}: max err {err:.3e} > {tol} * {scale:.3e}"


def route_on_device(router, x, n_tok, n_exp, hidden, top_k):
    k = min(top_k, n_exp)
    d = dict(experts=torch.full((n_tok, k), -1, dtype=torch.int32, device=DEV),
             weights=torch.zeros((n_tok, k), dtype=torch.float32, device=DEV),
             offsets=torch.full((n_exp + 1,), -1, dtype=torch.int32, device=DEV),
             pair_token=torch.full((n_tok * k,), -1, dtype=torch.int32, device=DEV),
             token_rows=torch.full((n_tok, k), -1, dtype=torch.int32, device=DEV))
    moe.route_dev(dev(router), dev(x), n_tok, n_exp, hidden, top_k, d["experts"], d["weights"], d["offsets"],
                  d["pair_token"], d["token_rows"])
    return d, k


@pytest.mark.parametrize("cfg", [(8, 2, 512, 4096), (8, 2, 1, 256), (64, 6, 33, 512), (5, 9, 17, 96), (3, 1, 300, 64),
                                 (256, 8, 4, 128)], ids=str)
def test_route_and_grouping(hip, ref, cfg):
    n_exp, top_k, n_tok, hidden = cfg
    say("moe route", cfg)
    router = synth.normal_f32(31 + n_exp, n_exp * hidden, 0.05)
    x = synth.normal_f32(32 + n_tok, n_tok * hidden)
    d, k = route_on_device(router, x, n_tok, n_exp, hidden, top_k)
    experts, weights = host(d["experts"]), host(d["weights"])
    for t in range(n_tok if n_tok <= 64 else 64):
        sel, wt = ref.moe_route(router, n_exp, hidden, top_k, x[t * hidden:(t + 1) * hidden])
        assert experts[t].tolist() == sel.tolist(), f"token {t}"
        assert np.max(np.abs(weights[t] - wt)) <= 1e-5, f"token {t}"
    assert np.all(np.abs(weights.sum(axis=1) - 1) < 1e-5) and np.all(np.diff(weights, axis=1) <= 0)
    # the tables are those of the host-side grouping of the same decisions, exactly
    offsets, tok, slot = moe.group_by_expert(experts, n_exp)
    assert np.array_equal(host(d["offsets"]), offsets)
    assert np.array_equal(host(d["pair_token"]), tok)
    assert np.array_equal(host(d["token_rows"]), moe.token_rows(offsets, tok, slot, n_tok, k))


def test_route_reference_cases(hip, ref):
    # moe.rs:324-401: one-hot router, uniform router (ties -> lowest indices, weights 1/k), top_k clamp
    h, n_exp = 4, 4
    router = np.zeros(n_exp * h, np.float32)
    router[0] = 1.0
    d, _ = route_on_device(router, np.array([1, 0, 0, 0], np.float32), 1, n_exp, h, 1)
    assert host(d["experts"]).tolist() == [[0]] and host(d["weights"]).tolist() == [[1.0]]
    d, _ = route_on_device(np.ones(16, np.float32), np.ones(4, np.float32), 1, 4, 4, 2)
    assert host(d["experts"]).tolist() == [[0, 1]] and host(d["weights"]).tolist() == [[0.5, 0.5]]
    d, k = route_on_device(np.ones(16, np.float32), np.ones(4, np.float32), 1, 4, 4, 10)
    assert k == 4 and host(d["experts"]).tolist() == [[0, 1, 2, 3]] and host(d["weights"]).tolist() == [[0.25] * 4]
    assert host(d["offsets"]).tolist() == [0, 1, 2, 3, 4]
    z = torch.zeros(64, dtype=torch.float32, device=DEV)
    zi = torch.zeros(64, dtype=torch.int32, device=DEV)
    with pytest.raises(hip.KernelError):  # moe.rs:403-424
        moe.route_dev(z, z, 1, 2, 4, 0, zi, z, zi, zi, zi)


def test_gather_quantize_and_combine(hip, ref):
    rng = np.random.default_rng(3)
    n_tok, k, hidden, n_exp = 37, 3, 320, 6
    x = synth.normal_f32(77, n_tok * hidden)
    experts = np.stack([rng.permutation(n_exp)[:k] for _ in range(n_tok)]).astype(np.int32)
    weights = rng.random((n_tok, k)).astype(np.float32)
    offsets, tok, slot = moe.group_by_expert(experts, n_exp)
    rows = moe.token_rows(offsets, tok, slot, n_tok, k)
    d_q8 = torch.empty(n_tok * k * hidden // 32 * 34, dtype=torch.uint8, device=DEV)
    moe.gather_quantize_dev(dev(x), dev(tok), n_tok * k, hidden, d_q8)
    want = np.concatenate([ref.quantize_q8_0(x[t * hidden:(t + 1) * hidden]) for t in tok])
    assert np.array_equal(host(d_q8), want)
    y = synth.normal_f32(78, n_tok * k * hidden).reshape(n_tok * k, hidden)
    d_out = torch.empty(n_tok * hidden, dtype=torch.float32, device=DEV)
    moe.combine_dev(dev(y), dev(rows), dev(weights), n_tok, k, hidden, d_out)
    want = np.zeros((n_tok, hidden), np.float32)
    for t in range(n_tok):
        for j in range(k):
            ref.load().oxq_ref_moe_accumulate(O._p(want[t]), O._p(np.ascontiguousarray(y[rows[t, j]])),
                                              float(weights[t, j]), hidden)
    assert np.array_equal(host(d_out).view(np.uint32), want.ravel().view(np.uint32))


def expert_weights(t, seed, n_exp, n_rows, n_cols):
    if t in (O.Q4_0, O.Q8_0, O.Q4_K, O.Q6_K, O.IQ4_XS):
        return np.concatenate([synth.weights(t, seed + e, n_rows, n_cols, 0.05) for e in range(n_exp)])
    return np.concatenate([O.random_blocks(t, seed + e, n_rows, n_cols) for e in range(n_exp)])


@pytest.mark.parametrize("types", [(O.Q4_K, O.Q4_K, O.Q6_K), (O.Q8_0, O.Q8_0, O.Q8_0), (O.Q4_0, O.IQ4_XS, O.Q4_0),
                                   (O.Q5_K, O.Q5_K, O.Q5_K), (O.Q3_K, O.Q3_K, O.Q2_K), (O.Q5_0, O.Q5_1, O.Q4_1)],
                         ids=["q4k_q4k_q6k", "q8_0", "q4_0_iq4xs", "q5k", "q3k_q3k_q2k", "q5_0_q5_1_q4_1"])
@pytest.mark.parametrize("shape", [(4, 2, 1, 256, 512), (8, 2, 3, 512, 256), (8, 2, 40, 512, 256), (6, 3, 130, 256, 768),
                                   (128, 8, 20, 512, 768), (128, 8, 4, 512, 768)], ids=str)  # (the last two: more experts than a wave has
                                                                                            # lanes, most with one row or none; 32 rows: one GEMV per row)
def test_moe_ffn_layer(hip, ref, types, shape):
    _moe_ffn_layer_case(hip, ref, types, shape)


@pytest.mark.parametrize("types", [(O.Q4_K, O.Q8_0, O.Q4_K), (O.IQ4_XS, O.Q4_0, O.IQ4_XS), (O.Q8_0, O.Q4_K, O.Q6_K)],
                         ids=["q4k_q8_0_q4k", "iq4xs_q4_0_iq4xs", "q8_0_q4k_q6k"])
@pytest.mark.parametrize("shape", [(8, 2, 24, 512, 256), (8, 2, 40, 1024, 512)], ids=str)
def test_moe_ffn_layer_gate_and_up_on_different_kernels(hip, ref, types, shape):
    """Gate in a format that the few-token kernel serves (it reads the caller's Q8_0 rows and re-lays nothing out) and
    up in a format of the same activation byte order that only the tile kernel serves, and the other way round: up
    must not take the workspace for prepared when gate's launch did not prepare it."""
    _moe_ffn_layer_case(hip, ref, types, shape)


@pytest.mark.parametrize("types", [(O.Q8_0, O.Q8_0, O.Q8_0), (O.Q4_0, O.Q5_0, O.Q8_1), (O.Q5_1, O.Q4_1, O.IQ4_NL)],
                         ids=["q8_0", "q4_0_q5_0_q8_1", "q5_1_q4_1_iq4nl"])
@pytest.mark.parametrize("shape", [(4, 2, 3, 288, 352), (4, 2, 40, 288, 352), (6, 3, 130, 352, 1408)], ids=str)
def test_moe_ffn_layer_rows_of_whole_32_blocks(hip, ref, types, shape):
    """Hidden and intermediate sizes that are multiples of 32 but not of 256 (expert matrices in the 32-weight
    formats, as GGUF files store tensors whose rows the 256-weight formats cannot take): the same layer, the same
    bars."""
    _moe_ffn_layer_case(hip, ref, types, shape)


def _moe_ffn_layer_case(hip, ref, types, shape):
    n_exp, top_k, n_tok, hidden, inter = shape
    tg, tu, td = types
    say("moe ffn", [O.NAMES[t] for t in types], shape)
    wg = expert_weights(tg, 100, n_exp, inter, hidden)
    wu = expert_weights(tu, 200, n_exp, inter, hidden)
    wd = expert_weights(td, 300, n_exp, hidden, inter)
    sg, su, sd = wg.size // n_exp, wu.size // n_exp, wd.size // n_exp
    router = synth.normal_f32(5, n_exp * hidden, 0.05)
    x = synth.normal_f32(6, n_tok * hidden)
    d_x = dev(x)
    d, k = route_on_device(router, x, n_tok, n_exp, hidden, top_k)
    pairs = n_tok * k
    need = moe.moe_ffn_workspace_bytes(types, pairs, hidden, inter)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    d_out = torch.full((n_tok * hidden,), 7.0, dtype=torch.float32, device=DEV)  # overwritten, moe.rs:240-242
    d_wg, d_wu, d_wd = dev(wg), dev(wu), dev(wd)
    moe.moe_ffn_dev((tg, d_wg, sg), (tu, d_wu, su), (td, d_wd, sd), n_exp, d_x, n_tok, k, d["offsets"],
                    d["pair_token"], d["token_rows"], d["weights"], 0, d_out, hidden, inter, ws)
    got = host(d_out).reshape(n_tok, hidden)

    # the same steps through the plain entry points: bit-identical
    d_q8 = torch.empty(pairs * hidden // 32 * 34, dtype=torch.uint8, device=DEV)
    moe.gather_quantize_dev(d_x, d["pair_token"], pairs, hidden, d_q8)
    g = torch.empty(pairs * inter, dtype=torch.float32, device=DEV)
    u = torch.empty(pairs * inter, dtype=torch.float32, device=DEV)
    y = torch.empty(pairs * hidden, dtype=torch.float32, device=DEV)
    hq = torch.empty(pairs * inter // 32 * 34, dtype=torch.uint8, device=DEV)

    def grouped(t, d_w, stride, d_acts, d_y, n, kk):
        kern = hip.HipKernel(t)
        w2 = torch.empty(kern.moe_gemm_workspace_bytes(pairs, n, kk), dtype=torch.uint8, device=DEV)
        kern.moe_gemm_q8_dev(d_w, stride, n_exp, d_acts, d["offsets"], pairs, 0, d_y, n, kk, w2)

    grouped(tg, d_wg, sg, d_q8, g, inter, hidden)
    grouped(tu, d_wu, su, d_q8, u, inter, hidden)
    L.swiglu_quantize_dev(g, u, None, hq)
    grouped(td, d_wd, sd, hq, y, hidden, inter)
    step = torch.empty(n_tok * hidden, dtype=torch.float32, device=DEV)
    moe.combine_dev(y, d["token_rows"], d["weights"], n_tok, k, hidden, step)
    assert np.array_equal(got.ravel().view(np.uint32), host(step).view(np.uint32))

    # stage by stage against the oracle, on a sample of tokens, each stage fed the device's own input
    experts, weights, rows = host(d["experts"]), host(d["weights"]), host(d["token_rows"])
    q8, gh, uh, hqh, yh = host(d_q8), host(g), host(u), host(hq), host(y).reshape(pairs, hidden)
    a_row, h_row = hidden // 32 * 34, inter // 32 * 34
    sample = sorted(set([0, n_tok - 1, n_tok // 2] + list(range(0, n_tok, 4))))
    flipped_h = bytes_h = flipped_chain = scales_chain = 0
    for t in sample:
        xt = x[t * hidden:(t + 1) * hidden]
        sel, wt = ref.moe_route(router, n_exp, hidden, top_k, xt)
        assert experts[t].tolist() == sel.tolist() and np.max(np.abs(weights[t] - wt)) <= 1e-5
        acc = np.zeros(hidden, np.float32)
        chain_before = flipped_chain + scales_chain
        for j, e in enumerate(sel):
            r = rows[t, j]
            acts = q8[r * a_row:(r + 1) * a_row]
            assert np.array_equal(acts, ref.quantize_q8_0(xt))
            g_ref = ref.matvec_q8_fused(tg, wg[e * sg:(e + 1) * sg], acts, inter, hidden)
            u_ref = ref.matvec_q8_fused(tu, wu[e * su:(e + 1) * su], acts, inter, hidden)
            assert_close(gh[r * inter:(r + 1) * inter], g_ref, f"gate t{t} e{e}")
            assert_close(uh[r * inter:(r + 1) * inter], u_ref, f"up t{t} e{e}")
            hq_ref = ref.quantize_q8_0(ref.swiglu(gh[r * inter:(r + 1) * inter], uh[r * inter:(r + 1) * inter]))
            mine = hqh[r * h_row:(r + 1) * h_row]
            # the device evaluates exp the way the C library does (oxq_device.hpp expf_libm), so on identical gate / up
            # values the bytes of h are the oracle's
            mb, rb_ = mine.reshape(-1, 34), hq_ref.reshape(-1, 34)
            assert np.array_equal(mb[:, :2], rb_[:, :2]), f"h scales t{t} e{e}"
            step = mb[:, 2:].view(np.int8).astype(np.int32) - rb_[:, 2:].view(np.int8).astype(np.int32)
            assert np.abs(step).max() <= 1, f"h bytes t{t} e{e}: a byte moved by more than one step"
            flipped_h += int(np.count_nonzero(step))
            bytes_h += mine.size
            # against the oracle's own chain (its gate / up, within 1e-5 of the device's, then libm): the same kind
            # of difference, counted over everything that feeds the down projection
            chain = ref.quantize_q8_0(ref.swiglu(g_ref, u_ref)).reshape(-1, 34)
            chain_step = mb[:, 2:].view(np.int8).astype(np.int32) - chain[:, 2:].view(np.int8).astype(np.int32)
            d_mine = mb[:, :2].copy().view(np.uint16).astype(np.int32).ravel()
            d_chain = chain[:, :2].copy().view(np.uint16).astype(np.int32).ravel()
            assert np.abs(d_mine - d_chain).max() <= 1, "a block scale of h moved by more than one f16 step"
            same_scale = d_mine == d_chain
            assert np.abs(chain_step[same_scale]).max(initial=0) <= 1
            flipped_chain += int(np.count_nonzero(chain_step[same_scale]))
            scales_chain += int(np.count_nonzero(~same_scale))
            e_ref = ref.matvec_q8_fused(td, wd[e * sd:(e + 1) * sd], mine, hidden, inter)
            assert_close(yh[r], e_ref, f"down t{t} e{e}")
            ref.load().oxq_ref_moe_accumulate(O._p(acc), O._p(np.ascontiguousarray(yh[r])), float(weights[t, j]),
                                              hidden)
        assert np.array_equal(got[t].view(np.uint32), acc.view(np.uint32)), f"combine t{t}"
        # end to end against MoeFfn::forward with quantized experts
        want, sel2, _ = ref.moe_forward_q(tg, router, wg, wu, wd, n_exp, hidden, inter, top_k, xt) \
            if tg == tu == td else (None, None, None)
        if want is not None:
            # a token whose h bytes are the oracle chain's bytes: the layer's output within the fp32 bar (2e-5: the
            # routing weights carry up to 1e-5 of their own); a byte of h that the last-place difference between the
            # device's and the oracle's gate / up moved across a rounding boundary is a whole quantization step
            same_h = flipped_chain + scales_chain == chain_before
            assert_close(got[t], want, f"end to end t{t}", tol=2e-5 if same_h else 2e-3)
    say(f"h bytes one step off the oracle's: {flipped_h} of {bytes_h} (same gate/up); oracle's gate/up: {flipped_chain} bytes, "
        f"{scales_chain} of {bytes_h // 34} block scales one f16 step off")
    assert flipped_h == 0, f"{flipped_h} of {bytes_h} Q8_0 bytes of h differ on identical gate / up values"
    assert flipped_chain <= max(2, bytes_h // 1000), f"{flipped_chain} of {bytes_h} Q8_0 bytes of h differ from the oracle's chain"
    assert scales_chain <= max(2, bytes_h // 34 // 100), f"{scales_chain} of {bytes_h // 34} block scales of h differ"


def test_moe_ffn_with_host_tables_and_errors(hip, ref):
    # tables made on the host (route_top_k + group_by_expert), max_rows known; an expert without rows
    n_exp, k, n_tok, hidden, inter = 5, 2, 9, 256, 256
    t = O.Q4_K
    wg, wu, wd = (expert_weights(t, s, n_exp, inter, hidden) for s in (1, 2, 3))
    stride = wg.size // n_exp
    logits = synth.normal_f32(9, n_tok * n_exp).reshape(n_tok, n_exp)
    logits[:, 3] = -50.0  # expert 3 is never chosen
    experts, weights = moe.route_top_k(logits, k)
    offsets, tok, slot = moe.group_by_expert(experts, n_exp)
    assert offsets[3] == offsets[4]
    rows = moe.token_rows(offsets, tok, slot, n_tok, k)
    x = synth.normal_f32(10, n_tok * hidden)
    ws = torch.empty(moe.moe_ffn_workspace_bytes((t, t, t), n_tok * k, hidden, inter), dtype=torch.uint8, device=DEV)
    d_out = torch.empty(n_tok * hidden, dtype=torch.float32, device=DEV)
    args = ((t, dev(wg), stride), (t, dev(wu), stride), (t, dev(wd), stride), n_exp, dev(x), n_tok, k, dev(offsets),
            dev(tok), dev(rows), dev(weights), int(np.diff(offsets).max()), d_out, hidden, inter)
    moe.moe_ffn_dev(*args, ws)
    got = host(d_out).reshape(n_tok, hidden)
    for tkn in range(n_tok):
        xq = ref.quantize_q8_0(x[tkn * hidden:(tkn + 1) * hidden])
        acc = np.zeros(hidden, np.float32)
        for j in range(k):
            e = experts[tkn, j]
            eo = ref.expert_forward_q(t, wg[e * stride:(e + 1) * stride], wu[e * stride:(e + 1) * stride],
                                      wd[e * stride:(e + 1) * stride], hidden, inter, xq)
            acc = acc + weights[tkn, j] * eo
        assert_close(got[tkn], acc, f"token {tkn}", tol=2e-3)
    with pytest.raises(hip.BufferTooSmall) as e:
        moe.moe_ffn_dev(*args, ws[:256])
    assert e.value.needed == ws.numel()
    with pytest.raises(hip.UnsupportedShape):  # the grouped kernel walks 256 columns at a time: rows of at least that
        moe.moe_ffn_dev((O.Q8_0, args[0][1], stride), (O.Q8_0, args[1][1], stride), (O.Q8_0, args[2][1], stride),
                        *args[3:-2], 224, inter, ws)
    assert moe.moe_ffn_workspace_bytes((O.Q8_0, O.Q8_0, O.Q8_0), n_tok * k, 224, inter) == 0
    assert moe.moe_ffn_workspace_bytes((O.Q8_0, O.Q8_0, O.Q8_0), n_tok * k, 288, inter) > 0
    with pytest.raises(hip.KernelError):  # top_k = 0, moe.rs:168-172
        moe.moe_ffn_dev(*args[:6], 0, *args[7:], ws)


def test_moe_forward_host_slices(hip, ref):
    """MoeFfn::forward through the host-slice entry point (the drop-in route), one token and a batch."""
    n_exp, k, hidden, inter = 4, 2, 256, 512
    t = O.Q4_K
    wg, wu, wd = (expert_weights(t, s, n_exp, inter, hidden) for s in (11, 12, 13))
    wd = expert_weights(O.Q6_K, 13, n_exp, hidden, inter)
    router = synth.normal_f32(14, n_exp * hidden, 0.05)
    layer = moe.MoeFfn(router, (t, wg), (t, wu), (O.Q6_K, wd), k, n_exp, hidden, inter)
    x = synth.normal_f32(15, 5 * hidden)
    sg, sd = wg.size // n_exp, wd.size // n_exp

    def want(xt):
        sel, wt = ref.moe_route(router, n_exp, hidden, k, xt)
        xq = ref.quantize_q8_0(xt)
        acc = np.zeros(hidden, np.float32)
        for e, w in zip(sel, wt):
            g = ref.matvec_q8_fused(t, wg[e * sg:(e + 1) * sg], xq, inter, hidden)
            u = ref.matvec_q8_fused(t, wu[e * sg:(e + 1) * sg], xq, inter, hidden)
            hq = ref.quantize_q8_0(ref.swiglu(g, u))
            eo = ref.matvec_q8_fused(O.Q6_K, wd[e * sd:(e + 1) * sd], hq, hidden, inter)
            acc = acc + np.float32(w) * eo
        return acc

    from oxillama_amd import capi
    lib = capi.load()
    for cache in (0, 1):
        lib.oxq_weight_cache_enable(cache)
        one = layer.forward(x[:hidden])
        assert_close(one, want(x[:hidden]), "one token", tol=2e-3)
        many = layer.forward_batch(x, 5).reshape(5, hidden)
        # one token is two rows (one GEMV launch per projection), five tokens ten (the matmul kernels): another
        # summation order, so the same row agrees to the layer's bar rather than bit for bit
        assert_close(many[0], one, "a token alone and in a batch", tol=2e-3)
        for i in range(5):
            assert_close(many[i], want(x[i * hidden:(i + 1) * hidden]), f"token {i}", tol=2e-3)
    # a byte cap that the three tensors do not fit under together: staging `down` must not evict (and free) the
    # `gate` or `up` that the same call staged a moment earlier -- such a call goes round the cache; and with room
    # for exactly the three, an older entry goes, not one of the call's own
    plain = layer.forward_batch(x, 5)
    other = synth.weights(t, 77, 64, hidden)
    xa = ref.quantize_q8_0(x[:hidden])
    for limit in (wg.nbytes + wu.nbytes + wd.nbytes - 1, 2 * wg.nbytes, wg.nbytes + wu.nbytes + wd.nbytes):
        lib.oxq_weight_cache_clear()
        lib.oxq_weight_cache_enable(1)
        lib.oxq_weight_cache_set_limit(limit)
        hip.HipKernel(t).matvec_q8_fused(other, xa, np.zeros(64, dtype=np.float32), 64, hidden)  # an older entry
        for _ in range(2):
            assert np.array_equal(layer.forward_batch(x, 5).view(np.uint32), plain.view(np.uint32)), limit
    lib.oxq_weight_cache_set_limit(16 << 30)
    lib.oxq_weight_cache_enable(0)
    lib.oxq_weight_cache_clear()
    # the reference's error cases (moe.rs:403-450, 307-322) after a working call
    layer.top_k = 0
    with pytest.raises(hip.KernelError):
        layer.forward(x[:hidden])
    layer.top_k = 10  # clamps to the expert count (moe.rs:381-401)
    assert_close(layer.forward(x[:hidden]), want_all(ref, layer, router, wg, wu, wd, x[:hidden]), "top_k clamp", tol=2e-3)
    bad = moe.MoeFfn(router[:-1], (t, wg), (t, wu), (O.Q6_K, wd), k, n_exp, hidden, inter)
    with pytest.raises(hip.DimensionMismatch) as e:
        bad.forward(x[:hidden])
    assert (e.value.expected, e.value.got) == (n_exp * hidden, n_exp * hidden - 1)
    bad = moe.MoeFfn(router, (t, wg[:-1]), (t, wu), (O.Q6_K, wd), k, n_exp, hidden, inter)
    with pytest.raises(hip.DimensionMismatch) as e:
        bad.forward(x[:hidden])
    assert (e.value.expected, e.value.got) == (wg.size, wg.size - 1)
    bad = moe.MoeFfn(router[:n_exp * 100], (t, wg), (t, wu), (O.Q6_K, wd), k, n_exp, 100, inter)
    with pytest.raises(hip.DimensionMismatch):  # sizes no longer fit hidden = 100
        bad.forward(x[:100])


def want_all(ref, layer, router, wg, wu, wd, xt):
    """All experts selected (top_k >= num_experts): weights are the plain softmax."""
    n_exp, hidden, inter = layer.num_experts, layer.hidden_size, layer.intermediate_size
    sel, wt = ref.moe_route(router, n_exp, hidden, layer.top_k, xt)
    assert len(sel) == n_exp
    xq = ref.quantize_q8_0(xt)
    sg, sd = wg.size // n_exp, wd.size // n_exp
    acc = np.zeros(hidden, np.float32)
    for e, w in zip(sel, wt):
        eo_in = ref.quantize_q8_0(ref.swiglu(ref.matvec_q8_fused(layer.gate[0], wg[e * sg:(e + 1) * sg], xq, inter, hidden),
                                             ref.matvec_q8_fused(layer.up[0], wu[e * sg:(e + 1) * sg], xq, inter, hidden)))
        acc = acc + np.float32(w) * ref.matvec_q8_fused(layer.down[0], wd[e * sd:(e + 1) * sd], eo_in, hidden, inter)
    return acc


def test_moe_layer_full_size_c5(hip, ref):
    """The whole layer at the C5 size (IQ4_XS, 8 experts of 14336 x 4096 / 4096 x 14336, 64 tokens, top-2): routing
    exact for every token; for every token the layer's output against the oracle's MoeFfn::forward on quantized
    experts (end-to-end bar), and the size-independent property that the weights of a token sum to one."""
    n_exp, top_k, n_tok, hidden, inter = 8, 2, 64, 4096, 14336
    t = O.IQ4_XS
    say("moe layer C5 full size: generating 749 MB of expert weights")
    wg = np.concatenate([synth.weights(t, 7000 + e, inter, hidden) for e in range(n_exp)])
    wu = np.concatenate([synth.weights(t, 7100 + e, inter, hidden) for e in range(n_exp)])
    wd = np.concatenate([synth.weights(t, 7200 + e, hidden, inter) for e in range(n_exp)])
    stride = wg.size // n_exp
    router = synth.normal_f32(9, n_exp * hidden, 0.05)
    x = synth.normal_f32(7, n_tok * hidden)
    d, k = route_on_device(router, x, n_tok, n_exp, hidden, top_k)
    experts, weights = host(d["experts"]), host(d["weights"])
    for tk in range(n_tok):
        sel, wt = ref.moe_route(router, n_exp, hidden, top_k, x[tk * hidden:(tk + 1) * hidden])
        assert experts[tk].tolist() == sel.tolist() and np.max(np.abs(weights[tk] - wt)) <= 1e-5
    assert np.all(np.abs(weights.sum(axis=1) - 1) < 1e-5)
    ws = torch.empty(moe.moe_ffn_workspace_bytes((t, t, t), n_tok * k, hidden, inter), dtype=torch.uint8, device=DEV)
    d_out = torch.empty(n_tok * hidden, dtype=torch.float32, device=DEV)
    d_wg, d_wu, d_wd = dev(wg), dev(wu), dev(wd)
    say("moe layer C5 full size: device run")
    moe.moe_ffn_dev((t, d_wg, stride), (t, d_wu, stride), (t, d_wd, stride), n_exp, dev(x), n_tok, k, d["offsets"],
                    d["pair_token"], d["token_rows"], d["weights"], 0, d_out, hidden, inter, ws)
    got = host(d_out).reshape(n_tok, hidden)
    assert np.all(np.isfinite(got))
    for tk in range(n_tok):  # every token (threaded oracle matvecs: a few seconds)
        if tk % 16 == 0:
            say("moe layer C5 full size: oracle token", tk)
        xt = x[tk * hidden:(tk + 1) * hidden]
        xq = ref.quantize_q8_0(xt)
        acc = np.zeros(hidden, np.float32)
        for j, e in enumerate(experts[tk]):
            g = ref.matvec_q8_fused_mt(t, wg[e * stride:(e + 1) * stride], xq, inter, hidden, 16)
            u = ref.matvec_q8_fused_mt(t, wu[e * stride:(e + 1) * stride], xq, inter, hidden, 16)
            hq = ref.quantize_q8_0(ref.swiglu(g, u))
            eo = ref.matvec_q8_fused_mt(t, wd[e * stride:(e + 1) * stride], hq, hidden, inter, 16)
            acc = acc + weights[tk, j] * eo
        assert_close(got[tk], acc, f"token {tk}", tol=2e-3)
    # the one-call entry point at the same size: the same bits for the batch; and the reference's own call, one
    # token (router launch that also groups and writes the activation rows, one GEMV launch per projection over the
    # two chosen experts), against the same oracle result
    say("moe layer C5 full size: oxq_moe_forward_dev, 64 tokens and one token")
    d_router, d_x = dev(router), dev(x)
    ws2 = torch.empty(moe.moe_forward_workspace_bytes((t, t, t), n_tok, top_k, n_exp, hidden, inter), dtype=torch.uint8,
                      device=DEV)
    d_out2 = torch.full((n_tok * hidden,), 7.0, dtype=torch.float32, device=DEV)
    moe.moe_forward_dev((t, d_wg, stride), (t, d_wu, stride), (t, d_wd, stride), n_exp, d_router, d_x, n_tok, top_k, d_out2,
                        hidden, inter, ws2)
    assert np.array_equal(host(d_out2).view(np.uint32), got.ravel().view(np.uint32))
    one = torch.full((hidden,), 7.0, dtype=torch.float32, device=DEV)
    moe.moe_forward_dev((t, d_wg, stride), (t, d_wu, stride), (t, d_wd, stride), n_exp, d_router, d_x[63 * hidden:], 1, top_k,
                        one, hidden, inter, ws2)
    assert_close(host(one), acc, "token 63 alone", tol=2e-3)
    assert_close(host(one), got[63], "token 63 alone against its row of the batch", tol=2e-3)


@pytest.mark.parametrize("cfg", [(8, 2, 1, 512, 256, O.IQ4_XS), (8, 1, 1, 256, 512, O.Q4_K), (8, 8, 1, 256, 256, O.Q6_K),
                                 (16, 9, 1, 256, 256, O.Q4_K), (3, 5, 1, 256, 256, O.Q8_0), (8, 2, 5, 256, 512, O.IQ4_XS),
                                 (8, 2, 40, 512, 256, O.Q4_K), (70, 2, 1, 256, 256, O.Q4_K)], ids=str)
def test_moe_forward_on_device_pointers(hip, ref, cfg):
    """oxq_moe_forward_dev (routing and experts in one call; for one token the router's launch also groups the
    choices and writes the activation rows) against oxq_moe_route_dev + oxq_moe_ffn_dev: the same bits, on a
    workspace that held other contents before; one token against the oracle's layer as well."""
    n_exp, top_k, n_tok, hidden, inter, t = cfg
    say("moe forward dev", cfg)
    wg = expert_weights(t, 100, n_exp, inter, hidden)
    wu = expert_weights(t, 200, n_exp, inter, hidden)
    wd = expert_weights(t, 300, n_exp, hidden, inter)
    stride_gu, stride_d = wg.size // n_exp, wd.size // n_exp
    router = synth.normal_f32(15, n_exp * hidden, 0.05)
    x = synth.normal_f32(16, n_tok * hidden)
    d_x, d_router, d_wg, d_wu, d_wd = dev(x), dev(router), dev(wg), dev(wu), dev(wd)
    d, k = route_on_device(router, x, n_tok, n_exp, hidden, top_k)
    ws = torch.empty(moe.moe_ffn_workspace_bytes((t, t, t), n_tok * k, hidden, inter), dtype=torch.uint8, device=DEV)
    want = torch.empty(n_tok * hidden, dtype=torch.float32, device=DEV)
    moe.moe_ffn_dev((t, d_wg, stride_gu), (t, d_wu, stride_gu), (t, d_wd, stride_d), n_exp, d_x, n_tok, k, d["offsets"],
                    d["pair_token"], d["token_rows"], d["weights"], 0, want, hidden, inter, ws)
    need = moe.moe_forward_workspace_bytes((t, t, t), n_tok, top_k, n_exp, hidden, inter)
    assert need > ws.numel()
    ws2 = torch.full((need,), 0xA5, dtype=torch.uint8, device=DEV)
    got = torch.full((n_tok * hidden,), 7.0, dtype=torch.float32, device=DEV)
    for _ in range(2):  # the second call finds the first one's tables and rows in the workspace
        moe.moe_forward_dev((t, d_wg, stride_gu), (t, d_wu, stride_gu), (t, d_wd, stride_d), n_exp, d_router, d_x, n_tok,
                            top_k, got, hidden, inter, ws2)
        assert np.array_equal(host(got).view(np.uint32), host(want).view(np.uint32))
    # the tables at the head of the workspace: experts | weights | offsets | pair_token | token_rows, 256-byte slots
    al = lambda n: (n + 255) & ~255
    raw = host(ws2)
    o = 0
    for name, n in (("experts", n_tok * k), ("weights", n_tok * k), ("offsets", n_exp + 1), ("pair_token", n_tok * k),
                    ("token_rows", n_tok * k)):
        assert np.array_equal(raw[o:o + 4 * n], host(d[name]).ravel().view(np.uint8)), name
        o += al(4 * n)
    with pytest.raises(Exception):
        moe.moe_forward_dev((t, d_wg, stride_gu), (t, d_wu, stride_gu), (t, d_wd, stride_d), n_exp, d_router, d_x, n_tok,
                            top_k, got, hidden, inter, ws2[:need - 256])
    if n_tok == 1:
        y_ref, sel, _ = ref.moe_forward_q(t, router, wg, wu, wd, n_exp, hidden, inter, top_k, x)
        assert np.array_equal(host(d["experts"]).ravel(), sel.astype(np.int32))
        assert_close(host(got), y_ref, "one token against the oracle", tol=2e-3)


def test_moe_forward_on_device_pointers_degenerate(hip):
    """No experts or no intermediate columns: the zeroed output (moe.rs:240-242); top_k == 0: InvalidConfig."""
    from oxillama_amd.quant import KernelError
    hidden = 256
    d_x = dev(synth.normal_f32(3, 2 * hidden))
    out = torch.full((2 * hidden,), 7.0, dtype=torch.float32, device=DEV)
    empty = torch.empty(256, dtype=torch.uint8, device=DEV)
    moe.moe_forward_dev((O.Q4_K, empty, 0), (O.Q4_K, empty, 0), (O.Q4_K, empty, 0), 0, empty, d_x, 2, 2, out, hidden, 256,
                        empty)
    assert not host(out).any()
    with pytest.raises(KernelError):
        moe.moe_forward_dev((O.Q4_K, empty, 0), (O.Q4_K, empty, 0), (O.Q4_K, empty, 0), 4, empty, d_x, 2, 0, out, hidden,
                            256, empty)
