"""The C-ABI library loads and exports every symbol include/oxq.h declares, and the
checks that precede any GPU work behave as the reference's do.  CPU only: no entry
point that would touch a device is called with valid arguments here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from oxillama_amd import capi, quant

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header="oxq.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(oxq_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_the_same_symbols():
    assert declared_symbols() == sorted(capi.SIGNATURES)
    assert declared_symbols("oxq_gguf.h") == sorted(capi.GGUF_SIGNATURES)
    assert declared_symbols("oxq_tuning.h") == sorted(capi.TUNING_SIGNATURES)


def test_boundary_header_holds_no_tuning_knob():
    # the reference-side shim binds oxq.h only: nothing there may be a launch-shape setter
    assert not [s for s in declared_symbols() if s.startswith("oxq_set_") or s == "oxq_last_launch"]


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(capi.LIB_PATH)
    for name in declared_symbols() + declared_symbols("oxq_gguf.h") + declared_symbols("oxq_tuning.h"):
        assert hasattr(lib, name), name


def test_format_metadata_matches_reference_tables():
    # crates/oxillama-gguf/src/types.rs:199-262
    lib = capi.load()
    table = {2: (32, 18, b"Q4_0"), 8: (32, 34, b"Q8_0"), 12: (256, 144, b"Q4_K"), 14: (256, 210, b"Q6_K"),
             23: (256, 136, b"IQ4_XS"), 3: (32, 20, b"Q4_1"), 6: (32, 22, b"Q5_0"), 7: (32, 24, b"Q5_1"),
             9: (32, 36, b"Q8_1"), 10: (256, 84, b"Q2_K"), 11: (256, 110, b"Q3_K"), 13: (256, 176, b"Q5_K"),
             20: (32, 18, b"IQ4_NL")}
    for t, (bs, bb, name) in table.items():
        assert lib.oxq_block_size(t) == bs and lib.oxq_block_bytes(t) == bb and lib.oxq_type_name(t) == name
        assert lib.oxq_get_kernel(t) == capi.OK
    for t in (0, 1, 15, 16, 24, 39):  # formats this library has no kernel for
        assert lib.oxq_block_size(t) == 0 and lib.oxq_type_name(t) is None
        assert lib.oxq_get_kernel(t) == capi.ERR_UNSUPPORTED_TYPE
    with pytest.raises(quant.UnsupportedType):
        quant.KernelDispatcher().get_kernel(15)


def test_status_names_follow_quant_error_variants():
    lib = capi.load()
    names = [lib.oxq_status_name(i).decode() for i in range(10)]
    assert names == ["Ok", "UnsupportedType", "BlockSizeMismatch", "DimensionMismatch", "KernelError",
                     "BlockCountMismatch", "BufferTooSmall", "Internal", "UnsupportedShape", "NoDevice"]


def test_quantize_rejects_unaligned_length_before_touching_the_gpu():
    # Q/quantize.rs:59-64
    with pytest.raises(quant.DimensionMismatch) as e:
        quant.quantize_f32_to_q8_0(np.zeros(31, dtype=np.float32))
    assert (e.value.expected, e.value.got) == (32, 31)


@pytest.mark.parametrize("t", [2, 8, 12, 14, 23, 3, 6, 7, 9, 10, 11, 13, 20])
def test_fused_validation_order_before_touching_the_gpu(t):
    # Q/reference/q4_k.rs:226-250: out, then weights, then activations
    k = quant.HipKernel(t)
    bs, bb = k.block_size(), k.block_bytes()
    n_rows, n_cols = 3, 2 * bs
    w = np.zeros(n_rows * 2 * bb, dtype=np.uint8)
    acts_needed = 2 * (bs // 32) * 34
    a = np.zeros(acts_needed, dtype=np.uint8)
    with pytest.raises(quant.DimensionMismatch) as e:
        k.matvec_q8_fused(w[:-1], a[:-1], np.zeros(2, dtype=np.float32), n_rows, n_cols)
    assert (e.value.expected, e.value.got) == (3, 2)
    with pytest.raises(quant.BufferTooSmall) as e:
        k.matvec_q8_fused(w[:-1], a[:-1], np.zeros(3, dtype=np.float32), n_rows, n_cols)
    assert (e.value.needed, e.value.available) == (w.size, w.size - 1)
    with pytest.raises(quant.BufferTooSmall) as e:
        k.matvec_q8_fused(w, a[:-1], np.zeros(3, dtype=np.float32), n_rows, n_cols)
    assert (e.value.needed, e.value.available) == (acts_needed, acts_needed - 1)
    with pytest.raises(quant.UnsupportedShape):  # the debug dump of the group sums wants whole blocks
        k.block_sums(w, a, n_rows, n_cols - 1)


@pytest.mark.parametrize("t", [2, 8, 12, 14, 23, 3, 6, 7, 9, 10, 11, 13, 20])
def test_dequant_and_gemv_argument_errors(t):
    k = quant.HipKernel(t)
    bs, bb = k.block_size(), k.block_bytes()
    with pytest.raises(quant.BufferTooSmall) as e:  # e.g. Q/reference/q4_0.rs:348-355
        k.dequant_block(np.zeros(4, dtype=np.uint8), np.zeros(bs, dtype=np.float32))
    assert (e.value.needed, e.value.available) == (bb, 4)
    with pytest.raises(quant.BufferTooSmall) as e:  # Q/reference/q4_0.rs:358-366
        k.dequant_block(np.zeros(bb, dtype=np.uint8), np.zeros(1, dtype=np.float32))
    assert (e.value.needed, e.value.available) == (bs, 1)
    tensor = quant.QuantTensor(np.zeros(2 * bb, dtype=np.uint8), [2, bs], t)
    with pytest.raises(quant.DimensionMismatch) as e:  # Q/reference/q4_0.rs:311-321
        k.gemv(tensor, np.zeros(4, dtype=np.float32), np.zeros(2, dtype=np.float32))
    assert (e.value.expected, e.value.got) == (bs, 4)
    with pytest.raises(quant.DimensionMismatch) as e:  # Q/reference/q4_0.rs:324-337
        k.gemv(tensor, np.zeros(bs, dtype=np.float32), np.zeros(1, dtype=np.float32))
    assert (e.value.expected, e.value.got) == (2, 1)


def test_quant_tensor_bookkeeping():
    # Q/types.rs:31-50
    t = quant.QuantTensor(np.zeros(144 * 6, dtype=np.uint8), [3, 512], 12)
    assert t.n_elements() == 1536 and t.n_blocks() == 6 and t.expected_data_size() == 864
    assert quant.QuantTensor(b"", [], 12).n_elements() == 0


def test_moe_forward_argument_errors_before_touching_the_gpu():
    # MoeFfn::validate / Expert::validate, crates/oxillama-arch/src/common/moe.rs:151-173, 33-58: router size,
    # top_k, then the experts' gate / up / down sizes; all of it is checked before any device work
    from oxillama_amd import moe
    n_exp, hidden, inter, t = 2, 256, 256, 12
    one = inter * (hidden // 256) * 144
    w = np.zeros(n_exp * one, dtype=np.uint8)
    router = np.zeros(n_exp * hidden, dtype=np.float32)
    x = np.zeros(hidden, dtype=np.float32)

    def layer(**kw):
        a = dict(router=router, gate=(t, w), up=(t, w), down=(t, w), top_k=1, num_experts=n_exp, hidden_size=hidden,
                 intermediate_size=inter)
        a.update(kw)
        return moe.MoeFfn(**a)

    with pytest.raises(quant.DimensionMismatch) as e:  # moe.rs:426-450
        layer(router=router[:-3]).forward(x)
    assert (e.value.expected, e.value.got) == (n_exp * hidden, n_exp * hidden - 3)
    with pytest.raises(quant.KernelError):  # moe.rs:403-424; comes before the experts' sizes
        layer(top_k=0, gate=(t, w[:-1])).forward(x)
    for name in ("gate", "up", "down"):  # moe.rs:307-322
        with pytest.raises(quant.DimensionMismatch) as e:
            layer(**{name: (t, w[:-1])}).forward(x)
        assert (e.value.expected, e.value.got) == (w.size, w.size - 1)
    with pytest.raises(quant.DimensionMismatch) as e:
        layer().forward(x[:100])
    assert (e.value.expected, e.value.got) == (hidden, 100)
    with pytest.raises(quant.DimensionMismatch) as e:
        layer().forward_batch(x, 1, out=np.zeros(5, dtype=np.float32))
    assert (e.value.expected, e.value.got) == (hidden, 5)
    with pytest.raises(quant.UnsupportedType):
        layer(gate=(15, w)).forward(x)
    # a layer without experts leaves the zeroed output (moe.rs:240-242)
    empty = moe.MoeFfn(np.zeros(0, np.float32), (t, w[:0]), (t, w[:0]), (t, w[:0]), 1, 0, hidden, inter)
    out = empty.forward_batch(np.ones(2 * hidden, np.float32), 2, out=np.full(2 * hidden, 7.0, np.float32))
    assert np.all(out == 0)
    lib = capi.load()
    assert lib.oxq_moe_route_dev(None, None, 1, 2, 4, 0, None, None, None, None, None, None) == capi.ERR_KERNEL
    assert lib.oxq_moe_route_dev(None, None, 1, 2000, 4, 1, None, None, None, None, None, None) == capi.ERR_UNSUPPORTED_SHAPE
    assert lib.oxq_moe_ffn_workspace_bytes(t, t, t, 8, 288, 256) == 0  # the grouped kernel walks 256 columns at a time
    assert lib.oxq_moe_ffn_workspace_bytes(t, t, t, 8, 256, 512) > 0
    # the formats of independent 32-weight blocks (8: Q8_0) take rows of any whole number of blocks from eight up
    assert lib.oxq_moe_ffn_workspace_bytes(8, 8, 8, 8, 288, 352) > 0
    assert lib.oxq_moe_ffn_workspace_bytes(8, 8, 8, 8, 224, 352) == 0
    assert lib.oxq_moe_ffn_workspace_bytes(8, 8, 8, 8, 300, 352) == 0


def test_gemm_workspace_size_is_a_function_of_the_shape():
    """oxq_gemm_q8_workspace_bytes: the re-tiled activations (token rows padded to 128 and 128 more, 46 bytes per
    token block, rounded to 256), plus -- for at most 16 token rows (32 on fewer than 8192 weight rows) of Q4_K / IQ4_XS / Q4_0 /
    Q6_K / Q8_0 / Q5_K and the other weight formats (all but Q8_1) on a matrix of at least 2^22 weights (2^25 where rows are shorter than 4096)
    that yields fewer than 448 groups of 128 rows -- the room for the few-token kernel's per-split sums:
    splits x m x n floats, splits = min(ceil(448 / groups), k / 1024, 16) taken in even numbers of super-blocks.
    For Q4_K the size is at least what the prefill kernel's planes take."""
    lib = capi.load()

    def planes(m, k):
        return ((k // 32) * ((m + 127) // 128 * 128 + 128) * 46 + 255) // 256 * 256

    q4k, iq4xs, q6k = 12, 23, 14
    w = lib.oxq_gemm_q8_workspace_bytes
    assert w(q4k, 16, 14336, 4096) == planes(16, 4096) + 4 * 16 * 14336 * 4            # 112 groups -> 4 splits of 4
    assert w(iq4xs, 9, 4096, 14336) == planes(9, 14336) + 14 * 9 * 4096 * 4            # 32 groups -> 14 splits of 4
    assert w(q4k, 11, 16384, 3584) == planes(11, 3584) + 3 * 11 * 16384 * 4            # 14 super-blocks: 6 + 6 + 2
    assert w(q4k, 16, 4096, 4096) == planes(16, 4096) + 4 * 16 * 4096 * 4              # 2^24 weights, rows of 4096: 4 splits of 4
    assert w(q4k, 16, 4096, 2048) == planes(16, 2048)                                  # below 2^25 weights in rows shorter than 4096
    assert w(q4k, 16, 512, 4096) == planes(16, 4096)                                   # below 2^22 weights
    assert w(q4k, 17, 14336, 4096) == planes(17, 4096)                                 # more than 16 rows on 8192 weight rows and more
    assert w(q4k, 17, 4096, 14336) == planes(17, 14336) + 14 * 17 * 4096 * 4           # ... up to 32 rows on fewer
    assert w(q6k, 16, 14336, 4096) == planes(16, 4096) + 4 * 16 * 14336 * 4            # Q6_K, Q8_0, Q4_0 alike
    assert w(13, 16, 14336, 4096) == planes(16, 4096) + 4 * 16 * 14336 * 4             # Q5_K too
    assert w(11, 16, 14336, 4096) == planes(16, 4096) + 4 * 16 * 14336 * 4             # Q3_K (and Q4_1, IQ4_NL, Q5_0, Q5_1)
    assert w(10, 16, 14336, 4096) == planes(16, 4096) + 4 * 16 * 14336 * 4             # Q2_K
    assert w(9, 16, 14336, 4096) == planes(16, 4096)                                   # Q8_1: no few-token kernel
    assert w(q4k, 16, 128256, 4096) == planes(16, 4096)                                # 1002 groups fill the chip
    # Q4_K: never less than the prefill kernel's planes (74 bytes per token block, token rows padded to 128)
    def prefill(m, k):
        return (k // 32) * ((m + 127) // 128 * 128) * 74
    assert w(q4k, 512, 14336, 4096) == max(planes(512, 4096), prefill(512, 4096)) == prefill(512, 4096)
    assert w(q6k, 512, 14336, 4096) == planes(512, 4096)
    assert w(q4k, 16, 14336, 4000) == 0                                                # k not a multiple of 256
    # the formats of independent 32-weight blocks: any whole number of blocks from eight up, planes padded to whole
    # groups of eight blocks
    q8_0, q5_0 = 8, 6
    assert w(q8_0, 64, 4864, 896) == planes(64, 1024)
    assert w(q5_0, 64, 896, 4864) == planes(64, 4864)                                  # 152 blocks: whole groups
    assert w(q8_0, 64, 4864, 288) == planes(64, 512)
    assert w(q8_0, 64, 4864, 224) == 0                                                 # fewer than eight blocks
    assert w(q8_0, 64, 4864, 300) == 0                                                 # ends inside a block
    assert w(q6k, 64, 4864, 288) == 0
