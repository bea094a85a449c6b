"""ctypes binding of liboxq_hip.so (the C ABI declared in include/oxq.h).

Plumbing for the Python tests and bench.py.  There is no fallback: if the HIP
library has not been built, loading raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("OXQ_HIP_LIB") or os.path.join(HERE, "liboxq_hip.so")

OK = 0
ERR_UNSUPPORTED_TYPE = 1
ERR_BLOCK_SIZE_MISMATCH = 2
ERR_DIMENSION_MISMATCH = 3
ERR_KERNEL = 4
ERR_BLOCK_COUNT_MISMATCH = 5
ERR_BUFFER_TOO_SMALL = 6
ERR_INTERNAL = 7
ERR_UNSUPPORTED_SHAPE = 8
ERR_NO_DEVICE = 9

TYPE_Q4_0, TYPE_Q8_0, TYPE_Q4_K, TYPE_Q6_K, TYPE_IQ4_XS = 2, 8, 12, 14, 23
TYPE_Q4_1, TYPE_Q5_0, TYPE_Q5_1, TYPE_Q8_1, TYPE_Q2_K, TYPE_Q3_K, TYPE_Q5_K, TYPE_IQ4_NL = 3, 6, 7, 9, 10, 11, 13, 20
GROUPS_OF_16 = (TYPE_Q6_K, TYPE_Q2_K, TYPE_Q3_K)  # formats whose exact integer sums cover 16 weights

# Every symbol include/oxq.h declares, with its signature.
_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_i32p = C.POINTER(C.c_int32)
_szp = C.POINTER(C.c_size_t)


class DeviceProps(C.Structure):
    _fields_ = [
        ("device", C.c_int),
        ("compute_units", C.c_int),
        ("clock_khz", C.c_int),
        ("memory_clock_khz", C.c_int),
        ("memory_bus_bits", C.c_int),
        ("total_memory", C.c_size_t),
        ("name", C.c_char * 128),
        ("arch", C.c_char * 64),
    ]


class GgufSummary(C.Structure):
    _fields_ = [("version", C.c_uint32), ("tensor_count", C.c_uint64), ("metadata_kv_count", C.c_uint64),
                ("n_tensors", C.c_uint64), ("n_metadata", C.c_uint64), ("alignment", C.c_uint64),
                ("data_offset", C.c_uint64), ("file_size", C.c_uint64)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_uint32), ("dims", C.c_uint64 * 4), ("type", C.c_uint32),
                ("offset", C.c_uint64), ("n_elements", C.c_uint64), ("data_size", C.c_uint64)]


class GgufValue(C.Structure):
    _fields_ = [("type", C.c_uint32), ("u", C.c_uint64), ("i", C.c_int64), ("f", C.c_double), ("str", C.c_void_p),
                ("str_len", C.c_size_t), ("elem_type", C.c_uint32), ("count", C.c_uint64), ("array_offset", C.c_uint64),
                ("array_bytes", C.c_uint64)]


# include/oxq_gguf.h
GGUF_SIGNATURES = {
    "oxq_gguf_open": (C.c_int, [C.c_char_p, C.POINTER(C.c_void_p)]),
    "oxq_gguf_open_bytes": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]),
    "oxq_gguf_close": (C.c_int, [C.c_void_p]),
    "oxq_gguf_get_summary": (C.c_int, [C.c_void_p, C.POINTER(GgufSummary)]),
    "oxq_gguf_tensor_at": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(GgufTensor)]),
    "oxq_gguf_find_tensor": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(GgufTensor)]),
    "oxq_gguf_tensor_data": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]),
    "oxq_gguf_meta_find": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(GgufValue)]),
    "oxq_gguf_meta_at": (C.c_int, [C.c_void_p, C.c_uint64, C.POINTER(C.c_char_p), C.POINTER(GgufValue)]),
    "oxq_gguf_meta_array_data": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t)]),
    "oxq_gguf_load_weights": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p)]),
    "oxq_gguf_upload_tensor": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t]),
}

SIGNATURES = {
    "oxq_init": (C.c_int, [C.c_int]),
    "oxq_shutdown": (C.c_int, []),
    "oxq_device_info": (C.c_int, [C.POINTER(DeviceProps)]),
    "oxq_last_error": (C.c_int, [_szp, _szp, C.c_char_p, C.c_size_t]),
    "oxq_status_name": (C.c_char_p, [C.c_int]),
    "oxq_block_size": (C.c_size_t, [C.c_uint32]),
    "oxq_block_bytes": (C.c_size_t, [C.c_uint32]),
    "oxq_type_name": (C.c_char_p, [C.c_uint32]),
    "oxq_get_kernel": (C.c_int, [C.c_uint32]),
    "oxq_dequant_block": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]),
    "oxq_quantize_f32_to_q8_0": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]),
    "oxq_matvec_q8_fused": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                      C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t]),
    "oxq_gemv": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, _szp, C.c_size_t, C.c_void_p,
                           C.c_size_t, C.c_void_p, C.c_size_t]),
    "oxq_gemm": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, _szp, C.c_size_t, C.c_void_p,
                           C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t]),
    "oxq_block_sums": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                 C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t]),
    "oxq_weight_cache_enable": (C.c_int, [C.c_int]),
    "oxq_weight_cache_clear": (C.c_int, []),
    "oxq_weight_cache_invalidate": (C.c_int, [C.c_void_p]),
    "oxq_weight_cache_set_limit": (C.c_int, [C.c_size_t]),
    "oxq_weight_cache_stats": (C.c_int, [_szp, _szp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "oxq_weights_register": (C.c_int, [C.c_uint32, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t,
                                       C.POINTER(C.c_void_p)]),
    "oxq_weights_release": (C.c_int, [C.c_void_p]),
    "oxq_weights_device_ptr": (C.c_void_p, [C.c_void_p]),
    "oxq_weights_nbytes": (C.c_size_t, [C.c_void_p]),
    "oxq_quantize_q8_0_dev": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]),
    "oxq_matvec_q8_fused_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                          C.c_size_t, C.c_int, C.c_void_p]),
    "oxq_matvec_q8_fused_multi_dev": (C.c_int, [C.c_uint32, C.c_size_t, C.POINTER(C.c_void_p), C.c_void_p,
                                                C.POINTER(C.c_void_p), C.c_size_t, C.c_size_t, C.c_int, C.c_void_p]),
    "oxq_gemv_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int,
                               C.c_void_p]),
    "oxq_gemv_f32_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                   C.c_int, C.c_void_p]),
    "oxq_select_activation_route": (C.c_int, [C.c_int]),
    "oxq_activation_route": (C.c_int, []),
    "oxq_gemv_multi_dev": (C.c_int, [C.c_uint32, C.c_size_t, C.POINTER(C.c_void_p), C.c_void_p,
                                     C.POINTER(C.c_void_p), C.c_size_t, C.c_size_t, C.c_int, C.c_void_p]),
    "oxq_gemm_q8_workspace_bytes": (C.c_size_t, [C.c_uint32, C.c_size_t, C.c_size_t, C.c_size_t]),
    "oxq_gemm_q8_static_max_workspace_bytes": (C.c_size_t, []),
    "oxq_gemm_q8_static_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                         C.c_size_t, C.c_int, C.c_void_p]),
    "oxq_gemm_q8_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                  C.c_size_t, C.c_size_t, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p]),
    "oxq_gemm_block_sums_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                          C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "oxq_gemm_scaled_sums_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                           C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "oxq_moe_gemm_q8_workspace_bytes": (C.c_size_t, [C.c_uint32, C.c_size_t, C.c_size_t, C.c_size_t]),
    "oxq_moe_gemm_q8_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p,
                                      C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int,
                                      C.c_void_p, C.c_size_t, C.c_void_p]),
    "oxq_lora_apply_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]),
    "oxq_linear_forward_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]),
    "oxq_linear_forward_multi_dev": (C.c_int, [C.c_uint32, C.c_size_t, C.POINTER(C.c_void_p), C.c_void_p,
                                               C.POINTER(C.c_void_p), C.POINTER(C.c_void_p),
                                               C.POINTER(C.c_size_t), C.c_size_t, C.c_void_p]),
    "oxq_linear_forward_batch_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                               C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t,
                                               C.c_void_p]),
    "oxq_linear_forward": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t), C.c_size_t,
                                     C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                     C.c_size_t, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t]),
    "oxq_linear_forward_batch": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t), C.c_size_t,
                                           C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                           C.c_size_t]),
    "oxq_swiglu_quantize_q8_0_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p,
                                               C.c_void_p]),
    "oxq_rmsnorm_quantize_q8_0_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_float, C.c_size_t, C.c_size_t,
                                                C.c_void_p, C.c_void_p, C.c_void_p]),
    "oxq_ffn_gate_up_swiglu_q8_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                C.c_size_t, C.c_size_t, C.c_void_p]),
    "oxq_ffn_workspace_bytes": (C.c_size_t, [C.c_size_t, C.c_size_t]),
    "oxq_ffn_swiglu_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32, C.c_void_p,
                                     C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t,
                                     C.c_void_p]),
    "oxq_moe_forward": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.c_uint32, C.c_void_p, C.c_size_t, C.c_uint32,
                                  C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t,
                                  C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t]),
    "oxq_moe_route_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p,
                                    C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "oxq_moe_gather_quantize_q8_0_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p,
                                                   C.c_void_p]),
    "oxq_moe_combine_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t,
                                      C.c_void_p, C.c_void_p]),
    "oxq_moe_ffn_workspace_bytes": (C.c_size_t, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_size_t, C.c_size_t,
                                                 C.c_size_t]),
    "oxq_moe_ffn_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.c_uint32, C.c_void_p, C.c_size_t, C.c_uint32,
                                  C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p,
                                  C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t,
                                  C.c_void_p, C.c_size_t, C.c_void_p]),
    "oxq_moe_forward_workspace_bytes": (C.c_size_t, [C.c_uint32, C.c_uint32, C.c_uint32, C.c_size_t, C.c_size_t,
                                                     C.c_size_t, C.c_size_t, C.c_size_t]),
    "oxq_moe_forward_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_size_t, C.c_uint32, C.c_void_p, C.c_size_t,
                                      C.c_uint32, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p,
                                      C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p,
                                      C.c_size_t, C.c_void_p]),
    "oxq_logits_edit_dev": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t,
                                      C.c_void_p, C.c_size_t, C.c_size_t, C.c_float, C.c_void_p]),
    "oxq_sample_candidates_dev": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.c_float, C.c_float,
                                            C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "oxq_topk_workspace_bytes": (C.c_size_t, [C.c_size_t, C.c_size_t]),
    "oxq_topk_dev": (C.c_int, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                               C.c_void_p]),
    "oxq_lm_head_topk_workspace_bytes": (C.c_size_t, [C.c_uint32, C.c_size_t, C.c_size_t, C.c_size_t]),
    "oxq_lm_head_topk_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t,
                                       C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "oxq_block_sums_dev": (C.c_int, [C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t,
                                     C.c_size_t, C.c_void_p]),
}

# include/oxq_tuning.h: launch-shape knobs for benchmarks and tests, outside the drop-in boundary.
TUNING_SIGNATURES = {
    "oxq_set_gemv_waves_per_cu": (C.c_int, [C.c_uint]),
    "oxq_set_gemv_rows_per_batch": (C.c_int, [C.c_uint]),
    "oxq_set_gemv_waves_per_row": (C.c_int, [C.c_uint]),
    "oxq_set_gemm_variant": (C.c_int, [C.c_int]),
    "oxq_set_gemm_tile_min_rows": (C.c_int, [C.c_uint]),
    "oxq_set_ffn_fusion": (C.c_int, [C.c_int]),
    "oxq_last_launch": (C.c_int, [C.c_char_p, C.c_size_t]),
    "oxq_set_gemv_phase_probe": (C.c_int, [C.c_void_p, C.c_size_t]),
}

_lib = None


def load():
    """Load liboxq_hip.so and attach signatures.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m oxillama_amd.build` "
            "(there is no CPU fallback for the HIP path)")
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in {**SIGNATURES, **GGUF_SIGNATURES, **TUNING_SIGNATURES}.items():
        fn = getattr(lib, name)  # AttributeError if the ABI lost a symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error():
    lib = load()
    a, b = C.c_size_t(0), C.c_size_t(0)
    msg = C.create_string_buffer(256)
    status = lib.oxq_last_error(C.byref(a), C.byref(b), msg, 256)
    return status, a.value, b.value, msg.value.decode("utf-8", "replace")
