"""Synthetic inputs for tests and benchmarks (host side, liboxq_synth.so).

Weights are drawn N(0, sigma) per row from a counter-seeded PRNG and encoded to
raw GGUF blocks; activations are N(0, 1).  See csrc/synth.cpp for the encoders.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboxq_synth.so")
_lib = None

BLOCK = {2: (32, 18), 8: (32, 34), 12: (256, 144), 14: (256, 210), 23: (256, 136)}


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m oxillama_amd.build`")
        lib = C.CDLL(LIB_PATH)
        lib.oxq_synth_normal_f32.restype = C.c_int
        lib.oxq_synth_normal_f32.argtypes = [C.c_uint64, C.c_float, C.c_void_p, C.c_size_t]
        lib.oxq_synth_encode.restype = C.c_int
        lib.oxq_synth_encode.argtypes = [C.c_uint32, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t]
        lib.oxq_synth_weights.restype = C.c_int
        lib.oxq_synth_weights.argtypes = [C.c_uint32, C.c_uint64, C.c_float, C.c_size_t, C.c_size_t,
                                          C.c_void_p, C.c_size_t, C.c_int]
        _lib = lib
    return _lib


def row_bytes(tensor_type, n_cols):
    bs, bb = BLOCK[int(tensor_type)]
    return n_cols // bs * bb


def normal_f32(seed, n, sigma=1.0):
    out = np.empty(n, dtype=np.float32)
    load().oxq_synth_normal_f32(seed, sigma, out.ctypes.data_as(C.c_void_p), n)
    return out


def encode(tensor_type, x):
    """x: float32 [n_rows, n_cols] -> uint8 raw blocks."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    n_rows, n_cols = x.shape
    out = np.empty(n_rows * row_bytes(tensor_type, n_cols), dtype=np.uint8)
    rc = load().oxq_synth_encode(int(tensor_type), x.ctypes.data_as(C.c_void_p), n_rows, n_cols,
                                 out.ctypes.data_as(C.c_void_p), out.size)
    if rc != 0:
        raise ValueError(f"cannot encode type {tensor_type} with n_cols={n_cols}")
    return out


def weights(tensor_type, seed, n_rows, n_cols, sigma=0.02, threads=None, out=None):
    """N(0, sigma) weights [n_rows x n_cols] encoded as raw GGUF blocks (uint8)."""
    n = n_rows * row_bytes(tensor_type, n_cols)
    if out is None:
        out = np.empty(n, dtype=np.uint8)
    assert out.size >= n and out.dtype == np.uint8
    threads = threads or min(16, os.cpu_count() or 1)
    rc = load().oxq_synth_weights(int(tensor_type), seed, sigma, n_rows, n_cols,
                                  out.ctypes.data_as(C.c_void_p), n, threads)
    if rc != 0:
        raise ValueError(f"cannot generate type {tensor_type} with n_cols={n_cols}")
    return out[:n]
