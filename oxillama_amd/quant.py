"""Python mirror of the reference's kernel interface for the quantized-matmul path.

Names, argument meaning and error behaviour follow the reference crate
(Q/ = crates/oxillama-quant/src):

  QuantError variants         Q/error.rs:10-71
  GgufTensorType              crates/oxillama-gguf/src/types.rs:72-262
  QuantTensor                 Q/types.rs:11-50
  QuantKernel (HipKernel)     Q/traits.rs:21-183
  KernelDispatcher.get_kernel Q/dispatch.rs:141
  quantize_f32_to_q8_0        Q/quantize.rs:58

Every method crosses the C ABI of liboxq_hip.so with numpy host buffers; the
compute runs on the GPU.  `HipKernel.*_dev` methods take torch CUDA tensors and
enqueue on torch's current stream without copies.
"""
import ctypes as C
import enum

import numpy as np

from . import capi


class QuantError(Exception):
    """Base of the reference's QuantError variants."""


class UnsupportedType(QuantError):
    def __init__(self, quant_type):
        super().__init__(f"unsupported quantization type: {quant_type}")
        self.quant_type = quant_type


class BlockSizeMismatch(QuantError):
    def __init__(self, expected, got):
        super().__init__(f"block size mismatch: expected {expected}, got {got}")
        self.expected, self.got = expected, got


class DimensionMismatch(QuantError):
    def __init__(self, expected, got):
        super().__init__(f"dimension mismatch: expected {expected}, got {got}")
        self.expected, self.got = expected, got


class KernelError(QuantError):
    def __init__(self, message):
        super().__init__(f"kernel error: {message}")
        self.message = message


class BlockCountMismatch(QuantError):
    def __init__(self, expected, got):
        super().__init__(f"block count mismatch: expected {expected} blocks, got {got}")
        self.expected, self.got = expected, got


class BufferTooSmall(QuantError):
    def __init__(self, needed, available):
        super().__init__(f"buffer too small: need {needed} bytes, have {available}")
        self.needed, self.available = needed, available


class Internal(QuantError):
    def __init__(self, message):
        super().__init__(f"internal error: {message}")
        self.message = message


class UnsupportedShape(QuantError):
    """Not a reference variant: the HIP tier declines the shape; use the CPU kernel."""

    def __init__(self, multiple_of, got):
        super().__init__(f"unsupported shape: n_cols {got} is not a multiple of {multiple_of}")
        self.multiple_of, self.got = multiple_of, got


class NoDevice(QuantError):
    """Not a reference variant: no usable GPU."""


def _raise(status):
    st, a, b, msg = capi.last_error()
    if status == capi.ERR_UNSUPPORTED_TYPE:
        raise UnsupportedType(a)
    if status == capi.ERR_BLOCK_SIZE_MISMATCH:
        raise BlockSizeMismatch(a, b)
    if status == capi.ERR_DIMENSION_MISMATCH:
        raise DimensionMismatch(a, b)
    if status == capi.ERR_KERNEL:
        raise KernelError(msg)
    if status == capi.ERR_BLOCK_COUNT_MISMATCH:
        raise BlockCountMismatch(a, b)
    if status == capi.ERR_BUFFER_TOO_SMALL:
        raise BufferTooSmall(a, b)
    if status == capi.ERR_UNSUPPORTED_SHAPE:
        raise UnsupportedShape(a, b)
    if status == capi.ERR_NO_DEVICE:
        raise NoDevice(msg)
    raise Internal(msg or f"status {status}")


def _check(status):
    if status != capi.OK:
        _raise(status)


class GgufTensorType(enum.IntEnum):
    Q4_0 = 2
    Q8_0 = 8
    Q4K = 12
    Q6K = 14
    Iq4Xs = 23
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_1 = 9
    Q2K = 10
    Q3K = 11
    Q5K = 13
    Iq4Nl = 20

    def block_size(self):
        return {2: 32, 8: 32, 12: 256, 14: 256, 23: 256, 3: 32, 6: 32, 7: 32, 9: 32, 10: 256, 11: 256, 13: 256,
                20: 32}[int(self)]

    def block_bytes(self):
        return {2: 18, 8: 34, 12: 144, 14: 210, 23: 136, 3: 20, 6: 22, 7: 24, 9: 36, 10: 84, 11: 110, 13: 176,
                20: 18}[int(self)]

    def type_name(self):
        return {2: "Q4_0", 8: "Q8_0", 12: "Q4_K", 14: "Q6_K", 23: "IQ4_XS", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 9: "Q8_1",
                10: "Q2_K", 11: "Q3_K", 13: "Q5_K", 20: "IQ4_NL"}[int(self)]


class QuantTensor:
    """Raw block data plus shape and type (Q/types.rs:11-50)."""

    def __init__(self, data, shape, tensor_type):
        self.data = np.ascontiguousarray(np.frombuffer(bytes(data), dtype=np.uint8)
                                         if not isinstance(data, np.ndarray) else data.view(np.uint8).ravel())
        self.shape = list(shape)
        self.tensor_type = tensor_type

    def n_elements(self):
        if not self.shape:
            return 0
        n = 1
        for s in self.shape:
            n *= s
        return n

    def n_blocks(self):
        bs = GgufTensorType(self.tensor_type).block_size()
        return -(-self.n_elements() // bs)

    def expected_data_size(self):
        return self.n_blocks() * GgufTensorType(self.tensor_type).block_bytes()


def _u8(buf):
    if isinstance(buf, np.ndarray):
        arr = np.ascontiguousarray(buf).view(np.uint8).ravel()
    else:
        arr = np.frombuffer(bytes(buf), dtype=np.uint8)
    return arr


def _ptr(arr):
    return arr.ctypes.data_as(C.c_void_p)


def quantize_f32_to_q8_0(data):
    """Q/quantize.rs:58: f32[n] -> n/32 Q8_0 blocks (34 bytes each), on the GPU."""
    lib = capi.load()
    x = np.ascontiguousarray(data, dtype=np.float32).ravel()
    out = np.zeros(x.size // 32 * 34, dtype=np.uint8)
    _check(lib.oxq_quantize_f32_to_q8_0(_ptr(x), x.size, _ptr(out), out.size))
    return out


class HipKernel:
    """QuantKernel implementation backed by liboxq_hip.so (Q/traits.rs:21-183)."""

    def __init__(self, tensor_type):
        self._lib = capi.load()
        self.tensor_type = int(tensor_type)
        _check(self._lib.oxq_get_kernel(self.tensor_type))

    # -- metadata ----------------------------------------------------------
    def block_size(self):
        return self._lib.oxq_block_size(self.tensor_type)

    def block_bytes(self):
        return self._lib.oxq_block_bytes(self.tensor_type)

    def name(self):
        return self._lib.oxq_type_name(self.tensor_type).decode()

    # -- host-slice trait methods -------------------------------------------
    def dequant_block(self, block, output):
        """output: float32 ndarray, filled in place (its length is checked)."""
        b = _u8(block)
        _check(self._lib.oxq_dequant_block(self.tensor_type, _ptr(b), b.size, _ptr(output), output.size))

    def gemv(self, quant_matrix, input, output):
        w = _u8(quant_matrix.data)
        shape = (C.c_size_t * len(quant_matrix.shape))(*quant_matrix.shape)
        x = np.ascontiguousarray(input, dtype=np.float32)
        _check(self._lib.oxq_gemv(self.tensor_type, _ptr(w), w.size, shape, len(quant_matrix.shape),
                                  _ptr(x), x.size, _ptr(output), output.size))

    def gemm(self, quant_matrix, input, output, m, n, k):
        w = _u8(quant_matrix.data)
        shape = (C.c_size_t * len(quant_matrix.shape))(*quant_matrix.shape)
        x = np.ascontiguousarray(input, dtype=np.float32)
        _check(self._lib.oxq_gemm(self.tensor_type, _ptr(w), w.size, shape, len(quant_matrix.shape),
                                  _ptr(x), x.size, _ptr(output), output.size, m, n, k))

    def matvec_q8_fused(self, weights, acts_q8, out, n_rows, n_cols):
        """out[r] += W[r,:] . acts  (accumulates, Q/traits.rs:84-86)."""
        w, a = _u8(weights), _u8(acts_q8)
        _check(self._lib.oxq_matvec_q8_fused(self.tensor_type, _ptr(w), w.size, _ptr(a), a.size,
                                             _ptr(out), out.size, n_rows, n_cols))

    def block_sums(self, weights, acts_q8, n_rows, n_cols):
        w, a = _u8(weights), _u8(acts_q8)
        groups = n_cols // (16 if self.tensor_type in capi.GROUPS_OF_16 else 32)
        sums = np.zeros(n_rows * groups, dtype=np.int32)
        _check(self._lib.oxq_block_sums(self.tensor_type, _ptr(w), w.size, _ptr(a), a.size,
                                        _ptr(sums), sums.size, n_rows, n_cols))
        return sums.reshape(n_rows, groups)

    # -- device-pointer route (torch CUDA tensors, current stream) ----------
    @staticmethod
    def _stream():
        import torch
        return C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def matvec_q8_fused_dev(self, d_weights, d_acts, d_out, n_rows, n_cols, accumulate=True):
        _check(self._lib.oxq_matvec_q8_fused_dev(self.tensor_type, d_weights.data_ptr(), d_acts.data_ptr(),
                                                 d_out.data_ptr(), n_rows, n_cols, int(accumulate),
                                                 self._stream()))

    def matvec_q8_fused_multi_dev(self, d_weights, d_acts, d_outs, n_rows, n_cols, accumulate=True):
        """Up to 4 matrices of one shape sharing d_acts, one launch (wq/wk/wv, ffn_gate/ffn_up)."""
        import ctypes as C
        n = len(d_weights)
        wp = (C.c_void_p * n)(*[w.data_ptr() for w in d_weights])
        op = (C.c_void_p * n)(*[o.data_ptr() for o in d_outs])
        _check(self._lib.oxq_matvec_q8_fused_multi_dev(self.tensor_type, n, wp, d_acts.data_ptr(), op, n_rows, n_cols,
                                                       int(accumulate), self._stream()))

    def gemv_dev(self, d_weights, d_x, d_out, n_rows, n_cols, accumulate=False):
        """fp32 activations in, quantized to Q8_0 inside the kernel (one launch)."""
        _check(self._lib.oxq_gemv_dev(self.tensor_type, d_weights.data_ptr(), d_x.data_ptr(), d_out.data_ptr(),
                                      n_rows, n_cols, int(accumulate), self._stream()))

    def gemv_f32_dev(self, d_weights, d_x, d_out, n_rows, n_cols, accumulate=False, d_bias=None):
        """QuantKernel::gemv with the reference's numerics: fp32 activations against weights dequantized in
        registers (oxq_gemv_f32_dev)."""
        _check(self._lib.oxq_gemv_f32_dev(self.tensor_type, d_weights.data_ptr(), d_x.data_ptr(),
                                          d_bias.data_ptr() if d_bias is not None else None, d_out.data_ptr(),
                                          n_rows, n_cols, int(accumulate), self._stream()))

    def gemv_multi_dev(self, d_weights, d_x, d_outs, n_rows, n_cols, accumulate=False):
        import ctypes as C
        n = len(d_weights)
        wp = (C.c_void_p * n)(*[w.data_ptr() for w in d_weights])
        op = (C.c_void_p * n)(*[o.data_ptr() for o in d_outs])
        _check(self._lib.oxq_gemv_multi_dev(self.tensor_type, n, wp, d_x.data_ptr(), op, n_rows, n_cols,
                                            int(accumulate), self._stream()))

    def gemm_workspace_bytes(self, m, n, k):
        return self._lib.oxq_gemm_q8_workspace_bytes(self.tensor_type, m, n, k)

    def gemm_q8_dev(self, d_weights, d_acts, d_out, m, n, k, accumulate=False, workspace=None):
        """workspace: uint8 CUDA tensor of gemm_workspace_bytes(m, n, k) bytes (256-byte aligned), or None."""
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_len = workspace.numel() if workspace is not None else 0
        _check(self._lib.oxq_gemm_q8_dev(self.tensor_type, d_weights.data_ptr(), d_acts.data_ptr(),
                                         d_out.data_ptr(), m, n, k, int(accumulate), ws_ptr, ws_len, self._stream()))

    def gemm_q8_static_dev(self, d_weights, d_acts, d_out, m, n, k, accumulate=False):
        """gemm_q8_dev on the library's static device scratch: allocates nothing (shapes up to the scratch size)."""
        _check(self._lib.oxq_gemm_q8_static_dev(self.tensor_type, d_weights.data_ptr(), d_acts.data_ptr(),
                                                d_out.data_ptr(), m, n, k, int(accumulate), self._stream()))

    def gemm_block_sums_dev(self, d_weights, d_acts, d_out, d_sums, m, n, k, workspace=None):
        ws_ptr = workspace.data_ptr() if workspace is not None else None
        ws_len = workspace.numel() if workspace is not None else 0
        _check(self._lib.oxq_gemm_block_sums_dev(self.tensor_type, d_weights.data_ptr(), d_acts.data_ptr(),
                                                 d_out.data_ptr(), d_sums.data_ptr(), m, n, k, ws_ptr, ws_len,
                                                 self._stream()))

    def gemm_scaled_sums_dev(self, d_weights, d_acts, d_out, d_sums, m, n, k, workspace):
        """The prefill kernel's debug dump: sub-block scale times integer group sum per (token, row, sub-block)."""
        _check(self._lib.oxq_gemm_scaled_sums_dev(self.tensor_type, d_weights.data_ptr(), d_acts.data_ptr(),
                                                  d_out.data_ptr(), d_sums.data_ptr(), m, n, k, workspace.data_ptr(),
                                                  workspace.numel(), self._stream()))

    def moe_gemm_workspace_bytes(self, total_rows, n, k):
        return self._lib.oxq_moe_gemm_q8_workspace_bytes(self.tensor_type, total_rows, n, k)

    def moe_gemm_q8_dev(self, d_weights, expert_stride, n_experts, d_acts, d_offsets, total_rows, max_rows, d_out,
                        n, k, workspace, accumulate=False, d_sums=None):
        """Grouped expert matmul: rows d_offsets[e]..d_offsets[e+1]-1 of d_acts times expert e's weights
        (d_weights + e * expert_stride bytes) -> the same rows of d_out [total_rows x n]."""
        _check(self._lib.oxq_moe_gemm_q8_dev(self.tensor_type, d_weights.data_ptr(), expert_stride, n_experts,
                                             d_acts.data_ptr(), d_offsets.data_ptr(), total_rows, max_rows,
                                             d_out.data_ptr(), d_sums.data_ptr() if d_sums is not None else None,
                                             n, k, int(accumulate), workspace.data_ptr(), workspace.numel(),
                                             self._stream()))

    def block_sums_dev(self, d_weights, d_acts, d_sums, n_rows, n_cols):
        _check(self._lib.oxq_block_sums_dev(self.tensor_type, d_weights.data_ptr(), d_acts.data_ptr(),
                                            d_sums.data_ptr(), n_rows, n_cols, self._stream()))


def quantize_q8_0_dev(d_x, d_out):
    lib = capi.load()
    _check(lib.oxq_quantize_q8_0_dev(d_x.data_ptr(), d_x.numel(), d_out.data_ptr(), HipKernel._stream()))


class KernelDispatcher:
    """get_kernel(type) -> kernel, or UnsupportedType (Q/dispatch.rs:141)."""

    def get_kernel(self, tensor_type):
        return HipKernel(tensor_type)


ROUTE_Q8, ROUTE_F32 = 0, 1


def select_activation_route(route):
    """How the fp32-input entry points (gemv, gemm, QuantLinear forward on host slices, linear forward on device
    without Q8_0 activations) treat their input: ROUTE_Q8 quantizes it to Q8_0 (the fused kernels), ROUTE_F32 runs
    the reference's gemv arithmetic (oxq_select_activation_route)."""
    _check(capi.load().oxq_select_activation_route(int(route)))


def activation_route():
    return capi.load().oxq_activation_route()


def init(device=0):
    _check(capi.load().oxq_init(device))


def device_info():
    props = capi.DeviceProps()
    _check(capi.load().oxq_device_info(C.byref(props)))
    return {
        "device": props.device,
        "compute_units": props.compute_units,
        "clock_khz": props.clock_khz,
        "memory_clock_khz": props.memory_clock_khz,
        "memory_bus_bits": props.memory_bus_bits,
        "total_memory": props.total_memory,
        "name": props.name.decode(),
        "arch": props.arch.decode(),
    }
