"""Python mirror of the reference's GGUF reader over liboxq_hip.so (include/oxq_gguf.h).

  GgufError variants   crates/oxillama-gguf/src/error.rs:14-60
  GgufModel            crates/oxillama-gguf/src/loader.rs:21-140 (load / from_bytes / tensor_data / architecture)
  GgufFile             crates/oxillama-gguf/src/parser.rs:17-90
  TensorInfo           crates/oxillama-gguf/src/tensor_info.rs:22-50
  load_quant_linear    crates/oxillama-arch/src/llama/model.rs:805-822 (here: the tensor lands in HBM)
"""
import ctypes as C

import numpy as np

from . import capi
from .quant import _check as _check_quant


class GgufError(Exception):
    pass


class InvalidMagic(GgufError):
    def __init__(self, magic):
        super().__init__(f"invalid GGUF magic number: expected 0x46554747, got 0x{magic:08X}")
        self.magic = magic


class UnsupportedVersion(GgufError):
    def __init__(self, version):
        super().__init__(f"unsupported GGUF version: {version} (supported: 1, 2, 3)")
        self.version = version


class UnexpectedEof(GgufError):
    def __init__(self, offset):
        super().__init__(f"unexpected end of file at offset {offset}")
        self.offset = offset


class InvalidMetadata(GgufError):
    pass


class UnsupportedQuantType(GgufError):
    def __init__(self, type_id):
        super().__init__(f"unsupported quantization type: id={type_id}")
        self.type_id = type_id


class TensorNotFound(GgufError):
    def __init__(self, name):
        super().__init__(f"tensor not found: '{name}'")
        self.name = name


class InvalidString(GgufError):
    def __init__(self, offset):
        super().__init__(f"invalid UTF-8 string at offset {offset}")
        self.offset = offset


class IoError(GgufError):
    pass


def _check(status):
    if status == capi.OK:
        return
    if status < 10:
        _check_quant(status)
    _, a, _, msg = capi.last_error()
    raise {10: lambda: InvalidMagic(a), 11: lambda: UnsupportedVersion(a), 12: lambda: UnexpectedEof(a),
           13: lambda: InvalidMetadata(msg), 14: lambda: UnsupportedQuantType(a), 15: lambda: TensorNotFound(msg),
           16: lambda: InvalidString(a), 17: lambda: IoError(msg)}.get(status, lambda: GgufError(msg))()


class TensorInfo:
    def __init__(self, t):
        self.name = t.name.decode()
        self.n_dims = t.n_dims
        self.dimensions = [int(t.dims[i]) for i in range(min(t.n_dims, 4))]
        self.tensor_type = t.type
        self.offset = t.offset
        self._n_elements, self._data_size = t.n_elements, t.data_size

    def n_elements(self):
        return self._n_elements

    def data_size(self):
        return self._data_size


class DeviceWeights:
    """A QuantTensor resident in HBM: shape = the stored dimensions, bytes unchanged."""

    def __init__(self, handle, info):
        self._lib = capi.load()
        self.handle = handle
        self.tensor_type = info.tensor_type
        self.shape = list(info.dimensions)
        self.nbytes = self._lib.oxq_weights_nbytes(handle)

    def device_ptr(self):
        return self._lib.oxq_weights_device_ptr(self.handle)

    def release(self):
        if self.handle:
            self._lib.oxq_weights_release(self.handle)
            self.handle = None


def _value(v):
    t = v.type
    if t in (0, 2, 4, 10):
        return int(v.u)
    if t in (1, 3, 5, 11):
        return int(v.i)
    if t in (6, 12):
        return float(v.f)
    if t == 7:
        return bool(v.u)
    if t == 8:
        return C.string_at(v.str, v.str_len).decode("utf-8")
    return ("array", v.elem_type, int(v.count))


class GgufModel:
    def __init__(self, handle):
        self._lib = capi.load()
        self._h = handle
        s = capi.GgufSummary()
        _check(self._lib.oxq_gguf_get_summary(self._h, C.byref(s)))
        self.version, self.tensor_count, self.metadata_kv_count = s.version, s.tensor_count, s.metadata_kv_count
        self.n_tensors, self.n_metadata = s.n_tensors, s.n_metadata
        self.alignment, self.data_offset, self._file_size = s.alignment, s.data_offset, s.file_size

    @classmethod
    def load(cls, path):
        lib = capi.load()
        h = C.c_void_p()
        _check(lib.oxq_gguf_open(str(path).encode(), C.byref(h)))
        return cls(h)

    @classmethod
    def from_bytes(cls, data):
        lib = capi.load()
        buf = np.frombuffer(bytes(data), dtype=np.uint8)
        h = C.c_void_p()
        _check(lib.oxq_gguf_open_bytes(buf.ctypes.data_as(C.c_void_p), buf.size, C.byref(h)))
        return cls(h)

    def close(self):
        if self._h:
            self._lib.oxq_gguf_close(self._h)
            self._h = None

    def file_size(self):
        return self._file_size

    def tensors(self):
        out = []
        for i in range(self.n_tensors):
            t = capi.GgufTensor()
            _check(self._lib.oxq_gguf_tensor_at(self._h, i, C.byref(t)))
            out.append(TensorInfo(t))
        return out

    def tensor(self, name):
        t = capi.GgufTensor()
        _check(self._lib.oxq_gguf_find_tensor(self._h, name.encode(), C.byref(t)))
        return TensorInfo(t)

    def tensor_data(self, name):
        """The tensor's bytes (a copy of the slice of the mapping)."""
        p, n = C.c_void_p(), C.c_size_t()
        _check(self._lib.oxq_gguf_tensor_data(self._h, name.encode(), C.byref(p), C.byref(n)))
        return np.frombuffer(C.string_at(p, n.value), dtype=np.uint8)

    def metadata(self, key):
        v = capi.GgufValue()
        _check(self._lib.oxq_gguf_meta_find(self._h, key.encode(), C.byref(v)))
        return _value(v)

    def metadata_array(self, key):
        """The elements of an array value: numbers, booleans or strings (tokenizer.ggml.tokens, scores,
        merges ...), decoded from the encoded bytes the library points at."""
        import struct
        v = capi.GgufValue()
        _check(self._lib.oxq_gguf_meta_find(self._h, key.encode(), C.byref(v)))
        p, n = C.c_void_p(), C.c_size_t()
        _check(self._lib.oxq_gguf_meta_array_data(self._h, key.encode(), C.byref(p), C.byref(n)))
        raw = C.string_at(p, n.value)
        fixed = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q", 12: "<d"}
        et, count = v.elem_type, int(v.count)
        if et in fixed:
            vals = [x[0] for x in struct.iter_unpack(fixed[et], raw)]
            assert len(vals) == count
            return [bool(x) for x in vals] if et == 7 else vals
        if et != 8:
            raise InvalidMetadata(f"{key}: arrays of arrays are not decoded")
        lfmt, lsz = ("<Q", 8) if self.version >= 3 else ("<I", 4)
        out, pos = [], 0
        for _ in range(count):
            (ln,) = struct.unpack_from(lfmt, raw, pos)
            out.append(raw[pos + lsz:pos + lsz + ln].decode("utf-8"))
            pos += lsz + ln
        return out

    def metadata_items(self):
        out = []
        for i in range(self.n_metadata):
            k, v = C.c_char_p(), capi.GgufValue()
            _check(self._lib.oxq_gguf_meta_at(self._h, i, C.byref(k), C.byref(v)))
            out.append((k.value.decode(), _value(v)))
        return out

    def architecture(self):
        v = self.metadata("general.architecture")
        if not isinstance(v, str):
            raise InvalidMetadata("general.architecture: expected string value")
        return v

    def model_name(self):
        try:
            v = self.metadata("general.name")
        except InvalidMetadata:
            return None
        return v if isinstance(v, str) else None

    def load_quant_linear(self, name):
        """The tensor as device-resident weights (file -> pinned staging -> HBM)."""
        info = self.tensor(name)
        h = C.c_void_p()
        _check(self._lib.oxq_gguf_load_weights(self._h, name.encode(), C.byref(h)))
        return DeviceWeights(h, info)

    def upload_tensor(self, name, d_dst):
        """Raw bytes of any tensor into a torch CUDA tensor (uint8 view is taken by byte size)."""
        _check(self._lib.oxq_gguf_upload_tensor(self._h, name.encode(), d_dst.data_ptr(),
                                                d_dst.numel() * d_dst.element_size()))
