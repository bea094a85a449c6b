"""Builders of GGUF file images for the tests, byte for byte as the reference's own tests assemble
them (crates/oxillama-gguf/src/parser.rs:232-275,352-372,520-613, loader.rs tests), plus a small
independent parser used to cross-check the library on randomized files.  Test infrastructure."""
import struct

MAGIC = 0x46554747
(U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64) = range(13)
_FMT = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
        F64: "<d"}
# block_size, block_bytes per tensor type id (crates/oxillama-gguf/src/types.rs:199-262)
LAYOUT = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
          10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292), 16: (256, 66),
          17: (256, 74), 18: (256, 98), 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82), 23: (256, 136),
          24: (1, 1), 25: (1, 2), 26: (1, 4), 27: (1, 8), 28: (1, 8), 29: (256, 56), 30: (1, 2), 31: (32, 18),
          32: (32, 18), 33: (32, 18), 34: (256, 54), 35: (256, 66), 36: (32, 34), 37: (32, 34), 38: (32, 34),
          39: (128, 18)}


def _len(version, n):
    return struct.pack("<Q", n) if version >= 3 else struct.pack("<I", n)


def string(version, s):
    b = s if isinstance(s, bytes) else s.encode()
    return _len(version, len(b)) + b


def value(version, vtype, v):
    if vtype == STRING:
        return string(version, v)
    if vtype == ARRAY:
        et, items = v
        return struct.pack("<I", et) + _len(version, len(items)) + b"".join(value(version, et, x) for x in items)
    return struct.pack(_FMT[vtype], v)


def align_up(n, a):
    return n if a == 0 or n % a == 0 else n + a - n % a


def build(version, kvs, tensors, data=b"", alignment=32, counts=None):
    """kvs: [(key, vtype, value)]; tensors: [(name, dims, type_id, offset)]; data: the data section."""
    out = struct.pack("<II", MAGIC, version)
    n_t, n_kv = counts if counts else (len(tensors), len(kvs))
    out += _len(version, n_t) + _len(version, n_kv)
    for key, vtype, v in kvs:
        out += string(version, key) + struct.pack("<I", vtype) + value(version, vtype, v)
    for name, dims, type_id, offset in tensors:
        out += string(version, name) + struct.pack("<I", len(dims))
        out += b"".join(_len(version, d) for d in dims)
        out += struct.pack("<I", type_id)
        out += struct.pack("<Q", offset) if version >= 2 else struct.pack("<I", offset)
    out += b"\0" * (align_up(len(out), alignment) - len(out))
    return out + data


# ---- an independent parser (straight from the layout above) -------------------------------------------

class Eof(Exception):
    pass


def parse(buf):
    pos = 0

    def rd(fmt):
        nonlocal pos
        n = struct.calcsize(fmt)
        if pos + n > len(buf):
            raise Eof(pos)
        v = struct.unpack_from(fmt, buf, pos)[0]
        pos += n
        return v

    magic, version = rd("<I"), rd("<I")
    assert magic == MAGIC and 1 <= version <= 3
    ln = (lambda: rd("<Q")) if version >= 3 else (lambda: rd("<I"))

    def rd_str():
        nonlocal pos
        n = ln()
        if pos + n > len(buf):
            raise Eof(pos)
        s = bytes(buf[pos:pos + n]).decode("utf-8")
        pos += n
        return s

    def rd_val(t):
        if t == STRING:
            return rd_str()
        if t == ARRAY:
            et = rd("<I")
            n = ln()
            return ("array", et, n, [rd_val(et) for _ in range(n)])
        if t == BOOL:
            return rd("<B") != 0
        return rd(_FMT[t])

    n_t, n_kv = ln(), ln()
    meta = {}
    for _ in range(n_kv):
        k = rd_str()
        meta[k] = rd_val(rd("<I"))
    tensors = {}
    for _ in range(n_t):
        name = rd_str()
        dims = [ln() for _ in range(rd("<I"))]
        tid = rd("<I")
        off = rd("<Q") if version >= 2 else rd("<I")
        tensors[name] = (dims, tid, off)
    al = meta.get("general.alignment", 32)
    if not isinstance(al, int) or isinstance(al, bool) or al < 0:
        al = 32
    return version, meta, tensors, align_up(pos, al), al
