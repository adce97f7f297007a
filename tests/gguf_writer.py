"""Byte-level GGUF writer for tests: builds files the way the reference's test builder does
(crates/rnb-loader/src/gguf/parser.rs:411-493: magic, version, counts, then hand-written records)."""
import struct

T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)
_FMT = {T_U8: "B", T_I8: "b", T_U16: "H", T_I16: "h", T_U32: "I", T_I32: "i", T_F32: "f", T_BOOL: "B",
        T_U64: "Q", T_I64: "q", T_F64: "d"}


class Builder:
    def __init__(self, version=3, tensor_count=None, kv_count=None, big_endian=False):
        self.e = ">" if big_endian else "<"
        self.buf = bytearray(b"GGUF") + struct.pack(self.e + "I", version)
        if tensor_count is not None:
            self.buf += struct.pack(self.e + "QQ", tensor_count, kv_count)

    def raw(self, b):
        self.buf += b
        return self

    def num(self, fmt, v):
        self.buf += struct.pack(self.e + fmt, v)
        return self

    def string(self, s):
        b = s if isinstance(s, bytes) else s.encode("utf-8")
        self.num("Q", len(b))
        self.buf += b
        return self

    def value(self, vtype, v, elem_type=None):
        if vtype == T_STR:
            return self.string(v)
        if vtype == T_ARR:
            self.num("I", elem_type).num("Q", len(v))
            for item in v:
                self.value(elem_type, item)
            return self
        return self.num(_FMT[vtype], v)

    def kv(self, key, vtype, v, elem_type=None):
        self.string(key).num("I", vtype)
        return self.value(vtype, v, elem_type)

    def tensor_info(self, name, dims_innermost_first, ggml_type, offset):
        self.string(name).num("I", len(dims_innermost_first))
        for d in dims_innermost_first:
            self.num("Q", d)
        return self.num("I", ggml_type).num("Q", offset)

    def pad(self, alignment=32):
        self.buf += b"\0" * ((alignment - len(self.buf) % alignment) % alignment)
        return self

    def build(self):
        return bytes(self.buf)


def write_model(path, metadata, tensors, alignment=32, set_alignment_key=False):
    """metadata: [(key, type, value[, elem_type])]; tensors: [(name, row_major_shape, ggml_type, bytes)].
    Returns {name: absolute file offset}."""
    md = list(metadata)
    if set_alignment_key:
        md.append(("general.alignment", T_U32, alignment))
    b = Builder(3, len(tensors), len(md))
    for item in md:
        b.kv(*item)
    offsets, rel = {}, 0
    for name, shape, ggml_type, data in tensors:
        rel += (alignment - rel % alignment) % alignment
        b.tensor_info(name, list(shape)[::-1], ggml_type, rel)
        offsets[name] = rel
        rel += len(data)
    b.pad(alignment)
    start = len(b.buf)
    for name, shape, ggml_type, data in tensors:
        b.buf += b"\0" * (start + offsets[name] - len(b.buf))
        b.buf += bytes(data)
    with open(path, "wb") as f:
        f.write(b.buf)
    return {k: start + v for k, v in offsets.items()}
