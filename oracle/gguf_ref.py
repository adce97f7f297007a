"""CPU restatement of the reference's GGUF header parser — TEST INFRASTRUCTURE ONLY (never imported by the product).

Follows crates/rnb-loader/src/gguf/parser.rs:247-407 (GGUFFile::parse), crates/rnb-loader/src/gguf/types.rs:5-41
(ggml type ids), crates/rnb-loader/src/convert.rs:28-83 (checked_tensor_size, ggml_quant_params) and :99-178
(map_tensors bounds).  Errors are raised as GGUFError whose text is the reference's LoaderError Display string
(crates/rnb-loader/src/error.rs:4-16).

Pins (tests/test_gguf.py): the reference's own parser and converter tests restated on byte strings built the way its
test builder builds them (parser.rs:411-717, convert.rs:186-392): minimal v3 file, tensor-info dimension reversal
[4, 8] -> [8, 4], data_start alignment, 64-bit metadata values, every rejection case with its message fragment, the
block-size table on the sizes the reference asserts (Q4_0 256 -> 144 B, Q4_K 512 -> 288 B, importance quants).
"""
import struct

MAX_STRING_LENGTH = 64 * 1024 * 1024
MAX_ARRAY_ELEMENTS = 4 * 1024 * 1024
MAX_ARRAY_NESTING = 64
MAX_METADATA_KEY_LENGTH = 65535
MAX_TENSOR_NAME_LENGTH = 64
USIZE_MAX = (1 << 64) - 1

# ggml type id -> (elements per block, bytes per block), convert.rs:46-83
QUANT_PARAMS = {
    0: (1, 4), 1: (1, 2), 30: (1, 2), 26: (1, 4), 24: (1, 1), 25: (1, 2), 27: (1, 8), 28: (1, 8),
    2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
    10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
    16: (256, 66), 17: (256, 74), 18: (256, 98), 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82),
    23: (256, 136), 29: (256, 56), 34: (256, 54), 35: (256, 66), 39: (32, 17), 40: (64, 36), 41: (128, 18),
    42: (64, 18),
}


class GGUFError(Exception):
    pass


def _parse_error(offset, msg):
    raise GGUFError(f"parse error at offset {offset}: {msg}")


class _Reader:
    def __init__(self, data):
        self.data = bytes(data)
        self.pos = 0

    def remaining(self):
        return len(self.data) - self.pos

    def take(self, n):
        if self.remaining() < n:
            _parse_error(self.pos, f"need {n} bytes, only {self.remaining()} remain")
        b = self.data[self.pos:self.pos + n]
        self.pos += n
        return b

    def num(self, fmt):
        return struct.unpack("<" + fmt, self.take(struct.calcsize(fmt)))[0]

    def string(self):
        n = self.num("Q")
        if n > MAX_STRING_LENGTH:
            _parse_error(self.pos - 8, f"string length {n} exceeds maximum supported length {MAX_STRING_LENGTH}")
        at = self.pos
        raw = self.take(n)
        try:
            return raw.decode("utf-8")
        except UnicodeDecodeError:
            _parse_error(at, "invalid UTF-8 in string")


_SCALARS = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 10: "Q", 11: "q", 12: "d"}


def _value(r, vtype, depth=0):
    if vtype > 12:
        _parse_error(r.pos, f"unknown GGUF value type: {vtype}")
    if depth > MAX_ARRAY_NESTING:
        _parse_error(r.pos, f"GGUF array nesting exceeds {MAX_ARRAY_NESTING} levels")
    if vtype in _SCALARS:
        return r.num(_SCALARS[vtype])
    if vtype == 7:
        at = r.pos
        b = r.num("B")
        if b > 1:
            _parse_error(at, f"invalid GGUF boolean value {b}; expected 0 or 1")
        return bool(b)
    if vtype == 8:
        return r.string()
    elem = r.num("I")
    if elem > 12:
        _parse_error(r.pos - 4, f"unknown GGUF value type: {elem}")
    count = r.num("Q")
    if count > MAX_ARRAY_ELEMENTS:
        _parse_error(r.pos - 8, f"array element count {count} exceeds maximum {MAX_ARRAY_ELEMENTS}")
    if count > r.remaining():
        _parse_error(r.pos, f"array element count {count} exceeds {r.remaining()} remaining bytes")
    return [_value(r, elem, depth + 1) for _ in range(count)]


def tensor_size(shape, ggml_type):
    """checked_tensor_size: byte size of a tensor with row-major `shape`."""
    if ggml_type not in QUANT_PARAMS:
        raise GGUFError(f"unsupported GGML type: {ggml_type}")
    block, nbytes = QUANT_PARAMS[ggml_type]
    row = shape[-1] if shape else 1
    if row % block:
        raise GGUFError(f"row has {row} elements, not divisible by block size {block}")
    numel = 1
    for d in shape:
        numel *= d
        if numel > USIZE_MAX:
            raise GGUFError("element count overflows usize")
    total = numel // block * nbytes
    if total > USIZE_MAX:
        raise GGUFError("tensor byte size overflows usize")
    return total


def parse(data):
    """GGUFFile::parse -> dict(version, metadata=[(key, type, value)], tensors=[dict], data_start, alignment)."""
    r = _Reader(data)
    if r.take(4) != b"GGUF":
        raise GGUFError("invalid GGUF magic bytes")
    at = r.pos
    vb = r.take(4)
    version = struct.unpack("<I", vb)[0]
    if version not in (2, 3):
        if struct.unpack(">I", vb)[0] in (2, 3):
            _parse_error(at, "big-endian GGUF is not supported by the mmap tensor runtime")
        raise GGUFError(f"unsupported GGUF version: {version}")
    tensor_count = r.num("Q")
    kv_count = r.num("Q")
    need = kv_count * 13 + tensor_count * 24
    if need > USIZE_MAX:
        _parse_error(r.pos, f"tensor count {tensor_count} and metadata count {kv_count} overflow header size")
    if need > r.remaining():
        _parse_error(r.pos, f"tensor count {tensor_count} and metadata count {kv_count} cannot fit in "
                            f"{r.remaining()} remaining bytes")
    metadata, keys = [], set()
    for _ in range(kv_count):
        key = r.string()
        klen = len(key.encode("utf-8"))
        if not key or klen > MAX_METADATA_KEY_LENGTH or not key.isascii():
            _parse_error(r.pos - klen, f"metadata key must be non-empty ASCII and at most {MAX_METADATA_KEY_LENGTH} bytes")
        if key in keys:
            _parse_error(r.pos - klen, f"duplicate metadata key '{key}'")
        keys.add(key)
        vtype = r.num("I")
        metadata.append((key, vtype, _value(r, vtype)))
    alignment = 32
    for key, vtype, value in metadata:
        if key == "general.alignment":
            if vtype not in (0, 1, 2, 3, 4, 5, 10, 11) or value < 0:
                _parse_error(0, "general.alignment must be a non-negative integer fitting usize")
            if value == 0 or value & (value - 1):
                _parse_error(0, f"general.alignment {value} must be a positive power of two")
            alignment = value
            break
    tensors, names = [], set()
    for _ in range(tensor_count):
        name = r.string()
        nlen = len(name.encode("utf-8"))
        if nlen >= MAX_TENSOR_NAME_LENGTH:
            _parse_error(r.pos - nlen, f"tensor name is {nlen} bytes; GGML requires fewer than {MAX_TENSOR_NAME_LENGTH}")
        if name in names:
            _parse_error(r.pos - nlen, f"duplicate tensor name '{name}'")
        names.add(name)
        n_dims = r.num("I")
        if n_dims > 4:
            _parse_error(r.pos - 4, f"tensor '{name}' has {n_dims} dimensions; GGUF supports at most 4")
        shape = [r.num("Q") for _ in range(n_dims)][::-1]
        ggml_type = r.num("I")
        if ggml_type not in QUANT_PARAMS:
            raise GGUFError(f"unsupported GGML type: {ggml_type}")
        offset = r.num("Q")
        if offset % alignment:
            _parse_error(r.pos - 8, f"tensor '{name}' offset {offset} is not aligned to {alignment} bytes")
        tensors.append({"name": name, "shape": shape, "ggml_type": ggml_type, "offset": offset})
    data_start = r.pos + (alignment - r.pos % alignment) % alignment
    if tensor_count > 0 and data_start > len(r.data):
        _parse_error(r.pos, f"tensor data starts at {data_start}, beyond file length {len(r.data)}")
    return {"version": version, "metadata": metadata, "tensors": tensors, "data_start": data_start,
            "alignment": alignment}


def map_tensors(parsed, file_len):
    """map_tensors bounds: name -> (absolute byte offset, byte count)."""
    out = {}
    for t in parsed["tensors"]:
        try:
            nbytes = tensor_size(t["shape"], t["ggml_type"])
        except GGUFError as exc:
            _parse_error(parsed["data_start"], f"tensor '{t['name']}' has invalid shape: {exc}")
        start = parsed["data_start"] + t["offset"]
        if start > USIZE_MAX:
            _parse_error(parsed["data_start"], f"tensor '{t['name']}' absolute offset overflows usize")
        end = start + nbytes
        if end > USIZE_MAX:
            _parse_error(start, f"tensor '{t['name']}' data end overflows usize")
        if end > file_len:
            _parse_error(start, f"tensor '{t['name']}' ends at {end}, beyond file length {file_len}")
        out[t["name"]] = (start, nbytes)
    return out
