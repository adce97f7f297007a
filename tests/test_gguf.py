"""GGUF reader: the product parser (librnb_hip.so, C ABI) against the Python restatement in oracle/gguf_ref.py,
both pinned on the reference's own parser / converter tests restated as byte strings
(crates/rnb-loader/src/gguf/parser.rs:494-717, crates/rnb-loader/src/convert.rs:186-392)."""
import math
import os

import numpy as np
import pytest

import runnburn_amd as rnb
from oracle import gguf_ref
from tests import gguf_writer as gw

U64_MAX = (1 << 64) - 1


def both_parse(data):
    """Parses with the oracle and the product and checks that they agree; returns the oracle's view."""
    ref = gguf_ref.parse(data)
    g = rnb.GGUFFile.parse(data)
    assert g.version == ref["version"] and g.alignment == ref["alignment"] and g.data_start == ref["data_start"]
    assert g.metadata_keys() == [k for k, _, _ in ref["metadata"]]
    for key, vtype, value in ref["metadata"]:
        assert g.metadata_type(key) == vtype
        got = g.metadata(key)
        if vtype == gw.T_ARR and value and isinstance(value[0], list):
            assert len(got) == len(value)
        elif isinstance(value, float):
            assert got == value or (math.isnan(got) and math.isnan(value))
        else:
            assert got == value, (key, got, value)
    assert len(g) == len(ref["tensors"])
    for i, t in enumerate(ref["tensors"]):
        pt = g.tensor_at(i)
        assert (pt.name, pt.shape, pt.ggml_type, pt.offset) == (t["name"], t["shape"], t["ggml_type"], t["offset"])
    g.close()
    return ref


def both_reject(data, fragment):
    with pytest.raises(gguf_ref.GGUFError) as ref:
        gguf_ref.parse(data)
    with pytest.raises(rnb.BackendError) as got:
        rnb.GGUFFile.parse(data)
    assert fragment in str(ref.value), str(ref.value)
    assert str(got.value) == str(ref.value)  # same text, offset included
    assert got.value.kind == "InvalidRequest"


def minimal(arch="llama"):
    return gw.Builder(3, 0, 1).kv("general.architecture", gw.T_STR, arch).pad().build()


def with_tensor(arch="llama"):
    b = gw.Builder(3, 1, 1).kv("general.architecture", gw.T_STR, arch)
    b.tensor_info("token_embd.weight", [4, 8], 0, 0).pad().raw(bytes(128))
    return b.build()


# ---- the reference's accepted files -----------------------------------------------------------

def test_minimal_v3():
    ref = both_parse(minimal())
    assert ref["version"] == 3 and ref["tensors"] == []
    assert ref["metadata"] == [("general.architecture", gw.T_STR, "llama")]
    assert ref["data_start"] % 32 == 0


def test_tensor_info_dimensions_are_reversed_to_row_major():
    ref = both_parse(with_tensor())
    assert ref["tensors"] == [{"name": "token_embd.weight", "shape": [8, 4], "ggml_type": 0, "offset": 0}]


def test_standard_64_bit_metadata():
    b = gw.Builder(3, 0, 3).kv("test.uint64", gw.T_U64, U64_MAX - 7).kv("test.int64", gw.T_I64, -1_234_567_890_123)
    ref = both_parse(b.kv("test.float64", gw.T_F64, math.pi).build())
    assert [v for _, _, v in ref["metadata"]] == [U64_MAX - 7, -1_234_567_890_123, math.pi]


def test_every_scalar_type_and_arrays_round_trip():
    b = gw.Builder(3, 0, 12)
    b.kv("a.u8", gw.T_U8, 200).kv("a.i8", gw.T_I8, -100).kv("a.u16", gw.T_U16, 65000).kv("a.i16", gw.T_I16, -30000)
    b.kv("a.u32", gw.T_U32, 4_000_000_000).kv("a.i32", gw.T_I32, -2_000_000_000).kv("a.f32", gw.T_F32, 0.5)
    b.kv("a.bool", gw.T_BOOL, 1).kv("a.str", gw.T_STR, "héllo")
    b.kv("a.tokens", gw.T_ARR, ["<s>", "</s>", "ÿ"], gw.T_STR).kv("a.ints", gw.T_ARR, [1, -2, 3], gw.T_I32)
    b.kv("a.floats", gw.T_ARR, [0.25, -8.0], gw.T_F32)
    ref = both_parse(b.build())
    assert ref["metadata"][8][2] == "héllo" and ref["metadata"][9][2] == ["<s>", "</s>", "ÿ"]


def test_version_2_and_custom_alignment():
    b = gw.Builder(2, 1, 1).kv("general.alignment", gw.T_U32, 64).tensor_info("w", [32], 8, 128).pad(64)
    ref = both_parse(b.raw(bytes(128 + 34)).build())
    assert ref["version"] == 2 and ref["alignment"] == 64 and ref["data_start"] % 64 == 0


# ---- the reference's rejections, message fragments from its tests ----------------------------------

def test_invalid_magic():
    both_reject(b"XXXX\x03\x00\x00\x00" + bytes(16), "invalid GGUF magic bytes")


def test_unsupported_version():
    both_reject(gw.Builder(1, 0, 0).build(), "unsupported GGUF version: 1")


def test_big_endian_is_named():
    both_reject(gw.Builder(3, 0, 0, big_endian=True).build(), "big-endian")


@pytest.mark.parametrize("build,fragment", [
    (lambda: gw.Builder(3, 0, 1).string("test.bool").num("I", 7).num("B", 2), "boolean"),
    (lambda: gw.Builder(3, 0, 1).kv("general.alignment", gw.T_U32, 24), "power of two"),
    (lambda: gw.Builder(3, 0, 1).kv("general.alignment", gw.T_U32, 12), "alignment"),
    (lambda: gw.Builder(3, 0, 1).kv("general.alignment", gw.T_U32, 0), "power of two"),
    (lambda: gw.Builder(3, 0, 1).kv("general.alignment", gw.T_I32, -32), "non-negative integer"),
    (lambda: gw.Builder(3, 0, 1).kv("general.alignment", gw.T_F32, 32.0), "non-negative integer"),
    (lambda: gw.Builder(3, 0, U64_MAX), "metadata count"),
    (lambda: gw.Builder(3, 0, 1_000_000), "cannot fit"),
    (lambda: gw.Builder(3, 0, 1).string("test.string").num("I", 8).num("Q", gguf_ref.MAX_STRING_LENGTH + 1),
     "string length"),
    (lambda: gw.Builder(3, 0, 1).string("test.array").num("I", 9).num("I", 0).num("Q", gguf_ref.MAX_ARRAY_ELEMENTS + 1),
     "array element count"),
    (lambda: gw.Builder(3, 0, 1).string("test.array").num("I", 9).num("I", 0).num("Q", 1000).raw(bytes(10)),
     "remaining bytes"),
    (lambda: gw.Builder(3, 0, 1).string("test.array").num("I", 9).num("I", 99).num("Q", 0), "unknown GGUF value type"),
    (lambda: gw.Builder(3, 0, 1).string("test.value").num("I", 13), "unknown GGUF value type"),
    (lambda: gw.Builder(3, 0, 2).kv("test.key", gw.T_U8, 1).kv("test.key", gw.T_U8, 2), "duplicate metadata key"),
    (lambda: gw.Builder(3, 0, 1).kv("", gw.T_U8, 1), "metadata key must be non-empty ASCII"),
    (lambda: gw.Builder(3, 0, 1).kv("clé", gw.T_U8, 1), "metadata key must be non-empty ASCII"),
    (lambda: gw.Builder(3, 0, 1).string(b"\xff\xfe").num("I", 0).num("B", 1), "invalid UTF-8"),
    (lambda: gw.Builder(3, 2, 0).tensor_info("duplicate.weight", [1], 0, 0).tensor_info("duplicate.weight", [1], 0, 32),
     "duplicate tensor name"),
    (lambda: gw.Builder(3, 1, 0).tensor_info("x" * 64, [1], 0, 0), "tensor name"),
    (lambda: gw.Builder(3, 1, 0).string("five.dims").num("I", 5).raw(bytes(64)), "at most 4"),
    (lambda: gw.Builder(3, 1, 0).tensor_info("odd.type", [1], 99, 0), "unsupported GGML type: 99"),
    (lambda: gw.Builder(3, 1, 0).tensor_info("odd.offset", [1], 0, 16), "is not aligned to 32 bytes"),
    (lambda: gw.Builder(3, 0, 1).string("cut.short").num("I", 10).raw(b"\x01\x02"), "need 8 bytes, only 2 remain"),
])
def test_rejections(build, fragment):
    both_reject(build().build(), fragment)


def test_nesting_limit():
    b = gw.Builder(3, 0, 1).string("deep").num("I", 9)
    for _ in range(70):
        b.num("I", 9).num("Q", 1)
    both_reject(b.raw(bytes(64)).build(), "nesting exceeds 64 levels")


def test_name_of_63_bytes_is_accepted():
    both_parse(gw.Builder(3, 1, 0).tensor_info("y" * 63, [1], 0, 0).pad().raw(bytes(4)).build())


# ---- tensor sizes and payload bounds (convert.rs) ------------------------------------------------------

@pytest.mark.parametrize("shape,ggml_type,expected", [
    ([4, 4], 0, 64), ([4, 4], 26, 64), ([4, 4], 1, 32), ([256], 2, 144), ([512], 12, 288), ([8, 4], 0, 128),
    ([256], 16, 66), ([256], 17, 74), ([256], 18, 98), ([256], 19, 50), ([256], 21, 110), ([256], 22, 82),
    ([256], 23, 136), ([256], 29, 56), ([256], 14, 210), ([14336, 4096], 12, 33030144), ([4096, 4096], 8, 17825792),
    ([128, 768, 2048], 12, 113246208), ([], 0, 4),
])
def test_tensor_sizes(shape, ggml_type, expected):
    assert gguf_ref.tensor_size(shape, ggml_type) == expected
    assert rnb.gguf_tensor_size(shape, ggml_type) == expected


def test_tensor_size_errors():
    for shape, t, frag in [([31], 2, "not divisible by block size 32"), ([3, 100], 12, "block size 256"),
                           ([1 << 40, 1 << 40], 0, "element count overflows usize"), ([4], 99, "unsupported GGML type")]:
        with pytest.raises(gguf_ref.GGUFError) as ref:
            gguf_ref.tensor_size(shape, t)
        with pytest.raises(rnb.BackendError) as got:
            rnb.gguf_tensor_size(shape, t)
        assert frag in str(ref.value) and str(got.value) == str(ref.value)


def test_map_tensors_bounds(tmp_path):
    data = with_tensor()
    ref = gguf_ref.parse(data)
    assert gguf_ref.map_tensors(ref, len(data)) == {"token_embd.weight": (ref["data_start"], 128)}
    g = rnb.GGUFFile.parse(data)
    g.map_tensors()
    t = g.tensor_at(0)
    assert (t.file_offset, t.n_bytes, t.data.size) == (ref["data_start"], 128, 128)
    g.close()
    # one byte short: the header still parses, map_tensors refuses (convert.rs:283-298)
    cut = data[:-1]
    ref = gguf_ref.parse(cut)
    with pytest.raises(gguf_ref.GGUFError) as e_ref:
        gguf_ref.map_tensors(ref, len(cut))
    g = rnb.GGUFFile.parse(cut)
    with pytest.raises(rnb.BackendError) as e_got:
        g.map_tensors()
    assert "beyond file length" in str(e_ref.value) and str(e_got.value) == str(e_ref.value)
    with pytest.raises(rnb.BackendError):
        g.tensor_at(0).data
    g.close()
    # and opening the truncated file from disk fails the same way
    p = tmp_path / "cut.gguf"
    p.write_bytes(cut)
    with pytest.raises(rnb.BackendError) as e_open:
        rnb.GGUFFile(str(p))
    assert str(e_open.value) == str(e_ref.value)


def test_map_tensors_rejects_row_not_divisible_by_block():
    b = gw.Builder(3, 1, 1).kv("general.architecture", gw.T_STR, "llama").tensor_info("test.weight", [31], 2, 0)
    data = b.pad().raw(bytes(18)).build()
    ref = gguf_ref.parse(data)
    with pytest.raises(gguf_ref.GGUFError) as e_ref:
        gguf_ref.map_tensors(ref, len(data))
    g = rnb.GGUFFile.parse(data)
    with pytest.raises(rnb.BackendError) as e_got:
        g.map_tensors()
    assert "block size" in str(e_ref.value) and str(e_got.value) == str(e_ref.value)
    g.close()


def test_open_missing_file_and_lookup_errors(tmp_path):
    with pytest.raises(rnb.BackendError) as e:
        rnb.GGUFFile(str(tmp_path / "absent.gguf"))
    assert e.value.kind == "ExecutionFailed" and str(e.value).startswith("I/O error:")
    g = rnb.GGUFFile.parse(with_tensor())
    with pytest.raises(rnb.BackendError) as e:
        g.tensor("nope")
    assert str(e.value) == "missing tensor: nope"
    with pytest.raises(rnb.BackendError) as e:
        g.metadata("nope")
    assert str(e.value) == "missing metadata key: nope"
    with pytest.raises(rnb.BackendError) as e:
        g.tensor_at(5)
    assert "out of range" in str(e.value)
    g.close()


def test_file_with_quantised_tensors_maps_untouched_bytes(tmp_path):
    """A model-shaped file: the bytes seen through the reader are the bytes written, at the offsets the oracle computes."""
    from oracle import oracle as o
    rows, cols = 6, 512
    w4 = o.make_weights(o.Q4_K, rows, cols, 1)
    w6 = o.make_weights(o.Q6_K, rows, cols, 2)
    w8 = o.make_weights(o.Q8_0, rows, cols, 3)
    norm = np.arange(cols, dtype=np.float32).view(np.uint8)
    path = str(tmp_path / "m.gguf")
    offs = gw.write_model(path, [("general.architecture", gw.T_STR, "llama"), ("llama.block_count", gw.T_U32, 1)],
                          [("blk.0.ffn_gate.weight", [rows, cols], 12, w4), ("blk.0.ffn_down.weight", [rows, cols], 14, w6),
                           ("output.weight", [rows, cols], 8, w8), ("output_norm.weight", [cols], 0, norm)])
    raw = open(path, "rb").read()
    ref = gguf_ref.parse(raw)
    mapped = gguf_ref.map_tensors(ref, len(raw))
    with rnb.GGUFFile(path) as g:
        assert g.metadata("general.architecture") == "llama" and g.metadata("llama.block_count") == 1
        for name, src in [("blk.0.ffn_gate.weight", w4), ("blk.0.ffn_down.weight", w6), ("output.weight", w8),
                          ("output_norm.weight", norm)]:
            t = g.tensor(name)
            assert (t.file_offset, t.n_bytes) == mapped[name] == (offs[name], src.size)
            assert t.file_offset % g.alignment == 0
            assert np.array_equal(t.data, src)
        assert g.tensor("blk.0.ffn_gate.weight").shape == [rows, cols]


# ---- split files: crates/rnb-loader/src/gguf/sharded.rs -------------------------------------------------------------------

def _shard(shard_no, shard_count, total_tensors, tensor_name, value, no_type=gw.T_U16, extra=(), count_type=gw.T_U16):
    """make_split_shard of sharded.rs:245-274: architecture, the three split keys, one F32 tensor of one element."""
    md = [("general.architecture", gw.T_STR, "llama")]
    if shard_no is not None:
        md.append(("split.no", no_type, shard_no))
    if shard_count is not None:
        md.append(("split.count", count_type, shard_count))
    if total_tensors is not None:
        md.append(("split.tensors.count", gw.T_U64, total_tensors))
    b = gw.Builder(3, 1 + len(extra), len(md))
    for item in md:
        b.kv(*item)
    b.tensor_info(tensor_name, [1], 0, 0)
    for i, name in enumerate(extra):
        b.tensor_info(name, [1], 0, 32 * (i + 1))
    b.pad(32)
    b.raw(np.float32(value).tobytes())
    for i, _ in enumerate(extra):
        b.pad(32)
        b.raw(np.float32(value + i + 1).tobytes())
    return b.build()


def test_single_file_keeps_the_direct_path(tmp_path):
    """sharded.rs:277-288: no split keys, one tensor."""
    path = tmp_path / "model.gguf"
    path.write_bytes(with_tensor())
    with rnb.GGUFFile(str(path)) as g:
        assert len(g) == 1 and g.tensor_at(0).name == "token_embd.weight"


@pytest.mark.parametrize("selected", [0, 1, 2])
def test_split_file_maps_every_shard_from_any_of_its_paths(tmp_path, selected):
    """sharded.rs:290-311 (from the first path) and the same from the other shards: the handle shows all tensors, each
    with the bytes of its own shard, and the metadata of shard zero."""
    names = ["first.weight", "second.weight", "third.weight"]
    values = [1.25, -2.5, 7.0]
    for i in range(3):
        data = _shard(i, 3, 3, names[i], values[i])
        (tmp_path / f"model-0000{i + 1}-of-00003.gguf").write_bytes(data)
    with rnb.GGUFFile(str(tmp_path / f"model-0000{selected + 1}-of-00003.gguf")) as g:
        assert len(g) == 3
        assert [t.name for t in g.tensors()] == names  # shard order
        for name, v in zip(names, values):
            t = g.tensor(name)
            assert t.n_bytes == 4 and bytes(t.data) == np.float32(v).tobytes()
        assert g.metadata("split.no") == 0 and g.metadata("general.architecture") == "llama"
        g.map_tensors()  # each tensor is checked against its own shard's length


def test_split_file_rejections(tmp_path):
    """Every check of load_mapped_gguf / validate_shard / resolve_shard_paths with its message text
    (`parse error at offset 0: invalid split GGUF: ...`)."""
    def write(name, data):
        (tmp_path / name).write_bytes(data)
        return str(tmp_path / name)

    def rejected(path, fragment):
        with pytest.raises(rnb.BackendError) as e:
            rnb.GGUFFile(path)
        assert e.value.kind == "InvalidRequest"
        assert str(e.value).startswith("parse error at offset 0: invalid split GGUF: ") and fragment in str(e.value), str(e.value)

    # a missing shard is named (sharded.rs:313-328)
    first = write("model-00001-of-00002.gguf", _shard(0, 2, 2, "first.weight", 1.25))
    rejected(first, "model-00002-of-00002.gguf")
    rejected(write("a-00001-of-00002.gguf", _shard(0, 0, 2, "w", 1.0)), "split.count must be positive")
    rejected(write("b-00001-of-00002.gguf", _shard(None, 2, 2, "w", 1.0)), "missing metadata key split.no")
    rejected(write("c-00001-of-00002.gguf", _shard(0, 2, None, "w", 1.0)), "missing metadata key split.tensors.count")
    rejected(write("d-00001-of-00002.gguf", _shard(2, 2, 2, "w", 1.0)), "split.no 2 is outside split.count 2")
    rejected(write("e-00001-of-00002.gguf", _shard(-1, 2, 2, "w", 1.0, no_type=gw.T_I16)),
             "metadata key split.no must be a non-negative integer")
    rejected(write("f-00001-of-00002.gguf", _shard("0", 2, 2, "w", 1.0, no_type=gw.T_STR)),
             "metadata key split.no must be a non-negative integer")
    # file names
    rejected(write("model-00001-of-00002.bin", _shard(0, 2, 2, "w", 1.0)), "split GGUF file name must end in .gguf")
    rejected(write("model.gguf", _shard(0, 2, 2, "w", 1.0)), "split GGUF file name must end in -00001-of-00001.gguf")
    rejected(write("00001-of-00002.gguf", _shard(0, 2, 2, "w", 1.0)), "split GGUF file name is missing its shard index")
    rejected(write("model-0000x-of-00002.gguf", _shard(0, 2, 2, "w", 1.0)), "split GGUF file name has an invalid shard suffix")
    rejected(write("-00001-of-00002.gguf", _shard(0, 2, 2, "w", 1.0)), "split GGUF file name has an invalid shard suffix")
    rejected(write("g-00002-of-00002.gguf", _shard(0, 2, 2, "w", 1.0)),
             "file name declares shard 2 of 2, metadata declares shard 1 of 2")
    rejected(write("h-00001-of-00003.gguf", _shard(0, 2, 2, "w", 1.0)),
             "file name declares shard 1 of 3, metadata declares shard 1 of 2")
    # the other shard disagrees with the selected one
    write("i-00001-of-00002.gguf", _shard(0, 2, 2, "w0", 1.0))
    write("i-00002-of-00002.gguf", _shard(0, 2, 2, "w1", 1.0))
    rejected(str(tmp_path / "i-00001-of-00002.gguf"), "expected shard 1, but its metadata declares split.no 0")
    write("j-00001-of-00002.gguf", _shard(0, 2, 2, "w0", 1.0))
    write("j-00002-of-00002.gguf", _shard(1, 3, 2, "w1", 1.0))
    rejected(str(tmp_path / "j-00001-of-00002.gguf"), "shard 1 declares split.count 3, expected 2")
    write("k-00001-of-00002.gguf", _shard(0, 2, 2, "w0", 1.0))
    write("k-00002-of-00002.gguf", _shard(1, 2, 5, "w1", 1.0))
    rejected(str(tmp_path / "k-00001-of-00002.gguf"), "shard 1 declares split.tensors.count 5, expected 2")
    write("l-00001-of-00002.gguf", _shard(0, 2, 2, "same.weight", 1.0))
    write("l-00002-of-00002.gguf", _shard(1, 2, 2, "same.weight", 2.0))
    rejected(str(tmp_path / "l-00001-of-00002.gguf"), "tensor 'same.weight' appears in more than one shard")
    write("m-00001-of-00002.gguf", _shard(0, 2, 3, "w0", 1.0))
    write("m-00002-of-00002.gguf", _shard(1, 2, 3, "w1", 1.0))
    rejected(str(tmp_path / "m-00001-of-00002.gguf"), "split.tensors.count declares 3 tensors but 2 were loaded")
    # a count no set of files can have: refused at the first missing file, without a list of that many names
    huge = 2 ** 64 - 1
    rejected(write(f"o-00001-of-{huge}.gguf", _shard(0, huge, 2, "w", 1.0, count_type=gw.T_U64)), f"o-00002-of-{huge}.gguf")
    # a shard that does not parse is named with its own error
    write("n-00001-of-00002.gguf", _shard(0, 2, 2, "w0", 1.0))
    write("n-00002-of-00002.gguf", b"GGUX" + bytes(60))
    rejected(str(tmp_path / "n-00001-of-00002.gguf"), "n-00002-of-00002.gguf': invalid GGUF magic bytes")


def test_split_file_index_widths_follow_the_selected_name(tmp_path):
    """resolve_shard_paths keeps the digit widths of the selected file's name (sharded.rs:223-234)."""
    (tmp_path / "m-1-of-2.gguf").write_bytes(_shard(0, 2, 2, "a", 1.0))
    (tmp_path / "m-2-of-2.gguf").write_bytes(_shard(1, 2, 2, "b", 2.0))
    with rnb.GGUFFile(str(tmp_path / "m-2-of-2.gguf")) as g:
        assert [t.name for t in g.tensors()] == ["a", "b"]


@pytest.mark.gpu
def test_gguf_tensors_run_from_the_untouched_upload(rnb, oracle, tmp_path):
    """File -> reader -> prewarm (upload as stored) -> GEMV / MoE on the mapped bytes == oracle on the same bytes."""
    o = oracle
    rows, cols = 40, 1024
    w4 = o.make_weights(o.Q4_K, rows, cols, 11)
    w6 = o.make_weights(o.Q6_K, rows, cols, 12)
    w8 = o.make_weights(o.Q8_0, rows, cols, 13)
    n_expert, n_ff, n_embd = 4, 256, 512
    gate = o.make_weights(o.Q4_K, n_expert * n_ff, n_embd, 21)
    up = o.make_weights(o.Q4_K, n_expert * n_ff, n_embd, 22)
    down = o.make_weights(o.Q6_K, n_expert * n_embd, n_ff, 23)
    path = str(tmp_path / "model.gguf")
    gw.write_model(path, [("general.architecture", gw.T_STR, "qwen3moe")],
                   [("blk.0.ffn_up.weight", [rows, cols], 12, w4), ("blk.0.ffn_down.weight", [rows, cols], 14, w6),
                    ("output.weight", [rows, cols], 8, w8),
                    ("blk.0.ffn_gate_exps.weight", [n_expert, n_ff, n_embd], 12, gate),
                    ("blk.0.ffn_up_exps.weight", [n_expert, n_ff, n_embd], 12, up),
                    ("blk.0.ffn_down_exps.weight", [n_expert, n_embd, n_ff], 14, down)])
    x = o.fill_normal(cols, 31, 1.0)
    with rnb.GGUFFile(path) as g:
        before = rnb.resident_bytes()[0]
        for t in g.tensors():
            t.prewarm()
        assert rnb.resident_bytes()[0] - before >= sum(t.n_bytes for t in g.tensors())
        up_before = rnb.transfer_counters()[0]
        for name, fn, q, src in [("blk.0.ffn_up.weight", rnb.q4k_gemv, o.Q4_K, w4),
                                 ("blk.0.ffn_down.weight", rnb.q6k_gemv, o.Q6_K, w6),
                                 ("output.weight", rnb.q8_0_gemv, o.Q8_0, w8)]:
            t = g.tensor(name)
            got = fn(t.data, t.shape[0], t.shape[1], x)
            ref = o.gemv(q, src, rows, cols, x)[0]
            assert np.allclose(got, ref, rtol=1e-3, atol=1e-3 * np.abs(ref).max()), name
        # the weights were already resident: only activations went up
        assert rnb.transfer_counters()[0] - up_before < 3 * (cols * 4 + 4096)
        # one expert of a stacked tensor = a sub-range of the pinned upload (fanout.rs:4-22 slicing)
        tg, tu, td = (g.tensor(f"blk.0.ffn_{k}_exps.weight") for k in ("gate", "up", "down"))
        assert tg.shape == [n_expert, n_ff, n_embd] and td.shape == [n_expert, n_embd, n_ff]
        ids = np.array([2, 0, 3], np.uint32)
        route = np.array([0.5, 0.3, 0.2], np.float32)
        toks = np.zeros(3, np.uint32)
        h = o.fill_normal(n_embd, 41, 1.0)
        got = rnb.qwen35_sparse_experts_selected_base_by_token(tg.data, tu.data, td.data, ids, route, toks, 1, o.Q6_K,
                                                               n_ff, n_embd, h)
        ref = o.moe_sparse_experts_by_token(gate, up, down, n_expert, ids, route, toks, 1, o.Q6_K, n_ff, n_embd, h)
        assert np.allclose(got, ref, rtol=1e-3, atol=1e-3 * np.abs(ref).max())
        for t in g.tensors():
            rnb.release(t.data)


def test_reader_survives_mutated_files_under_sanitizers(tmp_path):
    """tests/cpp/gguf_fuzz (built by __graft_entry__.build with the address and undefined-behaviour sanitizers on the
    host side): damaged copies of a valid file, every accessor exercised on what the parser accepts; then sets of shard
    files, consistent (must open from every shard with every tensor's own value) or damaged in one place (a split key's
    type or value, a missing key, a tensor name in two shards, a wrong total, a truncated shard)."""
    import subprocess

    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "gguf_fuzz")
    if not os.path.exists(exe):
        pytest.skip("tests/cpp/gguf_fuzz not built (run __graft_entry__.build())")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1")
    p = subprocess.run([exe, "60000", str(tmp_path)], capture_output=True, text=True, timeout=300, env=env)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-4000:]
    assert p.stdout.count("0 failure(s)") == 2, p.stdout[-2000:]


@pytest.mark.gpu
def test_split_model_tensors_upload_from_their_own_shard(rnb, oracle, tmp_path):
    """Two shards with one quantised matrix each, of different file lengths: prewarm + GEMV on the tensor of either shard,
    opened through the second shard's path, equals the oracle on that shard's bytes."""
    o = oracle
    mats = [(o.make_weights(o.Q4_K, 24, 512, 51), 24, 512, 12, o.Q4_K), (o.make_weights(o.Q6_K, 56, 1024, 52), 56, 1024, 14, o.Q6_K)]
    for no, (w, rows, cols, ggml_type, _) in enumerate(mats):
        md = [("general.architecture", gw.T_STR, "llama"), ("split.no", gw.T_U16, no), ("split.count", gw.T_U16, 2),
              ("split.tensors.count", gw.T_I32, 2)]
        gw.write_model(str(tmp_path / f"m-0000{no + 1}-of-00002.gguf"), md, [(f"blk.{no}.weight", [rows, cols], ggml_type, w)])
    with rnb.GGUFFile(str(tmp_path / "m-00002-of-00002.gguf")) as g:
        assert [t.name for t in g.tensors()] == ["blk.0.weight", "blk.1.weight"]
        for no, (w, rows, cols, _, q) in enumerate(mats):
            t = g.tensor(f"blk.{no}.weight")
            assert bytes(t.data) == w.tobytes()
            t.prewarm()
            x = o.fill_normal(cols, 60 + no, 1.0)
            got = (rnb.q4k_gemv if q == o.Q4_K else rnb.q6k_gemv)(t.data, rows, cols, x)
            ref = o.gemv(q, w, rows, cols, x)[0]
            assert np.allclose(got, ref, rtol=1e-3, atol=1e-3 * np.abs(ref).max())
