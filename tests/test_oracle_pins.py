"""Pins the CPU oracle WITHOUT running the reference (Rust; no toolchain here): every check is
either a known-answer vector held by the reference's own unit tests (cited per test), or an
independent numpy statement of the public format / a mathematical identity, chosen so that a
dropped term, wrong shift or transposed index fails."""
import math

import numpy as np
import pytest

from tests import npref

Q4_0, Q4_1, Q5_0, Q5_1, Q8_1 = 2, 3, 6, 7, 9
NIBBLE_FORMATS = (Q4_0, Q4_1, Q5_0, Q5_1)
LEGACY = NIBBLE_FORMATS
Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 8, 10, 11, 12, 13, 14


# ---- f16 ----------------------------------------------------------------------------

def test_f16_to_f32_all_bit_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_round_to_nearest_even(oracle):
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(0.02),
        rng.standard_normal(5000).astype(np.float32) * np.float32(1e-6),   # f16 subnormals / underflow
        rng.standard_normal(5000).astype(np.float32) * np.float32(3e4),    # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.9802322e-8,
                  6.1035156e-5, 6.0975552e-5, 1.0009766, 1.00048828125, 1.00146484375], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    # raw constants the reference's tests write by hand (quant_gemv.rs:1226-1227, 1451)
    assert oracle.f16_to_f32(0x3C00) == 1.0 and oracle.f16_to_f32(0x3800) == 0.5


# ---- 6-bit scale/min unpack -----------------------------------------------------------

def test_get_scale_min_k4_known_vector(oracle):
    # bytes used by crates/rnb-backend/cuda/src/runtime/tests.rs:12494, decoded by hand from
    # the format: j<4 low six bits; j>=4 low nibble / high nibble of byte j+4 plus top two bits.
    q = [3, 5, 7, 11, 13, 17, 19, 23, 0x21, 0x43, 0x65, 0x07]
    want = [(3, 13), (5, 17), (7, 19), (11, 23), (1, 2), (3, 4), (5, 6), (7, 0)]
    assert [oracle.get_scale_min_k4(j, q) for j in range(8)] == want
    # with top bits set: byte0 = 0xC3 -> scale4 gets (3<<4), byte4 = 0x8D -> min4 gets (2<<4)
    q2 = [0xC3, 5, 7, 11, 0x8D, 17, 19, 23, 0x21, 0x43, 0x65, 0x07]
    assert oracle.get_scale_min_k4(0, q2) == (3, 13)
    assert oracle.get_scale_min_k4(4, q2) == (1 | (3 << 4), 2 | (2 << 4))


def test_get_scale_min_k4_roundtrip_all_positions(oracle):
    rng = np.random.default_rng(2)
    for _ in range(200):
        sc = rng.integers(0, 64, 8)
        mn = rng.integers(0, 64, 8)
        q = npref.pack_scales_k4(sc, mn)
        got = [oracle.get_scale_min_k4(j, q) for j in range(8)]
        assert got == list(zip(sc.tolist(), mn.tolist()))


def test_nearest_int_is_round_half_even(oracle):
    for v, want in [(0.5, 0), (1.5, 2), (2.5, 2), (-0.5, 0), (-1.5, -2), (-2.5, -2), (3.49, 3), (-3.51, -4),
                    (4194303.0, 4194303), (-4194303.0, -4194303)]:
        assert oracle.nearest_int(v) == want


# ---- dequantisers: element order and arithmetic ------------------------------------------

def _random_q4k(rng, n):
    blocks = []
    for _ in range(n):
        blocks.append(npref.make_q4k_block(rng.uniform(1e-4, 5e-3), rng.uniform(1e-4, 5e-3),
                                           rng.integers(0, 64, 8), rng.integers(0, 64, 8),
                                           rng.integers(0, 16, 256)))
    return np.concatenate(blocks)


def _random_legacy(quant, rng, n):
    top = 32 if quant in (Q5_0, Q5_1) else 16
    return np.concatenate([npref.make_legacy_block(quant, rng.uniform(-1e-2, 1e-2), rng.uniform(-0.1, 0.1),
                                                   rng.integers(0, top, 32)) for _ in range(n)])


def _random_q2k(rng, n):
    return np.concatenate([npref.make_q2k_block(rng.uniform(1e-4, 5e-3), rng.uniform(1e-4, 5e-3), rng.integers(0, 16, 16),
                                                rng.integers(0, 16, 16), rng.integers(0, 4, 256)) for _ in range(n)])


def _random_q3k(rng, n):
    return np.concatenate([npref.make_q3k_block(rng.uniform(-5e-3, 5e-3), rng.integers(-32, 32, 16),
                                                rng.integers(-4, 4, 256)) for _ in range(n)])


def _random_q5k(rng, n):
    blocks = []
    for _ in range(n):
        blocks.append(npref.make_q5k_block(rng.uniform(1e-4, 5e-3), rng.uniform(1e-4, 5e-3),
                                           rng.integers(0, 64, 8), rng.integers(0, 64, 8),
                                           rng.integers(0, 32, 256)))
    return np.concatenate(blocks)


def _random_q6k(rng, n):
    blocks = []
    for _ in range(n):
        blocks.append(npref.make_q6k_block(rng.uniform(-5e-4, 5e-4), rng.integers(-128, 128, 16),
                                           rng.integers(0, 64, 256)))
    return np.concatenate(blocks)


def _random_q8_0(rng, n):
    return np.concatenate([npref.make_q8_0_block(rng.uniform(1e-4, 1e-2), rng.integers(-128, 128, 32))
                           for _ in range(n)])


def test_dequantize_q4k_places_each_nibble(oracle):
    # one-hot: a single nibble set -> exactly one output differs from the "-dmin*mn" background
    for elem in [0, 31, 32, 63, 64, 100, 255]:
        nib = np.zeros(256, dtype=np.uint8)
        nib[elem] = 9
        blk = npref.make_q4k_block(1.0, 0.0, np.arange(1, 9), np.zeros(8), nib)
        y = oracle.dequantize(Q4_K, blk)
        want = np.zeros(256, dtype=np.float32)
        want[elem] = 9.0 * (elem // 32 + 1)
        assert np.array_equal(y, want)
    rng = np.random.default_rng(3)
    blocks = _random_q4k(rng, 64)
    got = oracle.dequantize(Q4_K, blocks).astype(np.float64)
    want = npref.dequant_q4k_f64(blocks)
    assert np.allclose(got, want, rtol=0, atol=1e-7 * np.abs(want).max() * 4)


def test_q8_1_dequant_and_dot(oracle):
    """Q8_1 {f16 d, f16 s, i8 qs[32]}: crates/rnb-cpu/src/gemm/quant_gemv.rs:210-216 (element = d * q) and
    neon_quant.rs:236-253 (dot = d * d_x * sum(q * a); "the stored Q8_1 sum is not needed").  The reference holds no
    known-answer test for this format; pinned by hand-built bytes (every element position, s ignored), the closed
    form on constant vectors and the f64 identity against an independent numpy dequantiser."""
    q = (np.arange(32) * 7 % 255 - 127).astype(np.int8)
    blk = npref.make_q8_1_block(0.5, 123.0, q)
    assert blk.size == 36
    assert np.array_equal(oracle.dequantize(Q8_1, blk), q.astype(np.float32) * np.float32(0.5))
    assert np.array_equal(oracle.dequantize(Q8_1, npref.make_q8_1_block(0.5, -7.0, q)), oracle.dequantize(Q8_1, blk))
    for e in (0, 1, 15, 16, 31):
        one = np.zeros(32, np.int8)
        one[e] = -128
        want = np.zeros(32, np.float32)
        want[e] = -256.0
        assert np.array_equal(oracle.dequantize(Q8_1, npref.make_q8_1_block(2.0, 0.0, one)), want), e
    a = (np.arange(32) % 9 - 4).astype(np.int8)
    act = _q8_act(0.25, a)
    assert oracle.dot(Q8_1, npref.make_q8_1_block(2.0, 99.0, np.full(32, 3)), act) == 2.0 * 0.25 * 3 * float(a.astype(np.int64).sum())
    assert oracle.dot(Q8_1, blk, act) == 0.5 * 0.25 * float(np.dot(q.astype(np.int64), a.astype(np.int64)))
    rng = np.random.default_rng(69)
    for nb in (1, 3, 128):
        row = np.concatenate([npref.make_q8_1_block(rng.uniform(-1e-2, 1e-2), rng.uniform(-1, 1), rng.integers(-128, 128, 32))
                              for _ in range(nb)])
        x = rng.standard_normal(nb * 32).astype(np.float32)
        xa = oracle.quantize_q8(x)
        xq = (xa["d"].astype(np.float64)[:, None] * xa["qs"].astype(np.float64)).reshape(-1)
        want = float(np.dot(npref.dequant_q8_1_f64(row), xq))
        assert oracle.dot(Q8_1, row, xa, gold=True) == pytest.approx(want, rel=1e-11, abs=1e-12)
        assert abs(oracle.dot(Q8_1, row, xa) - want) <= 4e-7 * float(np.sum(np.abs(npref.dequant_q8_1_f64(row) * xq)))
    # the generator (ggml semantics, input generation only): round trip and the stored sum
    xw = oracle.fill_normal(32 * 200, 26, 0.02)
    w = oracle.quantize_row(Q8_1, xw)
    y = oracle.dequantize(Q8_1, w)
    assert np.sqrt(np.mean((xw - y) ** 2)) / np.sqrt(np.mean(xw ** 2)) < 0.01
    b = w.reshape(-1, 36)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
    ssum = b[:, 4:].copy().view(np.int8).astype(np.int64).sum(axis=1)
    assert np.allclose(b[:, 2:4].copy().view(np.float16).astype(np.float32).reshape(-1), d * ssum, rtol=2e-3, atol=1e-6)
    rows, cols = 3, 96
    wm = oracle.make_weights(Q8_1, rows, cols, 7)
    xs = oracle.fill_normal(2 * cols, 8, 1.0).reshape(2, cols)
    out = oracle.gemv(Q8_1, wm, rows, cols, xs)
    for si in range(2):
        xa = oracle.quantize_q8(xs[si])
        for r in range(rows):
            assert out[si, r] == np.float32(oracle.dot(Q8_1, wm[r * 108:(r + 1) * 108], xa))


@pytest.mark.parametrize("quant", NIBBLE_FORMATS)
def test_dequantize_legacy_formats_place_every_field(oracle, quant):
    """crates/rnb-cpu/src/quantize/dequant.rs:7-53 against hand-built bytes: one nibble, one high bit at a time."""
    nbytes, has_min, has_qh = npref.LEGACY_LAYOUT[quant]
    qs_off = 2 + (2 if has_min else 0) + (4 if has_qh else 0)
    offset = 0 if has_min else (16 if has_qh else 8)
    base = np.zeros(nbytes, np.uint8)
    base[0:2] = np.frombuffer(npref.f16_bytes(2.0), np.uint8)
    if has_min:
        base[2:4] = np.frombuffer(npref.f16_bytes(0.5), np.uint8)
    background = 0.5 if has_min else -2.0 * offset
    for i in (0, 7, 15):
        blk = base.copy()
        blk[qs_off + i] = 0xA3  # low nibble 3 -> element i, high nibble 10 -> element 16 + i
        want = np.full(32, background, np.float32)
        want[i] += 2.0 * 3
        want[16 + i] += 2.0 * 10
        assert np.array_equal(oracle.dequantize(quant, blk), want), i
    if has_qh:
        for e in (0, 9, 16, 31):
            blk = base.copy()
            blk[qs_off - 4 + e // 8] = 1 << (e % 8)
            want = np.full(32, background, np.float32)
            want[e] += 2.0 * 16
            assert np.array_equal(oracle.dequantize(quant, blk), want), e
    rng = np.random.default_rng(50 + quant)
    blocks = _random_legacy(quant, rng, 200)
    got = oracle.dequantize(quant, blocks).astype(np.float64)
    want = npref.dequant_legacy_f64(quant, blocks)
    assert np.allclose(got, want, rtol=0, atol=4e-7 * np.abs(want).max())


def test_dequantize_q2k_reference_vectors_and_placement(oracle):
    """crates/rnb-cpu/src/quantize/dequant.rs:898-927: the zero block, and qs[1] = 3 with all scales 1, d = 1,
    dmin = 0 -> out[1] = 3, out[4] = 0, out[33] = 0 (hand-built bytes); then every element one at a time."""
    assert np.all(oracle.dequantize(Q2_K, np.zeros(84, np.uint8)) == 0.0)
    blk = np.zeros(84, np.uint8)
    blk[0:16] = 1
    blk[16 + 1] = 3
    blk[80:82] = np.frombuffer(npref.f16_bytes(1.0), np.uint8)
    y = oracle.dequantize(Q2_K, blk)
    assert y[1] == 3.0 and y[4] == 0.0 and y[33] == 0.0 and np.count_nonzero(y) == 1
    for elem in (0, 15, 16, 31, 32, 47, 100, 127, 128, 200, 255):
        v = np.zeros(256, np.uint8)
        v[elem] = 2
        y = oracle.dequantize(Q2_K, npref.make_q2k_block(1.0, 0.0, np.arange(16) % 15 + 1, np.zeros(16), v))
        want = np.zeros(256, np.float32)
        want[elem] = 2.0 * ((elem // 16) % 15 + 1)
        assert np.array_equal(y, want), elem
    # mins: values 0 -> every element of sub-block j is -dmin * mn[j]
    y = oracle.dequantize(Q2_K, npref.make_q2k_block(0.0, 0.5, np.zeros(16), np.arange(16), np.zeros(256)))
    assert np.array_equal(y, np.repeat(-0.5 * np.arange(16), 16).astype(np.float32))
    rng = np.random.default_rng(41)
    blocks = _random_q2k(rng, 64)
    got = oracle.dequantize(Q2_K, blocks).astype(np.float64)
    want = npref.dequant_q2k_f64(blocks)
    assert np.allclose(got, want, rtol=0, atol=4e-7 * np.abs(want).max())


def test_dequantize_q3k_zero_block_and_placement(oracle):
    """crates/rnb-cpu/src/quantize/dequant.rs:1009-1019 (zero block); hand-built bytes for each field: with every
    stored scale 33 (signed 1), d = 1, qs = hmask = 0 every value is -4; setting one hmask bit lifts one element to 0;
    one 2-bit field adds its value."""
    assert np.all(oracle.dequantize(Q3_K, np.zeros(110, np.uint8)) == 0.0)
    base = np.zeros(110, np.uint8)
    base[96:104] = 0x11       # low nibbles of all sixteen codes: 1
    base[104:108] = 0xAA      # high two bits of all sixteen codes: 2 -> stored 33, signed 1
    base[108:110] = np.frombuffer(npref.f16_bytes(1.0), np.uint8)
    assert np.all(oracle.dequantize(Q3_K, base) == -4.0)
    for l, bit in ((0, 0), (5, 3), (31, 7), (16, 4)):
        blk = base.copy()
        blk[l] = 1 << bit
        want = np.full(256, -4.0, np.float32)
        want[128 * (bit // 4) + 32 * (bit % 4) + l] = 0.0
        assert np.array_equal(oracle.dequantize(Q3_K, blk), want), (l, bit)
    blk = base.copy()
    blk[32 + 32 + 7] = 0b10_01_11_00  # half 1, l = 7: pairs 0..3 hold 0, 3, 1, 2
    want = np.full(256, -4.0, np.float32)
    want[128 + 32 * np.arange(4) + 7] = np.array([0, 3, 1, 2], np.float32) - 4.0
    assert np.array_equal(oracle.dequantize(Q3_K, blk), want)
    # scales: each code on its own sub-block
    codes = np.arange(-8, 8) * 4
    y = oracle.dequantize(Q3_K, npref.make_q3k_block(0.5, codes, np.full(256, 3)))
    assert np.array_equal(y, np.repeat(0.5 * codes * 3, 16).astype(np.float32))
    rng = np.random.default_rng(42)
    blocks = _random_q3k(rng, 64)
    got = oracle.dequantize(Q3_K, blocks).astype(np.float64)
    want = npref.dequant_q3k_f64(blocks)
    assert np.allclose(got, want, rtol=0, atol=4e-7 * np.abs(want).max())


def test_dequantize_q5k_zero_block(oracle):
    """crates/rnb-cpu/src/quantize/dequant.rs:1036-1047 (test_dequant_q5_k_zero)."""
    assert np.all(oracle.dequantize(Q5_K, np.zeros(176, np.uint8)) == 0.0)


def test_dequantize_q5k_places_each_bit(oracle):
    """Hand-built bytes (no packer): one qh bit set -> exactly the element 64*(bit//2) + 32*(bit%2) + l gains 16
    (the placement crates/rnb-cpu/src/gemm/tile_q5k.rs:944-976 states: bit 2g of qh[l] for l < 32 of group g,
    bit 2g+1 for the upper half); one nibble set -> as for Q4_K, 48 bytes further into the block."""
    hdr = np.concatenate([np.frombuffer(npref.f16_bytes(1.0), np.uint8), np.frombuffer(npref.f16_bytes(0.0), np.uint8),
                          npref.pack_scales_k4(np.arange(1, 9), np.zeros(8))])
    for l in (0, 5, 31):
        for bit in range(8):
            blk = np.concatenate([hdr, np.zeros(32 + 128, np.uint8)])
            blk[16 + l] = 1 << bit
            y = oracle.dequantize(Q5_K, blk)
            want = np.zeros(256, np.float32)
            want[64 * (bit // 2) + 32 * (bit % 2) + l] = 16.0 * (bit + 1)  # scale of sub-block `bit` is bit + 1
            assert np.array_equal(y, want), (l, bit)
    for g, l in ((0, 0), (1, 7), (3, 31)):
        blk = np.concatenate([hdr, np.zeros(32 + 128, np.uint8)])
        blk[48 + 32 * g + l] = 0x93  # low nibble 3, high nibble 9
        y = oracle.dequantize(Q5_K, blk)
        want = np.zeros(256, np.float32)
        want[64 * g + l] = 3.0 * (2 * g + 1)
        want[64 * g + 32 + l] = 9.0 * (2 * g + 2)
        assert np.array_equal(y, want), (g, l)
    rng = np.random.default_rng(31)
    blocks = _random_q5k(rng, 64)
    got = oracle.dequantize(Q5_K, blocks).astype(np.float64)
    want = npref.dequant_q5k_f64(blocks)
    assert np.allclose(got, want, rtol=0, atol=1e-7 * np.abs(want).max() * 4)
    # packer and splitter are inverse on the five-bit values
    vals = rng.integers(0, 32, 256)
    assert np.array_equal(npref.split_q5k(npref.make_q5k_block(1.0, 1.0, np.zeros(8), np.zeros(8), vals))[4][0], vals)


def test_dequantize_q6k_places_each_value(oracle):
    for elem in [0, 15, 16, 31, 32, 64, 96, 127, 128, 200, 255]:
        q = np.full(256, 32, dtype=np.uint8)  # stored 32 == signed 0
        q[elem] = 32 + 7
        blk = npref.make_q6k_block(1.0, np.arange(1, 17), q)
        y = oracle.dequantize(Q6_K, blk)
        want = np.zeros(256, dtype=np.float32)
        want[elem] = 7.0 * (elem // 16 + 1)
        assert np.array_equal(y, want), elem
    rng = np.random.default_rng(4)
    blocks = _random_q6k(rng, 64)
    got = oracle.dequantize(Q6_K, blocks).astype(np.float64)
    want = npref.dequant_q6k_f64(blocks)
    assert np.allclose(got, want, rtol=0, atol=1e-6 * np.abs(want).max())


def test_dequantize_q8_0(oracle):
    rng = np.random.default_rng(5)
    blocks = _random_q8_0(rng, 50)
    got = oracle.dequantize(Q8_0, blocks).astype(np.float64)
    assert np.allclose(got, npref.dequant_q8_0_f64(blocks), rtol=1e-7, atol=0)


# ---- Q8_K activation quantiser: the reference's exact vectors --------------------------

def test_q8k_reference_vectors(oracle):
    """crates/rnb-cpu/src/gemm/activation_q8.rs:179-217"""
    z = oracle.quantize_q8k(np.zeros(256, np.float32))[0]
    assert z["d"] == 0.0 and not z["qs"].any() and not z["bsums"].any()

    ties = np.zeros(256, np.float32)
    ties[0] = 127.0
    ties[1:7] = [-0.5, -1.5, -2.5, 0.5, 1.5, 2.5]
    b = oracle.quantize_q8k(ties)[0]
    assert b["d"] == -1.0
    assert b["qs"][1:7].tolist() == [0, 2, 2, 0, -2, -2]

    fp = np.zeros(256, np.float32)
    fp[0], fp[1] = 127.0, -127.0
    b = oracle.quantize_q8k(fp)[0]
    assert b["d"] == -1.0 and b["qs"][:2].tolist() == [-127, 127]

    fn = np.zeros(256, np.float32)
    fn[0], fn[1] = -127.0, 127.0
    b = oracle.quantize_q8k(fn)[0]
    assert b["d"] == 1.0 and b["qs"][:2].tolist() == [-127, 127]

    bd = np.zeros(256, np.float32)
    bd[15], bd[16], bd[255] = -1.0, -2.0, 127.0
    b = oracle.quantize_q8k(bd)[0]
    assert b["bsums"][0] == 1 and b["bsums"][1] == 2
    assert not b["bsums"][2:15].any() and b["bsums"][15] == -127


def test_q8k_matches_numpy_statement(oracle):
    # the reference's batch generator (activation_q8.rs:221-224) plus gaussian data
    idx = np.arange(16 * 256)
    x1 = ((idx * 73 + 19) % 2001).astype(np.float32) - 1000.0
    x2 = np.random.default_rng(6).standard_normal(64 * 256).astype(np.float32)
    for x in (x1, x2):
        got = oracle.quantize_q8k(x)
        d, qs, bsums = npref.quantize_q8k_np(x)
        assert np.array_equal(got["d"].view(np.uint32), d.view(np.uint32))
        assert np.array_equal(got["qs"], qs)
        assert np.array_equal(got["bsums"], bsums)
    # d is 1/iscale, not max/-127: a value where the two differ in the last bit must follow 1/iscale
    x = np.zeros(256, np.float32)
    x[3] = np.float32(0.3)
    b = oracle.quantize_q8k(x)[0]
    iscale = np.float32(-127.0) / np.float32(0.3)
    assert b["d"] == np.float32(1.0) / iscale and b["qs"][3] == -127


def test_q8_activation_quantiser(oracle):
    """crates/rnb-cpu/src/gemm/activation_q8.rs:14-32: d = amax/127 (f32), round half AWAY, clamp [-128,127]."""
    x = np.zeros(32, np.float32)
    x[0] = 127.0
    x[1:7] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    b = oracle.quantize_q8(x)[0]
    assert b["d"] == 1.0
    assert b["qs"][:7].tolist() == [127, 1, 2, 3, -1, -2, -3]
    z = oracle.quantize_q8(np.zeros(32, np.float32))[0]
    assert z["d"] == 0.0 and not z["qs"].any()
    xr = np.random.default_rng(7).standard_normal(32 * 100).astype(np.float32)
    got = oracle.quantize_q8(xr)
    d, qs = npref.quantize_q8_np(xr)
    assert np.array_equal(got["d"].view(np.uint32), d.view(np.uint32))
    assert np.array_equal(got["qs"], qs)


def test_quantisers_on_non_finite_inputs(oracle):
    """What the Rust does with NaN and infinity, stated by hand from the source.  Q8_K
    (crates/rnb-cpu/src/gemm/activation_q8.rs:149-173): `ax > amax` is false for NaN, so a NaN never becomes the
    maximum and a block of NaNs returns the zero block; `(iscale * NaN).round_ties_even() as i32` is 0.  An infinite
    maximum gives iscale = -127/inf = -0.0 and d = 1/-0.0 = -inf; every product is +-0 or NaN, every code 0.  Q8
    (:14-32): f32::max ignores a NaN operand, `NaN.clamp(-128, 127) as i8` is 0; an infinite maximum gives d = inf,
    id = 0 and inf * 0 = NaN."""
    nan, inf = np.float32(np.nan), np.float32(np.inf)
    x = np.zeros(4 * 256, np.float32)
    x[0:256] = nan                                    # block 0: all NaN
    x[256:512] = np.linspace(-1.0, 1.0, 256, dtype=np.float32)
    clean = oracle.quantize_q8k(x[256:512].copy())[0]
    x[256 + 17] = nan                                 # block 1: one NaN among finite values
    x[512 + 3], x[512 + 4] = inf, 5.0                 # block 2: +inf
    x[768 + 9], x[768 + 200] = -inf, nan              # block 3: -inf and a NaN
    b = oracle.quantize_q8k(x)
    assert b["d"][0] == 0.0 and not b["qs"][0].any() and not b["bsums"][0].any()
    want = clean["qs"].copy()
    want[17] = 0
    assert b["d"][1].view(np.uint32) == clean["d"].view(np.uint32) and np.array_equal(b["qs"][1], want)
    assert np.array_equal(b["bsums"][1], want.astype(np.int16).reshape(16, 16).sum(axis=1))
    assert b["d"][2] == -inf and not b["qs"][2].any()
    assert b["d"][3] == inf and not b["qs"][3].any()   # max_val = -inf: iscale = +0.0, d = +inf
    y = np.zeros(3 * 32, np.float32)
    y[0:32] = np.arange(32, dtype=np.float32) - 16.0
    ref = oracle.quantize_q8(y[0:32].copy())[0]
    y[5] = nan
    y[32 + 1], y[32 + 2] = inf, 7.0
    y[64:96] = nan
    q = oracle.quantize_q8(y)
    want = ref["qs"].copy()
    want[5] = 0
    assert q["d"][0].view(np.uint32) == ref["d"].view(np.uint32) and np.array_equal(q["qs"][0], want)
    assert q["d"][1] == inf and not q["qs"][1].any()
    assert q["d"][2] == 0.0 and not q["qs"][2].any()


# ---- Q4_K x Q8_K dot ------------------------------------------------------------------

def _act_from_parts(d, qs, bsums=None):
    from oracle.oracle import Q8K_DTYPE

    qs = np.asarray(qs, dtype=np.int8).reshape(-1, 256)
    a = np.zeros(qs.shape[0], dtype=Q8K_DTYPE)
    a["d"] = d
    a["qs"] = qs
    a["bsums"] = qs.astype(np.int16).reshape(-1, 16, 16).sum(axis=2) if bsums is None else bsums
    return a


def test_q4k_dot_reference_closed_forms(oracle):
    """crates/rnb-cpu/src/gemm/tile_q4k.rs:2019-2151: zero input -> 0; zero scales -> 0; one sub-block -> 2560."""
    raw_scales = np.full(12, 10, np.uint8)
    blk = np.concatenate([np.frombuffer(npref.f16_bytes(1.0), np.uint8), np.frombuffer(npref.f16_bytes(0.5), np.uint8),
                          raw_scales, np.full(128, 0x88, np.uint8)])
    act = _act_from_parts(1.0, np.zeros(256, np.int8))
    assert oracle.dot(Q4_K, blk, act) == 0.0

    blk2 = np.concatenate([np.frombuffer(npref.f16_bytes(1.0), np.uint8), np.frombuffer(npref.f16_bytes(1.0), np.uint8),
                           np.zeros(12, np.uint8), np.full(128, 0x88, np.uint8)])
    act2 = _act_from_parts(1.0, np.zeros(256, np.int8), bsums=np.full((1, 16), 50, np.int16))
    assert oracle.dot(Q4_K, blk2, act2) == 0.0

    sc = np.zeros(12, np.uint8)
    sc[0] = 10
    blk3 = np.concatenate([np.frombuffer(npref.f16_bytes(1.0), np.uint8), np.frombuffer(npref.f16_bytes(0.0), np.uint8),
                           sc, np.full(128, 0x88, np.uint8)])
    q = np.zeros(256, np.int8)
    q[:32] = 1
    assert oracle.dot(Q4_K, blk3, _act_from_parts(1.0, q)) == 2560.0
    assert oracle.dot(Q4_K, blk3, _act_from_parts(1.0, q), avx2=True) == 2560.0


def test_q4k_dot_equals_f64_dequant_identity(oracle):
    """integer path == sum dequant(W)[i] * (d_x*q_x[i]) computed independently in f64 (the invariant of
    crates/rnb-cpu/src/gemm/avx2_dot.rs:949-983, here exact instead of loose)."""
    rng = np.random.default_rng(8)
    for nb in (1, 2, 7, 16):
        row = _random_q4k(rng, nb)
        x = rng.standard_normal(nb * 256).astype(np.float32)
        act = oracle.quantize_q8k(x)
        want = float(np.dot(npref.dequant_q4k_f64(row), npref.deq_act_q8k_f64(act)))
        gold = oracle.dot(Q4_K, row, act, gold=True)
        assert gold == pytest.approx(want, rel=1e-11, abs=1e-12)
        scale = float(np.sum(np.abs(npref.dequant_q4k_f64(row) * npref.deq_act_q8k_f64(act))))
        assert abs(oracle.dot(Q4_K, row, act) - want) <= 4e-7 * scale
        assert abs(oracle.dot(Q4_K, row, act, avx2=True) - want) <= 4e-7 * scale


def test_q4k_mins_use_32_wide_bsums(oracle):
    # dmin term only: nibbles 0, mins 1..8, bsums chosen per 16 -> summ = sum mn[k]*(bsums[2k]+bsums[2k+1])
    blk = npref.make_q4k_block(0.0, 1.0, np.zeros(8), np.arange(1, 9), np.zeros(256))
    bs = np.arange(1, 17, dtype=np.int16).reshape(1, 16)
    act = _act_from_parts(2.0, np.zeros(256, np.int8), bsums=bs)
    summ = sum((k + 1) * (bs[0, 2 * k] + bs[0, 2 * k + 1]) for k in range(8))
    assert oracle.dot(Q4_K, blk, act) == -2.0 * summ
    assert oracle.dot(Q4_K, blk, act, avx2=True) == -2.0 * summ


# ---- Q4_0 / Q4_1 / Q5_0 / Q5_1 x Q8 dots -------------------------------------------------

def _q8_act(d, q):
    a = np.zeros(1, dtype=np.dtype([("d", "<f4"), ("qs", "i1", (32,))]))
    a["d"] = d
    a["qs"] = np.asarray(q, np.int8)
    return a


@pytest.mark.parametrize("quant", NIBBLE_FORMATS)
def test_legacy_dot_known_vectors_and_identity(oracle, quant):
    """crates/rnb-cpu/src/gemm/neon_dot.rs:83-214 and neon_quant.rs:88-158 on hand vectors: all codes equal ->
    (code - offset) * sum(q) * d * d_x for the _0 formats, d_x * (d * code + m) * sum(q) for the _1 formats; then the
    f64 identity against an independent dequantiser."""
    _, has_min, has_qh = npref.LEGACY_LAYOUT[quant]
    q = (np.arange(32) % 9 - 4).astype(np.int8)
    sq = float(q.astype(np.int64).sum())
    code = 19 if has_qh else 11
    blk = npref.make_legacy_block(quant, 2.0, 0.25, np.full(32, code))
    got = oracle.dot(quant, blk, _q8_act(0.5, q))
    if has_min:
        assert got == 0.5 * (2.0 * code * sq + 0.25 * sq)
    else:
        assert got == (code - (16 if has_qh else 8)) * sq * (2.0 * 0.5)
    # one code differs: only that element's activation enters the difference
    codes = np.full(32, code)
    codes[21] += 3
    got2 = oracle.dot(quant, npref.make_legacy_block(quant, 2.0, 0.25, codes), _q8_act(0.5, q))
    assert got2 - got == 3 * float(q[21]) * 2.0 * 0.5
    rng = np.random.default_rng(60 + quant)
    for nb in (1, 3, 128):
        row = _random_legacy(quant, rng, nb)
        x = rng.standard_normal(nb * 32).astype(np.float32)
        act = oracle.quantize_q8(x)
        xq = (act["d"].astype(np.float64)[:, None] * act["qs"].astype(np.float64)).reshape(-1)
        want = float(np.dot(npref.dequant_legacy_f64(quant, row), xq))
        assert oracle.dot(quant, row, act, gold=True) == pytest.approx(want, rel=1e-11, abs=1e-12)
        scale = float(np.sum(np.abs(npref.dequant_legacy_f64(quant, row) * xq)))
        assert abs(oracle.dot(quant, row, act) - want) <= 4e-7 * scale


# ---- Q2_K / Q3_K x Q8_K dots ------------------------------------------------------------

def test_q2k_q3k_dot_known_vectors(oracle):
    """Hand-built blocks for crates/rnb-cpu/src/gemm/avx2_dot.rs:169-375: all values 1, one non-zero sub-block scale ->
    scale * (sum of that sub-block's 16 activations); mins against the 16-wide bsums; Q3_K's signed scales."""
    q = (np.arange(256) % 11 - 5).astype(np.int8)
    act = _act_from_parts(0.25, q)
    for j in range(16):
        sc = np.zeros(16, np.int64)
        sc[j] = 7
        blk = npref.make_q2k_block(2.0, 0.0, sc, np.zeros(16), np.ones(256))
        assert oracle.dot(Q2_K, blk, act) == 0.25 * 2.0 * 7 * float(q[16 * j:16 * j + 16].astype(np.int64).sum()), j
        codes = np.zeros(16, np.int64)
        codes[j] = -9
        blk3 = npref.make_q3k_block(2.0, codes, np.full(256, 3))
        assert oracle.dot(Q3_K, blk3, act) == 0.25 * 2.0 * -9 * 3 * float(q[16 * j:16 * j + 16].astype(np.int64).sum()), j
    blk = npref.make_q2k_block(0.0, 1.0, np.zeros(16), np.arange(16), np.zeros(256))
    bs = (np.arange(16, dtype=np.int16) * 3 - 20).reshape(1, 16)
    summ = int((np.arange(16) * bs[0].astype(np.int64)).sum())
    assert oracle.dot(Q2_K, blk, _act_from_parts(2.0, np.zeros(256, np.int8), bsums=bs)) == -2.0 * summ


@pytest.mark.parametrize("quant,maker,deq", [(Q2_K, _random_q2k, npref.dequant_q2k_f64),
                                             (Q3_K, _random_q3k, npref.dequant_q3k_f64)])
def test_q2k_q3k_dot_equals_f64_dequant_identity(oracle, quant, maker, deq):
    rng = np.random.default_rng(43 + quant)
    for nb in (1, 2, 7, 16):
        row = maker(rng, nb)
        x = rng.standard_normal(nb * 256).astype(np.float32)
        act = oracle.quantize_q8k(x)
        want = float(np.dot(deq(row), npref.deq_act_q8k_f64(act)))
        gold = oracle.dot(quant, row, act, gold=True)
        assert gold == pytest.approx(want, rel=1e-11, abs=1e-12)
        scale = float(np.sum(np.abs(deq(row) * npref.deq_act_q8k_f64(act))))
        assert abs(oracle.dot(quant, row, act) - want) <= 4e-7 * scale


# ---- Q5_K x Q8_K dot ------------------------------------------------------------------

def test_q5k_dot_fifth_bit_vectors(oracle):
    """Known answers for crates/rnb-cpu/src/gemm/neon_dot.rs:1742-1800 built by hand: d = 1, dmin = 0, sub-block
    scales 1..8, every nibble 0, one qh bit set in every byte -> the 32 elements of sub-block `bit` are 16, so the
    dot is 16 * (bit + 1) * sum of that sub-block's activations."""
    hdr = np.concatenate([np.frombuffer(npref.f16_bytes(1.0), np.uint8), np.frombuffer(npref.f16_bytes(0.0), np.uint8),
                          npref.pack_scales_k4(np.arange(1, 9), np.zeros(8))])
    q = (np.arange(256) % 7 - 3).astype(np.int8)
    act = _act_from_parts(0.5, q)
    for bit in range(8):
        blk = np.concatenate([hdr, np.full(32, 1 << bit, np.uint8), np.zeros(128, np.uint8)])
        want = 0.5 * 16.0 * (bit + 1) * float(q[32 * bit:32 * bit + 32].astype(np.int64).sum())
        assert oracle.dot(Q5_K, blk, act) == want, bit
    # with qh == 0 a Q5_K block is the Q4_K block with 32 zero bytes inserted
    rng = np.random.default_rng(32)
    row4 = _random_q4k(rng, 3).reshape(3, 144)
    row5 = np.concatenate([row4[:, :16], np.zeros((3, 32), np.uint8), row4[:, 16:]], axis=1).reshape(-1)
    act3 = oracle.quantize_q8k(rng.standard_normal(3 * 256).astype(np.float32))
    assert oracle.dot(Q5_K, row5, act3) == oracle.dot(Q4_K, row4.reshape(-1), act3)
    # dmin term: values 0, mins 1..8 -> summ over 32-wide bsums, as for Q4_K
    blk = npref.make_q5k_block(0.0, 1.0, np.zeros(8), np.arange(1, 9), np.zeros(256))
    bs = np.arange(1, 17, dtype=np.int16).reshape(1, 16)
    summ = sum((k + 1) * (bs[0, 2 * k] + bs[0, 2 * k + 1]) for k in range(8))
    assert oracle.dot(Q5_K, blk, _act_from_parts(2.0, np.zeros(256, np.int8), bsums=bs)) == -2.0 * summ


def test_q5k_dot_equals_f64_dequant_identity(oracle):
    rng = np.random.default_rng(33)
    for nb in (1, 2, 7, 16):
        row = _random_q5k(rng, nb)
        x = rng.standard_normal(nb * 256).astype(np.float32)
        act = oracle.quantize_q8k(x)
        want = float(np.dot(npref.dequant_q5k_f64(row), npref.deq_act_q8k_f64(act)))
        gold = oracle.dot(Q5_K, row, act, gold=True)
        assert gold == pytest.approx(want, rel=1e-11, abs=1e-12)
        scale = float(np.sum(np.abs(npref.dequant_q5k_f64(row) * npref.deq_act_q8k_f64(act))))
        assert abs(oracle.dot(Q5_K, row, act) - want) <= 4e-7 * scale


# ---- Q6_K x Q8_K dot ------------------------------------------------------------------

def test_q6k_dot_equals_f64_dequant_identity(oracle):
    rng = np.random.default_rng(9)
    for nb in (1, 3, 16, 56):
        row = _random_q6k(rng, nb)
        x = rng.standard_normal(nb * 256).astype(np.float32)
        act = oracle.quantize_q8k(x)
        want = float(np.dot(npref.dequant_q6k_f64(row), npref.deq_act_q8k_f64(act)))
        assert oracle.dot(Q6_K, row, act, gold=True) == pytest.approx(want, rel=1e-11, abs=1e-14)
        scale = float(np.sum(np.abs(npref.dequant_q6k_f64(row) * npref.deq_act_q8k_f64(act))))
        assert abs(oracle.dot(Q6_K, row, act) - want) <= 4e-7 * scale
        assert abs(oracle.dot(Q6_K, row, act, avx2=True) - want) <= 4e-7 * scale


def test_q6k_bsums_identity(oracle):
    """sum sc*(q-32)*x == sum sc*q*x - 32*sum sc[sb]*bsums[sb] (crates/rnb-cpu/src/gemm/avx2_dot.rs:824,880)."""
    rng = np.random.default_rng(10)
    row = _random_q6k(rng, 1)
    x = rng.standard_normal(256).astype(np.float32)
    act = oracle.quantize_q8k(x)
    d, sc, q = npref.split_q6k(row)
    u = (q + 32).reshape(16, 16)
    a = act["qs"][0].astype(np.int64).reshape(16, 16)
    lhs = int(np.sum(sc[0][:, None] * (u - 32) * a))
    rhs = int(np.sum(sc[0][:, None] * u * a)) - 32 * int(np.sum(sc[0] * act["bsums"][0].astype(np.int64)))
    assert lhs == rhs
    got = oracle.dot(Q6_K, row, act, gold=True)
    assert got == pytest.approx(float(d[0]) * float(act["d"][0]) * lhs, rel=1e-12)


# ---- Q8_0 ----------------------------------------------------------------------------

REF_Q8_0_BYTES = bytes([0x00, 0x3C] + list(range(1, 33)) + [0x00, 0x3C] + list(range(32, 0, -1)))


def test_q8_0_reference_seq_major_vector(oracle):
    """crates/rnb-cpu/src/gemm/quant_gemv.rs:1448-1464: rows 1..32 / 32..1, d = 1, x = 1 -> 528 everywhere,
    output index s*rows + row."""
    x = np.ones(64, np.float32)
    out = oracle.gemv_q8_0_f32act(REF_Q8_0_BYTES, 2, 32, x)
    assert out.shape == (2, 2) and np.all(out == 528.0)
    # distinguishable rows/tokens to pin the layout itself
    x2 = np.concatenate([np.ones(32, np.float32), 2 * np.ones(32, np.float32)])
    w = np.concatenate([npref.make_q8_0_block(1.0, np.ones(32)), npref.make_q8_0_block(1.0, 3 * np.ones(32))])
    out = oracle.gemv_q8_0_f32act(w, 2, 32, x2)
    assert out.ravel().tolist() == [32.0, 96.0, 64.0, 192.0]
    out_q = oracle.gemv(Q8_0, w, 2, 32, x2)
    assert np.allclose(out_q.ravel(), [32.0, 96.0, 64.0, 192.0], rtol=1e-6)


def test_q8_0_q8_matches_engine_oracle(oracle):
    """crates/rnb-llm/src/engine/tests.rs:6872-6896: out = d_x * sum(w*q) when d_w = 1."""
    values = np.array([(i % 7) - 3 for i in range(64)], dtype=np.int8)
    w = np.concatenate([npref.make_q8_0_block(1.0, values[:32]), npref.make_q8_0_block(1.0, values[32:])])
    x = (np.arange(32, dtype=np.float32) - 16.0) * 0.25
    act = oracle.quantize_q8(x)
    out = oracle.gemv(Q8_0, w, 2, 32, x)[0]
    for r in range(2):
        dot = int(np.dot(values[32 * r:32 * r + 32].astype(np.int64), act["qs"][0].astype(np.int64)))
        assert abs(out[r] - float(act["d"][0]) * dot) < 1e-5


def test_q8_0_q8_equals_f64_identity(oracle):
    rng = np.random.default_rng(11)
    row = _random_q8_0(rng, 128)
    x = rng.standard_normal(4096).astype(np.float32)
    act = oracle.quantize_q8(x)
    ax = (act["qs"].astype(np.float64) * act["d"].astype(np.float64)[:, None]).reshape(-1)
    want = float(np.dot(npref.dequant_q8_0_f64(row), ax))
    assert oracle.dot(Q8_0, row, act, gold=True) == pytest.approx(want, rel=1e-11)
    assert oracle.dot(Q8_0, row, act) == pytest.approx(want, rel=2e-5)
    assert oracle.dot_q8_0_f32(row, x) == pytest.approx(float(np.dot(npref.dequant_q8_0_f64(row), x.astype(np.float64))), rel=2e-5, abs=1e-5)


# ---- drivers --------------------------------------------------------------------------

@pytest.mark.parametrize("quant,maker", [(Q2_K, _random_q2k), (Q3_K, _random_q3k), (Q4_K, _random_q4k),
                                         (Q5_K, _random_q5k), (Q6_K, _random_q6k)])
def test_gemv_driver_layout_and_row_independence(oracle, quant, maker):
    rng = np.random.default_rng(12)
    rows, nb, seq = 5, 2, 3
    w = maker(rng, rows * nb)
    x = rng.standard_normal((seq, nb * 256)).astype(np.float32)
    out = oracle.gemv(quant, w, rows, nb * 256, x)
    rb = w.size // rows
    for s in range(seq):
        act = oracle.quantize_q8k(x[s])
        for r in range(rows):
            assert out[s, r] == np.float32(oracle.dot(quant, w[r * rb:(r + 1) * rb], act))
    gold = oracle.gemv(quant, w, rows, nb * 256, x, gold=True)
    assert np.allclose(out, gold, rtol=1e-4, atol=1e-6)
    if quant in (Q4_K, Q6_K):  # the vectorised baseline covers the benchmarked formats only
        fast = oracle.gemv(quant, w, rows, nb * 256, x, avx2=True)
        assert np.allclose(fast, gold, rtol=1e-4, atol=1e-6)
    # 1 thread == many threads, bitwise (rows are independent)
    assert np.array_equal(oracle.gemv(quant, w, rows, nb * 256, x, n_threads=1), out)


# ---- router ---------------------------------------------------------------------------

def test_router_reference_vectors(oracle):
    """crates/rnb-llm/src/engine/models/shared_expert_moe/routing.rs:272-318"""
    idx, w = oracle.route_topk([0.0, 4.0, 3.0, 2.0], 2)
    assert idx.tolist() == [1, 2] and abs(w.sum() - 1.0) < 1e-6 and w[0] > w[1]
    idx, w = oracle.route_topk([1.0, 4.0, 4.0, -2.0, 3.0], 3)
    assert idx.tolist() == [1, 2, 4]
    e4, e3 = 1.0, math.exp(-1.0)
    s = e4 + e4 + e3
    assert np.allclose(w, [e4 / s, e4 / s, e3 / s], atol=1e-6)


def test_router_against_numpy_sort(oracle):
    rng = np.random.default_rng(13)
    for _ in range(20):
        lg = rng.standard_normal(128).astype(np.float32)
        idx, w = oracle.route_topk(lg, 8)
        order = np.lexsort((np.arange(128), -lg))[:8]  # logit desc, ties -> lower id
        assert idx.tolist() == order.tolist()
        e = np.exp(lg[order].astype(np.float64) - float(lg[order[0]]))
        assert np.allclose(w, e / e.sum(), rtol=1e-5)


# ---- SiLU * up ------------------------------------------------------------------------

def test_silu_mul(oracle):
    g = np.array([0.0, 1.0, -1.0, 5.0, -20.0, 30.0], np.float32)
    u = np.array([2.0, 3.0, 4.0, -1.0, 1.0, 0.5], np.float32)
    want = g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64))) * u
    assert np.allclose(oracle.silu_mul(g, u), want, rtol=1e-6, atol=1e-12)


# ---- MoE ------------------------------------------------------------------------------

def test_gelu_mul_reference_vector_and_formula(oracle):
    """crates/rnb-cpu/src/kernels/activation.rs:166-173: gate [1, -1], up [2, 3] -> 1.6824, -0.4764 (1e-3)."""
    got = oracle.gelu_mul(np.array([1.0, -1.0], np.float32), np.array([2.0, 3.0], np.float32))
    assert abs(got[0] - 1.6824) < 1e-3 and abs(got[1] + 0.4764) < 1e-3
    g = (np.arange(2048) % 257).astype(np.float32) / np.float32(32.0) - np.float32(4.0)   # the inputs of activation.rs:181-186
    u = (np.arange(2048) % 113).astype(np.float32) / np.float32(64.0) - np.float32(0.75)
    g64 = g.astype(np.float64)
    want = 0.5 * g64 * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (g64 + 0.044715 * g64 ** 3))) * u
    assert np.allclose(oracle.gelu_mul(g, u), want, rtol=2e-6, atol=1e-7)
    assert oracle.gelu_mul(np.zeros(3, np.float32), np.ones(3, np.float32)).tolist() == [0.0, 0.0, 0.0]


def test_moe_matches_f32_dequant_statement(oracle):
    """The reference's CUDA-test oracle (crates/rnb-backend/cuda/src/runtime/tests.rs:29561-29584) is an
    f32-dequant statement of gate/up -> SiLU*up -> Q6_K down -> route-weighted sum; the integer path agrees
    with an independent f64 dequant statement up to activation-quantisation noise (~1e-2 relative)."""
    n_expert, n_ff, n_embd = 4, 256, 512
    w_gate = oracle.make_weights(Q4_K, n_expert * n_ff, n_embd, 101)
    w_up = oracle.make_weights(Q4_K, n_expert * n_ff, n_embd, 102)
    w_down = oracle.make_weights(Q6_K, n_expert * n_embd, n_ff, 103)
    x = oracle.fill_normal(2 * n_embd, 104).reshape(2, n_embd)
    expert_ids = np.array([2, 0, 3, 1, 2], np.uint32)
    token_ids = np.array([0, 0, 0, 1, 1], np.uint32)
    route = np.array([0.5, 0.3, 0.2, 0.6, 0.4], np.float32)
    out = oracle.moe_sparse_experts_by_token(w_gate, w_up, w_down, n_expert, expert_ids, route, token_ids, 2,
                                             Q6_K, n_ff, n_embd, x)
    G = npref.dequant_q4k_f64(w_gate).reshape(n_expert, n_ff, n_embd)
    U = npref.dequant_q4k_f64(w_up).reshape(n_expert, n_ff, n_embd)
    D = npref.dequant_q6k_f64(w_down).reshape(n_expert, n_embd, n_ff)
    want = np.zeros((2, n_embd))
    for e, t, r in zip(expert_ids, token_ids, route):
        g = G[e] @ x[t].astype(np.float64)
        u = U[e] @ x[t].astype(np.float64)
        a = g / (1.0 + np.exp(-g)) * u
        want[t] += r * (D[e] @ a)
    err = np.abs(out - want).max() / np.abs(want).max()
    assert err < 3e-2, err
    # exact composition: one slot == gemv(gate), gemv(up), silu, gemv(down) * w, bitwise
    pg = n_ff * (n_embd // 256) * 144
    pd = n_embd * (n_ff // 256) * 210
    g = oracle.gemv(Q4_K, w_gate[2 * pg:3 * pg], n_ff, n_embd, x[0])[0]
    u = oracle.gemv(Q4_K, w_up[2 * pg:3 * pg], n_ff, n_embd, x[0])[0]
    a = oracle.silu_mul(g, u)
    o = oracle.gemv(Q6_K, w_down[2 * pd:3 * pd], n_embd, n_ff, a)[0] * np.float32(0.5)
    one = oracle.moe_sparse_experts_by_token(w_gate, w_up, w_down, n_expert, [2], [0.5], [0], 1, Q6_K, n_ff,
                                             n_embd, x[0])
    assert np.array_equal(one[0], o)
    # token batching does not change a (token, expert) result: 1-token call == row of the 2-token call
    solo = oracle.moe_sparse_experts_by_token(w_gate, w_up, w_down, n_expert, expert_ids[:3], route[:3],
                                              [0, 0, 0], 1, Q6_K, n_ff, n_embd, x[0])
    assert np.array_equal(solo[0], out[0])


# ---- weight generators (input generation only) -----------------------------------------

def test_q4k_quantiser_roundtrip_property(oracle):
    """crates/rnb-cpu/src/quantize/quant.rs:766-798: quantise -> dequantise cosine >= 0.97.  Byte parity with
    the Rust quantiser is UNPINNED (cannot run it); GPU and oracle consume identical bytes regardless."""
    x = oracle.fill_normal(256 * 40, 21, 0.02)
    y = oracle.dequantize(Q4_K, oracle.quantize_row(Q4_K, x))
    cos = float(np.dot(x, y) / (np.linalg.norm(x) * np.linalg.norm(y)))
    assert cos >= 0.97
    assert np.sqrt(np.mean((x - y) ** 2)) / np.sqrt(np.mean(x ** 2)) < 0.1


def test_q5k_quantiser_roundtrip_property(oracle):
    """crates/rnb-cpu/src/quantize/quant.rs:732-764: the reference's own input and bound (cosine >= 0.98).  Byte
    parity with the Rust quantiser is UNPINNED (cannot run it); GPU and oracle consume identical bytes."""
    t = np.arange(1024, dtype=np.float32) * np.float32(0.019)
    x = (np.sin(t) * (1.0 + 0.3 * np.cos(t * np.float32(0.7)))).astype(np.float32)
    q = oracle.quantize_row(Q5_K, x)
    assert q.size == 4 * 176
    y = oracle.dequantize(Q5_K, q)
    assert float(np.dot(x, y) / (np.linalg.norm(x) * np.linalg.norm(y) + 1e-10)) >= 0.98
    xn = oracle.fill_normal(256 * 40, 23, 0.02)
    qn = oracle.quantize_row(Q5_K, xn)
    yn = oracle.dequantize(Q5_K, qn)
    assert np.sqrt(np.mean((xn - yn) ** 2)) / np.sqrt(np.mean(xn ** 2)) < 0.05
    d, dmin, sc, mn, val = npref.split_q5k(qn)
    assert sc.max() == 63 and val.max() == 31 and val.min() == 0


@pytest.mark.parametrize("quant,bound", [(Q4_0, 0.12), (Q4_1, 0.12), (Q5_0, 0.06), (Q5_1, 0.06)])
def test_legacy_generators_roundtrip(oracle, quant, bound):
    x = oracle.fill_normal(32 * 300, 25, 0.02)
    w = oracle.quantize_row(quant, x)
    y = oracle.dequantize(quant, w)
    assert np.sqrt(np.mean((x - y) ** 2)) / np.sqrt(np.mean(x ** 2)) < bound
    # the driver: out[s][r] == dot(row r, Q8(x_s)), seq-major
    rows, cols = 3, 96
    wm = oracle.make_weights(quant, rows, cols, 7)
    xs = oracle.fill_normal(2 * cols, 8, 1.0).reshape(2, cols)
    out = oracle.gemv(quant, wm, rows, cols, xs)
    rb = wm.size // rows
    for si in range(2):
        act = oracle.quantize_q8(xs[si])
        for r in range(rows):
            assert out[si, r] == np.float32(oracle.dot(quant, wm[r * rb:(r + 1) * rb], act))


def test_q2k_q3k_generators_roundtrip(oracle):
    """crates/rnb-cpu/src/quantize/quant.rs (q2k round-trip test: cosine > 0.90 on its sine input); the Q3_K
    generator is not the reference's.  Input generation only."""
    t = np.arange(1024, dtype=np.float32) * np.float32(0.013)
    x = (np.sin(t) * (1.0 + 0.2 * np.cos(t * np.float32(0.5)))).astype(np.float32)
    y = oracle.dequantize(Q2_K, oracle.quantize_row(Q2_K, x))
    assert float(np.dot(x, y) / (np.linalg.norm(x) * np.linalg.norm(y))) > 0.90
    xn = oracle.fill_normal(256 * 40, 24, 0.02)
    y2 = oracle.dequantize(Q2_K, oracle.quantize_row(Q2_K, xn))
    y3 = oracle.dequantize(Q3_K, oracle.quantize_row(Q3_K, xn))
    assert float(np.dot(xn, y2) / (np.linalg.norm(xn) * np.linalg.norm(y2))) > 0.90
    assert np.sqrt(np.mean((xn - y3) ** 2)) / np.sqrt(np.mean(xn ** 2)) < 0.25
    b3 = oracle.quantize_row(Q3_K, xn).reshape(-1, 110)
    assert b3[:, 0:32].any() and b3[:, 32:96].any()  # both bit planes in use


def test_q6k_q8_0_generators_roundtrip(oracle):
    x = oracle.fill_normal(256 * 40, 22, 0.02)
    y6 = oracle.dequantize(Q6_K, oracle.quantize_row(Q6_K, x))
    assert np.sqrt(np.mean((x - y6) ** 2)) / np.sqrt(np.mean(x ** 2)) < 0.03
    y8 = oracle.dequantize(Q8_0, oracle.quantize_row(Q8_0, x))
    assert np.sqrt(np.mean((x - y8) ** 2)) / np.sqrt(np.mean(x ** 2)) < 0.01
    # scales spread over the 6-bit / int8 range as for real weights
    d, dmin, sc, mn, nib = npref.split_q4k(oracle.quantize_row(Q4_K, x))
    assert sc.max() == 63 and nib.max() == 15 and nib.min() == 0


def test_generator_is_counter_based_and_normal(oracle):
    a = oracle.fill_normal(100000, 5, 1.0)
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1.0) < 0.02
    w1 = oracle.make_weights(Q4_K, 8, 512, 77, n_threads=1)
    w2 = oracle.make_weights(Q4_K, 8, 512, 77, n_threads=4)
    assert np.array_equal(w1, w2)
    row3 = oracle.quantize_row(Q4_K, oracle.fill_normal(8 * 512, 77, 0.02)[3 * 512:4 * 512])
    assert np.array_equal(w1[3 * 288:4 * 288], row3)


# ---- RMS norm ------------------------------------------------------------------------------------------

def test_rms_norm_reference_vectors_and_closed_forms(oracle):
    """crates/rnb-cpu/src/kernels/norm.rs:339-385: [1, 2, 3, 4] with unit weights gives x / sqrt(7.5 + 1e-5); the weighted
    and unit-offset forms multiply by w and 1 + w.  Against Python's own f64 arithmetic, then properties the
    mathematics fixes: a power-of-two scaling of x with eps = 0 leaves the output bits alone, a constant row of c
    gives sign(c) * w / sqrt(1 + eps / c^2), rows are independent."""
    import math

    x = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    one = oracle.rms_norm(x, np.ones(4, np.float32), 1e-5)[0]
    rms = math.sqrt(7.5 + float(np.float32(1e-5)))
    assert abs(one[0] - 1.0 / rms) < 1e-7 and abs(one[1] - 2.0 / rms) < 1e-7 and abs(one[3] - 4.0 / rms) < 2e-7
    w = np.array([1.0, 0.5, 2.0, 0.25], np.float32)
    got = oracle.rms_norm(x, w, 1e-5)[0]
    assert np.allclose(got, x.astype(np.float64) / rms * w, rtol=2e-7, atol=0)
    wu = np.array([0.0, -0.5, 1.0, -0.75], np.float32)
    gu = oracle.rms_norm(x, wu, 1e-5, unit_offset=True)[0]
    assert np.allclose(gu, x.astype(np.float64) / rms * (1.0 + wu), rtol=3e-7, atol=0)
    rng = np.random.default_rng(5)
    xr = rng.standard_normal(3 * 1536).astype(np.float32)
    wr = rng.standard_normal(1536).astype(np.float32)
    base = oracle.rms_norm(xr, wr, 0.0)
    assert np.array_equal(oracle.rms_norm(4.0 * xr, wr, 0.0).view(np.uint32), base.view(np.uint32))
    assert np.array_equal(oracle.rms_norm(xr[1536:3072], wr, 0.0)[0].view(np.uint32), base[1].view(np.uint32))
    f64 = xr.reshape(3, 1536).astype(np.float64)
    want = f64 / np.sqrt((f64 * f64).mean(axis=1, keepdims=True) + float(np.float32(1e-6))) * wr
    assert np.allclose(oracle.rms_norm(xr, wr, 1e-6), want, rtol=3e-7, atol=1e-9)
    assert np.allclose(oracle.rms_norm(xr, wr, 1e-6, unit_offset=True), want / wr * (1.0 + wr.astype(np.float64)), rtol=2e-6, atol=1e-8)
    c = np.full(256, -3.0, np.float32)
    assert np.allclose(oracle.rms_norm(c, np.ones(256, np.float32), 1e-5)[0], -1.0 / math.sqrt(1.0 + 1e-5 / 9.0), rtol=2e-7)


# ---- importance quants -------------------------------------------------------------------------------------------------

def _fnv1a_of_f32(values):
    h = 0xcbf29ce484222325
    for b in np.asarray(values, np.float32).tobytes():
        h = ((h ^ b) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
    return h


_ONE_F16 = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
_IQ_HASHES = {16: 0x0ead89a48d8fee11, 22: 0x69e6a32989d193d1, 18: 0xbcf1592321ede577, 23: 0x0c822de33756fd50}


@pytest.mark.parametrize("quant", [16, 22, 18, 23])
def test_iq_dequantisers_reproduce_the_references_known_answers(oracle, quant):
    """crates/rnb-cpu/src/quantize/iq.rs:258-334: the FNV-1a hash over the f32 bits of the decoded block whose byte i is
    73 i + 19 (mod 256) behind a leading f16 1.0 -- one known answer per format, which also fixes every codebook entry,
    sign and scale the block touches; and iq.rs:281-299: zero codes decode to +1.0 everywhere (IQ4_XS: scale -32 times
    the first table value, -127)."""
    n = oracle.BLOCK_BYTES[quant]
    blk = np.array([(i * 73 + 19) & 0xFF for i in range(n)], np.uint8)
    blk[:2] = _ONE_F16
    assert _fnv1a_of_f32(oracle.dequantize(quant, blk)) == _IQ_HASHES[quant]
    zero = np.zeros(n, np.uint8)
    zero[:2] = _ONE_F16
    want = 4064.0 if quant == 23 else 1.0
    assert np.array_equal(oracle.dequantize(quant, zero), np.full(256, want, np.float32))


def test_iq4_xs_reference_vector(oracle):
    """crates/rnb-cpu/src/gemm/dequant.rs:542-556: scales_h 0xaaaa, scales_l 0x11 -> every 6-bit scale is 33, i.e. +1;
    bytes 0xf0 -> low nibble 0 (-127) for the first 16 elements of a sub-block, high nibble 15 (113) for the other 16."""
    b = np.zeros(136, np.uint8)
    b[:2] = _ONE_F16
    b[2:4] = (0xAA, 0xAA)
    b[4:8] = 0x11
    b[8:] = 0xF0
    out = oracle.dequantize(23, b)
    assert out[0] == -127.0 and out[16] == 113.0 and out[32] == -127.0
    assert np.array_equal(out.reshape(8, 2, 16), np.broadcast_to(np.array([-127.0, 113.0], np.float32)[None, :, None], (8, 2, 16)))


def test_iq_codebooks_have_the_published_shape(oracle):
    """The packed codebooks expand to ggml's tables: the byte alphabets ({8, 25, 43}; 4 + 8 c with 62 for c = 7), the
    first and last entries, all entries distinct.  (The hashes above check the entries a block touches by value.)"""
    g2, g2s, g3 = oracle.iq_grid(0), oracle.iq_grid(1), oracle.iq_grid(2)
    assert g2.size == 256 and g2s.size == 1024 and g3.size == 256
    for g, nbytes in ((g2, 8), (g2s, 8)):
        by = g.view(np.uint8).reshape(-1, 8)[:, :nbytes]
        assert set(np.unique(by)) == {8, 25, 43}
        assert np.unique(g).size == g.size
    by3 = g3.astype(np.uint32).view(np.uint8).reshape(-1, 4)
    assert set(np.unique(by3)) == {4, 12, 20, 28, 36, 44, 52, 62}
    assert np.unique(g3).size == 256
    assert g2[0] == 0x0808080808080808 and g2[1] == 0x080808080808082B and g2s[0] == 0x0808080808080808 and g3[0] == 0x04040404


def _packed_inc_tables(path):
    """The three packed codebooks of an .inc file (16 bits per entry), by name."""
    import re

    text = open(path).read()
    out = {}
    for name, n in (("kIq2xxsPacked", 256), ("kIq2sPacked", 1024), ("kIq3xxsPacked", 256)):
        m = re.search(name + r"\[" + str(n) + r"\]\s*=\s*\{(.*?)\};", text, re.S)
        assert m, f"{name} not found in {path}"
        vals = [int(tok, 16) for tok in re.findall(r"0x[0-9a-fA-F]+", m.group(1))]
        assert len(vals) == n
        out[name] = vals
    return out


def _expand2(w):  # two bits per byte: 0 -> 8, 1 -> 25, 2 -> 43
    return sum((8, 25, 43)[(w >> (2 * j)) & 3] << (8 * j) for j in range(8))


def _expand3(w):  # three bits per byte: c -> 4 + 8 c, 7 -> 62
    return sum((62 if ((w >> (3 * j)) & 7) == 7 else 4 + 8 * ((w >> (3 * j)) & 7)) << (8 * j) for j in range(4))


def _digest(vals, width, signed=False):
    import hashlib

    return hashlib.sha256(b"".join(int(v).to_bytes(width, "little", signed=signed) for v in vals)).hexdigest()


def test_iq_codebooks_equal_the_references_tables_entry_for_entry(oracle):
    """Every entry of the three grids, the sign table and the IQ4_NL values against the reference's own tables
    (crates/rnb-core/src/quant_codebooks.rs:3, 13, 787, 1814; crates/rnb-cpu/src/quantize/iq.rs:9), through the digests and
    spot entries that tests/golden/make_iq_codebook_digests.py computed from the reference's text.  Three routes to the
    same numbers: the oracle's expanded tables; the product's packed file expanded here by the packing rule (the product
    and the oracle keep the same packed words, so a typo would be common to both: this is the check that is not); the
    sign rule `i | parity(i) << 7` and the IQ4_NL values as the oracle's dequantiser applies them."""
    import json
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    want = json.load(open(os.path.join(root, "tests", "golden", "iq_codebook_digests.json")))
    # the oracle's expansion
    for which, name, width in ((0, "IQ2XXS_GRID", 8), (1, "IQ2S_GRID", 8), (2, "IQ3XXS_GRID", 4)):
        g = oracle.iq_grid(which)
        assert g.size == want[name]["entries"]
        assert _digest(g.tolist(), width) == want[name]["sha256"], name
        for i, v in want[name]["spot"].items():
            assert int(g[int(i)]) == v
    # the product's and the oracle's packed files, expanded by the rule
    for rel in (("runnburn_amd", "csrc", "iq_grids_packed.inc"), ("oracle", "iq_grids.inc")):
        t = _packed_inc_tables(os.path.join(root, *rel))
        assert _digest([_expand2(w) for w in t["kIq2xxsPacked"]], 8) == want["IQ2XXS_GRID"]["sha256"], rel
        assert _digest([_expand2(w) for w in t["kIq2sPacked"]], 8) == want["IQ2S_GRID"]["sha256"], rel
        assert _digest([_expand3(w) for w in t["kIq3xxsPacked"]], 4) == want["IQ3XXS_GRID"]["sha256"], rel
    # the sign table: seven bits and their parity
    signs = [i | (bin(i).count("1") & 1) << 7 for i in range(128)]
    assert _digest(signs, 1) == want["KSIGNS_IQ2XS"]["sha256"]
    # the IQ4_NL values through the oracle's IQ4_XS dequantiser: d = 1, every group scale 33 (dl = 1), nibble k at element k
    blk = np.zeros(136, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.uint16(0xAAAA).tobytes(), np.uint8)  # high scale bits 2 for all eight groups: 32 + low nibble
    blk[4:8] = 0x11                                                   # low nibbles 1: ls = 33
    qs = blk[8:]
    for j in range(16):
        qs[j] = (j & 0x0F) | (((j + 1) & 0x0F) << 4)  # element j: nibble j; element j + 16: nibble j + 1
    vals = oracle.dequantize(23, blk)[:16].astype(np.int64).tolist()
    assert _digest(vals, 1, signed=True) == want["KVALUES_IQ4NL"]["sha256"]


@pytest.mark.parametrize("quant", [16, 22, 18, 23])
def test_iq_dots_equal_the_dequantised_statement(oracle, quant):
    """dot(W, Q8_K(x)) restated independently: f64 sum of dequantise(W) * (d_x * q_x).  The integer forms of
    crates/rnb-cpu/src/gemm/neon_quant.rs:273-411 must give the same number to f32 rounding, the f64 gold form to 1e-12;
    a wrong sign bit, scale nibble or element order shows as an O(1) relative error."""
    nb = 6
    w = oracle.make_weights(quant, 5, nb * 256, 4242 + quant)
    x = oracle.fill_normal(nb * 256, 99 + quant, 1.0)
    act = oracle.quantize_q8k(x)
    xq = (act["d"][:, None].astype(np.float64) * act["qs"].astype(np.float64)).ravel()
    rb = nb * oracle.BLOCK_BYTES[quant]
    for r in range(5):
        row = w[r * rb:(r + 1) * rb]
        want = float(np.dot(oracle.dequantize(quant, row).astype(np.float64), xq))
        scale = float(np.sqrt(np.sum(oracle.dequantize(quant, row).astype(np.float64) ** 2) * np.sum(xq ** 2)))
        assert abs(oracle.dot(quant, row, act, gold=True) - want) <= 1e-9 * scale
        assert abs(oracle.dot(quant, row, act) - want) <= 2e-6 * scale


def test_iq_dot_hand_built_blocks(oracle):
    """One block, activations 1 (Q8_K codes 127 at d = 1/127): IQ4_XS with every nibble 8 (value +1) and scale code 33
    (+1) gives 256 * 127 * (1/127) = 256 = the reference's d * d_x * block_sum; raising the scale code of sub-block 3
    alone to 47 (+15) adds 14 * 32.  IQ2_XXS zero codes (every element decodes to 1.0): 256 as well."""
    x = np.ones(256, np.float32)
    act = oracle.quantize_q8k(x)
    b = np.zeros(136, np.uint8)
    b[:2] = _ONE_F16
    b[2:4] = (0xAA, 0xAA)
    b[4:8] = 0x11
    b[8:] = 0x88
    assert oracle.dot(23, b, act) == pytest.approx(256.0, rel=1e-6)
    b2 = b.copy()
    b2[5] = 0xF1  # scales_l[1]: sub-block 2 keeps low nibble 1, sub-block 3 gets 15 -> code 2 << 4 | 15 = 47 -> +15
    assert oracle.dot(23, b2, act) == pytest.approx(256.0 + 14 * 32, rel=1e-6)
    z = np.zeros(66, np.uint8)
    z[:2] = _ONE_F16
    assert oracle.dot(16, z, act) == pytest.approx(256.0, rel=1e-6)
