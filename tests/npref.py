"""Independent numpy statements of the public GGUF block formats, written from the format
description (field order, bit positions) with reshape/bit-twiddling rather than the oracle's
loops, so that an index or shift mistake in the oracle fails a comparison against these."""
import numpy as np


def f16_bytes(v) -> bytes:
    return np.array([v], dtype=np.float16).tobytes()


# ---- Q4_0 / Q4_1 / Q5_0 / Q5_1 (32-element blocks) ------------------------------------

LEGACY_LAYOUT = {2: (18, False, False), 3: (20, True, False), 6: (22, False, True), 7: (24, True, True)}  # bytes, min, qh


def make_legacy_block(quant, d, m, codes) -> np.ndarray:
    """codes: 32 unsigned codes (0..15, or 0..31 for the 5-bit formats) in element order.  Layout: f16 d, [f16 m],
    [u32 qh], qs[16]; element i < 16 in the low nibble of qs[i], element 16 + i in its high nibble, fifth bit of
    element e in bit e of qh."""
    _, has_min, has_qh = LEGACY_LAYOUT[quant]
    c = np.asarray(codes, dtype=np.uint32)
    parts = [np.frombuffer(f16_bytes(d), dtype=np.uint8)]
    if has_min:
        parts.append(np.frombuffer(f16_bytes(m), dtype=np.uint8))
    if has_qh:
        qh = int((((c >> 4) & 1) << np.arange(32, dtype=np.uint32)).sum())
        parts.append(np.frombuffer(np.array([qh], dtype="<u4").tobytes(), dtype=np.uint8))
    parts.append(((c[:16] & 15) | ((c[16:] & 15) << 4)).astype(np.uint8))
    return np.concatenate(parts).astype(np.uint8)


def make_q8_1_block(d, s, values) -> np.ndarray:
    """Q8_1 {f16 d, f16 s, i8 qs[32]} (crates/rnb-cpu/src/quantize/blocks.rs:54-59); s is carried, never read."""
    return np.concatenate([np.frombuffer(f16_bytes(d), dtype=np.uint8), np.frombuffer(f16_bytes(s), dtype=np.uint8),
                           np.asarray(values, dtype=np.int8).view(np.uint8)]).astype(np.uint8)


def dequant_q8_1_f64(blocks) -> np.ndarray:
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 36)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64)
    return (b[:, 4:36].copy().view(np.int8).astype(np.float64) * d).reshape(-1)


def dequant_legacy_f64(quant, blocks) -> np.ndarray:
    nbytes, has_min, has_qh = LEGACY_LAYOUT[quant]
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, nbytes)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64)
    off = 2
    m = np.zeros_like(d)
    if has_min:
        m = b[:, 2:4].copy().view(np.float16).astype(np.float64)
        off = 4
    code = np.zeros((b.shape[0], 32), dtype=np.int64)
    if has_qh:
        qh = b[:, off:off + 4].copy().view("<u4").astype(np.int64)
        code += ((qh >> np.arange(32)) & 1) << 4
        off += 4
    qs = b[:, off:off + 16].astype(np.int64)
    code += np.concatenate([qs & 15, qs >> 4], axis=1)
    if has_min:
        return (code * d + m).reshape(-1)
    return ((code - (16 if has_qh else 8)) * d).reshape(-1)


# ---- Q2_K ---------------------------------------------------------------------------

def make_q2k_block(d, dmin, sc, mn, values) -> np.ndarray:
    """values: 256 two-bit values in element order; sc, mn: sixteen 4-bit codes.  Layout {scales[16], qs[64], f16 d,
    f16 dmin}: element 128h + 32p + l keeps its two bits at bit 2p of qs[32h + l]; its sub-block is (128h + 32p + l) / 16."""
    v = np.asarray(values, dtype=np.uint8).reshape(2, 4, 32)  # half, bit pair, l
    qs = np.zeros((2, 32), dtype=np.uint8)
    for p in range(4):
        qs |= (v[:, p, :] & 3) << (2 * p)
    scales = (np.asarray(sc, dtype=np.uint8) & 15) | ((np.asarray(mn, dtype=np.uint8) & 15) << 4)
    return np.concatenate([scales, qs.reshape(64), np.frombuffer(f16_bytes(d), dtype=np.uint8),
                           np.frombuffer(f16_bytes(dmin), dtype=np.uint8)]).astype(np.uint8)


def dequant_q2k_f64(blocks) -> np.ndarray:
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 84)
    sc = (b[:, 0:16] & 15).astype(np.float64)
    mn = (b[:, 0:16] >> 4).astype(np.float64)
    d = b[:, 80:82].copy().view(np.float16).astype(np.float64).reshape(-1, 1)
    dmin = b[:, 82:84].copy().view(np.float16).astype(np.float64).reshape(-1, 1)
    qs = b[:, 16:80].reshape(-1, 2, 1, 32).astype(np.int64)
    val = ((qs >> (2 * np.arange(4)).reshape(1, 1, 4, 1)) & 3).reshape(-1, 256)  # half, pair, l == element order
    return (np.repeat(sc * d, 16, axis=1) * val - np.repeat(mn * dmin, 16, axis=1)).reshape(-1)


# ---- Q3_K ---------------------------------------------------------------------------

def make_q3k_block(d, codes, values) -> np.ndarray:
    """values: 256 signed values -4..3 in element order; codes: sixteen signed sub-block scales -32..31.  Layout
    {hmask[32], qs[64], scales[12], f16 d}: the stored value v + 4 keeps its low two bits as for Q2_K and its third bit
    in bit 4h + p of hmask[l]; the stored scale code + 32 keeps its low four bits in nibble k/8 of byte k%8 and its
    high two in bit pair k/4 of byte 8 + k%4."""
    u = (np.asarray(values, dtype=np.int64) + 4).astype(np.uint8).reshape(2, 4, 32)
    qs = np.zeros((2, 32), dtype=np.uint8)
    hm = np.zeros(32, dtype=np.uint8)
    for h in range(2):
        for p in range(4):
            qs[h] |= (u[h, p] & 3) << (2 * p)
            hm |= ((u[h, p] >> 2) & 1) << (4 * h + p)
    st = (np.asarray(codes, dtype=np.int64) + 32).astype(np.uint8)
    sb = np.zeros(12, dtype=np.uint8)
    sb[0:8] = (st[0:8] & 15) | ((st[8:16] & 15) << 4)
    for k in range(16):
        sb[8 + k % 4] |= ((st[k] >> 4) & 3) << (2 * (k // 4))
    return np.concatenate([hm, qs.reshape(64), sb, np.frombuffer(f16_bytes(d), dtype=np.uint8)]).astype(np.uint8)


def dequant_q3k_f64(blocks) -> np.ndarray:
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 110)
    hm = b[:, 0:32].astype(np.int64)
    qs = b[:, 32:96].reshape(-1, 2, 1, 32).astype(np.int64)
    sb = b[:, 96:108].astype(np.int64)
    d = b[:, 108:110].copy().view(np.float16).astype(np.float64).reshape(-1, 1)
    low = (qs >> (2 * np.arange(4)).reshape(1, 1, 4, 1)) & 3                        # [n, half, pair, l]
    bit = (hm[:, None, :] >> np.arange(8)[None, :, None]) & 1                        # [n, 4*half + pair, l]
    val = (low + 4 * bit.reshape(-1, 2, 4, 32) - 4).reshape(-1, 256)
    k = np.arange(16)
    lo4 = np.where(k < 8, sb[:, k % 8] & 15, sb[:, k % 8] >> 4)
    hi2 = (sb[:, 8 + k % 4] >> (2 * (k // 4))) & 3
    code = (lo4 | (hi2 << 4)) - 32
    return (np.repeat(code * d, 16, axis=1) * val).reshape(-1)


# ---- Q4_K ---------------------------------------------------------------------------

def pack_scales_k4(sc, mn) -> np.ndarray:
    """Inverse of the 6-bit unpack: 8 scales + 8 mins (0..63) -> 12 bytes."""
    sc = np.asarray(sc, dtype=np.uint8)
    mn = np.asarray(mn, dtype=np.uint8)
    q = np.zeros(12, dtype=np.uint8)
    q[0:4] = (sc[0:4] & 63) | ((sc[4:8] >> 4) << 6)
    q[4:8] = (mn[0:4] & 63) | ((mn[4:8] >> 4) << 6)
    q[8:12] = (sc[4:8] & 15) | ((mn[4:8] & 15) << 4)
    return q


def make_q4k_block(d, dmin, sc, mn, nibbles) -> np.ndarray:
    """nibbles: 256 values 0..15 in element order."""
    nib = np.asarray(nibbles, dtype=np.uint8).reshape(4, 2, 32)  # group, lo/hi half, l
    qs = (nib[:, 0, :] | (nib[:, 1, :] << 4)).reshape(128)
    return np.concatenate([
        np.frombuffer(f16_bytes(d), dtype=np.uint8), np.frombuffer(f16_bytes(dmin), dtype=np.uint8),
        pack_scales_k4(sc, mn), qs]).astype(np.uint8)


def split_q4k(blocks: np.ndarray):
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(-1)
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float64).reshape(-1)
    s = b[:, 4:16].astype(np.int64)
    sc = np.concatenate([s[:, 0:4] & 63, (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)], axis=1)
    mn = np.concatenate([s[:, 4:8] & 63, (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)], axis=1)
    qs = b[:, 16:144].reshape(-1, 4, 32).astype(np.int64)
    nib = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 256)  # group, half, l
    return d, dmin, sc, mn, nib


def dequant_q4k_f64(blocks) -> np.ndarray:
    d, dmin, sc, mn, nib = split_q4k(blocks)
    scale = np.repeat(sc, 32, axis=1) * d[:, None]
    minv = np.repeat(mn, 32, axis=1) * dmin[:, None]
    return (scale * nib - minv).reshape(-1)


# ---- Q5_K ---------------------------------------------------------------------------

def make_q5k_block(d, dmin, sc, mn, values) -> np.ndarray:
    """values: 256 five-bit values 0..31 in element order.  Layout {f16 d, f16 dmin, scales[12], qh[32], qs[128]}:
    element 64g + 32h + l keeps its low four bits in nibble h of qs[32g + l] and its fifth bit in bit 2g + h of
    qh[l]."""
    v = np.asarray(values, dtype=np.uint8).reshape(4, 2, 32)  # group, lo/hi half, l
    qs = ((v[:, 0, :] & 15) | ((v[:, 1, :] & 15) << 4)).reshape(128)
    qh = np.zeros(32, dtype=np.uint8)
    for g in range(4):
        for h in range(2):
            qh |= ((v[g, h, :] >> 4) & 1) << (2 * g + h)
    return np.concatenate([
        np.frombuffer(f16_bytes(d), dtype=np.uint8), np.frombuffer(f16_bytes(dmin), dtype=np.uint8),
        pack_scales_k4(sc, mn), qh, qs]).astype(np.uint8)


def split_q5k(blocks: np.ndarray):
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 176)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(-1)
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float64).reshape(-1)
    s = b[:, 4:16].astype(np.int64)
    sc = np.concatenate([s[:, 0:4] & 63, (s[:, 8:12] & 15) | ((s[:, 0:4] >> 6) << 4)], axis=1)
    mn = np.concatenate([s[:, 4:8] & 63, (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)], axis=1)
    qh = b[:, 16:48].astype(np.int64)                       # [n, l]
    qs = b[:, 48:176].reshape(-1, 4, 32).astype(np.int64)   # [n, group, l]
    bits = (qh[:, None, :] >> np.arange(8)[None, :, None]) & 1          # [n, bit, l], bit = 2*group + half
    low = np.stack([qs & 15, qs >> 4], axis=2).reshape(-1, 8, 32)       # [n, 2*group + half, l]
    return d, dmin, sc, mn, (low + 16 * bits).reshape(-1, 256)


def dequant_q5k_f64(blocks) -> np.ndarray:
    d, dmin, sc, mn, val = split_q5k(blocks)
    scale = np.repeat(sc, 32, axis=1) * d[:, None]
    minv = np.repeat(mn, 32, axis=1) * dmin[:, None]
    return (scale * val - minv).reshape(-1)


# ---- Q6_K ---------------------------------------------------------------------------

def make_q6k_block(d, scales, q6) -> np.ndarray:
    """q6: 256 values 0..63 (stored value, i.e. signed value + 32) in element order."""
    q = np.asarray(q6, dtype=np.uint8).reshape(2, 4, 32)  # half, quarter, l
    ql = np.zeros((2, 64), dtype=np.uint8)
    qh = np.zeros((2, 32), dtype=np.uint8)
    ql[:, 0:32] = (q[:, 0] & 15) | ((q[:, 2] & 15) << 4)
    ql[:, 32:64] = (q[:, 1] & 15) | ((q[:, 3] & 15) << 4)
    qh[:] = (q[:, 0] >> 4) | ((q[:, 1] >> 4) << 2) | ((q[:, 2] >> 4) << 4) | ((q[:, 3] >> 4) << 6)
    return np.concatenate([ql.reshape(-1), qh.reshape(-1),
                           np.asarray(scales, dtype=np.int8).view(np.uint8),
                           np.frombuffer(f16_bytes(d), dtype=np.uint8)]).astype(np.uint8)


def split_q6k(blocks):
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 210)
    ql = b[:, 0:128].reshape(-1, 2, 2, 32).astype(np.int64)   # half, which-32, l
    qh = b[:, 128:192].reshape(-1, 2, 32).astype(np.int64)    # half, l
    sc = b[:, 192:208].copy().view(np.int8).astype(np.int64)  # 16
    d = b[:, 208:210].copy().view(np.float16).astype(np.float64).reshape(-1)
    quarters = [
        (ql[:, :, 0] & 15) | ((qh & 3) << 4),
        (ql[:, :, 1] & 15) | (((qh >> 2) & 3) << 4),
        (ql[:, :, 0] >> 4) | (((qh >> 4) & 3) << 4),
        (ql[:, :, 1] >> 4) | (((qh >> 6) & 3) << 4),
    ]
    q = np.stack(quarters, axis=2).reshape(-1, 256) - 32  # half, quarter, l -> element order
    return d, sc, q


def dequant_q6k_f64(blocks) -> np.ndarray:
    d, sc, q = split_q6k(blocks)
    return (np.repeat(sc, 16, axis=1) * d[:, None] * q).reshape(-1)


# ---- Q8_0 ---------------------------------------------------------------------------

def make_q8_0_block(d, qs) -> np.ndarray:
    return np.concatenate([np.frombuffer(f16_bytes(d), dtype=np.uint8),
                           np.asarray(qs, dtype=np.int8).view(np.uint8)]).astype(np.uint8)


def split_q8_0(blocks):
    b = np.asarray(blocks, dtype=np.uint8).reshape(-1, 34)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(-1)
    q = b[:, 2:34].copy().view(np.int8).astype(np.int64)
    return d, q


def dequant_q8_0_f64(blocks) -> np.ndarray:
    d, q = split_q8_0(blocks)
    return (q * d[:, None]).reshape(-1)


# ---- activations --------------------------------------------------------------------

def quantize_q8k_np(x):
    """Independent numpy statement of the Q8_K activation block (ggml quantize_row_q8_K_ref):
    first max-|x| element keeps its sign; iscale = -127/max; d = 1/iscale; q = min(127, rne(iscale*x))."""
    x = np.asarray(x, dtype=np.float32).reshape(-1, 256)
    nb = x.shape[0]
    d = np.zeros(nb, dtype=np.float32)
    qs = np.zeros((nb, 256), dtype=np.int8)
    for b in range(nb):
        i = int(np.argmax(np.abs(x[b])))  # numpy argmax returns the first maximum
        mv = x[b, i]
        if mv == 0:
            continue
        iscale = np.float32(-127.0) / mv
        d[b] = np.float32(1.0) / iscale
        v = np.rint((iscale * x[b]).astype(np.float32)).astype(np.int32)  # rint = half-to-even
        qs[b] = np.minimum(v, 127).astype(np.int8)
    bsums = qs.astype(np.int16).reshape(nb, 16, 16).sum(axis=2).astype(np.int16)
    return d, qs, bsums


def quantize_q8_np(x):
    x = np.asarray(x, dtype=np.float32).reshape(-1, 32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    p = (x * inv[:, None]).astype(np.float32)
    r = np.sign(p) * np.floor(np.abs(p) + np.float32(0.5))  # half away from zero
    return d, np.clip(r, -128, 127).astype(np.int8)


def deq_act_q8k_f64(blocks) -> np.ndarray:
    return (blocks["qs"].astype(np.float64) * blocks["d"].astype(np.float64)[:, None]).reshape(-1)


def close_rows(actual, expected, rel=1e-3, abs_floor=None):
    """The reference's abs-or-rel row check (crates/rnb-backend/cuda/src/runtime/tests.rs:28525-28541):
    |a-e| <= max(abs_tol, rel*|e|) with abs_tol = rel * rms(expected) unless given."""
    a = np.asarray(actual, dtype=np.float64).ravel()
    e = np.asarray(expected, dtype=np.float64).ravel()
    if abs_floor is None:
        abs_floor = rel * float(np.sqrt(np.mean(e * e))) if e.size else 0.0
    tol = np.maximum(abs_floor, rel * np.abs(e))
    diff = np.abs(a - e)
    bad = np.nonzero(diff > tol)[0]
    return bad, diff, tol
