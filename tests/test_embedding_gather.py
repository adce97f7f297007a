"""Embedding gather (quant_embedding_gather, crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:1827-1975): rows of a
block-quantised matrix picked by token id and dequantised on the device.  The device values are compared bit for bit with
the oracle's dequantisers (pinned on the reference's known answers in test_oracle_pins.py); the float formats with numpy."""
import numpy as np
import pytest

Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 2, 3, 6, 7, 8, 9, 10, 11, 12, 13, 14
IQ2_XXS, IQ3_XXS, IQ2_S, IQ4_XS = 16, 18, 22, 23
F32, F16, BF16 = 0, 1, 30
BLOCK_FORMATS = [Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, IQ2_XXS, IQ3_XXS, IQ2_S, IQ4_XS]


def _bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def _expected(oracle, quant, w, rows, cols, ids):
    row_bytes = cols // oracle.BLOCK_ELEMS[quant] * oracle.BLOCK_BYTES[quant]
    table = w.reshape(rows, row_bytes)
    return np.concatenate([oracle.dequantize(quant, table[i]) for i in ids])


@pytest.mark.gpu
@pytest.mark.parametrize("quant", BLOCK_FORMATS)
def test_gather_equals_the_dequantiser_bit_for_bit(rnb, oracle, quant):
    """Rows that are not resident (only the named rows travel), then the same matrix prewarmed (read in place), then the
    device-output form: all three give the dequantiser's bits, repeats and the first and last row included."""
    rows, cols = 37, 768
    w = oracle.make_weights(quant, rows, cols, 900 + quant)
    ids = np.array([4, 0, 4, 36, 17, 36, 1], dtype=np.uint32)
    want = _expected(oracle, quant, w, rows, cols, ids)
    got = rnb.quant_embedding_gather(quant, w, rows, cols, ids)
    assert np.array_equal(_bits(got), _bits(want))
    rnb.prewarm([w])
    try:
        before = rnb.residency_stats()
        again = rnb.quant_embedding_gather(quant, w, rows, cols, ids)
        after = rnb.residency_stats()
        assert after["hits"] == before["hits"] + 1 and after["misses"] == before["misses"]
        assert np.array_equal(_bits(again), _bits(want))
        out = rnb.DeviceBuffer(ids.size * cols * 4)
        rnb.quant_embedding_gather_dev(quant, w, rows, cols, ids, out)
        rnb.sync()
        assert np.array_equal(out.to_host(np.uint32), _bits(want))
        out.free()
    finally:
        rnb.release(w)


@pytest.mark.gpu
def test_gather_extreme_codes(rnb, oracle):
    """Every code value and both signs of every scale appear: blocks of random bytes with finite f16 scales."""
    rng = np.random.default_rng(77)
    for quant in BLOCK_FORMATS:
        bb, be = oracle.BLOCK_BYTES[quant], oracle.BLOCK_ELEMS[quant]
        rows, cols = 9, 2 * be if be == 256 else 8 * be
        nblk = rows * (cols // be)
        w = rng.integers(0, 256, size=(nblk, bb), dtype=np.uint8)
        # the f16 fields (d, and dmin / m where the format has one) get finite values
        f16 = (rng.standard_normal((nblk, 2)) * 0.05).astype(np.float16).view(np.uint8).reshape(nblk, 4)
        d_off = {Q2_K: 80, Q3_K: 108, Q6_K: 208}.get(quant, 0)
        two = quant in (Q4_1, Q5_1, Q8_1, Q2_K, Q4_K, Q5_K)
        w[:, d_off:d_off + (4 if two else 2)] = f16[:, :4 if two else 2]
        w = w.reshape(-1)
        ids = np.arange(rows, dtype=np.uint32)[::-1].copy()
        want = _expected(oracle, quant, w, rows, cols, ids)
        assert np.isfinite(want).all()
        got = rnb.quant_embedding_gather(quant, w, rows, cols, ids)
        assert np.array_equal(_bits(got), _bits(want)), quant


@pytest.mark.gpu
def test_gather_touches_every_codebook_entry(rnb, oracle):
    """The device tables are expanded at compile time from packed words by code of their own: blocks whose index bytes
    run through ALL 256 / 1024 / 256 grid entries (signs and scales random) must dequantise to the oracle's bits, whose
    tables are pinned entry for entry on the reference's (test_iq_codebooks_equal_the_references_tables_entry_for_entry)."""
    rng = np.random.default_rng(99)
    for quant, n_blocks in ((IQ2_XXS, 8), (IQ2_S, 32), (IQ3_XXS, 4)):
        bb = oracle.BLOCK_BYTES[quant]
        w = rng.integers(0, 256, size=(n_blocks, bb), dtype=np.uint8)
        w[:, 0:2] = np.frombuffer(np.float16(0.03125).tobytes(), np.uint8)
        seen = set()
        for k in range(n_blocks):
            if quant == IQ2_XXS:
                for ib in range(8):
                    for l in range(4):
                        w[k, 2 + 8 * ib + l] = 32 * k + 4 * ib + l
                        seen.add(32 * k + 4 * ib + l)
            elif quant == IQ2_S:
                for i in range(32):
                    w[k, 2 + i] = 32 * (k % 8) + i
                    seen.add((32 * (k % 8) + i) | (k // 8) << 8)
                w[k, 66:74] = 0x55 * (k // 8)  # the two high bits of every index of the block
            else:
                for i in range(64):
                    w[k, 2 + i] = 64 * k + i
                    seen.add(64 * k + i)
        assert len(seen) == (1024 if quant == IQ2_S else 256)
        w = w.reshape(-1)
        ids = np.arange(n_blocks, dtype=np.uint32)
        got = rnb.quant_embedding_gather(quant, w, n_blocks, 256, ids)
        want = _expected(oracle, quant, w, n_blocks, 256, ids)
        assert np.array_equal(_bits(got), _bits(want)), f"quant {quant}"


@pytest.mark.gpu
def test_gather_float_tables(rnb):
    rng = np.random.default_rng(5)
    rows, cols = 11, 96
    ids = np.array([10, 0, 3, 3], dtype=np.uint32)
    f = rng.standard_normal((rows, cols)).astype(np.float32)
    f[0, :6] = [0.0, -0.0, np.inf, -np.inf, 1e-42, -3e38]
    got = rnb.quant_embedding_gather(F32, f.view(np.uint8).reshape(-1), rows, cols, ids)
    assert np.array_equal(_bits(got), _bits(f[ids].reshape(-1)))
    with np.errstate(over="ignore"):
        h = f.astype(np.float16)  # -3e38 becomes -inf
    h[0, 4] = np.float16(6e-8)  # subnormal half
    got = rnb.quant_embedding_gather(F16, h.view(np.uint8).reshape(-1), rows, cols, ids)
    assert np.array_equal(_bits(got), _bits(h[ids].astype(np.float32).reshape(-1)))
    b = (f.view(np.uint32) >> 16).astype(np.uint16)
    got = rnb.quant_embedding_gather(BF16, b.view(np.uint8).reshape(-1), rows, cols, ids)
    assert np.array_equal(_bits(got), (b[ids].astype(np.uint32) << 16).reshape(-1))


@pytest.mark.gpu
def test_gather_moves_only_the_named_rows(rnb, oracle):
    """The reference's own case (cuda tests.rs:12551-12590): 6 x 512 Q4_K, ids [4, 0, 4, 5]: nothing becomes resident and
    four rows (not six) cross the bus."""
    rows, cols = 6, 512
    w = oracle.make_weights(Q4_K, rows, cols, 127)
    ids = np.array([4, 0, 4, 5], dtype=np.uint32)
    rnb.quant_embedding_gather(Q4_K, w, rows, cols, ids)  # sizes the staging buffers
    stats0, res0, (h2d0, d2h0) = rnb.residency_stats(), rnb.resident_bytes(), rnb.transfer_counters()
    got = rnb.quant_embedding_gather(Q4_K, w, rows, cols, ids)
    stats1, res1, (h2d1, d2h1) = rnb.residency_stats(), rnb.resident_bytes(), rnb.transfer_counters()
    assert stats1["admissions"] == stats0["admissions"] and stats1["h2d_bytes"] == stats0["h2d_bytes"] and res1 == res0
    assert h2d1 - h2d0 == ids.size * (cols // 256) * 144
    assert d2h1 - d2h0 == ids.size * cols * 4
    want = _expected(oracle, Q4_K, w, rows, cols, ids)
    assert np.abs(got - want).max() < 1e-6 and np.array_equal(_bits(got), _bits(want))


@pytest.mark.gpu
def test_gather_feeds_the_norm(rnb, oracle):
    """Token ids -> embedding rows on the device -> RMS norm + Q8_K -> projection, against the same chain from host rows."""
    rows, cols, out_rows = 50, 1024, 96
    emb = oracle.make_weights(Q6_K, rows, cols, 31)
    proj = oracle.make_weights(Q4_K, out_rows, cols, 32)
    ids = np.array([7, 49, 7], dtype=np.uint32)
    nw = np.linspace(0.5, 1.5, cols, dtype=np.float32)
    hidden = rnb.DeviceBuffer(ids.size * cols * 4)
    rnb.quant_embedding_gather_dev(Q6_K, emb, rows, cols, ids, hidden)
    nwd, pd = rnb.DeviceBuffer.from_host(nw), rnb.DeviceBuffer.from_host(proj)
    y = rnb.DeviceBuffer(ids.size * out_rows * 4)
    rnb.rms_norm_dev(hidden, nwd, 1e-6, ids.size, cols, None, quantize=True)
    rnb.gemv_quantized_dev(Q4_K, pd, out_rows, cols, ids.size, y)
    rnb.sync()
    got = y.to_host(np.float32).reshape(ids.size, out_rows)
    x = _expected(oracle, Q6_K, emb, rows, cols, ids).reshape(ids.size, cols)
    normed = oracle.rms_norm(x, nw, 1e-6)
    want = oracle.gemv(Q4_K, proj, out_rows, cols, normed)
    # the device norm rounds differently from the oracle's in the last place, which can move a quantised code by one
    assert np.abs(got - want).max() <= 1e-3 * np.sqrt((want.astype(np.float64) ** 2).mean())
    assert np.array_equal(_bits(got[0]), _bits(got[2]))
    for buf in (hidden, nwd, pd, y):
        buf.free()
