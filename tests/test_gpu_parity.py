"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle on identical
seeded inputs.  Activation quantisation must be bit-exact; f32 outputs must satisfy the reference's
abs-or-rel row check (crates/rnb-backend/cuda/src/runtime/tests.rs:28525-28541) with
rel = 1e-3 and abs floor = 1e-3 * rms(ref), and are additionally held to 2e-5 * rms against the
f64-accumulated form of the same integer arithmetic."""
import os
import numpy as np
import pytest

from tests import npref

pytestmark = pytest.mark.gpu

Q4_0, Q4_1, Q5_0, Q5_1, Q8_1 = 2, 3, 6, 7, 9
LEGACY = (Q4_0, Q4_1, Q5_0, Q5_1)
Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 8, 10, 11, 12, 13, 14
REL = 1e-3          # tolerance named by the task: max relative error 1e-3 per row
TIGHT = 2e-5        # what f32 summation-order differences actually allow, relative to rms


def check_close(got, ref, gold=None, label=""):
    assert np.all(np.isfinite(got)), f"{label}: non-finite output"
    bad, diff, tol = npref.close_rows(got, ref, rel=REL)
    assert bad.size == 0, f"{label}: {bad.size} rows outside max(1e-3*rms, 1e-3*|ref|); worst diff {diff.max()}"
    if gold is not None:
        g = np.asarray(gold, dtype=np.float64).ravel()
        rms = float(np.sqrt(np.mean(g * g))) or 1.0
        worst = float(np.abs(np.asarray(got, dtype=np.float64).ravel() - g).max())
        assert worst <= TIGHT * rms, f"{label}: |gpu - f64 gold| = {worst} > {TIGHT} * rms ({rms})"


def gemv_fn(rnb, quant, batch=False):
    table = {(Q4_0, False): rnb.q4_0_gemv, (Q4_0, True): rnb.q4_0_gemv_batch, (Q4_1, False): rnb.q4_1_gemv,
             (Q4_1, True): rnb.q4_1_gemv_batch, (Q5_0, False): rnb.q5_0_gemv, (Q5_0, True): rnb.q5_0_gemv_batch,
             (Q5_1, False): rnb.q5_1_gemv, (Q5_1, True): rnb.q5_1_gemv_batch, (Q2_K, False): rnb.q2k_gemv, (Q2_K, True): rnb.q2k_gemv_batch, (Q3_K, False): rnb.q3k_gemv,
             (Q3_K, True): rnb.q3k_gemv_batch, (Q4_K, False): rnb.q4k_gemv, (Q4_K, True): rnb.q4k_gemv_batch, (Q5_K, False): rnb.q5k_gemv,
             (Q5_K, True): rnb.q5k_gemv_batch, (Q6_K, False): rnb.q6k_gemv, (Q6_K, True): rnb.q6k_gemv_batch,
             (Q8_0, False): rnb.q8_0_gemv, (Q8_0, True): rnb.q8_0_gemv_batch,
             (Q8_1, False): rnb.q8_1_gemv, (Q8_1, True): rnb.q8_1_gemv_batch}
    return table[(quant, batch)]


# ---- activation quantisers: bit-exact ---------------------------------------------------------

def _q8k_inputs(oracle):
    rng = np.random.default_rng(100)
    cases = {}
    cases["gauss"] = oracle.fill_normal(512 * 4096 // 8, 1, 1.0)
    idx = np.arange(16 * 256)
    cases["ref_batch"] = ((idx * 73 + 19) % 2001).astype(np.float32) - 1000.0  # activation_q8.rs:221-224
    t = np.zeros(256 * 6, np.float32)
    t[256] = 127.0
    t[257:263] = [-0.5, -1.5, -2.5, 0.5, 1.5, 2.5]           # ties, activation_q8.rs:188-193
    t[512], t[513] = 127.0, -127.0                            # first-max sign rule
    t[768], t[769] = -127.0, 127.0
    t[1024 + 15], t[1024 + 16], t[1024 + 255] = -1.0, -2.0, 127.0  # bsums boundaries
    t[1280 + 200] = -3.0e-39                                  # subnormal-only block
    cases["reference_vectors"] = t
    tie = np.zeros(256, np.float32)
    tie[[7, 100, 255]] = [-2.0, 2.0, 2.0]                     # equal |x|: the first (negative) one must win
    cases["first_of_equal_magnitudes"] = tie
    cases["tiny_and_huge"] = np.concatenate([rng.standard_normal(256).astype(np.float32) * np.float32(1e-30),
                                             rng.standard_normal(256).astype(np.float32) * np.float32(1e30)])
    cases["half_integers"] = (rng.integers(-254, 255, 2048).astype(np.float32) * np.float32(0.5))
    nf = np.zeros(4 * 256, np.float32)                        # NaN and infinity: see test_quantisers_on_non_finite_inputs
    nf[0:256] = np.nan
    nf[256:512] = np.linspace(-1.0, 1.0, 256, dtype=np.float32)
    nf[256 + 17] = np.nan
    nf[512 + 3], nf[512 + 4] = np.inf, 5.0
    nf[768 + 9], nf[768 + 200] = -np.inf, np.nan
    cases["non_finite"] = nf
    return cases


def test_q8k_activation_quantiser_bit_exact(rnb, oracle):
    for name, x in _q8k_inputs(oracle).items():
        got = rnb.quantize_input_q8k(x)
        want = oracle.quantize_q8k(x)
        assert np.array_equal(got["d"].view(np.uint32), want["d"].view(np.uint32)), name
        assert np.array_equal(got["qs"], want["qs"]), name
        assert np.array_equal(got["bsums"], want["bsums"]), name
    b = rnb.quantize_input_q8k(_q8k_inputs(oracle)["reference_vectors"])
    assert b["d"][1] == -1.0 and b["qs"][1][1:7].tolist() == [0, 2, 2, 0, -2, -2]
    assert b["qs"][2][:2].tolist() == [-127, 127] and b["d"][3] == 1.0
    assert b["bsums"][4][0] == 1 and b["bsums"][4][1] == 2 and b["bsums"][4][15] == -127


def test_q8_activation_quantiser_bit_exact(rnb, oracle):
    rng = np.random.default_rng(101)
    xs = [oracle.fill_normal(4096, 2, 1.0), np.zeros(64, np.float32),
          rng.integers(-254, 255, 32 * 9).astype(np.float32) * np.float32(0.5),   # 9 blocks: ragged last wave
          rng.standard_normal(32 * 64 * 5 + 32).astype(np.float32) * np.float32(1e-20)]
    nf = np.zeros(3 * 32, np.float32)  # a NaN among finite values, an infinite block, a block of NaNs
    nf[0:32] = np.arange(32, dtype=np.float32) - 16.0
    nf[5] = np.nan
    nf[32 + 1], nf[32 + 2] = np.inf, 7.0
    nf[64:96] = np.nan
    xs.append(nf)
    for x in xs:
        got, want = rnb.quantize_input_q8(x), oracle.quantize_q8(x)
        assert np.array_equal(got["d"].view(np.uint32), want["d"].view(np.uint32))
        assert np.array_equal(got["qs"], want["qs"])


# ---- the reference's known-answer vectors through the device ------------------------------------

def test_reference_closed_forms_on_device(rnb):
    """crates/rnb-cpu/src/gemm/tile_q4k.rs:2019-2151 (0 / 0 / 2560 per row) and
    crates/rnb-cpu/src/gemm/quant_gemv.rs:1448-1464 (528, seq-major)."""
    rows = 8
    sc = np.zeros(8, np.int64)
    sc[0] = 10
    nib = np.full(256, 8)
    blk = npref.make_q4k_block(1.0, 0.0, sc, np.zeros(8), nib)
    w = np.tile(blk, rows)
    x = np.zeros(256, np.float32)
    x[:32] = 1.0  # Q8_K: d = -1/127, q = -127 -> d*q = 1 exactly per element
    out = rnb.q4k_gemv(w, rows, 256, x)
    assert np.allclose(out, 2560.0, rtol=1e-6)
    assert np.all(rnb.q4k_gemv(w, rows, 256, np.zeros(256, np.float32)) == 0.0)
    w0 = np.tile(npref.make_q4k_block(1.0, 1.0, np.zeros(8), np.zeros(8), nib), rows)
    assert np.all(rnb.q4k_gemv(w0, rows, 256, x) == 0.0)

    ref_bytes = np.frombuffer(bytes([0x00, 0x3C] + list(range(1, 33)) + [0x00, 0x3C] + list(range(32, 0, -1))),
                              dtype=np.uint8)
    out = rnb.q8_0_gemv_batch(ref_bytes, 2, 32, np.ones(64, np.float32))
    assert out.shape == (2, 2) and np.allclose(out, 528.0, rtol=1e-6)
    w2 = np.concatenate([npref.make_q8_0_block(1.0, np.ones(32)), npref.make_q8_0_block(1.0, 3 * np.ones(32))])
    x2 = np.concatenate([np.ones(32, np.float32), 2 * np.ones(32, np.float32)])
    assert np.allclose(rnb.q8_0_gemv_batch(w2, 2, 32, x2).ravel(), [32.0, 96.0, 64.0, 192.0], rtol=1e-6)


# ---- GEMV: shapes around every edge of the lane mapping ------------------------------------------

@pytest.mark.parametrize("quant", [Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, Q8_0])
@pytest.mark.parametrize("rows,nblk", [(1, 1), (3, 2), (4, 3), (5, 5), (7, 8), (9, 9), (64, 16), (33, 17), (6, 56),
                                       (5, 31), (130, 20), (9, 256), (2, 257)])
def test_gemv_small_shapes(rnb, oracle, quant, rows, nblk):
    cols = nblk * 256
    w = oracle.make_weights(quant, rows, cols, 1000 + rows * 31 + nblk)
    x = oracle.fill_normal(cols, 2000 + rows + nblk, 1.0)
    got = gemv_fn(rnb, quant)(w, rows, cols, x)
    ref = oracle.gemv(quant, w, rows, cols, x)[0]
    gold = oracle.gemv(quant, w, rows, cols, x, gold=True)[0]
    check_close(got, ref, gold, f"quant {quant} rows {rows} nblk {nblk}")


@pytest.mark.parametrize("quant", (Q8_0, Q8_1) + LEGACY)
@pytest.mark.parametrize("cols", [32, 96, 32 * 65, 32 * 129])
def test_block32_gemv_block_counts_off_the_wave_size(rnb, oracle, quant, cols):
    rows = 6
    w = oracle.make_weights(quant, rows, cols, 3000 + cols)
    x = oracle.fill_normal(cols, 3001 + cols, 1.0)
    check_close(gemv_fn(rnb, quant)(w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x)[0],
                oracle.gemv(quant, w, rows, cols, x, gold=True)[0], f"quant {quant} cols {cols}")


@pytest.mark.parametrize("quant", LEGACY)
def test_legacy_formats_shapes_batches_and_extremes(rnb, oracle, quant):
    """Q4_0 / Q4_1 / Q5_0 / Q5_1: decode shapes up to 4096x4096, small batches, and blocks at the ends of every field's
    range (all-max and all-zero codes, every fifth bit set, negative / zero / subnormal f16 scales and mins)."""
    for rows, cols in ((1, 32), (7, 1056), (300, 4096), (4096, 4096), (33, 11008)):
        w = oracle.make_weights(quant, rows, cols, 4000 + rows + quant)
        x = oracle.fill_normal(cols, 4001 + cols, 1.0)
        check_close(gemv_fn(rnb, quant)(w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x)[0],
                    oracle.gemv(quant, w, rows, cols, x, gold=True)[0], f"quant {quant} {rows}x{cols}")
        rnb.release(w)
    for seq in (2, 5, 17):
        rows, cols = 37, 768
        w = oracle.make_weights(quant, rows, cols, 4100 + quant)
        x = oracle.fill_normal(seq * cols, 4101 + seq, 1.0)
        got = gemv_fn(rnb, quant, True)(w, rows, cols, x)
        assert got.shape == (seq, rows)
        check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                    f"quant {quant} batch {seq}")
    rng = np.random.default_rng(29 + quant)
    top = 31 if quant in (Q5_0, Q5_1) else 15
    rows, nb32 = 8, 16
    x = oracle.fill_normal(nb32 * 32, 30, 1.0)
    x[64:96] = 0.0
    blocks = []
    for i in range(rows * nb32):
        codes = [np.full(32, top), np.zeros(32), rng.integers(0, top + 1, 32), np.full(32, 16 if top == 31 else 8)][i % 4]
        blocks.append(npref.make_legacy_block(quant, [1.0, -0.5, 6e-8, 0.0, 2.0 ** -14][i % 5], [0.25, -1.0, 0.0, 6e-8][i % 4],
                                              codes))
    w = np.concatenate(blocks)
    check_close(gemv_fn(rnb, quant)(w, rows, nb32 * 32, x), oracle.gemv(quant, w, rows, nb32 * 32, x)[0],
                oracle.gemv(quant, w, rows, nb32 * 32, x, gold=True)[0], f"quant {quant} extremes")


def test_q8_1_shapes_batches_and_extremes(rnb, oracle):
    """Q8_1 weights (crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:507-541): decode shapes (the large ones take the
    one-launch kernel), batches, and hand-built blocks with -128 / 127 codes, negative, zero and subnormal scales and an
    arbitrary stored sum (it must not be read)."""
    for rows, cols in ((1, 32), (7, 1056), (300, 4096), (4096, 4096), (33, 11008)):
        w = oracle.make_weights(Q8_1, rows, cols, 4200 + rows)
        x = oracle.fill_normal(cols, 4201 + cols, 1.0)
        check_close(rnb.q8_1_gemv(w, rows, cols, x), oracle.gemv(Q8_1, w, rows, cols, x)[0],
                    oracle.gemv(Q8_1, w, rows, cols, x, gold=True)[0], f"q8_1 {rows}x{cols}")
        rnb.release(w)
    for seq in (2, 5, 17):
        rows, cols = 37, 768
        w = oracle.make_weights(Q8_1, rows, cols, 4300)
        x = oracle.fill_normal(seq * cols, 4301 + seq, 1.0)
        got = rnb.q8_1_gemv_batch(w, rows, cols, x)
        assert got.shape == (seq, rows)
        check_close(got, oracle.gemv(Q8_1, w, rows, cols, x), oracle.gemv(Q8_1, w, rows, cols, x, gold=True), f"q8_1 batch {seq}")
    rng = np.random.default_rng(31)
    rows, nb32 = 8, 16
    x = oracle.fill_normal(nb32 * 32, 30, 1.0)
    x[64:96] = 0.0
    blocks = []
    for i in range(rows * nb32):
        codes = [np.full(32, 127), np.full(32, -128), rng.integers(-128, 128, 32), np.zeros(32)][i % 4]
        blocks.append(npref.make_q8_1_block([1.0, -0.5, 6e-8, 0.0, 2.0 ** -14][i % 5], [1e4, -3.0, 0.0][i % 3], codes))
    w = np.concatenate(blocks)
    check_close(rnb.q8_1_gemv(w, rows, nb32 * 32, x), oracle.gemv(Q8_1, w, rows, nb32 * 32, x)[0],
                oracle.gemv(Q8_1, w, rows, nb32 * 32, x, gold=True)[0], "q8_1 extremes")


def test_gemv_extreme_blocks(rnb, oracle):
    """all-max nibbles, negative Q6_K scales, zero / subnormal f16 scales, a zero activation block"""
    rng = np.random.default_rng(7)
    nblk, rows = 4, 8
    x = oracle.fill_normal(nblk * 256, 11, 1.0)
    x[256:512] = 0.0
    blocks = []
    for r in range(rows):
        for b in range(nblk):
            d = [1.0, 0.0, 6e-8, 2.0 ** -14][(r + b) % 4]
            blocks.append(npref.make_q4k_block(d, [0.5, 6e-8, 0.0, 1.0][(r + b) % 4], np.full(8, 63), np.full(8, 63),
                                               np.full(256, 15) if b % 2 == 0 else rng.integers(0, 16, 256)))
    w = np.concatenate(blocks)
    check_close(rnb.q4k_gemv(w, rows, nblk * 256, x), oracle.gemv(Q4_K, w, rows, nblk * 256, x)[0],
                oracle.gemv(Q4_K, w, rows, nblk * 256, x, gold=True)[0], "q4k extremes")
    blocks = []
    for r in range(rows):
        for b in range(nblk):
            d = [1.0, 0.0, 6e-8, 2.0 ** -14][(r + b) % 4]
            vals = [np.full(256, 31), rng.integers(0, 32, 256), np.tile([16, 15], 128), np.zeros(256)][(r + 2 * b) % 4]
            blocks.append(npref.make_q5k_block(d, [0.5, 6e-8, 0.0, 1.0][(r + b) % 4], np.full(8, 63), np.full(8, 63), vals))
    w = np.concatenate(blocks)
    check_close(rnb.q5k_gemv(w, rows, nblk * 256, x), oracle.gemv(Q5_K, w, rows, nblk * 256, x)[0],
                oracle.gemv(Q5_K, w, rows, nblk * 256, x, gold=True)[0], "q5k extremes")
    blocks = []
    for r in range(rows):
        for b in range(nblk):
            d = [1.0, -0.5, 6e-8, 0.0][(r + b) % 4]
            scales = np.full(16, -128) if b == 0 else rng.integers(-128, 128, 16)
            q = np.full(256, 63) if b == 1 else (np.zeros(256) if b == 2 else rng.integers(0, 64, 256))
            blocks.append(npref.make_q6k_block(d, scales, q))
    w = np.concatenate(blocks)
    check_close(rnb.q6k_gemv(w, rows, nblk * 256, x), oracle.gemv(Q6_K, w, rows, nblk * 256, x)[0],
                oracle.gemv(Q6_K, w, rows, nblk * 256, x, gold=True)[0], "q6k extremes")
    w = np.concatenate([npref.make_q8_0_block([1.0, 0.0, 6e-8, -2.0][i % 4],
                                              np.full(32, -128) if i % 3 == 0 else rng.integers(-128, 128, 32))
                        for i in range(rows * 32)])
    check_close(rnb.q8_0_gemv(w, rows, 1024, x), oracle.gemv(Q8_0, w, rows, 1024, x)[0],
                oracle.gemv(Q8_0, w, rows, 1024, x, gold=True)[0], "q8_0 extremes")


def test_unaligned_host_weights_and_subrange_residency(rnb, oracle):
    """Rows at odd host byte offsets must give identical results (crates/rnb-cpu/src/gemm/quant_gemv.rs:1257-1296);
    a sub-range of a resident parent resolves to parent + offset (crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:722-741)."""
    rows, cols = 16, 1024
    for quant in (Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, Q8_0):
        w = oracle.make_weights(quant, rows, cols, 42 + quant)
        x = oracle.fill_normal(cols, 43, 1.0)
        base = gemv_fn(rnb, quant)(w, rows, cols, x)
        buf = np.zeros(w.size + 3, np.uint8)
        buf[1:1 + w.size] = w
        shifted = buf[1:1 + w.size]
        assert shifted.ctypes.data % 2 == 1
        assert np.array_equal(gemv_fn(rnb, quant)(shifted, rows, cols, x), base)
        rnb.release(shifted)
        # parent resident, call with the second half of the rows
        rnb.prewarm([w])
        before = rnb.transfer_counters()[0]
        half = w[w.size // 2:]
        got = gemv_fn(rnb, quant)(half, rows // 2, cols, x)
        after = rnb.transfer_counters()[0]
        assert np.array_equal(got, base[rows // 2:])
        assert after - before == cols * 4, "the sub-range must not be uploaded again"
        rnb.release(w)


def test_resident_cache_notices_changed_bytes(rnb, oracle):
    rows, cols = 8, 512
    w = oracle.make_weights(Q4_K, rows, cols, 5).copy()
    x = oracle.fill_normal(cols, 6, 1.0)
    a = rnb.q4k_gemv(w, rows, cols, x)
    w[:] = oracle.make_weights(Q4_K, rows, cols, 6)
    b = rnb.q4k_gemv(w, rows, cols, x)
    check_close(b, oracle.gemv(Q4_K, w, rows, cols, x)[0], None, "changed bytes at the same address")
    assert not np.array_equal(a, b)
    rnb.release(w)


def test_unpinned_resident_never_serves_a_subrange(rnb, oracle):
    """Host memory of an unpinned resident may be freed and reused: a later, smaller weight tensor that lands
    inside the old address range must be uploaded, not resolved against the stale device copy."""
    rows, cols = 16, 512
    rb = cols // 256 * 144
    buf = np.zeros(rows * rb, np.uint8)
    buf[:] = oracle.make_weights(Q4_K, rows, cols, 31)
    x = oracle.fill_normal(cols, 32, 1.0)
    rnb.q4k_gemv(buf, rows, cols, x)                      # unpinned resident covering all of buf
    buf[:] = oracle.make_weights(Q4_K, rows, cols, 33)    # "freed and reused"
    inner = buf[4 * rb:12 * rb]
    got = rnb.q4k_gemv(inner, 8, cols, x)
    check_close(got, oracle.gemv(Q4_K, inner, 8, cols, x)[0], None, "sub-range of a stale unpinned resident")
    rnb.release(inner)
    rnb.q4k_gemv(buf, rows, cols, x)
    rnb.release(buf)


def test_gemv_into_and_zero_sized(rnb, oracle):
    rows, cols = 5, 512
    w = oracle.make_weights(Q6_K, rows, cols, 8)
    x = oracle.fill_normal(cols, 9, 1.0)
    out = np.full(rows + 3, -7.0, np.float32)
    rnb.q6k_gemv_into(w, rows, cols, x, out)
    assert np.array_equal(out[:rows], rnb.q6k_gemv(w, rows, cols, x)) and np.all(out[rows:] == -7.0)
    assert rnb.q4k_gemv(np.zeros(0, np.uint8), 0, 256, np.zeros(256, np.float32)).size == 0
    assert rnb.q4k_gemv_batch(np.zeros(144, np.uint8), 1, 256, np.zeros(0, np.float32)).shape == (0, 1)


@pytest.mark.parametrize("quant,rows,cols", [(Q4_K, 300, 4096), (Q4_K, 77, 2048), (Q4_K, 50, 768), (Q6_K, 300, 4096),
                                             (Q6_K, 64, 768), (Q8_0, 200, 4096), (Q8_0, 33, 1056), (Q6_K, 40, 14336),
                                             (Q5_K, 300, 4096), (Q5_K, 41, 1280), (Q5_K, 24, 14336),
                                             (Q2_K, 300, 4096), (Q2_K, 24, 14336), (Q3_K, 300, 4096), (Q3_K, 24, 14336),
                                             (Q4_K, 5, 256), (Q4_K, 20001, 256), (Q6_K, 9001, 1024), (Q5_K, 4099, 4096),
                                             (Q3_K, 8200, 2304), (Q8_0, 4100, 2048), (Q8_0, 5000, 2080), (2, 2100, 4096), (3, 8200, 1056),
                                             (6, 4100, 4096), (7, 90000, 96), (9, 4100, 2048), (9, 50, 96), (Q4_K, 4096, 14336), (Q6_K, 4099, 11008),
                                             (Q4_K, 37, 4352), (Q5_K, 300, 8192), (Q6_K, 9, 16384), (Q2_K, 100, 16640),
                                             (Q4_K, 33, 32768), (Q6_K, 21, 33024), (Q3_K, 4101, 5120), (Q6_K, 1030, 28672),
                                             (Q4_K, 20011, 8192), (Q2_K, 2050, 4608), (Q5_K, 7, 6144), (Q6_K, 8193, 8192),
                                             (Q4_K, 301, 12288), (Q2_K, 77, 8448), (Q6_K, 5, 12544),
                                             (Q5_K, 6200, 4352), (Q2_K, 10000, 4608), (Q3_K, 4097, 16384), (Q4_K, 1027, 13824)])
def test_gemv_dev_equals_split_quantise_then_gemv(rnb, oracle, quant, rows, cols):
    """rnb_hip_gemv_dev and its two halves (rnb_hip_quantize_dev + rnb_hip_gemv_quantized_dev, for callers that
    feed several matrices from one activation) run the same arithmetic: identical bits.  For K-quant rows of at most
    64 super-blocks, and 32-element formats with rows of at most 128 blocks, gemv_dev is a one-launch kernel whose
    workgroups quantise the token themselves (from 17 super-blocks on as split-K teams inside sixteen-wave workgroups,
    with one or two rows per team requested before the token is quantised; longer rows keep the separate quantiser);
    the shapes cover 1, 2 and 4 rows per wave, row counts that are no multiple of those or of the teams, more row groups
    than waves, launches of one to ten passes, and 2 to 9 K slices with full and partly idle last slices."""
    w = oracle.make_weights(quant, rows, cols, 900 + rows)
    x = oracle.fill_normal(cols, 901 + cols, 1.0)
    wd, xd = rnb.DeviceBuffer.from_host(w), rnb.DeviceBuffer.from_host(x)
    o1, o2 = rnb.DeviceBuffer(rows * 4), rnb.DeviceBuffer(rows * 4)
    rnb.gemv_dev(quant, wd, rows, cols, xd, 1, o1)
    rnb.quantize_dev(quant, xd, 1, cols)
    rnb.gemv_quantized_dev(quant, wd, rows, cols, 1, o2)
    rnb.sync()
    a, b = o1.to_host(np.float32), o2.to_host(np.float32)
    assert np.array_equal(a, b)
    check_close(a, oracle.gemv(quant, w, rows, cols, x)[0], oracle.gemv(quant, w, rows, cols, x, gold=True)[0],
                f"device-resident decode quant {quant} {rows}x{cols}")
    for buf in (wd, xd, o1, o2):
        buf.free()


@pytest.mark.parametrize("quant,rows,cols", [(Q6_K, 100, 5120), (Q6_K, 33, 14336), (Q4_K, 100, 5120), (Q5_K, 33, 11008),
                                             (Q6_K, 50, 2048)])
@pytest.mark.parametrize("shift", [1, 2, 3])
def test_gemv_sub_range_at_unaligned_device_address(rnb, oracle, quant, rows, cols, shift):
    """A matrix that is a sub-range of a resident parent, 1, 2 or 3 bytes in, is read at parent + offset on the device
    (crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:722-741) and gives the bits of the aligned one (the reference
    reads rows at any byte offset, crates/rnb-cpu/src/gemm/quant_gemv.rs:1257-1296).  Rows of 17 to 64 super-blocks: the
    one-launch kernel fetches Q6_K blocks without the odd-address path, so a Q6_K matrix at an odd address must take the
    quantiser + GEMV route."""
    w = oracle.make_weights(quant, rows, cols, 77 + rows)
    x = oracle.fill_normal(cols, 78, 1.0)
    base = gemv_fn(rnb, quant)(w, rows, cols, x)
    rnb.release(w)
    parent = np.zeros(w.size + 8, np.uint8)
    parent[shift:shift + w.size] = w
    rnb.prewarm([parent])
    before = rnb.transfer_counters()[0]
    got = gemv_fn(rnb, quant)(parent[shift:shift + w.size], rows, cols, x)
    assert rnb.transfer_counters()[0] - before == cols * 4, "the sub-range must not be uploaded again"
    assert np.array_equal(got, base)
    check_close(got, oracle.gemv(quant, w, rows, cols, x)[0], None, f"quant {quant} {rows}x{cols}")
    rnb.release(parent)


# ---- batches: seq-major layout, ragged token counts ----------------------------------------------

@pytest.mark.parametrize("quant", [Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, Q8_0])
@pytest.mark.parametrize("seq", [2, 3, 4, 9, 15, 33])
def test_gemv_batch_small(rnb, oracle, quant, seq):
    rows, cols = 37, 768
    w = oracle.make_weights(quant, rows, cols, 50 + quant)
    x = oracle.fill_normal(seq * cols, 60 + seq, 1.0)
    got = gemv_fn(rnb, quant, True)(w, rows, cols, x)
    assert got.shape == (seq, rows)
    check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                f"batch quant {quant} seq {seq}")


@pytest.mark.parametrize("quant,rows,cols", [(Q4_K, 300, 4096), (Q6_K, 131, 2048), (Q5_K, 70, 1024), (Q2_K, 257, 3072),
                                             (Q3_K, 90, 512), (Q6_K, 45, 14336), (Q4_K, 33, 8192), (Q3_K, 21, 5120),
                                             (Q8_0, 200, 4096), (Q8_0, 77, 1056), (Q4_0, 130, 4096), (Q5_1, 64, 2080),
                                             (Q4_1, 99, 96), (Q8_1, 50, 4096), (Q5_0, 41, 4096)])
def test_small_batches_equal_one_token_calls_bit_for_bit(rnb, oracle, quant, rows, cols):
    """Two to eight tokens run the GEMV kernels that fetch and unpack every weight block once and dot it against the
    activation slices of up to four tokens held in registers (row loop, K split for rows of more than 16 super-blocks,
    the 32-element formats with and without paired blocks): per token the same sums in the same order as the one-token
    kernel, so every row of the batch equals the one-token call."""
    w = oracle.make_weights(quant, rows, cols, 2300 + rows)
    one = gemv_fn(rnb, quant, batch=False)
    many = gemv_fn(rnb, quant, batch=True)
    x = oracle.fill_normal(8 * cols, 2301 + cols, 1.0)
    alone = np.stack([one(w, rows, cols, x[t * cols:(t + 1) * cols]) for t in range(8)])
    for seq in (2, 3, 4, 5, 7, 8):
        got = many(w, rows, cols, x[:seq * cols]).reshape(seq, rows)
        assert np.array_equal(got.view(np.uint32), alone[:seq].view(np.uint32)), (quant, rows, cols, seq)
    check_close(alone, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                f"small batches quant {quant} {rows}x{cols}")
    rnb.release(w)


@pytest.mark.parametrize("quant", [Q2_K, Q3_K, Q4_K, Q5_K, Q6_K])
def test_gemv_batch_long_rows(rnb, oracle, quant):
    """Rows longer than 16 super-blocks in small batches: the K-split kernel with groups of up to four tokens per pass
    (3, then 4 + 4 + 3, then 3 + 3); rows beyond the K-split kernel's 256 super-blocks keep one pass per token (the row
    loop walks them in passes of 16 super-blocks)."""
    for rows, cols, seq in ((21, 20 * 256, 3), (19, 20 * 256, 11), (5, 56 * 256, 6), (3, 257 * 256, 2)):
        w = oracle.make_weights(quant, rows, cols, 150 + quant)
        x = oracle.fill_normal(seq * cols, 160, 1.0)
        got = gemv_fn(rnb, quant, True)(w, rows, cols, x)
        check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                    f"long-row batch quant {quant} rows {rows} seq {seq}")


@pytest.mark.parametrize("rows,nblk,seq", [(32, 1, 32), (31, 2, 17), (33, 3, 17), (64, 4, 129), (100, 2, 33), (40, 20, 18),
                                           (1, 1, 17), (257, 5, 40), (4097, 1, 513), (8200, 2, 260), (2050, 9, 260),
                                           (8192, 8, 65)])
def test_q4k_gemm_mfma_ragged_tiles(rnb, oracle, rows, nblk, seq):
    """Q4_K batches on the matrix cores: shapes with fewer than 32 tiles of 256 rows x 64 tokens take the 128 x 32 / 64 kernel of
    gemm_blocks.hip, the last four the ping-pong kernel of gemm_q4k.hip: 153 and 165 tiles, both dimensions off the
    tile, then 45 and 64 tiles, where K is cut into two slices (5 + 4 blocks, 4 + 4) that a second kernel adds."""
    cols = nblk * 256
    w = oracle.make_weights(Q4_K, rows, cols, 70 + rows)
    x = oracle.fill_normal(seq * cols, 80 + seq, 1.0)
    got = rnb.q4k_gemv_batch(w, rows, cols, x)
    check_close(got, oracle.gemv(Q4_K, w, rows, cols, x), oracle.gemv(Q4_K, w, rows, cols, x, gold=True),
                f"gemm rows {rows} nblk {nblk} seq {seq}")


@pytest.mark.parametrize("rows,nblk,seq", [(32, 1, 32), (31, 2, 17), (33, 3, 17), (64, 4, 129), (100, 2, 33), (40, 20, 18),
                                           (1, 1, 17), (257, 5, 40), (129, 1, 65), (4096, 2, 64)])
def test_q6k_gemm_mfma_ragged_tiles(rnb, oracle, rows, nblk, seq):
    """Batches on Q6_K take the matrix-core GEMM (one K=16 instruction per sub-block, sub-block scales on
    the vector units): row and token counts off the 128 x 32 / 64 tile, one token tile and two."""
    cols = nblk * 256
    w = oracle.make_weights(Q6_K, rows, cols, 170 + rows)
    x = oracle.fill_normal(seq * cols, 180 + seq, 1.0)
    got = rnb.q6k_gemv_batch(w, rows, cols, x)
    check_close(got, oracle.gemv(Q6_K, w, rows, cols, x), oracle.gemv(Q6_K, w, rows, cols, x, gold=True),
                f"q6k gemm rows {rows} nblk {nblk} seq {seq}")
    # a token's row does not depend on the batch around it: the same bits with the tokens reversed
    rev = rnb.q6k_gemv_batch(w, rows, cols, x.reshape(seq, cols)[::-1].copy())
    assert np.array_equal(rev[::-1], got)


def test_q6k_gemm_extreme_blocks(rnb, oracle):
    """every 6-bit code at both ends of its range, scales -128 / 127 / 0, zero and subnormal d, zero activations"""
    rng = np.random.default_rng(19)
    rows, nblk, seq = 40, 3, 24
    blocks = []
    for i in range(rows * nblk):
        q = [np.full(256, 63), np.zeros(256), rng.integers(0, 64, 256), np.tile([0, 63], 128)][i % 4]
        sc = [np.full(16, 127), np.full(16, -128), rng.integers(-128, 128, 16), np.zeros(16)][(i // 4) % 4]
        blocks.append(npref.make_q6k_block([1.0, 6e-8, 0.0, 2.0 ** -14, -0.5][i % 5], sc, q))
    w = np.concatenate(blocks)
    x = oracle.fill_normal(seq * nblk * 256, 18, 1.0).reshape(seq, -1)
    x[3, 256:512] = 0.0
    x[5] = 0.0
    got = rnb.q6k_gemv_batch(w, rows, nblk * 256, x)
    assert np.all(got[5] == 0.0)
    check_close(got, oracle.gemv(Q6_K, w, rows, nblk * 256, x), oracle.gemv(Q6_K, w, rows, nblk * 256, x, gold=True),
                "q6k gemm extremes")


@pytest.mark.parametrize("rows,nblk,seq", [(32, 1, 32), (31, 2, 17), (33, 3, 17), (64, 4, 129), (100, 2, 33), (40, 20, 18),
                                           (1, 1, 17), (257, 5, 40), (129, 1, 65), (4096, 2, 64)])
def test_q5k_gemm_mfma_ragged_tiles(rnb, oracle, rows, nblk, seq):
    """Batches on Q5_K: one K=32 matrix instruction per sub-block, 6-bit scales on the vector units, the mins
    term through the quantiser's digits."""
    cols = nblk * 256
    w = oracle.make_weights(Q5_K, rows, cols, 470 + rows)
    x = oracle.fill_normal(seq * cols, 480 + seq, 1.0)
    got = rnb.q5k_gemv_batch(w, rows, cols, x)
    check_close(got, oracle.gemv(Q5_K, w, rows, cols, x), oracle.gemv(Q5_K, w, rows, cols, x, gold=True),
                f"q5k gemm rows {rows} nblk {nblk} seq {seq}")
    rev = rnb.q5k_gemv_batch(w, rows, cols, x.reshape(seq, cols)[::-1].copy())
    assert np.array_equal(rev[::-1], got)


def test_q5k_gemm_extreme_blocks(rnb, oracle):
    """all-31 and all-0 codes, alternating 16 / 15 (fifth bit on and off), scales and mins 63, zero / subnormal d and
    dmin, activations whose 32-element sums reach the digits' ends (all 127, all -127 -> rounds to -127), a zero token"""
    rng = np.random.default_rng(23)
    rows, nblk, seq = 40, 3, 24
    blocks = []
    for i in range(rows * nblk):
        vals = [np.full(256, 31), rng.integers(0, 32, 256), np.tile([16, 15], 128), np.zeros(256)][i % 4]
        blocks.append(npref.make_q5k_block([1.0, 0.0, 6e-8, 2.0 ** -14][i % 4], [0.5, 6e-8, 0.0, 1.0][(i // 2) % 4],
                                           np.full(8, 63) if i % 3 else rng.integers(0, 64, 8),
                                           np.full(8, 63) if i % 5 else rng.integers(0, 64, 8), vals))
    w = np.concatenate(blocks)
    x = oracle.fill_normal(seq * nblk * 256, 18, 1.0).reshape(seq, -1)
    x[3, 256:512] = 0.0
    x[5] = 0.0
    x[7] = 3.0       # every quantised value 127... the sign rule makes them -127: sums at the negative end
    x[8] = -3.0
    got = rnb.q5k_gemv_batch(w, rows, nblk * 256, x)
    assert np.all(got[5] == 0.0)
    check_close(got, oracle.gemv(Q5_K, w, rows, nblk * 256, x), oracle.gemv(Q5_K, w, rows, nblk * 256, x, gold=True),
                "q5k gemm extremes")


@pytest.mark.parametrize("quant,rows,cols,seq", [(Q4_K, 8192, 4096, 4), (Q4_K, 8192, 4096, 5), (Q5_K, 6144, 4096, 6),
                                                 (Q6_K, 4096, 5120, 6), (Q6_K, 4096, 5120, 7), (Q8_0, 4096, 4096, 6),
                                                 (Q8_0, 4096, 4096, 7), (Q8_1, 4096, 4096, 15), (Q4_K, 4096, 4096, 6),
                                                 (Q4_K, 4096, 4096, 8), (Q6_K, 2048, 4096, 8), (Q6_K, 2048, 4096, 11),
                                                 (Q4_0, 4096, 4096, 8), (Q4_0, 4096, 4096, 9), (Q2_K, 8192, 4096, 7),
                                                 (Q3_K, 8192, 4096, 9), (Q5_K, 6144, 4096, 12), (Q4_K, 8192, 4096, 12),
                                                 (Q5_1, 4096, 4096, 13)])
def test_gemm_few_tokens(rnb, oracle, quant, rows, cols, seq):
    """Either side of the token count at which a format's matrix-core GEMM takes over from the GEMV kernels that keep two
    to four tokens in registers (5 for Q4_K / Q5_K, 7 for Q6_K, Q2_K, Q3_K, Q8_0, Q8_1, 9 for the nibble formats; two more
    under 16 MB): on the GEMV side groups of 4, 3 + 3, 4 + 4 tokens, on the GEMM side a 32-token tile mostly empty (loads
    of the missing tokens repeat the last one, their results are not stored; up to 8 / 16 tokens the kernels that finish
    only the first 4 / 8 results of a lane)."""
    w = oracle.make_weights(quant, rows, cols, 1200 + seq)
    x = oracle.fill_normal(seq * cols, 1210 + seq, 1.0)
    got = gemv_fn(rnb, quant, batch=True)(w, rows, cols, x)
    check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                f"few tokens quant {quant} rows {rows} cols {cols} seq {seq}")
    rev = gemv_fn(rnb, quant, batch=True)(w, rows, cols, x.reshape(seq, cols)[::-1].copy())
    assert np.array_equal(rev[::-1], got)


@pytest.mark.parametrize("quant", [Q4_K, Q5_K, Q6_K, Q8_0, Q8_1, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K])
@pytest.mark.parametrize("rows,nblk,seq", [(128, 37, 17), (200, 11, 48), (4096, 16, 64), (1024, 8, 96)])
def test_gemm_k_slices(rnb, oracle, quant, rows, nblk, seq):
    """Grids too small for the chip are cut along K (blockIdx.z) and the slices' outputs added by a second kernel in
    slice order: 13 slices of 3 blocks and one of 1 (the cap of 16 slices asked for), slices of unequal length, and the
    two shapes where every slice has whole steps.  The sum does not depend on the batch around a token."""
    cols = nblk * 256
    w = oracle.make_weights(quant, rows, cols, 900 + rows)
    x = oracle.fill_normal(seq * cols, 910 + seq, 1.0)
    got = gemv_fn(rnb, quant, batch=True)(w, rows, cols, x)
    check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                f"k slices quant {quant} rows {rows} nblk {nblk} seq {seq}")
    rev = gemv_fn(rnb, quant, batch=True)(w, rows, cols, x.reshape(seq, cols)[::-1].copy())
    assert np.array_equal(rev[::-1], got)


@pytest.mark.parametrize("quant", [Q2_K, Q3_K])
@pytest.mark.parametrize("rows,nblk,seq", [(32, 1, 32), (31, 2, 17), (33, 3, 17), (64, 4, 129), (100, 2, 33), (1, 1, 17),
                                           (257, 5, 40), (129, 1, 65), (640, 3, 600)])
def test_q2k_q3k_gemm_mfma_ragged_tiles(rnb, oracle, quant, rows, nblk, seq):
    """Batches on Q2_K / Q3_K take the matrix-core GEMM (one K=16 instruction per 16-element sub-block, its scale on the
    vector units; Q2_K's mins through the activations' 16-element sums as two int8 digits): rows and tokens off the
    128 x 32 / 64 tile, one token tile and several, the last shape with 64-token workgroups."""
    cols = nblk * 256
    w = oracle.make_weights(quant, rows, cols, 370 + rows)
    x = oracle.fill_normal(seq * cols, 380 + seq, 1.0)
    got = gemv_fn(rnb, quant, True)(w, rows, cols, x)
    check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                f"q2k/q3k gemm quant {quant} rows {rows} nblk {nblk} seq {seq}")
    rev = gemv_fn(rnb, quant, True)(w, rows, cols, x.reshape(seq, cols)[::-1].copy())
    assert np.array_equal(rev[::-1], got)


@pytest.mark.parametrize("quant", [Q8_0, Q8_1, Q4_0, Q4_1, Q5_0, Q5_1])
@pytest.mark.parametrize("rows,cols,seq", [(32, 32, 17), (31, 96, 17), (33, 1056, 33), (130, 2080, 64), (257, 256, 65),
                                           (1, 4096, 17), (300, 288, 100)])
def test_q8_gemm_mfma_ragged_tiles(rnb, oracle, quant, rows, cols, seq):
    """Batches on the 32-element formats take the matrix-core GEMM (one K=32 instruction per block, the two f32 scales
    on the vector units; the nibble formats' codes are split, given their fifth bit and offset in packed bytes, the
    d n + m formats add m times the block's sum of activations from a second instruction against ones): block counts off
    the 8-block step, rows and tokens off the tile."""
    w = oracle.make_weights(quant, rows, cols, 270 + rows)
    x = oracle.fill_normal(seq * cols, 280 + seq, 1.0)
    got = gemv_fn(rnb, quant, True)(w, rows, cols, x)
    check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                f"q8 gemm quant {quant} rows {rows} cols {cols} seq {seq}")
    rev = gemv_fn(rnb, quant, True)(w, rows, cols, x.reshape(seq, cols)[::-1].copy())
    assert np.array_equal(rev[::-1], got)


def test_q4k_gemm_extreme_blocks(rnb, oracle):
    rng = np.random.default_rng(17)
    rows, nblk, seq = 40, 3, 24
    blocks = [npref.make_q4k_block([1.0, 0.0, 6e-8, 2.0 ** -14][i % 4], [0.5, 1.0, 0.0, 6e-8][i % 4],
                                   np.full(8, 63) if i % 2 else rng.integers(0, 64, 8), rng.integers(0, 64, 8),
                                   np.full(256, 15) if i % 3 == 0 else rng.integers(0, 16, 256))
              for i in range(rows * nblk)]
    w = np.concatenate(blocks)
    x = oracle.fill_normal(seq * nblk * 256, 18, 1.0).reshape(seq, -1)
    x[3, 256:512] = 0.0
    x[5] = 0.0
    got = rnb.q4k_gemv_batch(w, rows, nblk * 256, x)
    assert np.all(got[5] == 0.0)
    check_close(got, oracle.gemv(Q4_K, w, rows, nblk * 256, x), oracle.gemv(Q4_K, w, rows, nblk * 256, x, gold=True),
                "gemm extremes")


# ---- the BASELINE configurations at full size ------------------------------------------------------

def _full_gemv(rnb, oracle, quant, rows, cols, name):
    w = oracle.make_weights(quant, rows, cols, oracle.tensor_seed(name, "weight"))
    x = oracle.fill_normal(cols, oracle.tensor_seed(name, "x"), 1.0)
    got = gemv_fn(rnb, quant)(w, rows, cols, x)
    ref = oracle.gemv(quant, w, rows, cols, x)[0]
    gold = oracle.gemv(quant, w, rows, cols, x, gold=True)[0]
    check_close(got, ref, gold, name)
    # size-independent properties: x -> 2x doubles every output bit-for-bit (power-of-two scaling commutes
    # with the activation quantiser), x = 0 gives exact zeros, and reversing the row order reverses the output
    assert np.array_equal(gemv_fn(rnb, quant)(w, rows, cols, 2.0 * x), 2.0 * got)
    assert np.all(gemv_fn(rnb, quant)(w, rows, cols, np.zeros(cols, np.float32)) == 0.0)
    rb = w.size // rows
    w_rev = np.ascontiguousarray(w.reshape(rows, rb)[::-1]).reshape(-1)
    assert np.array_equal(gemv_fn(rnb, quant)(w_rev, rows, cols, x), got[::-1])
    rnb.release(w_rev)
    rnb.release(w)


def test_config1_q8_0_gemv_4096x4096(rnb, oracle):
    _full_gemv(rnb, oracle, Q8_0, 4096, 4096, "cfg1")


def test_config2_q4k_gemv_14336x4096(rnb, oracle):
    _full_gemv(rnb, oracle, Q4_K, 14336, 4096, "cfg2")


def test_config3a_q6k_gemv_4096x14336(rnb, oracle):
    _full_gemv(rnb, oracle, Q6_K, 4096, 14336, "cfg3a")


def test_config3b_q6k_gemv_lm_head_128256x4096(rnb, oracle):
    _full_gemv(rnb, oracle, Q6_K, 128256, 4096, "cfg3b")


@pytest.mark.parametrize("quant,rows,cols,seq", [(Q4_K, 21001, 4096, 1), (Q6_K, 15003, 4096, 1), (Q5_K, 17921, 4096, 3),
                                                 (Q4_K, 38839, 2304, 2), (Q2_K, 40001, 4096, 1), (Q3_K, 30001, 4096, 1),
                                                 (Q6_K, 15003, 4096, 4)])
def test_gemv_chunked_rows_kernel_large_matrices(rnb, oracle, quant, rows, cols, seq):
    """Matrices of 48 MB and more with rows of 9 to 16 super-blocks take the kernel whose waves each reduce a chunk of
    consecutive rows (two, four for Q6_K): row counts that are no multiple of the chunk, 9 super-blocks per row (idle
    lanes), and two to four tokens (their activation slices kept in registers, one pass over the matrix).  The arithmetic
    per row is the grid-stride kernel's, so the first 4096 rows alone, a matrix small enough for that kernel, give the
    same bits."""
    w = oracle.make_weights(quant, rows, cols, 7000 + rows)
    x = oracle.fill_normal(seq * cols, 7001 + rows, 1.0)
    fn = gemv_fn(rnb, quant, batch=seq > 1)
    got = fn(w, rows, cols, x).reshape(seq, rows)
    check_close(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
                f"chunked GEMV quant {quant} {rows}x{cols} seq {seq}")
    rb = w.size // rows
    head = w[:4096 * rb].copy()
    small = fn(head, 4096, cols, x).reshape(seq, 4096)
    assert np.array_equal(small.view(np.uint32), got[:, :4096].view(np.uint32))
    rnb.release(head)
    rnb.release(w)


def test_q5k_gemv_full_size_14336x4096_and_4096x14336(rnb, oracle):
    """Q5_K at the up- and down-projection shapes of the Q4_K / Q6_K configurations."""
    _full_gemv(rnb, oracle, Q5_K, 14336, 4096, "q5k_up")
    _full_gemv(rnb, oracle, Q5_K, 4096, 14336, "q5k_down")


def test_q2k_q3k_gemv_full_size_and_extremes(rnb, oracle):
    """Q2_K and Q3_K at the 14336x4096 shape of the Q4_K configuration, then blocks at the ends of every field's range
    (all-max and all-min values, scale codes -32 and 31, zero and subnormal f16 scales, a zero activation block)."""
    _full_gemv(rnb, oracle, Q2_K, 14336, 4096, "q2k_up")
    _full_gemv(rnb, oracle, Q3_K, 14336, 4096, "q3k_up")
    rng = np.random.default_rng(27)
    nblk, rows = 4, 8
    x = oracle.fill_normal(nblk * 256, 28, 1.0)
    x[512:768] = 0.0
    b2, b3 = [], []
    for r in range(rows):
        for b in range(nblk):
            d = [1.0, 0.0, 6e-8, 2.0 ** -14][(r + b) % 4]
            b2.append(npref.make_q2k_block(d, [0.5, 6e-8, 0.0, 1.0][(r + b) % 4], np.full(16, 15), np.full(16, 15),
                                           [np.full(256, 3), rng.integers(0, 4, 256), np.zeros(256)][(r + b) % 3]))
            b3.append(npref.make_q3k_block([1.0, -0.5, 6e-8, 0.0][(r + b) % 4],
                                           [np.full(16, -32), np.full(16, 31), rng.integers(-32, 32, 16)][(r + 2 * b) % 3],
                                           [np.full(256, -4), np.full(256, 3), rng.integers(-4, 4, 256)][(r + b) % 3]))
    for quant, blocks in ((Q2_K, b2), (Q3_K, b3)):
        w = np.concatenate(blocks)
        check_close(gemv_fn(rnb, quant)(w, rows, nblk * 256, x), oracle.gemv(quant, w, rows, nblk * 256, x)[0],
                    oracle.gemv(quant, w, rows, nblk * 256, x, gold=True)[0], f"quant {quant} extremes")


def test_q5k_fifth_bit_vectors_on_device(rnb):
    """The hand-built vectors that pin the oracle's Q5_K dot (one qh bit set in every byte, d = 1, dmin = 0,
    sub-block scales 1..8), through the device: 16 * (bit + 1) * sum of that sub-block's activations."""
    hdr = np.concatenate([np.frombuffer(npref.f16_bytes(1.0), np.uint8), np.frombuffer(npref.f16_bytes(0.0), np.uint8),
                          npref.pack_scales_k4(np.arange(1, 9), np.zeros(8))])
    x = np.zeros(256, np.float32)
    x[0] = 127.0                                   # Q8_K scale exactly 1: x == its quantised form
    x[1:] = (np.arange(1, 256) % 7 - 3).astype(np.float32)
    w = np.concatenate([np.concatenate([hdr, np.full(32, 1 << bit, np.uint8), np.zeros(128, np.uint8)])
                        for bit in range(8)])
    got = rnb.q5k_gemv(w, 8, 256, x)
    want = [16.0 * (bit + 1) * float(x[32 * bit:32 * bit + 32].sum()) for bit in range(8)]
    assert np.allclose(got, want, rtol=1e-6, atol=0), (got, want)


def test_config4_q4k_gemm_512x4096_to_14336(rnb, oracle):
    rows, cols, seq = 14336, 4096, 512
    w = oracle.make_weights(Q4_K, rows, cols, oracle.tensor_seed("cfg2", "weight"))
    x = oracle.fill_normal(seq * cols, oracle.tensor_seed("cfg4", "x"), 1.0)
    got = rnb.q4k_gemv_batch(w, rows, cols, x)
    assert got.shape == (seq, rows)
    rb = cols // 256 * 144
    # every one of the 14336 x 512 outputs against the oracle's AVX2 form of the block dot (pinned against the scalar
    # form and the reference's vectors in test_oracle_pins.py; seconds of CPU time on all cores) ...
    ref_all = oracle.gemv(Q4_K, w, rows, cols, x, avx2=oracle.have_avx2())
    check_close(got, ref_all, None, "cfg4 all rows, all tokens")
    # ... and three row bands (first, an interior band straddling tile edges, last) against the scalar form and its f64
    # statement at the tight tolerance
    for lo, hi in ((0, 160), (7001, 7161), (rows - 160, rows)):
        ws = w[lo * rb:hi * rb]
        ref = oracle.gemv(Q4_K, ws, hi - lo, cols, x)
        gold = oracle.gemv(Q4_K, ws, hi - lo, cols, x, gold=True)
        check_close(got[:, lo:hi], ref, gold, f"cfg4 rows {lo}:{hi}")
    # property: a token's result does not depend on its neighbours (permute tokens -> permuted output, bitwise)
    perm = np.random.default_rng(3).permutation(seq)
    got_p = rnb.q4k_gemv_batch(w, rows, cols, x.reshape(seq, cols)[perm])
    assert np.array_equal(got_p, got[perm])
    rnb.release(w)


# ---- sparse MoE ----------------------------------------------------------------------------------

def _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, seed, down_quant=Q6_K):
    gate = oracle.make_weights(Q4_K, n_expert * n_ff, n_embd, oracle.tensor_seed(f"moe{seed}", "gate"))
    up = oracle.make_weights(Q4_K, n_expert * n_ff, n_embd, oracle.tensor_seed(f"moe{seed}", "up"))
    down = oracle.make_weights(down_quant, n_expert * n_embd, n_ff, oracle.tensor_seed(f"moe{seed}", "down"))
    x = oracle.fill_normal(tokens * n_embd, oracle.tensor_seed(f"moe{seed}", "x"), 1.0)
    logits = oracle.fill_normal(tokens * n_expert, oracle.tensor_seed(f"moe{seed}", "logits"), 1.0)
    eids, route, tids = [], [], []
    for t in range(tokens):
        idx, wts = oracle.route_topk(logits[t * n_expert:(t + 1) * n_expert], k)
        eids += idx.tolist()
        route += wts.tolist()
        tids += [t] * len(idx)
    return gate, up, down, x, np.array(eids, np.uint32), np.array(route, np.float32), np.array(tids, np.uint32)


@pytest.mark.parametrize("tokens,down_quant", [(1, Q6_K), (3, Q6_K), (2, Q4_K), (1, Q5_K), (5, Q5_K), (40, Q5_K)])
def test_moe_small(rnb, oracle, tokens, down_quant):
    n_expert, n_ff, n_embd, k = 8, 512, 768, 3
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, 1, down_quant)
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    ref = oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    check_close(got, ref, None, f"moe tokens {tokens}")
    for w in (gate, up, down):
        rnb.release(w)


@pytest.mark.parametrize("n_ff,n_embd,k,down_quant", [(768, 2048, 8, Q6_K), (256, 512, 1, Q4_K), (512, 1280, 16, Q5_K),
                                                     (1024, 4096, 16, Q6_K), (256, 768, 17, Q6_K), (2304, 512, 8, Q4_K),
                                                     (512, 256, 5, Q5_K)])
def test_moe_one_token_equals_batch_row(rnb, oracle, n_ff, n_embd, k, down_quant):
    """One token takes the two-launch decode path (token and intermediates quantised inside the kernels, routing table
    in the kernel arguments) when it has at most 16 slots and 64 intermediate blocks; otherwise, and for batches of more
    than eight tokens, the general sequence.  Same arithmetic: the token alone equals its row in a nine-token batch bit
    for bit, with an expert repeated in the slot list, and both agree with the oracle."""
    n_expert = 20
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, 1, k, 77 + k, down_quant)
    if k >= 3:
        e[2] = e[0]  # the same expert twice in one token's list
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, 1, down_quant, n_ff, n_embd, x)
    ref = oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, 1, down_quant, n_ff, n_embd, x)
    check_close(got, ref, None, f"moe decode n_ff {n_ff} n_embd {n_embd} k {k}")
    x9 = np.concatenate([oracle.fill_normal(8 * n_embd, 5, 1.0), x])
    m = min(2, e.size)
    e9, r9 = np.concatenate([np.tile(e[:m], 8), e]), np.concatenate([np.tile(r[:m], 8), r])
    t9 = np.concatenate([np.repeat(np.arange(8, dtype=np.uint32), m), np.full(e.size, 8, np.uint32)])
    batch = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e9, r9, t9, 9, down_quant, n_ff, n_embd, x9)
    assert np.array_equal(batch[8], got[0])
    for w in (gate, up, down):
        rnb.release(w)


@pytest.mark.parametrize("tokens", [1, 3])
@pytest.mark.parametrize("shift", [1, 2])
def test_moe_decode_down_tensor_at_unaligned_device_address(rnb, oracle, tokens, shift):
    """The down tensor as a sub-range of a resident parent, one or two bytes in: read at parent + offset on the device.  The
    decode kernels fetch Q6_K blocks without the odd-address path, so at an odd address the call must take the general
    sequence; either way the bits of the aligned call (the same arithmetic in both sequences)."""
    n_expert, n_ff, n_embd, k = 6, 512, 768, 3
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, 9, Q6_K)
    base = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, Q6_K, n_ff, n_embd, x)
    rnb.release(down)
    parent = np.zeros(down.size + 8, np.uint8)
    parent[shift:shift + down.size] = down
    rnb.prewarm([parent])
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, parent[shift:shift + down.size], e, r, t, tokens, Q6_K,
                                                           n_ff, n_embd, x)
    assert np.array_equal(got, base)
    check_close(got, oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, tokens, Q6_K, n_ff, n_embd, x), None,
                f"moe decode, down tensor {shift} bytes in")
    for w in (gate, up, parent):
        rnb.release(w)


@pytest.mark.parametrize("tokens,n_ff,n_embd,k,down_quant", [(2, 768, 2048, 8, Q6_K), (3, 256, 512, 1, Q4_K), (4, 512, 1280, 16, Q5_K),
                                                            (8, 768, 2048, 8, Q6_K), (5, 1024, 768, 3, Q6_K), (8, 2304, 512, 7, Q4_K),
                                                            (7, 256, 4096, 9, Q5_K)])
def test_moe_small_batch_equals_general_sequence(rnb, oracle, tokens, n_ff, n_embd, k, down_quant):
    """Two to eight tokens with at most 64 slots take the decode kernels too (a workgroup of the first kernel quantises
    its slot's token, one of the second its token's intermediates).  The slot list comes interleaved (rank-major, not
    token by token), one token has no slot at all, and an expert is shared by several tokens.  Against the oracle, and
    bit for bit against the same tokens inside a batch of twelve, which takes the general sequence."""
    n_expert = 20
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, 170 + tokens, down_quant)
    e[(t == 1).nonzero()[0][:1]] = e[0]  # tokens 0 and 1 share an expert
    order = np.lexsort((t, np.concatenate([np.arange(k)] * tokens)))  # rank-major: token ids interleave
    e, r, t = e[order], r[order], t[order]
    if tokens >= 3:
        keep = t != 2  # token 2 is routed nowhere: its row must be exactly zero
        e, r, t = e[keep], r[keep], t[keep]
    assert e.size <= 64
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    ref = oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    check_close(got, ref, None, f"moe small batch tokens {tokens} k {k}")
    if tokens >= 3:
        assert np.all(got[2] == 0.0)
    pad = 12 - tokens
    x12 = np.concatenate([x, oracle.fill_normal(pad * n_embd, 6, 1.0)])
    e12 = np.concatenate([e, np.arange(pad, dtype=np.uint32) % n_expert])
    r12 = np.concatenate([r, np.full(pad, 0.5, np.float32)])
    t12 = np.concatenate([t, np.arange(tokens, 12, dtype=np.uint32)])
    big = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e12, r12, t12, 12, down_quant, n_ff, n_embd, x12)
    assert np.array_equal(big[:tokens], got)
    for w in (gate, up, down):
        rnb.release(w)


@pytest.mark.parametrize("tokens,n_expert,k,n_ff,n_embd,down_quant", [(16, 8, 2, 256, 256, Q6_K), (64, 3, 2, 512, 768, Q4_K),
                                                                     (100, 2, 2, 768, 512, Q5_K), (33, 20, 4, 300 * 0 + 512, 1280, Q6_K),
                                                                     (40, 5, 3, 1024, 256, Q4_K), (20, 64, 3, 256, 512, Q6_K),
                                                                     (64, 128, 8, 256, 1792, Q6_K), (48, 96, 8, 256, 1792, Q4_K)])
def test_moe_prefill_matrix_core_path(rnb, oracle, tokens, n_expert, k, n_ff, n_embd, down_quant):
    """16 or more tokens and at least 1.8 slots per routed expert on average: the grouped expert GEMMs on the matrix
    cores (32-token tiles per expert; experts with more than 32 tokens take several tiles, experts with few run mostly
    padding); the sixth case stays below that average and keeps the integer-dot kernels; in the last two the down
    kernel's workgroups walk four row tiles each (14 row tiles x ~100 expert groups: the last workgroup of a group gets two).
    Against the oracle, and a token's row must
    not depend on the batch: the same bits with the tokens in reverse order."""
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, 90 + tokens, down_quant)
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    ref = oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    check_close(got, ref, None, f"moe prefill tokens {tokens} experts {n_expert} down {down_quant}")
    xr = x.reshape(tokens, n_embd)[::-1].copy()
    tr = (tokens - 1 - t).astype(np.uint32)
    rev = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, tr, tokens, down_quant, n_ff, n_embd, xr)
    assert np.array_equal(rev[::-1], got)
    for w in (gate, up, down):
        rnb.release(w)


def test_moe_unrouted_token_and_empty_slot_list(rnb, oracle):
    n_expert, n_ff, n_embd = 4, 256, 256
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, 3, 2, 2)
    keep = t != 1  # token 1 gets no expert: its row must be exactly zero
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e[keep], r[keep], t[keep], 3, Q6_K, n_ff,
                                                           n_embd, x)
    ref = oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e[keep], r[keep], t[keep], 3, Q6_K, n_ff,
                                             n_embd, x)
    assert np.all(got[1] == 0.0)
    check_close(got, ref, None, "moe with an unrouted token")
    none = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e[:0], r[:0], t[:0], 3, Q6_K, n_ff, n_embd, x)
    assert none.shape == (3, n_embd) and np.all(none == 0.0)
    for w in (gate, up, down):
        rnb.release(w)


@pytest.mark.parametrize("tokens", [1, 64])
def test_config5_moe_qwen3_30b_a3b(rnb, oracle, tokens):
    n_expert, n_ff, n_embd, k = 128, 768, 2048, 8
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, 5)
    # callers hand prefill slots sorted by (expert, token) (crates/rnb-llm/.../shared_expert_moe/prefill.rs:1410-1458)
    if tokens > 1:
        order = np.lexsort((t, e))
        e, r, t = e[order], r[order], t[order]
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, Q6_K, n_ff, n_embd, x)
    ref = oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, tokens, Q6_K, n_ff, n_embd, x)
    check_close(got, ref, None, f"cfg5 tokens {tokens}")
    if tokens > 1:
        # a (token, expert) result does not depend on batching: token 7 alone (the decode kernels: per-lane f32 partial
        # sums) against row 7 of the batch (the matrix-core kernels: exact integer sums per block) agree to f32 rounding
        sel = t == 7
        solo = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e[sel], r[sel], np.zeros(sel.sum(), np.uint32),
                                                                1, Q6_K, n_ff, n_embd, x[7 * n_embd:8 * n_embd])
        assert np.abs(solo[0] - got[7]).max() <= 2e-5 * float(np.sqrt(np.mean(got[7].astype(np.float64) ** 2)))
    for w in (gate, up, down):
        rnb.release(w)


@pytest.mark.parametrize("q_rows,kv_rows,n_embd", [(4096, 1024, 4096), (5, 3, 512), (7, 2, 1280), (64, 0, 2048),
                                                     (0, 9, 768), (33, 33, 5120)])
def test_dense_q4k_attention_qkv_one_launch(rnb, oracle, q_rows, kv_rows, n_embd):
    """crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:916-985: three projections of one token from one quantised
    activation; for rows of up to 16 super-blocks each output equals the plain GEMV of its matrix bit for bit."""
    wq = oracle.make_weights(Q4_K, q_rows, n_embd, 600 + q_rows)
    wk = oracle.make_weights(Q4_K, kv_rows, n_embd, 601 + kv_rows)
    wv = oracle.make_weights(Q4_K, kv_rows, n_embd, 602 + kv_rows)
    x = oracle.fill_normal(n_embd, 603, 1.0)
    q = np.full(q_rows + 2, -3.0, np.float32)
    k = np.full(kv_rows + 1, -3.0, np.float32)
    v = np.full(kv_rows, -3.0, np.float32)
    rnb.dense_q4k_attention_qkv(wq, wk, wv, q_rows, kv_rows, n_embd, x, q, k, v)
    assert np.all(q[q_rows:] == -3.0) and np.all(k[kv_rows:] == -3.0)
    for got, w, rows, name in ((q[:q_rows], wq, q_rows, "q"), (k[:kv_rows], wk, kv_rows, "k"), (v, wv, kv_rows, "v")):
        if rows == 0:
            continue
        check_close(got, oracle.gemv(Q4_K, w, rows, n_embd, x)[0], oracle.gemv(Q4_K, w, rows, n_embd, x, gold=True)[0],
                    f"qkv {name} {rows}x{n_embd}")
        if n_embd <= 4096:  # longer rows: the plain GEMV splits K across waves, another f32 summation order
            assert np.array_equal(got, rnb.q4k_gemv(w, rows, n_embd, x)), name
        rnb.release(w)


def test_q8_0_gemv_argmax_matches_gemv(rnb, oracle):
    rows, cols = 3001, 1024
    w = oracle.make_weights(Q8_0, rows, cols, 510)
    x = oracle.fill_normal(cols, 511, 1.0)
    full = rnb.q8_0_gemv(w, rows, cols, x)
    idx, val = rnb.q8_0_gemv_argmax(w, rows, cols, x)
    assert idx == int(np.argmax(full)) and val == full[idx]
    assert rnb.q8_0_gemv_argmax_q8dot(w, rows, cols, x) == (idx, val)  # quant_api.rs:770-805: the same integer dots by name
    # two identical rows that win: the lower index is reported
    rb = cols // 32 * 34
    w2 = w.copy().reshape(rows, rb)
    w2[2500] = w2[idx]
    w2[17] = w2[idx]
    idx2, val2 = rnb.q8_0_gemv_argmax(w2.reshape(-1), rows, cols, x)
    assert idx2 == min(17, idx) and val2 == val


# ---- per-head Q8_0 projections (crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:824-882) ---------------------

@pytest.mark.parametrize("heads,rows_per_head,cols,tokens", [(3, 4, 96, 3), (16, 128, 512, 5), (64, 512, 128, 9), (5, 33, 1056, 2),
                                                             (1, 7, 4096, 1), (128, 64, 192, 6), (2, 300, 32, 4)])
def test_q8_0_head_gemv_batch(rnb, oracle, heads, rows_per_head, cols, tokens):
    """Every (token, head) group of the output is the Q8_0 GEMV of that head's rows on that token's vector for the head:
    bit for bit the one-token operator on the head's sub-matrix (what the reference's per-head path computes,
    crates/rnb-llm/src/engine/models/glm_dsa.rs:124-175), and within tolerance of the oracle; odd and even block counts
    (single and paired block fetches), token groups of 1 to 4, one head and many."""
    rows = heads * rows_per_head
    w = oracle.make_weights(Q8_0, rows, cols, 600 + heads)
    x = oracle.fill_normal(tokens * heads * cols, 601 + tokens, 1.0)
    got = rnb.q8_0_head_gemv_batch(w, heads, rows_per_head, cols, tokens, x)
    assert got.shape == (tokens, rows)
    hb = rows_per_head * (cols // 32) * 34
    xs = x.reshape(tokens, heads, cols)
    for h in sorted({0, heads // 2, heads - 1}):
        wh = w[h * hb:(h + 1) * hb].copy()
        ref = oracle.gemv(Q8_0, wh, rows_per_head, cols, xs[:, h].copy())
        gold = oracle.gemv(Q8_0, wh, rows_per_head, cols, xs[:, h].copy(), gold=True)
        mine = got[:, h * rows_per_head:(h + 1) * rows_per_head]
        check_close(mine, ref, gold, f"head batch head {h} of {heads}")
        for t in sorted({0, tokens - 1}):
            alone = rnb.q8_0_gemv(wh, rows_per_head, cols, xs[t, h].copy())
            assert np.array_equal(alone.view(np.uint32), mine[t].view(np.uint32)), (h, t)
        rnb.release(wh)
    rnb.release(w)


def test_q8_0_head_gemv_batch_reference_case(rnb, oracle):
    """The reference's own case (crates/rnb-backend/cuda/src/runtime/tests.rs:21118-21155): 3 heads x 4 rows x 96 columns,
    3 tokens, input ((i % 31) - 15) / 64, against dequantised weights times the f32 input (its cpu_q8_0_rows) within
    its tolerance of 0.01."""
    heads, rph, cols, tokens = 3, 4, 96, 3
    w = oracle.make_weights(Q8_0, heads * rph, cols, 181)
    x = (((np.arange(tokens * heads * cols) % 31).astype(np.float32)) - 15.0) * np.float32(0.015625)
    got = rnb.q8_0_head_gemv_batch(w, heads, rph, cols, tokens, x)
    hb = rph * (cols // 32) * 34
    xs = x.reshape(tokens, heads, cols)
    want = np.concatenate([oracle.gemv_q8_0_f32act(w[h * hb:(h + 1) * hb].copy(), rph, cols, xs[:, h].copy()) for h in range(heads)],
                          axis=1)
    assert np.abs(got - want).max() <= 0.01
    rnb.release(w)


# ---- dense SwiGLU FFN (crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:297-337) ----------------------------

def check_ffn(oracle, got, gate, up, down, down_quant, n_ff, n_embd, x, gelu, label):
    """The oracle's composition within the usual row check, plus what quantising the intermediate allows: act(gate) * up
    goes through expf / tanhf, whose last bit differs between the device and the host, and the two GEMV sums before it are
    added in different orders.  An element of the intermediate that lies within 1e-4 (relative) of a rounding boundary of
    its Q8_K / Q8 block may therefore be quantised one code apart; one code of element k is worth |W_down[r][k]| * d_block
    in output row r.  Rows are held to the usual tolerance plus that sum over the token's near-boundary elements (a few
    per token); every other difference fails."""
    seq = x.size // n_embd
    ref = (oracle.dense_gelu_ffn if gelu else oracle.dense_silu_ffn)(gate, up, down, down_quant, n_ff, n_embd, x)
    g = oracle.gemv(Q4_K, gate, n_ff, n_embd, x).ravel()
    u = oracle.gemv(Q4_K, up, n_ff, n_embd, x).ravel()
    mid = (oracle.gelu_mul if gelu else oracle.silu_mul)(g, u).reshape(seq, n_ff).astype(np.float64)
    blk = oracle.BLOCK_ELEMS[down_quant]
    m = mid.reshape(seq, n_ff // blk, blk)
    amax = np.abs(m).max(axis=2, keepdims=True)
    d = amax / 127.0                                    # one code step of the block, both quantisers
    v = np.divide(m, d, out=np.zeros_like(m), where=d > 0)
    near = np.abs(np.abs(v - np.floor(v)) - 0.5) < 1e-4 * np.maximum(1.0, np.abs(v))
    w = np.abs(oracle.dequantize(down_quant, down).reshape(n_embd, n_ff).astype(np.float64))
    step = np.broadcast_to(d, m.shape).reshape(seq, n_ff)
    near = near.reshape(seq, n_ff)
    slack = np.stack([w[:, near[t]] @ step[t, near[t]] for t in range(seq)])
    got = np.asarray(got, np.float64).reshape(seq, n_embd)
    r64 = ref.astype(np.float64).reshape(seq, n_embd)
    assert np.all(np.isfinite(got)), f"{label}: non-finite output"
    rms = float(np.sqrt(np.mean(r64 * r64))) or 1.0
    tol = np.maximum(REL * rms, REL * np.abs(r64)) + slack
    bad = np.abs(got - r64) > tol
    assert not bad.any(), (f"{label}: {int(bad.sum())} elements outside 1e-3 plus the quantiser's near-boundary slack "
                           f"(near-boundary elements per token: {near.sum(axis=1).tolist()}); worst excess "
                           f"{float((np.abs(got - r64) - tol).max())}")


@pytest.mark.parametrize("down_quant", [Q4_K, Q5_K, Q6_K, Q8_0, Q5_1])
@pytest.mark.parametrize("seq,n_ff,n_embd", [(2, 256, 256), (3, 768, 512), (5, 512, 4608), (17, 512, 768), (40, 1024, 256)])
def test_dense_silu_ffn_batch(rnb, oracle, down_quant, seq, n_ff, n_embd):
    """Decode-sized batches take the fused gate/up GEMV (groups of up to four tokens per pass over the two matrices), 9+
    tokens (these matrices are small) the MFMA GEMMs and the gated quantiser, rows longer than 16 super-blocks the unfused pair; all must equal the per-token composition of the
    oracle's pinned pieces."""
    gate = oracle.make_weights(Q4_K, n_ff, n_embd, 300 + seq)
    up = oracle.make_weights(Q4_K, n_ff, n_embd, 301 + seq)
    down = oracle.make_weights(down_quant, n_embd, n_ff, 302 + seq)
    x = oracle.fill_normal(seq * n_embd, 303 + seq, 1.0)
    got = rnb.dense_q4k_silu_ffn_batch(gate, up, down, down_quant, n_ff, n_embd, seq, x)
    assert got.shape == (seq, n_embd)
    check_ffn(oracle, got, gate, up, down, down_quant, n_ff, n_embd, x, False,
              f"dense ffn seq {seq} n_ff {n_ff} n_embd {n_embd} down {down_quant}")


@pytest.mark.parametrize("down_quant", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("seq,n_ff,n_embd", [(1, 512, 256), (1, 1024, 4608), (3, 768, 512), (17, 512, 768)])
def test_dense_gelu_ffn(rnb, oracle, down_quant, seq, n_ff, n_embd):
    """crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:182-293: the tanh-form GELU between the halves; one token
    through dense_q4k_gelu_ffn, more through the batch form (fused gate/up GEMV, long-row pair, MFMA GEMM routes)."""
    gate = oracle.make_weights(Q4_K, n_ff, n_embd, 320 + seq)
    up = oracle.make_weights(Q4_K, n_ff, n_embd, 321 + seq)
    down = oracle.make_weights(down_quant, n_embd, n_ff, 322 + seq)
    x = oracle.fill_normal(seq * n_embd, 323 + seq, 1.0)
    ref = oracle.dense_gelu_ffn(gate, up, down, down_quant, n_ff, n_embd, x)
    if seq == 1:
        got = rnb.dense_q4k_gelu_ffn(gate, up, down, down_quant, n_ff, n_embd, x).reshape(1, n_embd)
    else:
        got = rnb.dense_q4k_gelu_ffn_batch(gate, up, down, down_quant, n_ff, n_embd, seq, x)
    check_ffn(oracle, got, gate, up, down, down_quant, n_ff, n_embd, x, True,
              f"gelu ffn seq {seq} n_ff {n_ff} n_embd {n_embd} down {down_quant}")
    # and it is not the SiLU result
    assert not np.allclose(got, oracle.dense_silu_ffn(gate, up, down, down_quant, n_ff, n_embd, x), rtol=1e-3, atol=0)


@pytest.mark.parametrize("seq,down_quant", [(5, Q6_K), (6, Q4_K), (7, Q6_K), (9, Q4_K)])
def test_dense_silu_ffn_few_tokens_large_matrices(rnb, oracle, seq, down_quant):
    """Gate / up matrices of 16 MB and more (8192 x 4096 Q4_K) keep the fused gate/up GEMV up to six tokens (groups of
    3 + 2 and 3 + 3) and leave it for the GEMMs from seven on: gate and up GEMMs, SiLU * up quantised as it is made, down
    GEMM (K slices on these small grids)."""
    n_ff, n_embd = 8192, 4096
    gate = oracle.make_weights(Q4_K, n_ff, n_embd, 340 + seq)
    up = oracle.make_weights(Q4_K, n_ff, n_embd, 341 + seq)
    down = oracle.make_weights(down_quant, n_embd, n_ff, 342 + seq)
    x = oracle.fill_normal(seq * n_embd, 343 + seq, 1.0)
    got = rnb.dense_q4k_silu_ffn_batch(gate, up, down, down_quant, n_ff, n_embd, seq, x)
    check_ffn(oracle, got, gate, up, down, down_quant, n_ff, n_embd, x, False,
              f"dense ffn, large matrices, seq {seq} down {down_quant}")


def test_dense_silu_ffn_dev_single_token_and_residency(rnb, oracle):
    n_ff, n_embd = 1024, 512
    gate = oracle.make_weights(Q4_K, n_ff, n_embd, 310)
    up = oracle.make_weights(Q4_K, n_ff, n_embd, 311)
    down = oracle.make_weights(Q6_K, n_embd, n_ff, 312)
    x = oracle.fill_normal(n_embd, 313, 1.0)
    bufs = [rnb.DeviceBuffer.from_host(a) for a in (gate, up, down, x)]
    out = rnb.DeviceBuffer(n_embd * 4)
    rnb.dense_q4k_silu_ffn_dev(bufs[0], bufs[1], bufs[2], Q6_K, n_ff, n_embd, 1, bufs[3], out)
    got = out.to_host(np.float32).reshape(1, n_embd)
    check_close(got, oracle.dense_silu_ffn(gate, up, down, Q6_K, n_ff, n_embd, x), None, "dense ffn one token, device")
    for b in bufs + [out]:
        b.free()


def test_q6k_gemv_argmax_matches_gemv_and_tie_rule(rnb, oracle):
    """quant_api.rs:2170-2204; ties go to the lower row (quant_batch_and_ops.cuh:3299)."""
    rows, cols = 3000, 512
    w = oracle.make_weights(Q6_K, rows, cols, 500)
    x = oracle.fill_normal(cols, 501, 1.0)
    full = rnb.q6k_gemv(w, rows, cols, x)
    idx, val = rnb.q6k_gemv_argmax(w, rows, cols, x)
    assert idx == int(np.argmax(full)) and val == full[idx]
    ref = oracle.gemv(Q6_K, w, rows, cols, x)[0]
    assert idx == int(np.argmax(ref))
    # duplicate the winning row further down: the first occurrence must still win
    w2 = w.reshape(rows, -1).copy()
    w2[rows - 5] = w2[idx]
    w2[idx + 1 if idx + 1 < rows - 5 else 0] = w2[idx]
    idx2, val2 = rnb.q6k_gemv_argmax(w2.reshape(-1), rows, cols, x)
    assert idx2 == min(idx, idx + 1 if idx + 1 < rows - 5 else 0) and val2 == val
    one, v1 = rnb.q6k_gemv_argmax(w[:cols // 256 * 210], 1, cols, x)
    assert one == 0 and v1 == full[0]


# ---- HIP graph replay of the device-resident entry points --------------------------------------

@pytest.mark.parametrize("quant,rows,cols,seq", [(Q4_K, 512, 1024, 1), (Q6_K, 256, 2048, 24), (Q8_0, 300, 1024, 40),
                                                 (Q4_K, 2304, 2048, 260)])
def test_graph_replay_matches_eager(rnb, quant, rows, cols, seq):
    """The `_dev` entry points only enqueue on the library's stream, so a caller may capture them (after one eager call
    of the shape, which sizes the grow-only scratch): a decode GEMV in one launch, GEMMs cut into K slices plus their
    summing kernel, and the ping-pong GEMM with two slices.  Three replays with the input changed between them by eager
    uploads and synchronisations, each compared bit for bit with the eager result on the same input."""
    import ctypes as C
    import bench
    hip = bench.Hip()
    lib = rnb.lib()
    stream = C.c_void_p(rnb.stream_handle())
    rng = np.random.default_rng(4000 + rows)
    w = rnb.DeviceBuffer.from_host(bench.synth_weights(quant, rows, cols, 4100 + seq))
    xs = [rng.standard_normal(seq * cols).astype(np.float32) for _ in range(3)]
    x_dev = rnb.DeviceBuffer.from_host(xs[0])
    out_dev = rnb.DeviceBuffer(seq * rows * 4)
    eager = []
    for x in xs:
        assert lib.rnb_hip_dev_upload(x_dev.ptr, x.ctypes.data_as(C.c_void_p), x.nbytes) == 0
        rnb.gemv_dev(quant, w, rows, cols, x_dev, seq, out_dev)
        eager.append(out_dev.to_host(np.float32))
    graph, gexec = C.c_void_p(), C.c_void_p()
    hip.check(hip.rt.hipStreamBeginCapture(stream, 2), "hipStreamBeginCapture")
    try:
        rnb.gemv_dev(quant, w, rows, cols, x_dev, seq, out_dev)
    finally:
        rc = hip.rt.hipStreamEndCapture(stream, C.byref(graph))
    hip.check(rc, "hipStreamEndCapture")
    hip.check(hip.rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0), "hipGraphInstantiate")
    try:
        for x, want in zip(xs, eager):
            assert lib.rnb_hip_dev_upload(x_dev.ptr, x.ctypes.data_as(C.c_void_p), x.nbytes) == 0
            hip.check(hip.rt.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            rnb.sync()
            assert np.array_equal(out_dev.to_host(np.float32), want)
    finally:
        hip.rt.hipGraphExecDestroy(gexec)
        hip.rt.hipGraphDestroy(graph)
        for b in (w, x_dev, out_dev):
            b.free()


def test_graph_survives_scratch_growth_and_capture_refuses_growth(rnb):
    """A graph captured on a small shape keeps the scratch addresses of that moment.  A later, larger eager call grows
    the scratch: the replaced allocation is retired, not freed, once a capture has been seen, so the graph's replay
    still reads and writes live memory and gives the eager bits.  A capture whose call would itself have to grow the
    scratch is refused with a message, as is a host-pointer call (it would upload weights and synchronise); the
    no-allocation entry point captures without a warm-up."""
    import ctypes as C
    import bench
    hip = bench.Hip()
    lib = rnb.lib()
    stream = C.c_void_p(rnb.stream_handle())
    rng = np.random.default_rng(77)
    rows, cols, seq = 384, 1024, 6
    w = rnb.DeviceBuffer.from_host(bench.synth_weights(Q4_K, rows, cols, 78))
    x = rng.standard_normal(seq * cols).astype(np.float32)
    x_dev, out_dev = rnb.DeviceBuffer.from_host(x), rnb.DeviceBuffer(seq * rows * 4)
    rnb.gemv_dev(Q4_K, w, rows, cols, x_dev, seq, out_dev)  # eager: sizes the scratch for this shape
    want = out_dev.to_host(np.float32)
    graph, gexec = C.c_void_p(), C.c_void_p()
    hip.check(hip.rt.hipStreamBeginCapture(stream, 2), "hipStreamBeginCapture")
    try:
        rnb.gemv_dev(Q4_K, w, rows, cols, x_dev, seq, out_dev)
        # while capturing: a shape that needs more scratch than there is, and a host-pointer call, are refused
        big_seq = 4096
        xb, ob = rnb.DeviceBuffer(big_seq * cols * 4), rnb.DeviceBuffer(big_seq * rows * 4)
        with pytest.raises(rnb.BackendError) as err:
            rnb.gemv_dev(Q4_K, w, rows, cols, xb, big_seq, ob)
        assert err.value.kind == "InvalidRequest" and "capturing" in str(err.value)
        # entry points that free device memory synchronise the stream first: refused as well
        for call in (lambda: rnb.lib().rnb_hip_set_resident_budget(1 << 30), lambda: rnb.lib().rnb_hip_offload_unpinned(None),
                     lambda: rnb.lib().rnb_hip_release(x.ctypes.data_as(C.c_void_p), x.nbytes)):
            assert call() == 1 and "capturing" in rnb.last_error()  # RNB_HIP_INVALID_REQUEST
        # the no-allocation form of the same call is captured
        out2 = rnb.DeviceBuffer(seq * rows * 4)
        rnb.gemv_dev_noalloc(Q4_K, w, rows, cols, x_dev, seq, out2)
    finally:
        rc = hip.rt.hipStreamEndCapture(stream, C.byref(graph))
    hip.check(rc, "hipStreamEndCapture")
    hip.check(hip.rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0), "hipGraphInstantiate")
    try:
        # a larger eager call grows every scratch buffer the graph's nodes point into
        rnb.gemv_dev(Q4_K, w, rows, cols, xb, big_seq, ob)
        rnb.sync()
        for _ in range(3):
            assert lib.rnb_hip_dev_upload(out_dev.ptr, np.zeros(seq * rows, np.float32).ctypes.data_as(C.c_void_p),
                                          seq * rows * 4) == 0
            hip.check(hip.rt.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            rnb.sync()
            assert np.array_equal(out_dev.to_host(np.float32), want)
            assert np.array_equal(out2.to_host(np.float32), want)
            rnb.gemv_dev(Q4_K, w, rows, cols, xb, big_seq, ob)  # eager work between the replays
            rnb.sync()
    finally:
        hip.rt.hipGraphExecDestroy(gexec)
        hip.rt.hipGraphDestroy(graph)
        for b in (w, x_dev, out_dev, xb, ob, out2):
            b.free()


_FIRST_CAPTURE_SCRIPT = r"""
import ctypes as C, sys
import numpy as np
import bench
import runnburn_amd as rnb
Q4_K = 12
hip = bench.Hip()
stream = C.c_void_p(rnb.stream_handle())
rows, cols, seq = 384, 1024, 6
w = rnb.DeviceBuffer.from_host(bench.synth_weights(Q4_K, rows, cols, 78))
x = np.random.default_rng(77).standard_normal(seq * cols).astype(np.float32)
x_dev, out_dev = rnb.DeviceBuffer.from_host(x), rnb.DeviceBuffer(seq * rows * 4)
rnb.gemv_dev(Q4_K, w, rows, cols, x_dev, seq, out_dev)  # eager warm-up: the scratch now fits this shape
want = out_dev.to_host(np.float32)
graph, gexec = C.c_void_p(), C.c_void_p()
hip.check(hip.rt.hipStreamBeginCapture(stream, 2), "begin")
rnb.gemv_dev(Q4_K, w, rows, cols, x_dev, seq, out_dev)  # the only captured call: nothing has to grow
hip.check(hip.rt.hipStreamEndCapture(stream, C.byref(graph)), "end")
hip.check(hip.rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0), "instantiate")
big = 4096
xb, ob = rnb.DeviceBuffer(big * cols * 4), rnb.DeviceBuffer(big * rows * 4)
rnb.gemv_dev(Q4_K, w, rows, cols, xb, big, ob)  # grows every scratch buffer the graph points into
rnb.sync()
junk = [rnb.DeviceBuffer.from_host(np.full(1 << 20, 0x7f, np.uint8)) for _ in range(16)]  # reuse whatever was freed
for _ in range(3):
    rnb.lib().rnb_hip_dev_upload(out_dev.ptr, np.zeros(seq * rows, np.float32).ctypes.data_as(C.c_void_p), seq * rows * 4)
    hip.check(hip.rt.hipGraphLaunch(gexec, stream), "launch")
    rnb.sync()
    if not np.array_equal(out_dev.to_host(np.float32), want):
        print("REPLAY DIFFERS"); sys.exit(1)
    rnb.gemv_dev(Q4_K, w, rows, cols, xb, big, ob)
    rnb.sync()
print("REPLAY OK")
"""


def test_first_capture_of_a_process_with_fitting_calls_only_keeps_its_scratch(rnb):
    """In a fresh process: one eager call, then a capture whose only call fits the scratch that call left (so no buffer
    is asked to grow while capturing), then a larger eager call.  The library must have noticed the capture anyway and
    retire the replaced scratch instead of freeing it; the graph's replays give the eager bits."""
    import subprocess
    import sys as _sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([_sys.executable, "-c", _FIRST_CAPTURE_SCRIPT], cwd=root, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and "REPLAY OK" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-2000:]


# ---- the shared expert as a slot of the call: moe_view/fanout.rs:804-812 -------------------------------------------------

def _with_shared(oracle, n_expert, n_ff, n_embd, tokens, k, seed, down_quant):
    """A routed case plus a shared expert: its slot (id n_expert, weight = a gate scalar per token) is appended to every
    token's list, as the reference's decode call does.  The oracle sees the shared expert as expert n_expert of tensors
    one expert longer, which is what that id means."""
    gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, seed, down_quant)
    sg = oracle.make_weights(Q4_K, n_ff, n_embd, seed + 100)
    su = oracle.make_weights(Q4_K, n_ff, n_embd, seed + 101)
    sd = oracle.make_weights(down_quant, n_embd, n_ff, seed + 102)
    scal = 1.0 / (1.0 + np.exp(-oracle.fill_normal(tokens, seed + 103, 1.0)))  # sigmoid of the shared gate's logit
    es, rs, ts = [], [], []
    for tok in range(tokens):
        m = t == tok
        es += e[m].tolist() + [n_expert]
        rs += r[m].tolist() + [float(scal[tok])]
        ts += [tok] * (int(m.sum()) + 1)
    e, r, t = np.array(es, np.uint32), np.array(rs, np.float32), np.array(ts, np.uint32)
    longer = tuple(np.concatenate([a, b]) for a, b in ((gate, sg), (up, su), (down, sd)))
    return gate, up, down, (sg, su, sd), longer, x, e, r, t


@pytest.mark.parametrize("tokens,n_ff,n_embd,k,down_quant", [(1, 768, 2048, 8, Q6_K), (1, 512, 1280, 15, Q5_K), (1, 256, 512, 1, Q4_K),
                                                            (1, 256, 768, 17, Q6_K), (4, 768, 2048, 7, Q6_K), (8, 512, 768, 3, Q4_K),
                                                            (12, 768, 1024, 4, Q6_K), (40, 512, 768, 3, Q5_K)])
def test_moe_shared_expert_slot(rnb, oracle, tokens, n_ff, n_embd, k, down_quant):
    """Decode (two launches), small batches, the token-major and the expert-major general sequences, each with the
    shared expert as the last slot of every token: equal to the oracle run on tensors that hold the shared expert as
    expert n_expert, and bit-equal to the product run on those longer tensors without a shared expert."""
    n_expert = 12
    gate, up, down, shared, longer, x, e, r, t = _with_shared(oracle, n_expert, n_ff, n_embd, tokens, k, 300 + tokens + k, down_quant)
    got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, down_quant, n_ff, n_embd, x,
                                                           shared=shared)
    ref = oracle.moe_sparse_experts_by_token(*longer, n_expert + 1, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    check_close(got, ref, None, f"moe shared tokens {tokens} k {k}")
    same = rnb.qwen35_sparse_experts_selected_base_by_token(*longer, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    assert np.array_equal(got, same)
    # the shared expert alone (no routed slot)
    only = e == n_expert
    got1 = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e[only], r[only], t[only], tokens, down_quant,
                                                            n_ff, n_embd, x, shared=shared)
    ref1 = oracle.moe_sparse_experts_by_token(*longer, n_expert + 1, e[only], r[only], t[only], tokens, down_quant, n_ff,
                                              n_embd, x)
    check_close(got1, ref1, None, f"moe shared only tokens {tokens}")
    # without the tensors the id is refused
    with pytest.raises(rnb.BackendError) as err:
        rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    assert "expert id out of range" in str(err.value)
    for w in (gate, up, down, *shared, *longer):
        rnb.release(w)


def test_moe_shared_expert_slot_on_the_matrix_cores_dev(rnb, oracle):
    """64 tokens x top-4 of 16 experts + the shared expert for every token (a group of 64 slots), device buffers: the
    grouped matrix-core kernels read the shared tensors for that group."""
    n_expert, n_ff, n_embd, tokens, k = 16, 512, 1024, 64, 4
    gate, up, down, shared, longer, x, e, r, t = _with_shared(oracle, n_expert, n_ff, n_embd, tokens, k, 411, Q6_K)
    order = np.lexsort((t, e))  # the callers' (expert, token) order
    e, r, t = e[order], r[order], t[order]
    bufs = [rnb.DeviceBuffer.from_host(a) for a in (gate, up, down, *shared, x)]
    out_dev = rnb.DeviceBuffer(tokens * n_embd * 4)
    try:
        rnb.moe_sparse_experts_by_token_dev(bufs[0], bufs[1], bufs[2], n_expert, e, r, t, tokens, Q6_K, n_ff, n_embd, bufs[6],
                                            out_dev, shared=bufs[3:6])
        rnb.sync()
        got = out_dev.to_host(np.float32).reshape(tokens, n_embd).copy()
    finally:
        for b in bufs + [out_dev]:
            b.free()
    ref = oracle.moe_sparse_experts_by_token(*longer, n_expert + 1, e, r, t, tokens, Q6_K, n_ff, n_embd, x)
    from oracle import flips
    v = flips.moe_verdict(got, ref, *longer, n_expert + 1, e, r, t, tokens, Q6_K, n_ff, n_embd, x)
    assert v["ok"] or v["flip_aware_ok"], v


@pytest.mark.parametrize("tokens,n_expert,k,n_ff,n_embd,down_quant,shared", [(64, 128, 8, 1024, 512, Q6_K, False),
                                                                            (48, 60, 8, 1280, 768, Q5_K, False),
                                                                            (100, 128, 2, 512, 256, Q4_K, False),
                                                                            (16, 48, 8, 1024, 512, Q6_K, True)])
def test_moe_many_experts_wide_workgroups_ragged_row_tiles_dev(rnb, oracle, tokens, n_expert, k, n_ff, n_embd, down_quant, shared):
    """Many routed experts with few tokens each: the gate/up kernel runs six-wave workgroups (192 rows a tile) that
    walk two or three row tiles, and n_ff is no multiple of 192, so a group's last tile has idle waves and its last
    workgroup fewer tiles.  Device buffers, slots in the callers' (expert, token) order; the last case has the shared
    expert as the one group of sixteen tokens among groups of a few.  Against the oracle, and the same bits with the
    tokens in reverse order."""
    if shared:
        gate, up, down, sh, longer, x, e, r, t = _with_shared(oracle, n_expert, n_ff, n_embd, tokens, k, 700 + tokens, down_quant)
        ne = n_expert + 1
    else:
        gate, up, down, x, e, r, t = _moe_case(oracle, n_expert, n_ff, n_embd, tokens, k, 700 + tokens, down_quant)
        sh, longer, ne = (), (gate, up, down), n_expert
    order = np.lexsort((t, e))
    e, r, t = e[order], r[order], t[order]
    xr = x.reshape(tokens, n_embd)[::-1].copy()
    tr = (tokens - 1 - t).astype(np.uint32)
    order_r = np.lexsort((tr, e))
    bufs = [rnb.DeviceBuffer.from_host(a) for a in (gate, up, down, x, xr, *sh)]
    out_dev = rnb.DeviceBuffer(tokens * n_embd * 4)
    try:
        outs = []
        for xb, ee, rr, tt in ((bufs[3], e, r, t), (bufs[4], e[order_r], r[order_r], tr[order_r])):
            rnb.moe_sparse_experts_by_token_dev(bufs[0], bufs[1], bufs[2], n_expert, ee, rr, tt, tokens, down_quant, n_ff, n_embd,
                                                xb, out_dev, shared=bufs[5:8] if shared else None)
            rnb.sync()
            outs.append(out_dev.to_host(np.float32).reshape(tokens, n_embd).copy())
    finally:
        for b in bufs + [out_dev]:
            b.free()
    got, rev = outs
    ref = oracle.moe_sparse_experts_by_token(*longer, ne, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    from oracle import flips
    v = flips.moe_verdict(got, ref, *longer, ne, e, r, t, tokens, down_quant, n_ff, n_embd, x)
    assert v["ok"] or v["flip_aware_ok"], {key: v[key] for key in v if key != "flips"}
    assert np.array_equal(rev[::-1], got)
