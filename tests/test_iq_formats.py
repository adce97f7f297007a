"""IQ2_XXS / IQ2_S / IQ3_XXS / IQ4_XS GEMV on the device against the oracle (whose dequantisers reproduce the
reference's known-answer hashes, tests/test_oracle_pins.py): the operator surface of
crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:543-722 (gemv and gemv_batch per format, same validation texts)."""
import numpy as np
import pytest

IQ2_XXS, IQ3_XXS, IQ2_S, IQ4_XS = 16, 18, 22, 23
REL, TIGHT = 1e-3, 2e-5
LABEL = {IQ2_XXS: "IQ2_XXS", IQ3_XXS: "IQ3_XXS", IQ2_S: "IQ2_S", IQ4_XS: "IQ4_XS"}


def _fns(rnb, quant):
    return {IQ2_XXS: (rnb.iq2_xxs_gemv, rnb.iq2_xxs_gemv_batch), IQ3_XXS: (rnb.iq3_xxs_gemv, rnb.iq3_xxs_gemv_batch),
            IQ2_S: (rnb.iq2_s_gemv, rnb.iq2_s_gemv_batch), IQ4_XS: (rnb.iq4_xs_gemv, rnb.iq4_xs_gemv_batch)}[quant]


def _check(got, ref, gold, label):
    got, ref, gold = (np.asarray(a, np.float64) for a in (got, ref, gold))
    assert np.all(np.isfinite(got)), label
    rms = float(np.sqrt(np.mean(gold * gold))) or 1.0
    assert np.all(np.abs(got - ref) <= np.maximum(REL * rms, REL * np.abs(ref))), f"{label}: outside 1e-3 of the oracle"
    assert float(np.abs(got - gold).max()) <= TIGHT * rms, f"{label}: |gpu - f64 gold| {np.abs(got - gold).max()} > 2e-5 rms {rms}"


@pytest.mark.gpu
@pytest.mark.parametrize("quant", [IQ2_XXS, IQ2_S, IQ3_XXS, IQ4_XS])
@pytest.mark.parametrize("rows,cols", [(1, 256), (37, 768), (300, 4096), (4099, 2048), (64, 14336), (20000, 256)])
def test_iq_gemv_against_oracle(rnb, oracle, quant, rows, cols):
    """One token: rows of 1 to 56 blocks (idle lanes, several passes per row), more rows than waves."""
    w = oracle.make_weights(quant, rows, cols, 300 + quant + rows)
    x = oracle.fill_normal(cols, 17 + cols, 1.0)
    got = _fns(rnb, quant)[0](w, rows, cols, x)
    _check(got, oracle.gemv(quant, w, rows, cols, x)[0], oracle.gemv(quant, w, rows, cols, x, gold=True)[0],
           f"{LABEL[quant]} {rows}x{cols}")
    rnb.release(w)


@pytest.mark.gpu
@pytest.mark.parametrize("quant", [IQ2_XXS, IQ2_S, IQ3_XXS, IQ4_XS])
@pytest.mark.parametrize("seq", [2, 3, 4, 5, 33])
def test_iq_gemv_batch_layout(rnb, oracle, quant, seq):
    """Batch form: out[s * rows + r] (crates/rnb-cpu/src/gemm/quant_gemv.rs:1185-1196).  Up to four tokens every token's
    row equals the one-token call bit for bit (the GEMV decodes a block once and dots it against each token of the group
    with the one-token arithmetic); from five on the batch runs on the matrix cores (integer group sums, one f32 update
    per block) and agrees to rounding."""
    rows, cols = 203, 1024
    w = oracle.make_weights(quant, rows, cols, 800 + quant)
    x = oracle.fill_normal(seq * cols, 900 + seq, 1.0)
    one, batch = _fns(rnb, quant)
    got = batch(w, rows, cols, x).reshape(seq, rows)
    _check(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True), f"{LABEL[quant]} batch {seq}")
    for s in (0, seq - 1):
        alone = one(w, rows, cols, x[s * cols:(s + 1) * cols])
        if seq < 5:
            assert np.array_equal(got[s], alone)
        else:
            assert np.abs(got[s] - alone).max() <= 1e-5 * np.abs(alone).max()
    rnb.release(w)


@pytest.mark.gpu
@pytest.mark.parametrize("quant", [IQ2_XXS, IQ2_S, IQ3_XXS, IQ4_XS])
@pytest.mark.parametrize("rows,cols,seq", [(203, 1024, 5), (130, 256, 33), (129, 4096, 65), (4096, 2048, 96), (37, 14336, 17),
                                           (300, 768, 512), (8192, 512, 500)])
def test_iq_gemm_matrix_cores(rnb, oracle, quant, rows, cols, seq):
    """Batches of five tokens and more: ragged row and token tiles, 32- and 64-token workgroups (8192 rows x 500 tokens),
    K cut into slices on small grids (37 rows x 56 blocks: sixteen slices)."""
    w = oracle.make_weights(quant, rows, cols, 1200 + quant + rows)
    x = oracle.fill_normal(seq * cols, 1300 + seq, 1.0)
    got = _fns(rnb, quant)[1](w, rows, cols, x).reshape(seq, rows)
    _check(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True),
           f"{LABEL[quant]} gemm {rows}x{cols}x{seq}")
    rnb.release(w)


@pytest.mark.gpu
def test_iq_gemm_every_code_and_scale(rnb, oracle):
    """Blocks of random bytes (every grid index, sign pattern and scale value) with a finite d, eight tokens."""
    rng = np.random.default_rng(99)
    bb = {IQ2_XXS: 66, IQ2_S: 82, IQ3_XXS: 98, IQ4_XS: 136}
    for quant in (IQ2_XXS, IQ2_S, IQ3_XXS, IQ4_XS):
        rows, cols, seq = 160, 1024, 8
        w = rng.integers(0, 256, size=(rows * cols // 256, bb[quant]), dtype=np.uint8)
        w[:, 0:2] = (rng.standard_normal((w.shape[0], 1)) * 0.05).astype(np.float16).view(np.uint8).reshape(-1, 2)
        w = w.reshape(-1)
        x = oracle.fill_normal(seq * cols, 77 + quant, 1.0)
        got = _fns(rnb, quant)[1](w, rows, cols, x).reshape(seq, rows)
        _check(got, oracle.gemv(quant, w, rows, cols, x), oracle.gemv(quant, w, rows, cols, x, gold=True), f"{LABEL[quant]} random codes")
        rnb.release(w)


@pytest.mark.gpu
def test_iq4_xs_reference_block_on_device(rnb, oracle):
    """The reference's IQ4_XS vector (crates/rnb-cpu/src/gemm/dequant.rs:542-556: every scale +1, bytes 0xf0) against
    activations that quantise exactly (127 at one position of a block, zero elsewhere): the GEMV returns the dequantised
    element itself, -127 for an element in the first half of a sub-block and 113 in the second."""
    b = np.zeros(136, np.uint8)
    b[:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    b[2:4] = (0xAA, 0xAA)
    b[4:8] = 0x11
    b[8:] = 0xF0
    for pos, want in ((0, -127.0), (16, 113.0), (32, -127.0), (255, 113.0)):
        x = np.zeros(256, np.float32)
        x[pos] = 127.0
        got = rnb.iq4_xs_gemv(b, 1, 256, x)
        assert got[0] == want * 127.0
    rnb.release(b)


@pytest.mark.gpu
def test_iq_zero_codes_sum_the_activations(rnb, oracle):
    """crates/rnb-cpu/src/quantize/iq.rs:281-299: zero codes behind d = 1 decode to +1 everywhere, so the GEMV is the sum
    of the quantised activations."""
    x = np.zeros(512, np.float32)
    x[3], x[300] = 127.0, -127.0
    x[40] = 64.0
    for quant, nbytes, fn in ((IQ2_XXS, 66, rnb.iq2_xxs_gemv), (IQ2_S, 82, rnb.iq2_s_gemv), (IQ3_XXS, 98, rnb.iq3_xxs_gemv)):
        blk = np.zeros(nbytes, np.uint8)
        blk[:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
        w = np.tile(blk, 2)
        got = fn(w, 1, 512, x)
        assert got[0] == pytest.approx(127.0 + 64.0 - 127.0, abs=1e-4), LABEL[quant]
        rnb.release(w)


@pytest.mark.gpu
def test_iq_validation_texts(rnb):
    """quant_api.rs:651-722: the three checks, in order, with the reference's texts."""
    w = np.zeros(136 * 2, np.uint8)
    x = np.zeros(512, np.float32)
    with pytest.raises(rnb.BackendError, match="IQ4_XS cols must be divisible by 256, got 500"):
        rnb.iq4_xs_gemv(w, 1, 500, x)
    with pytest.raises(rnb.BackendError, match="IQ4_XS weight byte mismatch: got 272, expected 816"):
        rnb.iq4_xs_gemv(w, 3, 512, x)
    with pytest.raises(rnb.BackendError, match="IQ4_XS input length mismatch: got 256, expected 512"):
        rnb.iq4_xs_gemv(w, 1, 512, x[:256])
    with pytest.raises(rnb.BackendError, match="IQ2_XXS batch input length 500 is not divisible by cols 512"):
        rnb.iq2_xxs_gemv_batch(np.zeros(66 * 2, np.uint8), 1, 512, x[:500])
