"""rnb_hip_gemv_dev_noalloc: the device-resident GEMV / small-batch GEMM with its scratch (quantised activations,
K-slice partial sums) in the library's fixed device array instead of the grow-only buffers.  It runs the same kernels
on the same operands as rnb_hip_gemv_dev, so the outputs must be the same bits, call after call, also when a smaller
call follows a larger one over the array's stale contents."""
import numpy as np
import pytest

Q4_K, Q6_K, Q8_0 = 12, 14, 8


def _both(rnb, oracle, quant, rows, cols, seq, seed):
    w = oracle.make_weights(quant, rows, cols, seed)
    x = oracle.fill_normal(seq * cols, seed + 1, 1.0)
    wd, xd = rnb.DeviceBuffer.from_host(w), rnb.DeviceBuffer.from_host(x)
    o_ref, o_new = rnb.DeviceBuffer(seq * rows * 4), rnb.DeviceBuffer(seq * rows * 4)
    rnb.gemv_dev(quant, wd, rows, cols, xd, seq, o_ref)
    rnb.sync()
    ref = o_ref.to_host(np.float32)
    rnb.gemv_dev_noalloc(quant, wd, rows, cols, xd, seq, o_new)
    rnb.sync()
    got = o_new.to_host(np.float32)
    for buf in (wd, xd, o_ref, o_new):
        buf.free()
    return w, x, ref, got


@pytest.mark.gpu
@pytest.mark.parametrize("quant,big,small", [
    (Q4_K, (1024, 4096, 48), (300, 1024, 5)),      # MFMA GEMM with digits, then the GEMV that keeps several tokens in registers
    (Q6_K, (512, 14336, 24), (257, 5120, 1)),      # K cut into slices (workspace in the array), then split-K GEMV
    (Q8_0, (768, 4096, 40), (64, 96, 3)),          # 32-wide Q8 activations
    (Q4_K, (2048, 4096, 1), (40, 512, 2)),         # one-launch decode GEMV (no scratch), then a tiny batch
])
def test_noalloc_matches_gemv_dev_twice(rnb, oracle, quant, big, small):
    for i, (rows, cols, seq) in enumerate((big, small)):
        print(f"noalloc case quant={quant} rows={rows} cols={cols} seq={seq}", flush=True)
        w, x, ref, got = _both(rnb, oracle, quant, rows, cols, seq, 4100 + 10 * i + quant)
        assert np.array_equal(ref.view(np.uint32), got.view(np.uint32)), (quant, rows, cols, seq)
        # and against the oracle's f64 statement of the same integer dots: |gpu - gold| <= 2e-5 * rms(gold)
        gold = np.asarray(oracle.gemv(quant, w, rows, cols, x, gold=True), np.float64).ravel()
        rms = float(np.sqrt(np.mean(gold * gold))) or 1.0
        assert float(np.abs(got.astype(np.float64) - gold).max()) <= 2e-5 * rms


@pytest.mark.gpu
def test_noalloc_rejects_oversized_and_keeps_working(rnb, oracle):
    cap = rnb.gemv_dev_noalloc_scratch_bytes()
    assert cap == 8 << 20
    rows, cols = 16, 4096
    seq = cap // cols + 1  # the int8 activations alone exceed the array
    w = oracle.make_weights(Q4_K, rows, cols, 77)
    wd = rnb.DeviceBuffer.from_host(w)
    xd = rnb.DeviceBuffer(seq * cols * 4)
    od = rnb.DeviceBuffer(seq * rows * 4)
    with pytest.raises(rnb.BackendError) as err:
        rnb.gemv_dev_noalloc(Q4_K, wd, rows, cols, xd, seq, od)
    assert err.value.kind == "InvalidRequest" and "static scratch" in str(err.value)
    for buf in (wd, xd, od):
        buf.free()
    # the next call of a fitting shape is unaffected
    _, _, ref, got = _both(rnb, oracle, Q4_K, 128, 1024, 9, 78)
    assert np.array_equal(ref.view(np.uint32), got.view(np.uint32))
