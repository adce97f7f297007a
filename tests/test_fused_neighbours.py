"""The GEMV's device-resident neighbours: RMS norm (+ residual add) with a Q8_K output that feeds the GEMVs without a
quantiser launch, and the router (top-k + softmax over the selected logits).

Reference arithmetic: crates/rnb-cpu/src/kernels/norm.rs:140-225 (restated in oracle.rms_norm, pinned in
test_oracle_pins.py), crates/rnb-cpu/src/gemm/activation_q8.rs:149-173 (bit-exact quantiser),
crates/rnb-llm/src/engine/models/shared_expert_moe/routing.rs:18-64 (oracle.route_topk, pinned on routing.rs:272-318)."""
import numpy as np
import pytest

Q4_K, Q6_K = 12, 14


def _close(got, ref, rel):
    got = np.asarray(got, np.float64).ravel()
    ref = np.asarray(ref, np.float64).ravel()
    return bool(np.all(np.isfinite(got)) and np.all(np.abs(got - ref) <= rel * np.abs(ref) + 1e-12))


@pytest.mark.gpu
@pytest.mark.parametrize("seq,hidden,unit", [(1, 4096, False), (3, 2048, False), (5, 256, True), (7, 1536, True),
                                             (1, 14336, False), (33, 1024, False)])
def test_rms_norm_and_its_q8k_output(rnb, oracle, seq, hidden, unit):
    """f32 output against the oracle (the mean square is summed in another order, so the last bit of rms may differ: 3e-7
    relative); the Q8_K output is bit-for-bit the reference quantiser applied to the f32 output the kernel itself wrote,
    and the GEMV that follows from the activation scratch equals the GEMV of that f32 output, bit for bit."""
    rng = np.random.default_rng(hidden + seq)
    x = (rng.standard_normal(seq * hidden) * 3.0).astype(np.float32)
    w = (rng.standard_normal(hidden) * 0.5 + 1.0).astype(np.float32)
    eps = 1e-5
    xd, wd = rnb.DeviceBuffer.from_host(x), rnb.DeviceBuffer.from_host(w)
    o_plain, o_q = rnb.DeviceBuffer(seq * hidden * 4), rnb.DeviceBuffer(seq * hidden * 4)
    rnb.rms_norm_dev(xd, wd, eps, seq, hidden, o_plain, unit_offset=unit)
    rnb.rms_norm_dev(xd, wd, eps, seq, hidden, o_q, unit_offset=unit, quantize=True)
    rnb.sync()
    plain, withq = o_plain.to_host(np.float32), o_q.to_host(np.float32)
    assert np.array_equal(plain.view(np.uint32), withq.view(np.uint32))
    ref = oracle.rms_norm(x, w, eps, unit_offset=unit)
    assert _close(plain, ref, 3e-7 if not unit else 2e-6)
    # the activation scratch holds Q8_K(plain): a GEMV from it equals the one-call GEMV on `plain`, bit for bit, and
    # the oracle's GEMV on `plain`
    rows = 320
    wq = oracle.make_weights(Q4_K if hidden <= 4096 else Q6_K, rows, hidden, 600 + hidden)
    quant = Q4_K if hidden <= 4096 else Q6_K
    wqd = rnb.DeviceBuffer.from_host(wq)
    a, b = rnb.DeviceBuffer(seq * rows * 4), rnb.DeviceBuffer(seq * rows * 4)
    rnb.gemv_quantized_dev(quant, wqd, rows, hidden, seq, a)
    rnb.quantize_dev(quant, o_plain, seq, hidden)
    rnb.gemv_quantized_dev(quant, wqd, rows, hidden, seq, b)
    rnb.sync()
    ga, gb = a.to_host(np.float32), b.to_host(np.float32)
    assert np.array_equal(ga.view(np.uint32), gb.view(np.uint32))
    want = oracle.gemv(quant, wq, rows, hidden, plain)
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert float(np.abs(ga.reshape(seq, rows).astype(np.float64) - want).max()) <= 1e-3 * rms
    # out = None: only the quantised form
    rnb.rms_norm_dev(xd, wd, eps, seq, hidden, None, unit_offset=unit, quantize=True)
    rnb.gemv_quantized_dev(quant, wqd, rows, hidden, seq, b)
    rnb.sync()
    assert np.array_equal(b.to_host(np.float32).view(np.uint32), ga.view(np.uint32))
    for buf in (xd, wd, o_plain, o_q, wqd, a, b):
        buf.free()


@pytest.mark.gpu
@pytest.mark.parametrize("seq,hidden,post_unit,pre_unit", [(1, 4096, False, False), (4, 1024, True, False), (2, 2048, False, True)])
def test_rms_norm_add_then_rms_norm_quantize(rnb, oracle, seq, hidden, post_unit, pre_unit):
    rng = np.random.default_rng(900 + hidden)
    inp = rng.standard_normal(seq * hidden).astype(np.float32)
    res = (rng.standard_normal(seq * hidden) * 2.0).astype(np.float32)
    pw = (rng.standard_normal(hidden) * 0.3 + 1.0).astype(np.float32)
    qw = (rng.standard_normal(hidden) * 0.3 + 1.0).astype(np.float32)
    bufs = [rnb.DeviceBuffer.from_host(a) for a in (inp, pw, res, qw)]
    out = rnb.DeviceBuffer(seq * hidden * 4)
    rnb.rms_norm_add_rms_norm_quantize_dev(bufs[0], bufs[1], 1e-6, bufs[2], bufs[3], 1e-5, seq, hidden, out,
                                           post_unit_offset=post_unit, pre_unit_offset=pre_unit)
    rnb.sync()
    got_res, got_out = bufs[2].to_host(np.float32), out.to_host(np.float32)
    normed = oracle.rms_norm(inp, pw, 1e-6, unit_offset=post_unit).ravel()
    want_res = res + normed
    # the sum may cancel: the bound is relative to the addends, not to the sum
    assert np.all(np.abs(got_res.astype(np.float64) - want_res) <= 2e-6 * (np.abs(res) + np.abs(normed)) + 1e-12)
    # the second norm is checked on the residual the kernel itself produced (no compounding of the first's last bit)
    assert _close(got_out, oracle.rms_norm(got_res, qw, 1e-5, unit_offset=pre_unit), 3e-7 if not pre_unit else 2e-6)
    # and the scratch holds the reference quantiser's bits of got_out: the GEMV from it equals the GEMV on got_out
    rows = 128
    wq = oracle.make_weights(Q4_K, rows, hidden, 77)
    wqd = rnb.DeviceBuffer.from_host(wq)
    a, b = rnb.DeviceBuffer(seq * rows * 4), rnb.DeviceBuffer(seq * rows * 4)
    rnb.gemv_quantized_dev(Q4_K, wqd, rows, hidden, seq, a)
    rnb.gemv_dev(Q4_K, wqd, rows, hidden, out, seq, b)
    rnb.sync()
    assert np.array_equal(a.to_host(np.float32).view(np.uint32), b.to_host(np.float32).view(np.uint32))
    for buf in bufs + [out, wqd, a, b]:
        buf.free()


@pytest.mark.gpu
def test_rms_norm_rejects_bad_shapes(rnb):
    x = rnb.DeviceBuffer(4096)
    with pytest.raises(rnb.BackendError) as err:
        rnb.rms_norm_dev(x, x, 1e-5, 1, 300, x)
    assert err.value.kind == "InvalidRequest" and "divisible by 256" in str(err.value)
    x.free()


@pytest.mark.gpu
@pytest.mark.parametrize("tokens,n_expert,k", [(1, 128, 8), (64, 128, 8), (5, 8, 2), (3, 3, 8), (7, 300, 32), (2, 64, 1), (9, 512, 4)])
def test_router_topk_softmax(rnb, oracle, tokens, n_expert, k):
    """Expert ids must equal the oracle's exactly, ties and all; the softmax weights to a few units in the last place
    (the device's expf)."""
    rng = np.random.default_rng(n_expert * 31 + k)
    logits = rng.standard_normal(tokens * n_expert).astype(np.float32)
    lg = logits.reshape(tokens, n_expert)
    lg[0, : min(6, n_expert)] = 1.25           # ties among the largest: the lower ids win, in id order
    if tokens > 1:
        lg[1, :] = np.float32(0.5)             # all equal: ids 0 .. k-1
    if tokens > 2:
        lg[2, ::2] = np.float32(np.nan)        # NaN is never selected
        lg[2, 1] = np.float32(-np.inf)
    sel = min(k, n_expert)
    ld = rnb.DeviceBuffer.from_host(logits)
    idx_d, w_d = rnb.DeviceBuffer(tokens * sel * 4), rnb.DeviceBuffer(tokens * sel * 4)
    rnb.moe_route_topk_dev(ld, tokens, n_expert, k, idx_d, w_d)
    rnb.sync()
    idx, wts = idx_d.to_host(np.uint32).reshape(tokens, sel), w_d.to_host(np.float32).reshape(tokens, sel)
    for t in range(tokens):
        ri, rw = oracle.route_topk(lg[t], k)
        assert np.array_equal(idx[t], ri), (t, idx[t], ri)
        finite = np.isfinite(rw)
        assert np.array_equal(np.isfinite(wts[t]), finite)
        assert np.allclose(wts[t][finite], rw[finite], rtol=2e-6, atol=1e-9)
    for buf in (ld, idx_d, w_d):
        buf.free()
    with pytest.raises(rnb.BackendError):
        rnb.moe_route_topk_dev(ld, 1, 600, 8, idx_d, w_d)


@pytest.mark.gpu
@pytest.mark.parametrize("quant,rows,cols", [(Q4_K, 300, 4096), (Q6_K, 129, 2048), (Q6_K, 40, 14336)])
def test_gemv_with_device_input(rnb, oracle, quant, rows, cols):
    """crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:242-330: host-resident weights, a token that is already on
    the device (here: the output of the device RMS norm), result to the host; the same bits as the all-host call on the
    norm's output, and the reference's texts for its three checks."""
    fn = rnb.q4k_gemv_with_device_input if quant == Q4_K else rnb.q6k_gemv_with_device_input
    host = rnb.q4k_gemv if quant == Q4_K else rnb.q6k_gemv
    label = "Q4_K" if quant == Q4_K else "Q6_K"
    w = oracle.make_weights(quant, rows, cols, 5150 + rows)
    x = oracle.fill_normal(cols, 5151, 2.0)
    nw = np.ones(cols, np.float32)
    xd, wd = rnb.DeviceBuffer.from_host(x), rnb.DeviceBuffer.from_host(nw)
    normed = rnb.DeviceBuffer(cols * 4)
    rnb.rms_norm_dev(xd, wd, 1e-5, 1, cols, normed)
    out = np.zeros(rows + 3, np.float32)
    fn(w, rows, cols, normed, out)
    n_host = normed.to_host(np.float32)
    assert np.array_equal(out[:rows], host(w, rows, cols, n_host)) and np.all(out[rows:] == 0)
    want = oracle.gemv(quant, w, rows, cols, n_host)[0]
    rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    assert float(np.abs(out[:rows].astype(np.float64) - want).max()) <= 1e-3 * rms
    with pytest.raises(rnb.BackendError, match=f"{label} cols must be divisible by 256, got {cols + 1}"):
        fn(w, rows, cols + 1, normed, out)
    with pytest.raises(rnb.BackendError, match=f"{label} weight byte mismatch: got {w.size}, expected"):
        fn(w, rows + 1, cols, normed, out)
    with pytest.raises(rnb.BackendError, match=f"{label} output too small: got {rows - 1}, expected >= {rows}"):
        fn(w, rows, cols, normed, out[:rows - 1])
    rnb.release(w)
    for b in (xd, wd, normed):
        b.free()


@pytest.mark.gpu
def test_decode_layer_fragment_in_a_graph(rnb, oracle):
    """residual += post-norm(branch); pre-norm -> Q8_K in the activation scratch; two projections from that scratch and the
    router on one of their outputs, captured into one graph after an eager run of the same shapes (which sizes the
    scratch): three replays with new inputs uploaded between them, each compared bit for bit with the eager sequence on the
    same inputs.  No quantiser launch and no allocation happens inside the capture."""
    import ctypes as C
    import bench
    hip = bench.Hip()
    lib = rnb.lib()
    stream = C.c_void_p(rnb.stream_handle())
    hidden, rows_a, n_expert, k = 2048, 640, 64, 8
    rng = np.random.default_rng(2024)
    wa = rnb.DeviceBuffer.from_host(oracle.make_weights(Q4_K, rows_a, hidden, 31))
    wr = rnb.DeviceBuffer.from_host(oracle.make_weights(Q6_K, n_expert, hidden, 32))
    pw = rnb.DeviceBuffer.from_host((rng.standard_normal(hidden) * 0.2 + 1.0).astype(np.float32))
    qw = rnb.DeviceBuffer.from_host((rng.standard_normal(hidden) * 0.2 + 1.0).astype(np.float32))
    branch, resid = rnb.DeviceBuffer(hidden * 4), rnb.DeviceBuffer(hidden * 4)
    proj, logits = rnb.DeviceBuffer(rows_a * 4), rnb.DeviceBuffer(n_expert * 4)
    ids, wts = rnb.DeviceBuffer(k * 4), rnb.DeviceBuffer(k * 4)
    inputs = [(rng.standard_normal(hidden).astype(np.float32), rng.standard_normal(hidden).astype(np.float32)) for _ in range(3)]

    def upload(b, r):
        assert lib.rnb_hip_dev_upload(branch.ptr, b.ctypes.data_as(C.c_void_p), b.nbytes) == 0
        assert lib.rnb_hip_dev_upload(resid.ptr, r.ctypes.data_as(C.c_void_p), r.nbytes) == 0

    def enqueue():
        rnb.rms_norm_add_rms_norm_quantize_dev(branch, pw, 1e-6, resid, qw, 1e-5, 1, hidden, None)
        rnb.gemv_quantized_dev(Q4_K, wa, rows_a, hidden, 1, proj)
        rnb.gemv_quantized_dev(Q6_K, wr, n_expert, hidden, 1, logits)
        rnb.moe_route_topk_dev(logits, 1, n_expert, k, ids, wts)

    def results():
        rnb.sync()
        return (resid.to_host(np.float32), proj.to_host(np.float32), ids.to_host(np.uint32), wts.to_host(np.float32))

    eager = []
    for b, r in inputs:
        upload(b, r)
        enqueue()
        eager.append(results())
    graph, gexec = C.c_void_p(), C.c_void_p()
    hip.check(hip.rt.hipStreamBeginCapture(stream, 2), "hipStreamBeginCapture")
    try:
        enqueue()
    finally:
        rc = hip.rt.hipStreamEndCapture(stream, C.byref(graph))
    hip.check(rc, "hipStreamEndCapture")
    hip.check(hip.rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0), "hipGraphInstantiate")
    try:
        for (b, r), want in zip(inputs, eager):
            upload(b, r)
            hip.check(hip.rt.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            got = results()
            for g, w_ in zip(got, want):
                assert np.array_equal(g.view(np.uint32), w_.view(np.uint32))
    finally:
        hip.rt.hipGraphExecDestroy(gexec)
        hip.rt.hipGraphDestroy(graph)
        for buf in (wa, wr, pw, qw, branch, resid, proj, logits, ids, wts):
            buf.free()
