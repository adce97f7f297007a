"""Golden fixtures (tests/golden/, written by tests/golden/make_golden.py from the oracle):
 * CPU: the oracle still reproduces them bit-for-bit (regression pin of the checker);
 * GPU: the HIP library, through the Python binding and through the C++ host mirror, reproduces them."""
import os
import subprocess

import numpy as np
import pytest

from tests import npref

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")
CPP_BIN = os.path.join(HERE, "cpp", "host_mirror_test")
MATMUL_CASES = ["q4k_gemv", "q6k_gemv", "q8_0_gemv", "q4k_batch", "q6k_batch", "q8_0_batch", "q5k_gemv", "q5k_batch", "q2k_gemv",
                "q3k_batch", "q4_0_gemv", "q5_1_batch", "q8_1_gemv", "q6k_gemm", "q5k_gemm", "q8_0_gemm",
                "iq4_xs_gemv", "iq2_xxs_batch", "iq3_xxs_gemv", "iq2_s_batch"]
EMBED_CASES = ["q4k_gemv", "q6k_gemv", "q8_0_gemv", "iq2_s_batch"]


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(GOLD, "golden_small.npz"))


def test_oracle_reproduces_golden(oracle, gold):
    q = oracle.quantize_q8k(gold["actq_x"])
    assert np.array_equal(q["d"], gold["q8k_d"]) and np.array_equal(q["qs"], gold["q8k_qs"])
    assert np.array_equal(q["bsums"], gold["q8k_bsums"])
    q = oracle.quantize_q8(gold["actq_x"])
    assert np.array_equal(q["d"], gold["q8_d"]) and np.array_equal(q["qs"], gold["q8_qs"])
    for name in MATMUL_CASES:
        quant, rows, cols, seq = (int(v) for v in gold[f"{name}_shape"])
        out = oracle.gemv(quant, gold[f"{name}_w"], rows, cols, gold[f"{name}_x"])
        assert np.array_equal(out, gold[f"{name}_out"]), name
        raw = np.fromfile(os.path.join(GOLD, f"{name}_out.bin"), dtype="<f4")
        assert np.array_equal(raw, gold[f"{name}_out"].ravel())
    for name in EMBED_CASES:
        quant, rows, cols, _ = (int(v) for v in gold[f"{name}_shape"])
        table = gold[f"{name}_w"].reshape(rows, -1)
        emb = np.concatenate([oracle.dequantize(quant, table[i]) for i in gold[f"embed_{name}_ids"]])
        assert np.array_equal(emb.view(np.uint32), gold[f"embed_{name}_out"].view(np.uint32)), name
        raw = np.fromfile(os.path.join(GOLD, f"embed_{name}_out.bin"), dtype="<f4")
        assert np.array_equal(raw.view(np.uint32), emb.view(np.uint32))
    n_expert, n_ff, n_embd, tokens = (int(v) for v in gold["moe_shape"])
    out = oracle.moe_sparse_experts_by_token(gold["moe_gate"], gold["moe_up"], gold["moe_down"], n_expert,
                                             gold["moe_expert"], gold["moe_route"], gold["moe_token"], tokens, 14, n_ff,
                                             n_embd, gold["moe_x"])
    assert np.array_equal(out, gold["moe_out"])
    for tok in range(tokens):
        idx, wts = oracle.route_topk(gold["moe_logits"][tok * n_expert:(tok + 1) * n_expert], 2)
        assert np.array_equal(idx, gold["moe_expert"][2 * tok:2 * tok + 2])
        assert np.array_equal(wts, gold["moe_route"][2 * tok:2 * tok + 2])


def test_cpp_host_mirror_validation_messages():
    if not os.path.exists(CPP_BIN):
        pytest.skip("tests/cpp/host_mirror_test not built (run __graft_entry__.build())")
    p = subprocess.run([CPP_BIN, "validate"], capture_output=True, text=True, timeout=60)
    assert p.returncode == 0, p.stdout + p.stderr


@pytest.mark.gpu
def test_hip_reproduces_golden(rnb, gold):
    q = rnb.quantize_input_q8k(gold["actq_x"])
    assert np.array_equal(q["d"].view(np.uint32), gold["q8k_d"].view(np.uint32))
    assert np.array_equal(q["qs"], gold["q8k_qs"]) and np.array_equal(q["bsums"], gold["q8k_bsums"])
    q = rnb.quantize_input_q8(gold["actq_x"])
    assert np.array_equal(q["d"].view(np.uint32), gold["q8_d"].view(np.uint32)) and np.array_equal(q["qs"], gold["q8_qs"])
    fns = {"q4k_gemv": rnb.q4k_gemv, "q6k_gemv": rnb.q6k_gemv, "q8_0_gemv": rnb.q8_0_gemv,
           "q4k_batch": rnb.q4k_gemv_batch, "q6k_batch": rnb.q6k_gemv_batch, "q8_0_batch": rnb.q8_0_gemv_batch,
           "q5k_gemv": rnb.q5k_gemv, "q5k_batch": rnb.q5k_gemv_batch, "q2k_gemv": rnb.q2k_gemv,
           "q3k_batch": rnb.q3k_gemv_batch, "q4_0_gemv": rnb.q4_0_gemv, "q5_1_batch": rnb.q5_1_gemv_batch,
           "q8_1_gemv": rnb.q8_1_gemv, "q6k_gemm": rnb.q6k_gemv_batch, "q5k_gemm": rnb.q5k_gemv_batch,
           "q8_0_gemm": rnb.q8_0_gemv_batch, "iq4_xs_gemv": rnb.iq4_xs_gemv, "iq2_xxs_batch": rnb.iq2_xxs_gemv_batch,
           "iq3_xxs_gemv": rnb.iq3_xxs_gemv, "iq2_s_batch": rnb.iq2_s_gemv_batch}
    for name in MATMUL_CASES:
        _, rows, cols, _ = (int(v) for v in gold[f"{name}_shape"])
        w = np.ascontiguousarray(gold[f"{name}_w"])
        got = fns[name](w, rows, cols, gold[f"{name}_x"])
        bad, diff, _ = npref.close_rows(got, gold[f"{name}_out"], rel=1e-3)
        assert np.all(np.isfinite(got)) and bad.size == 0, (name, diff.max())
        rnb.release(w)
    for name in EMBED_CASES:  # embedding gather: the dequantiser's bits
        quant, rows, cols, _ = (int(v) for v in gold[f"{name}_shape"])
        got = rnb.quant_embedding_gather(quant, np.ascontiguousarray(gold[f"{name}_w"]), rows, cols, gold[f"embed_{name}_ids"])
        assert np.array_equal(got.view(np.uint32), gold[f"embed_{name}_out"].view(np.uint32)), name
    n_expert, n_ff, n_embd, tokens = (int(v) for v in gold["moe_shape"])
    g, u, d = (np.ascontiguousarray(gold[k]) for k in ("moe_gate", "moe_up", "moe_down"))
    got = rnb.qwen35_sparse_experts_selected_base_by_token(g, u, d, gold["moe_expert"], gold["moe_route"],
                                                           gold["moe_token"], tokens, 14, n_ff, n_embd, gold["moe_x"])
    bad, diff, _ = npref.close_rows(got, gold["moe_out"], rel=1e-3)
    assert bad.size == 0, diff.max()
    for w in (g, u, d):
        rnb.release(w)


@pytest.mark.gpu
def test_cpp_host_mirror_reproduces_golden(rnb):
    if not os.path.exists(CPP_BIN):
        pytest.skip("tests/cpp/host_mirror_test not built (run __graft_entry__.build())")
    p = subprocess.run([CPP_BIN, "run", GOLD], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, p.stdout + p.stderr
    assert "run: 0 failure(s)" in p.stdout
