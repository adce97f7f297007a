"""Writes the golden fixtures in this directory from the CPU oracle (run once; outputs are committed).

    python tests/golden/make_golden.py

golden_small.npz   inputs + expected outputs for small cases of every operator on the path, so that a
                   GPU box can check the HIP library with nothing but numpy.
<name>_{w,x,out}.bin  the same matmul cases as raw little-endian files (u8 weights, f32 input, f32 output)
embed_<name>_out.bin  rows [last, 0, 2, 2] of <name>_w.bin dequantised (f32), the embedding-gather cases
                   for the C++ host-mirror test (tests/cpp/host_mirror_test.cpp).
The vectors come from OUR oracle, which tests/test_oracle_pins.py pins against the reference's
known-answer tests; the reference itself (Rust) cannot run here.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as ora  # noqa: E402

Q4_0, Q5_1, Q8_1 = 2, 7, 9
Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 8, 10, 11, 12, 13, 14
IQ2_XXS, IQ3_XXS, IQ2_S, IQ4_XS = 16, 18, 22, 23


def main():
    out = {}
    # activation quantisers (bit-exact contract)
    x = ora.fill_normal(1024, 501, 1.0)
    x[0:7] = [127.0, -0.5, -1.5, -2.5, 0.5, 1.5, 2.5]
    x[300] = -9.0
    x[301] = 9.0
    x[512:768] = 0.0
    q8k = ora.quantize_q8k(x)
    out["actq_x"] = x
    out["q8k_d"], out["q8k_qs"], out["q8k_bsums"] = q8k["d"], q8k["qs"], q8k["bsums"]
    q8 = ora.quantize_q8(x)
    out["q8_d"], out["q8_qs"] = q8["d"], q8["qs"]
    # matmul cases: (name, quant, rows, cols, seq)
    for name, quant, rows, cols, seq in (("q4k_gemv", Q4_K, 24, 1024, 1), ("q6k_gemv", Q6_K, 20, 768, 1),
                                         ("q8_0_gemv", Q8_0, 16, 544, 1), ("q4k_batch", Q4_K, 40, 512, 19),
                                         ("q6k_batch", Q6_K, 9, 512, 3), ("q8_0_batch", Q8_0, 7, 96, 4),
                                         ("q5k_gemv", Q5_K, 22, 1280, 1), ("q5k_batch", Q5_K, 13, 512, 5),
                                         ("q2k_gemv", Q2_K, 18, 768, 1), ("q3k_batch", Q3_K, 11, 512, 6),
                                         ("q4_0_gemv", Q4_0, 21, 608, 1), ("q5_1_batch", Q5_1, 10, 160, 3),
                                         # 16+ tokens: the matrix-core GEMMs of the formats other than Q4_K
                                         ("q8_1_gemv", Q8_1, 19, 160, 1), ("q6k_gemm", Q6_K, 33, 512, 20),
                                         ("q5k_gemm", Q5_K, 40, 256, 17), ("q8_0_gemm", Q8_0, 35, 96, 18),
                                         # importance quants
                                         ("iq4_xs_gemv", IQ4_XS, 17, 768, 1), ("iq2_xxs_batch", IQ2_XXS, 12, 512, 3),
                                         ("iq3_xxs_gemv", IQ3_XXS, 14, 512, 1), ("iq2_s_batch", IQ2_S, 9, 256, 2)):
        w = ora.make_weights(quant, rows, cols, ora.tensor_seed(name, "w"))
        xin = ora.fill_normal(seq * cols, ora.tensor_seed(name, "x"), 1.0)
        ref = ora.gemv(quant, w, rows, cols, xin)
        out[f"{name}_w"], out[f"{name}_x"], out[f"{name}_out"] = w, xin, ref
        out[f"{name}_shape"] = np.array([quant, rows, cols, seq], np.int64)
        w.tofile(os.path.join(HERE, f"{name}_w.bin"))
        xin.astype("<f4").tofile(os.path.join(HERE, f"{name}_x.bin"))
        ref.astype("<f4").tofile(os.path.join(HERE, f"{name}_out.bin"))
    # embedding gather: rows [last, 0, 2, 2] of four of the matrices above, dequantised
    for name in ("q4k_gemv", "q6k_gemv", "q8_0_gemv", "iq2_s_batch"):
        quant, rows, cols, _ = (int(v) for v in out[f"{name}_shape"])
        ids = np.array([rows - 1, 0, 2, 2], np.uint32)
        table = out[f"{name}_w"].reshape(rows, -1)
        emb = np.concatenate([ora.dequantize(quant, table[i]) for i in ids])
        out[f"embed_{name}_ids"], out[f"embed_{name}_out"] = ids, emb
        emb.astype("<f4").tofile(os.path.join(HERE, f"embed_{name}_out.bin"))
    # MoE: 4 experts, 2 tokens, top-2
    n_expert, n_ff, n_embd = 4, 256, 512
    gate = ora.make_weights(Q4_K, n_expert * n_ff, n_embd, ora.tensor_seed("moe", "gate"))
    up = ora.make_weights(Q4_K, n_expert * n_ff, n_embd, ora.tensor_seed("moe", "up"))
    down = ora.make_weights(Q6_K, n_expert * n_embd, n_ff, ora.tensor_seed("moe", "down"))
    xm = ora.fill_normal(2 * n_embd, ora.tensor_seed("moe", "x"), 1.0)
    logits = ora.fill_normal(2 * n_expert, ora.tensor_seed("moe", "logits"), 1.0)
    e, r, t = [], [], []
    for tok in range(2):
        idx, wts = ora.route_topk(logits[tok * n_expert:(tok + 1) * n_expert], 2)
        e += idx.tolist()
        r += wts.tolist()
        t += [tok] * 2
    e, r, t = np.array(e, np.uint32), np.array(r, np.float32), np.array(t, np.uint32)
    out["moe_gate"], out["moe_up"], out["moe_down"], out["moe_x"] = gate, up, down, xm
    out["moe_logits"], out["moe_expert"], out["moe_route"], out["moe_token"] = logits, e, r, t
    out["moe_out"] = ora.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, 2, Q6_K, n_ff, n_embd, xm)
    out["moe_shape"] = np.array([n_expert, n_ff, n_embd, 2], np.int64)
    np.savez_compressed(os.path.join(HERE, "golden_small.npz"), **out)
    print("wrote", os.path.join(HERE, "golden_small.npz"))


if __name__ == "__main__":
    main()
