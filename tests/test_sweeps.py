"""Seeded sweeps of the two-stage operators (dense gated FFN, routed MoE) against the oracle, with a tolerance that
knows about re-quantisation flips.

Both operators quantise an intermediate, act(gate) * up, to Q8_K between their halves.  A difference of one unit in the
last place of that intermediate (the f32 summation order of the gate/up dots differs between any two implementations,
the reference's own SIMD and scalar paths included) can move one rounding: one int8 code changes by 1, and every output
that reads it moves by route * d_mid * w_down.  So an output may differ from the oracle's by the per-row tolerance of
the single-stage operators (max(1e-3 * rms, 1e-3 * |ref|)) PLUS a few such units; `flip_unit` below computes the unit
for every output from the oracle's own intermediate and the dequantised down weights.  The tests stop at the first
case outside it.

CPU: the oracle's down projection on an intermediate perturbed by one part in 1e7 shows the effect without any GPU.
GPU: the library against the oracle over shapes drawn from fixed seeds (all MoE paths: one-token decode, integer-dot
batches, matrix-core batches; FFN: GEMV and GEMM paths)."""
import numpy as np
import pytest

Q4_K, Q5_K, Q6_K = 12, 13, 14
REL = 1e-3
FLIPS = 3  # units of one re-quantisation flip allowed on top of the single-stage tolerance


def _mid_scales(oracle, gate, up, n_ff, n_embd, x_tok):
    """The oracle's intermediate of one token through one gate/up pair: (f32 mid, per-block Q8_K scale d_mid)."""
    g = oracle.gemv(Q4_K, gate, n_ff, n_embd, x_tok)[0]
    u = oracle.gemv(Q4_K, up, n_ff, n_embd, x_tok)[0]
    mid = oracle.silu_mul(g, u)
    return mid, np.abs(oracle.quantize_q8k(mid)["d"].astype(np.float64))


def _flip_unit(oracle, down, down_quant, n_embd, n_ff, d_mid):
    """max over k of |d_mid[block of k] * W_down[r][k]| for every output row r."""
    w = oracle.dequantize(down_quant, down).reshape(n_embd, n_ff).astype(np.float64)
    per_block = np.abs(w).reshape(n_embd, n_ff // 256, 256).max(axis=2)  # [row][block]
    return (per_block * d_mid[None, :]).max(axis=1)


def _within(got, ref, unit):
    ref = np.asarray(ref, np.float64)
    got = np.asarray(got, np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) or 1.0
    tol = np.maximum(REL * rms, REL * np.abs(ref)) + FLIPS * unit
    diff = np.abs(got - ref)
    plain = np.maximum(REL * rms, REL * np.abs(ref))
    return bool(np.all(np.isfinite(got)) and np.all(diff <= tol)), int(np.count_nonzero(diff > plain)), float(diff.max() / rms)


def _ffn_case(oracle, seed):
    rng = np.random.default_rng(seed)
    n_ff = int(rng.choice([256, 512, 1024, 1536]))
    n_embd = int(rng.choice([256, 512, 1024, 2048]))
    seq = int(rng.choice([1, 2, 3, 5, 8, 17, 33, 64]))
    dq = int(rng.choice([Q4_K, Q5_K, Q6_K]))
    gate = oracle.make_weights(Q4_K, n_ff, n_embd, 9000 + seed)
    up = oracle.make_weights(Q4_K, n_ff, n_embd, 9100 + seed)
    down = oracle.make_weights(dq, n_embd, n_ff, 9200 + seed)
    x = oracle.fill_normal(seq * n_embd, 9300 + seed, 1.0)
    return n_ff, n_embd, seq, dq, gate, up, down, x


def _ffn_units(oracle, case):
    n_ff, n_embd, seq, dq, gate, up, down, x = case
    units = np.empty((seq, n_embd))
    for s in range(seq):
        _, d_mid = _mid_scales(oracle, gate, up, n_ff, n_embd, x[s * n_embd:(s + 1) * n_embd])
        units[s] = _flip_unit(oracle, down, dq, n_embd, n_ff, d_mid)
    return units


def _moe_case(oracle, seed):
    rng = np.random.default_rng(seed)
    tokens = int(rng.choice([1, 2, 3, 5, 16, 17, 33, 64]))
    n_expert = int(rng.choice([2, 3, 8, 16]))
    k = min(int(rng.choice([1, 2, 4, 8])), n_expert)
    n_ff = int(rng.choice([256, 512, 768]))
    n_embd = int(rng.choice([256, 512, 1280]))
    dq = int(rng.choice([Q4_K, Q5_K, Q6_K]))
    gate = oracle.make_weights(Q4_K, n_expert * n_ff, n_embd, 7000 + seed)
    up = oracle.make_weights(Q4_K, n_expert * n_ff, n_embd, 7100 + seed)
    down = oracle.make_weights(dq, n_expert * n_embd, n_ff, 7200 + seed)
    x = oracle.fill_normal(tokens * n_embd, 7300 + seed, 1.0)
    logits = oracle.fill_normal(tokens * n_expert, 7400 + seed, 1.0)
    e, r, t = [], [], []
    for tok in range(tokens):
        idx, wts = oracle.route_topk(logits[tok * n_expert:(tok + 1) * n_expert], k)
        e += idx.tolist()
        r += wts.tolist()
        t += [tok] * len(idx)
    return (tokens, n_expert, n_ff, n_embd, dq, gate, up, down, x, np.array(e, np.uint32), np.array(r, np.float32),
            np.array(t, np.uint32))


def _moe_units(oracle, case):
    tokens, n_expert, n_ff, n_embd, dq, gate, up, down, x, e, r, t = case
    pg = gate.size // n_expert
    pd = down.size // n_expert
    units = np.zeros((tokens, n_embd))
    for slot in range(e.size):
        ex, tok = int(e[slot]), int(t[slot])
        _, d_mid = _mid_scales(oracle, gate[ex * pg:(ex + 1) * pg], up[ex * pg:(ex + 1) * pg], n_ff, n_embd,
                               x[tok * n_embd:(tok + 1) * n_embd])
        units[tok] += abs(float(r[slot])) * _flip_unit(oracle, down[ex * pd:(ex + 1) * pd], dq, n_embd, n_ff, d_mid)
    return units


# ---- CPU: the oracle's second stage on intermediates one part in 1e7 apart ----------------------------------------------

def test_oracle_second_stage_jumps_by_flips_only(oracle):
    """The dense FFN composed from the oracle's pieces, with the f32 intermediate act(gate) * up perturbed by one part in
    1e7 (at most a unit in the last place per element, what a different summation order of the gate/up dots does)
    before it is re-quantised: the down projection moves by whole re-quantisation flips, possibly beyond the plain
    tolerance, never beyond the flip-aware bound.  The first stage alone is continuous."""
    outside_plain = 0
    for seed in range(16):
        case = _ffn_case(oracle, 100 + seed)
        n_ff, n_embd, seq, dq, gate, up, down, x = case
        g = oracle.gemv(Q4_K, gate, n_ff, n_embd, x)
        u = oracle.gemv(Q4_K, up, n_ff, n_embd, x)
        mid = oracle.silu_mul(g.ravel(), u.ravel())
        rng = np.random.default_rng(seed)
        mid2 = (mid.astype(np.float64) * (1.0 + 1e-7 * rng.standard_normal(mid.size))).astype(np.float32)
        a = oracle.gemv(dq, down, n_embd, n_ff, mid)
        b = oracle.gemv(dq, down, n_embd, n_ff, mid2)
        ok, n_plain, worst = _within(b, a, _ffn_units(oracle, case))
        assert ok, f"FFN seed {seed}: second stage outside the flip-aware tolerance (worst {worst:.2e} of rms)"
        outside_plain += n_plain
    print(f"outputs outside the plain tolerance over 16 perturbed FFN intermediates: {outside_plain}")


# ---- GPU sweeps -----------------------------------------------------------------------------------------------------

@pytest.mark.gpu
def test_moe_sweep_against_oracle(rnb, oracle):
    for seed in range(40):
        case = _moe_case(oracle, seed)
        tokens, n_expert, n_ff, n_embd, dq, gate, up, down, x, e, r, t = case
        got = rnb.qwen35_sparse_experts_selected_base_by_token(gate, up, down, e, r, t, tokens, dq, n_ff, n_embd, x)
        ref = oracle.moe_sparse_experts_by_token(gate, up, down, n_expert, e, r, t, tokens, dq, n_ff, n_embd, x)
        ok, n_plain, worst = _within(got, ref, _moe_units(oracle, case))
        for wts in (gate, up, down):
            rnb.release(wts)
        assert ok, (f"MoE seed {seed} (tokens {tokens}, experts {n_expert}, k {e.size // tokens}, n_ff {n_ff}, n_embd {n_embd}, "
                    f"down {dq}): worst {worst:.2e} of rms, {n_plain} outputs outside the plain tolerance")


@pytest.mark.gpu
def test_dense_ffn_sweep_against_oracle(rnb, oracle):
    for seed in range(30):
        case = _ffn_case(oracle, seed)
        n_ff, n_embd, seq, dq, gate, up, down, x = case
        if seq == 1:
            got = rnb.dense_q4k_gelu_ffn(gate, up, down, dq, n_ff, n_embd, x)
            ref = oracle.dense_gelu_ffn(gate, up, down, dq, n_ff, n_embd, x)
        else:
            got = rnb.dense_q4k_silu_ffn_batch(gate, up, down, dq, n_ff, n_embd, seq, x)
            ref = oracle.dense_silu_ffn(gate, up, down, dq, n_ff, n_embd, x)
        units = _ffn_units(oracle, case)  # SiLU and GELU intermediates have the same order of magnitude
        ok, n_plain, worst = _within(np.asarray(got).reshape(seq, n_embd), np.asarray(ref).reshape(seq, n_embd), units)
        for wts in (gate, up, down):
            rnb.release(wts)
        assert ok, (f"FFN seed {seed} (seq {seq}, n_ff {n_ff}, n_embd {n_embd}, down {dq}): worst {worst:.2e} of rms, "
                    f"{n_plain} outputs outside the plain tolerance")
