"""Re-quantisation flips of the two-stage operators (routed MoE, gated FFN), as seen from the oracle.

TEST INFRASTRUCTURE ONLY (tests/, bench.py's cpu_baseline legs): nothing under runnburn_amd/ imports this module.

Both operators quantise an intermediate, act(gate) * up, to Q8_K between their halves
(crates/rnb-llm/src/engine/models/shared_expert_moe/prefill_cpu.rs:167-194).  The f32 summation order of the gate/up
dots differs between any two implementations (the reference's own SIMD and scalar paths included), so an intermediate
value may differ by a unit in the last place; where `value * iscale` sits that close to a half-integer the int8 code
moves by one, and every output that reads it moves by exactly `route * d_mid * W_down[row][element]`.

Two checks are built on that:
  * `moe_flip_units`: per output, the largest single-flip step (the bound used by the sweeps);
  * `moe_explain_by_flips`: the decisive one.  It lists the intermediates within `window` of a half-integer, fits
    `got - ref` with their flip vectors by least squares and reports the residual and the coefficients.  A difference
    that IS a flip has integer coefficients and a residual at f32 noise; an indexing or arithmetic defect does not.
"""
from __future__ import annotations

import numpy as np

from . import oracle as ora

Q4_K = ora.Q4_K
REL = 1e-3


def plain_tolerance(ref: np.ndarray) -> np.ndarray:
    """Per-row tolerance of the single-stage operators: max(1e-3 * rms, 1e-3 * |ref|)."""
    ref = np.asarray(ref, np.float64)
    rms = float(np.sqrt(np.mean(ref * ref))) or 1.0
    return np.maximum(REL * rms, REL * np.abs(ref))


class _SlotCache:
    """Intermediates and dequantised down matrices, by (expert, token) and by expert."""

    def __init__(self, gate_all, up_all, down_all, n_expert, down_quant, n_ff, n_embd, x):
        self.g, self.u, self.d = (ora._u8(a) for a in (gate_all, up_all, down_all))
        self.n_expert, self.dq, self.n_ff, self.n_embd = n_expert, down_quant, n_ff, n_embd
        self.x = ora._f32(x).reshape(-1, n_embd)
        self.pg = self.g.size // n_expert
        self.pd = self.d.size // n_expert
        self._mid, self._w = {}, {}

    def mid(self, expert: int, token: int):
        """(f32 intermediate, its Q8_K blocks) of one slot."""
        key = (expert, token)
        if key not in self._mid:
            sl = slice(expert * self.pg, (expert + 1) * self.pg)
            gg = ora.gemv(Q4_K, self.g[sl], self.n_ff, self.n_embd, self.x[token])[0]
            uu = ora.gemv(Q4_K, self.u[sl], self.n_ff, self.n_embd, self.x[token])[0]
            m = ora.silu_mul(gg, uu)
            self._mid[key] = (m, ora.quantize_q8k(m))
        return self._mid[key]

    def down(self, expert: int) -> np.ndarray:
        """Dequantised down matrix [n_embd][n_ff] of one expert (float64)."""
        if expert not in self._w:
            sl = slice(expert * self.pd, (expert + 1) * self.pd)
            key = self.d[sl].tobytes() if self.pd <= (1 << 22) else None
            for other, (k2, w2) in self._w.items():  # experts that are copies of each other share the matrix
                if key is not None and k2 == key:
                    self._w[expert] = (key, w2)
                    break
            else:
                w = ora.dequantize(self.dq, self.d[sl]).reshape(self.n_embd, self.n_ff).astype(np.float64)
                self._w[expert] = (key, w)
        return self._w[expert][1]


def moe_flip_units(gate_all, up_all, down_all, n_expert, expert_ids, route, token_ids, token_count, down_quant, n_ff,
                   n_embd, x) -> np.ndarray:
    """[token_count][n_embd]: sum over the token's slots of |route| * max_k |d_mid[block of k] * W_down[row][k]|."""
    c = _SlotCache(gate_all, up_all, down_all, n_expert, down_quant, n_ff, n_embd, x)
    units = np.zeros((token_count, n_embd))
    for s in range(len(expert_ids)):
        ex, tok = int(expert_ids[s]), int(token_ids[s])
        _, q = c.mid(ex, tok)
        d_mid = np.abs(q["d"].astype(np.float64))
        w = c.down(ex)
        per_block = np.abs(w).reshape(n_embd, n_ff // 256, 256).max(axis=2)
        units[tok] += abs(float(route[s])) * (per_block * d_mid[None, :]).max(axis=1)
    return units


def moe_explain_by_flips(got, ref, gate_all, up_all, down_all, n_expert, expert_ids, route, token_ids, token_count,
                         down_quant, n_ff, n_embd, x, window: float = 2e-3) -> dict:
    """Fit got - ref, token by token, with the flip vectors of the intermediates whose `value * iscale` lies within
    `window` of a half-integer.  Returns {"explained", "residual_over_rms", "flips": [(slot, element, distance, step)],
    "candidates"}: `explained` is true when the residual after the fit is f32 noise (<= 5e-6 of the output rms) and
    every coefficient is within 0.02 of an integer."""
    got = np.asarray(got, np.float64).reshape(token_count, n_embd)
    ref = np.asarray(ref, np.float64).reshape(token_count, n_embd)
    rms = float(np.sqrt(np.mean(ref * ref))) or 1.0
    c = _SlotCache(gate_all, up_all, down_all, n_expert, down_quant, n_ff, n_embd, x)
    flips, worst_resid, n_cand, integer = [], 0.0, 0, True
    for tok in range(token_count):
        diff = got[tok] - ref[tok]
        if np.abs(diff).max() <= 5e-6 * rms:
            continue
        cands, vecs, merged = [], [], {}
        for s in np.nonzero(np.asarray(token_ids) == tok)[0]:
            ex = int(expert_ids[s])
            m, q = c.mid(ex, tok)
            w = c.down(ex)
            for b in range(n_ff // 256):
                blk = m[b * 256:(b + 1) * 256].astype(np.float64)
                amax = blk[np.argmax(np.abs(blk))]
                if amax == 0.0:
                    continue
                v = blk * (-127.0 / amax)
                dist = np.abs(v - np.floor(v) - 0.5)
                for j in np.nonzero(dist < window)[0]:
                    # Slots whose experts are copies of one another see the same token with the same weights: the same
                    # intermediate, which rounds the same way in all of them.  Their flip vectors are parallel (they
                    # differ by the route weight only), so they are one candidate: the sum.
                    key = (b * 256 + int(j), float(m[b * 256 + j]), w[:, b * 256 + j].tobytes())
                    vec = float(route[s]) * float(q["d"][b]) * w[:, b * 256 + j]
                    if key in merged:
                        vecs[merged[key]] = vecs[merged[key]] + vec
                    else:
                        merged[key] = len(cands)
                        cands.append((int(s), b * 256 + int(j), float(dist[j])))
                        vecs.append(vec)
        n_cand += len(cands)
        if not cands:
            worst_resid = max(worst_resid, float(np.abs(diff).max() / rms))
            continue
        a = np.stack(vecs, axis=1)
        coef, *_ = np.linalg.lstsq(a, diff, rcond=None)
        worst_resid = max(worst_resid, float(np.abs(diff - a @ coef).max() / rms))
        for (s, el, dist), co in zip(cands, coef):
            if abs(co) > 0.02:
                flips.append((s, el, dist, float(co)))
                integer = integer and abs(co - round(co)) <= 0.02
    return {"explained": bool(worst_resid <= 5e-6 and integer), "residual_over_rms": worst_resid, "flips": flips,
            "candidates": n_cand}


def moe_verdict(got, ref, gate_all, up_all, down_all, n_expert, expert_ids, route, token_ids, token_count, down_quant,
                n_ff, n_embd, x) -> dict:
    """What bench.py and the tests report for one MoE call against the oracle: plain per-row tolerance first; if any
    output is outside it, whether the difference is made of whole re-quantisation flips."""
    got = np.asarray(got, np.float64).reshape(token_count, n_embd)
    ref = np.asarray(ref, np.float64).reshape(token_count, n_embd)
    tol = plain_tolerance(ref)
    diff = np.abs(got - ref)
    finite = bool(np.all(np.isfinite(got)))
    n_out = int(np.count_nonzero(diff > tol))
    res = {"ok": bool(finite and n_out == 0), "n_outside": n_out, "worst_over_tol": float((diff / tol).max()),
           "flip_aware_ok": bool(finite and n_out == 0)}
    if finite and n_out:
        ex = moe_explain_by_flips(got, ref, gate_all, up_all, down_all, n_expert, expert_ids, route, token_ids, token_count,
                                  down_quant, n_ff, n_embd, x)
        res["flip_aware_ok"] = ex["explained"]
        res["flips"] = [{"slot": s, "element": el, "distance_to_half": d, "step": co} for s, el, d, co in ex["flips"]]
        res["residual_over_rms_after_flips"] = ex["residual_over_rms"]
    return res
