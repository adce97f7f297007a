"""Resident-weight policy: the table logic on the CPU against a fake allocator (tests/cpp/residency_test.cpp), and on the
device with a byte budget below a call's working set: results still equal the oracle, the table stays inside the
budget, prewarmed ranges survive, the least recently used range is the one that goes.

Reference policy: crates/rnb-memory/src/byte_lru.rs:32-91, crates/rnb-memory/src/sparse_expert_cache.rs:221-250 and
:272-395, crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:1055-1079 and :1263-1459."""
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
Q4_K, Q6_K = 12, 14


def test_table_logic_against_fake_allocator():
    exe = os.path.join(HERE, "cpp", "residency_test")
    if not os.path.exists(exe):
        pytest.skip("tests/cpp/residency_test not built (run __graft_entry__.build())")
    env = dict(os.environ, ASAN_OPTIONS="abort_on_error=0", UBSAN_OPTIONS="halt_on_error=1")
    p = subprocess.run([exe], capture_output=True, text=True, timeout=120, env=env)
    assert p.returncode == 0, p.stdout[-3000:] + p.stderr[-3000:]
    assert " 0 failed" in p.stdout


def _close(got, ref):
    ref = np.asarray(ref, np.float64).ravel()
    got = np.asarray(got, np.float64).ravel()
    tol = np.maximum(1e-3 * np.sqrt(np.mean(ref * ref)), 1e-3 * np.abs(ref))
    return bool(np.all(np.isfinite(got)) and np.all(np.abs(got - ref) <= tol))


@pytest.fixture
def small_budget(rnb):
    """Starts from an empty unpinned table and restores the budget afterwards."""
    rnb.sync()
    rnb.offload_unpinned()
    before = rnb.residency_stats()["budget_bytes"]
    yield rnb
    rnb.offload_unpinned()
    rnb.set_resident_budget(before)


@pytest.mark.gpu
def test_calls_larger_than_the_budget_stay_correct(small_budget, oracle):
    """Dense FFN, QKV and MoE calls whose two or three weight ranges together exceed the budget, none prewarmed: a call
    never frees what it has resolved itself (the ranges that do not fit are uploaded for that call alone), so every
    result equals the oracle, and the table never exceeds the budget."""
    rnb = small_budget
    n_ff, n_embd, seq = 1024, 1024, 3
    gate = oracle.make_weights(Q4_K, n_ff, n_embd, 11)
    up = oracle.make_weights(Q4_K, n_ff, n_embd, 12)
    down = oracle.make_weights(Q6_K, n_embd, n_ff, 13)
    x = oracle.fill_normal(seq * n_embd, 14, 1.0)
    pinned0, _ = rnb.resident_bytes()
    budget = pinned0 + gate.nbytes + up.nbytes // 2  # room for one and a half of the three ranges
    rnb.set_resident_budget(budget)
    ref = oracle.dense_silu_ffn(gate, up, down, Q6_K, n_ff, n_embd, x)
    for _ in range(3):  # also once the reuse history has seen the ranges
        got = rnb.dense_q4k_silu_ffn_batch(gate, up, down, Q6_K, n_ff, n_embd, seq, x)
        assert _close(got, ref)
        assert rnb.resident_bytes()[0] <= budget
    st = rnb.residency_stats()
    assert st["temp_h2d_bytes"] > 0

    q_rows, kv_rows = 1024, 256
    qw = oracle.make_weights(Q4_K, q_rows, n_embd, 21)
    kw = oracle.make_weights(Q4_K, kv_rows, n_embd, 22)
    vw = oracle.make_weights(Q4_K, kv_rows, n_embd, 23)
    x1 = oracle.fill_normal(n_embd, 24, 1.0)
    q, k, v = (np.zeros(n, np.float32) for n in (q_rows, kv_rows, kv_rows))
    rnb.set_resident_budget(pinned0 + qw.nbytes // 2)  # not even the first range fits
    for _ in range(2):
        rnb.dense_q4k_attention_qkv(qw, kw, vw, q_rows, kv_rows, n_embd, x1, q, k, v)
        assert _close(q, oracle.gemv(Q4_K, qw, q_rows, n_embd, x1)) and _close(k, oracle.gemv(Q4_K, kw, kv_rows, n_embd, x1))
        assert _close(v, oracle.gemv(Q4_K, vw, kv_rows, n_embd, x1))
        assert rnb.resident_bytes()[0] <= pinned0 + qw.nbytes // 2

    n_expert, e_ff, e_embd = 8, 256, 512
    eg = oracle.make_weights(Q4_K, n_expert * e_ff, e_embd, 31)
    eu = oracle.make_weights(Q4_K, n_expert * e_ff, e_embd, 32)
    ed = oracle.make_weights(Q6_K, n_expert * e_embd, e_ff, 33)
    h = oracle.fill_normal(2 * e_embd, 34, 1.0)
    ids = np.array([1, 5, 2, 7], np.uint32)
    route = np.array([0.6, 0.4, 0.7, 0.3], np.float32)
    toks = np.array([0, 0, 1, 1], np.uint32)
    rnb.set_resident_budget(pinned0 + eg.nbytes + eu.nbytes // 3)
    mref = oracle.moe_sparse_experts_by_token(eg, eu, ed, n_expert, ids, route, toks, 2, Q6_K, e_ff, e_embd, h)
    for _ in range(2):
        got = rnb.qwen35_sparse_experts_selected_base_by_token(eg, eu, ed, ids, route, toks, 2, Q6_K, e_ff, e_embd, h)
        assert _close(got, mref)
        assert rnb.resident_bytes()[0] <= pinned0 + eg.nbytes + eu.nbytes // 3


@pytest.mark.gpu
def test_eviction_order_admission_and_prewarmed_ranges(small_budget, oracle):
    rnb = small_budget
    rows, cols = 512, 2048
    mats = [oracle.make_weights(Q4_K, rows, cols, 40 + i) for i in range(4)]
    a, b, c, p = mats
    nbytes = a.nbytes
    x = oracle.fill_normal(cols, 50, 1.0)
    refs = [oracle.gemv(Q4_K, m, rows, cols, x)[0] for m in mats]
    pinned0, entries0 = rnb.resident_bytes()
    rnb.prewarm([p])
    rnb.set_resident_budget(pinned0 + nbytes + 2 * nbytes + nbytes // 2)  # the prewarmed range and two and a half more
    s0 = rnb.residency_stats()
    assert _close(rnb.q4k_gemv(a, rows, cols, x), refs[0])
    assert _close(rnb.q4k_gemv(b, rows, cols, x), refs[1])
    assert _close(rnb.q4k_gemv(a, rows, cols, x), refs[0])  # a is now more recent than b
    s1 = rnb.residency_stats()
    assert s1["admissions"] - s0["admissions"] == 2 and s1["hits"] - s0["hits"] == 1
    # the first and second lookups of c do not pay for evicting a range of the same size (bytes * (earlier lookups + 1)
    # must EXCEED bytes + evicted bytes): those calls upload c for themselves only
    for n_seen in (1, 2):
        assert _close(rnb.q4k_gemv(c, rows, cols, x), refs[2])
        s2 = rnb.residency_stats()
        assert s2["evictions"] == s1["evictions"] and s2["temp_h2d_bytes"] - s1["temp_h2d_bytes"] == n_seen * nbytes
    # the third lookup does: b, the least recently used, goes; a and the prewarmed range stay
    assert _close(rnb.q4k_gemv(c, rows, cols, x), refs[2])
    s3 = rnb.residency_stats()
    assert s3["evictions"] - s2["evictions"] == 1 and s3["evicted_bytes"] - s2["evicted_bytes"] == nbytes
    assert rnb.resident_bytes() == (pinned0 + 3 * nbytes, entries0 + 3)
    assert _close(rnb.q4k_gemv(a, rows, cols, x), refs[0])
    assert _close(rnb.q4k_gemv(p, rows, cols, x), refs[3])
    s4 = rnb.residency_stats()
    assert s4["hits"] - s3["hits"] == 2 and s4["misses"] == s3["misses"]  # both were still resident
    assert _close(rnb.q4k_gemv(b, rows, cols, x), refs[1])                # b comes back, correct
    assert rnb.residency_stats()["misses"] - s4["misses"] == 1
    # offload frees what is not prewarmed
    freed = rnb.offload_unpinned()
    assert freed >= 2 * nbytes and rnb.resident_bytes()[0] == pinned0 + nbytes
    assert _close(rnb.q4k_gemv(p, rows, cols, x), refs[3])
    rnb.release(p)
