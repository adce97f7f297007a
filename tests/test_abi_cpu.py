"""No-GPU checks of the C-ABI library: it loads, exports every symbol include/rnb_hip.h declares,
validates requests with the reference's messages before touching a device, and reports a
distinguishable NoDevice status so callers can skip (crates/rnb-backend/cuda/src/runtime/tests.rs:22831-22834)."""
import os
import re

import numpy as np
import pytest

import runnburn_amd as rnb
from runnburn_amd import binding

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "rnb_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(rnb_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 25
    L = rnb.lib()
    for name in names:
        assert hasattr(L, name), f"{name} declared in include/rnb_hip.h but not exported"
    bound = {s[0] for s in binding.SYMBOLS}
    assert bound == set(names), (sorted(bound - set(names)), sorted(set(names) - bound))


def test_trait_facade():
    b = rnb.HipBackend()
    assert b.kind() == "Hip" and b.kind_ordinal() == 6
    caps = b.capabilities()
    assert caps == {"MatMul": True, "Attention": False, "Gdn": False, "MoE": True, "Sampler": False}
    assert b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q4_K) and b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q8_0)
    assert b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q5_K) and b.supports_quant(rnb.OP_MOE, rnb.GGML_Q5_K)
    assert b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q2_K) and b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q3_K)
    assert b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q4_0) and b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q5_1)
    assert b.supports_quant(rnb.OP_MATMUL, rnb.GGML_Q8_1)
    for iq in (rnb.GGML_IQ2_XXS, rnb.GGML_IQ2_S, rnb.GGML_IQ3_XXS, rnb.GGML_IQ4_XS):
        assert b.supports_quant(rnb.OP_MATMUL, iq) and not b.supports_quant(rnb.OP_MOE, iq)
    assert not b.supports_quant(rnb.OP_MATMUL, 17) and not b.supports_quant(rnb.OP_MOE, rnb.GGML_Q8_0)  # IQ2_XS; Q8_0 down
    with pytest.raises(rnb.BackendError) as ei:
        b.execute(object())
    assert ei.value.kind == "UnsupportedOp"


def _err(fn, *args, **kwargs):
    with pytest.raises(rnb.BackendError) as ei:
        fn(*args, **kwargs)
    return ei.value


def test_matmul_validation_messages_match_reference():
    """crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:189-206, 352-358, 2289-2307, 1992-2009"""
    z = np.zeros
    e = _err(rnb.q4k_gemv, z(144, np.uint8), 1, 255, z(255, np.float32))
    assert (e.kind, str(e)) == ("InvalidRequest", "Q4_K cols must be divisible by 256, got 255")
    e = _err(rnb.q4k_gemv, z(143, np.uint8), 1, 256, z(256, np.float32))
    assert str(e) == "Q4_K weight byte mismatch: got 143, expected 144"
    e = _err(rnb.q4k_gemv, z(144, np.uint8), 1, 256, z(255, np.float32))
    assert str(e) == "Q4_K input length mismatch: got 255, expected 256"
    out = np.zeros(1, np.float32)
    e = _err(rnb.q4k_gemv_into, z(288, np.uint8), 2, 256, z(256, np.float32), out)
    assert str(e) == "Q4_K shape mismatch: input=256 output=1 expected input=256 output>=2"
    e = _err(rnb.q4k_gemv_batch, z(144, np.uint8), 1, 256, z(300, np.float32))
    assert str(e) == "Q4_K batch input length 300 is not divisible by cols 256"
    # crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:374-496, 1983-2075
    for fn, label, nbytes in ((rnb.q4_0_gemv, "Q4_0", 18), (rnb.q4_1_gemv, "Q4_1", 20), (rnb.q5_0_gemv, "Q5_0", 22),
                              (rnb.q5_1_gemv, "Q5_1", 24), (rnb.q8_1_gemv, "Q8_1", 36)):
        e = _err(fn, z(nbytes, np.uint8), 1, 33, z(33, np.float32))
        assert str(e) == f"{label} cols must be divisible by 32, got 33"
        e = _err(fn, z(nbytes + 1, np.uint8), 1, 32, z(32, np.float32))
        assert str(e) == f"{label} weight byte mismatch: got {nbytes + 1}, expected {nbytes}"
        e = _err(fn, z(nbytes, np.uint8), 1, 32, z(31, np.float32))
        assert str(e) == f"{label} input length mismatch: got 31, expected 32"
    e = _err(rnb.q5_1_gemv_batch, z(24, np.uint8), 1, 32, z(40, np.float32))
    assert str(e) == "Q5_1 batch input length 40 is not divisible by cols 32"
    e = _err(rnb.q8_1_gemv_batch, z(36, np.uint8), 1, 32, z(40, np.float32))  # quant_api.rs:1737-1742
    assert str(e) == "Q8_1 batch input length 40 is not divisible by cols 32"
    # crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:73-181
    e = _err(rnb.q2k_gemv, z(84, np.uint8), 1, 100, z(100, np.float32))
    assert str(e) == "Q2_K cols must be divisible by 256, got 100"
    e = _err(rnb.q2k_gemv, z(85, np.uint8), 1, 256, z(256, np.float32))
    assert str(e) == "Q2_K weight byte mismatch: got 85, expected 84"
    e = _err(rnb.q3k_gemv, z(110, np.uint8), 1, 256, z(255, np.float32))
    assert str(e) == "Q3_K input length mismatch: got 255, expected 256"
    e = _err(rnb.q3k_gemv_batch, z(110, np.uint8), 1, 256, z(300, np.float32))
    assert str(e) == "Q3_K batch input length 300 is not divisible by cols 256"
    # crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:2207-2281, 3957-3993
    e = _err(rnb.q5k_gemv, z(176, np.uint8), 1, 100, z(100, np.float32))
    assert str(e) == "Q5_K cols must be divisible by 256, got 100"
    e = _err(rnb.q5k_gemv, z(175, np.uint8), 1, 256, z(256, np.float32))
    assert str(e) == "Q5_K weight byte mismatch: got 175, expected 176"
    e = _err(rnb.q5k_gemv, z(176, np.uint8), 1, 256, z(255, np.float32))
    assert str(e) == "Q5_K input length mismatch: got 255, expected 256"
    e = _err(rnb.q5k_gemv_into, z(352, np.uint8), 2, 256, z(256, np.float32), out)
    assert str(e) == "Q5_K shape mismatch: input=256 output=1 expected input=256 output>=2"
    e = _err(rnb.q5k_gemv_batch, z(176, np.uint8), 1, 256, z(300, np.float32))
    assert str(e) == "Q5_K batch input length 300 is not divisible by cols 256"
    e = _err(rnb.q6k_gemv, z(210, np.uint8), 1, 100, z(100, np.float32))
    assert str(e) == "Q6_K cols must be divisible by 256, got 100"
    e = _err(rnb.q6k_gemv, z(200, np.uint8), 1, 256, z(256, np.float32))
    assert str(e) == "Q6_K weight byte mismatch: got 200, expected 210"
    e = _err(rnb.q6k_gemv_batch, z(210, np.uint8), 1, 256, z(257, np.float32))
    assert str(e) == "Q6_K batch input length 257 is not divisible by cols 256"
    e = _err(rnb.q8_0_gemv, z(34, np.uint8), 1, 31, z(31, np.float32))
    assert str(e) == "Q8_0 cols must be divisible by 32, got 31"
    e = _err(rnb.q8_0_gemv, z(35, np.uint8), 1, 32, z(32, np.float32))
    assert str(e) == "Q8_0 weight byte mismatch: got 35, expected 34"
    e = _err(rnb.q8_0_gemv, z(34, np.uint8), 1, 32, z(33, np.float32))
    assert str(e) == "Q8_0 input length mismatch: got 33, expected 32"


def test_dense_gelu_ffn_validation_messages():
    """crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:191-232 (one token) and dense.rs:1712-1765 with "GELU"."""
    z = np.zeros
    g = z(256 * 144, np.uint8)
    f = rnb.dense_q4k_gelu_ffn
    e = _err(f, g, g, z(256 * 210, np.uint8), 14, 256, 256, z(255, np.float32))
    assert str(e) == "dense GELU FFN input length mismatch: got 255, expected 256"
    e = _err(f, g, g, z(256 * 210, np.uint8), 14, 250, 256, z(256, np.float32))
    assert str(e) == "dense GELU FFN dims must be divisible by 256, got n_ff=250 n_embd=256"
    e = _err(f, g, g, z(256 * 8 * 34, np.uint8), 8, 256, 256, z(256, np.float32))
    assert str(e) == "unsupported dense GELU FFN down quant code 8"
    e = _err(f, g[:-1], g, z(256 * 210, np.uint8), 14, 256, 256, z(256, np.float32))
    assert str(e) == "dense GELU FFN gate byte mismatch: got 36863, expected 36864"
    e = _err(f, g, g, z(256 * 176 + 2, np.uint8), 13, 256, 256, z(256, np.float32))
    assert str(e) == "dense GELU FFN down byte mismatch: got 45058, expected 45056"
    fb = rnb.dense_q4k_gelu_ffn_batch
    e = _err(fb, g, g, z(256 * 210, np.uint8), 14, 256, 256, 1, z(256, np.float32))
    assert str(e) == "dense GELU FFN batch requires seq_len > 1, got 1"
    e = _err(fb, g, g, z(10, np.uint8), 2, 256, 256, 2, z(512, np.float32))
    assert str(e) == "unsupported dense GELU FFN batch down quant code 2"
    e = _err(fb, g, g[:-2], z(256 * 210, np.uint8), 14, 256, 256, 2, z(512, np.float32))
    assert str(e) == "dense GELU FFN batch up byte mismatch: got 36862, expected 36864"


def test_dense_qkv_validation_messages():
    """crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:928-968"""
    z = np.zeros
    f = rnb.dense_q4k_attention_qkv
    w2, w1 = z(2 * 144, np.uint8), z(144, np.uint8)
    q, k, v = z(2, np.float32), z(1, np.float32), z(1, np.float32)
    e = _err(f, w2, w1, w1, 2, 1, 256, z(255, np.float32), q, k, v)
    assert str(e) == "dense QKV input length mismatch: got 255, expected 256"
    e = _err(f, w2, w1, w1, 2, 1, 100, z(100, np.float32), q, k, v)
    assert str(e) == "dense QKV cols must be divisible by 256, got 100"
    e = _err(f, w2, w1, w1, 2, 1, 256, z(256, np.float32), q[:1], k, v)
    assert str(e) == "dense QKV output length mismatch: q=1 k=1 v=1 expected q>=2 k/v>=1"
    e = _err(f, w2[:-1], w1, w1, 2, 1, 256, z(256, np.float32), q, k, v)
    assert str(e) == "dense QKV q byte mismatch: got 287, expected 288"
    e = _err(f, w2, w2, w1, 2, 1, 256, z(256, np.float32), q, k, v)
    assert str(e) == "dense QKV k byte mismatch: got 288, expected 144"
    e = _err(f, w2, w1, w2, 2, 1, 256, z(256, np.float32), q, k, v)
    assert str(e) == "dense QKV v byte mismatch: got 288, expected 144"


def test_argmax_entry_points_validate_like_their_gemv():
    z = np.zeros
    e = _err(rnb.q8_0_gemv_argmax, z(34, np.uint8), 1, 31, z(31, np.float32))
    assert str(e) == "Q8_0 cols must be divisible by 32, got 31"
    e = _err(rnb.q8_0_gemv_argmax, z(35, np.uint8), 1, 32, z(32, np.float32))
    assert str(e) == "Q8_0 weight byte mismatch: got 35, expected 34"
    e = _err(rnb.q6k_gemv_argmax, z(210, np.uint8), 1, 256, z(255, np.float32))
    assert str(e) == "Q6_K input length mismatch: got 255, expected 256"
    e = _err(rnb.q8_0_gemv_argmax, z(0, np.uint8), 0, 32, z(32, np.float32))
    assert str(e) == "Q8_0 argmax needs at least one row"


def test_shapes_beyond_32_bit_indexing_are_refused():
    z = np.zeros
    e = _err(rnb.q4k_gemv_batch, z(0, np.uint8), 0, 1 << 32, z(0, np.float32))
    assert str(e) == "Q4_K shape out of range: rows=0 cols=4294967296 seq_len=0"
    e = _err(rnb.q8_0_gemv_batch, z(0, np.uint8), 0, 1 << 31, z(0, np.float32))
    assert "shape out of range" in str(e)
    e = _err(rnb.qwen35_sparse_experts_selected_base_by_token, z(0, np.uint8), z(0, np.uint8), z(0, np.uint8), [], [], [],
             0, 14, 1 << 24, 256, z(0, np.float32))
    assert str(e) == "Qwen35 full-layer dims out of range"


def test_moe_validation_messages():
    """crates/rnb-backend/cuda/src/runtime/helpers.rs:1570-1600, 2747-2800"""
    z = np.zeros
    n_ff, n_embd = 256, 256
    per_gate, per_down = n_ff * 144, n_embd * 210
    g, u, d = z(2 * per_gate, np.uint8), z(2 * per_gate, np.uint8), z(2 * per_down, np.uint8)
    x = z(n_embd, np.float32)
    call = rnb.qwen35_sparse_experts_selected_base_by_token
    e = _err(call, g, u, d, [0], [1.0], [0], 1, 14, n_ff, n_embd, z(10, np.float32))
    assert str(e) == "Qwen35 full-layer input length mismatch: got 10, expected 256"
    e = _err(call, g, u, d, [0], [1.0], [0], 1, 14, 100, n_embd, x)
    assert str(e) == "Qwen35 full-layer dims must be divisible by 256, got n_ff=100 n_embd=256"
    e = _err(call, g, u, d, [0], [1.0], [1], 1, 14, n_ff, n_embd, x)
    assert str(e) == "Qwen35 full-layer token id out of range"
    e = _err(call, g, u, d, [0], [1.0], [0], 1, 10, n_ff, n_embd, x)
    assert e.kind == "UnsupportedOp" and "down quant code 10" in str(e)
    e = _err(call, g, u, d, [0], [1.0], [0], 1, 13, n_ff, n_embd, x)  # Q5_K down: 176-byte blocks expected
    assert str(e) == "Qwen35 selected-base down length mismatch: len=107520 expected=90112"
    e = _err(call, g[:-1], u, d, [0], [1.0], [0], 1, 14, n_ff, n_embd, x)
    assert str(e).startswith("Qwen35 selected-base gate length is not expert-aligned")
    e = _err(call, g, u[:per_gate], d, [0], [1.0], [0], 1, 14, n_ff, n_embd, x)
    assert str(e).startswith("Qwen35 selected-base up length mismatch")
    e = _err(call, g, u, d, [2], [1.0], [0], 1, 14, n_ff, n_embd, x)
    assert str(e).startswith("Qwen35 selected-base expert id out of range")
    e = _err(call, g, u, d, [0, 1], [1.0], [0], 1, 14, n_ff, n_embd, x)
    assert "length mismatch" in str(e)
    # the shared expert (slot id n_expert, moe_view/fanout.rs:804-812): all three tensors, one expert's bytes each
    sg, su, sd = z(per_gate, np.uint8), z(per_gate, np.uint8), z(per_down, np.uint8)
    e = _err(call, g, u, d, [3], [1.0], [0], 1, 14, n_ff, n_embd, x, shared=(sg, su, sd))
    assert str(e) == "Qwen35 selected-base expert id out of range: id=3 n_expert=2"
    e = _err(call, g, u, d, [2], [1.0], [0], 1, 14, n_ff, n_embd, x, shared=(sg, su, sd[:-1]))
    assert str(e) == ("Qwen35 shared expert length mismatch: gate=36864 up=36864 down=53759 expected gate=up=36864 "
                      "down=53760")
    e = _err(call, g, u, d, [2], [1.0], [0], 1, 14, n_ff, n_embd, x, shared=(sg, su[:10], sd))
    assert str(e).startswith("Qwen35 shared expert length mismatch")
    lib = rnb.binding.lib()
    ptr = lambda a: a.ctypes.data  # noqa: E731
    ids, rt, tk, out = np.array([2], np.uint32), np.ones(1, np.float32), z(1, np.uint32), z(n_embd, np.float32)
    rc = lib.rnb_hip_moe_sparse_experts_by_token(ptr(g), g.size, ptr(u), u.size, ptr(d), d.size, ptr(sg), sg.size, None, 0,
                                                 ptr(sd), sd.size, ptr(ids), ptr(rt), ptr(tk), 1, 1, 14, n_ff, n_embd,
                                                 ptr(x), x.size, ptr(out), out.size)
    assert rc == 1 and rnb.last_error() == "Qwen35 shared expert needs its gate, up and down tensors together"


def test_quantizer_validation():
    e = _err(rnb.quantize_input_q8k, np.zeros(100, np.float32))
    assert str(e) == "Q8_K input length must be divisible by 256, got 100"
    e = _err(rnb.quantize_input_q8, np.zeros(33, np.float32))
    assert str(e) == "Q8 input length must be divisible by 32, got 33"


def test_no_device_is_distinguishable_and_there_is_no_fallback():
    if rnb.device_available():
        pytest.skip("a device is present; the NoDevice path is exercised on CPU-only hosts")
    e = _err(rnb.q4k_gemv, np.zeros(144, np.uint8), 1, 256, np.zeros(256, np.float32))
    assert e.kind == "NoDevice" and str(e).startswith("no HIP device")
    assert rnb.stream_handle() == 0


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "runnburn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower().replace("test oracle", ""), f"{f} mentions the oracle"


def test_dense_ffn_validation_messages():
    """crates/rnb-backend/cuda/src/runtime/dense.rs:1712-1765"""
    z = np.zeros
    f = rnb.dense_q4k_silu_ffn_batch
    g = z(256 * 144, np.uint8)
    e = _err(f, g, g, z(256 * 210, np.uint8), 14, 256, 256, 1, z(256, np.float32))
    assert (e.kind, str(e)) == ("InvalidRequest", "dense SiLU FFN batch requires seq_len > 1, got 1")
    e = _err(f, g, g, z(256 * 210, np.uint8), 14, 256, 256, 2, z(500, np.float32))
    assert str(e) == "dense SiLU FFN batch input length mismatch: got 500, expected 512"
    e = _err(f, g, g, z(10, np.uint8), 14, 300, 256, 2, z(512, np.float32))
    assert str(e) == "dense SiLU FFN batch dims must align to gate/down blocks, got n_ff=300 down_block=256 n_embd=256"
    e = _err(f, g, g, z(10, np.uint8), 8, 250, 256, 2, z(512, np.float32))
    assert str(e) == "dense SiLU FFN batch dims must align to gate/down blocks, got n_ff=250 down_block=32 n_embd=256"
    e = _err(f, g, g, z(10, np.uint8), 2, 256, 256, 2, z(512, np.float32))
    assert str(e) == "unsupported dense SiLU FFN batch down quant code 2"
    e = _err(f, g[:-1], g, z(256 * 210, np.uint8), 14, 256, 256, 2, z(512, np.float32))
    assert str(e) == "dense SiLU FFN batch gate byte mismatch: got 36863, expected 36864"
    e = _err(f, g, g[:-2], z(256 * 210, np.uint8), 14, 256, 256, 2, z(512, np.float32))
    assert str(e) == "dense SiLU FFN batch up byte mismatch: got 36862, expected 36864"
    e = _err(f, g, g, z(256 * 210 + 1, np.uint8), 14, 256, 256, 2, z(512, np.float32))
    assert str(e) == "dense SiLU FFN batch down byte mismatch: got 53761, expected 53760"
    e = _err(f, g, g, z(256 * 176 - 1, np.uint8), 13, 256, 256, 2, z(512, np.float32))
    assert str(e) == "dense SiLU FFN batch down byte mismatch: got 45055, expected 45056"
    e = _err(f, g, g, z(256 * 8 * 24 + 1, np.uint8), 7, 256, 256, 2, z(512, np.float32))  # Q5_1 down: 24-byte blocks
    assert str(e) == "dense SiLU FFN batch down byte mismatch: got 49153, expected 49152"


def test_embedding_gather_validation_messages_match_reference():
    """crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:1854-1885: the format's Debug name, checks in this order."""
    z = np.zeros
    ids = np.array([0, 5], dtype=np.uint32)
    e = _err(rnb.quant_embedding_gather, rnb.GGML_Q4_K, z(144, np.uint8), 1, 255, ids)
    assert (e.kind, str(e)) == ("InvalidRequest", "Q4K embedding cols must be non-zero and divisible by 256, got 255")
    e = _err(rnb.quant_embedding_gather, rnb.GGML_Q8_0, z(34, np.uint8), 1, 0, ids)
    assert str(e) == "Q80 embedding cols must be non-zero and divisible by 32, got 0"
    # an empty id list returns before the other checks
    assert rnb.quant_embedding_gather(rnb.GGML_Q6_K, z(1, np.uint8), 4, 256, np.zeros(0, np.uint32)).size == 0
    e = _err(rnb.quant_embedding_gather, rnb.GGML_IQ2_XXS, z(66 * 5, np.uint8), 5, 256, ids)
    assert str(e) == "IQ2XXS embedding token id 5 is out of range for 5 rows"
    e = _err(rnb.quant_embedding_gather, rnb.GGML_Q6_K, z(210 * 6 - 1, np.uint8), 6, 256, ids)
    assert str(e) == "Q6K embedding weight byte mismatch: got 1259, expected 1260"
    e = _err(rnb.quant_embedding_gather, rnb.GGML_BF16, z(64 * 6 * 2 + 2, np.uint8), 6, 64, ids)
    assert str(e) == "BF16 embedding weight byte mismatch: got 770, expected 768"
    e = _err(rnb.quant_embedding_gather, 17, z(74 * 6, np.uint8), 6, 256, ids)
    assert e.kind == "UnsupportedOp"


def test_q8_0_head_batch_validation_messages_match_reference():
    """crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:832-866: dimensions, cols, weight bytes, input length, in
    this order."""
    z = np.zeros
    e = _err(rnb.q8_0_head_gemv_batch, z(34, np.uint8), 0, 4, 32, 2, z(64, np.float32))
    assert (e.kind, str(e)) == ("InvalidRequest", "Q8_0 head batch dimensions must be non-zero: heads=0 rows_per_head=4 tokens=2")
    e = _err(rnb.q8_0_head_gemv_batch, z(34, np.uint8), 3, 4, 32, 0, z(0, np.float32))
    assert str(e) == "Q8_0 head batch dimensions must be non-zero: heads=3 rows_per_head=4 tokens=0"
    e = _err(rnb.q8_0_head_gemv_batch, z(34, np.uint8), 3, 4, 48, 2, z(288, np.float32))
    assert str(e) == "Q8_0 head batch cols must be non-zero and divisible by 32, got 48"
    e = _err(rnb.q8_0_head_gemv_batch, z(34, np.uint8), 3, 4, 0, 2, z(0, np.float32))
    assert str(e) == "Q8_0 head batch cols must be non-zero and divisible by 32, got 0"
    e = _err(rnb.q8_0_head_gemv_batch, z(3 * 4 * 3 * 34 - 1, np.uint8), 3, 4, 96, 3, z(3 * 3 * 96, np.float32))
    assert str(e) == "Q8_0 head batch weight byte mismatch: got 1223, expected 1224"
    e = _err(rnb.q8_0_head_gemv_batch, z(3 * 4 * 3 * 34, np.uint8), 3, 4, 96, 3, z(3 * 3 * 96 - 1, np.float32))
    assert str(e) == "Q8_0 head batch input length mismatch: got 863, expected 864"

