"""ctypes binding of the CPU oracle (oracle/librnb_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg.  The shipped package (runnburn_amd) never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librnb_oracle.so")

Q4_0, Q4_1, Q5_0, Q5_1, Q8_1 = 2, 3, 6, 7, 9
LEGACY = (Q4_0, Q4_1, Q5_0, Q5_1, Q8_1)  # 32-element blocks other than Q8_0, dotted against 32-wide Q8 activations
Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K = 8, 10, 11, 12, 13, 14  # ggml type ids (crates/rnb-loader/src/gguf/types.rs:5-41)
IQ2_XXS, IQ3_XXS, IQ2_S, IQ4_XS = 16, 18, 22, 23  # importance quants (crates/rnb-cpu/src/quantize/iq.rs), against Q8_K activations
IQ = (IQ2_XXS, IQ3_XXS, IQ2_S, IQ4_XS)
BLOCK_BYTES = {Q4_0: 18, Q4_1: 20, Q5_0: 22, Q5_1: 24, Q8_0: 34, Q8_1: 36, Q2_K: 84, Q3_K: 110, Q4_K: 144, Q5_K: 176, Q6_K: 210,
               IQ2_XXS: 66, IQ3_XXS: 98, IQ2_S: 82, IQ4_XS: 136}
BLOCK_ELEMS = {Q4_0: 32, Q4_1: 32, Q5_0: 32, Q5_1: 32, Q8_0: 32, Q8_1: 32, Q2_K: 256, Q3_K: 256, Q4_K: 256, Q5_K: 256, Q6_K: 256,
               IQ2_XXS: 256, IQ3_XXS: 256, IQ2_S: 256, IQ4_XS: 256}

Q8K_DTYPE = np.dtype([("d", "<f4"), ("qs", "i1", (256,)), ("bsums", "<i2", (16,))])
Q8_DTYPE = np.dtype([("d", "<f4"), ("qs", "i1", (32,))])
assert Q8K_DTYPE.itemsize == 292 and Q8_DTYPE.itemsize == 36


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (make).  Returns the library path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-s"] + (["-B"] if force else []), check=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, sz, u32, u64, i32, f32 = C.c_void_p, C.c_size_t, C.c_uint32, C.c_uint64, C.c_int, C.c_float
        L.rnbo_f16_to_f32.restype = f32
        L.rnbo_f16_to_f32.argtypes = [C.c_uint16]
        L.rnbo_f32_to_f16.restype = C.c_uint16
        L.rnbo_f32_to_f16.argtypes = [f32]
        L.rnbo_nearest_int.restype = i32
        L.rnbo_nearest_int.argtypes = [f32]
        L.rnbo_get_scale_min_k4.restype = None
        L.rnbo_get_scale_min_k4.argtypes = [i32, vp, vp, vp]
        for name in ("rnbo_dequantize_q8_0", "rnbo_dequantize_q2_k", "rnbo_dequantize_q3_k", "rnbo_dequantize_q4_k",
                     "rnbo_dequantize_q5_k", "rnbo_dequantize_q6_k", "rnbo_dequantize_iq2_xxs", "rnbo_dequantize_iq2_s",
                     "rnbo_dequantize_iq3_xxs", "rnbo_dequantize_iq4_xs"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, sz, vp]
        for name in ("rnbo_quantize_q8k", "rnbo_quantize_q8"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, sz, vp]
        for name in ("rnbo_dot_q2k_q8k", "rnbo_dot_q3k_q8k", "rnbo_dot_q4k_q8k", "rnbo_dot_q5k_q8k", "rnbo_dot_q6k_q8k", "rnbo_dot_q8_0_q8", "rnbo_dot_q8_0_f32",
                     "rnbo_dot_q4k_q8k_avx2", "rnbo_dot_q6k_q8k_avx2"):
            getattr(L, name).restype = f32
            getattr(L, name).argtypes = [vp, vp, sz]
        for name in ("rnbo_dot_q2k_q8k_f64", "rnbo_dot_q3k_q8k_f64", "rnbo_dot_q4k_q8k_f64", "rnbo_dot_q5k_q8k_f64",
                     "rnbo_dot_q6k_q8k_f64", "rnbo_dot_q8_0_q8_f64"):
            getattr(L, name).restype = C.c_double
            getattr(L, name).argtypes = [vp, vp, sz]
        for name in ("rnbo_gemv", "rnbo_gemv_f64", "rnbo_gemv_avx2"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [u32, vp, sz, sz, vp, sz, vp, i32]
        L.rnbo_gemv_q8_0_f32act.restype = i32
        L.rnbo_gemv_q8_0_f32act.argtypes = [vp, sz, sz, vp, sz, vp, i32]
        for name in ("rnbo_silu_mul_inplace", "rnbo_gelu_mul_inplace"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, sz]
        L.rnbo_route_topk.restype = sz
        L.rnbo_route_topk.argtypes = [vp, sz, sz, vp, vp]
        for name in ("rnbo_moe_sparse_experts_by_token", "rnbo_moe_sparse_experts_by_token_avx2"):
            getattr(L, name).restype = i32
            getattr(L, name).argtypes = [vp, vp, vp, sz, vp, vp, vp, sz, sz, u32, sz, sz, vp, vp, i32]
        for name in ("rnbo_quantize_row_q2_k", "rnbo_quantize_row_q3_k", "rnbo_quantize_row_q4_k", "rnbo_quantize_row_q5_k",
                     "rnbo_quantize_row_q6_k", "rnbo_quantize_row_q8_0"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, sz, vp]
        L.rnbo_dequantize_legacy.restype = i32
        L.rnbo_dequantize_legacy.argtypes = [u32, vp, sz, vp]
        L.rnbo_dot_legacy_q8.restype = f32
        L.rnbo_dot_legacy_q8.argtypes = [u32, vp, vp, sz]
        L.rnbo_dot_legacy_q8_f64.restype = C.c_double
        L.rnbo_dot_legacy_q8_f64.argtypes = [u32, vp, vp, sz]
        L.rnbo_quantize_row_legacy.restype = i32
        L.rnbo_quantize_row_legacy.argtypes = [u32, vp, sz, vp]
        L.rnbo_fill_normal.restype = None
        L.rnbo_fill_normal.argtypes = [vp, sz, u64, f32]
        L.rnbo_make_weights.restype = i32
        L.rnbo_make_weights.argtypes = [u32, sz, sz, u64, f32, vp, i32]
        L.rnbo_have_avx2.restype = i32
        L.rnbo_have_avx2.argtypes = []
        L.rnbo_dot_iq_q8k.restype = f32
        L.rnbo_dot_iq_q8k.argtypes = [u32, vp, vp, sz]
        L.rnbo_dot_iq_q8k_f64.restype = C.c_double
        L.rnbo_dot_iq_q8k_f64.argtypes = [u32, vp, vp, sz]
        L.rnbo_iq_grid.restype = sz
        L.rnbo_iq_grid.argtypes = [i32, vp]
        _lib = L
    return _lib


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    if isinstance(a, (bytes, bytearray, memoryview)):
        a = np.frombuffer(a, dtype=np.uint8)
    return np.ascontiguousarray(a, dtype=np.uint8)


# ---- scalar helpers -----------------------------------------------------------------

def f16_to_f32(bits: int) -> float:
    return float(lib().rnbo_f16_to_f32(bits))


def f32_to_f16(value: float) -> int:
    return int(lib().rnbo_f32_to_f16(C.c_float(value)))


def nearest_int(value: float) -> int:
    return int(lib().rnbo_nearest_int(C.c_float(value)))


def get_scale_min_k4(j: int, q12) -> tuple[int, int]:
    q = _u8(q12)
    assert q.size == 12
    sc, mn = C.c_uint8(), C.c_uint8()
    lib().rnbo_get_scale_min_k4(j, _p(q), C.byref(sc), C.byref(mn))
    return sc.value, mn.value


# ---- dequantisers -------------------------------------------------------------------

def dequantize(quant: int, blocks) -> np.ndarray:
    b = _u8(blocks)
    n = b.size // BLOCK_BYTES[quant]
    assert n * BLOCK_BYTES[quant] == b.size
    out = np.empty(n * BLOCK_ELEMS[quant], dtype=np.float32)
    if quant in LEGACY:
        assert lib().rnbo_dequantize_legacy(quant, _p(b), n, _p(out)) == 0
        return out
    fn = {Q8_0: "rnbo_dequantize_q8_0", Q2_K: "rnbo_dequantize_q2_k", Q3_K: "rnbo_dequantize_q3_k",
          Q4_K: "rnbo_dequantize_q4_k", Q5_K: "rnbo_dequantize_q5_k", Q6_K: "rnbo_dequantize_q6_k",
          IQ2_XXS: "rnbo_dequantize_iq2_xxs", IQ2_S: "rnbo_dequantize_iq2_s", IQ3_XXS: "rnbo_dequantize_iq3_xxs",
          IQ4_XS: "rnbo_dequantize_iq4_xs"}[quant]
    getattr(lib(), fn)(_p(b), n, _p(out))
    return out


def iq_grid(which: int) -> np.ndarray:
    """The expanded codebook: 0 IQ2_XXS (256 entries of 8 bytes), 1 IQ2_S (1024 of 8), 2 IQ3_XXS (256 of 4, widened)."""
    out = np.zeros(1024, dtype=np.uint64)
    n = lib().rnbo_iq_grid(which, _p(out))
    return out[:n]


# ---- activation quantisers ----------------------------------------------------------

def quantize_q8k(x) -> np.ndarray:
    x = _f32(x).ravel()
    assert x.size % 256 == 0
    out = np.zeros(x.size // 256, dtype=Q8K_DTYPE)
    lib().rnbo_quantize_q8k(_p(x), x.size, _p(out))
    return out


def quantize_q8(x) -> np.ndarray:
    x = _f32(x).ravel()
    assert x.size % 32 == 0
    out = np.zeros(x.size // 32, dtype=Q8_DTYPE)
    lib().rnbo_quantize_q8(_p(x), x.size, _p(out))
    return out


# ---- row dots -----------------------------------------------------------------------

def dot(quant: int, row, act: np.ndarray, gold: bool = False, avx2: bool = False) -> float:
    r = _u8(row)
    nb = r.size // BLOCK_BYTES[quant]
    assert act.size == nb
    if quant in LEGACY:
        assert not avx2
        act = np.ascontiguousarray(act)
        fn = lib().rnbo_dot_legacy_q8_f64 if gold else lib().rnbo_dot_legacy_q8
        return float(fn(quant, _p(r), _p(act), nb))
    if quant in IQ:
        assert not avx2
        act = np.ascontiguousarray(act)
        fn = lib().rnbo_dot_iq_q8k_f64 if gold else lib().rnbo_dot_iq_q8k
        return float(fn(quant, _p(r), _p(act), nb))
    base = {Q8_0: "rnbo_dot_q8_0_q8", Q2_K: "rnbo_dot_q2k_q8k", Q3_K: "rnbo_dot_q3k_q8k", Q4_K: "rnbo_dot_q4k_q8k",
            Q5_K: "rnbo_dot_q5k_q8k", Q6_K: "rnbo_dot_q6k_q8k"}[quant]
    if gold:
        base += "_f64"
    elif avx2:
        base += "_avx2"
    act = np.ascontiguousarray(act)
    return float(getattr(lib(), base)(_p(r), _p(act), nb))


def dot_q8_0_f32(row, x) -> float:
    r, x = _u8(row), _f32(x)
    return float(lib().rnbo_dot_q8_0_f32(_p(r), _p(x), r.size // 34))


# ---- drivers ------------------------------------------------------------------------

def gemv(quant: int, w, rows: int, cols: int, x, gold: bool = False, avx2: bool = False,
         n_threads: int = 0) -> np.ndarray:
    """out[seq][rows]; x is [seq][cols] (or [cols])."""
    w, x = _u8(w), _f32(x)
    seq = x.size // cols
    assert x.size == seq * cols
    assert w.size == rows * (cols // BLOCK_ELEMS[quant]) * BLOCK_BYTES[quant]
    out = np.empty((seq, rows), dtype=np.float64 if gold else np.float32)
    fn = "rnbo_gemv_f64" if gold else ("rnbo_gemv_avx2" if avx2 else "rnbo_gemv")
    rc = getattr(lib(), fn)(quant, _p(w), rows, cols, _p(x), seq, _p(out), n_threads)
    if rc != 0:
        raise RuntimeError(f"{fn} failed with code {rc}")
    return out


def gemv_q8_0_f32act(w, rows: int, cols: int, x, n_threads: int = 0) -> np.ndarray:
    w, x = _u8(w), _f32(x)
    seq = x.size // cols
    out = np.empty((seq, rows), dtype=np.float32)
    rc = lib().rnbo_gemv_q8_0_f32act(_p(w), rows, cols, _p(x), seq, _p(out), n_threads)
    if rc != 0:
        raise RuntimeError(f"rnbo_gemv_q8_0_f32act failed with code {rc}")
    return out


# ---- MoE ----------------------------------------------------------------------------

def silu_mul(gate, up) -> np.ndarray:
    g, u = _f32(gate).copy(), _f32(up)
    lib().rnbo_silu_mul_inplace(_p(g), _p(u), g.size)
    return g


def gelu_mul(gate, up) -> np.ndarray:
    g, u = _f32(gate).copy(), _f32(up)
    lib().rnbo_gelu_mul_inplace(_p(g), _p(u), g.size)
    return g


def dense_gelu_ffn(gate, up, down, down_quant: int, n_ff: int, n_embd: int, x) -> np.ndarray:
    """As dense_silu_ffn with crates/rnb-cpu/src/kernels/activation.rs:91-98 (fused_gelu_mul) between the halves."""
    g = gemv(Q4_K, gate, n_ff, n_embd, x)
    u = gemv(Q4_K, up, n_ff, n_embd, x)
    mid = gelu_mul(g.ravel(), u.ravel()).reshape(g.shape)
    return gemv(down_quant, down, n_embd, n_ff, mid)


def dense_silu_ffn(gate, up, down, down_quant: int, n_ff: int, n_embd: int, x) -> np.ndarray:
    """Dense SwiGLU FFN per token, composed of pinned pieces exactly as the reference's CPU path composes them
    (gate/up GEMV on Q8_K(x), crates/rnb-cpu/src/kernels/activation.rs:73-89 fused_silu_mul, down GEMV on the
    re-quantised intermediate): out[seq][n_embd]."""
    g = gemv(Q4_K, gate, n_ff, n_embd, x)
    u = gemv(Q4_K, up, n_ff, n_embd, x)
    mid = silu_mul(g.ravel(), u.ravel()).reshape(g.shape)
    return gemv(down_quant, down, n_embd, n_ff, mid)


def rms_norm(x, weight, eps: float, unit_offset: bool = False) -> np.ndarray:
    """crates/rnb-cpu/src/kernels/norm.rs:180-196 (rms_norm_into_f64, the default of rms_norm_into: mean square summed in
    f64 in element order, rms = f32(sqrt(mean + eps)), out = (x / rms) * weight) and :211-224
    (rms_norm_unit_offset_into_scalar: f32 sum in element order, out = (x / rms) * (1 + weight)).  x is [rows][hidden]."""
    w = _f32(weight)
    rows = _f32(x).reshape(-1, w.size)
    out = np.empty_like(rows)
    e32 = np.float32(eps)
    for r in range(rows.shape[0]):
        row = rows[r]
        if unit_offset:
            total = np.cumsum(row * row, dtype=np.float32)[-1]  # cumsum accumulates strictly in order
            rms = np.sqrt(np.float32(total / np.float32(w.size)) + e32, dtype=np.float32)
            out[r] = (row / rms) * (np.float32(1.0) + w)
        else:
            r64 = row.astype(np.float64)
            total = np.cumsum(r64 * r64)[-1]
            rms = np.float32(np.sqrt(total / float(w.size) + float(e32)))
            out[r] = (row / rms) * w
    return out


def route_topk(logits, k: int) -> tuple[np.ndarray, np.ndarray]:
    lg = _f32(logits)
    idx = np.zeros(min(k, lg.size), dtype=np.uint32)
    w = np.zeros(min(k, lg.size), dtype=np.float32)
    n = lib().rnbo_route_topk(_p(lg), lg.size, k, _p(idx), _p(w))
    return idx[:n], w[:n]


def moe_sparse_experts_by_token(gate_all, up_all, down_all, n_expert: int, expert_ids, route, token_ids,
                                token_count: int, down_quant: int, n_ff: int, n_embd: int, x,
                                n_threads: int = 0, avx2: bool = False) -> np.ndarray:
    """`avx2`: the block dots of rnb-cpu's x86_64 path (same integer sums, another f32 order inside a row): the form
    that is timed as the CPU baseline; the checks use the scalar form."""
    g, u, d = _u8(gate_all), _u8(up_all), _u8(down_all)
    e = np.ascontiguousarray(expert_ids, dtype=np.uint32)
    r = _f32(route)
    t = np.ascontiguousarray(token_ids, dtype=np.uint32)
    x = _f32(x)
    assert x.size == token_count * n_embd
    out = np.empty((token_count, n_embd), dtype=np.float32)
    fn = lib().rnbo_moe_sparse_experts_by_token_avx2 if avx2 else lib().rnbo_moe_sparse_experts_by_token
    rc = fn(_p(g), _p(u), _p(d), n_expert, _p(e), _p(r), _p(t), e.size, token_count, down_quant, n_ff, n_embd, _p(x),
            _p(out), n_threads)
    if rc != 0:
        raise RuntimeError(f"rnbo_moe_sparse_experts_by_token{'_avx2' if avx2 else ''} failed with code {rc}")
    return out


# ---- input generation ---------------------------------------------------------------

def quantize_row(quant: int, x) -> np.ndarray:
    x = _f32(x).ravel()
    assert x.size % BLOCK_ELEMS[quant] == 0
    out = np.zeros(x.size // BLOCK_ELEMS[quant] * BLOCK_BYTES[quant], dtype=np.uint8)
    if quant in LEGACY:
        assert lib().rnbo_quantize_row_legacy(quant, _p(x), x.size, _p(out)) == 0
        return out
    fn = {Q8_0: "rnbo_quantize_row_q8_0", Q2_K: "rnbo_quantize_row_q2_k", Q3_K: "rnbo_quantize_row_q3_k",
          Q4_K: "rnbo_quantize_row_q4_k", Q5_K: "rnbo_quantize_row_q5_k", Q6_K: "rnbo_quantize_row_q6_k"}[quant]
    getattr(lib(), fn)(_p(x), x.size, _p(out))
    return out


def fill_normal(n: int, seed: int, sigma: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    lib().rnbo_fill_normal(_p(out), n, seed, sigma)
    return out


def make_weights(quant: int, rows: int, cols: int, seed: int, sigma: float = 0.02,
                 n_threads: int = 0) -> np.ndarray:
    out = np.empty(rows * (cols // BLOCK_ELEMS[quant]) * BLOCK_BYTES[quant], dtype=np.uint8)
    rc = lib().rnbo_make_weights(quant, rows, cols, seed, sigma, _p(out), n_threads)
    if rc != 0:
        raise RuntimeError(f"rnbo_make_weights failed with code {rc}")
    return out


def have_avx2() -> bool:
    return bool(lib().rnbo_have_avx2())


def tensor_seed(config: str, tensor: str, base: int = 20240607) -> int:
    """Seed per tensor = hash(config id, tensor name) mixed with the base seed (FNV-1a 64)."""
    h = 0xcbf29ce484222325
    for ch in f"{base}:{config}:{tensor}".encode():
        h = ((h ^ ch) * 0x100000001b3) & 0xFFFFFFFFFFFFFFFF
    return h
