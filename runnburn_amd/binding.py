"""ctypes binding of librnb_hip.so and the host-side mirror of the reference's operator functions."""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional, Sequence

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_PKG, "librnb_hip.so")

GGML_Q4_0, GGML_Q4_1, GGML_Q5_0, GGML_Q5_1, GGML_Q8_1 = 2, 3, 6, 7, 9
GGML_Q8_0, GGML_Q2_K, GGML_Q3_K, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 8, 10, 11, 12, 13, 14
GGML_IQ2_XXS, GGML_IQ3_XXS, GGML_IQ2_S, GGML_IQ4_XS = 16, 18, 22, 23
GGML_F32, GGML_F16, GGML_BF16 = 0, 1, 30  # embedding tables only
OP_MATMUL, OP_ATTENTION, OP_GDN, OP_MOE, OP_SAMPLER = 0, 1, 2, 3, 4
STATUS_NAMES = {0: "Ok", 1: "InvalidRequest", 2: "UnsupportedOp", 3: "ExecutionFailed", 4: "NoDevice"}

# every symbol include/rnb_hip.h declares: (name, restype, argtypes)
_vp, _sz, _u32, _u64p, _i = C.c_void_p, C.c_size_t, C.c_uint32, C.POINTER(C.c_uint64), C.c_int
_MATMUL_ARGS = [_vp, _sz, _sz, _sz, _vp, _sz, _vp, _sz]
SYMBOLS = [
    ("rnb_hip_backend_kind", _i, []),
    ("rnb_hip_backend_supports", _i, [_i]),
    ("rnb_hip_backend_supports_quant", _i, [_i, _u32]),
    ("rnb_hip_init", _i, []),
    ("rnb_hip_last_error", C.c_char_p, []),
    ("rnb_hip_device_name", _i, [C.c_char_p, _sz]),
    ("rnb_hip_sync", _i, []),
    ("rnb_hip_transfer_counters", _i, [_u64p, _u64p]),
    ("rnb_hip_stream", _vp, []),
    ("rnb_hip_prewarm", _i, [C.POINTER(_vp), C.POINTER(_sz), _sz]),
    ("rnb_hip_release", _i, [_vp, _sz]),
    ("rnb_hip_resident_bytes", _i, [_u64p, _u64p]),
    ("rnb_hip_calib_read", _i, [_vp, _sz, _i]),
    ("rnb_hip_calib_mfma_i8", _i, [_u32, _u32, _u64p]),
    ("rnb_hip_residency_stats", _i, [_u64p, _sz]),
    ("rnb_hip_set_resident_budget", _i, [C.c_uint64]),
    ("rnb_hip_offload_unpinned", _i, [_u64p]),
    ("rnb_hip_quantize_q8k", _i, [_vp, _sz, _vp, _sz]),
    ("rnb_hip_quantize_q8", _i, [_vp, _sz, _vp, _sz]),
    ("rnb_hip_q4k_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q4k_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q4_0_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q4_0_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q4_1_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q4_1_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q5_0_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q5_0_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q5_1_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q5_1_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q8_1_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q8_1_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q2k_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q2k_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q3k_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q3k_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q4k_gemv_with_device_input", _i, [_vp, _sz, _sz, _sz, _vp, _vp, _sz]),
    ("rnb_hip_q6k_gemv_with_device_input", _i, [_vp, _sz, _sz, _sz, _vp, _vp, _sz]),
    ("rnb_hip_quant_embedding_gather", _i, [_u32, _vp, _sz, _sz, _sz, _vp, _sz, _vp, _sz]),
    ("rnb_hip_quant_embedding_gather_dev", _i, [_u32, _vp, _sz, _sz, _sz, _vp, _sz, _vp]),
    ("rnb_hip_iq2_xxs_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_iq2_xxs_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_iq2_s_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_iq2_s_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_iq3_xxs_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_iq3_xxs_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_iq4_xs_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_iq4_xs_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q5k_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q5k_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q6k_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q6k_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q8_0_gemv", _i, _MATMUL_ARGS),
    ("rnb_hip_q8_0_gemv_batch", _i, _MATMUL_ARGS),
    ("rnb_hip_q8_0_head_gemv_batch", _i, [_vp, _sz, _sz, _sz, _sz, _sz, _vp, _sz, _vp, _sz]),
    ("rnb_hip_moe_sparse_experts_by_token", _i,
     [_vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _vp, _vp, _sz, _sz, _u32, _sz, _sz, _vp, _sz, _vp, _sz]),
    ("rnb_hip_dev_alloc", _vp, [_sz]),
    ("rnb_hip_dev_free", _i, [_vp]),
    ("rnb_hip_dev_upload", _i, [_vp, _vp, _sz]),
    ("rnb_hip_dev_download", _i, [_vp, _vp, _sz]),
    ("rnb_hip_gemv_dev", _i, [_u32, _vp, _sz, _sz, _vp, _sz, _vp]),
    ("rnb_hip_gemv_dev_noalloc", _i, [_u32, _vp, _sz, _sz, _vp, _sz, _vp]),
    ("rnb_hip_gemv_dev_noalloc_scratch_bytes", _sz, []),
    ("rnb_hip_quantize_dev", _i, [_u32, _vp, _sz, _sz]),
    ("rnb_hip_rms_norm_dev", _i, [_vp, _vp, C.c_float, _i, _sz, _sz, _vp]),
    ("rnb_hip_rms_norm_quantize_dev", _i, [_vp, _vp, C.c_float, _i, _sz, _sz, _vp]),
    ("rnb_hip_rms_norm_add_rms_norm_quantize_dev", _i, [_vp, _vp, C.c_float, _i, _vp, _vp, C.c_float, _i, _sz, _sz, _vp]),
    ("rnb_hip_moe_route_topk_dev", _i, [_vp, _sz, _sz, _sz, _vp, _vp]),
    ("rnb_hip_gemv_quantized_dev", _i, [_u32, _vp, _sz, _sz, _sz, _vp]),
    ("rnb_hip_moe_sparse_experts_by_token_dev", _i,
     [_vp, _vp, _vp, _sz, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _u32, _sz, _sz, _vp, _vp]),
    ("rnb_hip_q6k_gemv_argmax", _i, [_vp, _sz, _sz, _sz, _vp, _sz, C.POINTER(_u32), C.POINTER(C.c_float)]),
    ("rnb_hip_dense_q4k_attention_qkv", _i, [_vp, _sz, _vp, _sz, _vp, _sz, _sz, _sz, _sz, _vp, _sz, _vp, _sz, _vp, _sz, _vp, _sz]),
    ("rnb_hip_q8_0_gemv_argmax", _i, [_vp, _sz, _sz, _sz, _vp, _sz, C.POINTER(_u32), C.POINTER(C.c_float)]),
    ("rnb_hip_q8_0_gemv_argmax_q8dot", _i, [_vp, _sz, _sz, _sz, _vp, _sz, C.POINTER(_u32), C.POINTER(C.c_float)]),
    ("rnb_hip_dense_q4k_silu_ffn_batch", _i, [_vp, _sz, _vp, _sz, _vp, _sz, _u32, _sz, _sz, _sz, _vp, _sz, _vp, _sz]),
    ("rnb_hip_dense_q4k_gelu_ffn_batch", _i, [_vp, _sz, _vp, _sz, _vp, _sz, _u32, _sz, _sz, _sz, _vp, _sz, _vp, _sz]),
    ("rnb_hip_dense_q4k_gelu_ffn", _i, [_vp, _sz, _vp, _sz, _vp, _sz, _u32, _sz, _sz, _vp, _sz, _vp, _sz]),
    ("rnb_hip_dense_q4k_silu_ffn_dev", _i, [_vp, _vp, _vp, _u32, _sz, _sz, _sz, _vp, _vp]),
    ("rnb_hip_gguf_open", _i, [C.c_char_p, C.POINTER(_vp)]),
    ("rnb_hip_gguf_parse", _i, [_vp, _sz, C.POINTER(_vp)]),
    ("rnb_hip_gguf_map_tensors", _i, [_vp]),
    ("rnb_hip_gguf_close", None, [_vp]),
    ("rnb_hip_gguf_version", _u32, [_vp]),
    ("rnb_hip_gguf_alignment", C.c_uint64, [_vp]),
    ("rnb_hip_gguf_data_start", C.c_uint64, [_vp]),
    ("rnb_hip_gguf_tensor_count", _sz, [_vp]),
    ("rnb_hip_gguf_tensor_at", _i, [_vp, _sz, _vp]),
    ("rnb_hip_gguf_find_tensor", _i, [_vp, C.c_char_p, _vp]),
    ("rnb_hip_gguf_tensor_size", _i, [_u64p, _u32, _u32, _u64p]),
    ("rnb_hip_gguf_metadata_count", _sz, [_vp]),
    ("rnb_hip_gguf_metadata_key", C.c_char_p, [_vp, _sz]),
    ("rnb_hip_gguf_metadata_type", _i, [_vp, C.c_char_p]),
    ("rnb_hip_gguf_metadata_u64", _i, [_vp, C.c_char_p, _u64p]),
    ("rnb_hip_gguf_metadata_i64", _i, [_vp, C.c_char_p, C.POINTER(C.c_int64)]),
    ("rnb_hip_gguf_metadata_f64", _i, [_vp, C.c_char_p, C.POINTER(C.c_double)]),
    ("rnb_hip_gguf_metadata_str", C.c_char_p, [_vp, C.c_char_p]),
    ("rnb_hip_gguf_metadata_array", _i, [_vp, C.c_char_p, C.POINTER(_u32), _u64p]),
    ("rnb_hip_gguf_metadata_array_str", C.c_char_p, [_vp, C.c_char_p, C.c_uint64]),
    ("rnb_hip_gguf_metadata_array_f64", _i, [_vp, C.c_char_p, C.c_uint64, C.POINTER(C.c_double)]),
    ("rnb_hip_gguf_prewarm_tensor", _i, [_vp, _sz]),
]

Q8K_DTYPE = np.dtype([("d", "<f4"), ("qs", "i1", (256,)), ("bsums", "<i2", (16,))])
Q8_DTYPE = np.dtype([("d", "<f4"), ("qs", "i1", (32,))])


class BackendError(RuntimeError):
    """BackendError of crates/rnb-backend/api/src/lib.rs:55-108: kind + message."""

    def __init__(self, status: int, message: str):
        super().__init__(message)
        self.status = status
        self.kind = STATUS_NAMES.get(status, str(status))
        self.message = message


_lib: Optional[C.CDLL] = None


def lib_path() -> str:
    return _LIB_PATH


def lib() -> C.CDLL:
    """Loads the HIP extension.  Raises when it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(f"{_LIB_PATH} is missing: build it with `python -m runnburn_amd.build` "
                              "(hipcc --offload-arch=gfx950); runnburn_amd has no CPU fallback")
        L = C.CDLL(_LIB_PATH)
        for name, restype, argtypes in SYMBOLS:
            fn = getattr(L, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = L
    return _lib


def last_error() -> str:
    msg = lib().rnb_hip_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def _check(status: int) -> None:
    if status != 0:
        raise BackendError(status, last_error())


def device_available() -> bool:
    return lib().rnb_hip_init() == 0


def device_name() -> str:
    buf = C.create_string_buffer(256)
    _check(lib().rnb_hip_device_name(buf, 256))
    return buf.value.decode()


def sync() -> None:
    _check(lib().rnb_hip_sync())


def stream_handle() -> int:
    return int(lib().rnb_hip_stream() or 0)


def transfer_counters() -> tuple[int, int]:
    a, b = C.c_uint64(), C.c_uint64()
    _check(lib().rnb_hip_transfer_counters(C.byref(a), C.byref(b)))
    return a.value, b.value


def resident_bytes() -> tuple[int, int]:
    a, b = C.c_uint64(), C.c_uint64()
    _check(lib().rnb_hip_resident_bytes(C.byref(a), C.byref(b)))
    return a.value, b.value


RESIDENCY_STAT_NAMES = ("lookups", "hits", "sub_range_hits", "misses", "admissions", "evictions", "admitted_bytes",
                        "evicted_bytes", "h2d_bytes", "temp_h2d_bytes", "oom_retries", "budget_bytes")


def residency_stats() -> dict:
    """Counters of the resident-weight table (the fields of ExpertBundleCacheStats that apply) and its budget."""
    out = (C.c_uint64 * 12)()
    _check(lib().rnb_hip_residency_stats(out, 12))
    return dict(zip(RESIDENCY_STAT_NAMES, (int(v) for v in out)))


def set_resident_budget(nbytes: int) -> None:
    _check(lib().rnb_hip_set_resident_budget(int(nbytes)))


def offload_unpinned() -> int:
    freed = C.c_uint64()
    _check(lib().rnb_hip_offload_unpinned(C.byref(freed)))
    return int(freed.value)


def _bytes_view(w) -> np.ndarray:
    if isinstance(w, np.ndarray):
        if w.dtype != np.uint8 or not w.flags.c_contiguous:
            raise TypeError("weights must be a C-contiguous uint8 array (raw GGUF block bytes)")
        return w
    return np.frombuffer(w, dtype=np.uint8)


def _f32(x) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.float32)


def _ptr(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def prewarm(weights: Sequence) -> None:
    """prewarm_q4k_weights(&[&[u8]]), quant_api.rs:952"""
    views = [_bytes_view(w) for w in weights]
    n = len(views)
    ptrs = (_vp * n)(*[v.ctypes.data for v in views])
    lens = (_sz * n)(*[v.size for v in views])
    _check(lib().rnb_hip_prewarm(ptrs, lens, n))


def release(weights) -> None:
    v = _bytes_view(weights)
    _check(lib().rnb_hip_release(_ptr(v), v.size))


# ---- activation quantisers ---------------------------------------------------------------

def quantize_input_q8k(x) -> np.ndarray:
    """quantize_input_q8k, crates/rnb-cpu/src/gemm/activation_q8.rs:109-119, computed on the device."""
    x = _f32(x).ravel()
    out = np.zeros(x.size // 256 if x.size % 256 == 0 else 0, dtype=Q8K_DTYPE)
    _check(lib().rnb_hip_quantize_q8k(_ptr(x), x.size, _ptr(out), out.nbytes))
    return out


def quantize_input_q8(x) -> np.ndarray:
    """quantize_input_q8, crates/rnb-cpu/src/gemm/activation_q8.rs:14-32, computed on the device."""
    x = _f32(x).ravel()
    out = np.zeros(x.size // 32 if x.size % 32 == 0 else 0, dtype=Q8_DTYPE)
    _check(lib().rnb_hip_quantize_q8(_ptr(x), x.size, _ptr(out), out.nbytes))
    return out


# ---- operator surface ---------------------------------------------------------------------

def _gemv(fn_name: str, weights, rows: int, cols: int, x) -> np.ndarray:
    w, x = _bytes_view(weights), _f32(x).ravel()
    out = np.empty(rows, dtype=np.float32)
    _check(getattr(lib(), fn_name)(_ptr(w), w.size, rows, cols, _ptr(x), x.size, _ptr(out), out.size))
    return out


def _gemv_into(fn_name: str, weights, rows: int, cols: int, x, output: np.ndarray) -> None:
    w, x = _bytes_view(weights), _f32(x).ravel()
    if output.dtype != np.float32 or not output.flags.c_contiguous:
        raise TypeError("output must be a C-contiguous float32 array")
    _check(getattr(lib(), fn_name)(_ptr(w), w.size, rows, cols, _ptr(x), x.size, _ptr(output), output.size))


def _gemv_batch(fn_name: str, weights, rows: int, cols: int, x) -> np.ndarray:
    w, x = _bytes_view(weights), _f32(x).ravel()
    seq = x.size // cols if cols and x.size % cols == 0 else 0
    out = np.empty((seq, rows), dtype=np.float32)
    _check(getattr(lib(), fn_name)(_ptr(w), w.size, rows, cols, _ptr(x), x.size, _ptr(out), out.size))
    return out


def q4k_gemv(weights, rows, cols, input):  # noqa: A002 - the reference's argument name
    return _gemv("rnb_hip_q4k_gemv", weights, rows, cols, input)


def q4k_gemv_into(weights, rows, cols, input, output):  # noqa: A002
    _gemv_into("rnb_hip_q4k_gemv", weights, rows, cols, input, output)


def q4k_gemv_batch(weights, rows, cols, input):  # noqa: A002
    """seq_len = len(input) / cols; returns out[seq][rows]"""
    return _gemv_batch("rnb_hip_q4k_gemv_batch", weights, rows, cols, input)


def q4_0_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q4_0_gemv", weights, rows, cols, input)


def q4_0_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q4_0_gemv_batch", weights, rows, cols, input)


def q4_1_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q4_1_gemv", weights, rows, cols, input)


def q4_1_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q4_1_gemv_batch", weights, rows, cols, input)


def q5_0_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q5_0_gemv", weights, rows, cols, input)


def q5_0_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q5_0_gemv_batch", weights, rows, cols, input)


def q5_1_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q5_1_gemv", weights, rows, cols, input)


def q5_1_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q5_1_gemv_batch", weights, rows, cols, input)


def q8_1_gemv(weights, rows, cols, input):  # noqa: A002
    """crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:507-523."""
    return _gemv("rnb_hip_q8_1_gemv", weights, rows, cols, input)


def q8_1_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q8_1_gemv_batch", weights, rows, cols, input)


def _gemv_with_device_input(fn_name: str, weights, rows: int, cols: int, input_dev, output: np.ndarray) -> None:
    w = _bytes_view(weights)
    if output.dtype != np.float32 or not output.flags.c_contiguous:
        raise TypeError("output must be a C-contiguous float32 array")
    _check(getattr(lib(), fn_name)(_ptr(w), w.size, rows, cols, input_dev.ptr, _ptr(output), output.size))


def q4k_gemv_with_device_input(weights, rows, cols, input_dev, output):
    """quant_api.rs:288-330: host-resident Q4_K weights, one token on the device (a DeviceBuffer of cols floats), result
    into the caller's host array."""
    _gemv_with_device_input("rnb_hip_q4k_gemv_with_device_input", weights, rows, cols, input_dev, output)


def q6k_gemv_with_device_input(weights, rows, cols, input_dev, output):
    """quant_api.rs:242-284, the Q6_K form."""
    _gemv_with_device_input("rnb_hip_q6k_gemv_with_device_input", weights, rows, cols, input_dev, output)


def quant_embedding_gather(quant: int, weights, rows: int, cols: int, token_ids) -> np.ndarray:
    """quant_api.rs:1827-1975: the rows `token_ids` name, dequantised to f32 [len(token_ids)][cols]; `quant` is the ggml
    type id of any block format or of f32 / f16 / bf16."""
    w = _bytes_view(weights)
    ids = np.ascontiguousarray(token_ids, dtype=np.uint32)
    out = np.empty(ids.size * cols, dtype=np.float32)
    _check(lib().rnb_hip_quant_embedding_gather(quant, _ptr(w), w.size, rows, cols, _ptr(ids), ids.size, _ptr(out), out.size))
    return out


def quant_embedding_gather_dev(quant: int, weights, rows: int, cols: int, token_ids, out: "DeviceBuffer") -> None:
    """The same with the rows left on the device (launchers.rs:4062), e.g. as the input of rms_norm_dev."""
    w = _bytes_view(weights)
    ids = np.ascontiguousarray(token_ids, dtype=np.uint32)
    if out.nbytes < ids.size * cols * 4:
        raise ValueError("output buffer too small")
    _check(lib().rnb_hip_quant_embedding_gather_dev(quant, _ptr(w), w.size, rows, cols, _ptr(ids), ids.size, out.ptr))


def iq2_xxs_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_iq2_xxs_gemv", weights, rows, cols, input)


def iq2_xxs_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_iq2_xxs_gemv_batch", weights, rows, cols, input)


def iq2_s_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_iq2_s_gemv", weights, rows, cols, input)


def iq2_s_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_iq2_s_gemv_batch", weights, rows, cols, input)


def iq3_xxs_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_iq3_xxs_gemv", weights, rows, cols, input)


def iq3_xxs_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_iq3_xxs_gemv_batch", weights, rows, cols, input)


def iq4_xs_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_iq4_xs_gemv", weights, rows, cols, input)


def iq4_xs_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_iq4_xs_gemv_batch", weights, rows, cols, input)


def q2k_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q2k_gemv", weights, rows, cols, input)


def q2k_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q2k_gemv_batch", weights, rows, cols, input)


def q3k_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q3k_gemv", weights, rows, cols, input)


def q3k_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q3k_gemv_batch", weights, rows, cols, input)


def q5k_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q5k_gemv", weights, rows, cols, input)


def q5k_gemv_into(weights, rows, cols, input, output):  # noqa: A002
    _gemv_into("rnb_hip_q5k_gemv", weights, rows, cols, input, output)


def q5k_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q5k_gemv_batch", weights, rows, cols, input)


def q6k_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q6k_gemv", weights, rows, cols, input)


def q6k_gemv_into(weights, rows, cols, input, output):  # noqa: A002
    _gemv_into("rnb_hip_q6k_gemv", weights, rows, cols, input, output)


def q6k_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q6k_gemv_batch", weights, rows, cols, input)


def q8_0_gemv(weights, rows, cols, input):  # noqa: A002
    return _gemv("rnb_hip_q8_0_gemv", weights, rows, cols, input)


def q8_0_gemv_batch(weights, rows, cols, input):  # noqa: A002
    return _gemv_batch("rnb_hip_q8_0_gemv_batch", weights, rows, cols, input)


def q8_0_head_gemv_batch(weights, head_count: int, rows_per_head: int, cols: int, token_count: int, input) -> np.ndarray:  # noqa: A002
    """quant_api.rs:824-882: weights [head][rows_per_head][cols], input [token][head][cols]; returns
    out[token][head_count * rows_per_head]."""
    w, x = _bytes_view(weights), _f32(input).ravel()
    out = np.empty((token_count, head_count * rows_per_head), dtype=np.float32)
    _check(lib().rnb_hip_q8_0_head_gemv_batch(_ptr(w), w.size, head_count, rows_per_head, cols, token_count, _ptr(x), x.size,
                                              _ptr(out), out.size))
    return out


def qwen35_sparse_experts_selected_base_by_token(gate_all, up_all, down_all, expert_ids, route_weights, token_ids,
                                                 token_count: int, down_quant: int, n_ff: int, n_embd: int,
                                                 input, shared=None) -> np.ndarray:  # noqa: A002
    """api/qwen_moe_api.rs:2529-2541; returns out[token_count][n_embd].  `shared`: the shared expert's (gate, up, down)
    bytes; slots with expert id n_expert then run on it (the decode call's extra slot, moe_view/fanout.rs:804-812)."""
    g, u, d = _bytes_view(gate_all), _bytes_view(up_all), _bytes_view(down_all)
    sh = [_bytes_view(a) for a in shared] if shared is not None else []
    sh_args = [v for a in sh for v in (_ptr(a), a.size)] if sh else [None, 0, None, 0, None, 0]
    e = np.ascontiguousarray(expert_ids, dtype=np.uint32)
    r = _f32(route_weights).ravel()
    t = np.ascontiguousarray(token_ids, dtype=np.uint32)
    if not (e.size == r.size == t.size):
        raise BackendError(1, f"Qwen35 full-layer token-batch length mismatch: expert={e.size} route={r.size} "
                              f"token={t.size}")
    x = _f32(input).ravel()
    out = np.empty((token_count, n_embd), dtype=np.float32)
    _check(lib().rnb_hip_moe_sparse_experts_by_token(_ptr(g), g.size, _ptr(u), u.size, _ptr(d), d.size, *sh_args, _ptr(e),
                                                     _ptr(r), _ptr(t), e.size, token_count, down_quant, n_ff, n_embd,
                                                     _ptr(x), x.size, _ptr(out), out.size))
    return out


# ---- device-resident helpers (benchmarks, fused callers) -----------------------------------

class DeviceBuffer:
    """A hipMalloc'd range owned by the library's device."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        self.ptr = lib().rnb_hip_dev_alloc(self.nbytes)
        if not self.ptr:
            raise BackendError(3, last_error())

    @classmethod
    def from_host(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = cls(a.nbytes)
        _check(lib().rnb_hip_dev_upload(buf.ptr, _ptr(a), a.nbytes))
        return buf

    def to_host(self, dtype, count: Optional[int] = None) -> np.ndarray:
        dt = np.dtype(dtype)
        n = self.nbytes // dt.itemsize if count is None else count
        out = np.empty(n, dtype=dt)
        _check(lib().rnb_hip_dev_download(_ptr(out), self.ptr, out.nbytes))
        return out

    def free(self) -> None:
        if self.ptr:
            lib().rnb_hip_dev_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def calib_read(buf: DeviceBuffer, nbytes: int, non_temporal: bool = False) -> None:
    """Enqueue the read-only calibration kernel over the first nbytes of buf."""
    _check(lib().rnb_hip_calib_read(buf.ptr, nbytes, 1 if non_temporal else 0))


def calib_mfma_i8(iters: int, workgroups: int) -> int:
    """Enqueue the matrix-instruction-only calibration kernel; returns the integer operations it performs."""
    ops = C.c_uint64()
    _check(lib().rnb_hip_calib_mfma_i8(iters, workgroups, C.byref(ops)))
    return int(ops.value)


def gemv_dev(quant: int, w: DeviceBuffer, rows: int, cols: int, x: DeviceBuffer, seq_len: int,
             out: DeviceBuffer) -> None:
    """Enqueue activation quantisation + GEMV/GEMM on the library stream; does not synchronise."""
    _check(lib().rnb_hip_gemv_dev(quant, w.ptr, rows, cols, x.ptr, seq_len, out.ptr))


def gemv_dev_noalloc(quant: int, w: DeviceBuffer, rows: int, cols: int, x: DeviceBuffer, seq_len: int,
                     out: DeviceBuffer) -> None:
    """gemv_dev with its scratch in the library's fixed device array: never allocates; does not synchronise."""
    _check(lib().rnb_hip_gemv_dev_noalloc(quant, w.ptr, rows, cols, x.ptr, seq_len, out.ptr))


def gemv_dev_noalloc_scratch_bytes() -> int:
    return int(lib().rnb_hip_gemv_dev_noalloc_scratch_bytes())


def rms_norm_dev(x: DeviceBuffer, weight: DeviceBuffer, eps: float, seq_len: int, hidden: int, out: DeviceBuffer,
                 unit_offset: bool = False, quantize: bool = False) -> None:
    """RMS norm of [seq_len][hidden] rows; with quantize=True Q8_K(out) is also left in the activation scratch
    (out may then be None)."""
    fn = lib().rnb_hip_rms_norm_quantize_dev if quantize else lib().rnb_hip_rms_norm_dev
    _check(fn(x.ptr, weight.ptr, eps, 1 if unit_offset else 0, seq_len, hidden, out.ptr if out is not None else None))


def rms_norm_add_rms_norm_quantize_dev(inp: DeviceBuffer, post_weight: DeviceBuffer, post_eps: float, residual: DeviceBuffer,
                                       pre_weight: DeviceBuffer, pre_eps: float, seq_len: int, hidden: int,
                                       out: Optional[DeviceBuffer], post_unit_offset: bool = False,
                                       pre_unit_offset: bool = False) -> None:
    """residual += norm(inp, post_weight); out = norm(residual, pre_weight); Q8_K(out) -> activation scratch."""
    _check(lib().rnb_hip_rms_norm_add_rms_norm_quantize_dev(
        inp.ptr, post_weight.ptr, post_eps, 1 if post_unit_offset else 0, residual.ptr, pre_weight.ptr, pre_eps,
        1 if pre_unit_offset else 0, seq_len, hidden, out.ptr if out is not None else None))


def moe_route_topk_dev(logits: DeviceBuffer, token_count: int, n_expert: int, k: int, idx: DeviceBuffer,
                       weights: DeviceBuffer) -> None:
    """Per token: top-k expert ids (ties to the lower id) and the softmax over their logits, in rank order."""
    _check(lib().rnb_hip_moe_route_topk_dev(logits.ptr, token_count, n_expert, k, idx.ptr, weights.ptr))


def quantize_dev(quant: int, x: DeviceBuffer, seq_len: int, cols: int) -> None:
    """Fill the library's activation scratch from x (Q8 for Q8_0 weights, Q8_K otherwise)."""
    _check(lib().rnb_hip_quantize_dev(quant, x.ptr, seq_len, cols))


def gemv_quantized_dev(quant: int, w: DeviceBuffer, rows: int, cols: int, seq_len: int, out: DeviceBuffer) -> None:
    """GEMV/GEMM against the activation scratch filled by quantize_dev; does not synchronise."""
    _check(lib().rnb_hip_gemv_quantized_dev(quant, w.ptr, rows, cols, seq_len, out.ptr))


def moe_sparse_experts_by_token_dev(gate: DeviceBuffer, up: DeviceBuffer, down: DeviceBuffer, n_expert: int,
                                    expert_ids, route_weights, token_ids, token_count: int, down_quant: int,
                                    n_ff: int, n_embd: int, x: DeviceBuffer, out: DeviceBuffer, shared=None) -> None:
    """`shared`: three DeviceBuffers, the shared expert's gate, up and down (expert id n_expert in the slot list)."""
    sh = [b.ptr for b in shared] if shared is not None else [None, None, None]
    e = np.ascontiguousarray(expert_ids, dtype=np.uint32)
    r = _f32(route_weights).ravel()
    t = np.ascontiguousarray(token_ids, dtype=np.uint32)
    _check(lib().rnb_hip_moe_sparse_experts_by_token_dev(gate.ptr, up.ptr, down.ptr, n_expert, *sh, _ptr(e), _ptr(r),
                                                         _ptr(t), e.size, token_count, down_quant, n_ff, n_embd,
                                                         x.ptr, out.ptr))


# ---- trait facade --------------------------------------------------------------------------

class HipBackend:
    """Capability facade in the shape of `trait Backend` (crates/rnb-backend/api/src/lib.rs:1281-1285).
    Like CudaBackend::execute (crates/rnb-backend/cuda/src/lib.rs:193-195), execute() does not run
    requests: real work flows through the operator functions above."""

    def kind(self) -> str:
        return "Hip"

    def kind_ordinal(self) -> int:
        return lib().rnb_hip_backend_kind()

    def capabilities(self) -> dict:
        names = {OP_MATMUL: "MatMul", OP_ATTENTION: "Attention", OP_GDN: "Gdn", OP_MOE: "MoE", OP_SAMPLER: "Sampler"}
        return {name: bool(lib().rnb_hip_backend_supports(op)) for op, name in names.items()}

    def supports_quant(self, op: int, quant: int) -> bool:
        return bool(lib().rnb_hip_backend_supports_quant(op, quant))

    def execute(self, request) -> None:
        raise BackendError(2, "HipBackend::execute: requests are served by the operator functions "
                              "(q4k_gemv, q6k_gemv, q8_0_gemv, *_batch, qwen35_sparse_experts_*)")


def q6k_gemv_argmax(weights, rows: int, cols: int, input) -> tuple:  # noqa: A002
    """quant_api.rs:2170-2204 -> (row index, value)"""
    w, x = _bytes_view(weights), _f32(input).ravel()
    idx, val = _u32(), C.c_float()
    _check(lib().rnb_hip_q6k_gemv_argmax(_ptr(w), w.size, rows, cols, _ptr(x), x.size, C.byref(idx), C.byref(val)))
    return int(idx.value), float(val.value)


def dense_q4k_attention_qkv(q_weights, k_weights, v_weights, q_rows: int, kv_rows: int, n_embd: int, input,  # noqa: A002
                            q: np.ndarray, k: np.ndarray, v: np.ndarray) -> None:
    """api/dense_api.rs:916-985: writes q[:q_rows], k[:kv_rows], v[:kv_rows] (f32, C-contiguous, may be longer)."""
    qw, kw, vw = _bytes_view(q_weights), _bytes_view(k_weights), _bytes_view(v_weights)
    x = _f32(input).ravel()
    for name, a in (("q", q), ("k", k), ("v", v)):
        if a.dtype != np.float32 or not a.flags["C_CONTIGUOUS"]:
            raise TypeError(f"{name} must be a C-contiguous float32 array")
    _check(lib().rnb_hip_dense_q4k_attention_qkv(_ptr(qw), qw.size, _ptr(kw), kw.size, _ptr(vw), vw.size, q_rows, kv_rows,
                                                 n_embd, _ptr(x), x.size, _ptr(q), q.size, _ptr(k), k.size, _ptr(v), v.size))


def q8_0_gemv_argmax(weights, rows: int, cols: int, input) -> tuple:  # noqa: A002
    """quant_api.rs:733-768 -> (row index, value)"""
    w, x = _bytes_view(weights), _f32(input).ravel()
    idx, val = _u32(), C.c_float()
    _check(lib().rnb_hip_q8_0_gemv_argmax(_ptr(w), w.size, rows, cols, _ptr(x), x.size, C.byref(idx), C.byref(val)))
    return int(idx.value), float(val.value)


def q8_0_gemv_argmax_q8dot(weights, rows: int, cols: int, input) -> tuple:  # noqa: A002
    """quant_api.rs:770-805 -> (row index, value); the same integer dots as q8_0_gemv_argmax"""
    w, x = _bytes_view(weights), _f32(input).ravel()
    idx, val = _u32(), C.c_float()
    _check(lib().rnb_hip_q8_0_gemv_argmax_q8dot(_ptr(w), w.size, rows, cols, _ptr(x), x.size, C.byref(idx), C.byref(val)))
    return int(idx.value), float(val.value)


def dense_q4k_silu_ffn_batch(gate_weights, up_weights, down_weights, down_quant: int, n_ff: int, n_embd: int,
                             seq_len: int, input) -> np.ndarray:  # noqa: A002
    """api/dense_api.rs:297-337; returns out[seq_len][n_embd]."""
    g, u, d = _bytes_view(gate_weights), _bytes_view(up_weights), _bytes_view(down_weights)
    x = _f32(input).ravel()
    out = np.empty((seq_len, n_embd), dtype=np.float32)
    _check(lib().rnb_hip_dense_q4k_silu_ffn_batch(_ptr(g), g.size, _ptr(u), u.size, _ptr(d), d.size, down_quant, n_ff,
                                                  n_embd, seq_len, _ptr(x), x.size, _ptr(out), out.size))
    return out


def dense_q4k_gelu_ffn_batch(gate_weights, up_weights, down_weights, down_quant: int, n_ff: int, n_embd: int,
                             seq_len: int, input) -> np.ndarray:  # noqa: A002
    """api/dense_api.rs:256-293; returns out[seq_len][n_embd]."""
    g, u, d = _bytes_view(gate_weights), _bytes_view(up_weights), _bytes_view(down_weights)
    x = _f32(input).ravel()
    out = np.empty((seq_len, n_embd), dtype=np.float32)
    _check(lib().rnb_hip_dense_q4k_gelu_ffn_batch(_ptr(g), g.size, _ptr(u), u.size, _ptr(d), d.size, down_quant, n_ff,
                                                  n_embd, seq_len, _ptr(x), x.size, _ptr(out), out.size))
    return out


def dense_q4k_gelu_ffn(gate_weights, up_weights, down_weights, down_quant: int, n_ff: int, n_embd: int,
                       input) -> np.ndarray:  # noqa: A002
    """api/dense_api.rs:182-254: one token; returns out[n_embd]."""
    g, u, d = _bytes_view(gate_weights), _bytes_view(up_weights), _bytes_view(down_weights)
    x = _f32(input).ravel()
    out = np.empty(n_embd, dtype=np.float32)
    _check(lib().rnb_hip_dense_q4k_gelu_ffn(_ptr(g), g.size, _ptr(u), u.size, _ptr(d), d.size, down_quant, n_ff, n_embd,
                                            _ptr(x), x.size, _ptr(out), out.size))
    return out


def dense_q4k_silu_ffn_dev(gate: "DeviceBuffer", up: "DeviceBuffer", down: "DeviceBuffer", down_quant: int, n_ff: int,
                           n_embd: int, seq_len: int, x: "DeviceBuffer", out: "DeviceBuffer") -> None:
    _check(lib().rnb_hip_dense_q4k_silu_ffn_dev(gate.ptr, up.ptr, down.ptr, down_quant, n_ff, n_embd, seq_len, x.ptr,
                                                out.ptr))


# ---- GGUF container (crates/rnb-loader/src/gguf/parser.rs, crates/rnb-loader/src/convert.rs) ---------------------

class _GGUFTensorStruct(C.Structure):
    _fields_ = [("name", C.c_char_p), ("n_dims", C.c_uint32), ("shape", C.c_uint64 * 4), ("ggml_type", C.c_uint32),
                ("offset", C.c_uint64), ("file_offset", C.c_uint64), ("n_bytes", C.c_uint64), ("data", C.c_void_p)]


class GGUFTensor:
    """One row of the tensor table: TensorInfo (crates/rnb-loader/src/gguf/types.rs:103-110) plus where its bytes are."""

    def __init__(self, owner: "GGUFFile", index: int, st: _GGUFTensorStruct):
        self._owner = owner  # keeps the mapping alive while `data` is in use
        self.index = index
        self.name = st.name.decode()
        self.shape = [int(st.shape[i]) for i in range(st.n_dims)]
        self.ggml_type = int(st.ggml_type)
        self.offset = int(st.offset)
        self.file_offset = int(st.file_offset)
        self.n_bytes = int(st.n_bytes)
        self._addr = st.data

    @property
    def data(self) -> np.ndarray:
        """The tensor's bytes inside the mapping (no copy)."""
        if not self._addr:
            raise BackendError(1, f"tensor '{self.name}' does not lie inside the file")
        buf = (C.c_uint8 * self.n_bytes).from_address(self._addr)
        arr = np.frombuffer(buf, dtype=np.uint8)
        arr.flags.writeable = False
        return arr

    def prewarm(self) -> None:
        _check(lib().rnb_hip_gguf_prewarm_tensor(self._owner._h, self.index))


class GGUFFile:
    """GGUFFile::parse (+ map_tensors when opened from a path).  `GGUFFile(path)` maps the file;
    `GGUFFile.parse(bytes)` parses caller-owned bytes without the payload bounds checks."""

    def __init__(self, path: Optional[str] = None, *, _handle=None, _keep=None):
        self._keep = _keep
        if _handle is not None:
            self._h = _handle
            return
        h = _vp()
        _check(lib().rnb_hip_gguf_open(os.fsencode(path), C.byref(h)))
        self._h = h

    @classmethod
    def parse(cls, data) -> "GGUFFile":
        view = np.frombuffer(data, dtype=np.uint8) if not isinstance(data, np.ndarray) else data
        h = _vp()
        _check(lib().rnb_hip_gguf_parse(_ptr(view) if view.size else None, view.size, C.byref(h)))
        return cls(_handle=h, _keep=view)

    def map_tensors(self) -> None:
        _check(lib().rnb_hip_gguf_map_tensors(self._h))

    def close(self) -> None:
        if self._h:
            lib().rnb_hip_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def version(self) -> int:
        return int(lib().rnb_hip_gguf_version(self._h))

    @property
    def alignment(self) -> int:
        return int(lib().rnb_hip_gguf_alignment(self._h))

    @property
    def data_start(self) -> int:
        return int(lib().rnb_hip_gguf_data_start(self._h))

    def __len__(self) -> int:
        return int(lib().rnb_hip_gguf_tensor_count(self._h))

    def tensor_at(self, index: int) -> GGUFTensor:
        st = _GGUFTensorStruct()
        _check(lib().rnb_hip_gguf_tensor_at(self._h, index, C.byref(st)))
        return GGUFTensor(self, index, st)

    def tensors(self) -> list:
        return [self.tensor_at(i) for i in range(len(self))]

    def tensor(self, name: str) -> GGUFTensor:
        for i in range(len(self)):
            t = self.tensor_at(i)
            if t.name == name:
                return t
        st = _GGUFTensorStruct()
        _check(lib().rnb_hip_gguf_find_tensor(self._h, name.encode(), C.byref(st)))
        raise AssertionError("unreachable")

    def metadata_keys(self) -> list:
        n = int(lib().rnb_hip_gguf_metadata_count(self._h))
        return [lib().rnb_hip_gguf_metadata_key(self._h, i).decode() for i in range(n)]

    def metadata_type(self, key: str) -> int:
        return int(lib().rnb_hip_gguf_metadata_type(self._h, key.encode()))

    def metadata(self, key: str):
        """Value of a key as a Python object (int, float, bool, str or list)."""
        k = key.encode()
        t = self.metadata_type(key)
        if t < 0:
            v = C.c_uint64()
            _check(lib().rnb_hip_gguf_metadata_u64(self._h, k, C.byref(v)))  # raises "missing metadata key"
        if t in (0, 2, 4, 10):
            v = C.c_uint64()
            _check(lib().rnb_hip_gguf_metadata_u64(self._h, k, C.byref(v)))
            return int(v.value)
        if t in (1, 3, 5, 11):
            v = C.c_int64()
            _check(lib().rnb_hip_gguf_metadata_i64(self._h, k, C.byref(v)))
            return int(v.value)
        if t in (6, 12):
            v = C.c_double()
            _check(lib().rnb_hip_gguf_metadata_f64(self._h, k, C.byref(v)))
            return float(v.value)
        if t == 7:
            v = C.c_uint64()
            _check(lib().rnb_hip_gguf_metadata_u64(self._h, k, C.byref(v)))
            return bool(v.value)
        if t == 8:
            return lib().rnb_hip_gguf_metadata_str(self._h, k).decode()
        et, n = C.c_uint32(), C.c_uint64()
        _check(lib().rnb_hip_gguf_metadata_array(self._h, k, C.byref(et), C.byref(n)))
        if et.value == 8:
            return [lib().rnb_hip_gguf_metadata_array_str(self._h, k, i).decode() for i in range(n.value)]
        if et.value == 9:
            return [None] * n.value  # nested arrays are validated but not kept
        out = []
        for i in range(n.value):
            v = C.c_double()
            _check(lib().rnb_hip_gguf_metadata_array_f64(self._h, k, i, C.byref(v)))
            out.append(v.value if et.value in (6, 12) else (bool(v.value) if et.value == 7 else int(v.value)))
        return out


def gguf_tensor_size(shape: Sequence[int], ggml_type: int) -> int:
    """checked_tensor_size, crates/rnb-loader/src/convert.rs:28-43"""
    arr = (C.c_uint64 * max(1, len(shape)))(*shape)
    out = C.c_uint64()
    _check(lib().rnb_hip_gguf_tensor_size(arr, len(shape), ggml_type, C.byref(out)))
    return int(out.value)
