"""runnburn_amd -- MI355X (gfx950) backend for runNburn's quantized matmul hot path.

Python mirror of the reference's operator surface over the C ABI in include/rnb_hip.h.  The
functions keep the reference's names, argument meaning and error behaviour:
`Result<Vec<f32>, String>` becomes "return an array or raise BackendError(message)".

  q4k_gemv / q4k_gemv_into / q4k_gemv_batch   crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:183-238, 2283-2319
  q4_0 / q4_1 / q5_0 / q5_1 _gemv (+ _batch)  quant_api.rs:374-496
  q8_1_gemv (+ _batch)                         quant_api.rs:507-541
  q2k_gemv / q3k_gemv (+ _batch)              quant_api.rs:73-181
  iq2_xxs / iq2_s / iq3_xxs / iq4_xs _gemv (+ _batch)  quant_api.rs:543-722
  quant_embedding_gather                       quant_api.rs:1827-1975
  q5k_gemv / q5k_gemv_into / q5k_gemv_batch   quant_api.rs:2207-2281, 3957-3993
  q6k_gemv / q6k_gemv_into / q6k_gemv_batch   quant_api.rs:2071-2168, 3919-3955
  q8_0_gemv / q8_0_gemv_batch                 quant_api.rs:498-505, 807-822
  q8_0_head_gemv_batch                        quant_api.rs:824-882
  qwen35_sparse_experts_selected_base_by_token  api/qwen_moe_api.rs:2529-2541
  HipBackend                                  crates/rnb-backend/api/src/lib.rs:1281-1285 (trait Backend)

There is no CPU fallback: when librnb_hip.so is missing or no gfx950 device opens, every
operator raises.
"""
from __future__ import annotations

from .binding import (  # noqa: F401
    BackendError,
    HipBackend,
    DeviceBuffer,
    GGUFFile,
    GGUFTensor,
    gguf_tensor_size,
    GGML_Q4_0,
    GGML_Q4_1,
    GGML_Q5_0,
    GGML_Q5_1,
    GGML_Q8_1,
    GGML_Q2_K,
    GGML_Q3_K,
    GGML_Q4_K,
    GGML_Q5_K,
    GGML_Q6_K,
    GGML_Q8_0,
    OP_MATMUL,
    OP_MOE,
    STATUS_NAMES,
    dense_q4k_silu_ffn_batch,
    dense_q4k_silu_ffn_dev,
    device_available,
    device_name,
    calib_mfma_i8,
    calib_read,
    gemv_dev,
    gemv_dev_noalloc,
    gemv_dev_noalloc_scratch_bytes,
    gemv_quantized_dev,
    quantize_dev,
    rms_norm_dev,
    rms_norm_add_rms_norm_quantize_dev,
    moe_route_topk_dev,
    last_error,
    lib,
    lib_path,
    moe_sparse_experts_by_token_dev,
    prewarm,
    q4k_gemv,
    q4k_gemv_batch,
    q4k_gemv_into,
    q4_0_gemv,
    q4_0_gemv_batch,
    q4_1_gemv,
    q4_1_gemv_batch,
    q5_0_gemv,
    q5_0_gemv_batch,
    q5_1_gemv,
    q5_1_gemv_batch,
    q8_1_gemv,
    q8_1_gemv_batch,
    q4k_gemv_with_device_input,
    q6k_gemv_with_device_input,
    iq2_xxs_gemv,
    iq2_xxs_gemv_batch,
    iq2_s_gemv,
    iq2_s_gemv_batch,
    iq3_xxs_gemv,
    iq3_xxs_gemv_batch,
    iq4_xs_gemv,
    iq4_xs_gemv_batch,
    GGML_IQ2_XXS,
    GGML_IQ3_XXS,
    GGML_IQ2_S,
    GGML_IQ4_XS,
    GGML_F32,
    GGML_F16,
    GGML_BF16,
    quant_embedding_gather,
    quant_embedding_gather_dev,
    q2k_gemv,
    q2k_gemv_batch,
    q3k_gemv,
    q3k_gemv_batch,
    q5k_gemv,
    q5k_gemv_batch,
    q5k_gemv_into,
    q6k_gemv,
    q6k_gemv_batch,
    q6k_gemv_into,
    q6k_gemv_argmax,
    dense_q4k_attention_qkv,
    dense_q4k_gelu_ffn,
    dense_q4k_gelu_ffn_batch,
    q8_0_gemv_argmax,
    q8_0_gemv_argmax_q8dot,
    q8_0_gemv,
    q8_0_gemv_batch,
    q8_0_head_gemv_batch,
    quantize_input_q8,
    quantize_input_q8k,
    qwen35_sparse_experts_selected_base_by_token,
    release,
    resident_bytes,
    residency_stats,
    set_resident_budget,
    offload_unpinned,
    stream_handle,
    sync,
    transfer_counters,
)

__all__ = [name for name in dir() if not name.startswith("_")]
