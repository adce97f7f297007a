// Embedding gather: rows of a block-quantised matrix picked by token id and dequantised to f32
// (quant_embedding_gather, crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:1827-1975).  The kernel is the same for
// every format; a format supplies `octet(block, o, y)`: elements 8 o .. 8 o + 7 of one block, with the float operations
// of the reference's dequantiser in its order (crates/rnb-cpu/src/quantize/dequant.rs, iq.rs), so the values are the
// dequantiser's bit for bit.  One thread per eight elements: two 16-byte stores, consecutive threads consecutive.
#pragma once

#include "device_utils.h"

namespace rnb {

// ids == nullptr: output row t is matrix row t (the caller compacted the rows it needs)
template <typename F>
__global__ void __launch_bounds__(256)
    embed_gather_kernel(const uint8_t *__restrict__ w, size_t row_bytes, const uint32_t *__restrict__ ids,
                        uint32_t octets_per_row, float *__restrict__ out) {
    const uint32_t o = blockIdx.x * 256 + threadIdx.x;
    if (o >= octets_per_row) return;
    const uint32_t tok = blockIdx.y;
    const size_t row = ids != nullptr ? ids[tok] : tok;
    constexpr uint32_t kOctets = F::kElems / 8;
    const uint32_t blk = o / kOctets;
    float y[8];
    F::octet(w + row * row_bytes + static_cast<size_t>(blk) * F::kBytes, static_cast<int>(o - blk * kOctets), y);
    float4 *dst = reinterpret_cast<float4 *>(out + (static_cast<size_t>(tok) * octets_per_row + o) * 8);
    dst[0] = make_float4(y[0], y[1], y[2], y[3]);
    dst[1] = make_float4(y[4], y[5], y[6], y[7]);
}

// n_tokens <= 65535 per launch (grid.y); the caller cuts longer lists
template <typename F>
void launch_embed_gather_format(const uint8_t *w, size_t row_bytes, const uint32_t *ids, uint32_t n_tokens, uint32_t cols,
                                float *out, hipStream_t stream) {
    const uint32_t octets = cols / 8;
    hipLaunchKernelGGL((embed_gather_kernel<F>), dim3((octets + 255) / 256, n_tokens, 1), dim3(256), 0, stream, w, row_bytes,
                       ids, octets, out);
}

}  // namespace rnb
