// Dequantisers of the embedding gather for the 32-element formats, the K-quants and the float formats (the importance
// quants sit beside their codebooks in gemv_iq.hip).  Every `octet` follows the reference's dequantiser operation by
// operation: crates/rnb-cpu/src/quantize/dequant.rs:7-60 (32-element formats), :66-86 (Q2_K), :237-297 (Q3_K),
// :353-381 (Q4_K), :735-770 (Q5_K), :780-807 (Q6_K).  The library is compiled with -ffp-contract=off, so `a * b - c`
// is a multiply and a subtraction, as there.
#include "embed_gather.h"
#include "kernels.h"

namespace rnb {

namespace {

__device__ __forceinline__ uint32_t ld_u32_bytes(const uint8_t *p) {
    return static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8) | (static_cast<uint32_t>(p[2]) << 16) |
           (static_cast<uint32_t>(p[3]) << 24);
}

// ---- float formats: "blocks" of 32 elements, as the reference's table has them ------------------
struct DqF32 {
    static constexpr uint32_t kElems = 32, kBytes = 128;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = __uint_as_float(ld_u32_bytes(blk + 32 * o + 4 * i));
    }
};
struct DqF16 {
    static constexpr uint32_t kElems = 32, kBytes = 64;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = f16_bits_to_f32(blk[16 * o + 2 * i] | (blk[16 * o + 2 * i + 1] << 8));
    }
};
struct DqBF16 {
    static constexpr uint32_t kElems = 32, kBytes = 64;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++)
            y[i] = __uint_as_float((static_cast<uint32_t>(blk[16 * o + 2 * i]) << 16) |
                                   (static_cast<uint32_t>(blk[16 * o + 2 * i + 1]) << 24));
    }
};

// ---- 32-element formats ---------------------------------------------------------------------------
//   Q4_0 {f16 d, qs[16]}  (code - 8) d      Q4_1 {f16 d, f16 m, qs[16]}  code d + m
//   Q5_0 {f16 d, qh[4], qs[16]}  (code - 16) d      Q5_1 {f16 d, f16 m, qh[4], qs[16]}  code d + m
//   Q8_0 {f16 d, i8 qs[32]}  code d         Q8_1 {f16 d, f16 s, i8 qs[32]}  code d
// element e < 16: low nibble of qs[e]; 16 + e: high nibble of qs[e]; fifth bit of element e = bit e of qh
template <uint32_t kBlockBytes, int kQs, int kQh, bool kMin, int kOffset, bool kByteCodes>
struct DqBlock32 {
    static constexpr uint32_t kElems = 32, kBytes = kBlockBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const float d = ld_f16(blk);
        const float m = kMin ? ld_f16(blk + 2) : 0.0f;
        const uint32_t qh = kQh >= 0 ? ld_u32_bytes(blk + (kQh >= 0 ? kQh : 0)) : 0u;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int e = 8 * o + i;
            int code;
            if constexpr (kByteCodes) {
                code = static_cast<int8_t>(blk[kQs + e]);
            } else {
                code = e < 16 ? (blk[kQs + e] & 0x0f) : (blk[kQs + e - 16] >> 4);
                if constexpr (kQh >= 0) code |= static_cast<int>((qh >> e) & 1u) << 4;
            }
            if constexpr (kMin)
                y[i] = static_cast<float>(code) * d + m;
            else
                y[i] = (static_cast<float>(code) - static_cast<float>(kOffset)) * d;
        }
    }
};
using DqQ4_0 = DqBlock32<kQ4_0Bytes, 2, -1, false, 8, false>;
using DqQ4_1 = DqBlock32<kQ4_1Bytes, 4, -1, true, 0, false>;
using DqQ5_0 = DqBlock32<kQ5_0Bytes, 6, 2, false, 16, false>;
using DqQ5_1 = DqBlock32<kQ5_1Bytes, 8, 4, true, 0, false>;
using DqQ8_0 = DqBlock32<kQ8_0Bytes, 2, -1, false, 0, true>;
using DqQ8_1 = DqBlock32<kQ8_1Bytes, 4, -1, false, 0, true>;

// ---- K-quants -------------------------------------------------------------------------------------
// {u8 scales[16] (scale | min << 4), u8 qs[64], f16 d, f16 dmin}: sub-block j (16 elements) lives in half j / 8, bytes
// 16 (j % 2).. of that half's 32, bit pair (j % 8) / 2
struct DqQ2K {
    static constexpr uint32_t kElems = 256, kBytes = kQ2KBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int j = o >> 1, l0 = (o & 1) * 8;
        const float d = ld_f16(blk + 80), dmin = ld_f16(blk + 82);
        const float scale = d * static_cast<float>(blk[j] & 0x0f);
        const float mn = dmin * static_cast<float>(blk[j] >> 4);
        const int q_base = (j / 8) * 32 + (j % 2) * 16, shift = ((j % 8) / 2) * 2;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float q = static_cast<float>((blk[16 + q_base + l0 + i] >> shift) & 3);
            y[i] = q * scale - mn;
        }
    }
};

// {u8 hmask[32], u8 qs[64], u8 scales[12], f16 d}: element index = 128 n + 32 (shift / 2) + 16 h + l; 2-bit field minus
// 4 unless bit 4 n + shift / 2 of hmask[16 h + l] is set; 6-bit scale k = low nibble (k / 8 of byte k % 8) | two bits
// (pair k / 4 of byte 8 + k % 4) << 4, minus 32
struct DqQ3K {
    static constexpr uint32_t kElems = 256, kBytes = kQ3KBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int idx = 8 * o, n = idx >> 7, rem = idx & 127, sh = rem >> 5, h = (rem & 31) >> 4, l0 = rem & 15, is = idx >> 4;
        const uint8_t *sb = blk + 96;
        const int lo = is < 8 ? (sb[is] & 0x0f) : (sb[is - 8] >> 4);
        const int hi = (sb[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
        const int scale = static_cast<int8_t>(lo | (hi << 4));
        const float dl = ld_f16(blk + 108) * (static_cast<float>(scale) - 32.0f);
        const uint32_t m = 1u << (4 * n + sh);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int l = l0 + i;
            const int qv = (blk[32 + 32 * n + 16 * h + l] >> (2 * sh)) & 3;
            const int hv = (blk[16 * h + l] & m) ? 0 : 4;
            y[i] = dl * static_cast<float>(qv - hv);
        }
    }
};

// scale and min of sub-block j from the 12 packed bytes (get_scale_min_k4, crates/rnb-cpu/src/quantize/dequant.rs:340-351)
__device__ __forceinline__ void scale_min_k4(int j, const uint8_t *q, int *sc, int *mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 0x0f) | ((q[j - 4] >> 6) << 4);
        *mn = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

// Q4_K {f16 d, f16 dmin, u8 scales[12], u8 qs[128]}; Q5_K {f16 d, f16 dmin, u8 scales[12], u8 qh[32], u8 ql[128]}: group g
// (64 elements) = low nibbles of its 32 bytes, then their high nibbles; Q5_K's fifth bit of byte l: bit 2 g (low
// half) or 2 g + 1 (high half) of qh[l]
template <bool kFifth>
struct DqQ45K {
    static constexpr uint32_t kElems = 256, kBytes = kFifth ? kQ5KBytes : kQ4KBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int g = o >> 3, half = (o >> 2) & 1, l0 = (o & 3) * 8;
        int sc, mn;
        scale_min_k4(2 * g + half, blk + 4, &sc, &mn);
        const float d1 = ld_f16(blk) * static_cast<float>(sc);
        const float m1 = ld_f16(blk + 2) * static_cast<float>(mn);
        const uint8_t *ql = blk + (kFifth ? 48 : 16), *qh = blk + 16;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int l = l0 + i;
            const uint8_t byte = ql[32 * g + l];
            int v = half ? (byte >> 4) : (byte & 0x0f);
            if constexpr (kFifth) v += (qh[l] & (1u << (2 * g + half))) ? 16 : 0;
            y[i] = d1 * static_cast<float>(v) - m1;
        }
    }
};

// {u8 ql[128], u8 qh[64], i8 scales[16], f16 d}: element 128 n + 32 k + l: nibble (k >= 2: high) of ql[64 n + l + 32 (k & 1)],
// bits 2 k of qh[32 n + l], scale 8 n + l / 16 + 2 k; d * scale * (q - 32), left to right
struct DqQ6K {
    static constexpr uint32_t kElems = 256, kBytes = kQ6KBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int idx = 8 * o, n = idx >> 7, rem = idx & 127, k = rem >> 5, l0 = rem & 31;
        const float d = ld_f16(blk + 208);
        const float sc = static_cast<float>(static_cast<int8_t>(blk[192 + 8 * n + (l0 >> 4) + 2 * k]));
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int l = l0 + i;
            const uint8_t lb = blk[64 * n + l + 32 * (k & 1)];
            const int nib = k >= 2 ? (lb >> 4) : (lb & 0x0f);
            const int q = nib | (((blk[128 + 32 * n + l] >> (2 * k)) & 3) << 4);
            y[i] = d * sc * static_cast<float>(q - 32);
        }
    }
};

}  // namespace

bool embed_gather_supported(uint32_t quant) {
    switch (quant) {
    case kF32: case kF16: case kBF16: case kQ4_0: case kQ4_1: case kQ5_0: case kQ5_1: case kQ8_0: case kQ8_1:
    case kQ2K: case kQ3K: case kQ4K: case kQ5K: case kQ6K:
        return true;
    default: return is_iq_quant(quant);
    }
}

void launch_embed_gather(uint32_t quant, const uint8_t *w, size_t row_bytes, const uint32_t *ids, uint32_t n_tokens,
                         uint32_t cols, float *out, hipStream_t stream) {
    if (n_tokens == 0 || cols == 0) return;
    switch (quant) {
    case kF32: launch_embed_gather_format<DqF32>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kF16: launch_embed_gather_format<DqF16>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kBF16: launch_embed_gather_format<DqBF16>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ4_0: launch_embed_gather_format<DqQ4_0>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ4_1: launch_embed_gather_format<DqQ4_1>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ5_0: launch_embed_gather_format<DqQ5_0>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ5_1: launch_embed_gather_format<DqQ5_1>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ8_0: launch_embed_gather_format<DqQ8_0>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ8_1: launch_embed_gather_format<DqQ8_1>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ2K: launch_embed_gather_format<DqQ2K>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ3K: launch_embed_gather_format<DqQ3K>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ4K: launch_embed_gather_format<DqQ45K<false>>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ5K: launch_embed_gather_format<DqQ45K<true>>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kQ6K: launch_embed_gather_format<DqQ6K>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    default: launch_embed_gather_iq(quant, w, row_bytes, ids, n_tokens, cols, out, stream); break;
    }
}

}  // namespace rnb
