// Activation quantisation kernels (the wave-level quantisers live in act_quant.h).  One wave64 owns one 256-element span: each
// lane loads four consecutive floats with one 128-bit load, so a wave reads 1 KiB contiguously and
// writes 256 contiguous int8.  The library is compiled with -ffp-contract=off: every product is a
// single IEEE multiply, and `/` is hipcc's correctly rounded division sequence.
#include "act_quant.h"
#include "kernels.h"

namespace rnb {

namespace {

constexpr int kWavesPerWg = 4;

__global__ void __launch_bounds__(kWave *kWavesPerWg)
    quantize_q8k_kernel(const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ qs,
                        float *__restrict__ d_out, int16_t *__restrict__ bsums, uint8_t *__restrict__ digits) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t blk = static_cast<size_t>(blockIdx.x) * kWavesPerWg + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;  // wave-uniform
    q8k_quantize_span(x + blk * 256, lane, qs + blk * 256, d_out + blk, bsums + blk * 16,
                      digits != nullptr ? digits + blk * 16 : nullptr);
}

// The gated-FFN intermediate quantised as it is made: x = act(gate) * up element by element (SiLU or the tanh form of
// GELU, device_utils.h::act_mul), then quantize_q8k_kernel's routine; the f32 intermediate never travels through memory.
template <bool kGelu>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    quantize_q8k_gated_kernel(const float *__restrict__ gate, const float *__restrict__ up, size_t n_blocks,
                              int8_t *__restrict__ qs, float *__restrict__ d_out, int16_t *__restrict__ bsums,
                              uint8_t *__restrict__ digits) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t blk = static_cast<size_t>(blockIdx.x) * kWavesPerWg + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;  // wave-uniform
    const float4 g = reinterpret_cast<const float4 *>(gate + blk * 256)[lane];
    const float4 u = reinterpret_cast<const float4 *>(up + blk * 256)[lane];
    const float4 v = make_float4(act_mul<kGelu>(g.x, u.x), act_mul<kGelu>(g.y, u.y), act_mul<kGelu>(g.z, u.z),
                                 act_mul<kGelu>(g.w, u.w));
    q8k_quantize_vals(v, lane, qs + blk * 256, d_out + blk, bsums + blk * 16, digits != nullptr ? digits + blk * 16 : nullptr);
}

// Same as quantize_q8k_kernel with a copy job riding along: the workgroups past the quantiser's copy `n_words` words from
// `src`, which may be pinned host memory (the MoE routing tables of a batch: read over the bus by the kernel that runs
// anyway instead of a copy command with a launch and a gap of its own), to `dst` in device memory.
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    quantize_q8k_copy_kernel(const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ qs, float *__restrict__ d_out,
                             int16_t *__restrict__ bsums, uint8_t *__restrict__ digits, const uint32_t *__restrict__ src,
                             uint32_t n_words, uint32_t *__restrict__ dst, uint32_t quant_wgs) {
    if (blockIdx.x >= quant_wgs) {  // workgroup-uniform
        const uint32_t i = (blockIdx.x - quant_wgs) * (kWave * kWavesPerWg) + threadIdx.x;
        if (i < n_words) dst[i] = src[i];
        return;
    }
    const int lane = threadIdx.x & (kWave - 1);
    const size_t blk = static_cast<size_t>(blockIdx.x) * kWavesPerWg + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;  // wave-uniform
    q8k_quantize_span(x + blk * 256, lane, qs + blk * 256, d_out + blk, bsums + blk * 16,
                      digits != nullptr ? digits + blk * 16 : nullptr);
}

// Same as quantize_q8k_kernel; workgroup 0 additionally copies `n_words` routing-table words from the
// kernel argument to device memory (n_words <= 256 = one word per thread).
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    quantize_q8k_tables_kernel(const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ qs,
                               float *__restrict__ d_out, int16_t *__restrict__ bsums, const MoeInlineTables tables,
                               uint32_t n_words, uint32_t *__restrict__ tables_dev) {
    if (blockIdx.x == 0 && threadIdx.x < n_words) tables_dev[threadIdx.x] = tables.words[threadIdx.x];
    const int lane = threadIdx.x & (kWave - 1);
    const size_t blk = static_cast<size_t>(blockIdx.x) * kWavesPerWg + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;  // wave-uniform
    q8k_quantize_span(x + blk * 256, lane, qs + blk * 256, d_out + blk, bsums + blk * 16);
}

__global__ void __launch_bounds__(kWave *kWavesPerWg)
    quantize_q8_kernel(const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ qs,
                       float *__restrict__ d_out) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t span = static_cast<size_t>(blockIdx.x) * kWavesPerWg + (threadIdx.x >> 6);
    if (span * 8 >= n_blocks) return;  // wave-uniform
    const size_t left = n_blocks - span * 8;
    q8_quantize_span(x + span * 256, lane, left < 8 ? static_cast<int>(left) : 8, qs + span * 256, d_out + span * 8);
}

// arg-max with the reference's rule (larger value, ties to the lower index; a NaN never wins; the search starts from
// (-FLT_MAX, 0)): crates/rnb-backend/cuda/cuda/kernels/quant_batch_and_ops.cuh:3286-3328.  Stage 1 reduces `len`
// values to one candidate per workgroup, stage 2 (one workgroup, in = stage 1's candidates) to the result.
struct Best {
    float val;
    uint32_t idx;
};
__device__ __forceinline__ Best better(Best a, Best b) {
    return (b.val > a.val || (b.val == a.val && b.idx < a.idx)) ? b : a;
}
__global__ void __launch_bounds__(256)
    argmax_kernel(const float *__restrict__ values, const uint32_t *__restrict__ indices, uint32_t len,
                  float *__restrict__ out_values, uint32_t *__restrict__ out_indices) {
    __shared__ Best s_best[4];
    Best b{-3.4028234663852886e38f, 0u};
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < len; i += gridDim.x * blockDim.x)
        b = better(b, Best{values[i], indices != nullptr ? indices[i] : i});
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        Best o;
        o.val = __shfl_xor(b.val, off, kWave);
        o.idx = __shfl_xor(b.idx, off, kWave);
        b = better(b, o);
    }
    if ((threadIdx.x & (kWave - 1)) == 0) s_best[threadIdx.x >> 6] = b;
    __syncthreads();
    if (threadIdx.x == 0) {
        b = better(better(s_best[0], s_best[1]), better(s_best[2], s_best[3]));
        out_values[blockIdx.x] = b.val;
        out_indices[blockIdx.x] = b.idx;
    }
}

}  // namespace

void launch_argmax(const float *values, uint32_t len, float *scratch_values, uint32_t *scratch_indices, float *out_value,
                   uint32_t *out_index, hipStream_t stream) {
    const uint32_t blocks = len == 0 ? 1 : (len + 255) / 256 < 256 ? (len + 255) / 256 : 256;
    hipLaunchKernelGGL(argmax_kernel, dim3(blocks), dim3(256), 0, stream, values, nullptr, len, scratch_values,
                       scratch_indices);
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(256), 0, stream, scratch_values, scratch_indices, blocks, out_value,
                       out_index);
}

void launch_quantize_q8k(const float *x, size_t n_blocks, int8_t *qs, float *d, int16_t *bsums, uint8_t *digits,
                         hipStream_t stream) {
    if (n_blocks == 0) return;
    const unsigned grid = static_cast<unsigned>((n_blocks + kWavesPerWg - 1) / kWavesPerWg);
    hipLaunchKernelGGL(quantize_q8k_kernel, dim3(grid), dim3(kWave * kWavesPerWg), 0, stream, x, n_blocks, qs,
                       d, bsums, digits);
}

void launch_quantize_q8k_copy(const float *x, size_t n_blocks, int8_t *qs, float *d, int16_t *bsums, uint8_t *digits,
                              const uint32_t *words_src, uint32_t n_words, uint32_t *words_dst, hipStream_t stream) {
    const unsigned quant_wgs = static_cast<unsigned>((n_blocks + kWavesPerWg - 1) / kWavesPerWg);
    const unsigned copy_wgs = (n_words + kWave * kWavesPerWg - 1) / (kWave * kWavesPerWg);
    if (quant_wgs + copy_wgs == 0) return;
    hipLaunchKernelGGL(quantize_q8k_copy_kernel, dim3(quant_wgs + copy_wgs), dim3(kWave * kWavesPerWg), 0, stream, x, n_blocks,
                       qs, d, bsums, digits, words_src, n_words, words_dst, quant_wgs);
}

void launch_quantize_q8k_gated(const float *gate, const float *up, size_t n_blocks, bool gelu, int8_t *qs, float *d,
                               int16_t *bsums, uint8_t *digits, hipStream_t stream) {
    if (n_blocks == 0) return;
    const dim3 grid(static_cast<unsigned>((n_blocks + kWavesPerWg - 1) / kWavesPerWg)), block(kWave * kWavesPerWg);
    if (gelu)
        hipLaunchKernelGGL(quantize_q8k_gated_kernel<true>, grid, block, 0, stream, gate, up, n_blocks, qs, d, bsums, digits);
    else
        hipLaunchKernelGGL(quantize_q8k_gated_kernel<false>, grid, block, 0, stream, gate, up, n_blocks, qs, d, bsums, digits);
}

void launch_quantize_q8k_with_tables(const float *x, size_t n_blocks, int8_t *qs, float *d, int16_t *bsums,
                                     const MoeInlineTables &tables, uint32_t n_words, uint32_t *tables_dev,
                                     hipStream_t stream) {
    const unsigned grid = static_cast<unsigned>((n_blocks + kWavesPerWg - 1) / kWavesPerWg);
    hipLaunchKernelGGL(quantize_q8k_tables_kernel, dim3(grid ? grid : 1), dim3(kWave * kWavesPerWg), 0, stream, x,
                       n_blocks, qs, d, bsums, tables, n_words, tables_dev);
}

void launch_quantize_q8(const float *x, size_t n_blocks, int8_t *qs, float *d, hipStream_t stream) {
    if (n_blocks == 0) return;
    const size_t spans = (n_blocks + 7) / 8;
    const unsigned grid = static_cast<unsigned>((spans + kWavesPerWg - 1) / kWavesPerWg);
    hipLaunchKernelGGL(quantize_q8_kernel, dim3(grid), dim3(kWave * kWavesPerWg), 0, stream, x, n_blocks, qs, d);
}

}  // namespace rnb
