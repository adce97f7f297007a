// Activation quantisers, bit-exact with rnb-cpu.
//
//  Q8_K (256-wide): crates/rnb-cpu/src/gemm/activation_q8.rs:149-173 (quantize_q8k_block_ggml)
//  Q8   ( 32-wide): crates/rnb-cpu/src/gemm/activation_q8.rs:14-32   (quantize_input_q8)
//
// One wave64 owns one 256-element span: each lane loads four consecutive floats with one
// 128-bit load, so a wave reads 1 KiB contiguously and writes 256 contiguous int8.  The file is
// compiled with -ffp-contract=off: every product below is a single IEEE multiply, and `/` is
// hipcc's correctly rounded division sequence.
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

constexpr int kWavesPerWg = 4;

struct AbsMax {
    float amax;  // max |x|
    float val;   // the signed element that attained it first
    int idx;     // its index within the 256-span
};

// first occurrence wins: larger |x|, or equal |x| and smaller index
__device__ __forceinline__ AbsMax absmax_merge(AbsMax a, AbsMax b) {
    const bool take_b = (b.amax > a.amax) || (b.amax == a.amax && b.idx < a.idx);
    return take_b ? b : a;
}

__global__ void __launch_bounds__(kWave *kWavesPerWg)
    quantize_q8k_kernel(const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ qs,
                        float *__restrict__ d_out, int16_t *__restrict__ bsums) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t blk = static_cast<size_t>(blockIdx.x) * kWavesPerWg + (threadIdx.x >> 6);
    if (blk >= n_blocks) return;

    const float4 v = reinterpret_cast<const float4 *>(x + blk * 256)[lane];
    const float e[4] = {v.x, v.y, v.z, v.w};

    AbsMax m{0.0f, 0.0f, 4 * lane};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float ax = fabsf(e[i]);
        if (ax > m.amax) {  // strict: keeps the first of equal magnitudes
            m.amax = ax;
            m.val = e[i];
            m.idx = 4 * lane + i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        AbsMax o;
        o.amax = __shfl_xor(m.amax, off, kWave);
        o.val = __shfl_xor(m.val, off, kWave);
        o.idx = __shfl_xor(m.idx, off, kWave);
        m = absmax_merge(m, o);
    }

    float iscale = 0.0f, d = 0.0f;
    if (m.amax != 0.0f) {
        iscale = -127.0f / m.val;
        d = 1.0f / iscale;
    }

    int q[4];
    int part = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float prod = iscale * e[i];
        int r = __float2int_rn(prod);  // round half to even
        r = r > 127 ? 127 : r;         // upper clamp only
        q[i] = static_cast<int>(static_cast<int8_t>(r));
        part += q[i];
    }
    const uint32_t packed = (static_cast<uint32_t>(q[0]) & 0xffu) | ((static_cast<uint32_t>(q[1]) & 0xffu) << 8) |
                            ((static_cast<uint32_t>(q[2]) & 0xffu) << 16) |
                            ((static_cast<uint32_t>(q[3]) & 0xffu) << 24);
    reinterpret_cast<uint32_t *>(qs + blk * 256)[lane] = packed;

    const int sum16 = group_sum_i<4>(part);  // 4 lanes = 16 consecutive elements
    if ((lane & 3) == 0) bsums[blk * 16 + (lane >> 2)] = static_cast<int16_t>(sum16);
    if (lane == 0) d_out[blk] = d;
}

// A wave covers eight 32-element blocks; 8 lanes per block.
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    quantize_q8_kernel(const float *__restrict__ x, size_t n_blocks, int8_t *__restrict__ qs,
                       float *__restrict__ d_out) {
    const int lane = threadIdx.x & (kWave - 1);
    const size_t span = static_cast<size_t>(blockIdx.x) * kWavesPerWg + (threadIdx.x >> 6);
    const size_t blk = span * 8 + (lane >> 3);
    const bool live = blk < n_blocks;

    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (live) v = reinterpret_cast<const float4 *>(x + span * 256)[lane];
    const float e[4] = {v.x, v.y, v.z, v.w};
    float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
#pragma unroll
    for (int off = 4; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));

    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float prod = e[i] * id;
        float r = roundf(prod);  // half away from zero
        r = fminf(fmaxf(r, -128.0f), 127.0f);
        packed |= (static_cast<uint32_t>(static_cast<int>(r)) & 0xffu) << (8 * i);
    }
    if (live) {
        reinterpret_cast<uint32_t *>(qs + span * 256)[lane] = packed;
        if ((lane & 7) == 0) d_out[blk] = d;
    }
}

}  // namespace

void launch_quantize_q8k(const float *x, size_t n_blocks, int8_t *qs, float *d, int16_t *bsums,
                         hipStream_t stream) {
    if (n_blocks == 0) return;
    const unsigned grid = static_cast<unsigned>((n_blocks + kWavesPerWg - 1) / kWavesPerWg);
    hipLaunchKernelGGL(quantize_q8k_kernel, dim3(grid), dim3(kWave * kWavesPerWg), 0, stream, x, n_blocks, qs,
                       d, bsums);
}

void launch_quantize_q8(const float *x, size_t n_blocks, int8_t *qs, float *d, hipStream_t stream) {
    if (n_blocks == 0) return;
    const size_t spans = (n_blocks + 7) / 8;
    const unsigned grid = static_cast<unsigned>((spans + kWavesPerWg - 1) / kWavesPerWg);
    hipLaunchKernelGGL(quantize_q8_kernel, dim3(grid), dim3(kWave * kWavesPerWg), 0, stream, x, n_blocks, qs, d);
}

}  // namespace rnb
