// The GEMV's neighbours in a decode step that the reference's CUDA backend fuses around it:
//
//  RMS norm (+ residual add) -> Q8_K activation          crates/rnb-backend/cuda/cuda/kernels/quant_batch_and_ops.cuh:4031
//                                                         (rnb_rms_norm_f32) and :4275 (rnb_rms_norm_add_then_rms_norm_q8_1_f32;
//                                                         here the quantised form is rnb-cpu's Q8_K, not the CUDA backend's Q8_1)
//  router top-k + softmax over the selected logits        crates/rnb-llm/src/engine/models/shared_expert_moe/routing.rs:18-64
//
// Arithmetic of the norm is rnb-cpu's (crates/rnb-cpu/src/kernels/norm.rs:140-225): the mean square is accumulated in f64
// (rms_norm_into_f64, the default) and rms = f32(sqrt(mean + eps)); with the unit offset (scale = 1 + weight) in f32, as
// rms_norm_unit_offset_into_scalar does; out = (x / rms) * scale with one IEEE division and one multiplication.  The
// quantiser is the wave-level Q8_K routine of act_quant.h applied to those f32 values, so quantising the f32 output with
// rnb_hip_quantize_q8k gives the same bits.
#include "act_quant.h"
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

constexpr int kNormWaves = 4;
constexpr int kNormThreads = kWave * kNormWaves;

// sum over the workgroup, every thread gets the total; partial sums meet in wave order
template <typename T>
__device__ __forceinline__ T wg_sum(T v, T *s_part) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    const int wave = threadIdx.x >> 6;
    __syncthreads();  // s_part may still be read from an earlier call
    if ((threadIdx.x & 63) == 0) s_part[wave] = v;
    __syncthreads();
    T total = s_part[0];
#pragma unroll
    for (int w = 1; w < kNormWaves; w++) total += s_part[w];
    return total;
}

// rms of one row of `nb` 256-element blocks: wave w of the workgroup owns blocks w, w + 4, ..., lane l the elements
// 4l .. 4l+3 of a block
template <bool kUnit>
__device__ __forceinline__ float row_rms(const float *__restrict__ x, uint32_t nb, float eps, double *s_d, float *s_f) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float n = static_cast<float>(nb) * 256.0f;
    if constexpr (kUnit) {
        float acc = 0.0f;
        for (uint32_t b = wave; b < nb; b += kNormWaves) {
            const float4 v = reinterpret_cast<const float4 *>(x + static_cast<size_t>(b) * 256)[lane];
            acc += v.x * v.x;
            acc += v.y * v.y;
            acc += v.z * v.z;
            acc += v.w * v.w;
        }
        const float mean = wg_sum<float>(acc, s_f) / n;
        return sqrtf(mean + eps);
    } else {
        double acc = 0.0;
        for (uint32_t b = wave; b < nb; b += kNormWaves) {
            const float4 v = reinterpret_cast<const float4 *>(x + static_cast<size_t>(b) * 256)[lane];
            acc += static_cast<double>(v.x) * static_cast<double>(v.x);
            acc += static_cast<double>(v.y) * static_cast<double>(v.y);
            acc += static_cast<double>(v.z) * static_cast<double>(v.z);
            acc += static_cast<double>(v.w) * static_cast<double>(v.w);
        }
        const double mean = wg_sum<double>(acc, s_d) / static_cast<double>(n);
        return static_cast<float>(sqrt(mean + static_cast<double>(eps)));
    }
}

template <bool kUnit>
__device__ __forceinline__ float4 scale_of(const float *__restrict__ weight, uint32_t b, int lane) {
    float4 w = reinterpret_cast<const float4 *>(weight + static_cast<size_t>(b) * 256)[lane];
    if constexpr (kUnit) w = make_float4(1.0f + w.x, 1.0f + w.y, 1.0f + w.z, 1.0f + w.w);
    return w;
}

// One workgroup per token row.  kAdd: residual += norm(input, post_weight) first, then the row that is normalised with
// `weight` is the new residual; else it is `input`.  out_f32 and the Q8_K outputs are optional (null).
template <bool kAdd, bool kUnitPost, bool kUnit>
__global__ void __launch_bounds__(kNormThreads)
    rms_norm_kernel(const float *__restrict__ input, const float *__restrict__ post_weight, float post_eps,
                    float *__restrict__ residual, const float *__restrict__ weight, float eps, uint32_t nb,
                    float *__restrict__ out_f32, int8_t *__restrict__ qs, float *__restrict__ d_out,
                    int16_t *__restrict__ bsums, uint8_t *__restrict__ digits) {
    __shared__ double s_d[kNormWaves];
    __shared__ float s_f[kNormWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t row = blockIdx.x, hidden = static_cast<size_t>(nb) * 256;
    const float *x = input + row * hidden;
    if constexpr (kAdd) {
        float *res = residual + row * hidden;
        const float post_rms = row_rms<kUnitPost>(x, nb, post_eps, s_d, s_f);
        for (uint32_t b = wave; b < nb; b += kNormWaves) {
            const float4 v = reinterpret_cast<const float4 *>(x + static_cast<size_t>(b) * 256)[lane];
            const float4 w = scale_of<kUnitPost>(post_weight, b, lane);
            float4 r = reinterpret_cast<float4 *>(res + static_cast<size_t>(b) * 256)[lane];
            r.x += (v.x / post_rms) * w.x;
            r.y += (v.y / post_rms) * w.y;
            r.z += (v.z / post_rms) * w.z;
            r.w += (v.w / post_rms) * w.w;
            reinterpret_cast<float4 *>(res + static_cast<size_t>(b) * 256)[lane] = r;  // re-read below by the same thread
        }
        x = res;
    }
    const float rms = row_rms<kUnit>(x, nb, eps, s_d, s_f);
    for (uint32_t b = wave; b < nb; b += kNormWaves) {
        const float4 v = reinterpret_cast<const float4 *>(x + static_cast<size_t>(b) * 256)[lane];
        const float4 w = scale_of<kUnit>(weight, b, lane);
        const float4 o = make_float4((v.x / rms) * w.x, (v.y / rms) * w.y, (v.z / rms) * w.z, (v.w / rms) * w.w);
        if (out_f32 != nullptr) reinterpret_cast<float4 *>(out_f32 + row * hidden + static_cast<size_t>(b) * 256)[lane] = o;
        if (qs != nullptr) {
            const size_t blk = row * nb + b;
            q8k_quantize_vals(o, lane, qs + blk * 256, d_out + blk, bsums + blk * 16, digits != nullptr ? digits + blk * 16 : nullptr);
        }
    }
}

// One wave per token: every lane holds the logits e = lane, lane + 64, ... (at most kRouteMaxPerLane of them); `k`
// rounds of a wave-wide arg-max (larger value first, then the lower expert id) pick the experts in rank order, lane 0
// then forms the softmax over the selected logits in that order.
constexpr int kRouteMaxPerLane = 8;  // up to 512 experts
constexpr int kRouteMaxK = 32;

__global__ void __launch_bounds__(kWave)
    route_topk_kernel(const float *__restrict__ logits, uint32_t n_expert, uint32_t k, uint32_t *__restrict__ idx_out,
                      float *__restrict__ w_out) {
    const int lane = threadIdx.x;
    const size_t tok = blockIdx.x;
    const float *lg = logits + tok * n_expert;
    float v[kRouteMaxPerLane];
#pragma unroll
    for (int i = 0; i < kRouteMaxPerLane; i++) {
        const uint32_t e = lane + 64u * i;
        v[i] = e < n_expert ? lg[e] : -INFINITY;
    }
    uint32_t taken = 0;  // bit i: this lane's i-th logit has been selected
    const uint32_t sel = k < n_expert ? k : n_expert;
    float best_v[kRouteMaxK];
    uint32_t best_e[kRouteMaxK];
    for (uint32_t r = 0; r < sel; r++) {
        // this lane's best remaining candidate: larger value, then lower id (its ids grow with i)
        float cv = -INFINITY;
        uint32_t ce = 0xffffffffu;
#pragma unroll
        for (int i = 0; i < kRouteMaxPerLane; i++) {
            const uint32_t e = lane + 64u * i;
            const bool candidate = e < n_expert && !((taken >> i) & 1u) && !(v[i] != v[i]);  // a NaN is never selected
            if (candidate && (ce == 0xffffffffu || v[i] > cv)) {
                cv = v[i];
                ce = e;
            }
        }
        // wave-wide winner
        float wv = cv;
        uint32_t we = ce;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(wv, off, kWave);
            const uint32_t oe = __shfl_xor(we, off, kWave);
            const bool take = oe != 0xffffffffu && (we == 0xffffffffu || ov > wv || (ov == wv && oe < we));
            wv = take ? ov : wv;
            we = take ? oe : we;
        }
        best_v[r] = wv;
        best_e[r] = we;
        if (we != 0xffffffffu && (we & 63u) == static_cast<uint32_t>(lane)) taken |= 1u << (we >> 6);
    }
    if (lane == 0) {
        const float mx = best_v[0];
        float sum = 0.0f;
        float wts[kRouteMaxK];
        for (uint32_t r = 0; r < sel; r++) {
            wts[r] = expf(best_v[r] - mx);
            sum += wts[r];
        }
        for (uint32_t r = 0; r < sel; r++) {
            idx_out[tok * sel + r] = best_e[r];
            w_out[tok * sel + r] = sum != 0.0f ? wts[r] / sum : wts[r];
        }
    }
}

}  // namespace

void launch_rms_norm(const float *input, const float *post_weight, float post_eps, bool post_unit, float *residual,
                     const float *weight, float eps, bool unit, uint32_t seq, uint32_t nb, float *out_f32, int8_t *qs,
                     float *d, int16_t *bsums, uint8_t *digits, hipStream_t stream) {
    if (seq == 0 || nb == 0) return;
    const dim3 grid(seq), block(kNormThreads);
#define RNB_NORM(ADD, UP, U)                                                                                          \
    hipLaunchKernelGGL((rms_norm_kernel<ADD, UP, U>), grid, block, 0, stream, input, post_weight, post_eps, residual, \
                       weight, eps, nb, out_f32, qs, d, bsums, digits)
    if (residual == nullptr) {
        if (unit)
            RNB_NORM(false, false, true);
        else
            RNB_NORM(false, false, false);
    } else if (post_unit) {
        if (unit)
            RNB_NORM(true, true, true);
        else
            RNB_NORM(true, true, false);
    } else {
        if (unit)
            RNB_NORM(true, false, true);
        else
            RNB_NORM(true, false, false);
    }
#undef RNB_NORM
}

bool route_topk_supported(uint32_t n_expert, uint32_t k) {
    return n_expert >= 1 && n_expert <= 64u * kRouteMaxPerLane && k >= 1 && k <= kRouteMaxK;
}

void launch_route_topk(const float *logits, uint32_t tokens, uint32_t n_expert, uint32_t k, uint32_t *idx_out, float *w_out,
                       hipStream_t stream) {
    if (tokens == 0) return;
    hipLaunchKernelGGL(route_topk_kernel, dim3(tokens), dim3(kWave), 0, stream, logits, n_expert, k, idx_out, w_out);
}

}  // namespace rnb
