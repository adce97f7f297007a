// Decode GEMV kernels: one packed GGUF row x one quantised activation vector -> one f32.
//
//  Q4_K x Q8_K : crates/rnb-cpu/src/gemm/neon_dot.rs:884-916   (dot_q4_k_q8k_scalar)
//  Q6_K x Q8_K : crates/rnb-cpu/src/gemm/neon_dot.rs:2240-2288 (dot_q6_k_q8k_scalar)
//  Q8_0 x Q8   : crates/rnb-cpu/src/gemm/neon_dot.rs:376-436   (dot_q8_0_q8_neon)
//  driver      : crates/rnb-cpu/src/gemm/quant_gemv.rs:403-536, out[s*rows + row]
//
// These kernels are HBM-bound: every weight byte is read exactly once, with 8- or 16-byte loads
// per lane that tile each row contiguously.  A wave64 owns a row; groups of 8 lanes own a
// 256-element super-block (1 lane owns a 32-element Q8_0 block).  Integer sums per lane are exact
// (v_dot4_i32_i8); the per-block f32 scale is applied once per lane and the 64 partial sums are
// added across the wave, so results differ from the scalar reference only by f32 summation order.
#include "block_dots.h"
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

constexpr int kRowsPerWg = 4;  // one wave per row

__global__ void __launch_bounds__(kWave *kRowsPerWg)
    gemv_q4k_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                    const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
    const uint32_t tok = blockIdx.y;
    if (row >= rows) return;
    const uint8_t *rowp = w + static_cast<size_t>(row) * nb * kQ4KBytes;
    const size_t abase = static_cast<size_t>(tok) * nb;
    const int c = lane & 7;
    float acc = 0.0f;
    for (uint32_t b = lane >> 3; b < nb; b += 8) {
        acc += q4k_block_partial(rowp + static_cast<size_t>(b) * kQ4KBytes, aq + (abase + b) * 256, ad[abase + b],
                                 abs + (abase + b) * 16, c);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[static_cast<size_t>(tok) * rows + row] = acc;
}

__global__ void __launch_bounds__(kWave *kRowsPerWg)
    gemv_q6k_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                    float *__restrict__ out, uint32_t rows, uint32_t nb) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
    const uint32_t tok = blockIdx.y;
    if (row >= rows) return;
    const uint8_t *rowp = w + static_cast<size_t>(row) * nb * kQ6KBytes;
    const size_t abase = static_cast<size_t>(tok) * nb;
    const int sub = lane & 7;
    float acc = 0.0f;
    for (uint32_t b = lane >> 3; b < nb; b += 8) {
        acc += q6k_block_partial(rowp + static_cast<size_t>(b) * kQ6KBytes, aq + (abase + b) * 256, ad[abase + b], sub);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[static_cast<size_t>(tok) * rows + row] = acc;
}

// ---------------------------------------------------------------------------------------------
// Q8_0: block = {f16 d, i8 qs[32]}, 34 bytes, 2-byte aligned.  One lane per block.
// ---------------------------------------------------------------------------------------------
__global__ void __launch_bounds__(kWave *kRowsPerWg)
    gemv_q8_0_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                     float *__restrict__ out, uint32_t rows, uint32_t nb32) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
    const uint32_t tok = blockIdx.y;
    if (row >= rows) return;
    const uint8_t *rowp = w + static_cast<size_t>(row) * nb32 * kQ8_0Bytes;
    const size_t abase = static_cast<size_t>(tok) * nb32;
    float acc = 0.0f;
    for (uint32_t b = lane; b < nb32; b += kWave) {
        const uint8_t *blk = rowp + static_cast<size_t>(b) * kQ8_0Bytes;
        const float d = ld_f16(blk);
        const uint4 q0 = ld_u4_a2(blk + 2), q1 = ld_u4_a2(blk + 18);
        const uint4 a0 = *reinterpret_cast<const uint4 *>(aq + (abase + b) * 32);
        const uint4 a1 = *reinterpret_cast<const uint4 *>(aq + (abase + b) * 32 + 16);
        int p = 0;
        p = dot4(q0.x, a0.x, p);
        p = dot4(q0.y, a0.y, p);
        p = dot4(q0.z, a0.z, p);
        p = dot4(q0.w, a0.w, p);
        p = dot4(q1.x, a1.x, p);
        p = dot4(q1.y, a1.y, p);
        p = dot4(q1.z, a1.z, p);
        p = dot4(q1.w, a1.w, p);
        acc += (d * ad[abase + b]) * static_cast<float>(p);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[static_cast<size_t>(tok) * rows + row] = acc;
}

inline dim3 gemv_grid(uint32_t rows, uint32_t seq) { return dim3((rows + kRowsPerWg - 1) / kRowsPerWg, seq, 1); }

}  // namespace

void launch_gemv_q4k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                     hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    hipLaunchKernelGGL(gemv_q4k_kernel, gemv_grid(rows, seq), dim3(kWave * kRowsPerWg), 0, stream, w, act.qs, act.d,
                       act.bsums, out, rows, nb);
}

void launch_gemv_q6k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                     hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    hipLaunchKernelGGL(gemv_q6k_kernel, gemv_grid(rows, seq), dim3(kWave * kRowsPerWg), 0, stream, w, act.qs, act.d,
                       out, rows, nb);
}

void launch_gemv_q8_0(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb32, uint32_t seq,
                      hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    hipLaunchKernelGGL(gemv_q8_0_kernel, gemv_grid(rows, seq), dim3(kWave * kRowsPerWg), 0, stream, w, act.qs, act.d,
                       out, rows, nb32);
}

}  // namespace rnb
