// Prefill GEMM: Q4_K weights [rows][nb] x Q8_K activations [seq][nb] -> f32 out[seq][rows] on the
// int8 matrix cores (v_mfma_i32_32x32x32_i8).
//
// Arithmetic: the exact-integer block form of crates/rnb-cpu/src/gemm/tile_q4k.rs:1749-1800
// (q4k_q8k_exact_ref) / crates/rnb-cpu/src/gemm/neon_dot.rs:884-916:
//   out[s][r] = sum_b d_x[s][b] * (d[r][b] * sum_sb sc[r][b][sb] * P_sb  -  dmin[r][b] * sum_sb mn[r][b][sb] * bsum32[s][b][sb])
// with P_sb = sum_{k<32} nibble[r][b][32sb+k] * q[s][b][32sb+k].  One MFMA has K = 32 = one
// sub-block, so each MFMA result takes exactly one 6-bit scale.  Output layout out[s*rows + r]
// (crates/rnb-cpu/src/gemm/quant_gemv.rs:1185-1196).
//
// Tile mapping: the MFMA "M" index is the token, "N" is the weight row, so a lane's 16 results
// all belong to ONE weight row (lane % 32) and its scales are per-lane scalars.  Both operands
// take their 16 K-bytes per lane from the same K positions (16 * (lane / 32) + j), so the
// contraction is independent of how the hardware orders K inside the instruction.
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTile = 32;          // tokens and rows per wave tile
constexpr int kWavesPerWg = 4;     // 4 token tiles per workgroup share one row tile

__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemm_q4k_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                         const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                         uint32_t seq) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const uint32_t row0 = blockIdx.x * kTile;
    const uint32_t tok0 = (blockIdx.y * kWavesPerWg + wave) * kTile;
    if (tok0 >= seq) return;  // uniform per wave

    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t row = min(row0 + lrow, rows - 1);        // clamped loads, masked stores
    const uint32_t tok_a = min(tok0 + lrow, seq - 1);       // token whose bytes this lane feeds to the MFMA
    const uint8_t *rowp = w + static_cast<size_t>(row) * nb * kQ4KBytes;
    const int8_t *arow = aq + static_cast<size_t>(tok_a) * nb * 256 + 16 * khalf;

    // tokens of this lane's 16 results: i(r) = 8*(r/4) + 4*(lane/32) + (r%4)
    uint32_t tok_r[16];
#pragma unroll
    for (int r = 0; r < 16; r++) tok_r[r] = min(tok0 + 8 * (r >> 2) + 4 * khalf + (r & 3), seq - 1);

    float accf[16];
#pragma unroll
    for (int r = 0; r < 16; r++) accf[r] = 0.0f;

    for (uint32_t b = 0; b < nb; b++) {
        const uint8_t *blk = rowp + static_cast<size_t>(b) * kQ4KBytes;
        const uint4 hdr = *reinterpret_cast<const uint4 *>(blk);
        const float d = f16_bits_to_f32(hdr.x), dmin = f16_bits_to_f32(hdr.x >> 16);
        const Q4KScales s = unpack_q4k_scales(hdr.y, hdr.z, hdr.w);

        int acci[16];
#pragma unroll
        for (int r = 0; r < 16; r++) acci[r] = 0;

#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint4 q = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * g + 16 * khalf);
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int sb = 2 * g + h;
                v4i bw;
                bw.x = static_cast<int>((q.x >> (4 * h)) & 0x0f0f0f0fu);
                bw.y = static_cast<int>((q.y >> (4 * h)) & 0x0f0f0f0fu);
                bw.z = static_cast<int>((q.z >> (4 * h)) & 0x0f0f0f0fu);
                bw.w = static_cast<int>((q.w >> (4 * h)) & 0x0f0f0f0fu);
                const v4i av = *reinterpret_cast<const v4i *>(arow + static_cast<size_t>(b) * 256 + 32 * sb);
                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                const v16i p = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, bw, zero, 0, 0, 0);
                const int sc = byte_of(s.sc_lo, s.sc_hi, sb);
#pragma unroll
                for (int r = 0; r < 16; r++) acci[r] += sc * p[r];
            }
        }

#pragma unroll
        for (int r = 0; r < 16; r++) {
            const size_t ab = static_cast<size_t>(tok_r[r]) * nb + b;
            const uint4 bs0 = *reinterpret_cast<const uint4 *>(abs + ab * 16);
            const uint4 bs1 = *reinterpret_cast<const uint4 *>(abs + ab * 16 + 8);
            const uint32_t pairs[8] = {bs0.x, bs0.y, bs0.z, bs0.w, bs1.x, bs1.y, bs1.z, bs1.w};
            int summ = 0;
#pragma unroll
            for (int sb = 0; sb < 8; sb++) {
                const int bsum32 =
                    static_cast<int>(static_cast<int16_t>(pairs[sb] & 0xffffu)) + (static_cast<int>(pairs[sb]) >> 16);
                summ += byte_of(s.mn_lo, s.mn_hi, sb) * bsum32;
            }
            accf[r] += ad[ab] * (d * static_cast<float>(acci[r]) - dmin * static_cast<float>(summ));
        }
    }

    if (row0 + lrow < rows) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t tok = tok0 + 8 * (r >> 2) + 4 * khalf + (r & 3);
            if (tok < seq) out[static_cast<size_t>(tok) * rows + row0 + lrow] = accf[r];
        }
    }
}

}  // namespace

void launch_gemm_q4k_mfma(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                          hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    const dim3 grid((rows + kTile - 1) / kTile, (seq + kTile * kWavesPerWg - 1) / (kTile * kWavesPerWg), 1);
    hipLaunchKernelGGL(gemm_q4k_mfma_kernel, grid, dim3(kWave * kWavesPerWg), 0, stream, w, act.qs, act.d, act.bsums,
                       out, rows, nb, seq);
}

}  // namespace rnb
