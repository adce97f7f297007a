// Prefill GEMM: Q4_K weights [rows][nb] x Q8_K activations [seq][nb] -> f32 out[seq][rows] on the
// int8 matrix cores (v_mfma_i32_32x32x32_i8, 32 K-values = one Q4_K sub-block per instruction).
//
// Arithmetic: the exact-integer block form of crates/rnb-cpu/src/gemm/tile_q4k.rs:1749-1800
// (q4k_q8k_exact_ref) / crates/rnb-cpu/src/gemm/neon_dot.rs:884-916, per super-block b:
//   I = sum_sb sc[r][sb] * sum_k nib[r][32sb+k] * q[s][32sb+k]        (exact int32)
//   S = sum_sb mn[r][sb] * bsum32[s][sb]                              (exact int32)
//   out[s][r] += d_x[s][b] * (d[r][b] * float(I) - dmin[r][b] * float(S))
// Output layout out[s*rows + r] (crates/rnb-cpu/src/gemm/quant_gemv.rs:1185-1196).
//
// How the 6-bit sub-block scale gets onto an int8 MFMA without a per-sub-block pass over the
// accumulators: the scale is folded into the weight operand.  sc = lo + 8*hi with lo, hi in 0..7, so
// lo*nib and hi*nib (<= 105) are int8 values made from the packed nibbles with one packed 16-bit
// multiply per four weights; two MFMA chains accumulate I_lo and I_hi over the whole super-block and
// I = I_lo + 8*I_hi.  The mins term rides on the matrix cores as well: bsum32 = b0 + 64*b1 with int8
// digits, S = mn.b0 + 64 * mn.b1, two K=8 (zero-padded) MFMAs per super-block.
//
// Tiling: workgroup = 4 waves = 128 weight rows x 64 tokens; a wave owns 32 rows x 64 tokens (two
// 32x32 accumulator tiles).  The MFMA "M" index is the token and "N" the weight row, so a lane's 16
// results of a tile belong to ONE weight row (lane % 32): d, dmin and the scale digits are per-lane
// scalars.  Both operands are double-buffered in LDS, one super-block per stage: the packed 144-byte
// weight blocks of the 128 rows untouched and back to back, the token tile's int8 activations with a
// row stride of 272 B (128-bit reads of either are bank-conflict free).  The copy of the next stage is
// split in four and interleaved with the four 64-element groups of the current one, so only a few
// registers are ever in flight for it.  Both
// MFMA operands take their 16 K-bytes per lane from the same K positions (16*(lane/32) + j), so the
// contraction does not depend on how the hardware orders K inside the instruction.
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr int kWavesPerWg = 4;
constexpr int kThreads = kWave * kWavesPerWg;           // 256
constexpr int kRowsPerWave = 32;
constexpr int kRowsPerWg = kWavesPerWg * kRowsPerWave;  // 128
constexpr int kTokTiles = 2;                            // 32-token accumulator tiles per wave
constexpr int kToksPerWg = 32 * kTokTiles;              // 64
constexpr int kActStride = 272;                         // bytes per token row in LDS (256 + 16 pad)
constexpr int kStageActBytes = kToksPerWg * kActStride; // 17408
constexpr int kStageDxOff = kStageActBytes;             // f32 d_x[64]
constexpr int kStageDigOff = kStageDxOff + kToksPerWg * 4;    // 16 B per token: b0[8] | b1[8]
constexpr int kStageWOff = kStageDigOff + kToksPerWg * 16;    // packed weight blocks, 144 B per row
constexpr int kStageBytes = kStageWOff + kRowsPerWg * 144;    // 37120
constexpr int kActChunks = kToksPerWg * 16;             // 16-byte chunks of activations per stage (1024)
constexpr int kWChunks = kRowsPerWg * 9;                // 16-byte chunks of packed weights per stage (1152)
constexpr int kActCopies = kActChunks / kThreads;       // 4 per thread
constexpr int kWCopies = (kWChunks + kThreads - 1) / kThreads;  // 5 per thread (the last one half populated)

// four bytes (each <= 15) times a scalar <= 7 held in both 16-bit halves of `s2`: no carry between bytes
__device__ __forceinline__ int pk_scale(uint32_t nib4, uint32_t s2) {
    const u16x2 a = __builtin_bit_cast(u16x2, nib4), b = __builtin_bit_cast(u16x2, s2);
    return __builtin_bit_cast(int, static_cast<u16x2>(a * b));
}

__global__ void __launch_bounds__(kThreads, 2)
    gemm_q4k_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                         const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                         uint32_t seq) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t wg_row0 = blockIdx.x * kRowsPerWg;
    const uint32_t row0 = wg_row0 + wave * kRowsPerWave;
    const uint32_t tok0 = blockIdx.y * kToksPerWg;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;

    // ---- cooperative copy roles (loop invariant) ------------------------------------------------
    // activations: chunk c = i*256 + tid -> token c/16, column c%16: 16 consecutive lanes read 256 contiguous bytes
    const int8_t *act_base = aq + static_cast<size_t>(tok0) * nb * 256;  // workgroup-uniform bases, 32-bit lane offsets
    const uint8_t *w_base = w + static_cast<size_t>(wg_row0) * row_bytes;
    uint32_t act_src[kActCopies], act_dst[kActCopies];
#pragma unroll
    for (int i = 0; i < kActCopies; i++) {
        const uint32_t c = i * kThreads + tid;
        const uint32_t tok = min(tok0 + (c >> 4), seq - 1) - tok0;  // clamped loads, masked stores
        act_src[i] = tok * nb * 256 + (c & 15) * 16;
        act_dst[i] = (c >> 4) * kActStride + (c & 15) * 16;
    }
    // packed weights: chunk c -> row c/9, column c%9; LDS keeps the 144-byte blocks back to back
    uint32_t w_src[kWCopies];
#pragma unroll
    for (int i = 0; i < kWCopies; i++) {
        const uint32_t c = min(static_cast<uint32_t>(i * kThreads + tid), static_cast<uint32_t>(kWChunks - 1));
        const uint32_t r = (c * 7282u) >> 16;  // c / 9 for c < 1152
        const uint32_t row = min(wg_row0 + r, rows - 1) - wg_row0;
        w_src[i] = row * static_cast<uint32_t>(row_bytes) + (c - 9 * r) * 16;
    }
    const bool w_last_live = 4 * kThreads + tid < kWChunks;
    const uint32_t aux_tok = min(tok0 + (tid & 63), seq - 1);

    // One quarter (`part` in 0..3) of a stage: a 16-byte activation chunk and one or two 16-byte weight chunks
    // per thread.  Loads and LDS stores are separate steps so that a group of MFMAs runs between them.
    struct PartRegs {
        uint4 a, w0, w1;
    };
    auto part_load = [&](uint32_t b, int part) {
        PartRegs r;
        r.a = *reinterpret_cast<const uint4 *>(act_base + (act_src[part] + b * 256u));
        r.w0 = *reinterpret_cast<const uint4 *>(w_base + (w_src[part] + b * 144u));
        r.w1 = r.w0;  // only the last quarter carries a fifth weight chunk
        if (part == 3 && w_last_live) r.w1 = *reinterpret_cast<const uint4 *>(w_base + (w_src[4] + b * 144u));
        return r;
    };
    auto part_store = [&](const PartRegs &r, int buf, int part) {
        uint8_t *base = lds + buf * kStageBytes;
        *reinterpret_cast<uint4 *>(base + act_dst[part]) = r.a;
        *reinterpret_cast<uint4 *>(base + kStageWOff + (part * kThreads + tid) * 16) = r.w0;
        if (part == 3 && w_last_live) *reinterpret_cast<uint4 *>(base + kStageWOff + (4 * kThreads + tid) * 16) = r.w1;
    };
    // d_x (threads 0..63) and the 16 bsums (threads 64..127) of one token for super-block b
    struct AuxRegs {
        float dx;
        uint4 bs0, bs1;
    };
    auto aux_load = [&](uint32_t b) {
        AuxRegs r;
        r.dx = 0.0f;
        r.bs0 = r.bs1 = make_uint4(0, 0, 0, 0);
        if (tid < 64) {
            r.dx = ad[static_cast<size_t>(aux_tok) * nb + b];
        } else if (tid < 128) {
            const uint4 *bp = reinterpret_cast<const uint4 *>(abs + (static_cast<size_t>(aux_tok) * nb + b) * 16);
            r.bs0 = bp[0];
            r.bs1 = bp[1];
        }
        return r;
    };
    auto aux_store = [&](const AuxRegs &r, int buf) {
        uint8_t *base = lds + buf * kStageBytes;
        if (tid < 64) {
            reinterpret_cast<float *>(base + kStageDxOff)[tid] = r.dx;
        } else if (tid < 128) {
            // bsum32[k] = bsums[2k] + bsums[2k+1] = b0 + 64*b1, b0 in 0..63, b1 in -64..63
            const uint32_t pr[8] = {r.bs0.x, r.bs0.y, r.bs0.z, r.bs0.w, r.bs1.x, r.bs1.y, r.bs1.z, r.bs1.w};
            uint32_t dg[4] = {0, 0, 0, 0};  // b0[0..4) b0[4..8) b1[0..4) b1[4..8)
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const int bs = static_cast<int>(static_cast<int16_t>(pr[k] & 0xffffu)) + (static_cast<int>(pr[k]) >> 16);
                dg[k >> 2] |= static_cast<uint32_t>(bs & 63) << (8 * (k & 3));
                dg[2 + (k >> 2)] |= (static_cast<uint32_t>(bs >> 6) & 0xffu) << (8 * (k & 3));
            }
            reinterpret_cast<uint4 *>(base + kStageDigOff)[tid - 64] = make_uint4(dg[0], dg[1], dg[2], dg[3]);
        }
    };

    float accf[kTokTiles][16];
#pragma unroll
    for (int t = 0; t < kTokTiles; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) accf[t][r] = 0.0f;

#pragma unroll
    for (int part = 0; part < 4; part++) part_store(part_load(0, part), 0, part);
    aux_store(aux_load(0), 0);
    __syncthreads();

    for (uint32_t b = 0; b < nb; b++) {
        const int buf = b & 1;
        const bool has_next = b + 1 < nb;
        // prefetch for the next stage; on the last super-block the loads simply repeat this one and are dropped
        const uint32_t bn = has_next ? b + 1 : b;
        AuxRegs aux_next = aux_load(bn);
        PartRegs part_next = part_load(bn, 0);
        const uint8_t *sbase = lds + buf * kStageBytes;
        const uint8_t *wblk = sbase + kStageWOff + (wave * kRowsPerWave + lrow) * 144;
        const uint4 hdr = *reinterpret_cast<const uint4 *>(wblk);
        const float d = f16_bits_to_f32(hdr.x), dmin = f16_bits_to_f32(hdr.x >> 16);
        const Q4KScales sc = unpack_q4k_scales(hdr.y, hdr.z, hdr.w);

        const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        v16i acc_lo[kTokTiles], acc_hi[kTokTiles];
        // digits of the eight 6-bit scales, four per dword: sc = lo + 8*hi
        const uint32_t dlo[2] = {sc.sc_lo & 0x07070707u, sc.sc_hi & 0x07070707u};
        const uint32_t dhi[2] = {(sc.sc_lo >> 3) & 0x07070707u, (sc.sc_hi >> 3) & 0x07070707u};

#pragma unroll
        for (int g = 0; g < 4; g++) {
            if (g > 0) {  // the quarter loaded one group ago lands in LDS, the next one takes off
                if (has_next) part_store(part_next, buf ^ 1, g - 1);
                part_next = part_load(bn, g);
            }
            const uint4 q = *reinterpret_cast<const uint4 *>(wblk + 16 + 32 * g + 16 * khalf);
            const uint32_t qd[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int sb = 2 * g + h;
                // byte (sb & 3) of the digit dword replicated into both 16-bit halves (v_perm_b32, 0x0c = zero)
                const uint32_t sel = 0x0c000c00u | ((sb & 3) << 16) | (sb & 3);
                const uint32_t slo = __builtin_amdgcn_perm(0u, dlo[sb >> 2], sel);
                const uint32_t shi = __builtin_amdgcn_perm(0u, dhi[sb >> 2], sel);
                v4i wlo, whi;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t nib = (qd[i] >> (4 * h)) & 0x0f0f0f0fu;
                    wlo[i] = pk_scale(nib, slo);
                    whi[i] = pk_scale(nib, shi);
                }
#pragma unroll
                for (int t = 0; t < kTokTiles; t++) {
                    const v4i a = *reinterpret_cast<const v4i *>(sbase + (32 * t + lrow) * kActStride + 32 * sb + 16 * khalf);
                    acc_lo[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, wlo, sb == 0 ? zero16 : acc_lo[t], 0, 0, 0);
                    acc_hi[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, whi, sb == 0 ? zero16 : acc_hi[t], 0, 0, 0);
                }
            }
        }
        if (has_next) {
            part_store(part_next, buf ^ 1, 3);
            aux_store(aux_next, buf ^ 1);
        }

        // mins: K slots 0..7 of the lower K-half carry mn[0..8); everything else is zero
        v4i mnop = {0, 0, 0, 0};
        if (khalf == 0) {
            mnop[0] = static_cast<int>(sc.mn_lo);
            mnop[1] = static_cast<int>(sc.mn_hi);
        }
        const float neg_dmin = -dmin;
#pragma unroll
        for (int t = 0; t < kTokTiles; t++) {
            const uint4 dig = reinterpret_cast<const uint4 *>(sbase + kStageDigOff)[32 * t + lrow];
            const v4i op0 = {static_cast<int>(dig.x), static_cast<int>(dig.y), 0, 0};
            const v4i op1 = {static_cast<int>(dig.z), static_cast<int>(dig.w), 0, 0};
            const v16i s0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(op0, mnop, zero16, 0, 0, 0);
            const v16i s1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(op1, mnop, zero16, 0, 0, 0);
            // results r = 4*j + i of this lane belong to tokens 32t + 8j + 4*khalf + i
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 dx4 = reinterpret_cast<const float4 *>(sbase + kStageDxOff)[8 * t + 2 * j + khalf];
                const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = 4 * j + i;
                    const float fi = static_cast<float>(acc_lo[t][r] + 8 * acc_hi[t][r]);
                    const float fs = static_cast<float>(s0[r] + 64 * s1[r]);
                    // d*I - dmin*S and the accumulation use fused multiply-adds: same value as the reference
                    // formula up to one rounding per term
                    accf[t][r] = __builtin_fmaf(dx[i], __builtin_fmaf(neg_dmin, fs, d * fi), accf[t][r]);
                }
            }
        }
        __syncthreads();
    }

    if (row0 + lrow < rows) {
#pragma unroll
        for (int t = 0; t < kTokTiles; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t tok = tok0 + 32 * t + 8 * (r >> 2) + 4 * khalf + (r & 3);
                if (tok < seq) out[static_cast<size_t>(tok) * rows + row0 + lrow] = accf[t][r];
            }
    }
}

}  // namespace

void launch_gemm_q4k_mfma(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                          hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb == 0) return;
    static bool configured = false;
    if (!configured) {  // 2 stages x 37 KB exceed the default 64 KB dynamic LDS limit
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_mfma_kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kStageBytes);
        configured = true;
    }
    const dim3 grid((rows + kRowsPerWg - 1) / kRowsPerWg, (seq + kToksPerWg - 1) / kToksPerWg, 1);
    hipLaunchKernelGGL(gemm_q4k_mfma_kernel, grid, dim3(kThreads), 2 * kStageBytes, stream, w, act.qs, act.d, act.bsums,
                       out, rows, nb, seq);
}

}  // namespace rnb
