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
// Tiling: workgroup = 8 waves = 256 weight rows x 64 tokens; a wave owns 32 rows x 64 tokens (two
// 32x32 accumulator tiles).  The MFMA "M" index is the token and "N" the weight row, so a lane's 16
// results of a tile belong to ONE weight row (lane % 32): d, dmin and the scale digits are per-lane
// scalars.  Both MFMA operands take their 16 K-bytes per lane from the same K positions
// (16*(lane/32) + j), so the contraction does not depend on how the hardware orders K inside the
// instruction.
//
// Schedule: waves w and w+4 share a SIMD and run half a super-block apart.  While one is in its vector
// phase (float update of the previous super-block, LDS reads of the next one's packed weights) the
// other is in its matrix phase (scale the nibbles, 32 MFMAs fed from registers and LDS); a workgroup
// barrier swaps the roles.  All LDS fills are LDS-direct global loads issued two phases before their
// data is read, so no vector registers or VALU work go into the copies:
//   wbuf[2]  packed weight blocks of the 256 rows (144 B each, back to back)   read in the vector phase
//   abuf[2]  int8 activations of the 64 tokens (272 B stride: 128-bit reads
//            are bank-conflict free)                                            read in the matrix phase
//   aux[4]   the 64 activation scales d_x and 16 B of bsum digits per token     read one phase later
// Phase p (0-based) of group 0 handles super-block p/2; group 1 lags by one phase.
#include "device_utils.h"
#include "kernels.h"
#include <algorithm>

namespace rnb {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr int kActStride = 272;  // bytes per token row in LDS (256 + 16 pad): 128-bit reads are bank-conflict free

// four bytes (each <= 15) times a scalar <= 7 held in both 16-bit halves of `s2`: no carry between bytes
__device__ __forceinline__ int pk_scale(uint32_t nib4, uint32_t s2) {
    const u16x2 a = __builtin_bit_cast(u16x2, nib4), b = __builtin_bit_cast(u16x2, s2);
    return __builtin_bit_cast(int, static_cast<u16x2>(a * b));
}

constexpr int kPpWaves = 8;
constexpr int kPpThreads = kWave * kPpWaves;      // 512
constexpr int kPpRowsPerWg = kPpWaves * 32;       // 256
constexpr int kPpToks = 64;
constexpr int kPpWBuf = kPpRowsPerWg * 144;       // 36864
constexpr int kPpActBytes = kPpToks * kActStride; // 17408 = 17 x 1024
constexpr int kPpABuf = kPpActBytes;
constexpr int kPpWOff = 0;
constexpr int kPpAOff = 2 * kPpWBuf;
constexpr int kPpAuxOff = kPpAOff + 2 * kPpABuf;
constexpr int kPpAuxBytes = kPpToks * 4 + kPpToks * 16;  // d_x[64] then digits[64][16]
constexpr int kPpLdsBytes = kPpAuxOff + 4 * kPpAuxBytes;  // 113664
constexpr int kPpWInstr = kPpWBuf / 1024;         // 36 wave-wide 16-byte loads
constexpr int kPpAInstr = kPpActBytes / 1024;     // 17
constexpr int kPpWPerWave = (kPpWInstr + kPpWaves - 1) / kPpWaves;  // 5
constexpr int kPpAPerWave = (kPpAInstr + kPpWaves - 1) / kPpWaves;  // 3
constexpr uint32_t kMagicBits = 0x4B400000u;      // 1.5 * 2^23: int bits of 12582912.0f
constexpr float kMagic = 12582912.0f;

__global__ void __launch_bounds__(kPpThreads, 1)
    gemm_q4k_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                             const uint8_t *__restrict__ adig, float *__restrict__ out, uint32_t rows, uint32_t nb,
                             uint32_t seq, uint32_t nb_slice) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: what derives from it stays in SGPRs
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lptr_t)lds));
    const uint32_t wg_row0 = blockIdx.x * kPpRowsPerWg;
    const uint32_t row0 = wg_row0 + wave * 32;
    const uint32_t tok0 = blockIdx.y * kPpToks;
    const uint32_t row_bytes = nb * static_cast<uint32_t>(kQ4KBytes);
    const uint32_t last_row = rows - 1 - wg_row0, last_tok = seq - 1 - tok0;  // clamped loads, masked stores

    // ---- fill roles (loop invariant): workgroup-uniform bases, 32-bit lane offsets ----------------
    // K slice of this workgroup (blockIdx.z): nbs blocks from slice0 on, counted from 0 below (the bases move instead);
    // its sums go to the slice's own copy of the output
    const uint32_t slice0 = blockIdx.z * nb_slice, nbs = min(nb - slice0, nb_slice);
    out += static_cast<size_t>(blockIdx.z) * seq * rows;
    const uint8_t *w_base = w + static_cast<size_t>(wg_row0) * row_bytes + slice0 * 144u;
    const uint8_t *a_base = reinterpret_cast<const uint8_t *>(aq) + (static_cast<size_t>(tok0) * nb + slice0) * 256;
    const uint8_t *dig_base = adig + (static_cast<size_t>(tok0) * nb + slice0) * 16;
    const uint8_t *dx_base = reinterpret_cast<const uint8_t *>(ad) + (static_cast<size_t>(tok0) * nb + slice0) * 4;
    uint32_t w_off[kPpWPerWave], a_off[kPpAPerWave];
#pragma unroll
    for (int k = 0; k < kPpWPerWave; k++) {  // chunk c -> row c/9, 16-byte column c%9
        const uint32_t c = min((k * kPpWaves + wave) * 64 + lane, kPpWBuf / 16 - 1);
        const uint32_t r = c / 9u;
        w_off[k] = min(r, last_row) * row_bytes + (c - 9u * r) * 16u;
    }
#pragma unroll
    for (int k = 0; k < kPpAPerWave; k++) {  // chunk c -> token c/17, column c%17 (column 16 is the row padding)
        const uint32_t c = min((k * kPpWaves + wave) * 64 + lane, kPpActBytes / 16 - 1);
        const uint32_t t = c / 17u, col = c - 17u * t;
        a_off[k] = min(t, last_tok) * nb * 256u + (col & 15u) * 16u;
    }
    const uint32_t tok_lane = min(static_cast<uint32_t>(lane), last_tok);
    const uint32_t dig_off = tok_lane * nb * 16u, dx_off = tok_lane * nb * 4u;

    auto issue_w = [&](uint32_t b) {
        const uint32_t dst = lds0 + kPpWOff + (b & 1) * kPpWBuf;
        const uint8_t *src = w_base + b * 144u;
#pragma unroll
        for (int k = 0; k < kPpWPerWave; k++) {
            const int i = k * kPpWaves + wave;
            if (i < kPpWInstr) lds_fill16(src, w_off[k], dst + i * 1024);
        }
    };
    auto issue_a = [&](uint32_t b) {
        const uint32_t dst = lds0 + kPpAOff + (b & 1) * kPpABuf;
        const uint8_t *src = a_base + b * 256u;
#pragma unroll
        for (int k = 0; k < kPpAPerWave; k++) {
            const int i = k * kPpWaves + wave;
            if (i < kPpAInstr) lds_fill16(src, a_off[k], dst + i * 1024);
        }
        const uint32_t aux = lds0 + kPpAuxOff + (b & 3) * kPpAuxBytes;
        if (wave == 1) lds_fill16(dig_base + b * 16u, dig_off, aux + kPpToks * 4);
        if (wave == 2) lds_fill4(dx_base + b * 4u, dx_off, aux);
    };

    // ---- per-wave state carried between phases -------------------------------------------------
    float accf[2][16];
#pragma unroll
    for (int t = 0; t < 2; t++)
#pragma unroll
        for (int r = 0; r < 16; r++) accf[t][r] = 0.0f;
    v4i wlo[8], whi[8];          // scaled int8 weights of the current super-block, one operand per sub-block
    v4i mnop = {0, 0, 0, 0};     // mins, K slots 0..7 of the lower K-half
    v16i acc_lo[2], acc_hi[2];
    float d = 0.0f, neg_dmin = 0.0f, cm = 0.0f;

    // vector phase, part 2: unpack super-block b of this lane's row into MFMA operands
    auto prep = [&](uint32_t b) {
        const uint8_t *wblk = lds + kPpWOff + (b & 1) * kPpWBuf + (wave * 32 + lrow) * 144;
        const uint4 hdr = *reinterpret_cast<const uint4 *>(wblk);
        d = f16_bits_to_f32(hdr.x);
        const float dmin = f16_bits_to_f32(hdr.x >> 16);
        neg_dmin = -dmin;
        cm = dmin * kMagic;  // exact: 11-bit x 2-bit significands
        const Q4KScales sc = unpack_q4k_scales(hdr.y, hdr.z, hdr.w);
        const uint32_t dlo[2] = {sc.sc_lo & 0x07070707u, sc.sc_hi & 0x07070707u};
        const uint32_t dhi[2] = {(sc.sc_lo >> 3) & 0x07070707u, (sc.sc_hi >> 3) & 0x07070707u};
        mnop[0] = khalf == 0 ? static_cast<int>(sc.mn_lo) : 0;
        mnop[1] = khalf == 0 ? static_cast<int>(sc.mn_hi) : 0;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const uint4 q = *reinterpret_cast<const uint4 *>(wblk + 16 + 32 * g + 16 * khalf);
            const uint32_t qd[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int sb = 2 * g + h;
                const uint32_t sel = 0x0c000c00u | ((sb & 3) << 16) | (sb & 3);
                const uint32_t slo = __builtin_amdgcn_perm(0u, dlo[sb >> 2], sel);
                const uint32_t shi = __builtin_amdgcn_perm(0u, dhi[sb >> 2], sel);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const uint32_t nib = (qd[i] >> (4 * h)) & 0x0f0f0f0fu;
                    wlo[sb][i] = pk_scale(nib, slo);
                    whi[sb][i] = pk_scale(nib, shi);
                }
            }
        }
    };
    // matrix phase: I_lo, I_hi over the eight sub-blocks; the activation operands are read from LDS two
    // sub-blocks ahead of the MFMAs that take them
    auto matrix = [&](uint32_t b) {
        const uint8_t *abase = lds + kPpAOff + (b & 1) * kPpABuf + lrow * kActStride + 16 * khalf;
        const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        constexpr int kAhead = 2;
        v4i a[kAhead + 1][2];
#pragma unroll
        for (int sb = 0; sb < kAhead; sb++)
#pragma unroll
            for (int t = 0; t < 2; t++) a[sb][t] = *reinterpret_cast<const v4i *>(abase + 32 * t * kActStride + 32 * sb);
#pragma unroll
        for (int sb = 0; sb < 8; sb++) {
            if (sb + kAhead < 8) {
#pragma unroll
                for (int t = 0; t < 2; t++)
                    a[(sb + kAhead) % (kAhead + 1)][t] =
                        *reinterpret_cast<const v4i *>(abase + 32 * t * kActStride + 32 * (sb + kAhead));
            }
            // only vector/scalar ALU work may move across: the LDS reads above stay ahead of these MFMAs
            __builtin_amdgcn_sched_barrier(0x6);
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const v4i av = a[sb % (kAhead + 1)][t];
                acc_lo[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, wlo[sb], sb == 0 ? zero16 : acc_lo[t], 0, 0, 0);
                acc_hi[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, whi[sb], sb == 0 ? zero16 : acc_hi[t], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0x6);
        }
    };
    // vector phase, part 1: accf += d_x * (d * I - dmin * S) for the super-block whose I sums are in registers
    // (d, dmin and the mins operand still belong to it).  S = mn.b0 + 64 * mn.b1 takes two K=8 MFMAs per tile; the
    // second one starts from 64 * (first) + magic, so bits(acc_s) = magic + S read as a float and
    // fma(-dmin, that, dmin * magic) is -dmin * S rounded once.
    auto update = [&](uint32_t b) {
        const uint8_t *dxp = lds + kPpAuxOff + (b & 3) * kPpAuxBytes;
        const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        v16i acc_s[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            const uint4 dig = *reinterpret_cast<const uint4 *>(dxp + kPpToks * 4 + (32 * t + lrow) * 16);
            const v4i op0 = {static_cast<int>(dig.x), static_cast<int>(dig.y), 0, 0};
            const v4i op1 = {static_cast<int>(dig.z), static_cast<int>(dig.w), 0, 0};
            v16i c = __builtin_amdgcn_mfma_i32_32x32x32_i8(op1, mnop, zero16, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++) c[r] = static_cast<int>((static_cast<uint32_t>(c[r]) << 6) + kMagicBits);
            acc_s[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(op0, mnop, c, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 dx4 = reinterpret_cast<const float4 *>(dxp)[8 * t + 2 * j + khalf];
                const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = 4 * j + i;
                    const float fi = static_cast<float>(acc_lo[t][r] + 8 * acc_hi[t][r]);
                    const int s_bits = acc_s[t][r];  // a copy: bit-casting the vector element in place reads element 0
                    const float ws = __builtin_fmaf(neg_dmin, __int_as_float(s_bits), cm);
                    accf[t][r] = __builtin_fmaf(dx[i], __builtin_fmaf(d, fi, ws), accf[t][r]);
                }
            }
    };

    issue_w(0);
    issue_a(0);
    wait_fills();
    __builtin_amdgcn_s_barrier();

    if (wave < 4) {
        for (uint32_t b = 0; b < nbs; b++) {
            wait_fills();
            if (b + 1 < nbs) issue_w(b + 1);
            __builtin_amdgcn_s_setprio(1);  // the vector phase is the longer one: let it win issue slots
            if (b > 0) update(b - 1);
            prep(b);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_s_barrier();
            wait_fills();
            if (b + 1 < nbs) issue_a(b + 1);
            matrix(b);
            __builtin_amdgcn_s_barrier();
        }
    } else {
        wait_fills();
        if (1 < nbs) issue_w(1);
        __builtin_amdgcn_s_barrier();
        for (uint32_t b = 0; b < nbs; b++) {
            wait_fills();
            if (b + 1 < nbs) issue_a(b + 1);
            __builtin_amdgcn_s_setprio(1);  // the vector phase is the longer one: let it win issue slots
            if (b > 0) update(b - 1);
            prep(b);
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_s_barrier();
            wait_fills();
            if (b + 2 < nbs) issue_w(b + 2);
            matrix(b);
            if (b + 1 < nbs) __builtin_amdgcn_s_barrier();
        }
    }
    update(nbs - 1);

    if (row0 + lrow < rows) {
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t tok = tok0 + 32 * t + 8 * (r >> 2) + 4 * khalf + (r & 3);
                if (tok < seq) out[static_cast<size_t>(tok) * rows + row0 + lrow] = accf[t][r];
            }
    }
}

}  // namespace

// One workgroup fits a compute unit: up to 128 tiles the K range is cut so that the slices fill the 256 units once
// (a slice keeps at least 4 blocks); 4096 x 14336 x 512 tokens, 128 tiles: 125 -> 94 us
static uint32_t pp_slices(uint32_t rows, uint32_t nb, uint32_t seq) {
    const uint64_t tiles = static_cast<uint64_t>((rows + kPpRowsPerWg - 1) / kPpRowsPerWg) * ((seq + kPpToks - 1) / kPpToks);
    if (tiles == 0 || tiles > 128) return 1;
    const uint64_t s = std::min<uint64_t>(256 / tiles, nb / 4);
    return static_cast<uint32_t>(std::max<uint64_t>(1, s));
}

size_t gemm_q4k_slice_floats(uint32_t rows, uint32_t nb, uint32_t seq) {
    const uint32_t slices = pp_slices(rows, nb, seq);
    return slices > 1 ? static_cast<size_t>(slices) * seq * rows : 0;
}

void launch_gemm_q4k_mfma(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                          uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb == 0) return;
    static bool configured = false;  // 111 KB exceed the default 64 KB dynamic LDS limit
    if (!allow_dynamic_lds(reinterpret_cast<const void *>(gemm_q4k_mfma_kernel), kPpLdsBytes, &configured, "gemm_q4k_mfma_kernel"))
        return;
    const uint32_t slices = slice_out ? pp_slices(rows, nb, seq) : 1;
    const uint32_t nb_slice = (nb + slices - 1) / slices, nz = (nb + nb_slice - 1) / nb_slice;
    const dim3 grid((rows + kPpRowsPerWg - 1) / kPpRowsPerWg, (seq + kPpToks - 1) / kPpToks, nz);
    hipLaunchKernelGGL(gemm_q4k_mfma_kernel, grid, dim3(kPpThreads), kPpLdsBytes, stream, w, act.qs, act.d,
                       act.digits, nz > 1 ? slice_out : out, rows, nb, seq, nb_slice);
    if (nz > 1) launch_sum_slices(slice_out, out, static_cast<size_t>(seq) * rows, nz, stream);
}

}  // namespace rnb
