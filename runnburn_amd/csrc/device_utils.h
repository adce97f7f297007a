// Device-side helpers shared by the gfx950 kernels: wave64 reductions, unaligned vector loads,
// fp16 decode and the Q4_K 6-bit scale/min unpack.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rnb {

constexpr int kWave = 64;

// GGUF blocks of 210 / 34 bytes are only 2-byte aligned inside a row.  gfx950 global loads
// accept any alignment (the queue runs in unaligned access mode); the reduced-alignment
// typedefs keep the compiler from assuming more than is true.
typedef uint4 __attribute__((aligned(2))) uint4_a2;
typedef uint2 __attribute__((aligned(2))) uint2_a2;
typedef uint32_t __attribute__((aligned(2))) uint32_a2;

// loads known to sit on a 4-byte boundary
typedef uint4 __attribute__((aligned(4))) uint4_a4;
typedef uint2 __attribute__((aligned(4))) uint2_a4;

__device__ __forceinline__ uint4 ld_u4_a2(const uint8_t *p) { return *reinterpret_cast<const uint4_a2 *>(p); }
__device__ __forceinline__ uint2 ld_u2_a2(const uint8_t *p) { return *reinterpret_cast<const uint2_a2 *>(p); }
__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t *p) { return *reinterpret_cast<const uint32_a2 *>(p); }

// A batch of `seq` tokens cut into groups of equal size, at most four tokens each (the multi-token GEMV kernels keep a
// group's activation slices in registers and make one pass over the matrix per group): 5 -> 3 + 2, 7 -> 4 + 3, 8 -> 4 + 4.
struct TokenGroups {
    uint32_t groups, per;
};
inline TokenGroups token_groups(uint32_t seq) {
    const uint32_t groups = (seq + 3) / 4;
    return {groups, groups ? (seq + groups - 1) / groups : 0};
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t bits) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(bits & 0xffffu)));
}
__device__ __forceinline__ float ld_f16(const uint8_t *p) {
    return f16_bits_to_f32(*reinterpret_cast<const unsigned short *>(p));
}

// a * b for operands known to fit 24 signed bits (block sums times 6- or 8-bit scales): one full-rate multiply
// where the 32-bit form takes a quarter-rate one
__device__ __forceinline__ int mul24(int a, int b) { return __mul24(a, b); }

__device__ __forceinline__ int dot4(uint32_t a, uint32_t b, int c) {
    return __builtin_amdgcn_sdot4(static_cast<int>(a), static_cast<int>(b), c, false);
}

typedef __attribute__((address_space(3))) void *lptr_t;

// LDS-direct global loads: 64 lanes x 16 B (or 4 B), lane i's bytes land at LDS byte address dst + 16*i (4*i); the
// source is a wave-uniform base plus a 32-bit lane offset.  Written as assembly so that the compiler does not make
// every later LDS read wait for them: callers order fills and reads themselves with waits on vmcnt and barriers.
// (m0 needs one wait state before the load reads it.)
__device__ __forceinline__ void lds_fill16(const uint8_t *base, uint32_t lane_off, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(lane_off), "s"(base) : "memory");
}
__device__ __forceinline__ void lds_fill4(const uint8_t *base, uint32_t lane_off, uint32_t dst) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(dst), "v"(lane_off), "s"(base) : "memory");
}
__device__ __forceinline__ void wait_fills() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// gate activation times up, as crates/rnb-cpu/src/kernels/activation.rs:73-98: SiLU g / (1 + exp(-g)) or the tanh form
// of GELU, 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3)))
template <bool kGelu>
__device__ __forceinline__ float act_mul(float g, float up) {
    if constexpr (kGelu) {
        const float inner = g + 0.044715f * (g * g * g);
        return (0.5f * g) * (1.0f + tanhf(0.7978845608028654f * inner)) * up;
    } else {
        const float e = expf(-g);
        return (g / (1.0f + e)) * up;
    }
}

// Cross-lane sums on the DPP data path (no LDS traffic).  After seg_sum<W>(v) the LAST lane of every
// aligned W-lane segment (W = 4, 8, 16, 32 or 64) holds the sum over that segment.  The steps of a narrower width are
// the first steps of a wider one, so a segment's sum has the bits of a wider sum whose other lanes hold zeros.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_add(float v) {
    const int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, kRowMask, 0xf, false);
    return v + __builtin_bit_cast(float, t);
}
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_max(float v) {  // for non-negative v (lanes left out of the row mask read 0)
    const int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), kCtrl, kRowMask, 0xf, false);
    return fmaxf(v, __builtin_bit_cast(float, t));
}
template <int kWidth>
__device__ __forceinline__ float seg_sum(float v) {
    static_assert(kWidth == 4 || kWidth == 8 || kWidth == 16 || kWidth == 32 || kWidth == 64, "segment width");
    v = dpp_add<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
    if (kWidth >= 8) v = dpp_add<0x141, 0xf>(v);   // row_half_mirror
    if (kWidth >= 16) v = dpp_add<0x140, 0xf>(v);  // row_mirror: all 16 lanes of a row hold the row sum
    if (kWidth >= 32) v = dpp_add<0x142, 0xa>(v);  // row_bcast15 into rows 1 and 3
    if (kWidth >= 64) v = dpp_add<0x143, 0xc>(v);  // row_bcast31 into rows 2 and 3
    return v;
}

// sum over the 64 lanes of a wave through the LDS crossbar; every lane gets the total
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

template <int width>
__device__ __forceinline__ int group_sum_i(int v) {
#pragma unroll
    for (int off = width / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// The 12 scale bytes of a Q4_K block as three dwords -> four dwords of packed 6-bit values:
// sc[0..3], sc[4..7], mn[0..3], mn[4..7] (one byte each).
struct Q4KScales {
    uint32_t sc_lo, sc_hi, mn_lo, mn_hi;
};
__device__ __forceinline__ Q4KScales unpack_q4k_scales(uint32_t u0, uint32_t u1, uint32_t u2) {
    Q4KScales s;
    s.sc_lo = u0 & 0x3f3f3f3fu;
    s.mn_lo = u1 & 0x3f3f3f3fu;
    s.sc_hi = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
    s.mn_hi = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
    return s;
}
// byte j (0..7) of an (lo, hi) pair of packed dwords
__device__ __forceinline__ int byte_of(uint32_t lo, uint32_t hi, int j) {
    const uint32_t wsel = (j & 4) ? hi : lo;
    return static_cast<int>((wsel >> ((j & 3) * 8)) & 0xffu);
}

// Expert `e` of one projection: routed experts lie back to back in `all` (base + e * bytes_per_expert, the slicing of
// crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs:4-22); ids from n_routed up name the shared
// expert, a tensor of its own (fanout.rs:804-812).
__device__ __forceinline__ const uint8_t *expert_base(const uint8_t *all, const uint8_t *shared, uint32_t n_routed, uint32_t e,
                                                      size_t bytes_per_expert) {
    return e < n_routed ? all + static_cast<size_t>(e) * bytes_per_expert : shared;
}

}  // namespace rnb
