// Per-lane partial dot products of one GGUF super-block against one Q8_K activation block, shared by
// the decode GEMV and the gathered-MoE kernels.  FOUR lanes cooperate on a 256-element block (a wave64
// pass covers 16 blocks); the caller adds the partials across lanes.  Activations are held in
// registers (`Q4KAct` / `Q6KAct`) so that a wave which walks many rows loads them once.
// `KQuant<id>` at the end gives the kernels one interface over the K-quant formats.
#pragma once

#include "device_utils.h"
#include "kernels.h"

namespace rnb {

// ---------------------------------------------------------------------------------------------
// Q4_K: block = {f16 d, f16 dmin, u8 scales[12], u8 qs[128]}.  Lane g (0..3) of a block owns group g:
// qs[32g .. 32g+32) -> elements 64g + [0,32) in the low nibbles (scale 2g, min 2g) and
// 64g + 32 + [0,32) in the high nibbles (scale 2g+1, min 2g+1).
//   sumi = sc[2g]*dot(lo, a_lo) + sc[2g+1]*dot(hi, a_hi);  summ = mn[2g]*bsum32[2g] + mn[2g+1]*bsum32[2g+1]
//   partial = d_x * (d*sumi - dmin*summ)          crates/rnb-cpu/src/gemm/neon_dot.rs:884-916
// ---------------------------------------------------------------------------------------------
struct Q4KAct {
    uint4 lo0, lo1, hi0, hi1;  // 64 int8 activations of group g
    float dx;                  // Q8_K block scale
    int bs_lo, bs_hi;          // bsum32[2g], bsum32[2g+1]
};

__device__ __forceinline__ Q4KAct q4k_load_act(const int8_t *__restrict__ aq_blk, float dx,
                                               const int16_t *__restrict__ bs_blk, int g) {
    Q4KAct a;
    const int8_t *p = aq_blk + 64 * g;
    a.lo0 = *reinterpret_cast<const uint4 *>(p);
    a.lo1 = *reinterpret_cast<const uint4 *>(p + 16);
    a.hi0 = *reinterpret_cast<const uint4 *>(p + 32);
    a.hi1 = *reinterpret_cast<const uint4 *>(p + 48);
    a.dx = dx;
    const uint2 bp = *reinterpret_cast<const uint2 *>(bs_blk + 4 * g);  // bsums[4g .. 4g+4)
    a.bs_lo = static_cast<int>(static_cast<int16_t>(bp.x & 0xffffu)) + (static_cast<int>(bp.x) >> 16);
    a.bs_hi = static_cast<int>(static_cast<int16_t>(bp.y & 0xffffu)) + (static_cast<int>(bp.y) >> 16);
    return a;
}

struct Q4KRegs {
    uint4 h, qa, qb;  // 16-byte header, 32 bytes of packed nibbles
};

__device__ __forceinline__ Q4KRegs q4k_load_block(const uint8_t *__restrict__ blk, int g) {
    Q4KRegs r;
    r.h = *reinterpret_cast<const uint4 *>(blk);
    r.qa = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * g);
    r.qb = *reinterpret_cast<const uint4 *>(blk + 32 + 32 * g);
    return r;
}

// A block slice decoded once (nibbles split, scales and mins picked) so that it can be dotted with
// several tokens' activations: the batched MoE kernels keep a row in this form while walking tokens.
struct Q4KPrep {
    uint4 lo0, lo1, hi0, hi1;  // 32 low and 32 high nibbles, one per byte
    float d, dmin;
    int sc0, sc1, mn0, mn1;
};

__device__ __forceinline__ Q4KPrep q4k_prepare(const Q4KRegs &r, int g) {
    Q4KPrep p;
    p.d = f16_bits_to_f32(r.h.x);
    p.dmin = f16_bits_to_f32(r.h.x >> 16);
    const Q4KScales s = unpack_q4k_scales(r.h.y, r.h.z, r.h.w);
    const uint32_t scw = (g & 2) ? s.sc_hi : s.sc_lo, mnw = (g & 2) ? s.mn_hi : s.mn_lo;
    const int sh = (g & 1) * 16;
    p.sc0 = (scw >> sh) & 0xff;
    p.sc1 = (scw >> (sh + 8)) & 0xff;
    p.mn0 = (mnw >> sh) & 0xff;
    p.mn1 = (mnw >> (sh + 8)) & 0xff;
    p.lo0 = make_uint4(r.qa.x & 0x0f0f0f0fu, r.qa.y & 0x0f0f0f0fu, r.qa.z & 0x0f0f0f0fu, r.qa.w & 0x0f0f0f0fu);
    p.lo1 = make_uint4(r.qb.x & 0x0f0f0f0fu, r.qb.y & 0x0f0f0f0fu, r.qb.z & 0x0f0f0f0fu, r.qb.w & 0x0f0f0f0fu);
    p.hi0 = make_uint4((r.qa.x >> 4) & 0x0f0f0f0fu, (r.qa.y >> 4) & 0x0f0f0f0fu, (r.qa.z >> 4) & 0x0f0f0f0fu,
                       (r.qa.w >> 4) & 0x0f0f0f0fu);
    p.hi1 = make_uint4((r.qb.x >> 4) & 0x0f0f0f0fu, (r.qb.y >> 4) & 0x0f0f0f0fu, (r.qb.z >> 4) & 0x0f0f0f0fu,
                       (r.qb.w >> 4) & 0x0f0f0f0fu);
    return p;
}

__device__ __forceinline__ float q4k_dot(const Q4KPrep &p, const Q4KAct &a) {
    int i0 = 0, i1 = 0;
    i0 = dot4(p.lo0.x, a.lo0.x, i0);
    i0 = dot4(p.lo0.y, a.lo0.y, i0);
    i0 = dot4(p.lo0.z, a.lo0.z, i0);
    i0 = dot4(p.lo0.w, a.lo0.w, i0);
    i0 = dot4(p.lo1.x, a.lo1.x, i0);
    i0 = dot4(p.lo1.y, a.lo1.y, i0);
    i0 = dot4(p.lo1.z, a.lo1.z, i0);
    i0 = dot4(p.lo1.w, a.lo1.w, i0);
    i1 = dot4(p.hi0.x, a.hi0.x, i1);
    i1 = dot4(p.hi0.y, a.hi0.y, i1);
    i1 = dot4(p.hi0.z, a.hi0.z, i1);
    i1 = dot4(p.hi0.w, a.hi0.w, i1);
    i1 = dot4(p.hi1.x, a.hi1.x, i1);
    i1 = dot4(p.hi1.y, a.hi1.y, i1);
    i1 = dot4(p.hi1.z, a.hi1.z, i1);
    i1 = dot4(p.hi1.w, a.hi1.w, i1);
    // |i| <= 32 * 31 * 127 and |bsum32| <= 32 * 127 against 6-bit scales: every product fits 24 bits
    const int sumi = mul24(p.sc0, i0) + mul24(p.sc1, i1);
    const int summ = mul24(p.mn0, a.bs_lo) + mul24(p.mn1, a.bs_hi);
    return a.dx * (p.d * static_cast<float>(sumi) - p.dmin * static_cast<float>(summ));
}

__device__ __forceinline__ float q4k_partial(const Q4KRegs &r, const Q4KAct &a, int g) {
    return q4k_dot(q4k_prepare(r, g), a);
}

// ---------------------------------------------------------------------------------------------
// Q5_K: block = {f16 d, f16 dmin, u8 scales[12], u8 qh[32], u8 qs[128]}, 176 bytes.  Q4_K's element order
// with a fifth bit: element 64g + l takes bit 2g of qh[l], element 64g + 32 + l bit 2g+1.  Lane g reads the
// header, all of qh and its 32 bytes of qs; once the fifth bits are merged the values (0..31) sit one per
// byte exactly as a prepared Q4_K slice does, so the activation state and the dot are Q4_K's.
//                                                        crates/rnb-cpu/src/gemm/neon_dot.rs:1742-1800
// ---------------------------------------------------------------------------------------------
struct Q5KRegs {
    uint4 h, qh0, qh1, qa, qb;
};

__device__ __forceinline__ Q5KRegs q5k_load_block(const uint8_t *__restrict__ blk, int g) {
    Q5KRegs r;
    r.h = *reinterpret_cast<const uint4 *>(blk);
    r.qh0 = *reinterpret_cast<const uint4 *>(blk + 16);
    r.qh1 = *reinterpret_cast<const uint4 *>(blk + 32);
    r.qa = *reinterpret_cast<const uint4 *>(blk + 48 + 32 * g);
    r.qb = *reinterpret_cast<const uint4 *>(blk + 64 + 32 * g);
    return r;
}

__device__ __forceinline__ Q4KPrep q5k_prepare(const Q5KRegs &r, int g) {
    Q4KRegs r4;
    r4.h = r.h;
    r4.qa = r.qa;
    r4.qb = r.qb;
    Q4KPrep p = q4k_prepare(r4, g);
    const int s = 2 * g;  // bit s -> low-nibble half, bit s+1 -> high-nibble half; moved to bit 4 of each byte
#define RNB_Q5_BITS(dst_lo, dst_hi, src, k)                          \
    p.dst_lo.k |= ((r.src.k >> s) & 0x01010101u) << 4;               \
    p.dst_hi.k |= ((r.src.k >> (s + 1)) & 0x01010101u) << 4;
    RNB_Q5_BITS(lo0, hi0, qh0, x)
    RNB_Q5_BITS(lo0, hi0, qh0, y)
    RNB_Q5_BITS(lo0, hi0, qh0, z)
    RNB_Q5_BITS(lo0, hi0, qh0, w)
    RNB_Q5_BITS(lo1, hi1, qh1, x)
    RNB_Q5_BITS(lo1, hi1, qh1, y)
    RNB_Q5_BITS(lo1, hi1, qh1, z)
    RNB_Q5_BITS(lo1, hi1, qh1, w)
#undef RNB_Q5_BITS
    return p;
}

// ---------------------------------------------------------------------------------------------
// Q6_K: block = {u8 ql[128], u8 qh[64], i8 scales[16], f16 d}, 210 bytes, 2-byte aligned.
// Lane q (0..3) of a block owns half n = q>>1, l = 16*(q&1) .. +16: 16 bytes each of ql[64n+l],
// ql[64n+32+l], qh[32n+l] -> 64 six-bit values, 16 per activation quarter 128n + 32i + l (i = 0..3),
// scale index 8n + (q&1) + 2i.  (q6 - 32) is applied as dot(q6, a) - 32*sum(a); the activation sums
// are part of the held activation state.                 crates/rnb-cpu/src/gemm/neon_dot.rs:2240-2288
// ---------------------------------------------------------------------------------------------
struct Q6KAct {
    uint4 a0, a1, a2, a3;  // 16 int8 activations of each quarter
    int s0, s1, s2, s3;    // their sums
    float dx;
};

// The sum of the 16 activations starting at element 16*j is the Q8_K block's bsums[j]: quarter i of lane q starts
// at element 128n + 32i + 16(q&1), so its sum is bsums[8n + 2i + (q&1)].
__device__ __forceinline__ Q6KAct q6k_load_act(const int8_t *__restrict__ aq_blk, float dx,
                                               const int16_t *__restrict__ bs_blk, int q) {
    Q6KAct a;
    const int8_t *p = aq_blk + 128 * (q >> 1) + 16 * (q & 1);
    a.a0 = *reinterpret_cast<const uint4 *>(p);
    a.a1 = *reinterpret_cast<const uint4 *>(p + 32);
    a.a2 = *reinterpret_cast<const uint4 *>(p + 64);
    a.a3 = *reinterpret_cast<const uint4 *>(p + 96);
    const uint4 bs = *reinterpret_cast<const uint4 *>(bs_blk + 8 * (q >> 1));  // bsums[8n .. 8n+8)
    const int sh = 16 * (q & 1);                                               // even or odd entry of each pair
    a.s0 = static_cast<int>(bs.x << (16 - sh)) >> 16;
    a.s1 = static_cast<int>(bs.y << (16 - sh)) >> 16;
    a.s2 = static_cast<int>(bs.z << (16 - sh)) >> 16;
    a.s3 = static_cast<int>(bs.w << (16 - sh)) >> 16;
    a.dx = dx;
    return a;
}

// A lane's share of a block as loaded.  Every other 210-byte block starts 2 bytes off a 4-byte boundary, and 16-byte
// loads from such addresses are slow (forcing them onto 4-byte boundaries, wrong data: 4096 x 14336 11.3 -> 10.6 us,
// 14336 x 4096 11.2 -> 10.3, 128256 x 4096 71.6 -> 67.8).  So every piece is fetched from the boundary below it (m = 0 or
// 2 bytes early) and lacks its last m bytes, which are the first bytes of the piece that follows it in the block; that
// piece is in a register of a lane of the same quad (the four lanes of a block hold its twelve 16-byte pieces and the
// scales, in memory order A00 A01 B00 B01 A10 A11 B10 B11 H00 H01 H10 H11 S0 S1), and q6k_prepare puts the pieces right
// with six quad-permute moves, five selects and fourteen funnel shifts: no load more than before, and none waited for
// before the block is used.  The dword at byte 206 carries the scales' last two bytes and d.  (Fetching one dword more per
// piece instead, nine loads for five, was slower than the misaligned loads everywhere.)
struct Q6KRegs {
    uint4 A, B, H;  // as fetched: m bytes early
    uint2 S;
    uint32_t t;     // bytes 206..209 of the block
    uint32_t sh;    // 8 m: the funnel shift that puts the pieces right
};

// kEvenBase: the caller has checked that the matrix starts at an even address.  Without the odd-address path the four
// loads stay whole in the compiled code; with it the compiler merges the two paths into single-dword loads that it
// groups again later, not always as they were (a piece fetched as 1 + 3 dwords needs a register copy and a wait where
// a kernel assigns the register set).
template <bool kEvenBase = false>
__device__ __forceinline__ Q6KRegs q6k_load_block(const uint8_t *__restrict__ blk, int q) {
    Q6KRegs r;
    const int n = q >> 1, th = q & 1;
    uint32_t m = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(blk)) & 3u;
    if (!kEvenBase && (m & 1u)) {  // a matrix at an odd address (the same for every lane): the pieces themselves, whatever it costs
        r.A = ld_u4_a2(blk + 64 * n + 16 * th);
        r.B = ld_u4_a2(blk + 64 * n + 32 + 16 * th);
        r.H = ld_u4_a2(blk + 128 + 32 * n + 16 * th);
        r.S = ld_u2_a2(blk + 192 + 8 * n);
        m = 0;
    } else {
        const uint8_t *base = blk - m;
        r.A = *reinterpret_cast<const uint4_a4 *>(base + 64 * n + 16 * th);
        r.B = *reinterpret_cast<const uint4_a4 *>(base + 64 * n + 32 + 16 * th);
        r.H = *reinterpret_cast<const uint4_a4 *>(base + 128 + 32 * n + 16 * th);
        r.S = *reinterpret_cast<const uint2_a4 *>(base + 192 + 8 * n);
    }
    r.t = ld_u32_a2(blk + 206);
    r.sh = 8 * m;
    return r;
}

template <int kL0, int kL1, int kL2, int kL3>
__device__ __forceinline__ uint32_t quad_take(uint32_t v) {  // lane i of a quad reads lane kLi's v
    return static_cast<uint32_t>(
        __builtin_amdgcn_update_dpp(0, static_cast<int>(v), kL0 | (kL1 << 2) | (kL2 << 4) | (kL3 << 6), 0xf, 0xf, false));
}

__device__ __forceinline__ int sext8(uint32_t v, int shift) {
    return static_cast<int>(static_cast<int8_t>((v >> shift) & 0xffu));
}

struct Q6KPrep {
    uint4 u0, u1, u2, u3;  // 16 six-bit values (0..63) of each activation quarter, one per byte
    int s0, s1, s2, s3;    // their sub-block scales
    float d;
};

// All four lanes of a quad must be active (they exchange the pieces' first dwords).
__device__ __forceinline__ Q6KPrep q6k_prepare(const Q6KRegs &raw, int q) {
    Q6KPrep p;
    // the first dword of the piece after each of this lane's pieces, then the pieces moved into place
    const int n = q >> 1, th = q & 1;
    const uint32_t a1 = quad_take<1, 0, 3, 2>(raw.A.x), b1 = quad_take<1, 0, 3, 2>(raw.B.x);
    const uint32_t ar = quad_take<1, 2, 3, 0>(raw.A.x), hr = quad_take<1, 2, 3, 0>(raw.H.x), sr = quad_take<1, 2, 3, 0>(raw.S.x);
    const uint32_t s2 = quad_take<2, 3, 0, 1>(raw.S.x);
    const uint32_t after_a = th ? b1 : a1;
    const uint32_t after_b = th ? (n ? hr : ar) : b1;
    const uint32_t after_h = q == 3 ? sr : hr;
    const uint32_t after_s = n ? raw.t : s2;
    const uint32_t sh = raw.sh;
    struct {
        uint4 A, B, H;
        uint2 S;
    } r;
    r.A = make_uint4(__builtin_amdgcn_alignbit(raw.A.y, raw.A.x, sh), __builtin_amdgcn_alignbit(raw.A.z, raw.A.y, sh),
                     __builtin_amdgcn_alignbit(raw.A.w, raw.A.z, sh), __builtin_amdgcn_alignbit(after_a, raw.A.w, sh));
    r.B = make_uint4(__builtin_amdgcn_alignbit(raw.B.y, raw.B.x, sh), __builtin_amdgcn_alignbit(raw.B.z, raw.B.y, sh),
                     __builtin_amdgcn_alignbit(raw.B.w, raw.B.z, sh), __builtin_amdgcn_alignbit(after_b, raw.B.w, sh));
    r.H = make_uint4(__builtin_amdgcn_alignbit(raw.H.y, raw.H.x, sh), __builtin_amdgcn_alignbit(raw.H.z, raw.H.y, sh),
                     __builtin_amdgcn_alignbit(raw.H.w, raw.H.z, sh), __builtin_amdgcn_alignbit(after_h, raw.H.w, sh));
    r.S = make_uint2(__builtin_amdgcn_alignbit(raw.S.y, raw.S.x, sh), __builtin_amdgcn_alignbit(after_s, raw.S.y, sh));
    const int is = (q & 1) * 8;  // l / 16 selects scale byte 0 or 1 of each pair
    p.s0 = sext8(r.S.x, is);
    p.s1 = sext8(r.S.x, is + 16);
    p.s2 = sext8(r.S.y, is);
    p.s3 = sext8(r.S.y, is + 16);
    p.d = f16_bits_to_f32(raw.t >> 16);
#define RNB_Q6_UNPACK(k)                                                          \
    p.u0.k = (r.A.k & 0x0f0f0f0fu) | ((r.H.k & 0x03030303u) << 4);                \
    p.u1.k = (r.B.k & 0x0f0f0f0fu) | ((r.H.k & 0x0c0c0c0cu) << 2);                \
    p.u2.k = ((r.A.k >> 4) & 0x0f0f0f0fu) | (r.H.k & 0x30303030u);                \
    p.u3.k = ((r.B.k >> 4) & 0x0f0f0f0fu) | ((r.H.k & 0xc0c0c0c0u) >> 2);
    RNB_Q6_UNPACK(x)
    RNB_Q6_UNPACK(y)
    RNB_Q6_UNPACK(z)
    RNB_Q6_UNPACK(w)
#undef RNB_Q6_UNPACK
    return p;
}

__device__ __forceinline__ int dot16(const uint4 &u, const uint4 &a) {
    int s = 0;
    s = dot4(u.x, a.x, s);
    s = dot4(u.y, a.y, s);
    s = dot4(u.z, a.z, s);
    s = dot4(u.w, a.w, s);
    return s;
}

__device__ __forceinline__ float q6k_dot(const Q6KPrep &p, const Q6KAct &a) {
    const int p0 = dot16(p.u0, a.a0), p1 = dot16(p.u1, a.a1), p2 = dot16(p.u2, a.a2), p3 = dot16(p.u3, a.a3);
    // |p - 32 s| <= 16 * 63 * 127 + 32 * 16 * 127 against int8 scales: every product fits 24 bits
    const int sumi = mul24(p.s0, p0 - 32 * a.s0) + mul24(p.s1, p1 - 32 * a.s1) + mul24(p.s2, p2 - 32 * a.s2) +
                     mul24(p.s3, p3 - 32 * a.s3);
    return (p.d * a.dx) * static_cast<float>(sumi);
}

__device__ __forceinline__ float q6k_partial(const Q6KRegs &r, const Q6KAct &a, int q) {
    return q6k_dot(q6k_prepare(r, q), a);
}

// ---------------------------------------------------------------------------------------------
// Q2_K: block = {u8 scales[16] (scale | min << 4), u8 qs[64], f16 d, f16 dmin}, 84 bytes, 4-byte aligned.
// Q3_K: block = {u8 hmask[32], u8 qs[64], u8 scales[12], f16 d}, 110 bytes, 2-byte aligned.
// Both keep sixteen 16-element sub-blocks and lay qs out alike: byte 32n + l holds elements 128n + 32i + l in bit
// pair i.  Lane q owns half n = q>>1, l = 16*(q&1) .. +16, i.e. one 16-byte piece of qs and, as for Q6_K, the four
// activation quarters 128n + 32i + 16*(q&1) with sub-block index 8n + 2i + (q&1): activation state is Q6KAct.
//   Q2_K: sum_i sc_i * dot(u_i, a_i) and sum_i mn_i * bsums_i           crates/rnb-cpu/src/gemm/avx2_dot.rs:169-242
//   Q3_K: value = u - 4 + 4 * hbit (bit 4n + i of hmask[l]), signed scale = 6-bit code - 32; (u + 4 hbit - 4) is applied
//         as dot(u | hbit << 2, a) - 4 * sum(a)                          crates/rnb-cpu/src/gemm/avx2_dot.rs:247-375
// ---------------------------------------------------------------------------------------------
struct Q2KRegs {
    uint4 q;        // 16 bytes of packed 2-bit values
    uint2 s;        // scale bytes 8n .. 8n+8
    uint32_t dd;    // f16 d | f16 dmin << 16
};

__device__ __forceinline__ Q2KRegs q2k_load_block(const uint8_t *__restrict__ blk, int q) {
    Q2KRegs r;
    r.q = ld_u4_a2(blk + 16 + 32 * (q >> 1) + 16 * (q & 1));
    r.s = ld_u2_a2(blk + 8 * (q >> 1));
    r.dd = ld_u32_a2(blk + 80);
    return r;
}

struct Q2KPrep {
    uint4 u0, u1, u2, u3;  // 16 two-bit (Q3_K: three-bit) values of each activation quarter, one per byte
    int s0, s1, s2, s3;    // sub-block scales
    int m0, m1, m2, m3;    // sub-block mins (Q2_K only)
    float d, dmin;
};

__device__ __forceinline__ Q2KPrep q2k_prepare(const Q2KRegs &r, int q) {
    Q2KPrep p;
    const int sh = 8 * (q & 1);  // sub-block 8n + 2i + (q&1): byte (q&1) of each 16-bit pair
    const uint32_t b0 = (r.s.x >> sh) & 0xffu, b1 = (r.s.x >> (16 + sh)) & 0xffu;
    const uint32_t b2 = (r.s.y >> sh) & 0xffu, b3 = (r.s.y >> (16 + sh)) & 0xffu;
    p.s0 = b0 & 15; p.m0 = b0 >> 4;
    p.s1 = b1 & 15; p.m1 = b1 >> 4;
    p.s2 = b2 & 15; p.m2 = b2 >> 4;
    p.s3 = b3 & 15; p.m3 = b3 >> 4;
    p.d = f16_bits_to_f32(r.dd);
    p.dmin = f16_bits_to_f32(r.dd >> 16);
#define RNB_Q2_UNPACK(k)                      \
    p.u0.k = r.q.k & 0x03030303u;             \
    p.u1.k = (r.q.k >> 2) & 0x03030303u;      \
    p.u2.k = (r.q.k >> 4) & 0x03030303u;      \
    p.u3.k = (r.q.k >> 6) & 0x03030303u;
    RNB_Q2_UNPACK(x)
    RNB_Q2_UNPACK(y)
    RNB_Q2_UNPACK(z)
    RNB_Q2_UNPACK(w)
#undef RNB_Q2_UNPACK
    return p;
}

__device__ __forceinline__ float q2k_dot(const Q2KPrep &p, const Q6KAct &a) {
    const int sumi = mul24(p.s0, dot16(p.u0, a.a0)) + mul24(p.s1, dot16(p.u1, a.a1)) + mul24(p.s2, dot16(p.u2, a.a2)) +
                     mul24(p.s3, dot16(p.u3, a.a3));
    const int summ = mul24(p.m0, a.s0) + mul24(p.m1, a.s1) + mul24(p.m2, a.s2) + mul24(p.m3, a.s3);
    return (a.dx * p.d) * static_cast<float>(sumi) - (a.dx * p.dmin) * static_cast<float>(summ);
}

struct Q3KRegs {
    uint4 q, hm;       // 16 bytes of packed low bits, the 16 hmask bytes of the same l range
    uint2 s01;         // scale bytes 0..7 (low nibbles of codes 0..7, high nibbles of codes 8..15)
    uint32_t s2;       // scale bytes 8..11 (two high bits of every code)
    uint32_t d_bits;
};

__device__ __forceinline__ Q3KRegs q3k_load_block(const uint8_t *__restrict__ blk, int q) {
    Q3KRegs r;
    r.hm = ld_u4_a2(blk + 16 * (q & 1));
    r.q = ld_u4_a2(blk + 32 + 32 * (q >> 1) + 16 * (q & 1));
    r.s01 = ld_u2_a2(blk + 96);
    r.s2 = ld_u32_a2(blk + 104);
    r.d_bits = *reinterpret_cast<const unsigned short *>(blk + 108);
    return r;
}

// code k = 8n + 2i + h: low nibble from nibble n of byte k%8 = 2i + h, high bits from bit pair k/4 = 2n + i/2 of
// byte 8 + k%4 = 8 + 2(i%2) + h
__device__ __forceinline__ int q3k_code(const Q3KRegs &r, int n, int i, int h) {
    const uint32_t lo_word = (i < 2) ? r.s01.x : r.s01.y;
    const uint32_t lo = (lo_word >> (8 * (2 * (i & 1) + h) + 4 * n)) & 15u;
    const uint32_t hi = (r.s2 >> (8 * (2 * (i & 1) + h) + 2 * (2 * n + (i >> 1)))) & 3u;
    return static_cast<int>(lo | (hi << 4)) - 32;
}

__device__ __forceinline__ Q2KPrep q3k_prepare(const Q3KRegs &r, int q) {
    Q2KPrep p;
    const int n = q >> 1, h = q & 1;
    p.s0 = q3k_code(r, n, 0, h);
    p.s1 = q3k_code(r, n, 1, h);
    p.s2 = q3k_code(r, n, 2, h);
    p.s3 = q3k_code(r, n, 3, h);
    p.m0 = p.m1 = p.m2 = p.m3 = 0;
    p.d = f16_bits_to_f32(r.d_bits);
    p.dmin = 0.0f;
    const int hb = 4 * n;  // hmask bit of quarter i is 4n + i
#define RNB_Q3_UNPACK(k)                                                               \
    p.u0.k = (r.q.k & 0x03030303u) | (((r.hm.k >> hb) & 0x01010101u) << 2);            \
    p.u1.k = ((r.q.k >> 2) & 0x03030303u) | (((r.hm.k >> (hb + 1)) & 0x01010101u) << 2); \
    p.u2.k = ((r.q.k >> 4) & 0x03030303u) | (((r.hm.k >> (hb + 2)) & 0x01010101u) << 2); \
    p.u3.k = ((r.q.k >> 6) & 0x03030303u) | (((r.hm.k >> (hb + 3)) & 0x01010101u) << 2);
    RNB_Q3_UNPACK(x)
    RNB_Q3_UNPACK(y)
    RNB_Q3_UNPACK(z)
    RNB_Q3_UNPACK(w)
#undef RNB_Q3_UNPACK
    return p;
}

__device__ __forceinline__ float q3k_dot(const Q2KPrep &p, const Q6KAct &a) {
    const int sumi = mul24(p.s0, dot16(p.u0, a.a0) - 4 * a.s0) + mul24(p.s1, dot16(p.u1, a.a1) - 4 * a.s1) +
                     mul24(p.s2, dot16(p.u2, a.a2) - 4 * a.s2) + mul24(p.s3, dot16(p.u3, a.a3) - 4 * a.s3);
    return (a.dx * p.d) * static_cast<float>(sumi);
}

// ---------------------------------------------------------------------------------------------
// One interface over the K-quant formats for the kernels that are templated on the ggml type id.
// `bs_blk` points at the activation block's 16 int16 sums.
// ---------------------------------------------------------------------------------------------
template <uint32_t kQuant>
struct KQuant;

template <>
struct KQuant<kQ2K> {
    static constexpr size_t kBytes = kQ2KBytes;
    using Act = Q6KAct;
    using Regs = Q2KRegs;
    using Prep = Q2KPrep;
    static __device__ __forceinline__ Act load_act(const int8_t *aq_blk, float dx, const int16_t *bs_blk, int q) {
        return q6k_load_act(aq_blk, dx, bs_blk, q);
    }
    static __device__ __forceinline__ Regs load_block(const uint8_t *blk, int q) { return q2k_load_block(blk, q); }
    static __device__ __forceinline__ Regs load_block_even(const uint8_t *blk, int q) { return q2k_load_block(blk, q); }
    static __device__ __forceinline__ Prep prepare(const Regs &r, int q) { return q2k_prepare(r, q); }
    static __device__ __forceinline__ float dot(const Prep &p, const Act &a) { return q2k_dot(p, a); }
};

template <>
struct KQuant<kQ3K> {
    static constexpr size_t kBytes = kQ3KBytes;
    using Act = Q6KAct;
    using Regs = Q3KRegs;
    using Prep = Q2KPrep;
    static __device__ __forceinline__ Act load_act(const int8_t *aq_blk, float dx, const int16_t *bs_blk, int q) {
        return q6k_load_act(aq_blk, dx, bs_blk, q);
    }
    static __device__ __forceinline__ Regs load_block(const uint8_t *blk, int q) { return q3k_load_block(blk, q); }
    static __device__ __forceinline__ Regs load_block_even(const uint8_t *blk, int q) { return q3k_load_block(blk, q); }
    static __device__ __forceinline__ Prep prepare(const Regs &r, int q) { return q3k_prepare(r, q); }
    static __device__ __forceinline__ float dot(const Prep &p, const Act &a) { return q3k_dot(p, a); }
};

template <>
struct KQuant<kQ4K> {
    static constexpr size_t kBytes = kQ4KBytes;
    using Act = Q4KAct;
    using Regs = Q4KRegs;
    using Prep = Q4KPrep;
    static __device__ __forceinline__ Act load_act(const int8_t *aq_blk, float dx, const int16_t *bs_blk, int g) {
        return q4k_load_act(aq_blk, dx, bs_blk, g);
    }
    static __device__ __forceinline__ Regs load_block(const uint8_t *blk, int g) { return q4k_load_block(blk, g); }
    static __device__ __forceinline__ Regs load_block_even(const uint8_t *blk, int g) { return q4k_load_block(blk, g); }
    static __device__ __forceinline__ Prep prepare(const Regs &r, int g) { return q4k_prepare(r, g); }
    static __device__ __forceinline__ float dot(const Prep &p, const Act &a) { return q4k_dot(p, a); }
};

template <>
struct KQuant<kQ5K> {
    static constexpr size_t kBytes = kQ5KBytes;
    using Act = Q4KAct;
    using Regs = Q5KRegs;
    using Prep = Q4KPrep;
    static __device__ __forceinline__ Act load_act(const int8_t *aq_blk, float dx, const int16_t *bs_blk, int g) {
        return q4k_load_act(aq_blk, dx, bs_blk, g);
    }
    static __device__ __forceinline__ Regs load_block(const uint8_t *blk, int g) { return q5k_load_block(blk, g); }
    static __device__ __forceinline__ Regs load_block_even(const uint8_t *blk, int g) { return q5k_load_block(blk, g); }
    static __device__ __forceinline__ Prep prepare(const Regs &r, int g) { return q5k_prepare(r, g); }
    static __device__ __forceinline__ float dot(const Prep &p, const Act &a) { return q4k_dot(p, a); }
};

template <>
struct KQuant<kQ6K> {
    static constexpr size_t kBytes = kQ6KBytes;
    using Act = Q6KAct;
    using Regs = Q6KRegs;
    using Prep = Q6KPrep;
    static __device__ __forceinline__ Act load_act(const int8_t *aq_blk, float dx, const int16_t *bs_blk, int q) {
        return q6k_load_act(aq_blk, dx, bs_blk, q);
    }
    static __device__ __forceinline__ Regs load_block(const uint8_t *blk, int q) { return q6k_load_block(blk, q); }
    // for a matrix at an even address (checked on the host)
    static __device__ __forceinline__ Regs load_block_even(const uint8_t *blk, int q) { return q6k_load_block<true>(blk, q); }
    static __device__ __forceinline__ Prep prepare(const Regs &r, int q) { return q6k_prepare(r, q); }
    static __device__ __forceinline__ float dot(const Prep &p, const Act &a) { return q6k_dot(p, a); }
};

template <uint32_t kQuant>
__device__ __forceinline__ float kquant_partial(const typename KQuant<kQuant>::Regs &r,
                                                const typename KQuant<kQuant>::Act &a, int g) {
    return KQuant<kQuant>::dot(KQuant<kQuant>::prepare(r, g), a);
}

}  // namespace rnb
