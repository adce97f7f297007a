// Pieces shared by the matrix-core kernels for the formats whose scale groups are applied on the vector units
// (gemm_blocks.hip: dense prefill GEMMs; moe_mfma.hip: the grouped expert GEMMs): how a lane that owns a weight row
// loads its share of a block, turns a scale group into an int8 MFMA operand, and how a workgroup stages its tokens'
// quantised activations in LDS.  Lane = (row lane % 32, K-half lane / 32).
#pragma once

#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kGbWaves = 4;
constexpr int kGbThreads = kWave * kGbWaves;
constexpr int kGbRows = 32 * kGbWaves;  // 128 rows per workgroup
constexpr int kGbStride64 = 264;   // bytes per staged token row for 64-bit operand reads (256 + 8): bank-conflict free
constexpr int kGbStride128 = 272;  // ... and for 128-bit operand reads (256 + 16, keeps them 16-byte aligned)

// ---------------------------------------------------------------------------------------------
// Q6_K: block = {ql[128], qh[64], i8 scales[16], f16 d}, 210 bytes, 2-byte aligned.  Element 128h + 32p + l
// (h = half, p = quarter, l < 32) = ((ql[64h + 32(p&1) + l] >> 4(p>>1)) & 15 | ((qh[32h + l] >> 2p) & 3) << 4) - 32, its
// 16-element sub-block is 8h + 2p + l/16.  The lane of K-half k takes l = 16(sb&1) + 8k .. +8 of every sub-block.
// ---------------------------------------------------------------------------------------------
struct Q6Half {
    uint2 ql[2][2];  // [p & 1][l / 16]
    uint2 qh[2];     // [l / 16]
};
struct Q6Row {
    Q6Half h[2];
    uint4 scales;
    float d;
};

__device__ __forceinline__ Q6Row q6_load_row(const uint8_t *__restrict__ blk, int khalf) {
    Q6Row r;
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int lh = 0; lh < 2; lh++) r.h[h].ql[a][lh] = ld_u2_a2(blk + 64 * h + 32 * a + 16 * lh + 8 * khalf);
#pragma unroll
        for (int lh = 0; lh < 2; lh++) r.h[h].qh[lh] = ld_u2_a2(blk + 128 + 32 * h + 16 * lh + 8 * khalf);
    }
    r.scales = ld_u4_a2(blk + 192);
    r.d = ld_f16(blk + 208);
    return r;
}

// four 6-bit values (low 4 bits in `nib`, high 2 bits already at bit 4 in `two`) minus 32, as signed bytes: the sum
// v + 0x60 never carries between bytes (v <= 63), and flipping bit 7 of v + 96 gives v - 32 modulo 256
__device__ __forceinline__ uint32_t q6_signed(uint32_t nib, uint32_t two) {
    return ((nib | two) + 0x60606060u) ^ 0x80808080u;
}

template <int kSb>
__device__ __forceinline__ long q6_operand(const Q6Row &r) {
    constexpr int h = kSb >> 3, p = (kSb >> 1) & 3, lh = kSb & 1;
    const uint2 ql = r.h[h].ql[p & 1][lh], qh = r.h[h].qh[lh];
    uint32_t n0, n1, t0, t1;
    if constexpr ((p >> 1) == 0) {
        n0 = ql.x & 0x0f0f0f0fu;
        n1 = ql.y & 0x0f0f0f0fu;
    } else {
        n0 = (ql.x >> 4) & 0x0f0f0f0fu;
        n1 = (ql.y >> 4) & 0x0f0f0f0fu;
    }
    if constexpr (p == 0) {
        t0 = (qh.x << 4) & 0x30303030u;
        t1 = (qh.y << 4) & 0x30303030u;
    } else if constexpr (p == 1) {
        t0 = (qh.x << 2) & 0x30303030u;
        t1 = (qh.y << 2) & 0x30303030u;
    } else if constexpr (p == 2) {
        t0 = qh.x & 0x30303030u;
        t1 = qh.y & 0x30303030u;
    } else {
        t0 = (qh.x >> 2) & 0x30303030u;
        t1 = (qh.y >> 2) & 0x30303030u;
    }
    const uint32_t lo = q6_signed(n0, t0), hi = q6_signed(n1, t1);
    return static_cast<long>(static_cast<unsigned long>(lo) | (static_cast<unsigned long>(hi) << 32));
}

template <int kSb>
__device__ __forceinline__ int q6_scale(const Q6Row &r) {
    const uint32_t word = kSb < 4 ? r.scales.x : (kSb < 8 ? r.scales.y : (kSb < 12 ? r.scales.z : r.scales.w));
    return static_cast<int>(__builtin_amdgcn_sbfe(static_cast<int>(word), 8 * (kSb & 3), 8));
}

// ---------------------------------------------------------------------------------------------
// Route of a wave's 32 weight rows from global memory to the lanes that own them.  A lane that reads its own row
// directly makes every load instruction touch 64 cache lines, and the vector cache, which looks up one line a cycle,
// becomes the limit long before the matrix cores.  Here consecutive lanes take consecutive 16-byte pieces of a row
// (kPieces per row step, so one instruction covers whole lines), the pieces go to a strip of LDS private to the wave
// with rows kStride bytes apart, and each lane reads its row back from there.  Only the wave itself touches the strip:
// LDS accesses of one wave execute in order, so no barrier is involved.
// ---------------------------------------------------------------------------------------------
template <int kPieces>
struct RowRoute {
    static constexpr int kN = (32 * kPieces + kWave - 1) / kWave;  // load instructions per row step
    uint32_t goff[kN];  // byte offset of this lane's piece from the wave's first row (rows past the end: the last row)
    uint32_t loff[kN];  // where it goes in the strip
    uint4 v[kN];
};

template <int kPieces, int kStride>
__device__ __forceinline__ void route_setup(RowRoute<kPieces> &rt, uint32_t rows_left, size_t row_bytes, int lane) {
#pragma unroll
    for (int i = 0; i < RowRoute<kPieces>::kN; i++) {
        const uint32_t c = min(static_cast<uint32_t>(lane) + i * kWave, 32u * kPieces - 1);
        const uint32_t r = c / kPieces, j = c - r * kPieces;
        rt.goff[i] = static_cast<uint32_t>(min(r, rows_left - 1) * row_bytes) + 16 * j;
        rt.loff[i] = r * kStride + 16 * j;
    }
}

template <int kPieces>
__device__ __forceinline__ void route_load(RowRoute<kPieces> &rt, const uint8_t *__restrict__ base) {
#pragma unroll
    for (int i = 0; i < RowRoute<kPieces>::kN; i++) rt.v[i] = ld_u4_a2(base + rt.goff[i]);
}

// 64-bit stores: the strip's row stride is a multiple of 8, not of 16, to keep the per-row reads off each other's banks
template <int kPieces>
__device__ __forceinline__ void route_store(const RowRoute<kPieces> &rt, uint8_t *strip, int lane) {
#pragma unroll
    for (int i = 0; i < RowRoute<kPieces>::kN; i++) {
        if ((i + 1) * kWave <= 32 * kPieces || lane + i * kWave < 32 * kPieces) {
            *reinterpret_cast<uint2 *>(strip + rt.loff[i]) = make_uint2(rt.v[i].x, rt.v[i].y);
            *reinterpret_cast<uint2 *>(strip + rt.loff[i] + 8) = make_uint2(rt.v[i].z, rt.v[i].w);
        }
    }
}

// 128-bit stores, for strips whose row stride is a multiple of 16
template <int kPieces>
__device__ __forceinline__ void route_store16(const RowRoute<kPieces> &rt, uint8_t *strip, int lane) {
#pragma unroll
    for (int i = 0; i < RowRoute<kPieces>::kN; i++) {
        if ((i + 1) * kWave <= 32 * kPieces || lane + i * kWave < 32 * kPieces)
            *reinterpret_cast<uint4 *>(strip + rt.loff[i]) = rt.v[i];
    }
}

constexpr int kQ6Pieces = 13;        // ql, qh and scales: 208 bytes; d is read by the row's lanes themselves
constexpr int kQ6StripStride = 216;  // 54 dwords: the 32 rows' 64-bit reads fall on 32 different bank pairs

// The same route for Q6_K rows whose blocks do not all start on a 4-byte boundary (rows of an odd number of blocks: every
// other row and every other block starts 2 bytes off), where the 16-byte loads of RowRoute take the address path about
// a fifth longer (128 experts x top-8 at 64 tokens, loads forced onto 4-byte boundaries: down kernel 51 -> 45 us).
// A piece is fetched from the boundary below it, and the two bytes it lacks come from the lane that holds the next
// piece (one DPP move inside a row of sixteen lanes); a fourteenth slot per row fetches the block's last 16 bytes for
// piece twelve.  Sixteen slots a row, four rows an instruction, eight instructions a block.  The instructions of a
// request are four rows apart and 4 * row_bytes is a multiple of 4, so one shift serves them all.  Needs rows and base
// at even addresses and whole 32-row tiles (no clamping of rows past the end).
struct Q6RouteDw {
    static constexpr int kN = 8;
    uint32_t goff[kN];  // byte offset of this lane's piece from the wave's first row, were the row's block aligned
    uint32_t loff;      // where the piece of instruction 0 goes in the strip; instruction i is four rows further
    uint32_t sh;        // funnel shift of the request in flight: 0 or 16 bits
    uint4 v[kN];
};
__device__ __forceinline__ void q6dw_setup(Q6RouteDw &rt, uint32_t row_bytes, int lane) {
    const uint32_t rr = static_cast<uint32_t>(lane) >> 4, j = lane & 15;
#pragma unroll
    for (int i = 0; i < Q6RouteDw::kN; i++) rt.goff[i] = (4 * i + rr) * row_bytes + (j < 13 ? 16 * j : 192);
    rt.loff = rr * kQ6StripStride + 16 * (j < 13 ? j : 12);
    rt.sh = 0;
}
// base: block b of the wave's first row, the same for every lane (a scalar base and a 32-bit lane offset leave the
// address arithmetic to the load instruction; the offsets count from four bytes below the base so that they stay
// unsigned: the first piece of the wave's first row sits at offset -m)
__device__ __forceinline__ void q6dw_load(Q6RouteDw &rt, const uint8_t *__restrict__ base, int lane) {
    const uint32_t j = lane & 15;
    const uint32_t m = (static_cast<uint32_t>(reinterpret_cast<uintptr_t>(base)) + rt.goff[0]) & 2u;  // the row's block start mod 4
    // pieces start m bytes early; slot 13 takes bytes 192 + m .. 208 + m of the block
    const uint32_t adj = j < 13 ? 4u - m : 4u + m;
    rt.sh = 8 * m;
    const uint8_t *below = base - 4;
#pragma unroll
    for (int i = 0; i < Q6RouteDw::kN; i++)
        rt.v[i] = *reinterpret_cast<const uint4_a4 *>(below + static_cast<size_t>(rt.goff[i] + adj));
}
__device__ __forceinline__ void q6dw_store(const Q6RouteDw &rt, uint8_t *strip, int lane) {
    const uint32_t j = lane & 15;
#pragma unroll
    for (int i = 0; i < Q6RouteDw::kN; i++) {
        const uint4 v = rt.v[i];
        // the dword after this piece: the next slot's first one, or for piece twelve the block's last four bytes
        const uint32_t give = j == 13 ? v.w : v.x;
        const uint32_t nx = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(give), 0x101, 0xf, 0xf, false));  // row_shl:1
        const uint32_t o0 = __builtin_amdgcn_alignbit(v.y, v.x, rt.sh), o1 = __builtin_amdgcn_alignbit(v.z, v.y, rt.sh);
        const uint32_t o2 = __builtin_amdgcn_alignbit(v.w, v.z, rt.sh), o3 = __builtin_amdgcn_alignbit(nx, v.w, rt.sh);
        if (j < 13) {
            uint8_t *dst = strip + rt.loff + i * 4 * kQ6StripStride;
            *reinterpret_cast<uint2 *>(dst) = make_uint2(o0, o1);
            *reinterpret_cast<uint2 *>(dst + 8) = make_uint2(o2, o3);
        }
    }
}

// a lane's share of a Q6_K block from the wave's strip (same pieces as q6_load_row, without d)
__device__ __forceinline__ void q6_row_from_strip(Q6Row &r, const uint8_t *row, int khalf) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int lh = 0; lh < 2; lh++)
                r.h[h].ql[a][lh] = *reinterpret_cast<const uint2 *>(row + 64 * h + 32 * a + 16 * lh + 8 * khalf);
#pragma unroll
        for (int lh = 0; lh < 2; lh++)
            r.h[h].qh[lh] = *reinterpret_cast<const uint2 *>(row + 128 + 32 * h + 16 * lh + 8 * khalf);
    }
    const uint2 s0 = *reinterpret_cast<const uint2 *>(row + 192), s1 = *reinterpret_cast<const uint2 *>(row + 200);
    r.scales = make_uint4(s0.x, s0.y, s1.x, s1.y);
}

// cooperative copy of the workgroup's tokens' quantised activations of one 256-element block into LDS
template <int kToks>
struct Stage {
    static constexpr int kChunks = kToks * 32 / kGbThreads;  // 8-byte chunks per thread
    uint2 v[kChunks];
    float dx;
};

template <int kToks>
__device__ __forceinline__ void stage_load(Stage<kToks> &st, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                           uint32_t tok0, uint32_t last_tok, size_t blocks_per_tok, size_t b, int tid) {
#pragma unroll
    for (int i = 0; i < Stage<kToks>::kChunks; i++) {
        const uint32_t c = static_cast<uint32_t>(tid) + i * kGbThreads;
        const uint32_t t = min(tok0 + (c >> 5), last_tok);
        st.v[i] = *reinterpret_cast<const uint2 *>(aq + (static_cast<size_t>(t) * blocks_per_tok + b) * 256 + (c & 31) * 8);
    }
    st.dx = 0.0f;
    if (tid < kToks) st.dx = ad[static_cast<size_t>(min(tok0 + tid, last_tok)) * blocks_per_tok + b];
}

template <int kToks>
__device__ __forceinline__ void stage_store(const Stage<kToks> &st, uint8_t *abuf, float *dxbuf, int tid) {
#pragma unroll
    for (int i = 0; i < Stage<kToks>::kChunks; i++) {
        const uint32_t c = static_cast<uint32_t>(tid) + i * kGbThreads;
        *reinterpret_cast<uint2 *>(abuf + (c >> 5) * kGbStride64 + (c & 31) * 8) = st.v[i];
    }
    if (tid < kToks) dxbuf[tid] = st.dx;
}

struct Q5Row {
    uint4 hdr, qh;
    uint4 qs[4];
};

template <int kSb>
__device__ __forceinline__ uint32_t q5_codes(uint32_t qs, uint32_t qh) {
    const uint32_t nib = (kSb & 1) ? (qs >> 4) & 0x0f0f0f0fu : qs & 0x0f0f0f0fu;
    const uint32_t fifth = kSb <= 4 ? (qh << (4 - kSb)) & 0x10101010u : (qh >> (kSb - 4)) & 0x10101010u;
    return nib | fifth;
}

// four bytes (each <= 15) times a scalar <= 7 held in both 16-bit halves of `s2`: no carry between bytes
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ int pk_scale(uint32_t nib4, uint32_t s2) {
    const u16x2_t a = __builtin_bit_cast(u16x2_t, nib4), b = __builtin_bit_cast(u16x2_t, s2);
    return __builtin_bit_cast(int, static_cast<u16x2_t>(a * b));
}

// Q4_K / Q5_K row share of a block: header, (fifth bits,) the K-half's 16 bytes of every 32-byte nibble group
template <bool kFifth>
__device__ __forceinline__ Q5Row q45_load_row(const uint8_t *__restrict__ blk, int khalf) {
    Q5Row r;
    r.hdr = ld_u4_a2(blk);
    r.qh = make_uint4(0, 0, 0, 0);
    if constexpr (kFifth) r.qh = ld_u4_a2(blk + 16 + 16 * khalf);
#pragma unroll
    for (int g = 0; g < 4; g++) r.qs[g] = ld_u4_a2(blk + (kFifth ? 48 : 16) + 32 * g + 16 * khalf);
    return r;
}

// Q4_K rows through the wave's strip: a block is nine 16-byte pieces; rows 144 bytes (36 dwords) apart, which keeps the
// 32 rows' 128-bit reads on different banks
constexpr int kQ4Pieces = 9;
constexpr int kQ4StripStride = 144;
constexpr int kQ4StripBytes = 32 * kQ4StripStride;
__device__ __forceinline__ void q4_row_from_strip(Q5Row &r, const uint8_t *row, int khalf) {
    r.hdr = *reinterpret_cast<const uint4 *>(row);
    r.qh = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int g = 0; g < 4; g++) r.qs[g] = *reinterpret_cast<const uint4 *>(row + 16 + 32 * g + 16 * khalf);
}

template <int kSb, bool kFifth>
__device__ __forceinline__ v4i q45_operand(const Q5Row &r) {
    const uint4 qs = r.qs[kSb >> 1];
    if constexpr (kFifth) {
        return v4i{static_cast<int>(q5_codes<kSb>(qs.x, r.qh.x)), static_cast<int>(q5_codes<kSb>(qs.y, r.qh.y)),
                   static_cast<int>(q5_codes<kSb>(qs.z, r.qh.z)), static_cast<int>(q5_codes<kSb>(qs.w, r.qh.w))};
    } else {
        constexpr int sh = (kSb & 1) * 4;
        return v4i{static_cast<int>((qs.x >> sh) & 0x0f0f0f0fu), static_cast<int>((qs.y >> sh) & 0x0f0f0f0fu),
                   static_cast<int>((qs.z >> sh) & 0x0f0f0f0fu), static_cast<int>((qs.w >> sh) & 0x0f0f0f0fu)};
    }
}

}  // namespace

}  // namespace rnb
