// Gathered sparse-MoE experts for batches (prefill) on the matrix cores: the grouped form of gemm_blocks.hip.
// Slots are sorted by expert on the host (api.cpp); workgroup (row tile, expert group) walks the group's slots in tiles
// of 32 tokens: the tokens' quantised activations are gathered into LDS by the sorted lists, the expert's weight rows go
// from global memory to the registers of the lane that owns the row, one int8 matrix instruction per scale group, the
// group's scale on the vector units (see gemm_blocks.hip).  With a handful of tokens per expert most of a 32-token tile
// is padding, which costs no arithmetic: the work per tile is the same whatever the number of live tokens, where the
// integer-dot kernels of moe.hip cost per token (measured crossover on 128 experts x top-8: 64 tokens).  Padding costs
// no LDS either: only the live tokens are staged, the matrix instruction's padding lanes read the last live token's
// row, and the launch sizes the image for the largest group of the call, so that several workgroups share a compute
// unit when the groups are small.
//   gate/up   mid[slot][n_ff] = silu(Wg[e] . a_tok) * (Wu[e] . a_tok), both Q4_K: the two matrices share the activation
//             operand of every instruction                        fanout.rs:260-327, activation.rs:73-89
//   down      slot_out[slot][n_embd] = route[slot] * (Wd[e] . Q8_K(mid[slot])), Q4_K, Q5_K or Q6_K; mid is quantised as the
//             kernel stages it (no quantiser launch between the two kernels)
// (crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs, crates/rnb-cpu/src/kernels/activation.rs)
#include "act_quant.h"
#include "device_utils.h"
#include "kernels.h"
#include "mfma_blocks.h"
#include <algorithm>
#include <type_traits>

namespace rnb {

namespace {

constexpr int kMmToks = 32;  // tokens per tile
constexpr int kQ4FillInstr = (32 * kQ4Pieces + kWave - 1) / kWave;  // 5 wave-wide 16-byte loads per 32 rows of a Q4_K block
constexpr int kQ4FillBytes = kQ4FillInstr * 1024;                   // what they write: 32 x 144 bytes of rows + the tail
constexpr int kMmGateUpStripBytes = kGbWaves * 2 * kQ4FillBytes;    // gate and up strips of the four waves

// the tile's list entries: activation row, output row (0xffffffff past the end of the group) and output scale
struct TileMap {
    uint32_t act_row[kMmToks];
    uint32_t out_row[kMmToks];
    float scale[kMmToks];
};

__device__ __forceinline__ void tile_map_fill(TileMap &m, const uint32_t *__restrict__ act_idx, const uint32_t *__restrict__ out_idx,
                                              const float *__restrict__ out_scale, uint32_t first, uint32_t n_live, int tid) {
    if (tid < kMmToks) {
        const bool live = static_cast<uint32_t>(tid) < n_live;
        const uint32_t p = first + (live ? static_cast<uint32_t>(tid) : n_live - 1);  // padding repeats the last entry
        m.act_row[tid] = act_idx[p];
        const uint32_t o = out_idx[p];
        m.out_row[tid] = live ? o : 0xffffffffu;
        m.scale[tid] = out_scale != nullptr ? out_scale[o] : 1.0f;
    }
}

// the tile's quantised activations of block b (256 int8 per token, 8-byte chunks), scale and digits
template <int kThreads>
struct TileStage {
    static constexpr int kN = (kMmToks * 32 + kThreads - 1) / kThreads;  // chunks per thread
    uint2 v[kN];
    float dx;
    uint4 dig;
};

template <bool kDigits, int kThreads>
__device__ __forceinline__ void tile_stage_load(TileStage<kThreads> &st, const TileMap &m, const int8_t *__restrict__ aq,
                                                const float *__restrict__ ad, const uint8_t *__restrict__ adig, size_t nb,
                                                size_t b, int tid, uint32_t live) {
#pragma unroll
    for (int i = 0; i < TileStage<kThreads>::kN; i++) {
        const uint32_t c = static_cast<uint32_t>(tid) + i * kThreads;
        st.v[i] = make_uint2(0, 0);
        if ((c >> 5) < live)
            st.v[i] = *reinterpret_cast<const uint2 *>(aq + (static_cast<size_t>(m.act_row[c >> 5]) * nb + b) * 256 + (c & 31) * 8);
    }
    st.dx = 0.0f;
    st.dig = make_uint4(0, 0, 0, 0);
    if (tid < kMmToks) {
        const size_t blk = static_cast<size_t>(m.act_row[tid]) * nb + b;
        st.dx = ad[blk];
        if constexpr (kDigits) st.dig = *reinterpret_cast<const uint4 *>(adig + blk * 16);
    }
}

template <int kStride, bool kDigits, int kThreads>
__device__ __forceinline__ void tile_stage_store(const TileStage<kThreads> &st, uint8_t *abuf, float *dxbuf, uint4 *digbuf, int tid,
                                                 uint32_t live) {
#pragma unroll
    for (int i = 0; i < TileStage<kThreads>::kN; i++) {
        const uint32_t c = static_cast<uint32_t>(tid) + i * kThreads;
        if ((c >> 5) < live) *reinterpret_cast<uint2 *>(abuf + (c >> 5) * kStride + (c & 31) * 8) = st.v[i];
    }
    if (tid < kMmToks) {
        dxbuf[tid] = st.dx;
        if constexpr (kDigits) digbuf[tid] = st.dig;
    }
}

// One super-block of one 32-token tile against one Q4_K / Q5_K row share: I = sum_sb sc * (codes . a) and the mins sum
// S = sum_sb mn * bsum32 (through the digits); returns d * I - dmin * S per result in `val`.
// kJ = 1, 2 or 4: only the results of the tile's first 8 kJ tokens are finished on the vector units (result r of a lane
// is token 8 * (r / 4) + 4 * khalf + r % 4, so they are the lane's first 4 kJ results); the matrix instructions always
// compute all 32 tokens, which costs nothing extra.
// The matrix instruction of sub-block SB is issued before the results of sub-block SB - 1 are scaled: a wave that has
// its SIMD to itself would otherwise sit out the instruction's latency (16 passes) eight times per block.
#define RNB_Q45_ISSUE(SB, ROW, ACC, SC)                                                                  \
    {                                                                                                    \
        const v4i bop = q45_operand<SB, kFifth>(ROW);                                                    \
        SC = byte_of(sc8.sc_lo, sc8.sc_hi, SB);                                                          \
        ACC = __builtin_amdgcn_mfma_i32_32x32x32_i8(aops.v[SB], bop, zero16, 0, 0, 0);                   \
        asm volatile("" : "+v"(ACC)); /* pins the instruction in front of the fence */                  \
        __builtin_amdgcn_sched_barrier(0);                                                               \
    }
#define RNB_Q45_TAKE(ACC, SC, TOT)                                                                       \
    {                                                                                                    \
        _Pragma("unroll") for (int i = 0; i < 4 * kJ; i++) {                                             \
            TOT[i] += mul24(ACC[i], SC);                                                                 \
            asm volatile("" : "+v"(TOT[i])); /* keep the eight additions a chain, not a tree */          \
        }                                                                                                \
        asm volatile("" ::"v"(ACC)); /* all sixteen result registers stay the instruction's until here */ \
        __builtin_amdgcn_sched_barrier(0);                                                               \
    }
#define RNB_Q45_SUB_BLOCK(SB, ROW, TOT)                                                                  \
    {                                                                                                    \
        if constexpr (((SB) & 1) == 0) {                                                                 \
            RNB_Q45_ISSUE(SB, ROW, acc_a, sc_a)                                                          \
            if constexpr ((SB) > 0) RNB_Q45_TAKE(acc_b, sc_b, TOT)                                       \
        } else {                                                                                         \
            RNB_Q45_ISSUE(SB, ROW, acc_b, sc_b)                                                          \
            RNB_Q45_TAKE(acc_a, sc_a, TOT)                                                               \
        }                                                                                                \
    }

// The lane's activation operands of one block: token lrow's 16 bytes of each 32-element sub-block.  Read from the
// image in one batch, before the first matrix instruction, and used for both matrices of a gate/up step: read one by
// one in front of their instructions they cost an LDS round trip per sub-block, which a wave alone on its SIMD sits out.
struct TileOps128 {
    v4i v[8];
};
__device__ __forceinline__ void tile_ops_load(TileOps128 &o, const uint8_t *abase) {
#pragma unroll
    for (int sb = 0; sb < 8; sb++) o.v[sb] = *reinterpret_cast<const v4i *>(abase + 32 * sb);
}
struct TileOps64 {
    long v[16];
};
__device__ __forceinline__ void tile_ops_load(TileOps64 &o, const uint8_t *abase) {
#pragma unroll
    for (int sb = 0; sb < 16; sb++) o.v[sb] = *reinterpret_cast<const long *>(abase + 16 * sb);
}

template <bool kFifth, int kJ>
__device__ __forceinline__ void q45_block_tile(const Q5Row &row, const TileOps128 &aops, const uint4 dig, int khalf,
                                               float (&val)[4 * kJ]) {
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const Q4KScales sc8 = unpack_q4k_scales(row.hdr.y, row.hdr.z, row.hdr.w);
    int tot[4 * kJ];
    // With at most 16 live tokens the scale costs 4 kJ <= 8 multiply-adds per sub-block on the results: fewer vector
    // instructions than folding it into the operand (8 per sub-block and a second matrix instruction), which pays for
    // whole tiles only.
    if constexpr (kFifth || kJ < 4) {
#pragma unroll
        for (int i = 0; i < 4 * kJ; i++) tot[i] = 0;
        v16i acc_a, acc_b;
        int sc_a, sc_b;
        RNB_Q45_SUB_BLOCK(0, row, tot)
        RNB_Q45_SUB_BLOCK(1, row, tot)
        RNB_Q45_SUB_BLOCK(2, row, tot)
        RNB_Q45_SUB_BLOCK(3, row, tot)
        RNB_Q45_SUB_BLOCK(4, row, tot)
        RNB_Q45_SUB_BLOCK(5, row, tot)
        RNB_Q45_SUB_BLOCK(6, row, tot)
        RNB_Q45_SUB_BLOCK(7, row, tot)
        RNB_Q45_TAKE(acc_b, sc_b, tot)
    } else {
        // Q4_K: the scale folded into the operand (sc = lo + 8 * hi, two accumulator chains), as in gemm_blocks.hip
        const uint32_t dlo[2] = {sc8.sc_lo & 0x07070707u, sc8.sc_hi & 0x07070707u};
        const uint32_t dhi[2] = {(sc8.sc_lo >> 3) & 0x07070707u, (sc8.sc_hi >> 3) & 0x07070707u};
        v16i acc_lo = zero16, acc_hi = zero16;
#define RNB_Q4_FOLD_SUB_BLOCK(SB)                                                                        \
    {                                                                                                    \
        const v4i nib = q45_operand<SB, false>(row);                                                     \
        constexpr uint32_t sel = 0x0c000c00u | (((SB) & 3) << 16) | ((SB) & 3);                          \
        const uint32_t slo = __builtin_amdgcn_perm(0u, dlo[(SB) >> 2], sel);                             \
        const uint32_t shi = __builtin_amdgcn_perm(0u, dhi[(SB) >> 2], sel);                             \
        const v4i wlo = {pk_scale(nib[0], slo), pk_scale(nib[1], slo), pk_scale(nib[2], slo), pk_scale(nib[3], slo)}; \
        const v4i whi = {pk_scale(nib[0], shi), pk_scale(nib[1], shi), pk_scale(nib[2], shi), pk_scale(nib[3], shi)}; \
        acc_lo = __builtin_amdgcn_mfma_i32_32x32x32_i8(aops.v[SB], wlo, acc_lo, 0, 0, 0);                \
        acc_hi = __builtin_amdgcn_mfma_i32_32x32x32_i8(aops.v[SB], whi, acc_hi, 0, 0, 0);                \
    }
        RNB_Q4_FOLD_SUB_BLOCK(0)
        RNB_Q4_FOLD_SUB_BLOCK(1)
        RNB_Q4_FOLD_SUB_BLOCK(2)
        RNB_Q4_FOLD_SUB_BLOCK(3)
        RNB_Q4_FOLD_SUB_BLOCK(4)
        RNB_Q4_FOLD_SUB_BLOCK(5)
        RNB_Q4_FOLD_SUB_BLOCK(6)
        RNB_Q4_FOLD_SUB_BLOCK(7)
#undef RNB_Q4_FOLD_SUB_BLOCK
#pragma unroll
        for (int i = 0; i < 4 * kJ; i++) tot[i] = acc_lo[i] + 8 * acc_hi[i];
    }
    const float d = f16_bits_to_f32(row.hdr.x), dmin = f16_bits_to_f32(row.hdr.x >> 16);
    // K slots 0..7 of the lower K-half carry the eight mins (weights) and the eight digits (tokens)
    const long mnop = khalf == 0 ? static_cast<long>(static_cast<unsigned long>(sc8.mn_lo) | (static_cast<unsigned long>(sc8.mn_hi) << 32)) : 0L;
    const long op0 = khalf == 0 ? static_cast<long>(static_cast<unsigned long>(dig.x) | (static_cast<unsigned long>(dig.y) << 32)) : 0L;
    const long op1 = khalf == 0 ? static_cast<long>(static_cast<unsigned long>(dig.z) | (static_cast<unsigned long>(dig.w) << 32)) : 0L;
    const v16i c0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(op0, mnop, zero16, 0, 0, 0);
    const v16i c1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(op1, mnop, zero16, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4 * kJ; i++) val[i] = d * static_cast<float>(tot[i]) - dmin * static_cast<float>(c0[i] + 64 * c1[i]);
}
#undef RNB_Q45_SUB_BLOCK
#undef RNB_Q45_TAKE
#undef RNB_Q45_ISSUE

// ... and against one Q6_K row share: returns d * sum_sb sc * ((q - 32) . a)
#define RNB_Q6_TILE_ISSUE(SB, ACC, SC)                                                                   \
    {                                                                                                    \
        const long bop = q6_operand<SB>(row);                                                            \
        SC = q6_scale<SB>(row);                                                                          \
        ACC = __builtin_amdgcn_mfma_i32_32x32x16_i8(aops.v[SB], bop, zero16, 0, 0, 0);                   \
        asm volatile("" : "+v"(ACC));                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                               \
    }
#define RNB_Q6_TILE_TAKE(ACC, SC)                                                                        \
    {                                                                                                    \
        _Pragma("unroll") for (int i = 0; i < 4 * kJ; i++) {                                             \
            tot[i] += mul24(ACC[i], SC);                                                                 \
            asm volatile("" : "+v"(tot[i]));                                                             \
        }                                                                                                \
        asm volatile("" ::"v"(ACC)); /* all sixteen result registers stay the instruction's until here */ \
        __builtin_amdgcn_sched_barrier(0);                                                               \
    }
// issue sub-block SB, then scale the results of SB - 1 (see RNB_Q45_SUB_BLOCK)
#define RNB_Q6_TILE_SUB_BLOCK(SB)                                                                        \
    {                                                                                                    \
        if constexpr (((SB) & 1) == 0) {                                                                 \
            RNB_Q6_TILE_ISSUE(SB, acc_a, sc_a)                                                           \
            if constexpr ((SB) > 0) RNB_Q6_TILE_TAKE(acc_b, sc_b)                                        \
        } else {                                                                                         \
            RNB_Q6_TILE_ISSUE(SB, acc_b, sc_b)                                                           \
            RNB_Q6_TILE_TAKE(acc_a, sc_a)                                                                \
        }                                                                                                \
    }
template <int kJ>
__device__ __forceinline__ void q6_block_tile(const Q6Row &row, const TileOps64 &aops, float (&val)[4 * kJ]) {
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    int tot[4 * kJ];
#pragma unroll
    for (int i = 0; i < 4 * kJ; i++) tot[i] = 0;
    v16i acc_a, acc_b;
    int sc_a, sc_b;
    RNB_Q6_TILE_SUB_BLOCK(0)
    RNB_Q6_TILE_SUB_BLOCK(1)
    RNB_Q6_TILE_SUB_BLOCK(2)
    RNB_Q6_TILE_SUB_BLOCK(3)
    RNB_Q6_TILE_SUB_BLOCK(4)
    RNB_Q6_TILE_SUB_BLOCK(5)
    RNB_Q6_TILE_SUB_BLOCK(6)
    RNB_Q6_TILE_SUB_BLOCK(7)
    RNB_Q6_TILE_SUB_BLOCK(8)
    RNB_Q6_TILE_SUB_BLOCK(9)
    RNB_Q6_TILE_SUB_BLOCK(10)
    RNB_Q6_TILE_SUB_BLOCK(11)
    RNB_Q6_TILE_SUB_BLOCK(12)
    RNB_Q6_TILE_SUB_BLOCK(13)
    RNB_Q6_TILE_SUB_BLOCK(14)
    RNB_Q6_TILE_SUB_BLOCK(15)
    RNB_Q6_TILE_TAKE(acc_b, sc_b)
#pragma unroll
    for (int i = 0; i < 4 * kJ; i++) val[i] = row.d * static_cast<float>(tot[i]);
}
#undef RNB_Q6_TILE_SUB_BLOCK
#undef RNB_Q6_TILE_TAKE
#undef RNB_Q6_TILE_ISSUE

// accf[r] += d_x[token of result r] * val[r]; result r of a tile is token 8 * (r / 4) + 4 * khalf + r % 4
template <int kJ>
__device__ __forceinline__ void tile_scale_add(const float *dxbuf, int khalf, const float (&val)[4 * kJ], float (&accf)[4 * kJ]) {
#pragma unroll
    for (int j = 0; j < kJ; j++) {
        const float4 dx4 = reinterpret_cast<const float4 *>(dxbuf)[2 * j + khalf];
        const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
        for (int i = 0; i < 4; i++) accf[4 * j + i] += dx[i] * val[4 * j + i];
    }
}

// LDS image of one tile: every 256-element block of the tile's live tokens, staged once and then only read
//   act[nb][toks][kStride] | d_x[nb][32] | digits[nb][32] (16 bytes each; absent for Q6_K weights)
// toks <= 32 is the number of token rows the launch made room for (the largest group of the call, capped at a tile)
template <int kStride, bool kDigits>
struct TileImage {
    static __host__ __device__ size_t act_bytes(uint32_t nb, uint32_t toks) { return static_cast<size_t>(nb) * toks * kStride; }
    static __host__ __device__ size_t bytes(uint32_t nb, uint32_t toks = kMmToks) {
        return act_bytes(nb, toks) + static_cast<size_t>(nb) * kMmToks * (4 + (kDigits ? 16 : 0));
    }
    uint8_t *base;
    uint32_t nb, toks;
    __device__ uint8_t *act(uint32_t b) const { return base + static_cast<size_t>(b) * toks * kStride; }
    __device__ float *dx(uint32_t b) const { return reinterpret_cast<float *>(base + act_bytes(nb, toks)) + b * kMmToks; }
    __device__ uint4 *dig(uint32_t b) const {
        return reinterpret_cast<uint4 *>(base + act_bytes(nb, toks) + static_cast<size_t>(nb) * kMmToks * 4) + b * kMmToks;
    }
};

template <int kThreads, int kStride, bool kDigits>
__device__ __forceinline__ void tile_image_fill(const TileImage<kStride, kDigits> &img, const TileMap &m,
                                                const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                                const uint8_t *__restrict__ adig, int tid, uint32_t live) {
    const uint32_t nb = img.nb;
    for (uint32_t b = 0; b < nb; b += 2) {  // two blocks' loads in flight before their stores
        TileStage<kThreads> st0, st1;
        const uint32_t b1 = b + 1 < nb ? b + 1 : b;
        tile_stage_load<kDigits, kThreads>(st0, m, aq, ad, adig, nb, b, tid, live);
        tile_stage_load<kDigits, kThreads>(st1, m, aq, ad, adig, nb, b1, tid, live);
        tile_stage_store<kStride, kDigits, kThreads>(st0, img.act(b), img.dx(b), img.dig(b), tid, live);
        tile_stage_store<kStride, kDigits, kThreads>(st1, img.act(b1), img.dx(b1), img.dig(b1), tid, live);
    }
}

// ---------------------------------------------------------------------------------------------
// gate + up + SiLU * up.  Grid (row tiles of 128, expert groups).  The tile's activations are staged once, all blocks;
// after that the waves run without barriers, each streaming its 32 rows of both matrices one block ahead.  The rows
// come in by whole cache lines as LDS-direct loads into the wave's two strips (consecutive lanes take consecutive
// 16-byte pieces of a row, see RowRoute for why; no vector registers hold the data in flight), and each lane reads its
// row's share back from there.  Dynamic LDS: the four waves' strips, then the tile image.
// ---------------------------------------------------------------------------------------------
template <int kJ, int kW>
__global__ void __attribute__((amdgpu_flat_work_group_size(kWave * kW, kWave * kW), amdgpu_waves_per_eu(2)))
    moe_gate_up_mfma_kernel(const uint8_t *__restrict__ gate_all, const uint8_t *__restrict__ up_all,
                            const uint8_t *__restrict__ gate_shared, const uint8_t *__restrict__ up_shared, uint32_t n_routed,
                            const int8_t *__restrict__ aq, const float *__restrict__ ad, const uint8_t *__restrict__ adig,
                            const uint32_t *__restrict__ grp_expert, const uint32_t *__restrict__ grp_start,
                            const uint32_t *__restrict__ sorted_slot, const uint32_t *__restrict__ sorted_token,
                            float *__restrict__ mid, uint32_t n_ff, uint32_t nb, uint32_t img_toks, uint32_t tiles_per_wg) {
    constexpr bool kFifth = false;
    constexpr int kPair = 2 * kQ4FillBytes;  // a gate strip and an up strip
    extern __shared__ __attribute__((aligned(16))) uint8_t s_dyn[];
    __shared__ TileMap s_map;
    const TileImage<kGbStride128, true> img{s_dyn + kW * kPair, nb, img_toks};
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: LDS-direct loads take their target from a scalar register
    const int lrow = lane & 31, khalf = lane >> 5;
    uint8_t *strips = s_dyn + wave * kPair;
    const uint32_t lds_strips = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lptr_t)strips));
    const uint32_t grp = blockIdx.y;
    const uint32_t expert = grp_expert[grp], start = grp_start[grp], count = grp_start[grp + 1] - start;
    const uint32_t row_bytes = nb * static_cast<uint32_t>(kQ4KBytes);
    const size_t per_expert = static_cast<size_t>(n_ff) * row_bytes;
    const uint8_t *gate_e = expert_base(gate_all, gate_shared, n_routed, expert, per_expert),
                  *up_e = expert_base(up_all, up_shared, n_routed, expert, per_expert);
    // The workgroup walks tiles_per_wg row tiles against one staged token tile (map and image are made once: a chain of
    // dependent loads); the weight blocks of the whole walk form one stream of rt_n * nb steps, requested one step
    // ahead across row tiles.  (Two steps ahead into a second pair of strips measured no faster: 53.3 against 50.6 us.)
    const uint32_t row_tiles = (n_ff + 32 * kW - 1) / (32 * kW);
    const uint32_t rt0 = blockIdx.x * tiles_per_wg, rt_n = min(tiles_per_wg, row_tiles - rt0);
    // The request cursor.  Row tile rt: the wave's first row (a wave wholly past the end streams the last row and stores
    // nothing) and its pieces.  Piece c = 64 i + lane of the wave's 32 x 9 pieces of a block: row c / 9, 16-byte column
    // c % 9; it lands at byte 16 c of the strip, which puts the rows 144 bytes apart (rows past the end of the matrix
    // repeat the last row; the pieces past 288 of the fifth instruction repeat the last piece and land behind the rows)
    const uint8_t *gbase, *ubase;
    uint32_t goff[kQ4FillInstr];
    uint32_t req_b = 0, req_rt = 0;  // next block / row tile to request
    auto set_tile = [&](uint32_t rt) {
        const uint32_t first = min((rt0 + rt) * (32 * kW) + wave * 32, n_ff - 1);
        const size_t woff = static_cast<size_t>(first) * row_bytes;
        gbase = gate_e + woff;
        ubase = up_e + woff;
#pragma unroll
        for (int i = 0; i < kQ4FillInstr; i++) {
            const uint32_t c = min(static_cast<uint32_t>(lane) + i * kWave, 32u * kQ4Pieces - 1);
            const uint32_t r = c / kQ4Pieces, j = c - r * kQ4Pieces;
            goff[i] = min(r, n_ff - first - 1) * row_bytes + 16 * j;
        }
    };
    // the next step of the walk into the strips (past the end: the last step again, unused)
    auto request = [&]() {
        // the strips' previous contents have been read out (the reads are ahead of these fills in program order; make
        // sure they have executed)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const uint32_t dst = lds_strips;
        const uint8_t *gsrc = gbase + req_b * static_cast<uint32_t>(kQ4KBytes), *usrc = ubase + req_b * static_cast<uint32_t>(kQ4KBytes);
#pragma unroll
        for (int i = 0; i < kQ4FillInstr; i++) lds_fill16(gsrc, goff[i], dst + i * 1024);
#pragma unroll
        for (int i = 0; i < kQ4FillInstr; i++) lds_fill16(usrc, goff[i], dst + kQ4FillBytes + i * 1024);
        if (req_b + 1 < nb) {
            req_b++;
        } else if (req_rt + 1 < rt_n) {
            req_rt++;
            req_b = 0;
            set_tile(req_rt);
        }
    };
    auto take = [&](Q5Row &g, Q5Row &u) {
        wait_fills();
        q4_row_from_strip(g, strips + lrow * kQ4StripStride, khalf);
        q4_row_from_strip(u, strips + kQ4FillBytes + lrow * kQ4StripStride, khalf);
    };

    for (uint32_t tile0 = 0; tile0 < count; tile0 += img_toks) {
        // the first weight blocks do not depend on the token lists: requested before them
        req_b = req_rt = 0;
        set_tile(0);
        request();
        const uint32_t live = min(count - tile0, img_toks);
        const uint32_t arow = min(static_cast<uint32_t>(lrow), live - 1);  // padding lanes read the last live row
        if (tile0) __syncthreads();  // the previous tile's readers of the map and the image are done
        tile_map_fill(s_map, sorted_token, sorted_slot, nullptr, start + tile0, live, tid);
        __syncthreads();
        tile_image_fill<kWave * kW>(img, s_map, aq, ad, adig, tid, live);
        Q5Row cg, cu;
        take(cg, cu);
        __syncthreads();
        // a tile of at most eight live tokens (most groups of a routed batch) finishes only a lane's first four results
        auto walk = [&](auto jtag) {
            constexpr int kJl = decltype(jtag)::value;
            for (uint32_t rt = 0; rt < rt_n; rt++) {
                const uint32_t row = (rt0 + rt) * (32 * kW) + wave * 32 + lrow;
                float accg[4 * kJl], accu[4 * kJl];
#pragma unroll
                for (int i = 0; i < 4 * kJl; i++) accg[i] = accu[i] = 0.0f;
                for (uint32_t b = 0; b < nb; b++) {
                    request();  // the step after this one
                    const uint8_t *abase = img.act(b) + arow * kGbStride128 + 16 * khalf;
                    const uint4 dig = img.dig(b)[lrow];
                    float val[4 * kJl];
                    TileOps128 aops;
                    tile_ops_load(aops, abase);
                    q45_block_tile<kFifth, kJl>(cg, aops, dig, khalf, val);
                    tile_scale_add<kJl>(img.dx(b), khalf, val, accg);
                    q45_block_tile<kFifth, kJl>(cu, aops, dig, khalf, val);
                    tile_scale_add<kJl>(img.dx(b), khalf, val, accu);
                    take(cg, cu);  // (after the last step: a repeat of it, unused)
                }
                if (row < n_ff) {
#pragma unroll
                    for (int r = 0; r < 4 * kJl; r++) {
                        const uint32_t slot = s_map.out_row[8 * (r >> 2) + 4 * khalf + (r & 3)];
                        if (slot != 0xffffffffu) mid[static_cast<size_t>(slot) * n_ff + row] = act_mul<false>(accg[r], accu[r]);
                    }
                }
            }
        };
        if constexpr (kJ == 2) {  // (the 32-token kernel keeps its one form: its groups are large)
            if (live <= 8)  // workgroup-uniform
                walk(std::integral_constant<int, 1>{});
            else
                walk(std::integral_constant<int, 2>{});
        } else {
            walk(std::integral_constant<int, kJ>{});
        }
    }
}

// ---------------------------------------------------------------------------------------------
// down projection of the re-quantised intermediate, scaled by the route weight.  Grid (row tiles of 128, expert groups).
// ---------------------------------------------------------------------------------------------
template <uint32_t kQuant, int kJ>
__global__ void __launch_bounds__(kGbThreads, 2)
    moe_down_mfma_kernel(const uint8_t *__restrict__ down_all, const uint8_t *__restrict__ down_shared, uint32_t n_routed,
                         const float *__restrict__ mid,
                         const uint32_t *__restrict__ grp_expert,
                         const uint32_t *__restrict__ grp_start, const uint32_t *__restrict__ sorted_slot,
                         const float *__restrict__ slot_route, float *__restrict__ slot_out, uint32_t n_embd, uint32_t nb,
                         uint32_t tiles_per_wg, uint32_t img_toks) {
    constexpr bool kSix = kQuant == kQ6K;
    constexpr bool kFifth = kQuant == kQ5K;
    constexpr int kStride = kSix ? kGbStride64 : kGbStride128;
    constexpr size_t kBlockBytes = kSix ? kQ6KBytes : (kFifth ? kQ5KBytes : kQ4KBytes);
    extern __shared__ __attribute__((aligned(16))) uint8_t s_dyn[];
    __shared__ TileMap s_map;
    const TileImage<kStride, !kSix> img{s_dyn, nb, img_toks};
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: the wave's row addresses are scalar bases plus lane offsets
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t grp = blockIdx.y;
    const uint32_t expert = grp_expert[grp], start = grp_start[grp], count = grp_start[grp + 1] - start;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint8_t *down_e = expert_base(down_all, down_shared, n_routed, expert, n_embd * row_bytes);
    // The workgroup walks tiles_per_wg row tiles of 128 against one staged token tile: map and image are made once,
    // and the weight blocks of the whole walk form one stream that is requested one block ahead across row tiles.
    const uint32_t row_tiles = (n_embd + kGbRows - 1) / kGbRows;
    const uint32_t rt0 = blockIdx.x * tiles_per_wg, rt_n = min(tiles_per_wg, row_tiles - rt0);
    const uint32_t steps = rt_n * nb;
    auto row_of = [&](uint32_t rt) { return (rt0 + rt) * kGbRows + wave * 32 + lrow; };
    auto block_ptr = [&](uint32_t rt, uint32_t b) {
        return down_e + static_cast<size_t>(min(row_of(rt), n_embd - 1)) * row_bytes + b * kBlockBytes;
    };
    // Q6_K rows come in by whole cache lines through the wave's strip of LDS (RowRoute: the lane-owns-row loads of
    // q6_load_row touch 64 lines per instruction); the other formats' 16-byte loads go straight to the lane
    __shared__ int16_t s_bsums[kGbWaves][16];  // the quantiser's 16-element sums: not used by these kernels
    __shared__ __attribute__((aligned(16))) uint8_t s_w[kSix ? kGbWaves : 1][kSix ? 32 * kQ6StripStride : 16];
    uint8_t *strip = s_w[kSix ? wave : 0];
    // (n_embd is a multiple of 128 and down_all is 16-byte aligned: whole tiles, even addresses, as Q6RouteDw needs)
    Q6RouteDw route;
    if constexpr (kSix) q6dw_setup(route, static_cast<uint32_t>(row_bytes), lane);
    float d_next = 0.0f;
    const uint32_t d_off = static_cast<uint32_t>(lrow) * static_cast<uint32_t>(row_bytes) + 208;  // the lane's row's d from the wave's first row
    auto q6_request = [&](uint32_t rt, uint32_t b) {  // block b of row tile rt: pieces into route.v, d into d_next
        const uint32_t first = (rt0 + rt) * kGbRows + wave * 32;  // the wave's first row (whole tiles: no row past the end)
        const uint8_t *base = down_e + static_cast<size_t>(first) * row_bytes + b * kBlockBytes;
        q6dw_load(route, base, lane);
        d_next = ld_f16(base + static_cast<size_t>(d_off));
    };
    auto q6_take = [&](Q6Row &r) {
        q6dw_store(route, strip, lane);
        q6_row_from_strip(r, strip + lrow * kQ6StripStride, khalf);
        r.d = d_next;
    };

    for (uint32_t tile0 = 0; tile0 < count; tile0 += img_toks) {
        Q6Row c6{};
        Q5Row c5{};
        // the first weight block does not depend on the token lists: requested before them
        if constexpr (kSix)
            q6_request(0, 0);
        else
            c5 = q45_load_row<kFifth>(block_ptr(0, 0), khalf);
        if (tile0) __syncthreads();
        const uint32_t live = min(count - tile0, img_toks);
        const uint32_t arow = min(static_cast<uint32_t>(lrow), live - 1);
        tile_map_fill(s_map, sorted_slot, sorted_slot, slot_route, start + tile0, live, tid);
        __syncthreads();
        // the tile's slots' intermediates (f32, [slot][nb * 256]) are quantised to Q8_K as they are staged, with the
        // stand-alone quantiser's wave-level routine (the same bits): wave w takes (token, block) pairs w, w + 4, ...,
        // four loads in flight.  The workgroups of a group's other row tiles repeat this; it is a few blocks each.
        {
            const uint32_t pairs = live * nb;
            for (uint32_t p0 = wave; p0 < pairs; p0 += 4 * kGbWaves) {
                float4 v[4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t p = p0 + k * kGbWaves;
                    v[k] = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (p < pairs) {
                        const uint32_t t = p / nb, b = p - t * nb;
                        v[k] = reinterpret_cast<const float4 *>(mid + (static_cast<size_t>(s_map.act_row[t]) * nb + b) * 256)[lane];
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const uint32_t p = p0 + k * kGbWaves;
                    if (p < pairs) {  // wave-uniform
                        const uint32_t t = p / nb, b = p - t * nb;
                        q8k_quantize_vals(v[k], lane, reinterpret_cast<int8_t *>(img.act(b) + t * kStride), &img.dx(b)[t], s_bsums[wave],
                                          kSix ? nullptr : reinterpret_cast<uint8_t *>(&img.dig(b)[t]));
                    }
                }
            }
        }
        if constexpr (kSix) q6_take(c6);
        __syncthreads();
        // a tile of at most eight live tokens (most groups of a routed batch) finishes only a lane's first four results
        auto walk = [&](auto jtag) {
        constexpr int kJl = decltype(jtag)::value;
        float accf[4 * kJl];
#pragma unroll
        for (int i = 0; i < 4 * kJl; i++) accf[i] = 0.0f;
        uint32_t rt = 0, b = 0;
        for (uint32_t s = 0; s < steps; s++) {
            uint32_t rtn = rt, bn = b + 1;  // the step after this one; the last step reloads its own block, unused
            if (bn == nb) {
                bn = 0;
                rtn = rt + 1;
            }
            if (s + 1 == steps) {
                rtn = rt;
                bn = b;
            }
            Q5Row n5{};
            float val[4 * kJl];
            if constexpr (kSix) {
                q6_request(rtn, bn);
                TileOps64 aops;
                tile_ops_load(aops, img.act(b) + arow * kStride + 8 * khalf);
                q6_block_tile<kJl>(c6, aops, val);
            } else {
                n5 = q45_load_row<kFifth>(block_ptr(rtn, bn), khalf);
                TileOps128 aops;
                tile_ops_load(aops, img.act(b) + arow * kStride + 16 * khalf);
                q45_block_tile<kFifth, kJl>(c5, aops, img.dig(b)[lrow], khalf, val);
            }
            tile_scale_add<kJl>(img.dx(b), khalf, val, accf);
            if constexpr (kSix) q6_take(c6);
            c5 = n5;
            if (b + 1 == nb) {  // the row tile is complete
                const uint32_t row = row_of(rt);
                if (row < n_embd) {
#pragma unroll
                    for (int r = 0; r < 4 * kJl; r++) {
                        const int t = 8 * (r >> 2) + 4 * khalf + (r & 3);
                        const uint32_t slot = s_map.out_row[t];
                        // fanout.rs:306-308: the expert's output times the slot's route weight
                        if (slot != 0xffffffffu)
                            slot_out[static_cast<size_t>(slot) * n_embd + row] = accf[r] * s_map.scale[t];
                    }
                }
#pragma unroll
                for (int i = 0; i < 4 * kJl; i++) accf[i] = 0.0f;
            }
            rt = rtn;
            b = bn;
        }
        };
        if constexpr (kJ == 2) {
            if (live <= 8)  // workgroup-uniform
                walk(std::integral_constant<int, 1>{});
            else
                walk(std::integral_constant<int, 2>{});
        } else {
            walk(std::integral_constant<int, kJ>{});
        }
    }
}

// raises a kernel's dynamic LDS limit above the default 64 KB, once per kernel (K is a distinct type per kernel only
// through the tag)
template <int kTag, typename K>
bool allow_lds(K kernel, size_t bytes) {
    static bool done = false;
    return allow_dynamic_lds(reinterpret_cast<const void *>(kernel), bytes, &done, "MoE matrix-core kernel");
}

}  // namespace

// the tile image (all blocks of the tile's tokens) must fit the LDS of a compute unit beside the waves' strips and the
// small static arrays; a tile holds as many tokens as fit, at most 32
constexpr size_t kMmLdsLimit = 150 * 1024;
constexpr size_t kMmGateUpImageLimit = kMmLdsLimit - kMmGateUpStripBytes;
constexpr size_t kMmQ6DownLdsLimit = kMmLdsLimit - kGbWaves * 32 * kQ6StripStride;
constexpr uint32_t kMmMinToks = 16;  // below this the matrix-core path re-reads the weights too often to pay

template <int kStride, bool kDigits>
static uint32_t tile_tokens_that_fit(size_t limit, uint32_t nb) {
    uint32_t toks = kMmToks;
    while (toks > 0 && TileImage<kStride, kDigits>::bytes(nb, toks) > limit) toks--;
    return toks;
}
static uint32_t gate_up_tile_tokens(uint32_t nb_in) { return tile_tokens_that_fit<kGbStride128, true>(kMmGateUpImageLimit, nb_in); }
static uint32_t down_tile_tokens(uint32_t nb_mid, uint32_t down_quant) {
    return down_quant == kQ6K ? tile_tokens_that_fit<kGbStride64, false>(kMmQ6DownLdsLimit, nb_mid)
                              : tile_tokens_that_fit<kGbStride128, true>(kMmLdsLimit, nb_mid);
}

bool moe_mfma_supported(uint32_t nb_in, uint32_t nb_mid, uint32_t down_quant) {
    return nb_in >= 1 && nb_mid >= 1 && gate_up_tile_tokens(nb_in) >= kMmMinToks && down_tile_tokens(nb_mid, down_quant) >= kMmMinToks;
}

void launch_moe_gate_up_mfma(const uint8_t *gate_all, const uint8_t *up_all, const MoeShared &shared, ActView act,
                             MoeGroups groups, float *mid, uint32_t n_ff, uint32_t nb_in, hipStream_t stream) {
    if (groups.n_groups == 0 || n_ff == 0) return;
    const uint32_t toks = std::min<uint32_t>(std::max<uint32_t>(groups.max_group, 1), gate_up_tile_tokens(nb_in));
    if (toks == 0) return;  // moe_mfma_supported said no
    const size_t image = TileImage<kGbStride128, true>::bytes(nb_in, toks);
    // A wave's time is its chain of steps, and the chain is mostly instruction and LDS latency that only another wave on
    // the SIMD hides (without its fills the kernel still takes 40 of its 50 us); a grid of more workgroups than fit at once
    // runs in rounds, and a last round that is partly empty costs as much as a full one.  So: the widest workgroup (six
    // waves = 192 rows, else four = 128) for which merging up to three row tiles into one walk brings the grid down to
    // one workgroup per compute unit, map and image made once per walk.  128 experts x top-8 at 64 tokens (126 groups):
    // four waves 1 / 2 / 3 tiles per workgroup 55.4 / 58.4 / 50.6 us (2 leaves half the units with two workgroups and
    // half with one), six waves x 2 tiles 48.8 us, eight waves x 1 (two rounds) 61.6, twelve waves 67-74.
    int waves = kGbWaves;
    uint32_t tiles_per_wg = 1;
    for (const int w : {6, 4}) {
        if (w != kGbWaves && (toks > 16 || static_cast<size_t>(w) * 2 * kQ4FillBytes + image > kMmLdsLimit)) continue;
        const uint32_t tiles = (n_ff + 32 * w - 1) / (32 * w);
        const uint32_t t = static_cast<uint32_t>((static_cast<uint64_t>(tiles) * groups.n_groups + 255) / 256);
        if (t >= 1 && t <= 3 && t <= tiles && static_cast<uint64_t>((tiles + t - 1) / t) * groups.n_groups <= 256 &&
            (t > 1 || w == 4)) {
            waves = w;
            tiles_per_wg = t;
            break;
        }
    }
    const size_t lds = static_cast<size_t>(waves) * 2 * kQ4FillBytes + image;
    const uint32_t rows_per_wg = 32 * waves, row_tiles = (n_ff + rows_per_wg - 1) / rows_per_wg;
    const dim3 grid((row_tiles + tiles_per_wg - 1) / tiles_per_wg, groups.n_groups, 1);
    // tiles of at most 8 / 16 / 32 tokens: the kernel finishes only that many results per lane
#define RNB_LAUNCH_GUW(J, W)                                                                                          \
    if (!allow_lds<J * 16 + W>(moe_gate_up_mfma_kernel<J, W>, kMmLdsLimit)) return;                                   \
    hipLaunchKernelGGL((moe_gate_up_mfma_kernel<J, W>), grid, dim3(kWave * W), lds, stream, gate_all, up_all, shared.gate, \
                       shared.up, shared.n_routed, act.qs, act.d, act.digits, groups.expert, groups.start,            \
                       groups.sorted_slot, groups.sorted_token, mid, n_ff, nb_in, toks, tiles_per_wg)
    if (toks > 16) {
        RNB_LAUNCH_GUW(4, kGbWaves);
    } else if (waves == 6) {
        if (toks <= 8) {
            RNB_LAUNCH_GUW(1, 6);
        } else {
            RNB_LAUNCH_GUW(2, 6);
        }
    } else if (toks <= 8) {
        RNB_LAUNCH_GUW(1, kGbWaves);
    } else {
        RNB_LAUNCH_GUW(2, kGbWaves);
    }
#undef RNB_LAUNCH_GUW
}

void launch_moe_down_mfma(const uint8_t *down_all, const MoeShared &shared, uint32_t down_quant, const float *mid, MoeGroups groups,
                          const float *slot_route, float *slot_out, uint32_t n_embd, uint32_t nb_mid, hipStream_t stream) {
    if (groups.n_groups == 0 || n_embd == 0) return;
    // A workgroup's setup (group, map, image: a chain of dependent loads) costs more than a row tile's few blocks, and
    // about three workgroups fit a compute unit: row tiles are merged (up to 4 per workgroup) until the grid fits them at
    // once (cfg5's shape, 16 row tiles x 126 groups, 64 tokens: 1 / 2 / 4 / 8 tiles per workgroup 72 / 62 / 59 / 62 us)
    const uint32_t row_tiles = (n_embd + kGbRows - 1) / kGbRows;
    uint32_t tiles_per_wg = 1;
    while (tiles_per_wg < 4 && static_cast<uint64_t>((row_tiles + tiles_per_wg - 1) / tiles_per_wg) * groups.n_groups > 768)
        tiles_per_wg *= 2;
    const dim3 grid((row_tiles + tiles_per_wg - 1) / tiles_per_wg, groups.n_groups, 1), block(kGbThreads);
    const uint32_t toks = std::min<uint32_t>(std::max<uint32_t>(groups.max_group, 1), down_tile_tokens(nb_mid, down_quant));
    if (toks == 0) return;
#define RNB_LAUNCH_DMJ(Q, J, LDS)                                                                                     \
    if (!allow_lds<static_cast<int>(Q) * 8 + J>(moe_down_mfma_kernel<Q, J>, Q == kQ6K ? kMmQ6DownLdsLimit : kMmLdsLimit)) return; \
    hipLaunchKernelGGL((moe_down_mfma_kernel<Q, J>), grid, block, LDS, stream, down_all, shared.down, shared.n_routed, mid, \
                       groups.expert, groups.start, groups.sorted_slot, slot_route, slot_out, n_embd, nb_mid, tiles_per_wg, toks)
#define RNB_LAUNCH_DM(Q, LDS)                                                                                         \
    if (toks <= 8) {                                                                                                  \
        RNB_LAUNCH_DMJ(Q, 1, LDS);                                                                                    \
    } else if (toks <= 16) {                                                                                          \
        RNB_LAUNCH_DMJ(Q, 2, LDS);                                                                                    \
    } else {                                                                                                          \
        RNB_LAUNCH_DMJ(Q, 4, LDS);                                                                                    \
    }
    if (down_quant == kQ6K) {
        RNB_LAUNCH_DM(kQ6K, (TileImage<kGbStride64, false>::bytes(nb_mid, toks)));
    } else if (down_quant == kQ5K) {
        RNB_LAUNCH_DM(kQ5K, (TileImage<kGbStride128, true>::bytes(nb_mid, toks)));
    } else {
        RNB_LAUNCH_DM(kQ4K, (TileImage<kGbStride128, true>::bytes(nb_mid, toks)));
    }
#undef RNB_LAUNCH_DM
#undef RNB_LAUNCH_DMJ
}

}  // namespace rnb
