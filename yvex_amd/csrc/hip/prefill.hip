// Row-batch (prefill-width) grouped expert projections on the int8 matrix cores of gfx950.
//
// A work item is (bucket, tile of up to 128 ordered pairs, tile of 128 weight rows: 64 gate rows
// and the 64 matching up rows when the SwiGLU is fused). The workgroup has four waves, one per
// SIMD; each owns 32 weight rows and multiplies them by all of the item's Q8_K activation rows
// with V_MFMA_I32_32X32X32_I8, so one activation fragment read from LDS feeds two matrix
// instructions of 32 passes in total and the decode of a weight is shared by up to 128 tokens.
//
//   A operand (weights): built in registers. Lane (r, h) = (lane % 32, lane / 32) owns weight
//       row r and the groups 4h .. 4h + 3 of the current superblock (128 columns); K chunk m of
//       the superblock is, for that lane, the 16 weights 16 (m % 2) .. + 15 of group 4h + m / 2.
//       The order of K inside a matrix instruction is free as long as both operands agree.
//       The IQ2_XXS value of one weight is level * sign * (2s+1), up to 43 * 31 = 1333, so it is
//       split into two int8 limbs, value = 128 * hi + lo with hi in [1, 11] and lo in
//       [-120, 63], and every K chunk costs two matrix instructions. For one scale there are only
//       three levels, so the six signed limb values of a group fit two registers and one
//       V_PERM_B32 per four weights picks them: the selector byte of a weight is its level code
//       (0..2) plus 4 when it is negative. Three LDS tables feed this: level codes of a codebook
//       entry (8 bytes, 32 replicas: no two lanes of a half-wave share a bank), sign selectors
//       of a 7-bit sign field (8 bytes, 16 replicas) and the limb words of a scale (16 bytes,
//       16 replicas).
//   B operand (activations): the tile's int8 blocks of one stage period (four superblocks of 32
//       tokens, two of 64 or one of 128), copied from global memory straight into LDS
//       (GLOBAL_LOAD_LDS_DWORDX4), double buffered. 16-byte piece c of token t sits at piece
//       position c ^ (t % 16), so the 16 lanes that read one fragment column together hit 16
//       different bank groups.
//   C: per (superblock, 32-token block) two int32 accumulators of 32 x 32; T = 128 * C_hi + C_lo
//       is the exact integer superblock sum of the reference's primitive
//       (src/backend/cuda/kernel_primitives.h:287-313), scaled into fp32 as
//       ((0.125 * d_w) * d_a) * T and summed over superblocks.
//   Output: the wave's fp32 sums go through LDS once per item so that every store instruction
//       writes whole 64-byte runs of an output row.
//
// Same inputs, outputs and rounding points as the decode-width sweeps in moe.hip
// (src/backend/cuda/tensorcore.cu:378-702 is the reference's counterpart, unused there).
#include "common.hpp"
#include "launch.hpp"
#include "grouped.hpp"

namespace yvex {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr unsigned kRowWaves = 4u;
constexpr unsigned kRowThreads = 64u * kRowWaves;
constexpr unsigned kTileTokens = 128u;
constexpr unsigned kActPitch = 256u;                       // one Q8_K block's int8 payload
// LDS map (absolute byte offsets; the dynamic allocation starts at 0, checked at kernel start).
constexpr unsigned kCodeBase = 0u;                          // 256 entries x 32 replicas x 8 bytes
constexpr unsigned kSelBase = 65536u;                       // 128 sign fields x 16 replicas x 8 bytes
constexpr unsigned kLutBase = kSelBase + 128u * 16u * 8u;   // 16 scales x 16 replicas x 16 bytes
constexpr unsigned kRowScaleBase = kLutBase + 16u * 16u * 16u;   // 4 waves x 2 x 32 floats
constexpr unsigned kPairInfoBase = kRowScaleBase + kRowWaves * 2u * 128u;   // {out row, route weight} x 128
// Item numbering: first full 128-pair tile of every bucket (257 words), then per class of last,
// partial, tile (65-127, 33-64, 1-32 pairs) a count and the list of its buckets (u16).
constexpr unsigned kTileStartBase = kPairInfoBase + kTileTokens * 8u;
constexpr unsigned kClassCountBase = kTileStartBase + 260u * 4u;
constexpr unsigned kClassListBase = kClassCountBase + 16u;
constexpr unsigned kTrashBase = kClassListBase + 3u * 256u * 2u;   // 256 bytes nobody reads
constexpr unsigned kStageBase = (kTrashBase + 256u + 255u) & ~255u;
constexpr unsigned kStageActs = kTileTokens * kActPitch;
constexpr unsigned kStageBytes = kStageActs + kTileTokens * 4u;   // + one fp32 scale per slot
// the finished tile on its way out: 128 tokens x (128 values + 4 of padding) fp32
constexpr unsigned kOutPitch = 132u * 4u;
constexpr unsigned kOutBytes = kTileTokens * kOutPitch;
constexpr unsigned kMfmaLdsBytes = kStageBase + (2u * kStageBytes > kOutBytes ? 2u * kStageBytes : kOutBytes);
static_assert(kMfmaLdsBytes <= 160u * 1024u, "one workgroup per compute unit");

struct MfmaArgs {
    GroupedProblem pr;
    unsigned width;          // reduction width
    unsigned out_rows;       // weight rows per expert
    double limit;
    int *status;
};

__device__ __forceinline__ void lds_write_uint4(unsigned address, uint4 v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) uint4 *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_write_uint2(unsigned address, uint2 v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) uint2 *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_write_u32(unsigned address, unsigned v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) unsigned *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_write_u16(unsigned address, unsigned v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) unsigned short *>(address) = (unsigned short)v;
#else
    (void)address;
    (void)v;
#endif
}
// One 16-byte LDS read as a vector value (a struct of four words may reach the backend as four
// scalar loads and come out as two 8-byte reads).
__device__ __forceinline__ v4i lds_read_v4i(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const v4i *>(address);
#else
    (void)address;
    return v4i{0, 0, 0, 0};
#endif
}
__device__ __forceinline__ unsigned lds_read_u16(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const unsigned short *>(address);
#else
    (void)address;
    return 0u;
#endif
}
__device__ __forceinline__ unsigned lds_read_u32(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const unsigned *>(address);
#else
    (void)address;
    return 0u;
#endif
}

// Asynchronous copy global -> LDS (GLOBAL_LOAD_LDS): lane l of the wave writes `bytes` bytes at
// lds_base + l * bytes; nothing passes through registers. Written as assembly so the compiler
// does not put a conservative wait in front of every later LDS read: the kernel waits with
// vmcnt(0) (loads retire in order, so the compiler's own counted waits stay correct) before
// the barrier that publishes the data.
__device__ __forceinline__ void copy_to_lds_16(const void *global, unsigned lds_base)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :: "s"(lds_base), "v"(global) : "memory");   // m0 is reserved: the compiler reloads it before any use of its own
#else
    (void)global;
    (void)lds_base;
#endif
}
__device__ __forceinline__ void copy_to_lds_4(const void *global, unsigned lds_base)
{
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                 :: "s"(lds_base), "v"(global) : "memory");   // m0 is reserved: the compiler reloads it before any use of its own
#else
    (void)global;
    (void)lds_base;
#endif
}

// Limb pair of one magnitude: low limb in bits 0-7, high limb in bits 8-15.
__device__ __forceinline__ unsigned iq2_limbs(unsigned level, unsigned factor)
{
    const unsigned magnitude = level * factor;
    unsigned hi = (magnitude + 64u) >> 7;
    if (hi == 0u) hi = 1u;
    const int lo = (int)magnitude - 128 * (int)hi;
    return ((unsigned)lo & 255u) | (hi << 8);
}

__device__ __forceinline__ void mfma_tables_fill()
{
    // level codes: byte l of the entry is 0, 1 or 2 for level 8, 25 or 43 of weight l
    for (unsigned index = threadIdx.x; index < 256u * 32u; index += blockDim.x) {
        const uint2 m = iq2_magnitude_entry(index >> 5);
        uint2 codes = make_uint2(0u, 0u);
#pragma unroll
        for (unsigned l = 0; l < 4u; ++l) {
            const unsigned a = (m.x >> (8u * l)) & 255u, b = (m.y >> (8u * l)) & 255u;
            codes.x |= (a == 8u ? 0u : a == 25u ? 1u : 2u) << (8u * l);
            codes.y |= (b == 8u ? 0u : b == 25u ? 1u : 2u) << (8u * l);
        }
        lds_write_uint2(kCodeBase + index * 8u, codes);
    }
    // sign selectors: byte l is 4 when weight l is negative (7 stored bits + parity)
    for (unsigned index = threadIdx.x; index < 128u * 16u; index += blockDim.x) {
        const uint2 m = iq2_signmask_entry(index >> 4);
        lds_write_uint2(kSelBase + index * 8u, make_uint2(m.x & 0x04040404u, m.y & 0x04040404u));
    }
    // limb words of scale s: {+lo, -lo, +hi, -hi}, byte c = limb of level code c
    for (unsigned index = threadIdx.x; index < 16u * 16u; index += blockDim.x) {
        const unsigned factor = 2u * (index >> 4) + 1u;
        unsigned lo = 0u, hi = 0u;
        const unsigned levels[3] = {8u, 25u, 43u};
#pragma unroll
        for (unsigned c = 0; c < 3u; ++c) {
            const unsigned pair = iq2_limbs(levels[c], factor);
            lo |= (pair & 255u) << (8u * c);
            hi |= (pair >> 8) << (8u * c);
        }
        // byte-wise negation: no limb is zero, so (x ^ 0xff) + 1 never carries; byte 3 stays 0
        const unsigned neg_lo = ((lo ^ 0x00ffffffu) + 0x00010101u) & 0x00ffffffu;
        const unsigned neg_hi = ((hi ^ 0x00ffffffu) + 0x00010101u) & 0x00ffffffu;
        lds_write_uint4(kLutBase + index * 16u, make_uint4(lo, neg_lo, hi, neg_hi));
    }
}

// What one work item needs to know about its place in the problem.
struct MfmaItem {
    unsigned long long expert, pair0;
    unsigned tokens, row_tile;
};

// The aligned dwords around a lane's 32 code bytes of one superblock, and the dword that holds
// the superblock's fp16 scale.
struct RawCodes {
    uint4 x0, x1;
    unsigned x2, scale_word;
};

__device__ __forceinline__ uint4 load_uint4_dword_aligned(const unsigned char *p)
{
    uint4 v;
    __builtin_memcpy(&v, __builtin_assume_aligned(p, 4), 16);
    return v;
}
__device__ __forceinline__ unsigned load_u32_aligned(const unsigned char *p)
{
    return *reinterpret_cast<const unsigned *>(p);
}

// Where in the 8 NTB slots of a superblock each piece of the next superblock's decode runs:
// settle (records out of the loaded dwords, row scale to LDS), then per group g the nine table
// lookups L(g), the selector words S(g), and per K chunk m the permutes P(m) that overwrite the
// chunk's operands once the last token block has used them.
template <unsigned NTB>
struct DecodePlan {
    static constexpr unsigned kSlots = 8u * NTB;
    static constexpr unsigned lookup_slot(unsigned g)
    {
        return NTB == 4u ? 1u + 6u * g : NTB == 2u ? 2u * g : g;
    }
    static constexpr unsigned select_slot(unsigned g)
    {
        return NTB == 4u ? 4u + 6u * g : NTB == 2u ? 2u * g + 2u : g + 2u;
    }
    static constexpr unsigned permute_slot(unsigned m)
    {
        // after the last token block's matrix instructions on chunk m, and after S(m / 2)
        const unsigned last_use = kSlots - 8u + m;
        const unsigned ready = select_slot(m / 2u) + 1u;
        return last_use > ready ? last_use : ready;
    }
};

// One work item with NTB live 32-token blocks (NTB is 1, 2 or 4).
//
// The stage in LDS holds 128 "slots" of 256 activation bytes + one scale. An item with fewer than
// 97 tokens fills them with S = 4 / NTB consecutive superblocks of its NTB * 32 tokens (slot =
// superblock within the period * NTB * 32 + token), so that every period between two barriers
// carries the same copies and 32 "time slots" of two matrix instructions each.
//
// Time slot (u, tb, m) = superblock u of the period, token block tb, K chunk m. Around its two
// matrix instructions (low and high limb) the slot carries, a few instructions at a time, the
// rest of the work: the LDS read of the activation fragment two slots ahead, the scaling of two
// rows of the previous token block's integer sums into the fp32 accumulators, one piece of the
// decode of the next superblock's weights, and this period's share of the copies and loads.
// The loop body is one period in one basic block (requests past the end are clamped, and
// superblocks past the end run with a zero row scale), so the compiler's wait counts stay exact
// and accumulators never leave registers.
template <bool FUSED_UP, unsigned NTB>
__device__ __forceinline__ void rows_item(const MfmaArgs &a, const MfmaItem &it)
{
    const GroupedProblem &pr = a.pr;
    constexpr unsigned S = 4u / NTB;                 // superblocks per stage period
    constexpr unsigned T = NTB * 32u;                // token slots of one superblock
    constexpr unsigned kSbSlots = 8u * NTB;
    constexpr unsigned kPeriodSlots = 32u;
    constexpr unsigned kBarrierSlot = kPeriodSlots - 3u;
    using Plan = DecodePlan<NTB>;
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned r = lane & 31u, h = lane >> 5;
    constexpr unsigned kItemRows = FUSED_UP ? 64u : 128u;
    const unsigned superblocks = a.width >> 8;
    const unsigned last = superblocks - 1u;

    // ---- the weight row of this lane: rows 0-15 of a wave are gate rows and rows 16-31 the
    // matching up rows when the SwiGLU is fused ----
    const unsigned char *weight_row;
    {
        unsigned row;
        bool is_up = false;
        if constexpr (FUSED_UP) {
            row = it.row_tile * kItemRows + wave * 16u + (r & 15u);
            is_up = r >= 16u;
        } else {
            row = it.row_tile * kItemRows + wave * 32u + r;
        }
        if (row >= a.out_rows) row = a.out_rows - 1u;
        weight_row = is_up
            ? pr.up + it.expert * pr.up_expert_bytes + (unsigned long long)row * pr.up_row_bytes
            : pr.gate + it.expert * pr.expert_bytes + (unsigned long long)row * pr.row_bytes;
    }
    // Superblocks are 66 bytes, so the lane's 32 code bytes start on 2-byte boundaries, and vector
    // loads that are not dword-aligned run at less than half rate: the lane loads the aligned
    // dwords around them (two 16-byte loads and a ninth dword, which repeats the eighth when the
    // codes are aligned so that nothing past the dword holding the last code byte is touched)
    // and shifts the records into place.
    const unsigned row_misalign = (unsigned)(unsigned long long)weight_row & 3u;
    const unsigned char *row_aligned = weight_row - row_misalign;
    const unsigned code_offset = row_misalign + 2u + 32u * h;       // of superblock 0's codes from row_aligned
    auto load_raw = [&](unsigned sb) {
        sb = sb < last ? sb : last;
        RawCodes out;
        const unsigned at = code_offset + sb * 66u;
        const unsigned char *from = row_aligned + (at & ~3u);
        out.x0 = load_uint4_dword_aligned(from);
        out.x1 = load_uint4_dword_aligned(from + 16u);
        out.x2 = load_u32_aligned(from + ((at & 3u) ? 32u : 28u));
        out.scale_word = load_u32_aligned(row_aligned + ((row_misalign + sb * 66u) & ~3u));
        return out;
    };

    // ---- activation rows this lane copies: wave w owns the 4-slot groups w, w + 4, ... ----
    // Lane l of a group moves piece position l % 16 of slot 4 g + l / 16; LDS receives the wave's
    // 64 pieces back to back, so the swizzle is applied on the global side.
    constexpr unsigned kCopies = kTileTokens / (4u * kRowWaves);
    auto token_row = [&](unsigned token) {
        const unsigned live = token < it.tokens ? token : it.tokens - 1u;   // padding repeats a row
        const unsigned long long ordered = it.pair0 + live;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long arow = pr.act_by_ordered_pair ? ordered : source / pr.topk;
        return (const unsigned char *)pr.activations + arow * pr.act_stride;
    };
    const unsigned char *copy_from[kCopies];
    unsigned copy_step[kCopies];            // superblock of the slot within its period
#pragma unroll
    for (unsigned j = 0; j < kCopies; ++j) {
        const unsigned slot = 4u * (wave + kRowWaves * j) + (lane >> 4);
        const unsigned token = slot % T;
        copy_step[j] = slot / T;
        copy_from[j] = token_row(token) + 4u + 16u * ((lane & 15u) ^ (token & 15u));
    }
    // Waves 0 and 1 also copy the 128 slot scales, laid out [superblock][token % 32][token block]
    // so that a lane reads the scales of its NTB tokens with one LDS read. The other waves run the
    // same instruction on one address for all lanes (one cache line: next to free) into bytes
    // nobody reads, which is cheaper than a branch around the copy.
    const unsigned char *scale_from;
    unsigned scale_step;
    {
        const unsigned index = wave < 2u ? 64u * wave + lane : 0u;
        const unsigned within = index % T;
        scale_step = index / T;
        scale_from = token_row((within % NTB) * 32u + within / NTB);
    }
    const unsigned scale_to = wave < 2u ? kStageActs + wave * 256u : 0xffffffffu;

    constexpr unsigned kCopyPieces = kCopies + 1u;
    auto copy_piece = [&](unsigned period, unsigned stage, unsigned j) {
        const unsigned base = kStageBase + stage * kStageBytes;
        if (j < kCopies) {
            unsigned sb = period * S + copy_step[j];
            sb = sb < last ? sb : last;
            copy_to_lds_16(copy_from[j] + (unsigned long long)sb * kQ8KBytes,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(base + (wave + kRowWaves * j) * 1024u)));
        } else {
            unsigned sb = period * S + scale_step;
            sb = sb < last ? sb : last;
            copy_to_lds_4(scale_from + (unsigned long long)sb * kQ8KBytes,
                          (unsigned)__builtin_amdgcn_readfirstlane(
                              (int)(scale_to != 0xffffffffu ? base + scale_to : kTrashBase)));
        }
    };

    // ---- decode state of the superblock after the current one ----
    const unsigned code_lane = kCodeBase + (lane & 31u) * 8u;
    const unsigned sel_lane = kSelBase + (lane & 15u) * 8u;
    const unsigned lut_lane = kLutBase + (lane & 15u) * 16u;
    const unsigned row_scale_at = kRowScaleBase + wave * 256u;      // + 128 for odd superblocks
    unsigned grids[4], aux[4];
    uint2 codes[2][4], signs[2][4];      // [g & 1]: of the groups whose lookups are in flight
    uint4 limbs[4];                      // limb words per group
    unsigned sel[4][8];                  // selector words per group
    v4i a_lo[8], a_hi[8];                // A operands of the current superblock, per K chunk

    // records out of the loaded dwords, and the row's scale into LDS for the lanes that hold
    // this row's sums (zero past the end: such superblocks add nothing)
    auto settle = [&](const RawCodes &raw, unsigned sb) {
        const unsigned clamped = sb < last ? sb : last;
        const unsigned shift = (code_offset + clamped * 66u) & 3u;
        const unsigned w[9] = {raw.x0.x, raw.x0.y, raw.x0.z, raw.x0.w, raw.x1.x, raw.x1.y, raw.x1.z, raw.x1.w, raw.x2};
#pragma unroll
        for (unsigned g = 0; g < 4u; ++g) {
            grids[g] = __builtin_amdgcn_alignbyte(w[2u * g + 1u], w[2u * g], shift);
            aux[g] = __builtin_amdgcn_alignbyte(w[2u * g + 2u], w[2u * g + 1u], shift);
        }
        const unsigned scale_shift = ((row_misalign + clamped * 66u) & 3u) * 8u;
        const unsigned scale16 = (raw.scale_word >> scale_shift) & 0xffffu;
        const float mine = sb < superblocks ? 0.125f * f16_bits_to_float(scale16) : 0.0f;
        lds_write_u32(row_scale_at + (sb & 1u) * 128u + r * 4u, __float_as_uint(mine));
    };
    auto lookup = [&](unsigned g) {
#pragma unroll
        for (unsigned j = 0; j < 4u; ++j) {
            codes[g & 1u][j] = lds_read_uint2(__builtin_amdgcn_perm(grids[g], code_lane, 0x0c0c0400u + (j << 8)));
            const unsigned field = j == 0u ? aux[g] << 7 : j == 1u ? aux[g] : aux[g] >> (7u * j - 7u);
            signs[g & 1u][j] = lds_read_uint2((field & 0x3f80u) | sel_lane);
        }
        limbs[g] = lds_read_uint4(((aux[g] >> 20) & 0xf00u) | lut_lane);
    };
    auto select = [&](unsigned g) {
#pragma unroll
        for (unsigned j = 0; j < 4u; ++j) {
            sel[g][2u * j] = codes[g & 1u][j].x | signs[g & 1u][j].x;
            sel[g][2u * j + 1u] = codes[g & 1u][j].y | signs[g & 1u][j].y;
        }
    };
    auto permute = [&](unsigned m) {
        const unsigned g = m >> 1, first = 4u * (m & 1u);
        a_lo[m] = v4i{(int)__builtin_amdgcn_perm(limbs[g].y, limbs[g].x, sel[g][first]),
                      (int)__builtin_amdgcn_perm(limbs[g].y, limbs[g].x, sel[g][first + 1u]),
                      (int)__builtin_amdgcn_perm(limbs[g].y, limbs[g].x, sel[g][first + 2u]),
                      (int)__builtin_amdgcn_perm(limbs[g].y, limbs[g].x, sel[g][first + 3u])};
        a_hi[m] = v4i{(int)__builtin_amdgcn_perm(limbs[g].w, limbs[g].z, sel[g][first]),
                      (int)__builtin_amdgcn_perm(limbs[g].w, limbs[g].z, sel[g][first + 1u]),
                      (int)__builtin_amdgcn_perm(limbs[g].w, limbs[g].z, sel[g][first + 2u]),
                      (int)__builtin_amdgcn_perm(limbs[g].w, limbs[g].z, sel[g][first + 3u])};
    };

    // ---- activation fragments: piece 8 h + m of slot r (+ 32 tb + T u) ----
    unsigned piece_at[8];
    auto enter_stage = [&](unsigned base) {
#pragma unroll
        for (unsigned m = 0; m < 8u; ++m) {
            // kept opaque so that the slot offset stays the instruction's immediate
            piece_at[m] = base + r * kActPitch + ((((8u * h) ^ (r & 15u)) ^ m) << 4);
            asm volatile("" : "+v"(piece_at[m]));
        }
    };
    auto stage_base = [&](unsigned period) { return kStageBase + (period & 1u) * kStageBytes; };

    // ---- prologue ----
    RawCodes raw[S];
    // The first superblocks of the weight rows are asked for before anything else: their trip to
    // HBM runs under the index loads and copies of the activation side.
    RawCodes first_raw = load_raw(0u);
#pragma unroll
    for (unsigned x = 1; x <= S; ++x) raw[x % S] = load_raw(x);

    __syncthreads();   // every wave is done with the previous item's stage and output tile
#pragma unroll
    for (unsigned j = 0; j < kCopyPieces; ++j) copy_piece(0u, 0u, j);
    // where each pair's results go and its route weight, for the publishing pass
    if (tid < kTileTokens && tid < it.tokens) {
        const unsigned long long ordered = it.pair0 + tid;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long out_index = pr.out_by_source_pair ? source : ordered;
        const float route_weight = pr.route_weights ? pr.route_weights[source] : 1.0f;
        lds_write_uint2(kPairInfoBase + tid * 8u, make_uint2((unsigned)out_index, __float_as_uint(route_weight)));
    }
    settle(first_raw, 0u);
#pragma unroll
    for (unsigned g = 0; g < 4u; ++g) {
        lookup(g);
        select(g);
    }
#pragma unroll
    for (unsigned m = 0; m < 8u; ++m) permute(m);
    __builtin_amdgcn_s_waitcnt(0x0070u);   // vmcnt(0) lgkmcnt(0): the copies above have landed
    __syncthreads();

    float acc[NTB][16];
#pragma unroll
    for (unsigned tb = 0; tb < NTB; ++tb)
#pragma unroll
        for (unsigned i = 0; i < 16u; ++i) acc[tb][i] = 0.0f;
    float rs[16];                    // row scales of the rows this lane holds sums of
#pragma unroll
    for (unsigned i = 0; i < 16u; ++i) rs[i] = 0.0f;
    float ts[NTB];                   // activation scales of this lane's token per token block
    float ts_before = 0.0f;          // of the last token block of the superblock before
#pragma unroll
    for (unsigned tb = 0; tb < NTB; ++tb) ts[tb] = 0.0f;
    v16i sum_lo[2], sum_hi[2];       // [phase & 1]: integer sums of a token block, scaled one phase later
#pragma unroll
    for (unsigned i = 0; i < 16u; ++i) {
        sum_lo[1][i] = 0;
        sum_hi[1][i] = 0;
    }
    v4i frag[2];                     // [slot & 1]: re-requested for two slots on as soon as it is used
    enter_stage(stage_base(0u));
    frag[0] = lds_read_v4i(piece_at[0]);
    frag[1] = lds_read_v4i(piece_at[1]);

    auto scale_rows = [&](unsigned parity, unsigned tb_of, float token_scale, unsigned m) {
#pragma unroll
        for (unsigned i = 2u * m; i < 2u * m + 2u; ++i) {
            const int total = (sum_hi[parity][i] << 7) + sum_lo[parity][i];
            acc[tb_of][i] = __builtin_fmaf(rs[i] * token_scale, (float)total, acc[tb_of][i]);
        }
    };

    const unsigned periods = (superblocks + S - 1u) / S;
    for (unsigned period = 0; period < periods; ++period) {
        const unsigned base = stage_base(period);
#pragma unroll
        for (unsigned u = 0; u < S; ++u) {
            const unsigned sb = period * S + u;           // this superblock
#pragma unroll
            for (unsigned tb = 0; tb < NTB; ++tb) {
                const unsigned phase = u * NTB + tb;
                const unsigned parity = phase & 1u;
#pragma unroll
                for (unsigned m = 0; m < 8u; ++m) {
                    const unsigned slot = phase * 8u + m;         // within the period
                    const unsigned sb_slot = tb * 8u + m;         // within the superblock
                    // ---- two matrix instructions ----
                    const v4i b = frag[slot & 1u];
                    if (m == 0u) {
                        v16i zero;
#pragma unroll
                        for (unsigned i = 0; i < 16u; ++i) zero[i] = 0;
                        sum_lo[parity] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_lo[0], b, zero, 0, 0, 0);
                        sum_hi[parity] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_hi[0], b, zero, 0, 0, 0);
                    } else {
                        sum_lo[parity] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_lo[m], b, sum_lo[parity], 0, 0, 0);
                        sum_hi[parity] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_hi[m], b, sum_hi[parity], 0, 0, 0);
                    }
                    // ---- this superblock's token scales at its start ----
                    if (sb_slot == 0u) {
                        ts_before = ts[NTB - 1u];
                        const unsigned at = base + kStageActs + (u * T + r * NTB) * 4u;
                        if constexpr (NTB == 4u) {
                            const uint4 v = lds_read_uint4(at);
                            ts[0] = __uint_as_float(v.x);
                            ts[1] = __uint_as_float(v.y);
                            ts[2] = __uint_as_float(v.z);
                            ts[3] = __uint_as_float(v.w);
                        } else if constexpr (NTB == 2u) {
                            const uint2 v = lds_read_uint2(at);
                            ts[0] = __uint_as_float(v.x);
                            ts[1] = __uint_as_float(v.y);
                        } else {
                            ts[0] = __uint_as_float(lds_read_u32(at));
                        }
                    }
                    // ---- the fragment two slots on (past the barrier slot the addresses already
                    // point into the next period's stage) ----
                    {
                        const unsigned within = (slot + 2u) % kPeriodSlots;
                        const unsigned phase_of = within / 8u;
                        frag[slot & 1u] = lds_read_v4i(piece_at[within % 8u] +
                                                       ((phase_of / NTB) * T + (phase_of % NTB) * 32u) * kActPitch);
                    }
                    // ---- scaling of two rows of the token block before this one ----
                    scale_rows(parity ^ 1u, tb ? tb - 1u : NTB - 1u, tb ? ts[tb - 1u] : ts_before, m);
                    // ---- this superblock's share of the decode of the next one ----
                    if (sb_slot == 0u) settle(raw[(u + 1u) % S], sb + 1u);
                    if (sb_slot == 1u) raw[(u + 1u) % S] = load_raw(sb + 1u + S);
#pragma unroll
                    for (unsigned g = 0; g < 4u; ++g) {
                        if (sb_slot == Plan::select_slot(g)) select(g);
                        if (sb_slot == Plan::lookup_slot(g)) lookup(g);
                    }
#pragma unroll
                    for (unsigned k = 0; k < 8u; ++k)
                        if (sb_slot == Plan::permute_slot(k)) permute(k);
                    // ---- the row scales of this superblock, once the last sums of the one before
                    // have been scaled ----
                    if (sb_slot == 7u) {
#pragma unroll
                        for (unsigned q = 0; q < 4u; ++q) {
                            const uint4 v = lds_read_uint4(row_scale_at + (sb & 1u) * 128u + (8u * q + 4u * h) * 4u);
                            rs[4u * q] = __uint_as_float(v.x);
                            rs[4u * q + 1u] = __uint_as_float(v.y);
                            rs[4u * q + 2u] = __uint_as_float(v.z);
                            rs[4u * q + 3u] = __uint_as_float(v.w);
                        }
                    }
                    // ---- the next period's copies, one a slot ----
                    if (slot < kCopyPieces) copy_piece(period + 1u, (period + 1u) & 1u, slot);
                    if (slot == kBarrierSlot) {
                        // every activation read of this period has returned and the next period's
                        // copies have landed: after the barrier nobody reads this stage again
                        __builtin_amdgcn_s_waitcnt(0x0070u);
                        __syncthreads();
                        const unsigned flip = (period & 1u) ? 0u - kStageBytes : kStageBytes;
#pragma unroll
                        for (unsigned k = 0; k < 8u; ++k) piece_at[k] += flip;
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }
    // the last token block of the last superblock
#pragma unroll
    for (unsigned m = 0; m < 8u; ++m) scale_rows(1u, NTB - 1u, ts[NTB - 1u], m);

    // ---- publish: the lane holds, for tokens 32 tb + r, rows 8 q + 4 h + j of its 32 (j < 4) ----
    // The tile goes through LDS as [token][value], values 0-63 the gate sums and 64-127 the up
    // sums of the item's 64 row pairs when fused, else the 128 rows' sums.
#pragma unroll
    for (unsigned tb = 0; tb < NTB; ++tb)
#pragma unroll
        for (unsigned q = 0; q < 4u; ++q) {
            unsigned column;
            if constexpr (FUSED_UP) column = (q >= 2u ? 64u : 0u) + wave * 16u + 8u * (q & 1u) + 4u * h;
            else column = wave * 32u + 8u * q + 4u * h;
            lds_write_uint4(kStageBase + (tb * 32u + r) * kOutPitch + column * 4u,
                            make_uint4(__float_as_uint(acc[tb][4u * q]), __float_as_uint(acc[tb][4u * q + 1u]),
                                       __float_as_uint(acc[tb][4u * q + 2u]), __float_as_uint(acc[tb][4u * q + 3u])));
        }
    __syncthreads();
    auto store4 = [&](unsigned long long out_index, unsigned row, const float (&value)[4]) {
        const bool good = finite_f32(value[0]) && finite_f32(value[1]) && finite_f32(value[2]) &&
                          finite_f32(value[3]);
        if (!good) raise_status(a.status, 1);
        else if (row + 3u < a.out_rows)
            *reinterpret_cast<float4 *>(pr.out + out_index * a.out_rows + row) =
                make_float4(value[0], value[1], value[2], value[3]);
        else
            for (unsigned j = 0; j < 4u; ++j)
                if (row + j < a.out_rows) pr.out[out_index * a.out_rows + row + j] = value[j];
    };
    constexpr unsigned kQuads = kItemRows / 4u;       // groups of four output values per token
    const float limit_f32 = (float)a.limit;
#pragma unroll 1
    for (unsigned unit = tid; unit < T * kQuads; unit += kRowThreads) {
        const unsigned token = unit / kQuads, quad = unit % kQuads;
        if (token >= it.tokens) break;
        const uint2 info = lds_read_uint2(kPairInfoBase + token * 8u);
        const unsigned row = it.row_tile * kItemRows + 4u * quad;
        if (row >= a.out_rows) continue;
        const uint4 g = lds_read_uint4(kStageBase + token * kOutPitch + quad * 16u);
        if constexpr (FUSED_UP) {
            const uint4 up = lds_read_uint4(kStageBase + token * kOutPitch + 256u + quad * 16u);
            const float route_weight = __uint_as_float(info.y);
            const float value[4] = {
                swiglu_bf16_fast(__uint_as_float(g.x), __uint_as_float(up.x), route_weight, a.limit, limit_f32),
                swiglu_bf16_fast(__uint_as_float(g.y), __uint_as_float(up.y), route_weight, a.limit, limit_f32),
                swiglu_bf16_fast(__uint_as_float(g.z), __uint_as_float(up.z), route_weight, a.limit, limit_f32),
                swiglu_bf16_fast(__uint_as_float(g.w), __uint_as_float(up.w), route_weight, a.limit, limit_f32)};
            store4(info.x, row, value);
        } else {
            const float value[4] = {bf16_round(__uint_as_float(g.x)), bf16_round(__uint_as_float(g.y)),
                                    bf16_round(__uint_as_float(g.z)), bf16_round(__uint_as_float(g.w))};
            store4(info.x, row, value);
        }
    }
}

template <bool FUSED_UP>
__global__ __launch_bounds__(kRowThreads) void mfma_iq2_kernel(MfmaArgs a)
{
    extern __shared__ __align__(16) unsigned char mfma_lds[];
    if (lds_address_of(mfma_lds) != 0u) {   // the lookups address LDS by absolute byte offsets
        if (threadIdx.x == 0u) raise_status(a.status, 2);
        return;
    }
    const GroupedProblem &pr = a.pr;
    const unsigned tid = threadIdx.x;
    const bool fixed = pr.expert_ids == nullptr;
    const unsigned buckets = fixed ? 1u : (unsigned)pr.counts[0];

    mfma_tables_fill();
    if (tid == 0u) {
        // Full 128-pair tiles come first in the item list, then the partial last tiles by size,
        // largest first: every workgroup, walking the list with the grid's stride, gets the same
        // share of each kind of item, and the short items come last.
        unsigned cursor = 0u, members[3] = {0u, 0u, 0u};
        for (unsigned b = 0; b < buckets && b < 256u; ++b) {
            lds_write_u32(kTileStartBase + 4u * b, cursor);
            const unsigned long long n = fixed ? pr.pairs : pr.bucket_populations[b];
            cursor += (unsigned)(n / kTileTokens);
            const unsigned rest = (unsigned)(n % kTileTokens);
            if (rest) {
                const unsigned c = rest > 64u ? 0u : rest > 32u ? 1u : 2u;
                lds_write_u16(kClassListBase + (c * 256u + members[c]) * 2u, b);
                ++members[c];
            }
        }
        lds_write_u32(kTileStartBase + 4u * (buckets < 256u ? buckets : 256u), cursor);
        for (unsigned c = 0; c < 3u; ++c) lds_write_u32(kClassCountBase + 4u * c, members[c]);
    }
    __syncthreads();
    if (buckets == 0u || buckets > 256u) {
        if (tid == 0u && buckets > 256u) raise_status(a.status, 2);
        return;
    }

    // weight rows (gate/up row pairs when fused) per work item
    constexpr unsigned kItemRows = FUSED_UP ? 64u : 128u;
    const unsigned row_tiles = (a.out_rows + kItemRows - 1u) / kItemRows;
    const unsigned long long full_items = (unsigned long long)lds_read_u32(kTileStartBase + 4u * buckets) * row_tiles;
    unsigned members[3];
    unsigned long long items = full_items;
    for (unsigned c = 0; c < 3u; ++c) {
        members[c] = lds_read_u32(kClassCountBase + 4u * c);
        items += (unsigned long long)members[c] * row_tiles;
    }

    for (unsigned long long item = blockIdx.x; item < items; item += gridDim.x) {
        // ---- which bucket, row tile and token tile ----
        unsigned bucket, token_tile;
        MfmaItem it;
        if (item < full_items) {
            unsigned low = 0u, high = buckets;   // the last bucket whose first full tile is <= item's
            while (low + 1u < high) {
                const unsigned middle = (low + high) >> 1;
                if ((unsigned long long)lds_read_u32(kTileStartBase + 4u * middle) * row_tiles <= item)
                    low = middle;
                else
                    high = middle;
            }
            const unsigned tile_first = lds_read_u32(kTileStartBase + 4u * low);
            const unsigned bucket_tiles = lds_read_u32(kTileStartBase + 4u * (low + 1u)) - tile_first;
            const unsigned long long local = item - (unsigned long long)tile_first * row_tiles;
            if (!bucket_tiles) {
                if (tid == 0u) raise_status(a.status, 2);
                continue;
            }
            bucket = low;
            token_tile = (unsigned)(local % bucket_tiles);
            it.row_tile = (unsigned)(local / bucket_tiles);
        } else {
            unsigned long long rest = item - full_items;
            unsigned c = 0u;
            while (c < 2u && rest >= (unsigned long long)members[c] * row_tiles) {
                rest -= (unsigned long long)members[c] * row_tiles;
                ++c;
            }
            if (!members[c]) {
                if (tid == 0u) raise_status(a.status, 2);
                continue;
            }
            bucket = lds_read_u16(kClassListBase + (c * 256u + (unsigned)(rest % members[c])) * 2u);
            it.row_tile = (unsigned)(rest / members[c]);
            const unsigned long long n = fixed ? pr.pairs : pr.bucket_populations[bucket];
            token_tile = (unsigned)(n / kTileTokens);
        }
        const unsigned long long first = fixed ? 0ull : pr.bucket_offsets[bucket];
        const unsigned long long population = fixed ? pr.pairs : pr.bucket_populations[bucket];
        it.expert = fixed ? 0ull : pr.expert_ids[bucket];
        if (bucket >= buckets || it.expert >= pr.experts || first + population > pr.pairs ||
            (unsigned long long)token_tile * kTileTokens >= population || it.row_tile >= row_tiles) {
            if (tid == 0u) raise_status(a.status, 2);
            continue;
        }
        const unsigned long long left = population - (unsigned long long)token_tile * kTileTokens;
        it.pair0 = first + (unsigned long long)token_tile * kTileTokens;
        it.tokens = left < kTileTokens ? (unsigned)left : kTileTokens;
        if (it.tokens <= 32u) rows_item<FUSED_UP, 1u>(a, it);
        else if (it.tokens <= 64u) rows_item<FUSED_UP, 2u>(a, it);
        else rows_item<FUSED_UP, 4u>(a, it);
    }
}

static int mfma_grid()
{
    static int units = 0;
    if (!units) {
        int device = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&device) != hipSuccess || hipGetDeviceProperties(&prop, device) != hipSuccess) {
            (void)hipGetLastError();
            return 256;
        }
        units = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    return units;
}

template <bool FUSED_UP>
static int launch_mfma(const MfmaArgs &a, hipStream_t stream)
{
    static bool configured = false;
    if (!configured) {
        if (hipFuncSetAttribute((const void *)mfma_iq2_kernel<FUSED_UP>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaLdsBytes) != hipSuccess)
            (void)hipGetLastError();
        configured = true;
    }
    mfma_iq2_kernel<FUSED_UP><<<mfma_grid(), kRowThreads, kMfmaLdsBytes, stream>>>(a);
    return check_launch("moe_rows_mfma");
}

}  // namespace yvex

using namespace yvex;


extern "C" int yvex_hip_moe_up_rows(const yvex_hip_expert_weights *w, const void *act_q8k,
                                    const float *route_weights, const uint64_t *order,
                                    const uint64_t *expert_ids, const uint64_t *bucket_offsets,
                                    const uint64_t *bucket_populations, const uint64_t *counts,
                                    uint64_t pairs, uint64_t topk, uint64_t experts, double limit,
                                    float *intermediate, int *status, yvex_hip_stream stream)
{
    if (!w || !w->gate || !w->up || !act_q8k || !intermediate || !status || !pairs || !topk ||
        !experts || !(limit > 0.0) || (expert_ids && (!bucket_offsets || !bucket_populations || !counts)))
        return ST_INVALID_ARG;
    if (w->gate_qtype != QT_IQ2_XXS || w->up_qtype != QT_IQ2_XXS) return ST_UNSUPPORTED;
    int rc = check_matrix(w->gate_qtype, w->hidden, w->gate_row_bytes);
    if (rc) return rc;
    if (w->up_row_bytes != w->gate_row_bytes) return ST_BOUNDS;
    if (pairs > 0xffffffffull || w->intermediate > 0xffffffffull || w->intermediate % 4u) return ST_BOUNDS;
    MfmaArgs a{};
    const WorklistView wl{order, expert_ids, bucket_offsets, bucket_populations, nullptr, counts};
    fill_up_problem(a.pr, w, act_q8k, 1, route_weights, wl, pairs, topk, experts, intermediate);
    a.width = (unsigned)w->hidden;
    a.out_rows = (unsigned)w->intermediate;
    a.limit = limit;
    a.status = status;
    return launch_mfma<true>(a, as_stream(stream));
}

extern "C" int yvex_hip_moe_down_rows(const yvex_hip_expert_weights *w, const void *intermediate_q8k,
                                      const uint64_t *order, const uint64_t *expert_ids,
                                      const uint64_t *bucket_offsets,
                                      const uint64_t *bucket_populations, const uint64_t *counts,
                                      uint64_t pairs, uint64_t experts, float *pair_outputs,
                                      int *status, yvex_hip_stream stream)
{
    if (!w || !w->down || !intermediate_q8k || !pair_outputs || !status || !pairs || !experts ||
        (expert_ids && (!bucket_offsets || !bucket_populations || !counts)))
        return ST_INVALID_ARG;
    if (w->down_qtype != QT_IQ2_XXS) return ST_UNSUPPORTED;
    int rc = check_matrix(w->down_qtype, w->intermediate, w->down_row_bytes);
    if (rc) return rc;
    if (pairs > 0xffffffffull || w->hidden > 0xffffffffull || w->hidden % 4u) return ST_BOUNDS;
    MfmaArgs a{};
    const WorklistView wl{order, expert_ids, bucket_offsets, bucket_populations, nullptr, counts};
    fill_down_problem(a.pr, w, intermediate_q8k, 1, wl, pairs, experts, pair_outputs);
    a.width = (unsigned)w->intermediate;
    a.out_rows = (unsigned)w->hidden;
    a.limit = 1.0;
    a.status = status;
    return launch_mfma<false>(a, as_stream(stream));
}
