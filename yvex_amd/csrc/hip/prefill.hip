// Row-batch (prefill-width) grouped expert projections on the int8 matrix cores of gfx950.
//
// A work item is (bucket, tile of 128 ordered pairs, tile of weight rows). The workgroup's eight
// waves split the weight rows, 16 each (four gate blocks and the four matching up blocks when the
// SwiGLU is fused); every wave multiplies its rows by the item's 128 Q8_K activation rows with
// V_MFMA_I32_16X16X64_I8. Two waves share a SIMD, so one wave's decode and scaling arithmetic
// runs under the other's matrix instructions.
//
//   A operand (weights): each lane builds the 16 weights it owns straight into registers. The
//       IQ2_XXS value of one weight is level * sign * (2s+1), up to 43 * 31 = 1333, so it is
//       split into two int8 limbs, value = 128 * hi + lo with hi in [1, 11] and lo in
//       [-120, 63]. For a given scale there are only three levels, so the six signed limb
//       values of a group fit two registers and one V_PERM_B32 per four weights picks them:
//       the selector byte of a weight is its level code (0..2) plus 4 when it is negative.
//       Three small conflict-free LDS tables feed this: level codes of a codebook entry
//       (8 bytes), sign selectors of a 7-bit sign field (8 bytes) and the limb words of a
//       scale (16 bytes).
//   B operand (activations): the 128 x 256 int8 block of the current superblock, copied from
//       global memory straight into LDS (GLOBAL_LOAD_LDS_DWORDX4, no registers in between),
//       double buffered. 16-byte piece c of token t sits at piece position c ^ (t % 16), so the
//       16 lanes that read one fragment column together hit 16 different bank groups.
//   C: per superblock two int32 accumulators per 16 x 16 block; T = 128 * C_hi + C_lo is the
//       exact integer superblock sum of the reference's primitive
//       (src/backend/cuda/kernel_primitives.h:287-313), scaled into fp32 as
//       ((0.125 * d_w) * d_a) * T and summed over superblocks.
//
// Same inputs, outputs and rounding points as the decode-width sweeps in moe.hip
// (src/backend/cuda/tensorcore.cu:378-702 is the reference's counterpart, unused there).
#include "common.hpp"
#include "launch.hpp"
#include "grouped.hpp"

namespace yvex {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr unsigned kTileTokens = 128u;
constexpr unsigned kActPitch = 256u;                       // one Q8_K block's int8 payload
// LDS map. Codebook entry e owns the 256 bytes at 256 e: sixteen replicas of its 8 level codes
// in the first half; the second half of entries 0-127 holds sixteen replicas of the sign
// selectors of sign field e.
constexpr unsigned kCodeBase = 0u;
constexpr unsigned kSelBase = 128u;
constexpr unsigned kLutBase = 65536u;                       // 16 scales x 16 replicas x 16 bytes
constexpr unsigned kStageBase = kLutBase + 16u * 16u * 16u;
constexpr unsigned kStageActs = kTileTokens * kActPitch;
constexpr unsigned kStageBytes = kStageActs + kTileTokens * 4u;   // + one fp32 scale per token
// Weight windows: per wave two slots; a slot holds, for each of the wave's 16 rows, the 80
// bytes (five 16-byte pieces) around one superblock. Rows 0-11 lie at 80 r, rows 12-15 at
// 1024 + 80 (r - 12): the two copies that fill a slot each write lane * 16.
constexpr unsigned kWeightBase = kStageBase + 2u * kStageBytes;
constexpr unsigned kWeightSlot = 1024u + 4u * 80u;
// Item numbering: first full 128-pair tile of every bucket (257 words), then per class of last,
// partial, tile (65-127, 33-64, 17-32, 1-16 pairs) a count and the list of its buckets (u16).
constexpr unsigned kTileStartBase = kWeightBase + 8u * 2u * kWeightSlot;
constexpr unsigned kClassCountBase = kTileStartBase + 260u * 4u;
constexpr unsigned kClassListBase = kClassCountBase + 16u;
constexpr unsigned kTrashBase = kClassListBase + 4u * 256u * 2u;   // 256 bytes nobody reads
// per pair of the item: {output row index, route weight}, read when the item publishes
constexpr unsigned kPairInfoBase = kTrashBase + 256u;
constexpr unsigned kMfmaLdsBytes = kPairInfoBase + kTileTokens * 8u;

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
__device__ __forceinline__ void lds_write_u32(unsigned address, unsigned v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) unsigned *>(address) = v;
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
__device__ __forceinline__ void lds_write_u16(unsigned address, unsigned v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) unsigned short *>(address) = (unsigned short)v;
#else
    (void)address;
    (void)v;
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
// does not put a conservative wait in front of every later LDS read: the caller waits with
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

// The same 16-byte copy for lanes 0-19 only (the other lanes neither read nor write).
__device__ __forceinline__ void copy_to_lds_16_first20(const void *global, unsigned lds_base)
{
#if defined(__HIP_DEVICE_COMPILE__)
    unsigned long long saved;
    asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 0xfffff\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %2, off\n\ts_mov_b64 exec, %0"
                 : "=&s"(saved) : "s"(lds_base), "v"(global) : "memory");
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

__device__ __forceinline__ void lds_write_uint2(unsigned address, uint2 v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) uint2 *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}

__device__ __forceinline__ void mfma_tables_fill()
{
    // level codes: byte l of the entry is 0, 1 or 2 for level 8, 25 or 43 of weight l
    for (unsigned index = threadIdx.x; index < 256u * 16u; index += blockDim.x) {
        const uint2 m = iq2_magnitude_entry(index >> 4);
        uint2 codes = make_uint2(0u, 0u);
#pragma unroll
        for (unsigned l = 0; l < 4u; ++l) {
            const unsigned a = (m.x >> (8u * l)) & 255u, b = (m.y >> (8u * l)) & 255u;
            codes.x |= (a == 8u ? 0u : a == 25u ? 1u : 2u) << (8u * l);
            codes.y |= (b == 8u ? 0u : b == 25u ? 1u : 2u) << (8u * l);
        }
        lds_write_uint2(kCodeBase + (index >> 4) * 256u + (index & 15u) * 8u, codes);
    }
    // sign selectors: byte l is 4 when weight l is negative (7 stored bits + parity)
    for (unsigned index = threadIdx.x; index < 128u * 16u; index += blockDim.x) {
        const uint2 m = iq2_signmask_entry(index >> 4);
        lds_write_uint2(kSelBase + (index >> 4) * 256u + (index & 15u) * 8u,
                        make_uint2(m.x & 0x04040404u, m.y & 0x04040404u));
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

// Twelve aligned bytes that hold one 8-byte group record starting 0 or 2 bytes in.
struct alignas(4) RawGroup {
    unsigned x, y, z;
};

// The lane's four group records and block scale of one superblock of its weight row.
struct Codes {
    uint2 c[4];
    unsigned scale16;
};
// Table words of the lane's sixteen weights in one K step.
struct Lookup {
    uint2 codes[2], signs[2];
    uint4 limbs;
};

// One work item with NB live 16-token blocks (NB is 1, 2, 4 or 8). Eight waves, two per SIMD, each
// owning one 16-row block.
//
// The stage in LDS holds 128 "slots" of 256 activation bytes + one scale. An item with fewer than
// 128 tokens fills them with S consecutive superblocks of its NB * 16 tokens (slot = superblock
// within the period * NB * 16 + token), so that every period between two barriers carries about
// the same matrix work and the same copies whatever NB is.
//
// A step is one superblock. Its instruction stream is laid out by hand as 4 * NB slots of two
// matrix instructions (low and high limb of one K step of one token block), and between them,
// a few vector instructions at a time, everything else: the scaling of the previous token
// block's integer sums into the fp32 accumulators, the table lookups and byte permutes that
// build the next superblock's A operands, the LDS reads of the next token block's fragments.
// The loop body holds D steps back to back in one basic block (requests past the end are
// clamped, and steps past the end run with a zero row scale), so the compiler's wait counts stay
// exact and accumulators never leave registers.
template <bool FUSED_UP, unsigned NB>
__device__ __forceinline__ void mfma_item(const MfmaArgs &a, const MfmaItem &it)
{
    const GroupedProblem &pr = a.pr;
    constexpr unsigned kWaves = 8u;
    constexpr unsigned S = NB >= 8u ? 1u : NB == 4u ? 2u : 4u;   // superblocks per stage period
    constexpr unsigned D = S < 2u ? 2u : S;                      // steps per loop turn (even)
    constexpr unsigned T = NB * 16u;                             // token slots of one superblock
    constexpr unsigned kStagedSlots = S * T;
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned li = lane & 15u, kb = lane >> 4;
    constexpr unsigned kItemRows = FUSED_UP ? 64u : 128u;
    const unsigned code_lane = kCodeBase + (lane & 15u) * 8u;
    const unsigned sel_lane = kSelBase + (lane & 15u) * 8u;
    const unsigned lut_lane = kLutBase + (lane & 15u) * 16u;
    const unsigned superblocks = a.width >> 8;
    const unsigned last = superblocks - 1u;

    // ---- the weight row of this lane: waves 0-3 hold gate blocks and waves 4-7 the matching up
    // blocks when the SwiGLU is fused ----
    unsigned out_row_base;
    bool is_up = false;
    if constexpr (FUSED_UP) {
        out_row_base = it.row_tile * kItemRows + (wave & 3u) * 16u;
        is_up = wave >= 4u;
    } else {
        out_row_base = it.row_tile * kItemRows + wave * 16u;
    }
    auto row_pointer = [&](unsigned r) {     // weight row r of the wave's 16
        unsigned row = out_row_base + r;
        if (row >= a.out_rows) row = a.out_rows - 1u;
        return is_up
            ? pr.up + it.expert * pr.up_expert_bytes + (unsigned long long)row * pr.up_row_bytes
            : pr.gate + it.expert * pr.expert_bytes + (unsigned long long)row * pr.row_bytes;
    };
    // Superblocks are 66 bytes, so they start on 2-byte boundaries, and vector loads that are
    // not dword-aligned run at less than half rate. The wave copies, for each of its rows, the
    // aligned 68 bytes that hold the superblock into its LDS slot, as five 16-byte pieces (the
    // fifth one ends with those 68 bytes, so nothing past the dword that holds the superblock's
    // last byte is touched: an aligned dword with a valid byte lies in a mapped page). Two
    // copies fill a slot: lanes 0-59 of the first serve rows 0-11, lanes 0-19 of the second
    // rows 12-15. Every row is fetched once per step by five lanes instead of by all four lane
    // groups record by record: the memory pipeline's cost per instruction grows with the number
    // of cache lines it touches.
    const unsigned row_misalign = (unsigned)(unsigned long long)row_pointer(li) & 3u;   // of the lane's own row
    const unsigned lane_group = kb >> 1;                      // groups 2 ks + lane_group
    const unsigned char *window_from[2];    // aligned row start + piece offset, of the row this lane copies
    unsigned window_misalign[2];
#pragma unroll
    for (unsigned c = 0; c < 2u; ++c) {
        const unsigned served = c == 0u ? (lane < 60u ? lane : 0u) : (lane < 20u ? 60u + lane : 60u);
        const unsigned piece_index = served % 5u;
        const unsigned char *from = row_pointer(served / 5u);
        window_misalign[c] = (unsigned)(unsigned long long)from & 3u;
        window_from[c] = from - window_misalign[c] + (piece_index < 4u ? 16u * piece_index : 52u);
    }
    const unsigned weight_slots = kWeightBase + wave * 2u * kWeightSlot;
    const unsigned row_at = li < 12u ? li * 80u : 1024u + (li - 12u) * 80u;   // of the lane's row in a slot
    constexpr unsigned kFetchPieces = 2u;
    auto fetch_piece = [&](unsigned slot, unsigned sb, unsigned c) {
        sb = sb < last ? sb : last;
        const unsigned char *from = window_from[c] + ((window_misalign[c] + sb * 66u) & ~3u);
        const unsigned to = (unsigned)__builtin_amdgcn_readfirstlane((int)(weight_slots + slot * kWeightSlot + c * 1024u));
        if (c == 0u) copy_to_lds_16(from, to);
        else copy_to_lds_16_first20(from, to);
    };
    auto fetch_codes = [&](unsigned slot, unsigned sb) {
#pragma unroll
        for (unsigned c = 0; c < kFetchPieces; ++c) fetch_piece(slot, sb, c);
    };
    // The first two superblocks of the weight rows are asked for before anything else: their
    // trip to HBM runs under the index loads and copies of the activation side below.
    fetch_codes(0u, 0u);
    fetch_codes(1u, 1u);

    // ---- activation rows this lane copies: wave w owns the 4-slot groups w, w + kWaves, ... ----
    // Lane l of a group moves piece position l % 16 of slot 4 g + l / 16; LDS receives the wave's
    // 64 pieces back to back, so the swizzle is applied on the global side.
    constexpr unsigned kCopies = kStagedSlots / (4u * kWaves);
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
        const unsigned slot = 4u * (wave + kWaves * j) + (lane >> 4);
        const unsigned token = slot % T;
        copy_step[j] = slot / T;
        copy_from[j] = token_row(token) + 4u + 16u * ((lane & 15u) ^ (token & 15u));
    }
    // Waves 0 and 1 also copy the 128 slot scales. The other waves run the same instruction on
    // one address for all lanes (one cache line: next to free) into bytes nobody reads, which is
    // cheaper than a branch around the copy.
    const unsigned scale_slot = wave < 2u ? 64u * wave + lane : 0u;
    const unsigned char *scale_from = token_row(scale_slot % T);
    const unsigned scale_step = scale_slot / T;
    const unsigned scale_to = wave < 2u ? kStageActs + wave * 256u : 0xffffffffu;

    // The copies and loads of a step are issued one piece at a time between its matrix
    // instructions: a burst of them fills the memory pipeline's queue and holds the wave, and
    // with it its matrix instructions, until the queue drains.
    constexpr unsigned kCopyPieces = kCopies + 1u;
    auto copy_piece = [&](unsigned period, unsigned stage, unsigned j) {
        const unsigned base = kStageBase + stage * kStageBytes;
        if (j < kCopies) {
            unsigned sb = period * S + copy_step[j];
            sb = sb < last ? sb : last;
            copy_to_lds_16(copy_from[j] + (unsigned long long)sb * kQ8KBytes,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(base + (wave + kWaves * j) * 1024u)));
        } else {
            unsigned sb = period * S + scale_step;
            sb = sb < last ? sb : last;
            copy_to_lds_4(scale_from + (unsigned long long)sb * kQ8KBytes,
                          (unsigned)__builtin_amdgcn_readfirstlane(
                              (int)(scale_to != 0xffffffffu ? base + scale_to : kTrashBase)));
        }
    };
    auto copy_activations = [&](unsigned period, unsigned stage) {
#pragma unroll
        for (unsigned j = 0; j < kCopyPieces; ++j) copy_piece(period, stage, j);
    };
    // Records of superblock sb out of the slot fetch_codes(slot, sb) filled. With o = (row start
    // + 2 sb) mod 4 (0 or 2) the fp16 scale sits o bytes into the window and the record of group
    // G at o + 2 + 8 G: in dwords 2 G (+1 when o is 2), shifted by 2 bytes when o is 0. Window
    // dword 16 is the last dword of the fifth piece.
    auto settle_codes = [&](unsigned slot, unsigned sb) {
        sb = sb < last ? sb : last;
        Codes out;
        const unsigned o = (row_misalign + 2u * sb) & 3u;
        const unsigned shift = (o + 2u) & 3u;
        const unsigned row_base = weight_slots + slot * kWeightSlot + row_at;
        const unsigned first = row_base + 8u * lane_group + (o & 2u) * 2u;    // dword 2 g (+1) of the window
        out.scale16 = (lds_read_u32(row_base) >> (8u * o)) & 0xffffu;
#pragma unroll
        for (unsigned ks = 0; ks < 4u; ++ks) {
            unsigned x, y, z;
            if (ks < 3u) {
                x = lds_read_u32(first + 16u * ks);
                y = lds_read_u32(first + 16u * ks + 4u);
                z = lds_read_u32(first + 16u * ks + 8u);
            } else {
                // dwords 12 + 2 g (+1) and the two behind it; 16 lives 12 bytes further on, and
                // 17 is never part of a record (it is read as 16 and shifted out)
                const unsigned d0 = 12u + 2u * lane_group + (o >> 1);
                const unsigned d1 = d0 + 1u, d2 = d0 + 2u < 16u ? d0 + 2u : 16u;
                x = lds_read_u32(row_base + 4u * d0);
                y = lds_read_u32(row_base + 4u * d1 + (d1 == 16u ? 12u : 0u));
                z = lds_read_u32(row_base + 4u * d2 + (d2 == 16u ? 12u : 0u));
            }
            out.c[ks].x = __builtin_amdgcn_alignbyte(y, x, shift);
            out.c[ks].y = __builtin_amdgcn_alignbyte(z, y, shift);
        }
        return out;
    };
    // the lane's sixteen weights of K step ks: subgroups 2 (kb & 1) and 2 (kb & 1) + 1 of its group
    auto lookup = [&](const Codes &codes, unsigned ks) {
        Lookup out;
        const unsigned grids = codes.c[ks].x >> (16u * (kb & 1u));
        const unsigned aux = codes.c[ks].y;
        const unsigned signs = aux >> (14u * (kb & 1u));
        out.codes[0] = lds_read_uint2(__builtin_amdgcn_perm(grids, code_lane, 0x0c0c0400u));
        out.codes[1] = lds_read_uint2(__builtin_amdgcn_perm(grids, code_lane, 0x0c0c0500u));
        out.signs[0] = lds_read_uint2(((signs << 8) & 0x7f00u) | sel_lane);
        out.signs[1] = lds_read_uint2(((signs << 1) & 0x7f00u) | sel_lane);
        out.limbs = lds_read_uint4(((aux >> 20) & 0xf00u) | lut_lane);
        return out;
    };
    auto weights_from_lookup = [&](const Lookup &lk, v4i &a_lo, v4i &a_hi) {
        const unsigned s0 = lk.codes[0].x | lk.signs[0].x, s1 = lk.codes[0].y | lk.signs[0].y;
        const unsigned s2 = lk.codes[1].x | lk.signs[1].x, s3 = lk.codes[1].y | lk.signs[1].y;
        a_lo = v4i{(int)__builtin_amdgcn_perm(lk.limbs.y, lk.limbs.x, s0),
                   (int)__builtin_amdgcn_perm(lk.limbs.y, lk.limbs.x, s1),
                   (int)__builtin_amdgcn_perm(lk.limbs.y, lk.limbs.x, s2),
                   (int)__builtin_amdgcn_perm(lk.limbs.y, lk.limbs.x, s3)};
        a_hi = v4i{(int)__builtin_amdgcn_perm(lk.limbs.w, lk.limbs.z, s0),
                   (int)__builtin_amdgcn_perm(lk.limbs.w, lk.limbs.z, s1),
                   (int)__builtin_amdgcn_perm(lk.limbs.w, lk.limbs.z, s2),
                   (int)__builtin_amdgcn_perm(lk.limbs.w, lk.limbs.z, s3)};
    };
    // fp32 scales of C rows 4 kb + r of superblock sb (zero past the end: such steps add nothing)
    auto row_scales = [&](const Codes &codes, unsigned sb, float (&out)[4]) {
        const float mine = sb < superblocks ? 0.125f * f16_bits_to_float(codes.scale16) : 0.0f;
#pragma unroll
        for (unsigned r = 0; r < 4u; ++r) out[r] = __shfl(mine, (int)(4u * kb + r), 64);
    };
    // LDS offsets of this lane's fragment pieces: piece 4 ks + kb of slot 16 b + li
    unsigned piece[4];
#pragma unroll
    for (unsigned ks = 0; ks < 4u; ++ks) piece[ks] = li * kActPitch + (((4u * ks + kb) ^ li) << 4);

    float acc[NB][4];
#pragma unroll
    for (unsigned tb = 0; tb < NB; ++tb)
#pragma unroll
        for (unsigned r = 0; r < 4u; ++r) acc[tb][r] = 0.0f;

    // ---- pipeline state; every index below is a compile-time constant after unrolling ----
    // (weight windows: LDS slot x & 1 holds superblock x, copied two steps before its records
    // are taken out)
    v4i a_lo[2][4], a_hi[2][4];      // [x & 1]: A operands of superblock x, all four K steps
    float rs[2][4];                  // [x & 1]: row scales of superblock x
    v4i frags[4];                    // B fragment of K step ks: re-requested for the next token block
                                     // as soon as the current one has used it
    float ts[2];                     // [g & 1]: activation scale of token block g (counted over steps)
    v4i sum_lo[2], sum_hi[2];        // [g & 1]: its integer sums, scaled one token block later
    // Fragment addresses: stage base + piece offset live in registers (kept opaque so that the
    // block offset, under 32 KB, stays the instruction's immediate instead of a separate OR).
    unsigned piece_at[4];
    auto enter_stage = [&](unsigned base) {
#pragma unroll
        for (unsigned ks = 0; ks < 4u; ++ks) {
            piece_at[ks] = base + piece[ks];
            asm volatile("" : "+v"(piece_at[ks]));
        }
    };
    auto request = [&](unsigned block, unsigned ks) {   // block: 16-slot block of the entered stage
        frags[ks] = lds_read_v4i(piece_at[ks] + block * 16u * kActPitch);
    };
    auto request_scale = [&](unsigned base, unsigned block, unsigned g) {
        ts[g & 1u] = __uint_as_float(lds_read_u32(base + kStageActs + 4u * (block * 16u + li)));
    };
    auto stage_of = [&](unsigned step) { return kStageBase + ((step / S) & 1u) * kStageBytes; };

    __syncthreads();   // every wave is done with the previous item's stages
    copy_activations(0u, 0u);
    // where each pair's results go and its route weight, for the publishing pass
    if (tid < kTileTokens && tid < it.tokens) {
        const unsigned long long ordered = it.pair0 + tid;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long out_index = pr.out_by_source_pair ? source : ordered;
        const float route_weight = pr.route_weights ? pr.route_weights[source] : 1.0f;
        lds_write_uint2(kPairInfoBase + tid * 8u, make_uint2((unsigned)out_index, __float_as_uint(route_weight)));
    }
    {
        __builtin_amdgcn_s_waitcnt(0x0f70u);   // vmcnt(0): every copy above has landed
        const Codes first = settle_codes(0u, 0u);
        // the slot's reads have returned before it is refilled
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        fetch_codes(0u, 2u);
        __syncthreads();
        enter_stage(stage_of(0u));
#pragma unroll
        for (unsigned ks = 0; ks < 3u; ++ks) request(0u, ks);
        request_scale(stage_of(0u), 0u, 0u);
        row_scales(first, 0u, rs[0]);
        Lookup lk[4];
#pragma unroll
        for (unsigned ks = 0; ks < 4u; ++ks) lk[ks] = lookup(first, ks);
#pragma unroll
        for (unsigned ks = 0; ks < 4u; ++ks) weights_from_lookup(lk[ks], a_lo[0][ks], a_hi[0][ks]);
    }
    sum_lo[1] = v4i{0, 0, 0, 0};
    sum_hi[1] = v4i{0, 0, 0, 0};
    ts[1] = 0.0f;
#pragma unroll
    for (unsigned r = 0; r < 4u; ++r) rs[1][r] = 0.0f;

    // scaling of the integer sums of token block g - 1 into the accumulators, one C row per call
    auto scale_row = [&](unsigned g_prev, unsigned tb_prev, float row_scale, float token_scale, unsigned r) {
        const int total = (sum_hi[g_prev & 1u][r] << 7) + sum_lo[g_prev & 1u][r];
        acc[tb_prev][r] = __builtin_fmaf(row_scale * token_scale, (float)total, acc[tb_prev][r]);
    };

    const unsigned steps = (superblocks + D - 1u) / D * D;
    for (unsigned t0 = 0; t0 < steps; t0 += D) {
#pragma unroll
        for (unsigned u = 0; u < D; ++u) {
            const unsigned t = t0 + u;                    // this step's superblock; u == t % D
            const unsigned base = stage_of(t);
            // the next superblock's records leave the ring; the one D steps on enters it piece
            // by piece below, behind this period's copies
            // (copies are invisible to the compiler's wait counts; they complete in order, so
            // waiting until only the copies issued after a slot's two are in flight covers it)
            constexpr unsigned kAfterPeriodStart = 2u + kCopyPieces;
            if (((u + D - 1u) % D) % S == 0u)
                __builtin_amdgcn_s_waitcnt(0x0f70u | (kAfterPeriodStart & 15u) | ((kAfterPeriodStart >> 4) << 14));
            else
                __builtin_amdgcn_s_waitcnt(0x0f72u);
            const Codes next = settle_codes((u + 1u) & 1u, t + 1u);
            constexpr unsigned kSlots = 4u * NB;
            const unsigned memory_pieces = (u % S == 0u ? kCopyPieces : 0u) + kFetchPieces;
            float rs_before[4];                           // of the step before this one
#pragma unroll
            for (unsigned r = 0; r < 4u; ++r) rs_before[r] = rs[(u + 1u) & 1u][r];
            row_scales(next, t + 1u, rs[(u + 1u) & 1u]);
            Lookup lk[4];
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (unsigned tb = 0; tb < NB; ++tb) {
                const unsigned g = u * NB + tb;           // parity of the global token-block count
                const float ts_before = ts[(g + 1u) & 1u];   // of the token block before this one
#pragma unroll
                for (unsigned ks = 0; ks < 4u; ++ks) {
                    const unsigned q = tb * 4u + ks;
                    // across a period end the next token block's scale and fragments are
                    // requested after the barrier instead
                    const bool next_here = tb + 1u < NB || u % S != S - 1u;
                    const unsigned next_block = (u % S) * NB + tb + 1u;
                    if (ks == 0u && next_here) request_scale(base, next_block, g + 1u);
                    const v4i b = frags[ks];
                    if (ks == 0u) {
                        sum_lo[g & 1u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_lo[u & 1u][0], b, v4i{0, 0, 0, 0}, 0, 0, 0);
                        sum_hi[g & 1u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_hi[u & 1u][0], b, v4i{0, 0, 0, 0}, 0, 0, 0);
                    } else {
                        sum_lo[g & 1u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_lo[u & 1u][ks], b, sum_lo[g & 1u], 0, 0, 0);
                        sum_hi[g & 1u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_hi[u & 1u][ks], b, sum_hi[g & 1u], 0, 0, 0);
                    }
                    // fragment ks - 1 is free now: its next use is one token block on (fragment 3
                    // of this token block still has to be asked for when ks is 0)
                    if (ks == 0u) request(next_block - 1u, 3u);
                    else if (next_here) request(next_block, ks - 1u);
                    // one C row of the previous token block (the previous step's last one for tb 0)
                    scale_row(g + 1u, tb ? tb - 1u : NB - 1u, tb ? rs[u & 1u][ks] : rs_before[ks], ts_before, ks);
                    // this step's copies and loads, spread evenly
#pragma unroll
                    for (unsigned v = 0; v < kCopyPieces + kFetchPieces; ++v) {
                        if (v >= memory_pieces || v * kSlots / memory_pieces != q) continue;
                        const unsigned first_fetch = memory_pieces - kFetchPieces;
                        if (v < first_fetch) copy_piece(t / S + 1u, (t / S + 1u) & 1u, v);
                        else {
                            // the reads that took this slot's records out have returned
                            if (v == first_fetch) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                            fetch_piece((u + 1u) & 1u, t + 3u, v - first_fetch);
                        }
                    }
                    // the next superblock's A operands: eight pieces (lookups L, permutes W of the
                    // four K steps) spread evenly over the slots, every W at least two slots
                    // behind its L
#pragma unroll
                    for (unsigned i = 0; i < 8u; ++i) {
                        if (i * NB / 2u != q) continue;
                        unsigned is_w, k;
                        if (NB >= 8u) {
                            is_w = i & 1u;
                            k = i >> 1;
                        } else {
                            is_w = (i == 2u || i == 4u || i >= 6u) ? 1u : 0u;
                            k = is_w ? (i == 2u ? 0u : i == 4u ? 1u : i - 4u) : (i < 2u ? i : (i + 1u) / 2u);
                        }
                        if (is_w) weights_from_lookup(lk[k], a_lo[(u + 1u) & 1u][k], a_hi[(u + 1u) & 1u][k]);
                        else lk[k] = lookup(next, k);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (u % S == S - 1u) {
                // the copies of the next period are older than the 2 S window copies issued since
                __builtin_amdgcn_s_waitcnt(0x0f70u | ((2u * S) & 15u) | (((2u * S) >> 4) << 14));
                __syncthreads();
                enter_stage(stage_of(t + 1u));
#pragma unroll
                for (unsigned ks = 0; ks < 3u; ++ks) request(0u, ks);
                request_scale(stage_of(t + 1u), 0u, (u + 1u) * NB);
            }
        }
    }
    // the last token block of the last step
#pragma unroll
    for (unsigned r = 0; r < 4u; ++r) scale_row(D * NB - 1u, NB - 1u, rs[(D - 1u) & 1u][r], ts[(D * NB - 1u) & 1u], r);

    // ---- publish: the lane holds C rows 4 kb + r of its block for tokens tb * 16 + li ----
    auto store4 = [&](unsigned long long out_index, unsigned row, const float (&value)[4]) {
        const bool good = finite_f32(value[0]) && finite_f32(value[1]) && finite_f32(value[2]) &&
                          finite_f32(value[3]);
        if (!good) raise_status(a.status, 1);
        else if (row + 3u < a.out_rows)
            *reinterpret_cast<float4 *>(pr.out + out_index * a.out_rows + row) =
                make_float4(value[0], value[1], value[2], value[3]);
        else
            for (unsigned r = 0; r < 4u; ++r)
                if (row + r < a.out_rows) pr.out[out_index * a.out_rows + row + r] = value[r];
    };
    if constexpr (FUSED_UP) {
        // Gate wave w and up wave w + 4 hold the two inputs of every SwiGLU. All waves put their
        // blocks into LDS (the stages are free after the last barrier); gate waves then finish
        // token blocks [0, G) of their row block, up waves blocks [G, NB), in a loop that is not
        // unrolled: the activation with its guarded fast path is long, and sixteen copies of it
        // cost more in registers than they save.
        constexpr unsigned G = (NB + 1u) / 2u;
        const bool is_gate = wave < 4u;
        const unsigned pair_wave = wave & 3u;
#pragma unroll
        for (unsigned tb = 0; tb < NB; ++tb)
            lds_write_uint4(kStageBase + ((wave * NB + tb) * 64u + lane) * 16u,
                            make_uint4(__float_as_uint(acc[tb][0]), __float_as_uint(acc[tb][1]),
                                       __float_as_uint(acc[tb][2]), __float_as_uint(acc[tb][3])));
        __syncthreads();
        const unsigned tb_end = is_gate ? G : NB;
        const float limit_f32 = (float)a.limit;
#pragma unroll 1
        for (unsigned tb = is_gate ? 0u : G; tb < tb_end; ++tb) {
            const unsigned token = tb * 16u + li;
            const uint4 g = lds_read_uint4(kStageBase + ((pair_wave * NB + tb) * 64u + lane) * 16u);
            const uint4 u = lds_read_uint4(kStageBase + (((pair_wave + 4u) * NB + tb) * 64u + lane) * 16u);
            if (token < it.tokens) {
                const uint2 info = lds_read_uint2(kPairInfoBase + token * 8u);
                const float route_weight = __uint_as_float(info.y);
                const float value[4] = {
                    swiglu_bf16_fast(__uint_as_float(g.x), __uint_as_float(u.x), route_weight, a.limit, limit_f32),
                    swiglu_bf16_fast(__uint_as_float(g.y), __uint_as_float(u.y), route_weight, a.limit, limit_f32),
                    swiglu_bf16_fast(__uint_as_float(g.z), __uint_as_float(u.z), route_weight, a.limit, limit_f32),
                    swiglu_bf16_fast(__uint_as_float(g.w), __uint_as_float(u.w), route_weight, a.limit, limit_f32)};
                store4(info.x, out_row_base + 4u * kb, value);
            }
        }
    } else {
#pragma unroll
        for (unsigned tb = 0; tb < NB; ++tb) {
            const unsigned token = tb * 16u + li;
            if (token < it.tokens) {
                const uint2 info = lds_read_uint2(kPairInfoBase + token * 8u);
                const float value[4] = {bf16_round(acc[tb][0]), bf16_round(acc[tb][1]),
                                        bf16_round(acc[tb][2]), bf16_round(acc[tb][3])};
                store4(info.x, out_row_base + 4u * kb, value);
            }
        }
    }
}

template <bool FUSED_UP>
__global__ __launch_bounds__(512) void mfma_iq2_kernel(MfmaArgs a)
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
        unsigned cursor = 0u, members[4] = {0u, 0u, 0u, 0u};
        for (unsigned b = 0; b < buckets && b < 256u; ++b) {
            lds_write_u32(kTileStartBase + 4u * b, cursor);
            const unsigned long long n = fixed ? pr.pairs : pr.bucket_populations[b];
            cursor += (unsigned)(n / kTileTokens);
            const unsigned rest = (unsigned)(n % kTileTokens);
            if (rest) {
                const unsigned c = rest > 64u ? 0u : rest > 32u ? 1u : rest > 16u ? 2u : 3u;
                lds_write_u16(kClassListBase + (c * 256u + members[c]) * 2u, b);
                ++members[c];
            }
        }
        lds_write_u32(kTileStartBase + 4u * (buckets < 256u ? buckets : 256u), cursor);
        for (unsigned c = 0; c < 4u; ++c) lds_write_u32(kClassCountBase + 4u * c, members[c]);
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
    unsigned members[4];
    unsigned long long items = full_items;
    for (unsigned c = 0; c < 4u; ++c) {
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
            while (c < 3u && rest >= (unsigned long long)members[c] * row_tiles) {
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
        if (it.tokens <= 16u) mfma_item<FUSED_UP, 1u>(a, it);
        else if (it.tokens <= 32u) mfma_item<FUSED_UP, 2u>(a, it);
        else if (it.tokens <= 64u) mfma_item<FUSED_UP, 4u>(a, it);
        else mfma_item<FUSED_UP, 8u>(a, it);
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
    mfma_iq2_kernel<FUSED_UP><<<mfma_grid(), 512u, kMfmaLdsBytes, stream>>>(a);
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
