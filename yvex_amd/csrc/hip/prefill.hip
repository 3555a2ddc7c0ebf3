// Row-batch (prefill-width) grouped expert projections on the int8 matrix cores of gfx950.
//
// A work item is (bucket, tile of up to 64 ordered pairs, tile of 256 weight rows: 128 gate rows
// and the 128 matching up rows when the SwiGLU is fused). The workgroup has eight waves, two per
// SIMD; each owns 32 weight rows and multiplies them by all of the item's Q8_K activation rows
// with V_MFMA_I32_32X32X32_I8. A wave cannot run vector instructions under its own matrix
// instruction, the other wave of its SIMD can, so two waves a SIMD is the shape that lets decode
// and scaling arithmetic overlap the matrix pipe, and 256 registers a wave is what decides the
// tile: 32 rows x 64 tokens of int32 limb sums and double-precision row sums.
//
//   A operand (weights): built in registers, one K chunk (32 columns) ahead of its use. Lane
//       (r, h) = (lane % 32, lane / 32) owns weight row r and the groups 4h .. 4h + 3 of the
//       current superblock (128 columns); K chunk m of the superblock is, for that lane, the 16
//       weights 16 (m % 2) .. + 15 of group 4h + m / 2. The order of K inside a matrix
//       instruction is free as long as both operands agree.
//       The IQ2_XXS value of one weight is level * sign * (2s+1), up to 43 * 31 = 1333, so it is
//       split into two int8 limbs, value = 128 * hi + lo with hi in [1, 11] and lo in
//       [-120, 63], and every K chunk costs two matrix instructions per token block. For one
//       scale there are only three levels, so the six signed limb values of a group fit two
//       registers and one V_PERM_B32 per four weights picks them: the selector byte of a weight
//       is its level code (0..2) plus 4 when it is negative. Three LDS tables feed this, sixteen
//       replicas each so that the lanes of a quarter-wave never share a bank: level codes of a
//       codebook entry (8 bytes), sign selectors of a 7-bit sign field (8 bytes) and the limb
//       words of a scale (16 bytes).
//   Weight bytes: each wave copies, per superblock, the aligned 68 bytes around the superblock of
//       each of its 32 rows into an LDS window (GLOBAL_LOAD_LDS_DWORDX4, every cache line
//       fetched once), two superblocks ahead; the lanes take their records out with three
//       16-byte LDS reads from a piece-major window (no two lanes of sixteen on one bank; dword
//       reads of rows 80 bytes apart put four lanes on a bank).
//   B operand (activations): the tile's int8 blocks of one superblock, copied from global memory
//       straight into LDS, in a ring of stages. 16-byte piece c of token t sits at piece position
//       c ^ (t % 16), so the 16 lanes that read one fragment column together hit 16 different
//       bank groups.
//   C: per (superblock, 32-token block) two int32 accumulators of 32 x 32; T = 128 * C_hi + C_lo
//       is the exact integer superblock sum of the reference's primitive
//       (src/backend/cuda/kernel_primitives.h:287-313), scaled into the float term
//       ((0.125 * d_w) * d_a) * T; a row's terms are added in double, in superblock order, and
//       the sum is rounded to float once, which is what the CPU path computes for a row (double
//       accumulation over a row's blocks, src/gguf/quant_compute.c:152-172): every value
//       rounded to bfloat16 afterwards rounds as it does there.
//   Output: accumulator i of lane (r, h) is token r's sum for row 8 (i / 4) + 4 h + i % 4 of the
//       wave's 32 (gate sums in the first eight, the matching up sums in the last eight when
//       fused), so a lane stores four consecutive rows of its token, 16 bytes, straight from its
//       registers; the stores of a wave complete whole cache lines, which the L2 merges.
//
// Same inputs, outputs and rounding points as the decode-width sweeps in moe.hip
// (src/backend/cuda/tensorcore.cu:378-702 is the reference's counterpart, unused there).
#include "common.hpp"
#include "launch.hpp"
#include "grouped.hpp"
#include "lds_copy.hpp"

namespace yvex {

constexpr unsigned kRowWaves = 8u;                          // two per SIMD
constexpr unsigned kRowThreads = 64u * kRowWaves;
constexpr unsigned kTileTokens = 64u;
constexpr unsigned kActPitch = 256u;                       // one Q8_K block's int8 payload
// LDS map (absolute byte offsets; the dynamic allocation starts at 0, checked at kernel start).
// Codebook entry e owns the 256 bytes at 256 e: sixteen replicas of its 8 level codes in the
// first half; the second half of entries 0-127 holds sixteen replicas of the sign selectors of
// sign field e.
constexpr unsigned kCodeBase = 0u;
constexpr unsigned kSelBase = 128u;
constexpr unsigned kLutBase = 65536u;                       // 16 scales x 16 replicas x 16 bytes
constexpr unsigned kRowScaleBase = kLutBase + 16u * 16u * 16u;   // 8 waves x 2 x 32 floats
constexpr unsigned kPairInfoBase = kRowScaleBase + kRowWaves * 2u * 128u;   // {out row, route weight} x 64
// Item numbering: first full 64-pair tile of every bucket (257 words), then per class of last,
// partial, tile (33-63, 1-32 pairs) a count and the list of its buckets (u16).
constexpr unsigned kTileStartBase = kPairInfoBase + kTileTokens * 8u;
constexpr unsigned kClassCountBase = kTileStartBase + 260u * 4u;
constexpr unsigned kClassListBase = kClassCountBase + 16u;
constexpr unsigned kTrashBase = kClassListBase + 2u * 256u * 2u;   // 256 bytes nobody reads
// Weight windows: per wave two buffers of six 16-byte pieces for each of the wave's 32 rows,
// piece-major (piece p of row r at slot 32 p + r; three full copies fill a buffer): the pieces a
// lane's record lies in are three conflict-free 16-byte reads. Canonical bytes: the aligned 68
// bytes around a superblock (pieces at 0, 16, 32, 48 and 52, the sixth repeats the fifth); the
// image: the two 36-byte lane records (pieces at 0, 16, 32 and at 36, 52, 56).
constexpr unsigned kWindowBase = (kTrashBase + 256u + 255u) & ~255u;
constexpr unsigned kWindowBytes = 32u * 96u;
constexpr unsigned kStageBase = kWindowBase + kRowWaves * 2u * kWindowBytes;
// activation stages: a ring of 4 / NTB stages of NTB x 32 slots (256 bytes each) + 64 scales
constexpr unsigned kStageRingBytes = 128u * kActPitch + 4u * 256u;
constexpr unsigned kMfmaLdsBytes = kStageBase + kStageRingBytes;
static_assert(kMfmaLdsBytes <= 160u * 1024u, "one workgroup per compute unit");

struct MfmaArgs {
    GroupedProblem pr;
    unsigned width;          // reduction width
    unsigned out_rows;       // weight rows per expert
    double limit;
    int *status;
    int plain_output;        // plain projection: outputs stay fp32 instead of being rounded to bf16
    int image;               // weights are the sweep image (72-byte records) instead of canonical bytes
};

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

// A work item whose bucket record has been requested from memory but not looked at yet.
struct MfmaItemRequest {
    int state;                      // 0: requested, 1: the lists are inconsistent (skip it), 2: past the last item
    bool partial;                   // the bucket's last, partial token tile
    unsigned bucket, token_tile, row_tile;
    unsigned long long first, population, expert;
};

// The item a workgroup runs after the current one.
struct MfmaNextItem {
    MfmaItem it;
    int state;                      // as above (0: it holds the item)
    bool ahead;                     // the current item's last rounds of copies fetch its first two windows
    long long shift;                // from a weight row of the current item to the same row of this one
};

// One work item with NTB live 32-token blocks (NTB is 1 or 2).
//
// Time slot (sb, m) = superblock sb, K chunk m: 2 NTB matrix instructions (low and high limb for
// every token block) on the chunk's operands, which were built during the slot before: the
// weights of a superblock are decoded chunk by chunk just ahead of their use, two chunks' worth
// of operand registers in all. Between the matrix instructions the slot carries the LDS reads of
// the activation fragments two slots ahead, the table lookups of the chunk two slots ahead,
// the selector words and permutes of the next chunk, and its share of the copies. After the
// last chunk the integer sums of the superblock are scaled and added to the row sums. Two waves
// share a SIMD: while one waits for its own matrix instructions or scales its sums the other's
// instructions run.
//
// Everything that comes from memory inside the loop arrives by GLOBAL_LOAD_LDS copies, whose
// completion the kernel counts by hand (they retire in order):
//   * activations: a ring of R = 4 / NTB stages of NTB x 32 slots (256 int8 + one scale each);
//     the copies of superblock sb + R are issued right after the barrier of superblock sb, which
//     every wave passes once all its reads of that stage have returned;
//   * weights: per wave two windows holding, for each of its 32 rows, the aligned 68 bytes
//     around one superblock (five 16-byte pieces a row, the fifth ending with the dword that
//     holds the superblock's last byte, so nothing behind it is touched; the image: the three
//     pieces that hold each of the two lane records), stored piece-major. Each cache line of a
//     row is fetched once; taking the records out of the window is LDS work. Loading the
//     records lane by lane from global memory touched every row's line four times per
//     superblock, and the memory pipeline spends about two cycles per line an instruction
//     touches: with eight waves that was the longest pole of the step.
// The loop body is one superblock in one basic block (requests past the end are clamped, and
// superblocks past the end run with a zero row scale), so nothing leaves registers.
//
// Between two items of a workgroup: the item that follows is looked up while the first copies of
// this one are in flight (`request_next` before them, `resolve_next` once they have landed), and
// when it has the same shape the loop's last rounds of window copies, which have no superblock
// of this item left to fetch, fetch its first two windows instead (`prefetched` tells the
// item that they are there). Its first activation stage cannot come early: the publishing pass
// uses the stages' memory.
template <bool FUSED_UP, unsigned NTB, bool IMAGE, class Request, class Resolve>
__device__ __forceinline__ void rows_item(const MfmaArgs &a, const MfmaItem &it, bool prefetched,
                                          Request &&request_next, Resolve &&resolve_next, MfmaNextItem &next)
{
    const GroupedProblem &pr = a.pr;
    constexpr unsigned R = 4u / NTB;                 // activation stages
    constexpr unsigned T = NTB * 32u;                // token slots of one stage
    constexpr unsigned kStageBytes = T * kActPitch + 256u;
    constexpr unsigned kBarrierSlot = 5u;
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned r = lane & 31u, h = lane >> 5;
    constexpr unsigned kItemRows = FUSED_UP ? 128u : 256u;
    const unsigned superblocks = a.width >> 8;
    const unsigned last = superblocks - 1u;

    // ---- weight rows: rows 0-15 of a wave are gate rows and rows 16-31 the matching up rows
    // when the SwiGLU is fused ----
    auto row_pointer = [&](unsigned wave_row) {
        unsigned row;
        bool is_up = false;
        if constexpr (FUSED_UP) {
            row = it.row_tile * kItemRows + wave * 16u + (wave_row & 15u);
            is_up = wave_row >= 16u;
        } else {
            row = it.row_tile * kItemRows + wave * 32u + wave_row;
        }
        if (row >= a.out_rows) row = a.out_rows - 1u;
        return is_up
            ? pr.up + it.expert * pr.up_expert_bytes + (unsigned long long)row * pr.up_row_bytes
            : pr.gate + it.expert * pr.expert_bytes + (unsigned long long)row * pr.row_bytes;
    };
    // Superblocks are 66 bytes, so they start on 2-byte boundaries, and vector accesses that are
    // not dword-aligned run at less than half rate: a window starts at the aligned dword that
    // holds the superblock's first byte. Copy k of a window moves pieces 64 k + lane of the
    // wave's 160 (row = piece / 5).
    const unsigned row_misalign = (unsigned)(unsigned long long)row_pointer(r) & 3u;    // of the lane's own row
    const unsigned char *window_from[3];    // row start + piece offset, of the row this lane copies
#pragma unroll
    for (unsigned k = 0; k < 3u; ++k) {
        if constexpr (IMAGE) {
            // The 72-byte record of a row's superblock is two lane records of 36 bytes (dword
            // aligned): bytes 0-35 lie in the pieces at 0, 16 and 32, bytes 36-71 in the pieces at
            // 36, 52 and 56 (the last one ends with the record, so nothing behind it is touched).
            const unsigned piece = 2u * k + (lane >> 5);        // slot 64 k + lane = 32 piece + row
            const unsigned at = piece < 3u ? 16u * piece : piece == 3u ? 36u : piece == 4u ? 52u : 56u;
            window_from[k] = row_pointer(lane & 31u) + at;
        } else {
            // The aligned 68 bytes around a superblock lie in the pieces at 0, 16, 32, 48 and 52
            // (the last ends with the dword that holds the superblock's last byte); the sixth slot
            // repeats the fifth.
            const unsigned piece = 2u * k + (lane >> 5);
            window_from[k] = row_pointer(lane & 31u) + (piece < 4u ? 16u * piece : 52u);
        }
    }
    const unsigned window_base = kWindowBase + wave * 2u * kWindowBytes;
    // Windows past the last superblock: windows 0 and 1 of the next item (by parity, so that a
    // third one repeats the first) when they are fetched ahead, else the last window again.
    long long ahead_shift = 0;
    bool ahead = false;
    auto weight_piece = [&](unsigned sb, unsigned k) {
        const unsigned to = (unsigned)__builtin_amdgcn_readfirstlane(
            (int)(window_base + (sb & 1u) * kWindowBytes + k * 1024u));
        const bool past = sb > last;
        const unsigned record = !past ? sb : ahead ? (sb - superblocks) & 1u : last;
        const long long offset = (past ? ahead_shift : 0ll) + (long long)(record * (IMAGE ? 72u : 66u));
        const unsigned char *from = IMAGE
            ? window_from[k] + offset
            : (const unsigned char *)((unsigned long long)(window_from[k] + offset) & ~3ull);
        copy_to_lds_16(from, to);
    };

    // ---- activation rows this lane copies: wave w owns the 4-slot groups w (and w + 8) ----
    // Lane l of a group moves piece position l % 16 of slot 4 g + l / 16; LDS receives the wave's
    // 64 pieces back to back, so the swizzle is applied on the global side.
    auto token_row = [&](unsigned token) {
        const unsigned live = token < it.tokens ? token : it.tokens - 1u;   // padding repeats a row
        const unsigned long long ordered = it.pair0 + live;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long arow = pr.act_by_ordered_pair ? ordered : source / pr.topk;
        return (const unsigned char *)pr.activations + arow * pr.act_stride;
    };
    const unsigned char *copy_from[NTB];
#pragma unroll
    for (unsigned j = 0; j < NTB; ++j) {
        const unsigned token = 4u * (wave + kRowWaves * j) + (lane >> 4);
        copy_from[j] = token_row(token) + 4u + 16u * ((lane & 15u) ^ (token & 15u));
    }
    // Wave 0 also copies the stage's slot scales, laid out [token % 32][token block] so that a lane
    // reads the scales of its NTB tokens with one LDS read. The other waves run the same
    // instruction on one address for all lanes (one cache line: next to free) into bytes nobody
    // reads, which is cheaper than a branch around the copy.
    const unsigned char *scale_from;
    {
        const unsigned index = wave == 0u ? lane % T : 0u;
        scale_from = token_row((index % NTB) * 32u + index / NTB);
    }
    // Where each pair's results go and its route weight, for the publishing pass: requested now,
    // put into LDS once the previous item's publishing pass is over.
    const bool info_lane = tid < kTileTokens && tid < it.tokens;
    unsigned info_out = 0u;
    float info_weight = 1.0f;
    if (info_lane) {
        const unsigned long long ordered = it.pair0 + tid;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        info_out = (unsigned)(pr.out_by_source_pair ? source : ordered);
        if (pr.route_weights) info_weight = pr.route_weights[source];
    }
    auto request = request_next();
    constexpr unsigned kActPieces = NTB + 1u;
    auto act_piece = [&](unsigned sb, unsigned j) {
        const unsigned base = kStageBase + (sb % R) * kStageBytes;
        sb = sb < last ? sb : last;
        if (j < NTB) {
            copy_to_lds_16(copy_from[j] + (unsigned long long)sb * kQ8KBytes,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(base + (wave + kRowWaves * j) * 1024u)));
        } else {
            copy_to_lds_4(scale_from + (unsigned long long)sb * kQ8KBytes,
                          (unsigned)__builtin_amdgcn_readfirstlane(
                              (int)(wave == 0u ? base + T * kActPitch : kTrashBase)));
        }
    };
    // the copies issued after the barrier of superblock sb: the stage and the window just released
    constexpr unsigned kRoundPieces = kActPieces + 3u;
    auto round_piece = [&](unsigned sb, unsigned j) {
        if (j < kActPieces) act_piece(sb + R, j);
        else weight_piece(sb + 3u, j - kActPieces);
    };

    // ---- decode state ----
    const unsigned code_lane = kCodeBase + (lane & 15u) * 8u;
    const unsigned sel_lane = kSelBase + (lane & 15u) * 8u;
    const unsigned lut_lane = kLutBase + (lane & 15u) * 16u;
    const unsigned row_scale_at = kRowScaleBase + wave * 256u;      // + 128 for odd superblocks
    unsigned grids[4], aux[4];           // group records of the superblock being decoded
    unsigned head = 0u;                  // image: fp16 scale | the four group scales of this half << 16
    uint2 codes[2][2], signs[2][2];      // [chunk & 1]: table words of the chunk's two subgroups
    uint4 limbs[2];                      // [group & 1]: limb words of a group
    v4i a_lo[2], a_hi[2];                // [chunk & 1]: A operands of a K chunk

    // Records of superblock sb out of its window, and the row's scale into LDS for the lanes that
    // hold this row's sums (zero past the end: such superblocks add nothing). With o = (row start
    // + 66 sb) mod 4 (0 or 2) the fp16 scale sits o bytes into the window and the lane's 32 code
    // bytes at o + 2 + 32 h: in aligned dwords 8 h + o / 2 onwards, shifted by 2 bytes when o is
    // 0. Aligned dword 16 is the last dword of the fifth piece.
    auto settle = [&](unsigned sb) {
        if constexpr (IMAGE) {
            // The lane's record is nine dwords: pieces 3 h and 3 h + 1 whole, and of piece 3 h + 2
            // the first dword (bytes 32-35 of the row's 72) or the last (bytes 68-71).
            const unsigned at = window_base + (sb & 1u) * kWindowBytes + (3u * h * 32u + r) * 16u;
            const v4i first = lds_read_v4i(at), second = lds_read_v4i(at + 512u), third = lds_read_v4i(at + 1024u);
            head = (unsigned)first[0];
            grids[0] = (unsigned)first[1];
            aux[0] = (unsigned)first[2];
            grids[1] = (unsigned)first[3];
            aux[1] = (unsigned)second[0];
            grids[2] = (unsigned)second[1];
            aux[2] = (unsigned)second[2];
            grids[3] = (unsigned)second[3];
            aux[3] = (unsigned)(h ? third[3] : third[0]);
            const float mine = sb < superblocks ? 0.125f * f16_bits_to_float(head & 0xffffu) : 0.0f;
            lds_write_u32(row_scale_at + (sb & 1u) * 128u + r * 4u, __float_as_uint(mine));
            return;
        }
        const unsigned clamped = sb < last ? sb : last;
        const unsigned o = (row_misalign + 2u * clamped) & 3u;
        // Aligned dwords 8 h .. 8 h + 8 of the window: pieces 2 h and 2 h + 1 whole, and the dword
        // behind them (the first of piece 2, or the last of the fifth piece, which is aligned
        // dword 16). The lane's nine dwords start at dword 8 h + o / 2 of the window.
        const unsigned at = window_base + (sb & 1u) * kWindowBytes + (2u * h * 32u + r) * 16u;
        const v4i first = lds_read_v4i(at), second = lds_read_v4i(at + 512u), third = lds_read_v4i(at + 1024u);
        const unsigned d[9] = {(unsigned)first[0], (unsigned)first[1], (unsigned)first[2], (unsigned)first[3],
                               (unsigned)second[0], (unsigned)second[1], (unsigned)second[2], (unsigned)second[3],
                               (unsigned)(h ? third[3] : third[0])};
        unsigned w[9];
#pragma unroll
        for (unsigned i = 0; i < 8u; ++i) w[i] = o ? d[i + 1u] : d[i];
        w[8] = d[8];           // (the ninth is only part of a record when o is 0)
        // the fp16 scale sits o bytes into the window: in the first dword of the first half's lanes,
        // which are the ones that publish it
        const unsigned scale16 = ((unsigned)first[0] >> (8u * o)) & 0xffffu;
        const unsigned shift = (o + 2u) & 3u;
#pragma unroll
        for (unsigned g = 0; g < 4u; ++g) {
            grids[g] = __builtin_amdgcn_alignbyte(w[2u * g + 1u], w[2u * g], shift);
            aux[g] = __builtin_amdgcn_alignbyte(w[2u * g + 2u], w[2u * g + 1u], shift);
        }
        const float mine = sb < superblocks ? 0.125f * f16_bits_to_float(scale16) : 0.0f;
        lds_write_u32(h ? kTrashBase : row_scale_at + (sb & 1u) * 128u + r * 4u, __float_as_uint(mine));
    };
    // table lookups of K chunk c: subgroups 2 (c & 1) and 2 (c & 1) + 1 of group c / 2
    auto lookup = [&](unsigned c) {
        const unsigned g = c >> 1;
#pragma unroll
        for (unsigned i = 0; i < 2u; ++i) {
            const unsigned j = 2u * (c & 1u) + i;
            codes[c & 1u][i] = lds_read_uint2(__builtin_amdgcn_perm(grids[g], code_lane, 0x0c0c0400u + (j << 8)));
            if constexpr (IMAGE) {      // the field has a byte of its own
                signs[c & 1u][i] = lds_read_uint2(__builtin_amdgcn_perm(aux[g], sel_lane, 0x0c0c0400u + (j << 8)));
            } else {
                const unsigned field = j == 0u ? aux[g] << 8 : j == 1u ? aux[g] << 1 : aux[g] >> (7u * j - 8u);
                signs[c & 1u][i] = lds_read_uint2((field & 0x7f00u) | sel_lane);
            }
        }
        if ((c & 1u) == 0u)
            limbs[g & 1u] = lds_read_uint4((IMAGE ? (head >> (8u + 4u * g)) & 0xf00u : (aux[g] >> 20) & 0xf00u) | lut_lane);
    };
    // selector words and permutes of K chunk c
    auto build = [&](unsigned c) {
        const uint4 lw = limbs[(c >> 1) & 1u];
        const unsigned s0 = codes[c & 1u][0].x | signs[c & 1u][0].x, s1 = codes[c & 1u][0].y | signs[c & 1u][0].y;
        const unsigned s2 = codes[c & 1u][1].x | signs[c & 1u][1].x, s3 = codes[c & 1u][1].y | signs[c & 1u][1].y;
        a_lo[c & 1u] = v4i{(int)__builtin_amdgcn_perm(lw.y, lw.x, s0), (int)__builtin_amdgcn_perm(lw.y, lw.x, s1),
                           (int)__builtin_amdgcn_perm(lw.y, lw.x, s2), (int)__builtin_amdgcn_perm(lw.y, lw.x, s3)};
        a_hi[c & 1u] = v4i{(int)__builtin_amdgcn_perm(lw.w, lw.z, s0), (int)__builtin_amdgcn_perm(lw.w, lw.z, s1),
                           (int)__builtin_amdgcn_perm(lw.w, lw.z, s2), (int)__builtin_amdgcn_perm(lw.w, lw.z, s3)};
    };

    // ---- activation fragments: piece 8 h + m of slot r (+ 32 tb) of the current stage; stage
    // bases are multiples of 256, so the piece position is bits 4-7 of the address ----
    unsigned frag_at = kStageBase + r * kActPitch + (((8u * h) ^ (r & 15u)) << 4);

    // ---- prologue ----
    // Copies in flight when the loop starts are those of its own schedule: a round (stage sb + R,
    // window sb + 3) is issued after the barrier of superblock sb, four pieces in slots 6 and 7 and
    // the rest at the start of the next superblock, so rounds -(R - 1) .. -1 are issued here
    // (windows 0 and 1 are needed before them; the rounds before -1 repeat window 1, which keeps
    // the counts below the same for every superblock).
    lds_barrier();     // every wave is done with the previous item's stages and pair records (its stores may still be on their way)
    if (prefetched) {      // windows 0 and 1 came with the previous item's last rounds
#pragma unroll
        for (unsigned j = 0; j < kActPieces; ++j) act_piece(0u, j);
        __builtin_amdgcn_s_waitcnt(0x0f70u);   // vmcnt(0): stage 0 has landed
    } else {
#pragma unroll
        for (unsigned k = 0; k < 3u; ++k) weight_piece(0u, k);
#pragma unroll
        for (unsigned j = 0; j < kActPieces; ++j) act_piece(0u, j);
#pragma unroll
        for (unsigned k = 0; k < 3u; ++k) weight_piece(1u, k);
        __builtin_amdgcn_s_waitcnt(0x0f73u);   // vmcnt(3): window 0 and stage 0 have landed
    }
    if (info_lane) lds_write_uint2(kPairInfoBase + tid * 8u, make_uint2(info_out, __float_as_uint(info_weight)));
    // The next item, and whether its first windows can ride on this item's last rounds: both
    // items cover whole row tiles of equal geometry (then the same lane copies the same piece of
    // the same row, one fixed distance on), and the window parity comes out right.
    resolve_next(request, next);
    next.ahead = false;
    next.shift = 0;
    if (next.state == 0 && superblocks >= 4u && (superblocks & 1u) == 0u &&
        (!FUSED_UP || (pr.expert_bytes == pr.up_expert_bytes && pr.row_bytes == pr.up_row_bytes)) &&
        (unsigned long long)(it.row_tile + 1u) * kItemRows <= a.out_rows &&
        (unsigned long long)(next.it.row_tile + 1u) * kItemRows <= a.out_rows) {
        next.ahead = true;
        next.shift = ((long long)next.it.expert - (long long)it.expert) * (long long)pr.expert_bytes +
                     ((long long)next.it.row_tile - (long long)it.row_tile) * (long long)kItemRows * (long long)pr.row_bytes;
    }
    ahead = next.ahead;
    ahead_shift = next.shift;
    settle(0u);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the window's reads have returned before it is refilled
#pragma unroll
    for (unsigned x = 1; x + 1u < R; ++x) {
#pragma unroll
        for (unsigned j = 0; j < kActPieces; ++j) act_piece(x, j);
#pragma unroll
        for (unsigned k = 0; k < 3u; ++k) weight_piece(1u, k);
    }
#pragma unroll
    for (unsigned j = 0; j < 4u; ++j) round_piece(0u - 1u, j);
    lookup(0u);
    lookup(1u);
    build(0u);
    __syncthreads();   // every wave's share of stage 0 has landed

    double acc[NTB][16];            // row sums: float terms added in double, in superblock order
#pragma unroll
    for (unsigned tb = 0; tb < NTB; ++tb)
#pragma unroll
        for (unsigned i = 0; i < 16u; ++i) acc[tb][i] = 0.0;
    v16i sum_lo[NTB], sum_hi[NTB];   // integer sums of the running superblock
    v4i frag[2][NTB];                // [slot & 1]: re-requested for two slots on as soon as it is used
#pragma unroll
    for (unsigned tb = 0; tb < NTB; ++tb) {
        frag[0][tb] = lds_read_v4i(frag_at + tb * 32u * kActPitch);
        frag[1][tb] = lds_read_v4i((frag_at ^ 16u) + tb * 32u * kActPitch);
    }
    // Waits, counted in copies issued later than the one needed:
    //   * before settle(sb + 1) at slot 5: window sb + 1 belongs to round sb - 2, so one full
    //     round (sb - 1) may be in flight;
    //   * at the barrier of superblock sb: stage sb + 1 belongs to round sb + 1 - R, so the
    //     window of that round and R - 2 full rounds may be in flight.
    constexpr unsigned kSettleInFlight = kRoundPieces;
    constexpr unsigned kBarrierInFlight = 3u + (R - 2u) * kRoundPieces;

    for (unsigned sb = 0; sb < superblocks; ++sb) {
        float rs[16];                // row scales of the rows this lane holds sums of
        float ts[NTB];               // activation scales of this lane's token per token block
        const unsigned stage = kStageBase + (sb % R) * kStageBytes;
#pragma unroll
        for (unsigned m = 0; m < 8u; ++m) {
            // ---- 2 NTB matrix instructions with the rest of the slot's work between them, a
            // few instructions at a time ----
            auto matrix = [&](unsigned tb, bool high) {
                const v4i b = frag[m & 1u][tb];
                v16i zero;
#pragma unroll
                for (unsigned i = 0; i < 16u; ++i) zero[i] = 0;
                if (!high) sum_lo[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_lo[m & 1u], b, m ? sum_lo[tb] : zero, 0, 0, 0);
                else sum_hi[tb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_hi[m & 1u], b, m ? sum_hi[tb] : zero, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            };
            const unsigned next_chunk = (m + 1u) & 7u;
            const uint4 lw = limbs[(next_chunk >> 1) & 1u];
            unsigned selector[4];
            matrix(0u, false);
            // the table lookups of the chunk two slots on
            lookup((m + 2u) & 7u);
            __builtin_amdgcn_sched_barrier(0);
            matrix(0u, true);
            // selector words and low limbs of the next chunk
            selector[0] = codes[next_chunk & 1u][0].x | signs[next_chunk & 1u][0].x;
            selector[1] = codes[next_chunk & 1u][0].y | signs[next_chunk & 1u][0].y;
            selector[2] = codes[next_chunk & 1u][1].x | signs[next_chunk & 1u][1].x;
            selector[3] = codes[next_chunk & 1u][1].y | signs[next_chunk & 1u][1].y;
#pragma unroll
            for (unsigned i = 0; i < 4u; ++i) a_lo[next_chunk & 1u][i] = (int)__builtin_amdgcn_perm(lw.y, lw.x, selector[i]);
            if constexpr (NTB == 2u) {
                __builtin_amdgcn_sched_barrier(0);
                matrix(1u, false);
            }
            // high limbs of the next chunk
#pragma unroll
            for (unsigned i = 0; i < 4u; ++i) a_hi[next_chunk & 1u][i] = (int)__builtin_amdgcn_perm(lw.w, lw.z, selector[i]);
            if constexpr (NTB == 2u) {
                __builtin_amdgcn_sched_barrier(0);
                matrix(1u, true);
            }
            // ---- the fragments two slots on (past the barrier slot the addresses already
            // point into the next superblock's stage) ----
            {
                unsigned piece = frag_at ^ (((m + 2u) & 7u) << 4);
                asm volatile("" : "+v"(piece));   // kept opaque so that the token block offset stays the instruction's immediate
#pragma unroll
                for (unsigned tb = 0; tb < NTB; ++tb) frag[m & 1u][tb] = lds_read_v4i(piece + tb * 32u * kActPitch);
            }
            if (m == 5u) {
                // chunk 7's lookups are on their way: the next superblock's records replace this
                // one's (its window has landed: see the counts above)
                __builtin_amdgcn_s_waitcnt(0x0f70u | (kSettleInFlight & 15u) | ((kSettleInFlight >> 4) << 14));
                settle(sb + 1u);
            }
            if (m == 4u) {
                // this superblock's token scales, while its stage is still held
                const unsigned at = stage + T * kActPitch + r * NTB * 4u;
                if constexpr (NTB == 2u) {
                    const uint2 v = lds_read_uint2(at);
                    ts[0] = __uint_as_float(v.x);
                    ts[1] = __uint_as_float(v.y);
                } else {
                    ts[0] = __uint_as_float(lds_read_u32(at));
                }
            }
            if (m == 6u) {
                // the row scales of this superblock, for the scaling below
#pragma unroll
                for (unsigned q = 0; q < 4u; ++q) {
                    const uint4 v = lds_read_uint4(row_scale_at + (sb & 1u) * 128u + (8u * q + 4u * h) * 4u);
                    rs[4u * q] = __uint_as_float(v.x);
                    rs[4u * q + 1u] = __uint_as_float(v.y);
                    rs[4u * q + 2u] = __uint_as_float(v.z);
                    rs[4u * q + 3u] = __uint_as_float(v.w);
                }
            }
            if (m == kBarrierSlot) {
                // Every read of this superblock's stage and of the next one's window has returned
                // and this wave's share of the next stage has landed: after the barrier nobody
                // reads this stage again and the next one is complete.
                __builtin_amdgcn_s_waitcnt(0x0070u | (kBarrierInFlight & 15u) | ((kBarrierInFlight >> 4) << 14));
                __syncthreads();
                const unsigned flip = (sb % R == R - 1u) ? 0u - (R - 1u) * kStageBytes : kStageBytes;
                frag_at += flip;
            }
            // ---- the round of copies into the stage and the window just released: two pieces a
            // slot behind the barrier, the rest at the start of the next superblock ----
            if (m > kBarrierSlot) {
                round_piece(sb, 2u * (m - kBarrierSlot - 1u));
                round_piece(sb, 2u * (m - kBarrierSlot - 1u) + 1u);
            }
            if (m < kRoundPieces - 4u) round_piece(sb - 1u, 4u + m);
            // ---- the superblock's sums are complete: ((0.125 d_w) d_a) (128 hi + lo) ----
            if (m == 7u) {
#pragma unroll
                for (unsigned tb = 0; tb < NTB; ++tb)
#pragma unroll
                    for (unsigned i = 0; i < 16u; ++i) {
                        const int total = (sum_hi[tb][i] << 7) + sum_lo[tb][i];
                        const float term = rs[i] * ts[tb] * (float)total;    // each product rounded to float
                        acc[tb][i] += (double)term;
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // ---- publish: the lane holds, for tokens 32 tb + r, rows 8 q + 4 h + j of its wave's 32
    // (j < 4): when fused, q 0-1 are gate rows and q 2-3 the matching up rows ----
    // The values go from the registers straight to memory, 16 bytes a lane: the two halves of a
    // wave complete 32 bytes of a token's row per store, the four (two) stores of a token block
    // a whole cache line (half of one), which the L2 merges before it writes them back. No LDS,
    // no barrier: the stores drain while the next item starts, and copies past the end that are
    // still in flight land in stages and windows nobody reads before the next item has waited
    // for copies of its own, which the same wave issues later to the same places.
    const float limit_f32 = (float)a.limit;
    const bool whole_quads = (a.out_rows & 3u) == 0u;
    bool bad = false;
#pragma unroll
    for (unsigned tb = 0; tb < NTB; ++tb) {
        const unsigned token = tb * 32u + r;
        const uint2 info = lds_read_uint2(kPairInfoBase + token * 8u);   // (stale past the item's last token: not used)
        float *const out_row = pr.out + (unsigned long long)info.x * a.out_rows;
#pragma unroll
        for (unsigned q = 0; q < (FUSED_UP ? 2u : 4u); ++q) {
            const unsigned row = it.row_tile * kItemRows + wave * (FUSED_UP ? 16u : 32u) + 8u * q + 4u * h;
            float value[4];
            bool good = true;
            if constexpr (FUSED_UP) {
                const float route_weight = __uint_as_float(info.y);
#pragma unroll
                for (unsigned j = 0; j < 4u; ++j)
                    value[j] = swiglu_bf16_fast((float)acc[tb][4u * q + j], (float)acc[tb][4u * (q + 2u) + j], route_weight,
                                                a.limit, limit_f32);
            } else {
#pragma unroll
                for (unsigned j = 0; j < 4u; ++j) {
                    value[j] = (float)acc[tb][4u * q + j];
                    good &= finite_f32(value[j]);
                    if (!a.plain_output) value[j] = bf16_round_number(value[j]);   // (a NaN has just been noted)
                }
            }
#pragma unroll
            for (unsigned j = 0; j < 4u; ++j) {
                const bool finite = finite_f32(value[j]);
                good &= finite;
            }
            const bool live = (token < it.tokens) & (row < a.out_rows);
            bad |= live & !good;
            if (live & good) {
                if (whole_quads) {
                    *reinterpret_cast<float4 *>(out_row + row) = make_float4(value[0], value[1], value[2], value[3]);
                } else {
#pragma unroll
                    for (unsigned j = 0; j < 4u; ++j)
                        if (row + j < a.out_rows) out_row[row + j] = value[j];
                }
            }
        }
    }
    if (bad) raise_status(a.status, 1);
    // An item with another number of token blocks lays its stages out differently, so that its
    // copies come from other waves than this item's copies to the same bytes: then this item's
    // last copies land first (the next item's opening barrier makes that hold for every wave).
    const unsigned blocks_next = next.state != 0 ? 0u : next.it.tokens <= 32u ? 1u : 2u;
    if (blocks_next != NTB) __builtin_amdgcn_s_waitcnt(0x0070u);   // vmcnt(0)
}

template <bool FUSED_UP, bool IMAGE>
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

    // The buckets' populations are requested before the tables are built (one round trip to
    // memory under the fill instead of one per bucket after it).
    unsigned long long population_here = 0ull;
    if (tid < 256u && tid < buckets) population_here = fixed ? pr.pairs : pr.bucket_populations[tid];
    mfma_tables_fill();
    // Full 64-pair tiles come first in the item list, then the partial last tiles by size,
    // largest first: every workgroup, walking the list with the grid's stride, gets the same
    // share of each kind of item, and the short items come last. Bucket b's first full tile is
    // the number of full tiles before it (a scan over the 256 bucket slots); its place in its
    // class of partial tiles (more than 32 pairs, or fewer) is its rank among the buckets of
    // that class, in bucket order, from ballots and per-wave totals.
    {
        const unsigned lane = tid & 63u, wave = tid >> 6;
        const unsigned full = tid < 256u ? (unsigned)(population_here / kTileTokens) : 0u;
        const unsigned rest = tid < 256u ? (unsigned)(population_here % kTileTokens) : 0u;
        const unsigned cls = rest == 0u ? 2u : rest > 32u ? 0u : 1u;
        unsigned inclusive = full;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const unsigned below = (unsigned)__shfl_up((int)inclusive, offset, kWave);
            if ((int)lane >= offset) inclusive += below;
        }
        unsigned rank[2];
#pragma unroll
        for (unsigned c = 0; c < 2u; ++c) {
            const unsigned long long members = __ballot(cls == c);
            rank[c] = (unsigned)__popcll(members & ((1ull << lane) - 1ull));
            if (lane == 0u && wave < 4u) lds_write_u32(kTrashBase + 16u + (c * 4u + wave) * 4u, (unsigned)__popcll(members));
        }
        if (lane == 63u && wave < 4u) lds_write_u32(kTrashBase + wave * 4u, inclusive);
        __syncthreads();
        if (tid < 256u) {
            unsigned before = 0u, class_before[2] = {0u, 0u};
            for (unsigned w = 0; w < wave; ++w) {
                before += lds_read_u32(kTrashBase + w * 4u);
                class_before[0] += lds_read_u32(kTrashBase + 16u + w * 4u);
                class_before[1] += lds_read_u32(kTrashBase + 16u + (4u + w) * 4u);
            }
            lds_write_u32(kTileStartBase + 4u * tid, before + inclusive - full);
            if (tid == 255u) lds_write_u32(kTileStartBase + 4u * 256u, before + inclusive);
            if (cls < 2u) lds_write_u16(kClassListBase + (cls * 256u + class_before[cls] + rank[cls]) * 2u, tid);
        }
        if (tid < 2u) {
            unsigned total = 0u;
            for (unsigned w = 0; w < 4u; ++w) total += lds_read_u32(kTrashBase + 16u + (tid * 4u + w) * 4u);
            lds_write_u32(kClassCountBase + 4u * tid, total);
        }
    }
    __syncthreads();
    if (buckets == 0u || buckets > 256u) {
        if (tid == 0u && buckets > 256u) raise_status(a.status, 2);
        return;
    }

    // weight rows (gate/up row pairs when fused) per work item
    constexpr unsigned kItemRows = FUSED_UP ? 128u : 256u;
    const unsigned row_tiles = (a.out_rows + kItemRows - 1u) / kItemRows;
    const unsigned long long full_items = (unsigned long long)lds_read_u32(kTileStartBase + 4u * buckets) * row_tiles;
    unsigned members[2];
    unsigned long long items = full_items;
    for (unsigned c = 0; c < 2u; ++c) {
        members[c] = lds_read_u32(kClassCountBase + 4u * c);
        items += (unsigned long long)members[c] * row_tiles;
    }

    // ---- which bucket, row tile and token tile an item is: the bucket's record is requested... ----
    auto request_item = [&](unsigned long long item) {
        MfmaItemRequest q;
        q.state = 0;
        q.partial = false;
        q.bucket = q.token_tile = q.row_tile = 0u;
        q.first = q.population = q.expert = 0ull;
        if (item >= items) {
            q.state = 2;
            return q;
        }
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
                q.state = 1;
                return q;
            }
            q.bucket = low;
            q.token_tile = (unsigned)(local % bucket_tiles);
            q.row_tile = (unsigned)(local / bucket_tiles);
        } else {
            unsigned long long rest = item - full_items;
            unsigned c = 0u;
            if (rest >= (unsigned long long)members[0] * row_tiles) {
                rest -= (unsigned long long)members[0] * row_tiles;
                c = 1u;
            }
            if (!members[c]) {
                q.state = 1;
                return q;
            }
            q.bucket = lds_read_u16(kClassListBase + (c * 256u + (unsigned)(rest % members[c])) * 2u);
            q.row_tile = (unsigned)(rest / members[c]);
            q.partial = true;               // its token tile is the one after the bucket's full tiles
        }
        if (q.bucket >= buckets) {
            q.state = 1;
            return q;
        }
        q.first = fixed ? 0ull : pr.bucket_offsets[q.bucket];
        q.population = fixed ? pr.pairs : pr.bucket_populations[q.bucket];
        q.expert = fixed ? 0ull : pr.expert_ids[q.bucket];
        return q;
    };
    // ---- ... and looked at later. Every lane holds the same values: the item is kept in scalar
    // registers. ----
    auto uniform32 = [](unsigned v) { return (unsigned)__builtin_amdgcn_readfirstlane((int)v); };
    auto uniform64 = [&](unsigned long long v) {
        return (unsigned long long)uniform32((unsigned)v) | ((unsigned long long)uniform32((unsigned)(v >> 32)) << 32);
    };
    auto resolve_item = [&](const MfmaItemRequest &q, MfmaNextItem &out) {
        out.ahead = false;
        out.shift = 0;
        out.state = (int)uniform32((unsigned)q.state);
        if (out.state == 2) return;
        const unsigned long long first = uniform64(q.first), population = uniform64(q.population);
        const unsigned token_tile = uniform32(q.partial ? (unsigned)(population / kTileTokens) : q.token_tile);
        out.it.expert = uniform64(q.expert);
        out.it.row_tile = uniform32(q.row_tile);
        if (out.state != 0 || out.it.expert >= pr.experts || first + population > pr.pairs ||
            (unsigned long long)token_tile * kTileTokens >= population || out.it.row_tile >= row_tiles) {
            if (tid == 0u) raise_status(a.status, 2);
            out.state = 1;
            return;
        }
        const unsigned long long left = population - (unsigned long long)token_tile * kTileTokens;
        out.it.pair0 = first + (unsigned long long)token_tile * kTileTokens;
        out.it.tokens = left < kTileTokens ? (unsigned)left : kTileTokens;
    };

    unsigned long long item = blockIdx.x;
    MfmaNextItem current;
    resolve_item(request_item(item), current);
    bool prefetched = false;
    while (current.state != 2) {
        MfmaNextItem next;
        const unsigned long long following = item + gridDim.x;
        auto request_next = [&] { return request_item(following); };
        if (current.state == 0) {
            if (current.it.tokens <= 32u)
                rows_item<FUSED_UP, 1u, IMAGE>(a, current.it, prefetched, request_next, resolve_item, next);
            else
                rows_item<FUSED_UP, 2u, IMAGE>(a, current.it, prefetched, request_next, resolve_item, next);
        } else {
            resolve_item(request_next(), next);
        }
        prefetched = current.state == 0 && next.ahead;
        current = next;
        item = following;
    }
}

template <bool FUSED_UP, bool IMAGE>
static int launch_mfma_variant(const MfmaArgs &a, hipStream_t stream)
{
    YVEX_ALLOW_DYNAMIC_LDS((mfma_iq2_kernel<FUSED_UP, IMAGE>), kMfmaLdsBytes);
    mfma_iq2_kernel<FUSED_UP, IMAGE><<<compute_units(), kRowThreads, kMfmaLdsBytes, stream>>>(a);
    return check_launch("moe_rows_mfma");
}

template <bool FUSED_UP>
static int launch_mfma(const MfmaArgs &a, hipStream_t stream)
{
    return a.image ? launch_mfma_variant<FUSED_UP, true>(a, stream)
                   : launch_mfma_variant<FUSED_UP, false>(a, stream);
}

// A plain projection through the row-batch kernel: every input row in one bucket of expert 0.
int launch_iq2_rows_dense(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                          uint64_t row_bytes, const void *act_q8k, uint64_t input_rows, float *out,
                          bool round_bf16, int *status, hipStream_t stream)
{
    int rc = check_matrix(QT_IQ2_XXS, row_width, row_bytes);
    if (rc) return rc;
    if (input_rows > 0xffffffffull || row_count > 0xffffffffull || row_count % 4u) return ST_BOUNDS;
    yvex_hip_expert_weights w{};
    w.down = encoded;
    w.down_qtype = QT_IQ2_XXS;
    w.hidden = row_count;
    w.intermediate = row_width;
    w.down_row_bytes = row_bytes;
    w.down_expert_bytes = row_bytes * row_count;
    MfmaArgs a{};
    const WorklistView none{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    fill_down_problem(a.pr, &w, act_q8k, 1, none, input_rows, 1u, out);
    a.width = (unsigned)row_width;
    a.out_rows = (unsigned)row_count;
    a.limit = 1.0;
    a.status = status;
    a.plain_output = round_bf16 ? 0 : 1;
    return launch_mfma<false>(a, stream);
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
    if (w->gate_qtype != w->up_qtype || (w->gate_qtype != QT_IQ2_XXS && w->gate_qtype != QT_Q4_K))
        return ST_UNSUPPORTED;
    int rc = w->gate_up_image
        ? check_image_matrix(w->gate_qtype, w->hidden, w->gate_row_bytes, w->gate, w->gate_expert_bytes)
        : check_matrix(w->gate_qtype, w->hidden, w->gate_row_bytes);
    if (rc) return rc;
    if (w->up_row_bytes != w->gate_row_bytes) return ST_BOUNDS;
    if (w->gate_up_image && (((uintptr_t)w->up & 3u) || (w->up_expert_bytes & 3u))) return ST_INVALID_ARG;
    if (pairs > 0xffffffffull || w->intermediate > 0xffffffffull || w->intermediate % 4u) return ST_BOUNDS;
    MfmaArgs a{};
    const WorklistView wl{order, expert_ids, bucket_offsets, bucket_populations, nullptr, counts};
    fill_up_problem(a.pr, w, act_q8k, 1, route_weights, wl, pairs, topk, experts, intermediate);
    if (w->gate_qtype == QT_Q4_K)
        return launch_q4k_rows_grouped(a.pr, QT_Q4_K, true, w->hidden, w->intermediate, limit, status, as_stream(stream));
    a.width = (unsigned)w->hidden;
    a.out_rows = (unsigned)w->intermediate;
    a.limit = limit;
    a.status = status;
    a.image = w->gate_up_image != 0;
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
    if (w->down_qtype != QT_IQ2_XXS && w->down_qtype != QT_Q4_K && w->down_qtype != QT_Q2_K) return ST_UNSUPPORTED;
    int rc = w->down_image
        ? check_image_matrix(w->down_qtype, w->intermediate, w->down_row_bytes, w->down, w->down_expert_bytes)
        : check_matrix(w->down_qtype, w->intermediate, w->down_row_bytes);
    if (rc) return rc;
    if (pairs > 0xffffffffull || w->hidden > 0xffffffffull || w->hidden % 4u) return ST_BOUNDS;
    MfmaArgs a{};
    const WorklistView wl{order, expert_ids, bucket_offsets, bucket_populations, nullptr, counts};
    fill_down_problem(a.pr, w, intermediate_q8k, 1, wl, pairs, experts, pair_outputs);
    if (w->down_qtype == QT_Q4_K || w->down_qtype == QT_Q2_K)
        return launch_q4k_rows_grouped(a.pr, w->down_qtype, false, w->intermediate, w->hidden, 1.0, status,
                                       as_stream(stream));
    a.width = (unsigned)w->intermediate;
    a.out_rows = (unsigned)w->hidden;
    a.limit = 1.0;
    a.status = status;
    a.image = w->down_image != 0;
    return launch_mfma<false>(a, as_stream(stream));
}
