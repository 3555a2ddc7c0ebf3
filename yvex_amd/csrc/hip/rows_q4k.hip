// Q4_K (and Q2_K) expert weights against a row batch of Q8_K activations on the int8 matrix cores, operands
// staged through LDS (src/backend/cuda/tensorcore.cu:378-702 is the reference's counterpart, for
// its own formats).
//
// Arithmetic per 256-value superblock as in dense_q4k.hip: the weight operand carries
// sc_j * nibble as two int8 limbs of base 8, one K step of V_MFMA_I32_32X32X32_I8 is one 32-value
// sub-block, the int32 accumulators run over the whole superblock, the minimum term is one more
// K step of depth 8, and
//     value = (d_a * d) * float(dot) - (d_a * dmin) * float(minimum)
// (a float, every operation rounded) is added to the row sums in double, superblock by
// superblock, and a sum is rounded to float once when it is published: the row dot the CPU path
// forms (double accumulation over a row's blocks, src/gguf/quant_compute.c:152-172).
//
// What differs is how the operands arrive. A lane that fetches its own 16-byte pieces of a
// 144-byte weight block and of a 292-byte activation block touches up to 64 cache lines per load
// instruction, and the memory pipeline in front of L1 spends about two cycles per line: some
// 2800 cycles per superblock and wave against 1150 cycles of matrix instructions. Here every
// piece is copied into LDS once per workgroup by GLOBAL_LOAD_LDS instructions whose lanes walk
// consecutive pieces of consecutive rows (a dozen lines an instruction), one superblock ahead of
// the arithmetic, and the operands are LDS reads:
//   * a workgroup of four waves owns a token tile (up to 64 ordered pairs of one bucket) and 128
//     weight rows (64 when gate and up are multiplied side by side: rows 0-15 of a wave are gate
//     rows and rows 16-31 the matching up rows, so a lane ends up holding both factors of the
//     SwiGLU); all waves work on the same superblock and share its activations;
//   * activations: [buffer][token][16 pieces of the 256 int8]; piece c of token t sits at
//     position c ^ (t % 16), applied on the global side of the copy, so the 16 lanes that read
//     one operand column together hit 16 different bank groups; the block scales and the
//     sixteen 16-value sums (bsums) have arrays of their own;
//   * weights: per wave [buffer][32 rows][144 bytes] as in memory (a pitch of 36 dwords keeps 16
//     rows on 16 different bank groups).
// One barrier per superblock publishes the next superblock's copies and retires the reads of
// the buffer they will overwrite.
//
// Q2_K weight rows (a plain projection: the down experts of the reference's model file, whose own
// tensor-core down kernel serves this format only, src/backend/cuda/tensorcore.cu:628-702) run
// through the same tiles, copies and publication. Their operand is simpler: a 2-bit code times its
// sub-block's 4-bit scale is at most 45, one int8 limb, so a K step (two 16-value sub-blocks) is
// one matrix instruction a token block; the minimum term is a K step of depth 16 against the
// Q8_K block's sixteen sums; rows are copied as dwords (84-byte superblocks), pitch 21 dwords.
#include "common.hpp"
#include "launch.hpp"
#include "grouped.hpp"
#include "lds_copy.hpp"

namespace yvex {

namespace {

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

// One 16-byte LDS read (as a vector value, so that it stays one instruction).
__device__ __forceinline__ uint4 read16(unsigned address)
{
    const v4i v = lds_read_v4i(address);
    return make_uint4((unsigned)v[0], (unsigned)v[1], (unsigned)v[2], (unsigned)v[3]);
}

constexpr unsigned kQ4Waves = 4u;
constexpr unsigned kQ4Threads = kQ4Waves * 64u;
constexpr unsigned kQ4Tokens = 64u;                       // token slots of a tile
constexpr unsigned kQ4WeightBytes = 32u * 144u;           // one wave's rows of one superblock
// LDS map (byte addresses; the dynamic block starts at LDS address 0)
constexpr unsigned kQ4WeightBase = 0u;                                          // [wave][buffer]
constexpr unsigned kQ4ActBase = kQ4WeightBase + kQ4Waves * 2u * kQ4WeightBytes; // [buffer][token][256]
constexpr unsigned kQ4ScaleBase = kQ4ActBase + 2u * kQ4Tokens * 256u;           // [buffer][token] f32
constexpr unsigned kQ4BsumBase = kQ4ScaleBase + 2u * kQ4Tokens * 4u;            // [buffer][token][32]
constexpr unsigned kQ4RowScaleBase = kQ4BsumBase + 2u * kQ4Tokens * 32u;        // [wave][d, dmin][32] f32
constexpr unsigned kQ4MetaBase = kQ4RowScaleBase + kQ4Waves * 2u * 32u * 4u;    // tile lookup
constexpr unsigned kQ4TrashBase = kQ4MetaBase + 64u;                            // 1 KB nobody reads
constexpr unsigned kQ4LdsBytes = kQ4TrashBase + 1024u;

struct RowsQ4kArgs {
    GroupedProblem pr;
    unsigned blocks;         // superblocks per weight row
    unsigned out_rows;       // weight rows per expert
    double limit;
    int *status;
    // plain projection (one bucket holding every input row): out[token * out_stride + row]
    int plain, output_bf16;
    const float *additive;
    unsigned long long out_stride;
};

// Two int8 limbs of sc * nibble for the four nibbles of one dword, value = 8 hi + lo (see
// dense_q4k.hip).
__device__ __forceinline__ void q4k_limbs(unsigned x, unsigned sc, unsigned &lo, unsigned &hi)
{
    const unsigned nibbles = x & 0x0f0f0f0fu;
    const unsigned low = (sc & 7u) * 0x00010001u, high = ((sc >> 3) & 7u) * 0x00010001u;
    lo = __builtin_bit_cast(unsigned, __builtin_bit_cast(u16x2, nibbles) * __builtin_bit_cast(u16x2, low));
    hi = __builtin_bit_cast(unsigned, __builtin_bit_cast(u16x2, nibbles) * __builtin_bit_cast(u16x2, high));
}

// Pair sums of the 16 int16 block sums as two int8 limbs (value = 128 hi + lo, lo in 0..127).
__device__ __forceinline__ void q4k_bsum_limbs(const uint4 (&b)[2], uint2 &lo, uint2 &hi)
{
    const unsigned w[8] = {b[0].x, b[0].y, b[0].z, b[0].w, b[1].x, b[1].y, b[1].z, b[1].w};
    unsigned l[2] = {0u, 0u}, u[2] = {0u, 0u};
#pragma unroll
    for (unsigned s = 0; s < 8u; ++s) {
        const int pair = (int)(short)(w[s] & 0xffffu) + ((int)w[s] >> 16);
        l[s >> 2] |= ((unsigned)pair & 127u) << (8u * (s & 3u));
        u[s >> 2] |= ((unsigned)(pair >> 7) & 255u) << (8u * (s & 3u));
    }
    lo = make_uint2(l[0], l[1]);
    hi = make_uint2(u[0], u[1]);
}

// The sixteen int16 block sums as two int8 limbs (value = 128 hi + lo, lo in 0..127), in order.
__device__ __forceinline__ void q2k_bsum_limbs(const uint4 (&b)[2], v4i &lo, v4i &hi)
{
    const unsigned w[8] = {b[0].x, b[0].y, b[0].z, b[0].w, b[1].x, b[1].y, b[1].z, b[1].w};
#pragma unroll
    for (unsigned i = 0; i < 4u; ++i) {
        unsigned l = 0u, u = 0u;
#pragma unroll
        for (unsigned k = 0; k < 4u; ++k) {
            const unsigned word = w[2u * i + k / 2u];
            const int sum = k % 2u ? (int)word >> 16 : (int)(short)(word & 0xffffu);
            l |= ((unsigned)sum & 127u) << (8u * k);
            u |= ((unsigned)(sum >> 7) & 255u) << (8u * k);
        }
        lo[i] = (int)l;
        hi[i] = (int)u;
    }
}

struct Q4Tile {
    unsigned long long expert, first;
    unsigned tokens;
};

// One (token tile, row tile) with NT live 32-token blocks.
template <unsigned QT, bool FUSED, unsigned NT>
__device__ __forceinline__ void rows_q4k_tile(const RowsQ4kArgs &g, const Q4Tile &tile)
{
    static_assert(QT == QT_Q4_K || (QT == QT_Q2_K && !FUSED), "Q4_K rows, or Q2_K rows of a plain projection");
    const GroupedProblem &pr = g.pr;
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned r = lane & 31u, h = lane >> 5;
    constexpr unsigned kWgRows = FUSED ? 64u : 128u;        // output rows of a workgroup
    constexpr unsigned kWaveRows = FUSED ? 16u : 32u;
    const unsigned row0 = blockIdx.x * kWgRows + wave * kWaveRows;   // first output row of this wave
    const unsigned last_block = g.blocks - 1u;

    auto token_row = [&](unsigned token) -> const unsigned char * {
        const unsigned live = token < tile.tokens ? token : tile.tokens - 1u;   // padding repeats a row
        const unsigned long long ordered = tile.first + live;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long act_row = pr.act_by_ordered_pair ? ordered : source / pr.topk;
        return (const unsigned char *)pr.activations + act_row * pr.act_stride;
    };

    // ---- copy sources ----
    // Q4_K weights: piece p = lane + 64 k of this wave's 288 (row p / 9, 16-byte piece p % 9).
    // Q2_K weights: dword p = lane + 64 k of this wave's 672 (row p / 21, dword p % 21: superblocks
    // of 84 bytes are dword-aligned, not more); the eleventh round's upper half repeats the last
    // dword into padding behind the rows.
    constexpr unsigned kRounds = QT == QT_Q2_K ? 11u : 5u;
    constexpr unsigned kPieces = QT == QT_Q2_K ? 21u : 9u, kPieceBytes = QT == QT_Q2_K ? 4u : 16u;
    constexpr unsigned kSuperblockBytes = QT == QT_Q2_K ? 84u : 144u;
    const unsigned char *weight_from[kRounds];
#pragma unroll
    for (unsigned k = 0; k < kRounds; ++k) {
        const unsigned piece = lane + 64u * k;
        const unsigned served = piece < 32u * kPieces ? piece : 32u * kPieces - 1u;
        const unsigned wave_row = served / kPieces;
        unsigned row = row0 + (FUSED ? (wave_row & 15u) : wave_row);
        if (row >= g.out_rows) row = g.out_rows - 1u;        // a ragged edge repeats the last row
        const bool is_up = FUSED && wave_row >= 16u;
        const unsigned char *base = is_up
            ? pr.up + tile.expert * pr.up_expert_bytes + (unsigned long long)row * pr.up_row_bytes
            : pr.gate + tile.expert * pr.expert_bytes + (unsigned long long)row * pr.row_bytes;
        weight_from[k] = base + kPieceBytes * (served % kPieces);
    }
    // activations: position q = tid + 256 k of the tile's 1024 (token q / 16, position q % 16
    // holds piece position ^ (token % 16))
    const unsigned char *act_from[2u * NT];
#pragma unroll
    for (unsigned k = 0; k < 2u * NT; ++k) {
        const unsigned q = tid + 256u * k;
        const unsigned token = q >> 4;
        act_from[k] = token_row(token) + 4u + 16u * ((q & 15u) ^ (token & 15u));
    }
    // wave 0: the block scales (lane = token); waves 1, 2: the bsums (two 16-byte pieces a token)
    const unsigned char *extra_from;
    if (wave == 0u) {
        extra_from = token_row(lane);
    } else {
        const unsigned index = 64u * ((wave - 1u) & 1u) + lane;
        extra_from = token_row(index >> 1) + 260u + 16u * (index & 1u);
    }
    const unsigned weight_base = kQ4WeightBase + wave * 2u * kQ4WeightBytes;
    auto copies = [&](unsigned sb) {
        const unsigned buffer = sb & 1u;
        const unsigned clamped = sb < last_block ? sb : last_block;
        const unsigned long long w_at = (unsigned long long)clamped * kSuperblockBytes;
        const unsigned long long a_at = (unsigned long long)clamped * kQ8KBytes;
        const unsigned w_to = weight_base + buffer * kQ4WeightBytes;
        if constexpr (QT == QT_Q2_K) {
#pragma unroll
            for (unsigned k = 0; k < kRounds; ++k)
                copy_to_lds_4(weight_from[k] + w_at, (unsigned)__builtin_amdgcn_readfirstlane((int)(w_to + 256u * k)));
        } else {
#pragma unroll
            for (unsigned k = 0; k < 4u; ++k)
                copy_to_lds_16(weight_from[k] + w_at, (unsigned)__builtin_amdgcn_readfirstlane((int)(w_to + 1024u * k)));
            copy_to_lds_16_first32(weight_from[4] + w_at, (unsigned)__builtin_amdgcn_readfirstlane((int)(w_to + 4096u)));
        }
#pragma unroll
        for (unsigned k = 0; k < 2u * NT; ++k)
            copy_to_lds_16(act_from[k] + a_at,
                           (unsigned)__builtin_amdgcn_readfirstlane(
                               (int)(kQ4ActBase + buffer * kQ4Tokens * 256u + 16u * (64u * wave + 256u * k))));
        // (wave 3 and, with one token block, part of the others copy into bytes nobody reads,
        // which is cheaper than a branch around the instruction)
        if (wave == 0u)
            copy_to_lds_4(extra_from + a_at,
                          (unsigned)__builtin_amdgcn_readfirstlane((int)(kQ4ScaleBase + buffer * kQ4Tokens * 4u)));
        else
            copy_to_lds_16(extra_from + a_at,
                           (unsigned)__builtin_amdgcn_readfirstlane(
                               (int)(wave == 3u ? kQ4TrashBase
                                                : kQ4BsumBase + buffer * kQ4Tokens * 32u + 1024u * (wave - 1u))));
    };

    double acc[NT][16];      // row sums: a float term per superblock, added in double in superblock order
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[nt][i] = 0.0;

    __syncthreads();      // the previous tile's reads (none in this kernel: one tile a workgroup) are done
    copies(0u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    const unsigned row_scale_at = kQ4RowScaleBase + wave * 256u;
    for (unsigned sb = 0; sb < g.blocks; ++sb) {
        const unsigned buffer = sb & 1u;
        if (sb + 1u < g.blocks) copies(sb + 1u);

        // ---- this lane's weight row of the superblock ----
        const unsigned w_at = weight_base + buffer * kQ4WeightBytes + r * kSuperblockBytes;
        const unsigned a_at = kQ4ActBase + buffer * kQ4Tokens * 256u + r * 256u;
        v16i lo_sum[NT], hi_sum[NT];     // Q2_K: one limb, lo_sum alone
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) lo_sum[nt][i] = hi_sum[nt][i] = 0;
        v4i m_op = {0, 0, 0, 0};         // the minimums of the row's sub-blocks, on the h = 0 half
        if constexpr (QT == QT_Q2_K) {
            // Public ggml block_q2_K (src/backend/cuda/kernel_primitives.h:314-341 is the product):
            // sixteen bytes (scale | minimum << 4) of the 16-value sub-blocks, 64 bytes of 2-bit
            // codes (byte l of half p holds values 128 p + 32 s + l at bit 2 s), fp16 d and dmin.
            // K step c = 4 p + s is the sub-blocks 2 c and 2 c + 1: lane (r, h) scales the sixteen
            // codes of sub-block 2 c + h (at most 3 * 15 = 45, one int8 limb), so one matrix
            // instruction per step and token block.
            const unsigned scale_words[4] = {lds_read_u32(w_at), lds_read_u32(w_at + 4u), lds_read_u32(w_at + 8u),
                                             lds_read_u32(w_at + 12u)};
            const unsigned dd = lds_read_u32(w_at + 80u);
            if (h == 0u) {
                lds_write_u32(row_scale_at + 4u * r, __float_as_uint(f16_bits_to_float(dd & 0xffffu)));
                lds_write_u32(row_scale_at + 128u + 4u * r, __float_as_uint(f16_bits_to_float(dd >> 16)));
#pragma unroll
                for (unsigned i = 0; i < 4u; ++i) m_op[i] = (int)((scale_words[i] >> 4) & 0x0f0f0f0fu);
            }
#pragma unroll
            for (unsigned p = 0; p < 2u; ++p) {
                unsigned q[4];
#pragma unroll
                for (unsigned i = 0; i < 4u; ++i) q[i] = lds_read_u32(w_at + 16u + 32u * p + 16u * h + 4u * i);
#pragma unroll
                for (unsigned sft = 0; sft < 4u; ++sft) {
                    const unsigned c = 4u * p + sft;
                    // scale byte 2 c + h: word c / 2, byte (2 c) % 4 + h
                    const unsigned sc = (scale_words[c >> 1] >> (8u * ((2u * c) & 3u) + 8u * h)) & 15u;
                    const u16x2 twice = __builtin_bit_cast(u16x2, sc * 0x00010001u);
                    v4i a;
#pragma unroll
                    for (unsigned i = 0; i < 4u; ++i)
                        // two bytes a 16-bit lane: (code * sc) stays inside its byte
                        a[i] = (int)__builtin_bit_cast(unsigned,
                                                       __builtin_bit_cast(u16x2, (q[i] >> (2u * sft)) & 0x03030303u) * twice);
#pragma unroll
                    for (unsigned nt = 0; nt < NT; ++nt) {
                        const v4i b = lds_read_v4i(a_at + nt * 32u * 256u + 16u * ((2u * c + h) ^ (r & 15u)));
                        lo_sum[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, lo_sum[nt], 0, 0, 0);
                    }
                }
            }
        } else {
            const uint4 head = read16(w_at);             // d | dmin << 16, then the 12 scale bytes
            const unsigned s0 = head.y, s1 = head.z, s2 = head.w;
            const unsigned sc_pack[2] = {s0 & 0x3f3f3f3fu, (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)};
            const unsigned mn_pack[2] = {s1 & 0x3f3f3f3fu, ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)};
            if (h == 0u) {
                lds_write_u32(row_scale_at + 4u * r, __float_as_uint(f16_bits_to_float(head.x & 0xffffu)));
                lds_write_u32(row_scale_at + 128u + 4u * r, __float_as_uint(f16_bits_to_float(head.x >> 16)));
                // minimum term: m_j (bytes 0..7 of the h = 0 half, zeros elsewhere) against the pair sums
                m_op[0] = (int)mn_pack[0];
                m_op[1] = (int)mn_pack[1];
            }
#pragma unroll
            for (unsigned j = 0; j < 4u; ++j) {
                const uint4 q = read16(w_at + 16u + 32u * j + 16u * h);
#pragma unroll
                for (unsigned half = 0; half < 2u; ++half) {
                    const unsigned c = 2u * j + half;
                    const unsigned sc = (sc_pack[c >> 2] >> (8u * (c & 3u))) & 255u;
                    const unsigned shift = 4u * half;
                    v4i a_lo, a_hi;
                    unsigned lo, hi;
                    q4k_limbs(q.x >> shift, sc, lo, hi); a_lo[0] = (int)lo; a_hi[0] = (int)hi;
                    q4k_limbs(q.y >> shift, sc, lo, hi); a_lo[1] = (int)lo; a_hi[1] = (int)hi;
                    q4k_limbs(q.z >> shift, sc, lo, hi); a_lo[2] = (int)lo; a_hi[2] = (int)hi;
                    q4k_limbs(q.w >> shift, sc, lo, hi); a_lo[3] = (int)lo; a_hi[3] = (int)hi;
#pragma unroll
                    for (unsigned nt = 0; nt < NT; ++nt) {
                        const v4i b = lds_read_v4i(a_at + nt * 32u * 256u + 16u * ((2u * c + h) ^ (r & 15u)));
                        lo_sum[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_lo, b, lo_sum[nt], 0, 0, 0);
                        hi_sum[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_hi, b, hi_sum[nt], 0, 0, 0);
                    }
                }
            }
        }
        // d and dmin of the sixteen rows this lane accumulates (written above by the wave itself)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt) {
            const unsigned token = nt * 32u + r;
            const float da = __uint_as_float(lds_read_u32(kQ4ScaleBase + buffer * kQ4Tokens * 4u + 4u * token));
            v4i b_lo = {0, 0, 0, 0}, b_hi = {0, 0, 0, 0};
            if (h == 0u) {
                const unsigned at = kQ4BsumBase + buffer * kQ4Tokens * 32u + 32u * token;
                const uint4 bsums[2] = {read16(at), read16(at + 16u)};
                if constexpr (QT == QT_Q2_K) {
                    q2k_bsum_limbs(bsums, b_lo, b_hi);       // a minimum per 16 values: the sums as they are
                } else {
                    uint2 bl, bh;
                    q4k_bsum_limbs(bsums, bl, bh);
                    b_lo[0] = (int)bl.x; b_lo[1] = (int)bl.y;
                    b_hi[0] = (int)bh.x; b_hi[1] = (int)bh.y;
                }
            }
            v16i zero;
#pragma unroll
            for (int i = 0; i < 16; ++i) zero[i] = 0;
            const v16i min_lo = __builtin_amdgcn_mfma_i32_32x32x32_i8(m_op, b_lo, zero, 0, 0, 0);
            const v16i min_hi = __builtin_amdgcn_mfma_i32_32x32x32_i8(m_op, b_hi, zero, 0, 0, 0);
#pragma unroll
            for (unsigned q4 = 0; q4 < 4u; ++q4) {
                const uint4 d = read16(row_scale_at + 4u * (8u * q4 + 4u * h));
                const uint4 mn = read16(row_scale_at + 128u + 4u * (8u * q4 + 4u * h));
                const float d_of[4] = {__uint_as_float(d.x), __uint_as_float(d.y), __uint_as_float(d.z),
                                       __uint_as_float(d.w)};
                const float dmin_of[4] = {__uint_as_float(mn.x), __uint_as_float(mn.y), __uint_as_float(mn.z),
                                          __uint_as_float(mn.w)};
#pragma unroll
                for (unsigned k = 0; k < 4u; ++k) {
                    const unsigned i = 4u * q4 + k;
                    const int dot = QT == QT_Q2_K ? lo_sum[nt][i] : (hi_sum[nt][i] << 3) + lo_sum[nt][i];
                    const int minimum = (min_hi[i] << 7) + min_lo[i];
                    const float left = (da * d_of[k]) * (float)dot;
                    const float right = (da * dmin_of[k]) * (float)minimum;
                    acc[nt][i] += (double)(left - right);
                }
            }
        }
        // the next superblock's copies have landed and every wave is done with this one's buffers
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // ---- publish: lane (token r, half h) holds rows 8 (i / 4) + 4 h + i % 4 of the wave's 32 ----
    // Four rows at a time, 16 bytes a lane where the output's geometry allows it (the two halves
    // of a wave then complete 32 bytes of a token's row per store and a token block's stores a
    // whole cache line, which the L2 merges before writing it back); values that are not finite
    // are noted and reported once, so that the pass has few branches.
    const float limit_f32 = (float)g.limit;
    const unsigned long long out_stride = g.plain ? g.out_stride : (unsigned long long)g.out_rows;
    const bool quads = ((g.out_rows | (unsigned)out_stride) & 3u) == 0u &&
                       ((unsigned long long)pr.out & 15ull) == 0ull &&
                       (!(g.plain && g.additive) || ((unsigned long long)g.additive & 15ull) == 0ull);
    bool bad = false;
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt) {
        const unsigned token = nt * 32u + r;
        if (token >= tile.tokens) continue;
        const unsigned long long ordered = tile.first + token;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long out_index = pr.out_by_source_pair ? source : ordered;
        const float route_weight = pr.route_weights ? pr.route_weights[source] : 1.0f;
        constexpr unsigned kQuads = FUSED ? 2u : 4u;
#pragma unroll
        for (unsigned q4 = 0; q4 < kQuads; ++q4) {
            const unsigned row = row0 + 8u * q4 + 4u * h;
            if (row >= g.out_rows) continue;
            const unsigned long long at = out_index * out_stride + row;
            float value[4];
            bool fine[4] = {true, true, true, true};
            if constexpr (FUSED) {
#pragma unroll
                for (unsigned k = 0; k < 4u; ++k)
                    value[k] = swiglu_bf16_fast((float)acc[nt][4u * q4 + k], (float)acc[nt][4u * q4 + k + 8u], route_weight,
                                                g.limit, limit_f32);
            } else {
                const bool add = g.plain && g.additive;
                float extra[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                if (add) {
                    if (quads) {
                        const float4 e = *reinterpret_cast<const float4 *>(g.additive + at);
                        extra[0] = e.x; extra[1] = e.y; extra[2] = e.z; extra[3] = e.w;
                    } else {
#pragma unroll
                        for (unsigned k = 0; k < 4u; ++k)
                            if (row + k < g.out_rows) extra[k] = g.additive[at + k];
                    }
                }
                const bool round = g.plain ? g.output_bf16 != 0 : true;
#pragma unroll
                for (unsigned k = 0; k < 4u; ++k) {
                    value[k] = add ? (float)acc[nt][4u * q4 + k] + extra[k] : (float)acc[nt][4u * q4 + k];
                    fine[k] = finite_f32(value[k]);          // (the rounding below is for numbers)
                    if (round) value[k] = bf16_round_number(value[k]);
                }
            }
#pragma unroll
            for (unsigned k = 0; k < 4u; ++k) fine[k] &= finite_f32(value[k]);
            if (quads & fine[0] & fine[1] & fine[2] & fine[3]) {
                *reinterpret_cast<float4 *>(pr.out + at) = make_float4(value[0], value[1], value[2], value[3]);
            } else {
                // value by value: rows past the last one are not touched, and a value that is
                // not finite is reported instead of stored
#pragma unroll
                for (unsigned k = 0; k < 4u; ++k) {
                    if (row + k >= g.out_rows) continue;
                    bad |= !fine[k];
                    if (fine[k]) pr.out[at + k] = value[k];
                }
            }
        }
    }
    if (bad) raise_status(g.status, 1);
}

template <unsigned QT, bool FUSED>
__global__ __launch_bounds__(kQ4Threads, 2) void rows_q4k_kernel(RowsQ4kArgs g)
{
    extern __shared__ __align__(16) unsigned char rows_q4k_lds[];
    if (lds_address_of(rows_q4k_lds) != 0u) {   // operands are addressed by absolute LDS offsets
        if (threadIdx.x == 0u) raise_status(g.status, 2);
        return;
    }
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const GroupedProblem &pr = g.pr;
    // which bucket holds token tile blockIdx.y (tiles of 64 ordered pairs, numbered bucket by bucket)
    if (threadIdx.x < 6u) lds_write_u32(kQ4MetaBase + 4u * threadIdx.x, 0u);
    __syncthreads();
    if (!pr.expert_ids) {
        if (threadIdx.x == 0u) {
            const unsigned long long first = (unsigned long long)blockIdx.y * kQ4Tokens;
            const unsigned tokens = first < pr.pairs
                ? (unsigned)(pr.pairs - first < kQ4Tokens ? pr.pairs - first : kQ4Tokens) : 0u;
            lds_write_u32(kQ4MetaBase + 8u, (unsigned)first);
            lds_write_u32(kQ4MetaBase + 12u, (unsigned)(first >> 32));
            lds_write_u32(kQ4MetaBase + 16u, tokens);
        }
    } else {
        const unsigned buckets = (unsigned)pr.counts[0];
        const unsigned long long population = threadIdx.x < buckets ? pr.bucket_populations[threadIdx.x] : 0ull;
        const unsigned tiles = (unsigned)((population + kQ4Tokens - 1ull) / kQ4Tokens);
        unsigned inclusive = tiles;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const unsigned below = __shfl_up(inclusive, offset, kWave);
            if ((int)lane >= offset) inclusive += below;
        }
        if (lane == 63u) lds_write_u32(kQ4MetaBase + 32u + 4u * wave, inclusive);
        __syncthreads();
        unsigned before = 0u;
        for (unsigned w = 0; w < wave; ++w) before += lds_read_u32(kQ4MetaBase + 32u + 4u * w);
        inclusive += before;
        const unsigned exclusive = inclusive - tiles;
        if (tiles && blockIdx.y >= exclusive && blockIdx.y < inclusive) {
            const unsigned long long inside = (unsigned long long)(blockIdx.y - exclusive) * kQ4Tokens;
            const unsigned long long expert = pr.expert_ids[threadIdx.x];
            const unsigned long long first = pr.bucket_offsets[threadIdx.x] + inside;
            lds_write_u32(kQ4MetaBase, (unsigned)expert);
            lds_write_u32(kQ4MetaBase + 4u, (unsigned)(expert >> 32));
            lds_write_u32(kQ4MetaBase + 8u, (unsigned)first);
            lds_write_u32(kQ4MetaBase + 12u, (unsigned)(first >> 32));
            lds_write_u32(kQ4MetaBase + 16u, (unsigned)(population - inside < kQ4Tokens ? population - inside : kQ4Tokens));
        }
    }
    __syncthreads();
    Q4Tile tile;
    tile.expert = (unsigned long long)lds_read_u32(kQ4MetaBase) | ((unsigned long long)lds_read_u32(kQ4MetaBase + 4u) << 32);
    tile.first = (unsigned long long)lds_read_u32(kQ4MetaBase + 8u) | ((unsigned long long)lds_read_u32(kQ4MetaBase + 12u) << 32);
    tile.tokens = lds_read_u32(kQ4MetaBase + 16u);
    if (!tile.tokens) return;                               // a tile number past the last bucket
    if (tile.expert >= pr.experts || tile.first + tile.tokens > pr.pairs) {
        if (threadIdx.x == 0u) raise_status(g.status, 2);
        return;
    }
    if (tile.tokens > 32u) rows_q4k_tile<QT, FUSED, 2u>(g, tile);
    else rows_q4k_tile<QT, FUSED, 1u>(g, tile);
}

template <unsigned QT, bool FUSED>
int launch_rows_q4k(const RowsQ4kArgs &g, dim3 grid, hipStream_t stream)
{
    YVEX_ALLOW_DYNAMIC_LDS((rows_q4k_kernel<QT, FUSED>), kQ4LdsBytes);
    rows_q4k_kernel<QT, FUSED><<<grid, kQ4Threads, kQ4LdsBytes, stream>>>(g);
    return check_launch("rows_q4k");
}

}  // namespace

int launch_q4k_rows_grouped(const GroupedProblem &problem, unsigned qtype, bool fused, uint64_t width,
                            uint64_t out_rows, double limit, int *status, hipStream_t stream)
{
    if (qtype != QT_Q4_K && !(qtype == QT_Q2_K && !fused)) return ST_UNSUPPORTED;
    if (!width || width % 256u || !out_rows || out_rows > 0x7fffffffull) return ST_BOUNDS;
    const uint64_t superblock = qtype == QT_Q2_K ? 84u : 144u;
    // (Q4_K rows are copied in 16-byte pieces, Q2_K rows in dwords)
    const uintptr_t misaligned = qtype == QT_Q2_K ? 3u : 15u;
    if (problem.row_bytes != width / 256u * superblock || (fused && problem.up_row_bytes != problem.row_bytes))
        return ST_BOUNDS;
    if (((uintptr_t)problem.gate & misaligned) || (fused && ((uintptr_t)problem.up & 15u)) ||
        ((uintptr_t)problem.activations & 3u) || (problem.expert_bytes & misaligned) ||
        (fused && (problem.up_expert_bytes & 15u)) || (problem.act_stride & 3u))
        return ST_INVALID_ARG;
    if (problem.experts > 256u && problem.expert_ids) return ST_BOUNDS;
    const uint64_t row_tiles = (out_rows + (fused ? 63u : 127u)) / (fused ? 64u : 128u);
    // token tiles: every bucket may end in a partial tile
    const uint64_t token_tiles = problem.expert_ids ? (uint64_t)problem.pairs / kQ4Tokens + problem.experts
                                                    : ((uint64_t)problem.pairs + kQ4Tokens - 1u) / kQ4Tokens;
    if (row_tiles > 0x7fffffffull || token_tiles > 65535ull) return ST_BOUNDS;
    RowsQ4kArgs g{problem, (unsigned)(width / 256u), (unsigned)out_rows, limit, status, 0, 0, nullptr, 0ull};
    const dim3 grid((unsigned)row_tiles, (unsigned)token_tiles);
    if (qtype == QT_Q2_K) return launch_rows_q4k<QT_Q2_K, false>(g, grid, stream);
    return fused ? launch_rows_q4k<QT_Q4_K, true>(g, grid, stream) : launch_rows_q4k<QT_Q4_K, false>(g, grid, stream);
}

// A plain projection of many input rows: one bucket that holds them all, outputs left in fp32
// (or rounded when the caller asks for bf16), additive rows allowed.
int launch_q4k_rows_staged(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                           uint64_t row_bytes, const void *act_q8k, uint64_t input_rows,
                           const float *additive, float *out, uint64_t out_stride, bool output_bf16,
                           int *status, hipStream_t stream)
{
    if (!row_count || !input_rows || row_width % 256u || row_width / 256u * 144u != row_bytes ||
        row_count > 0x7fffffffull || input_rows > 0xffffffffull)
        return ST_BOUNDS;
    if (((uintptr_t)encoded & 15u) || ((uintptr_t)act_q8k & 3u)) return ST_INVALID_ARG;
    GroupedProblem problem{};
    problem.gate = encoded;
    problem.row_bytes = row_bytes;
    problem.activations = act_q8k;
    problem.act_stride = row_width / 256u * kQ8KBytes;
    problem.act_by_ordered_pair = 1;
    problem.pairs = (unsigned)input_rows;
    problem.topk = 1u;
    problem.experts = 1u;
    problem.out = out;
    const uint64_t row_tiles = (row_count + 127u) / 128u;
    const uint64_t token_tiles = (input_rows + kQ4Tokens - 1u) / kQ4Tokens;
    if (token_tiles > 65535ull) return ST_BOUNDS;
    RowsQ4kArgs g{problem, (unsigned)(row_width / 256u), (unsigned)row_count, 0.0, status, 1, output_bf16 ? 1 : 0,
                  additive, out_stride};
    return launch_rows_q4k<QT_Q4_K, false>(g, dim3((unsigned)row_tiles, (unsigned)token_tiles), stream);
}

}  // namespace yvex
