// Q8_0 weight rows against a batch of Q8_K input rows on the int8 matrix cores: the dense
// projection at prefill width (the reference turns its tensor-core kernels on from 16 input rows
// for every format that takes Q8 activations, src/backend/cuda/private.h:461-464,
// src/backend/cuda/qtype.c:252-255).
//
// Arithmetic, as the reference's primitive forms it for one 256-value superblock
// (src/backend/cuda/kernel_primitives.h:342-359) and the CPU path adds a row's superblocks
// (src/gguf/quant_compute.c:152-172):
//     dot_b = sum_i q_i * a_i                              (int32, exact: one K step of V_MFMA_I32_32X32X32_I8)
//     total = fmaf(d_b * d_a, float(dot_b), total)         b = 0 .. 7 in order, floats, from zero
//     row  += double(total)                                superblock by superblock, rounded to float once
// A block has a scale of its own, so every matrix instruction starts from zero and its sixteen
// results a lane are converted, scaled and chained on the vector ALU (three instructions each).
//
// A workgroup owns 32 weight rows x 32 input rows; its four waves take every fourth superblock
// (eight blocks, 272 bytes a row) and their partial tiles are added in wave order, so results do
// not depend on timing. The input rows are the A operand and the weight rows the B operand: lane (r, h) holds bytes 16 h .. 16 h + 15 of input row r's block and
// of weight row r's block, and accumulator i of that lane is weight row r against input row
// 8 (i / 4) + 4 h + i % 4, so a block's scale is one value a lane. Blocks start on 2-byte
// boundaries (34 bytes each): the codes of an even block are read as five aligned dwords and
// shifted into place, those of an odd block are dword-aligned as they lie.
#include "common.hpp"
#include "launch.hpp"
#include "lds_copy.hpp"

namespace yvex {

namespace {

struct DenseQ80Args {
    const unsigned char *encoded;
    unsigned long long row_count, row_bytes;
    unsigned blocks;                         // superblocks (256 columns) per row
    const unsigned char *act;                // Q8_K rows, blocks * 292 bytes each
    unsigned long long input_rows;
    const float *additive;
    float *out;
    unsigned long long out_stride;
    int output_bf16;
    int *status;
};

// What a lane needs of one superblock: its half of the eight blocks' codes (their scales lie in
// the same windows) and its half of one input row's blocks.
struct Q80Inputs {
    uint4 codes[8];         // even blocks: the aligned window two bytes in front of the codes
    unsigned tail[4];       // even blocks: the dword behind the window
    uint4 a[8];
    float act_scale;
};

__device__ __forceinline__ void q80_load(const unsigned char *wrow, const unsigned char *arow, unsigned sb,
                                         unsigned h, Q80Inputs &in)
{
    const unsigned char *w = wrow + (unsigned long long)sb * 272ull;     // dword-aligned
#pragma unroll
    for (unsigned c = 0; c < 8u; ++c) {
        // block c starts at 34 c: two bytes past a dword boundary when c is odd
        const unsigned codes = 34u * c + 2u + 16u * h;
        if (c % 2u == 0u) {
            const unsigned *p = reinterpret_cast<const unsigned *>(w + codes - 2u);
            in.codes[c] = make_uint4(p[0], p[1], p[2], p[3]);
            in.tail[c / 2u] = p[4];
        } else {
            const unsigned *p = reinterpret_cast<const unsigned *>(w + codes);
            in.codes[c] = make_uint4(p[0], p[1], p[2], p[3]);
        }
    }
    const unsigned char *a = arow + (unsigned long long)sb * kQ8KBytes;
    in.act_scale = *reinterpret_cast<const float *>(a);
#pragma unroll
    for (unsigned c = 0; c < 8u; ++c) {
        const unsigned *p = reinterpret_cast<const unsigned *>(a + 4u + 32u * c + 16u * h);
        in.a[c] = make_uint4(p[0], p[1], p[2], p[3]);
    }
}

constexpr unsigned kPlainWaves = 4u;

__global__ __launch_bounds__(64 * kPlainWaves) void dense_q8_0_kernel(DenseQ80Args g)
{
    // per wave: the scales of the input rows whose blocks its lanes hold; then the partial tiles
    __shared__ __align__(16) float row_scale[kPlainWaves][32];
    __shared__ double partial[kPlainWaves - 1u][16][64];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned r = lane & 31u, h = lane >> 5;
    const unsigned long long row0 = (unsigned long long)blockIdx.x * 32ull;
    const unsigned long long tok0 = (unsigned long long)blockIdx.y * 32ull;
    unsigned long long wr = row0 + r;
    if (wr >= g.row_count) wr = g.row_count - 1ull;              // a ragged edge repeats the last row
    const unsigned char *wrow = g.encoded + wr * g.row_bytes;
    unsigned long long t = tok0 + r;
    if (t >= g.input_rows) t = g.input_rows - 1ull;
    const unsigned char *arow = g.act + t * ((unsigned long long)g.blocks * kQ8KBytes);
    double acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0;

    Q80Inputs cur;
    q80_load(wrow, arow, wave < g.blocks ? wave : 0u, h, cur);
    for (unsigned sb = wave; sb < g.blocks; sb += kPlainWaves) {
        // the next superblock's bytes travel while this one is worked on
        Q80Inputs nxt;
        q80_load(wrow, arow, sb + kPlainWaves < g.blocks ? sb + kPlainWaves : sb, h, nxt);

        // The block scales lie in the windows already: an even block's in front of its codes (the
        // low half of the first dword of the lane with h = 0), an odd block's behind the codes of
        // the block before it (the high half of the tail dword of the lane with h = 1). Each half
        // packs its four and takes the other half's from the lane 32 away.
        unsigned mine[2], theirs[2];
#pragma unroll
        for (unsigned j = 0; j < 2u; ++j) {
            const unsigned first = h ? cur.tail[2u * j] >> 16 : cur.codes[4u * j].x & 0xffffu;
            const unsigned second = h ? cur.tail[2u * j + 1u] >> 16 : cur.codes[4u * j + 2u].x & 0xffffu;
            mine[j] = first | (second << 16);
            theirs[j] = (unsigned)__shfl_xor((int)mine[j], 32, 64);
        }
        float d_w[8];
#pragma unroll
        for (unsigned c = 0; c < 8u; ++c) {
            const unsigned pack = (c % 2u == h) ? mine[c / 4u] : theirs[c / 4u];     // blocks c with c % 2 == h are mine
            d_w[c] = f16_bits_to_float((c / 2u) % 2u ? pack >> 16 : pack & 0xffffu);
        }
        // the input rows' scales to the lanes that hold their sums
        row_scale[wave][r] = cur.act_scale;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        float d_a[16], total[16];       // the input rows' scales; the superblock's chain of eight terms
#pragma unroll
        for (unsigned q4 = 0; q4 < 4u; ++q4) {
            const float4 d = *reinterpret_cast<const float4 *>(&row_scale[wave][8u * q4 + 4u * h]);
            d_a[4u * q4] = d.x; d_a[4u * q4 + 1u] = d.y; d_a[4u * q4 + 2u] = d.z; d_a[4u * q4 + 3u] = d.w;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) total[i] = 0.0f;
#pragma unroll
        for (unsigned c = 0; c < 8u; ++c) {
            v4i codes;
            if (c % 2u == 0u) {
                const uint4 q = cur.codes[c];
                codes[0] = (int)__builtin_amdgcn_alignbyte(q.y, q.x, 2u);
                codes[1] = (int)__builtin_amdgcn_alignbyte(q.z, q.y, 2u);
                codes[2] = (int)__builtin_amdgcn_alignbyte(q.w, q.z, 2u);
                codes[3] = (int)__builtin_amdgcn_alignbyte(cur.tail[c / 2u], q.w, 2u);
            } else {
                codes[0] = (int)cur.codes[c].x; codes[1] = (int)cur.codes[c].y;
                codes[2] = (int)cur.codes[c].z; codes[3] = (int)cur.codes[c].w;
            }
            v16i zero;
#pragma unroll
            for (int i = 0; i < 16; ++i) zero[i] = 0;
            const v4i tokens = {(int)cur.a[c].x, (int)cur.a[c].y, (int)cur.a[c].z, (int)cur.a[c].w};
            const v16i dot = __builtin_amdgcn_mfma_i32_32x32x32_i8(tokens, codes, zero, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 16; ++i) total[i] = __builtin_fmaf(d_w[c] * d_a[i], (float)dot[i], total[i]);
            // (left alone the scheduler issues the matrix instructions of all blocks first and
            // keeps their results)
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] += (double)total[i];
        // (the next superblock's scales are not written before every lane has read these)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        cur = nxt;
    }

    if (wave) {
#pragma unroll
        for (int i = 0; i < 16; ++i) partial[wave - 1u][i][lane] = acc[i];
    }
    __syncthreads();
    if (wave) return;
    // lane (r, h): weight row r against sixteen input rows; a store instruction writes 32
    // consecutive floats of two output rows
    const unsigned long long row = row0 + r;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const unsigned long long token = tok0 + 8u * (i >> 2) + 4u * h + (i & 3);
        double wide = acc[i];
#pragma unroll
        for (unsigned w = 0; w + 1u < kPlainWaves; ++w) wide += partial[w][i][lane];
        const float sum = (float)wide;
        if (row >= g.row_count || token >= g.input_rows) continue;
        const unsigned long long at = token * g.out_stride + row;
        const float value = g.additive ? sum + g.additive[at] : sum;
        if (!finite_f32(value)) raise_status(g.status, 1);
        else g.out[at] = g.output_bf16 ? bf16_round(value) : value;
    }
}

// The same product for batches that offer every compute unit a tile of 128 weight rows x 64
// input rows: the operands of one superblock pass through LDS. GLOBAL_LOAD_LDS instructions whose
// lanes walk consecutive 16-byte pieces of consecutive rows (a dozen cache lines an instruction
// where the kernel above touches up to 64) fill the other of two buffers while this one is
// multiplied; one barrier per superblock. A weight row keeps its 272 bytes and an input row's 256
// codes get the same pitch, its scale (the row's first 16 bytes) as a seventeenth piece behind
// them, so the 16-byte operand reads of 16 lanes fall on 16 different bank groups. The window of
// a block's codes is not 16-byte aligned in its row: a lane reads the two aligned pieces around
// it and picks its dwords (the offsets are compile-time constants).
//
// Eight waves, two per SIMD, each 32 weight rows x 32 input rows over the whole row width: no
// partial tiles. Here the input rows are the A operand and the weight rows the B operand, so lane
// (r, h) holds weight row r against input rows 8 (i / 4) + 4 h + i % 4: the block's scale is one
// value a lane (read from the row's bytes in LDS) and the input rows' scales, needed once a
// superblock, are sixteen broadcast reads.
//
// ROW_BLOCKS = 4: the tile above (512 lanes, 104 KB of LDS, a workgroup a compute unit);
// ROW_BLOCKS = 2: 64 weight rows, four waves, 70 KB, two workgroups a compute unit, for batches
// that have too few of the large tiles.
// TOKEN_BLOCKS = 1 (with ROW_BLOCKS = 8: 256 weight rows x 32 input rows, 153 KB): batches of up to
// 32 input rows against a matrix too large for the caches, an output head at decode width, where
// the second block of input rows would be padding and half of every wave's work with it.
constexpr unsigned kStagedPitch = 272u;
constexpr unsigned staged_lds_bytes(unsigned row_blocks, unsigned token_blocks = 2u)
{
    return 2u * (32u * row_blocks + 32u * token_blocks) * kStagedPitch;
}

__device__ __forceinline__ uint4 read16(unsigned address)
{
    const v4i v = lds_read_v4i(address);
    return make_uint4((unsigned)v[0], (unsigned)v[1], (unsigned)v[2], (unsigned)v[3]);
}

template <unsigned ROW_BLOCKS, unsigned TOKEN_BLOCKS = 2u>
__global__ __launch_bounds__(64 * ROW_BLOCKS * TOKEN_BLOCKS) void dense_q8_0_staged_kernel(DenseQ80Args g)
{
    constexpr unsigned kStagedThreads = 64u * ROW_BLOCKS * TOKEN_BLOCKS, kStagedRows = 32u * ROW_BLOCKS;
    constexpr unsigned kStagedTokens = 32u * TOKEN_BLOCKS;
    constexpr unsigned kStagedActBytes = kStagedTokens * kStagedPitch;                  // one buffer
    constexpr unsigned kStagedWeightBytes = kStagedRows * kStagedPitch;                 // one buffer
    constexpr unsigned kStagedWeightBase = 0u;                                          // [buffer]
    constexpr unsigned kStagedActBase = kStagedWeightBase + 2u * kStagedWeightBytes;    // [buffer]
    constexpr unsigned kWeightRounds = kStagedRows * 17u / kStagedThreads;              // full rounds of copies
    constexpr unsigned kWeightRest = (kStagedRows * 17u - kWeightRounds * kStagedThreads) / 64u;   // waves of the last
    constexpr unsigned kActRounds = kStagedTokens * 17u / kStagedThreads;
    constexpr unsigned kActRest = (kStagedTokens * 17u - kActRounds * kStagedThreads) / 64u;
    constexpr unsigned kActTail = (kStagedTokens * 17u - kActRounds * kStagedThreads) % 64u;    // lanes of one more wave
    static_assert((kStagedRows * 17u) % 64u == 0u && (kActTail == 0u || kActTail == 32u), "whole or half waves copy");
    static_assert(kWeightRounds + 1u <= 10u && kActRounds + 1u <= 5u, "copy sources");
    extern __shared__ __align__(16) unsigned char dense_q8_0_lds[];
    if (lds_address_of(dense_q8_0_lds) != 0u) {   // operands are addressed by absolute LDS offsets
        if (threadIdx.x == 0u) raise_status(g.status, 2);
        return;
    }
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned r = lane & 31u, h = lane >> 5;
    const unsigned row_block = wave % ROW_BLOCKS, token_block = wave / ROW_BLOCKS;
    const unsigned long long row0 = (unsigned long long)blockIdx.x * kStagedRows;
    const unsigned long long tok0 = (unsigned long long)blockIdx.y * kStagedTokens;
    const unsigned rows_here = (unsigned)(g.row_count - row0 < kStagedRows ? g.row_count - row0 : kStagedRows);
    const unsigned toks_here = (unsigned)(g.input_rows - tok0 < kStagedTokens ? g.input_rows - tok0 : kStagedTokens);
    const unsigned long long act_row_bytes = (unsigned long long)g.blocks * kQ8KBytes;

    // ---- copy sources (a ragged edge repeats the tile's last row) ----
    // weights: piece q = tid + threads * k of the tile's rows x 17; input rows: piece q of 64 x 17,
    // the seventeenth being the 16 bytes at the row's start
    const unsigned char *weight_from[kWeightRounds + 1u], *act_from[kActRounds + 1u];
#pragma unroll
    for (unsigned k = 0; k < kWeightRounds + 1u; ++k) {
        unsigned q = tid + kStagedThreads * k;
        if (q >= kStagedRows * 17u) q = kStagedRows * 17u - 1u;            // (waves that do not copy this round)
        const unsigned row = q / 17u, piece = q - row * 17u;
        weight_from[k] = g.encoded + (row0 + (row < rows_here ? row : rows_here - 1u)) * g.row_bytes + 16u * piece;
    }
#pragma unroll
    for (unsigned k = 0; k < kActRounds + 1u; ++k) {
        unsigned q = tid + kStagedThreads * k;
        if (q >= kStagedTokens * 17u) q = kStagedTokens * 17u - 1u;
        const unsigned token = q / 17u, piece = q - token * 17u;
        act_from[k] = g.act + (tok0 + (token < toks_here ? token : toks_here - 1u)) * act_row_bytes +
                      (piece < 16u ? 4u + 16u * piece : 0u);
    }
    const unsigned last_block = g.blocks - 1u;
    auto copies = [&](unsigned sb) {
        const unsigned buffer = sb & 1u;
        const unsigned clamped = sb < last_block ? sb : last_block;
        const unsigned long long w_at = (unsigned long long)clamped * 272ull;
        const unsigned long long a_at = (unsigned long long)clamped * kQ8KBytes;
        const unsigned w_to = kStagedWeightBase + buffer * kStagedWeightBytes + 1024u * wave;
        const unsigned a_to = kStagedActBase + buffer * kStagedActBytes + 1024u * wave;
#pragma unroll
        for (unsigned k = 0; k < kWeightRounds; ++k)
            copy_to_lds_16(weight_from[k] + w_at,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(w_to + 16u * kStagedThreads * k)));
        if (wave < kWeightRest)
            copy_to_lds_16(weight_from[kWeightRounds] + w_at,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(w_to + 16u * kStagedThreads * kWeightRounds)));
#pragma unroll
        for (unsigned k = 0; k < kActRounds; ++k)
            copy_to_lds_16(act_from[k] + a_at,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(a_to + 16u * kStagedThreads * k)));
        if (wave < kActRest)
            copy_to_lds_16(act_from[kActRounds] + a_at,
                           (unsigned)__builtin_amdgcn_readfirstlane((int)(a_to + 16u * kStagedThreads * kActRounds)));
        else if (kActTail && wave == kActRest)
            copy_to_lds_16_first32(act_from[kActRounds] + a_at,
                                   (unsigned)__builtin_amdgcn_readfirstlane((int)(a_to + 16u * kStagedThreads * kActRounds)));
    };

    double acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0;

    copies(0u);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    for (unsigned sb = 0; sb < g.blocks; ++sb) {
        const unsigned buffer = sb & 1u;
        if (sb + 1u < g.blocks) copies(sb + 1u);
        const unsigned w_row = kStagedWeightBase + buffer * kStagedWeightBytes + (32u * row_block + r) * kStagedPitch;
        const unsigned a_tile = kStagedActBase + buffer * kStagedActBytes + 32u * token_block * kStagedPitch;

        float d_a[16], total[16];   // the input rows' scales; the superblock's chain of eight terms
#pragma unroll
        for (unsigned i = 0; i < 16u; ++i) {
            const unsigned token = 8u * (i >> 2) + 4u * h + (i & 3u);
            d_a[i] = __uint_as_float(lds_read_u32(a_tile + token * kStagedPitch + 256u));
            total[i] = 0.0f;
        }
        // Three stages in flight, or a wave would run its LDS reads, its matrix instruction and the
        // scaling of the results one after the other: in step k the operands of block k are
        // read, block k - 1 is multiplied and the results of block k - 2 are scaled (vector
        // instructions that issue while the matrix pipe works).
        uint4 lo[2], hi[2];
        v4i tokens[2];
        unsigned scale_bits[2];
        v16i dot[2];
        float d_w[2];
#pragma unroll
        for (unsigned k = 0; k < 10u; ++k) {
            if (k < 8u) {
                const unsigned c = k, slot = c % 2u;
                const unsigned start = c % 2u == 0u ? 34u * c : 34u * c + 2u;      // the lane's window: + 16 h
                lo[slot] = read16(w_row + 16u * h + (start & ~15u));
                // (an even block's window is 20 bytes, an odd block's 16: only block 7's fits one piece)
                hi[slot] = c % 2u == 0u || (start & 15u) ? read16(w_row + 16u * h + (start & ~15u) + 16u) : lo[slot];
                scale_bits[slot] = lds_read_u16(w_row + 34u * c);
                tokens[slot] = lds_read_v4i(a_tile + r * kStagedPitch + 16u * (2u * c + h));
            }
            if (k >= 1u && k < 9u) {
                const unsigned c = k - 1u, slot = c % 2u;
                const unsigned start = c % 2u == 0u ? 34u * c : 34u * c + 2u;
                const unsigned at = (start & 15u) / 4u;
                const unsigned q[8] = {lo[slot].x, lo[slot].y, lo[slot].z, lo[slot].w,
                                       hi[slot].x, hi[slot].y, hi[slot].z, hi[slot].w};
                v4i codes;
                if (c % 2u == 0u) {
#pragma unroll
                    for (unsigned j = 0; j < 4u; ++j)
                        codes[j] = (int)__builtin_amdgcn_alignbyte(q[at + j + 1u], q[at + j], 2u);
                } else {
#pragma unroll
                    for (unsigned j = 0; j < 4u; ++j) codes[j] = (int)q[at + j];
                }
                v16i zero;
#pragma unroll
                for (int i = 0; i < 16; ++i) zero[i] = 0;
                dot[slot] = __builtin_amdgcn_mfma_i32_32x32x32_i8(tokens[slot], codes, zero, 0, 0, 0);
                d_w[slot] = f16_bits_to_float(scale_bits[slot]);
            }
            if (k >= 2u) {
                const unsigned slot = k % 2u;           // block k - 2
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    total[i] = __builtin_fmaf(d_w[slot] * d_a[i], (float)dot[slot][i], total[i]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] += (double)total[i];
        // the next superblock's copies have landed and every wave is done with this one's buffers
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // lane (r, h): weight row r of the wave's 32 against sixteen input rows; a store instruction
    // writes 32 consecutive floats of two output rows
    const unsigned long long row = row0 + 32u * row_block + r;
    if (row >= g.row_count) return;
    bool bad = false;
#pragma unroll
    for (unsigned i = 0; i < 16u; ++i) {
        const unsigned long long token = tok0 + 32u * token_block + 8u * (i >> 2) + 4u * h + (i & 3u);
        if (token >= g.input_rows) continue;
        const unsigned long long at = token * g.out_stride + row;
        const float sum = (float)acc[i];
        const float value = g.additive ? sum + g.additive[at] : sum;
        if (!finite_f32(value)) bad = true;
        else g.out[at] = g.output_bf16 ? bf16_round(value) : value;
    }
    if (bad) raise_status(g.status, 1);
}

}  // namespace

int launch_q8_0_rows_dense(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                           uint64_t row_bytes, const void *act_q8k, uint64_t input_rows,
                           const float *additive, float *out, uint64_t out_stride, bool output_bf16,
                           int *status, hipStream_t stream)
{
    if (!row_count || !input_rows || row_width % 256u || row_width / 32u * 34u != row_bytes)
        return ST_BOUNDS;
    if (((uintptr_t)encoded & 3u) || ((uintptr_t)act_q8k & 3u)) return ST_INVALID_ARG;
    const uint64_t row_tiles = (row_count + 31u) / 32u;
    if (row_tiles > 0x7fffffffull || row_width / 256u > 0xffffffffull) return ST_BOUNDS;
    DenseQ80Args g{encoded, row_count, row_bytes, (unsigned)(row_width / 256u),
                   (const unsigned char *)act_q8k, input_rows, additive, out, out_stride,
                   output_bf16 ? 1 : 0, status};
    // Which tiles: a pass over the row width costs a workgroup about the same whatever the device's
    // load (measured at 16 superblocks a row, microseconds: 17 unstaged and 27 once two such
    // workgroups share a compute unit, 29 on the 64-row staged tile and 43 once two of them share
    // a compute unit, 35 on the 128-row tile), so the choice is the number of rounds each shape needs.
    const uint64_t token_tiles32 = (input_rows + 31u) / 32u;
    const uint64_t token_tiles64 = (input_rows + 63u) / 64u;
    if (token_tiles32 > 65535ull) return ST_BOUNDS;
    const uint64_t units = (uint64_t)compute_units();
    // up to 32 input rows against a matrix with a 256-row tile for every compute unit (an output
    // head at decode width, 129 280 x 7168: 306 us on the 128 x 64 tiles, half of them padding;
    // memory time 173 us)
    if (!((uintptr_t)encoded & 15u) && input_rows <= 32u && units && (row_count + 255u) / 256u >= units) {
        YVEX_ALLOW_DYNAMIC_LDS((dense_q8_0_staged_kernel<8u, 1u>), staged_lds_bytes(8u, 1u));
        dense_q8_0_staged_kernel<8u, 1u><<<dim3((unsigned)((row_count + 255u) / 256u), 1), 512, staged_lds_bytes(8u, 1u),
                                           stream>>>(g);
        return check_launch("dense_q8_0_staged");
    }
    if (!((uintptr_t)encoded & 15u) && units) {
        const uint64_t plain = row_tiles * token_tiles32;
        const uint64_t tall = (row_count + 127u) / 128u * token_tiles64, low = (row_count + 63u) / 64u * token_tiles64;
        const double plain_cost = plain <= units ? 17.0 : 27.0 * (double)((plain + 2u * units - 1u) / (2u * units));
        const double low_share = 43.0 * (double)low / (double)(2u * units);
        const double low_cost = low <= units ? 29.0 : (low_share > 43.0 ? low_share : 43.0);
        const double tall_cost = 35.0 * (double)((tall + units - 1u) / units);
        if (tall_cost < plain_cost && tall_cost <= low_cost) {
            YVEX_ALLOW_DYNAMIC_LDS(dense_q8_0_staged_kernel<4u>, staged_lds_bytes(4u));
            dense_q8_0_staged_kernel<4u><<<dim3((unsigned)((row_count + 127u) / 128u), (unsigned)token_tiles64), 512,
                                          staged_lds_bytes(4u), stream>>>(g);
            return check_launch("dense_q8_0_staged");
        }
        if (low_cost < plain_cost) {
            YVEX_ALLOW_DYNAMIC_LDS(dense_q8_0_staged_kernel<2u>, staged_lds_bytes(2u));
            dense_q8_0_staged_kernel<2u><<<dim3((unsigned)((row_count + 63u) / 64u), (unsigned)token_tiles64), 256,
                                          staged_lds_bytes(2u), stream>>>(g);
            return check_launch("dense_q8_0_staged");
        }
    }
    dense_q8_0_kernel<<<dim3((unsigned)row_tiles, (unsigned)token_tiles32), 64 * kPlainWaves, 0, stream>>>(g);
    return check_launch("dense_q8_0");
}

}  // namespace yvex
