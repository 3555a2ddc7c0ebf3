// Decode-width expert sweeps specialised for IQ2_XXS (and, with the same item list, streams and
// finishing pass, Q4_K rows and the Q2_K rows of a down projection) weights and Q8_K activations
// on gfx950. The notes below are about IQ2_XXS; what differs for Q4_K rows stands above
// `Q4kHalf`, for Q2_K rows above `Q2kHalf`.
//
// Same contract as the generic grouped kernel in moe.hip (src/backend/cuda/moe_kernels.cu:431-582
// is the reference's counterpart), built around the instruction budget of this one format: at
// 2.0625 bits per weight the vector ALU, not HBM, is the first limit, so every 32-weight unit is
// decoded with as few vector instructions as the format allows.
//
//   * magnitudes: one 16-byte LDS read returns the eight level bytes of a codebook entry and their
//     negations; signs: one 8-byte LDS read returns two byte-permute selectors for the 7 stored
//     sign bits plus parity; V_PERM_B32 then picks +level or -level per byte. Four signed weights
//     cost one vector instruction after the two reads.
//   * a sweep serves up to four (row, rank) pairs of a bucket, whose Q8_K columns stay in
//     registers (128 columns per lane), so an expert's bytes are decoded once for most buckets.
//   * the exact int32 superblock sum (kernel_primitives.h:287-313) is formed in the lane pair
//     that shares a superblock and scaled to fp32 as ((0.125 d_w) d_a) T (gate on even lanes, up
//     on odd lanes, or two row groups of the down projection): one float term per superblock,
//     the same float the CPU path forms. Every lane parks its term in an LDS window; when the
//     window is full a lane per weight row adds that row's terms in double, in superblock
//     order, and rounds the sum to float once: the row dot is bit for bit the sum the CPU path
//     computes (double accumulation over the blocks of a row, src/gguf/quant_compute.c:152-172),
//     so every value that is rounded to bfloat16 afterwards rounds as it does there.
//
// A work item is (bucket, tile of up to 32 row iterations, sweep). One workgroup per compute
// unit stays resident and its waves draw items from the workgroup's share of the list.
//
// IMAGE: the weights come from the backend's own re-packing of the canonical bytes (built once at
// residency time, the canonical tensor stays the authority), made for this kernel's instruction
// budget. A superblock is two records of 36 bytes, one per lane of the pair that shares it:
//     dword 0      f16 d of the superblock | the four 4-bit group scales of this half << 16
//     dword 1 + 2j the four codebook bytes of group j of this half
//     dword 2 + 2j its four 7-bit sign fields, one to a byte
// so every load is dword-aligned with nothing to shift into place, a sign lookup address is one
// byte permute like a codebook lookup address (the canonical 7-bit fields need a shift and a
// mask each), and the scale arrives with the lane's own record. 72 bytes against 66.
#include "common.hpp"
#include "launch.hpp"
#include "grouped.hpp"

namespace yvex {

constexpr unsigned kSweepWaves = 8u;           // two per SIMD: the sweep of four pairs needs their registers
constexpr unsigned kSweepThreads = kSweepWaves * 64u;
constexpr int kSweepPairs = 4;                 // pairs of one bucket served by one sweep
constexpr unsigned kSweepIters = 32u;          // weight-row iterations per work item (at most)
constexpr int kSweepAheadSmall = 1;            // rows requested ahead of the one decoded, sweeps of one or two pairs
constexpr unsigned kSweepLongPercent = 75u;    // share of the weight rows that goes out in full-length items
constexpr unsigned kSweepShortDiv = 2u;        // the rest goes out in items of 1 / kSweepShortDiv of that length

// LDS map (byte addresses; the dynamic block starts at LDS address 0)
constexpr unsigned kMagBase = 0u;              // 256 entries x 16 replicas x {+lo, +hi, -lo, -hi}
constexpr unsigned kSelBase = 65536u;          // 128 entries x 32 replicas x {selector lo, hi}
constexpr unsigned kTicketAddress = kSelBase + 128u * 32u * 8u;   // work-item counter of the workgroup
constexpr unsigned kParkBase = kTicketAddress + 32u;
// Per wave: a window of kWindowLines lines of 64 float terms (one line per iteration and packed
// value: even lanes' terms in the first 32 words, odd lanes' in the last 32, a weight row's
// terms next to each other in superblock order), then the (gate, up) row sums of a fused item
// ([stream][pair][row of the item]) for the SwiGLU pass at its end.
constexpr unsigned kWindowLines = 16u;
constexpr unsigned kWindowBytes = kWindowLines * 256u;
constexpr unsigned kFusedItemRows = 32u;       // weight row pairs per fused work item
constexpr unsigned kResultBytes = 2u * 4u * kFusedItemRows * 4u;
constexpr unsigned kParkBytes = kWindowBytes + kResultBytes;
// Sweeps listed by the number of pairs they serve (4, 3, 2, 1): four class sizes, four class
// starts (cursors while the list is built) and one word per sweep:
// {whole problem is one bucket : 1, shared expert's problem : 1, bucket : 14, sweep of the bucket : 16}.
constexpr unsigned kClassMaxSweeps = 4096u;
constexpr unsigned kClassCountBase = kParkBase + kSweepWaves * kParkBytes;
constexpr unsigned kClassWaveBase = kClassCountBase + 32u;    // per wave and class: entries of a turn
constexpr unsigned kClassListBase = kClassCountBase + 32u + kSweepWaves * 16u;
// What opens an item without a round trip to memory: expert, first ordered pair and population of
// every routed bucket, and {source pair, route weight} of every ordered pair when the routed
// problem has at most kPairCacheMax of them (decode widths; wider batches read them from memory).
constexpr unsigned kBucketBase = kClassListBase + kClassMaxSweeps * 4u;   // 256 x {expert, first, population}
constexpr unsigned kPairCacheBase = kBucketBase + 256u * 12u;
constexpr unsigned kPairCacheMax = 608u;
constexpr unsigned kSweepLdsBytes = kPairCacheBase + kPairCacheMax * 8u;
static_assert(kSweepLdsBytes <= 160u * 1024u, "the sweep's tables, lists and caches must fit the LDS of a compute unit");

__device__ __forceinline__ void lds_store_u32(unsigned address, unsigned v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) unsigned *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_store_uint2(unsigned address, uint2 v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) uint2 *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ void lds_store_uint4(unsigned address, uint4 v)
{
#if defined(__HIP_DEVICE_COMPILE__)
    *reinterpret_cast<__attribute__((address_space(3))) uint4 *>(address) = v;
#else
    (void)address;
    (void)v;
#endif
}
__device__ __forceinline__ uint2 lds_load_uint2(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const uint2 *>(address);
#else
    (void)address;
    return make_uint2(0u, 0u);
#endif
}
__device__ __forceinline__ unsigned lds_load_u32(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const unsigned *>(address);
#else
    (void)address;
    return 0u;
#endif
}

__device__ __forceinline__ void sweep_tables_fill()
{
    // (the codebook digits of a thread's entries are requested together: one round trip to
    // memory, not one per entry)
    constexpr unsigned kTurns = 256u * 16u / kSweepThreads;
    static_assert(256u * 16u % kSweepThreads == 0u && 128u * 32u % kSweepThreads == 0u,
                  "every thread fills the same number of table entries");
    unsigned digits[kTurns];
#pragma unroll
    for (unsigned t = 0; t < kTurns; ++t) digits[t] = k_iq2_digits[(threadIdx.x + t * kSweepThreads) >> 4];
#pragma unroll
    for (unsigned t = 0; t < kTurns; ++t) {
        const unsigned i = threadIdx.x + t * kSweepThreads;
        const uint2 m = iq2_magnitude_of_digits(digits[t]);
        // byte-wise negation: every level is >= 8, so (x ^ 0xff) + 1 never carries
        lds_store_uint4(kMagBase + i * 16u,
                        make_uint4(m.x, m.y, (m.x ^ 0xffffffffu) + 0x01010101u,
                                   (m.y ^ 0xffffffffu) + 0x01010101u));
    }
#pragma unroll
    for (unsigned i = threadIdx.x; i < 128u * 32u; i += kSweepThreads) {
        const unsigned s7 = i >> 5;
        const unsigned s = s7 | ((__popc(s7) & 1u) << 7);
        // selector byte k = k (take +level, source 1) or k + 4 (take -level, source 0)
        unsigned lo = 0x03020100u, hi = 0x03020100u;
#pragma unroll
        for (unsigned l = 0; l < 4u; ++l) {
            if ((s >> l) & 1u) lo += 4u << (8u * l);
            if ((s >> (l + 4u)) & 1u) hi += 4u << (8u * l);
        }
        lds_store_uint2(kSelBase + i * 8u, make_uint2(lo, hi));
    }
}

// A lane's share of one IQ2_XXS weight row: half a superblock, 32 packed bytes plus the scale.
// Superblocks are 66 bytes, so the codes start on a 2-byte boundary, and vector loads that are
// not dword-aligned run at less than half rate on this part. Every load here is dword-aligned:
// eight dwords from the aligned address at or below the codes and a ninth whose place depends on
// the lane; the consumer shifts the codes into place with byte-align instructions. Each load
// instruction costs the memory pipeline about two cycles per cache line its lanes touch, so the
// fp16 scale gets no instruction of its own. Rows start on dword boundaries and superblocks are
// 66 bytes, so in even superblocks the codes start two bytes into their aligned window: the
// ninth dword is the end of the codes, and the scale is the low half of the first dword of the
// superblock's first half. In odd superblocks the codes fill eight aligned dwords exactly and
// the ninth load fetches the dword whose high half is the scale.
struct Iq2Half {
    uint4 lo, hi;
    unsigned tail;
    // rows: wave-uniform address of the iteration's first weight row; the rest are this lane's
    // byte offsets from it (scalar base + 32-bit lane offset addressing)
    __device__ __forceinline__ void load(const unsigned char *rows, unsigned codes_at, unsigned tail_at)
    {
        lo = *reinterpret_cast<const uint4 *>(rows + codes_at);          // 4-byte aligned
        hi = *reinterpret_cast<const uint4 *>(rows + codes_at + 16u);
        tail = *reinterpret_cast<const unsigned *>(rows + tail_at);
    }
};

struct SweepLane {
    unsigned lanes_per_row, rows_per_iter;
    unsigned sub, super, half;
    bool live;
    unsigned mag_lane;     // (lane % 16) * 16
    unsigned sel_lane;     // kSelBase + (lane % 32) * 8
    unsigned code_shift;   // bytes the codes sit above their aligned load address: 0 or 2
    unsigned scale_shift;  // bits the fp16 scale sits above its aligned load address: 0 or 16
    unsigned park;         // this wave's term window
    unsigned term_slot;    // the lane's word inside a line of the window (byte offset)
    unsigned results;      // the wave's row sums of a fused item
    unsigned terms;        // superblocks of a weight row: the float terms of one row sum
    unsigned row_shift;    // log2(rows_per_iter)
};

__device__ __forceinline__ int dot4_from_zero(unsigned a, unsigned b)
{
#if defined(__HIP_DEVICE_COMPILE__)
    int d;
    asm("v_dot4_i32_i8 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
#else
    (void)a;
    (void)b;
    return 0;
#endif
}

template <int CTRL>
__device__ __forceinline__ float dpp_add(float v)
{
    return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}

// Exact integer sums of this lane's four units of each of STREAMS weight rows against N
// activation rows. The work is cut into eight stages of half a unit per stream (two codebook
// lookups, two selector lookups, sixteen weights); the LDS reads of stage s + DEPTH are issued
// before stage s is consumed, so their latency runs under the permutes and dot products of the
// stages between. A stage holds independent dependency chains (one per stream, or the even and
// odd products of a single stream), because a dependent vector instruction issues only about
// nine cycles after its producer.
template <int STREAMS, int N, bool IMAGE>
__device__ __forceinline__ void iq2_half_dots(const Iq2Half (&c)[STREAMS], const SweepLane &g,
                                              const unsigned (&act)[N][32], int (&total)[STREAMS][N])
{
    constexpr int kStages = 8;
    constexpr int DEPTH = STREAMS == 2 ? 1 : 2;
    constexpr int CHAINS = STREAMS == 2 ? 1 : 2;   // accumulators per (stream, pair)
    unsigned q[STREAMS][8];
#pragma unroll
    for (int w = 0; w < STREAMS; ++w) {
        const unsigned raw[9] = {c[w].lo.x, c[w].lo.y, c[w].lo.z, c[w].lo.w,
                                 c[w].hi.x, c[w].hi.y, c[w].hi.z, c[w].hi.w, c[w].tail};
#pragma unroll
        for (int i = 0; i < 8; ++i)
            q[w][i] = IMAGE ? raw[i] : __builtin_amdgcn_alignbyte(raw[i + 1], raw[i], g.code_shift);
#pragma unroll
        for (int p = 0; p < N; ++p) total[w][p] = 0;
    }
    uint4 mag[DEPTH + 1][STREAMS][2];
    uint2 sel[DEPTH + 1][STREAMS][2];
    auto issue = [&](int stage) {
        const int k = stage >> 1, h = stage & 1, slot = stage % (DEPTH + 1);
#pragma unroll
        for (int w = 0; w < STREAMS; ++w) {
            const unsigned grids = q[w][2 * k], aux = q[w][2 * k + 1];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const unsigned j = 2u * (unsigned)h + (unsigned)jj;
                // magnitude address = index byte j << 8 | replica offset
                const unsigned ma = __builtin_amdgcn_perm(grids, g.mag_lane, 0x0c0c0400u + (j << 8));
                // selector address = sign field j moved to bit 8 | replica offset: the image holds
                // the field in byte j (the table base's third byte comes from the replica word),
                // the canonical word holds it at bit 7j
                unsigned sa;
                if constexpr (IMAGE) {
                    sa = __builtin_amdgcn_perm(aux, g.sel_lane, 0x0c020400u + (j << 8));
                } else {
                    const unsigned moved = 7u * j >= 8u ? aux >> (7u * j - 8u) : aux << (8u - 7u * j);
                    sa = (moved & 0x7f00u) | g.sel_lane;
                }
                mag[slot][w][jj] = lds_read_uint4(ma);
                sel[slot][w][jj] = lds_read_uint2(sa);
            }
        }
    };
#pragma unroll
    for (int stage = 0; stage < DEPTH; ++stage) issue(stage);
    int d[STREAMS][N][CHAINS];
#pragma unroll
    for (int stage = 0; stage < kStages; ++stage) {
        if (stage + DEPTH < kStages) issue(stage + DEPTH);
        __builtin_amdgcn_sched_barrier(0);
        const int k = stage >> 1, h = stage & 1, slot = stage % (DEPTH + 1);
        unsigned weights[STREAMS][4];
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int w = 0; w < STREAMS; ++w) {
                weights[w][2 * jj] = __builtin_amdgcn_perm(mag[slot][w][jj].z, mag[slot][w][jj].x, sel[slot][w][jj].x);
                weights[w][2 * jj + 1] = __builtin_amdgcn_perm(mag[slot][w][jj].w, mag[slot][w][jj].y, sel[slot][w][jj].y);
            }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int p = 0; p < N; ++p)
#pragma unroll
                for (int w = 0; w < STREAMS; ++w) {
                    const int chain = i % CHAINS;
                    const unsigned x = act[p][8 * k + 4 * h + i];
                    // the first product of a chain starts from the constant zero
                    if (h == 0 && i < CHAINS) d[w][p][chain] = dot4_from_zero(weights[w][i], x);
                    else d[w][p][chain] = dot4(weights[w][i], x, d[w][p][chain]);
                }
        if (h == 1) {
#pragma unroll
            for (int w = 0; w < STREAMS; ++w) {
                // 2 s + 1: bit 27 of the canonical word is a sign bit, forced to 1; the image
                // keeps the scale of group k in bits 16 + 4k of the record's first dword
                const int factor = IMAGE ? (int)(((c[w].tail >> (15 + 4 * k)) & 0x1eu) | 1u)
                                         : (int)((q[w][2 * k + 1] >> 27) | 1u);
#pragma unroll
                for (int p = 0; p < N; ++p) {
                    int sum = d[w][p][0];
                    if (CHAINS == 2) sum += d[w][p][1];
                    total[w][p] += __mul24(sum, factor);   // |sum| < 2^23
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// ---- Q4_K rows in the same sweeps ---------------------------------------------------------------
//
// A lane's share of one Q4_K weight row: the superblock's 16-byte head (d, dmin, the twelve bytes
// of 6-bit scales and minimums) and the 64 code bytes of its half (sub-blocks 4 h .. 4 h + 3:
// two chunks of 32 bytes, low nibbles one sub-block and high nibbles the next). Superblocks are
// 144 bytes, so every load is 16-byte aligned relative to the row.
struct Q4kHalf {
    uint4 head;
    uint4 q[4];
    __device__ __forceinline__ void load(const unsigned char *rows, unsigned codes_at, unsigned head_at)
    {
        head = *reinterpret_cast<const uint4 *>(rows + head_at);
#pragma unroll
        for (int i = 0; i < 4; ++i) q[i] = *reinterpret_cast<const uint4 *>(rows + codes_at + 16u * i);
    }
};

// ---- Q2_K rows in the same sweeps (the down experts of the reference's model file) --------------
//
// A lane's share of one Q2_K weight row (public ggml block_q2_K, 84 bytes: sixteen bytes
// scale | minimum << 4 of the 16-value sub-blocks, 64 bytes of 2-bit codes, fp16 d and dmin): the
// 32 code bytes of its half (byte l holds the values 32 s + l of the half at bit 2 s), the half's
// eight scale bytes and the dword of d and dmin. Superblocks are dword-aligned, not more.
struct Q2kHalf {
    uint4 q[2];
    uint2 scales;
    unsigned dd;
    __device__ __forceinline__ void load(const unsigned char *rows, unsigned codes_at, unsigned scales_at,
                                         unsigned dd_at)
    {
        q[0] = *reinterpret_cast<const uint4 *>(rows + codes_at);
        q[1] = *reinterpret_cast<const uint4 *>(rows + codes_at + 16u);
        scales = *reinterpret_cast<const uint2 *>(rows + scales_at);
        dd = *reinterpret_cast<const unsigned *>(rows + dd_at);
    }
};

template <unsigned QT>
struct SweepHalf {
    using type = Iq2Half;
};
template <>
struct SweepHalf<QT_Q4_K> {
    using type = Q4kHalf;
};
template <>
struct SweepHalf<QT_Q2_K> {
    using type = Q2kHalf;
};

// Exact integer sums of this lane's eight Q2_K sub-blocks of each of STREAMS weight rows against N
// activation rows: dot = sum over sub-blocks of scale * (codes . activations), minimum = sum of
// minimum * (sum of the sub-block's sixteen activations), the two terms of the reference's
// primitive (src/backend/cuda/kernel_primitives.h:314-341). A code is a shift and a mask away.
template <int STREAMS, int N>
__device__ __forceinline__ void q2k_half_dots(const Q2kHalf (&c)[STREAMS], const unsigned (&act)[N][32],
                                              const int (&act_sums)[N][8], int (&dot)[STREAMS][N],
                                              int (&minimum)[STREAMS][N])
{
#pragma unroll
    for (int w = 0; w < STREAMS; ++w) {
        const unsigned packed[2] = {c[w].scales.x, c[w].scales.y};
        const unsigned words[8] = {c[w].q[0].x, c[w].q[0].y, c[w].q[0].z, c[w].q[0].w,
                                   c[w].q[1].x, c[w].q[1].y, c[w].q[1].z, c[w].q[1].w};
#pragma unroll
        for (int p = 0; p < N; ++p) {
            int m = 0;
#pragma unroll
            for (int sub = 0; sub < 8; ++sub)       // 15 * 16 * 128 * 8 < 2^23
                m += __mul24((int)((packed[sub >> 2] >> (8 * (sub & 3) + 4)) & 15u), act_sums[p][sub]);
            minimum[w][p] = m;
            dot[w][p] = 0;
        }
#pragma unroll
        for (int shift = 0; shift < 4; ++shift) {
            int first[N], second[N];     // sub-blocks 2 shift (bytes 0-15) and 2 shift + 1 (bytes 16-31)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const unsigned codes = (words[i] >> (2 * shift)) & 0x03030303u;
#pragma unroll
                for (int p = 0; p < N; ++p) {
                    if (i < 4) first[p] = i == 0 ? dot4_from_zero(codes, act[p][8 * shift + i])
                                                  : dot4(codes, act[p][8 * shift + i], first[p]);
                    else second[p] = i == 4 ? dot4_from_zero(codes, act[p][8 * shift + i])
                                            : dot4(codes, act[p][8 * shift + i], second[p]);
                }
            }
            const int sc_first = (int)((packed[shift >> 1] >> (16 * (shift & 1))) & 15u);
            const int sc_second = (int)((packed[shift >> 1] >> (16 * (shift & 1) + 8)) & 15u);
#pragma unroll
            for (int p = 0; p < N; ++p)   // |sum| <= 3 * 128 * 16 < 2^13
                dot[w][p] += __mul24(first[p], sc_first) + __mul24(second[p], sc_second);
        }
    }
}

// Exact integer sums of this lane's four sub-blocks of each of STREAMS weight rows against N
// activation rows: dot = sum over sub-blocks of scale * (nibbles . activations), minimum = sum of
// minimum * (sum of the sub-block's activations), the two terms of the reference's primitive
// (src/backend/cuda/kernel_primitives.h:315-340). No tables: a nibble is a mask away.
template <int STREAMS, int N>
__device__ __forceinline__ void q4k_half_dots(const Q4kHalf (&c)[STREAMS], const SweepLane &g,
                                              const unsigned (&act)[N][32], const int (&act_sums)[N][4],
                                              int (&dot)[STREAMS][N], int (&minimum)[STREAMS][N])
{
#pragma unroll
    for (int w = 0; w < STREAMS; ++w) {
        const unsigned s0 = c[w].head.y, s1 = c[w].head.z, s2 = c[w].head.w;
        // the four scales and the four minimums of this half, one to a byte
        const unsigned scales = g.half ? ((s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)) : (s0 & 0x3f3f3f3fu);
        const unsigned minimums = g.half ? (((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u))
                                         : (s1 & 0x3f3f3f3fu);
#pragma unroll
        for (int p = 0; p < N; ++p) {
            int m = 0;
#pragma unroll
            for (int sub = 0; sub < 4; ++sub)
                m += __mul24((int)((minimums >> (8 * sub)) & 255u), act_sums[p][sub]);   // 63 * 32 * 127 * 4 < 2^23
            minimum[w][p] = m;
            dot[w][p] = 0;
        }
#pragma unroll
        for (int chunk = 0; chunk < 2; ++chunk) {
            const unsigned words[8] = {c[w].q[2 * chunk].x, c[w].q[2 * chunk].y, c[w].q[2 * chunk].z,
                                       c[w].q[2 * chunk].w, c[w].q[2 * chunk + 1].x, c[w].q[2 * chunk + 1].y,
                                       c[w].q[2 * chunk + 1].z, c[w].q[2 * chunk + 1].w};
            int low[N], high[N];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const unsigned lo = words[i] & 0x0f0f0f0fu, hi = (words[i] >> 4) & 0x0f0f0f0fu;
#pragma unroll
                for (int p = 0; p < N; ++p) {
                    low[p] = i == 0 ? dot4_from_zero(lo, act[p][16 * chunk + i]) : dot4(lo, act[p][16 * chunk + i], low[p]);
                    high[p] = i == 0 ? dot4_from_zero(hi, act[p][16 * chunk + 8 + i])
                                     : dot4(hi, act[p][16 * chunk + 8 + i], high[p]);
                }
            }
#pragma unroll
            for (int p = 0; p < N; ++p)   // |sum| <= 15 * 127 * 32 < 2^16
                dot[w][p] += __mul24(low[p], (int)((scales >> (16 * chunk)) & 255u)) +
                             __mul24(high[p], (int)((scales >> (16 * chunk + 8)) & 255u));
        }
    }
}

// One sweep over the item's weight rows [row_begin, row_end) for N live pairs.
// MODE 0: one weight row group (the rows of one iteration) at a time; MODE 1: a gate row group
// and the matching up row group, SwiGLU in the finishing pass; MODE 2: two consecutive row groups
// of one matrix, which share the activation columns as gate and up rows do: the fixed cost of an
// iteration (requests, waits, reduction, loop control) is spent once per two groups.
template <int MODE, int N, bool IMAGE, unsigned QT>
__device__ __forceinline__ void iq2_sweep(const GroupedArgs &a, const GroupedProblem &pr,
                                          const SweepLane &g, const unsigned char *gate_e,
                                          const unsigned char *up_e, unsigned long long first_ordered,
                                          unsigned row_begin, unsigned row_end, bool pairs_in_lds)
{
    constexpr bool FUSED = MODE == 1;
    constexpr bool TWIN = MODE != 0;     // two streams of weight rows against the same activation columns
    constexpr bool Q4 = QT == QT_Q4_K, Q2 = QT == QT_Q2_K;
    constexpr bool KQ = Q4 || Q2;        // formats with a minimum term
    static_assert(!(KQ && IMAGE), "the image is a layout of IQ2_XXS rows");
    const unsigned lane = threadIdx.x & 63u;
    const bool odd = (lane & 1u) != 0u;
    // packed values per iteration: (first, second stream) of pair v with two streams, else pairs (2v, 2v + 1)
    constexpr int PV = TWIN ? N : (N + 1) / 2;

    // ---- the sweep's activation rows: this lane's 128 columns stay in registers ----
    unsigned act[N][32];
    // the sums of the activations under each of the lane's sub-blocks: four of 32 (Q4_K), eight of 16 (Q2_K)
    int act_sums[N][Q4 ? 4 : Q2 ? 8 : 1];
    float act_scale[N];
    float route_weight[N];
    unsigned long long out_index[N];
#pragma unroll
    for (int p = 0; p < N; ++p) {
        const unsigned long long ordered = first_ordered + p;
        unsigned long long source;
        if (pairs_in_lds) {      // wave-uniform
            const uint2 cached = lds_load_uint2(kPairCacheBase + 8u * (unsigned)ordered);
            source = cached.x;
            route_weight[p] = __uint_as_float(cached.y);
        } else {
            source = pr.order ? pr.order[ordered] : ordered;
            route_weight[p] = pr.route_weights ? pr.route_weights[source] : 1.0f;
        }
        const unsigned long long arow = pr.act_by_ordered_pair ? ordered : source / pr.topk;
        out_index[p] = pr.out_by_source_pair ? source : ordered;
        const unsigned char *blk = (const unsigned char *)pr.activations + arow * pr.act_stride +
                                   (unsigned long long)(g.live ? g.super : 0u) * kQ8KBytes;
        // lanes past the last row group multiply zeros
        act_scale[p] = g.live ? *reinterpret_cast<const float *>(blk) : 0.0f;
        const unsigned char *qv = blk + 4u + 128u * g.half;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            uint4 v;
            __builtin_memcpy(&v, qv + 16 * k, 16);
            act[p][4 * k] = g.live ? v.x : 0u;
            act[p][4 * k + 1] = g.live ? v.y : 0u;
            act[p][4 * k + 2] = g.live ? v.z : 0u;
            act[p][4 * k + 3] = g.live ? v.w : 0u;
        }
        if constexpr (Q4) {
            // the block's sixteen sums of 16 activations follow its 256 values: eight belong to this half
            uint4 sums;
            __builtin_memcpy(&sums, blk + 260u + 16u * g.half, 16);
            const unsigned pairs_of_sums[4] = {sums.x, sums.y, sums.z, sums.w};
#pragma unroll
            for (int sub = 0; sub < 4; ++sub)
                act_sums[p][sub] = g.live ? (int)(short)(pairs_of_sums[sub] & 0xffffu) + (int)(short)(pairs_of_sums[sub] >> 16)
                                          : 0;
        } else if constexpr (Q2) {
            uint4 sums;
            __builtin_memcpy(&sums, blk + 260u + 16u * g.half, 16);
            const unsigned pairs_of_sums[4] = {sums.x, sums.y, sums.z, sums.w};
#pragma unroll
            for (int sub = 0; sub < 8; ++sub)
                act_sums[p][sub] = !g.live ? 0 : sub % 2 ? (int)pairs_of_sums[sub / 2] >> 16
                                                         : (int)(short)(pairs_of_sums[sub / 2] & 0xffffu);
        } else {
            act_sums[p][0] = 0;
        }
    }
    // the activation scale each lane applies to packed value v
    float packed_scale[PV];
#pragma unroll
    for (int v = 0; v < PV; ++v) {
        if constexpr (TWIN) packed_scale[v] = act_scale[v];
        else packed_scale[v] = odd ? (2 * v + 1 < N ? act_scale[2 * v + 1 < N ? 2 * v + 1 : 0] : 0.0f)
                                   : act_scale[2 * v];
    }

    const unsigned rows_per_turn = MODE == 2 ? 2u * g.rows_per_iter : g.rows_per_iter;
    const unsigned rows = row_end - row_begin;               // a multiple of rows_per_turn
    const unsigned iterations = rows / rows_per_turn;         // <= kSweepIters
    // wave-uniform row bases advance by a scalar stride; the lane's place inside an iteration's
    // rows is a constant 32-bit offset
    const unsigned char *gate_rows = gate_e + (unsigned long long)row_begin * pr.row_bytes;
    const unsigned long long second_row_bytes = FUSED ? pr.up_row_bytes : pr.row_bytes;
    const unsigned char *up_rows = FUSED ? up_e + (unsigned long long)row_begin * pr.up_row_bytes
        : MODE == 2 ? gate_rows + (unsigned long long)g.rows_per_iter * pr.row_bytes : nullptr;
    const unsigned long long gate_step = (unsigned long long)rows_per_turn * pr.row_bytes;
    const unsigned long long up_step = (unsigned long long)rows_per_turn * second_row_bytes;
    const unsigned lane_row = g.live ? g.sub : 0u, lane_super = g.live ? g.super : 0u;
    // (row bases and row strides are multiples of four bytes: checked on the host)
    constexpr unsigned kSuperBytes = Q4 ? 144u : Q2 ? 84u : IMAGE ? 72u : 66u;
    const unsigned gate_block = lane_row * (unsigned)pr.row_bytes + lane_super * kSuperBytes;
    const unsigned up_block = lane_row * (unsigned)second_row_bytes + lane_super * kSuperBytes;
    // image: the lane's record is its first dword (scale and group scales) and eight more
    // (Q4_K: the half's 64 code bytes behind the 16-byte head, which is the "tail" load)
    // (Q2_K: the half's 32 code bytes behind the sixteen scale bytes; "tail" is the half's eight scale bytes)
    const unsigned gate_codes_at = Q4 ? gate_block + 16u + 64u * g.half
        : Q2 ? gate_block + 16u + 32u * g.half
        : IMAGE ? gate_block + 36u * g.half + 4u
                : (gate_block + 2u + 32u * g.half) & ~3u;   // + code_shift = codes
    const unsigned up_codes_at = Q4 ? up_block + 16u + 64u * g.half
        : Q2 ? up_block + 16u + 32u * g.half
        : IMAGE ? up_block + 36u * g.half + 4u : (up_block + 2u + 32u * g.half) & ~3u;
    // ninth dword: the end of the codes where they start two bytes in, else the scale's dword
    const unsigned gate_tail_at = Q4 ? gate_block : Q2 ? gate_block + 8u * g.half : IMAGE ? gate_codes_at - 4u
                                        : g.code_shift ? gate_codes_at + 32u : gate_block & ~3u;
    const unsigned up_tail_at = Q4 ? up_block : Q2 ? up_block + 8u * g.half
        : IMAGE ? up_codes_at - 4u : g.code_shift ? up_codes_at + 32u : up_block & ~3u;
    // Ring of packed rows: the bytes of iteration it + AHEAD are requested before iteration it is
    // decoded, so about AHEAD iterations of arithmetic cover the HBM latency.
    // The loop body is one basic block: every turn requests a row (the last ones clamped to the
    // final row) and every lane stores (lanes that hold no result write to a spare word), so no
    // branch sits between a request and the wait that consumes it and the waits stay counted.
    constexpr int AHEAD = N <= 2 ? kSweepAheadSmall : 1;   // rows requested ahead of the one decoded
    constexpr int STREAMS = TWIN ? 2 : 1;
    using Half = typename SweepHalf<QT>::type;
    Half ring[AHEAD + 1][STREAMS];
    const unsigned last = iterations - 1u;
    auto request = [&](Half (&slot)[STREAMS], unsigned it) {
        const unsigned clamped = it < last ? it : last;
        if constexpr (Q2) {
            slot[0].load(gate_rows + clamped * gate_step, gate_codes_at, gate_tail_at, gate_block + 80u);
            if constexpr (TWIN)
                slot[1].load(up_rows + clamped * up_step, up_codes_at, up_tail_at, up_block + 80u);
        } else {
            slot[0].load(gate_rows + clamped * gate_step, gate_codes_at, gate_tail_at);
            if constexpr (TWIN)
                slot[1].load(up_rows + clamped * up_step, up_codes_at, up_tail_at);
        }
    };
    // The first requests are kept in ring order: the loop's first wait is counted against the
    // loads issued after the slot it consumes, on the entry path and on the back edge alike.
#pragma unroll
    for (int ahead = 0; ahead < AHEAD; ++ahead) {
        __builtin_amdgcn_sched_barrier(0);
        request(ring[ahead], (unsigned)ahead);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- the window's row sums: a lane per (line, parity, row of the iteration) adds that
    // row's float terms in double, in superblock order, and rounds once ----
    // A fused item keeps the sums for the SwiGLU pass at its end; a plain projection rounds to
    // bfloat16 and stores here.
    const unsigned R = g.rows_per_iter;
    auto flush = [&](unsigned first_iteration, unsigned count) {
        // LDS operations of one wave complete in order, so the terms parked above are visible here
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const unsigned sums = (count * (unsigned)PV * 2u) << g.row_shift;
        const unsigned segment_bytes = 128u >> g.row_shift;       // a row's terms of one parity
        for (unsigned s = lane; s < sums; s += 64u) {
            const unsigned line = s >> (g.row_shift + 1u), rest = s & (2u * R - 1u);
            const unsigned parity = rest >> g.row_shift, group = rest & (R - 1u);
            const unsigned at = g.park + line * 256u + parity * 128u + group * segment_bytes;
            double sum = 0.0;
            unsigned k = 0u;
            for (; k + 4u <= g.terms; k += 4u) {
                const uint4 t = lds_read_uint4(at + 4u * k);
                sum += (double)__uint_as_float(t.x);
                sum += (double)__uint_as_float(t.y);
                sum += (double)__uint_as_float(t.z);
                sum += (double)__uint_as_float(t.w);
            }
            for (; k < g.terms; ++k) sum += (double)__uint_as_float(lds_load_u32(at + 4u * k));
            const float row_sum = (float)sum;
            const unsigned iteration = first_iteration + line / (unsigned)PV, v = line % (unsigned)PV;
            if constexpr (FUSED) {
                const unsigned local = (iteration << g.row_shift) + group;      // < kFusedItemRows
                lds_store_u32(g.results + ((parity * (unsigned)N + v) * kFusedItemRows + local) * 4u,
                              __float_as_uint(row_sum));
            } else {
                // two row groups an iteration: pair v, group `parity`; one: pairs 2v and 2v + 1
                const unsigned p = TWIN ? v : 2u * v + parity;
                const unsigned row = row_begin + (TWIN ? ((2u * iteration + parity) << g.row_shift)
                                                       : (iteration << g.row_shift)) + group;
                unsigned long long oi = out_index[0];
#pragma unroll
                for (int q = 1; q < N; ++q)
                    if (p == (unsigned)q) oi = out_index[q];
                const float value = bf16_round(row_sum);
                if (p < (unsigned)N) {
                    if (!finite_f32(value)) raise_status(a.status, 1);
                    else pr.out[oi * a.out_rows + row] = value;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // iterations a window holds (a multiple of the turns of one trip through the loop below)
    constexpr unsigned kWindowIters = (kWindowLines / (unsigned)PV) / (AHEAD + 1) * (AHEAD + 1);
    static_assert(kWindowIters >= AHEAD + 1, "a window holds at least one trip's lines");

    for (unsigned window_begin = 0; window_begin < iterations; window_begin += kWindowIters) {
      const unsigned window_end = window_begin + kWindowIters < iterations ? window_begin + kWindowIters : iterations;
      unsigned park_at = g.park + g.term_slot;
      for (unsigned it0 = window_begin; it0 < window_end; it0 += AHEAD + 1) {
#pragma unroll
      for (int turn = 0; turn <= AHEAD; ++turn) {
        const unsigned it = it0 + (unsigned)turn;   // may run past the last row by AHEAD turns
        request(ring[(turn + AHEAD) % (AHEAD + 1)], it + AHEAD);
        const Half (&now)[STREAMS] = ring[turn];
        int total_gate[N], total_up[N];
        int min_gate[N], min_up[N];          // Q4_K: the sums of the minimum term
        {
            int totals[STREAMS][N], minimums[STREAMS][N];
            if constexpr (Q4) {
                q4k_half_dots<STREAMS, N>(now, g, act, act_sums, totals, minimums);
            } else if constexpr (Q2) {
                q2k_half_dots<STREAMS, N>(now, act, act_sums, totals, minimums);
            } else {
                iq2_half_dots<STREAMS, N, IMAGE>(now, g, act, totals);
#pragma unroll
                for (int w = 0; w < STREAMS; ++w)
#pragma unroll
                    for (int p = 0; p < N; ++p) minimums[w][p] = 0;
            }
#pragma unroll
            for (int p = 0; p < N; ++p) {
                total_gate[p] = totals[0][p];
                total_up[p] = totals[STREAMS - 1][p];
                min_gate[p] = minimums[0][p];
                min_up[p] = minimums[STREAMS - 1][p];
            }
        }
        // the two lanes of a superblock add their halves: exact int32 superblock sums
#pragma unroll
        for (int p = 0; p < N; ++p) {
            total_gate[p] += dpp_move<0xb1, 0xf>(total_gate[p]);
            if constexpr (TWIN) total_up[p] += dpp_move<0xb1, 0xf>(total_up[p]);
            if constexpr (KQ) {
                min_gate[p] += dpp_move<0xb1, 0xf>(min_gate[p]);
                if constexpr (TWIN) min_up[p] += dpp_move<0xb1, 0xf>(min_up[p]);
            }
        }
        // The even lane of a pair scales the first stream and the odd lane the last one. An odd
        // lane holds the second half of its superblock, so where the scale rides in the first
        // half's codes it comes from the neighbour.
        const Half &mine = odd ? now[STREAMS - 1] : now[0];
        float weight_scale, weight_minimum = 0.0f;
        if constexpr (Q4) {
            weight_scale = f16_bits_to_float(mine.head.x & 0xffffu);       // d
            weight_minimum = f16_bits_to_float(mine.head.x >> 16);         // dmin
        } else if constexpr (Q2) {
            weight_scale = f16_bits_to_float(mine.dd & 0xffffu);
            weight_minimum = f16_bits_to_float(mine.dd >> 16);
        } else if constexpr (IMAGE) {
            weight_scale = 0.125f * f16_bits_to_float(mine.tail & 0xffffu);
        } else {
            // (the exchange runs in every lane: it reads its neighbour, which must be executing it)
            const unsigned neighbour_word = (unsigned)dpp_move<0xb1, 0xf>((int)now[STREAMS - 1].lo.x);
            const unsigned first_word = odd ? neighbour_word : now[0].lo.x;
            weight_scale = 0.125f * f16_bits_to_float(
                ((g.code_shift ? first_word : mine.tail) >> g.scale_shift) & 0xffffu);
        }
#pragma unroll
        for (int v = 0; v < PV; ++v) {
            int t, m = 0;
            if constexpr (TWIN) t = odd ? total_up[v] : total_gate[v];
            else t = odd ? total_gate[2 * v + 1 < N ? 2 * v + 1 : 2 * v] : total_gate[2 * v];
            float value;
            if constexpr (KQ) {
                if constexpr (TWIN) m = odd ? min_up[v] : min_gate[v];
                else m = odd ? min_gate[2 * v + 1 < N ? 2 * v + 1 : 2 * v] : min_gate[2 * v];
                // (d_a d) dot - (d_a dmin) minimum, each product rounded: the order of the reference's primitive
                const float left = packed_scale[v] * weight_scale * (float)t;
                const float right = packed_scale[v] * weight_minimum * (float)m;
                value = left - right;
            } else {
                value = weight_scale * packed_scale[v] * (float)t;
            }
            // every lane parks its term (lanes past the last row group park zeros nobody adds)
            lds_store_u32(park_at, __float_as_uint(value));
            park_at += 256u;
        }
      }
      }
      flush(window_begin, window_end - window_begin);
    }

    // ---- finish a fused item: SwiGLU of the (gate, up) row sums, coalesced stores ----
    if constexpr (FUSED) {
        const unsigned outputs = rows * (unsigned)N;
        for (unsigned o = lane; o < outputs; o += 64u) {
            const unsigned p = o / rows, local = o % rows;      // consecutive lanes: consecutive rows
            const float first = __uint_as_float(lds_load_u32(g.results + (p * kFusedItemRows + local) * 4u));
            const float second = __uint_as_float(
                lds_load_u32(g.results + (((unsigned)N + p) * kFusedItemRows + local) * 4u));
            float rw = route_weight[0];
            unsigned long long oi = out_index[0];
#pragma unroll
            for (int q = 1; q < N; ++q)
                if (p == (unsigned)q) {
                    rw = route_weight[q];
                    oi = out_index[q];
                }
            const float value = swiglu_bf16_fast(first, second, rw, a.limit, (float)a.limit);
            if (!finite_f32(value)) raise_status(a.status, 1);
            else pr.out[oi * a.out_rows + row_begin + local] = value;
        }
        __builtin_amdgcn_wave_barrier();
    }
}

template <int MODE, bool IMAGE, unsigned QT>
__global__ __launch_bounds__(kSweepThreads) void iq2_sweep_kernel(GroupedArgs a)
{
    constexpr bool FUSED = MODE == 1;
    extern __shared__ __align__(16) unsigned char sweep_lds[];
    if (lds_address_of(sweep_lds) != 0u) {   // the lookups address LDS by absolute byte offsets
        if (threadIdx.x == 0u) raise_status(a.status, 2);
        return;
    }
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    // The bucket count and this thread's bucket population are requested before the tables are
    // built, so that their round trips to memory run under the table fill instead of after it.
    const GroupedProblem &routed = a.problem[0];
    const bool routed_fixed = routed.expert_ids == nullptr;
    const unsigned buckets = routed_fixed ? 1u : (unsigned)routed.counts[0];
    unsigned population_here = 0u;
    if (!routed_fixed && tid < 256u && tid < routed.experts)
        population_here = (unsigned)routed.bucket_populations[tid];
    // ... and so are the routed buckets' experts and first pairs and the pairs' sources, which
    // the items will find in LDS
    unsigned long long expert_here = 0ull, first_here = 0ull;
    if (!routed_fixed && tid < 256u && tid < routed.experts) {
        expert_here = routed.expert_ids[tid];
        first_here = routed.bucket_offsets[tid];
    }
    const bool pairs_in_lds = !routed_fixed && routed.order != nullptr && routed.pairs <= kPairCacheMax;
    static_assert(kPairCacheMax <= 2u * kSweepThreads, "two cached pairs a thread");
    unsigned long long source_here[2] = {~0ull, ~0ull};
    if (pairs_in_lds) {
#pragma unroll
        for (unsigned k = 0; k < 2u; ++k)
            if (tid + k * kSweepThreads < routed.pairs) source_here[k] = routed.order[tid + k * kSweepThreads];
    }
    if constexpr (QT == QT_IQ2_XXS) sweep_tables_fill();     // (Q4_K rows need no tables)
    if (tid == 0u) lds_store_u32(kTicketAddress, 0u);
    if (pairs_in_lds) {
        float weight_here[2];
#pragma unroll
        for (unsigned k = 0; k < 2u; ++k)   // a source outside the problem reads no weight here; the sweep's own checks refuse it
            weight_here[k] = routed.route_weights && source_here[k] < routed.pairs
                ? routed.route_weights[source_here[k]] : 1.0f;
#pragma unroll
        for (unsigned k = 0; k < 2u; ++k)
            if (tid + k * kSweepThreads < routed.pairs)
                lds_store_uint2(kPairCacheBase + 8u * (tid + k * kSweepThreads),
                                make_uint2(source_here[k] < 0xffffffffull ? (unsigned)source_here[k] : 0xffffffffu,
                                           __float_as_uint(weight_here[k])));
    }

    if (!routed_fixed && buckets > 256u) {
        if (tid == 0u) raise_status(a.status, 2);
        return;
    }
    if (!routed_fixed && tid < buckets) {
        // (values past 32 bits fail the item's range check through their low words' sum only by
        // accident, so they are clamped to a value that always fails it)
        lds_store_u32(kBucketBase + 12u * tid, expert_here < 0xffffffffull ? (unsigned)expert_here : 0xffffffffu);
        lds_store_u32(kBucketBase + 12u * tid + 4u, first_here < 0xffffffffull ? (unsigned)first_here : 0xffffffffu);
        lds_store_u32(kBucketBase + 12u * tid + 8u, population_here);
    }

    const unsigned units = a.width >> 5;
    SweepLane g;
    g.lanes_per_row = units / 4u;                                  // 16 .. 64, checked on the host
    g.rows_per_iter = (g.lanes_per_row % 16u) == 0u && 64u % g.lanes_per_row == 0u
        ? 64u / g.lanes_per_row : 1u;
    g.sub = lane / g.lanes_per_row;
    const unsigned seg = lane % g.lanes_per_row;
    g.live = g.sub < g.rows_per_iter;
    g.super = seg >> 1;
    g.half = seg & 1u;
    // superblock `super` starts 66 * super bytes into a row whose start is dword-aligned
    const unsigned block_start = 66u * (g.live ? g.super : 0u);
    g.code_shift = (block_start + 2u + 32u * g.half) & 3u;
    g.scale_shift = 8u * (block_start & 3u);
    g.mag_lane = (lane & 15u) * 16u;
    g.sel_lane = kSelBase + (lane & 31u) * 8u;
    g.park = kParkBase + wave * kParkBytes;
    g.results = g.park + kWindowBytes;
    g.terms = g.lanes_per_row / 2u;
    g.row_shift = g.rows_per_iter == 4u ? 2u : g.rows_per_iter == 2u ? 1u : 0u;
    {
        // a line of the window: parity, then the rows of an iteration, then the row's superblocks
        const unsigned span = 64u >> g.row_shift;                  // lanes of a weight row's slot
        g.term_slot = ((lane & 1u) * 32u + (lane / span) * (span / 2u) + (lane % span) / 2u) * 4u;
    }

    // The first part of the weight rows is cut into long items (kSweepIters iterations), the rest
    // into short ones that come last in the item list: the waves of the grid finish within a short
    // item of each other instead of a long one, and only the short items pay the fixed cost of an
    // item (its activation columns, the first requests, the finishing pass) more often.
    // (a fused item keeps its row sums in LDS until its SwiGLU pass: kFusedItemRows rows)

    // Work items: sweeps by class, the ones that serve four pairs first (the shared expert's are
    // all of that kind), then three, two, one; inside a class sweep by sweep, each over its tiles
    // (neighbouring items are neighbouring tiles of one expert). A sweep's cost grows with its
    // pairs and workgroup b owns items b, b + grid, ...: listed by class every workgroup gets the
    // same share of every kind.
    // Every workgroup must arrive at the same list, so a sweep's place is computed, not drawn:
    // a bucket of n pairs has n / 4 sweeps of the first class, which start at the number of such
    // sweeps in the buckets before it (a scan over the bucket slots), and, when n % 4 pairs are
    // left, one sweep of class 4 - n % 4, whose place is the bucket's rank among the buckets that
    // have one of that class (ballots and per-wavefront totals). The shared expert's pairs count
    // as a bucket in front of the routed ones.
    // list word: {whole problem is one bucket : 1, shared expert's problem : 1, bucket : 14, sweep of the bucket : 16}
    static_assert(kSweepPairs == 4, "the sweep list has one class per number of pairs served, four of them");
    unsigned all_sweeps;
    {
        const GroupedProblem &extra = a.problem[a.problems > 1u ? 1u : 0u];
        const unsigned extra_pairs = a.problems > 1u ? extra.pairs : 0u;
        const unsigned extra_full = extra_pairs / 4u, extra_class = extra_pairs % 4u ? 4u - extra_pairs % 4u : 0u;
        // this thread's slot: bucket tid of the routed problem (or the whole problem as slot 0)
        unsigned pairs_here = 0u;
        if (routed_fixed) pairs_here = tid == 0u ? routed.pairs : 0u;
        else if (tid < buckets) pairs_here = population_here;
        const unsigned full = pairs_here / 4u;
        const unsigned cls = pairs_here % 4u ? 4u - pairs_here % 4u : 0u;     // 0: no partial sweep
        unsigned inclusive = full;
#pragma unroll
        for (int offset = 1; offset < 64; offset <<= 1) {
            const unsigned below = (unsigned)__shfl_up((int)inclusive, offset, kWave);
            if ((int)lane >= offset) inclusive += below;
        }
        unsigned rank[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (unsigned c = 1; c < 4u; ++c) {
            const unsigned long long members = __ballot(cls == c);
            rank[c] = (unsigned)__popcll(members & ((1ull << lane) - 1ull));
            if (lane == 0u) lds_store_u32(kClassWaveBase + (wave * 4u + c) * 4u, (unsigned)__popcll(members));
        }
        if (lane == 63u) lds_store_u32(kClassWaveBase + wave * 16u, inclusive);       // class 0: full sweeps of the wave's slots
        __syncthreads();
        unsigned before[4] = {0u, 0u, 0u, 0u}, total[4] = {0u, 0u, 0u, 0u};
        for (unsigned w = 0; w < kSweepWaves; ++w)
#pragma unroll
            for (unsigned c = 0; c < 4u; ++c) {
                const unsigned n = lds_load_u32(kClassWaveBase + (w * 4u + c) * 4u);
                if (w < wave) before[c] += n;
                total[c] += n;
            }
        total[0] += extra_full;
        if (extra_class) total[extra_class] += 1u;
        all_sweeps = total[0] + total[1] + total[2] + total[3];
        if (all_sweeps > kClassMaxSweeps) {          // the launch wrapper bounds the pairs
            if (tid == 0u) raise_status(a.status, 2);
            return;
        }
        unsigned start[4];
        start[0] = 0u;
#pragma unroll
        for (unsigned c = 1; c < 4u; ++c) start[c] = start[c - 1u] + total[c - 1u];
        const unsigned tag = routed_fixed ? 0x80000000u : tid << 16;
        {
            const unsigned at = extra_full + before[0] + inclusive - full;
            for (unsigned k = 0; k < full; ++k) lds_store_u32(kClassListBase + 4u * (at + k), tag | (k & 0xffffu));
        }
        if (cls)
            lds_store_u32(kClassListBase + 4u * (start[cls] + (extra_class == cls ? 1u : 0u) + before[cls] + rank[cls]),
                          tag | (full & 0xffffu));
        // the shared expert's sweeps: in front of their classes
        for (unsigned k = tid; k < extra_full; k += kSweepThreads)
            lds_store_u32(kClassListBase + 4u * k, 0xc0000000u | (k & 0xffffu));
        if (tid == 0u && extra_class)
            lds_store_u32(kClassListBase + 4u * start[extra_class], 0xc0000000u | (extra_full & 0xffffu));
        if (tid < 4u) lds_store_u32(kClassCountBase + 4u * tid, total[tid]);
        __syncthreads();
    }
    // A batch of a few rows has few sweeps: its items are made shorter (down to four iterations)
    // until every wave of the grid has one, which matters more there than an item's fixed cost.
    unsigned item_rows = FUSED ? kFusedItemRows : kSweepIters * g.rows_per_iter * (MODE == 2 ? 2u : 1u);
    {
        const unsigned least = 4u * g.rows_per_iter * (MODE == 2 ? 2u : 1u);
        const unsigned waves = gridDim.x * kSweepWaves;
        while (item_rows / 2u >= least && all_sweeps * (a.out_rows / item_rows) < waves) item_rows /= 2u;
    }
    const unsigned short_rows = item_rows / kSweepShortDiv;
    const unsigned long_tiles = (unsigned)((unsigned long long)a.out_rows * kSweepLongPercent / 100u / item_rows);
    const unsigned long_rows = long_tiles * item_rows;
    const unsigned short_tiles = (a.out_rows - long_rows + short_rows - 1u) / short_rows;
    const unsigned total_long = all_sweeps * long_tiles;
    const unsigned total_items = total_long + all_sweeps * short_tiles;
    // Workgroup b owns items b, b + grid, b + 2 grid, ...; its waves draw positions in that list
    // from a counter in LDS, so a wave that met light items takes more of them.
    auto draw = [&]() -> unsigned {
        unsigned got = 0u;
        if (lane == 0u)
            got = __hip_atomic_fetch_add(
                reinterpret_cast<__attribute__((address_space(3))) unsigned *>(kTicketAddress), 1u,
                __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return (unsigned)__builtin_amdgcn_readfirstlane((int)got) * gridDim.x + blockIdx.x;
    };
    for (unsigned listed = draw(); listed < total_items; listed = draw()) {
        const bool is_short = listed >= total_long;
        const unsigned item = is_short ? listed - total_long : listed;   // within its zone of rows
        const unsigned tiles = is_short ? short_tiles : long_tiles;
        const unsigned rows_of_item = is_short ? short_rows : item_rows;
        // class of the item, then (sweep of the class list, tile)
        unsigned start = 0u, size = 0u, position = item;
        bool found = false;
        for (unsigned c = 0; c < 4u && !found; ++c) {
            size = lds_load_u32(kClassCountBase + 4u * c);
            if (position < size * tiles) {
                found = true;
            } else {
                position -= size * tiles;
                start += size;
            }
        }
        if (!found) {
            if (lane == 0u) raise_status(a.status, 2);
            continue;
        }
        const unsigned tile = position % tiles;
        const unsigned word = lds_load_u32(kClassListBase + 4u * (start + position / tiles));
        const GroupedProblem &pr = a.problem[(word & 0x40000000u) && a.problems > 1u ? 1u : 0u];
        unsigned long long expert = 0ull, first = 0ull, population = pr.pairs;
        const bool is_routed = !(word & 0x40000000u);
        if (!(word & 0x80000000u)) {
            const unsigned bucket = (word >> 16) & 0x3fffu;
            if (is_routed) {          // the routed problem's buckets were copied at kernel start
                expert = lds_load_u32(kBucketBase + 12u * bucket);
                first = lds_load_u32(kBucketBase + 12u * bucket + 4u);
                population = lds_load_u32(kBucketBase + 12u * bucket + 8u);
            } else {
                expert = pr.expert_ids[bucket];
                first = pr.bucket_offsets[bucket];
                population = pr.bucket_populations[bucket];
            }
        }
        const unsigned long long pass = (unsigned long long)(word & 0xffffu) * kSweepPairs;
        if (expert >= pr.experts || first + population > pr.pairs || pass >= population) {
            if (lane == 0u) raise_status(a.status, 2);
            continue;
        }
        const unsigned char *gate_e = pr.gate + expert * pr.expert_bytes;
        const unsigned char *up_e = FUSED ? pr.up + expert * pr.up_expert_bytes : nullptr;
        const unsigned row_begin = (is_short ? long_rows : 0u) + tile * rows_of_item;
        const unsigned row_end = row_begin + rows_of_item < a.out_rows ? row_begin + rows_of_item : a.out_rows;
        const unsigned long long live = population - pass;
        const bool cached = pairs_in_lds && is_routed;
        if (kSweepPairs >= 4 && live >= 4ull)
            iq2_sweep<MODE, kSweepPairs >= 4 ? 4 : 1, IMAGE, QT>(a, pr, g, gate_e, up_e, first + pass, row_begin, row_end, cached);
        else if (kSweepPairs >= 3 && live >= 3ull)
            iq2_sweep<MODE, kSweepPairs >= 3 ? 3 : 1, IMAGE, QT>(a, pr, g, gate_e, up_e, first + pass, row_begin, row_end, cached);
        else if (live >= 2ull)
            iq2_sweep<MODE, 2, IMAGE, QT>(a, pr, g, gate_e, up_e, first + pass, row_begin, row_end, cached);
        else
            iq2_sweep<MODE, 1, IMAGE, QT>(a, pr, g, gate_e, up_e, first + pass, row_begin, row_end, cached);
    }
}

bool iq2_sweep_supported(unsigned qtype, unsigned width, unsigned out_rows, unsigned long long pairs, bool image)
{
    if (qtype != QT_IQ2_XXS && qtype != QT_Q4_K && qtype != QT_Q2_K) return false;
    if (image && qtype != QT_IQ2_XXS) return false;
    if (pairs > kClassMaxSweeps) return false;            // every sweep serves at least one pair
    const unsigned lanes_per_row = width / 128u;
    if (width % 256u != 0u || lanes_per_row < 16u || lanes_per_row > 64u) return false;
    // IQ2_XXS rows must start on dword boundaries (Q4_K rows are multiples of 144 bytes, Q2_K rows of 84)
    if (qtype == QT_IQ2_XXS && !image && (width / 256u * 66u) % 4u != 0u) return false;
    const unsigned rows_per_iter = lanes_per_row % 16u == 0u && 64u % lanes_per_row == 0u
        ? 64u / lanes_per_row : 1u;
    return out_rows % rows_per_iter == 0u;   // an iteration never reads past the last row
}

template <int MODE, bool IMAGE, unsigned QT>
static int launch_iq2_sweep_variant(const GroupedArgs &a, hipStream_t stream)
{
    YVEX_ALLOW_DYNAMIC_LDS((iq2_sweep_kernel<MODE, IMAGE, QT>), kSweepLdsBytes);
    iq2_sweep_kernel<MODE, IMAGE, QT><<<compute_units(), kSweepThreads, kSweepLdsBytes, stream>>>(a);
    return check_launch("moe_sweep");
}

template <bool IMAGE, unsigned QT>
static int launch_iq2_sweep_mode(const GroupedArgs &a, int mode, hipStream_t stream)
{
    return mode == 1 ? launch_iq2_sweep_variant<1, IMAGE, QT>(a, stream)
         : mode == 2 ? launch_iq2_sweep_variant<2, IMAGE, QT>(a, stream)
                     : launch_iq2_sweep_variant<0, IMAGE, QT>(a, stream);
}

int launch_iq2_sweep(const GroupedArgs &a, unsigned qtype, bool fused, bool image, hipStream_t stream)
{
    // a projection that is not fused takes two row groups an iteration where the rows allow it
    // (every item then holds whole pairs of groups: the short items are half a long one)
    const unsigned lanes_per_row = a.width / 128u;
    const unsigned rows_per_iter = lanes_per_row % 16u == 0u && 64u % lanes_per_row == 0u ? 64u / lanes_per_row : 1u;
    const int mode = fused ? 1 : a.out_rows % (2u * rows_per_iter) == 0u ? 2 : 0;
    if (qtype == QT_Q4_K) return image ? ST_UNSUPPORTED : launch_iq2_sweep_mode<false, QT_Q4_K>(a, mode, stream);
    if (qtype == QT_Q2_K) {      // the down experts: a plain projection
        if (image || fused) return ST_UNSUPPORTED;
        return mode == 2 ? launch_iq2_sweep_variant<2, false, QT_Q2_K>(a, stream)
                         : launch_iq2_sweep_variant<0, false, QT_Q2_K>(a, stream);
    }
    if (qtype != QT_IQ2_XXS) return ST_UNSUPPORTED;
    return image ? launch_iq2_sweep_mode<true, QT_IQ2_XXS>(a, mode, stream)
                 : launch_iq2_sweep_mode<false, QT_IQ2_XXS>(a, mode, stream);
}

// ---- the image: canonical IQ2_XXS superblocks re-packed for the sweeps -------------------------

// One thread per half superblock: nine dwords out of the 66 canonical bytes.
__global__ __launch_bounds__(256) void iq2_sweep_image_kernel(const unsigned char *canonical,
                                                              unsigned long long blocks, unsigned *image)
{
    const unsigned long long at = (unsigned long long)blockIdx.x * 256ull + threadIdx.x;
    if (at >= 2ull * blocks) return;
    const unsigned long long block = at >> 1;
    const unsigned half = (unsigned)(at & 1ull);
    const unsigned char *b = canonical + block * 66ull;
    unsigned *record = image + at * 9ull;
    unsigned scales = 0u;
#pragma unroll
    for (unsigned j = 0; j < 4u; ++j) {
        const unsigned char *group = b + 2u + 8u * (4u * half + j);
        const unsigned grids = load_u32(group), aux = load_u32(group + 4u);
        record[1u + 2u * j] = grids;
        record[2u + 2u * j] = (aux & 127u) | (((aux >> 7) & 127u) << 8) | (((aux >> 14) & 127u) << 16) |
                              (((aux >> 21) & 127u) << 24);
        scales |= (aux >> 28) << (4u * j);
    }
    record[0] = load_u16(b) | (scales << 16);
}

}  // namespace yvex

extern "C" uint64_t yvex_hip_iq2_sweep_image_bytes(uint64_t blocks) { return blocks * 72u; }

extern "C" int yvex_hip_iq2_sweep_image_build(const uint8_t *canonical, uint64_t blocks, void *image,
                                              yvex_hip_stream stream)
{
    if (!canonical || !image || !blocks || ((uintptr_t)image & 3u)) return yvex::ST_INVALID_ARG;
    const uint64_t groups = (2u * blocks + 255u) / 256u;
    if (groups > 0x7fffffffull) return yvex::ST_BOUNDS;
    yvex::iq2_sweep_image_kernel<<<(unsigned)groups, 256, 0, yvex::as_stream(stream)>>>(canonical, blocks,
                                                                                         (unsigned *)image);
    return yvex::check_launch("iq2_sweep_image");
}
