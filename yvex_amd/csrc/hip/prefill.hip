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
constexpr unsigned kCodeBase = 0u;                          // 256 entries x 32 replicas x 8 bytes
constexpr unsigned kSelBase = 65536u;                       // 128 entries x 16 replicas x 8 bytes
constexpr unsigned kLutBase = kSelBase + 128u * 16u * 8u;   // 16 scales x 16 replicas x 16 bytes
constexpr unsigned kStageBase = kLutBase + 16u * 16u * 16u;
constexpr unsigned kStageActs = kTileTokens * kActPitch;
constexpr unsigned kStageBytes = kStageActs + kTileTokens * 4u;   // + one fp32 scale per token
constexpr unsigned kTileStartBase = kStageBase + 2u * kStageBytes;
constexpr unsigned kMfmaLdsBytes = kTileStartBase + 260u * 4u;

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

// Twelve aligned bytes that hold one 8-byte group record starting 0 or 2 bytes in.
struct alignas(4) RawGroup {
    unsigned x, y, z;
};

// One work item with NB live 16-token blocks (NB is 1, 2, 4 or 8). Eight waves, two per SIMD, each
// owning one 16-row block. Every loop below has a fixed trip count and the superblock body is one
// basic block (requests past the end are clamped, not guarded), so accumulators never leave
// registers and the compiler's wait counts stay exact.
template <bool FUSED_UP, unsigned NB>
__device__ __forceinline__ void mfma_item(const MfmaArgs &a, const MfmaItem &it)
{
    const GroupedProblem &pr = a.pr;
    constexpr unsigned kWaves = 8u;
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned li = lane & 15u, kb = lane >> 4;
    constexpr unsigned kItemRows = FUSED_UP ? 64u : 128u;
    constexpr unsigned kStagedTokens = NB * 16u;
    const unsigned code_lane = kCodeBase + (lane & 31u) * 8u;
    const unsigned sel_lane = kSelBase + (lane & 15u) * 8u;
    const unsigned lut_lane = kLutBase + (lane & 15u) * 16u;
    const unsigned superblocks = a.width >> 8;

    // ---- activation rows this lane copies: wave w owns the 4-token groups w, w + kWaves, ... ----
    // Lane l of a group moves piece position l % 16 of token 4 g + l / 16; LDS receives the
    // wave's 64 pieces back to back, so the swizzle is applied on the global side.
    constexpr unsigned kCopies = (kStagedTokens / 4u + kWaves - 1u) / kWaves;
    auto token_row = [&](unsigned token) {
        const unsigned live = token < it.tokens ? token : it.tokens - 1u;   // padding repeats a row
        const unsigned long long ordered = it.pair0 + live;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long arow = pr.act_by_ordered_pair ? ordered : source / pr.topk;
        return (const unsigned char *)pr.activations + arow * pr.act_stride;
    };
    const unsigned char *copy_from[kCopies];
#pragma unroll
    for (unsigned j = 0; j < kCopies; ++j) {
        const unsigned token = 4u * (wave + kWaves * j) + (lane >> 4);
        copy_from[j] = token_row(token) + 4u + 16u * ((lane & 15u) ^ (token & 15u));
    }
    // waves 0 and 1 also copy the block scales of tokens 64 w + lane
    const unsigned char *scale_from = token_row(64u * (wave & 1u) + lane);

    // ---- the weight row of this lane: waves 0-3 hold gate blocks and waves 4-7 the matching up
    // blocks when the SwiGLU is fused ----
    unsigned out_row_base;
    const unsigned char *weight_row;
    {
        bool is_up = false;
        if constexpr (FUSED_UP) {
            out_row_base = it.row_tile * kItemRows + (wave & 3u) * 16u;
            is_up = wave >= 4u;
        } else {
            out_row_base = it.row_tile * kItemRows + wave * 16u;
        }
        unsigned row = out_row_base + li;
        if (row >= a.out_rows) row = a.out_rows - 1u;
        weight_row = is_up
            ? pr.up + it.expert * pr.up_expert_bytes + (unsigned long long)row * pr.up_row_bytes
            : pr.gate + it.expert * pr.expert_bytes + (unsigned long long)row * pr.row_bytes;
    }
    // Superblocks are 66 bytes, so group records start on 2-byte boundaries, and vector loads
    // that are not dword-aligned run at less than half rate: the lane loads twelve aligned bytes
    // around each record and shifts them into place. Records of superblock sb start
    // (row start + 2 sb + 2) mod 4 bytes past a dword, the fp16 scale (row start + 2 sb) mod 4.
    const unsigned row_misalign = (unsigned)(unsigned long long)weight_row & 3u;
    const unsigned char *row_aligned = weight_row - row_misalign;
    const unsigned lane_group = kb >> 1;                      // groups 2 ks + lane_group

    float acc[NB][4];
#pragma unroll
    for (unsigned tb = 0; tb < NB; ++tb)
#pragma unroll
        for (unsigned r = 0; r < 4u; ++r) acc[tb][r] = 0.0f;

    RawGroup raw[4];
    unsigned raw_scale;
    auto copy_activations = [&](unsigned sb, unsigned stage) {
        const unsigned base = kStageBase + stage * kStageBytes;
#pragma unroll
        for (unsigned j = 0; j < kCopies; ++j) {
            const unsigned group = wave + kWaves * j;            // wave-uniform
            if (group * 4u < kStagedTokens)
                copy_to_lds_16(copy_from[j] + (unsigned long long)sb * kQ8KBytes,
                               (unsigned)__builtin_amdgcn_readfirstlane((int)(base + group * 1024u)));
        }
        if (wave < 2u && wave * 64u < kStagedTokens)
            copy_to_lds_4(scale_from + (unsigned long long)sb * kQ8KBytes,
                          (unsigned)__builtin_amdgcn_readfirstlane((int)(base + kStageActs + wave * 256u)));
    };
    auto fetch_codes = [&](unsigned sb) {
        const unsigned block = row_misalign + sb * 66u;         // from row_aligned
        raw_scale = *reinterpret_cast<const unsigned *>(row_aligned + (block & ~3u));
#pragma unroll
        for (unsigned ks = 0; ks < 3u; ++ks)
            raw[ks] = *reinterpret_cast<const RawGroup *>(
                row_aligned + ((block + 2u + 8u * (2u * ks + lane_group)) & ~3u));
        // The last record of a superblock may be the last bytes of the tensor: its third dword
        // is read only when it holds bytes of the record (an aligned dword with a valid byte
        // lies in a mapped page), otherwise the second dword is read again.
        const unsigned start = block + 2u + 8u * (6u + lane_group);
        const unsigned char *at = row_aligned + (start & ~3u);
        const uint2 head = *reinterpret_cast<const uint2 *>(at);
        raw[3].x = head.x;
        raw[3].y = head.y;
        raw[3].z = *reinterpret_cast<const unsigned *>(at + 4u + 2u * (start & 3u));
    };
    uint2 now_codes[4];
    unsigned now_scale16;
    auto settle_codes = [&](unsigned sb) {   // the registers fetch_codes(sb) filled -> records
        const unsigned shift = (row_misalign + 2u * sb + 2u) & 3u;
        now_scale16 = (raw_scale >> (8u * ((row_misalign + 2u * sb) & 3u))) & 0xffffu;
#pragma unroll
        for (unsigned ks = 0; ks < 4u; ++ks) {
            now_codes[ks].x = __builtin_amdgcn_alignbyte(raw[ks].y, raw[ks].x, shift);
            now_codes[ks].y = __builtin_amdgcn_alignbyte(raw[ks].z, raw[ks].y, shift);
        }
    };
    // LDS offsets of this lane's fragment pieces: piece 4 ks + kb of token 16 tb + li
    unsigned piece[4];
#pragma unroll
    for (unsigned ks = 0; ks < 4u; ++ks) piece[ks] = li * kActPitch + (((4u * ks + kb) ^ li) << 4);

    __syncthreads();   // every wave is done with the previous item's stages
    copy_activations(0u, 0u);
    fetch_codes(0u);
    __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): the copies above have landed in LDS
    settle_codes(0u);
    __syncthreads();

    const unsigned last = superblocks - 1u;
    for (unsigned sb = 0; sb < superblocks; ++sb) {
        const unsigned base = kStageBase + (sb & 1u) * kStageBytes;
        const unsigned ahead = sb < last ? sb + 1u : last;     // the last turn repeats a request
        copy_activations(ahead, (sb & 1u) ^ 1u);
        fetch_codes(ahead);

        v4i sum_lo[NB], sum_hi[NB];
#pragma unroll
        for (unsigned tb = 0; tb < NB; ++tb) {
            sum_lo[tb] = v4i{0, 0, 0, 0};
            sum_hi[tb] = v4i{0, 0, 0, 0};
        }
        // Software pipeline over phases (K step, group of up to four token blocks): the
        // activation fragments of the next phase and the table lookups of the next K step are
        // requested before the current phase's matrix instructions are issued, so their LDS
        // latency runs under those instructions.
        constexpr unsigned kGroups = NB > 4u ? 2u : 1u;      // groups per K step
        constexpr unsigned kGroupSize = NB / kGroups;
        constexpr unsigned kPhases = 4u * kGroups;
        uint2 codes_of[2], signs_of[2];
        uint4 limbs_of;
        auto lookup = [&](unsigned ks) {
            // the lane's sixteen weights: subgroups 2 (kb & 1) and 2 (kb & 1) + 1 of its group
            const unsigned grids = now_codes[ks].x >> (16u * (kb & 1u));
            const unsigned aux = now_codes[ks].y;
            const unsigned signs = aux >> (14u * (kb & 1u));
            codes_of[0] = lds_read_uint2(__builtin_amdgcn_perm(grids, code_lane, 0x0c0c0400u));
            codes_of[1] = lds_read_uint2(__builtin_amdgcn_perm(grids, code_lane, 0x0c0c0500u));
            signs_of[0] = lds_read_uint2(((signs << 7) & 0x3f80u) | sel_lane);
            signs_of[1] = lds_read_uint2((signs & 0x3f80u) | sel_lane);
            limbs_of = lds_read_uint4(((aux >> 20) & 0xf00u) | lut_lane);
        };
        v4i a_lo, a_hi;
        auto weights_from_lookup = [&]() {
            const unsigned s0 = codes_of[0].x | signs_of[0].x, s1 = codes_of[0].y | signs_of[0].y;
            const unsigned s2 = codes_of[1].x | signs_of[1].x, s3 = codes_of[1].y | signs_of[1].y;
            a_lo = v4i{(int)__builtin_amdgcn_perm(limbs_of.y, limbs_of.x, s0),
                       (int)__builtin_amdgcn_perm(limbs_of.y, limbs_of.x, s1),
                       (int)__builtin_amdgcn_perm(limbs_of.y, limbs_of.x, s2),
                       (int)__builtin_amdgcn_perm(limbs_of.y, limbs_of.x, s3)};
            a_hi = v4i{(int)__builtin_amdgcn_perm(limbs_of.w, limbs_of.z, s0),
                       (int)__builtin_amdgcn_perm(limbs_of.w, limbs_of.z, s1),
                       (int)__builtin_amdgcn_perm(limbs_of.w, limbs_of.z, s2),
                       (int)__builtin_amdgcn_perm(limbs_of.w, limbs_of.z, s3)};
        };
        uint4 frags[2][kGroupSize];
        auto request = [&](unsigned phase, uint4 (&into)[kGroupSize]) {
            const unsigned ks = phase / kGroups, group = phase % kGroups;
#pragma unroll
            for (unsigned i = 0; i < kGroupSize; ++i)
                into[i] = lds_read_uint4(base + piece[ks] + (group * kGroupSize + i) * 16u * kActPitch);
        };
        lookup(0u);
        request(0u, frags[0]);
        weights_from_lookup();
#pragma unroll
        for (unsigned phase = 0; phase < kPhases; ++phase) {
            const unsigned ks = phase / kGroups, group = phase % kGroups;
            if (phase + 1u < kPhases) request(phase + 1u, frags[(phase + 1u) & 1u]);
            if (group == 0u && ks + 1u < 4u) lookup(ks + 1u);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (unsigned i = 0; i < kGroupSize; ++i) {
                const unsigned tb = group * kGroupSize + i;
                const uint4 rawb = frags[phase & 1u][i];
                const v4i b = v4i{(int)rawb.x, (int)rawb.y, (int)rawb.z, (int)rawb.w};
                sum_lo[tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_lo, b, sum_lo[tb], 0, 0, 0);
                sum_hi[tb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_hi, b, sum_hi[tb], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (group == kGroups - 1u && ks + 1u < 4u) weights_from_lookup();
        }
        // ---- exact superblock sums -> fp32 ----
        float row_scale[4];
        {
            const float mine = 0.125f * f16_bits_to_float(now_scale16);
#pragma unroll
            for (unsigned r = 0; r < 4u; ++r) row_scale[r] = __shfl(mine, (int)(4u * kb + r), 64);
        }
#pragma unroll
        for (unsigned tb = 0; tb < NB; ++tb) {
            const float token_scale =
                __uint_as_float(lds_read_u32(base + kStageActs + 4u * (tb * 16u + li)));
#pragma unroll
            for (unsigned r = 0; r < 4u; ++r) {
                const int total = (sum_hi[tb][r] << 7) + sum_lo[tb][r];
                acc[tb][r] = __builtin_fmaf(row_scale[r] * token_scale, (float)total, acc[tb][r]);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0): the next stage is complete in LDS
        settle_codes(ahead);
        __syncthreads();
    }

    // ---- publish: the lane holds C rows 4 kb + r of its block for tokens tb * 16 + li ----
    auto store4 = [&](unsigned token, unsigned row, const float (&value)[4]) {
        const unsigned long long ordered = it.pair0 + token;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long out_index = pr.out_by_source_pair ? source : ordered;
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
    auto route_weight_of = [&](unsigned token) {
        const unsigned long long source = pr.order ? pr.order[it.pair0 + token] : it.pair0 + token;
        return pr.route_weights ? pr.route_weights[source] : 1.0f;
    };
    if constexpr (FUSED_UP) {
        // Gate wave w and up wave w + 4 hold the two inputs of every SwiGLU. They swap token
        // blocks through LDS (the stages are free after the last barrier): gate waves finish
        // blocks [0, G), up waves finish blocks [G, NB).
        constexpr unsigned G = (NB + 1u) / 2u;
        const bool is_gate = wave < 4u;
        const unsigned slot = kStageBase + ((wave & 3u) * 2u + (is_gate ? 0u : 1u)) * 4096u;
        const unsigned peer = kStageBase + ((wave & 3u) * 2u + (is_gate ? 1u : 0u)) * 4096u;
        if (is_gate) {
#pragma unroll
            for (unsigned tb = G; tb < NB; ++tb)
                lds_write_uint4(slot + ((tb - G) * 64u + lane) * 16u,
                                make_uint4(__float_as_uint(acc[tb][0]), __float_as_uint(acc[tb][1]),
                                           __float_as_uint(acc[tb][2]), __float_as_uint(acc[tb][3])));
        } else {
#pragma unroll
            for (unsigned tb = 0; tb < G; ++tb)
                lds_write_uint4(slot + (tb * 64u + lane) * 16u,
                                make_uint4(__float_as_uint(acc[tb][0]), __float_as_uint(acc[tb][1]),
                                           __float_as_uint(acc[tb][2]), __float_as_uint(acc[tb][3])));
        }
        __syncthreads();
        if (is_gate) {
#pragma unroll
            for (unsigned tb = 0; tb < G; ++tb) {
                const unsigned token = tb * 16u + li;
                const uint4 other = lds_read_uint4(peer + (tb * 64u + lane) * 16u);
                if (token < it.tokens) {
                    const float route_weight = route_weight_of(token);
                    const float value[4] = {
                        swiglu_bf16(acc[tb][0], __uint_as_float(other.x), route_weight, a.limit),
                        swiglu_bf16(acc[tb][1], __uint_as_float(other.y), route_weight, a.limit),
                        swiglu_bf16(acc[tb][2], __uint_as_float(other.z), route_weight, a.limit),
                        swiglu_bf16(acc[tb][3], __uint_as_float(other.w), route_weight, a.limit)};
                    store4(token, out_row_base + 4u * kb, value);
                }
            }
        } else {
#pragma unroll
            for (unsigned tb = G; tb < NB; ++tb) {
                const unsigned token = tb * 16u + li;
                const uint4 other = lds_read_uint4(peer + ((tb - G) * 64u + lane) * 16u);
                if (token < it.tokens) {
                    const float route_weight = route_weight_of(token);
                    const float value[4] = {
                        swiglu_bf16(__uint_as_float(other.x), acc[tb][0], route_weight, a.limit),
                        swiglu_bf16(__uint_as_float(other.y), acc[tb][1], route_weight, a.limit),
                        swiglu_bf16(__uint_as_float(other.z), acc[tb][2], route_weight, a.limit),
                        swiglu_bf16(__uint_as_float(other.w), acc[tb][3], route_weight, a.limit)};
                    store4(token, out_row_base + 4u * kb, value);
                }
            }
        }
    } else {
#pragma unroll
        for (unsigned tb = 0; tb < NB; ++tb) {
            const unsigned token = tb * 16u + li;
            if (token < it.tokens) {
                const float value[4] = {bf16_round(acc[tb][0]), bf16_round(acc[tb][1]),
                                        bf16_round(acc[tb][2]), bf16_round(acc[tb][3])};
                store4(token, out_row_base + 4u * kb, value);
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
        // first 128-pair tile of every bucket
        unsigned cursor = 0u;
        for (unsigned b = 0; b < buckets && b < 256u; ++b) {
            lds_write_u32(kTileStartBase + 4u * b, cursor);
            const unsigned long long n = fixed ? pr.pairs : pr.bucket_populations[b];
            cursor += (unsigned)((n + kTileTokens - 1u) / kTileTokens);
        }
        lds_write_u32(kTileStartBase + 4u * (buckets < 256u ? buckets : 256u), cursor);
    }
    __syncthreads();
    if (buckets == 0u || buckets > 256u) {
        if (tid == 0u && buckets > 256u) raise_status(a.status, 2);
        return;
    }

    // weight rows (gate/up row pairs when fused) per work item
    constexpr unsigned kItemRows = FUSED_UP ? 64u : 128u;
    const unsigned row_tiles = (a.out_rows + kItemRows - 1u) / kItemRows;
    const unsigned long long token_tiles = lds_read_u32(kTileStartBase + 4u * buckets);
    const unsigned long long items = token_tiles * row_tiles;

    for (unsigned long long item = blockIdx.x; item < items; item += gridDim.x) {
        // ---- which bucket, row tile and token tile ----
        unsigned low = 0u, high = buckets;
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
        const unsigned token_tile = bucket_tiles ? (unsigned)(local % bucket_tiles) : 0u;
        const unsigned long long first = fixed ? 0ull : pr.bucket_offsets[low];
        const unsigned long long population = fixed ? pr.pairs : pr.bucket_populations[low];
        MfmaItem it;
        it.expert = fixed ? 0ull : pr.expert_ids[low];
        it.row_tile = bucket_tiles ? (unsigned)(local / bucket_tiles) : 0u;
        if (!bucket_tiles || it.expert >= pr.experts || first + population > pr.pairs ||
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
