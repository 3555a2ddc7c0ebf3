// MoE routing, expert-major worklist, and the decode-width grouped expert kernels for gfx950.
//
// The grouped kernels walk buckets (one expert plus the ordered (row, rank) pairs routed to it)
// so an expert's packed bytes are streamed from HBM once per bucket and reused for every pair in
// it. Lanes own fixed column ranges of the activation rows and keep them in registers; weight
// rows stream through with unaligned 16-byte loads; integer superblock sums are exact.
//
// Behaviour restated from src/backend/cuda/moe_kernels.cu:180-291 (routing), :294-402
// (worklist), :431-616 (grouped up/down, reduce, combine) and src/graph/moe.c:497-622.
#include "common.hpp"
#include "launch.hpp"
#include "units.hpp"
#include "grouped.hpp"
#include "q8k.hpp"

namespace yvex {

// ---- routing --------------------------------------------------------------------------------

// The scores alone, as the token-local operation publishes them beside the logits
// (src/backend/cuda/moe_kernels.cu:29-55).
__global__ __launch_bounds__(256) void route_scores_kernel(
    const float *__restrict__ logits, unsigned count, int scoring, float *__restrict__ scores, int *status)
{
    const unsigned i = blockIdx.x * 256u + threadIdx.x;
    if (i >= count) return;
    const double s = route_score((double)logits[i], scoring);
    const float published = (float)s;
    if (!(s == s) || !finite_f32(published)) raise_status(status, 1);
    scores[i] = published;
}

// One wavefront per row; each lane scores four experts (experts <= 256).
// Largest value of the 64 lanes, in every lane: butterflies inside each row of 16 lanes, then the
// rows' results carried upward (lane 15 into the next row, lane 31 into the upper half) and the
// last lane read back.
template <int CTRL, int ROWS>
__device__ __forceinline__ unsigned dpp_max_u32(unsigned v)
{
    const unsigned other = (unsigned)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, ROWS, 0xf, false);
    return other > v ? other : v;
}

__device__ __forceinline__ unsigned wave_max_u32(unsigned v)
{
    v = dpp_max_u32<0xb1, 0xf>(v);    // quad_perm [1, 0, 3, 2]
    v = dpp_max_u32<0x4e, 0xf>(v);    // quad_perm [2, 3, 0, 1]
    v = dpp_max_u32<0x141, 0xf>(v);   // row_half_mirror
    v = dpp_max_u32<0x140, 0xf>(v);   // row_mirror
    v = dpp_max_u32<0x142, 0xa>(v);   // row_bcast15 into rows 1 and 3
    v = dpp_max_u32<0x143, 0xc>(v);   // row_bcast31 into rows 2 and 3
    return (unsigned)__builtin_amdgcn_readlane((int)v, 63);
}

// What a lane reads of one row: the logits (or the scores a launch before this one has
// published: the float a double-precision score rounds to, what route_row works out from a logit
// otherwise) and the correction biases of experts 4 lane .. 4 lane + 3. The loads depend on
// nothing and sit under no condition on the lane (a lane past the last expert reads the last
// one's again), so a caller can ask for a row's values while it routes the row before: under
// `if (e < experts)` they were issued, and waited for, one expert after another.
struct RouteInputs {
    float value[4], bias[4];
};

__device__ __forceinline__ void route_inputs_load(RouteInputs &in, const float *__restrict__ values,
                                                  const float *__restrict__ bias, unsigned long long row,
                                                  unsigned lane, unsigned experts)
{
#pragma unroll
    for (unsigned i = 0; i < 4u; ++i) {
        const unsigned e = lane * 4u + i < experts ? lane * 4u + i : experts - 1u;
        in.value[i] = values[row * experts + e];
        in.bias[i] = bias ? bias[e] : 0.0f;
    }
}

// One row by one wavefront. `published`: in.value holds scores, not logits.
__device__ __forceinline__ void route_row(
    const RouteInputs &in, bool published, unsigned long long row, unsigned lane,
    unsigned experts, unsigned topk, int scoring, int normalize, double scaling,
    unsigned long long *__restrict__ selected, float *__restrict__ weights, int *status)
{
    float score[4];
    unsigned long long key[4];
#pragma unroll
    for (unsigned i = 0; i < 4u; ++i) {
        const unsigned e = lane * 4u + i;
        score[i] = 0.0f;
        key[i] = 0ull;
        if (e < experts) {
            if (published) {
                score[i] = in.value[i];
            } else {
                const double s = route_score((double)in.value[i], scoring);
                score[i] = (float)s;      // (a NaN stays a NaN)
            }
            float biased = in.bias[i] + score[i];
            if (!finite_f32(score[i]) || !finite_f32(biased)) raise_status(status, 1);
            biased += 0.0f;   // -0 and +0 must compare equal
            const unsigned bits = __float_as_uint(biased);
            const unsigned sortable = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
            // larger score first, then the lower expert ordinal; +1 keeps live keys non-zero
            key[i] = ((unsigned long long)sortable << 32) | (unsigned long long)(0xfffffffeu - e + 1u);
        }
    }
    double total = 0.0;
    float picked_score = 0.0f;   // lane r keeps the score of rank r
    for (unsigned rank = 0; rank < topk; ++rank) {
        unsigned long long best = key[0];
#pragma unroll
        for (unsigned i = 1; i < 4u; ++i) best = key[i] > best ? key[i] : best;
        // The wave's best key in two steps that need no cross-lane permutes through LDS: the
        // largest score word, then the first lane holding it (a lane's ordinals are below the
        // next lane's, and its own best already is its lowest ordinal with that score).
        const unsigned top = wave_max_u32((unsigned)(best >> 32));
        const unsigned long long holders = __ballot((unsigned)(best >> 32) == top);
        const unsigned winner = (unsigned)__builtin_ctzll(holders);
        const unsigned e = 0xffffffffu - (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(best & 0xffffffffull),
                                                                             (int)winner);
        float s = 0.0f;
#pragma unroll
        for (unsigned i = 0; i < 4u; ++i)
            if (lane * 4u + i == e) {
                s = score[i];
                key[i] = 0ull;
            }
        // (the winner's ordinal is the same in every lane: a lane read, no permute through LDS)
        s = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(s), (int)(e >> 2)));
        total += (double)s;                 // rank order, in double (src/graph/moe.c:566-574)
        if (lane == rank) picked_score = s;
        if (lane == 0u) selected[row * topk + rank] = e;
    }
    if (normalize && !(total > 0.0 && total < 1.0e300)) raise_status(status, 1);
    if (lane < topk) {
        double value = (double)picked_score;
        if (normalize) value /= total;
        value *= scaling;
        const float w = (float)value;
        if (!finite_f32(w)) raise_status(status, 1);
        weights[row * topk + lane] = w;
    }
}

__global__ __launch_bounds__(256) void route_rows_kernel(
    const float *__restrict__ logits, const float *__restrict__ bias, unsigned long long rows,
    unsigned experts, unsigned topk, int scoring, int normalize, double scaling,
    unsigned long long *__restrict__ selected, float *__restrict__ weights, int *status)
{
    const unsigned long long row = (unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6);
    if (row >= rows) return;
    RouteInputs in;
    route_inputs_load(in, logits, bias, row, threadIdx.x & 63u, experts);
    route_row(in, false, row, threadIdx.x & 63u, experts, topk, scoring, normalize, scaling, selected,
              weights, status);
}

// Hash router (src/backend/cuda/moe_kernels.cu:222-245, src/graph/moe.c:539-582): a row's experts
// are the first topk ordinals of its token's row of an I32 table; weights as for the learned
// router. One wavefront per row, lane r holds rank r. An ordinal outside the expert range, a
// repeated one or a token outside the table is a contract violation (status 2).
__global__ __launch_bounds__(256) void route_hash_rows_kernel(
    const float *__restrict__ logits, const unsigned char *__restrict__ table,
    const unsigned *__restrict__ token_ids, unsigned long long rows, unsigned experts, unsigned topk,
    unsigned long long table_rows, unsigned long long table_row_bytes, int single_row, int scoring,
    int normalize, double scaling, unsigned long long *__restrict__ selected,
    float *__restrict__ weights, int *status)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned long long row = (unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6);
    if (row >= rows) return;
    const unsigned long long token = token_ids[row];
    if (token >= table_rows) {
        if (lane == 0u) raise_status(status, 2);
        return;
    }
    const int *ordinals = reinterpret_cast<const int *>(table + (single_row ? 0ull : token * table_row_bytes));
    const int mine = lane < topk ? ordinals[lane] : -1;
    const bool live = lane < topk;
    bool bad = live && (mine < 0 || (unsigned)mine >= experts);
    float score = 0.0f;
    if (live && !bad) {
        const double s = route_score((double)logits[row * experts + (unsigned)mine], scoring);
        score = (float)s;
        if (!(s == s) || !finite_f32(score)) raise_status(status, 1);
    }
    double total = 0.0;
    for (unsigned rank = 0; rank < topk; ++rank) {
        const int other = __shfl(mine, (int)rank, kWave);
        bad |= live && rank < lane && other == mine;
        total += (double)__shfl(score, (int)rank, kWave);      // rank order, in double
    }
    if (bad) raise_status(status, 2);
    if (normalize && !(total > 0.0 && total < 1.0e300)) raise_status(status, 1);
    if (live) {
        double value = (double)score;
        if (normalize) value /= total;
        value *= scaling;
        const float w = (float)value;
        if (!finite_f32(w)) raise_status(status, 1);
        weights[row * topk + lane] = w;
        selected[row * topk + lane] = bad ? 0ull : (unsigned long long)mine;
    }
}

// ---- worklist -------------------------------------------------------------------------------
//
// A row never routes to the same expert twice, so each expert's pairs are a set of rows: one bit
// per (expert, row) in LDS. Bucket order is expert order, order inside a bucket is row order,
// which is exactly the stable counting sort of pairs by expert (src/graph/worklist.c:380-393).

constexpr unsigned kWorklistMaxRows = 4096u;

// The whole worklist by one workgroup; shared_words is its dynamic LDS (worklist_lds_bytes).
__device__ __forceinline__ void worklist_block(
    const unsigned long long *__restrict__ selected, unsigned pairs, unsigned topk,
    unsigned experts, unsigned long long *__restrict__ order,
    unsigned long long *__restrict__ expert_ids, unsigned long long *__restrict__ bucket_offsets,
    unsigned long long *__restrict__ bucket_populations,
    unsigned long long *__restrict__ sweep_offsets, unsigned long long *__restrict__ counts,
    int *status, unsigned *shared_words, bool with_below)
{
    const unsigned rows = pairs / topk;
    const unsigned words = (rows + 31u) / 32u;            // bitmap words per expert
    unsigned *bitmap = shared_words;                       // [experts][words]
    unsigned *population = bitmap + experts * words;       // [experts]
    unsigned *offset = population + experts;               // [experts + 1]
    unsigned *slot = offset + experts + 1u;                // [experts] bucket index or ~0
    __shared__ unsigned bad;
    const unsigned tid = threadIdx.x;
    for (unsigned i = tid; i < experts * words; i += blockDim.x) bitmap[i] = 0u;
    if (tid == 0u) {
        bad = 0u;
        slot[experts + 1536u] = 0u;   // running maximum of the populations (scan[1536])
    }
    __syncthreads();
    for (unsigned p = tid; p < pairs; p += blockDim.x) {
        const unsigned long long e = selected[p];
        if (e >= experts) {
            bad = 1u;
            continue;
        }
        const unsigned row = p / topk;
        const unsigned old = atomicOr(&bitmap[(unsigned)e * words + (row >> 5)], 1u << (row & 31u));
        if (old & (1u << (row & 31u))) bad = 1u;   // duplicate expert inside one row
    }
    __syncthreads();
    // rows below each bitmap word that chose the expert (16 bits: at most 4096 rows), kept when
    // the table fits beside the bitmap
    unsigned short *below = reinterpret_cast<unsigned short *>(slot + experts + 1537u);
    for (unsigned e = tid; e < experts; e += blockDim.x) {
        unsigned n = 0u;
        for (unsigned w = 0; w < words; ++w) {
            if (with_below) below[e * words + w] = (unsigned short)n;
            n += __popc(bitmap[e * words + w]);
        }
        population[e] = n;
    }
    __syncthreads();
    // Inclusive prefix sums over the experts (<= 256: the first four wavefronts) of population,
    // sweep count and occupancy: a shuffle scan inside each wavefront, the wavefronts' totals
    // through LDS (one barrier); every expert then publishes its own bucket.
    unsigned *scan = slot + experts;                       // [4][3] wavefront totals; [1536] running maximum
    const unsigned n_mine = tid < experts ? population[tid] : 0u;
    unsigned sum_n = n_mine, sum_sweeps = (n_mine + (unsigned)kPass - 1u) / (unsigned)kPass,
             sum_used = n_mine ? 1u : 0u;
    if (tid < 256u) {
#pragma unroll
        for (int step = 1; step < 64; step <<= 1) {
            const unsigned a = (unsigned)__shfl_up((int)sum_n, step, kWave);
            const unsigned b = (unsigned)__shfl_up((int)sum_sweeps, step, kWave);
            const unsigned c = (unsigned)__shfl_up((int)sum_used, step, kWave);
            if ((int)(tid & 63u) >= step) {
                sum_n += a;
                sum_sweeps += b;
                sum_used += c;
            }
        }
        if ((tid & 63u) == 63u) {
            scan[3u * (tid >> 6)] = sum_n;
            scan[3u * (tid >> 6) + 1u] = sum_sweeps;
            scan[3u * (tid >> 6) + 2u] = sum_used;
        }
    }
    __syncthreads();
    unsigned total_pairs = 0u, total_sweeps = 0u, bucket_count = 0u;
    for (unsigned w = 0; w < 4u; ++w) {
        const unsigned a = scan[3u * w], b = scan[3u * w + 1u], c = scan[3u * w + 2u];
        if (w < (tid >> 6)) {
            sum_n += a;
            sum_sweeps += b;
            sum_used += c;
        }
        total_pairs += a;
        total_sweeps += b;
        bucket_count += c;
    }
    if (tid < experts) {
        const unsigned n = n_mine;
        const unsigned cursor = sum_n - n;
        const unsigned sweeps_before = sum_sweeps - (n + (unsigned)kPass - 1u) / (unsigned)kPass;
        const unsigned bucket = sum_used - (n ? 1u : 0u);
        offset[tid] = cursor;
        if (n) {
            expert_ids[bucket] = tid;
            bucket_offsets[bucket] = cursor;
            bucket_populations[bucket] = n;
            sweep_offsets[bucket] = sweeps_before;
        }
        if (tid >= bucket_count) {                         // unused tail of the bucket arrays
            expert_ids[tid] = 0ull;
            bucket_populations[tid] = 0ull;
            bucket_offsets[tid + 1u] = total_pairs;
            sweep_offsets[tid + 1u] = total_sweeps;
        }
    }
    if (tid == 0u) {
        offset[experts] = total_pairs;
        bucket_offsets[bucket_count] = total_pairs;
        sweep_offsets[bucket_count] = total_sweeps;
        counts[0] = bucket_count;
        counts[2] = total_pairs;
        counts[3] = total_sweeps;
        if (total_pairs != pairs) bad = 1u;
    }
    // largest population: one atomic per wave after a wave-wide maximum
    {
        unsigned n = tid < experts ? population[tid] : 0u;
#pragma unroll
        for (int offset_lanes = 32; offset_lanes > 0; offset_lanes >>= 1) {
            const unsigned other = (unsigned)__shfl_xor((int)n, offset_lanes, kWave);
            n = other > n ? other : n;
        }
        if ((tid & 63u) == 0u && tid < 256u) atomicMax(&scan[1536u], n);
    }
    __syncthreads();
    if (tid == 0u) counts[1] = scan[1536u];
    // every pair finds its own place: its bucket's start plus the rows below its own that chose
    // the same expert (pairs of a bucket stay in row order, which is the stable order)
    for (unsigned p = tid; p < pairs; p += blockDim.x) {
        const unsigned long long e = selected[p];
        if (e >= experts) continue;
        const unsigned row = p / topk, w = row >> 5;
        const unsigned *mine = bitmap + (unsigned)e * words;
        unsigned before = __popc(mine[w] & ((1u << (row & 31u)) - 1u));
        if (with_below) before += below[(unsigned)e * words + w];
        else
            for (unsigned k = 0; k < w; ++k) before += __popc(mine[k]);
        order[offset[e] + before] = p;
    }
    __syncthreads();
    if (tid == 0u && bad) raise_status(status, 2);
}

__global__ __launch_bounds__(1024) void worklist_kernel(
    const unsigned long long *__restrict__ selected, unsigned pairs, unsigned topk,
    unsigned experts, unsigned long long *__restrict__ order,
    unsigned long long *__restrict__ expert_ids, unsigned long long *__restrict__ bucket_offsets,
    unsigned long long *__restrict__ bucket_populations,
    unsigned long long *__restrict__ sweep_offsets, unsigned long long *__restrict__ counts,
    int *status, int with_below)
{
    extern __shared__ unsigned shared_words[];
    worklist_block(selected, pairs, topk, experts, order, expert_ids, bucket_offsets, bucket_populations,
                   sweep_offsets, counts, status, shared_words, with_below != 0);
}

// A decode batch's preparation in one launch instead of three: workgroup 0 routes the rows (one
// wavefront a row, sixteen at a time) and then builds the worklist from what it wrote; every
// other workgroup quantizes sixteen Q8_K blocks of the input rows, which depend on neither.
constexpr unsigned kPrepareMaxRows = 128u;

__global__ __launch_bounds__(1024) void decode_prepare_kernel(
    const float *__restrict__ logits, const float *__restrict__ bias, unsigned rows, unsigned experts,
    unsigned topk, int scoring, int normalize, double scaling, unsigned long long *selected,
    float *__restrict__ weights, unsigned long long *__restrict__ order,
    unsigned long long *__restrict__ expert_ids, unsigned long long *__restrict__ bucket_offsets,
    unsigned long long *__restrict__ bucket_populations, unsigned long long *__restrict__ sweep_offsets,
    unsigned long long *__restrict__ counts, const float *__restrict__ values, unsigned blocks,
    unsigned long long input_stride, unsigned char *__restrict__ encoded, int *status,
    const float *__restrict__ scores)
{
    extern __shared__ unsigned shared_words[];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    if (blockIdx.x != 0u) {
        const unsigned task = (blockIdx.x - 1u) * 16u + wave;
        if (task >= rows * blocks) return;
        const unsigned row = task / blocks, block = task % blocks;
        q8k_quantize_block(values + (unsigned long long)row * input_stride + block * 256u + lane * 4u,
                           encoded + (unsigned long long)task * kQ8KBytes, lane, status);
        return;
    }
    // a wave's rows one after another, the next row's values on their way while this one is routed
    const float *values_in = scores ? scores : logits;
    RouteInputs current;
    if (wave < rows) route_inputs_load(current, values_in, bias, wave, lane, experts);
    for (unsigned row = wave; row < rows; row += 16u) {
        RouteInputs next;
        route_inputs_load(next, values_in, bias, row + 16u < rows ? row + 16u : row, lane, experts);
        route_row(current, scores != nullptr, row, lane, experts, topk, scoring, normalize, scaling, selected,
                  weights, status);
        current = next;
    }
    __syncthreads();   // the selections written above are read back by other waves below
    worklist_block(selected, rows * topk, topk, experts, order, expert_ids, bucket_offsets,
                   bucket_populations, sweep_offsets, counts, status, shared_words, true);
}

// ---- grouped expert projections ---------------------------------------------------------------
//
// Persistent kernel: one 512-thread workgroup per compute unit builds the conflict-free lookup
// tables once, then each of its waves walks a strided list of work items. An item is
// (bucket, tile of weight rows, sweep): a bucket's expert bytes stream from HBM once per sweep
// and every sweep serves up to kPass pairs of the bucket.

constexpr int kRowsInFlight = 1;  // weight-row groups a wave decodes back to back
constexpr int kGroupedThreads = 512;     // two waves per SIMD: with three, a sweep's activation columns spill out of 168 registers
constexpr int kGroupedWaves = kGroupedThreads / 64;
constexpr unsigned kItemRowsMax = 16u;   // gate/up row pairs per item when the SwiGLU is fused

struct LaneGeometry {
    unsigned rows_per_wave, reduce_width, sub, seg, unit0, super;
    bool lane_live;
    unsigned wave;
};

// One sweep of a wave over the item's weight rows [row_begin, row_end) with N live pairs.
// Each iteration handles kRows row groups; the packed bytes of the next iteration are requested
// before the current one is decoded, so HBM latency hides behind the decode.
template <unsigned QT, bool Q8, bool FUSED_UP, int N, typename Tables>
__device__ __forceinline__ void grouped_sweep(
    const GroupedArgs &a, const GroupedProblem &pr, const Tables &tables, const LaneGeometry &g,
    const unsigned char *gate_e, const unsigned char *up_e, unsigned long long first_ordered,
    unsigned row_begin, unsigned row_end, float *park, float *terms)
{
    constexpr int kStreams = FUSED_UP ? 2 : 1;
    constexpr int kRows = Q8 ? kRowsInFlight : 1;
    // ---- the sweep's activation rows: this lane's 128 columns stay in registers (Q8_K) ----
    unsigned act[N][Q8 ? kUnitsPerLane * 8 : 1];
    float act_scale[N];
    int act_bsum[N][(QT == QT_Q4_K || QT == QT_Q2_K) ? 8 : 1];
    const unsigned char *act_row[N];
    float route_weight[N];
    unsigned long long out_index[N];
#pragma unroll
    for (int p = 0; p < N; ++p) {
        const unsigned long long ordered = first_ordered + p;
        const unsigned long long source = pr.order ? pr.order[ordered] : ordered;
        const unsigned long long arow = pr.act_by_ordered_pair ? ordered : source / pr.topk;
        act_row[p] = (const unsigned char *)pr.activations + arow * pr.act_stride;
        route_weight[p] = pr.route_weights ? pr.route_weights[source] : 1.0f;
        out_index[p] = pr.out_by_source_pair ? source : ordered;
        act_scale[p] = 0.0f;
        if constexpr (Q8) {
            const unsigned char *blk = act_row[p] + (unsigned long long)g.super * kQ8KBytes;
            act_scale[p] = *reinterpret_cast<const float *>(blk);
            const unsigned char *q = blk + 4u + 32u * (g.unit0 & 7u);   // 4-byte aligned payload
#pragma unroll
            for (int k = 0; k < kUnitsPerLane * 2; ++k) {
                uint4 v;
                __builtin_memcpy(&v, q + 16 * k, 16);
                act[p][4 * k] = v.x;
                act[p][4 * k + 1] = v.y;
                act[p][4 * k + 2] = v.z;
                act[p][4 * k + 3] = v.w;
            }
            if constexpr (QT == QT_Q4_K || QT == QT_Q2_K) {
                const short *bs = reinterpret_cast<const short *>(blk + 260u) + 2u * (g.unit0 & 7u);
#pragma unroll
                for (int i = 0; i < 8; ++i) act_bsum[p][i] = bs[i];
            }
        }
    }

    const unsigned stride = kRows * g.rows_per_wave;
    LaneChunk<QT> next[kRows][kStreams];
    auto request = [&](unsigned base) {
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            const unsigned want = base + r * g.rows_per_wave + g.sub;
            const unsigned safe_row = (g.lane_live && want < row_end) ? want : row_begin;
            next[r][0].load(gate_e + (unsigned long long)safe_row * pr.row_bytes, g.unit0);
            if constexpr (FUSED_UP)
                next[r][1].load(up_e + (unsigned long long)safe_row * pr.up_row_bytes, g.unit0);
        }
    };
    request(row_begin);

    for (unsigned base = row_begin; base < row_end; base += stride) {
        LaneChunk<QT> chunk[kRows][kStreams];
#pragma unroll
        for (int r = 0; r < kRows; ++r)
#pragma unroll
            for (int w = 0; w < kStreams; ++w) chunk[r][w] = next[r][w];
        if (base + stride < row_end) request(base + stride);

        float sums[kRows][kStreams][N];
        double wide[Q8 ? 1 : kRows][Q8 ? 1 : kStreams][Q8 ? 1 : N];   // F32 activations: the lane's sums in double
        unsigned row[kRows];
        bool row_live[kRows];
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            row[r] = base + r * g.rows_per_wave + g.sub;
            row_live[r] = g.lane_live && row[r] < row_end;
#pragma unroll
            for (int w = 0; w < kStreams; ++w) {
                const LaneChunk<QT> &c = chunk[r][w];
                int whole_dot[N], whole_min[N];
                int unit_dots[N][UnitTraits<QT>::kIntegerCombine ? 1 : kUnitsPerLane];   // Q8_0: a dot per 32-value block
#pragma unroll
                for (int p = 0; p < N; ++p) {
                    whole_dot[p] = whole_min[p] = 0;
                    sums[r][w][p] = 0.0f;
                    if constexpr (!Q8) wide[r][w][p] = 0.0;
                }
#pragma unroll
                for (int k = 0; k < kUnitsPerLane; ++k) {
                    Unit unit;
                    c.decode(tables, k, g.unit0, unit);
#pragma unroll
                    for (int p = 0; p < N; ++p) {
                        if constexpr (Q8) {
                            const unsigned *av = &act[p][8 * k];
                            int d = 0, d2 = 0;
                            if constexpr (QT == QT_Q2_K) {
#pragma unroll
                                for (int i = 0; i < 4; ++i) {
                                    d = dot4(unit.w[i], av[i], d);
                                    d2 = dot4(unit.w[4 + i], av[4 + i], d2);
                                }
                                d = __mul24(unit.factor, d) + __mul24(unit.factor2, d2);
                            } else {
#pragma unroll
                                for (int i = 0; i < 8; ++i) d = dot4(unit.w[i], av[i], d);
                                if constexpr (QT != QT_Q8_0) d = __mul24(d, unit.factor);
                            }
                            if constexpr (UnitTraits<QT>::kIntegerCombine) {
                                whole_dot[p] += d;
                                if constexpr (QT == QT_Q4_K || QT == QT_Q2_K)
                                    whole_min[p] += unit.min1 * act_bsum[p][2 * k] +
                                                    unit.min2 * act_bsum[p][2 * k + 1];
                            } else {
                                unit_dots[p][k] = d;
                            }
                        } else {
                            const float *x = reinterpret_cast<const float *>(act_row[p]) +
                                             32ull * (g.unit0 + k);
                            wide[r][w][p] = chunk_unit_dot_f64<QT>(c, k, unit, x, wide[r][w][p]);
                        }
                    }
                }
                if constexpr (Q8 && UnitTraits<QT>::kIntegerCombine) {
                    // two neighbouring lanes hold the halves of one superblock: finish the exact
                    // integer sum; both compute the float value, the odd lane contributes zero
#pragma unroll
                    for (int p = 0; p < N; ++p) {
                        UnitSum t;
                        t.dot = group_sum_i32<2>(whole_dot[p]);
                        t.min = 0;
                        if constexpr (QT != QT_IQ2_XXS) t.min = group_sum_i32<2>(whole_min[p]);
                        const float v = c.combine(act_scale[p], t);
                        sums[r][w][p] = (g.seg & 1u) ? 0.0f : v;
                    }
                }
                if constexpr (Q8 && !UnitTraits<QT>::kIntegerCombine) {
                    // Q8_0: the term of a Q8_K block is one chain of eight fused multiply-adds over
                    // its eight 32-value blocks (kernel_primitives.h:342-359). The even lane of the
                    // pair runs the first four links, the odd lane goes on from there and holds the
                    // block's term.
#pragma unroll
                    for (int p = 0; p < N; ++p) {
                        float total = 0.0f;
#pragma unroll
                        for (int k = 0; k < kUnitsPerLane; ++k)
                            total = __builtin_fmaf(c.unit_scale(k) * act_scale[p], (float)unit_dots[p][k], total);
                        float carried = dpp_move_f32<0xa0, 0xf>(total);     // quad_perm [0,0,2,2]: the even neighbour's
#pragma unroll
                        for (int k = 0; k < kUnitsPerLane; ++k)
                            carried = __builtin_fmaf(c.unit_scale(k) * act_scale[p], (float)unit_dots[p][k], carried);
                        sums[r][w][p] = (g.seg & 1u) ? carried : 0.0f;
                    }
                }
            }
        }
        // ---- sum across the lanes of each row, then publish ----
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            if constexpr (Q8) {
                // One float term per superblock sits in a lane of its pair (the even one; Q8_0: the
                // odd one). The row's first lane adds them in double, in superblock order, and
                // rounds once: the row dot of the CPU path (src/gguf/quant_compute.c:152-172 adds a
                // row's blocks in double).
                const unsigned lane = threadIdx.x & 63u;
                constexpr unsigned kTermLane = UnitTraits<QT>::kIntegerCombine ? 0u : 1u;
                const unsigned blocks = a.width >> 8;
#pragma unroll
                for (int w = 0; w < kStreams; ++w)
#pragma unroll
                    for (int p = 0; p < N; ++p)
                        terms[(w * N + p) * 64 + lane] = row_live[r] ? sums[r][w][p] : 0.0f;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                if (row_live[r] && g.seg == 0u) {
#pragma unroll
                    for (int w = 0; w < kStreams; ++w)
#pragma unroll
                        for (int p = 0; p < N; ++p) {
                            double sum = 0.0;
                            for (unsigned k = 0; k < blocks; ++k)
                                sum += (double)terms[(w * N + p) * 64 + lane + 2u * k + kTermLane];
                            sums[r][w][p] = (float)sum;
                        }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            } else {
                // F32 activations: the lanes' double sums added in double, rounded once
                // (the CPU row dot: src/gguf/quant_compute.c:152-172)
#pragma unroll
                for (int w = 0; w < kStreams; ++w)
#pragma unroll
                    for (int p = 0; p < N; ++p) {
                        double sum = row_live[r] ? wide[r][w][p] : 0.0;
                        for (unsigned offset = g.reduce_width >> 1; offset; offset >>= 1)
                            sum += __shfl_xor(sum, (int)offset, kWave);
                        sums[r][w][p] = (float)sum;
                    }
            }
            if constexpr (FUSED_UP) {
                // park (gate, up); the SwiGLU runs once per item with every lane busy
                const unsigned local = row[r] - row_begin;
                if (row_live[r] && g.seg == 0u && local < kItemRowsMax) {
#pragma unroll
                    for (int p = 0; p < N; ++p) {
                        park[(0u * kItemRowsMax + local) * kPass + p] = sums[r][0][p];
                        park[(1u * kItemRowsMax + local) * kPass + p] = sums[r][1][p];
                    }
                }
            } else if (row_live[r] && g.seg == 0u) {
#pragma unroll
                for (int p = 0; p < N; ++p) {
                    const float value = bf16_round(sums[r][0][p]);
                    if (!finite_f32(value)) raise_status(a.status, 1);
                    else pr.out[out_index[p] * a.out_rows + row[r]] = value;
                }
            }
        }
    }
    if constexpr (FUSED_UP) {
        // LDS operations of one wave complete in order: no barrier between park and read
        const unsigned lane = threadIdx.x & 63u;
        const unsigned local = lane >> 2;
        const int p = (int)(lane & 3u);
        const unsigned out_row = row_begin + local;
        if (local < kItemRowsMax && out_row < row_end && p < N) {
            float rw = route_weight[0];
            unsigned long long oi = out_index[0];
#pragma unroll
            for (int q = 1; q < N; ++q) {
                if (p == q) {
                    rw = route_weight[q];
                    oi = out_index[q];
                }
            }
            const float value = swiglu_bf16(park[(0u * kItemRowsMax + local) * kPass + p],
                                            park[(1u * kItemRowsMax + local) * kPass + p], rw, a.limit);
            if (!finite_f32(value)) raise_status(a.status, 1);
            else pr.out[oi * a.out_rows + out_row] = value;
        }
    }
}

template <unsigned QT>
struct GroupedTables {
    using type = Iq2Tables;   // unused placeholder for qtypes without lookup tables
};
template <>
struct GroupedTables<QT_IQ2_XXS> {
    using type = Iq2TablesWide;
};

template <unsigned QT, bool Q8, bool FUSED_UP>
__global__ __launch_bounds__(kGroupedThreads) void grouped_kernel(GroupedArgs a)
{
    extern __shared__ __align__(16) unsigned char grouped_lds[];
    typename GroupedTables<QT>::type tables;
    unsigned char *after_tables = grouped_lds;
    if constexpr (QT == QT_IQ2_XXS) {
        // the lookups address LDS directly: the dynamic block must start at LDS address 0
        if (lds_address_of(grouped_lds) != 0u) {
            if (threadIdx.x == 0u) raise_status(a.status, 2);
            return;
        }
        tables = iq2_tables_wide_fill(grouped_lds);
        after_tables = grouped_lds + kIq2WideBytes;
        __syncthreads();
    }
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    float *park = reinterpret_cast<float *>(after_tables) + wave * (2u * kItemRowsMax * kPass);
    // per wave: the float terms of an iteration, one word per (stream, pair, lane)
    float *terms = reinterpret_cast<float *>(after_tables) + kGroupedWaves * (2u * kItemRowsMax * kPass) +
                   wave * (2u * kPass * 64u);

    const unsigned units = a.width >> 5;                          // multiple of 8
    const unsigned lanes_per_row = units / kUnitsPerLane;         // even, <= 64
    const bool pow2 = (lanes_per_row & (lanes_per_row - 1u)) == 0u;
    LaneGeometry g;
    g.rows_per_wave = pow2 ? 64u / lanes_per_row : 1u;
    g.reduce_width = pow2 ? lanes_per_row : 64u;
    g.sub = lane / lanes_per_row;
    g.seg = lane % lanes_per_row;
    g.lane_live = g.sub < g.rows_per_wave;
    g.unit0 = g.seg * kUnitsPerLane;                              // four units, one superblock
    g.super = g.unit0 >> 3;
    g.wave = wave;

    const unsigned tiles = (a.out_rows + a.item_rows - 1u) / a.item_rows;
    const unsigned long long wave_id = (unsigned long long)blockIdx.x * kGroupedWaves + wave;
    const unsigned long long wave_count = (unsigned long long)gridDim.x * kGroupedWaves;

    // The shared expert's items come first (their number is known at launch), then the routed
    // buckets the device-built worklist reports.
    for (int which = (int)a.problems - 1; which >= 0; --which) {
        const GroupedProblem &pr = a.problem[which];
        const bool fixed = pr.expert_ids == nullptr;
        // a work item is one sweep over one tile; sweeps are numbered across all buckets
        const unsigned long long buckets = fixed ? 1ull : pr.counts[0];
        const unsigned long long sweeps = fixed ? pr.sweeps : pr.counts[3];
        const unsigned long long items = sweeps * tiles;
        // stagger the second list so the waves that ran short on the first start it
        const unsigned long long shift = which == 0 && a.problems > 1
            ? ((unsigned long long)tiles * a.problem[1].sweeps) % wave_count : 0ull;
        unsigned long long item = (wave_id + wave_count - shift) % wave_count;
        for (; item < items; item += wave_count) {
            // Items of one bucket are contiguous and, inside a bucket, the sweeps over one tile
            // are neighbours: neighbouring waves stream the same bytes at the same time, so only
            // the first of them goes to HBM.
            unsigned long long expert = 0ull, first = 0ull, population = pr.pairs;
            unsigned long long local = item, bucket_sweeps = sweeps;
            if (!fixed) {
                // last bucket whose first item is <= item
                unsigned long long low = 0ull, high = buckets;
                while (low + 1ull < high) {
                    const unsigned long long middle = (low + high) >> 1;
                    if (pr.sweep_offsets[middle] * tiles <= item) low = middle;
                    else high = middle;
                }
                expert = pr.expert_ids[low];
                first = pr.bucket_offsets[low];
                population = pr.bucket_populations[low];
                local = item - pr.sweep_offsets[low] * tiles;
                bucket_sweeps = pr.sweep_offsets[low + 1ull] - pr.sweep_offsets[low];
            }
            if (bucket_sweeps == 0ull) {
                if (lane == 0u) raise_status(a.status, 2);
                continue;
            }
            const unsigned tile = (unsigned)(local / bucket_sweeps);
            const unsigned long long pass = (local % bucket_sweeps) * kPass;
            if (expert >= pr.experts || first + population > pr.pairs || pass >= population ||
                tile >= tiles) {
                if (lane == 0u) raise_status(a.status, 2);
                continue;
            }
            const unsigned char *gate_e = pr.gate + expert * pr.expert_bytes;
            const unsigned char *up_e = FUSED_UP ? pr.up + expert * pr.up_expert_bytes : nullptr;
            const unsigned row_begin = tile * a.item_rows;
            const unsigned row_end = row_begin + a.item_rows < a.out_rows ? row_begin + a.item_rows
                                                                          : a.out_rows;
            if (population - pass >= 2ull)
                grouped_sweep<QT, Q8, FUSED_UP, 2>(a, pr, tables, g, gate_e, up_e, first + pass,
                                                   row_begin, row_end, park, terms);
            else
                grouped_sweep<QT, Q8, FUSED_UP, 1>(a, pr, tables, g, gate_e, up_e, first + pass,
                                                   row_begin, row_end, park, terms);
        }
    }
}

// LANES columns per thread (4 when the width allows 16-byte accesses); each column's sum runs in
// rank order, so the result does not depend on LANES.
template <int LANES>
__global__ __launch_bounds__(256) void reduce_combine_kernel(
    const float *__restrict__ pair_outputs, unsigned long long rows, unsigned topk,
    unsigned long long hidden, const float *__restrict__ shared, float *__restrict__ routed,
    float *__restrict__ combined, int *status)
{
    struct alignas(4 * LANES) Pack {
        float v[LANES];
    };
    const unsigned long long index = ((unsigned long long)blockIdx.x * 256ull + threadIdx.x) * LANES;
    if (index >= rows * hidden) return;
    const unsigned long long row = index / hidden, column = index % hidden;
    Pack total;
#pragma unroll
    for (int i = 0; i < LANES; ++i) total.v[i] = 0.0f;
    const float *source = pair_outputs + row * topk * hidden + column;
    unsigned rank = 0;
    for (; rank + 4u <= topk; rank += 4u) {     // four ranks' loads in flight, added in rank order
        Pack part[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) part[k] = *reinterpret_cast<const Pack *>(source + (rank + k) * hidden);
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int i = 0; i < LANES; ++i) total.v[i] += part[k].v[i];
    }
    for (; rank < topk; ++rank) {
        const Pack part = *reinterpret_cast<const Pack *>(source + rank * hidden);
#pragma unroll
        for (int i = 0; i < LANES; ++i) total.v[i] += part.v[i];
    }
    bool good = true;
#pragma unroll
    for (int i = 0; i < LANES; ++i) good = good && finite_f32(total.v[i]);
    if (!good) {
        raise_status(status, 1);
        return;
    }
    if (routed) *reinterpret_cast<Pack *>(routed + index) = total;
    if (combined && shared) {
        const Pack base = *reinterpret_cast<const Pack *>(shared + index);
        Pack value;
#pragma unroll
        for (int i = 0; i < LANES; ++i) {
            value.v[i] = bf16_round(total.v[i] + base.v[i]);
            good = good && finite_f32(value.v[i]);
        }
        if (!good) raise_status(status, 1);
        else *reinterpret_cast<Pack *>(combined + index) = value;
    }
}

template <unsigned QT, bool Q8, bool FUSED>
static int launch_grouped_variant(const GroupedArgs &a, hipStream_t stream)
{
    const size_t lds = (QT == QT_IQ2_XXS ? kIq2WideBytes : 0u) +
                       (size_t)kGroupedWaves * 2u * kItemRowsMax * kPass * sizeof(float) +
                       (size_t)kGroupedWaves * 2u * kPass * 64u * sizeof(float);
    YVEX_ALLOW_DYNAMIC_LDS((grouped_kernel<QT, Q8, FUSED>), lds);
    grouped_kernel<QT, Q8, FUSED><<<compute_units(), kGroupedThreads, lds, stream>>>(a);
    return check_launch("moe_grouped");
}

template <unsigned QT>
static int launch_grouped(const GroupedArgs &a, bool q8, bool fused, hipStream_t stream)
{
    if (fused) return q8 ? launch_grouped_variant<QT, true, true>(a, stream)
                         : launch_grouped_variant<QT, false, true>(a, stream);
    return q8 ? launch_grouped_variant<QT, true, false>(a, stream)
              : launch_grouped_variant<QT, false, false>(a, stream);
}

static int dispatch_grouped(unsigned qtype, const GroupedArgs &a, bool q8, bool fused,
                            hipStream_t stream)
{
    bool aligned = true;   // the specialised sweeps load dwords: bases and strides must allow it
    for (unsigned i = 0; i < a.problems; ++i) {
        const GroupedProblem &pr = a.problem[i];
        aligned = aligned && ((uintptr_t)pr.gate % 4u == 0u) && pr.expert_bytes % 4u == 0u &&
                  (!pr.up || ((uintptr_t)pr.up % 4u == 0u && pr.up_expert_bytes % 4u == 0u));
    }
    unsigned long long all_pairs = 0ull;
    for (unsigned i = 0; i < a.problems; ++i) all_pairs += a.problem[i].pairs;
    // (Q2_K rows have the sweeps for a plain projection, the down experts, only)
    if (q8 && aligned && !(qtype == QT_Q2_K && fused) &&
        iq2_sweep_supported(qtype, a.width, a.out_rows, all_pairs, a.image != 0))
        return launch_iq2_sweep(a, qtype, fused, a.image != 0, stream);
    if (a.image) return ST_UNSUPPORTED;      // only the specialised sweeps read the image
    switch (qtype) {
    case QT_IQ2_XXS: return launch_grouped<QT_IQ2_XXS>(a, q8, fused, stream);
    case QT_Q4_K: return launch_grouped<QT_Q4_K>(a, q8, fused, stream);
    case QT_Q8_0: return launch_grouped<QT_Q8_0>(a, q8, fused, stream);
    case QT_Q2_K: return launch_grouped<QT_Q2_K>(a, q8, fused, stream);
    default: return ST_UNSUPPORTED;
    }
}

}  // namespace yvex

using namespace yvex;

extern "C" int yvex_hip_moe_route_rows(const float *logits, const float *bias, uint64_t rows,
                                       uint64_t experts, uint64_t topk, int scoring,
                                       int normalize, double scaling, uint64_t *selected,
                                       float *weights, int *status, yvex_hip_stream stream)
{
    if (!logits || !selected || !weights || !status || !rows || !experts || experts > 256u ||
        !topk || topk > 16u || topk > experts ||
        (scoring != YVEX_HIP_SCORING_SQRT_SOFTPLUS && scoring != YVEX_HIP_SCORING_SIGMOID))
        return ST_INVALID_ARG;
    const uint64_t grid = (rows + 3u) / 4u;
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    route_rows_kernel<<<(unsigned)grid, 256, 0, as_stream(stream)>>>(
        logits, bias, rows, (unsigned)experts, (unsigned)topk, scoring, normalize, scaling,
        (unsigned long long *)selected, weights, status);
    return check_launch("moe_route_rows");
}

extern "C" int yvex_hip_moe_route_hash_rows(const float *logits, const uint8_t *table,
                                            const uint32_t *token_ids, uint64_t rows,
                                            uint64_t experts, uint64_t topk, uint64_t table_rows,
                                            uint64_t table_row_bytes, int single_row, int scoring,
                                            int normalize,
                                            double scaling, uint64_t *selected, float *weights,
                                            int *status, yvex_hip_stream stream)
{
    if (!logits || !table || !token_ids || !selected || !weights || !status || !rows || !experts ||
        experts > 256u || !topk || topk > 16u || topk > experts || !table_rows ||
        ((uintptr_t)table & 3u) ||
        (scoring != YVEX_HIP_SCORING_SQRT_SOFTPLUS && scoring != YVEX_HIP_SCORING_SIGMOID))
        return ST_INVALID_ARG;
    if (table_row_bytes < topk * 4u || (table_row_bytes & 3u)) return ST_BOUNDS;
    const uint64_t grid = (rows + 3u) / 4u;
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    route_hash_rows_kernel<<<(unsigned)grid, 256, 0, as_stream(stream)>>>(
        logits, table, token_ids, rows, (unsigned)experts, (unsigned)topk, table_rows, table_row_bytes,
        single_row, scoring, normalize, scaling, (unsigned long long *)selected, weights, status);
    return check_launch("moe_route_hash_rows");
}

extern "C" int yvex_hip_moe_route_scores(const float *logits, uint64_t count, int scoring,
                                         float *scores, int *status, yvex_hip_stream stream)
{
    if (!logits || !scores || !status || !count || count > 0x7fffffffull ||
        (scoring != YVEX_HIP_SCORING_SQRT_SOFTPLUS && scoring != YVEX_HIP_SCORING_SIGMOID))
        return ST_INVALID_ARG;
    route_scores_kernel<<<(unsigned)((count + 255u) / 256u), 256, 0, as_stream(stream)>>>(
        logits, (unsigned)count, scoring, scores, status);
    return check_launch("moe_route_scores");
}

constexpr size_t kWorklistLdsLimit = 160u * 1024u - 64u;

// Dynamic LDS of the worklist workgroup; *with_below says whether the 16-bit table of rows below
// each bitmap word fits as well.
static size_t worklist_lds_bytes(uint64_t experts, uint64_t rows, int *with_below)
{
    const uint64_t words = (rows + 31u) / 32u;
    const size_t base = (size_t)(experts * words + 3u * experts + 1u + 1537u) * sizeof(unsigned);
    const size_t table = (size_t)(experts * words) * sizeof(unsigned short);
    *with_below = base + table <= kWorklistLdsLimit;
    return *with_below ? base + table : base;
}

extern "C" int yvex_hip_worklist_build(const uint64_t *selected, uint64_t pairs, uint64_t topk,
                                       uint64_t experts, uint64_t *order, uint64_t *expert_ids,
                                       uint64_t *bucket_offsets, uint64_t *bucket_populations,
                                       uint64_t *sweep_offsets, uint64_t *counts, int *status,
                                       yvex_hip_stream stream)
{
    if (!selected || !order || !expert_ids || !bucket_offsets || !bucket_populations ||
        !sweep_offsets || !counts ||
        !status || !pairs || !topk || !experts || experts > 256u || pairs % topk)
        return ST_INVALID_ARG;
    const uint64_t rows = pairs / topk;
    if (rows > kWorklistMaxRows) return ST_BOUNDS;
    int with_below = 0;
    const size_t lds = worklist_lds_bytes(experts, rows, &with_below);
    YVEX_ALLOW_DYNAMIC_LDS(worklist_kernel, kWorklistLdsLimit);
    if (lds > kWorklistLdsLimit) return ST_BOUNDS;
    worklist_kernel<<<1, 1024, lds, as_stream(stream)>>>(
        (const unsigned long long *)selected, (unsigned)pairs, (unsigned)topk, (unsigned)experts,
        (unsigned long long *)order, (unsigned long long *)expert_ids,
        (unsigned long long *)bucket_offsets, (unsigned long long *)bucket_populations,
        (unsigned long long *)sweep_offsets, (unsigned long long *)counts, status, with_below);
    return check_launch("worklist_build");
}

extern "C" int yvex_hip_moe_prepare_supported(uint64_t rows, uint64_t experts, uint64_t topk)
{
    return rows != 0u && rows <= kPrepareMaxRows && experts != 0u && experts <= 256u && topk != 0u &&
           topk <= experts && topk <= 16u;
}

static int launch_moe_prepare(const float *logits, const float *scores, const float *bias, uint64_t rows,
                              uint64_t experts, uint64_t topk, int scoring, int normalize, double scaling,
                              uint64_t *selected, float *weights, uint64_t *order, uint64_t *expert_ids,
                              uint64_t *bucket_offsets, uint64_t *bucket_populations, uint64_t *sweep_offsets,
                              uint64_t *counts, const float *values, uint64_t width, uint64_t input_stride,
                              uint8_t *encoded, int *status, yvex_hip_stream stream)
{
    if ((!logits && !scores) || !selected || !weights || !order || !expert_ids || !bucket_offsets ||
        !bucket_populations || !sweep_offsets || !counts || !status || (scoring != 0 && scoring != 1))
        return ST_INVALID_ARG;
    if (!yvex_hip_moe_prepare_supported(rows, experts, topk)) return ST_UNSUPPORTED;
    uint64_t tasks = 0u;
    if (values) {
        if (!encoded || !width || width % 256u || input_stride < width || width / 256u > 0xffffu)
            return ST_INVALID_ARG;
        tasks = rows * (width / 256u);
    }
    int with_below = 0;
    const size_t lds = worklist_lds_bytes(experts, rows, &with_below);   // always fits at these sizes
    if (!with_below) return ST_BOUNDS;
    decode_prepare_kernel<<<(unsigned)(1u + (tasks + 15u) / 16u), 1024, lds, as_stream(stream)>>>(
        logits, bias, (unsigned)rows, (unsigned)experts, (unsigned)topk, scoring, normalize, scaling,
        (unsigned long long *)selected, weights, (unsigned long long *)order,
        (unsigned long long *)expert_ids, (unsigned long long *)bucket_offsets,
        (unsigned long long *)bucket_populations, (unsigned long long *)sweep_offsets,
        (unsigned long long *)counts, values, (unsigned)(width / 256u), input_stride, encoded, status, scores);
    return check_launch("moe_prepare");
}

extern "C" int yvex_hip_moe_prepare(const float *logits, const float *bias, uint64_t rows, uint64_t experts,
                                    uint64_t topk, int scoring, int normalize, double scaling,
                                    uint64_t *selected, float *weights, uint64_t *order,
                                    uint64_t *expert_ids, uint64_t *bucket_offsets,
                                    uint64_t *bucket_populations, uint64_t *sweep_offsets, uint64_t *counts,
                                    const float *values, uint64_t width, uint64_t input_stride,
                                    uint8_t *encoded, int *status, yvex_hip_stream stream)
{
    if (!logits) return ST_INVALID_ARG;
    return launch_moe_prepare(logits, nullptr, bias, rows, experts, topk, scoring, normalize, scaling, selected,
                              weights, order, expert_ids, bucket_offsets, bucket_populations, sweep_offsets,
                              counts, values, width, input_stride, encoded, status, stream);
}

extern "C" int yvex_hip_moe_prepare_scored(const float *scores, const float *bias, uint64_t rows,
                                           uint64_t experts, uint64_t topk, int normalize, double scaling,
                                           uint64_t *selected, float *weights, uint64_t *order,
                                           uint64_t *expert_ids, uint64_t *bucket_offsets,
                                           uint64_t *bucket_populations, uint64_t *sweep_offsets,
                                           uint64_t *counts, const float *values, uint64_t width,
                                           uint64_t input_stride, uint8_t *encoded, int *status,
                                           yvex_hip_stream stream)
{
    if (!scores) return ST_INVALID_ARG;
    return launch_moe_prepare(nullptr, scores, bias, rows, experts, topk, 0, normalize, scaling, selected, weights,
                              order, expert_ids, bucket_offsets, bucket_populations, sweep_offsets, counts,
                              values, width, input_stride, encoded, status, stream);
}

extern "C" int yvex_hip_moe_up(const yvex_hip_expert_weights *w, const void *activations,
                               int act_q8, const float *route_weights, const uint64_t *order,
                               const uint64_t *expert_ids, const uint64_t *bucket_offsets,
                               const uint64_t *bucket_populations, const uint64_t *sweep_offsets,
                               const uint64_t *counts, uint64_t pairs, uint64_t topk,
                               uint64_t experts, double limit,
                               float *intermediate, const yvex_hip_expert_weights *shared,
                               uint64_t shared_rows, float *shared_intermediate, int *status,
                               yvex_hip_stream stream)
{
    if (!w || !w->gate || !w->up || !activations || !intermediate || !status || !pairs || !topk ||
        !experts || !(limit > 0.0) || (act_q8 != 0 && act_q8 != 1) ||
        (expert_ids && (!bucket_offsets || !bucket_populations || !sweep_offsets || !counts)) ||
        (shared && (!shared->gate || !shared->up || !shared_rows || !shared_intermediate)))
        return ST_INVALID_ARG;
    if (w->gate_qtype != w->up_qtype) return ST_UNSUPPORTED;
    int rc = w->gate_up_image
        ? check_image_matrix(w->gate_qtype, w->hidden, w->gate_row_bytes, w->gate, w->gate_expert_bytes)
        : check_matrix(w->gate_qtype, w->hidden, w->gate_row_bytes);
    if (rc) return rc;
    if (w->gate_up_image && (!act_q8 || ((uintptr_t)w->up & 3u) || (w->up_expert_bytes & 3u)))
        return ST_UNSUPPORTED;
    if (w->up_row_bytes != w->gate_row_bytes) return ST_BOUNDS;
    if (pairs > 0xffffffffull || w->intermediate > 0xffffffffull || shared_rows > 0xffffffffull)
        return ST_BOUNDS;
    if (shared && (!same_shape(w, shared) || shared->gate_row_bytes != w->gate_row_bytes ||
                   shared->up_row_bytes != w->up_row_bytes ||
                   (shared->gate_up_image != 0) != (w->gate_up_image != 0)))
        return ST_UNSUPPORTED;   // launch the shared expert on its own instead
    GroupedArgs a{};
    const WorklistView wl{order, expert_ids, bucket_offsets, bucket_populations, sweep_offsets, counts};
    fill_up_problem(a.problem[0], w, activations, act_q8, route_weights, wl, pairs, topk, experts,
                    intermediate);
    a.problems = 1u;
    if (shared) {
        const WorklistView none{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
        fill_up_problem(a.problem[1], shared, activations, act_q8, nullptr, none, shared_rows, 1u,
                        1u, shared_intermediate);
        a.problems = 2u;
    }
    a.width = (unsigned)w->hidden;
    a.out_rows = (unsigned)w->intermediate;
    a.item_rows = kItemRowsMax;
    a.limit = limit;
    a.status = status;
    a.image = w->gate_up_image != 0;
    return dispatch_grouped(w->gate_qtype, a, act_q8 != 0, true, as_stream(stream));
}

extern "C" int yvex_hip_moe_down(const yvex_hip_expert_weights *w, const void *intermediate,
                                 int act_q8, const uint64_t *order, const uint64_t *expert_ids,
                                 const uint64_t *bucket_offsets,
                                 const uint64_t *bucket_populations, const uint64_t *sweep_offsets,
                                 const uint64_t *counts, uint64_t pairs, uint64_t experts,
                                 float *pair_outputs,
                                 const yvex_hip_expert_weights *shared, uint64_t shared_rows,
                                 const void *shared_intermediate, float *shared_outputs,
                                 int *status, yvex_hip_stream stream)
{
    if (!w || !w->down || !intermediate || !pair_outputs || !status || !pairs || !experts ||
        (act_q8 != 0 && act_q8 != 1) ||
        (expert_ids && (!bucket_offsets || !bucket_populations || !sweep_offsets || !counts)) ||
        (shared && (!shared->down || !shared_rows || !shared_intermediate || !shared_outputs)))
        return ST_INVALID_ARG;
    int rc = w->down_image
        ? check_image_matrix(w->down_qtype, w->intermediate, w->down_row_bytes, w->down, w->down_expert_bytes)
        : check_matrix(w->down_qtype, w->intermediate, w->down_row_bytes);
    if (rc) return rc;
    if (w->down_image && !act_q8) return ST_UNSUPPORTED;
    if (pairs > 0xffffffffull || w->hidden > 0xffffffffull || shared_rows > 0xffffffffull)
        return ST_BOUNDS;
    if (shared && (!same_shape(w, shared) || shared->down_row_bytes != w->down_row_bytes ||
                   (shared->down_image != 0) != (w->down_image != 0)))
        return ST_UNSUPPORTED;
    GroupedArgs a{};
    const WorklistView wl{order, expert_ids, bucket_offsets, bucket_populations, sweep_offsets, counts};
    fill_down_problem(a.problem[0], w, intermediate, act_q8, wl, pairs, experts, pair_outputs);
    a.problems = 1u;
    if (shared) {
        const WorklistView none{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
        fill_down_problem(a.problem[1], shared, shared_intermediate, act_q8, none, shared_rows, 1u,
                          shared_outputs);
        a.problems = 2u;
    }
    a.width = (unsigned)w->intermediate;
    a.out_rows = (unsigned)w->hidden;
    a.item_rows = 64u;
    a.limit = 1.0;
    a.status = status;
    a.image = w->down_image != 0;
    return dispatch_grouped(w->down_qtype, a, act_q8 != 0, false, as_stream(stream));
}

// The clamped SiLU-gated products of given gate and up sums (src/graph/moe.c:605-611), rounded
// to bfloat16 as the fused kernels round them; out may be either input.
__global__ __launch_bounds__(256) void swiglu_rows_kernel(const float *gate, const float *up,
                                                          unsigned long long count, double limit, float *out,
                                                          int *status)
{
    const unsigned long long at = (unsigned long long)blockIdx.x * 256ull + threadIdx.x;
    if (at >= count) return;
    const float value = swiglu_bf16_fast(gate[at], up[at], 1.0f, limit, (float)limit);
    if (!finite_f32(value)) raise_status(status, 1);
    else out[at] = value;
}

extern "C" int yvex_hip_moe_swiglu_rows(const float *gate, const float *up, uint64_t count, double limit,
                                        float *out, int *status, yvex_hip_stream stream)
{
    if (!gate || !up || !out || !status || !count || !(limit > 0.0)) return ST_INVALID_ARG;
    const uint64_t grid = (count + 255u) / 256u;
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    swiglu_rows_kernel<<<(unsigned)grid, 256, 0, as_stream(stream)>>>(gate, up, count, limit, out, status);
    return check_launch("moe_swiglu_rows");
}

extern "C" int yvex_hip_moe_reduce_combine(const float *pair_outputs, uint64_t rows,
                                           uint64_t topk, uint64_t hidden, const float *shared,
                                           float *routed, float *combined, int *status,
                                           yvex_hip_stream stream)
{
    if (!pair_outputs || !status || !rows || !topk || !hidden || (!routed && !combined) ||
        (combined && !shared) || topk > 0xffffffffull)
        return ST_INVALID_ARG;
    if (rows > UINT64_MAX / hidden) return ST_BOUNDS;
    const uintptr_t addresses = (uintptr_t)pair_outputs | (uintptr_t)shared | (uintptr_t)routed |
                                (uintptr_t)combined;
    const bool quads = hidden % 4u == 0u && addresses % 16u == 0u;
    const uint64_t grid = (rows * hidden / (quads ? 4u : 1u) + 255u) / 256u;
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    if (quads)
        reduce_combine_kernel<4><<<(unsigned)grid, 256, 0, as_stream(stream)>>>(
            pair_outputs, rows, (unsigned)topk, hidden, shared, routed, combined, status);
    else
        reduce_combine_kernel<1><<<(unsigned)grid, 256, 0, as_stream(stream)>>>(
            pair_outputs, rows, (unsigned)topk, hidden, shared, routed, combined, status);
    return check_launch("moe_reduce_combine");
}
