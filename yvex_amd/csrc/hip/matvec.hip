// Encoded matvec (dense projection / output head), gather and the int32 block-sum probe.
//
// One 64-lane wavefront owns one encoded weight row and up to T activation rows; lanes walk the
// row in 32-weight units, so one unit's packed bytes are decoded once and reused for every
// activation row of the tile. Q8_K activations go through v_dot4 integer dots whose exact sums
// are reduced across the eight lanes of a superblock before the single float scaling; F32
// activations use fused multiply-adds. Results are summed across the wave with shuffles.
//
// Behaviour restated from src/backend/cuda/kernels.cu:529-626 (matvec), :784-830 (gather) and
// src/backend/cuda/kernel_primitives.h:218-255,566-596 (row dots).
#include <type_traits>
#include "common.hpp"
#include "launch.hpp"
#include "units.hpp"

namespace yvex {

struct MatvecArgs {
    const unsigned char *encoded;
    unsigned long long row_count, row_width, row_bytes;
    const void *input;
    unsigned long long input_rows, input_stride;
    const float *additive;
    float *out;
    unsigned long long out_stride;
    int output_bf16;
    int *status;
    double *parts;           // split projections: [split][input row][weight row] partial sums
    float *scores;           // join of a split projection: the router scores of the outputs as well
    int scoring;
};

__device__ __forceinline__ void matvec_publish(const MatvecArgs &a, unsigned long long in,
                                               unsigned long long row, float sum)
{
    const unsigned long long at = in * a.out_stride + row;
    float value = a.additive ? sum + a.additive[at] : sum;
    if (!finite_f32(value)) raise_status(a.status, 1);
    else a.out[at] = a.output_bf16 ? bf16_round(value) : value;
}

// Slow exact path for a row whose F32 sum overflowed before opposite terms cancelled
// (kernels.cu:616-620): the whole wave recomputes it in double.
__device__ float matvec_recover_f64(const unsigned char *row, const float *x,
                                    unsigned long long width, unsigned qtype)
{
    double sum = 0.0;
    for (unsigned long long i = threadIdx.x & 63u; i < width; i += 64u)
        sum += (double)qtype_value(row, i, qtype) * (double)x[i];
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, kWave);
    return (float)sum;
}

// U: 64-unit chunks of the row whose loads are issued together before the first of them is used.
// A wave walks one row front to back; with one chunk in flight it waits a full memory latency per
// chunk (weights, then the activation bytes that go with them), which bounds a long matrix such as
// an output head well below what the same loads reach when nothing waits on them.
// EVEN: every row starts on an even address (even base address and even row bytes).
// STAGE (one F32 input row): the workgroup copies the input row into LDS once, 16-byte pieces
// swizzled inside each 128-byte unit, and its four waves read their units from there. A lane owns
// 32 consecutive values, so read from global memory each of its eight 16-byte loads touches 64
// different cache lines, which the memory pipeline serves at about two cycles a line.
template <unsigned QT, bool Q8, int T, int U, bool EVEN, bool STAGE = false>
__global__ __launch_bounds__(256) void matvec_block_kernel(MatvecArgs a)
{
    __shared__ Iq2Tables tables;
    extern __shared__ __align__(16) float4 staged_row[];
    const unsigned long long in0 = (unsigned long long)blockIdx.y * T;
    if constexpr (STAGE) {
        const float4 *source = reinterpret_cast<const float4 *>((const float *)a.input + in0 * a.input_stride);
        const unsigned pieces = (unsigned)(a.row_width >> 2);
        for (unsigned p = threadIdx.x; p < pieces; p += 256u)
            staged_row[(p & ~7u) | ((p ^ (p >> 3)) & 7u)] = source[p];
    }
    if constexpr (QT == QT_IQ2_XXS) iq2_tables_fill(tables);
    if constexpr (QT == QT_IQ2_XXS || STAGE) __syncthreads();
    const unsigned lane = threadIdx.x & 63u;
    const unsigned long long row = (unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6);
    if (row >= a.row_count) return;
    const unsigned char *wrow = a.encoded + row * a.row_bytes;
    const unsigned units = (unsigned)(a.row_width >> 5);
    const unsigned long long act_row_bytes = (a.row_width >> 8) * kQ8KBytes;
    // Q8_K activations against superblock formats: a superblock's float term is formed in the
    // order of the reference's device primitive and the terms of a row are added in double and
    // rounded once, as the CPU path adds a row's blocks (src/gguf/quant_compute.c:152-172): the
    // result is that path's, bit for bit. Q8_0 rows chain their eight terms of a superblock as
    // the primitive chains them (total = fmaf(d_b * d_a, float(dot_b), total), b = 0 .. 7, from
    // zero: kernel_primitives.h:342-359) across the eight lanes that hold the superblock's blocks.
    // F32 activations keep float partial sums, inside the tolerance of the dense projections.
    constexpr bool kWide = Q8 && (UnitTraits<QT>::kIntegerCombine || QT == QT_Q8_0);
    using Sum = typename std::conditional<kWide, double, float>::type;
    Sum acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = (Sum)0;

    // Every lane runs the same trip count so the superblock shuffles below stay converged.
    for (unsigned base = 0; base < units; base += 64u * U) {
        Unit unit[U];
        unsigned uu[U];
        bool live[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const unsigned u = base + 64u * j + lane;
            live[j] = u < units;
            uu[j] = live[j] ? u : units - 1u;
            unit_load<QT, EVEN ? 1 : -1>(tables, wrow, uu[j], unit[j]);
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if (j > 0 && base + 64u * j >= units) break;      // wave-uniform: no chunk here
#pragma unroll
            for (int t = 0; t < T; ++t) {
                unsigned long long in = in0 + t;
                if (in >= a.input_rows) in = a.input_rows - 1ull;   // clamped rows are never written
                if constexpr (Q8) {
                    const unsigned char *act = (const unsigned char *)a.input + in * act_row_bytes +
                                               (unsigned long long)(uu[j] >> 3) * kQ8KBytes;
                    UnitSum s = unit_dot_q8<QT>(unit[j], act, uu[j] & 7u);
                    const float act_scale = *reinterpret_cast<const float *>(act);
                    if constexpr (UnitTraits<QT>::kIntegerCombine) {
                        if (!live[j]) s.dot = s.min = 0;
                        s.dot = group_sum_i32<8>(s.dot);
                        if constexpr (QT != QT_IQ2_XXS) s.min = group_sum_i32<8>(s.min);
                        if (live[j] && (uu[j] & 7u) == 0u)
                            acc[t] += (Sum)super_combine<QT>(wrow + (uu[j] >> 3) * UnitTraits<QT>::kSuperBytes,
                                                             act_scale, s);
                    } else {
                        // lane b of a group of eight holds block b. The start gives lane 0 its
                        // chain (block 0 onto zero); step k gives lane k the chain through block k
                        // from lane k - 1's value of the step before, so after seven steps the last
                        // lane holds the superblock's total. What a lane holds after its own step
                        // is read by nobody and may be anything (units past the row's end belong
                        // to no superblock: a row is whole superblocks)
                        const float scale = f16_bits_to_float((unsigned short)unit[j].scale_bits) * act_scale;
                        const float value = (float)s.dot;
                        float total = __builtin_fmaf(scale, value, 0.0f);
#pragma unroll
                        for (int step = 1; step < 8; ++step) {
                            const float before = __int_as_float(
                                __builtin_amdgcn_update_dpp(0, __float_as_int(total), 0x111, 0xf, 0xf, false));   // row_shr:1
                            total = __builtin_fmaf(scale, value, before);
                        }
                        acc[t] += (Sum)(live[j] && (lane & 7u) == 7u ? total : 0.0f);
                    }
                } else if constexpr (STAGE) {
                    float4 x4[8];
#pragma unroll
                    for (unsigned i = 0; i < 8u; ++i) x4[i] = staged_row[8u * uu[j] + (i ^ (uu[j] & 7u))];
                    const float v = unit_dot_f32_values<QT>(unit[j], wrow, uu[j], x4);
                    if (live[j]) acc[t] += v;
                } else {
                    const float *x = (const float *)a.input + in * a.input_stride + 32ull * uu[j];
                    const float v = unit_dot_f32<QT>(unit[j], wrow, uu[j], x);
                    if (live[j]) acc[t] += v;
                }
            }
        }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
        float sum;
        if constexpr (kWide) {
            double wide = acc[t];
#pragma unroll
            for (int offset = 32; offset > 0; offset >>= 1) wide += __shfl_xor(wide, offset, kWave);
            sum = (float)wide;
        } else {
            sum = group_sum_f32<64>(acc[t]);
        }
        const unsigned long long in = in0 + t;
        if (in >= a.input_rows) continue;
        if constexpr (!Q8) {
            if (!finite_f32(sum) && *a.status == 0)
                sum = matvec_recover_f64(wrow, (const float *)a.input + in * a.input_stride,
                                         a.row_width, QT);
        }
        if (lane == 0u) matvec_publish(a, in, row, sum);
    }
}

// A unit against 32 int8 activations held in registers; `sums` = the two 16-value sums of the
// activations as Q8_K stores them (low and high half of the dword).
template <unsigned QT>
__device__ __forceinline__ UnitSum unit_dot_regs(const Unit &unit, const unsigned *a, unsigned sums)
{
    const int first = (int)(short)(sums & 0xffffu), second = (int)(short)(sums >> 16);
    UnitSum out;
    if constexpr (QT == QT_Q2_K) {
        int d1 = 0, d2 = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            d1 = dot4(unit.w[i], a[i], d1);
            d2 = dot4(unit.w[4 + i], a[4 + i], d2);
        }
        out.dot = unit.factor * d1 + unit.factor2 * d2;
        out.min = unit.min1 * first + unit.min2 * second;
    } else {
        int d = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) d = dot4(unit.w[i], a[i], d);
        out.dot = unit.factor * d;
        out.min = QT == QT_Q4_K ? unit.min1 * (first + second) : 0;
    }
    return out;
}

// A lane's half superblock (units 4 half .. 4 half + 3 of superblock sb) of a weight row that
// starts on a dword boundary. The 32 record bytes of an IQ2_XXS half start on a 2-byte boundary,
// and vector loads that are not dword-aligned run at less than half rate: the aligned dwords
// that hold them are loaded and shifted into place, and the superblock's fp16 scale comes out
// of the aligned dword that holds it (never a byte outside the row's own or its neighbours').
template <unsigned QT>
__device__ __forceinline__ void half_superblock_load(LaneChunk<QT> &chunk, const unsigned char *wrow,
                                                     unsigned sb, unsigned half)
{
    if constexpr (QT == QT_IQ2_XXS) {
        const unsigned char *b = wrow + sb * 66u;
        const unsigned char *p = b + 2u + 32u * half;
        const unsigned shift = (unsigned)(unsigned long long)p & 3u;       // 0 or 2
        const unsigned *at = reinterpret_cast<const unsigned *>(p - shift);
        unsigned raw[9];
#pragma unroll
        for (int i = 0; i < 8; ++i) raw[i] = at[i];
        raw[8] = at[shift ? 8 : 0];                       // (aligned records end with the eighth)
        const unsigned head = *reinterpret_cast<const unsigned *>(b - ((unsigned long long)b & 2ull));
#pragma unroll
        for (int i = 0; i < 8; ++i) chunk.q[i] = __builtin_amdgcn_alignbyte(raw[i + 1], raw[i], shift);
        chunk.d16 = ((unsigned long long)b & 2ull) ? head >> 16 : head & 0xffffu;
    } else {
        chunk.load(wrow, 8u * sb + 4u * half);
    }
}

// One Q8_K input row against superblock-format weight rows, for matrices of a few megabytes
// whose launch is over before the memory system is busy: what counts is the number of memory
// round trips a wave waits for one after another. A lane owns half a superblock (four units)
// of its weight row and L lanes share the row, so a wave holds 64 / L rows; every byte the lane
// needs (weight record, superblock header, activation bytes, their scale and sums) is asked for
// by loads that depend on nothing, issued together, and (IQ2_XXS) the codebook tables are
// built in LDS while those are in flight: one round trip, where the general kernel above
// waits for several in turn (unit after unit, then the header for the lane that combines).
// The float term of a superblock and the double-precision row sum are the general kernel's.
template <unsigned QT, int L>
__global__ __launch_bounds__(256) void dense_row_q8k_kernel(MatvecArgs a)
{
    __shared__ Iq2Tables tables;
    constexpr unsigned kRows = 64u / L;
    const unsigned lane = threadIdx.x & 63u, slot = lane % L;
    unsigned long long row = ((unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6)) * kRows + lane / L;
    const bool row_live = row < a.row_count;
    if (!row_live) row = a.row_count - 1ull;          // (no early exit: the barrier below)
    const unsigned char *wrow = a.encoded + row * a.row_bytes;
    const unsigned halves = (unsigned)(a.row_width >> 7);
    // (asked for ahead of the weight bytes: loads come back in order, and the tables are to be
    // built while the weight bytes are on their way, not after them)
    unsigned digits = 0u;
    if constexpr (QT == QT_IQ2_XXS) digits = k_iq2_digits[threadIdx.x];
    double acc = 0.0;
    for (unsigned base = 0; base < halves; base += L) {
        // a superblock's two lanes are live or clamped together (halves and L are even)
        const bool live = base + slot < halves;
        const unsigned hs = live ? base + slot : halves - 1u;
        const unsigned sb = hs >> 1, half = hs & 1u;
        LaneChunk<QT> chunk;
        half_superblock_load<QT>(chunk, wrow, sb, half);
        const unsigned char *block = (const unsigned char *)a.input + (unsigned long long)sb * kQ8KBytes;
        const unsigned *values = reinterpret_cast<const unsigned *>(block + 4u + 128u * half);
        unsigned act[32], sums[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int i = 0; i < 32; ++i) act[i] = values[i];
        if constexpr (QT != QT_IQ2_XXS) {
            const unsigned *s = reinterpret_cast<const unsigned *>(block + 260u + 16u * half);
#pragma unroll
            for (int i = 0; i < 4; ++i) sums[i] = s[i];
        }
        const float act_scale = *reinterpret_cast<const float *>(block);
        if constexpr (QT == QT_IQ2_XXS) {
            if (base == 0u) {                             // (the same trip for every thread)
                asm volatile("" : "+v"(digits));          // (the entry is not to be worked out, and waited for, ahead of the loads above)
                tables.magnitudes[threadIdx.x] = iq2_magnitude_of_digits(digits);   // 256 threads, 256 entries
                if (threadIdx.x < 128u) tables.signmask[threadIdx.x] = iq2_signmask_entry(threadIdx.x);
                __syncthreads();
            }
        }
        UnitSum total{0, 0};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            Unit unit;
            chunk.decode(tables, k, 8u * sb + 4u * half, unit);
            const UnitSum s = unit_dot_regs<QT>(unit, act + 8 * k, sums[k]);
            total.dot += s.dot;
            total.min += s.min;
        }
        total.dot += dpp_move<0xb1, 0xf>(total.dot);      // the superblock's other half
        if constexpr (QT != QT_IQ2_XXS) total.min += dpp_move<0xb1, 0xf>(total.min);
        const float term = chunk.combine(act_scale, total);
        if (live && half == 0u) acc += (double)term;
    }
    acc = group_sum_f64_last<L>(acc);
    if (row_live && slot == (unsigned)L - 1u) matvec_publish(a, 0ull, row, (float)acc);
}

// The same for a few Q8_K input rows (rows of up to 8192 columns, which L lanes hold whole): the
// lane's four units are decoded once and stay in registers, and the input rows go by one after
// another, the next one's bytes asked for before the current one is multiplied.
struct RowActs {
    unsigned values[32];
    unsigned sums[4];
    float scale;
};

template <unsigned QT>
__device__ __forceinline__ void row_acts_load(RowActs &r, const unsigned char *block, unsigned half)
{
    const unsigned *values = reinterpret_cast<const unsigned *>(block + 4u + 128u * half);
#pragma unroll
    for (int i = 0; i < 32; ++i) r.values[i] = values[i];
    if constexpr (QT != QT_IQ2_XXS) {
        const unsigned *s = reinterpret_cast<const unsigned *>(block + 260u + 16u * half);
#pragma unroll
        for (int i = 0; i < 4; ++i) r.sums[i] = s[i];
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) r.sums[i] = 0u;
    }
    r.scale = *reinterpret_cast<const float *>(block);
}

template <unsigned QT, int L>
__global__ __launch_bounds__(256) void dense_fewrows_q8k_kernel(MatvecArgs a)
{
    __shared__ Iq2Tables tables;
    constexpr unsigned kRows = 64u / L;
    const unsigned lane = threadIdx.x & 63u, slot = lane % L;
    unsigned long long row = ((unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6)) * kRows + lane / L;
    const bool row_live = row < a.row_count;
    if (!row_live) row = a.row_count - 1ull;
    const unsigned char *wrow = a.encoded + row * a.row_bytes;
    const unsigned halves = (unsigned)(a.row_width >> 7);             // <= L
    const unsigned long long act_row_bytes = (a.row_width >> 8) * kQ8KBytes;
    unsigned digits = 0u;
    if constexpr (QT == QT_IQ2_XXS) digits = k_iq2_digits[threadIdx.x];
    const bool live = slot < halves;
    const unsigned hs = live ? slot : halves - 1u;
    const unsigned sb = hs >> 1, half = hs & 1u;
    LaneChunk<QT> chunk;
    half_superblock_load<QT>(chunk, wrow, sb, half);
    const unsigned char *block = (const unsigned char *)a.input + (unsigned long long)sb * kQ8KBytes;
    RowActs current;
    row_acts_load<QT>(current, block, half);
    if constexpr (QT == QT_IQ2_XXS) {
        asm volatile("" : "+v"(digits));
        tables.magnitudes[threadIdx.x] = iq2_magnitude_of_digits(digits);
        if (threadIdx.x < 128u) tables.signmask[threadIdx.x] = iq2_signmask_entry(threadIdx.x);
        __syncthreads();
    }
    Unit units[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) chunk.decode(tables, k, 8u * sb + 4u * half, units[k]);
    for (unsigned long long in = 0; in < a.input_rows; ++in) {
        RowActs next;
        const unsigned long long ahead = in + 1ull < a.input_rows ? in + 1ull : in;
        row_acts_load<QT>(next, block + ahead * act_row_bytes, half);
        UnitSum total{0, 0};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const UnitSum s = unit_dot_regs<QT>(units[k], current.values + 8 * k, current.sums[k]);
            total.dot += s.dot;
            total.min += s.min;
        }
        total.dot += dpp_move<0xb1, 0xf>(total.dot);
        if constexpr (QT != QT_IQ2_XXS) total.min += dpp_move<0xb1, 0xf>(total.min);
        const float term = chunk.combine(current.scale, total);
        const double sum = group_sum_f64_last<L>(live && half == 0u ? (double)term : 0.0);
        if (row_live && slot == (unsigned)L - 1u) matvec_publish(a, in, row, (float)sum);
        current = next;
    }
}

// F32 / F16 / BF16 weight rows: lanes stride the row element-wise. Products and sums run in
// double, as the CPU row dot forms them (src/gguf/quant_compute.c:152-172: double(value) *
// double(x) added in double, rounded to float once); the product of two floats is exact in
// double, so only the order of the double additions differs from the serial loop, far below
// what the final rounding to float keeps.
template <int T>
__global__ __launch_bounds__(256) void matvec_scalar_kernel(MatvecArgs a, unsigned qtype)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned long long row = (unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6);
    const unsigned long long in0 = (unsigned long long)blockIdx.y * T;
    if (row >= a.row_count) return;
    const unsigned char *wrow = a.encoded + row * a.row_bytes;
    double acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.0;
    for (unsigned long long i = lane; i < a.row_width; i += 64u) {
        const float w = qtype_value(wrow, i, qtype);
        if (!finite_f32(w)) raise_status(a.status, 1);
#pragma unroll
        for (int t = 0; t < T; ++t) {
            unsigned long long in = in0 + t;
            if (in >= a.input_rows) in = a.input_rows - 1ull;
            acc[t] += (double)w * (double)((const float *)a.input)[in * a.input_stride + i];
        }
    }
#pragma unroll
    for (int t = 0; t < T; ++t) {
        double sum = acc[t];
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, kWave);
        const unsigned long long in = in0 + t;
        if (in >= a.input_rows) continue;
        if (lane == 0u) matvec_publish(a, in, row, (float)sum);
    }
}

// F32, F16 or BF16 weight rows against fewer than eight F32 input rows (the router and mixing
// projections of a batch of one to seven tokens; a projection or an output head kept in 16-bit
// floats): the lane-strided kernel above walks a row one load at a time, a wave a row: a
// 256 x 7168 F32 router took 90 us of memory round trips, a 129 280 x 7168 F16 head streamed at
// 1.1 TB/s. Here a workgroup owns
// one weight row, its 256 threads take 16-byte pieces of it side by side (a 4 KB stretch a
// step), DEPTH steps of weight and input loads are in flight before the first product, and the
// four waves' double-precision sums are joined through LDS in wave order. Products and sums in
// double as above.
// WAVE_ROW: a wave a weight row (four rows a workgroup, no barrier) for matrices of many rows,
// where the device is full either way and a workgroup a row is a launch and a barrier a row.
template <unsigned QT, int T, int DEPTH, bool WAVE_ROW>
__global__ __launch_bounds__(256) void matvec_scalar_few_kernel(MatvecArgs a)
{
    constexpr unsigned kSpan = WAVE_ROW ? 64u : 256u;       // threads that share a row
    typedef float v4f __attribute__((ext_vector_type(4)));
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    constexpr int kColumns = QT == QT_F32 ? 4 : 8;           // weights in a 16-byte piece
    constexpr int kInputs = kColumns / 4;                    // 16-byte pieces of an input row beside it
    __shared__ double partial[3][T];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned long long row = WAVE_ROW ? (unsigned long long)blockIdx.x * 4ull + wave : blockIdx.x;
    const unsigned long long in0 = (unsigned long long)blockIdx.y * T;
    if (WAVE_ROW && row >= a.row_count) return;
    const unsigned self = WAVE_ROW ? lane : threadIdx.x;
    const v4u *w4 = reinterpret_cast<const v4u *>(a.encoded + row * a.row_bytes);
    const v4f *x4[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const unsigned long long in = in0 + t < a.input_rows ? in0 + t : a.input_rows - 1ull;   // clamped rows are never written
        x4[t] = reinterpret_cast<const v4f *>((const float *)a.input + in * a.input_stride);
    }
    const unsigned pieces = (unsigned)(a.row_width / kColumns);
    double acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.0;
    unsigned bad = 0u;
    for (unsigned base = 0; base < pieces; base += kSpan * DEPTH) {
        const unsigned first = base + self;
        // steps of this turn that hold a piece for some thread (the same for the whole
        // workgroup: a step with none is not loaded at all, a short row costs what it holds)
        const unsigned steps = (pieces - base + kSpan - 1u) / kSpan;
        v4u raw[DEPTH];
        v4f x[T][DEPTH][kInputs];
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            if ((unsigned)u < steps) {
                const unsigned at = first + kSpan * u < pieces ? first + kSpan * u : pieces - 1u;
                raw[u] = w4[at];
#pragma unroll
                for (int t = 0; t < T; ++t)
#pragma unroll
                    for (int j = 0; j < kInputs; ++j) x[t][u][j] = x4[t][at * kInputs + j];
            } else {
                raw[u] = v4u{0u, 0u, 0u, 0u};
#pragma unroll
                for (int t = 0; t < T; ++t)
#pragma unroll
                    for (int j = 0; j < kInputs; ++j) x[t][u][j] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            // (a thread past the end of the row repeated the last piece: its inputs count as
            // zeros. A branch here would pull each step's loads behind it, one wait a step)
            const bool live = first + kSpan * u < pieces;
            float w[kColumns];
#pragma unroll
            for (int c = 0; c < kColumns; ++c) {
                if constexpr (QT == QT_F32) {
                    w[c] = __uint_as_float(raw[u][c]);
                } else {
                    const unsigned bits = (raw[u][c >> 1] >> (16 * (c & 1))) & 0xffffu;
                    w[c] = QT == QT_BF16 ? __uint_as_float(bits << 16) : f16_bits_to_float(bits);
                }
                bad |= (unsigned)!finite_f32(w[c]);
            }
#pragma unroll
            for (int t = 0; t < T; ++t)
#pragma unroll
                for (int c = 0; c < kColumns; ++c)
                    acc[t] += (double)w[c] * (double)(live ? x[t][u][c >> 2][c & 3] : 0.0f);
        }
    }
    if (bad) raise_status(a.status, 1);
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
        for (int offset = 32; offset > 0; offset >>= 1) acc[t] += __shfl_xor(acc[t], offset, kWave);
        if (!WAVE_ROW && wave && lane == 0u) partial[wave - 1u][t] = acc[t];
    }
    if constexpr (WAVE_ROW) {
        if (lane != 0u) return;
#pragma unroll
        for (int t = 0; t < T; ++t)
            if (in0 + t < a.input_rows) matvec_publish(a, in0 + t, row, (float)acc[t]);
        return;
    }
    __syncthreads();
    if (threadIdx.x != 0u) return;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (in0 + t >= a.input_rows) continue;
        const double sum = acc[t] + partial[0][t] + partial[1][t] + partial[2][t];
        matvec_publish(a, in0 + t, row, (float)sum);
    }
}

template <unsigned QT, bool WAVE_ROW>
static int launch_scalar_few_rows(const MatvecArgs &a, hipStream_t s)
{
    const unsigned long long grid_x = WAVE_ROW ? (a.row_count + 3ull) / 4ull : a.row_count;
    if (a.input_rows == 1ull)
        matvec_scalar_few_kernel<QT, 1, 8, WAVE_ROW><<<dim3((unsigned)grid_x, 1), 256, 0, s>>>(a);
    else if (a.input_rows == 2ull)
        matvec_scalar_few_kernel<QT, 2, 8, WAVE_ROW><<<dim3((unsigned)grid_x, 1), 256, 0, s>>>(a);
    else
        matvec_scalar_few_kernel<QT, 4, 4, WAVE_ROW><<<dim3((unsigned)grid_x, (unsigned)((a.input_rows + 3ull) / 4ull)),
                                                       256, 0, s>>>(a);
    return check_launch("matvec_scalar_few");
}

template <unsigned QT>
static int launch_scalar_few(const MatvecArgs &a, hipStream_t s)
{
    // (sixteen waves a compute unit either way from 4096 rows on)
    return a.row_count >= 4096ull ? launch_scalar_few_rows<QT, true>(a, s) : launch_scalar_few_rows<QT, false>(a, s);
}

// F32 weight rows against a batch of F32 input rows (a router or mixing projection over a row
// batch) on the double-precision matrix cores: a workgroup of WAVES waves owns 16 weight rows x
// 16 input rows on V_MFMA_F64_16X16X4_F64 and its waves split the row width. Lane (i, q) loads
// four consecutive floats of weight row i and of input row i at offset 16 j + 4 q. A product of
// two floats is exact in double and the sums run in double, which is how the CPU row dot forms
// them (src/gguf/quant_compute.c:152-172); only the order of the double additions differs from
// its serial loop, so the float the sum rounds to is the CPU path's. The partial tiles of the
// waves (and of the workgroups that split the width: blockIdx.z, joined by a second launch in
// split order) are doubles, added in a fixed order.
// Four consecutive weights (column a multiple of four) of a row of F32, F16 or BF16 values, or of
// Q8_0 blocks (scale times code, exact in float: the value the CPU decoder forms,
// src/gguf/quant_block.c:715-881), as floats.
template <unsigned QT>
__device__ __forceinline__ float4 scalar_weights4(const unsigned char *row, unsigned long long column)
{
    if constexpr (QT == QT_F32) {
        return *reinterpret_cast<const float4 *>(row + 4ull * column);
    } else if constexpr (QT == QT_Q8_0) {
        const unsigned char *block = row + 34ull * (column >> 5);
        const float d = f16_bits_to_float(*reinterpret_cast<const unsigned short *>(block));
        const unsigned char *codes = block + 2u + (unsigned)(column & 31ull);      // on a 2-byte boundary
        const unsigned lo = *reinterpret_cast<const unsigned short *>(codes);
        const unsigned hi = *reinterpret_cast<const unsigned short *>(codes + 2);
        return make_float4(d * (float)(signed char)(lo & 255u), d * (float)(signed char)(lo >> 8),
                           d * (float)(signed char)(hi & 255u), d * (float)(signed char)(hi >> 8));
    } else {
        const uint2 v = *reinterpret_cast<const uint2 *>(row + 2ull * column);
        if constexpr (QT == QT_F16)
            return make_float4(f16_bits_to_float(v.x & 0xffffu), f16_bits_to_float(v.x >> 16),
                               f16_bits_to_float(v.y & 0xffffu), f16_bits_to_float(v.y >> 16));
        else
            return make_float4(bf16_bits_to_float(v.x & 0xffffu), bf16_bits_to_float(v.x >> 16),
                               bf16_bits_to_float(v.y & 0xffffu), bf16_bits_to_float(v.y >> 16));
    }
}

template <unsigned WAVES, unsigned QT = QT_F32>
__global__ __launch_bounds__(WAVES * 64) void matvec_f32_tile16_kernel(MatvecArgs a)
{
    typedef double v4d __attribute__((ext_vector_type(4)));
    __shared__ double partial[WAVES - 1u][4][64];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned i16 = lane & 15u, q = lane >> 4;
    unsigned long long wrow = (unsigned long long)blockIdx.x * 16ull + i16;
    unsigned long long in = (unsigned long long)blockIdx.y * 16ull + i16;
    if (wrow >= a.row_count) wrow = a.row_count - 1ull;      // a ragged edge repeats the last row
    if (in >= a.input_rows) in = a.input_rows - 1ull;
    const unsigned long long share = a.row_width / ((unsigned long long)gridDim.z * WAVES);   // a multiple of 16
    const unsigned long long begin = ((unsigned long long)blockIdx.z * WAVES + wave) * share + 4u * q;
    const unsigned char *wp = a.encoded + wrow * a.row_bytes;       // columns from `begin` on
    const float *xp = (const float *)a.input + in * a.input_stride + begin;
    const unsigned steps = (unsigned)(share / 16ull);
    v4d acc = {0.0, 0.0, 0.0, 0.0};
    unsigned bad = 0u;
    // four steps of loads stay in flight ahead of the matrix instructions that use them
    const unsigned groups = (steps + 3u) / 4u;
    float4 w[4], x[4];
#pragma unroll
    for (unsigned j = 0; j < 4u; ++j) {
        const unsigned at = 16u * (j < steps ? j : steps - 1u);
        w[j] = scalar_weights4<QT>(wp, begin + at);
        x[j] = *reinterpret_cast<const float4 *>(xp + at);
    }
    for (unsigned group = 0; group < groups; ++group) {
        float4 wn[4], xn[4];
        if (group + 1u < groups) {
#pragma unroll
            for (unsigned j = 0; j < 4u; ++j) {
                const unsigned step = 4u * (group + 1u) + j;
                const unsigned at = 16u * (step < steps ? step : steps - 1u);
                wn[j] = scalar_weights4<QT>(wp, begin + at);
                xn[j] = *reinterpret_cast<const float4 *>(xp + at);
            }
        }
#pragma unroll
        for (unsigned j = 0; j < 4u; ++j) {
            if (4u * group + j >= steps) break;
            bad |= (unsigned)!finite_f32(w[j].x) | (unsigned)!finite_f32(w[j].y) |
                   (unsigned)!finite_f32(w[j].z) | (unsigned)!finite_f32(w[j].w);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[j].x, (double)x[j].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[j].y, (double)x[j].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[j].z, (double)x[j].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[j].w, (double)x[j].w, acc, 0, 0, 0);
        }
#pragma unroll
        for (unsigned j = 0; j < 4u; ++j) {
            w[j] = wn[j];
            x[j] = xn[j];
        }
    }
    if (bad) raise_status(a.status, 1);
    if (wave) {
#pragma unroll
        for (int k = 0; k < 4; ++k) partial[wave - 1u][k][lane] = acc[k];
    }
    __syncthreads();
    if (wave) return;
    const unsigned long long out_in = (unsigned long long)blockIdx.y * 16ull + i16;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        // accumulator k of lane (i, q): weight row 4 k + q, input row i
        const unsigned long long row = (unsigned long long)blockIdx.x * 16ull + 4u * k + q;
        double sum = acc[k];
#pragma unroll
        for (unsigned wv = 0; wv + 1u < WAVES; ++wv) sum += partial[wv][k][lane];
        if (row >= a.row_count || out_in >= a.input_rows) continue;
        if (a.parts) {
            a.parts[((unsigned long long)blockIdx.z * a.input_rows + out_in) * a.row_count + row] = sum;
            continue;
        }
        matvec_publish(a, out_in, row, (float)sum);
    }
}

// The same product for a batch of 256 input rows or more (the router projection of a prefill
// batch): with one 16 x 16 tile a workgroup every wave loads its own operands, four bytes for
// every matrix-core flop, and the launch runs at what the caches deliver (33 TFLOP/s where the
// instruction alone sustains 75). Here a workgroup of eight waves (two a SIMD, so that one
// multiplies while the other waits) owns 32 weight rows x 64 input rows and stages 128 columns
// of both in LDS (a 528-byte pitch keeps the sixteen rows that one 16-byte read phase touches
// on sixteen different bank groups), the next chunk's loads in flight while the current one is
// multiplied; wave w multiplies the 16-row half w % 2 of the weight block by input rows
// 16 (w / 2) .. + 15. Sums and rounding as above.
constexpr unsigned kF32BlockColumns = 128u, kF32BlockPitch = kF32BlockColumns * 4u + 16u;
constexpr unsigned kF32BlockWeightRows = 32u, kF32BlockInputRows = 64u;
constexpr unsigned kF32BlockLdsBytes = 2u * (kF32BlockWeightRows + kF32BlockInputRows) * kF32BlockPitch;

template <unsigned QT>
__global__ __launch_bounds__(512) void matvec_f32_block_kernel(MatvecArgs a)
{
    typedef double v4d __attribute__((ext_vector_type(4)));
    typedef float v4f __attribute__((ext_vector_type(4)));
    constexpr unsigned kRows = kF32BlockWeightRows + kF32BlockInputRows;
    constexpr unsigned kPieces = kF32BlockColumns / 4u;                   // 16-byte pieces a row
    constexpr unsigned kHeld = kRows * kPieces / 512u;
    extern __shared__ __align__(16) unsigned char staged[];               // [2][kRows * kF32BlockPitch]
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned i16 = lane & 15u, q = lane >> 4;
    // staging: piece p = threadIdx.x + 512 j of the chunk is columns 4 (p % 32) .. + 3 of staged
    // row p / 32 (weight rows first, then input rows); 32 lanes read one row's 512 bytes
    const unsigned char *source[kHeld];       // (weight rows: F32, F16 or BF16 values; input rows: F32)
    unsigned target[kHeld];
#pragma unroll
    for (unsigned j = 0; j < kHeld; ++j) {
        const unsigned p = threadIdx.x + 512u * j, row = p / kPieces, piece = p % kPieces;
        if (row < kF32BlockWeightRows) {
            unsigned long long wrow = (unsigned long long)blockIdx.x * kF32BlockWeightRows + row;
            if (wrow >= a.row_count) wrow = a.row_count - 1ull;          // a ragged edge repeats the last row
            source[j] = a.encoded + wrow * a.row_bytes;       // (a weight row: columns from 4 * piece on)
        } else {
            unsigned long long in = (unsigned long long)blockIdx.y * kF32BlockInputRows + (row - kF32BlockWeightRows);
            if (in >= a.input_rows) in = a.input_rows - 1ull;
            source[j] = (const unsigned char *)((const float *)a.input + in * a.input_stride + 4u * piece);
        }
        target[j] = row * kF32BlockPitch + 16u * piece;
    }
    const unsigned chunks = (unsigned)(a.row_width / kF32BlockColumns);
    v4f held[kHeld];
    unsigned bad = 0u;
    // piece j of this thread is a piece of a weight row for the first two j, of an input row after
    auto fetch = [&](unsigned j, unsigned chunk) -> v4f {
        if (512u * (j + 1u) <= kF32BlockWeightRows * kPieces) {
            const unsigned piece = (threadIdx.x + 512u * j) % kPieces;
            const float4 w = scalar_weights4<QT>(source[j], (unsigned long long)chunk * kF32BlockColumns + 4u * piece);
            return v4f{w.x, w.y, w.z, w.w};
        }
        return *reinterpret_cast<const v4f *>(source[j] + (unsigned long long)chunk * kF32BlockColumns * 4ull);
    };
#pragma unroll
    for (unsigned j = 0; j < kHeld; ++j) held[j] = fetch(j, 0u);
#pragma unroll
    for (unsigned j = 0; j < kHeld; ++j) {
        if (512u * (j + 1u) <= kF32BlockWeightRows * kPieces)
            bad |= (unsigned)!finite_f32(held[j][0]) | (unsigned)!finite_f32(held[j][1]) |
                   (unsigned)!finite_f32(held[j][2]) | (unsigned)!finite_f32(held[j][3]);
        *reinterpret_cast<v4f *>(&staged[target[j]]) = held[j];
    }
    __syncthreads();
    v4d acc = {0.0, 0.0, 0.0, 0.0};
    const unsigned weight_at = (16u * (wave & 1u) + i16) * kF32BlockPitch + 16u * q;
    const unsigned input_at = (kF32BlockWeightRows + 16u * (wave >> 1) + i16) * kF32BlockPitch + 16u * q;
    for (unsigned chunk = 0; chunk < chunks; ++chunk) {
        // (the last turn asks for its own chunk again and stages it where nobody reads it: no
        // branch around the loads, whose registers would otherwise be kept in scratch memory)
        const unsigned ahead = chunk + 1u < chunks ? chunk + 1u : chunk;
#pragma unroll
        for (unsigned j = 0; j < kHeld; ++j)
            held[j] = fetch(j, ahead);
        const unsigned char *now = staged + (chunk & 1u) * (kRows * kF32BlockPitch);
        unsigned char *next = staged + ((chunk + 1u) & 1u) * (kRows * kF32BlockPitch);
#pragma unroll
        for (unsigned step = 0; step < kF32BlockColumns / 16u; ++step) {
            if (step == kF32BlockColumns / 32u) {
                // half way: the loads have had four steps to arrive, and the stores have four
                // more to land before the barrier
#pragma unroll
                for (unsigned j = 0; j < kHeld; ++j) {
                    // (the weight rows are the first pieces: a non-finite weight is reported by
                    // the thread that stages it, once, not by the sixteen lanes that multiply it)
                    if (512u * (j + 1u) <= kF32BlockWeightRows * kPieces)
                        bad |= (unsigned)!finite_f32(held[j][0]) | (unsigned)!finite_f32(held[j][1]) |
                               (unsigned)!finite_f32(held[j][2]) | (unsigned)!finite_f32(held[j][3]);
                    *reinterpret_cast<v4f *>(next + target[j]) = held[j];
                }
            }
            const v4f x = *reinterpret_cast<const v4f *>(now + input_at + 64u * step);
            const v4f w = *reinterpret_cast<const v4f *>(now + weight_at + 64u * step);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[0], (double)x[0], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[1], (double)x[1], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[2], (double)x[2], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f64_16x16x4f64((double)w[3], (double)x[3], acc, 0, 0, 0);
        }
        // the next chunk is complete, and nobody reads this one any more when it is overwritten
        __syncthreads();
    }
    if (bad) raise_status(a.status, 1);
    const unsigned long long in = (unsigned long long)blockIdx.y * kF32BlockInputRows + 16u * (wave >> 1) + i16;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        // accumulator k of lane (i, q): weight row 4 k + q of the tile, input row i
        const unsigned long long row = (unsigned long long)blockIdx.x * kF32BlockWeightRows + 16u * (wave & 1u) + 4u * k + q;
        if (row < a.row_count && in < a.input_rows) matvec_publish(a, in, row, (float)acc[k]);
    }
}

// Second launch of a split projection: the partial sums of one output added in split order.
__global__ __launch_bounds__(256) void matvec_f32_join_kernel(MatvecArgs a, unsigned splits)
{
    const unsigned long long outputs = a.input_rows * a.row_count;
    const unsigned long long at = (unsigned long long)blockIdx.x * 256ull + threadIdx.x;
    if (at >= outputs) return;
    const unsigned long long in = at / a.row_count, row = at % a.row_count;
    double sum = a.parts[at];
    for (unsigned z = 1; z < splits; ++z) sum += a.parts[z * outputs + at];
    matvec_publish(a, in, row, (float)sum);
    if (a.scores) {
        // the router's score of this logit: the routing launch behind this one then has no
        // double-precision exponentials left in its one workgroup
        const double s = route_score((double)(float)sum, a.scoring);
        const float published = (float)s;
        if (!(s == s) || !finite_f32(published)) raise_status(a.status, 1);
        a.scores[in * a.row_count + row] = published;
    }
}

// int32 block sums of the Q8_K path, produced by the same unit code the matvec runs.
template <unsigned QT>
__global__ __launch_bounds__(256) void block_dots_kernel(
    const unsigned char *encoded, unsigned long long row_count, unsigned long long row_width,
    unsigned long long row_bytes, const unsigned char *input, unsigned long long input_rows,
    int *sums)
{
    __shared__ Iq2Tables tables;
    if constexpr (QT == QT_IQ2_XXS) {
        iq2_tables_fill(tables);
        __syncthreads();
    }
    const unsigned lane = threadIdx.x & 63u;
    const unsigned long long row = (unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6);
    const unsigned long long in = blockIdx.y;
    if (row >= row_count || in >= input_rows) return;
    const unsigned char *wrow = encoded + row * row_bytes;
    const unsigned units = (unsigned)(row_width >> 5);
    const unsigned long long blocks = row_width >> 8;
    for (unsigned base = 0; base < units; base += 64u) {
        const unsigned u = base + lane;
        const bool live = u < units;
        const unsigned uu = live ? u : units - 1u;
        Unit unit;
        unit_load<QT>(tables, wrow, uu, unit);
        const unsigned char *act = input + (in * blocks + (uu >> 3)) * kQ8KBytes;
        UnitSum s = unit_dot_q8<QT>(unit, act, uu & 7u);
        if constexpr (UnitTraits<QT>::kIntegerCombine) {
            if (!live) s.dot = s.min = 0;
            s.dot = group_sum_i32<8>(s.dot);
            s.min = group_sum_i32<8>(s.min);
            if (live && (uu & 7u) == 0u) {
                int *o = sums + ((in * row_count + row) * blocks + (uu >> 3)) * 2ull;
                o[0] = s.dot;
                o[1] = s.min;
            }
        } else if (live) {
            sums[(in * row_count + row) * blocks * 8ull + uu] = s.dot;
        }
    }
}

// Serial double-precision row dot by one thread, element by element: the parity probe of the
// qtype decoders (src/backend/cuda/kernels.cu:112-124). Same order and arithmetic as the CPU row
// dot, so the two agree to the last bit wherever the decoders do.
__global__ void row_dot_serial_kernel(const unsigned char *__restrict__ encoded,
                                      const float *__restrict__ vector, unsigned long long elements,
                                      unsigned qtype, float *out)
{
    if (blockIdx.x != 0u || threadIdx.x != 0u) return;
    double sum = 0.0;
    for (unsigned long long index = 0; index < elements; ++index)
        sum += (double)qtype_value(encoded, index, qtype) * (double)vector[index];
    out[0] = (float)sum;
}

__global__ __launch_bounds__(256) void gather_kernel(
    const unsigned char *encoded, unsigned qtype, unsigned long long row_count,
    unsigned long long row_width, unsigned long long row_bytes, const unsigned *row_ids,
    unsigned long long selected, float *out, int *status)
{
    const unsigned long long index = (unsigned long long)blockIdx.x * 256ull + threadIdx.x;
    if (index >= selected * row_width) return;
    const unsigned long long s = index / row_width, column = index % row_width;
    const unsigned long long row = row_ids ? row_ids[s] : s;
    if (row >= row_count) {
        raise_status(status, 2);
        return;
    }
    const float value = qtype_value(encoded + row * row_bytes, column, qtype);
    if (!finite_f32(value)) raise_status(status, 1);
    else out[index] = value;
}

template <unsigned QT, bool Q8, bool EVEN>
static int launch_block_even(const MatvecArgs &a, hipStream_t stream)
{
    const unsigned long long grid_x = (a.row_count + 3ull) / 4ull;
    if (grid_x > 0x7fffffffull) return ST_BOUNDS;
    if (a.input_rows == 1ull) {
        // Q8_K activations: four chunks (8192 columns) in flight for a matrix that takes many
        // rounds of waves, and for rows of more than one chunk, whose chunks would otherwise each
        // wait a memory round trip of their own
        const bool deep = Q8 && (a.row_count * a.row_bytes >= (64ull << 20) || a.row_width > 2048ull);
        // one F32 input row of up to 12 288 values (48 KB) is staged in LDS
        const bool stage = !Q8 && a.row_width <= 12288ull && !((uintptr_t)a.input & 15u);
        if (deep) matvec_block_kernel<QT, Q8, 1, Q8 ? 4 : 1, EVEN><<<dim3((unsigned)grid_x, 1), 256, 0, stream>>>(a);
        else if (stage)
            matvec_block_kernel<QT, Q8, 1, 1, EVEN, !Q8><<<dim3((unsigned)grid_x, 1), 256,
                                                            (size_t)a.row_width * 4u, stream>>>(a);
        else matvec_block_kernel<QT, Q8, 1, 1, EVEN><<<dim3((unsigned)grid_x, 1), 256, 0, stream>>>(a);
    } else {
        const unsigned long long grid_y = (a.input_rows + 3ull) / 4ull;
        if (grid_y > 65535ull) return ST_BOUNDS;
        matvec_block_kernel<QT, Q8, 4, 1, EVEN><<<dim3((unsigned)grid_x, (unsigned)grid_y), 256, 0, stream>>>(a);
    }
    return check_launch("matvec");
}

template <unsigned QT, int L>
static int launch_dense_row(const MatvecArgs &a, hipStream_t stream)
{
    const unsigned long long grid = (a.row_count + 4ull * (64u / L) - 1ull) / (4ull * (64u / L));
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    dense_row_q8k_kernel<QT, L><<<(unsigned)grid, 256, 0, stream>>>(a);
    return check_launch("matvec.row");
}

// One Q8_K input row against superblock-format rows on dword boundaries: the row kernel, whatever
// the size of the matrix (a 470 MB Q4_K matrix streams at 4.8 TB/s through it, at 2.4 TB/s
// through the general kernel, whose lanes wait for the superblock header on their own).
template <unsigned QT>
static bool dense_row_applies(const MatvecArgs &a)
{
    return UnitTraits<QT>::kIntegerCombine && a.input_rows == 1ull &&
           !((unsigned long long)a.encoded & 3ull) && !(a.row_bytes & 3ull);
}

template <unsigned QT, int L>
static int launch_dense_fewrows(const MatvecArgs &a, hipStream_t stream)
{
    const unsigned long long grid = (a.row_count + 4ull * (64u / L) - 1ull) / (4ull * (64u / L));
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    dense_fewrows_q8k_kernel<QT, L><<<(unsigned)grid, 256, 0, stream>>>(a);
    return check_launch("matvec.fewrows");
}

template <unsigned QT>
static bool dense_fewrows_applies(const MatvecArgs &a)
{
    // (measured against the general kernel on 2048 x 7168 and 7168 x 2048 matrices: ahead up to
    // a dozen input rows, and at any number below 32 where a row is 2048 columns or fewer)
    return UnitTraits<QT>::kIntegerCombine && a.input_rows >= 2ull && a.input_rows < 32ull &&
           (a.input_rows <= 12ull || a.row_width <= 2048ull) &&
           a.row_width <= 8192ull && a.row_count * a.row_bytes < (64ull << 20) &&
           !((unsigned long long)a.encoded & 3ull) && !(a.row_bytes & 3ull);
}

template <unsigned QT>
static int launch_dense_fewrows_width(const MatvecArgs &a, hipStream_t stream)
{
    const unsigned long long halves = a.row_width >> 7;
    if (halves <= 8ull) return launch_dense_fewrows<QT, 8>(a, stream);
    if (halves <= 16ull) return launch_dense_fewrows<QT, 16>(a, stream);
    if (halves <= 32ull) return launch_dense_fewrows<QT, 32>(a, stream);
    return launch_dense_fewrows<QT, 64>(a, stream);
}

template <unsigned QT>
static int launch_dense_row_width(const MatvecArgs &a, hipStream_t stream)
{
    const unsigned long long halves = a.row_width >> 7;
    if (halves <= 8ull) return launch_dense_row<QT, 8>(a, stream);
    if (halves <= 16ull) return launch_dense_row<QT, 16>(a, stream);
    if (halves <= 32ull) return launch_dense_row<QT, 32>(a, stream);
    return launch_dense_row<QT, 64>(a, stream);
}

template <unsigned QT, bool Q8>
static int launch_block(const MatvecArgs &a, hipStream_t stream)
{
    if constexpr (Q8 && UnitTraits<QT>::kIntegerCombine) {
        if (dense_row_applies<QT>(a)) return launch_dense_row_width<QT>(a, stream);
        if (dense_fewrows_applies<QT>(a)) return launch_dense_fewrows_width<QT>(a, stream);
    }
    const bool even = (((unsigned long long)a.encoded | a.row_bytes) & 1ull) == 0ull;
    return even ? launch_block_even<QT, Q8, true>(a, stream) : launch_block_even<QT, Q8, false>(a, stream);
}

template <unsigned QT>
static int launch_block_q(const MatvecArgs &a, bool q8, hipStream_t stream)
{
    return q8 ? launch_block<QT, true>(a, stream) : launch_block<QT, false>(a, stream);
}

}  // namespace yvex

using namespace yvex;

// Rows of F32, F16 or BF16 values against eight or more F32 input rows: 16 x 16 tiles on the
// double-precision matrix cores; a small batch offers few tiles, so sixteen waves split the row
// width, a large one has tiles enough for four, or for the staged kernel.
template <unsigned QT>
static int launch_scalar_rows(const MatvecArgs &a, hipStream_t s)
{
    const unsigned long long grid_x = (a.row_count + 15ull) / 16ull, grid_y = (a.input_rows + 15ull) / 16ull;
    if (grid_x > 0x7fffffffull || grid_y > 65535ull) return ST_BOUNDS;
    if (a.input_rows < 256ull) {
        matvec_f32_tile16_kernel<16, QT><<<dim3((unsigned)grid_x, (unsigned)grid_y), 1024, 0, s>>>(a);
    } else if (a.row_width % kF32BlockColumns == 0ull &&
               (a.row_count + kF32BlockWeightRows - 1ull) / kF32BlockWeightRows *
                   ((a.input_rows + kF32BlockInputRows - 1ull) / kF32BlockInputRows) >= 3ull * compute_units() / 4ull) {
        // (a block a compute unit or close to it: the staged kernel walks the row width
        // chunk by chunk, 3 us each, and is behind the small tiles on a grid that leaves
        // most of the device idle: 161 us against 46 us for 256 rows by 256)
        const unsigned long long block_y = (a.input_rows + kF32BlockInputRows - 1ull) / kF32BlockInputRows;
        if (block_y > 65535ull) return ST_BOUNDS;
        YVEX_ALLOW_DYNAMIC_LDS(matvec_f32_block_kernel<QT>, kF32BlockLdsBytes);
        matvec_f32_block_kernel<QT><<<dim3((unsigned)((a.row_count + kF32BlockWeightRows - 1ull) / kF32BlockWeightRows),
                                       (unsigned)block_y), 512, kF32BlockLdsBytes, s>>>(a);
    } else {
        matvec_f32_tile16_kernel<4, QT><<<dim3((unsigned)grid_x, (unsigned)grid_y), 256, 0, s>>>(a);
    }
    return check_launch("matvec_f32_tile16");
}

extern "C" int yvex_hip_matvec(const uint8_t *encoded, unsigned int qtype, uint64_t row_count,
                               uint64_t row_width, uint64_t row_bytes, const void *input,
                               int input_q8, uint64_t input_rows, uint64_t input_stride,
                               const float *additive, float *out, uint64_t out_stride,
                               int output_bf16, int *status, yvex_hip_stream stream)
{
    unsigned block, bytes;
    if (!encoded || !input || !out || !status || !row_count || !row_width || !input_rows ||
        out_stride < row_count || (input_q8 != 0 && input_q8 != 1))
        return ST_INVALID_ARG;
    if (!qtype_geometry(qtype, block, bytes)) return ST_UNSUPPORTED;
    if (row_width % block || row_width / block * bytes != row_bytes) return ST_BOUNDS;
    if (row_width > 0xffffffffull * 32ull) return ST_BOUNDS;
    if (((uintptr_t)input & 3u) || ((uintptr_t)out & 3u)) return ST_INVALID_ARG;
    MatvecArgs a{encoded, row_count, row_width, row_bytes, input, input_rows, input_stride,
                 additive, out, out_stride, output_bf16, status, nullptr, nullptr, 0};
    hipStream_t s = as_stream(stream);
    const bool scalar = qtype == QT_F32 || qtype == QT_F16 || qtype == QT_BF16 || qtype == QT_I32;
    if (input_q8 && (scalar || row_width % 256u)) return ST_UNSUPPORTED;
    if (!input_q8) {
        if (input_stride < row_width) return ST_INVALID_ARG;
        if (!scalar && (((uintptr_t)input & 15u) || (input_stride & 3u))) return ST_INVALID_ARG;
    }
    // IQ2_XXS rows against a batch of Q8_K input rows: the int8 matrix-core kernel of the
    // row-batch expert path, as one bucket that holds every input row (the reference turns its
    // tensor-core kernels on from 16 input rows, src/backend/cuda/private.h:461-464; measured
    // here the sweep below stays faster up to 31 rows: 17 us against 22 us for 7168 x 2048 at 16). Same exact
    // int32 superblock sums and the same float terms as the sweep below, added in double in
    // superblock order there and here: the same bits.
    if (qtype == QT_IQ2_XXS && input_q8 && input_rows >= 32ull && !additive &&
        out_stride == row_count && row_count % 4ull == 0ull && !((uintptr_t)encoded & 3u) &&
        !(row_bytes & 3ull) && row_width / 32ull <= 64ull * 4ull && !((uintptr_t)out & 15u))
        return launch_iq2_rows_dense(encoded, row_count, row_width, row_bytes, input, input_rows, out,
                                     output_bf16 != 0, status, s);
    // Q4_K rows against two or more Q8_K input rows: matrix cores (the reference's threshold is 16
    // input rows; here the 16-token tiles beat the general kernel below from two rows on, 10.5 us
    // against 12.2 us at 2 and 19.7 us at 15 rows for 2048 x 7168; the few-rows kernel, where it
    // applies, is ahead of both at two and three rows: 6.0 and 7.1 us against 8.6)
    if (qtype == QT_Q4_K && input_q8 && input_rows >= 2ull && !((uintptr_t)encoded & 15u) &&
        !(input_rows < 4ull && dense_fewrows_applies<QT_Q4_K>(a)))
        return launch_q4k_rows_dense(encoded, row_count, row_width, row_bytes, input, input_rows, additive,
                                     out, out_stride, output_bf16 != 0, status, s);
    // Q8_0 rows against a batch of Q8_K input rows: matrix cores from the reference's threshold on
    // (src/backend/cuda/private.h:461-464); below it the lane-strided kernel, which reads the
    // matrix once per input row: fine while the matrix stays in the caches (4096 x 4096, 18 MB:
    // 10 us up to four rows, 12.5 at eight, 19 at fifteen; the matrix cores 13.5 us throughout),
    // but 7168 x 7168 (55 MB) takes 15 us for one row, 21 for two and 66 for fifteen where the
    // matrix cores take 18.5, and an output head of 129 280 x 7168 171 us for one row, 336 for two
    // and 1.5 ms for fifteen where they take 200 to 235
    const unsigned long long matrix_bytes = row_count * row_bytes;
    if (qtype == QT_Q8_0 && input_q8 && !((uintptr_t)encoded & 3u) &&
        (input_rows >= 16ull || (input_rows >= 2ull && matrix_bytes >= (32ull << 20)) ||
         (input_rows >= 12ull && matrix_bytes >= (8ull << 20))))
        return launch_q8_0_rows_dense(encoded, row_count, row_width, row_bytes, input, input_rows, additive, out,
                                      out_stride, output_bf16 != 0, status, s);
    // F32 rows against a batch of F32 input rows: the double-precision matrix cores; rows of F16
    // and BF16 values take the same kernels (the conversion to double is exact for them as well),
    // and so do Q8_0 rows against F32 input rows (a caller that switched the Q8 activation policy
    // off: the decoded weight, scale times code, is exact in float; 4096 x 4096 by 2048 rows 20.9 ms
    // on the lane-strided kernel)
    if ((qtype == QT_F32 || qtype == QT_F16 || qtype == QT_BF16 || (qtype == QT_Q8_0 && !input_q8)) &&
        input_rows >= 8ull && !(((uintptr_t)encoded | (uintptr_t)input) & 15u) && !(input_stride & 3ull) &&
        row_width % (input_rows < 256ull ? 256ull : 64ull) == 0ull)
        return qtype == QT_F32 ? launch_scalar_rows<QT_F32>(a, s)
             : qtype == QT_F16 ? launch_scalar_rows<QT_F16>(a, s)
             : qtype == QT_BF16 ? launch_scalar_rows<QT_BF16>(a, s) : launch_scalar_rows<QT_Q8_0>(a, s);
    // (fewer than eight input rows, or a row width the matrix-core kernels do not take: 16-bit
    // rows have no other fast kernel and stay here at any number of input rows, four a workgroup)
    if (((qtype == QT_F32 && input_rows < 8ull) ||
         ((qtype == QT_F16 || qtype == QT_BF16) && (input_rows + 3ull) / 4ull <= 65535ull)) &&
        row_count <= 0x7fffffffull && !(((uintptr_t)encoded | (uintptr_t)input) & 15u) && !(input_stride & 3ull) &&
        !(row_bytes & 15ull)) {      // (whole 16-byte pieces a row: a multiple of 4 or 8 columns)
        if (qtype == QT_F32) return launch_scalar_few<QT_F32>(a, s);
        return qtype == QT_F16 ? launch_scalar_few<QT_F16>(a, s) : launch_scalar_few<QT_BF16>(a, s);
    }
    if (scalar) {
        const unsigned long long grid_x = (row_count + 3ull) / 4ull;
        if (grid_x > 0x7fffffffull) return ST_BOUNDS;
        if (input_rows == 1ull) {
            matvec_scalar_kernel<1><<<dim3((unsigned)grid_x, 1), 256, 0, s>>>(a, qtype);
        } else {
            const unsigned long long grid_y = (input_rows + 3ull) / 4ull;
            if (grid_y > 65535ull) return ST_BOUNDS;
            matvec_scalar_kernel<4><<<dim3((unsigned)grid_x, (unsigned)grid_y), 256, 0, s>>>(a, qtype);
        }
        return check_launch("matvec_scalar");
    }
    switch (qtype) {
    case QT_IQ2_XXS: return launch_block_q<QT_IQ2_XXS>(a, input_q8, s);
    case QT_Q8_0: return launch_block_q<QT_Q8_0>(a, input_q8, s);
    case QT_Q4_K: return launch_block_q<QT_Q4_K>(a, input_q8, s);
    case QT_Q2_K: return launch_block_q<QT_Q2_K>(a, input_q8, s);
    default: return ST_UNSUPPORTED;
    }
}

extern "C" int yvex_hip_block_dots_i32(const uint8_t *encoded, unsigned int qtype,
                                       uint64_t row_count, uint64_t row_width,
                                       uint64_t row_bytes, const uint8_t *input_q8,
                                       uint64_t input_rows, int32_t *sums, int *status,
                                       yvex_hip_stream stream)
{
    unsigned block, bytes;
    if (!encoded || !input_q8 || !sums || !status || !row_count || !row_width || !input_rows)
        return ST_INVALID_ARG;
    if (!qtype_geometry(qtype, block, bytes)) return ST_UNSUPPORTED;
    if (row_width % 256u || row_width / block * bytes != row_bytes) return ST_BOUNDS;
    if (((uintptr_t)input_q8 & 3u) || input_rows > 65535ull) return ST_INVALID_ARG;
    const unsigned long long grid_x = (row_count + 3ull) / 4ull;
    if (grid_x > 0x7fffffffull) return ST_BOUNDS;
    dim3 grid((unsigned)grid_x, (unsigned)input_rows);
    hipStream_t s = as_stream(stream);
    switch (qtype) {
    case QT_IQ2_XXS:
        block_dots_kernel<QT_IQ2_XXS><<<grid, 256, 0, s>>>(encoded, row_count, row_width,
                                                           row_bytes, input_q8, input_rows, sums);
        break;
    case QT_Q8_0:
        block_dots_kernel<QT_Q8_0><<<grid, 256, 0, s>>>(encoded, row_count, row_width, row_bytes,
                                                        input_q8, input_rows, sums);
        break;
    case QT_Q4_K:
        block_dots_kernel<QT_Q4_K><<<grid, 256, 0, s>>>(encoded, row_count, row_width, row_bytes,
                                                        input_q8, input_rows, sums);
        break;
    case QT_Q2_K:
        block_dots_kernel<QT_Q2_K><<<grid, 256, 0, s>>>(encoded, row_count, row_width, row_bytes,
                                                        input_q8, input_rows, sums);
        break;
    default: return ST_UNSUPPORTED;
    }
    return check_launch("block_dots");
}

extern "C" int yvex_hip_gather(const uint8_t *encoded, unsigned int qtype, uint64_t row_count,
                               uint64_t row_width, uint64_t row_bytes, const uint32_t *row_ids,
                               uint64_t selected, float *out, int *status,
                               yvex_hip_stream stream)
{
    unsigned block, bytes;
    if (!encoded || !out || !status || !row_count || !row_width || !selected) return ST_INVALID_ARG;
    if (!qtype_geometry(qtype, block, bytes)) return ST_UNSUPPORTED;
    if (row_width % block || row_width / block * bytes != row_bytes) return ST_BOUNDS;
    if (selected > UINT64_MAX / row_width) return ST_BOUNDS;
    const unsigned long long grid = (selected * row_width + 255ull) / 256ull;
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    gather_kernel<<<(unsigned)grid, 256, 0, as_stream(stream)>>>(
        encoded, qtype, row_count, row_width, row_bytes, row_ids, selected, out, status);
    return check_launch("gather");
}

extern "C" int yvex_hip_row_dot(const uint8_t *encoded, unsigned int qtype, const float *vector,
                                uint64_t elements, float *out, yvex_hip_stream stream)
{
    unsigned block, bytes;
    if (!encoded || !vector || !out || !elements) return ST_INVALID_ARG;
    if (!qtype_geometry(qtype, block, bytes)) return ST_UNSUPPORTED;
    if (elements % block) return ST_BOUNDS;
    row_dot_serial_kernel<<<1, 1, 0, as_stream(stream)>>>(encoded, vector, elements, qtype, out);
    return check_launch("row_dot");
}

// Splits of an F32 projection over a decode-width batch: per-wave shares of 128 columns. A larger
// batch against a few weight rows (the mixing projection of a prefill batch: 24 rows) is split
// too, as often as brings its 16 x 16 tiles to about two thousand.
static unsigned f32_rows_splits(uint64_t row_count, uint64_t row_width, uint64_t input_rows)
{
    if (input_rows < 8u || row_width % 128u) return 0u;
    if (input_rows >= 256u) {
        const uint64_t tiles = (row_count + 15u) / 16u * ((input_rows + 15u) / 16u);
        if (tiles >= 1024u) return 0u;
        for (unsigned splits = (unsigned)(2048u / tiles < 16u ? 2048u / tiles : 16u); splits >= 2u; --splits)
            if (row_width % (64ull * splits) == 0u) return splits;
        return 0u;
    }
    // 512 columns a split (128 a wave) where that gives 2 to 64 splits; a wider row takes the
    // most splits up to 64 that leave every wave a multiple of 16 columns
    if (row_width % 512u == 0u && row_width / 512u >= 2u && row_width / 512u <= 64u)
        return (unsigned)(row_width / 512u);
    if (row_width < 64u * 512u) return 0u;
    for (unsigned splits = 64u; splits >= 2u; --splits)
        if (row_width % (64ull * splits) == 0u) return splits;
    return 0u;
}

extern "C" uint64_t yvex_hip_matvec_f32_scratch_bytes(uint64_t row_count, uint64_t row_width,
                                                      uint64_t input_rows)
{
    const unsigned splits = f32_rows_splits(row_count, row_width, input_rows);
    return splits ? (uint64_t)splits * input_rows * row_count * sizeof(double) : 0u;
}

// Whether the projection runs as partial tiles plus a join (two launches) or as one launch.
static bool f32_rows_split_applies(const float *weights, uint64_t row_count, uint64_t row_width,
                                   const float *input, uint64_t input_rows, uint64_t input_stride,
                                   const void *scratch, uint64_t scratch_bytes)
{
    const unsigned splits = f32_rows_splits(row_count, row_width, input_rows);
    const uint64_t need = yvex_hip_matvec_f32_scratch_bytes(row_count, row_width, input_rows);
    return splits && scratch && scratch_bytes >= need && !((uintptr_t)scratch & 7u) &&
           !(((uintptr_t)weights | (uintptr_t)input) & 15u) && !(input_stride & 3ull) && weights && input &&
           row_count && input_stride >= row_width;
}

extern "C" unsigned int yvex_hip_matvec_f32_rows_launches(const float *weights, uint64_t row_count,
                                                          uint64_t row_width, const float *input,
                                                          uint64_t input_rows, uint64_t input_stride,
                                                          const void *scratch, uint64_t scratch_bytes)
{
    return f32_rows_split_applies(weights, row_count, row_width, input, input_rows, input_stride, scratch,
                                  scratch_bytes) ? 2u : 1u;
}

static int launch_f32_rows_split(const MatvecArgs &a, yvex_hip_stream stream);

extern "C" int yvex_hip_matvec_f32_rows(const float *weights, uint64_t row_count, uint64_t row_width,
                                        const float *input, uint64_t input_rows, uint64_t input_stride,
                                        const float *additive, float *out, uint64_t out_stride,
                                        int output_bf16, void *scratch, uint64_t scratch_bytes,
                                        int *status, yvex_hip_stream stream)
{
    if (!f32_rows_split_applies(weights, row_count, row_width, input, input_rows, input_stride, scratch,
                                scratch_bytes) || !out || !status || out_stride < row_count)
        return yvex_hip_matvec((const uint8_t *)weights, QT_F32, row_count, row_width, row_width * 4u, input, 0,
                               input_rows, input_stride, additive, out, out_stride, output_bf16, status,
                               stream);
    MatvecArgs a{(const unsigned char *)weights, row_count, row_width, row_width * 4u, input, input_rows,
                 input_stride, additive, out, out_stride, output_bf16, status, (double *)scratch, nullptr, 0};
    return launch_f32_rows_split(a, stream);
}

// The split projection with the router's score of every output published beside it
// (`scores`, dense [input row][weight row]): the scores are computed by the join's many
// workgroups instead of the routing launch's one. Only where the split applies (two launches,
// as yvex_hip_matvec_f32_rows_launches says); anything else is refused.
extern "C" int yvex_hip_matvec_f32_rows_scored(const float *weights, uint64_t row_count, uint64_t row_width,
                                               const float *input, uint64_t input_rows,
                                               uint64_t input_stride, float *out, uint64_t out_stride,
                                               float *scores, int scoring, void *scratch,
                                               uint64_t scratch_bytes, int *status, yvex_hip_stream stream)
{
    if (!out || !scores || !status || out_stride < row_count || (scoring != 0 && scoring != 1) ||
        ((uintptr_t)out & 3u) || ((uintptr_t)scores & 3u))
        return ST_INVALID_ARG;
    if (!f32_rows_split_applies(weights, row_count, row_width, input, input_rows, input_stride, scratch,
                                scratch_bytes))
        return ST_UNSUPPORTED;
    MatvecArgs a{(const unsigned char *)weights, row_count, row_width, row_width * 4u, input, input_rows,
                 input_stride, nullptr, out, out_stride, 0, status, (double *)scratch, scores, scoring};
    return launch_f32_rows_split(a, stream);
}

static int launch_f32_rows_split(const MatvecArgs &a, yvex_hip_stream stream)
{
    const uint64_t row_count = a.row_count, input_rows = a.input_rows;
    const unsigned splits = f32_rows_splits(row_count, a.row_width, input_rows);
    hipStream_t s = as_stream(stream);
    const uint64_t grid_x = (row_count + 15u) / 16u, grid_y = (input_rows + 15u) / 16u;
    const uint64_t outputs = input_rows * row_count;
    if (grid_x > 0x7fffffffull || grid_y > 65535ull || (outputs + 255u) / 256u > 0x7fffffffull) return ST_BOUNDS;
    matvec_f32_tile16_kernel<4><<<dim3((unsigned)grid_x, (unsigned)grid_y, splits), 256, 0, s>>>(a);
    int rc = check_launch("matvec_f32_rows.parts");
    if (rc) return rc;
    matvec_f32_join_kernel<<<(unsigned)((outputs + 255u) / 256u), 256, 0, s>>>(a, splits);
    return check_launch("matvec_f32_rows.join");
}
