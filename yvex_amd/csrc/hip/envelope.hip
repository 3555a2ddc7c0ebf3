// Residual-stream envelope around the expert math, for gfx950.
//
// A layer's input row holds `streams` residual streams of `width` values. Ingress collapses them
// into one row with sigmoid gates, builds the stream-mixing matrix (row softmax followed by
// alternating row and column normalisations), applies the weighted RMS norm and publishes bf16
// values; egress spreads the layer's output back over the streams. Behaviour restated from
// src/graph/numeric.c:630-877 (the arithmetic and its order), src/graph/moe.c:446-495 (how the
// MoE composes it) and src/backend/cuda/kernels.cu:867-910,1243-1428 (the device twins, which
// round the incoming residual to bf16 first).
//
// Both kernels are bound by reading the rows once; the gates and the mixing matrix are a few
// dozen double-precision operations per row.
#include "common.hpp"
#include "launch.hpp"

namespace yvex {

constexpr unsigned kEnvelopeThreads = 256;
constexpr unsigned kEnvelopeMaxStreams = 7;       // (streams + 2) * streams <= 64 mixing rows
constexpr unsigned kEnvelopeMaxWidth = 16384;     // the reference's bound (src/graph/moe.c:453-455)

__device__ __forceinline__ bool finite_f64(double v)
{
    return (__double_as_longlong(v) & 0x7ff0000000000000ll) != 0x7ff0000000000000ll;
}

// Sum over the workgroup, the same value in every thread: a butterfly inside each wavefront,
// then the four wavefront totals in order. The order is fixed, so a row's result does not
// depend on where it runs.
__device__ __forceinline__ double workgroup_sum(double v, double *slots)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
    if ((threadIdx.x & 63u) == 0u) slots[threadIdx.x >> 6] = v;
    __syncthreads();
    const double total = ((slots[0] + slots[1]) + slots[2]) + slots[3];
    __syncthreads();
    return total;
}

__device__ __forceinline__ double sigmoid_f64(double value)
{
    if (value >= 0.0) return 1.0 / (1.0 + exp(-value));
    const double direct = exp(value);
    return direct / (1.0 + direct);
}

// One workgroup per row.
__global__ __launch_bounds__(kEnvelopeThreads) void mhc_ingress_kernel(
    const float *__restrict__ rows, const float *__restrict__ mixes, const float *__restrict__ scale,
    const float *__restrict__ base, const float *__restrict__ norm, unsigned streams, unsigned width,
    unsigned iterations, double rms_epsilon, double mhc_epsilon, double post_multiplier,
    float *__restrict__ normalized, float *__restrict__ post, float *__restrict__ combination,
    int *status)
{
    extern __shared__ __align__(16) float collapsed[];   // width values
    __shared__ double slots[4];
    __shared__ double gate[8];
    __shared__ float mixing[64];
    const unsigned tid = threadIdx.x;
    const unsigned long long row = blockIdx.x;
    const unsigned expanded = streams * width, mixing_rows = (streams + 2u) * streams;
    const float *in = rows + row * expanded;
    const float *mix = mixes + row * mixing_rows;
    bool bad = false;

    // mean square of the bf16-rounded residual
    double squares = 0.0;
    for (unsigned lane = tid; lane < expanded; lane += kEnvelopeThreads) {
        const float v = bf16_round(in[lane]);
        bad |= !finite_f32(v);
        squares += (double)v * (double)v;
    }
    if (tid < mixing_rows) bad |= !finite_f32(base[tid]) || !finite_f32(mix[tid]);
    if (tid < 3u) bad |= !finite_f32(scale[tid]);
    const double inverse = 1.0 / sqrt(workgroup_sum(squares, slots) / (double)expanded + rms_epsilon);
    bad |= !finite_f64(inverse);

    if (tid < streams) {
        const double pre = sigmoid_f64((double)mix[tid] * inverse * (double)scale[0] + (double)base[tid]);
        gate[tid] = pre + mhc_epsilon;
        post[row * streams + tid] = (float)(post_multiplier * sigmoid_f64(
            (double)mix[streams + tid] * inverse * (double)scale[1] + (double)base[streams + tid]));
        for (unsigned target = 0; target < streams; ++target) {
            const unsigned index = 2u * streams + tid * streams + target;
            mixing[tid * streams + target] =
                (float)((double)mix[index] * inverse * (double)scale[2] + (double)base[index]);
        }
    }
    __syncthreads();

    // collapsed row: float accumulation over the streams in order, then bf16
    double collapsed_squares = 0.0;
    for (unsigned lane = tid; lane < width; lane += kEnvelopeThreads) {
        float total = 0.0f;
        for (unsigned s = 0; s < streams; ++s)
            total += (float)(gate[s] * (double)bf16_round(in[s * width + lane]));
        bad |= !finite_f32(total);
        const float published = bf16_round(total);
        collapsed[lane] = published;
        collapsed_squares += (double)published * (double)published;
    }

    // mixing matrix: one thread per element; every thread of the row (or column) forms the same
    // total in the same order, then all write after a barrier
    const unsigned cells = streams * streams;
    const bool cell = tid < cells;
    const unsigned r = cell ? tid / streams : 0u, c = cell ? tid % streams : 0u;
    {
        double maximum = -__builtin_inf(), total = 0.0, mine = 0.0;
        for (unsigned k = 0; k < streams; ++k) maximum = fmax(maximum, (double)mixing[r * streams + k]);
        for (unsigned k = 0; k < streams; ++k) {
            const double value = exp((double)mixing[r * streams + k] - maximum);
            total += value;
            if (k == c) mine = value;
        }
        __syncthreads();
        if (cell) {
            bad |= !finite_f64(total) || !(total > 0.0);
            mixing[tid] = (float)((double)(float)mine / total + mhc_epsilon);
        }
        __syncthreads();
    }
    for (unsigned it = 0; it < iterations; ++it) {
        if (it != 0u) {
            double total = 0.0;
            for (unsigned k = 0; k < streams; ++k) total += (double)mixing[r * streams + k];
            __syncthreads();
            if (cell) {
                bad |= !finite_f64(total);
                mixing[tid] = (float)((double)mixing[tid] / (total + mhc_epsilon));
            }
            __syncthreads();
        }
        double total = 0.0;
        for (unsigned k = 0; k < streams; ++k) total += (double)mixing[k * streams + c];
        __syncthreads();
        if (cell) {
            bad |= !finite_f64(total);
            mixing[tid] = (float)((double)mixing[tid] / (total + mhc_epsilon));
        }
        __syncthreads();
    }
    if (cell) combination[row * cells + tid] = mixing[tid];

    // weighted RMS norm of the collapsed row, published as bf16
    const double mean = workgroup_sum(collapsed_squares, slots) / (double)width;
    const double norm_inverse = 1.0 / sqrt(mean + rms_epsilon);
    bad |= !finite_f64(norm_inverse);
    for (unsigned lane = tid; lane < width; lane += kEnvelopeThreads) {
        const float weight = norm[lane];
        double v = (double)collapsed[lane] * norm_inverse;
        v *= (double)weight;
        const float value = (float)v;
        bad |= !finite_f32(weight) || !finite_f64(v) || !finite_f32(value);
        normalized[row * width + lane] = bf16_round(value);
    }
    if (bad) raise_status(status, 1);
}

// One thread per (row, lane): the lane's value in every stream is read once and every target
// stream's output is formed from it.
__global__ __launch_bounds__(kEnvelopeThreads) void mhc_egress_kernel(
    const float *__restrict__ core, const float *__restrict__ rows, const float *__restrict__ post,
    const float *__restrict__ combination, unsigned long long row_count, unsigned streams,
    unsigned width, unsigned blocks_per_row, float *__restrict__ output, int *status)
{
    const unsigned long long row = blockIdx.x / blocks_per_row;
    const unsigned lane = (blockIdx.x % blocks_per_row) * kEnvelopeThreads + threadIdx.x;
    if (row >= row_count || lane >= width) return;
    const unsigned expanded = streams * width;
    const float *in = rows + row * expanded;
    const float *mixing = combination + row * streams * streams;
    const double value = (double)core[row * width + lane];
    double residual[kEnvelopeMaxStreams];
#pragma unroll
    for (unsigned s = 0; s < kEnvelopeMaxStreams; ++s)
        residual[s] = s < streams ? (double)bf16_round(in[s * width + lane]) : 0.0;
    bool bad = false;
    for (unsigned target = 0; target < streams; ++target) {
        double total = (double)post[row * streams + target] * value;
#pragma unroll
        for (unsigned s = 0; s < kEnvelopeMaxStreams; ++s)
            if (s < streams) total += (double)mixing[s * streams + target] * residual[s];
        const float published = (float)total;
        bad |= !finite_f64(total) || !finite_f32(published);
        output[row * expanded + target * width + lane] = bf16_round(published);
    }
    if (bad) raise_status(status, 1);
}

}  // namespace yvex

using namespace yvex;

static bool envelope_shape_ok(uint64_t row_count, uint64_t streams, uint64_t width)
{
    return row_count && streams && streams <= kEnvelopeMaxStreams && width && width <= kEnvelopeMaxWidth &&
           row_count <= 0x7fffffffull / ((width + kEnvelopeThreads - 1u) / kEnvelopeThreads);
}

extern "C" int yvex_hip_mhc_ingress(const float *rows, const float *mixes, const float *scale,
                                    const float *base, const float *norm, uint64_t row_count,
                                    uint64_t streams, uint64_t width, uint64_t iterations,
                                    double rms_epsilon, double mhc_epsilon, double post_multiplier,
                                    float *normalized, float *post, float *combination, int *status,
                                    yvex_hip_stream stream)
{
    if (!rows || !mixes || !scale || !base || !norm || !normalized || !post || !combination || !status)
        return ST_INVALID_ARG;
    if (!envelope_shape_ok(row_count, streams, width) || !iterations || iterations > 0xffffffffull)
        return ST_BOUNDS;
    if (!(rms_epsilon > 0.0) || !(mhc_epsilon > 0.0) || !(post_multiplier > 0.0) ||
        rms_epsilon > 1.0e300 || mhc_epsilon > 1.0e300 || post_multiplier > 1.0e300)
        return ST_INVALID_ARG;
    static bool prepared = false;
    if (!prepared) {
        if (hipFuncSetAttribute((const void *)mhc_ingress_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)(kEnvelopeMaxWidth * sizeof(float))) != hipSuccess) {
            set_last_error_text("mhc_ingress: the collapsed row does not fit in LDS");
            return ST_BACKEND;
        }
        prepared = true;
    }
    mhc_ingress_kernel<<<(unsigned)row_count, kEnvelopeThreads, (unsigned)(width * sizeof(float)),
                         as_stream(stream)>>>(
        rows, mixes, scale, base, norm, (unsigned)streams, (unsigned)width, (unsigned)iterations,
        rms_epsilon, mhc_epsilon, post_multiplier, normalized, post, combination, status);
    return check_launch("mhc_ingress");
}

extern "C" int yvex_hip_mhc_egress(const float *core, const float *rows, const float *post,
                                   const float *combination, uint64_t row_count, uint64_t streams,
                                   uint64_t width, float *output, int *status, yvex_hip_stream stream)
{
    if (!core || !rows || !post || !combination || !output || !status || output == rows)
        return ST_INVALID_ARG;
    if (!envelope_shape_ok(row_count, streams, width)) return ST_BOUNDS;
    const unsigned blocks_per_row = (unsigned)((width + kEnvelopeThreads - 1u) / kEnvelopeThreads);
    mhc_egress_kernel<<<(unsigned)(row_count * blocks_per_row), kEnvelopeThreads, 0, as_stream(stream)>>>(
        core, rows, post, combination, row_count, (unsigned)streams, (unsigned)width, blocks_per_row,
        output, status);
    return check_launch("mhc_egress");
}
