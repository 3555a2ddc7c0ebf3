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
#include <type_traits>

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
// then the wavefront totals in order. The order is fixed, so a row's result does not depend on
// where it runs.
template <unsigned WAVES>
__device__ __forceinline__ double workgroup_sum(double v, double *slots)
{
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
    if ((threadIdx.x & 63u) == 0u) slots[threadIdx.x >> 6] = v;
    __syncthreads();
    double total = slots[0];
#pragma unroll
    for (unsigned w = 1; w < WAVES; ++w) total += slots[w];
    __syncthreads();
    return total;
}

__device__ __forceinline__ double sigmoid_f64(double value)
{
    if (value >= 0.0) return 1.0 / (1.0 + exp(-value));
    const double direct = exp(value);
    return direct / (1.0 + direct);
}

__device__ __forceinline__ float4 bf16_round4(float4 v)
{
    return make_float4(bf16_round(v.x), bf16_round(v.y), bf16_round(v.z), bf16_round(v.w));
}

// A coefficient vector (scale, base, norm) as the layer stores it, F32 or BF16 values, decoded
// where they are used (the reference decodes them into F32 buffers with launches of their own,
// src/backend/cuda/moe.c:1226-1240; the decoded value is the same float).
__device__ __forceinline__ float coefficient(const void *values, unsigned qtype, unsigned index)
{
    if (qtype == QT_F32) return static_cast<const float *>(values)[index];
    return __uint_as_float((unsigned)static_cast<const unsigned short *>(values)[index] << 16);
}

// Four consecutive coefficients from a 16-byte (F32) or 8-byte (BF16) aligned address.
__device__ __forceinline__ float4 coefficient4(const void *values, unsigned qtype, unsigned quad)
{
    if (qtype == QT_F32) return static_cast<const float4 *>(values)[quad];
    const uint2 v = static_cast<const uint2 *>(values)[quad];
    return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                       __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
}

// One workgroup per row. The row is read twice (mean square, then the gated sum of the streams);
// both passes keep four 16-byte loads per thread in flight, because a row is a short stream and
// a loop that waits for each load in turn spends its time on latency; long rows take 1024
// threads for the same reason. Rows whose width is not a multiple of four take the scalar loops.
template <unsigned THREADS>
__global__ __launch_bounds__(THREADS) void mhc_ingress_kernel(
    const float *__restrict__ rows, const float *__restrict__ mixes, const void *__restrict__ scale_values,
    const void *__restrict__ base_values, const void *__restrict__ norm, unsigned scale_qtype,
    unsigned base_qtype, unsigned norm_qtype, unsigned streams, unsigned width,
    unsigned iterations, double rms_epsilon, double mhc_epsilon, double post_multiplier,
    float *__restrict__ normalized, float *__restrict__ post, float *__restrict__ combination,
    int quads, int *status)
{
    __shared__ float base[64], scale[3];      // (streams + 2) * streams <= 63 mixing rows
    extern __shared__ __align__(16) float collapsed[];   // width values
    __shared__ double slots[THREADS / 64u];
    __shared__ double gate[8];
    constexpr unsigned kBatch = 4;
    constexpr unsigned kWorkers = THREADS - 64u;     // the second pass leaves the first wavefront out
    const unsigned tid = threadIdx.x;
    const unsigned long long row = blockIdx.x;
    const unsigned expanded = streams * width, mixing_rows = (streams + 2u) * streams;
    const float *in = rows + row * expanded;
    const float *mix = mixes + row * mixing_rows;
    bool bad = false;    // quads: width is a multiple of four and every row starts 16-byte aligned

    // mean square of the bf16-rounded residual
    double squares = 0.0;
    if (quads) {
        const float4 *in4 = reinterpret_cast<const float4 *>(in);
        const unsigned count = expanded >> 2;
        for (unsigned first = tid; first < count; first += THREADS * kBatch) {
            float4 v[kBatch];
#pragma unroll
            for (unsigned u = 0; u < kBatch; ++u) {
                const unsigned at = first + u * THREADS;
                v[u] = at < count ? in4[at] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
#pragma unroll
            for (unsigned u = 0; u < kBatch; ++u) {
                const float4 r = bf16_round4(v[u]);
                bad |= !finite_f32(r.x) || !finite_f32(r.y) || !finite_f32(r.z) || !finite_f32(r.w);
                squares += (double)r.x * (double)r.x;
                squares += (double)r.y * (double)r.y;
                squares += (double)r.z * (double)r.z;
                squares += (double)r.w * (double)r.w;
            }
        }
    } else {
        for (unsigned lane = tid; lane < expanded; lane += THREADS) {
            const float v = bf16_round(in[lane]);
            bad |= !finite_f32(v);
            squares += (double)v * (double)v;
        }
    }
    if (tid < mixing_rows) {
        base[tid] = coefficient(base_values, base_qtype, tid);
        bad |= !finite_f32(base[tid]) || !finite_f32(mix[tid]);
    }
    if (tid < 3u) {
        scale[tid] = coefficient(scale_values, scale_qtype, tid);
        bad |= !finite_f32(scale[tid]);
    }
    // (the barriers inside the sum publish base and scale to the threads that read them below)
    const double inverse = 1.0 / sqrt(workgroup_sum<THREADS / 64u>(squares, slots) / (double)expanded + rms_epsilon);
    bad |= !finite_f64(inverse);

    if (tid < streams) {
        const double pre = sigmoid_f64((double)mix[tid] * inverse * (double)scale[0] + (double)base[tid]);
        gate[tid] = pre + mhc_epsilon;
        post[row * streams + tid] = (float)(post_multiplier * sigmoid_f64(
            (double)mix[streams + tid] * inverse * (double)scale[1] + (double)base[streams + tid]));
    }
    __syncthreads();

    // The mixing matrix lives in the first wavefront, one element per lane, and never touches
    // memory: a row (or column) total is gathered with lane reads in index order, so every lane
    // of the row forms the same double-precision sum the serial code forms. It is a chain of
    // dependent divisions several microseconds long, so the other wavefronts run the second pass
    // over the row meanwhile.
    const unsigned cells = streams * streams;
    if (tid < 64u) {
        const bool cell = tid < cells;
        const unsigned r = cell ? tid / streams : 0u, c = cell ? tid % streams : 0u;
        const unsigned index = 2u * streams + (cell ? tid : 0u);
        float m = (float)((double)mix[index] * inverse * (double)scale[2] + (double)base[index]);
        double maximum = -__builtin_inf(), total = 0.0, mine = 0.0;
        for (unsigned k = 0; k < streams; ++k)
            maximum = fmax(maximum, (double)__shfl(m, (int)(r * streams + k), kWave));
        for (unsigned k = 0; k < streams; ++k) {
            const double value = exp((double)__shfl(m, (int)(r * streams + k), kWave) - maximum);
            total += value;
            if (k == c) mine = value;
        }
        bad |= cell && (!finite_f64(total) || !(total > 0.0));
        m = (float)((double)(float)mine / total + mhc_epsilon);
        for (unsigned it = 0; it < iterations; ++it) {
            if (it != 0u) {
                double across = 0.0;
                for (unsigned k = 0; k < streams; ++k) across += (double)__shfl(m, (int)(r * streams + k), kWave);
                bad |= cell && !finite_f64(across);
                m = (float)((double)m / (across + mhc_epsilon));
            }
            double down = 0.0;
            for (unsigned k = 0; k < streams; ++k) down += (double)__shfl(m, (int)(k * streams + c), kWave);
            bad |= cell && !finite_f64(down);
            m = (float)((double)m / (down + mhc_epsilon));
        }
        if (cell) combination[row * cells + tid] = m;
    }

    // collapsed row: float accumulation over the streams in order, then bf16
    double collapsed_squares = 0.0;
    if (tid < 64u) {
        // busy with the mixing matrix above
    } else if (quads && streams <= kBatch) {
        const float4 *in4 = reinterpret_cast<const float4 *>(in);
        const unsigned count = width >> 2;
        for (unsigned at = tid - 64u; at < count; at += kWorkers) {
            float4 v[kBatch];
#pragma unroll
            for (unsigned s = 0; s < kBatch; ++s)
                v[s] = s < streams ? in4[s * count + at] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            float4 total = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
            for (unsigned s = 0; s < kBatch; ++s) {
                if (s < streams) {
                    const float4 r = bf16_round4(v[s]);
                    total.x += (float)(gate[s] * (double)r.x);
                    total.y += (float)(gate[s] * (double)r.y);
                    total.z += (float)(gate[s] * (double)r.z);
                    total.w += (float)(gate[s] * (double)r.w);
                }
            }
            bad |= !finite_f32(total.x) || !finite_f32(total.y) || !finite_f32(total.z) || !finite_f32(total.w);
            const float4 published = bf16_round4(total);
            reinterpret_cast<float4 *>(collapsed)[at] = published;
            collapsed_squares += (double)published.x * (double)published.x;
            collapsed_squares += (double)published.y * (double)published.y;
            collapsed_squares += (double)published.z * (double)published.z;
            collapsed_squares += (double)published.w * (double)published.w;
        }
    } else {
        for (unsigned lane = tid - 64u; lane < width; lane += kWorkers) {
            float total = 0.0f;
            for (unsigned s = 0; s < streams; ++s)
                total += (float)(gate[s] * (double)bf16_round(in[s * width + lane]));
            bad |= !finite_f32(total);
            const float published = bf16_round(total);
            collapsed[lane] = published;
            collapsed_squares += (double)published * (double)published;
        }
    }

    // weighted RMS norm of the collapsed row, published as bf16 (the barriers inside the sum
    // order the collapsed values before any thread reads them)
    const double mean = workgroup_sum<THREADS / 64u>(collapsed_squares, slots) / (double)width;
    const double norm_inverse = 1.0 / sqrt(mean + rms_epsilon);
    bad |= !finite_f64(norm_inverse);
    if (quads && streams <= kBatch) {
        float4 *out4 = reinterpret_cast<float4 *>(normalized + row * width);
        const unsigned count = width >> 2;
        for (unsigned at = tid; at < count; at += THREADS) {
            const float4 w = coefficient4(norm, norm_qtype, at), v = reinterpret_cast<const float4 *>(collapsed)[at];
            const float in_lane[4] = {v.x, v.y, v.z, v.w}, weight[4] = {w.x, w.y, w.z, w.w};
            float value[4];
#pragma unroll
            for (unsigned i = 0; i < 4u; ++i) {
                double d = (double)in_lane[i] * norm_inverse;
                d *= (double)weight[i];
                value[i] = (float)d;
                bad |= !finite_f32(weight[i]) || !finite_f64(d) || !finite_f32(value[i]);
            }
            out4[at] = bf16_round4(make_float4(value[0], value[1], value[2], value[3]));
        }
    } else {
        for (unsigned lane = tid; lane < width; lane += THREADS) {
            const float weight = coefficient(norm, norm_qtype, lane);
            double v = (double)collapsed[lane] * norm_inverse;
            v *= (double)weight;
            const float value = (float)v;
            bad |= !finite_f32(weight) || !finite_f64(v) || !finite_f32(value);
            normalized[row * width + lane] = bf16_round(value);
        }
    }
    if (bad) raise_status(status, 1);
}

// One thread per (row, four lanes): the lanes' values in every stream are read once and every
// target stream's outputs are formed from them.
template <unsigned LANES>
__global__ __launch_bounds__(kEnvelopeThreads) void mhc_egress_kernel(
    const float *__restrict__ core, const float *__restrict__ rows, const float *__restrict__ post,
    const float *__restrict__ combination, unsigned long long row_count, unsigned streams,
    unsigned width, unsigned blocks_per_row, float *__restrict__ output, int *status)
{
    using Pack = typename std::conditional<LANES == 4u, float4, float>::type;
    const unsigned long long row = blockIdx.x / blocks_per_row;
    const unsigned lane = ((blockIdx.x % blocks_per_row) * kEnvelopeThreads + threadIdx.x) * LANES;
    if (row >= row_count || lane >= width) return;
    const unsigned expanded = streams * width;
    const float *in = rows + row * expanded;
    const float *mixing = combination + row * streams * streams;
    Pack loaded[kEnvelopeMaxStreams + 1u];
    loaded[kEnvelopeMaxStreams] = *reinterpret_cast<const Pack *>(core + row * width + lane);
#pragma unroll
    for (unsigned s = 0; s < kEnvelopeMaxStreams; ++s)
        if (s < streams) loaded[s] = *reinterpret_cast<const Pack *>(in + s * width + lane);
    double value[LANES], residual[kEnvelopeMaxStreams][LANES];
#pragma unroll
    for (unsigned i = 0; i < LANES; ++i) {
        value[i] = (double)reinterpret_cast<const float *>(&loaded[kEnvelopeMaxStreams])[i];
#pragma unroll
        for (unsigned s = 0; s < kEnvelopeMaxStreams; ++s)
            residual[s][i] = s < streams ? (double)bf16_round(reinterpret_cast<const float *>(&loaded[s])[i]) : 0.0;
    }
    bool bad = false;
    for (unsigned target = 0; target < streams; ++target) {
        const double gain = (double)post[row * streams + target];
        double weight[kEnvelopeMaxStreams];
#pragma unroll
        for (unsigned s = 0; s < kEnvelopeMaxStreams; ++s)
            weight[s] = s < streams ? (double)mixing[s * streams + target] : 0.0;
        Pack packed;
#pragma unroll
        for (unsigned i = 0; i < LANES; ++i) {
            double total = gain * value[i];
#pragma unroll
            for (unsigned s = 0; s < kEnvelopeMaxStreams; ++s)
                if (s < streams) total += weight[s] * residual[s][i];
            const float published = (float)total;
            bad |= !finite_f64(total) || !finite_f32(published);
            reinterpret_cast<float *>(&packed)[i] = bf16_round(published);
        }
        *reinterpret_cast<Pack *>(output + row * expanded + target * width + lane) = packed;
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

static int launch_mhc_ingress(const float *rows, const float *mixes, const void *scale, unsigned scale_qtype,
                              const void *base, unsigned base_qtype, const void *norm, unsigned norm_qtype,
                              uint64_t row_count, uint64_t streams, uint64_t width, uint64_t iterations,
                              double rms_epsilon, double mhc_epsilon, double post_multiplier,
                              float *normalized, float *post, float *combination, int *status,
                              yvex_hip_stream stream)
{
    if (!rows || !mixes || !scale || !base || !norm || !normalized || !post || !combination || !status)
        return ST_INVALID_ARG;
    const unsigned qtypes[3] = {scale_qtype, base_qtype, norm_qtype};
    const void *const vectors[3] = {scale, base, norm};
    for (int k = 0; k < 3; ++k) {
        if (qtypes[k] != QT_F32 && qtypes[k] != QT_BF16) return ST_UNSUPPORTED;
        if ((uintptr_t)vectors[k] & (qtypes[k] == QT_F32 ? 3u : 1u)) return ST_INVALID_ARG;
    }
    if (!envelope_shape_ok(row_count, streams, width) || !iterations || iterations > 0xffffffffull)
        return ST_BOUNDS;
    if (!(rms_epsilon > 0.0) || !(mhc_epsilon > 0.0) || !(post_multiplier > 0.0) ||
        rms_epsilon > 1.0e300 || mhc_epsilon > 1.0e300 || post_multiplier > 1.0e300)
        return ST_INVALID_ARG;
    static std::once_flag once;
    static bool prepared = false;
    std::call_once(once, [] {
        prepared =
            hipFuncSetAttribute((const void *)mhc_ingress_kernel<256>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)(kEnvelopeMaxWidth * sizeof(float))) == hipSuccess &&
            hipFuncSetAttribute((const void *)mhc_ingress_kernel<1024>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)(kEnvelopeMaxWidth * sizeof(float))) == hipSuccess;
        if (!prepared) (void)hipGetLastError();
    });
    if (!prepared) {
        set_last_error_text("mhc_ingress: the collapsed row does not fit in LDS");
        return ST_BACKEND;
    }
    const int quads = width % 4u == 0u && !(((uintptr_t)rows | (uintptr_t)normalized) & 15u) &&
                      !((uintptr_t)norm & (norm_qtype == QT_F32 ? 15u : 7u));
    const unsigned lds = (unsigned)(width * sizeof(float));
    if (streams * width >= 8192u)
        mhc_ingress_kernel<1024><<<(unsigned)row_count, 1024, lds, as_stream(stream)>>>(
            rows, mixes, scale, base, norm, scale_qtype, base_qtype, norm_qtype, (unsigned)streams,
            (unsigned)width, (unsigned)iterations, rms_epsilon, mhc_epsilon, post_multiplier, normalized, post,
            combination, quads, status);
    else
        mhc_ingress_kernel<256><<<(unsigned)row_count, 256, lds, as_stream(stream)>>>(
            rows, mixes, scale, base, norm, scale_qtype, base_qtype, norm_qtype, (unsigned)streams,
            (unsigned)width, (unsigned)iterations, rms_epsilon, mhc_epsilon, post_multiplier, normalized, post,
            combination, quads, status);
    return check_launch("mhc_ingress");
}

extern "C" int yvex_hip_mhc_ingress(const float *rows, const float *mixes, const float *scale,
                                    const float *base, const float *norm, uint64_t row_count,
                                    uint64_t streams, uint64_t width, uint64_t iterations,
                                    double rms_epsilon, double mhc_epsilon, double post_multiplier,
                                    float *normalized, float *post, float *combination, int *status,
                                    yvex_hip_stream stream)
{
    return launch_mhc_ingress(rows, mixes, scale, QT_F32, base, QT_F32, norm, QT_F32, row_count, streams, width,
                              iterations, rms_epsilon, mhc_epsilon, post_multiplier, normalized, post,
                              combination, status, stream);
}

extern "C" int yvex_hip_mhc_ingress_encoded(const float *rows, const float *mixes, const void *scale,
                                            unsigned int scale_qtype, const void *base,
                                            unsigned int base_qtype, const void *norm,
                                            unsigned int norm_qtype, uint64_t row_count, uint64_t streams,
                                            uint64_t width, uint64_t iterations, double rms_epsilon,
                                            double mhc_epsilon, double post_multiplier, float *normalized,
                                            float *post, float *combination, int *status,
                                            yvex_hip_stream stream)
{
    return launch_mhc_ingress(rows, mixes, scale, scale_qtype, base, base_qtype, norm, norm_qtype, row_count,
                              streams, width, iterations, rms_epsilon, mhc_epsilon, post_multiplier, normalized,
                              post, combination, status, stream);
}

extern "C" int yvex_hip_mhc_egress(const float *core, const float *rows, const float *post,
                                   const float *combination, uint64_t row_count, uint64_t streams,
                                   uint64_t width, float *output, int *status, yvex_hip_stream stream)
{
    if (!core || !rows || !post || !combination || !output || !status || output == rows)
        return ST_INVALID_ARG;
    if (!envelope_shape_ok(row_count, streams, width)) return ST_BOUNDS;
    const bool quads = width % 4u == 0u && !(((uintptr_t)core | (uintptr_t)rows | (uintptr_t)output) & 15u);
    const uint64_t threads = quads ? width / 4u : width;
    const unsigned blocks_per_row = (unsigned)((threads + kEnvelopeThreads - 1u) / kEnvelopeThreads);
    if (quads)
        mhc_egress_kernel<4><<<(unsigned)(row_count * blocks_per_row), kEnvelopeThreads, 0, as_stream(stream)>>>(
            core, rows, post, combination, row_count, (unsigned)streams, (unsigned)width, blocks_per_row,
            output, status);
    else
        mhc_egress_kernel<1><<<(unsigned)(row_count * blocks_per_row), kEnvelopeThreads, 0, as_stream(stream)>>>(
            core, rows, post, combination, row_count, (unsigned)streams, (unsigned)width, blocks_per_row,
            output, status);
    return check_launch("mhc_egress");
}
