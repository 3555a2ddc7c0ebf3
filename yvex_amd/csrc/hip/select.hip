// Greedy selection over rows of logits: the largest value of a row, the lowest index that holds
// it and how many elements hold it, computed on the device so that a 129 280-entry logits row
// never has to cross to the host to pick a token.
//
// Behaviour restated from src/backend/cuda/kernels.cu:59-110 (yvex_argmax_f32): values start
// from -FLT_MAX with no index, a larger value replaces the candidate and resets the tie count
// to one, an equal value keeps the lower index and counts a tie; any non-finite element raises
// status 1 and the row publishes nothing.
//
// One workgroup of 1024 threads per row (the reference runs 128): a single 517 KB row is
// bounded by what one compute unit can pull from cache, about 4 us; several rows run side by
// side.
#include "common.hpp"
#include "launch.hpp"

namespace yvex {

struct Candidate {
    float best;
    unsigned index;               // 0xffffffff: none yet
    unsigned long long ties;
};

__device__ __forceinline__ void candidate_take(Candidate &c, float value, unsigned index)
{
    if (value > c.best) {
        c.best = value;
        c.index = index;
        c.ties = 1ull;
    } else if (value == c.best) {
        if (index < c.index) c.index = index;
        ++c.ties;
    }
}

__device__ __forceinline__ void candidate_merge(Candidate &c, const Candidate &other)
{
    if (other.best > c.best) {
        c = other;
    } else if (other.best == c.best) {
        if (other.index < c.index) c.index = other.index;
        c.ties += other.ties;
    }
}

// Candidate of the elements [begin, end) of one row, held by thread 0 of the workgroup on return
// (`ok` false when the span holds a non-finite value). THREADS threads.
//
// Two passes without branches, a compare-heavy single pass being bound by the vector ALUs: first
// the largest finite value of the span (and whether anything is not finite), then, with the span
// coming from cache, the lowest index and the count of the elements equal to it. Loads are 16
// bytes over the aligned middle of the span and issued eight at a time.
template <unsigned THREADS>
__device__ __forceinline__ Candidate span_candidate(const float *row, unsigned long long begin,
                                                    unsigned long long end, int *status, bool &ok)
{
    __shared__ float best_of[THREADS / 64u];
    __shared__ unsigned index_of[THREADS / 64u];
    __shared__ unsigned long long ties_of[THREADS / 64u];
    __shared__ int failed;
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    if (tid == 0u) failed = 0;
    __syncthreads();
    const float *v = row + begin;
    const unsigned long long count_all = end - begin;
    const unsigned long long address = (unsigned long long)v;
    unsigned long long head = ((16ull - (address & 15ull)) & 15ull) / 4ull;
    if (head > count_all) head = count_all;
    const unsigned long long quads = (count_all - head) / 4ull;
    const unsigned long long tail = head + 4ull * quads;
    const float4 *v4 = reinterpret_cast<const float4 *>(v + head);
    constexpr unsigned kBatch = 8u;
    constexpr float kLowest = -3.402823466e+38F;

    float top = kLowest;
    bool bad = false;
    auto rise = [&](float value) {
        bad |= !finite_f32(value);
        top = fmaxf(top, value);              // a NaN operand is dropped, an infinity is flagged above
    };
    for (unsigned long long i = tid; i < head; i += THREADS) rise(v[i]);
    for (unsigned long long q0 = 0; q0 < quads; q0 += (unsigned long long)THREADS * kBatch) {
        float4 x[kBatch];
#pragma unroll
        for (unsigned k = 0; k < kBatch; ++k) {
            const unsigned long long q = q0 + tid + (unsigned long long)k * THREADS;
            x[k] = v4[q < quads ? q : quads - 1ull];      // a repeated element changes no maximum
        }
#pragma unroll
        for (unsigned k = 0; k < kBatch; ++k) {
            rise(x[k].x);
            rise(x[k].y);
            rise(x[k].z);
            rise(x[k].w);
        }
    }
    for (unsigned long long i = tail + tid; i < count_all; i += THREADS) rise(v[i]);
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) top = fmaxf(top, __shfl_xor(top, offset, kWave));
    if (lane == 0u) best_of[wave] = top;
    if (bad) {
        raise_status(status, 1);
        failed = 1;
    }
    __syncthreads();
    ok = failed == 0;
    if (!ok) return Candidate{kLowest, 0xffffffffu, 0ull};
#pragma unroll
    for (unsigned w = 0; w < THREADS / 64u; ++w) top = fmaxf(top, best_of[w]);
    __syncthreads();                          // best_of is reused below

    // (the span's values cannot all lie below the starting value, the lowest finite float: `top`
    // is a value of the span)
    Candidate mine{top, 0xffffffffu, 0ull};
    auto count = [&](float value, unsigned long long index, bool inside) {
        const bool hit = inside && value == top;
        const unsigned at = (unsigned)(begin + index);
        mine.index = hit && at < mine.index ? at : mine.index;
        mine.ties += hit ? 1ull : 0ull;
    };
    for (unsigned long long i = tid; i < head; i += THREADS) count(v[i], i, true);
    for (unsigned long long q0 = 0; q0 < quads; q0 += (unsigned long long)THREADS * kBatch) {
        float4 x[kBatch];
#pragma unroll
        for (unsigned k = 0; k < kBatch; ++k) {
            const unsigned long long q = q0 + tid + (unsigned long long)k * THREADS;
            x[k] = v4[q < quads ? q : quads - 1ull];
        }
#pragma unroll
        for (unsigned k = 0; k < kBatch; ++k) {
            const unsigned long long q = q0 + tid + (unsigned long long)k * THREADS;
            const bool inside = q < quads;
            const unsigned long long at = head + 4ull * q;
            count(x[k].x, at, inside);
            count(x[k].y, at + 1ull, inside);
            count(x[k].z, at + 2ull, inside);
            count(x[k].w, at + 3ull, inside);
        }
    }
    for (unsigned long long i = tail + tid; i < count_all; i += THREADS) count(v[i], i, true);
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        Candidate other;
        other.best = __shfl_xor(mine.best, offset, kWave);
        other.index = (unsigned)__shfl_xor((int)mine.index, offset, kWave);
        other.ties = (unsigned long long)__shfl_xor((long long)mine.ties, offset, kWave);
        candidate_merge(mine, other);
    }
    if (lane == 0u) {
        best_of[wave] = mine.best;
        index_of[wave] = mine.index;
        ties_of[wave] = mine.ties;
    }
    __syncthreads();
    Candidate all{best_of[0], index_of[0], ties_of[0]};
    if (tid == 0u)
        for (unsigned w = 1; w < THREADS / 64u; ++w)
            candidate_merge(all, Candidate{best_of[w], index_of[w], ties_of[w]});
    return all;
}

constexpr unsigned kSelectThreads = 1024u;    // one workgroup per row
constexpr unsigned kSpanThreads = 256u;       // several workgroups per row
constexpr unsigned kSpanElements = 8192u;

__global__ __launch_bounds__(kSelectThreads) void argmax_rows_kernel(
    const float *values, unsigned long long row_count, unsigned long long row_width,
    unsigned *selected_tokens, float *selected_values, unsigned long long *tie_counts, int *status)
{
    const unsigned long long row = blockIdx.x;
    if (row >= row_count) return;
    bool ok;
    const Candidate all = span_candidate<kSelectThreads>(values + row * row_width, 0ull, row_width, status, ok);
    if (threadIdx.x == 0u && ok) {
        selected_tokens[row] = all.index;
        selected_values[row] = all.best;
        tie_counts[row] = all.ties;
    }
}

// A long row split over blockIdx.x spans of kSpanElements: partial candidates into scratch
// ({float best, u32 index, u64 ties} per span), merged by argmax_merge_kernel.
struct SpanResult {
    float best;
    unsigned index;
    unsigned long long ties;
};

__global__ __launch_bounds__(kSpanThreads) void argmax_spans_kernel(
    const float *values, unsigned long long row_count, unsigned long long row_width,
    SpanResult *partial, int *status)
{
    const unsigned long long row = blockIdx.y, span = blockIdx.x;
    const unsigned long long begin = span * kSpanElements;
    if (row >= row_count || begin >= row_width) return;
    const unsigned long long end = begin + kSpanElements < row_width ? begin + kSpanElements : row_width;
    bool ok;
    const Candidate all = span_candidate<kSpanThreads>(values + row * row_width, begin, end, status, ok);
    if (threadIdx.x == 0u)
        partial[row * gridDim.x + span] = ok ? SpanResult{all.best, all.index, all.ties}
                                             : SpanResult{-3.402823466e+38F, 0xffffffffu, 0ull};
}

__global__ __launch_bounds__(64) void argmax_merge_kernel(
    const SpanResult *partial, unsigned spans, unsigned long long row_count, unsigned *selected_tokens,
    float *selected_values, unsigned long long *tie_counts)
{
    const unsigned long long row = blockIdx.x;
    if (row >= row_count) return;
    const unsigned lane = threadIdx.x;
    Candidate mine{-3.402823466e+38F, 0xffffffffu, 0ull};
    bool bad = false;         // a span that met a non-finite value counts no element at all
    for (unsigned s = lane; s < spans; s += 64u) {
        const SpanResult r = partial[row * spans + s];
        if (!r.ties) bad = true;
        candidate_merge(mine, Candidate{r.best, r.index, r.ties});
    }
    // only the row that holds the bad value publishes nothing, as when one workgroup scans a row;
    // a status left by other work on the stream does not silence the rows of this launch
    if (__any(bad)) return;
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        Candidate other;
        other.best = __shfl_xor(mine.best, offset, kWave);
        other.index = (unsigned)__shfl_xor((int)mine.index, offset, kWave);
        other.ties = (unsigned long long)__shfl_xor((long long)mine.ties, offset, kWave);
        candidate_merge(mine, other);
    }
    if (lane == 0u) {
        selected_tokens[row] = mine.index;
        selected_values[row] = mine.best;
        tie_counts[row] = mine.ties;
    }
}

// Span results for callers that cannot allocate: one array per device, held until the process
// ends. 16 384 span results cover 64 rows of 262 144 values, or one row of 134 million.
constexpr uint64_t kStaticSpanResults = 16384u;
constexpr int kStaticDevices = 16;
static __device__ __align__(256) unsigned char scratch[kStaticSpanResults * sizeof(SpanResult)];
static std::mutex static_scratch_lock;
static void *static_scratch_of[kStaticDevices];      // device address of `scratch`, per device

// The device address of this device's copy of the array, looked up once per device with that
// device current. The array's name is only a host-side handle for this lookup.
static int static_scratch_address(void **out)
{
    int device = -1;
    hipError_t code = hipGetDevice(&device);
    if (code != hipSuccess || device < 0 || device >= kStaticDevices) {
        if (code != hipSuccess) set_last_error("argmax_f32_static: hipGetDevice", code);
        else set_last_error_text("argmax_f32_static: device ordinal is outside the table");
        (void)hipGetLastError();
        return ST_BACKEND;
    }
    std::lock_guard<std::mutex> guard(static_scratch_lock);
    if (!static_scratch_of[device]) {
        void *address = nullptr;
        code = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (code != hipSuccess || !address) {
            set_last_error("argmax_f32_static: hipGetSymbolAddress", code);
            (void)hipGetLastError();
            return ST_BACKEND;
        }
        static_scratch_of[device] = address;
    }
    *out = static_scratch_of[device];
    return ST_OK;
}

}  // namespace yvex

using namespace yvex;

extern "C" uint64_t yvex_hip_argmax_scratch_bytes(uint64_t row_count, uint64_t row_width)
{
    const uint64_t spans = (row_width + kSpanElements - 1u) / kSpanElements;
    return spans > 1u ? row_count * spans * sizeof(SpanResult) : 0u;
}

extern "C" int yvex_hip_argmax_f32(const float *values, uint64_t row_count, uint64_t row_width,
                                   uint32_t *selected_tokens, float *selected_values,
                                   uint64_t *tie_counts, void *scratch, uint64_t scratch_bytes,
                                   int *status, yvex_hip_stream stream)
{
    if (!values || !row_count || !row_width || !selected_tokens || !selected_values || !tie_counts ||
        !status)
        return ST_INVALID_ARG;
    if (row_count > 65535ull || row_width > 0xffffffffull) return ST_BOUNDS;
    if (((uintptr_t)values & 3u) || ((uintptr_t)scratch & 7u)) return ST_INVALID_ARG;
    const uint64_t need = yvex_hip_argmax_scratch_bytes(row_count, row_width);
    hipStream_t s = as_stream(stream);
    if (need && scratch && scratch_bytes >= need) {
        const unsigned spans = (unsigned)((row_width + kSpanElements - 1u) / kSpanElements);
        argmax_spans_kernel<<<dim3(spans, (unsigned)row_count), kSpanThreads, 0, s>>>(
            values, row_count, row_width, (SpanResult *)scratch, status);
        int rc = check_launch("argmax_f32.spans");
        if (rc) return rc;
        argmax_merge_kernel<<<(unsigned)row_count, 64, 0, s>>>(
            (const SpanResult *)scratch, spans, row_count, selected_tokens, selected_values,
            (unsigned long long *)tie_counts);
        return check_launch("argmax_f32.merge");
    }
    argmax_rows_kernel<<<(unsigned)row_count, kSelectThreads, 0, s>>>(
        values, row_count, row_width, selected_tokens, selected_values,
        (unsigned long long *)tie_counts, status);
    return check_launch("argmax_f32");
}

extern "C" uint64_t yvex_hip_argmax_static_capacity(void) { return sizeof(scratch); }

extern "C" int yvex_hip_argmax_f32_static(const float *values, uint64_t row_count, uint64_t row_width,
                                          uint32_t *selected_tokens, float *selected_values,
                                          uint64_t *tie_counts, int *status, yvex_hip_stream stream)
{
    if (!values || !row_count || !row_width || !selected_tokens || !selected_values || !tie_counts ||
        !status)
        return ST_INVALID_ARG;
    if (row_count > 65535ull || row_width > 0xffffffffull) return ST_BOUNDS;
    const uint64_t need = yvex_hip_argmax_scratch_bytes(row_count, row_width);
    if (need > sizeof(scratch)) {
        set_last_error_text("argmax_f32_static: rows x spans exceed the 16384 span results of the "
                            "static scratch array; use yvex_hip_argmax_f32 with a workspace");
        return ST_BOUNDS;
    }
    void *spans = nullptr;
    if (need) {
        const int rc = static_scratch_address(&spans);
        if (rc) return rc;
    }
    // every span result the merge reads is written by the span launch before it: nothing in the
    // array has to start at zero
    return yvex_hip_argmax_f32(values, row_count, row_width, selected_tokens, selected_values,
                               tie_counts, spans, need, status, stream);
}
