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

constexpr unsigned kSelectThreads = 1024u;

__global__ __launch_bounds__(kSelectThreads) void argmax_rows_kernel(
    const float *values, unsigned long long row_count, unsigned long long row_width,
    unsigned *selected_tokens, float *selected_values, unsigned long long *tie_counts, int *status)
{
    __shared__ float best_of[kSelectThreads / 64u];
    __shared__ unsigned index_of[kSelectThreads / 64u];
    __shared__ unsigned long long ties_of[kSelectThreads / 64u];
    __shared__ int failed;
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned long long row = blockIdx.x;
    if (row >= row_count) return;
    if (tid == 0u) failed = 0;
    __syncthreads();
    const float *v = values + row * row_width;
    Candidate mine{-3.402823466e+38F, 0xffffffffu, 0ull};
    bool bad = false;
    auto look = [&](float value, unsigned index) {
        if (!finite_f32(value)) bad = true;
        else candidate_take(mine, value, index);
    };
    // 16-byte loads over the aligned middle of the row, scalar loads at its ends
    const unsigned long long address = (unsigned long long)v;
    unsigned long long head = ((16ull - (address & 15ull)) & 15ull) / 4ull;
    if (head > row_width) head = row_width;
    const unsigned long long quads = (row_width - head) / 4ull;
    for (unsigned long long i = tid; i < head; i += kSelectThreads) look(v[i], (unsigned)i);
    const float4 *v4 = reinterpret_cast<const float4 *>(v + head);
    for (unsigned long long q = tid; q < quads; q += kSelectThreads) {
        const float4 x = v4[q];
        const unsigned at = (unsigned)(head + 4ull * q);
        look(x.x, at);
        look(x.y, at + 1u);
        look(x.z, at + 2u);
        look(x.w, at + 3u);
    }
    for (unsigned long long i = head + 4ull * quads + tid; i < row_width; i += kSelectThreads)
        look(v[i], (unsigned)i);

    if (bad) {
        raise_status(status, 1);
        failed = 1;
    }
    // wave, then workgroup
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
    if (tid == 0u && !failed) {
        Candidate all{best_of[0], index_of[0], ties_of[0]};
        for (unsigned w = 1; w < kSelectThreads / 64u; ++w)
            candidate_merge(all, Candidate{best_of[w], index_of[w], ties_of[w]});
        selected_tokens[row] = all.index;
        selected_values[row] = all.best;
        tie_counts[row] = all.ties;
    }
}

}  // namespace yvex

using namespace yvex;

extern "C" int yvex_hip_argmax_f32(const float *values, uint64_t row_count, uint64_t row_width,
                                   uint32_t *selected_tokens, float *selected_values,
                                   uint64_t *tie_counts, int *status, yvex_hip_stream stream)
{
    if (!values || !row_count || !row_width || !selected_tokens || !selected_values || !tie_counts ||
        !status)
        return ST_INVALID_ARG;
    if (row_count > 0x7fffffffull || row_width > 0xffffffffull) return ST_BOUNDS;
    if ((uintptr_t)values & 3u) return ST_INVALID_ARG;
    argmax_rows_kernel<<<(unsigned)row_count, kSelectThreads, 0, as_stream(stream)>>>(
        values, row_count, row_width, selected_tokens, selected_values,
        (unsigned long long *)tie_counts, status);
    return check_launch("argmax_f32");
}
