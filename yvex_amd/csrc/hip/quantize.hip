// Q8_K activation quantizer for gfx950: one 64-lane wavefront per 256-value block (q8k.hpp).
#include "common.hpp"
#include "q8k.hpp"
#include "launch.hpp"

namespace yvex {

__global__ __launch_bounds__(256) void q8k_quantize_kernel(
    const float *__restrict__ values, unsigned long long rows, unsigned long long blocks,
    unsigned long long input_stride, unsigned char *__restrict__ encoded, int *status)
{
    const unsigned lane = threadIdx.x & 63u;
    const unsigned long long task = (unsigned long long)blockIdx.x * 4ull + (threadIdx.x >> 6);
    if (task >= rows * blocks) return;
    const unsigned long long row = task / blocks, block = task % blocks;
    q8k_quantize_block(values + row * input_stride + block * 256ull + lane * 4u, encoded + task * kQ8KBytes,
                       lane, status);
}

// Rows of a split input laid end to end, each value rounded to bf16 as the reference's split
// projection rounds it (src/backend/cuda/kernels.cu:736-782).
__global__ __launch_bounds__(256) void concat_rows_bf16_kernel(
    const float *__restrict__ head, const float *__restrict__ tail, unsigned long long rows,
    unsigned head_width, unsigned tail_width, float *__restrict__ out, int *status)
{
    const unsigned width = head_width + tail_width;
    const unsigned long long index = (unsigned long long)blockIdx.x * 256ull + threadIdx.x;
    if (index >= rows * width) return;
    const unsigned long long row = index / width;
    const unsigned column = (unsigned)(index % width);
    const float value = bf16_round(column < head_width ? head[row * head_width + column]
                                                       : tail[row * tail_width + (column - head_width)]);
    if (!finite_f32(value)) raise_status(status, 1);
    out[index] = value;
}

}  // namespace yvex

using namespace yvex;

extern "C" int yvex_hip_q8k_quantize(const float *values, uint64_t rows, uint64_t width,
                                     uint64_t input_stride, uint8_t *encoded, int *status,
                                     yvex_hip_stream stream)
{
    if (!values || !encoded || !status || !rows || !width || width % 256u ||
        input_stride < width || ((uintptr_t)encoded & 3u) || ((uintptr_t)values & 3u))
        return ST_INVALID_ARG;
    const uint64_t blocks = width / 256u;
    if (rows > UINT64_MAX / blocks) return ST_BOUNDS;
    const uint64_t tasks = rows * blocks, grid = (tasks + 3u) / 4u;
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    q8k_quantize_kernel<<<(unsigned)grid, 256, 0, as_stream(stream)>>>(
        values, rows, blocks, input_stride, encoded, status);
    return check_launch("q8k_quantize");
}

extern "C" int yvex_hip_concat_rows_bf16(const float *head, const float *tail, uint64_t rows,
                                         uint64_t head_width, uint64_t tail_width, float *out,
                                         int *status, yvex_hip_stream stream)
{
    if (!head || !tail || !out || !status || !rows || !head_width || !tail_width) return ST_INVALID_ARG;
    if (head_width + tail_width > 0xffffffffull || rows > UINT64_MAX / (head_width + tail_width))
        return ST_BOUNDS;
    const uint64_t grid = (rows * (head_width + tail_width) + 255u) / 256u;
    if (grid > 0x7fffffffull) return ST_BOUNDS;
    concat_rows_bf16_kernel<<<(unsigned)grid, 256, 0, as_stream(stream)>>>(
        head, tail, rows, (unsigned)head_width, (unsigned)tail_width, out, status);
    return check_launch("concat_rows_bf16");
}
