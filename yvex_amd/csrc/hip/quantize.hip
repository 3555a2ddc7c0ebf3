// Q8_K activation quantizer for gfx950: one 64-lane wavefront per 256-value block, four values
// per lane, max-|x| search and the sixteen 16-value sums done with cross-lane shuffles.
// Behaviour restated from src/backend/cuda/kernels.cu:436-489.
#include "common.hpp"
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
    const float *x = values + row * input_stride + block * 256ull + lane * 4u;
    unsigned char *out = encoded + task * kQ8KBytes;
    float v[4];
    unsigned long long key = 0ull;
    bool bad = false;
#pragma unroll
    for (unsigned i = 0; i < 4u; ++i) {
        v[i] = x[i];
        const unsigned bits = __float_as_uint(v[i]);
        bad |= !finite_f32(v[i]);
        // order by |x|, then by lowest index; the low bit carries the sign of the winner
        const unsigned long long k = ((unsigned long long)(bits & 0x7fffffffu) << 32) |
                                     ((unsigned long long)(255u - (lane * 4u + i)) << 1) |
                                     (bits >> 31);
        key = k > key ? k : key;
    }
    if (bad) raise_status(status, 1);
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const unsigned long long other = __shfl_xor(key, offset, kWave);
        key = other > key ? other : key;
    }
    const float magnitude = __uint_as_float((unsigned)(key >> 32));
    const float signed_max = (key & 1ull) ? -magnitude : magnitude;
    const float inverse = magnitude == 0.0f ? 0.0f : -127.0f / signed_max;
    if (lane == 0u) *reinterpret_cast<float *>(out) = inverse == 0.0f ? 0.0f : 1.0f / inverse;
    unsigned packed = 0u;
    int sum = 0;
#pragma unroll
    for (unsigned i = 0; i < 4u; ++i) {
        int q = inverse == 0.0f ? 0 : __float2int_rn(inverse * v[i]);
        q = q > 127 ? 127 : q < -128 ? -128 : q;
        sum += q;
        packed |= ((unsigned)q & 255u) << (8u * i);
    }
    *reinterpret_cast<unsigned *>(out + 4u + lane * 4u) = packed;
    sum = group_sum_i32<4>(sum);   // four lanes hold sixteen consecutive values
    if ((lane & 3u) == 0u) *reinterpret_cast<short *>(out + 260u + (lane >> 2) * 2u) = (short)sum;
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
