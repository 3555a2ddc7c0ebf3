// One Q8_K block by one 64-lane wavefront: four values per lane, max-|x| search and the sixteen
// 16-value sums done with cross-lane shuffles. Behaviour restated from
// src/backend/cuda/kernels.cu:436-489.
#pragma once
#include "common.hpp"

namespace yvex {

// x: this lane's four values of the block; out: the block's 292 bytes.
__device__ __forceinline__ void q8k_quantize_block(const float *__restrict__ x, unsigned char *__restrict__ out,
                                                   unsigned lane, int *status)
{
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

}  // namespace yvex
