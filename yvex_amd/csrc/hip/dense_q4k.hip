// Q4_K weight rows against a batch of Q8_K input rows on the int8 matrix cores: the dense
// projection at prefill width (16 input rows and more; the reference turns its tensor-core
// kernels on there, src/backend/cuda/private.h:461-464).
//
// Arithmetic, per 256-value superblock (public ggml block_q4_K against the Q8_K block of
// src/backend/cuda/kernel_primitives.h:274-312, in the shape of the reference's Q2_K primitive,
// kernel_primitives.h:314-341):
//     dot     = sum_j sc_j * sum_{i in sub-block j} nibble_i * a_i        (int32, exact)
//     minimum = sum_j m_j  * (bsums[2j] + bsums[2j+1])                    (int32, exact)
//     value   = (d_a * d) * float(dot) - (d_a * dmin) * float(minimum)    (two products, one subtraction)
// and the superblock values of a row are added in double and rounded to float once, as the
// CPU path adds a row's blocks (src/gguf/quant_compute.c:152-172).
//
// A 32-value sub-block is exactly the reduction depth of V_MFMA_I32_32X32X32_I8. The weight
// operand carries sc_j * nibble (at most 63 * 15 = 945) as two int8 limbs, value = 8 hi + lo
// with lo = (sc_j mod 8) * nibble and hi = (sc_j div 8) * nibble, both at most 105, so each
// sub-block costs two matrix instructions per 32 tokens and the int32 accumulators run over the
// whole superblock without rescaling. The minimum term is one more reduction of depth 8 (the m_j
// against the pair sums of bsums, in two limbs of base 128) through the same instruction.
//
// A workgroup owns 32 weight rows x 32 or 64 tokens; its four waves take every fourth
// superblock and their double-precision partial tiles are added in wave order, so results do not depend on
// timing. Lane (r, h) of a wave holds bytes 16h..16h+15 of weight row r's sub-block as the A
// operand and the same bytes of token r's activations as the B operand; accumulator i of that
// lane is weight row 8 (i / 4) + 4 h + i % 4 against token r.
#include "common.hpp"
#include "launch.hpp"
#include "grouped.hpp"

namespace yvex {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct DenseQ4kArgs {
    const unsigned char *encoded;
    unsigned long long row_count, row_bytes;
    unsigned blocks;                         // superblocks per row
    const unsigned char *act;                // Q8_K rows, blocks * 292 bytes each
    unsigned long long input_rows;
    const float *additive;
    float *out;
    unsigned long long out_stride;
    int output_bf16;
    int *status;
};

// What one wave needs of one superblock: the weight row's block and NT token blocks.
template <unsigned NT>
struct SuperInputs {
    unsigned head;          // f16 d | f16 dmin << 16
    uint3 scales;           // the 12 scale bytes
    uint4 qs[4];            // this lane's 16 bytes of each 32-byte nibble group
    float act_scale[NT];
    uint4 a[NT][8];         // this lane's 16 bytes of each sub-block's activations
    uint4 bsums[NT][2];     // the 16 int16 sums of 16 activations each
};

template <unsigned NT>
__device__ __forceinline__ void load_super(const DenseQ4kArgs &g, const unsigned char *wrow,
                                           const unsigned char *const (&arow)[NT], unsigned sb,
                                           unsigned h, SuperInputs<NT> &in)
{
    const unsigned char *w = wrow + (unsigned long long)sb * 144ull;
    in.head = *reinterpret_cast<const unsigned *>(w);
    in.scales = *reinterpret_cast<const uint3 *>(w + 4u);
#pragma unroll
    for (unsigned j = 0; j < 4u; ++j) in.qs[j] = *reinterpret_cast<const uint4 *>(w + 16u + 32u * j + 16u * h);
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt) {
        const unsigned char *a = arow[nt] + (unsigned long long)sb * kQ8KBytes;
        in.act_scale[nt] = *reinterpret_cast<const float *>(a);
#pragma unroll
        for (unsigned c = 0; c < 8u; ++c) {
            // the activation bytes start 4 bytes into the block: dword-aligned, read as dwords
            const unsigned *p = reinterpret_cast<const unsigned *>(a + 4u + 32u * c + 16u * h);
            in.a[nt][c] = make_uint4(p[0], p[1], p[2], p[3]);
        }
        const unsigned *b = reinterpret_cast<const unsigned *>(a + 260u);
        in.bsums[nt][0] = make_uint4(b[0], b[1], b[2], b[3]);
        in.bsums[nt][1] = make_uint4(b[4], b[5], b[6], b[7]);
    }
    (void)g;
}

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

// Two int8 limbs of sc * nibble for the four nibbles of one dword (already shifted so that the
// wanted nibble of every byte sits in its low four bits), value = 8 hi + lo. The 6-bit scale is
// split as sc = 8 s_hi + s_lo with both parts in 0..7: a limb byte nibble * s is at most 105, so
// one 16-bit lane multiply scales two bytes at once without a carry from one into the next.
__device__ __forceinline__ void limbs(unsigned x, unsigned sc, unsigned &lo, unsigned &hi)
{
    const unsigned nibbles = x & 0x0f0f0f0fu;
    const unsigned low = (sc & 7u) * 0x00010001u, high = ((sc >> 3) & 7u) * 0x00010001u;
    lo = __builtin_bit_cast(unsigned, __builtin_bit_cast(u16x2, nibbles) * __builtin_bit_cast(u16x2, low));
    hi = __builtin_bit_cast(unsigned, __builtin_bit_cast(u16x2, nibbles) * __builtin_bit_cast(u16x2, high));
}

__device__ __forceinline__ v4i as_v4i(uint4 v)
{
    v4i r = {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
    return r;
}

// Pair sums of the 16 int16 block sums as two int8 limbs (value = 128 hi + lo, lo in 0..127).
__device__ __forceinline__ void bsum_limbs(const uint4 (&b)[2], uint2 &lo, uint2 &hi)
{
    const unsigned w[8] = {b[0].x, b[0].y, b[0].z, b[0].w, b[1].x, b[1].y, b[1].z, b[1].w};
    unsigned l[2] = {0u, 0u}, u[2] = {0u, 0u};
#pragma unroll
    for (unsigned s = 0; s < 8u; ++s) {
        const int pair = (int)(short)(w[s] & 0xffffu) + ((int)w[s] >> 16);
        l[s >> 2] |= ((unsigned)pair & 127u) << (8u * (s & 3u));
        u[s >> 2] |= ((unsigned)(pair >> 7) & 255u) << (8u * (s & 3u));
    }
    lo = make_uint2(l[0], l[1]);
    hi = make_uint2(u[0], u[1]);
}

template <unsigned NT>
__global__ __launch_bounds__(256) void dense_q4k_kernel(DenseQ4kArgs g)
{
    // per wave: d and dmin of its 32 rows for the superblock in hand; then the partial tiles
    __shared__ __align__(16) float row_scale[4][2][32];
    __shared__ double partial[3][NT][16][64];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned r = lane & 31u, h = lane >> 5;
    const unsigned long long row0 = (unsigned long long)blockIdx.x * 32ull;
    const unsigned long long tok0 = (unsigned long long)blockIdx.y * (32ull * NT);
    unsigned long long wr = row0 + r;
    if (wr >= g.row_count) wr = g.row_count - 1ull;              // a ragged edge repeats the last row
    const unsigned char *wrow = g.encoded + wr * g.row_bytes;
    const unsigned char *arow[NT];
    const unsigned long long act_row_bytes = (unsigned long long)g.blocks * kQ8KBytes;
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt) {
        unsigned long long t = tok0 + 32ull * nt + r;
        if (t >= g.input_rows) t = g.input_rows - 1ull;
        arow[nt] = g.act + t * act_row_bytes;
    }
    double acc[NT][16];
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[nt][i] = 0.0;

    SuperInputs<NT> cur;
    if (wave < g.blocks) load_super<NT>(g, wrow, arow, wave, h, cur);
    for (unsigned sb = wave; sb < g.blocks; sb += 4u) {
        // the next superblock's bytes travel while this one is worked on
        SuperInputs<NT> nxt;
        const unsigned ahead = sb + 4u < g.blocks ? sb + 4u : sb;
        load_super<NT>(g, wrow, arow, ahead, h, nxt);

        // scales and minima of the eight sub-blocks, four to a dword (ggml get_scale_min_k4)
        const unsigned s0 = cur.scales.x, s1 = cur.scales.y, s2 = cur.scales.z;
        const unsigned sc_pack[2] = {s0 & 0x3f3f3f3fu, (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)};
        const unsigned mn_pack[2] = {s1 & 0x3f3f3f3fu, ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)};
        if (h == 0u) {
            row_scale[wave][0][r] = f16_bits_to_float(cur.head & 0xffffu);
            row_scale[wave][1][r] = f16_bits_to_float(cur.head >> 16);
        }

        v16i lo_sum[NT], hi_sum[NT];
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) lo_sum[nt][i] = hi_sum[nt][i] = 0;
#pragma unroll
        for (unsigned c = 0; c < 8u; ++c) {
            const unsigned sc = (sc_pack[c >> 2] >> (8u * (c & 3u))) & 255u;
            const uint4 q = cur.qs[c >> 1];
            const unsigned shift = (c & 1u) * 4u;
            v4i a_lo, a_hi;
            unsigned lo, hi;
            limbs(q.x >> shift, sc, lo, hi); a_lo[0] = (int)lo; a_hi[0] = (int)hi;
            limbs(q.y >> shift, sc, lo, hi); a_lo[1] = (int)lo; a_hi[1] = (int)hi;
            limbs(q.z >> shift, sc, lo, hi); a_lo[2] = (int)lo; a_hi[2] = (int)hi;
            limbs(q.w >> shift, sc, lo, hi); a_lo[3] = (int)lo; a_hi[3] = (int)hi;
#pragma unroll
            for (unsigned nt = 0; nt < NT; ++nt) {
                const v4i b = as_v4i(cur.a[nt][c]);
                lo_sum[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_lo, b, lo_sum[nt], 0, 0, 0);
                hi_sum[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a_hi, b, hi_sum[nt], 0, 0, 0);
            }
        }
        // minimum term: m_j (bytes 0..7 of the h = 0 half, zeros elsewhere) against the pair sums
        v4i m_op = {0, 0, 0, 0};
        if (h == 0u) {
            m_op[0] = (int)mn_pack[0];
            m_op[1] = (int)mn_pack[1];
        }
        v16i min_lo[NT], min_hi[NT];
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt) {
            uint2 bl, bh;
            bsum_limbs(cur.bsums[nt], bl, bh);
            v4i b_lo = {0, 0, 0, 0}, b_hi = {0, 0, 0, 0};
            if (h == 0u) {
                b_lo[0] = (int)bl.x; b_lo[1] = (int)bl.y;
                b_hi[0] = (int)bh.x; b_hi[1] = (int)bh.y;
            }
            v16i zero;
#pragma unroll
            for (int i = 0; i < 16; ++i) zero[i] = 0;
            min_lo[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(m_op, b_lo, zero, 0, 0, 0);
            min_hi[nt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(m_op, b_hi, zero, 0, 0, 0);
        }
        // d and dmin of the sixteen rows this lane accumulates (written above by the wave itself)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        float d_of[16], dmin_of[16];
#pragma unroll
        for (unsigned q4 = 0; q4 < 4u; ++q4) {
            const float4 d = *reinterpret_cast<const float4 *>(&row_scale[wave][0][8u * q4 + 4u * h]);
            const float4 m = *reinterpret_cast<const float4 *>(&row_scale[wave][1][8u * q4 + 4u * h]);
            d_of[4u * q4] = d.x; d_of[4u * q4 + 1u] = d.y; d_of[4u * q4 + 2u] = d.z; d_of[4u * q4 + 3u] = d.w;
            dmin_of[4u * q4] = m.x; dmin_of[4u * q4 + 1u] = m.y; dmin_of[4u * q4 + 2u] = m.z;
            dmin_of[4u * q4 + 3u] = m.w;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt) {
            const float da = cur.act_scale[nt];
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int dot = (hi_sum[nt][i] << 3) + lo_sum[nt][i];
                const int minimum = (min_hi[nt][i] << 7) + min_lo[nt][i];
                const float left = (da * d_of[i]) * (float)dot;
                const float right = (da * dmin_of[i]) * (float)minimum;
                acc[nt][i] += (double)(left - right);
            }
        }
        cur = nxt;
    }

    if (wave) {
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 16; ++i) partial[wave - 1u][nt][i][lane] = acc[nt][i];
    }
    __syncthreads();
    if (wave) return;
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt) {
        const unsigned long long token = tok0 + 32ull * nt + r;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const unsigned long long row = row0 + 8u * (i >> 2) + 4u * h + (i & 3);
            const float sum = (float)(((acc[nt][i] + partial[0][nt][i][lane]) + partial[1][nt][i][lane]) +
                                      partial[2][nt][i][lane]);
            if (row >= g.row_count || token >= g.input_rows) continue;
            const unsigned long long at = token * g.out_stride + row;
            const float value = g.additive ? sum + g.additive[at] : sum;
            if (!finite_f32(value)) raise_status(g.status, 1);
            else g.out[at] = g.output_bf16 ? bf16_round(value) : value;
        }
    }
}

// The same product for 16 to 32 input rows on V_MFMA_I32_16X16X64_I8: a workgroup owns 16
// weight rows x 16 or 32 tokens, so a batch of 16 wastes no token slot and twice as many
// workgroups share the matrix; eight waves (two per SIMD) take every eighth superblock. One K
// step is a 64-value nibble group, i.e. two sub-blocks, which is fine because the limbs already
// carry their sub-block's scale. Lane (r, q) holds bytes 16q..16q+15 of weight row r's group as
// the A operand (q = 0, 1: low nibbles of nibble bytes 16q.., the first sub-block; q = 2, 3:
// high nibbles of nibble bytes 16(q-2).., the second) and the same positions of token r's
// activations as the B operand; accumulator i of that lane is weight row 4 q + i against token r.
template <unsigned NT>
__global__ __launch_bounds__(512) void dense_q4k16_kernel(DenseQ4kArgs g)
{
    typedef int v4s __attribute__((ext_vector_type(4)));
    __shared__ __align__(16) float row_scale[8][2][16];
    __shared__ double partial[7][NT][4][64];
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned r = lane & 15u, q = lane >> 4;
    const unsigned long long row0 = (unsigned long long)blockIdx.x * 16ull;
    const unsigned long long tok0 = (unsigned long long)blockIdx.y * (16ull * NT);
    unsigned long long wr = row0 + r;
    if (wr >= g.row_count) wr = g.row_count - 1ull;
    const unsigned char *wrow = g.encoded + wr * g.row_bytes;
    const unsigned char *arow[NT];
    const unsigned long long act_row_bytes = (unsigned long long)g.blocks * kQ8KBytes;
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt) {
        unsigned long long t = tok0 + 16ull * nt + r;
        if (t >= g.input_rows) t = g.input_rows - 1ull;
        arow[nt] = g.act + t * act_row_bytes;
    }
    double acc[NT][4];
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[nt][i] = 0.0;

    for (unsigned sb = wave; sb < g.blocks; sb += 8u) {
        const unsigned char *w = wrow + (unsigned long long)sb * 144ull;
        const unsigned head = *reinterpret_cast<const unsigned *>(w);
        const uint3 scales = *reinterpret_cast<const uint3 *>(w + 4u);
        uint4 qs[4];
#pragma unroll
        for (unsigned j = 0; j < 4u; ++j)
            qs[j] = *reinterpret_cast<const uint4 *>(w + 16u + 32u * j + 16u * (q & 1u));
        uint4 a[NT][4], bsums[NT][2];
        float da[NT];
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt) {
            const unsigned char *ab = arow[nt] + (unsigned long long)sb * kQ8KBytes;
            da[nt] = *reinterpret_cast<const float *>(ab);
#pragma unroll
            for (unsigned j = 0; j < 4u; ++j) {
                const unsigned *p = reinterpret_cast<const unsigned *>(ab + 4u + 64u * j + 16u * q);
                a[nt][j] = make_uint4(p[0], p[1], p[2], p[3]);
            }
            const unsigned *b = reinterpret_cast<const unsigned *>(ab + 260u);
            bsums[nt][0] = make_uint4(b[0], b[1], b[2], b[3]);
            bsums[nt][1] = make_uint4(b[4], b[5], b[6], b[7]);
        }
        const unsigned s0 = scales.x, s1 = scales.y, s2 = scales.z;
        const unsigned sc_pack[2] = {s0 & 0x3f3f3f3fu, (s2 & 0x0f0f0f0fu) | ((s0 >> 2) & 0x30303030u)};
        const unsigned mn_pack[2] = {s1 & 0x3f3f3f3fu, ((s2 >> 4) & 0x0f0f0f0fu) | ((s1 >> 2) & 0x30303030u)};
        if (q == 0u) {
            row_scale[wave][0][r] = f16_bits_to_float(head & 0xffffu);
            row_scale[wave][1][r] = f16_bits_to_float(head >> 16);
        }
        v4s lo_sum[NT], hi_sum[NT];
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) lo_sum[nt][i] = hi_sum[nt][i] = 0;
        const unsigned high = q >> 1;                          // this lane decodes the high nibbles
#pragma unroll
        for (unsigned j = 0; j < 4u; ++j) {
            // sub-block 2 j + high: its scale is byte (2 j + high) of the packed scales
            const unsigned sc = (sc_pack[j >> 1] >> (16u * (j & 1u) + 8u * high)) & 255u;
            const unsigned shift = 4u * high;
            v4i a_lo, a_hi;
            unsigned lo, hi;
            limbs(qs[j].x >> shift, sc, lo, hi); a_lo[0] = (int)lo; a_hi[0] = (int)hi;
            limbs(qs[j].y >> shift, sc, lo, hi); a_lo[1] = (int)lo; a_hi[1] = (int)hi;
            limbs(qs[j].z >> shift, sc, lo, hi); a_lo[2] = (int)lo; a_hi[2] = (int)hi;
            limbs(qs[j].w >> shift, sc, lo, hi); a_lo[3] = (int)lo; a_hi[3] = (int)hi;
#pragma unroll
            for (unsigned nt = 0; nt < NT; ++nt) {
                const v4i b = as_v4i(a[nt][j]);
                lo_sum[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_lo, b, lo_sum[nt], 0, 0, 0);
                hi_sum[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_hi, b, hi_sum[nt], 0, 0, 0);
            }
        }
        v4i m_op = {0, 0, 0, 0};
        if (q == 0u) {
            m_op[0] = (int)mn_pack[0];
            m_op[1] = (int)mn_pack[1];
        }
        v4s min_lo[NT], min_hi[NT];
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt) {
            uint2 bl, bh;
            bsum_limbs(bsums[nt], bl, bh);
            v4i b_lo = {0, 0, 0, 0}, b_hi = {0, 0, 0, 0};
            if (q == 0u) {
                b_lo[0] = (int)bl.x; b_lo[1] = (int)bl.y;
                b_hi[0] = (int)bh.x; b_hi[1] = (int)bh.y;
            }
            const v4s zero = {0, 0, 0, 0};
            min_lo[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(m_op, b_lo, zero, 0, 0, 0);
            min_hi[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(m_op, b_hi, zero, 0, 0, 0);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const float4 d4 = *reinterpret_cast<const float4 *>(&row_scale[wave][0][4u * q]);
        const float4 m4 = *reinterpret_cast<const float4 *>(&row_scale[wave][1][4u * q]);
        const float d_of[4] = {d4.x, d4.y, d4.z, d4.w}, dmin_of[4] = {m4.x, m4.y, m4.z, m4.w};
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dot = (hi_sum[nt][i] << 3) + lo_sum[nt][i];
                const int minimum = (min_hi[nt][i] << 7) + min_lo[nt][i];
                const float left = (da[nt] * d_of[i]) * (float)dot;
                const float right = (da[nt] * dmin_of[i]) * (float)minimum;
                acc[nt][i] += (double)(left - right);
            }
    }

    if (wave) {
#pragma unroll
        for (unsigned nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) partial[wave - 1u][nt][i][lane] = acc[nt][i];
    }
    __syncthreads();
    if (wave) return;
#pragma unroll
    for (unsigned nt = 0; nt < NT; ++nt) {
        const unsigned long long token = tok0 + 16ull * nt + r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const unsigned long long row = row0 + 4u * q + (unsigned)i;
            double wide = acc[nt][i];
#pragma unroll
            for (unsigned wv = 0; wv < 7u; ++wv) wide += partial[wv][nt][i][lane];
            const float sum = (float)wide;
            if (row >= g.row_count || token >= g.input_rows) continue;
            const unsigned long long at = token * g.out_stride + row;
            const float value = g.additive ? sum + g.additive[at] : sum;
            if (!finite_f32(value)) raise_status(g.status, 1);
            else g.out[at] = g.output_bf16 ? bf16_round(value) : value;
        }
    }
}

}  // namespace

int launch_q4k_rows_dense(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                          uint64_t row_bytes, const void *act_q8k, uint64_t input_rows,
                          const float *additive, float *out, uint64_t out_stride, bool output_bf16,
                          int *status, hipStream_t stream)
{
    if (!row_count || !input_rows || row_width % 256u || row_width / 256u * 144u != row_bytes)
        return ST_BOUNDS;
    if (((uintptr_t)encoded & 15u) || ((uintptr_t)act_q8k & 3u)) return ST_INVALID_ARG;
    const uint64_t row_tiles = (row_count + 31u) / 32u;
    if (row_tiles > 0x7fffffffull || row_width / 256u > 0xffffffffull) return ST_BOUNDS;
    DenseQ4kArgs g{encoded, row_count, row_bytes, (unsigned)(row_width / 256u),
                   (const unsigned char *)act_q8k, input_rows, additive, out, out_stride,
                   output_bf16 ? 1 : 0, status};
    if (input_rows <= 32u) {
        const uint64_t small_tiles = (row_count + 15u) / 16u;
        if (small_tiles > 0x7fffffffull) return ST_BOUNDS;
        if (input_rows <= 16u) dense_q4k16_kernel<1><<<dim3((unsigned)small_tiles, 1), 512, 0, stream>>>(g);
        else dense_q4k16_kernel<2><<<dim3((unsigned)small_tiles, 1), 512, 0, stream>>>(g);
    } else {
        const uint64_t token_tiles = (input_rows + 63u) / 64u;
        if (token_tiles > 65535ull) return ST_BOUNDS;
        // enough (128 rows x 64 tokens) tiles for every compute unit: operands staged through LDS
        if ((row_count + 127u) / 128u * token_tiles >= compute_units())
            return launch_q4k_rows_staged(encoded, row_count, row_width, row_bytes, act_q8k, input_rows,
                                          additive, out, out_stride, output_bf16, status, stream);
        // A workgroup's pass over the row width takes about as long on a full device as on an
        // empty one, so while the smaller tiles still fit the device in one round they are the
        // faster ones (2048 x 7168 at 64 rows: 25 us on 32 x 64 tiles, 17 us on 32 x 32, 16 us on
        // 16 x 32; at 256 rows 29, 33 and 49 us).
        const uint64_t token_tiles32 = (input_rows + 31u) / 32u, small_tiles = (row_count + 15u) / 16u;
        const uint64_t units = (uint64_t)compute_units();
        if (small_tiles * token_tiles32 <= units)
            dense_q4k16_kernel<2><<<dim3((unsigned)small_tiles, (unsigned)token_tiles32), 512, 0, stream>>>(g);
        else if (row_tiles * token_tiles32 <= units)
            dense_q4k_kernel<1><<<dim3((unsigned)row_tiles, (unsigned)token_tiles32), 256, 0, stream>>>(g);
        else
            dense_q4k_kernel<2><<<dim3((unsigned)row_tiles, (unsigned)token_tiles), 256, 0, stream>>>(g);
    }
    return check_launch("dense_q4k");
}

}  // namespace yvex
