// Device-side building blocks shared by every gfx950 kernel of the quantized matmul path:
// scalar conversion rules, the IQ2_XXS lookup tables kept in LDS, and per-qtype "unit"
// decoders that turn 32 packed weights into eight dwords of signed int8.
//
// Reference behaviour restated here: src/backend/cuda/kernel_primitives.h:49-142 (scalar
// rules, sign parity), :274-359 (integer block dots). Wavefronts are 64 lanes wide.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../../include/yvex_iq2xxs_grid.h"

namespace yvex {

constexpr int kWave = 64;
constexpr unsigned kQ8KBytes = 292u;

enum QType : unsigned {
    QT_F32 = 0, QT_F16 = 1, QT_Q8_0 = 8, QT_Q2_K = 10, QT_Q4_K = 12, QT_Q8_K = 15,
    QT_IQ2_XXS = 16, QT_I32 = 26, QT_BF16 = 30, QT_MXFP4 = 39
};

// Kernel status word: 0 ok, 1 non-finite numerics, 2 contract violation
// (same convention as src/backend/cuda/kernels.cu:555-564).
__device__ __forceinline__ void raise_status(int *status, int code)
{
    atomicCAS(status, 0, code);
}

__device__ __forceinline__ float f16_bits_to_float(unsigned bits)
{
    // binary16 -> binary32 is exact for every finite code including subnormals.
    return (float)__builtin_bit_cast(_Float16, (unsigned short)bits);
}

__device__ __forceinline__ float bf16_bits_to_float(unsigned bits)
{
    return __uint_as_float(bits << 16);
}

// Round-to-nearest-even binary32 -> bfloat16, returned widened (kernel_primitives.h:89-99).
__device__ __forceinline__ float bf16_round(float value)
{
    unsigned bits = __float_as_uint(value);
    unsigned upper = bits >> 16, lower = bits & 0xffffu;
    if ((bits & 0x7f800000u) == 0x7f800000u && (bits & 0x007fffffu))
        return __uint_as_float((upper | 0x40u) << 16);
    if (lower > 0x8000u || (lower == 0x8000u && (upper & 1u))) upper++;
    return __uint_as_float(upper << 16);
}

// The same rounding without branches, for values that are not NaN (to nearest, ties to even; a
// value that rounds past the largest finite number becomes infinite, as above).
__device__ __forceinline__ float bf16_round_number(float value)
{
    const unsigned bits = __float_as_uint(value);
    return __uint_as_float((bits + 0x7fffu + ((bits >> 16) & 1u)) & 0xffff0000u);
}

__device__ __forceinline__ bool finite_f32(float v)
{
    return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u;
}

// Router score of a logit in double (src/graph/moe.c:497-537): sigmoid, or the square root of the
// softplus. `sigmoid` is YVEX_HIP_SCORING_SIGMOID of the launch-level header.
__device__ __forceinline__ double route_score(double v, int scoring)
{
    if (scoring == 1)
        return v >= 0.0 ? 1.0 / (1.0 + exp(-v)) : exp(v) / (1.0 + exp(v));
    const double softplus = v > 0.0 ? v + log1p(exp(-v)) : log1p(exp(v));
    return sqrt(softplus);
}

__device__ __forceinline__ unsigned load_u16(const unsigned char *p)
{
    unsigned short v;
    __builtin_memcpy(&v, p, 2);
    return v;
}
__device__ __forceinline__ unsigned load_u32(const unsigned char *p)
{
    unsigned v;
    __builtin_memcpy(&v, p, 4);   // global loads may be 2-byte aligned; the hardware allows it
    return v;
}
__device__ __forceinline__ uint2 load_u32x2(const unsigned char *p)
{
    uint2 v;
    __builtin_memcpy(&v, p, 8);
    return v;
}

__device__ __forceinline__ int dot4(unsigned a, unsigned b, int acc)
{
    return __builtin_amdgcn_sdot4((int)a, (int)b, acc, false);
}

// ---- wave-wide reductions (64 lanes) -------------------------------------------------------
//
// Sums over aligned groups of WIDTH lanes, returned in every lane of the group. Steps inside a
// row of 16 lanes are data-parallel-primitive moves that run at ALU rate (no LDS crossbar);
// the two steps that cross rows use the row broadcasts and a scalar read-back.

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_move(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xf, false);
}

template <int WIDTH>
__device__ __forceinline__ int group_sum_i32(int v)
{
    static_assert(WIDTH == 1 || WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16 ||
                  WIDTH == 32 || WIDTH == 64, "power of two up to the wave");
    if constexpr (WIDTH >= 2) v += dpp_move<0xb1, 0xf>(v);    // quad_perm [1,0,3,2]
    if constexpr (WIDTH >= 4) v += dpp_move<0x4e, 0xf>(v);    // quad_perm [2,3,0,1]
    if constexpr (WIDTH >= 8) v += dpp_move<0x141, 0xf>(v);   // row_half_mirror
    if constexpr (WIDTH >= 16) v += dpp_move<0x140, 0xf>(v);  // row_mirror
    if constexpr (WIDTH >= 32) v += dpp_move<0x142, 0xa>(v);  // row_bcast15 into rows 1 and 3
    if constexpr (WIDTH == 64) {
        v += dpp_move<0x143, 0xc>(v);                          // row_bcast31 into rows 2 and 3
        v = __builtin_amdgcn_readlane(v, 63);
    } else if constexpr (WIDTH == 32) {
        const int low = __builtin_amdgcn_readlane(v, 31), high = __builtin_amdgcn_readlane(v, 63);
        v = (threadIdx.x & 32u) ? high : low;
    }
    return v;
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move_f32(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf,
                                                      false));
}

template <int WIDTH>
__device__ __forceinline__ float group_sum_f32(float v)
{
    static_assert(WIDTH == 1 || WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16 ||
                  WIDTH == 32 || WIDTH == 64, "power of two up to the wave");
    if constexpr (WIDTH >= 2) v += dpp_move_f32<0xb1, 0xf>(v);
    if constexpr (WIDTH >= 4) v += dpp_move_f32<0x4e, 0xf>(v);
    if constexpr (WIDTH >= 8) v += dpp_move_f32<0x141, 0xf>(v);
    if constexpr (WIDTH >= 16) v += dpp_move_f32<0x140, 0xf>(v);
    if constexpr (WIDTH >= 32) v += dpp_move_f32<0x142, 0xa>(v);
    if constexpr (WIDTH == 64) {
        v += dpp_move_f32<0x143, 0xc>(v);
        v = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
    } else if constexpr (WIDTH == 32) {
        const int low = __builtin_amdgcn_readlane(__float_as_int(v), 31);
        const int high = __builtin_amdgcn_readlane(__float_as_int(v), 63);
        v = __int_as_float((threadIdx.x & 32u) ? high : low);
    }
    return v;
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_move_f64(double v)
{
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, ROW_MASK, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, ROW_MASK, 0xf, false);
    return __hiloint2double(hi, lo);
}

// Double-precision sum over aligned groups of WIDTH lanes, valid in the LAST lane of every group
// (the other lanes hold partial sums).
template <int WIDTH>
__device__ __forceinline__ double group_sum_f64_last(double v)
{
    static_assert(WIDTH == 1 || WIDTH == 2 || WIDTH == 4 || WIDTH == 8 || WIDTH == 16 ||
                  WIDTH == 32 || WIDTH == 64, "power of two up to the wave");
    if constexpr (WIDTH >= 2) v += dpp_move_f64<0xb1, 0xf>(v);
    if constexpr (WIDTH >= 4) v += dpp_move_f64<0x4e, 0xf>(v);
    if constexpr (WIDTH >= 8) v += dpp_move_f64<0x141, 0xf>(v);
    if constexpr (WIDTH >= 16) v += dpp_move_f64<0x140, 0xf>(v);
    if constexpr (WIDTH >= 32) v += dpp_move_f64<0x142, 0xa>(v);   // rows 1 and 3 take rows 0 and 2
    if constexpr (WIDTH == 64) v += dpp_move_f64<0x143, 0xc>(v);   // rows 2 and 3 take row 1
    return v;
}

// Same with the width known only at run time (wave-uniform).
__device__ __forceinline__ float group_sum_f32_dynamic(float v, unsigned width)
{
    switch (width) {
    case 2: return group_sum_f32<2>(v);
    case 4: return group_sum_f32<4>(v);
    case 8: return group_sum_f32<8>(v);
    case 16: return group_sum_f32<16>(v);
    case 32: return group_sum_f32<32>(v);
    case 64: return group_sum_f32<64>(v);
    default: return v;
    }
}

// ---- IQ2_XXS lookup tables in LDS ----------------------------------------------------------
//
// magnitudes[idx] : eight bytes (8/25/43) for codebook entry idx, 2 KB.
// signmask[s7]    : eight bytes 0xff/0x00 for the 7 stored sign bits plus the parity bit, 1 KB.
// A signed int8x4 is (magnitude ^ mask) + (mask & 0x01010101): every magnitude is >= 8, so the
// +1 never carries into the next byte.

__constant__ unsigned short k_iq2_digits[256] = {YVEX_IQ2XXS_GRID_VALUES};

struct Iq2Tables {
    uint2 magnitudes[256];
    uint2 signmask[128];
    // magnitudes, byte masks and the +1 bytes of subgroup j of one 32-weight group
    __device__ __forceinline__ void lookup(unsigned grids, unsigned aux, unsigned j, uint2 &m,
                                           uint2 &mask, uint2 &one) const
    {
        m = magnitudes[(grids >> (8u * j)) & 255u];
        mask = signmask[(aux >> (7u * j)) & 127u];
        one = make_uint2(mask.x & 0x01010101u, mask.y & 0x01010101u);
    }
};

// The eight levels of a codebook entry from its sixteen digit bits.
__device__ __forceinline__ uint2 iq2_magnitude_of_digits(unsigned digits)
{
    unsigned lo = 0u, hi = 0u;
#pragma unroll
    for (unsigned l = 0; l < 4u; ++l) {
        const unsigned a = (digits >> (2u * l)) & 3u, b = (digits >> (2u * l + 8u)) & 3u;
        lo |= (a == 0u ? 8u : a == 1u ? 25u : 43u) << (8u * l);
        hi |= (b == 0u ? 8u : b == 1u ? 25u : 43u) << (8u * l);
    }
    return make_uint2(lo, hi);
}

__device__ __forceinline__ uint2 iq2_magnitude_entry(unsigned i)
{
    return iq2_magnitude_of_digits(k_iq2_digits[i]);
}

__device__ __forceinline__ uint2 iq2_signmask_entry(unsigned i)
{
    const unsigned s = i | ((__popc(i) & 1u) << 7);
    unsigned lo = 0u, hi = 0u;
#pragma unroll
    for (unsigned l = 0; l < 4u; ++l) {
        if ((s >> l) & 1u) lo |= 0xffu << (8u * l);
        if ((s >> (l + 4u)) & 1u) hi |= 0xffu << (8u * l);
    }
    return make_uint2(lo, hi);
}

__device__ __forceinline__ void iq2_tables_fill(Iq2Tables &t)
{
    for (unsigned i = threadIdx.x; i < 256u; i += blockDim.x) t.magnitudes[i] = iq2_magnitude_entry(i);
    for (unsigned i = threadIdx.x; i < 128u; i += blockDim.x) t.signmask[i] = iq2_signmask_entry(i);
}

// The same tables replicated 32 times for the persistent kernels. Replica r of entry e sits at
// [e * 32 + r] and a lane always reads replica (lane % 32), so the 32 lanes of a half-wave hit
// 32 different bank groups whatever entries they ask for: random lookups never conflict.
// Layout in LDS (128 KB of the CU's 160 KB):
//   [0, 64 KB)      magnitudes: 256 entries x 32 replicas x 8 bytes
//   [64 KB, 128 KB) signs:      128 entries x 32 replicas x 16 bytes {mask.x, mask.y, one.x, one.y}
// Byte addresses are assembled with one byte-permute (magnitudes) or one shift-or (signs).
constexpr unsigned kIq2Replicas = 32u;
constexpr unsigned kIq2SignBase = 256u * kIq2Replicas * 8u;
constexpr unsigned kIq2WideBytes = kIq2SignBase + 128u * kIq2Replicas * 16u;

// LDS reads by byte address. The host pass of the compiler never executes these.
__device__ __forceinline__ uint2 lds_read_uint2(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const uint2 *>(address);
#else
    (void)address;
    return make_uint2(0u, 0u);
#endif
}
__device__ __forceinline__ uint4 lds_read_uint4(unsigned address)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<__attribute__((address_space(3))) const uint4 *>(address);
#else
    (void)address;
    return make_uint4(0u, 0u, 0u, 0u);
#endif
}
__device__ __forceinline__ unsigned lds_address_of(const void *shared_pointer)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return (unsigned)(size_t)(__attribute__((address_space(3))) const void *)shared_pointer;
#else
    (void)shared_pointer;
    return 0u;
#endif
}

struct Iq2TablesWide {
    unsigned lane_magnitude;   // (lane % 32) * 8
    unsigned lane_sign;        // kIq2SignBase + (lane % 32) * 16
    __device__ __forceinline__ void lookup(unsigned grids, unsigned aux, unsigned j, uint2 &m,
                                           uint2 &mask, uint2 &one) const
    {
        // The tables start at LDS address 0, so these byte offsets are LDS addresses.
        // magnitude address = (index byte j) << 8 | lane offset: bytes {lane, index, 0, 0}
        const unsigned ma = __builtin_amdgcn_perm(grids, lane_magnitude, 0x0c0c0400u + (j << 8));
        // sign address = field j (7 bits at bit 7j) moved to bit 9, or-ed with the lane offset
        const unsigned moved = 7u * j >= 9u ? aux >> (7u * j - 9u) : aux << (9u - 7u * j);
        const unsigned sa = (moved & 0xfe00u) | lane_sign;
        m = lds_read_uint2(ma);
        const uint4 s = lds_read_uint4(sa);
        mask = make_uint2(s.x, s.y);
        one = make_uint2(s.z, s.w);
    }
};

__device__ __forceinline__ Iq2TablesWide iq2_tables_wide_fill(unsigned char *lds)
{
    uint2 *mag = reinterpret_cast<uint2 *>(lds);
    uint4 *sgn = reinterpret_cast<uint4 *>(lds + kIq2SignBase);
    for (unsigned i = threadIdx.x; i < 256u * kIq2Replicas; i += blockDim.x)
        mag[i] = iq2_magnitude_entry(i / kIq2Replicas);
    for (unsigned i = threadIdx.x; i < 128u * kIq2Replicas; i += blockDim.x) {
        const uint2 m = iq2_signmask_entry(i / kIq2Replicas);
        sgn[i] = make_uint4(m.x, m.y, m.x & 0x01010101u, m.y & 0x01010101u);
    }
    const unsigned replica = threadIdx.x & (kIq2Replicas - 1u);
    return Iq2TablesWide{replica * 8u, kIq2SignBase + replica * 16u};
}

// 32 weights of one IQ2_XXS group -> eight int8x4 dwords; returns the odd factor 2s+1.
// A signed byte is (magnitude ^ mask) + one: magnitudes are >= 8 so the +1 never carries.
template <typename Tables>
__device__ __forceinline__ int iq2_unit(const Tables &t, unsigned grids, unsigned aux,
                                        unsigned w[8])
{
#pragma unroll
    for (unsigned j = 0; j < 4u; ++j) {
        uint2 m, mask, one;
        t.lookup(grids, aux, j, m, mask, one);
        w[2 * j] = (m.x ^ mask.x) + one.x;
        w[2 * j + 1] = (m.y ^ mask.y) + one.y;
    }
    return (int)(2u * (aux >> 28) + 1u);
}

// Same group decoded straight from the 2-bit digits, for kernels without the LDS tables.
__device__ __forceinline__ int iq2_level(unsigned digits, unsigned signs, unsigned l)
{
    unsigned d = (digits >> (2u * l)) & 3u;
    int level = d == 0u ? 8 : d == 1u ? 25 : 43;
    return (signs >> l) & 1u ? -level : level;
}
__device__ __forceinline__ unsigned iq2_sign_byte(unsigned low7)
{
    return low7 | ((__popc(low7) & 1u) << 7);
}

// ---- Q4_K helpers (public ggml block_q4_K: f16 d, f16 dmin, 12 scale bytes, 128 nibble bytes)

__device__ __forceinline__ void q4k_scale_min(const unsigned char *scales, unsigned j,
                                              unsigned &sc, unsigned &mn)
{
    if (j < 4u) {
        sc = scales[j] & 63u;
        mn = scales[j + 4u] & 63u;
    } else {
        sc = (scales[j + 4u] & 15u) | ((scales[j - 4u] >> 6) << 4);
        mn = (scales[j + 4u] >> 4) | ((scales[j] >> 6) << 4);
    }
}

// ---- per-element decode, used by gather / row decode and as the slow exact path ------------
// Mirrors qtype_value (kernel_primitives.h:143-217) for the admitted qtypes; NaN otherwise.
__device__ inline float qtype_value(const unsigned char *row, unsigned long long index,
                                    unsigned qtype)
{
    switch (qtype) {
    case QT_F32: return __uint_as_float(load_u32(row + index * 4ull));
    case QT_F16: return f16_bits_to_float(load_u16(row + index * 2ull));
    case QT_BF16: return bf16_bits_to_float(load_u16(row + index * 2ull));
    case QT_I32: return (float)(int)load_u32(row + index * 4ull);
    case QT_Q8_0: {
        const unsigned char *b = row + (index >> 5) * 34ull;
        return f16_bits_to_float(load_u16(b)) * (float)(signed char)b[2u + (index & 31u)];
    }
    case QT_IQ2_XXS: {
        const unsigned char *b = row + (index >> 8) * 66ull;
        unsigned in = (unsigned)(index & 255u), g = in >> 5, j = (in >> 3) & 3u, l = in & 7u;
        unsigned grids = load_u32(b + 2u + 8u * g), aux = load_u32(b + 6u + 8u * g);
        float gs = f16_bits_to_float(load_u16(b)) * (0.5f + (float)(aux >> 28)) * 0.25f;
        int level = iq2_level(k_iq2_digits[(grids >> (8u * j)) & 255u],
                              iq2_sign_byte((aux >> (7u * j)) & 127u), l);
        return gs * (float)(level < 0 ? -level : level) * (level < 0 ? -1.0f : 1.0f);
    }
    case QT_Q4_K: {
        const unsigned char *b = row + (index >> 8) * 144ull;
        unsigned in = (unsigned)(index & 255u), j = in >> 5, l = in & 31u, sc, mn;
        unsigned byte = b[16u + 32u * (j >> 1) + l];
        q4k_scale_min(b + 4u, j, sc, mn);
        float d = f16_bits_to_float(load_u16(b)) * (float)sc;
        float m = f16_bits_to_float(load_u16(b + 2u)) * (float)mn;
        return d * (float)((j & 1u) ? byte >> 4 : byte & 15u) - m;
    }
    case QT_Q2_K: {
        const unsigned char *b = row + (index >> 8) * 84ull;
        unsigned in = (unsigned)(index & 255u), sub = in >> 4, lane = in & 15u;
        unsigned shift = ((sub & 7u) >> 1) * 2u;
        unsigned code = (b[16u + (sub >> 3) * 32u + (sub & 1u) * 16u + lane] >> shift) & 3u;
        float scale = f16_bits_to_float(load_u16(b + 80u)) * (float)(b[sub] & 15u);
        float minimum = f16_bits_to_float(load_u16(b + 82u)) * (float)(b[sub] >> 4);
        return scale * (float)code - minimum;
    }
    default: return __uint_as_float(0x7fc00000u);
    }
}

__host__ __device__ inline bool qtype_geometry(unsigned qtype, unsigned &block, unsigned &bytes)
{
    switch (qtype) {
    case QT_F32: block = 1; bytes = 4; return true;
    case QT_F16: case QT_BF16: block = 1; bytes = 2; return true;
    case QT_I32: block = 1; bytes = 4; return true;
    case QT_Q8_0: block = 32; bytes = 34; return true;
    case QT_Q2_K: block = 256; bytes = 84; return true;
    case QT_Q4_K: block = 256; bytes = 144; return true;
    case QT_IQ2_XXS: block = 256; bytes = 66; return true;
    default: block = 0; bytes = 0; return false;
    }
}

}  // namespace yvex
