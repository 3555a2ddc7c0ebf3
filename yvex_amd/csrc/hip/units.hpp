// Per-qtype "unit" arithmetic: one unit is 32 consecutive weights of a row (one IQ2_XXS group,
// one Q8_0 block, one Q4_K sub-block, two Q2_K sub-blocks). Eight units make one 256-value
// superblock, which pairs with exactly one Q8_K activation block.
//
// Integer definitions follow src/backend/cuda/kernel_primitives.h:287-359; the int32 results
// are exact, so they equal the CPU restatement bit for bit whatever the lane mapping.
#pragma once

#include "common.hpp"

namespace yvex {

// Integer partial of one unit against one Q8_K block: x = scaled dot, y = scaled min-sum.
struct UnitSum {
    int dot;
    int min;
};

template <unsigned QT>
struct UnitTraits;

template <>
struct UnitTraits<QT_IQ2_XXS> {
    static constexpr unsigned kSuperBytes = 66u;
    static constexpr bool kIntegerCombine = true;   // ints reduce across the superblock first
};
template <>
struct UnitTraits<QT_Q4_K> {
    static constexpr unsigned kSuperBytes = 144u;
    static constexpr bool kIntegerCombine = true;
};
template <>
struct UnitTraits<QT_Q2_K> {
    static constexpr unsigned kSuperBytes = 84u;
    static constexpr bool kIntegerCombine = true;
};
template <>
struct UnitTraits<QT_Q8_0> {
    static constexpr unsigned kSuperBytes = 272u;   // eight 34-byte blocks
    static constexpr bool kIntegerCombine = false;  // every unit carries its own f16 scale
};

// Decoded unit: eight int8x4 dwords plus what scales them.
struct Unit {
    unsigned w[8];
    int factor;      // IQ2_XXS 2s+1; Q4_K sc; Q2_K sc of the first 16 values
    int factor2;     // Q2_K sc of the second 16 values (else = factor)
    int min1, min2;  // Q4_K: m (min2 = m); Q2_K: m of each half; else 0
    unsigned scale_bits;  // Q8_0: the block's fp16 scale, taken from the dwords loaded for the codes
};

// EVEN: 1 = the caller knows the row starts on an even address, 0 = it does not, -1 = look.
template <unsigned QT, int EVEN = -1>
__device__ __forceinline__ void unit_load(const Iq2Tables &tables, const unsigned char *row,
                                          unsigned u, Unit &unit)
{
    const bool even = EVEN < 0 ? ((unsigned long long)row & 1ull) == 0ull : EVEN != 0;
    const unsigned sb = u >> 3, g = u & 7u;
    // Group records and Q8_0 blocks start on 2-byte boundaries, and vector loads that are not
    // dword-aligned run at under half rate on this part: load the aligned dwords that hold the
    // bytes and shift them into place. A dword is only read when it holds a byte of the record
    // (so it lies in a mapped page); rows on odd addresses take the byte-granular path.
    if constexpr (QT == QT_IQ2_XXS) {
        const unsigned char *p = row + sb * 66u + 2u + 8u * g;
        uint2 packed;
        if (even) {
            const unsigned shift = (unsigned)(unsigned long long)p & 3u;       // 0 or 2
            const unsigned char *at = p - shift;
            const uint2 head = *reinterpret_cast<const uint2 *>(at);
            const unsigned tail = *reinterpret_cast<const unsigned *>(at + 4u + 2u * shift);
            packed.x = __builtin_amdgcn_alignbyte(head.y, head.x, shift);
            packed.y = __builtin_amdgcn_alignbyte(tail, head.y, shift);
        } else {
            packed = load_u32x2(p);
        }
        unit.factor = unit.factor2 = iq2_unit(tables, packed.x, packed.y, unit.w);
        unit.min1 = unit.min2 = 0;
    } else if constexpr (QT == QT_Q8_0) {
        const unsigned char *b = row + u * 34u + 2u;
        if (even) {
            const unsigned shift = (unsigned)(unsigned long long)b & 3u;       // 0 or 2
            const unsigned char *at = b - shift;
            const uint4 lo = *reinterpret_cast<const uint4 *>(at);
            const uint4 hi = *reinterpret_cast<const uint4 *>(at + 16u);
            // Ninth dword: with the codes two bytes into their window it holds their last two
            // bytes, and the scale is the low half of the first dword; with the codes aligned
            // the eight dwords are complete and the ninth is the dword before them, whose high
            // half is the scale (for the first block of a row that dword may lie before the
            // tensor, so that one block reads its scale on its own).
            const bool before = shift == 0u && u != 0u;
            const unsigned tail = *reinterpret_cast<const unsigned *>(shift ? at + 32u : before ? at - 4u : at);
            const unsigned raw[9] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w, tail};
#pragma unroll
            for (int i = 0; i < 8; ++i) unit.w[i] = __builtin_amdgcn_alignbyte(raw[i + 1], raw[i], shift);
            unit.scale_bits = shift ? (lo.x & 0xffffu) : before ? (tail >> 16) : (unsigned)load_u16(b - 2u);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint2 v = load_u32x2(b + 8 * i);
                unit.w[2 * i] = v.x;
                unit.w[2 * i + 1] = v.y;
            }
            unit.scale_bits = load_u16(b - 2u);
        }
        unit.factor = unit.factor2 = 1;
        unit.min1 = unit.min2 = 0;
    } else if constexpr (QT == QT_Q4_K) {
        const unsigned char *b = row + sb * 144u;
        uint4 lo, hi;
        __builtin_memcpy(&lo, b + 16u + 32u * (g >> 1), 16);
        __builtin_memcpy(&hi, b + 32u + 32u * (g >> 1), 16);
        unsigned v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        const unsigned shift = (g & 1u) * 4u;
#pragma unroll
        for (int i = 0; i < 8; ++i) unit.w[i] = (v[i] >> shift) & 0x0f0f0f0fu;
        unsigned sc, mn;
        q4k_scale_min(b + 4u, g, sc, mn);
        unit.factor = unit.factor2 = (int)sc;
        unit.min1 = unit.min2 = (int)mn;
    } else if constexpr (QT == QT_Q2_K) {
        const unsigned char *b = row + sb * 84u;
        const unsigned char *q = b + 16u + (g >> 2) * 32u;
        const unsigned shift = 2u * (g & 3u);
#pragma unroll
        for (int i = 0; i < 8; ++i) unit.w[i] = (load_u32(q + 4 * i) >> shift) & 0x03030303u;
        unit.factor = b[2u * g] & 15u;
        unit.factor2 = b[2u * g + 1u] & 15u;
        unit.min1 = b[2u * g] >> 4;
        unit.min2 = b[2u * g + 1u] >> 4;
    }
}

// ---- a lane's share of one weight row, loaded first and decoded later -----------------------
//
// The grouped kernels give every lane four consecutive units (half a superblock) of each weight
// row. LaneChunk keeps those packed bytes in registers so all loads of an iteration can be in
// flight before the first decode starts.

template <unsigned QT>
struct LaneChunk;

template <>
struct LaneChunk<QT_IQ2_XXS> {
    unsigned q[8];
    unsigned d16;
    __device__ __forceinline__ void load(const unsigned char *row, unsigned unit0)
    {
        const unsigned char *b = row + (unit0 >> 3) * 66u;
        uint4 lo, hi;
        d16 = load_u16(b);
        __builtin_memcpy(&lo, b + 2u + 8u * (unit0 & 7u), 16);
        __builtin_memcpy(&hi, b + 18u + 8u * (unit0 & 7u), 16);
        q[0] = lo.x; q[1] = lo.y; q[2] = lo.z; q[3] = lo.w;
        q[4] = hi.x; q[5] = hi.y; q[6] = hi.z; q[7] = hi.w;
    }
    template <typename Tables>
    __device__ __forceinline__ void decode(const Tables &t, int k, unsigned, Unit &unit) const
    {
        unit.factor = unit.factor2 = iq2_unit(t, q[2 * k], q[2 * k + 1], unit.w);
        unit.min1 = unit.min2 = 0;
    }
    __device__ __forceinline__ float combine(float act_scale, UnitSum sum) const
    {
        return 0.125f * f16_bits_to_float(d16) * act_scale * (float)sum.dot;
    }
};

template <>
struct LaneChunk<QT_Q4_K> {
    unsigned q[16];     // two 32-byte nibble chunks
    unsigned head[4];   // f16 d, f16 dmin, 12 scale bytes
    __device__ __forceinline__ void load(const unsigned char *row, unsigned unit0)
    {
        const unsigned char *b = row + (unit0 >> 3) * 144u;
        uint4 v;
        __builtin_memcpy(&v, b, 16);
        head[0] = v.x; head[1] = v.y; head[2] = v.z; head[3] = v.w;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            __builtin_memcpy(&v, b + 16u + 32u * ((unit0 & 7u) >> 1) + 16u * i, 16);
            q[4 * i] = v.x; q[4 * i + 1] = v.y; q[4 * i + 2] = v.z; q[4 * i + 3] = v.w;
        }
    }
    // Unit k of the lane's four (unit0 is a multiple of four: the lane owns the first or the
    // second half of the superblock). The 6-bit scale and minimum of unit g are, for g < 4, the
    // low bits of scale bytes g and g + 4, and for g >= 4 the nibbles of byte g + 4 with the top
    // bits of bytes g - 4 and g (public ggml block_q4_K). With k a constant every byte sits at a
    // fixed place of the header words, and which half the lane owns is a select, not a branch
    // over an indexed array.
    template <typename Tables>
    __device__ __forceinline__ void decode(const Tables &, int k, unsigned unit0, Unit &unit) const
    {
        const bool second = (unit0 & 4u) != 0u;
        const unsigned shift = ((unsigned)k & 1u) * 4u;
#pragma unroll
        for (int i = 0; i < 8; ++i) unit.w[i] = (q[8 * (k >> 1) + i] >> shift) & 0x0f0f0f0fu;
        const unsigned s0 = (head[1] >> (8u * k)) & 255u, s1 = (head[2] >> (8u * k)) & 255u,
                       s2 = (head[3] >> (8u * k)) & 255u;
        const unsigned sc = second ? (s2 & 15u) | ((s0 >> 6) << 4) : s0 & 63u;
        const unsigned mn = second ? (s2 >> 4) | ((s1 >> 6) << 4) : s1 & 63u;
        unit.factor = unit.factor2 = (int)sc;
        unit.min1 = unit.min2 = (int)mn;
    }
    __device__ __forceinline__ float combine(float act_scale, UnitSum sum) const
    {
        const float left = act_scale * f16_bits_to_float(head[0] & 0xffffu) * (float)sum.dot;
        const float right = act_scale * f16_bits_to_float(head[0] >> 16) * (float)sum.min;
        return left - right;
    }
};

template <>
struct LaneChunk<QT_Q2_K> {
    unsigned q[8];       // one 32-byte plane chunk shared by the lane's four units
    unsigned scales[2];  // eight scale/min bytes
    unsigned dd;         // f16 d, f16 dmin
    __device__ __forceinline__ void load(const unsigned char *row, unsigned unit0)
    {
        const unsigned char *b = row + (unit0 >> 3) * 84u;
        uint4 lo, hi;
        __builtin_memcpy(&lo, b + 16u + ((unit0 & 7u) >> 2) * 32u, 16);
        __builtin_memcpy(&hi, b + 32u + ((unit0 & 7u) >> 2) * 32u, 16);
        q[0] = lo.x; q[1] = lo.y; q[2] = lo.z; q[3] = lo.w;
        q[4] = hi.x; q[5] = hi.y; q[6] = hi.z; q[7] = hi.w;
        uint2 sc = load_u32x2(b + 2u * (unit0 & 7u));
        scales[0] = sc.x;
        scales[1] = sc.y;
        dd = load_u32(b + 80u);
    }
    template <typename Tables>
    __device__ __forceinline__ void decode(const Tables &, int k, unsigned, Unit &unit) const
    {
        const unsigned shift = 2u * (unsigned)k;   // unit0 & 3 == 0
#pragma unroll
        for (int i = 0; i < 8; ++i) unit.w[i] = (q[i] >> shift) & 0x03030303u;
        const unsigned pair = (scales[k >> 1] >> (16u * (k & 1))) & 0xffffu;
        unit.factor = pair & 15u;
        unit.min1 = (pair >> 4) & 15u;
        unit.factor2 = (pair >> 8) & 15u;
        unit.min2 = pair >> 12;
    }
    __device__ __forceinline__ float combine(float act_scale, UnitSum sum) const
    {
        const float left = act_scale * f16_bits_to_float(dd & 0xffffu) * (float)sum.dot;
        const float right = act_scale * f16_bits_to_float(dd >> 16) * (float)sum.min;
        return left - right;
    }
};

template <>
struct LaneChunk<QT_Q8_0> {
    unsigned q[32];
    unsigned d16[4];
    __device__ __forceinline__ void load(const unsigned char *row, unsigned unit0)
    {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const unsigned char *b = row + (unit0 + k) * 34u;
            uint4 lo, hi;
            d16[k] = load_u16(b);
            __builtin_memcpy(&lo, b + 2u, 16);
            __builtin_memcpy(&hi, b + 18u, 16);
            q[8 * k] = lo.x; q[8 * k + 1] = lo.y; q[8 * k + 2] = lo.z; q[8 * k + 3] = lo.w;
            q[8 * k + 4] = hi.x; q[8 * k + 5] = hi.y; q[8 * k + 6] = hi.z; q[8 * k + 7] = hi.w;
        }
    }
    template <typename Tables>
    __device__ __forceinline__ void decode(const Tables &, int k, unsigned, Unit &unit) const
    {
#pragma unroll
        for (int i = 0; i < 8; ++i) unit.w[i] = q[8 * k + i];
        unit.factor = unit.factor2 = 1;
        unit.min1 = unit.min2 = 0;
    }
    __device__ __forceinline__ float unit_scale(int k) const { return f16_bits_to_float(d16[k]); }
    __device__ __forceinline__ float combine(float, UnitSum) const { return 0.0f; }
};

// Unit against Q8_K block `act` (292 bytes, 4-byte aligned); g = unit index inside the block.
template <unsigned QT>
__device__ __forceinline__ UnitSum unit_dot_q8(const Unit &unit, const unsigned char *act,
                                               unsigned g)
{
    const unsigned *a = reinterpret_cast<const unsigned *>(act + 4u + 32u * g);
    UnitSum out;
    if constexpr (QT == QT_Q2_K) {
        int d1 = 0, d2 = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            d1 = dot4(unit.w[i], a[i], d1);
            d2 = dot4(unit.w[4 + i], a[4 + i], d2);
        }
        const short *bs = reinterpret_cast<const short *>(act + 260u);
        out.dot = unit.factor * d1 + unit.factor2 * d2;
        out.min = unit.min1 * (int)bs[2u * g] + unit.min2 * (int)bs[2u * g + 1u];
    } else {
        int d = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) d = dot4(unit.w[i], a[i], d);
        out.dot = unit.factor * d;
        if constexpr (QT == QT_Q4_K) {
            const short *bs = reinterpret_cast<const short *>(act + 260u);
            out.min = unit.min1 * ((int)bs[2u * g] + (int)bs[2u * g + 1u]);
        } else {
            out.min = 0;
        }
    }
    return out;
}

// Float value of one superblock from its exact integer sums, float operations in the order
// the reference's device primitives use (kernel_primitives.h:312, :336-340).
template <unsigned QT>
__device__ __forceinline__ float super_combine(const unsigned char *super, float act_scale,
                                               UnitSum sum)
{
    if constexpr (QT == QT_IQ2_XXS) {
        return 0.125f * f16_bits_to_float(load_u16(super)) * act_scale * (float)sum.dot;
    } else if constexpr (QT == QT_Q4_K) {
        float left = act_scale * f16_bits_to_float(load_u16(super)) * (float)sum.dot;
        float right = act_scale * f16_bits_to_float(load_u16(super + 2u)) * (float)sum.min;
        return left - right;
    } else if constexpr (QT == QT_Q2_K) {
        float left = act_scale * f16_bits_to_float(load_u16(super + 80u)) * (float)sum.dot;
        float right = act_scale * f16_bits_to_float(load_u16(super + 82u)) * (float)sum.min;
        return left - right;
    } else {
        return 0.0f;
    }
}

// Q8_0: every unit scales itself (kernel_primitives.h:353-357).
__device__ __forceinline__ float q8_0_unit_value(const Unit &unit, float act_scale, int dot)
{
    return f16_bits_to_float((unsigned short)unit.scale_bits) * act_scale * (float)dot;
}

// Unit against 32 F32 activations. Returns the unit's contribution to the row dot.
template <unsigned QT>
__device__ __forceinline__ float unit_dot_f32_values(const Unit &unit, const unsigned char *row,
                                                     unsigned u, const float4 (&x4)[8])
{
    const unsigned sb = u >> 3;
    float s1 = 0.0f, s2 = 0.0f, xs1 = 0.0f, xs2 = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 v = x4[i];
        const unsigned w = unit.w[i];
        float p = 0.0f;
        p = fmaf((float)(signed char)(w & 255u), v.x, p);
        p = fmaf((float)(signed char)((w >> 8) & 255u), v.y, p);
        p = fmaf((float)(signed char)((w >> 16) & 255u), v.z, p);
        p = fmaf((float)(signed char)(w >> 24), v.w, p);
        if (i < 4) s1 += p; else s2 += p;
        if constexpr (QT == QT_Q4_K || QT == QT_Q2_K) {
            const float xs = (v.x + v.y) + (v.z + v.w);
            if (i < 4) xs1 += xs; else xs2 += xs;
        }
    }
    if constexpr (QT == QT_IQ2_XXS) {
        const unsigned char *b = row + sb * 66u;
        float gs = f16_bits_to_float(load_u16(b)) * (0.5f + (float)((unit.factor - 1) >> 1)) * 0.25f;
        return gs * (s1 + s2);
    } else if constexpr (QT == QT_Q8_0) {
        // its own 2-byte load: with F32 activations the scale is needed late and this form measured faster
        return f16_bits_to_float(load_u16(row + u * 34u)) * (s1 + s2);
    } else if constexpr (QT == QT_Q4_K) {
        const unsigned char *b = row + sb * 144u;
        float d = f16_bits_to_float(load_u16(b)) * (float)unit.factor;
        float m = f16_bits_to_float(load_u16(b + 2u)) * (float)unit.min1;
        return d * (s1 + s2) - m * (xs1 + xs2);
    } else {
        const unsigned char *b = row + sb * 84u;
        float d = f16_bits_to_float(load_u16(b + 80u)), dm = f16_bits_to_float(load_u16(b + 82u));
        return (d * (float)unit.factor * s1 - dm * (float)unit.min1 * xs1) +
               (d * (float)unit.factor2 * s2 - dm * (float)unit.min2 * xs2);
    }
}

template <unsigned QT>
__device__ __forceinline__ float unit_dot_f32(const Unit &unit, const unsigned char *row,
                                              unsigned u, const float *x)
{
    float4 x4[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) x4[i] = *reinterpret_cast<const float4 *>(x + 4 * i);
    return unit_dot_f32_values<QT>(unit, row, u, x4);
}

// Partial sums of one decoded unit against 32 F32 activations: halves of 16 values each, and
// (for the affine qtypes) the matching sums of the activations themselves.
struct UnitF32 {
    float s1, s2, xs1, xs2;
};

template <bool AFFINE>
__device__ __forceinline__ UnitF32 unit_dot_f32_core(const Unit &unit, const float *x)
{
    UnitF32 r{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 v = *reinterpret_cast<const float4 *>(x + 4 * i);
        const unsigned w = unit.w[i];
        float p = 0.0f;
        p = fmaf((float)(signed char)(w & 255u), v.x, p);
        p = fmaf((float)(signed char)((w >> 8) & 255u), v.y, p);
        p = fmaf((float)(signed char)((w >> 16) & 255u), v.z, p);
        p = fmaf((float)(signed char)(w >> 24), v.w, p);
        if (i < 4) r.s1 += p; else r.s2 += p;
        if constexpr (AFFINE) {
            const float xs = (v.x + v.y) + (v.z + v.w);
            if (i < 4) r.xs1 += xs; else r.xs2 += xs;
        }
    }
    return r;
}

// Contribution of unit k of a LaneChunk to the row dot with F32 activations x (32 floats).
template <unsigned QT>
__device__ __forceinline__ float chunk_unit_dot_f32(const LaneChunk<QT> &c, int k, const Unit &unit,
                                                    const float *x)
{
    const UnitF32 r = unit_dot_f32_core<QT == QT_Q4_K || QT == QT_Q2_K>(unit, x);
    if constexpr (QT == QT_IQ2_XXS) {
        const float gs = f16_bits_to_float(c.d16) * (0.5f + (float)((unit.factor - 1) >> 1)) * 0.25f;
        return gs * (r.s1 + r.s2);
    } else if constexpr (QT == QT_Q8_0) {
        return f16_bits_to_float(c.d16[k]) * (r.s1 + r.s2);
    } else if constexpr (QT == QT_Q4_K) {
        const float d = f16_bits_to_float(c.head[0] & 0xffffu) * (float)unit.factor;
        const float m = f16_bits_to_float(c.head[0] >> 16) * (float)unit.min1;
        return d * (r.s1 + r.s2) - m * (r.xs1 + r.xs2);
    } else {
        const float d = f16_bits_to_float(c.dd & 0xffffu), dm = f16_bits_to_float(c.dd >> 16);
        return (d * (float)unit.factor * r.s1 - dm * (float)unit.min1 * r.xs1) +
               (d * (float)unit.factor2 * r.s2 - dm * (float)unit.min2 * r.xs2);
    }
}

// Unit k of a LaneChunk against 32 F32 activations as the CPU row dot forms it
// (src/gguf/quant_compute.c:152-172): every weight decoded to the float the block decoder gives
// (src/gguf/quant_block.c:745-881, the float operations in its order), the product with its
// activation and the running sum in double. `sum` carries the lane's running sum on.
template <unsigned QT>
__device__ __forceinline__ double chunk_unit_dot_f64(const LaneChunk<QT> &c, int k, const Unit &unit,
                                                     const float *x, double sum)
{
    float scale1, scale2, minimum1 = 0.0f, minimum2 = 0.0f;
    if constexpr (QT == QT_IQ2_XXS) {
        scale1 = scale2 = f16_bits_to_float(c.d16) * (0.5f + (float)((unit.factor - 1) >> 1)) * 0.25f;
    } else if constexpr (QT == QT_Q8_0) {
        scale1 = scale2 = f16_bits_to_float(c.d16[k]);
    } else if constexpr (QT == QT_Q4_K) {
        scale1 = scale2 = f16_bits_to_float(c.head[0] & 0xffffu) * (float)unit.factor;
        minimum1 = minimum2 = f16_bits_to_float(c.head[0] >> 16) * (float)unit.min1;
    } else {
        scale1 = f16_bits_to_float(c.dd & 0xffffu) * (float)unit.factor;
        scale2 = f16_bits_to_float(c.dd & 0xffffu) * (float)unit.factor2;
        minimum1 = f16_bits_to_float(c.dd >> 16) * (float)unit.min1;
        minimum2 = f16_bits_to_float(c.dd >> 16) * (float)unit.min2;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 v = *reinterpret_cast<const float4 *>(x + 4 * i);
        const float xs[4] = {v.x, v.y, v.z, v.w};
        const unsigned w = unit.w[i];
        const float scale = i < 4 ? scale1 : scale2, minimum = i < 4 ? minimum1 : minimum2;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const float code = (float)(signed char)((w >> (8 * b)) & 255u);
            float value = scale * code;
            if constexpr (QT == QT_Q4_K || QT == QT_Q2_K) value = value - minimum;
            sum += (double)value * (double)xs[b];
        }
    }
    return sum;
}

}  // namespace yvex
