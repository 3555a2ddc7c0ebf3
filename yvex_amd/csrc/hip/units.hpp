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
};

template <unsigned QT>
__device__ __forceinline__ void unit_load(const Iq2Tables &tables, const unsigned char *row,
                                          unsigned u, Unit &unit)
{
    const unsigned sb = u >> 3, g = u & 7u;
    if constexpr (QT == QT_IQ2_XXS) {
        uint2 packed = load_u32x2(row + sb * 66u + 2u + 8u * g);
        unit.factor = unit.factor2 = iq2_unit(tables, packed.x, packed.y, unit.w);
        unit.min1 = unit.min2 = 0;
    } else if constexpr (QT == QT_Q8_0) {
        const unsigned char *b = row + u * 34u + 2u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint2 v = load_u32x2(b + 8 * i);
            unit.w[2 * i] = v.x;
            unit.w[2 * i + 1] = v.y;
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
__device__ __forceinline__ float q8_0_unit_value(const unsigned char *row, unsigned u,
                                                 float act_scale, int dot)
{
    return f16_bits_to_float(load_u16(row + u * 34u)) * act_scale * (float)dot;
}

// Unit against 32 F32 activations. Returns the unit's contribution to the row dot.
template <unsigned QT>
__device__ __forceinline__ float unit_dot_f32(const Unit &unit, const unsigned char *row,
                                              unsigned u, const float *x)
{
    const unsigned sb = u >> 3;
    float s1 = 0.0f, s2 = 0.0f, xs1 = 0.0f, xs2 = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float4 v = *reinterpret_cast<const float4 *>(x + 4 * i);
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

}  // namespace yvex
