/*
 * CPU oracle for the quantized-weight matmul path. TEST INFRASTRUCTURE ONLY: see the header
 * for what pins each function. Every function cites the reference lines it restates.
 */
#include "yvex_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "../include/yvex_iq2xxs_grid.h"

static const uint16_t yvo_iq2_grid[256] = {YVEX_IQ2XXS_GRID_VALUES};

static uint16_t load_u16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static uint32_t load_u32(const uint8_t *p)
{
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) |
           ((uint32_t)p[3] << 24);
}
static float bits_float(uint32_t bits)
{
    float out;
    memcpy(&out, &bits, sizeof(out));
    return out;
}
static uint32_t float_bits(float value)
{
    uint32_t bits;
    memcpy(&bits, &value, sizeof(bits));
    return bits;
}
static int as_i8(uint8_t byte) { return byte < 128u ? (int)byte : (int)byte - 256; }

/* ---- scalar rules: src/gguf/quant_scalar.c:40-143 ---- */

float yvo_f16_decode(uint16_t bits)
{
    uint32_t sign = ((uint32_t)bits & 0x8000u) << 16;
    uint32_t exponent = (bits >> 10) & 0x1fu;
    uint32_t mantissa = bits & 0x3ffu;
    if (exponent == 0u) {
        int shift = 0;
        if (mantissa == 0u) return bits_float(sign);
        /* subnormal half: normalise the 10-bit fraction */
        while (!(mantissa & 0x400u)) {
            mantissa <<= 1;
            shift++;
        }
        return bits_float(sign | ((uint32_t)(113 - shift) << 23) | ((mantissa & 0x3ffu) << 13));
    }
    if (exponent == 31u)
        return bits_float(sign | 0x7f800000u | (mantissa << 13) | (mantissa ? 0x00400000u : 0u));
    return bits_float(sign | ((exponent + 112u) << 23) | (mantissa << 13));
}

uint16_t yvo_f16_encode(float value)
{
    uint32_t bits = float_bits(value);
    uint32_t sign = (bits >> 16) & 0x8000u;
    uint32_t exponent = (bits >> 23) & 0xffu;
    uint32_t mantissa = bits & 0x7fffffu;
    uint32_t result;
    if (exponent == 0xffu)
        return (uint16_t)(mantissa ? (sign | 0x7e00u | ((mantissa >> 13) & 0x1ffu))
                                   : (sign | 0x7c00u));
    if (exponent > 142u) return (uint16_t)(sign | 0x7c00u);
    if (exponent < 113u) {
        uint32_t full, shift, quotient, rest, half;
        if (exponent < 102u) return (uint16_t)sign;
        full = mantissa | 0x800000u;
        shift = 126u - exponent;
        quotient = full >> shift;
        rest = full & ((1u << shift) - 1u);
        half = 1u << (shift - 1u);
        if (rest > half || (rest == half && (quotient & 1u))) quotient++;
        return (uint16_t)(sign | quotient);
    }
    result = ((exponent - 112u) << 10) | (mantissa >> 13);
    {
        uint32_t rest = mantissa & 0x1fffu;
        if (rest > 0x1000u || (rest == 0x1000u && (result & 1u))) result++;
    }
    if ((result & 0x7c00u) == 0x7c00u) result &= 0x7c00u;
    return (uint16_t)(sign | result);
}

float yvo_bf16_decode(uint16_t bits) { return bits_float((uint32_t)bits << 16); }

uint16_t yvo_bf16_encode(float value)
{
    uint32_t bits = float_bits(value);
    uint32_t upper = bits >> 16, lower = bits & 0xffffu;
    if ((bits & 0x7f800000u) == 0x7f800000u && (bits & 0x7fffffu)) return (uint16_t)(upper | 0x40u);
    if (lower > 0x8000u || (lower == 0x8000u && (upper & 1u))) upper++;
    return (uint16_t)upper;
}

float yvo_bf16_round(float value) { return yvo_bf16_decode(yvo_bf16_encode(value)); }

float yvo_e8m0_decode(uint8_t bits)
{
    if (bits == 0xffu) return NAN;
    return bits_float(bits == 0u ? 0x00400000u : (uint32_t)bits << 23);
}

/* ---- geometry and admission: src/gguf/qtype.c:15-104, quant_registry.c:50-103 ---- */

static const struct { unsigned short block, bytes; } yvo_geometry[YVO_QTYPE_COUNT] = {
    [0] = {1, 4},     [1] = {1, 2},     [2] = {32, 18},   [3] = {32, 20},   [6] = {32, 22},
    [7] = {32, 24},   [8] = {32, 34},   [9] = {32, 36},   [10] = {256, 84}, [11] = {256, 110},
    [12] = {256, 144}, [13] = {256, 176}, [14] = {256, 210}, [15] = {256, 292}, [16] = {256, 66},
    [17] = {256, 74}, [18] = {256, 98}, [19] = {256, 50}, [20] = {32, 18},  [21] = {256, 110},
    [22] = {256, 82}, [23] = {256, 136}, [24] = {1, 1},   [25] = {1, 2},    [26] = {1, 4},
    [27] = {1, 8},    [28] = {1, 8},    [29] = {256, 56}, [30] = {1, 2},    [34] = {256, 54},
    [35] = {256, 66}, [39] = {32, 17},  [40] = {64, 36},  [41] = {128, 18}, [42] = {64, 18},
};

int yvo_qtype_geometry(unsigned int qtype, unsigned int *block_size, unsigned int *block_bytes)
{
    if (qtype >= YVO_QTYPE_COUNT || !yvo_geometry[qtype].block) return 0;
    if (block_size) *block_size = yvo_geometry[qtype].block;
    if (block_bytes) *block_bytes = yvo_geometry[qtype].bytes;
    return 1;
}

int yvo_qtype_reference_cpu_compute(unsigned int qtype)
{
    switch (qtype) {
    case YVO_QTYPE_F32: case YVO_QTYPE_F16: case YVO_QTYPE_BF16: case YVO_QTYPE_I32:
    case YVO_QTYPE_Q8_0: case YVO_QTYPE_Q2_K: case YVO_QTYPE_IQ2_XXS: case YVO_QTYPE_MXFP4:
        return 1;
    default:
        return 0;
    }
}

int yvo_qtype_admitted(unsigned int qtype)
{
    return yvo_qtype_reference_cpu_compute(qtype) || qtype == YVO_QTYPE_Q4_K;
}

/* ---- block codecs ---- */

/* src/gguf/quant_block.c:160-186 */
int yvo_q8_0_encode_block(const float *source, uint8_t *encoded)
{
    float maximum = 0.0f, scale, inverse;
    uint16_t bits;
    int i;
    for (i = 0; i < 32; ++i) {
        float magnitude = fabsf(source[i]);
        if (magnitude > maximum) maximum = magnitude;
    }
    bits = yvo_f16_encode(maximum / 127.0f);
    encoded[0] = (uint8_t)(bits & 0xffu);
    encoded[1] = (uint8_t)(bits >> 8);
    scale = yvo_f16_decode(bits);
    if (!isfinite(scale) || scale < 0.0f || (maximum > 0.0f && scale == 0.0f)) return 0;
    inverse = scale != 0.0f ? 1.0f / scale : 0.0f;
    for (i = 0; i < 32; ++i) {
        int q = (int)roundf(source[i] * inverse);
        q = q < -127 ? -127 : q > 127 ? 127 : q;
        encoded[2 + i] = (uint8_t)(q & 0xff);
    }
    return 1;
}

/* src/gguf/quant_block.c:378-386 */
static unsigned int iq2_sign_byte(unsigned int low7)
{
    unsigned int parity = 0u, v = low7;
    for (; v; v >>= 1) parity ^= v & 1u;
    return low7 | (parity << 7);
}

/* src/gguf/quant_block.c:745-767 */
static void decode_iq2_xxs(const uint8_t *encoded, float *out)
{
    float d = yvo_f16_decode(load_u16(encoded));
    unsigned int g, j, l;
    for (g = 0; g < 8u; ++g) {
        uint32_t grids = load_u32(encoded + 2u + 8u * g);
        uint32_t aux = load_u32(encoded + 6u + 8u * g);
        float gs = d * (0.5f + (float)(aux >> 28)) * 0.25f;
        for (j = 0; j < 4u; ++j) {
            unsigned int digits = yvo_iq2_grid[(grids >> (8u * j)) & 255u];
            unsigned int signs = iq2_sign_byte((aux >> (7u * j)) & 127u);
            for (l = 0; l < 8u; ++l) {
                unsigned int digit = (digits >> (2u * l)) & 3u;
                float level = digit == 0u ? 8.0f : digit == 1u ? 25.0f : 43.0f;
                out[32u * g + 8u * j + l] = gs * level * ((signs >> l) & 1u ? -1.0f : 1.0f);
            }
        }
    }
}

/* src/gguf/quant_block.c:715-743 */
static void decode_q2_k(const uint8_t *encoded, float *out)
{
    float d = yvo_f16_decode(load_u16(encoded + 80u));
    float dmin = yvo_f16_decode(load_u16(encoded + 82u));
    unsigned int i;
    for (i = 0; i < 256u; ++i) {
        unsigned int sub = i / 16u, lane = i % 16u;
        unsigned int shift = ((sub % 8u) / 2u) * 2u;
        unsigned int byte = 16u + (sub / 8u) * 32u + (sub % 2u) * 16u + lane;
        unsigned int code = (encoded[byte] >> shift) & 3u;
        float scale = d * (float)(encoded[sub] & 15u);
        float minimum = dmin * (float)(encoded[sub] >> 4);
        out[i] = scale * (float)code - minimum;
    }
}

/* Public ggml get_scale_min_k4: 6-bit scale and min of sub-block j from 12 packed bytes. */
static void q4k_scale_min(const uint8_t *scales, unsigned int j, unsigned int *sc, unsigned int *mn)
{
    if (j < 4u) {
        *sc = scales[j] & 63u;
        *mn = scales[j + 4u] & 63u;
    } else {
        *sc = (scales[j + 4u] & 15u) | ((scales[j - 4u] >> 6) << 4);
        *mn = (scales[j + 4u] >> 4) | ((scales[j] >> 6) << 4);
    }
}

/* Public ggml dequantize_row_q4_K over block_q4_K {f16 d; f16 dmin; u8 scales[12]; u8 qs[128]}.
 * The reference has no Q4_K codec (src/gguf/quant_registry.c:67): parity unpinned. */
static void decode_q4_k(const uint8_t *encoded, float *out)
{
    float d = yvo_f16_decode(load_u16(encoded));
    float dmin = yvo_f16_decode(load_u16(encoded + 2u));
    const uint8_t *scales = encoded + 4u, *qs = encoded + 16u;
    unsigned int chunk, l;
    for (chunk = 0; chunk < 4u; ++chunk) {
        unsigned int sc1, m1, sc2, m2;
        float d1, d2, min1, min2;
        q4k_scale_min(scales, 2u * chunk, &sc1, &m1);
        q4k_scale_min(scales, 2u * chunk + 1u, &sc2, &m2);
        d1 = d * (float)sc1;
        min1 = dmin * (float)m1;
        d2 = d * (float)sc2;
        min2 = dmin * (float)m2;
        for (l = 0; l < 32u; ++l) {
            out[64u * chunk + l] = d1 * (float)(qs[32u * chunk + l] & 15u) - min1;
            out[64u * chunk + 32u + l] = d2 * (float)(qs[32u * chunk + l] >> 4) - min2;
        }
    }
}

/* src/gguf/quant_block.c:769-881 */
int yvo_decode_block(unsigned int qtype, const uint8_t *encoded, float *out)
{
    static const float mxfp4[16] = {0.0f, 1.0f, 2.0f, 3.0f, 4.0f, 6.0f, 8.0f, 12.0f,
                                    -0.0f, -1.0f, -2.0f, -3.0f, -4.0f, -6.0f, -8.0f, -12.0f};
    unsigned int i;
    if (!encoded || !out) return YVO_ERR_INVALID_ARG;
    switch (qtype) {
    case YVO_QTYPE_F32:
        out[0] = bits_float(load_u32(encoded));
        return YVO_OK;
    case YVO_QTYPE_F16:
        out[0] = yvo_f16_decode(load_u16(encoded));
        return YVO_OK;
    case YVO_QTYPE_BF16:
        out[0] = yvo_bf16_decode(load_u16(encoded));
        return YVO_OK;
    case YVO_QTYPE_I32: {
        uint32_t bits = load_u32(encoded);
        int32_t v = bits <= 0x7fffffffu ? (int32_t)bits : -1 - (int32_t)(0xffffffffu - bits);
        out[0] = (float)v;
        return YVO_OK;
    }
    case YVO_QTYPE_Q8_0: {
        float d = yvo_f16_decode(load_u16(encoded));
        if (!isfinite(d) || d < 0.0f) return YVO_ERR_FORMAT;
        for (i = 0; i < 32u; ++i) out[i] = d * (float)as_i8(encoded[2u + i]);
        return YVO_OK;
    }
    case YVO_QTYPE_MXFP4: {
        float scale = yvo_e8m0_decode(encoded[0]) * 0.5f;
        if (!isfinite(scale)) return YVO_ERR_FORMAT;
        for (i = 0; i < 16u; ++i) {
            out[i] = mxfp4[encoded[1u + i] & 15u] * scale;
            out[i + 16u] = mxfp4[encoded[1u + i] >> 4] * scale;
            if (!isfinite(out[i]) || !isfinite(out[i + 16u])) return YVO_ERR_FORMAT;
        }
        return YVO_OK;
    }
    case YVO_QTYPE_Q2_K: {
        float d = yvo_f16_decode(load_u16(encoded + 80u));
        float dmin = yvo_f16_decode(load_u16(encoded + 82u));
        if (!isfinite(d) || !isfinite(dmin) || d < 0.0f || dmin < 0.0f) return YVO_ERR_FORMAT;
        decode_q2_k(encoded, out);
        return YVO_OK;
    }
    case YVO_QTYPE_IQ2_XXS: {
        float d = yvo_f16_decode(load_u16(encoded));
        if (!isfinite(d) || d < 0.0f) return YVO_ERR_FORMAT;
        decode_iq2_xxs(encoded, out);
        return YVO_OK;
    }
    case YVO_QTYPE_Q4_K: {
        /* Same scale policy as the reference applies to Q2_K's two affine scales. */
        float d = yvo_f16_decode(load_u16(encoded));
        float dmin = yvo_f16_decode(load_u16(encoded + 2u));
        if (!isfinite(d) || !isfinite(dmin) || d < 0.0f || dmin < 0.0f) return YVO_ERR_FORMAT;
        decode_q4_k(encoded, out);
        return YVO_OK;
    }
    default:
        return YVO_ERR_UNSUPPORTED;
    }
}

/* ---- row dot: src/gguf/quant_compute.c:116-181 ---- */

int yvo_cpu_dot(unsigned int qtype, const uint8_t *encoded, size_t encoded_bytes,
                const float *vector, uint64_t elements, float *out)
{
    unsigned int block_size, block_bytes;
    uint64_t blocks, block, lane;
    double sum = 0.0;
    float values[256];
    if (!encoded || !vector || !out || !elements) return YVO_ERR_INVALID_ARG;
    if (!yvo_qtype_admitted(qtype) || !yvo_qtype_geometry(qtype, &block_size, &block_bytes))
        return YVO_ERR_UNSUPPORTED;
    if (elements % block_size) return YVO_ERR_BOUNDS;
    blocks = elements / block_size;
    if (blocks > SIZE_MAX / block_bytes || (size_t)blocks * block_bytes != encoded_bytes)
        return YVO_ERR_BOUNDS;
    for (block = 0; block < blocks; ++block) {
        int rc = yvo_decode_block(qtype, encoded + (size_t)block * block_bytes, values);
        if (rc != YVO_OK) return rc;
        for (lane = 0; lane < block_size; ++lane) {
            double term = (double)values[lane] * vector[block * block_size + lane];
            if (!isfinite(term) || !isfinite(sum + term)) return YVO_ERR_FORMAT;
            sum += term;
        }
    }
    *out = (float)sum;
    return isfinite(*out) ? YVO_OK : YVO_ERR_BOUNDS;
}

static int row_bytes_of(unsigned int qtype, uint64_t row_width, uint64_t *row_bytes)
{
    unsigned int block_size, block_bytes;
    if (!yvo_qtype_geometry(qtype, &block_size, &block_bytes)) return YVO_ERR_UNSUPPORTED;
    if (!row_width || row_width % block_size) return YVO_ERR_BOUNDS;
    *row_bytes = row_width / block_size * block_bytes;
    return YVO_OK;
}

/* src/graph/moe.c:430-444: one cpu_dot per row, per input row. */
int yvo_matvec(unsigned int qtype, const uint8_t *encoded, uint64_t row_count,
               uint64_t row_width, const float *input, uint64_t input_rows, float *out)
{
    uint64_t row_bytes, in, row;
    int rc = row_bytes_of(qtype, row_width, &row_bytes);
    if (rc != YVO_OK) return rc;
    for (in = 0; in < input_rows; ++in)
        for (row = 0; row < row_count; ++row) {
            rc = yvo_cpu_dot(qtype, encoded + row * row_bytes, (size_t)row_bytes,
                             input + in * row_width, row_width, &out[in * row_count + row]);
            if (rc != YVO_OK) return rc;
        }
    return YVO_OK;
}

typedef struct {
    unsigned int qtype;
    const uint8_t *encoded;
    uint64_t row_begin, row_end, row_count, row_width, input_rows;
    const float *input;
    float *out;
    int rc;
} matvec_slice;

static void *matvec_worker(void *opaque)
{
    matvec_slice *s = (matvec_slice *)opaque;
    uint64_t row_bytes, in, row;
    s->rc = row_bytes_of(s->qtype, s->row_width, &row_bytes);
    if (s->rc != YVO_OK) return NULL;
    for (in = 0; in < s->input_rows; ++in)
        for (row = s->row_begin; row < s->row_end; ++row) {
            int rc = yvo_cpu_dot(s->qtype, s->encoded + row * row_bytes, (size_t)row_bytes,
                                 s->input + in * s->row_width, s->row_width,
                                 &s->out[in * s->row_count + row]);
            if (rc != YVO_OK) {
                s->rc = rc;
                return NULL;
            }
        }
    return NULL;
}

int yvo_matvec_threads(unsigned int qtype, const uint8_t *encoded, uint64_t row_count,
                       uint64_t row_width, const float *input, uint64_t input_rows,
                       float *out, unsigned int threads)
{
    pthread_t handles[64];
    matvec_slice slices[64];
    unsigned int t, started = 0;
    int rc = YVO_OK;
    if (threads <= 1u)
        return yvo_matvec(qtype, encoded, row_count, row_width, input, input_rows, out);
    if (threads > 64u) threads = 64u;
    for (t = 0; t < threads; ++t) {
        slices[t] = (matvec_slice){qtype, encoded, row_count * t / threads,
                                   row_count * (t + 1u) / threads, row_count, row_width,
                                   input_rows, input, out, YVO_OK};
        if (pthread_create(&handles[t], NULL, matvec_worker, &slices[t]) != 0) break;
        started++;
    }
    for (t = 0; t < started; ++t) {
        pthread_join(handles[t], NULL);
        if (slices[t].rc != YVO_OK && rc == YVO_OK) rc = slices[t].rc;
    }
    if (started != threads) return YVO_ERR;
    return rc;
}

/* src/backend/cuda/kernels.cu:784-830: decode selected rows to float. */
int yvo_decode_rows(unsigned int qtype, const uint8_t *encoded, uint64_t row_width,
                    const uint32_t *row_ids, uint64_t selected, float *out)
{
    unsigned int block_size, block_bytes;
    uint64_t row_bytes, s, b;
    int rc = row_bytes_of(qtype, row_width, &row_bytes);
    if (rc != YVO_OK) return rc;
    if (!yvo_qtype_admitted(qtype)) return YVO_ERR_UNSUPPORTED;
    yvo_qtype_geometry(qtype, &block_size, &block_bytes);
    for (s = 0; s < selected; ++s) {
        const uint8_t *row = encoded + (uint64_t)(row_ids ? row_ids[s] : s) * row_bytes;
        for (b = 0; b < row_width / block_size; ++b) {
            rc = yvo_decode_block(qtype, row + b * block_bytes, out + s * row_width + b * block_size);
            if (rc != YVO_OK) return rc;
        }
    }
    return YVO_OK;
}

/* ---- Q8_K activations: src/backend/cuda/kernels.cu:436-489, tests/unit/cuda/quant_qtype.c:161-186 ---- */

int yvo_q8k_quantize(const float *values, uint64_t rows, uint64_t width, uint8_t *encoded)
{
    uint64_t blocks = width / 256u, task;
    if (!values || !encoded || !width || width % 256u) return YVO_ERR_INVALID_ARG;
    for (task = 0; task < rows * blocks; ++task) {
        const float *x = values + task * 256u;
        uint8_t *block = encoded + task * 292u;
        float best_abs = 0.0f, best = 0.0f, inverse, d;
        int i, k;
        for (i = 0; i < 256; ++i) {
            if (!isfinite(x[i])) return YVO_ERR_FORMAT;
            /* first strict maximum, as the host twin does; an exact |tie| with the device's
             * pairwise tree only flips the sign of d and of every q together */
            if (fabsf(x[i]) > best_abs) {
                best_abs = fabsf(x[i]);
                best = x[i];
            }
        }
        inverse = best_abs == 0.0f ? 0.0f : -127.0f / best;
        d = inverse == 0.0f ? 0.0f : 1.0f / inverse;
        memcpy(block, &d, 4);
        for (i = 0; i < 256; ++i) {
            int q = inverse == 0.0f ? 0 : (int)lrintf(inverse * x[i]); /* ties to even */
            q = q > 127 ? 127 : q < -128 ? -128 : q;
            block[4 + i] = (uint8_t)(q & 0xff);
        }
        for (k = 0; k < 16; ++k) {
            int sum = 0;
            int16_t s16;
            for (i = 0; i < 16; ++i) sum += as_i8(block[4 + 16 * k + i]);
            s16 = (int16_t)sum;
            memcpy(block + 260 + 2 * k, &s16, 2);
        }
    }
    return YVO_OK;
}

void yvo_q8k_dequantize(const uint8_t *encoded, uint64_t blocks, float *out)
{
    uint64_t b;
    int i;
    for (b = 0; b < blocks; ++b) {
        float d;
        memcpy(&d, encoded + b * 292u, 4);
        for (i = 0; i < 256; ++i) out[b * 256u + i] = d * (float)as_i8(encoded[b * 292u + 4 + i]);
    }
}

static int q8k_bsum(const uint8_t *act, unsigned int k)
{
    int16_t v;
    memcpy(&v, act + 260u + 2u * k, 2);
    return v;
}

/* ---- integer block dots ---- */

/* src/backend/cuda/kernel_primitives.h:287-313 */
int32_t yvo_block_dot_iq2xxs_q8k(const uint8_t *w, const uint8_t *a)
{
    int32_t total = 0;
    unsigned int g, j, l;
    for (g = 0; g < 8u; ++g) {
        uint32_t grids = load_u32(w + 2u + 8u * g);
        uint32_t aux = load_u32(w + 6u + 8u * g);
        int32_t group = 0;
        for (j = 0; j < 4u; ++j) {
            unsigned int digits = yvo_iq2_grid[(grids >> (8u * j)) & 255u];
            unsigned int signs = iq2_sign_byte((aux >> (7u * j)) & 127u);
            for (l = 0; l < 8u; ++l) {
                unsigned int digit = (digits >> (2u * l)) & 3u;
                int level = digit == 0u ? 8 : digit == 1u ? 25 : 43;
                if ((signs >> l) & 1u) level = -level;
                group += level * as_i8(a[4u + 32u * g + 8u * j + l]);
            }
        }
        total += group * (int32_t)(2u * (aux >> 28) + 1u);
    }
    return total;
}

/* src/backend/cuda/kernel_primitives.h:342-359 */
void yvo_block_dot_q8_0_q8k(const uint8_t *w, const uint8_t *a, int32_t dots[8])
{
    unsigned int b, i;
    for (b = 0; b < 8u; ++b) {
        int32_t dot = 0;
        for (i = 0; i < 32u; ++i) dot += as_i8(w[34u * b + 2u + i]) * as_i8(a[4u + 32u * b + i]);
        dots[b] = dot;
    }
}

/* Q4_K x Q8_K in the shape of the reference's Q2_K primitive (kernel_primitives.h:314-341):
 * dot = sum_j sc_j * sum_{i in j} nibble_i * a_i ; minimum = sum_j m_j * (bsums[2j] + bsums[2j+1]). */
void yvo_block_dot_q4k_q8k(const uint8_t *w, const uint8_t *a, int32_t *dot, int32_t *minimum)
{
    const uint8_t *scales = w + 4u, *qs = w + 16u;
    int32_t d = 0, m = 0;
    unsigned int j, l;
    for (j = 0; j < 8u; ++j) {
        unsigned int sc, mn, chunk = j / 2u, high = j & 1u;
        int32_t sub = 0;
        q4k_scale_min(scales, j, &sc, &mn);
        for (l = 0; l < 32u; ++l) {
            unsigned int byte = qs[32u * chunk + l];
            sub += (int32_t)(high ? byte >> 4 : byte & 15u) * as_i8(a[4u + 32u * j + l]);
        }
        d += (int32_t)sc * sub;
        m += (int32_t)mn * (q8k_bsum(a, 2u * j) + q8k_bsum(a, 2u * j + 1u));
    }
    *dot = d;
    *minimum = m;
}

/* src/backend/cuda/kernel_primitives.h:314-341 */
void yvo_block_dot_q2k_q8k(const uint8_t *w, const uint8_t *a, int32_t *dot, int32_t *minimum)
{
    int32_t d = 0, m = 0;
    unsigned int sub, lane;
    for (sub = 0; sub < 16u; ++sub) {
        unsigned int shift = ((sub % 8u) / 2u) * 2u;
        unsigned int base = 16u + (sub / 8u) * 32u + (sub % 2u) * 16u;
        int32_t part = 0;
        for (lane = 0; lane < 16u; ++lane)
            part += (int32_t)((w[base + lane] >> shift) & 3u) * as_i8(a[4u + 16u * sub + lane]);
        d += (int32_t)(w[sub] & 15u) * part;
        m += (int32_t)(w[sub] >> 4) * q8k_bsum(a, sub);
    }
    *dot = d;
    *minimum = m;
}

/* Float combination of one block exactly as the device primitives order it
 * (kernel_primitives.h:312, :336-340, :353-357). */
float yvo_block_dot_float(unsigned int qtype, const uint8_t *w, const uint8_t *a)
{
    float da;
    memcpy(&da, a, 4);
    if (qtype == YVO_QTYPE_IQ2_XXS) {
        float dw = yvo_f16_decode(load_u16(w));
        return 0.125f * dw * da * (float)yvo_block_dot_iq2xxs_q8k(w, a);
    }
    if (qtype == YVO_QTYPE_Q8_0) {
        int32_t dots[8];
        float total = 0.0f;
        unsigned int b;
        yvo_block_dot_q8_0_q8k(w, a, dots);
        for (b = 0; b < 8u; ++b)
            total = fmaf(yvo_f16_decode(load_u16(w + 34u * b)) * da, (float)dots[b], total);
        return total;
    }
    if (qtype == YVO_QTYPE_Q4_K || qtype == YVO_QTYPE_Q2_K) {
        int32_t dot, minimum;
        float d, dmin;
        if (qtype == YVO_QTYPE_Q4_K) {
            yvo_block_dot_q4k_q8k(w, a, &dot, &minimum);
            d = yvo_f16_decode(load_u16(w));
            dmin = yvo_f16_decode(load_u16(w + 2u));
        } else {
            yvo_block_dot_q2k_q8k(w, a, &dot, &minimum);
            d = yvo_f16_decode(load_u16(w + 80u));
            dmin = yvo_f16_decode(load_u16(w + 82u));
        }
        /* two rounded products, then one rounded subtraction: no fused contraction */
        {
            volatile float left = da * d * (float)dot;
            volatile float right = da * dmin * (float)minimum;
            return left - right;
        }
    }
    return NAN;
}

int yvo_q8_row_dot(unsigned int qtype, const uint8_t *row, uint64_t row_width,
                   const uint8_t *act, float *out)
{
    uint64_t blocks = row_width / 256u, b;
    unsigned int weight_bytes;
    double sum = 0.0;
    if (!row || !act || !out || !row_width || row_width % 256u) return YVO_ERR_BOUNDS;
    switch (qtype) {
    case YVO_QTYPE_IQ2_XXS: weight_bytes = 66u; break;
    case YVO_QTYPE_Q8_0: weight_bytes = 272u; break;
    case YVO_QTYPE_Q4_K: weight_bytes = 144u; break;
    case YVO_QTYPE_Q2_K: weight_bytes = 84u; break;
    default: return YVO_ERR_UNSUPPORTED;
    }
    for (b = 0; b < blocks; ++b)
        sum += (double)yvo_block_dot_float(qtype, row + b * weight_bytes, act + b * 292u);
    *out = (float)sum;
    return isfinite(*out) ? YVO_OK : YVO_ERR_FORMAT;
}

int yvo_q8_matvec(unsigned int qtype, const uint8_t *encoded, uint64_t row_count,
                  uint64_t row_width, const uint8_t *act, uint64_t input_rows, float *out)
{
    uint64_t row_bytes, in, row;
    int rc = row_bytes_of(qtype, row_width, &row_bytes);
    if (rc != YVO_OK) return rc;
    for (in = 0; in < input_rows; ++in)
        for (row = 0; row < row_count; ++row) {
            rc = yvo_q8_row_dot(qtype, encoded + row * row_bytes, row_width,
                                act + in * (row_width / 256u) * 292u, &out[in * row_count + row]);
            if (rc != YVO_OK) return rc;
        }
    return YVO_OK;
}

/* ---- router: src/graph/moe.c:497-585 ---- */

static double score_sqrt_softplus(double v)
{
    double softplus = v > 0.0 ? v + log1p(exp(-v)) : log1p(exp(v));
    return sqrt(softplus);
}

static double score_sigmoid(double v)
{
    return v >= 0.0 ? 1.0 / (1.0 + exp(-v)) : exp(v) / (1.0 + exp(v));
}

/* table_row != NULL is the hash router (moe.c:539-559): the selection comes from the token's
 * row of expert ordinals and the bias plays no part. */
static int route_one(const float *logits, const float *bias, const int32_t *table_row,
                     uint64_t experts, uint64_t topk, int scoring, int normalize, double scaling,
                     float *scores_out, uint64_t *selected, float *weights)
{
    float scores[256], biased[256];
    uint64_t e, rank, prior;
    double total = 0.0;
    if (!logits || !selected || !weights || !experts || experts > 256u || !topk || topk > 16u ||
        topk > experts)
        return YVO_ERR_INVALID_ARG;
    for (e = 0; e < experts; ++e) {
        double s = scoring == YVO_SCORING_SIGMOID ? score_sigmoid(logits[e])
                                                  : score_sqrt_softplus(logits[e]);
        if (!isfinite(s)) return YVO_ERR_FORMAT;
        scores[e] = (float)s;
        biased[e] = (bias ? bias[e] : 0.0f) + scores[e];
        if (scores_out) scores_out[e] = scores[e];
    }
    for (rank = 0; table_row && rank < topk; ++rank) {
        if (table_row[rank] < 0 || (uint64_t)table_row[rank] >= experts) return YVO_ERR_FORMAT;
        selected[rank] = (uint64_t)table_row[rank];
    }
    for (rank = 0; !table_row && rank < topk; ++rank) { /* src/graph/moe.c:503-518 */
        uint64_t best = UINT64_MAX;
        for (e = 0; e < experts; ++e) {
            int used = 0;
            for (prior = 0; prior < rank; ++prior) used |= selected[prior] == e;
            if (!used && (best == UINT64_MAX || biased[e] > biased[best] ||
                          (biased[e] == biased[best] && e < best)))
                best = e;
        }
        selected[rank] = best;
    }
    for (rank = 0; rank < topk; ++rank) {
        for (prior = 0; prior < rank; ++prior)       /* moe.c:561-566 */
            if (selected[prior] == selected[rank]) return YVO_ERR_FORMAT;
        weights[rank] = scores[selected[rank]];
        total += weights[rank];
    }
    if (normalize && (!isfinite(total) || total <= 0.0)) return YVO_ERR_FORMAT;
    for (rank = 0; rank < topk; ++rank) {
        double value = weights[rank];
        if (normalize) value /= total;
        value *= scaling;
        weights[rank] = (float)value;
    }
    return YVO_OK;
}

int yvo_moe_route(const float *logits, const float *bias, uint64_t experts, uint64_t topk,
                  int scoring, int normalize, double scaling, float *scores_out,
                  uint64_t *selected, float *weights)
{
    return route_one(logits, bias, NULL, experts, topk, scoring, normalize, scaling, scores_out,
                     selected, weights);
}

int yvo_moe_route_hash(const float *logits, const int32_t *table, uint64_t table_rows,
                       uint64_t table_row_bytes, uint64_t token, uint64_t experts, uint64_t topk,
                       int scoring, int normalize, double scaling, float *scores_out,
                       uint64_t *selected, float *weights)
{
    if (!table || table_row_bytes < topk * 4u || (table_row_bytes & 3u)) return YVO_ERR_BOUNDS;
    if (token >= table_rows) return YVO_ERR_BOUNDS;
    return route_one(logits, NULL, table + token * (table_row_bytes / 4u), experts, topk, scoring,
                     normalize, scaling, scores_out, selected, weights);
}

/* ---- expert FFN: src/graph/moe.c:587-622 ---- */

static int project(unsigned int qtype, const uint8_t *weight, uint64_t rows, uint64_t width,
                   const float *input, int act_q8, float *out)
{
    if (!act_q8) return yvo_matvec(qtype, weight, rows, width, input, 1u, out);
    {
        uint8_t *q = (uint8_t *)malloc((size_t)(width / 256u) * 292u);
        int rc;
        if (!q) return YVO_ERR_NOMEM;
        rc = yvo_q8k_quantize(input, 1u, width, q);
        if (rc == YVO_OK) rc = yvo_q8_matvec(qtype, weight, rows, width, q, 1u, out);
        free(q);
        return rc;
    }
}

int yvo_moe_expert(unsigned int gate_qtype, const uint8_t *gate, unsigned int up_qtype,
                   const uint8_t *up, unsigned int down_qtype, const uint8_t *down,
                   uint64_t hidden, uint64_t intermediate, const float *input,
                   float route_weight, double limit, int act_q8, float *output,
                   float *intermediate_out, float *unrounded_out)
{
    float *g, *u, *h;
    uint64_t i;
    int rc;
    if (!gate || !up || !down || !input || !output || !isfinite(route_weight))
        return YVO_ERR_INVALID_ARG;
    g = (float *)malloc(sizeof(float) * 3u * (size_t)intermediate);
    if (!g) return YVO_ERR_NOMEM;
    u = g + intermediate;
    h = u + intermediate;
    rc = project(gate_qtype, gate, intermediate, hidden, input, act_q8, g);
    if (rc == YVO_OK) rc = project(up_qtype, up, intermediate, hidden, input, act_q8, u);
    for (i = 0; rc == YVO_OK && i < intermediate; ++i) {
        double gv = fmin(g[i], limit);
        double uv = fmax(-limit, fmin(u[i], limit));
        double silu = gv >= 0.0 ? gv / (1.0 + exp(-gv)) : gv * exp(gv) / (1.0 + exp(gv));
        h[i] = yvo_bf16_round((float)(silu * uv * route_weight));
        if (!isfinite(h[i])) rc = YVO_ERR_FORMAT;
    }
    if (rc == YVO_OK && intermediate_out) memcpy(intermediate_out, h, sizeof(float) * intermediate);
    if (rc == YVO_OK) rc = project(down_qtype, down, hidden, intermediate, h, act_q8, output);
    for (i = 0; rc == YVO_OK && i < hidden; ++i) {
        if (unrounded_out) unrounded_out[i] = output[i];
        output[i] = yvo_bf16_round(output[i]);
        if (!isfinite(output[i])) rc = YVO_ERR_FORMAT;
    }
    free(g);
    return rc;
}

/* ---- greedy selection: src/backend/cuda/kernels.cu:59-110 ---- */

int yvo_argmax_f32(const float *values, uint64_t row_count, uint64_t row_width,
                   uint32_t *selected_tokens, float *selected_values, uint64_t *tie_counts)
{
    uint64_t row, index;
    int status = 0;
    if (!values || !row_count || !row_width || !selected_tokens || !selected_values || !tie_counts)
        return YVO_ERR_INVALID_ARG;
    for (row = 0; row < row_count; ++row) {
        const float *v = values + row * row_width;
        float best = -3.402823466e+38F;
        uint64_t best_index = ~(uint64_t)0, tied = 0;
        int bad = 0;
        for (index = 0; index < row_width; ++index) {
            float value = v[index];
            if (!isfinite(value)) bad = 1;
            else if (value > best) best = value, best_index = index, tied = 1;
            else if (value == best) {
                if (index < best_index) best_index = index;
                tied++;
            }
        }
        if (bad) {
            status = 1;
            continue;
        }
        selected_tokens[row] = (uint32_t)best_index;
        selected_values[row] = best;
        tie_counts[row] = tied;
    }
    return status;
}

/* ---- residual-stream envelope around the expert math ---- */

/* src/graph/numeric.c:630-666: mean of squares in double, one rounding to float per value */
int yvo_rms_norm(float *values, uint64_t count, const float *weights, double epsilon)
{
    double mean = 0.0, inverse;
    uint64_t i;
    if (!values || !count || !weights || !isfinite(epsilon) || epsilon <= 0.0)
        return YVO_ERR_INVALID_ARG;
    for (i = 0; i < count; ++i) {
        if (!isfinite(values[i]) || !isfinite(weights[i])) return YVO_ERR_FORMAT;
        mean += (double)values[i] * (double)values[i];
    }
    mean /= (double)count;
    inverse = 1.0 / sqrt(mean + epsilon);
    if (!isfinite(inverse)) return YVO_ERR_FORMAT;
    for (i = 0; i < count; ++i) {
        double v = (double)values[i] * inverse;
        v *= (double)weights[i];
        if (!isfinite(v)) return YVO_ERR_FORMAT;
        values[i] = (float)v;
    }
    return YVO_OK;
}

/* src/graph/numeric.c:691-702 */
static double envelope_sigmoid(double value)
{
    if (value >= 0.0) return 1.0 / (1.0 + exp(-value));
    {
        double direct = exp(value);
        return direct / (1.0 + direct);
    }
}

/* src/graph/numeric.c:704-750: row softmax (+ epsilon), then alternating row and column
 * normalisations; the first iteration normalises columns only */
static int envelope_sinkhorn(float *m, uint64_t n, uint64_t iterations, double epsilon)
{
    uint64_t r, c, it;
    for (r = 0; r < n; ++r) {
        double maximum = -(double)INFINITY, total = 0.0;
        for (c = 0; c < n; ++c) maximum = fmax(maximum, m[r * n + c]);
        for (c = 0; c < n; ++c) {
            double value = exp((double)m[r * n + c] - maximum);
            m[r * n + c] = (float)value;
            total += value;
        }
        if (!isfinite(total) || total <= 0.0) return 0;
        for (c = 0; c < n; ++c) m[r * n + c] = (float)((double)m[r * n + c] / total + epsilon);
    }
    for (it = 0; it < iterations; ++it) {
        if (it != 0) {
            for (r = 0; r < n; ++r) {
                double total = 0.0;
                for (c = 0; c < n; ++c) total += m[r * n + c];
                if (!isfinite(total)) return 0;
                for (c = 0; c < n; ++c)
                    m[r * n + c] = (float)((double)m[r * n + c] / (total + epsilon));
            }
        }
        for (c = 0; c < n; ++c) {
            double total = 0.0;
            for (r = 0; r < n; ++r) total += m[r * n + c];
            if (!isfinite(total)) return 0;
            for (r = 0; r < n; ++r)
                m[r * n + c] = (float)((double)m[r * n + c] / (total + epsilon));
        }
    }
    return 1;
}

/* src/graph/numeric.c:752-826 with dense strides */
int yvo_mhc_pre(const float *residual, const float *mixes, const float *scale, const float *base,
                uint64_t tokens, uint64_t streams, uint64_t width, uint64_t iterations,
                double rms_epsilon, double mhc_epsilon, double post_multiplier, float *collapsed,
                float *post, float *combination)
{
    const uint64_t expanded = streams * width, mixing_rows = (streams + 2u) * streams;
    uint64_t token, stream, target, lane;
    if (!residual || !mixes || !scale || !base || !collapsed || !post || !combination || !tokens ||
        !streams || !width || !iterations || !(rms_epsilon > 0.0) || !(mhc_epsilon > 0.0) ||
        !(post_multiplier > 0.0) || !isfinite(rms_epsilon) || !isfinite(mhc_epsilon) ||
        !isfinite(post_multiplier))
        return YVO_ERR_BOUNDS;
    for (lane = 0; lane < 3u; ++lane)
        if (!isfinite(scale[lane])) return YVO_ERR_FORMAT;
    for (lane = 0; lane < mixing_rows; ++lane)
        if (!isfinite(base[lane])) return YVO_ERR_FORMAT;
    for (token = 0; token < tokens; ++token) {
        const float *res = residual + token * expanded;
        const float *mix = mixes + token * mixing_rows;
        float *out = collapsed + token * width;
        float *po = post + token * streams;
        float *comb = combination + token * streams * streams;
        double squares = 0.0, inverse;
        memset(out, 0, (size_t)width * sizeof(*out));
        for (lane = 0; lane < expanded; ++lane) {
            if (!isfinite(res[lane])) return YVO_ERR_FORMAT;
            squares += (double)res[lane] * (double)res[lane];
        }
        inverse = 1.0 / sqrt(squares / (double)expanded + rms_epsilon);
        if (!isfinite(inverse)) return YVO_ERR_FORMAT;
        for (stream = 0; stream < streams; ++stream) {
            double pre = envelope_sigmoid((double)mix[stream] * inverse * (double)scale[0] +
                                          (double)base[stream]);
            po[stream] = (float)(post_multiplier * envelope_sigmoid(
                (double)mix[streams + stream] * inverse * (double)scale[1] +
                (double)base[streams + stream]));
            for (target = 0; target < streams; ++target) {
                uint64_t index = 2u * streams + stream * streams + target;
                comb[stream * streams + target] =
                    (float)((double)mix[index] * inverse * (double)scale[2] + (double)base[index]);
            }
            for (lane = 0; lane < width; ++lane)
                out[lane] += (float)((pre + mhc_epsilon) * (double)res[stream * width + lane]);
        }
        if (!envelope_sinkhorn(comb, streams, iterations, mhc_epsilon)) return YVO_ERR_FORMAT;
        for (lane = 0; lane < width; ++lane) {
            if (!isfinite(out[lane])) return YVO_ERR_FORMAT;
            out[lane] = yvo_bf16_round(out[lane]);
        }
    }
    return YVO_OK;
}

/* src/graph/numeric.c:828-877 with dense strides: combination rows are sources, columns targets */
int yvo_mhc_post(const float *core, const float *residual, const float *post,
                 const float *combination, uint64_t tokens, uint64_t streams, uint64_t width,
                 float *output)
{
    uint64_t token, target, source, lane;
    if (!core || !residual || !post || !combination || !output || !tokens || !streams || !width)
        return YVO_ERR_BOUNDS;
    for (token = 0; token < tokens; ++token) {
        const float *c = core + token * width, *res = residual + token * streams * width;
        const float *po = post + token * streams, *comb = combination + token * streams * streams;
        float *out = output + token * streams * width;
        for (target = 0; target < streams; ++target)
            for (lane = 0; lane < width; ++lane) {
                double value = (double)po[target] * (double)c[lane];
                for (source = 0; source < streams; ++source)
                    value += (double)comb[source * streams + target] *
                             (double)res[source * width + lane];
                if (!isfinite(value)) return YVO_ERR_FORMAT;
                out[target * width + lane] = (float)value;
            }
        for (lane = 0; lane < streams * width; ++lane) {
            if (!isfinite(out[lane])) return YVO_ERR_FORMAT;
            out[lane] = yvo_bf16_round(out[lane]);
        }
    }
    return YVO_OK;
}

/* src/graph/moe.c:446-495: mixes = function . expanded row through the CPU row dot, ingress,
 * weighted RMS norm, bf16 publication. scale, base and norm arrive decoded (moe.c:405-428
 * copies F32, widens BF16 and converts I32). */
int yvo_moe_ffn_prepare(unsigned int function_qtype, const uint8_t *function,
                        const float *expanded, const float *scale, const float *base,
                        const float *norm, uint64_t tokens, uint64_t streams, uint64_t width,
                        uint64_t iterations, double rms_epsilon, double mhc_epsilon,
                        double post_multiplier, float *normalized, float *post, float *combination)
{
    const uint64_t expanded_width = streams * width, mixing_rows = (streams + 2u) * streams;
    float mix[64];
    uint64_t token;
    int rc;
    if (!function || !expanded || !norm || !normalized || mixing_rows > 64u || width > 16384u)
        return YVO_ERR_INVALID_ARG;
    for (token = 0; token < tokens; ++token) {
        float *row = normalized + token * width;
        uint64_t lane;
        rc = yvo_matvec(function_qtype, function, mixing_rows, expanded_width,
                        expanded + token * expanded_width, 1, mix);
        if (rc != YVO_OK) return rc;
        rc = yvo_mhc_pre(expanded + token * expanded_width, mix, scale, base, 1, streams, width,
                         iterations, rms_epsilon, mhc_epsilon, post_multiplier, row,
                         post + token * streams, combination + token * streams * streams);
        if (rc != YVO_OK) return rc;
        rc = yvo_rms_norm(row, width, norm, rms_epsilon);
        if (rc != YVO_OK) return rc;
        for (lane = 0; lane < width; ++lane) {
            if (!isfinite(row[lane])) return YVO_ERR_FORMAT;
            row[lane] = yvo_bf16_round(row[lane]);
        }
    }
    return YVO_OK;
}

/* ---- worklist: src/graph/worklist.c:369-441 ---- */

int yvo_worklist_build(const uint64_t *selected_experts, const float *route_weights,
                       uint64_t pair_count, uint64_t experts_per_row, uint64_t expert_count,
                       uint64_t *expert_ids, uint64_t *bucket_offsets,
                       uint64_t *bucket_populations, uint64_t *source_pairs,
                       uint64_t *source_rows, uint64_t *destination_rows,
                       float *ordered_weights, uint64_t *bucket_count)
{
    uint64_t expert, pair, cursor = 0, bucket = 0;
    if (!selected_experts || !route_weights || !experts_per_row || !expert_count ||
        pair_count % experts_per_row)
        return YVO_ERR_INVALID_ARG;
    for (pair = 0; pair < pair_count; ++pair)
        if (selected_experts[pair] >= expert_count || !isfinite(route_weights[pair]))
            return YVO_ERR_FORMAT;
    for (expert = 0; expert < expert_count; ++expert) {
        uint64_t start = cursor;
        for (pair = 0; pair < pair_count; ++pair) {
            if (selected_experts[pair] != expert) continue;
            source_pairs[cursor] = pair;
            source_rows[cursor] = pair / experts_per_row;
            destination_rows[cursor] = pair;
            ordered_weights[cursor] = route_weights[pair];
            cursor++;
        }
        if (cursor == start) continue;
        expert_ids[bucket] = expert;
        bucket_offsets[bucket] = start;
        bucket_populations[bucket] = cursor - start;
        bucket++;
    }
    bucket_offsets[bucket] = cursor;
    if (cursor != pair_count) return YVO_ERR_STATE;
    *bucket_count = bucket;
    return YVO_OK;
}

/* ---- layer over a row batch: src/runtime/moe.c:596-632 ---- */

typedef struct {
    const yvo_moe_layer_args *args;
    const float *inputs, *logits;
    uint64_t *selected;
    float *weights, *routed, *shared, *combined;
    uint64_t row_begin, row_end;
    int rc;
} layer_slice;

static void *layer_worker(void *opaque)
{
    layer_slice *s = (layer_slice *)opaque;
    const yvo_moe_layer_args *a = s->args;
    uint64_t gate_row, down_row, gate_expert, down_expert, row, rank, c;
    float *expert_out = (float *)malloc(sizeof(float) * 3u * (size_t)a->hidden);
    float *routed, *shared;
    s->rc = YVO_OK;
    if (!expert_out) {
        s->rc = YVO_ERR_NOMEM;
        return NULL;
    }
    routed = expert_out + a->hidden;
    shared = routed + a->hidden;
    if (row_bytes_of(a->gate_qtype, a->hidden, &gate_row) != YVO_OK ||
        row_bytes_of(a->down_qtype, a->intermediate, &down_row) != YVO_OK) {
        s->rc = YVO_ERR_BOUNDS;
        free(expert_out);
        return NULL;
    }
    gate_expert = gate_row * a->intermediate;
    down_expert = down_row * a->hidden;
    for (row = s->row_begin; row < s->row_end && s->rc == YVO_OK; ++row) {
        const float *x = s->inputs + row * a->hidden;
        uint64_t *sel = s->selected + row * a->topk;
        float *w = s->weights + row * a->topk;
        s->rc = route_one(s->logits + row * a->experts, a->router_bias,
                          a->hash_selected ? a->hash_selected + row * a->topk : NULL, a->experts,
                          a->topk, a->scoring, a->normalize, a->scaling, NULL, sel, w);
        memset(routed, 0, sizeof(float) * a->hidden);
        for (rank = 0; rank < a->topk && s->rc == YVO_OK; ++rank) {
            uint64_t e = sel[rank];
            s->rc = yvo_moe_expert(a->gate_qtype, a->routed_gate + e * gate_expert, a->up_qtype,
                                   a->routed_up + e * gate_expert, a->down_qtype,
                                   a->routed_down + e * down_expert, a->hidden, a->intermediate,
                                   x, w[rank], a->activation_limit, a->act_q8, expert_out, NULL,
                                   NULL);
            for (c = 0; c < a->hidden; ++c) routed[c] += expert_out[c];
        }
        memset(shared, 0, sizeof(float) * a->hidden);
        if (s->rc == YVO_OK && a->shared_gate)
            s->rc = yvo_moe_expert(a->gate_qtype, a->shared_gate, a->up_qtype, a->shared_up,
                                   a->down_qtype, a->shared_down, a->hidden, a->intermediate, x,
                                   1.0f, a->activation_limit, a->act_q8, shared, NULL, NULL);
        for (c = 0; c < a->hidden && s->rc == YVO_OK; ++c) {
            if (s->routed) s->routed[row * a->hidden + c] = routed[c];
            if (s->shared) s->shared[row * a->hidden + c] = shared[c];
            s->combined[row * a->hidden + c] = yvo_bf16_round(routed[c] + shared[c]);
        }
    }
    free(expert_out);
    return NULL;
}

int yvo_moe_layer(const yvo_moe_layer_args *args, const float *inputs, const float *logits,
                  uint64_t *selected, float *weights, float *routed, float *shared,
                  float *combined)
{
    pthread_t handles[64];
    layer_slice slices[64];
    unsigned int threads, t, started = 0;
    int rc = YVO_OK;
    if (!args || !inputs || !logits || !selected || !weights || !combined)
        return YVO_ERR_INVALID_ARG;
    threads = args->threads ? args->threads : 1u;
    if (threads > 64u) threads = 64u;
    if (threads > args->rows) threads = (unsigned int)(args->rows ? args->rows : 1u);
    for (t = 0; t < threads; ++t) {
        slices[t] = (layer_slice){args, inputs, logits, selected, weights, routed, shared,
                                  combined, args->rows * t / threads,
                                  args->rows * (t + 1u) / threads, YVO_OK};
        if (threads == 1u) {
            layer_worker(&slices[0]);
            return slices[0].rc;
        }
        if (pthread_create(&handles[t], NULL, layer_worker, &slices[t]) != 0) break;
        started++;
    }
    for (t = 0; t < started; ++t) {
        pthread_join(handles[t], NULL);
        if (slices[t].rc != YVO_OK && rc == YVO_OK) rc = slices[t].rc;
    }
    return started == threads ? rc : YVO_ERR;
}

/* ---- synthetic data ---- */

static uint64_t splitmix64(uint64_t *state)
{
    uint64_t z = (*state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

void yvo_rng_seed(yvo_rng *rng, uint64_t seed, const char *tensor_name)
{
    uint64_t hash = 0xcbf29ce484222325ull, state;
    int i;
    for (; tensor_name && *tensor_name; ++tensor_name)
        hash = (hash ^ (uint8_t)*tensor_name) * 0x100000001b3ull; /* FNV-1a */
    state = seed ^ hash;
    for (i = 0; i < 4; ++i) rng->s[i] = splitmix64(&state);
}

static uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

uint64_t yvo_rng_next(yvo_rng *rng) /* xoshiro256** */
{
    uint64_t *s = rng->s, result = rotl64(s[1] * 5u, 7) * 9u, t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}

double yvo_rng_uniform(yvo_rng *rng) { return (double)(yvo_rng_next(rng) >> 11) * 0x1.0p-53; }

void yvo_rng_normal_f32(yvo_rng *rng, float *out, uint64_t count, double sigma)
{
    uint64_t i;
    for (i = 0; i < count; i += 2u) {
        double u1 = 1.0 - yvo_rng_uniform(rng), u2 = yvo_rng_uniform(rng);
        double radius = sqrt(-2.0 * log(u1)), angle = 6.283185307179586476925 * u2;
        out[i] = (float)(sigma * radius * cos(angle));
        if (i + 1u < count) out[i + 1u] = (float)(sigma * radius * sin(angle));
    }
}

void yvo_rng_bytes(yvo_rng *rng, uint8_t *out, uint64_t count)
{
    uint64_t i = 0;
    while (i < count) {
        uint64_t word = yvo_rng_next(rng);
        int k;
        for (k = 0; k < 8 && i < count; ++k, ++i) out[i] = (uint8_t)(word >> (8 * k));
    }
}

static uint16_t positive_scale_f16(yvo_rng *rng, double sigma)
{
    float n;
    yvo_rng_normal_f32(rng, &n, 1u, 1.0);
    return yvo_f16_encode((float)(fabs((double)n) * sigma + sigma * 0.25));
}

void yvo_fill_iq2xxs(yvo_rng *rng, uint8_t *encoded, uint64_t blocks, double scale_sigma)
{
    uint64_t b;
    yvo_rng_bytes(rng, encoded, blocks * 66u);
    for (b = 0; b < blocks; ++b) {
        uint16_t d = positive_scale_f16(rng, scale_sigma);
        encoded[66u * b] = (uint8_t)(d & 0xffu);
        encoded[66u * b + 1u] = (uint8_t)(d >> 8);
    }
}

void yvo_fill_q4k(yvo_rng *rng, uint8_t *encoded, uint64_t blocks, double scale_sigma)
{
    uint64_t b;
    yvo_rng_bytes(rng, encoded, blocks * 144u);
    for (b = 0; b < blocks; ++b) {
        uint16_t d = positive_scale_f16(rng, scale_sigma);
        uint16_t dmin = positive_scale_f16(rng, scale_sigma * 8.0);
        encoded[144u * b] = (uint8_t)(d & 0xffu);
        encoded[144u * b + 1u] = (uint8_t)(d >> 8);
        encoded[144u * b + 2u] = (uint8_t)(dmin & 0xffu);
        encoded[144u * b + 3u] = (uint8_t)(dmin >> 8);
    }
}

void yvo_fill_q8_0_from_normal(yvo_rng *rng, uint8_t *encoded, uint64_t blocks, double sigma)
{
    float values[32];
    uint64_t b;
    for (b = 0; b < blocks; ++b) {
        yvo_rng_normal_f32(rng, values, 32u, sigma);
        yvo_q8_0_encode_block(values, encoded + 34u * b);
    }
}
