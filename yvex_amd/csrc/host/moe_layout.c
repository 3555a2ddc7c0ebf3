/*
 * Derived storage for one routed expert tensor: the size and the byte re-packing the reference
 * defines in src/backend/cuda/layout.c:23-167 (yvex_cuda_moe_derived_layout_plan / _build).
 * Host byte work over the caller's buffers; the canonical GGUF bytes stay the authority and the
 * derived image can be rebuilt from them at any time.
 *
 * Sections, each starting on a multiple of 64 bytes, padding zero:
 *   IQ2_XXS  [2 B scale per superblock, block order] [64 B codes per superblock, block order]
 *   Q2_K     rows of one expert are taken in neighbouring pairs (even, odd); a unit is one
 *            (pair, block):
 *            [8 B per unit: d, dmin of the even row, d, dmin of the odd row]
 *            [32 B per unit: sub-block scales 0-7 even, 0-7 odd, 8-15 even, 8-15 odd]
 *            [128 B per unit: the 16 code words, even row's word then odd row's word]
 */
#include "private.h"

#include <stdint.h>
#include <string.h>

#define SUPERBLOCK 256ull
#define IQ2_XXS_BYTES 66ull
#define Q2_K_BYTES 84ull
#define SECTION_ALIGN 64ull

typedef struct {
    unsigned long long blocks_per_row, rows_per_expert, blocks;   /* blocks = all rows x blocks_per_row */
    unsigned long long units;          /* Q2_K: (row pair, block) units */
    unsigned long long second, third;  /* offsets of the sections behind the first */
    unsigned long long total;
} layout_sections;

static int product(unsigned long long a, unsigned long long b, unsigned long long *out)
{
    return !__builtin_mul_overflow(a, b, out);
}

/* *out = the next multiple of 64 at or above base + count * each. */
static int section_end(unsigned long long base, unsigned long long count, unsigned long long each,
                       int align, unsigned long long *out)
{
    unsigned long long bytes, end;
    if (!product(count, each, &bytes) || __builtin_add_overflow(base, bytes, &end)) return 0;
    if (align) {
        if (__builtin_add_overflow(end, SECTION_ALIGN - 1ull, &end)) return 0;
        end &= ~(SECTION_ALIGN - 1ull);
    }
    *out = end;
    return 1;
}

static int layout_sections_of(const yvex_physical_execution_decision *decision, layout_sections *s,
                              yvex_error *err)
{
    static const char where[] = "rocm.moe.layout";
    unsigned long long block_bytes, canonical;
    int routed;
    if (!decision || !s)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where, "derived MoE layout decision is incomplete");
    routed = decision->consumer == YVEX_EXECUTION_CONSUMER_ROUTED_GATE_UP ||
             decision->consumer == YVEX_EXECUTION_CONSUMER_ROUTED_DOWN;
    if (decision->layout != YVEX_EXECUTION_LAYOUT_DERIVED_BACKEND || !decision->derived_asset_required ||
        decision->expert_count <= 1ull || !routed ||
        decision->canonical_row_count % decision->expert_count != 0ull ||
        decision->canonical_row_width % SUPERBLOCK != 0ull)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where, "derived MoE layout decision is incomplete");
    memset(s, 0, sizeof(*s));
    s->rows_per_expert = decision->canonical_row_count / decision->expert_count;
    s->blocks_per_row = decision->canonical_row_width / SUPERBLOCK;
    if (!product(decision->canonical_row_count, s->blocks_per_row, &s->blocks))
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "derived MoE block geometry overflowed");
    if (decision->canonical_qtype == YVEX_GGUF_QTYPE_IQ2_XXS) {
        block_bytes = IQ2_XXS_BYTES;
        if (!section_end(0ull, s->blocks, 2ull, 1, &s->second) ||
            !section_end(s->second, s->blocks, 64ull, 0, &s->total))
            return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "derived IQ2 geometry overflowed");
    } else if (decision->canonical_qtype == YVEX_GGUF_QTYPE_Q2_K) {
        unsigned long long pairs;
        block_bytes = Q2_K_BYTES;
        if (s->rows_per_expert % 2ull != 0ull ||
            !product(decision->expert_count, s->rows_per_expert / 2ull, &pairs) ||
            !product(pairs, s->blocks_per_row, &s->units) ||
            !section_end(0ull, s->units, 8ull, 1, &s->second) ||
            !section_end(s->second, s->units, 32ull, 1, &s->third) ||
            !section_end(s->third, s->units, 128ull, 0, &s->total))
            return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "derived Q2 geometry overflowed");
    } else {
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, where, "derived MoE layout qtype is not admitted");
    }
    if (!product(s->blocks, block_bytes, &canonical) || canonical != decision->encoded_bytes ||
        s->total < decision->encoded_bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where,
                                "derived MoE layout differs from canonical geometry");
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_moe_derived_layout_plan(const yvex_physical_execution_decision *decision,
                                      unsigned long long *storage_bytes, yvex_error *err)
{
    layout_sections s;
    int rc;
    if (!storage_bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.layout",
                                "derived MoE storage output is required");
    *storage_bytes = 0ull;
    rc = layout_sections_of(decision, &s, err);
    if (rc == YVEX_OK) *storage_bytes = s.total;
    return rc;
}

static void pack_iq2_xxs(const layout_sections *s, const unsigned char *canonical, unsigned char *derived)
{
    unsigned char *scales = derived, *codes = derived + s->second;
    unsigned long long b;
    for (b = 0ull; b < s->blocks; ++b, canonical += IQ2_XXS_BYTES, scales += 2, codes += 64) {
        memcpy(scales, canonical, 2u);
        memcpy(codes, canonical + 2, 64u);
    }
}

/* One Q2_K block (16 scale bytes, 64 code bytes, d, dmin) of the row with this parity into the
 * three records of its unit. */
static void pack_q2_k_block(const unsigned char *block, unsigned int parity, unsigned char *factors,
                            unsigned char *scales, unsigned char *codes)
{
    unsigned int w;
    memcpy(factors + 4u * parity, block + 80, 4u);
    memcpy(scales + 8u * parity, block, 8u);             /* sub-blocks 0-7 */
    memcpy(scales + 16u + 8u * parity, block + 8, 8u);   /* sub-blocks 8-15 */
    for (w = 0u; w < 16u; ++w) memcpy(codes + 8u * w + 4u * parity, block + 16u + 4u * w, 4u);
}

static void pack_q2_k(const layout_sections *s, unsigned long long experts, const unsigned char *canonical,
                      unsigned char *derived)
{
    unsigned long long rows = experts * s->rows_per_expert, row, b;
    for (row = 0ull; row < rows; ++row) {
        /* rows_per_expert is even, so row / 2 counts the pairs across experts as well */
        unsigned long long unit = (row / 2ull) * s->blocks_per_row;
        unsigned int parity = (unsigned int)(row & 1ull);
        for (b = 0ull; b < s->blocks_per_row; ++b, ++unit, canonical += Q2_K_BYTES)
            pack_q2_k_block(canonical, parity, derived + unit * 8ull, derived + s->second + unit * 32ull,
                            derived + s->third + unit * 128ull);
    }
}

int yvex_rocm_moe_derived_layout_build(const yvex_physical_execution_decision *decision,
                                       const unsigned char *canonical, unsigned long long canonical_bytes,
                                       unsigned char *derived, unsigned long long storage_bytes,
                                       yvex_error *err)
{
    layout_sections s;
    int rc = layout_sections_of(decision, &s, err);
    if (rc != YVEX_OK) return rc;
    if (!canonical || !derived || canonical == derived || canonical_bytes != decision->encoded_bytes ||
        storage_bytes != s.total || storage_bytes > (unsigned long long)SIZE_MAX)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.layout",
                                "separate exact derived MoE storage is required");
    memset(derived, 0, (size_t)storage_bytes);
    if (decision->canonical_qtype == YVEX_GGUF_QTYPE_IQ2_XXS) pack_iq2_xxs(&s, canonical, derived);
    else pack_q2_k(&s, decision->expert_count, canonical, derived);
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}
