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
 *
 * A decision whose kernel family is the gfx950 expert sweep asks for this backend's own image of
 * an IQ2_XXS tensor instead, the one its decode sweeps read (the reference has no counterpart;
 * DERIVED_BACKEND storage is the backend's to define, layout.c:23-93 only fixes the hook):
 *   72 B per superblock, block order, two records of nine little-endian dwords, one per half
 *   superblock (four groups of 32 weights):
 *     dword 0        fp16 superblock scale | the four 4-bit group scales << 16 (group j at 16 + 4 j)
 *     dword 1 + 2 j  the four codebook indices of group j
 *     dword 2 + 2 j  the four 7-bit sign fields of group j, one to a byte
 *   Rows start on dword boundaries at any width, no load needs re-aligning, a sign field is
 *   addressed with one byte permute and the scale arrives with the codes. The shared expert may
 *   be imaged as well (expert_count 1), so that it stays in the routed experts' launch.
 */
#include "private.h"

#include <stdint.h>
#include <string.h>

#define SUPERBLOCK 256ull
#define IQ2_XXS_BYTES 66ull
#define Q2_K_BYTES 84ull
#define SECTION_ALIGN 64ull
#define SWEEP_IMAGE_BYTES 72ull

typedef struct {
    unsigned long long blocks_per_row, rows_per_expert, blocks;   /* blocks = all rows x blocks_per_row */
    unsigned long long units;          /* Q2_K: (row pair, block) units */
    unsigned long long second, third;  /* offsets of the sections behind the first */
    unsigned long long total;
    int sweep_image;
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
    int routed, sweep_image;
    if (!decision || !s)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where, "derived MoE layout decision is incomplete");
    routed = decision->consumer == YVEX_EXECUTION_CONSUMER_ROUTED_GATE_UP ||
             decision->consumer == YVEX_EXECUTION_CONSUMER_ROUTED_DOWN;
    sweep_image = !strncmp(decision->kernel_family, YVEX_MOE_KERNEL_GFX950_EXPERT_SWEEP,
                           sizeof(decision->kernel_family));
    if (sweep_image && decision->consumer == YVEX_EXECUTION_CONSUMER_SHARED_EXPERT) routed = 1;
    if (decision->layout != YVEX_EXECUTION_LAYOUT_DERIVED_BACKEND || !decision->derived_asset_required ||
        decision->expert_count < (sweep_image ? 1ull : 2ull) || !routed ||
        decision->canonical_row_count % decision->expert_count != 0ull ||
        decision->canonical_row_width % SUPERBLOCK != 0ull)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where, "derived MoE layout decision is incomplete");
    memset(s, 0, sizeof(*s));
    s->rows_per_expert = decision->canonical_row_count / decision->expert_count;
    s->blocks_per_row = decision->canonical_row_width / SUPERBLOCK;
    if (!product(decision->canonical_row_count, s->blocks_per_row, &s->blocks))
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "derived MoE block geometry overflowed");
    if (sweep_image) {
        if (decision->canonical_qtype != YVEX_GGUF_QTYPE_IQ2_XXS)
            return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, where,
                                    "the expert sweeps read an image of IQ2_XXS tensors only");
        block_bytes = IQ2_XXS_BYTES;
        s->sweep_image = 1;
        if (!product(s->blocks, SWEEP_IMAGE_BYTES, &s->total))
            return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "derived IQ2 geometry overflowed");
    } else if (decision->canonical_qtype == YVEX_GGUF_QTYPE_IQ2_XXS) {
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

static void store_le32(unsigned char *to, uint32_t v)
{
    to[0] = (unsigned char)v;
    to[1] = (unsigned char)(v >> 8);
    to[2] = (unsigned char)(v >> 16);
    to[3] = (unsigned char)(v >> 24);
}

/* The sweep image: the same re-packing yvex_hip_iq2_sweep_image_build performs on the device. */
static void pack_sweep_image(const layout_sections *s, const unsigned char *canonical, unsigned char *derived)
{
    unsigned long long b;
    for (b = 0ull; b < s->blocks; ++b, canonical += IQ2_XXS_BYTES) {
        const uint32_t d = (uint32_t)canonical[0] | ((uint32_t)canonical[1] << 8);
        unsigned int half, j;
        for (half = 0u; half < 2u; ++half, derived += SWEEP_IMAGE_BYTES / 2ull) {
            uint32_t scales = 0u;
            for (j = 0u; j < 4u; ++j) {
                const unsigned char *group = canonical + 2u + 8u * (4u * half + j);
                const uint32_t aux = (uint32_t)group[4] | ((uint32_t)group[5] << 8) |
                                     ((uint32_t)group[6] << 16) | ((uint32_t)group[7] << 24);
                memcpy(derived + 4u + 8u * j, group, 4u);
                store_le32(derived + 8u + 8u * j, (aux & 127u) | (((aux >> 7) & 127u) << 8) |
                                                      (((aux >> 14) & 127u) << 16) |
                                                      (((aux >> 21) & 127u) << 24));
                scales |= (aux >> 28) << (4u * j);
            }
            store_le32(derived, d | (scales << 16));
        }
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
    if (s.sweep_image) {
        pack_sweep_image(&s, canonical, derived);
        yvex_rocm_error_clear(err);
        return YVEX_OK;
    }
    memset(derived, 0, (size_t)storage_bytes);
    if (decision->canonical_qtype == YVEX_GGUF_QTYPE_IQ2_XXS) pack_iq2_xxs(&s, canonical, derived);
    else pack_q2_k(&s, decision->expert_count, canonical, derived);
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

/* The sweep image of a tensor whose canonical bytes are already on the device, built there (the
 * reference builds on the host and uploads; its residency step, src/runtime/residency.c:457-600,
 * has no device-side builder). The image never crosses the host link. Synchronous. */
int yvex_rocm_moe_sweep_image_build_resident(yvex_rocm_backend *backend,
                                             const yvex_physical_execution_decision *decision,
                                             unsigned long long canonical_address,
                                             unsigned long long image_address,
                                             unsigned long long storage_bytes, yvex_error *err)
{
    static const char where[] = "rocm.moe.layout.resident";
    layout_sections s;
    int device_status = 0, rc;
    if (!backend) return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, where, "backend is required");
    rc = layout_sections_of(decision, &s, err);
    if (rc != YVEX_OK) return rc;
    if (!s.sweep_image)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, where,
                                "only the expert sweeps' image is built on the device");
    if (!canonical_address || !image_address || storage_bytes != s.total || (image_address & 3ull) ||
        (canonical_address < image_address + s.total && image_address < canonical_address + decision->encoded_bytes))
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, where,
                                "separate exact derived MoE storage is required");
    rc = yvex_rocm_require_kernels(backend, where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_launch_result(yvex_hip_iq2_sweep_image_build((const uint8_t *)(uintptr_t)canonical_address,
                                                                s.blocks, (void *)(uintptr_t)image_address,
                                                                backend->stream), where, err);
    if (rc != YVEX_OK) return rc;
    rc = yvex_rocm_finish(backend, where, &device_status, err);
    if (rc != YVEX_OK) return rc;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}
