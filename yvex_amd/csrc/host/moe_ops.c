/*
 * MoE row-batch operations of the ROCm backend (host side) and the host worklist builder.
 * Restates the contract of src/backend/cuda/moe.c:113-183 (workspace), :905-990 (activation and
 * kernel-family policy), :1826-1981 (execute / complete / operations table) and the sorting core
 * of src/graph/worklist.c:369-441. All device work is enqueued on the backend's stream through
 * the launch-level ABI; one synchronisation per layer publishes status, routing and worklist facts.
 */
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "private.h"

#define ALIGN 256ull

static unsigned long long align_up(unsigned long long v) { return (v + ALIGN - 1ull) & ~(ALIGN - 1ull); }

static unsigned long long monotonic_ns(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (unsigned long long)ts.tv_sec * 1000000000ull + (unsigned long long)ts.tv_nsec;
}

/* Byte ranges bump-allocated from the attached workspace, in this order. */
typedef struct {
    unsigned long long input_q8, logits, bias, selected, weights;
    unsigned long long order, expert_ids, bucket_offsets, bucket_populations, sweep_offsets, counts;
    unsigned long long intermediate, intermediate_q8, pair_outputs;
    unsigned long long shared_intermediate, shared_intermediate_q8, shared_outputs, routed;
    /* residual-stream envelope (layers whose plan names mixing rows) */
    unsigned long long mixes, scale, base, norm, normalized, post, combination, combined;
    unsigned long long tokens;    /* hash router: the rows' token ids */
    int joined_intermediates;     /* shared expert's intermediate rows follow the routed pairs' */
    unsigned long long total;
} moe_ranges;

/* Layers that carry residual streams run the reference's ingress and egress around the expert
 * math (src/backend/cuda/moe.c:1210-1254,1533-1541); a plan without mixing rows hands this
 * backend rows that are already normalised. Geometry as src/graph/numeric.c:668-689 asks. */
static int moe_envelope(const yvex_moe_layer_plan *layer)
{
    return layer->mhc_mixing_rows != 0ull;
}

int yvex_rocm_moe_envelope_geometry(const yvex_moe_layer_plan *layer)
{
    unsigned long long streams = layer->residual_streams;
    return streams >= 1ull && streams <= 7ull && layer->hidden_width <= 16384ull &&
           layer->expanded_width == streams * layer->hidden_width &&
           layer->mhc_mixing_rows == (streams + 2ull) * streams &&
           layer->mhc_sinkhorn_iterations > 0ull && layer->mhc_sinkhorn_iterations <= 0xffffffffull &&
           isfinite(layer->rms_epsilon) && layer->rms_epsilon > 0.0 &&
           isfinite(layer->mhc_epsilon) && layer->mhc_epsilon > 0.0 &&
           isfinite(layer->mhc_post_multiplier) && layer->mhc_post_multiplier > 0.0;
}

static int moe_layout(const yvex_moe_layer_plan *layer, unsigned long long rows, moe_ranges *r)
{
    unsigned long long cursor = 0ull, pairs, hidden, routed_i, shared_i, experts, streams;
    if (!layer || !rows || rows > YVEX_ROCM_MOE_MAX_ROWS || !layer->hidden_width ||
        !layer->routed_experts || layer->routed_experts > 256ull || !layer->experts_per_token ||
        layer->experts_per_token > YVEX_MOE_MAX_SELECTED ||
        layer->experts_per_token > layer->routed_experts || !layer->expert_intermediate_width ||
        layer->hidden_width > (1ull << 20) || layer->expert_intermediate_width > (1ull << 20) ||
        layer->shared_intermediate_width > (1ull << 20) || layer->shared_experts > 1ull ||
        (moe_envelope(layer) && !yvex_rocm_moe_envelope_geometry(layer)))
        return 0;
    streams = moe_envelope(layer) ? layer->residual_streams : 0ull;
    pairs = rows * layer->experts_per_token;
    hidden = layer->hidden_width;
    routed_i = layer->expert_intermediate_width;
    shared_i = layer->shared_experts ? layer->shared_intermediate_width : 0ull;
    experts = layer->routed_experts;
#define TAKE(field, bytes) do { r->field = cursor; cursor = align_up(cursor + (bytes)); } while (0)
    TAKE(input_q8, rows * ((hidden + 255ull) / 256ull) * 292ull);
    TAKE(logits, rows * experts * sizeof(float));
    TAKE(bias, experts * sizeof(float));
    TAKE(selected, pairs * sizeof(unsigned long long));
    TAKE(weights, pairs * sizeof(float));
    TAKE(order, pairs * sizeof(unsigned long long));
    TAKE(expert_ids, experts * sizeof(unsigned long long));
    TAKE(bucket_offsets, (experts + 1ull) * sizeof(unsigned long long));
    TAKE(bucket_populations, experts * sizeof(unsigned long long));
    TAKE(sweep_offsets, (experts + 1ull) * sizeof(unsigned long long));
    TAKE(counts, 4ull * sizeof(unsigned long long));
    /* With a shared expert of the routed width its intermediate rows are laid right behind the
     * routed pairs' (F32 and Q8_K alike), so one launch quantizes both. Q8_K rows are read with
     * 16-byte loads, which the offset must respect. */
    r->joined_intermediates = shared_i == routed_i && routed_i % 256ull == 0ull &&
                              (pairs * (routed_i / 256ull) * 292ull) % 16ull == 0ull &&
                              (pairs * routed_i * sizeof(float)) % 16ull == 0ull;
    if (r->joined_intermediates) {
        TAKE(intermediate, (pairs + rows) * routed_i * sizeof(float));
        TAKE(intermediate_q8, (pairs + rows) * (routed_i / 256ull) * 292ull);
        r->shared_intermediate = r->intermediate + pairs * routed_i * sizeof(float);
        r->shared_intermediate_q8 = r->intermediate_q8 + pairs * (routed_i / 256ull) * 292ull;
    } else {
        TAKE(intermediate, pairs * routed_i * sizeof(float));
        TAKE(intermediate_q8, pairs * ((routed_i + 255ull) / 256ull) * 292ull);
    }
    TAKE(pair_outputs, pairs * hidden * sizeof(float));
    if (!r->joined_intermediates) {
        TAKE(shared_intermediate, rows * shared_i * sizeof(float));
        TAKE(shared_intermediate_q8, rows * ((shared_i + 255ull) / 256ull) * 292ull);
    }
    TAKE(shared_outputs, rows * hidden * sizeof(float));
    TAKE(routed, rows * hidden * sizeof(float));
    if (streams) {
        TAKE(mixes, rows * layer->mhc_mixing_rows * sizeof(float));
        TAKE(scale, 3ull * sizeof(float));
        TAKE(base, layer->mhc_mixing_rows * sizeof(float));
        TAKE(norm, hidden * sizeof(float));
        TAKE(normalized, rows * hidden * sizeof(float));
        TAKE(post, rows * streams * sizeof(float));
        TAKE(combination, rows * streams * streams * sizeof(float));
        TAKE(combined, rows * hidden * sizeof(float));
    }
    if (layer->router_class == YVEX_MOE_ROUTER_HASH_TOKEN_ID) TAKE(tokens, rows * sizeof(unsigned int));
#undef TAKE
    r->total = cursor + ALIGN;   /* slack for aligning the workspace base itself */
    return 1;
}

int yvex_rocm_moe_workspace_required(const yvex_moe_layer_plan *layer, unsigned long long row_count,
                                  unsigned long long *bytes, yvex_error *err)
{
    moe_ranges ranges;
    if (bytes) *bytes = 0ull;
    if (!bytes || !moe_layout(layer, row_count, &ranges))
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.workspace",
                                "MoE layer geometry or row count is outside this backend's bounds");
    *bytes = ranges.total;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

static int q8_eligible(unsigned int qtype)
{
    return qtype == YVEX_GGUF_QTYPE_Q8_0 || qtype == YVEX_GGUF_QTYPE_Q2_K ||
           qtype == YVEX_GGUF_QTYPE_Q4_K || qtype == YVEX_GGUF_QTYPE_IQ2_XXS;
}

static int family_admitted(const char *family)
{
    return family && (!strcmp(family, YVEX_MOE_KERNEL_PORTABLE_EXPERT_ROW) ||
                      !strcmp(family, YVEX_MOE_KERNEL_PORTABLE_ENCODED_ROW) ||
                      !strcmp(family, YVEX_MOE_KERNEL_GFX950_EXPERT_SWEEP));
}

/* Activation / kernel-family policy of one expert triple (moe.c:905-990). */
static int expert_policy(const yvex_moe_weight_view *gate, const yvex_moe_weight_view *up,
                         const yvex_moe_weight_view *down, unsigned long long input_width,
                         unsigned long long intermediate_width, int *act_q8, int *image, yvex_error *err)
{
    int gate_encoded, up_encoded, down_encoded;
    *image = 0;
    if (gate->activation > YVEX_EXECUTION_ACTIVATION_DEVICE_ENCODED ||
        up->activation > YVEX_EXECUTION_ACTIVATION_DEVICE_ENCODED ||
        down->activation > YVEX_EXECUTION_ACTIVATION_DEVICE_ENCODED)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.policy",
                                "MoE activation policy is invalid");
    gate_encoded = gate->activation == YVEX_EXECUTION_ACTIVATION_DEVICE_ENCODED;
    up_encoded = up->activation == YVEX_EXECUTION_ACTIVATION_DEVICE_ENCODED;
    down_encoded = down->activation == YVEX_EXECUTION_ACTIVATION_DEVICE_ENCODED;
    if (gate_encoded != up_encoded)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.policy",
                                "MoE gate/up activations disagree");
    if (gate_encoded && (!gate->kernel_family || !up->kernel_family ||
                         strcmp(gate->kernel_family, up->kernel_family) != 0))
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.policy",
                                "compiled MoE gate and up kernel-family decisions disagree");
    /* moe.c:933-958: layouts must agree (FORMAT). The reference's row-batch path executes no
     * derived image at all (UNSUPPORTED); this one executes the one image its expert sweeps
     * read: IQ2_XXS tensors, device-encoded activations, the gfx950 sweep family on all three
     * views. Any other derived view is refused as there. */
    /* One exception to the agreement: Q2_K down rows have no image (the sweeps read them as they
     * lie), so canonical Q2_K down rows beside imaged IQ2_XXS gate and up rows are admitted, the
     * pairing of the reference's model file. *image: bit 0 gate and up, bit 1 down. */
    {
        const int gate_derived = gate->layout == YVEX_EXECUTION_LAYOUT_DERIVED_BACKEND;
        const int down_derived = down->layout == YVEX_EXECUTION_LAYOUT_DERIVED_BACKEND;
        const int q2k_down_as_it_lies = gate_derived && !down_derived && down->qtype == YVEX_GGUF_QTYPE_Q2_K;
        if (gate->layout != up->layout || (gate_derived != down_derived && !q2k_down_as_it_lies))
            return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.policy",
                                    "compiled routed MoE layouts disagree");
        if (gate_derived) {
            if (!gate_encoded || !down_encoded || !down->kernel_family ||
                strcmp(gate->kernel_family, YVEX_MOE_KERNEL_GFX950_EXPERT_SWEEP) != 0 ||
                strcmp(down->kernel_family, YVEX_MOE_KERNEL_GFX950_EXPERT_SWEEP) != 0 ||
                gate->qtype != YVEX_GGUF_QTYPE_IQ2_XXS || up->qtype != YVEX_GGUF_QTYPE_IQ2_XXS ||
                (down_derived && down->qtype != YVEX_GGUF_QTYPE_IQ2_XXS))
                return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.policy",
                                        "the row-batch path executes canonical rows, or the expert sweeps' "
                                        "image of IQ2_XXS tensors with device-encoded activations");
            *image = down_derived ? 3 : 1;
        }
    }
    if ((gate_encoded && !family_admitted(gate->kernel_family)) ||
        (down_encoded && !family_admitted(down->kernel_family)))
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.policy",
                                "compiled MoE kernel family is not admitted by the rocm backend");
    if (gate_encoded != down_encoded)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.policy",
                                "gate/up and down projections must share one activation class");
    if (gate_encoded && (input_width % 256ull || intermediate_width % 256ull ||
                         !q8_eligible(gate->qtype) || !q8_eligible(up->qtype) ||
                         !q8_eligible(down->qtype)))
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.policy",
                                "compiled MoE activation is incompatible with its qtype geometry");
    *act_q8 = gate_encoded;
    return YVEX_OK;
}

/* Check one weight view against the geometry the plan implies and find its device address. */
int yvex_rocm_moe_view_check(const yvex_rocm_backend *backend, const yvex_moe_weight_view *view,
                             unsigned long long row_width, unsigned long long row_count,
                             unsigned long long *device_address, int *resident, yvex_error *err)
{
    const yvex_rocm_numeric_capability *capability = yvex_rocm_quant_numeric_capability_at(view->qtype);
    const yvex_rocm_qtype_geometry *geometry = yvex_rocm_gguf_qtype_geometry_find(view->qtype);
    if (!capability || !geometry || !capability->device_compute_available)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.weights",
                                "qtype has no device compute on this backend");
    if (view->layout == YVEX_EXECUTION_LAYOUT_DERIVED_BACKEND)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.weights",
                                "this operation takes canonical rows, not a derived image");
    if (view->row_width != row_width || view->row_count != row_count || !geometry->block_size ||
        row_width % geometry->block_size ||
        row_width / geometry->block_size * geometry->bytes_per_block != view->row_bytes ||
        view->row_bytes > ULLONG_MAX / (row_count ? row_count : 1ull) ||
        view->row_bytes * row_count != view->encoded_bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.weights",
                                "MoE weight view geometry disagrees with the layer plan");
    *resident = 1;
    *device_address = 0ull;
    if (view->device_address) {
        *device_address = view->device_address;
        return YVEX_OK;
    }
    if (!view->encoded)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.weights", "MoE weight view has no bytes");
    if (!yvex_rocm_resolve(backend, view->encoded, view->encoded_bytes, device_address)) {
        *resident = 0;
        *device_address = 0ull;
    }
    return YVEX_OK;
}

static int view_resolve(const yvex_rocm_backend *backend, const yvex_moe_weight_view *view,
                        unsigned long long row_width, unsigned long long row_count,
                        unsigned long long *device_address, yvex_error *err)
{
    int resident = 0;
    int rc = yvex_rocm_moe_view_check(backend, view, row_width, row_count, device_address, &resident, err);
    if (rc == YVEX_OK && !resident)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.weights",
                                "MoE weight view is not inside the attached resident arena");
    return rc;
}

/* A view of the expert sweeps' image (src/runtime/moe.c:297-300 hands a derived binding over the
 * same way): row geometry and encoded_bytes describe the canonical tensor, `encoded` (or
 * device_address) and storage_bytes the image, 72 bytes per superblock. */
static int image_view_resolve(const yvex_rocm_backend *backend, const yvex_moe_weight_view *view,
                              unsigned long long row_width, unsigned long long row_count,
                              unsigned long long *device_address, yvex_error *err)
{
    unsigned long long blocks;
    if (view->row_width != row_width || view->row_count != row_count || row_width % 256ull ||
        view->row_bytes != row_width / 256ull * 66ull ||
        __builtin_mul_overflow(row_width / 256ull, row_count, &blocks) || blocks > ULLONG_MAX / 72ull ||
        view->encoded_bytes != blocks * 66ull || view->storage_bytes != blocks * 72ull)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.weights",
                                "MoE weight image disagrees with the layer plan");
    if (view->device_address) {
        *device_address = view->device_address;
    } else if (!view->encoded ||
               !yvex_rocm_resolve(backend, view->encoded, view->storage_bytes, device_address)) {
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.weights",
                                "MoE weight image is not inside the attached resident arena");
    }
    if (*device_address & 3ull)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.weights",
                                "MoE weight image must start on a dword boundary");
    return YVEX_OK;
}

static int expert_view_resolve(const yvex_rocm_backend *backend, const yvex_moe_weight_view *view, int image,
                               unsigned long long row_width, unsigned long long row_count,
                               unsigned long long *device_address, yvex_error *err)
{
    return image ? image_view_resolve(backend, view, row_width, row_count, device_address, err)
                 : view_resolve(backend, view, row_width, row_count, device_address, err);
}

static void fill_expert_weights(yvex_hip_expert_weights *w, const yvex_moe_weight_view *gate,
                                const yvex_moe_weight_view *up, const yvex_moe_weight_view *down,
                                unsigned long long gate_address, unsigned long long up_address,
                                unsigned long long down_address, unsigned long long hidden,
                                unsigned long long intermediate, int image)
{
    /* image: bit 0 the gate and up matrices, bit 1 the down matrix */
    const unsigned long long gate_row = (image & 1) ? hidden / 256ull * 72ull : gate->row_bytes;
    const unsigned long long up_row = (image & 1) ? hidden / 256ull * 72ull : up->row_bytes;
    const unsigned long long down_row = (image & 2) ? intermediate / 256ull * 72ull : down->row_bytes;
    w->gate = (const uint8_t *)(uintptr_t)gate_address;
    w->up = (const uint8_t *)(uintptr_t)up_address;
    w->down = (const uint8_t *)(uintptr_t)down_address;
    w->gate_qtype = gate->qtype;
    w->up_qtype = up->qtype;
    w->down_qtype = down->qtype;
    w->hidden = hidden;
    w->intermediate = intermediate;
    w->gate_row_bytes = gate_row;
    w->up_row_bytes = up_row;
    w->down_row_bytes = down_row;
    w->gate_expert_bytes = gate_row * intermediate;
    w->up_expert_bytes = up_row * intermediate;
    w->down_expert_bytes = down_row * hidden;
    w->gate_up_image = image & 1;
    w->down_image = (image >> 1) & 1;
}

/* Expert weights the matrix-core row-batch kernels take: gate and up of one format, IQ2_XXS (16)
 * or Q4_K (12); the down matrix of either or Q2_K (10), the pairing the reference's own
 * tensor-core kernels serve (IQ2_XXS gate and up, src/backend/cuda/tensorcore.cu:563-564; Q2_K
 * down, tensorcore.cu:660). */
static int matrix_core_qtypes(const yvex_hip_expert_weights *w)
{
    return w->gate_qtype == w->up_qtype && (w->gate_qtype == 16u || w->gate_qtype == 12u) &&
           (w->down_qtype == 16u || w->down_qtype == 12u || w->down_qtype == 10u);
}

static int same_expert_shape(const yvex_hip_expert_weights *a, const yvex_hip_expert_weights *b)
{
    return a->gate_qtype == b->gate_qtype && a->up_qtype == b->up_qtype &&
           a->down_qtype == b->down_qtype && a->hidden == b->hidden &&
           a->intermediate == b->intermediate && a->gate_up_image == b->gate_up_image &&
           a->down_image == b->down_image;
}

/* ---- launch graphs -------------------------------------------------------------------------
 * The launch sequence of a row batch depends only on facts the host knows before the first
 * kernel: the layer's geometry and policies, the weight views, the row count, and the device
 * addresses of rows, outputs, weights and workspace. The reference keys a captured graph on the
 * same topology (src/backend/cuda/moe.c:1545-1643) and replays it unless the job asks for eager
 * execution (moe.c:1650-1681). Here a key seen for the first time runs eagerly, the second time
 * it is captured and launched, and from then on it is replayed; sixteen keys are kept, the least
 * recently used one making room. Everything a kernel argument is computed from is in the key,
 * so a replay submits exactly the launches the eager sequence would. */
enum { GRAPH_SLOTS = 16, GRAPH_KEY_WORDS = 176 };

typedef struct {
    unsigned long long words[GRAPH_KEY_WORDS];
    unsigned int count;
    int overflow;
} graph_key;

typedef struct {
    graph_key key;
    yvex_hip_graph graph;              /* NULL: seen once, ran eagerly */
    unsigned long long launches, last_use;
    int used;
    int eager_only;                    /* a launch wrapper refused this job while it was recorded */
} graph_slot;

struct yvex_rocm_moe_graphs {
    graph_slot slots[GRAPH_SLOTS];
    unsigned long long clock;
    int refused;                       /* a capture failed: this backend stays eager */
};

static void key_word(graph_key *key, unsigned long long value)
{
    if (key->count < GRAPH_KEY_WORDS) key->words[key->count++] = value;
    else key->overflow = 1;
}

static void key_real(graph_key *key, double value)
{
    unsigned long long bits = 0ull;
    memcpy(&bits, &value, sizeof(bits));
    key_word(key, bits);
}

static void key_layer(graph_key *key, const yvex_moe_layer_plan *layer)
{
    key_word(key, (unsigned long long)layer->router_class);
    key_word(key, (unsigned long long)layer->scoring);
    key_word(key, (unsigned long long)layer->topk_policy);
    key_word(key, (unsigned long long)layer->activation);
    key_word(key, layer->hidden_width);
    key_word(key, layer->residual_streams);
    key_word(key, layer->expanded_width);
    key_word(key, layer->mhc_mixing_rows);
    key_word(key, layer->mhc_sinkhorn_iterations);
    key_word(key, layer->routed_experts);
    key_word(key, layer->shared_experts);
    key_word(key, layer->experts_per_token);
    key_word(key, layer->expert_intermediate_width);
    key_word(key, layer->shared_intermediate_width);
    key_word(key, layer->hash_table_rows);
    key_word(key, layer->hash_table_columns);
    key_word(key, layer->correction_bias_width);
    key_real(key, layer->rms_epsilon);
    key_real(key, layer->mhc_epsilon);
    key_real(key, layer->mhc_post_multiplier);
    key_real(key, layer->routed_scaling_factor);
    key_real(key, layer->activation_limit);
    key_word(key, (unsigned long long)layer->requires_token_ids);
    key_word(key, (unsigned long long)layer->requires_correction_bias);
    key_word(key, (unsigned long long)layer->normalize_topk_probabilities);
}

static void key_view(graph_key *key, const yvex_moe_weight_view *view, unsigned long long address)
{
    key_word(key, view->qtype);
    key_word(key, (unsigned long long)view->layout);
    key_word(key, (unsigned long long)view->activation);
    key_word(key, view->encoded_bytes);
    key_word(key, view->row_bytes);
    key_word(key, view->row_width);
    key_word(key, view->row_count);
    key_word(key, address);
}

static graph_slot *graph_find(struct yvex_rocm_moe_graphs *cache, const graph_key *key)
{
    unsigned int i;
    for (i = 0u; i < GRAPH_SLOTS; ++i)
        if (cache->slots[i].used && cache->slots[i].key.count == key->count &&
            !memcmp(cache->slots[i].key.words, key->words, key->count * sizeof(key->words[0])))
            return &cache->slots[i];
    return NULL;
}

static graph_slot *graph_admit(struct yvex_rocm_moe_graphs *cache, const graph_key *key)
{
    unsigned int i, oldest = 0u;
    for (i = 0u; i < GRAPH_SLOTS; ++i) {
        if (!cache->slots[i].used) { oldest = i; break; }
        if (cache->slots[i].last_use < cache->slots[oldest].last_use) oldest = i;
    }
    if (cache->slots[oldest].used && cache->slots[oldest].graph)
        (void)yvex_hip_graph_destroy(cache->slots[oldest].graph);
    memset(&cache->slots[oldest], 0, sizeof(cache->slots[oldest]));
    cache->slots[oldest].key = *key;
    cache->slots[oldest].used = 1;
    return &cache->slots[oldest];
}

/* Graphs name device addresses: whoever frees or re-attaches what they point into drops them.
 * The caller has synchronised the stream (or nothing was ever launched). */
void yvex_rocm_moe_graphs_release(yvex_rocm_backend *backend)
{
    unsigned int i;
    if (!backend || !backend->moe_graphs) return;
    for (i = 0u; i < GRAPH_SLOTS; ++i)
        if (backend->moe_graphs->slots[i].used && backend->moe_graphs->slots[i].graph)
            (void)yvex_hip_graph_destroy(backend->moe_graphs->slots[i].graph);
    free(backend->moe_graphs);
    backend->moe_graphs = NULL;
}

/* The structural half of yvex_expert_worklist_policy_seal (src/graph/worklist.c:252-272): width 1
 * admitted, width 0 and bit 63 not, a narrow family named, and a tensor-core minimum that is an
 * admitted width below 63 with a family of its own. */
static int worklist_policy_valid(const yvex_expert_worklist_policy *policy)
{
    int tensor_core;
    if (!policy || policy->schema_version != YVEX_EXPERT_WORKLIST_POLICY_SCHEMA_V1 ||
        !(policy->supported_width_mask & 2ull) || (policy->supported_width_mask & 1ull) ||
        (policy->supported_width_mask >> 63u) || !policy->narrow_kernel_family[0])
        return 0;
    tensor_core = policy->tensor_core_minimum != 0ull;
    if (tensor_core != (policy->tensor_core_kernel_family[0] != '\0')) return 0;
    if (tensor_core &&
        (policy->tensor_core_minimum >= 63ull ||
         !(policy->supported_width_mask & (1ull << policy->tensor_core_minimum)) ||
         !strncmp(policy->narrow_kernel_family, policy->tensor_core_kernel_family,
                  sizeof(policy->narrow_kernel_family))))
        return 0;
    return 1;
}

static int moe_execute_rows(yvex_rocm_backend *backend, const yvex_moe_layer_job *job,
                            const yvex_moe_row_batch *rows, const yvex_moe_row_batch_output *output,
                            yvex_moe_row_batch_result *result, yvex_error *err)
{
    const yvex_moe_layer_plan *layer = job ? job->layer : NULL;
    const yvex_moe_weight_view *views = job ? job->weights : NULL;
    yvex_hip_expert_weights routed, shared;
    moe_ranges ranges;
    unsigned long long base, pairs, hidden, experts, topk, row_count, launches = 0ull;
    unsigned long long router_address = 0ull, bias_address = 0ull, addresses[6] = {0};
    unsigned long long envelope_addresses[4] = {0}, streams = 0ull, expanded;
    unsigned long long d2h = 0ull, started, counts[4] = {0}, status_launches = 0ull;
    const void *activations;
    const float *bias_rows;
    void *combined_target;
    unsigned long long table_address = 0ull;
    int matrix_allowed = 1, envelope, hash_router, unsupported_width, routed_q8 = 0, shared_q8 = 0, routed_image = 0, shared_image = 0, has_shared, merged, row_batch, shared_row_batch, shared_dense, device_status = 0, rc, defer, scored = 0;
    void *status;
    yvex_hip_stream stream;
    enum { GRAPH_EAGER = 0, GRAPH_CAPTURE, GRAPH_REPLAY } graph_mode = GRAPH_EAGER;
    graph_slot *graph_target = NULL;
    if (result) memset(result, 0, sizeof(*result));
    /* src/backend/cuda/moe.c:1840-1852: batch and policy come together, are structurally valid,
     * describe the same rows, and a profile identity needs both; a width outside the policy's
     * mask is UNSUPPORTED, the rest INVALID_ARG */
    unsupported_width = job && rows && job->worklist_policy &&
                        (rows->row_count >= 63ull ||
                         !(job->worklist_policy->supported_width_mask & (1ull << rows->row_count)));
    if (!backend || !job || !layer || !rows || !output || !result ||
        backend->kind != YVEX_BACKEND_KIND_ROCM ||
        ((job->execution_batch == NULL) != (job->worklist_policy == NULL)) ||
        (job->execution_batch &&
         (job->execution_batch->schema_version != YVEX_EXECUTION_BATCH_SCHEMA_V1 ||
          !worklist_policy_valid(job->worklist_policy) ||
          job->execution_batch->row_count != rows->row_count ||
          job->execution_batch->provenance != rows->provenance ||
          job->execution_batch->phase != rows->phase)) ||
        (rows->execution_profile_identity && (!job->execution_batch || !job->worklist_policy)) ||
        unsupported_width)
        return unsupported_width
            ? yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.rows",
                               "row count is outside the sealed supported width mask")
            : yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.rows",
                               "width-N MoE owners, execution batch or worklist policy are invalid");
    if (
        rows->schema_version != YVEX_MOE_ROW_BATCH_SCHEMA_V1 || !rows->row_count ||
        rows->row_count > YVEX_ROCM_MOE_MAX_ROWS || rows->row_width != layer->expanded_width ||
        rows->row_stride != rows->row_width ||
        !yvex_rocm_tensor_owner_is(backend, rows->device_rows) ||
        !yvex_rocm_tensor_owner_is(backend, rows->device_outputs) ||
        rows->device_rows == rows->device_outputs || !rows->device_rows->is_written ||
        rows->device_rows->dtype != YVEX_DTYPE_F32 || rows->device_outputs->dtype != YVEX_DTYPE_F32 ||
        rows->device_rows->bytes < rows->row_count * rows->row_width * sizeof(float) ||
        rows->device_outputs->bytes < rows->row_count * rows->row_width * sizeof(float))
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.rows",
                                "width-N MoE owners, geometry or admitted width are invalid");
    envelope = moe_envelope(layer);
    hash_router = layer->router_class == YVEX_MOE_ROUTER_HASH_TOKEN_ID;
    if ((!envelope && layer->expanded_width != layer->hidden_width) ||
        (!hash_router && layer->router_class != YVEX_MOE_ROUTER_LEARNED_HIDDEN_STATE) ||
        (layer->scoring != YVEX_MOE_SCORING_SQRT_SOFTPLUS && layer->scoring != YVEX_MOE_SCORING_SIGMOID))
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.rows",
                                "other router classes, other scoring policies and expanded rows without mixing rows are outside this backend");
    if (envelope && !yvex_rocm_moe_envelope_geometry(layer))
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.rows",
                                "residual-stream geometry is invalid");
    streams = envelope ? layer->residual_streams : 0ull;
    expanded = layer->expanded_width;
    row_count = rows->row_count;
    hidden = layer->hidden_width;
    experts = layer->routed_experts;
    topk = layer->experts_per_token;
    if (!moe_layout(layer, row_count, &ranges))
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.rows",
                                "MoE layer geometry is outside this backend's bounds");
    pairs = row_count * topk;
    if ((output->selected_experts || output->selected_weights) && output->selection_capacity < pairs)
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.rows", "selection capacity is too small");
    if ((output->combined_rows && output->combined_capacity < row_count * hidden) ||
        (output->routed_rows && output->routed_capacity < row_count * hidden) ||
        (output->shared_rows && output->shared_capacity < row_count * hidden) ||
        (envelope && output->post_rows && output->post_capacity < row_count * streams) ||
        (envelope && output->combination_rows &&
         output->combination_capacity < row_count * streams * streams))
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.rows", "host output capacity is too small");
    if (hash_router) {
        /* src/graph/moe.c:539-549: one in-vocabulary token id per row, an I32 table */
        const yvex_moe_weight_view *table = &views[YVEX_MOE_WEIGHT_ROUTER_TABLE];
        unsigned long long r;
        if (!rows->token_ids || !rows->token_ids_present || !layer->hash_table_rows ||
            table->qtype != YVEX_GGUF_QTYPE_I32 || table->row_bytes < topk * 4ull || (table->row_bytes & 3ull))
            return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.rows",
                                    "MoE hash router requires one in-vocabulary token ID");
        for (r = 0ull; r < row_count; ++r)
            if (rows->token_ids[r] >= layer->hash_table_rows)
                return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.rows",
                                        "MoE hash router requires one in-vocabulary token ID");
    }
    if (job->cancel_requested && job->cancel_requested(job->cancel_context))
        return yvex_rocm_refuse(err, YVEX_ERR_CANCELLED, "rocm.moe.rows",
                                "width-N MoE was cancelled before launch");
    if (!backend->workspace_device_tensor || backend->workspace_bytes < ranges.total)
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, "rocm.moe.rows",
                                "width-N MoE workspace was not preflighted");
    has_shared = layer->shared_experts == 1ull;
    rc = expert_policy(&views[YVEX_MOE_WEIGHT_ROUTED_GATE], &views[YVEX_MOE_WEIGHT_ROUTED_UP],
                       &views[YVEX_MOE_WEIGHT_ROUTED_DOWN], hidden, layer->expert_intermediate_width,
                       &routed_q8, &routed_image, err);
    if (rc == YVEX_OK && has_shared)
        rc = expert_policy(&views[YVEX_MOE_WEIGHT_SHARED_GATE], &views[YVEX_MOE_WEIGHT_SHARED_UP],
                           &views[YVEX_MOE_WEIGHT_SHARED_DOWN], hidden, layer->shared_intermediate_width,
                           &shared_q8, &shared_image, err);
    if (rc != YVEX_OK) return rc;
    /* The sealed worklist policy decides whether the matrix-core regime may run at all
     * (src/backend/cuda/moe.c:913-951, 1341-1361): a minimum of zero keeps it off, a minimum above
     * the batch's rows keeps it off for this batch, and a regime named by another family than
     * this backend's is refused. A job without a policy leaves the choice to the backend. */
    if (job->worklist_policy && job->worklist_policy->tensor_core_minimum) {
        if (strcmp(job->worklist_policy->tensor_core_kernel_family, YVEX_MOE_KERNEL_GFX950_MATRIX_CORE_EXPERT) != 0)
            return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.policy",
                                    "compiled matrix-core MoE worklist regime is unavailable");
        matrix_allowed = row_count >= job->worklist_policy->tensor_core_minimum;
    } else if (job->worklist_policy) {
        matrix_allowed = 0;
    }
    /* weights: router [experts x hidden], optional bias [1 x experts], expert-major matrices */
    rc = view_resolve(backend, &views[YVEX_MOE_WEIGHT_ROUTER], hidden, experts, &router_address, err);
    if (rc == YVEX_OK && !hash_router && layer->requires_correction_bias)
        rc = view_resolve(backend, &views[YVEX_MOE_WEIGHT_ROUTER_BIAS], experts, 1ull, &bias_address, err);
    if (rc == YVEX_OK && hash_router) {
        const yvex_moe_weight_view *table = &views[YVEX_MOE_WEIGHT_ROUTER_TABLE];
        rc = view_resolve(backend, table, table->row_width, table->row_count, &table_address, err);
        if (rc == YVEX_OK && table->row_count != 1ull && table->row_count < layer->hash_table_rows)
            rc = yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.weights",
                                  "MoE hash table holds fewer rows than the plan names");
    }
    if (rc == YVEX_OK)
        rc = expert_view_resolve(backend, &views[YVEX_MOE_WEIGHT_ROUTED_GATE], routed_image & 1, hidden,
                                 experts * layer->expert_intermediate_width, &addresses[0], err);
    if (rc == YVEX_OK)
        rc = expert_view_resolve(backend, &views[YVEX_MOE_WEIGHT_ROUTED_UP], routed_image & 1, hidden,
                                 experts * layer->expert_intermediate_width, &addresses[1], err);
    if (rc == YVEX_OK)
        rc = expert_view_resolve(backend, &views[YVEX_MOE_WEIGHT_ROUTED_DOWN], (routed_image >> 1) & 1,
                                 layer->expert_intermediate_width, experts * hidden, &addresses[2], err);
    if (rc == YVEX_OK && has_shared)
        rc = expert_view_resolve(backend, &views[YVEX_MOE_WEIGHT_SHARED_GATE], shared_image & 1, hidden,
                                 layer->shared_intermediate_width, &addresses[3], err);
    if (rc == YVEX_OK && has_shared)
        rc = expert_view_resolve(backend, &views[YVEX_MOE_WEIGHT_SHARED_UP], shared_image & 1, hidden,
                                 layer->shared_intermediate_width, &addresses[4], err);
    if (rc == YVEX_OK && has_shared)
        rc = expert_view_resolve(backend, &views[YVEX_MOE_WEIGHT_SHARED_DOWN], (shared_image >> 1) & 1,
                                 layer->shared_intermediate_width, hidden, &addresses[5], err);
    if (rc == YVEX_OK && envelope) {
        /* ingress coefficients: the mixing function is a matrix over the expanded row, the rest
         * are flat rows of F32, BF16 or I32 values (src/graph/moe.c:405-428) */
        static const int flat_slots[3] = {YVEX_MOE_WEIGHT_MHC_SCALE, YVEX_MOE_WEIGHT_MHC_BASE,
                                          YVEX_MOE_WEIGHT_FFN_NORM};
        const unsigned long long flat_widths[3] = {3ull, layer->mhc_mixing_rows, hidden};
        int k;
        rc = view_resolve(backend, &views[YVEX_MOE_WEIGHT_MHC_FUNCTION], expanded,
                          layer->mhc_mixing_rows, &envelope_addresses[0], err);
        for (k = 0; rc == YVEX_OK && k < 3; ++k) {
            unsigned int q = views[flat_slots[k]].qtype;
            if (q != 0u && q != 30u && q != 26u)
                rc = yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.rows",
                                      "MoE FFN coefficients cannot be decoded");
            else
                rc = view_resolve(backend, &views[flat_slots[k]], flat_widths[k], 1ull,
                                  &envelope_addresses[1 + k], err);
        }
    }
    if (rc != YVEX_OK) return rc;
    if (!(layer->activation_limit > 0.0) || !isfinite(layer->activation_limit) ||
        !isfinite(layer->routed_scaling_factor))
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.rows",
                                "activation limit and routed scaling must be finite");
    rc = yvex_rocm_require_kernels(backend, "rocm.moe.rows", err);
    if (rc != YVEX_OK) return rc;

    rows->device_outputs->is_written = 0;
    started = monotonic_ns();
    yvex_rocm_workspace_reset(backend);
    if (!yvex_rocm_backend_workspace_acquire(backend, ranges.total - ALIGN, ALIGN, &base))
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, "rocm.moe.rows", "workspace acquisition failed");
    fill_expert_weights(&routed, &views[YVEX_MOE_WEIGHT_ROUTED_GATE], &views[YVEX_MOE_WEIGHT_ROUTED_UP],
                        &views[YVEX_MOE_WEIGHT_ROUTED_DOWN], addresses[0], addresses[1], addresses[2],
                        hidden, layer->expert_intermediate_width, routed_image);
    if (has_shared)
        fill_expert_weights(&shared, &views[YVEX_MOE_WEIGHT_SHARED_GATE], &views[YVEX_MOE_WEIGHT_SHARED_UP],
                            &views[YVEX_MOE_WEIGHT_SHARED_DOWN], addresses[3], addresses[4], addresses[5],
                            hidden, layer->shared_intermediate_width, shared_image);
    /* Row batches whose buckets average six pairs or more (four with Q4_K gate and up rows) go to
     * the int8 matrix-core kernels (IQ2_XXS or Q4_K weights, Q8_K activations); below that the decode
     * sweeps, which read an expert's bytes once per four pairs, are faster: with 256 experts and
     * top-8 the two families cross at about 170 rows (IQ2_XXS) and 128 rows (Q4_K). The
     * reference switches its tensor-core kernels on from 16 input rows
     * (src/backend/cuda/private.h:461-464). Both kernel families read the sweep image of
     * IQ2_XXS experts as well as canonical bytes, and both publish the same bits (a row's terms
     * are added in double in block order in either), so the choice is one of speed only; a
     * sealed worklist policy can keep the matrix-core regime off (matrix_allowed). */
    row_batch = matrix_allowed && routed_q8 && matrix_core_qtypes(&routed) &&
                pairs >= (routed.gate_qtype == 12u ? 4ull : 6ull) * experts;
    shared_row_batch = row_batch && has_shared && shared_q8 && matrix_core_qtypes(&shared);
    merged = !row_batch && has_shared && shared_q8 == routed_q8 && same_expert_shape(&routed, &shared);
    /* A Q8_0 shared expert (the format the reference's model file keeps it in, its default for every
     * tensor outside the routed experts: src/graph/families/deepseek_v4.c:1550-1557) is three dense
     * projections of every row, and the dense Q8_0 kernels give the CPU path's bits at any number of
     * rows: gate and up sums, the SwiGLU stage, quantization, down. The up sums
     * borrow the pair-output range, which nothing uses between the router and the routed down
     * projection. */
    shared_dense = has_shared && shared_q8 && !merged && !shared_row_batch && !shared_image &&
                   shared.gate_qtype == 8u && shared.up_qtype == 8u && shared.down_qtype == 8u &&
                   layer->shared_intermediate_width <= topk * hidden;
    if (yvex_rocm_seam("YVEX_TEST_ROCM_LAUNCH_FAILURE"))
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.moe.rows.launch",
                                "kernel launch failed (test seam)");
    status = backend->device_status;
    stream = backend->stream;
#define AT(field) ((void *)(uintptr_t)(base + ranges.field))
    /* token ids come from the caller's host buffer on every call, so they travel ahead of the
     * kernels and never inside a graph; they pass through pinned memory of the backend, so a
     * deferred batch queues the copy and returns without waiting for the stream */
    if (hash_router && yvex_rocm_upload_queued(backend, AT(tokens), rows->token_ids,
                                               row_count * sizeof(unsigned int)) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.moe.rows.token-ids", yvex_hip_last_error());
    /* The kernels' status word is cleared where a phase starts, not per batch: a batch whose
     * completion is deferred leaves what it raised for the barrier to find, whatever runs behind
     * it (the word only ever changes from zero). Like the token ids, outside any graph. */
    if (!backend->pending_completion) {
        rc = yvex_rocm_status_reset(backend, "rocm.moe.rows.status", err);
        if (rc != YVEX_OK) return rc;
        status_launches = 1ull;
    }
    if (!job->eager_execution && !(backend->moe_graphs && backend->moe_graphs->refused)) {
        graph_key key;
        unsigned long long slot_address[YVEX_MOE_WEIGHT_COUNT] = {0};
        int k;
        slot_address[YVEX_MOE_WEIGHT_FFN_NORM] = envelope_addresses[3];
        slot_address[YVEX_MOE_WEIGHT_MHC_FUNCTION] = envelope_addresses[0];
        slot_address[YVEX_MOE_WEIGHT_MHC_BASE] = envelope_addresses[2];
        slot_address[YVEX_MOE_WEIGHT_MHC_SCALE] = envelope_addresses[1];
        slot_address[YVEX_MOE_WEIGHT_ROUTER] = router_address;
        slot_address[YVEX_MOE_WEIGHT_ROUTER_TABLE] = table_address;
        slot_address[YVEX_MOE_WEIGHT_ROUTER_BIAS] = bias_address;
        for (k = 0; k < 6; ++k) slot_address[YVEX_MOE_WEIGHT_ROUTED_GATE + k] = addresses[k];
        key.count = 0u;
        key.overflow = 0;
        key_word(&key, row_count);
        key_word(&key, (unsigned long long)row_batch);
        key_word(&key, (unsigned long long)(uintptr_t)status);
        key_word(&key, (unsigned long long)(uintptr_t)stream);
        key_word(&key, base);
        key_word(&key, backend->workspace_bytes);
        key_word(&key, backend->resident_generation);
        key_word(&key, (unsigned long long)(uintptr_t)rows->device_rows->data);
        key_word(&key, (unsigned long long)(uintptr_t)rows->device_outputs->data);
        key_layer(&key, layer);
        for (k = 0; k < YVEX_MOE_WEIGHT_COUNT; ++k) key_view(&key, &views[k], slot_address[k]);
        if (!backend->moe_graphs) backend->moe_graphs = calloc(1u, sizeof(*backend->moe_graphs));
        if (backend->moe_graphs && !key.overflow) {
            graph_slot *slot = graph_find(backend->moe_graphs, &key);
            if (!slot) slot = graph_admit(backend->moe_graphs, &key);   /* first sight: eager */
            else if (!slot->eager_only) graph_mode = slot->graph ? GRAPH_REPLAY : GRAPH_CAPTURE;
            slot->last_use = ++backend->moe_graphs->clock;
            graph_target = slot;
        }
    }
sequence:
    rc = YVEX_OK;
    launches = 0ull;
    if (graph_mode == GRAPH_CAPTURE && yvex_hip_capture_begin(stream) != 0) {
        backend->moe_graphs->refused = 1;
        graph_mode = GRAPH_EAGER;
    }
#define LAUNCH(call, where)                                             \
    do {                                                                \
        if (rc == YVEX_OK && graph_mode != GRAPH_REPLAY) {              \
            rc = yvex_rocm_launch_result((call), (where), err);         \
            if (rc == YVEX_OK) launches++;                              \
        }                                                               \
    } while (0)
    if (has_shared && !merged)
        LAUNCH(yvex_hip_fill_u32(AT(shared_outputs), 0u, row_count * hidden, stream), "rocm.moe.rows.zero");
    activations = rows->device_rows->data;
    combined_target = rows->device_outputs->data;
    if (envelope) {
        /* src/backend/cuda/moe.c:1210-1254: mixes = function . expanded row, coefficients decoded
         * to F32, then ingress and the weighted norm in one kernel */
        const yvex_moe_weight_view *function = &views[YVEX_MOE_WEIGHT_MHC_FUNCTION];
        static const int flat_slots[3] = {YVEX_MOE_WEIGHT_MHC_SCALE, YVEX_MOE_WEIGHT_MHC_BASE,
                                          YVEX_MOE_WEIGHT_FFN_NORM};
        void *flat_targets[3];
        int k, fused_coefficients;
        flat_targets[0] = AT(scale);
        flat_targets[1] = AT(base);
        flat_targets[2] = AT(norm);
        /* F32 mixing rows over a decode-width batch: two dozen weight rows are four tiles, so the
         * row width is split over the whole device like the router's, the partial sums in the
         * pair-output range (116 us unsplit for 24 x 28672 against 32 rows, 11 us split) */
        if (function->qtype == YVEX_GGUF_QTYPE_F32) {
            unsigned long long need = yvex_hip_matvec_f32_scratch_bytes(layer->mhc_mixing_rows, expanded, row_count);
            int lend = need && need <= pairs * hidden * sizeof(float);
            unsigned int mixing_launches = yvex_hip_matvec_f32_rows_launches(
                (const float *)(uintptr_t)envelope_addresses[0], layer->mhc_mixing_rows, expanded,
                (const float *)rows->device_rows->data, row_count, expanded, lend ? AT(pair_outputs) : NULL,
                lend ? need : 0ull);
            LAUNCH(yvex_hip_matvec_f32_rows((const float *)(uintptr_t)envelope_addresses[0],
                                            layer->mhc_mixing_rows, expanded,
                                            (const float *)rows->device_rows->data, row_count, expanded, NULL,
                                            (float *)AT(mixes), layer->mhc_mixing_rows, 0,
                                            lend ? AT(pair_outputs) : NULL, lend ? need : 0ull, (int *)status,
                                            stream), "rocm.moe.rows.mhc-function");
            if (rc == YVEX_OK && mixing_launches == 2u && graph_mode != GRAPH_REPLAY) launches++;
        } else
        LAUNCH(yvex_hip_matvec((const uint8_t *)(uintptr_t)envelope_addresses[0], function->qtype,
                               layer->mhc_mixing_rows, expanded, function->row_bytes,
                               rows->device_rows->data, 0, row_count, expanded, NULL,
                               (float *)AT(mixes), layer->mhc_mixing_rows, 0, (int *)status, stream),
               "rocm.moe.rows.mhc-function");
        /* coefficient vectors stored as F32 or BF16 values are decoded by the ingress itself;
         * I32 ones go through the decode launches first */
        fused_coefficients = 1;
        for (k = 0; k < 3; ++k) {
            unsigned int q = views[flat_slots[k]].qtype;
            if (q == YVEX_GGUF_QTYPE_F32) fused_coefficients &= !(envelope_addresses[1 + k] & 3ull);
            else if (q == YVEX_GGUF_QTYPE_BF16) fused_coefficients &= !(envelope_addresses[1 + k] & 1ull);
            else fused_coefficients = 0;
        }
        if (fused_coefficients)
            LAUNCH(yvex_hip_mhc_ingress_encoded((const float *)rows->device_rows->data, (const float *)AT(mixes),
                                                (const void *)(uintptr_t)envelope_addresses[1],
                                                views[flat_slots[0]].qtype,
                                                (const void *)(uintptr_t)envelope_addresses[2],
                                                views[flat_slots[1]].qtype,
                                                (const void *)(uintptr_t)envelope_addresses[3],
                                                views[flat_slots[2]].qtype, row_count, streams, hidden,
                                                layer->mhc_sinkhorn_iterations, layer->rms_epsilon,
                                                layer->mhc_epsilon, layer->mhc_post_multiplier,
                                                (float *)AT(normalized), (float *)AT(post),
                                                (float *)AT(combination), (int *)status, stream),
                   "rocm.moe.rows.mhc-ingress");
        else {
        for (k = 0; k < 3; ++k)
            LAUNCH(yvex_hip_gather((const uint8_t *)(uintptr_t)envelope_addresses[1 + k],
                                   views[flat_slots[k]].qtype, 1ull, views[flat_slots[k]].row_width,
                                   views[flat_slots[k]].row_bytes, NULL, 1ull, (float *)flat_targets[k],
                                   (int *)status, stream), "rocm.moe.rows.mhc-coefficients");
        LAUNCH(yvex_hip_mhc_ingress((const float *)rows->device_rows->data, (const float *)AT(mixes),
                                    (const float *)AT(scale), (const float *)AT(base),
                                    (const float *)AT(norm), row_count, streams, hidden,
                                    layer->mhc_sinkhorn_iterations, layer->rms_epsilon,
                                    layer->mhc_epsilon, layer->mhc_post_multiplier,
                                    (float *)AT(normalized), (float *)AT(post),
                                    (float *)AT(combination), (int *)status, stream),
               "rocm.moe.rows.mhc-ingress");
        }
        activations = AT(normalized);
        combined_target = AT(combined);
    }
    /* router: logits = router . row (F32 activations, as src/backend/cuda/moe.c:1259-1284). F32
     * router weights over a decode-width batch are split over the whole device; their partial
     * sums use the pair-output range, which nothing else touches before the down projection. */
    if (views[YVEX_MOE_WEIGHT_ROUTER].qtype == YVEX_GGUF_QTYPE_F32) {
        unsigned long long need = yvex_hip_matvec_f32_scratch_bytes(experts, hidden, row_count);
        int lend = need && need <= pairs * hidden * sizeof(float);
        /* (the wrapper says how many launches it makes for these operands: the count below and
         * the node count of a captured graph must agree) */
        unsigned int router_launches = yvex_hip_matvec_f32_rows_launches(
            (const float *)(uintptr_t)router_address, experts, hidden, (const float *)activations, row_count,
            hidden, lend ? AT(pair_outputs) : NULL, lend ? need : 0ull);
        /* the split projection's second launch publishes the learned router's scores as well
         * (into the combine's output range, which nothing reads or writes before the combine):
         * the preparation launch, whose one routing workgroup everything behind it waits for,
         * then starts from them */
        scored = router_launches == 2u && !hash_router && hidden >= experts &&
                 yvex_hip_moe_prepare_supported(row_count, experts, topk);
        if (scored)
            LAUNCH(yvex_hip_matvec_f32_rows_scored((const float *)(uintptr_t)router_address, experts, hidden,
                                                   (const float *)activations, row_count, hidden,
                                                   (float *)AT(logits), experts, (float *)AT(routed),
                                                   (int)layer->scoring, AT(pair_outputs), need,
                                                   (int *)status, stream), "rocm.moe.rows.router");
        else
        LAUNCH(yvex_hip_matvec_f32_rows((const float *)(uintptr_t)router_address, experts, hidden,
                                        (const float *)activations, row_count, hidden, NULL,
                                        (float *)AT(logits), experts, 0, lend ? AT(pair_outputs) : NULL,
                                        lend ? need : 0ull, (int *)status, stream), "rocm.moe.rows.router");
        if (rc == YVEX_OK && router_launches == 2u && graph_mode != GRAPH_REPLAY) launches++;   /* partials, then their sum */
    } else
    LAUNCH(yvex_hip_matvec((const uint8_t *)(uintptr_t)router_address, views[YVEX_MOE_WEIGHT_ROUTER].qtype,
                           experts, hidden, views[YVEX_MOE_WEIGHT_ROUTER].row_bytes,
                           activations, 0, row_count, hidden, NULL, (float *)AT(logits),
                           experts, 0, (int *)status, stream), "rocm.moe.rows.router");
    if (hash_router) {
        LAUNCH(yvex_hip_moe_route_hash_rows((const float *)AT(logits), (const uint8_t *)(uintptr_t)table_address,
                                            (const uint32_t *)AT(tokens), row_count, experts, topk,
                                            layer->hash_table_rows,
                                            views[YVEX_MOE_WEIGHT_ROUTER_TABLE].row_bytes,
                                            views[YVEX_MOE_WEIGHT_ROUTER_TABLE].row_count == 1ull,
                                            (int)layer->scoring, layer->normalize_topk_probabilities,
                                            layer->routed_scaling_factor, (uint64_t *)AT(selected),
                                            (float *)AT(weights), (int *)status, stream),
               "rocm.moe.rows.route");
    }
    /* a correction bias stored as F32 values is read where it lies; any other encoding is
     * decoded into the workspace first */
    bias_rows = NULL;
    if (!hash_router && layer->requires_correction_bias)
        bias_rows = views[YVEX_MOE_WEIGHT_ROUTER_BIAS].qtype == YVEX_GGUF_QTYPE_F32 && !(bias_address & 3ull)
                        ? (const float *)(uintptr_t)bias_address : (const float *)AT(bias);
    if (bias_rows && bias_rows == (const float *)AT(bias))
        LAUNCH(yvex_hip_gather((const uint8_t *)(uintptr_t)bias_address, views[YVEX_MOE_WEIGHT_ROUTER_BIAS].qtype,
                               1ull, experts, views[YVEX_MOE_WEIGHT_ROUTER_BIAS].row_bytes, NULL, 1ull,
                               (float *)AT(bias), (int *)status, stream), "rocm.moe.rows.bias");
    /* a decode-width batch with the learned router: routing, worklist and input quantization
     * share one launch */
    const int need_q8 = routed_q8 || (has_shared && shared_q8);
    if (scored) {
        LAUNCH(yvex_hip_moe_prepare_scored((const float *)AT(routed),
                                           bias_rows,
                                           row_count, experts, topk, layer->normalize_topk_probabilities,
                                           layer->routed_scaling_factor, (uint64_t *)AT(selected),
                                           (float *)AT(weights), (uint64_t *)AT(order),
                                           (uint64_t *)AT(expert_ids), (uint64_t *)AT(bucket_offsets),
                                           (uint64_t *)AT(bucket_populations),
                                           (uint64_t *)AT(sweep_offsets), (uint64_t *)AT(counts),
                                           need_q8 ? (const float *)activations : NULL, hidden, hidden,
                                           need_q8 ? (uint8_t *)AT(input_q8) : NULL, (int *)status, stream),
               "rocm.moe.rows.prepare");
    } else if (!hash_router && yvex_hip_moe_prepare_supported(row_count, experts, topk)) {
        LAUNCH(yvex_hip_moe_prepare((const float *)AT(logits),
                                    bias_rows,
                                    row_count, experts, topk, (int)layer->scoring,
                                    layer->normalize_topk_probabilities, layer->routed_scaling_factor,
                                    (uint64_t *)AT(selected), (float *)AT(weights), (uint64_t *)AT(order),
                                    (uint64_t *)AT(expert_ids), (uint64_t *)AT(bucket_offsets),
                                    (uint64_t *)AT(bucket_populations), (uint64_t *)AT(sweep_offsets),
                                    (uint64_t *)AT(counts), need_q8 ? (const float *)activations : NULL,
                                    hidden, hidden, need_q8 ? (uint8_t *)AT(input_q8) : NULL,
                                    (int *)status, stream), "rocm.moe.rows.prepare");
    } else {
        if (!hash_router)
            LAUNCH(yvex_hip_moe_route_rows((const float *)AT(logits),
                                           bias_rows,
                                           row_count, experts, topk, (int)layer->scoring,
                                           layer->normalize_topk_probabilities,
                                           layer->routed_scaling_factor, (uint64_t *)AT(selected),
                                           (float *)AT(weights), (int *)status, stream),
                   "rocm.moe.rows.route");
        LAUNCH(yvex_hip_worklist_build((const uint64_t *)AT(selected), pairs, topk, experts,
                                       (uint64_t *)AT(order), (uint64_t *)AT(expert_ids),
                                       (uint64_t *)AT(bucket_offsets), (uint64_t *)AT(bucket_populations),
                                       (uint64_t *)AT(sweep_offsets), (uint64_t *)AT(counts), (int *)status,
                                       stream), "rocm.moe.rows.worklist");
        if (need_q8)
            LAUNCH(yvex_hip_q8k_quantize((const float *)activations, row_count, hidden, hidden,
                                         (uint8_t *)AT(input_q8), (int *)status, stream), "rocm.moe.rows.q8");
    }
    if (row_batch)
        LAUNCH(yvex_hip_moe_up_rows(&routed, AT(input_q8), (const float *)AT(weights),
                                    (const uint64_t *)AT(order), (const uint64_t *)AT(expert_ids),
                                    (const uint64_t *)AT(bucket_offsets),
                                    (const uint64_t *)AT(bucket_populations), (const uint64_t *)AT(counts),
                                    pairs, topk, experts, layer->activation_limit,
                                    (float *)AT(intermediate), (int *)status, stream),
               "rocm.moe.rows.up-matrix");
    else
    LAUNCH(yvex_hip_moe_up(&routed, routed_q8 ? AT(input_q8) : (void *)(uintptr_t)activations, routed_q8,
                           (const float *)AT(weights), (const uint64_t *)AT(order),
                           (const uint64_t *)AT(expert_ids), (const uint64_t *)AT(bucket_offsets),
                           (const uint64_t *)AT(bucket_populations), (const uint64_t *)AT(sweep_offsets),
                           (const uint64_t *)AT(counts), pairs, topk, experts, layer->activation_limit,
                           (float *)AT(intermediate), merged ? &shared : NULL, merged ? row_count : 0ull,
                           merged ? (float *)AT(shared_intermediate) : NULL, (int *)status, stream),
           "rocm.moe.rows.up");
    if (shared_row_batch)
        LAUNCH(yvex_hip_moe_up_rows(&shared, AT(input_q8), NULL, NULL, NULL, NULL, NULL, NULL, row_count,
                                    1ull, 1ull, layer->activation_limit, (float *)AT(shared_intermediate),
                                    (int *)status, stream), "rocm.moe.rows.shared-up-matrix");
    else if (shared_dense) {
        LAUNCH(yvex_hip_matvec(shared.gate, shared.gate_qtype, layer->shared_intermediate_width, hidden,
                               shared.gate_row_bytes, AT(input_q8), 1, row_count, hidden, NULL,
                               (float *)AT(shared_intermediate), layer->shared_intermediate_width, 0,
                               (int *)status, stream), "rocm.moe.rows.shared-gate-dense");
        LAUNCH(yvex_hip_matvec(shared.up, shared.up_qtype, layer->shared_intermediate_width, hidden,
                               shared.up_row_bytes, AT(input_q8), 1, row_count, hidden, NULL,
                               (float *)AT(pair_outputs), layer->shared_intermediate_width, 0,
                               (int *)status, stream), "rocm.moe.rows.shared-up-dense");
        LAUNCH(yvex_hip_moe_swiglu_rows((const float *)AT(shared_intermediate), (const float *)AT(pair_outputs),
                                        row_count * layer->shared_intermediate_width, layer->activation_limit,
                                        (float *)AT(shared_intermediate), (int *)status, stream),
               "rocm.moe.rows.shared-swiglu");
    } else if (has_shared && !merged)
        LAUNCH(yvex_hip_moe_up(&shared, shared_q8 ? AT(input_q8) : (void *)(uintptr_t)activations,
                               shared_q8, NULL, NULL, NULL, NULL, NULL, NULL, NULL, row_count, 1ull, 1ull,
                               layer->activation_limit, (float *)AT(shared_intermediate), NULL, 0ull, NULL,
                               (int *)status, stream), "rocm.moe.rows.shared-up");
    if (routed_q8 && has_shared && shared_q8 && ranges.joined_intermediates)
        LAUNCH(yvex_hip_q8k_quantize((const float *)AT(intermediate), pairs + row_count,
                                     layer->expert_intermediate_width, layer->expert_intermediate_width,
                                     (uint8_t *)AT(intermediate_q8), (int *)status, stream),
               "rocm.moe.rows.q8-mid");
    else if (routed_q8)
        LAUNCH(yvex_hip_q8k_quantize((const float *)AT(intermediate), pairs, layer->expert_intermediate_width,
                                     layer->expert_intermediate_width, (uint8_t *)AT(intermediate_q8),
                                     (int *)status, stream), "rocm.moe.rows.q8-mid");
    if (has_shared && shared_q8 && !(routed_q8 && ranges.joined_intermediates))
        LAUNCH(yvex_hip_q8k_quantize((const float *)AT(shared_intermediate), row_count,
                                     layer->shared_intermediate_width, layer->shared_intermediate_width,
                                     (uint8_t *)AT(shared_intermediate_q8), (int *)status, stream),
               "rocm.moe.rows.q8-shared-mid");
    if (row_batch)
        LAUNCH(yvex_hip_moe_down_rows(&routed, AT(intermediate_q8), (const uint64_t *)AT(order),
                                      (const uint64_t *)AT(expert_ids), (const uint64_t *)AT(bucket_offsets),
                                      (const uint64_t *)AT(bucket_populations), (const uint64_t *)AT(counts),
                                      pairs, experts, (float *)AT(pair_outputs), (int *)status, stream),
               "rocm.moe.rows.down-matrix");
    else
    LAUNCH(yvex_hip_moe_down(&routed, routed_q8 ? AT(intermediate_q8) : AT(intermediate), routed_q8,
                             (const uint64_t *)AT(order), (const uint64_t *)AT(expert_ids),
                             (const uint64_t *)AT(bucket_offsets), (const uint64_t *)AT(bucket_populations),
                             (const uint64_t *)AT(sweep_offsets), (const uint64_t *)AT(counts), pairs,
                             experts, (float *)AT(pair_outputs), merged ? &shared : NULL,
                             merged ? row_count : 0ull,
                             merged ? (shared_q8 ? AT(shared_intermediate_q8) : AT(shared_intermediate)) : NULL,
                             merged ? (float *)AT(shared_outputs) : NULL, (int *)status, stream),
           "rocm.moe.rows.down");
    if (shared_row_batch)
        LAUNCH(yvex_hip_moe_down_rows(&shared, AT(shared_intermediate_q8), NULL, NULL, NULL, NULL, NULL,
                                      row_count, 1ull, (float *)AT(shared_outputs), (int *)status, stream),
               "rocm.moe.rows.shared-down-matrix");
    else if (shared_dense)
        LAUNCH(yvex_hip_matvec(shared.down, shared.down_qtype, hidden, layer->shared_intermediate_width,
                               shared.down_row_bytes, AT(shared_intermediate_q8), 1, row_count,
                               layer->shared_intermediate_width, NULL, (float *)AT(shared_outputs), hidden, 1,
                               (int *)status, stream), "rocm.moe.rows.shared-down-dense");
    else if (has_shared && !merged)
        LAUNCH(yvex_hip_moe_down(&shared, shared_q8 ? AT(shared_intermediate_q8) : AT(shared_intermediate),
                                 shared_q8, NULL, NULL, NULL, NULL, NULL, NULL, row_count, 1ull,
                                 (float *)AT(shared_outputs), NULL, 0ull, NULL, NULL, (int *)status, stream),
               "rocm.moe.rows.shared-down");
    if (!has_shared)
        LAUNCH(yvex_hip_fill_u32(AT(shared_outputs), 0u, row_count * hidden, stream), "rocm.moe.rows.zero");
    LAUNCH(yvex_hip_moe_reduce_combine((const float *)AT(pair_outputs), row_count, topk, hidden,
                                       (const float *)AT(shared_outputs), (float *)AT(routed),
                                       (float *)combined_target, (int *)status, stream),
           "rocm.moe.rows.combine");
    if (envelope)
        LAUNCH(yvex_hip_mhc_egress((const float *)AT(combined), (const float *)rows->device_rows->data,
                                   (const float *)AT(post), (const float *)AT(combination), row_count,
                                   streams, hidden, (float *)rows->device_outputs->data, (int *)status,
                                   stream), "rocm.moe.rows.mhc-egress");
    if (graph_mode == GRAPH_CAPTURE) {
        /* a recording that fails, or holds anything but kernels, is dropped for good and the
         * batch runs eagerly: the stream has executed nothing yet */
        uint64_t nodes = 0u;
        if (rc != YVEX_OK) {
            /* a launch wrapper refused this job's geometry: the job fails eagerly too, and only
             * its own slot stops recording; other topologies keep their graphs */
            (void)yvex_hip_capture_abort(stream);
            graph_target->eager_only = 1;
            graph_mode = GRAPH_EAGER;
            goto sequence;
        }
        if (yvex_hip_capture_end(stream, &graph_target->graph, &nodes) != 0 || nodes != launches) {
            if (graph_target->graph) (void)yvex_hip_graph_destroy(graph_target->graph);
            graph_target->graph = NULL;
            backend->moe_graphs->refused = 1;
            graph_mode = GRAPH_EAGER;
            goto sequence;
        }
        graph_target->launches = launches;
    }
    if (graph_mode != GRAPH_EAGER) {
        launches = graph_target->launches;
        rc = yvex_rocm_launch_result(yvex_hip_graph_launch(graph_target->graph, stream),
                                     "rocm.moe.rows.graph", err);
    }
    if (rc != YVEX_OK) {
        /* a job that fails on first sight is not remembered: its next call is a first sight again */
        if (graph_target && !graph_target->graph) graph_target->used = 0;
        return rc;
    }

    defer = job->device_completion && job->device_completion->defer;
    result->graph_launches = graph_mode != GRAPH_EAGER;
    result->graph_captures = graph_mode == GRAPH_CAPTURE;
    result->graph_replays = graph_mode == GRAPH_REPLAY;
    result->schema_version = YVEX_MOE_ROW_BATCH_RESULT_SCHEMA_V4;
    result->execution_class = YVEX_EXECUTION_CLASS_DEVICE_NATIVE;
    result->row_count = row_count;
    result->row_expert_pairs = pairs;
    result->kernel_launches = launches + status_launches;
    result->tensor_core_launches = (row_batch ? 2ull : 0ull) + (shared_row_batch ? 2ull : 0ull);
    result->shared_expert_operations = has_shared ? row_count : 0ull;
    result->grouped_expert_operations = pairs;
    result->active_weight_base_bytes = views[YVEX_MOE_WEIGHT_ROUTER].encoded_bytes +
        (has_shared ? views[YVEX_MOE_WEIGHT_SHARED_GATE].encoded_bytes +
                      views[YVEX_MOE_WEIGHT_SHARED_UP].encoded_bytes +
                      views[YVEX_MOE_WEIGHT_SHARED_DOWN].encoded_bytes : 0ull);
    result->active_weight_per_unique_expert_bytes =
        routed.gate_expert_bytes + routed.up_expert_bytes + routed.down_expert_bytes;
    if (envelope)
        result->active_weight_base_bytes += views[YVEX_MOE_WEIGHT_MHC_FUNCTION].encoded_bytes +
            views[YVEX_MOE_WEIGHT_MHC_SCALE].encoded_bytes + views[YVEX_MOE_WEIGHT_MHC_BASE].encoded_bytes +
            views[YVEX_MOE_WEIGHT_FFN_NORM].encoded_bytes;
    result->memory.activation_bytes = 2ull * row_count * expanded * sizeof(float);
    result->memory.temporary_bytes = ranges.total;
    result->memory.measured_operations = 1ull;
    if (defer) {
        backend->pending_completion = 1;
        result->device_completion_pending = 1;
        rows->device_outputs->is_written = 1;   /* ordered on the backend stream */
        result->total_ns = monotonic_ns() - started;
        yvex_rocm_error_clear(err);
        return YVEX_OK;
    }
    /* one synchronisation publishes status, worklist facts, routing and optional host copies */
    {
        unsigned long long sync_started = monotonic_ns();
        rc = yvex_rocm_finish(backend, "rocm.moe.rows.sync", &device_status, err);
        result->synchronization_ns = monotonic_ns() - sync_started;
    }
    d2h += sizeof(int);
    if (rc == YVEX_OK && device_status)
        rc = yvex_rocm_refuse(err, device_status == 1 ? YVEX_ERR_FORMAT : YVEX_ERR_BACKEND,
                              "rocm.moe.rows", device_status == 1
                                  ? "width-N MoE produced invalid numerics"
                                  : "width-N MoE kernels met a contract violation");
#define DOWNLOAD(dst, field, bytes)                                                          \
    do {                                                                                     \
        if (rc == YVEX_OK && (dst)) {                                                        \
            if (yvex_hip_memcpy_d2h((dst), AT(field), (bytes), stream) != 0)                 \
                rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.moe.rows.download",       \
                                      yvex_hip_last_error());                                \
            else { d2h += (bytes); result->download_count++; }                               \
        }                                                                                    \
    } while (0)
    {
        unsigned long long *counts_host = counts;
        DOWNLOAD(counts_host, counts, sizeof(counts));
    }
    DOWNLOAD(output->selected_experts, selected, pairs * sizeof(unsigned long long));
    DOWNLOAD(output->selected_weights, weights, pairs * sizeof(float));
    DOWNLOAD(output->routed_rows, routed, row_count * hidden * sizeof(float));
    DOWNLOAD(output->shared_rows, shared_outputs, row_count * hidden * sizeof(float));
    if (envelope) {
        DOWNLOAD(output->post_rows, post, row_count * streams * sizeof(float));
        DOWNLOAD(output->combination_rows, combination, row_count * streams * streams * sizeof(float));
    }
    if (rc == YVEX_OK && output->combined_rows) {
        if (yvex_hip_memcpy_d2h(output->combined_rows, combined_target,
                                row_count * hidden * sizeof(float), stream) != 0)
            rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.moe.rows.download", yvex_hip_last_error());
        else { d2h += row_count * hidden * sizeof(float); result->download_count++; }
    }
#undef DOWNLOAD
#undef LAUNCH
#undef AT
    if (rc != YVEX_OK) {
        memset(result, 0, sizeof(*result));
        return rc;
    }
    backend->memory.d2h_bytes += d2h - sizeof(int);
    result->completed = 1;
    result->unique_experts = counts[0];
    result->worklists.schema_version = 1u;
    result->worklists.worklist_count = 1ull;
    result->worklists.pair_count = counts[2];
    result->worklists.bucket_count = counts[0];
    result->worklists.maximum_bucket_population = counts[1];
    /* every pair of a batch runs in one regime (src/graph/worklist.c:407-425 counts per bucket) */
    result->worklists.tensor_core_eligible_pairs = row_batch ? counts[2] : 0ull;
    result->worklists.tensor_core_executed_pairs = row_batch ? counts[2] : 0ull;
    result->worklists.narrow_pairs = row_batch ? 0ull : counts[2];
    result->worklists.width_histogram[row_count < YVEX_EXPERT_WORKLIST_HISTOGRAM_CAP
                                          ? row_count : YVEX_EXPERT_WORKLIST_HISTOGRAM_CAP - 1u] = 1ull;
    result->worklists.provenance_counts[rows->provenance <= YVEX_EXECUTION_BATCH_COMPILED_COMPATIBLE
                                            ? rows->provenance : 0] = 1ull;
    result->expert_subviews_accessed = 3ull * counts[0] + (has_shared ? 3ull : 0ull);
    result->encoded_bytes_read = result->active_weight_base_bytes +
                                 result->active_weight_per_unique_expert_bytes * counts[0];
    result->memory.active_weight_bytes = result->encoded_bytes_read;
    result->memory.complete = 1;
    result->d2h_bytes = d2h;
    result->stream_synchronizations = 1ull;
    result->total_ns = monotonic_ns() - started;
    rows->device_outputs->is_written = 1;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

static int moe_complete_rows(yvex_rocm_backend *backend, int barrier_observed,
                             yvex_moe_row_batch_result *result, yvex_error *err)
{
    unsigned long long started = 0ull;
    int device_status = 0, rc = YVEX_OK;
    if (result) memset(result, 0, sizeof(*result));
    if (!backend || !result || (barrier_observed != 0 && barrier_observed != 1) ||
        backend->kind != YVEX_BACKEND_KIND_ROCM)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.complete",
                                "MoE completion owner is invalid");
    if (!backend->host_only) {
        started = monotonic_ns();
        rc = yvex_rocm_finish(backend, "rocm.moe.rows.phase-sync", &device_status, err);
        if (rc == YVEX_OK) backend->pending_completion = 0;   /* the barrier was reached: the next phase starts clean */
        if (rc == YVEX_OK && device_status)
            rc = yvex_rocm_refuse(err, device_status == 1 ? YVEX_ERR_FORMAT : YVEX_ERR_BACKEND,
                                  "rocm.moe.complete", "deferred width-N MoE reported a device failure");
    }
    if (rc != YVEX_OK) return rc;
    backend->pending_completion = 0;
    result->schema_version = YVEX_MOE_ROW_BATCH_RESULT_SCHEMA_V4;
    result->completed = 1;
    result->execution_class = YVEX_EXECUTION_CLASS_DEVICE_NATIVE;
    result->stream_synchronizations = barrier_observed ? 0ull : 1ull;
    result->synchronization_ns = started ? monotonic_ns() - started : 0ull;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

static const yvex_rocm_moe_operations moe_operations = {
    yvex_rocm_moe_derived_layout_plan, yvex_rocm_moe_derived_layout_build, yvex_rocm_moe_workspace_required,
    moe_execute_rows,
    moe_complete_rows};

const yvex_rocm_moe_operations *yvex_rocm_backend_moe_operations_get(const yvex_rocm_backend *backend)
{
    if (!backend || backend->kind != YVEX_BACKEND_KIND_ROCM || !backend->kernels_available ||
        backend->status == YVEX_BACKEND_STATUS_FAILED)
        return NULL;
    return &moe_operations;
}

/* ---- host worklist: src/graph/worklist.c:369-441 ---------------------------------------------- */

int yvex_rocm_expert_worklist_build(const unsigned long long *selected_experts,
                               const float *route_weights, unsigned long long pair_count,
                               unsigned long long experts_per_row, unsigned long long expert_count,
                               const yvex_expert_worklist_storage *storage,
                               yvex_expert_worklist_observation *observation, yvex_error *err)
{
    unsigned long long expert, pair, cursor = 0ull, bucket = 0ull, maximum = 0ull;
    if (observation) memset(observation, 0, sizeof(*observation));
    if (!selected_experts || !route_weights || !storage || !observation || !experts_per_row ||
        !expert_count || expert_count > 256ull || experts_per_row > expert_count || !pair_count ||
        pair_count % experts_per_row || !storage->expert_ids || !storage->bucket_offsets ||
        !storage->bucket_populations || !storage->source_pairs || !storage->source_rows ||
        !storage->destination_rows || !storage->route_weights ||
        storage->bucket_capacity < expert_count || storage->pair_capacity < pair_count)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "worklist.build",
                                "expert worklist request or storage is invalid");
    for (pair = 0ull; pair < pair_count; ++pair)
        if (selected_experts[pair] >= expert_count || !isfinite(route_weights[pair]))
            return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "worklist.build",
                                    "routed pair has an invalid expert or weight");
    for (expert = 0ull; expert < expert_count; ++expert) {
        unsigned long long start = cursor, population;
        for (pair = 0ull; pair < pair_count; ++pair) {
            if (selected_experts[pair] != expert) continue;
            storage->source_pairs[cursor] = pair;
            storage->source_rows[cursor] = pair / experts_per_row;
            storage->destination_rows[cursor] = pair;
            storage->route_weights[cursor] = route_weights[pair];
            cursor++;
        }
        population = cursor - start;
        if (!population) continue;
        storage->expert_ids[bucket] = expert;
        storage->bucket_offsets[bucket] = start;
        storage->bucket_populations[bucket] = population;
        if (population > maximum) maximum = population;
        observation->population_histogram[population < YVEX_EXPERT_WORKLIST_HISTOGRAM_CAP
                                              ? population : YVEX_EXPERT_WORKLIST_HISTOGRAM_CAP - 1u]++;
        bucket++;
    }
    storage->bucket_offsets[bucket] = cursor;
    if (cursor != pair_count)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, "worklist.build",
                                "expert worklist did not emit every routed pair");
    observation->schema_version = 1u;
    observation->worklist_count = 1ull;
    observation->pair_count = pair_count;
    observation->bucket_count = bucket;
    observation->maximum_bucket_population = maximum;
    observation->narrow_pairs = pair_count;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}
