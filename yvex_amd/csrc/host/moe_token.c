/*
 * Token-local MoE operation of the ROCm backend: one row, experts handed over one at a time.
 * Same contract as the reference's yvex_backend_moe_begin / add_expert / finish / close
 * (include/yvex/internal/moe.h:308-319, src/backend/cuda/moe.c:516-842): begin runs the
 * residual-stream ingress and the router and publishes the routing, every add_expert runs one
 * expert FFN on F32 activations, finish sums the routed experts in the order they were added,
 * combines with the shared expert, rounds to bf16 and, when the job names a device output, runs
 * the egress onto the residual streams.
 *
 * All ranges of an execution form one block of device memory: taken from the attached workspace
 * when it has room (as the reference does, moe.c:565-566), else allocated for the execution.
 * Weight views that lie outside the attached resident arena are uploaded into staging ranges of
 * that block (moe.c:205-245), one per projection so that gate, up and down of an expert are on
 * the device together. Nothing here computes on tensor data.
 */
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "private.h"

#define ALIGN 256ull

struct yvex_rocm_moe_execution {
    yvex_rocm_backend *backend;
    const yvex_moe_layer_job *job;
    void *block;
    int owns_block;                       /* allocated here rather than taken from the workspace */
    unsigned long long expanded, mixes, scale, base, norm, normalized, post, combination;
    unsigned long long logits, scores, bias, selected, weights, slot_weights, token;
    unsigned long long order, expert_ids, bucket_offsets, bucket_populations, sweep_offsets, counts;
    unsigned long long intermediate, pair_outputs, shared_output, routed, combined, staging;
    unsigned long long staging_bytes;
    unsigned long long stage_offset[3], stage_capacity[3];   /* gate, up, down of one expert */
    unsigned long long routed_added;
    int shared_added, finished, grouped_selected;
    unsigned long long h2d, d2h, d2d, launches, uploads, downloads, direct_weights, subviews;
    unsigned long long synchronizations, synchronization_ns;
    unsigned long long started_ns, ingress_ns, routing_ns, routed_ns, shared_ns;
};

static unsigned long long now_ns(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (unsigned long long)ts.tv_sec * 1000000000ull + (unsigned long long)ts.tv_nsec;
}

static unsigned long long align_up(unsigned long long v) { return (v + ALIGN - 1ull) & ~(ALIGN - 1ull); }

#define AT(field) ((void *)((unsigned char *)x->block + x->field))

static int launched(yvex_rocm_moe_execution *x, int code, const char *where, yvex_error *err)
{
    int rc = yvex_rocm_launch_result(code, where, err);
    if (rc == YVEX_OK) x->launches++;
    return rc;
}

static int upload(yvex_rocm_moe_execution *x, void *dst, const void *src, unsigned long long bytes,
                  const char *where, yvex_error *err)
{
    if (yvex_hip_memcpy_h2d(dst, src, bytes, x->backend->stream) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
    x->h2d += bytes;
    return YVEX_OK;
}

static int download(yvex_rocm_moe_execution *x, void *dst, const void *src, unsigned long long bytes,
                    const char *where, yvex_error *err)
{
    if (!dst) return YVEX_OK;
    if (yvex_hip_memcpy_d2h(dst, src, bytes, x->backend->stream) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
    x->d2h += bytes;
    x->downloads++;
    return YVEX_OK;
}

/* Device address of a weight view: resident, or uploaded into the staging range at `offset`
 * (src/backend/cuda/moe.c:226-245). */
static int weight_address_in(yvex_rocm_moe_execution *x, const yvex_moe_weight_view *view,
                             unsigned long long row_width, unsigned long long row_count,
                             unsigned long long offset, unsigned long long capacity,
                             unsigned long long *address, const char *where, yvex_error *err);

/* A coefficient or router matrix staged alone: the whole staging range is its own. */
static int weight_address(yvex_rocm_moe_execution *x, const yvex_moe_weight_view *view,
                          unsigned long long row_width, unsigned long long row_count,
                          unsigned long long offset, unsigned long long *address, const char *where,
                          yvex_error *err)
{
    return weight_address_in(x, view, row_width, row_count, offset,
                             offset <= x->staging_bytes ? x->staging_bytes - offset : 0ull, address, where, err);
}

static int weight_address_in(yvex_rocm_moe_execution *x, const yvex_moe_weight_view *view,
                             unsigned long long row_width, unsigned long long row_count,
                             unsigned long long offset, unsigned long long capacity,
                             unsigned long long *address, const char *where, yvex_error *err)
{
    int resident = 0;
    int rc = yvex_rocm_moe_view_check(x->backend, view, row_width, row_count, address, &resident, err);
    if (rc != YVEX_OK) return rc;
    if (resident) {
        x->direct_weights++;
        return YVEX_OK;
    }
    if (offset > x->staging_bytes || capacity > x->staging_bytes - offset || view->encoded_bytes > capacity)
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where,
                                "selected MoE encoded weight exceeds its stable staging range");
    rc = upload(x, (unsigned char *)AT(staging) + offset, view->encoded, view->encoded_bytes, where, err);
    if (rc == YVEX_OK) {
        *address = (unsigned long long)(uintptr_t)((unsigned char *)AT(staging) + offset);
        x->uploads++;
    }
    return rc;
}

/* Stream synchronisation and the kernels' status word (moe.c:277-296). */
static int sync_status(yvex_rocm_moe_execution *x, const char *where, yvex_error *err)
{
    int device_status = 0, rc;
    unsigned long long started = now_ns();
    rc = yvex_rocm_finish(x->backend, where, &device_status, err);
    x->synchronization_ns += now_ns() - started;
    x->synchronizations++;
    x->d2h += sizeof(int);
    if (rc == YVEX_OK && device_status)
        rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where,
                              "MoE kernel reported invalid or non-finite numerics");
    return rc;
}

static int flat_qtype(unsigned int qtype) { return qtype == 0u || qtype == 30u || qtype == 26u; }

static int plan_ranges(yvex_rocm_moe_execution *x, const yvex_moe_layer_plan *layer)
{
    unsigned long long cursor = 0ull, hidden = layer->hidden_width, streams = layer->residual_streams;
    unsigned long long experts = layer->routed_experts, topk = layer->experts_per_token;
    unsigned long long widest = layer->expert_intermediate_width * topk;
    unsigned long long staging = 0ull;
    unsigned int slot;
    if (layer->shared_intermediate_width > widest) widest = layer->shared_intermediate_width;
#define TAKE(field, bytes) do { x->field = cursor; cursor = align_up(cursor + (bytes)); } while (0)
    TAKE(expanded, layer->expanded_width * sizeof(float));
    TAKE(mixes, layer->mhc_mixing_rows * sizeof(float));
    TAKE(scale, 3ull * sizeof(float));
    TAKE(base, layer->mhc_mixing_rows * sizeof(float));
    TAKE(norm, hidden * sizeof(float));
    TAKE(normalized, hidden * sizeof(float));
    TAKE(post, streams * sizeof(float));
    TAKE(combination, streams * streams * sizeof(float));
    TAKE(logits, experts * sizeof(float));
    TAKE(scores, experts * sizeof(float));
    TAKE(bias, experts * sizeof(float));
    TAKE(selected, topk * sizeof(unsigned long long));
    TAKE(weights, topk * sizeof(float));
    TAKE(slot_weights, YVEX_MOE_MAX_SELECTED * sizeof(float));
    TAKE(token, sizeof(unsigned int));
    TAKE(order, topk * sizeof(unsigned long long));
    TAKE(expert_ids, experts * sizeof(unsigned long long));
    TAKE(bucket_offsets, (experts + 1ull) * sizeof(unsigned long long));
    TAKE(bucket_populations, experts * sizeof(unsigned long long));
    TAKE(sweep_offsets, (experts + 1ull) * sizeof(unsigned long long));
    TAKE(counts, 4ull * sizeof(unsigned long long));
    TAKE(intermediate, widest * sizeof(float));
    TAKE(pair_outputs, YVEX_MOE_MAX_SELECTED * hidden * sizeof(float));
    TAKE(shared_output, hidden * sizeof(float));
    TAKE(routed, hidden * sizeof(float));
    TAKE(combined, hidden * sizeof(float));
    /* staging for views outside the arena: gate, up and down of one expert side by side (the
     * sweeps read gate and up together), each range as large as the largest expert matrix of its
     * projection over the routed and the shared slots; or the largest ingress / router
     * coefficient matrix, staged alone (moe.c:552-568 sizes one matrix at a time) */
    for (slot = 0u; slot < 3u; ++slot) {
        unsigned long long part = x->job->weights[YVEX_MOE_WEIGHT_ROUTED_GATE + slot].encoded_bytes /
                                  (experts ? experts : 1ull);
        if (x->job->weights[YVEX_MOE_WEIGHT_SHARED_GATE + slot].encoded_bytes > part)
            part = x->job->weights[YVEX_MOE_WEIGHT_SHARED_GATE + slot].encoded_bytes;
        x->stage_offset[slot] = staging;
        x->stage_capacity[slot] = align_up(part);
        staging += x->stage_capacity[slot];
    }
    for (slot = 0u; slot <= YVEX_MOE_WEIGHT_ROUTER_BIAS; ++slot)
        if (x->job->weights[slot].encoded_bytes > staging && slot != YVEX_MOE_WEIGHT_ROUTER_TABLE)
            staging = x->job->weights[slot].encoded_bytes;
    x->staging_bytes = align_up(staging);
    TAKE(staging, x->staging_bytes);
#undef TAKE
    return cursor <= (1ull << 40);
}

/* src/backend/cuda/moe.c:372-414 */
static int prepare_input(yvex_rocm_moe_execution *x, yvex_error *err)
{
    const yvex_moe_layer_job *job = x->job;
    const yvex_moe_layer_plan *layer = job->layer;
    const yvex_moe_weight_view *function = &job->weights[YVEX_MOE_WEIGHT_MHC_FUNCTION];
    static const int flat_slots[3] = {YVEX_MOE_WEIGHT_MHC_SCALE, YVEX_MOE_WEIGHT_MHC_BASE,
                                      YVEX_MOE_WEIGHT_FFN_NORM};
    const unsigned long long flat_widths[3] = {3ull, layer->mhc_mixing_rows, layer->hidden_width};
    void *flat_targets[3];
    unsigned long long address = 0ull;
    yvex_hip_stream stream = x->backend->stream;
    int *status = x->backend->device_status;
    int rc, k;
    flat_targets[0] = AT(scale);
    flat_targets[1] = AT(base);
    flat_targets[2] = AT(norm);
    rc = weight_address(x, function, layer->expanded_width, layer->mhc_mixing_rows, 0ull, &address,
                        "rocm.moe.mhc-function", err);
    if (rc == YVEX_OK)
        rc = launched(x, yvex_hip_matvec((const uint8_t *)(uintptr_t)address, function->qtype,
                                         layer->mhc_mixing_rows, layer->expanded_width,
                                         function->row_bytes, AT(expanded), 0, 1ull,
                                         layer->expanded_width, NULL, (float *)AT(mixes),
                                         layer->mhc_mixing_rows, 0, status, stream),
                      "rocm.moe.mhc-function", err);
    for (k = 0; rc == YVEX_OK && k < 3; ++k) {
        const yvex_moe_weight_view *view = &job->weights[flat_slots[k]];
        if (!flat_qtype(view->qtype))
            return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.mhc-coefficients",
                                    "MoE FFN coefficients cannot be decoded");
        rc = weight_address(x, view, flat_widths[k], 1ull, 0ull, &address, "rocm.moe.mhc-coefficients", err);
        if (rc == YVEX_OK)
            rc = launched(x, yvex_hip_gather((const uint8_t *)(uintptr_t)address, view->qtype, 1ull,
                                             view->row_width, view->row_bytes, NULL, 1ull,
                                             (float *)flat_targets[k], status, stream),
                          "rocm.moe.mhc-coefficients", err);
    }
    if (rc == YVEX_OK)
        rc = launched(x, yvex_hip_mhc_ingress((const float *)AT(expanded), (const float *)AT(mixes),
                                              (const float *)AT(scale), (const float *)AT(base),
                                              (const float *)AT(norm), 1ull, layer->residual_streams,
                                              layer->hidden_width, layer->mhc_sinkhorn_iterations,
                                              layer->rms_epsilon, layer->mhc_epsilon,
                                              layer->mhc_post_multiplier, (float *)AT(normalized),
                                              (float *)AT(post), (float *)AT(combination), status, stream),
                      "rocm.moe.mhc-ingress", err);
    return rc;
}

/* src/backend/cuda/moe.c:416-514 */
static int route(yvex_rocm_moe_execution *x, yvex_moe_layer_result *result, yvex_error *err)
{
    const yvex_moe_layer_job *job = x->job;
    const yvex_moe_layer_plan *layer = job->layer;
    const yvex_moe_weight_view *router = &job->weights[YVEX_MOE_WEIGHT_ROUTER];
    const yvex_moe_weight_view *bias = &job->weights[YVEX_MOE_WEIGHT_ROUTER_BIAS];
    unsigned long long address = 0ull, experts = layer->routed_experts, topk = layer->experts_per_token;
    yvex_hip_stream stream = x->backend->stream;
    int *status = x->backend->device_status;
    int evidence = !job->device_output || job->evidence_level == YVEX_ATTENTION_EVIDENCE_FULL;
    int hash_router = layer->router_class == YVEX_MOE_ROUTER_HASH_TOKEN_ID;
    int rc = weight_address(x, router, layer->hidden_width, experts, 0ull, &address,
                            "rocm.moe.router-projection", err);
    if (rc == YVEX_OK)
        rc = launched(x, yvex_hip_matvec((const uint8_t *)(uintptr_t)address, router->qtype, experts,
                                         layer->hidden_width, router->row_bytes, AT(normalized), 0, 1ull,
                                         layer->hidden_width, NULL, (float *)AT(logits), experts, 0,
                                         status, stream), "rocm.moe.router-projection", err);
    if (rc == YVEX_OK && !hash_router && layer->requires_correction_bias) {
        if (!flat_qtype(bias->qtype))
            return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.router-bias",
                                    "router bias cannot be decoded");
        rc = weight_address(x, bias, experts, 1ull, 0ull, &address, "rocm.moe.router-bias", err);
        if (rc == YVEX_OK)
            rc = launched(x, yvex_hip_gather((const uint8_t *)(uintptr_t)address, bias->qtype, 1ull,
                                             experts, bias->row_bytes, NULL, 1ull, (float *)AT(bias),
                                             status, stream), "rocm.moe.router-bias", err);
    }
    if (rc == YVEX_OK && evidence)
        rc = launched(x, yvex_hip_moe_route_scores((const float *)AT(logits), experts, (int)layer->scoring,
                                                   (float *)AT(scores), status, stream),
                      "rocm.moe.scores", err);
    if (rc == YVEX_OK && hash_router) {
        /* src/graph/moe.c:539-549 and moe.c:437-456 of the CUDA backend: the token's table row */
        const yvex_moe_weight_view *table = &job->weights[YVEX_MOE_WEIGHT_ROUTER_TABLE];
        unsigned int token = job->token_id;
        if (!job->token_id_present || token >= layer->hash_table_rows || table->qtype != YVEX_GGUF_QTYPE_I32 ||
            table->row_bytes < topk * 4ull || (table->row_bytes & 3ull) ||
            (table->row_count != 1ull && table->row_count < layer->hash_table_rows))
            return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.route",
                                    "MoE hash router requires one in-vocabulary token ID");
        rc = weight_address(x, table, table->row_width, table->row_count, 0ull, &address,
                            "rocm.moe.hash-table", err);
        if (rc == YVEX_OK) rc = upload(x, AT(token), &token, sizeof(token), "rocm.moe.hash-row", err);
        if (rc == YVEX_OK)
            rc = launched(x, yvex_hip_moe_route_hash_rows((const float *)AT(logits),
                                                          (const uint8_t *)(uintptr_t)address,
                                                          (const uint32_t *)AT(token), 1ull, experts, topk,
                                                          layer->hash_table_rows, table->row_bytes,
                                                          table->row_count == 1ull, (int)layer->scoring,
                                                          layer->normalize_topk_probabilities,
                                                          layer->routed_scaling_factor,
                                                          (uint64_t *)AT(selected), (float *)AT(weights),
                                                          status, stream), "rocm.moe.route", err);
    }
    if (rc == YVEX_OK && !hash_router)
        rc = launched(x, yvex_hip_moe_route_rows((const float *)AT(logits),
                                                 layer->requires_correction_bias ? (const float *)AT(bias) : NULL,
                                                 1ull, experts, topk, (int)layer->scoring,
                                                 layer->normalize_topk_probabilities,
                                                 layer->routed_scaling_factor, (uint64_t *)AT(selected),
                                                 (float *)AT(weights), status, stream),
                      "rocm.moe.route", err);
    result->router.selected_count = topk;
    if (rc == YVEX_OK && evidence) {
        rc = download(x, result->router.router_logits, AT(logits), experts * sizeof(float),
                      "rocm.moe.logits-download", err);
        if (rc == YVEX_OK)
            rc = download(x, result->router.router_scores, AT(scores), experts * sizeof(float),
                          "rocm.moe.scores-download", err);
    }
    if (rc == YVEX_OK && !x->grouped_selected) {
        rc = download(x, result->router.selected_experts, AT(selected), topk * sizeof(unsigned long long),
                      "rocm.moe.selected-download", err);
        if (rc == YVEX_OK)
            rc = download(x, result->router.selected_weights, AT(weights), topk * sizeof(float),
                          "rocm.moe.weights-download", err);
        if (rc == YVEX_OK) rc = sync_status(x, "rocm.moe.route-sync", err);
    }
    return rc;
}

static void fill_weights(yvex_hip_expert_weights *w, const yvex_moe_weight_view *gate,
                         const yvex_moe_weight_view *up, const yvex_moe_weight_view *down,
                         const unsigned long long address[3], unsigned long long hidden,
                         unsigned long long intermediate)
{
    memset(w, 0, sizeof(*w));      /* canonical rows: no sweep image */
    w->gate = (const uint8_t *)(uintptr_t)address[0];
    w->up = (const uint8_t *)(uintptr_t)address[1];
    w->down = (const uint8_t *)(uintptr_t)address[2];
    w->gate_qtype = gate->qtype;
    w->up_qtype = up->qtype;
    w->down_qtype = down->qtype;
    w->hidden = hidden;
    w->intermediate = intermediate;
    w->gate_row_bytes = gate->row_bytes;
    w->up_row_bytes = up->row_bytes;
    w->down_row_bytes = down->row_bytes;
    w->gate_expert_bytes = gate->row_bytes * intermediate;
    w->up_expert_bytes = up->row_bytes * intermediate;
    w->down_expert_bytes = down->row_bytes * hidden;
}

/* The selected experts at once from the resident expert-major matrices (moe.c:584-672). */
static int add_selected(yvex_rocm_moe_execution *x, yvex_error *err)
{
    const yvex_moe_layer_job *job = x->job;
    const yvex_moe_layer_plan *layer = job->layer;
    const yvex_moe_weight_view *gate = &job->weights[YVEX_MOE_WEIGHT_ROUTED_GATE];
    const yvex_moe_weight_view *up = &job->weights[YVEX_MOE_WEIGHT_ROUTED_UP];
    const yvex_moe_weight_view *down = &job->weights[YVEX_MOE_WEIGHT_ROUTED_DOWN];
    unsigned long long address[3] = {0}, experts = layer->routed_experts, topk = layer->experts_per_token;
    unsigned long long started = now_ns();
    yvex_hip_expert_weights w;
    yvex_hip_stream stream = x->backend->stream;
    int *status = x->backend->device_status;
    int resident = 0, rc;
    if (gate->layout == YVEX_EXECUTION_LAYOUT_DERIVED_BACKEND)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.grouped",
                                "selected-expert execution takes canonical rows");
    rc = yvex_rocm_moe_view_check(x->backend, gate, layer->hidden_width,
                                  experts * layer->expert_intermediate_width, &address[0], &resident, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_moe_view_check(x->backend, up, layer->hidden_width,
                                      experts * layer->expert_intermediate_width, &address[1], &resident, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_moe_view_check(x->backend, down, layer->expert_intermediate_width,
                                      experts * layer->hidden_width, &address[2], &resident, err);
    if (rc != YVEX_OK) return rc;
    fill_weights(&w, gate, up, down, address, layer->hidden_width, layer->expert_intermediate_width);
    rc = launched(x, yvex_hip_worklist_build((const uint64_t *)AT(selected), topk, topk, experts,
                                             (uint64_t *)AT(order), (uint64_t *)AT(expert_ids),
                                             (uint64_t *)AT(bucket_offsets), (uint64_t *)AT(bucket_populations),
                                             (uint64_t *)AT(sweep_offsets), (uint64_t *)AT(counts), status, stream),
                  "rocm.moe.grouped-worklist", err);
    if (rc == YVEX_OK)
        rc = launched(x, yvex_hip_moe_up(&w, AT(normalized), 0, (const float *)AT(weights),
                                         (const uint64_t *)AT(order), (const uint64_t *)AT(expert_ids),
                                         (const uint64_t *)AT(bucket_offsets),
                                         (const uint64_t *)AT(bucket_populations),
                                         (const uint64_t *)AT(sweep_offsets), (const uint64_t *)AT(counts),
                                         topk, topk, experts, layer->activation_limit,
                                         (float *)AT(intermediate), NULL, 0ull, NULL, status, stream),
                      "rocm.moe.grouped-up", err);
    if (rc == YVEX_OK)
        rc = launched(x, yvex_hip_moe_down(&w, AT(intermediate), 0, (const uint64_t *)AT(order),
                                           (const uint64_t *)AT(expert_ids), (const uint64_t *)AT(bucket_offsets),
                                           (const uint64_t *)AT(bucket_populations),
                                           (const uint64_t *)AT(sweep_offsets), (const uint64_t *)AT(counts),
                                           topk, experts, (float *)AT(pair_outputs), NULL, 0ull, NULL, NULL,
                                           status, stream), "rocm.moe.grouped-down", err);
    if (rc == YVEX_OK) {
        x->routed_added = topk;
        x->direct_weights += 3ull;
        x->subviews += topk * 3ull;
        x->routed_ns += now_ns() - started;
    }
    return rc;
}

int yvex_rocm_backend_moe_begin(yvex_rocm_moe_execution **out, yvex_rocm_backend *backend,
                           const yvex_moe_layer_job *job, yvex_moe_layer_result *result,
                           yvex_error *err)
{
    const yvex_moe_layer_plan *layer = job ? job->layer : NULL;
    yvex_rocm_moe_execution *x;
    unsigned long long expanded_bytes, total;
    int rc;
    if (out) *out = NULL;
    if (!out || !backend || !job || !layer || !result || !job->expanded_input ||
        backend->kind != YVEX_BACKEND_KIND_ROCM || !result->combined_output ||
        result->combined_capacity < layer->hidden_width || !result->post ||
        result->post_capacity < layer->residual_streams || !result->combination ||
        result->combination_capacity < layer->residual_streams * layer->residual_streams)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.begin", "MoE begin arguments are invalid");
    if ((job->device_input || job->device_output) &&
        (!yvex_rocm_tensor_owner_is(backend, job->device_input) ||
         !yvex_rocm_tensor_owner_is(backend, job->device_output) ||
         job->device_input->dtype != YVEX_DTYPE_F32 || job->device_output->dtype != YVEX_DTYPE_F32 ||
         job->device_input->bytes < layer->expanded_width * sizeof(float) ||
         job->device_output->bytes < layer->expanded_width * sizeof(float) ||
         job->device_input == job->device_output))
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.begin",
                                "MoE device activation views are incompatible");
    if (!layer->mhc_mixing_rows || !yvex_rocm_moe_envelope_geometry(layer) || !layer->routed_experts ||
        layer->routed_experts > 256ull || !layer->experts_per_token ||
        layer->experts_per_token > YVEX_MOE_MAX_SELECTED ||
        layer->experts_per_token > layer->routed_experts || !layer->expert_intermediate_width ||
        layer->expert_intermediate_width > (1ull << 20) || layer->shared_intermediate_width > (1ull << 20))
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.begin",
                                "MoE layer geometry is outside this backend's bounds");
    if ((layer->router_class != YVEX_MOE_ROUTER_LEARNED_HIDDEN_STATE &&
         layer->router_class != YVEX_MOE_ROUTER_HASH_TOKEN_ID) ||
        (layer->scoring != YVEX_MOE_SCORING_SQRT_SOFTPLUS && layer->scoring != YVEX_MOE_SCORING_SIGMOID))
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.begin",
                                "other router classes and scoring policies are outside this backend");
    if (!(layer->activation_limit > 0.0) || !isfinite(layer->activation_limit) ||
        !isfinite(layer->routed_scaling_factor))
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.begin",
                                "activation limit and routed scaling must be finite");
    if (job->device_input && !job->device_input->is_written)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "rocm.moe.begin", "device input was never written");
    rc = yvex_rocm_require_kernels(backend, "rocm.moe.begin", err);
    if (rc != YVEX_OK) return rc;
    if (job->cancel_requested && job->cancel_requested(job->cancel_context))
        return yvex_rocm_refuse(err, YVEX_ERR_CANCELLED, "rocm.moe.begin", "MoE execution was cancelled");
    x = (yvex_rocm_moe_execution *)calloc(1u, sizeof(*x));
    if (!x) return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, "rocm.moe.begin", "MoE owner allocation failed");
    x->backend = backend;
    x->job = job;
    x->started_ns = now_ns();
    /* the caller decides by the same rule whether it still has to add the routed experts
     * (src/backend/cuda/moe.c:557-561, src/runtime/moe.c:654-660) */
    x->grouped_selected = job->device_output && job->evidence_level != YVEX_ATTENTION_EVIDENCE_FULL &&
                          job->weights[YVEX_MOE_WEIGHT_ROUTED_GATE].device_address &&
                          job->weights[YVEX_MOE_WEIGHT_ROUTED_UP].device_address &&
                          job->weights[YVEX_MOE_WEIGHT_ROUTED_DOWN].device_address;
    if (!plan_ranges(x, layer)) {
        free(x);
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.begin", "MoE range extent overflowed");
    }
    total = x->staging + x->staging_bytes;
    {
        /* the attached workspace when it has room (no allocation on the token path), else a
         * block of the execution's own */
        unsigned long long base = 0ull;
        yvex_rocm_workspace_reset(backend);
        if (backend->workspace_device_tensor &&
            yvex_rocm_backend_workspace_acquire(backend, total, ALIGN, &base)) {
            x->block = (void *)(uintptr_t)base;
        } else if (yvex_hip_malloc(&x->block, total) != 0) {
            free(x);
            return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, "rocm.moe.begin", yvex_hip_last_error());
        } else {
            x->owns_block = 1;
        }
    }
    expanded_bytes = layer->expanded_width * sizeof(float);
    rc = backend->pending_completion   /* deferred row batches own the word until their barrier */
        ? YVEX_OK
        : launched(x, yvex_hip_fill_u32(backend->device_status, 0u, 1u, backend->stream), "rocm.moe.status", err);
    if (rc == YVEX_OK)       /* slots never added read as zero in the rank-ordered sum */
        rc = launched(x, yvex_hip_fill_u32(AT(pair_outputs), 0u,
                                           (x->routed - x->pair_outputs) / sizeof(float), backend->stream),
                      "rocm.moe.zero", err);
    if (rc == YVEX_OK) {
        if (job->device_input) {
            if (yvex_hip_memcpy_d2d(AT(expanded), job->device_input->data, expanded_bytes, backend->stream) != 0)
                rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.moe.device-input", yvex_hip_last_error());
            else x->d2d += expanded_bytes;
        } else {
            rc = upload(x, AT(expanded), job->expanded_input, expanded_bytes, "rocm.moe.input", err);
        }
    }
    if (rc == YVEX_OK) rc = prepare_input(x, err);
    if (rc == YVEX_OK) {
        unsigned long long routing_started = now_ns();
        x->ingress_ns = routing_started - x->started_ns;
        rc = route(x, result, err);
        if (rc == YVEX_OK) x->routing_ns = now_ns() - routing_started;
    }
    if (rc == YVEX_OK && x->grouped_selected) rc = add_selected(x, err);
    if (rc != YVEX_OK) {
        (void)yvex_rocm_backend_moe_close(&x, NULL);
        return rc;
    }
    *out = x;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_moe_add_expert(yvex_rocm_moe_execution *x, const yvex_moe_weight_view *gate,
                                const yvex_moe_weight_view *up, const yvex_moe_weight_view *down,
                                float route_weight, int shared, yvex_error *err)
{
    const yvex_moe_layer_plan *layer = x && x->job ? x->job->layer : NULL;
    unsigned long long address[3] = {0}, width, started = now_ns();
    yvex_hip_expert_weights w;
    yvex_hip_stream stream;
    float *target;
    int *status;
    int rc;
    if (!x || !layer || !gate || !up || !down || x->finished || gate->row_count != up->row_count ||
        down->row_width != gate->row_count || down->row_count != layer->hidden_width)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.expert", "MoE expert geometry is invalid");
    width = gate->row_count;
    if (!width || width > (shared ? layer->shared_intermediate_width
                                  : layer->expert_intermediate_width * layer->experts_per_token) ||
        (!shared && x->routed_added >= YVEX_MOE_MAX_SELECTED) || (shared && x->shared_added))
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "rocm.moe.expert",
                                "MoE expert exceeds the ranges planned at begin");
    stream = x->backend->stream;
    status = x->backend->device_status;
    rc = weight_address_in(x, gate, layer->hidden_width, width, x->stage_offset[0], x->stage_capacity[0],
                           &address[0], "rocm.moe.expert-gate", err);
    if (rc == YVEX_OK)
        rc = weight_address_in(x, up, layer->hidden_width, width, x->stage_offset[1], x->stage_capacity[1],
                               &address[1], "rocm.moe.expert-up", err);
    if (rc == YVEX_OK)
        rc = weight_address_in(x, down, width, layer->hidden_width, x->stage_offset[2],
                               x->stage_capacity[2], &address[2], "rocm.moe.expert-down", err);
    if (rc != YVEX_OK) return rc;
    fill_weights(&w, gate, up, down, address, layer->hidden_width, width);
    if (!shared) {
        unsigned int bits;
        memcpy(&bits, &route_weight, sizeof(bits));
        rc = launched(x, yvex_hip_fill_u32((float *)AT(slot_weights) + x->routed_added, bits, 1u, stream),
                      "rocm.moe.route-weight", err);
    }
    /* single-expert forms of the sweeps: one pair, F32 activations (moe.c:674-737) */
    if (rc == YVEX_OK)
        rc = launched(x, yvex_hip_moe_up(&w, AT(normalized), 0,
                                         shared ? NULL : (const float *)AT(slot_weights) + x->routed_added,
                                         NULL, NULL, NULL, NULL, NULL, NULL, 1ull, 1ull, 1ull,
                                         layer->activation_limit, (float *)AT(intermediate), NULL, 0ull, NULL,
                                         status, stream), "rocm.moe.expert-up", err);
    target = shared ? (float *)AT(shared_output)
                    : (float *)AT(pair_outputs) + x->routed_added * layer->hidden_width;
    if (rc == YVEX_OK)
        rc = launched(x, yvex_hip_moe_down(&w, AT(intermediate), 0, NULL, NULL, NULL, NULL, NULL, NULL, 1ull,
                                           1ull, target, NULL, 0ull, NULL, NULL, status, stream),
                      "rocm.moe.expert-down", err);
    if (rc == YVEX_OK) {
        if (shared) {
            x->shared_added = 1;
            x->shared_ns += now_ns() - started;
        } else {
            x->routed_added++;
            x->subviews += 3ull;
            x->routed_ns += now_ns() - started;
        }
        yvex_rocm_error_clear(err);
    }
    return rc;
}

int yvex_rocm_backend_moe_finish(yvex_rocm_moe_execution *x, yvex_moe_layer_result *result, yvex_error *err)
{
    const yvex_moe_layer_plan *layer = x && x->job ? x->job->layer : NULL;
    unsigned long long hidden, streams;
    yvex_hip_stream stream;
    int *status;
    int rc, evidence;
    if (!x || !layer || !result || x->finished)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.finish", "MoE finish is invalid");
    hidden = layer->hidden_width;
    streams = layer->residual_streams;
    if (!result->routed_output || result->routed_capacity < hidden || !result->shared_output ||
        result->shared_capacity < hidden)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.moe.finish",
                                "MoE routed/shared publication capacity is invalid");
    stream = x->backend->stream;
    status = x->backend->device_status;
    evidence = !x->job->device_output || x->job->evidence_level == YVEX_ATTENTION_EVIDENCE_FULL;
    /* routed = experts in the order added, combined = bf16(routed + shared): moe.c:752-770 */
    rc = launched(x, yvex_hip_moe_reduce_combine((const float *)AT(pair_outputs), 1ull,
                                                 x->routed_added ? x->routed_added : 1ull, hidden,
                                                 (const float *)AT(shared_output), (float *)AT(routed),
                                                 (float *)AT(combined), status, stream),
                  "rocm.moe.combine", err);
    if (rc == YVEX_OK && x->job->device_output) {
        x->job->device_output->is_written = 0;
        rc = launched(x, yvex_hip_mhc_egress((const float *)AT(combined), (const float *)AT(expanded),
                                             (const float *)AT(post), (const float *)AT(combination), 1ull,
                                             streams, hidden, (float *)x->job->device_output->data, status,
                                             stream), "rocm.moe.deferred-post", err);
    }
    if (rc == YVEX_OK && x->grouped_selected) {
        rc = download(x, result->router.selected_experts, AT(selected),
                      layer->experts_per_token * sizeof(unsigned long long), "rocm.moe.selected-publication", err);
        if (rc == YVEX_OK)
            rc = download(x, result->router.selected_weights, AT(weights),
                          layer->experts_per_token * sizeof(float), "rocm.moe.weights-publication", err);
    }
    if (rc == YVEX_OK && evidence) {
        rc = download(x, result->combined_output, AT(combined), hidden * sizeof(float), "rocm.moe.output-download", err);
        if (rc == YVEX_OK)
            rc = download(x, result->routed_output, AT(routed), hidden * sizeof(float), "rocm.moe.routed-download", err);
        if (rc == YVEX_OK)
            rc = download(x, result->shared_output, AT(shared_output), hidden * sizeof(float),
                          "rocm.moe.shared-download", err);
        if (rc == YVEX_OK)
            rc = download(x, result->post, AT(post), streams * sizeof(float), "rocm.moe.post-download", err);
        if (rc == YVEX_OK)
            rc = download(x, result->combination, AT(combination), streams * streams * sizeof(float),
                          "rocm.moe.combination-download", err);
    }
    if (rc == YVEX_OK) rc = sync_status(x, "rocm.moe.finish-sync", err);
    if (rc != YVEX_OK) return rc;
    if (x->job->device_output) x->job->device_output->is_written = 1;
    if (x->job->device_input && x->job->device_output) {
        result->memory.activation_bytes = 2ull * layer->expanded_width * sizeof(float);
        result->memory.temporary_bytes = x->staging + x->staging_bytes;
    }
    result->expert_subviews_accessed += x->subviews;
    result->host_to_device_bytes += x->h2d;
    result->device_to_host_bytes += x->d2h;
    result->kernel_launches += x->launches;
    result->upload_count += x->uploads;
    result->download_count += x->downloads;
    result->cache_hits += x->direct_weights;
    result->cache_misses += x->uploads;
    result->device_to_device_bytes += x->d2d;
    result->stream_synchronizations += x->synchronizations;
    result->synchronization_ns += x->synchronization_ns;
    result->ingress_ns += x->ingress_ns;
    result->routing_ns += x->routing_ns;
    result->routed_ns += x->routed_ns;
    result->shared_ns += x->shared_ns;
    result->total_ns += now_ns() - x->started_ns;
    x->backend->memory.h2d_bytes += x->h2d;
    x->backend->memory.d2h_bytes += x->d2h - x->synchronizations * sizeof(int);   /* counted by the sync */
    x->finished = 1;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_moe_close(yvex_rocm_moe_execution **execution, yvex_error *err)
{
    if (!execution || !*execution) {
        yvex_rocm_error_clear(err);
        return YVEX_OK;
    }
    if ((*execution)->block && (*execution)->owns_block) {
        /* kernels of an abandoned execution may still be reading the block */
        (void)yvex_hip_stream_sync((*execution)->backend->stream);
        if (yvex_hip_free((*execution)->block) != 0)
            return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.moe.close", yvex_hip_last_error());
    }
    free(*execution);
    *execution = NULL;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}
