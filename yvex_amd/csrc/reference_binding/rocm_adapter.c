/*
 * Reference-side binding of libyvex_rocm.so: the file a yailabs/yvex maintainer adds to the
 * reference tree (as src/backend/rocm/adapter.c) to run the quantized-weight matmul path on an
 * MI355X. It is compiled with the reference's own headers, not into libyvex_rocm.so; this
 * repository only checks that it compiles against them.
 *
 * The reference's backend object (struct yvex_backend, src/backend/private.h:66-95) stays the
 * owner its core and runtime see. The ROCm backend object of the library sits behind `impl`;
 * the vtable below forwards the lifecycle and tensor entries of src/backend/private.h:10-64, and
 * the operation entry points forward the calls the CUDA backend serves for this path:
 * yvex_backend_cuda_encoded_matvec / _gather (include/yvex/internal/backend.h:332-343), the MoE
 * row-batch operations table (include/yvex/internal/moe.h:273-297) and the token-local MoE
 * operation (moe.h:308-319).
 *
 * Residency and workspace are attached on the reference's object by its own generic code
 * (src/backend/residency.c:19-112, src/backend/core.c workspace functions); rocm_follow() carries
 * a changed attachment over to the library before an operation runs. The library publishes a
 * resident arena to HBM at attach, so the first operation after a new generation pays the upload.
 */
#include <stdatomic.h>
#include <stdlib.h>
#include <string.h>

#include <yvex/internal/backend.h>
#include <yvex/internal/moe.h>

#include "backend/private.h"

#define YVEX_ROCM_REFERENCE_TYPES
#include "yvex_rocm.h"

typedef struct {
    yvex_rocm_backend *backend;
    unsigned long long resident_generation;          /* what the library has attached */
    const yvex_device_tensor *resident_tensor;
    const yvex_device_tensor *workspace_tensor;
    unsigned long long workspace_bytes;
} rocm_impl;

static rocm_impl *rocm_of(const yvex_backend *backend)
{
    return backend && backend->kind == YVEX_BACKEND_KIND_ROCM ? (rocm_impl *)backend->impl : NULL;
}

/* Carry the owner's current resident arena and workspace over to the library. */
static int rocm_follow(yvex_backend *backend, yvex_error *err)
{
    rocm_impl *impl = rocm_of(backend);
    int rc = YVEX_OK;
    if (!impl) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "rocm.adapter", "a ROCm backend is required");
        return YVEX_ERR_INVALID_ARG;
    }
    /* a shared session attaches what its owner has published: the owner goes first */
    if (backend->resource_owner && backend->resource_owner != backend) {
        rc = rocm_follow(backend->resource_owner, err);
        if (rc != YVEX_OK) return rc;
    }
    if (impl->resident_generation != backend->resident_generation ||
        impl->resident_tensor != backend->resident_device_tensor) {
        if (backend->resident_device_tensor)
            rc = yvex_rocm_backend_resident_attach(impl->backend, backend->resident_host_base,
                                                   backend->resident_host_bytes,
                                                   backend->resident_device_tensor,
                                                   backend->resident_generation, err);
        else
            rc = yvex_rocm_backend_resident_detach(impl->backend, err);
        if (rc != YVEX_OK) return rc;
        impl->resident_generation = backend->resident_generation;
        impl->resident_tensor = backend->resident_device_tensor;
    }
    if (impl->workspace_tensor != backend->workspace_device_tensor ||
        impl->workspace_bytes != backend->workspace_bytes) {
        if (backend->workspace_device_tensor)
            rc = yvex_rocm_backend_workspace_attach(impl->backend, backend->workspace_device_tensor,
                                                    backend->workspace_bytes, err);
        else
            yvex_rocm_backend_workspace_detach(impl->backend);
        if (rc != YVEX_OK) return rc;
        impl->workspace_tensor = backend->workspace_device_tensor;
        impl->workspace_bytes = backend->workspace_bytes;
    }
    return YVEX_OK;
}

/* ---- vtable: src/backend/private.h:10-64 ------------------------------------------------------ */

static int rocm_close(yvex_backend *backend, yvex_error *err)
{
    rocm_impl *impl = rocm_of(backend);
    int rc = impl ? yvex_rocm_backend_close_checked(&impl->backend, err) : YVEX_OK;
    if (rc != YVEX_OK) return rc;              /* the owner stays for a checked retry */
    free(impl);
    backend->impl = NULL;
    return YVEX_OK;
}

static int rocm_memory_stats(const yvex_backend *backend, yvex_backend_memory_stats *out, yvex_error *err)
{
    return yvex_rocm_backend_get_memory_stats(rocm_of(backend)->backend, out, err);
}

static int rocm_bandwidth_probe(yvex_backend *backend, yvex_backend_bandwidth_evidence *out, yvex_error *err)
{
    return yvex_rocm_backend_bandwidth_probe(rocm_of(backend)->backend, out, err);
}

static int rocm_tensor_alloc(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                             yvex_device_tensor **out, yvex_error *err)
{
    return yvex_rocm_backend_tensor_alloc(rocm_of(backend)->backend, desc, out, err);
}

static int rocm_resident_alloc(yvex_backend *backend, const yvex_backend_tensor_desc *desc,
                               yvex_device_tensor **out, unsigned char **host, yvex_error *err)
{
    return yvex_rocm_backend_resident_alloc(rocm_of(backend)->backend, desc, out, host, err);
}

static int rocm_resident_prefetch_supported(const yvex_backend *backend)
{
    return rocm_of(backend) != NULL;
}

static int rocm_resident_prefetch(yvex_backend *backend, yvex_device_tensor *tensor,
                                  unsigned long long *prefetched, yvex_error *err)
{
    return yvex_rocm_backend_resident_prefetch(rocm_of(backend)->backend, tensor, prefetched, err);
}

static int rocm_tensor_free(yvex_backend *backend, yvex_device_tensor *tensor, yvex_error *err)
{
    return yvex_rocm_backend_tensor_release(rocm_of(backend)->backend, &tensor, err);
}

static int rocm_tensor_write(yvex_backend *backend, yvex_device_tensor *tensor, const void *src,
                             unsigned long long len, yvex_error *err)
{
    return yvex_rocm_backend_tensor_write(rocm_of(backend)->backend, tensor, src, len, err);
}

static int rocm_tensor_read(yvex_backend *backend, const yvex_device_tensor *tensor, void *dst,
                            unsigned long long len, yvex_error *err)
{
    return yvex_rocm_backend_tensor_read(rocm_of(backend)->backend, tensor, dst, len, err);
}

static int rocm_tensor_copy(yvex_backend *backend, yvex_device_tensor *dst,
                            const yvex_device_tensor *src, yvex_error *err)
{
    return yvex_rocm_backend_tensor_copy(rocm_of(backend)->backend, dst, src, err);
}

static int rocm_sync(yvex_backend *backend, yvex_error *err)
{
    return yvex_rocm_backend_sync(rocm_of(backend)->backend, err);
}

static int rocm_query_capability(const yvex_backend *backend, yvex_backend_operation_variant variant,
                                 yvex_backend_capability_result *out, yvex_error *err)
{
    return yvex_rocm_backend_query_capability(rocm_of(backend)->backend, variant, out, err);
}

/* Entries left NULL (embed, rms_norm, rope, matmul, mlp, attention, virtual tensors, host
 * workspace) are outside this path; the core refuses a NULL entry as unsupported. */
static const yvex_backend_vtable rocm_vtable = {
    .close = rocm_close,
    .memory_stats = rocm_memory_stats,
    .bandwidth_probe = rocm_bandwidth_probe,
    .tensor_alloc = rocm_tensor_alloc,
    .resident_alloc = rocm_resident_alloc,
    .resident_prefetch_supported = rocm_resident_prefetch_supported,
    .resident_prefetch = rocm_resident_prefetch,
    .tensor_free = rocm_tensor_free,
    .tensor_write = rocm_tensor_write,
    .tensor_read = rocm_tensor_read,
    .tensor_copy = rocm_tensor_copy,
    .tensor_copy_async = rocm_tensor_copy,          /* one stream: a copy is ordered on it */
    .sync = rocm_sync,
    .query_capability = rocm_query_capability,
};

/* Called from yvex_backend_open (src/backend/core.c:197-200) beside the CUDA arm. */
int yvex_backend_open_rocm_impl(yvex_backend **out, const char *device,
                                unsigned long long memory_limit_bytes, yvex_error *err)
{
    yvex_backend_options options;
    yvex_backend *backend;
    rocm_impl *impl;
    int rc;
    if (!out) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "yvex_backend_open", "out is required");
        return YVEX_ERR_INVALID_ARG;
    }
    *out = NULL;
    backend = (yvex_backend *)calloc(1u, sizeof(*backend));
    impl = (rocm_impl *)calloc(1u, sizeof(*impl));
    if (!backend || !impl) {
        free(backend);
        free(impl);
        yvex_error_set(err, YVEX_ERR_NOMEM, "yvex_backend_open", "backend allocation failed");
        return YVEX_ERR_NOMEM;
    }
    memset(&options, 0, sizeof(options));
    options.kind = YVEX_BACKEND_KIND_ROCM;
    options.device = device;
    options.memory_limit_bytes = memory_limit_bytes;
    rc = yvex_rocm_backend_open(&impl->backend, &options, err);
    /* tensors name the reference's object as their owner, so backend_tensor_owner_is holds */
    if (rc == YVEX_OK) rc = yvex_rocm_backend_bind_owner(impl->backend, backend, err);
    if (rc != YVEX_OK) {
        if (impl->backend) (void)yvex_rocm_backend_close_checked(&impl->backend, NULL);
        free(impl);
        free(backend);
        return rc;
    }
    backend->kind = YVEX_BACKEND_KIND_ROCM;
    backend->status = yvex_rocm_backend_status_of(impl->backend);
    backend->vtable = &rocm_vtable;
    backend->impl = impl;
    backend->resource_owner = backend;
    backend->tensor_id_next = 1ull;
    backend->stats.memory_limit_bytes = memory_limit_bytes;
    *out = backend;
    return YVEX_OK;
}

/* The ROCm counterpart of yvex_backend_open_shared_cuda (include/yvex/internal/backend.h:254-255,
 * src/backend/cuda/backend.c:1913-2000): session-local state that borrows one model-owned backend.
 * The lease on the owner is the child count in its lifecycle word, which the reference's
 * yvex_backend_close_checked releases (src/backend/core.c:283-343). */
int yvex_backend_open_shared_rocm(yvex_backend **out, yvex_backend *context_owner,
                                  unsigned long long memory_limit_bytes, yvex_error *err)
{
    yvex_backend *backend;
    rocm_impl *impl, *owner_impl = rocm_of(context_owner);
    unsigned long long observed;
    int rc;
    if (out) *out = NULL;
    if (!out || !owner_impl || context_owner->resource_owner != context_owner) {
        yvex_error_set(err, YVEX_ERR_INVALID_ARG, "rocm.shared.open", "one owning ROCm backend is required");
        return YVEX_ERR_INVALID_ARG;
    }
    backend = (yvex_backend *)calloc(1u, sizeof(*backend));
    impl = (rocm_impl *)calloc(1u, sizeof(*impl));
    if (!backend || !impl) {
        free(backend);
        free(impl);
        yvex_error_set(err, YVEX_ERR_NOMEM, "rocm.shared.open", "shared ROCm session allocation failed");
        return YVEX_ERR_NOMEM;
    }
    observed = atomic_load_explicit(&context_owner->lifecycle, memory_order_acquire);
    for (;;) {
        if (observed & YVEX_BACKEND_LIFECYCLE_CLOSING) {
            free(backend);
            free(impl);
            yvex_error_set(err, YVEX_ERR_STATE, "rocm.shared.open", "owning ROCm backend is closing");
            return YVEX_ERR_STATE;
        }
        if (atomic_compare_exchange_weak_explicit(&context_owner->lifecycle, &observed, observed + 1ull,
                                                  memory_order_acq_rel, memory_order_acquire))
            break;
    }
    rc = yvex_rocm_backend_open_shared(&impl->backend, owner_impl->backend, memory_limit_bytes, err);
    if (rc == YVEX_OK) rc = yvex_rocm_backend_bind_owner(impl->backend, backend, err);
    if (rc != YVEX_OK) {
        if (impl->backend) (void)yvex_rocm_backend_close_checked(&impl->backend, NULL);
        atomic_fetch_sub_explicit(&context_owner->lifecycle, 1ull, memory_order_acq_rel);
        free(impl);
        free(backend);
        return rc;
    }
    backend->kind = YVEX_BACKEND_KIND_ROCM;
    backend->status = yvex_rocm_backend_status_of(impl->backend);
    backend->vtable = &rocm_vtable;
    backend->impl = impl;
    backend->resource_owner = context_owner;
    backend->shared_owner_registered = 1;
    backend->tensor_id_next = 1ull;
    backend->stats.memory_limit_bytes = memory_limit_bytes;
    backend->device_info = context_owner->device_info;
    *out = backend;
    return YVEX_OK;
}

/* ---- dense projection, output head, gather: include/yvex/internal/backend.h:332-343 ---------- */

int yvex_backend_rocm_encoded_matvec(
    yvex_backend *backend, const unsigned char *resident_encoded, unsigned long long encoded_bytes,
    unsigned int qtype, unsigned long long row_count, unsigned long long row_width,
    unsigned long long row_bytes, unsigned long long input_rows, const yvex_device_tensor *input,
    const yvex_device_tensor *input_tail, unsigned long long input_head_width,
    const yvex_device_tensor *additive, yvex_device_tensor *output, int activation_q8,
    yvex_backend_cuda_operation_facts *facts, yvex_error *err)
{
    int rc = rocm_follow(backend, err);
    if (rc != YVEX_OK) return rc;
    /* the facts structure has the same members in the same order in both libraries */
    return yvex_rocm_encoded_matvec(rocm_of(backend)->backend, resident_encoded, encoded_bytes, qtype,
                                    row_count, row_width, row_bytes, input_rows, input, input_tail,
                                    input_head_width, additive, output, activation_q8,
                                    (yvex_rocm_operation_facts *)facts, err);
}

int yvex_backend_rocm_encoded_gather(
    yvex_backend *backend, const unsigned char *resident_encoded, unsigned long long encoded_bytes,
    unsigned int qtype, unsigned long long row_count, unsigned long long row_width,
    unsigned long long row_bytes, const unsigned int *row_ids, unsigned long long selected_rows,
    yvex_device_tensor *output, yvex_backend_cuda_operation_facts *facts, yvex_error *err)
{
    int rc = rocm_follow(backend, err);
    if (rc != YVEX_OK) return rc;
    return yvex_rocm_encoded_gather(rocm_of(backend)->backend, resident_encoded, encoded_bytes, qtype,
                                    row_count, row_width, row_bytes, row_ids, selected_rows, output,
                                    (yvex_rocm_operation_facts *)facts, err);
}

/* ---- MoE row batch: include/yvex/internal/moe.h:273-297 ---------------------------------------- */

static int rocm_workspace_required(const yvex_moe_layer_plan *layer, unsigned long long rows,
                                   unsigned long long *bytes, yvex_error *err)
{
    return yvex_rocm_moe_workspace_required(layer, rows, bytes, err);
}

static int rocm_execute_rows(yvex_backend *backend, const yvex_moe_layer_job *job,
                             const yvex_moe_row_batch *rows, const yvex_moe_row_batch_output *output,
                             yvex_moe_row_batch_result *result, yvex_error *err)
{
    const yvex_rocm_moe_operations *ops;
    int rc = rocm_follow(backend, err);
    if (rc != YVEX_OK) return rc;
    ops = yvex_rocm_backend_moe_operations_get(rocm_of(backend)->backend);
    if (!ops) {
        yvex_error_set(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.rows", "ROCm MoE kernels are unavailable");
        return YVEX_ERR_UNSUPPORTED;
    }
    return ops->execute_rows(rocm_of(backend)->backend, job, rows, output, result, err);
}

static int rocm_complete_rows(yvex_backend *backend, int barrier_observed,
                              yvex_moe_row_batch_result *result, yvex_error *err)
{
    const yvex_rocm_moe_operations *ops = yvex_rocm_backend_moe_operations_get(rocm_of(backend)->backend);
    if (!ops) {
        yvex_error_set(err, YVEX_ERR_UNSUPPORTED, "rocm.moe.complete", "ROCm MoE kernels are unavailable");
        return YVEX_ERR_UNSUPPORTED;
    }
    return ops->complete_rows(rocm_of(backend)->backend, barrier_observed, result, err);
}

/* Returned by yvex_backend_moe_operations_get (src/backend/cuda/moe.c:1968) for kind ROCM. */
const yvex_backend_moe_operations *yvex_backend_rocm_moe_operations_get(const yvex_backend *backend)
{
    static const yvex_backend_moe_operations table = {
        .derived_layout_plan = yvex_rocm_moe_derived_layout_plan,
        .derived_layout_build = yvex_rocm_moe_derived_layout_build,
        .workspace_required = rocm_workspace_required,
        .execute_rows = rocm_execute_rows,
        .complete_rows = rocm_complete_rows,
    };
    rocm_impl *impl = rocm_of(backend);
    return impl && yvex_rocm_backend_moe_operations_get(impl->backend) ? &table : NULL;
}

/* ---- token-local MoE operation: include/yvex/internal/moe.h:308-319 ---------------------------- */

int yvex_backend_rocm_moe_begin(yvex_backend_moe_execution **out, yvex_backend *backend,
                                const yvex_moe_layer_job *job, yvex_moe_layer_result *result,
                                yvex_error *err)
{
    int rc = rocm_follow(backend, err);
    if (rc != YVEX_OK) return rc;
    return yvex_rocm_backend_moe_begin((yvex_rocm_moe_execution **)out, rocm_of(backend)->backend, job,
                                       result, err);
}

int yvex_backend_rocm_moe_add_expert(yvex_backend_moe_execution *execution,
                                     const yvex_moe_weight_view *gate, const yvex_moe_weight_view *up,
                                     const yvex_moe_weight_view *down, float route_weight, int shared,
                                     yvex_error *err)
{
    return yvex_rocm_backend_moe_add_expert((yvex_rocm_moe_execution *)execution, gate, up, down,
                                            route_weight, shared, err);
}

int yvex_backend_rocm_moe_finish(yvex_backend_moe_execution *execution, yvex_moe_layer_result *result,
                                 yvex_error *err)
{
    return yvex_rocm_backend_moe_finish((yvex_rocm_moe_execution *)execution, result, err);
}

int yvex_backend_rocm_moe_close(yvex_backend_moe_execution **execution, yvex_error *err)
{
    return yvex_rocm_backend_moe_close((yvex_rocm_moe_execution **)execution, err);
}
