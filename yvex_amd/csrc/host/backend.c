/*
 * The ROCm backend object: lifecycle, owned tensors, resident weight arena, device workspace and
 * capability queries. Restates the contract of src/backend/core.c:176-205 (open),
 * src/backend/private.h:95-162 (ownership, workspace reset), src/backend/residency.c:19-112
 * (resident attach / resolve) and tests/test_cuda_failclosed.sh:61-82 (a backend whose kernels
 * are absent still allocates, writes and reads tensors but refuses every compute variant).
 */
#include <limits.h>
#include <stdlib.h>
#include <string.h>

#include "private.h"

static unsigned long long next_owner_id = 1ull;

int yvex_rocm_refuse(yvex_error *err, yvex_status code, const char *where, const char *message)
{
    yvex_rocm_error_set(err, code, where, message);
    return code;
}

int yvex_rocm_seam(const char *name)
{
    const char *value = getenv(name);
    return value && value[0] && strcmp(value, "0") != 0;
}

int yvex_rocm_tensor_owner_is(const yvex_rocm_backend *backend, const yvex_device_tensor *tensor)
{
    return backend && tensor && (const void *)tensor->owner == backend->public_owner &&
           tensor->owner_id == backend->owner_id;
}

int yvex_rocm_backend_tensor_owned_by(const yvex_rocm_backend *backend, const yvex_device_tensor *tensor)
{
    return yvex_rocm_tensor_owner_is(backend, tensor);
}

void yvex_rocm_workspace_reset(yvex_rocm_backend *backend)
{
    if (backend) backend->workspace_cursor = 0ull;
}

int yvex_rocm_launch_result(int rc, const char *where, yvex_error *err)
{
    if (rc == 0) return YVEX_OK;
    if (rc == YVEX_ERR_BACKEND)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
    return yvex_rocm_refuse(err, (yvex_status)rc, where, "kernel launch refused the operand geometry");
}

int yvex_rocm_require_kernels(const yvex_rocm_backend *backend, const char *where, yvex_error *err)
{
    if (!backend || backend->status == YVEX_BACKEND_STATUS_FAILED)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, where, "backend is failed or closing");
    if (!backend->kernels_available)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, where,
                                "operation variant unsupported: kernel-bundle-absent");
    return YVEX_OK;
}

int yvex_rocm_status_reset(yvex_rocm_backend *backend, const char *where, yvex_error *err)
{
    /* row batches whose completion is deferred own the word until their barrier: an operation
     * that runs between them must not erase what they raised (it then reports it as its own) */
    if (backend->pending_completion) return YVEX_OK;
    return yvex_rocm_launch_result(yvex_hip_fill_u32(backend->device_status, 0u, 1u, backend->stream),
                                   where, err);
}

int yvex_rocm_finish(yvex_rocm_backend *backend, const char *where, int *device_status, yvex_error *err)
{
    int rc;
    *device_status = 0;
    if (yvex_rocm_seam("YVEX_TEST_ROCM_SYNC_FAILURE"))
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, "synchronisation failed (test seam)");
    /* the copy below synchronises the stream after the last kernel */
    rc = yvex_hip_memcpy_d2h(device_status, backend->device_status, sizeof(int), backend->stream);
    if (rc != 0) {
        backend->status = YVEX_BACKEND_STATUS_FAILED;
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
    }
    backend->memory.d2h_bytes += sizeof(int);
    return YVEX_OK;
}

int yvex_rocm_upload_queued(yvex_rocm_backend *backend, void *device, const void *host,
                            unsigned long long bytes)
{
    const unsigned long long piece = (bytes + 63ull) & ~63ull;
    if (!bytes) return 0;
    /* nothing deferred: every earlier copy out of the staging memory has been waited for */
    if (!backend->pending_completion) backend->token_staging_cursor = 0ull;
    if (backend->token_staging_cursor == 0ull && backend->token_staging_bytes < piece) {
        unsigned long long want = piece < (64ull << 10) ? (64ull << 10) : piece * 2ull;
        void *fresh = NULL;
        if (yvex_hip_stream_sync(backend->stream) != 0) return -1;
        if (backend->token_staging) (void)yvex_hip_host_free(backend->token_staging);
        backend->token_staging = NULL;
        backend->token_staging_bytes = 0ull;
        if (yvex_hip_host_alloc(&fresh, want) == 0) {
            backend->token_staging = (unsigned char *)fresh;
            backend->token_staging_bytes = want;
        }
    }
    if (!backend->token_staging ||
        backend->token_staging_bytes - backend->token_staging_cursor < piece)
        return yvex_hip_memcpy_h2d(device, host, bytes, backend->stream);   /* waits for the copy */
    memcpy(backend->token_staging + backend->token_staging_cursor, host, (size_t)bytes);
    if (yvex_hip_memcpy_h2d_queued(device, backend->token_staging + backend->token_staging_cursor, bytes,
                                   backend->stream) != 0)
        return -1;
    backend->token_staging_cursor += piece;
    return 0;
}

int yvex_rocm_backend_open(yvex_rocm_backend **out, const yvex_backend_options *options, yvex_error *err)
{
    yvex_rocm_backend *backend;
    int device = 0, host_only;
    if (out) *out = NULL;
    if (!out || !options)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.open",
                                "backend output and options are required");
    if (options->kind != YVEX_BACKEND_KIND_ROCM)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, "backend.open",
                                "this library implements the rocm backend only");
    if (options->device && options->device[0]) {
        char *end = NULL;
        long parsed = strtol(options->device, &end, 10);
        if (!end || *end || parsed < 0 || parsed > 1023)
            return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.open",
                                    "device must be a device ordinal");
        device = (int)parsed;
    }
    host_only = yvex_rocm_seam("YVEX_TEST_ROCM_NO_DEVICE");
    if (!host_only && device >= yvex_hip_device_count())
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.open",
                                "no rocm device is available: device-unavailable");
    backend = (yvex_rocm_backend *)calloc(1, sizeof(*backend));
    if (!backend) return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, "backend.open", "out of host memory");
    backend->kind = YVEX_BACKEND_KIND_ROCM;
    backend->owner_id = __atomic_fetch_add(&next_owner_id, 1ull, __ATOMIC_RELAXED);   /* sessions may be opened from several threads */
    backend->public_owner = backend;
    backend->device_index = device;
    backend->host_only = host_only;
    backend->memory.memory_limit_bytes = options->memory_limit_bytes;
    if (!host_only) {
        void *status_word = NULL;
        char name[64], arch[64];
        uint64_t total = 0, free_bytes = 0;
        int units = 0;
        if (yvex_hip_device_info(device, name, sizeof(name), arch, sizeof(arch), &total,
                                 &free_bytes, &units) != 0 ||
            yvex_hip_stream_create(&backend->stream) != 0 ||
            yvex_hip_malloc(&status_word, 256u) != 0) {
            if (backend->stream) yvex_hip_stream_destroy(backend->stream);
            free(backend);
            return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.open", yvex_hip_last_error());
        }
        backend->device_status = (int *)status_word;
        backend->kernels_available = !yvex_rocm_seam("YVEX_TEST_ROCM_BUNDLE_FAILURE") &&
                                     strncmp(arch, "gfx950", 6) == 0 && yvex_hip_kernels_loadable();
        if (backend->kernels_available &&
            (yvex_hip_fill_u32(backend->device_status, 0u, 1u, backend->stream) != 0 ||
             yvex_hip_stream_sync(backend->stream) != 0))
            backend->kernels_available = 0;
    }
    backend->status = backend->kernels_available ? YVEX_BACKEND_STATUS_READY
                                                 : YVEX_BACKEND_STATUS_CONTEXT_READY;
    backend->resource_owner = backend;
    *out = backend;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

/* Session-local state that borrows one owning backend's device and resident arena
 * (yvex_backend_open_shared_cuda, src/backend/cuda/backend.c:1913-2000): a stream, a status word,
 * memory accounting under its own limit, tensors, a workspace and launch graphs of its own. The
 * owner's arena is attached to the child without another upload (yvex_rocm_backend_resident_attach).
 * The owner refuses to close while a child is open. One caller at a time per backend, as ever;
 * different backends of one owner may run from different threads. */
int yvex_rocm_backend_open_shared(yvex_rocm_backend **out, yvex_rocm_backend *context_owner,
                                  unsigned long long memory_limit_bytes, yvex_error *err)
{
    yvex_rocm_backend *backend;
    if (out) *out = NULL;
    if (!out || !context_owner || context_owner->kind != YVEX_BACKEND_KIND_ROCM ||
        context_owner->resource_owner != context_owner)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.shared.open",
                                "one owning rocm backend is required");
    if (context_owner->status == YVEX_BACKEND_STATUS_FAILED)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, "rocm.shared.open",
                                "owning rocm backend became unavailable");
    backend = (yvex_rocm_backend *)calloc(1, sizeof(*backend));
    if (!backend)
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, "rocm.shared.open", "shared rocm session allocation failed");
    backend->kind = YVEX_BACKEND_KIND_ROCM;
    backend->owner_id = __atomic_fetch_add(&next_owner_id, 1ull, __ATOMIC_RELAXED);   /* sessions may be opened from several threads */
    backend->public_owner = backend;
    backend->device_index = context_owner->device_index;
    backend->host_only = context_owner->host_only;
    backend->memory.memory_limit_bytes = memory_limit_bytes;
    if (!backend->host_only) {
        void *status_word = NULL;
        if (yvex_hip_stream_create(&backend->stream) != 0 || yvex_hip_malloc(&status_word, 256u) != 0) {
            if (backend->stream) yvex_hip_stream_destroy(backend->stream);
            free(backend);
            return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.shared.open", yvex_hip_last_error());
        }
        backend->device_status = (int *)status_word;
        backend->kernels_available = context_owner->kernels_available;
        if (backend->kernels_available &&
            (yvex_hip_fill_u32(backend->device_status, 0u, 1u, backend->stream) != 0 ||
             yvex_hip_stream_sync(backend->stream) != 0))
            backend->kernels_available = 0;
    }
    backend->status = backend->kernels_available ? YVEX_BACKEND_STATUS_READY
                                                 : YVEX_BACKEND_STATUS_CONTEXT_READY;
    backend->resource_owner = context_owner;
    __atomic_add_fetch(&context_owner->shared_children, 1ull, __ATOMIC_ACQ_REL);
    *out = backend;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_close_checked(yvex_rocm_backend **backend_ref, yvex_error *err)
{
    yvex_rocm_backend *backend = backend_ref ? *backend_ref : NULL;
    if (!backend_ref)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.close", "owner is required");
    if (!backend) {
        yvex_rocm_error_clear(err);
        return YVEX_OK;
    }
    if (backend->live_tensors)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, "backend.close",
                                "backend still owns live tensors");
    if (__atomic_load_n(&backend->shared_children, __ATOMIC_ACQUIRE))
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, "backend.close",
                                "backend still serves shared sessions");
    if (yvex_rocm_seam("YVEX_TEST_ROCM_CLEANUP_FAILURE")) {
        backend->status = YVEX_BACKEND_STATUS_FAILED;   /* owner kept for a checked retry */
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.close",
                                "resource discharge failed (test seam)");
    }
    if (!backend->host_only) {
        if (yvex_hip_stream_sync(backend->stream) == 0) yvex_rocm_moe_graphs_release(backend);
        if (yvex_hip_stream_sync(backend->stream) == 0 && yvex_hip_host_free(backend->token_staging) == 0) {
            backend->token_staging = NULL;
            backend->token_staging_bytes = 0ull;
        }
        if (yvex_hip_stream_sync(backend->stream) != 0 || backend->token_staging ||
            yvex_hip_free(backend->device_status) != 0 ||
            yvex_hip_stream_destroy(backend->stream) != 0) {
            backend->status = YVEX_BACKEND_STATUS_FAILED;
            return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.close", yvex_hip_last_error());
        }
    }
    if (backend->resource_owner && backend->resource_owner != backend)
        __atomic_sub_fetch(&backend->resource_owner->shared_children, 1ull, __ATOMIC_ACQ_REL);
    free(backend);
    *backend_ref = NULL;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_bind_owner(yvex_rocm_backend *backend, const void *owner, yvex_error *err)
{
    if (!backend || !owner)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.bind", "backend and owner are required");
    if (backend->live_tensors)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, "backend.bind",
                                "the owner is bound before the first tensor is allocated");
    backend->public_owner = owner;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

yvex_backend_kind yvex_rocm_backend_kind_of(const yvex_rocm_backend *backend)
{
    return backend ? backend->kind : YVEX_BACKEND_KIND_CPU;
}

yvex_backend_status yvex_rocm_backend_status_of(const yvex_rocm_backend *backend)
{
    return backend ? backend->status : YVEX_BACKEND_STATUS_FAILED;
}

int yvex_rocm_backend_get_memory_stats(const yvex_rocm_backend *backend, yvex_backend_memory_stats *out,
                                  yvex_error *err)
{
    if (!backend || !out)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.memory", "owner and output required");
    *out = backend->memory;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

static unsigned long long median_of_five(const unsigned long long *values)
{
    unsigned long long v[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned int i, j;
    memcpy(v, values, sizeof(v));
    for (i = 1u; i < YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT; ++i) {
        unsigned long long x = v[i];
        for (j = i; j && v[j - 1u] > x; --j) v[j] = v[j - 1u];
        v[j] = x;
    }
    return v[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT / 2u];
}

/* src/backend/cuda/backend.c:1386-1640 (cuda_bandwidth_probe) */
int yvex_rocm_backend_bandwidth_probe(yvex_rocm_backend *backend, yvex_backend_bandwidth_evidence *out,
                                      yvex_error *err)
{
    const unsigned long long working_set = 1ull << 30, iterations = 4ull;
    void *source = NULL, *destination = NULL;
    unsigned int sample;
    int rc;
    if (out) memset(out, 0, sizeof(*out));
    if (!backend || !out || backend->kind != YVEX_BACKEND_KIND_ROCM)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.bandwidth", "backend and output are required");
    rc = yvex_rocm_require_kernels(backend, "rocm.bandwidth", err);
    if (rc != YVEX_OK) return rc;
    if (backend->pending_completion)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, "rocm.bandwidth",
                                "a deferred operation is pending on the backend stream");
    if (yvex_hip_malloc(&source, working_set) != 0 || yvex_hip_malloc(&destination, working_set) != 0) {
        (void)yvex_hip_free(source);
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, "rocm.bandwidth", yvex_hip_last_error());
    }
    rc = yvex_rocm_launch_result(yvex_hip_fill_u32(source, 0x5a5a5a5au, working_set / 4ull, backend->stream),
                                 "rocm.bandwidth.fill", err);
    out->schema_version = YVEX_BACKEND_BANDWIDTH_SCHEMA_V1;
    out->working_set_bytes = working_set;
    out->iterations = iterations;
    out->sample_count = YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT;
    /* one untimed pass of each kind first */
    if (rc == YVEX_OK) {
        uint64_t ignored = 0u;
        rc = yvex_rocm_launch_result(yvex_hip_bandwidth_sample(source, NULL, working_set, 1ull,
                                                               (uint32_t *)destination, &ignored,
                                                               backend->stream), "rocm.bandwidth.warmup", err);
        if (rc == YVEX_OK)
            rc = yvex_rocm_launch_result(yvex_hip_bandwidth_sample(source, destination, working_set, 1ull, NULL,
                                                                   &ignored, backend->stream),
                                         "rocm.bandwidth.warmup.copy", err);
    }
    for (sample = 0u; rc == YVEX_OK && sample < YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT; ++sample) {
        uint64_t elapsed = 0u;       /* the read kernel's sink is a word of the copy target */
        rc = yvex_rocm_launch_result(yvex_hip_bandwidth_sample(source, NULL, working_set, iterations,
                                                               (uint32_t *)destination, &elapsed,
                                                               backend->stream), "rocm.bandwidth.stream", err);
        out->stream_elapsed_ns[sample] = elapsed;
    }
    for (sample = 0u; rc == YVEX_OK && sample < YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT; ++sample) {
        uint64_t elapsed = 0u;
        rc = yvex_rocm_launch_result(yvex_hip_bandwidth_sample(source, destination, working_set, iterations, NULL,
                                                               &elapsed, backend->stream),
                                     "rocm.bandwidth.copy", err);
        out->copy_elapsed_ns[sample] = elapsed;
    }
    if (rc == YVEX_OK) {
        unsigned long long read_ns = median_of_five(out->stream_elapsed_ns);
        unsigned long long copy_ns = median_of_five(out->copy_elapsed_ns);
        if (!read_ns || !copy_ns)
            rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.bandwidth", "a timed sample took no time");
        else {
            out->sustainable_read_bytes_per_second =
                (unsigned long long)((double)working_set * (double)iterations * 1.0e9 / (double)read_ns);
            out->sustainable_copy_bytes_per_second =
                (unsigned long long)((double)working_set * (double)iterations * 1.0e9 / (double)copy_ns);
        }
    }
    if (yvex_hip_stream_sync(backend->stream) != 0 && rc == YVEX_OK)
        rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.bandwidth.sync", yvex_hip_last_error());
    (void)yvex_hip_free(source);
    (void)yvex_hip_free(destination);
    if (rc != YVEX_OK) {
        memset(out, 0, sizeof(*out));
        return rc;
    }
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_sync(yvex_rocm_backend *backend, yvex_error *err)
{
    if (!backend) return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.sync", "owner is required");
    if (backend->host_only) {
        yvex_rocm_error_clear(err);
        return YVEX_OK;
    }
    if (yvex_rocm_seam("YVEX_TEST_ROCM_SYNC_FAILURE") || yvex_hip_stream_sync(backend->stream) != 0) {
        backend->status = YVEX_BACKEND_STATUS_FAILED;
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.sync", "stream synchronisation failed");
    }
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_query_capability(const yvex_rocm_backend *backend,
                                  yvex_backend_operation_variant variant,
                                  yvex_backend_capability_result *out, yvex_error *err)
{
    int tensor_variant;
    if (out) memset(out, 0, sizeof(*out));
    if (!backend || !out || (int)variant < 0 || variant >= YVEX_BACKEND_VARIANT_COUNT)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.capability",
                                "owner, variant and output are required");
    tensor_variant = variant <= YVEX_BACKEND_VARIANT_TENSOR_COPY;
    out->backend_kind = backend->kind;
    out->variant = variant;
    out->input_dtype = out->output_dtype = YVEX_DTYPE_F32;
    out->weight_dtype = YVEX_DTYPE_UNKNOWN;
    out->context_available = backend->status != YVEX_BACKEND_STATUS_FAILED;
    out->kernel_bundle_available = backend->kernels_available;
    if (backend->status == YVEX_BACKEND_STATUS_FAILED) {
        out->state = YVEX_BACKEND_CAPABILITY_FAILED;
        out->reason = YVEX_BACKEND_CAPABILITY_REASON_CONTEXT_UNAVAILABLE;
    } else if (tensor_variant) {
        out->state = YVEX_BACKEND_CAPABILITY_SUPPORTED;
        out->function_available = 1;
    } else if (variant != YVEX_BACKEND_VARIANT_QTYPE_ROW_DOT &&
               variant != YVEX_BACKEND_VARIANT_ATTENTION_ENCODED) {
        out->state = YVEX_BACKEND_CAPABILITY_UNSUPPORTED;   /* other operators are not on this path */
        out->reason = YVEX_BACKEND_CAPABILITY_REASON_VARIANT_UNSUPPORTED;
    } else if (!backend->kernels_available) {
        out->state = YVEX_BACKEND_CAPABILITY_UNSUPPORTED;
        out->reason = YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT;
    } else {
        out->state = YVEX_BACKEND_CAPABILITY_SUPPORTED;
        out->function_available = 1;
    }
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

/* ---- tensors -------------------------------------------------------------------------------- */

static int memory_can_add(const yvex_rocm_backend *backend, unsigned long long bytes)
{
    const yvex_backend_memory_stats *m = &backend->memory;
    if (bytes > ULLONG_MAX - m->allocated_bytes) return 0;
    return !m->memory_limit_bytes || m->allocated_bytes + bytes <= m->memory_limit_bytes;
}

static int tensor_create(yvex_rocm_backend *backend, const yvex_backend_tensor_desc *desc, int resident,
                         yvex_device_tensor **out, const char *where, yvex_error *err)
{
    yvex_device_tensor *tensor;
    void *device = NULL, *host = NULL;
    unsigned int i;
    if (out) *out = NULL;
    if (!backend || !desc || !out || !desc->bytes || desc->rank > YVEX_TENSOR_MAX_DIMS)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, where, "owner and tensor geometry are required");
    if (backend->status == YVEX_BACKEND_STATUS_FAILED)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, where, "backend is failed or closing");
    if (!memory_can_add(backend, desc->bytes))
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where, "allocation exceeds the backend memory limit");
    tensor = (yvex_device_tensor *)calloc(1, sizeof(*tensor));
    if (!tensor) return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where, "out of host memory");
    if (backend->host_only) {
        device = calloc(1, (size_t)desc->bytes);
        if (device && resident) host = device;   /* unified in the no-device seam */
    } else {
        if (yvex_hip_malloc(&device, desc->bytes) != 0) device = NULL;
        if (device && resident && yvex_hip_host_alloc(&host, desc->bytes) != 0) {
            yvex_hip_free(device);
            device = NULL;
        }
    }
    if (!device) {
        free(tensor);
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where, "device allocation failed");
    }
    tensor->owner = (yvex_rocm_backend *)backend->public_owner;
    tensor->owner_id = backend->owner_id;
    if (desc->name) {
        size_t n = strlen(desc->name) + 1u;
        tensor->name = (char *)malloc(n);
        if (tensor->name) memcpy(tensor->name, desc->name, n);
    }
    tensor->dtype = desc->dtype;
    tensor->rank = desc->rank;
    for (i = 0; i < desc->rank; ++i) tensor->dims[i] = desc->dims[i];
    tensor->bytes = desc->bytes;
    tensor->data = (unsigned char *)device;
    tensor->host_data = (unsigned char *)host;
    tensor->backend_allocation = device;
    tensor->resident_bytes = resident ? desc->bytes : 0ull;
    tensor->host_accessible = host != NULL;
    backend->memory.allocated_bytes += desc->bytes;
    backend->memory.allocation_count++;
    backend->memory.allocation_events++;
    if (backend->memory.allocated_bytes > backend->memory.peak_allocated_bytes)
        backend->memory.peak_allocated_bytes = backend->memory.allocated_bytes;
    backend->live_tensors++;
    *out = tensor;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_tensor_alloc(yvex_rocm_backend *backend, const yvex_backend_tensor_desc *desc,
                              yvex_device_tensor **out, yvex_error *err)
{
    return tensor_create(backend, desc, 0, out, "backend.tensor.alloc", err);
}

int yvex_rocm_backend_tensor_release(yvex_rocm_backend *backend, yvex_device_tensor **tensor_ref,
                                yvex_error *err)
{
    yvex_device_tensor *tensor = tensor_ref ? *tensor_ref : NULL;
    if (!backend || !tensor_ref)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.tensor.release", "owner is required");
    if (!tensor) {
        yvex_rocm_error_clear(err);
        return YVEX_OK;
    }
    if (!yvex_rocm_tensor_owner_is(backend, tensor))
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "backend.tensor.release",
                                "tensor belongs to another backend");
    if (yvex_rocm_seam("YVEX_TEST_ROCM_CLEANUP_FAILURE"))
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.tensor.release",
                                "release failed (test seam); the owner keeps the tensor");
    if (backend->resident_device_tensor == tensor) yvex_rocm_backend_resident_detach(backend, NULL);
    if (backend->workspace_device_tensor == tensor) yvex_rocm_backend_workspace_detach(backend);
    if (backend->host_only) {
        free(tensor->backend_allocation);
    } else {
        if (yvex_hip_stream_sync(backend->stream) != 0 || yvex_hip_free(tensor->backend_allocation) != 0)
            return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.tensor.release", yvex_hip_last_error());
        if (tensor->host_data) yvex_hip_host_free(tensor->host_data);
    }
    backend->memory.allocated_bytes -= tensor->bytes;
    backend->memory.allocation_count--;
    backend->memory.release_events++;
    backend->live_tensors--;
    free(tensor->name);
    free(tensor);
    *tensor_ref = NULL;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

static int rw_validate(const char *where, const yvex_rocm_backend *backend, const yvex_device_tensor *tensor,
                       const void *host, unsigned long long len, yvex_error *err)
{
    if (!backend || !tensor || !host)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, where, "owner, tensor and host buffer are required");
    if (backend->status == YVEX_BACKEND_STATUS_FAILED)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, where, "backend is failed or closing");
    if (!yvex_rocm_tensor_owner_is(backend, tensor))
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where, "tensor belongs to another backend");
    if (!len || len > tensor->bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "transfer length exceeds the tensor");
    return YVEX_OK;
}

int yvex_rocm_backend_tensor_write(yvex_rocm_backend *backend, yvex_device_tensor *tensor, const void *src,
                              unsigned long long len, yvex_error *err)
{
    int rc = rw_validate("backend.tensor.write", backend, tensor, src, len, err);
    if (rc != YVEX_OK) return rc;
    if (backend->host_only) memcpy(tensor->data, src, (size_t)len);
    else if (yvex_hip_memcpy_h2d(tensor->data, src, len, backend->stream) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.tensor.write", yvex_hip_last_error());
    backend->memory.h2d_bytes += len;
    tensor->is_written = 1;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_tensor_read(yvex_rocm_backend *backend, const yvex_device_tensor *tensor, void *dst,
                             unsigned long long len, yvex_error *err)
{
    int rc = rw_validate("backend.tensor.read", backend, tensor, dst, len, err);
    if (rc != YVEX_OK) return rc;
    if (!tensor->is_written)
        return yvex_rocm_refuse(err, YVEX_ERR_STATE, "backend.tensor.read", "tensor was never written");
    if (backend->host_only) memcpy(dst, tensor->data, (size_t)len);
    else if (yvex_hip_memcpy_d2h(dst, tensor->data, len, backend->stream) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.tensor.read", yvex_hip_last_error());
    backend->memory.d2h_bytes += len;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_tensor_copy(yvex_rocm_backend *backend, yvex_device_tensor *dst,
                             const yvex_device_tensor *src, yvex_error *err)
{
    if (!backend || !dst || !src)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.tensor.copy", "owner and tensors are required");
    if (!yvex_rocm_tensor_owner_is(backend, dst) || !yvex_rocm_tensor_owner_is(backend, src) ||
        !src->is_written || dst->bytes != src->bytes || dst == src)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, "backend.tensor.copy",
                                "copy needs two distinct written tensors of equal size and one owner");
    if (backend->host_only) memcpy(dst->data, src->data, (size_t)src->bytes);
    else if (yvex_hip_memcpy_d2d(dst->data, src->data, src->bytes, backend->stream) != 0 ||
             yvex_hip_stream_sync(backend->stream) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "backend.tensor.copy", yvex_hip_last_error());
    dst->is_written = 1;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

/* ---- resident arena -------------------------------------------------------------------------- */

int yvex_rocm_backend_resident_alloc(yvex_rocm_backend *backend, const yvex_backend_tensor_desc *desc,
                                yvex_device_tensor **out, unsigned char **host, yvex_error *err)
{
    int rc;
    if (host) *host = NULL;
    if (!host) return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.resident.alloc", "host output is required");
    rc = tensor_create(backend, desc, 1, out, "backend.resident.alloc", err);
    if (rc == YVEX_OK) *host = (*out)->host_data;
    return rc;
}

static int resident_upload(yvex_rocm_backend *backend, const yvex_device_tensor *tensor,
                           unsigned long long offset, unsigned long long bytes, const char *where,
                           yvex_error *err)
{
    if (backend->host_only || !bytes) return YVEX_OK;   /* the seam's shadow is the storage */
    if (yvex_hip_memcpy_h2d(tensor->data + offset, tensor->host_data + offset, bytes, backend->stream) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
    backend->memory.h2d_bytes += bytes;
    return YVEX_OK;
}

int yvex_rocm_backend_resident_prefetch(yvex_rocm_backend *backend, yvex_device_tensor *tensor,
                                   unsigned long long *prefetched_bytes, yvex_error *err)
{
    int rc;
    if (prefetched_bytes) *prefetched_bytes = 0ull;
    if (!backend || !tensor || !prefetched_bytes || !yvex_rocm_tensor_owner_is(backend, tensor) ||
        !tensor->host_data || !tensor->resident_bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.resident.prefetch",
                                "a backend-owned resident tensor is required");
    rc = resident_upload(backend, tensor, 0ull, tensor->resident_bytes, "backend.resident.prefetch", err);
    if (rc != YVEX_OK) return rc;
    tensor->is_written = 1;
    *prefetched_bytes = tensor->resident_bytes;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_resident_attach(yvex_rocm_backend *backend, const unsigned char *host_base,
                                 unsigned long long bytes, const yvex_device_tensor *tensor,
                                 unsigned long long generation, yvex_error *err)
{
    unsigned long long offset;
    int rc;
    if (backend && backend->resource_owner && backend->resource_owner != backend && host_base && bytes &&
        tensor && generation && yvex_rocm_tensor_owner_is(backend->resource_owner, tensor)) {
        /* a shared session attaches the arena its owner has published (src/backend/residency.c:47-57:
         * same base, same generation, the owner's device address): nothing is uploaded again */
        const yvex_rocm_backend *owner = backend->resource_owner;
        if (backend->resident_host_base)
            return yvex_rocm_refuse(err, YVEX_ERR_STATE, "backend.resident.attach",
                                    "backend residency mapping is already attached");
        if (owner->resident_host_base != host_base || owner->resident_host_bytes < bytes ||
            owner->resident_generation != generation || !owner->resident_device_address)
            return yvex_rocm_refuse(err, YVEX_ERR_STATE, "backend.resident.attach",
                                    "the owning backend has no matching resident arena attached");
        backend->resident_host_base = host_base;
        backend->resident_host_bytes = bytes;
        backend->resident_device_tensor = tensor;
        backend->resident_device_address = owner->resident_device_address;
        backend->resident_generation = generation;
        yvex_rocm_error_clear(err);
        return YVEX_OK;
    }
    if (!backend || !host_base || !bytes || !tensor || !generation ||
        !yvex_rocm_tensor_owner_is(backend, tensor) || !tensor->host_data ||
        host_base < tensor->host_data)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.resident.attach",
                                "a backend-owned resident tensor and a range inside its host shadow are required");
    offset = (unsigned long long)(host_base - tensor->host_data);
    if (offset > tensor->bytes || bytes > tensor->bytes - offset)
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, "backend.resident.attach",
                                "resident range leaves the tensor");
    /* publication point: the shadow range becomes visible to the device here */
    rc = resident_upload(backend, tensor, offset, bytes, "backend.resident.attach", err);
    if (rc != YVEX_OK) return rc;
    ((yvex_device_tensor *)tensor)->is_written = 1;
    backend->resident_host_base = host_base;
    backend->resident_host_bytes = bytes;
    backend->resident_device_tensor = tensor;
    backend->resident_device_address = (unsigned long long)(uintptr_t)(tensor->data + offset);
    backend->resident_generation = generation;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_resident_detach(yvex_rocm_backend *backend, yvex_error *err)
{
    if (backend) {
        backend->resident_host_base = NULL;
        backend->resident_host_bytes = 0ull;
        backend->resident_device_tensor = NULL;
        backend->resident_device_address = 0ull;
        backend->resident_generation = 0ull;
    }
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_backend_resident_resolve(const yvex_rocm_backend *backend, const unsigned char *host,
                                  unsigned long long bytes, unsigned long long *device_address)
{
    uintptr_t base, pointer;
    unsigned long long offset;
    if (device_address) *device_address = 0ull;
    if (!backend || backend->status == YVEX_BACKEND_STATUS_FAILED || !host || !bytes ||
        !device_address || !backend->resident_host_base)
        return YVEX_BACKEND_RESIDENT_MISS;
    base = (uintptr_t)backend->resident_host_base;
    pointer = (uintptr_t)host;
    if (pointer < base) return YVEX_BACKEND_RESIDENT_MISS;
    offset = (unsigned long long)(pointer - base);
    if (offset > backend->resident_host_bytes || bytes > backend->resident_host_bytes - offset)
        return YVEX_BACKEND_RESIDENT_MISS;
    if (backend->resident_device_address > ULLONG_MAX - offset) return YVEX_BACKEND_RESIDENT_INVALID;
    *device_address = backend->resident_device_address + offset;
    return YVEX_BACKEND_RESIDENT_HIT;
}

int yvex_rocm_resolve(const yvex_rocm_backend *backend, const unsigned char *host,
                      unsigned long long bytes, unsigned long long *device_address)
{
    return yvex_rocm_backend_resident_resolve(backend, host, bytes, device_address) ==
           YVEX_BACKEND_RESIDENT_HIT;
}

/* ---- workspace -------------------------------------------------------------------------------- */

int yvex_rocm_backend_workspace_attach(yvex_rocm_backend *backend, const yvex_device_tensor *tensor,
                                  unsigned long long bytes, yvex_error *err)
{
    if (!backend || !tensor || !bytes || !yvex_rocm_tensor_owner_is(backend, tensor) ||
        bytes > tensor->bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "backend.workspace.attach",
                                "a backend-owned tensor at least as large as the workspace is required");
    backend->workspace_device_tensor = tensor;
    backend->workspace_bytes = bytes;
    backend->workspace_cursor = 0ull;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

void yvex_rocm_backend_workspace_detach(yvex_rocm_backend *backend)
{
    if (!backend) return;
    backend->workspace_device_tensor = NULL;
    backend->workspace_bytes = backend->workspace_cursor = 0ull;
}

int yvex_rocm_backend_workspace_acquire(yvex_rocm_backend *backend, unsigned long long bytes,
                                   unsigned long long alignment, unsigned long long *device_address)
{
    unsigned long long base, start;
    if (device_address) *device_address = 0ull;
    if (!backend || !device_address || !bytes || !backend->workspace_device_tensor || !alignment ||
        (alignment & (alignment - 1ull)))
        return 0;
    base = (unsigned long long)(uintptr_t)backend->workspace_device_tensor->data;
    start = (base + backend->workspace_cursor + alignment - 1ull) & ~(alignment - 1ull);
    if (start - base > backend->workspace_bytes || bytes > backend->workspace_bytes - (start - base))
        return 0;
    backend->workspace_cursor = start - base + bytes;
    *device_address = start;
    return 1;
}
