/*
 * Greedy row selection on the ROCm backend: the largest logit of each row, the lowest token that
 * holds it and the number of tokens that hold it, selected on the device so that only 16 bytes
 * per row cross to the host instead of the logits row (517 KB for a 129 280-token vocabulary).
 * Host side only: validation, workspace, launch, completion, downloads, facts.
 * Restates sampling_cuda_select_greedy_rows (src/backend/cuda/sampling.c:284-392), the
 * select_greedy_rows entry of yvex_backend_sampling_operations
 * (include/yvex/internal/sampling.h:129-137).
 */
#include <limits.h>
#include <math.h>
#include <string.h>

#include "private.h"

static int mul_u64(unsigned long long a, unsigned long long b, unsigned long long *out)
{
    if (a && b > ULLONG_MAX / a) return 0;
    *out = a * b;
    return 1;
}

int yvex_rocm_select_greedy_rows(
    yvex_rocm_backend *backend, const yvex_device_tensor *logits, unsigned long long row_count,
    unsigned long long row_width, unsigned int *selected_tokens, float *selected_values,
    unsigned long long *tie_counts, yvex_rocm_operation_facts *facts, yvex_error *err)
{
    const char *where = "rocm.sampling.greedy";
    unsigned long long value_count, value_bytes, token_bytes, selected_bytes, tie_bytes;
    unsigned long long temporary_bytes, tokens_device = 0ull, values_device = 0ull, ties_device = 0ull, row;
    unsigned long long scratch_bytes, scratch_device = 0ull;
    int device_status = 0, rc;
    if (facts) memset(facts, 0, sizeof(*facts));
    if (!backend || backend->kind != YVEX_BACKEND_KIND_ROCM || !logits || !selected_tokens ||
        !selected_values || !tie_counts || !facts || !row_count || !row_width ||
        row_count > UINT_MAX || row_width > UINT_MAX ||
        !mul_u64(row_count, row_width, &value_count) ||
        !mul_u64(value_count, sizeof(float), &value_bytes) ||
        !mul_u64(row_count, sizeof(*selected_tokens), &token_bytes) ||
        !mul_u64(row_count, sizeof(*selected_values), &selected_bytes) ||
        !mul_u64(row_count, sizeof(*tie_counts), &tie_bytes) ||
        !yvex_rocm_tensor_owner_is(backend, logits) || logits->dtype != YVEX_DTYPE_F32 ||
        !logits->is_written || logits->bytes < value_bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where,
                                "greedy row selection geometry or ownership is incompatible");
    temporary_bytes = token_bytes + selected_bytes + tie_bytes + sizeof(int);
    memset(selected_tokens, 0, (size_t)token_bytes);
    memset(selected_values, 0, (size_t)selected_bytes);
    memset(tie_counts, 0, (size_t)tie_bytes);
    rc = yvex_rocm_require_kernels(backend, where, err);
    if (rc != YVEX_OK) return rc;
    yvex_rocm_workspace_reset(backend);
    if (!yvex_rocm_backend_workspace_acquire(backend, tie_bytes, 256ull, &ties_device) ||
        !yvex_rocm_backend_workspace_acquire(backend, token_bytes, 256ull, &tokens_device) ||
        !yvex_rocm_backend_workspace_acquire(backend, selected_bytes, 256ull, &values_device))
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where,
                                "greedy row selection needs an attached workspace for its results");
    /* long rows are shared among the compute units when the workspace has room for the partial
     * results; otherwise one workgroup scans a row */
    scratch_bytes = yvex_hip_argmax_scratch_bytes(row_count, row_width);
    if (scratch_bytes && !yvex_rocm_backend_workspace_acquire(backend, scratch_bytes, 256ull, &scratch_device))
        scratch_bytes = 0ull, scratch_device = 0ull;
    if (yvex_rocm_seam("YVEX_TEST_ROCM_LAUNCH_FAILURE"))
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.sampling.greedy.launch",
                                "kernel launch failed (test seam)");
    rc = yvex_rocm_status_reset(backend, where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_launch_result(
            yvex_hip_argmax_f32((const float *)logits->data, row_count, row_width,
                                (uint32_t *)(uintptr_t)tokens_device, (float *)(uintptr_t)values_device,
                                (uint64_t *)(uintptr_t)ties_device, (void *)(uintptr_t)scratch_device,
                                scratch_bytes, backend->device_status, backend->stream),
            "rocm.sampling.greedy.launch", err);
#define READ(target_, source_, bytes_)                                                         \
    if (rc == YVEX_OK &&                                                                       \
        yvex_hip_memcpy_d2h((target_), (const void *)(uintptr_t)(source_), (bytes_), backend->stream) != 0) \
        rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error())
    READ(selected_tokens, tokens_device, token_bytes);
    READ(selected_values, values_device, selected_bytes);
    READ(tie_counts, ties_device, tie_bytes);
#undef READ
    if (rc == YVEX_OK) rc = yvex_rocm_finish(backend, "rocm.sampling.greedy.sync", &device_status, err);
    for (row = 0ull; rc == YVEX_OK && row < row_count; ++row)
        if (device_status || selected_tokens[row] >= row_width || !isfinite(selected_values[row]) ||
            !tie_counts[row])
            rc = yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where,
                                  "greedy row selection produced invalid bounded facts");
    if (rc != YVEX_OK) {
        memset(selected_tokens, 0, (size_t)token_bytes);
        memset(selected_values, 0, (size_t)selected_bytes);
        memset(tie_counts, 0, (size_t)tie_bytes);
        return rc;
    }
    facts->d2h_bytes = temporary_bytes;
    facts->kernel_launches = scratch_bytes ? 2ull : 1ull;
    facts->download_count = 4ull;
    facts->stream_synchronizations = 1ull;
    facts->activation_bytes = value_bytes;
    facts->temporary_bytes = temporary_bytes;
    facts->compulsory_memory_facts_available = 1;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}
