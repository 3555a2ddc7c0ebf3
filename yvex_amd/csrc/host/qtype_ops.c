/*
 * Encoded matvec (dense projection / output head) and encoded gather on the ROCm backend.
 * Host side only: validation, fail-closed admission, workspace, launch, completion, facts.
 * Restates src/backend/cuda/qtype.c:220-405 (matvec) and :411-521 (gather).
 */
#include <limits.h>
#include <string.h>

#include "private.h"

static int mul_u64(unsigned long long a, unsigned long long b, unsigned long long *out)
{
    if (a && b > ULLONG_MAX / a) return 0;
    *out = a * b;
    return 1;
}

/* Fail-closed admission: the qtype must have a row with device compute, and the row geometry
 * must be exact. Runs on the host so a refused qtype never reaches a kernel. */
static int qtype_admit(unsigned int qtype, unsigned long long row_width, unsigned long long row_bytes,
                       const char *where, yvex_error *err)
{
    const yvex_rocm_numeric_capability *capability = yvex_rocm_quant_numeric_capability_at(qtype);
    const yvex_rocm_qtype_geometry *geometry = yvex_rocm_gguf_qtype_geometry_find(qtype);
    unsigned long long expected;
    if (!capability || !geometry || !capability->device_compute_available)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, where,
                                "qtype has no device compute on this backend");
    if (!geometry->block_size || row_width % geometry->block_size ||
        !mul_u64(row_width / geometry->block_size, geometry->bytes_per_block, &expected) ||
        expected != row_bytes)
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where,
                                "row width is not block divisible or the row byte count is inconsistent");
    return YVEX_OK;
}

static int q8_eligible(unsigned int qtype)
{
    return qtype == YVEX_GGUF_QTYPE_Q8_0 || qtype == YVEX_GGUF_QTYPE_Q2_K ||
           qtype == YVEX_GGUF_QTYPE_Q4_K || qtype == YVEX_GGUF_QTYPE_IQ2_XXS;
}

int yvex_rocm_encoded_matvec(
    yvex_rocm_backend *backend, const unsigned char *resident_encoded,
    unsigned long long encoded_bytes, unsigned int qtype, unsigned long long row_count,
    unsigned long long row_width, unsigned long long row_bytes, unsigned long long input_rows,
    const yvex_device_tensor *input, const yvex_device_tensor *input_tail,
    unsigned long long input_head_width, const yvex_device_tensor *additive,
    yvex_device_tensor *output, int activation_q8, yvex_rocm_operation_facts *facts,
    yvex_error *err)
{
    const char *where = "rocm.encoded-matvec";
    unsigned long long device_address = 0ull, input_bytes, output_bytes, activation_bytes;
    unsigned long long total_bytes, q8_bytes = 0ull, q8_address = 0ull, launches = 0ull;
    unsigned long long head_bytes, tail_bytes = 0ull, joined_bytes = 0ull, joined_address = 0ull;
    const void *activations;
    int q8_path, device_status = 0, rc, split_input = input_tail != NULL;
    if (facts) memset(facts, 0, sizeof(*facts));
    if (activation_q8 != 0 && activation_q8 != 1)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, "rocm.encoded-matvec.activation",
                                "activation Q8 policy must be explicitly disabled or enabled");
    /* split input (speculation): row = head[0..input_head_width) ++ tail, qtype.c:256-281 */
    if (!backend || backend->kind != YVEX_BACKEND_KIND_ROCM || !resident_encoded || !encoded_bytes ||
        !row_count || !input_rows || !row_width || !row_bytes || !facts || !input || !output ||
        split_input != (input_head_width != 0ull) || (split_input && input_head_width >= row_width))
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where,
                                "resident encoded matvec geometry or ownership is incompatible");
    rc = qtype_admit(qtype, row_width, row_bytes, where, err);
    if (rc != YVEX_OK) return rc;
    if (!mul_u64(input_rows, split_input ? input_head_width : row_width, &head_bytes) ||
        !mul_u64(head_bytes, sizeof(float), &head_bytes) ||
        (split_input && (!mul_u64(input_rows, row_width - input_head_width, &tail_bytes) ||
                         !mul_u64(tail_bytes, sizeof(float), &tail_bytes))) ||
        !mul_u64(input_rows, row_width, &input_bytes) || !mul_u64(input_bytes, sizeof(float), &input_bytes) ||
        !mul_u64(input_rows, row_count, &output_bytes) ||
        !mul_u64(output_bytes, sizeof(float), &output_bytes) ||
        !mul_u64(row_count, row_bytes, &total_bytes) || total_bytes != encoded_bytes ||
        !yvex_rocm_tensor_owner_is(backend, input) || !input->is_written ||
        input->dtype != YVEX_DTYPE_F32 || input->bytes < head_bytes ||
        (split_input && (!yvex_rocm_tensor_owner_is(backend, input_tail) || !input_tail->is_written ||
                         input_tail->dtype != YVEX_DTYPE_F32 || input_tail->bytes < tail_bytes ||
                         input_tail == output)) ||
        !yvex_rocm_tensor_owner_is(backend, output) || output->dtype != YVEX_DTYPE_F32 ||
        output->bytes < output_bytes || output == input ||
        (additive && (!yvex_rocm_tensor_owner_is(backend, additive) ||
                      additive->dtype != YVEX_DTYPE_F32 || !additive->is_written ||
                      additive->bytes < output_bytes || additive == output)) ||
        !yvex_rocm_resolve(backend, resident_encoded, encoded_bytes, &device_address))
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where,
                                "resident encoded matvec geometry or ownership is incompatible");
    activation_bytes = input_bytes + output_bytes + (additive ? output_bytes : 0ull);
    q8_path = activation_q8 && !split_input && row_width % 256ull == 0ull && q8_eligible(qtype);
    output->is_written = 0;
    rc = yvex_rocm_require_kernels(backend, where, err);
    if (rc != YVEX_OK) return rc;
    yvex_rocm_workspace_reset(backend);
    if (q8_path) {
        if (!mul_u64(input_rows * (row_width / 256ull), 292ull, &q8_bytes))
            return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "Q8 activation workspace exceeds bounds");
        if (!yvex_rocm_backend_workspace_acquire(backend, q8_bytes, 256ull, &q8_address))
            return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where,
                                    "Q8 activation needs an attached workspace of rows * width/256 * 292 bytes");
    }
    if (split_input) {
        joined_bytes = input_bytes;
        if (!yvex_rocm_backend_workspace_acquire(backend, joined_bytes, 256ull, &joined_address))
            return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where,
                                    "a split input needs an attached workspace of rows * width * 4 bytes");
    }
    if (yvex_rocm_seam("YVEX_TEST_ROCM_LAUNCH_FAILURE"))
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.encoded-matvec.launch",
                                "kernel launch failed (test seam)");
    rc = yvex_rocm_status_reset(backend, where, err);
    activations = input->data;
    if (rc == YVEX_OK && split_input) {
        rc = yvex_rocm_launch_result(
            yvex_hip_concat_rows_bf16((const float *)input->data, (const float *)input_tail->data, input_rows,
                                      input_head_width, row_width - input_head_width,
                                      (float *)(uintptr_t)joined_address, backend->device_status,
                                      backend->stream), "rocm.encoded-matvec.split", err);
        if (rc == YVEX_OK) launches++;
        activations = (const void *)(uintptr_t)joined_address;
    }
    if (rc == YVEX_OK && q8_path) {
        rc = yvex_rocm_launch_result(
            yvex_hip_q8k_quantize((const float *)input->data, input_rows, row_width, row_width,
                                  (uint8_t *)(uintptr_t)q8_address, backend->device_status,
                                  backend->stream),
            "rocm.encoded-matvec.q8", err);
        if (rc == YVEX_OK) launches++;
    }
    if (rc == YVEX_OK) {
        rc = yvex_rocm_launch_result(
            yvex_hip_matvec((const uint8_t *)(uintptr_t)device_address, qtype, row_count, row_width,
                            row_bytes, q8_path ? (const void *)(uintptr_t)q8_address : activations,
                            q8_path, input_rows, row_width, additive ? (const float *)additive->data : NULL,
                            (float *)output->data, row_count, 0, backend->device_status, backend->stream),
            "rocm.encoded-matvec.launch", err);
        if (rc == YVEX_OK) launches++;
    }
    if (rc == YVEX_OK) rc = yvex_rocm_finish(backend, "rocm.encoded-matvec.sync", &device_status, err);
    if (rc == YVEX_OK && device_status)
        rc = yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where,
                              "encoded projection produced invalid numerics");
    if (rc != YVEX_OK) return rc;
    output->is_written = 1;
    facts->d2h_bytes = sizeof(int);
    facts->kernel_launches = launches + 1ull;   /* status reset included */
    facts->download_count = 1ull;
    facts->stream_synchronizations = 1ull;
    facts->active_weight_bytes = encoded_bytes;
    facts->activation_bytes = activation_bytes;
    facts->temporary_bytes = sizeof(int) + q8_bytes + joined_bytes;
    facts->compulsory_memory_facts_available = 1;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

int yvex_rocm_encoded_gather(
    yvex_rocm_backend *backend, const unsigned char *resident_encoded,
    unsigned long long encoded_bytes, unsigned int qtype, unsigned long long row_count,
    unsigned long long row_width, unsigned long long row_bytes, const unsigned int *row_ids,
    unsigned long long selected_rows, yvex_device_tensor *output,
    yvex_rocm_operation_facts *facts, yvex_error *err)
{
    const char *where = "rocm.encoded-gather";
    unsigned long long device_address = 0ull, output_bytes, total_bytes, ids_address = 0ull, i;
    int device_status = 0, rc;
    if (facts) memset(facts, 0, sizeof(*facts));
    if (!backend || backend->kind != YVEX_BACKEND_KIND_ROCM || !resident_encoded || !encoded_bytes ||
        !row_count || !row_width || !row_bytes || !row_ids || !selected_rows || !output || !facts)
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, where, "gather arguments are required");
    rc = qtype_admit(qtype, row_width, row_bytes, where, err);
    if (rc != YVEX_OK) return rc;
    for (i = 0; i < selected_rows; ++i)
        if (row_ids[i] >= row_count)
            return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "selected row is outside the matrix");
    if (!mul_u64(selected_rows, row_width, &output_bytes) ||
        !mul_u64(output_bytes, sizeof(float), &output_bytes) ||
        !mul_u64(row_count, row_bytes, &total_bytes) || total_bytes != encoded_bytes ||
        !yvex_rocm_tensor_owner_is(backend, output) || output->dtype != YVEX_DTYPE_F32 ||
        output->bytes < output_bytes ||
        !yvex_rocm_resolve(backend, resident_encoded, encoded_bytes, &device_address))
        return yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where,
                                "resident gather geometry or ownership is incompatible");
    output->is_written = 0;
    rc = yvex_rocm_require_kernels(backend, where, err);
    if (rc != YVEX_OK) return rc;
    yvex_rocm_workspace_reset(backend);
    if (!yvex_rocm_backend_workspace_acquire(backend, selected_rows * sizeof(unsigned int), 256ull, &ids_address))
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where,
                                "gather needs an attached workspace for the row identifiers");
    if (yvex_rocm_seam("YVEX_TEST_ROCM_LAUNCH_FAILURE"))
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, "rocm.encoded-gather.launch",
                                "kernel launch failed (test seam)");
    if (yvex_hip_memcpy_h2d((void *)(uintptr_t)ids_address, row_ids, selected_rows * sizeof(unsigned int),
                            backend->stream) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
    rc = yvex_rocm_status_reset(backend, where, err);
    if (rc == YVEX_OK)
        rc = yvex_rocm_launch_result(
            yvex_hip_gather((const uint8_t *)(uintptr_t)device_address, qtype, row_count, row_width,
                            row_bytes, (const uint32_t *)(uintptr_t)ids_address, selected_rows,
                            (float *)output->data, backend->device_status, backend->stream),
            "rocm.encoded-gather.launch", err);
    if (rc == YVEX_OK) rc = yvex_rocm_finish(backend, "rocm.encoded-gather.sync", &device_status, err);
    if (rc == YVEX_OK && device_status)
        rc = yvex_rocm_refuse(err, YVEX_ERR_FORMAT, where, "encoded gather produced invalid numerics");
    if (rc != YVEX_OK) return rc;
    output->is_written = 1;
    facts->h2d_bytes = selected_rows * sizeof(unsigned int);
    facts->d2h_bytes = sizeof(int);
    facts->kernel_launches = 2ull;
    facts->upload_count = facts->download_count = 1ull;
    facts->stream_synchronizations = 2ull;
    facts->active_weight_bytes = selected_rows * row_bytes;
    facts->activation_bytes = output_bytes;
    facts->temporary_bytes = sizeof(int) + selected_rows * sizeof(unsigned int);
    facts->compulsory_memory_facts_available = 1;
    yvex_rocm_error_clear(err);
    return YVEX_OK;
}

/* src/backend/cuda/qtype.c:523-700: one encoded row times one vector, host pointers in, one float
 * out, computed on the device by the serial double-precision probe kernel. The device
 * temporaries live for the call only. */
int yvex_rocm_quant_row_dot(yvex_rocm_backend *backend, unsigned int qtype, const unsigned char *encoded,
                            size_t encoded_bytes, const float *vector, unsigned long long elements,
                            float *out, void *failure, yvex_error *err)
{
    const char *where = "rocm.quant.row_dot";
    const yvex_rocm_numeric_capability *capability = yvex_rocm_quant_numeric_capability_at(qtype);
    const yvex_rocm_qtype_geometry *geometry = yvex_rocm_gguf_qtype_geometry_find(qtype);
    unsigned long long vector_bytes, weight_offset, total;
    void *block = NULL;
    int rc;
    (void)failure;      /* the reference's failure record belongs to its quantization pipeline */
    yvex_rocm_error_clear(err);
    if (!backend || backend->kind != YVEX_BACKEND_KIND_ROCM || !encoded || !vector || !out || !elements ||
        ((uintptr_t)vector & 3u) || ((uintptr_t)out & 3u) ||
        ((qtype == YVEX_GGUF_QTYPE_F32 || qtype == YVEX_GGUF_QTYPE_I32) && ((uintptr_t)encoded & 3u)) ||
        ((qtype == 1u || qtype == 30u) && ((uintptr_t)encoded & 1u)))
        return yvex_rocm_refuse(err, YVEX_ERR_INVALID_ARG, where,
                                "encoded row, aligned vector/result, and backend are required");
    if (!capability || !geometry || !capability->device_compute_available)
        return yvex_rocm_refuse(err, YVEX_ERR_UNSUPPORTED, where,
                                "qtype has no dedicated device numeric contract");
    if (!geometry->block_size || elements % geometry->block_size)
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where,
                                "qtype row does not satisfy canonical block geometry");
    if (elements / geometry->block_size > ULLONG_MAX / geometry->bytes_per_block ||
        elements / geometry->block_size * geometry->bytes_per_block != encoded_bytes ||
        !mul_u64(elements, sizeof(float), &vector_bytes))
        return yvex_rocm_refuse(err, YVEX_ERR_BOUNDS, where, "encoded row byte geometry is inconsistent");
    rc = yvex_rocm_require_kernels(backend, where, err);
    if (rc != YVEX_OK) return rc;
    weight_offset = (vector_bytes + 255ull) & ~255ull;
    total = weight_offset + ((encoded_bytes + 255ull) & ~255ull) + 256ull;
    if (yvex_hip_malloc(&block, total) != 0)
        return yvex_rocm_refuse(err, YVEX_ERR_NOMEM, where, yvex_hip_last_error());
    {
        unsigned char *base = (unsigned char *)block;
        float *device_out = (float *)(base + total - 256ull);
        if (yvex_hip_memcpy_h2d(base, vector, vector_bytes, backend->stream) != 0 ||
            yvex_hip_memcpy_h2d(base + weight_offset, encoded, encoded_bytes, backend->stream) != 0)
            rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
        if (rc == YVEX_OK)
            rc = yvex_rocm_launch_result(yvex_hip_row_dot(base + weight_offset, qtype, (const float *)base,
                                                          elements, device_out, backend->stream),
                                         "rocm.quant.row_dot.launch", err);
        if (rc == YVEX_OK && yvex_hip_memcpy_d2h(out, device_out, sizeof(float), backend->stream) != 0)
            rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, yvex_hip_last_error());
    }
    if (yvex_hip_free(block) != 0 && rc == YVEX_OK)
        rc = yvex_rocm_refuse(err, YVEX_ERR_BACKEND, where, "device temporary cleanup failed");
    if (rc == YVEX_OK) {
        backend->memory.h2d_bytes += vector_bytes + encoded_bytes;
        backend->memory.d2h_bytes += sizeof(float);
        yvex_rocm_error_clear(err);
    }
    return rc;
}
