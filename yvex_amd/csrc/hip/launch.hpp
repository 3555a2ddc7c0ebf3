// Host-side helpers shared by the launch wrappers: status codes, error text, launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "../../../include/yvex_rocm_kernels.h"

namespace yvex {

enum Status : int {
    ST_OK = 0, ST_ERR = -1, ST_NOMEM = -2, ST_FORMAT = -4, ST_UNSUPPORTED = -5,
    ST_BACKEND = -6, ST_BOUNDS = -7, ST_STATE = -8, ST_INVALID_ARG = -10
};

void set_last_error(const char *where, hipError_t code);
void set_last_error_text(const char *text);

inline int check_launch(const char *where)
{
    hipError_t code = hipGetLastError();
    if (code != hipSuccess) {
        set_last_error(where, code);
        return ST_BACKEND;
    }
    return ST_OK;
}

// Compute units of the current device (read once, thread-safe).
int compute_units();

// Raise a kernel's dynamic LDS limit once per process; safe when several threads launch.
#define YVEX_ALLOW_DYNAMIC_LDS(kernel, bytes)                                                   \
    do {                                                                                        \
        static std::once_flag once_;                                                            \
        std::call_once(once_, [] {                                                              \
            if (hipFuncSetAttribute((const void *)(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                    (int)(bytes)) != hipSuccess)                                \
                (void)hipGetLastError();                                                        \
        });                                                                                     \
    } while (0)

// IQ2_XXS rows x Q8_K input rows on the int8 matrix cores as a plain projection (prefill.hip).
int launch_iq2_rows_dense(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                          uint64_t row_bytes, const void *act_q8k, uint64_t input_rows, float *out,
                          bool round_bf16, int *status, hipStream_t stream);

// Q8_0 rows x Q8_K input rows on the int8 matrix cores (dense_q8_0.hip).
int launch_q8_0_rows_dense(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                           uint64_t row_bytes, const void *act_q8k, uint64_t input_rows,
                           const float *additive, float *out, uint64_t out_stride, bool output_bf16,
                           int *status, hipStream_t stream);

// Q4_K rows x Q8_K input rows on the int8 matrix cores (dense_q4k.hip).
int launch_q4k_rows_dense(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                          uint64_t row_bytes, const void *act_q8k, uint64_t input_rows,
                          const float *additive, float *out, uint64_t out_stride, bool output_bf16,
                          int *status, hipStream_t stream);
// The same product with its operands staged through LDS, for batches that fill every compute
// unit with (128 rows x 64 tokens) tiles (rows_q4k.hip).
int launch_q4k_rows_staged(const uint8_t *encoded, uint64_t row_count, uint64_t row_width,
                          uint64_t row_bytes, const void *act_q8k, uint64_t input_rows,
                          const float *additive, float *out, uint64_t out_stride, bool output_bf16,
                          int *status, hipStream_t stream);

inline hipStream_t as_stream(yvex_hip_stream s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace yvex
