// Host-side helpers shared by the launch wrappers: status codes, error text, launch checks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

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

inline hipStream_t as_stream(yvex_hip_stream s) { return reinterpret_cast<hipStream_t>(s); }

}  // namespace yvex
