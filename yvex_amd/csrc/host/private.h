/*
 * Private state of the ROCm backend object. Mirrors the shape of the reference's backend owner
 * (src/backend/private.h:66-162): status word, memory accounting, one attached resident arena,
 * one attached device workspace with a bump cursor that every operation resets.
 */
#ifndef YVEX_ROCM_PRIVATE_H
#define YVEX_ROCM_PRIVATE_H

#include "yvex_rocm.h"
#include "yvex_rocm_kernels.h"

struct yvex_rocm_backend {
    yvex_backend_kind kind;
    yvex_backend_status status;
    unsigned long long owner_id;
    /* what this backend's tensors name as their owner: the backend itself, or the object an
     * embedding library wraps it in (yvex_rocm_backend_bind_owner) */
    const void *public_owner;
    int device_index;
    int host_only;             /* YVEX_TEST_ROCM_NO_DEVICE: tensors in host memory, no kernels */
    int kernels_available;
    yvex_hip_stream stream;
    yvex_backend_memory_stats memory;
    unsigned long long live_tensors;
    /* resident arena: host shadow range -> device range */
    const unsigned char *resident_host_base;
    unsigned long long resident_host_bytes;
    const yvex_device_tensor *resident_device_tensor;
    unsigned long long resident_device_address;
    unsigned long long resident_generation;
    /* device workspace */
    const yvex_device_tensor *workspace_device_tensor;
    unsigned long long workspace_bytes, workspace_cursor;
    /* device status word shared by the operations of this backend */
    int *device_status;
    int pending_completion;
    /* launch graphs of the row-batch MoE operation, keyed on topology and device addresses */
    struct yvex_rocm_moe_graphs *moe_graphs;
    /* shared sessions (src/backend/cuda/backend.c:1913-2000): a child borrows the device and the
     * resident arena of `resource_owner` (itself for an owning backend) and keeps a stream, a
     * status word, tensors, a workspace and launch graphs of its own; an owner counts its
     * children and does not close while one is open */
    struct yvex_rocm_backend *resource_owner;
    unsigned long long shared_children;
    /* pinned host memory the token ids of hash-routed row batches are copied through, so that the
     * upload is queued on the stream instead of waited for; deferred batches each take a fresh
     * piece, and the cursor returns to the start once nothing is pending on the stream */
    unsigned char *token_staging;
    unsigned long long token_staging_bytes, token_staging_cursor;
};

/* Drop every cached launch graph (the stream is idle or was never used). */
void yvex_rocm_moe_graphs_release(yvex_rocm_backend *backend);

int yvex_rocm_refuse(yvex_error *err, yvex_status code, const char *where, const char *message);
int yvex_rocm_seam(const char *name);
int yvex_rocm_tensor_owner_is(const yvex_rocm_backend *backend, const yvex_device_tensor *tensor);
void yvex_rocm_workspace_reset(yvex_rocm_backend *backend);
/* Kernels present and the backend healthy, else the typed refusal of a missing bundle. */
int yvex_rocm_require_kernels(const yvex_rocm_backend *backend, const char *where, yvex_error *err);
/* Map a launch-level return code (negative yvex_status) to an error. */
int yvex_rocm_launch_result(int rc, const char *where, yvex_error *err);
/* Stream synchronise + read the device status word. */
int yvex_rocm_finish(yvex_rocm_backend *backend, const char *where, int *device_status, yvex_error *err);
/* Clear the status word on the stream, unless deferred row batches are waiting for their barrier. */
int yvex_rocm_status_reset(yvex_rocm_backend *backend, const char *where, yvex_error *err);
/* Resolve a weight view: device_address if given, else the resident arena mapping. */
/* Queue `bytes` of caller-owned host memory for upload to `device` on the backend's stream; the
 * caller's buffer may be reused as soon as this returns. */
int yvex_rocm_upload_queued(yvex_rocm_backend *backend, void *device, const void *host,
                            unsigned long long bytes);
int yvex_rocm_resolve(const yvex_rocm_backend *backend, const unsigned char *host,
                      unsigned long long bytes, unsigned long long *device_address);

/* Residual-stream geometry of a layer plan (src/graph/numeric.c:668-689) within this backend's
 * bounds: at most 7 streams, width at most 16384. */
int yvex_rocm_moe_envelope_geometry(const yvex_moe_layer_plan *layer);
/* Check a weight view against the shape the plan implies (FORMAT), its qtype against the device
 * capability rows (UNSUPPORTED), and find its device address; *resident = 0 when the bytes lie
 * outside the attached arena and carry no device address (the address is then left 0). */
int yvex_rocm_moe_view_check(const yvex_rocm_backend *backend, const yvex_moe_weight_view *view,
                             unsigned long long row_width, unsigned long long row_count,
                             unsigned long long *device_address, int *resident, yvex_error *err);

#endif
