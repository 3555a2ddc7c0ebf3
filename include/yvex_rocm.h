/*
 * C ABI of the MI355X (gfx950) backend for YVEX's quantized-weight matmul path.
 *
 * This header is what a libyvex build binds instead of its CUDA backend for the operations on
 * this path. Names, argument meaning, status codes and fail-closed behaviour follow the
 * reference's backend contract; every declaration cites the reference interface it replaces.
 * Structures that cross the boundary keep the reference's field names and order.
 *
 * Conventions (include/yvex/core.h:13-48, src/backend/cuda/qtype.c:246,299,391-392):
 *   - every entry point returns a yvex_status (0 = OK, negative = refusal);
 *   - the last parameter is a yvex_error that is cleared on success and may be NULL;
 *   - output facts are zeroed on entry and published only on success;
 *   - an output tensor is marked written only by a successful operation;
 *   - nothing here ever falls back to another backend or to the CPU.
 */
#ifndef YVEX_ROCM_H
#define YVEX_ROCM_H

/* The structures, enumerations and constants this header shares with the reference are declared
 * below with the reference's names and layout (a test compares both, field by field). A
 * translation unit of the reference itself, which already has them from <yvex/...>, defines
 * YVEX_ROCM_REFERENCE_TYPES before including this header and gets only the library's own types
 * and entry points (all named yvex_rocm_*). */

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status and error: include/yvex/core.h:13-48 ------------------------------------------ */

#ifndef YVEX_ROCM_REFERENCE_TYPES
typedef enum {
    YVEX_OK = 0,
    YVEX_ERR = -1,
    YVEX_ERR_NOMEM = -2,
    YVEX_ERR_IO = -3,
    YVEX_ERR_FORMAT = -4,
    YVEX_ERR_UNSUPPORTED = -5,
    YVEX_ERR_BACKEND = -6,
    YVEX_ERR_BOUNDS = -7,
    YVEX_ERR_STATE = -8,
    YVEX_ERR_CANCELLED = -9,
    YVEX_ERR_INVALID_ARG = -10,
    YVEX_ERR_TIMEOUT = -11
} yvex_status;

#define YVEX_ERROR_WHERE_CAP 96
#define YVEX_ERROR_MESSAGE_CAP 256
typedef struct {
    yvex_status code;
    char where[YVEX_ERROR_WHERE_CAP];
    char message[YVEX_ERROR_MESSAGE_CAP];
} yvex_error;
#endif

const char *yvex_rocm_status_name(yvex_status status);
void yvex_rocm_error_clear(yvex_error *err);
void yvex_rocm_error_set(yvex_error *err, yvex_status code, const char *where, const char *message);
int yvex_rocm_error_is_set(const yvex_error *err);
yvex_status yvex_rocm_error_code(const yvex_error *err);

/* ---- qtype identity, geometry and fail-closed admission ----------------------------------- */
/* include/yvex/qtype.h:19-63, src/gguf/qtype.c:15-104, src/gguf/quant_registry.c:50-117 */

#ifndef YVEX_ROCM_REFERENCE_TYPES
enum {
    YVEX_GGUF_QTYPE_F32 = 0, YVEX_GGUF_QTYPE_F16 = 1, YVEX_GGUF_QTYPE_Q8_0 = 8,
    YVEX_GGUF_QTYPE_Q2_K = 10, YVEX_GGUF_QTYPE_Q4_K = 12, YVEX_GGUF_QTYPE_Q8_K = 15,
    YVEX_GGUF_QTYPE_IQ2_XXS = 16, YVEX_GGUF_QTYPE_I32 = 26, YVEX_GGUF_QTYPE_BF16 = 30,
    YVEX_GGUF_QTYPE_MXFP4 = 39, YVEX_GGUF_QTYPE_ABI_UPSTREAM_MAX_ID = 42
};

typedef enum {
    YVEX_GGUF_QTYPE_IDENTITY_ADMITTED = 0,
    YVEX_GGUF_QTYPE_IDENTITY_REMOVED = 1,
    YVEX_GGUF_QTYPE_IDENTITY_RESERVED = 2,
    YVEX_GGUF_QTYPE_IDENTITY_OUTSIDE_BASELINE = 3,
    YVEX_GGUF_QTYPE_IDENTITY_UNKNOWN = 4
} yvex_gguf_qtype_identity_status;
#endif

typedef struct {
    unsigned int qtype;
    const char *name;
    yvex_gguf_qtype_identity_status identity;
    unsigned int block_size, bytes_per_block;
} yvex_rocm_qtype_geometry;

/* Replaces yvex_gguf_qtype_geometry_find (src/gguf/qtype.c:119-124): NULL above ID 42. */
const yvex_rocm_qtype_geometry *yvex_rocm_gguf_qtype_geometry_find(unsigned int qtype);

typedef enum {
    YVEX_ROCM_QUANT_REFUSAL_NONE = 0,
    YVEX_ROCM_QUANT_REFUSAL_ENCODER_UNAVAILABLE,
    YVEX_ROCM_QUANT_REFUSAL_REMOVED_IDENTITY,
    YVEX_ROCM_QUANT_REFUSAL_OUTSIDE_PINNED_BASELINE
} yvex_rocm_quant_refusal;

/* One row per qtype ID, index == ID (src/gguf/quant_registry.c:50-103). device_compute is the
 * reference's dedicated_cuda_compute_available restated for this backend. Relative to the
 * reference, exactly one row is extended: Q4_K is admitted with device compute; MXFP4 is
 * admitted for storage but has no kernel in this backend yet (device_compute = 0). */
typedef struct {
    unsigned int qtype;
    int known, storage_admitted, reference_decoder_available;
    int dedicated_cpu_compute_available, device_compute_available;
    int extension_of_reference;
    yvex_rocm_quant_refusal refusal;
} yvex_rocm_numeric_capability;

/* Replaces yvex_quant_numeric_capability_at (src/gguf/quant_registry.c:114-118). */
const yvex_rocm_numeric_capability *yvex_rocm_quant_numeric_capability_at(unsigned int qtype);

/* ---- backend object: include/yvex/backend.h:13-152 ----------------------------------------- */

typedef struct yvex_rocm_backend yvex_rocm_backend;
#ifndef YVEX_ROCM_REFERENCE_TYPES
typedef struct yvex_device_tensor yvex_device_tensor;

typedef enum {
    YVEX_BACKEND_KIND_CPU = 0,
    YVEX_BACKEND_KIND_CUDA,
    YVEX_BACKEND_KIND_METAL,
    YVEX_BACKEND_KIND_ROCM
} yvex_backend_kind;

typedef enum {
    YVEX_BACKEND_STATUS_READY = 0,
    YVEX_BACKEND_STATUS_CONTEXT_READY,
    YVEX_BACKEND_STATUS_UNSUPPORTED,
    YVEX_BACKEND_STATUS_FAILED
} yvex_backend_status;

typedef struct {
    yvex_backend_kind kind;
    const char *device;                 /* NULL or "0".."N": device ordinal */
    unsigned long long memory_limit_bytes;
} yvex_backend_options;

typedef struct {
    unsigned long long allocated_bytes;
    unsigned long long allocation_count, allocation_events, release_events;
    unsigned long long h2d_bytes, d2h_bytes;
    unsigned long long peak_allocated_bytes;
    unsigned long long memory_limit_bytes;
} yvex_backend_memory_stats;

/* include/yvex/model.h:18-58, same values. Raw encoded bytes (resident arenas, workspaces)
 * travel as I8 tensors. */
typedef enum {
    YVEX_DTYPE_UNKNOWN = 0,
    YVEX_DTYPE_F32,
    YVEX_DTYPE_F16,
    YVEX_DTYPE_BF16,
    YVEX_DTYPE_F64,
    YVEX_DTYPE_I8,
    YVEX_DTYPE_I16,
    YVEX_DTYPE_I32,
    YVEX_DTYPE_I64,
    YVEX_DTYPE_Q4_0, YVEX_DTYPE_Q4_1, YVEX_DTYPE_Q5_0, YVEX_DTYPE_Q5_1, YVEX_DTYPE_Q8_0,
    YVEX_DTYPE_Q8_1,
    YVEX_DTYPE_Q2_K, YVEX_DTYPE_Q3_K, YVEX_DTYPE_Q4_K, YVEX_DTYPE_Q5_K, YVEX_DTYPE_Q6_K,
    YVEX_DTYPE_Q8_K,
    YVEX_DTYPE_IQ2_XXS, YVEX_DTYPE_IQ2_XS, YVEX_DTYPE_IQ3_XXS, YVEX_DTYPE_IQ1_S,
    YVEX_DTYPE_IQ4_NL, YVEX_DTYPE_IQ3_S, YVEX_DTYPE_IQ2_S, YVEX_DTYPE_IQ4_XS, YVEX_DTYPE_IQ1_M,
    YVEX_DTYPE_TQ1_0, YVEX_DTYPE_TQ2_0, YVEX_DTYPE_MXFP4
} yvex_dtype;

#define YVEX_TENSOR_MAX_DIMS 4
typedef struct {
    const char *name;
    yvex_dtype dtype;
    unsigned int rank;
    unsigned long long dims[YVEX_TENSOR_MAX_DIMS];
    unsigned long long bytes;
} yvex_backend_tensor_desc;

/* include/yvex/internal/backend.h:256-269, same fields in the same order. */
struct yvex_device_tensor {
    yvex_rocm_backend *owner;
    unsigned long long owner_id;
    char *name;
    yvex_dtype dtype;
    unsigned int rank;
    unsigned long long dims[YVEX_TENSOR_MAX_DIMS];
    unsigned long long bytes;
    unsigned char *data, *host_data;    /* device address; host shadow of a resident tensor */
    void *backend_allocation;
    unsigned long long resident_bytes;
    int virtual_reserved;
    int is_written, host_accessible, borrowed_host;
};

typedef enum {
    YVEX_BACKEND_VARIANT_TENSOR_ALLOC = 0,
    YVEX_BACKEND_VARIANT_TENSOR_ZERO,
    YVEX_BACKEND_VARIANT_TENSOR_WRITE,
    YVEX_BACKEND_VARIANT_TENSOR_READ,
    YVEX_BACKEND_VARIANT_TENSOR_COPY,
    YVEX_BACKEND_VARIANT_QTYPE_ROW_DOT = 15,
    YVEX_BACKEND_VARIANT_ATTENTION_ENCODED = 16,   /* the encoded matvec / MoE family */
    YVEX_BACKEND_VARIANT_COUNT = 17
} yvex_backend_operation_variant;

typedef enum {
    YVEX_BACKEND_CAPABILITY_UNSUPPORTED = 0,
    YVEX_BACKEND_CAPABILITY_SUPPORTED,
    YVEX_BACKEND_CAPABILITY_FAILED
} yvex_backend_capability_state;

typedef enum {
    YVEX_BACKEND_CAPABILITY_REASON_NONE = 0,
    YVEX_BACKEND_CAPABILITY_REASON_DRIVER_UNAVAILABLE,
    YVEX_BACKEND_CAPABILITY_REASON_DEVICE_UNAVAILABLE,
    YVEX_BACKEND_CAPABILITY_REASON_CONTEXT_UNAVAILABLE,
    YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_ABSENT,
    YVEX_BACKEND_CAPABILITY_REASON_KERNEL_BUNDLE_REJECTED,
    YVEX_BACKEND_CAPABILITY_REASON_FUNCTION_MISSING,
    YVEX_BACKEND_CAPABILITY_REASON_VARIANT_UNSUPPORTED,
    YVEX_BACKEND_CAPABILITY_REASON_LAUNCH_FAILED,
    YVEX_BACKEND_CAPABILITY_REASON_SYNCHRONIZATION_FAILED,
    YVEX_BACKEND_CAPABILITY_REASON_CLEANUP_FAILED
} yvex_backend_capability_reason;

typedef struct {
    yvex_backend_kind backend_kind;
    yvex_backend_operation_variant variant;
    yvex_backend_capability_state state;
    yvex_backend_capability_reason reason;
    yvex_dtype input_dtype, weight_dtype, output_dtype;
    int context_available, kernel_bundle_available, function_available;
} yvex_backend_capability_result;
#endif

/* Replaces yvex_backend_open (src/backend/core.c:176-205) for kind ROCM; every other kind
 * answers UNSUPPORTED. Test seams, read from the environment like the reference's
 * YVEX_TEST_CUDA_* (src/backend/cuda/capability.c:183, backend.c:275-453):
 *   YVEX_TEST_ROCM_NO_DEVICE=1       open without a GPU: tensors live in host memory, every
 *                                    kernel variant is unsupported (kernel-bundle-absent)
 *   YVEX_TEST_ROCM_BUNDLE_FAILURE=1  a GPU is present but its kernels are treated as absent
 *   YVEX_TEST_ROCM_LAUNCH_FAILURE=1 / _SYNC_FAILURE=1 / _CLEANUP_FAILURE=1
 *                                    the next launch / synchronise / release reports failure */
int yvex_rocm_backend_open(yvex_rocm_backend **out, const yvex_backend_options *options, yvex_error *err);
/* For a library that wraps this backend in an object of its own (the reference's struct
 * yvex_backend with this backend behind `impl`): tensors allocated from now on name `owner` in
 * their `owner` field, and ownership checks compare against it, so the embedding library's own
 * checks (src/backend/private.h:95-101) hold on them. No reference counterpart; bound once, before
 * the first allocation. */
int yvex_rocm_backend_bind_owner(yvex_rocm_backend *backend, const void *owner, yvex_error *err);
/* yvex_backend_open_shared_cuda (include/yvex/internal/backend.h:254-255,
 * src/backend/cuda/backend.c:1913-2000): session-local state that borrows one owning backend's
 * device and resident arena. The child has a stream, a device status word, memory accounting
 * under its own limit, tensors, a workspace and launch graphs of its own, so sessions that share
 * one set of resident weights each run their own row batches; attaching the owner's arena to a
 * child (yvex_rocm_backend_resident_attach with the owner's resident tensor, the same host base
 * and generation the owner attached) uploads nothing. The owner must itself be an owning
 * backend (INVALID_ARG otherwise) and refuses to close while a child is open (STATE). */
int yvex_rocm_backend_open_shared(yvex_rocm_backend **out, yvex_rocm_backend *context_owner,
                                  unsigned long long memory_limit_bytes, yvex_error *err);
/* include/yvex/backend.h:142-152: a cleanup failure keeps *backend non-NULL for a retry. */
int yvex_rocm_backend_close_checked(yvex_rocm_backend **backend, yvex_error *err);
yvex_backend_kind yvex_rocm_backend_kind_of(const yvex_rocm_backend *backend);
yvex_backend_status yvex_rocm_backend_status_of(const yvex_rocm_backend *backend);
int yvex_rocm_backend_get_memory_stats(const yvex_rocm_backend *backend, yvex_backend_memory_stats *out,
                                  yvex_error *err);
int yvex_rocm_backend_sync(yvex_rocm_backend *backend, yvex_error *err);
int yvex_rocm_backend_query_capability(const yvex_rocm_backend *backend,
                                  yvex_backend_operation_variant variant,
                                  yvex_backend_capability_result *out, yvex_error *err);

/* include/yvex/internal/backend.h:174-185,302: what the device sustains, measured at the
 * caller's request (the reference publishes it in its backend report, src/backend/core.c:1801).
 * Five samples each of four streaming reads and four device-to-device copies of a 1 GiB working
 * set (allocated for the probe and released again); the rates are working set x iterations over
 * the median sample, the copy counting its payload once. A discrete-HBM device has no coherent
 * host path: those fields stay zero. The identity fields are the reference runtime's SHA-256
 * seals and stay empty here. */
#ifndef YVEX_ROCM_REFERENCE_TYPES
#define YVEX_BACKEND_BANDWIDTH_SCHEMA_V1 1u
#define YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT 5u
typedef struct {
    unsigned int schema_version;
    unsigned long long working_set_bytes, iterations, sample_count;
    unsigned long long stream_elapsed_ns[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned long long copy_elapsed_ns[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned long long coherent_host_elapsed_ns[YVEX_BACKEND_BANDWIDTH_SAMPLE_COUNT];
    unsigned long long sustainable_read_bytes_per_second, sustainable_copy_bytes_per_second;
    unsigned long long sustainable_coherent_host_bytes_per_second;
    char kernel_bundle_identity[65], identity[65];
} yvex_backend_bandwidth_evidence;
#endif
int yvex_rocm_backend_bandwidth_probe(yvex_rocm_backend *backend, yvex_backend_bandwidth_evidence *out,
                                      yvex_error *err);

/* include/yvex/backend.h:177-204 */
int yvex_rocm_backend_tensor_alloc(yvex_rocm_backend *backend, const yvex_backend_tensor_desc *desc,
                              yvex_device_tensor **out, yvex_error *err);
int yvex_rocm_backend_tensor_release(yvex_rocm_backend *backend, yvex_device_tensor **tensor,
                                yvex_error *err);
int yvex_rocm_backend_tensor_write(yvex_rocm_backend *backend, yvex_device_tensor *tensor, const void *src,
                              unsigned long long len, yvex_error *err);
int yvex_rocm_backend_tensor_read(yvex_rocm_backend *backend, const yvex_device_tensor *tensor, void *dst,
                             unsigned long long len, yvex_error *err);
int yvex_rocm_backend_tensor_copy(yvex_rocm_backend *backend, yvex_device_tensor *dst,
                             const yvex_device_tensor *src, yvex_error *err);
int yvex_rocm_backend_tensor_owned_by(const yvex_rocm_backend *backend, const yvex_device_tensor *tensor);

/* ---- resident weights: include/yvex/internal/backend.h:270-301, src/backend/residency.c ---- */
/*
 * The reference maps one pointer that the CPU writes and the GPU reads (unified memory). On a
 * discrete-HBM MI355X the same calls are kept with these meanings: resident_alloc gives a device
 * allocation in HBM plus a pinned host shadow returned through *host; resident_attach is the
 * publication point that uploads [host_base, host_base + bytes) into HBM; later writes to the
 * shadow become visible at the next attach or prefetch. resolve maps a borrowed pointer inside
 * the shadow to device_base + offset exactly as src/backend/residency.c:89-112 does.
 */
#ifndef YVEX_ROCM_REFERENCE_TYPES
typedef enum {
    YVEX_BACKEND_RESIDENT_INVALID = -1,
    YVEX_BACKEND_RESIDENT_MISS = 0,
    YVEX_BACKEND_RESIDENT_HIT = 1
} yvex_backend_resident_result;
#endif

int yvex_rocm_backend_resident_alloc(yvex_rocm_backend *backend, const yvex_backend_tensor_desc *desc,
                                yvex_device_tensor **out, unsigned char **host, yvex_error *err);
int yvex_rocm_backend_resident_prefetch(yvex_rocm_backend *backend, yvex_device_tensor *tensor,
                                   unsigned long long *prefetched_bytes, yvex_error *err);
int yvex_rocm_backend_resident_attach(yvex_rocm_backend *backend, const unsigned char *host_base,
                                 unsigned long long bytes, const yvex_device_tensor *tensor,
                                 unsigned long long generation, yvex_error *err);
int yvex_rocm_backend_resident_detach(yvex_rocm_backend *backend, yvex_error *err);
int yvex_rocm_backend_resident_resolve(const yvex_rocm_backend *backend, const unsigned char *host,
                                  unsigned long long bytes, unsigned long long *device_address);

/* include/yvex/internal/backend.h:350-354: bump-allocated device scratch, reset per operation. */
int yvex_rocm_backend_workspace_attach(yvex_rocm_backend *backend, const yvex_device_tensor *tensor,
                                  unsigned long long bytes, yvex_error *err);
void yvex_rocm_backend_workspace_detach(yvex_rocm_backend *backend);
int yvex_rocm_backend_workspace_acquire(yvex_rocm_backend *backend, unsigned long long bytes,
                                   unsigned long long alignment,
                                   unsigned long long *device_address);

/* ---- dense projection, output head, gather ------------------------------------------------- */

/* include/yvex/internal/backend.h:325-331 (yvex_backend_cuda_operation_facts). */
typedef struct yvex_rocm_operation_facts {
    unsigned long long h2d_bytes, d2h_bytes, d2d_bytes, kernel_launches, upload_count;
    unsigned long long download_count, stream_synchronizations, device_synchronizations;
    unsigned long long active_weight_bytes, state_bytes;
    unsigned long long activation_bytes, temporary_bytes, tensor_core_launches;
    int compulsory_memory_facts_available;
} yvex_rocm_operation_facts;

/* Replaces yvex_backend_cuda_encoded_matvec (include/yvex/internal/backend.h:332-337,
 * src/backend/cuda/qtype.c:220-405). output[in, row] = dot(encoded row, input row in)
 * (+ additive). activation_q8 = 1 quantizes the F32 input rows to Q8_K on device first.
 * Refusals: activation_q8 not 0/1 -> INVALID_ARG; qtype unknown, removed, outside the baseline
 * or without device compute -> UNSUPPORTED (on the host, before any launch); geometry, byte
 * count, ownership, unwritten input, additive aliasing output, resident MISS -> FORMAT; kernels
 * absent -> UNSUPPORTED; non-finite numerics seen on device -> FORMAT. With input_tail the rows
 * are split (the reference's speculation path, qtype.c:256-281, kernels.cu:736-782): row r is
 * input[r, 0..input_head_width) followed by input_tail[r, ...], every value rounded to bf16, the
 * Q8 activation policy is ignored, and the attached workspace must hold rows * width floats. */
int yvex_rocm_encoded_matvec(
    yvex_rocm_backend *backend, const unsigned char *resident_encoded,
    unsigned long long encoded_bytes, unsigned int qtype, unsigned long long row_count,
    unsigned long long row_width, unsigned long long row_bytes, unsigned long long input_rows,
    const yvex_device_tensor *input, const yvex_device_tensor *input_tail,
    unsigned long long input_head_width, const yvex_device_tensor *additive,
    yvex_device_tensor *output, int activation_q8, yvex_rocm_operation_facts *facts,
    yvex_error *err);

/* Replaces yvex_backend_cuda_encoded_gather (include/yvex/internal/backend.h:338-342,
 * src/backend/cuda/qtype.c:411-521): decode selected rows to F32. row_ids is a host array. */
int yvex_rocm_encoded_gather(
    yvex_rocm_backend *backend, const unsigned char *resident_encoded,
    unsigned long long encoded_bytes, unsigned int qtype, unsigned long long row_count,
    unsigned long long row_width, unsigned long long row_bytes, const unsigned int *row_ids,
    unsigned long long selected_rows, yvex_device_tensor *output,
    yvex_rocm_operation_facts *facts, yvex_error *err);

/* ---- greedy selection over logits rows ---------------------------------------------------- */

/* Replaces the select_greedy_rows entry of yvex_backend_sampling_operations
 * (include/yvex/internal/sampling.h:129-137, src/backend/cuda/sampling.c:284-392): for each of
 * row_count rows of row_width F32 logits held by a tensor of this backend, the largest value,
 * the lowest token holding it and the number of tokens holding it, written to host arrays. The
 * device results live in the attached workspace for the call. Refusals: geometry, ownership,
 * dtype, unwritten logits -> FORMAT; no workspace -> NOMEM; kernels absent -> UNSUPPORTED; a
 * non-finite logit, a token outside the row or a zero tie count -> FORMAT, outputs zeroed. */
int yvex_rocm_select_greedy_rows(
    yvex_rocm_backend *backend, const yvex_device_tensor *logits, unsigned long long row_count,
    unsigned long long row_width, unsigned int *selected_tokens, float *selected_values,
    unsigned long long *tie_counts, yvex_rocm_operation_facts *facts, yvex_error *err);

/* The qtype parity probe, yvex_cuda_quant_row_dot (src/backend/cuda/qtype.c:523-700): one encoded
 * row (host bytes) times one vector (host floats), computed on the device by one thread in double
 * precision in element order, as src/backend/cuda/kernels.cu:112-124 does, so it equals the CPU
 * row dot wherever the decoders agree. Refusals: missing or misaligned arguments INVALID_ARG,
 * qtype without device compute UNSUPPORTED, elements not a whole number of blocks or a byte count
 * that disagrees BOUNDS, kernels absent UNSUPPORTED. failure is accepted for call compatibility
 * and left untouched (the reference's record belongs to its quantization pipeline). */
int yvex_rocm_quant_row_dot(yvex_rocm_backend *backend, unsigned int qtype, const unsigned char *encoded,
                            size_t encoded_bytes, const float *vector, unsigned long long elements,
                            float *out, void *failure, yvex_error *err);

/* ---- MoE row batch: include/yvex/internal/moe.h ------------------------------------------- */

#ifndef YVEX_ROCM_REFERENCE_TYPES
#define YVEX_SHA256_HEX_CAP 65u
#define YVEX_MOE_MAX_SELECTED 16u
#define YVEX_MOE_ROW_BATCH_SCHEMA_V1 1u
#define YVEX_MOE_ROW_BATCH_RESULT_SCHEMA_V4 4u
#define YVEX_EXPERT_WORKLIST_HISTOGRAM_CAP 17u
/* Kernel families this backend admits in a weight view (moe.h:20-23 list the CUDA ones). */
#define YVEX_MOE_KERNEL_PORTABLE_ENCODED_ROW "portable-encoded-row"
#define YVEX_MOE_KERNEL_PORTABLE_EXPERT_ROW "portable-expert-row"
#endif
#define YVEX_MOE_KERNEL_GFX950_EXPERT_SWEEP "gfx950-int8-dot-expert-sweep"
/* The family a sealed worklist policy names in tensor_core_kernel_family to admit this backend's
 * int8 matrix-core expert kernels (the reference names its own, moe.h:22, and refuses any other:
 * src/backend/cuda/moe.c:937-951). With a policy present the matrix-core regime runs only when
 * tensor_core_minimum is non-zero and the batch has at least that many rows; execute_rows then
 * still picks the faster of its two kernel families, which publish the same bits. */
#define YVEX_MOE_KERNEL_GFX950_MATRIX_CORE_EXPERT "gfx950-int8-matrix-core-expert"

#ifndef YVEX_ROCM_REFERENCE_TYPES
typedef enum {
    YVEX_MOE_ROUTER_HASH_TOKEN_ID = 0,
    YVEX_MOE_ROUTER_LEARNED_HIDDEN_STATE
} yvex_moe_router_class;
/* moe.h:35 has SQRT_SOFTPLUS only; SIGMOID is this build's addition for the benchmark layer. */
typedef enum {
    YVEX_MOE_SCORING_SQRT_SOFTPLUS = 0,
    YVEX_MOE_SCORING_SIGMOID = 1
} yvex_moe_scoring_policy;
typedef enum { YVEX_MOE_TOPK_NOAUX_TC = 0 } yvex_moe_topk_policy;
typedef enum { YVEX_MOE_ACTIVATION_SILU = 0 } yvex_moe_activation;

typedef enum {
    YVEX_MOE_WEIGHT_FFN_NORM = 0,
    YVEX_MOE_WEIGHT_MHC_FUNCTION,
    YVEX_MOE_WEIGHT_MHC_BASE,
    YVEX_MOE_WEIGHT_MHC_SCALE,
    YVEX_MOE_WEIGHT_ROUTER,
    YVEX_MOE_WEIGHT_ROUTER_TABLE,
    YVEX_MOE_WEIGHT_ROUTER_BIAS,
    YVEX_MOE_WEIGHT_ROUTED_GATE,
    YVEX_MOE_WEIGHT_ROUTED_UP,
    YVEX_MOE_WEIGHT_ROUTED_DOWN,
    YVEX_MOE_WEIGHT_SHARED_GATE,
    YVEX_MOE_WEIGHT_SHARED_UP,
    YVEX_MOE_WEIGHT_SHARED_DOWN,
    YVEX_MOE_WEIGHT_COUNT
} yvex_moe_weight_slot;

typedef enum {
    YVEX_EXECUTION_LAYOUT_CANONICAL_ROW = 0,
    YVEX_EXECUTION_LAYOUT_CONTIGUOUS_DENSE,
    YVEX_EXECUTION_LAYOUT_EXPERT_MAJOR,
    YVEX_EXECUTION_LAYOUT_DERIVED_BACKEND
} yvex_execution_layout_class;

typedef enum {
    YVEX_EXECUTION_ACTIVATION_HOST_F32 = 0,
    YVEX_EXECUTION_ACTIVATION_DEVICE_F32,
    YVEX_EXECUTION_ACTIVATION_DEVICE_F16,
    YVEX_EXECUTION_ACTIVATION_DEVICE_ENCODED
} yvex_execution_activation_class;

typedef enum {
    YVEX_EXECUTION_CLASS_PORTABLE_REFERENCE = 0,
    YVEX_EXECUTION_CLASS_DEVICE_NATIVE,
    YVEX_EXECUTION_CLASS_FORENSIC_REFERENCE
} yvex_execution_class;

typedef enum {
    YVEX_EXECUTION_BATCH_SINGLE_ROW = 0,
    YVEX_EXECUTION_BATCH_SPECULATIVE_VERIFICATION,
    YVEX_EXECUTION_BATCH_MULTI_SESSION,
    YVEX_EXECUTION_BATCH_PREFILL,
    YVEX_EXECUTION_BATCH_COMPILED_COMPATIBLE
} yvex_execution_batch_provenance;

/* moe.h:54-64 */
typedef struct {
    unsigned long long tensor_id, expert_index;
    int role;
    unsigned int qtype;
    yvex_execution_layout_class layout;
    yvex_execution_activation_class activation;
    const char *kernel_family;
    const unsigned char *encoded;        /* host pointer inside the attached resident arena */
    size_t encoded_bytes, storage_bytes;
    unsigned long long row_bytes, row_width, row_count, device_address;
} yvex_moe_weight_view;

/* moe.h:65-84 */
typedef struct {
    unsigned int schema_version;
    unsigned long long ordinal, layer_index, predictor_index;
    int tensor_scope;
    yvex_moe_router_class router_class;
    yvex_moe_scoring_policy scoring;
    yvex_moe_topk_policy topk_policy;
    yvex_moe_activation activation;
    unsigned long long hidden_width, residual_streams, expanded_width;
    unsigned long long mhc_mixing_rows, mhc_sinkhorn_iterations;
    unsigned long long routed_experts, shared_experts, experts_per_token;
    unsigned long long expert_intermediate_width, shared_intermediate_width;
    unsigned long long hash_table_rows, hash_table_columns, correction_bias_width;
    double rms_epsilon, mhc_epsilon, mhc_post_multiplier;
    double routed_scaling_factor, activation_limit;
    int requires_token_ids, requires_correction_bias, normalize_topk_probabilities;
    unsigned long long tensor_ids[YVEX_MOE_WEIGHT_COUNT];
    unsigned int qtypes[YVEX_MOE_WEIGHT_COUNT];
    char layer_identity[YVEX_SHA256_HEX_CAP];
} yvex_moe_layer_plan;

/* execution_batch.h:42-66: who the rows of a batch belong to. The reference seals the identity
 * fields with SHA-256 (yvex_execution_batch_seal); that seal belongs to its runtime and is not
 * re-derived here: this backend checks the fields execute_rows compares with the row batch
 * (schema, row_count, provenance, phase; src/backend/cuda/moe.c:1845-1852). */
#define YVEX_EXECUTION_BATCH_SCHEMA_V1 1u
#define YVEX_EXPERT_WORKLIST_POLICY_SCHEMA_V1 1u
typedef struct {
    unsigned long long execution_generation, state_generation;
    char identity[YVEX_SHA256_HEX_CAP];
} yvex_execution_batch_source;
typedef struct {
    unsigned long long source_index, source_row, sequence_position;
    unsigned long long candidate_ordinal, publication_ordinal;
    int candidate_present;
} yvex_execution_batch_row;
typedef struct {
    unsigned int schema_version;
    yvex_execution_batch_provenance provenance;
    unsigned int phase;
    unsigned long long row_count, source_count, model_generation;
    const yvex_execution_batch_source *sources;
    const yvex_execution_batch_row *rows;
    char runtime_model_identity[YVEX_SHA256_HEX_CAP];
    char runtime_binding_identity[YVEX_SHA256_HEX_CAP];
    char physical_variant_identity[YVEX_SHA256_HEX_CAP];
    char execution_profile_identity[YVEX_SHA256_HEX_CAP];
    char operation_identity[YVEX_SHA256_HEX_CAP];
    char identity[YVEX_SHA256_HEX_CAP];
} yvex_execution_batch;

/* execution_batch.h:86-93 */
typedef struct {
    unsigned int schema_version;
    unsigned long long supported_width_mask;   /* bit n set: a batch of n rows is admitted */
    unsigned long long tensor_core_minimum;
    char narrow_kernel_family[64];
    char tensor_core_kernel_family[64];
    char identity[YVEX_SHA256_HEX_CAP];
} yvex_expert_worklist_policy;

/* execution_batch.h:128-137 */
typedef struct {
    unsigned int schema_version;
    unsigned long long worklist_count, pair_count, bucket_count;
    unsigned long long maximum_bucket_population;
    unsigned long long tensor_core_eligible_pairs, tensor_core_executed_pairs;
    unsigned long long narrow_pairs, tail_rows;
    unsigned long long width_histogram[YVEX_EXPERT_WORKLIST_HISTOGRAM_CAP];
    unsigned long long population_histogram[YVEX_EXPERT_WORKLIST_HISTOGRAM_CAP];
    unsigned long long provenance_counts[YVEX_EXECUTION_BATCH_COMPILED_COMPATIBLE + 1u];
} yvex_expert_worklist_observation;

/* execution.h:329-333 */
typedef struct {
    unsigned long long active_weight_bytes, state_bytes, activation_bytes, temporary_bytes;
    unsigned long long measured_operations, missing_operations;
    int complete;
} yvex_execution_memory_facts;

typedef struct {
    int defer;
    void *host;
} yvex_moe_device_completion;

/* moe.h:182-197. execution_batch and worklist_policy come together or not at all; when present
 * they are checked against the row batch as moe.c:1845-1852 does (their SHA-256 seals excepted). */
typedef struct {
    const yvex_moe_layer_plan *layer;
    yvex_moe_weight_view weights[YVEX_MOE_WEIGHT_COUNT];
    const float *expanded_input;
    const yvex_device_tensor *device_input;
    yvex_device_tensor *device_output;
    unsigned int token_id;
    int token_id_present;
    int (*cancel_requested)(void *context);
    void *cancel_context;
    int evidence_level;
    int eager_execution;
    const yvex_moe_device_completion *device_completion;
    const yvex_execution_batch *execution_batch;
    const yvex_expert_worklist_policy *worklist_policy;
} yvex_moe_layer_job;

/* moe.h:221-236 */
typedef struct {
    unsigned int schema_version;
    unsigned long long row_count, row_width, row_stride;
    const float *expanded_rows;
    const yvex_device_tensor *device_rows;
    yvex_device_tensor *device_outputs;
    const unsigned int *token_ids;
    int token_ids_present;
    yvex_execution_batch_provenance provenance;
    unsigned int phase;
    yvex_execution_class execution_class;
    const char *execution_profile_identity;
    const void *execution_sources;
    const void *execution_rows;
    unsigned long long execution_source_count;
    int complete_after_operation;
} yvex_moe_row_batch;

/* moe.h:238-246: optional host copies; NULL pointers are skipped. */
typedef struct {
    float *combined_rows, *routed_rows, *shared_rows, *post_rows, *combination_rows;
    unsigned long long combined_capacity, routed_capacity, shared_capacity;
    unsigned long long post_capacity, combination_capacity;
    unsigned long long *selected_experts;
    float *selected_weights;
    unsigned long long selection_capacity;
} yvex_moe_row_batch_output;

/* moe.h:248-271 */
typedef struct {
    unsigned int schema_version;
    int completed, execution_profile_available, device_completion_pending;
    yvex_execution_class execution_class;
    unsigned long long row_count, row_expert_pairs, unique_experts;
    yvex_expert_worklist_observation worklists;
    unsigned long long grouped_expert_operations, shared_expert_operations;
    unsigned long long expert_subviews_accessed, encoded_bytes_read;
    unsigned long long h2d_bytes, d2h_bytes, d2d_bytes, kernel_launches;
    unsigned long long tensor_core_launches;
    unsigned long long graph_launches, graph_captures, graph_replays;
    unsigned long long upload_count, download_count, cache_hits, cache_misses;
    unsigned long long stream_synchronizations, device_synchronizations;
    unsigned long long active_weight_base_bytes;
    unsigned long long active_weight_per_unique_expert_bytes;
    yvex_execution_memory_facts memory;
    unsigned long long total_ns, synchronization_ns;
    char execution_profile_identity[YVEX_SHA256_HEX_CAP];
    char execution_batch_identity[YVEX_SHA256_HEX_CAP];
    char worklist_policy_identity[YVEX_SHA256_HEX_CAP];
    char expert_worklist_identity[YVEX_SHA256_HEX_CAP];
    char routing_digest[YVEX_SHA256_HEX_CAP];
    char execution_identity[YVEX_SHA256_HEX_CAP];
} yvex_moe_row_batch_result;

/* include/yvex/internal/execution.h:56-71,79-84,108-112: the classes a physical-execution
 * decision names. */
typedef enum {
    YVEX_EXECUTION_CONSUMER_EMBEDDING = 0,
    YVEX_EXECUTION_CONSUMER_ATTENTION_PROJECTION,
    YVEX_EXECUTION_CONSUMER_ATTENTION_STATE,
    YVEX_EXECUTION_CONSUMER_MOE_ROUTER,
    YVEX_EXECUTION_CONSUMER_ROUTED_GATE_UP,
    YVEX_EXECUTION_CONSUMER_ROUTED_DOWN,
    YVEX_EXECUTION_CONSUMER_SHARED_EXPERT,
    YVEX_EXECUTION_CONSUMER_FINAL_NORMALIZATION,
    YVEX_EXECUTION_CONSUMER_OUTPUT_HEAD,
    YVEX_EXECUTION_CONSUMER_DRAFT_FEATURE_PROJECTION,
    YVEX_EXECUTION_CONSUMER_DRAFT_BACKBONE,
    YVEX_EXECUTION_CONSUMER_MARKOV,
    YVEX_EXECUTION_CONSUMER_CONFIDENCE,
    YVEX_EXECUTION_CONSUMER_COUNT
} yvex_execution_consumer_class;

#define YVEX_EXECUTION_TEXT_CAP 64u

/* include/yvex/internal/execution.h:129-155, field for field (the tensor role and scope, the
 * placement, sharing, backend-requirement and evidence classes are plain enums there and are
 * carried as int here: the layout functions never read them). */
typedef struct {
    unsigned int schema_version;
    unsigned long long terminal_tensor_id;
    int role, scope;
    unsigned long long layer_index, predictor_index, expert_count;
    unsigned int canonical_qtype;
    unsigned long long canonical_row_width, canonical_row_count;
    unsigned long long encoded_offset, encoded_bytes, alignment;
    yvex_execution_consumer_class consumer;
    yvex_execution_layout_class layout;
    int placement, sharing;
    yvex_execution_activation_class activation;
    unsigned long long supported_width_mask, maximum_context, worklist_width_mask;
    unsigned long long tensor_core_minimum;
    int required_backend;
    unsigned int required_compute_major, required_compute_minor;
    int evidence;
    yvex_execution_class fallback;
    int derived_asset_required;
    char kernel_family[YVEX_EXECUTION_TEXT_CAP];
    char tensor_core_kernel_family[YVEX_EXECUTION_TEXT_CAP];
    char terminal_identity[YVEX_SHA256_HEX_CAP];
    char decision_identity[YVEX_SHA256_HEX_CAP];
} yvex_physical_execution_decision;
#endif

/* moe.h:277-297. execute_rows follows src/backend/cuda/moe.c:1826-1923: with mixing rows in the
 * layer plan it runs the residual-stream ingress (mixing projection, gates, Sinkhorn matrix,
 * weighted RMS norm; moe.c:1210-1254), the experts on the normalised rows and the egress onto the
 * streams (moe.c:1533-1541); rows are then row_count x expanded_width. Without mixing rows the
 * rows are taken as normalised hidden rows and the output is bf16(routed + shared).
 * derived_layout_plan/build replace yvex_cuda_moe_derived_layout_plan/build
 * (src/backend/cuda/layout.c:95-167): the storage size and the deterministic re-packing of one
 * routed expert tensor, as host byte work over the caller's buffers. IQ2_XXS: the two scale bytes
 * of every superblock in block order, then (from the next multiple of 64) its 64 code bytes in
 * block order. Q2_K: per pair of neighbouring rows of one expert and block, 8 bytes (d, dmin of
 * the even row, then of the odd row), then from a 64-aligned offset 32 bytes of sub-block scales
 * (two halves of 16: even row's 8 bytes, odd row's 8 bytes), then from a 64-aligned offset 128
 * code bytes (the rows' 4-byte words interleaved). Padding is zero. A decision whose
 * kernel_family is YVEX_MOE_KERNEL_GFX950_EXPERT_SWEEP asks for this backend's own image of an
 * IQ2_XXS tensor instead (routed or shared expert): 72 bytes per superblock in block order, two
 * records of nine little-endian dwords, one per half superblock {fp16 superblock scale | the four
 * 4-bit group scales << 16; then per group of 32 weights its four codebook indices and its four
 * 7-bit sign fields, one to a byte}. The reference's row-batch path refuses every
 * DERIVED_BACKEND view (moe.c:939-958); execute_rows here runs that one image (IQ2_XXS,
 * device-encoded activations, the sweep family on gate, up and down) on the decode sweeps and on
 * the matrix-core kernels, and answers UNSUPPORTED for any other derived view. Q2_K down rows
 * have no image: canonical Q2_K down rows beside imaged IQ2_XXS gate and up rows are admitted,
 * the one pairing of layouts that need not agree. */
typedef struct {
    int (*derived_layout_plan)(const yvex_physical_execution_decision *decision,
                               unsigned long long *storage_bytes, yvex_error *err);
    int (*derived_layout_build)(const yvex_physical_execution_decision *decision,
                                const unsigned char *canonical,
                                unsigned long long canonical_bytes, unsigned char *derived,
                                unsigned long long storage_bytes, yvex_error *err);
    int (*workspace_required)(const yvex_moe_layer_plan *layer, unsigned long long row_count,
                              unsigned long long *bytes, yvex_error *err);
    /*
     * One MoE layer over an ordered row batch (replaces moe_cuda_execute_rows,
     * src/backend/cuda/moe.c:1826-1923): router projection, scoring and top-k, expert-major
     * worklist, routed experts (gate/up -> clamped SwiGLU -> bf16 -> down -> bf16, summed in rank
     * order), shared expert, combined = bf16(routed + shared) into batch->device_outputs.
     * Without mixing rows batch->device_rows holds the already normalised hidden rows
     * [row_count, hidden_width]; with them, the residual streams [row_count, expanded_width].
     * Mandatory refusals kept from the reference: row count outside
     * worklist_policy->supported_width_mask -> UNSUPPORTED before anything is touched
     * (moe.c:1840-1862); gate/up activation or kernel family disagreement -> FORMAT
     * (moe.c:923-928); unknown kernel family -> UNSUPPORTED (moe.c:961-969); workspace missing or
     * too small -> NOMEM; cancellation -> CANCELLED; non-finite numerics -> FORMAT.
     */
    int (*execute_rows)(yvex_rocm_backend *backend, const yvex_moe_layer_job *job,
                        const yvex_moe_row_batch *batch, const yvex_moe_row_batch_output *output,
                        yvex_moe_row_batch_result *result, yvex_error *err);
    /* The barrier of batches whose jobs asked for deferred completion
     * (job->device_completion->defer; src/runtime/moe.c:1567-1576 closes a phase's layers with one
     * call): synchronises the backend's stream and reports what any of them raised (non-finite
     * numerics -> FORMAT, a kernel's contract check -> BACKEND). The kernels' status word is
     * cleared when a phase starts, not between its batches, so a failure of an early batch is
     * still there at the barrier; an operation run between deferred batches reports it as its own. */
    int (*complete_rows)(yvex_rocm_backend *backend, int barrier_observed,
                         yvex_moe_row_batch_result *result, yvex_error *err);
} yvex_rocm_moe_operations;

/* The two layout entries of the table above, callable without a backend (they touch no device):
 * replace yvex_cuda_moe_derived_layout_plan/build, src/backend/cuda/private.h:400-402. */
int yvex_rocm_moe_derived_layout_plan(const yvex_physical_execution_decision *decision,
                                      unsigned long long *storage_bytes, yvex_error *err);
int yvex_rocm_moe_derived_layout_build(const yvex_physical_execution_decision *decision,
                                       const unsigned char *canonical,
                                       unsigned long long canonical_bytes, unsigned char *derived,
                                       unsigned long long storage_bytes, yvex_error *err);

/* No counterpart in the reference, whose residency step builds derived storage on the host and
 * uploads it (src/runtime/residency.c:457-600): the image a gfx950-sweep decision asks for, of a
 * tensor whose canonical bytes are on the device already, built there. decision is what
 * derived_layout_plan took; canonical_address holds decision->encoded_bytes, image_address
 * storage_bytes (dword-aligned, no overlap). Synchronous on the backend's stream. A view of the
 * result carries layout DERIVED_BACKEND, the family YVEX_MOE_KERNEL_GFX950_EXPERT_SWEEP,
 * activation DEVICE_ENCODED, the canonical row geometry and encoded_bytes, storage_bytes, and the
 * image's device_address (or `encoded` inside the attached arena). execute_rows runs such experts
 * on the decode sweeps and, for wide batches, on the matrix-core kernels, both of which read the
 * image: it can be the only resident form of the experts. Every other operation takes canonical
 * rows (UNSUPPORTED). */
int yvex_rocm_moe_sweep_image_build_resident(yvex_rocm_backend *backend,
                                             const yvex_physical_execution_decision *decision,
                                             unsigned long long canonical_address,
                                             unsigned long long image_address,
                                             unsigned long long storage_bytes, yvex_error *err);

/* The workspace_required entry of the table below, callable without a backend (it depends on
 * the layer plan and the row count alone). */
int yvex_rocm_moe_workspace_required(const yvex_moe_layer_plan *layer, unsigned long long row_count,
                                     unsigned long long *bytes, yvex_error *err);

/* moe.h:295-296: NULL unless the backend is ROCM and its kernels are loadable. */
const yvex_rocm_moe_operations *yvex_rocm_backend_moe_operations_get(const yvex_rocm_backend *backend);

/* ---- GGUF tensor directory and resident loading: include/yvex/gguf.h:142-195 ------------------- */

#ifndef YVEX_ROCM_REFERENCE_TYPES
#define YVEX_GGUF_MAX_DIMS 4u

/* include/yvex/gguf.h:142-154 */
typedef struct {
    const char *name;
    unsigned long long name_len;
    unsigned int rank;
    unsigned long long dims[YVEX_GGUF_MAX_DIMS];
    unsigned int ggml_type;
    const char *ggml_type_name;
    unsigned long long relative_offset, absolute_offset, storage_bytes, absolute_end_offset;
    int range_addressable;
} yvex_gguf_tensor_info;
#endif

typedef struct yvex_rocm_gguf yvex_rocm_gguf;

/* Structural reader with the rules and refusal codes of the reference's yvex_gguf_open
 * (src/gguf/core.c:1163-1249, :52-79): version 3 only (UNSUPPORTED), bad magic / rank / dimension
 * / alignment / key grammar / duplicate names (FORMAT), truncation and extents beyond the file
 * (BOUNDS), qtypes without storage geometry (UNSUPPORTED). It takes a path where the reference
 * takes its artifact handle. Scalar and string metadata are kept; arrays are walked and dropped. */
int yvex_rocm_gguf_open_path(yvex_rocm_gguf **out, const char *path, yvex_error *err);
void yvex_rocm_gguf_close(yvex_rocm_gguf *gguf);
unsigned long long yvex_rocm_gguf_metadata_count(const yvex_rocm_gguf *gguf);
int yvex_rocm_gguf_metadata_u64(const yvex_rocm_gguf *gguf, const char *key, unsigned long long *out);
int yvex_rocm_gguf_metadata_f64(const yvex_rocm_gguf *gguf, const char *key, double *out);
int yvex_rocm_gguf_metadata_string(const yvex_rocm_gguf *gguf, const char *key, const char **text,
                              unsigned long long *len);
unsigned long long yvex_rocm_gguf_tensor_count(const yvex_rocm_gguf *gguf);
const yvex_gguf_tensor_info *yvex_rocm_gguf_tensor_at(const yvex_rocm_gguf *gguf, unsigned long long index);
const yvex_gguf_tensor_info *yvex_rocm_gguf_tensor_find(const yvex_rocm_gguf *gguf, const char *name);
unsigned long long yvex_rocm_gguf_tensor_data_offset(const yvex_rocm_gguf *gguf);
unsigned int yvex_rocm_gguf_alignment(const yvex_rocm_gguf *gguf);
unsigned long long yvex_rocm_gguf_file_size(const yvex_rocm_gguf *gguf);

/* The reference's runtime maps an artifact's tensor-data section into the resident arena and
 * hands the backend borrowed pointers into it (src/runtime/residency.c, contract text
 * include/yvex/internal/backend.h:283-288). Here: one resident arena of the section's size, the
 * bytes read from the file into its host shadow, one attach (the upload to HBM). A weight view
 * of a named tensor is then host_base + relative_offset with rows of dims[0] values; tensors of
 * rank 3 are expert-major (rows = dims[1] * dims[2]). The view's activation class and kernel
 * family are the caller's to set. */
int yvex_rocm_gguf_resident_load(yvex_rocm_backend *backend, const yvex_rocm_gguf *gguf,
                                         unsigned long long generation, yvex_device_tensor **arena,
                                         unsigned char **host_base, yvex_error *err);
int yvex_rocm_gguf_weight_view(const yvex_rocm_gguf *gguf, const unsigned char *host_base,
                                       const char *name, yvex_moe_weight_view *view, yvex_error *err);

/* ---- token-local MoE operation: include/yvex/internal/moe.h:161-166,198-214,308-319 ------------ */

#ifndef YVEX_ROCM_REFERENCE_TYPES
#define YVEX_RUNTIME_DESCRIPTOR_QTYPE_CAP 43u
#define YVEX_ATTENTION_EVIDENCE_FULL 3      /* include/yvex/internal/graph.h:250-255 */

typedef struct {
    unsigned long long selected_count;
    unsigned long long selected_experts[YVEX_MOE_MAX_SELECTED];
    float router_logits[256], router_scores[256];
    float selected_weights[YVEX_MOE_MAX_SELECTED];
} yvex_moe_router_result;

typedef struct {
    float *combined_output, *post, *combination;
    unsigned long long combined_capacity, post_capacity, combination_capacity;
    float *routed_output, *shared_output;
    unsigned long long routed_capacity, shared_capacity;
    yvex_moe_router_result router;
    unsigned long long expert_subviews_accessed, encoded_bytes_read;
    unsigned long long host_to_device_bytes, device_to_host_bytes, kernel_launches;
    unsigned long long cache_hits, cache_misses, upload_count, download_count;
    unsigned long long stream_synchronizations, device_synchronizations, device_to_device_bytes;
    yvex_execution_memory_facts memory;
    unsigned long long ingress_ns, routing_ns, routed_ns, shared_ns, post_ns, total_ns;
    unsigned long long synchronization_ns;
    unsigned long long qtype_counts[YVEX_RUNTIME_DESCRIPTOR_QTYPE_CAP];
    char routed_digest[YVEX_SHA256_HEX_CAP], shared_digest[YVEX_SHA256_HEX_CAP];
    char combined_digest[YVEX_SHA256_HEX_CAP], routing_digest[YVEX_SHA256_HEX_CAP];
} yvex_moe_layer_result;
#endif

/* One row, experts handed over one at a time by a caller that loads them on demand
 * (src/backend/cuda/moe.c:516-842; the caller is src/runtime/moe.c:647-720).
 *
 * begin: uploads job->expanded_input (or copies job->device_input), runs the residual-stream
 *   ingress and the router, and publishes result->router (logits and scores unless a device
 *   output is named and evidence is below FULL). When job->device_output is set, evidence is
 *   below FULL and the three routed weight views carry a device_address, the selected experts
 *   run on the device at once and the caller adds the shared expert only (the caller applies
 *   the same rule, src/runtime/moe.c:654-660).
 * add_expert: intermediate = bf16(silu(min(g, L)) * clamp(u, +-L) * weight) with weight 1 for the
 *   shared expert, output = bf16(down . intermediate), kept for the rank-ordered sum (at most
 *   YVEX_MOE_MAX_SELECTED routed experts). Weight views outside the resident arena are uploaded
 *   to a staging range owned by the execution.
 * finish: routed = sum in the order added, combined = bf16(routed + shared); with a device
 *   output the egress writes it; host copies as moe.c:775-803 publishes them.
 * close: releases the execution (safe on NULL). A kernel status other than zero surfaces as
 * BACKEND, as moe.c:277-296 reports it. */
typedef struct yvex_rocm_moe_execution yvex_rocm_moe_execution;
int yvex_rocm_backend_moe_begin(yvex_rocm_moe_execution **out, yvex_rocm_backend *backend,
                           const yvex_moe_layer_job *job, yvex_moe_layer_result *result,
                           yvex_error *err);
int yvex_rocm_backend_moe_add_expert(yvex_rocm_moe_execution *execution,
                                const yvex_moe_weight_view *gate, const yvex_moe_weight_view *up,
                                const yvex_moe_weight_view *down, float route_weight, int shared,
                                yvex_error *err);
int yvex_rocm_backend_moe_finish(yvex_rocm_moe_execution *execution, yvex_moe_layer_result *result,
                            yvex_error *err);
int yvex_rocm_backend_moe_close(yvex_rocm_moe_execution **execution, yvex_error *err);

/* Largest row batch execute_rows accepts in one call. */
#define YVEX_ROCM_MOE_MAX_ROWS 4096ull

/* ---- expert worklist on the host: include/yvex/internal/execution_batch.h:95-169 ----------- */

#ifndef YVEX_ROCM_REFERENCE_TYPES
typedef struct {
    unsigned long long *expert_ids, *bucket_offsets, *bucket_populations;
    unsigned long long *source_pairs, *source_rows, *destination_rows;
    float *route_weights;
    unsigned long long bucket_capacity, pair_capacity;
} yvex_expert_worklist_storage;
#endif

/* Replaces the sorting core of yvex_expert_worklist_build (src/graph/worklist.c:369-441):
 * stable counting sort of pairs by expert. bucket_offsets needs bucket_capacity + 1 entries.
 * An expert ordinal >= expert_count or a non-finite weight -> FORMAT; storage too small or
 * pair_count not a multiple of experts_per_row -> INVALID_ARG. */
int yvex_rocm_expert_worklist_build(const unsigned long long *selected_experts,
                               const float *route_weights, unsigned long long pair_count,
                               unsigned long long experts_per_row,
                               unsigned long long expert_count,
                               const yvex_expert_worklist_storage *storage,
                               yvex_expert_worklist_observation *observation, yvex_error *err);

#ifdef __cplusplus
}
#endif
#endif
