"""ctypes mirror of include/yvex_rocm.h: the structures and entry points of the C11 backend.

Field order follows the header one to one. Nothing here computes; it only lets Python callers
(the tests, which read like the reference's unit tests) reach the C ABI.
"""
from __future__ import annotations

import ctypes as C

from . import load_library

OK, ERR, NOMEM, IO, FORMAT, UNSUPPORTED, BACKEND, BOUNDS, STATE, CANCELLED, INVALID_ARG, TIMEOUT = \
    0, -1, -2, -3, -4, -5, -6, -7, -8, -9, -10, -11
KIND_CPU, KIND_CUDA, KIND_METAL, KIND_ROCM = 0, 1, 2, 3
STATUS_READY, STATUS_CONTEXT_READY, STATUS_UNSUPPORTED, STATUS_FAILED = 0, 1, 2, 3
DTYPE_F32, DTYPE_I8, DTYPE_I32 = 1, 5, 7
VARIANT_TENSOR_ALLOC, VARIANT_QTYPE_ROW_DOT, VARIANT_ATTENTION_ENCODED = 0, 15, 16
CAP_UNSUPPORTED, CAP_SUPPORTED, CAP_FAILED = 0, 1, 2
REASON_NONE, REASON_KERNEL_BUNDLE_ABSENT, REASON_VARIANT_UNSUPPORTED = 0, 4, 7
RESIDENT_INVALID, RESIDENT_MISS, RESIDENT_HIT = -1, 0, 1
ROUTER_HASH, ROUTER_LEARNED = 0, 1
SCORING_SQRT_SOFTPLUS, SCORING_SIGMOID = 0, 1
LAYOUT_CANONICAL_ROW, LAYOUT_EXPERT_MAJOR, LAYOUT_DERIVED = 0, 2, 3
ACT_HOST_F32, ACT_DEVICE_F32, ACT_DEVICE_F16, ACT_DEVICE_ENCODED = 0, 1, 2, 3
BATCH_MULTI_SESSION, BATCH_PREFILL = 2, 3
W_FFN_NORM, W_MHC_FUNCTION, W_MHC_BASE, W_MHC_SCALE, W_ROUTER, W_ROUTER_TABLE, W_ROUTER_BIAS, \
    W_ROUTED_GATE, W_ROUTED_UP, W_ROUTED_DOWN, W_SHARED_GATE, W_SHARED_UP, W_SHARED_DOWN, W_COUNT = range(14)
FAMILY_PORTABLE_EXPERT_ROW = b"portable-expert-row"
FAMILY_GFX950 = b"gfx950-int8-dot-expert-sweep"
FAMILY_GFX950_MATRIX_CORE = b"gfx950-int8-matrix-core-expert"
HEX = 65
ULL = C.c_ulonglong


class Error(C.Structure):
    _fields_ = [("code", C.c_int), ("where", C.c_char * 96), ("message", C.c_char * 256)]


class BackendOptions(C.Structure):
    _fields_ = [("kind", C.c_int), ("device", C.c_char_p), ("memory_limit_bytes", ULL)]


class MemoryStats(C.Structure):
    _fields_ = [(n, ULL) for n in ("allocated_bytes", "allocation_count", "allocation_events",
                                   "release_events", "h2d_bytes", "d2h_bytes",
                                   "peak_allocated_bytes", "memory_limit_bytes")]


class BandwidthEvidence(C.Structure):
    _fields_ = [("schema_version", C.c_uint), ("working_set_bytes", ULL), ("iterations", ULL),
                ("sample_count", ULL), ("stream_elapsed_ns", ULL * 5), ("copy_elapsed_ns", ULL * 5),
                ("coherent_host_elapsed_ns", ULL * 5), ("sustainable_read_bytes_per_second", ULL),
                ("sustainable_copy_bytes_per_second", ULL),
                ("sustainable_coherent_host_bytes_per_second", ULL),
                ("kernel_bundle_identity", C.c_char * 65), ("identity", C.c_char * 65)]


class TensorDesc(C.Structure):
    _fields_ = [("name", C.c_char_p), ("dtype", C.c_int), ("rank", C.c_uint), ("dims", ULL * 4),
                ("bytes", ULL)]


class DeviceTensor(C.Structure):
    _fields_ = [("owner", C.c_void_p), ("owner_id", ULL), ("name", C.c_char_p), ("dtype", C.c_int),
                ("rank", C.c_uint), ("dims", ULL * 4), ("bytes", ULL), ("data", C.c_void_p),
                ("host_data", C.c_void_p), ("backend_allocation", C.c_void_p),
                ("resident_bytes", ULL), ("virtual_reserved", C.c_int), ("is_written", C.c_int),
                ("host_accessible", C.c_int), ("borrowed_host", C.c_int)]


class CapabilityResult(C.Structure):
    _fields_ = [("backend_kind", C.c_int), ("variant", C.c_int), ("state", C.c_int),
                ("reason", C.c_int), ("input_dtype", C.c_int), ("weight_dtype", C.c_int),
                ("output_dtype", C.c_int), ("context_available", C.c_int),
                ("kernel_bundle_available", C.c_int), ("function_available", C.c_int)]


class OperationFacts(C.Structure):
    _fields_ = [(n, ULL) for n in ("h2d_bytes", "d2h_bytes", "d2d_bytes", "kernel_launches",
                                   "upload_count", "download_count", "stream_synchronizations",
                                   "device_synchronizations", "active_weight_bytes", "state_bytes",
                                   "activation_bytes", "temporary_bytes", "tensor_core_launches")] + \
               [("compulsory_memory_facts_available", C.c_int)]


class QtypeGeometry(C.Structure):
    _fields_ = [("qtype", C.c_uint), ("name", C.c_char_p), ("identity", C.c_int),
                ("block_size", C.c_uint), ("bytes_per_block", C.c_uint)]


class NumericCapability(C.Structure):
    _fields_ = [("qtype", C.c_uint), ("known", C.c_int), ("storage_admitted", C.c_int),
                ("reference_decoder_available", C.c_int),
                ("dedicated_cpu_compute_available", C.c_int), ("device_compute_available", C.c_int),
                ("extension_of_reference", C.c_int), ("refusal", C.c_int)]


class WeightView(C.Structure):
    _fields_ = [("tensor_id", ULL), ("expert_index", ULL), ("role", C.c_int), ("qtype", C.c_uint),
                ("layout", C.c_int), ("activation", C.c_int), ("kernel_family", C.c_char_p),
                ("encoded", C.c_void_p), ("encoded_bytes", C.c_size_t), ("storage_bytes", C.c_size_t),
                ("row_bytes", ULL), ("row_width", ULL), ("row_count", ULL), ("device_address", ULL)]


class LayerPlan(C.Structure):
    _fields_ = [("schema_version", C.c_uint), ("ordinal", ULL), ("layer_index", ULL),
                ("predictor_index", ULL), ("tensor_scope", C.c_int), ("router_class", C.c_int),
                ("scoring", C.c_int), ("topk_policy", C.c_int), ("activation", C.c_int),
                ("hidden_width", ULL), ("residual_streams", ULL), ("expanded_width", ULL),
                ("mhc_mixing_rows", ULL), ("mhc_sinkhorn_iterations", ULL),
                ("routed_experts", ULL), ("shared_experts", ULL), ("experts_per_token", ULL),
                ("expert_intermediate_width", ULL), ("shared_intermediate_width", ULL),
                ("hash_table_rows", ULL), ("hash_table_columns", ULL), ("correction_bias_width", ULL),
                ("rms_epsilon", C.c_double), ("mhc_epsilon", C.c_double),
                ("mhc_post_multiplier", C.c_double), ("routed_scaling_factor", C.c_double),
                ("activation_limit", C.c_double), ("requires_token_ids", C.c_int),
                ("requires_correction_bias", C.c_int), ("normalize_topk_probabilities", C.c_int),
                ("tensor_ids", ULL * W_COUNT), ("qtypes", C.c_uint * W_COUNT),
                ("layer_identity", C.c_char * HEX)]


class WorklistPolicy(C.Structure):
    _fields_ = [("schema_version", C.c_uint), ("supported_width_mask", ULL),
                ("tensor_core_minimum", ULL), ("narrow_kernel_family", C.c_char * 64),
                ("tensor_core_kernel_family", C.c_char * 64), ("identity", C.c_char * HEX)]


class ExecutionBatch(C.Structure):
    _fields_ = [("schema_version", C.c_uint), ("provenance", C.c_int), ("phase", C.c_uint),
                ("row_count", ULL), ("source_count", ULL), ("model_generation", ULL),
                ("sources", C.c_void_p), ("rows", C.c_void_p)] + \
               [(n, C.c_char * HEX) for n in ("runtime_model_identity", "runtime_binding_identity",
                                              "physical_variant_identity", "execution_profile_identity",
                                              "operation_identity", "identity")]


class WorklistObservation(C.Structure):
    _fields_ = [("schema_version", C.c_uint), ("worklist_count", ULL), ("pair_count", ULL),
                ("bucket_count", ULL), ("maximum_bucket_population", ULL),
                ("tensor_core_eligible_pairs", ULL), ("tensor_core_executed_pairs", ULL),
                ("narrow_pairs", ULL), ("tail_rows", ULL), ("width_histogram", ULL * 17),
                ("population_histogram", ULL * 17), ("provenance_counts", ULL * 5)]


class MemoryFacts(C.Structure):
    _fields_ = [(n, ULL) for n in ("active_weight_bytes", "state_bytes", "activation_bytes",
                                   "temporary_bytes", "measured_operations", "missing_operations")] + \
               [("complete", C.c_int)]


class DeviceCompletion(C.Structure):
    _fields_ = [("defer", C.c_int), ("host", C.c_void_p)]


CANCEL_FN = C.CFUNCTYPE(C.c_int, C.c_void_p)


class LayerJob(C.Structure):
    _fields_ = [("layer", C.POINTER(LayerPlan)), ("weights", WeightView * W_COUNT),
                ("expanded_input", C.c_void_p), ("device_input", C.c_void_p),
                ("device_output", C.c_void_p), ("token_id", C.c_uint), ("token_id_present", C.c_int),
                ("cancel_requested", CANCEL_FN), ("cancel_context", C.c_void_p),
                ("evidence_level", C.c_int), ("eager_execution", C.c_int),
                ("device_completion", C.POINTER(DeviceCompletion)),
                ("execution_batch", C.POINTER(ExecutionBatch)),
                ("worklist_policy", C.POINTER(WorklistPolicy))]


class GgufTensorInfo(C.Structure):
    _fields_ = [("name", C.c_char_p), ("name_len", ULL), ("rank", C.c_uint), ("dims", ULL * 4),
                ("ggml_type", C.c_uint), ("ggml_type_name", C.c_char_p), ("relative_offset", ULL),
                ("absolute_offset", ULL), ("storage_bytes", ULL), ("absolute_end_offset", ULL),
                ("range_addressable", C.c_int)]


class RouterResult(C.Structure):
    _fields_ = [("selected_count", ULL), ("selected_experts", ULL * 16),
                ("router_logits", C.c_float * 256), ("router_scores", C.c_float * 256),
                ("selected_weights", C.c_float * 16)]


class LayerResult(C.Structure):
    _fields_ = [("combined_output", C.c_void_p), ("post", C.c_void_p), ("combination", C.c_void_p),
                ("combined_capacity", ULL), ("post_capacity", ULL), ("combination_capacity", ULL),
                ("routed_output", C.c_void_p), ("shared_output", C.c_void_p),
                ("routed_capacity", ULL), ("shared_capacity", ULL), ("router", RouterResult)] + \
               [(n, ULL) for n in ("expert_subviews_accessed", "encoded_bytes_read", "host_to_device_bytes",
                                   "device_to_host_bytes", "kernel_launches", "cache_hits", "cache_misses",
                                   "upload_count", "download_count", "stream_synchronizations",
                                   "device_synchronizations", "device_to_device_bytes")] + \
               [("memory", MemoryFacts)] + \
               [(n, ULL) for n in ("ingress_ns", "routing_ns", "routed_ns", "shared_ns", "post_ns",
                                   "total_ns", "synchronization_ns")] + \
               [("qtype_counts", ULL * 43)] + \
               [(n, C.c_char * HEX) for n in ("routed_digest", "shared_digest", "combined_digest",
                                              "routing_digest")]


class RowBatch(C.Structure):
    _fields_ = [("schema_version", C.c_uint), ("row_count", ULL), ("row_width", ULL),
                ("row_stride", ULL), ("expanded_rows", C.c_void_p),
                ("device_rows", C.POINTER(DeviceTensor)), ("device_outputs", C.POINTER(DeviceTensor)),
                ("token_ids", C.c_void_p), ("token_ids_present", C.c_int), ("provenance", C.c_int),
                ("phase", C.c_uint), ("execution_class", C.c_int),
                ("execution_profile_identity", C.c_char_p), ("execution_sources", C.c_void_p),
                ("execution_rows", C.c_void_p), ("execution_source_count", ULL),
                ("complete_after_operation", C.c_int)]


class RowBatchOutput(C.Structure):
    _fields_ = [("combined_rows", C.c_void_p), ("routed_rows", C.c_void_p),
                ("shared_rows", C.c_void_p), ("post_rows", C.c_void_p),
                ("combination_rows", C.c_void_p), ("combined_capacity", ULL),
                ("routed_capacity", ULL), ("shared_capacity", ULL), ("post_capacity", ULL),
                ("combination_capacity", ULL), ("selected_experts", C.c_void_p),
                ("selected_weights", C.c_void_p), ("selection_capacity", ULL)]


class RowBatchResult(C.Structure):
    _fields_ = [("schema_version", C.c_uint), ("completed", C.c_int),
                ("execution_profile_available", C.c_int), ("device_completion_pending", C.c_int),
                ("execution_class", C.c_int), ("row_count", ULL), ("row_expert_pairs", ULL),
                ("unique_experts", ULL), ("worklists", WorklistObservation)] + \
               [(n, ULL) for n in ("grouped_expert_operations", "shared_expert_operations",
                                   "expert_subviews_accessed", "encoded_bytes_read", "h2d_bytes",
                                   "d2h_bytes", "d2d_bytes", "kernel_launches",
                                   "tensor_core_launches", "graph_launches", "graph_captures",
                                   "graph_replays", "upload_count", "download_count", "cache_hits",
                                   "cache_misses", "stream_synchronizations",
                                   "device_synchronizations", "active_weight_base_bytes",
                                   "active_weight_per_unique_expert_bytes")] + \
               [("memory", MemoryFacts), ("total_ns", ULL), ("synchronization_ns", ULL)] + \
               [(n, C.c_char * HEX) for n in ("execution_profile_identity",
                                              "execution_batch_identity", "worklist_policy_identity",
                                              "expert_worklist_identity", "routing_digest",
                                              "execution_identity")]


class ExecutionDecision(C.Structure):
    """yvex_physical_execution_decision, include/yvex/internal/execution.h:129-155."""
    _fields_ = [("schema_version", C.c_uint), ("terminal_tensor_id", ULL), ("role", C.c_int),
                ("scope", C.c_int), ("layer_index", ULL), ("predictor_index", ULL), ("expert_count", ULL),
                ("canonical_qtype", C.c_uint), ("canonical_row_width", ULL), ("canonical_row_count", ULL),
                ("encoded_offset", ULL), ("encoded_bytes", ULL), ("alignment", ULL),
                ("consumer", C.c_int), ("layout", C.c_int), ("placement", C.c_int), ("sharing", C.c_int),
                ("activation", C.c_int), ("supported_width_mask", ULL), ("maximum_context", ULL),
                ("worklist_width_mask", ULL), ("tensor_core_minimum", ULL), ("required_backend", C.c_int),
                ("required_compute_major", C.c_uint), ("required_compute_minor", C.c_uint),
                ("evidence", C.c_int), ("fallback", C.c_int), ("derived_asset_required", C.c_int),
                ("kernel_family", C.c_char * 64), ("tensor_core_kernel_family", C.c_char * 64),
                ("terminal_identity", C.c_char * HEX), ("decision_identity", C.c_char * HEX)]


CONSUMER_ROUTED_GATE_UP, CONSUMER_ROUTED_DOWN, CONSUMER_SHARED_EXPERT = 4, 5, 6


class MoeOperations(C.Structure):
    _fields_ = [
        ("derived_layout_plan", C.CFUNCTYPE(C.c_int, C.POINTER(ExecutionDecision), C.POINTER(ULL),
                                            C.POINTER(Error))),
        ("derived_layout_build", C.CFUNCTYPE(C.c_int, C.POINTER(ExecutionDecision), C.c_void_p, ULL, C.c_void_p, ULL,
                                             C.POINTER(Error))),
        ("workspace_required", C.CFUNCTYPE(C.c_int, C.POINTER(LayerPlan), ULL, C.POINTER(ULL),
                                           C.POINTER(Error))),
        ("execute_rows", C.CFUNCTYPE(C.c_int, C.c_void_p, C.POINTER(LayerJob), C.POINTER(RowBatch),
                                     C.POINTER(RowBatchOutput), C.POINTER(RowBatchResult),
                                     C.POINTER(Error))),
        ("complete_rows", C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.POINTER(RowBatchResult),
                                      C.POINTER(Error))),
    ]


class WorklistStorage(C.Structure):
    _fields_ = [("expert_ids", C.c_void_p), ("bucket_offsets", C.c_void_p),
                ("bucket_populations", C.c_void_p), ("source_pairs", C.c_void_p),
                ("source_rows", C.c_void_p), ("destination_rows", C.c_void_p),
                ("route_weights", C.c_void_p), ("bucket_capacity", ULL), ("pair_capacity", ULL)]


# Every symbol include/yvex_rocm.h declares; the CPU test suite checks the library exports all.
EXPORTS = [
    "yvex_rocm_status_name", "yvex_rocm_error_clear", "yvex_rocm_error_set", "yvex_rocm_error_is_set", "yvex_rocm_error_code",
    "yvex_rocm_gguf_qtype_geometry_find", "yvex_rocm_quant_numeric_capability_at",
    "yvex_rocm_backend_open", "yvex_rocm_backend_bind_owner", "yvex_rocm_backend_close_checked", "yvex_rocm_backend_open_shared", "yvex_rocm_backend_kind_of",
    "yvex_rocm_backend_status_of", "yvex_rocm_backend_get_memory_stats", "yvex_rocm_backend_sync",
    "yvex_rocm_backend_query_capability", "yvex_rocm_backend_bandwidth_probe", "yvex_rocm_backend_tensor_alloc", "yvex_rocm_backend_tensor_release",
    "yvex_rocm_backend_tensor_write", "yvex_rocm_backend_tensor_read", "yvex_rocm_backend_tensor_copy",
    "yvex_rocm_backend_tensor_owned_by", "yvex_rocm_backend_resident_alloc", "yvex_rocm_backend_resident_prefetch",
    "yvex_rocm_backend_resident_attach", "yvex_rocm_backend_resident_detach", "yvex_rocm_backend_resident_resolve",
    "yvex_rocm_backend_workspace_attach", "yvex_rocm_backend_workspace_detach",
    "yvex_rocm_backend_workspace_acquire", "yvex_rocm_encoded_matvec",
    "yvex_rocm_encoded_gather", "yvex_rocm_select_greedy_rows", "yvex_rocm_quant_row_dot",
    "yvex_rocm_backend_moe_operations_get", "yvex_rocm_backend_moe_begin", "yvex_rocm_backend_moe_add_expert",
    "yvex_rocm_backend_moe_finish", "yvex_rocm_backend_moe_close",
    "yvex_rocm_expert_worklist_build", "yvex_rocm_moe_derived_layout_plan", "yvex_rocm_moe_derived_layout_build",
    "yvex_rocm_moe_sweep_image_build_resident",
    "yvex_rocm_moe_workspace_required",
    "yvex_rocm_gguf_open_path", "yvex_rocm_gguf_close", "yvex_rocm_gguf_metadata_count", "yvex_rocm_gguf_metadata_u64",
    "yvex_rocm_gguf_metadata_f64", "yvex_rocm_gguf_metadata_string", "yvex_rocm_gguf_tensor_count", "yvex_rocm_gguf_tensor_at",
    "yvex_rocm_gguf_tensor_find", "yvex_rocm_gguf_tensor_data_offset", "yvex_rocm_gguf_alignment", "yvex_rocm_gguf_file_size",
    "yvex_rocm_gguf_resident_load", "yvex_rocm_gguf_weight_view",
]
KERNEL_EXPORTS = [
    "yvex_hip_q8k_quantize", "yvex_hip_concat_rows_bf16", "yvex_hip_row_dot", "yvex_hip_matvec", "yvex_hip_matvec_f32_rows", "yvex_hip_matvec_f32_scratch_bytes", "yvex_hip_matvec_f32_rows_launches", "yvex_hip_matvec_f32_rows_scored", "yvex_hip_block_dots_i32", "yvex_hip_gather",
    "yvex_hip_argmax_f32", "yvex_hip_argmax_scratch_bytes", "yvex_hip_argmax_f32_static",
    "yvex_hip_argmax_static_capacity",
    "yvex_hip_moe_route_rows", "yvex_hip_moe_route_scores", "yvex_hip_moe_route_hash_rows", "yvex_hip_worklist_build", "yvex_hip_moe_prepare", "yvex_hip_moe_prepare_scored",
    "yvex_hip_moe_prepare_supported", "yvex_hip_moe_up", "yvex_hip_moe_down", "yvex_hip_iq2_sweep_image_bytes", "yvex_hip_iq2_sweep_image_build",
    "yvex_hip_moe_up_rows", "yvex_hip_moe_down_rows", "yvex_hip_moe_swiglu_rows",
    "yvex_hip_moe_reduce_combine", "yvex_hip_mhc_ingress", "yvex_hip_mhc_ingress_encoded", "yvex_hip_mhc_egress",
    "yvex_hip_stream_read", "yvex_hip_bandwidth_sample", "yvex_hip_clock_probe", "yvex_hip_fill_u32",
    "yvex_hip_capture_begin", "yvex_hip_capture_end", "yvex_hip_capture_abort", "yvex_hip_graph_launch",
    "yvex_hip_graph_destroy",
    "yvex_hip_device_count", "yvex_hip_device_info", "yvex_hip_device_clocks", "yvex_hip_malloc", "yvex_hip_free",
    "yvex_hip_host_alloc", "yvex_hip_host_free", "yvex_hip_memcpy_h2d", "yvex_hip_memcpy_h2d_queued", "yvex_hip_memcpy_d2h",
    "yvex_hip_memcpy_d2d", "yvex_hip_stream_create", "yvex_hip_stream_destroy",
    "yvex_hip_stream_sync", "yvex_hip_kernels_loadable", "yvex_hip_last_error",
]


def library():
    lib = load_library()
    lib.yvex_rocm_status_name.restype = C.c_char_p
    lib.yvex_rocm_gguf_qtype_geometry_find.restype = C.POINTER(QtypeGeometry)
    lib.yvex_rocm_quant_numeric_capability_at.restype = C.POINTER(NumericCapability)
    lib.yvex_rocm_backend_moe_operations_get.restype = C.POINTER(MoeOperations)
    lib.yvex_rocm_backend_moe_operations_get.argtypes = [C.c_void_p]
    lib.yvex_rocm_quant_row_dot.argtypes = [C.c_void_p, C.c_uint, C.c_void_p, C.c_size_t, C.c_void_p, ULL,
                                            C.POINTER(C.c_float), C.c_void_p, C.POINTER(Error)]
    lib.yvex_rocm_moe_derived_layout_plan.argtypes = [C.POINTER(ExecutionDecision), C.POINTER(ULL),
                                                      C.POINTER(Error)]
    lib.yvex_rocm_moe_derived_layout_build.argtypes = [C.POINTER(ExecutionDecision), C.c_void_p, ULL,
                                                       C.c_void_p, ULL, C.POINTER(Error)]
    lib.yvex_rocm_moe_sweep_image_build_resident.argtypes = [C.c_void_p, C.POINTER(ExecutionDecision), ULL, ULL,
                                                             ULL, C.POINTER(Error)]
    lib.yvex_rocm_gguf_open_path.argtypes = [C.POINTER(C.c_void_p), C.c_char_p, C.POINTER(Error)]
    lib.yvex_rocm_gguf_close.argtypes = [C.c_void_p]
    lib.yvex_rocm_gguf_close.restype = None
    for name in ("yvex_rocm_gguf_metadata_count", "yvex_rocm_gguf_tensor_count", "yvex_rocm_gguf_tensor_data_offset",
                 "yvex_rocm_gguf_file_size"):
        getattr(lib, name).argtypes = [C.c_void_p]
        getattr(lib, name).restype = ULL
    lib.yvex_rocm_gguf_alignment.argtypes = [C.c_void_p]
    lib.yvex_rocm_gguf_alignment.restype = C.c_uint
    lib.yvex_rocm_gguf_metadata_u64.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(ULL)]
    lib.yvex_rocm_gguf_metadata_f64.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_double)]
    lib.yvex_rocm_gguf_metadata_string.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_char_p), C.POINTER(ULL)]
    lib.yvex_rocm_gguf_tensor_at.argtypes = [C.c_void_p, ULL]
    lib.yvex_rocm_gguf_tensor_at.restype = C.POINTER(GgufTensorInfo)
    lib.yvex_rocm_gguf_tensor_find.argtypes = [C.c_void_p, C.c_char_p]
    lib.yvex_rocm_gguf_tensor_find.restype = C.POINTER(GgufTensorInfo)
    lib.yvex_rocm_gguf_resident_load.argtypes = [C.c_void_p, C.c_void_p, ULL,
                                                         C.POINTER(C.POINTER(DeviceTensor)),
                                                         C.POINTER(C.c_void_p), C.POINTER(Error)]
    lib.yvex_rocm_gguf_weight_view.argtypes = [C.c_void_p, C.c_void_p, C.c_char_p,
                                                       C.POINTER(WeightView), C.POINTER(Error)]
    lib.yvex_rocm_backend_moe_begin.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.POINTER(LayerJob),
                                           C.POINTER(LayerResult), C.POINTER(Error)]
    lib.yvex_rocm_backend_moe_add_expert.argtypes = [C.c_void_p, C.POINTER(WeightView), C.POINTER(WeightView),
                                                C.POINTER(WeightView), C.c_float, C.c_int, C.POINTER(Error)]
    lib.yvex_rocm_backend_moe_finish.argtypes = [C.c_void_p, C.POINTER(LayerResult), C.POINTER(Error)]
    lib.yvex_rocm_backend_moe_close.argtypes = [C.POINTER(C.c_void_p), C.POINTER(Error)]
    lib.yvex_rocm_backend_open.argtypes = [C.POINTER(C.c_void_p), C.POINTER(BackendOptions), C.POINTER(Error)]
    lib.yvex_rocm_backend_close_checked.argtypes = [C.POINTER(C.c_void_p), C.POINTER(Error)]
    lib.yvex_rocm_backend_open_shared.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, ULL, C.POINTER(Error)]
    lib.yvex_rocm_backend_tensor_alloc.argtypes = [C.c_void_p, C.POINTER(TensorDesc),
                                              C.POINTER(C.POINTER(DeviceTensor)), C.POINTER(Error)]
    lib.yvex_rocm_backend_tensor_release.argtypes = [C.c_void_p, C.POINTER(C.POINTER(DeviceTensor)),
                                                C.POINTER(Error)]
    lib.yvex_rocm_backend_tensor_write.argtypes = [C.c_void_p, C.POINTER(DeviceTensor), C.c_void_p, ULL,
                                              C.POINTER(Error)]
    lib.yvex_rocm_backend_tensor_read.argtypes = [C.c_void_p, C.POINTER(DeviceTensor), C.c_void_p, ULL,
                                             C.POINTER(Error)]
    lib.yvex_rocm_backend_tensor_copy.argtypes = [C.c_void_p, C.POINTER(DeviceTensor),
                                             C.POINTER(DeviceTensor), C.POINTER(Error)]
    lib.yvex_rocm_backend_resident_alloc.argtypes = [C.c_void_p, C.POINTER(TensorDesc),
                                                C.POINTER(C.POINTER(DeviceTensor)),
                                                C.POINTER(C.c_void_p), C.POINTER(Error)]
    lib.yvex_rocm_backend_resident_attach.argtypes = [C.c_void_p, C.c_void_p, ULL, C.POINTER(DeviceTensor),
                                                 ULL, C.POINTER(Error)]
    lib.yvex_rocm_backend_resident_detach.argtypes = [C.c_void_p, C.POINTER(Error)]
    lib.yvex_rocm_backend_resident_resolve.argtypes = [C.c_void_p, C.c_void_p, ULL, C.POINTER(ULL)]
    lib.yvex_rocm_backend_resident_prefetch.argtypes = [C.c_void_p, C.POINTER(DeviceTensor),
                                                   C.POINTER(ULL), C.POINTER(Error)]
    lib.yvex_rocm_backend_workspace_attach.argtypes = [C.c_void_p, C.POINTER(DeviceTensor), ULL,
                                                  C.POINTER(Error)]
    lib.yvex_rocm_backend_workspace_detach.argtypes = [C.c_void_p]
    lib.yvex_rocm_backend_workspace_acquire.argtypes = [C.c_void_p, ULL, ULL, C.POINTER(ULL)]
    lib.yvex_rocm_backend_query_capability.argtypes = [C.c_void_p, C.c_int, C.POINTER(CapabilityResult),
                                                  C.POINTER(Error)]
    lib.yvex_rocm_backend_get_memory_stats.argtypes = [C.c_void_p, C.POINTER(MemoryStats), C.POINTER(Error)]
    lib.yvex_rocm_backend_sync.argtypes = [C.c_void_p, C.POINTER(Error)]
    lib.yvex_rocm_backend_kind_of.argtypes = [C.c_void_p]
    lib.yvex_rocm_backend_status_of.argtypes = [C.c_void_p]
    lib.yvex_rocm_backend_tensor_owned_by.argtypes = [C.c_void_p, C.POINTER(DeviceTensor)]
    lib.yvex_rocm_encoded_matvec.argtypes = [
        C.c_void_p, C.c_void_p, ULL, C.c_uint, ULL, ULL, ULL, ULL, C.POINTER(DeviceTensor),
        C.POINTER(DeviceTensor), ULL, C.POINTER(DeviceTensor), C.POINTER(DeviceTensor), C.c_int,
        C.POINTER(OperationFacts), C.POINTER(Error)]
    lib.yvex_rocm_encoded_gather.argtypes = [
        C.c_void_p, C.c_void_p, ULL, C.c_uint, ULL, ULL, ULL, C.c_void_p, ULL,
        C.POINTER(DeviceTensor), C.POINTER(OperationFacts), C.POINTER(Error)]
    lib.yvex_rocm_select_greedy_rows.argtypes = [
        C.c_void_p, C.POINTER(DeviceTensor), ULL, ULL, C.c_void_p, C.c_void_p, C.c_void_p,
        C.POINTER(OperationFacts), C.POINTER(Error)]
    lib.yvex_rocm_expert_worklist_build.argtypes = [C.c_void_p, C.c_void_p, ULL, ULL, ULL,
                                               C.POINTER(WorklistStorage),
                                               C.POINTER(WorklistObservation), C.POINTER(Error)]
    return lib
