"""Python-side callers of the launch-level C ABI (include/yvex_rocm_kernels.h).

torch is used for device memory and the current stream only; every computation goes through
``libyvex_rocm.so``. Tensors must live on the GPU and be contiguous.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import load_library

F32, F16, Q8_0, Q2_K, Q4_K, Q8_K, IQ2_XXS, I32, BF16 = 0, 1, 8, 10, 12, 15, 16, 26, 30
SQRT_SOFTPLUS, SIGMOID = 0, 1

_GEOMETRY = {F32: (1, 4), F16: (1, 2), BF16: (1, 2), I32: (1, 4), Q8_0: (32, 34), Q2_K: (256, 84),
             Q4_K: (256, 144), IQ2_XXS: (256, 66), Q8_K: (256, 292)}


class KernelError(RuntimeError):
    def __init__(self, name: str, rc: int):
        lib = load_library()
        lib.yvex_hip_last_error.restype = C.c_char_p
        text = lib.yvex_hip_last_error().decode(errors="replace")
        super().__init__(f"{name} returned {rc} {text}")
        self.rc = rc


class ExpertWeights(C.Structure):
    _fields_ = [("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p),
                ("gate_qtype", C.c_uint), ("up_qtype", C.c_uint), ("down_qtype", C.c_uint),
                ("hidden", C.c_uint64), ("intermediate", C.c_uint64),
                ("gate_row_bytes", C.c_uint64), ("up_row_bytes", C.c_uint64),
                ("down_row_bytes", C.c_uint64),
                ("gate_expert_bytes", C.c_uint64), ("up_expert_bytes", C.c_uint64),
                ("down_expert_bytes", C.c_uint64), ("gate_up_image", C.c_int), ("down_image", C.c_int)]


def row_bytes(qtype: int, width: int) -> int:
    block, nbytes = _GEOMETRY[qtype]
    if width % block:
        raise ValueError("row width is not block divisible")
    return width // block * nbytes


def _ptr(t):
    if t is None:
        return C.c_void_p(0)
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError("device, contiguous tensors only")
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _call(name, *args):
    fn = getattr(load_library(), name)
    fn.restype = C.c_int
    rc = fn(*args)
    if rc != 0:
        raise KernelError(name, rc)


def new_status(device="cuda"):
    return torch.zeros(1, dtype=torch.int32, device=device)


def q8k_quantize(values: torch.Tensor, status: torch.Tensor, out: torch.Tensor | None = None):
    rows, width = values.shape
    if out is None:
        out = torch.empty(rows * (width // 256) * 292, dtype=torch.uint8, device=values.device)
    _call("yvex_hip_q8k_quantize", _ptr(values), C.c_uint64(rows), C.c_uint64(width),
          C.c_uint64(values.stride(0)), _ptr(out), _ptr(status), _stream())
    return out


def matvec(encoded, qtype, row_count, row_width, inputs, *, input_q8=False, input_rows=None,
           additive=None, output_bf16=False, status=None, out=None):
    if input_rows is None:
        input_rows = inputs.shape[0]
    if out is None:
        out = torch.empty((input_rows, row_count), dtype=torch.float32, device=encoded.device)
    stride = row_width if input_q8 else inputs.stride(0)
    out_stride = out.stride(0) if out.dim() == 2 else row_count      # `additive` shares the output's stride
    _call("yvex_hip_matvec", _ptr(encoded), C.c_uint(qtype), C.c_uint64(row_count),
          C.c_uint64(row_width), C.c_uint64(row_bytes(qtype, row_width)), _ptr(inputs),
          C.c_int(int(input_q8)), C.c_uint64(input_rows), C.c_uint64(stride), _ptr(additive),
          _ptr(out), C.c_uint64(out_stride), C.c_int(int(output_bf16)), _ptr(status), _stream())
    return out


def matvec_f32_rows(weights, inputs, status, *, additive=None, output_bf16=False, scratch=None, out=None):
    """F32 weight rows [rows, width] against F32 input rows with the split-projection scratch:
    None allocates what yvex_hip_matvec_f32_scratch_bytes asks for, False passes none."""
    row_count, row_width = weights.shape
    input_rows = inputs.shape[0]
    lib = load_library()
    lib.yvex_hip_matvec_f32_scratch_bytes.restype = C.c_uint64
    need = lib.yvex_hip_matvec_f32_scratch_bytes(C.c_uint64(row_count), C.c_uint64(row_width),
                                                 C.c_uint64(input_rows))
    if scratch is None and need:
        scratch = torch.empty(need, dtype=torch.uint8, device=weights.device)
    if scratch is False:
        scratch = None
    if out is None:
        out = torch.empty((input_rows, row_count), dtype=torch.float32, device=weights.device)
    _call("yvex_hip_matvec_f32_rows", _ptr(weights), C.c_uint64(row_count), C.c_uint64(row_width),
          _ptr(inputs), C.c_uint64(input_rows), C.c_uint64(inputs.stride(0)), _ptr(additive), _ptr(out),
          C.c_uint64(row_count), C.c_int(int(output_bf16)), _ptr(scratch),
          C.c_uint64(scratch.numel() if scratch is not None else 0), _ptr(status), _stream())
    return out


def matvec_f32_rows_scored(weights, inputs, scoring, status):
    """The split router projection with the scores beside the logits: (logits, scores)."""
    row_count, row_width = weights.shape
    input_rows = inputs.shape[0]
    lib = load_library()
    lib.yvex_hip_matvec_f32_scratch_bytes.restype = C.c_uint64
    need = lib.yvex_hip_matvec_f32_scratch_bytes(C.c_uint64(row_count), C.c_uint64(row_width),
                                                 C.c_uint64(input_rows))
    scratch = torch.empty(max(need, 8), dtype=torch.uint8, device=weights.device)
    out = torch.empty((input_rows, row_count), dtype=torch.float32, device=weights.device)
    scores = torch.empty((input_rows, row_count), dtype=torch.float32, device=weights.device)
    _call("yvex_hip_matvec_f32_rows_scored", _ptr(weights), C.c_uint64(row_count), C.c_uint64(row_width),
          _ptr(inputs), C.c_uint64(input_rows), C.c_uint64(inputs.stride(0)), _ptr(out),
          C.c_uint64(row_count), _ptr(scores), C.c_int(scoring), _ptr(scratch), C.c_uint64(need),
          _ptr(status), _stream())
    return out, scores


def block_dots_i32(encoded, qtype, row_count, row_width, act_q8, input_rows, status):
    blocks = row_width // 256
    shape = (input_rows, row_count, blocks * 8) if qtype == Q8_0 else (input_rows, row_count, blocks, 2)
    sums = torch.zeros(shape, dtype=torch.int32, device=encoded.device)
    _call("yvex_hip_block_dots_i32", _ptr(encoded), C.c_uint(qtype), C.c_uint64(row_count),
          C.c_uint64(row_width), C.c_uint64(row_bytes(qtype, row_width)), _ptr(act_q8),
          C.c_uint64(input_rows), _ptr(sums), _ptr(status), _stream())
    return sums


def gather(encoded, qtype, row_count, row_width, row_ids, status):
    selected = row_count if row_ids is None else row_ids.numel()
    out = torch.empty((selected, row_width), dtype=torch.float32, device=encoded.device)
    _call("yvex_hip_gather", _ptr(encoded), C.c_uint(qtype), C.c_uint64(row_count),
          C.c_uint64(row_width), C.c_uint64(row_bytes(qtype, row_width)), _ptr(row_ids),
          C.c_uint64(selected), _ptr(out), _ptr(status), _stream())
    return out


def argmax_f32(values, status, out=None, scratch=None):
    """Greedy selection per row of a [rows, width] F32 tensor: (tokens u32, values f32, ties u64).
    scratch: None = allocate what splitting long rows needs, False = one workgroup per row."""
    rows, width = values.shape
    if out is None:
        out = (torch.zeros(rows, dtype=torch.int32, device=values.device),
               torch.zeros(rows, dtype=torch.float32, device=values.device),
               torch.zeros(rows, dtype=torch.int64, device=values.device))
    tokens, best, ties = out
    lib = load_library()
    lib.yvex_hip_argmax_scratch_bytes.restype = C.c_uint64
    need = lib.yvex_hip_argmax_scratch_bytes(C.c_uint64(rows), C.c_uint64(width))
    if scratch is None and need:
        scratch = torch.empty(need, dtype=torch.uint8, device=values.device)
    if scratch is False:
        scratch = None
    _call("yvex_hip_argmax_f32", _ptr(values), C.c_uint64(rows), C.c_uint64(width), _ptr(tokens),
          _ptr(best), _ptr(ties), _ptr(scratch), C.c_uint64(scratch.numel() if scratch is not None else 0),
          _ptr(status), _stream())
    return tokens, best, ties


def moe_route_hash_rows(logits, table, token_ids, topk, scoring, normalize, scaling, status, table_rows=None):
    """Hash router: table is an int32 [rows, columns] tensor, token_ids int32 [n]."""
    rows, experts = logits.shape
    selected = torch.zeros((rows, topk), dtype=torch.int64, device=logits.device)
    weights = torch.zeros((rows, topk), dtype=torch.float32, device=logits.device)
    single = table.shape[0] == 1 and table_rows is not None
    _call("yvex_hip_moe_route_hash_rows", _ptr(logits), _ptr(table), _ptr(token_ids), C.c_uint64(rows),
          C.c_uint64(experts), C.c_uint64(topk), C.c_uint64(table_rows or table.shape[0]),
          C.c_uint64(table.shape[1] * 4), C.c_int(int(single)), C.c_int(scoring), C.c_int(int(normalize)),
          C.c_double(scaling), _ptr(selected), _ptr(weights), _ptr(status), _stream())
    return selected, weights


def mhc_ingress(rows, mixes, scale, base, norm, *, streams, width, iterations, rms_epsilon,
                mhc_epsilon, post_multiplier, status, out=None):
    """Residual-stream ingress + weighted RMS norm: (normalized [n, width], post [n, streams],
    combination [n, streams, streams])."""
    count = rows.shape[0]
    if out is None:
        out = (torch.empty((count, width), dtype=torch.float32, device=rows.device),
               torch.empty((count, streams), dtype=torch.float32, device=rows.device),
               torch.empty((count, streams, streams), dtype=torch.float32, device=rows.device))
    normalized, post, combination = out
    _call("yvex_hip_mhc_ingress", _ptr(rows), _ptr(mixes), _ptr(scale), _ptr(base), _ptr(norm),
          C.c_uint64(count), C.c_uint64(streams), C.c_uint64(width), C.c_uint64(iterations),
          C.c_double(rms_epsilon), C.c_double(mhc_epsilon), C.c_double(post_multiplier),
          _ptr(normalized), _ptr(post), _ptr(combination), _ptr(status), _stream())
    return normalized, post, combination


def mhc_egress(core, rows, post, combination, *, streams, width, status, out=None):
    """Residual-stream egress: [n, streams * width] bf16-valued F32 rows."""
    count = core.shape[0]
    if out is None:
        out = torch.empty((count, streams * width), dtype=torch.float32, device=core.device)
    _call("yvex_hip_mhc_egress", _ptr(core), _ptr(rows), _ptr(post), _ptr(combination),
          C.c_uint64(count), C.c_uint64(streams), C.c_uint64(width), _ptr(out), _ptr(status), _stream())
    return out


def moe_route_rows(logits, bias, topk, scoring, normalize, scaling, status):
    rows, experts = logits.shape
    selected = torch.empty((rows, topk), dtype=torch.int64, device=logits.device)
    weights = torch.empty((rows, topk), dtype=torch.float32, device=logits.device)
    _call("yvex_hip_moe_route_rows", _ptr(logits), _ptr(bias), C.c_uint64(rows),
          C.c_uint64(experts), C.c_uint64(topk), C.c_int(scoring), C.c_int(int(normalize)),
          C.c_double(scaling), _ptr(selected), _ptr(weights), _ptr(status), _stream())
    return selected, weights


class Worklist:
    """Device-resident expert-major worklist (all int64 tensors hold unsigned 64-bit values)."""

    def __init__(self, pairs: int, experts: int, device):
        self.order = torch.empty(pairs, dtype=torch.int64, device=device)
        self.expert_ids = torch.empty(experts, dtype=torch.int64, device=device)
        self.bucket_offsets = torch.empty(experts + 1, dtype=torch.int64, device=device)
        self.bucket_populations = torch.empty(experts, dtype=torch.int64, device=device)
        self.sweep_offsets = torch.empty(experts + 1, dtype=torch.int64, device=device)
        self.counts = torch.zeros(4, dtype=torch.int64, device=device)


def worklist_build(selected, experts, status, worklist: Worklist | None = None) -> Worklist:
    rows, topk = selected.shape
    pairs = rows * topk
    wl = worklist or Worklist(pairs, experts, selected.device)
    _call("yvex_hip_worklist_build", _ptr(selected), C.c_uint64(pairs), C.c_uint64(topk),
          C.c_uint64(experts), _ptr(wl.order), _ptr(wl.expert_ids), _ptr(wl.bucket_offsets),
          _ptr(wl.bucket_populations), _ptr(wl.sweep_offsets), _ptr(wl.counts), _ptr(status),
          _stream())
    return wl


def moe_prepare_supported(rows: int, experts: int, topk: int) -> bool:
    fn = load_library().yvex_hip_moe_prepare_supported
    fn.restype = C.c_int
    return bool(fn(C.c_uint64(rows), C.c_uint64(experts), C.c_uint64(topk)))


def moe_prepare(logits, bias, topk, scoring, normalize, scaling, status, worklist: Worklist,
                values=None, encoded=None):
    """Routing, worklist and (with values) the Q8_K quantization of the input rows in one launch."""
    rows, experts = logits.shape
    selected = torch.empty((rows, topk), dtype=torch.int64, device=logits.device)
    weights = torch.empty((rows, topk), dtype=torch.float32, device=logits.device)
    width = 0 if values is None else values.shape[1]
    stride = 0 if values is None else values.stride(0)
    wl = worklist
    _call("yvex_hip_moe_prepare", _ptr(logits), _ptr(bias), C.c_uint64(rows), C.c_uint64(experts),
          C.c_uint64(topk), C.c_int(scoring), C.c_int(int(normalize)), C.c_double(scaling), _ptr(selected),
          _ptr(weights), _ptr(wl.order), _ptr(wl.expert_ids), _ptr(wl.bucket_offsets),
          _ptr(wl.bucket_populations), _ptr(wl.sweep_offsets), _ptr(wl.counts), _ptr(values),
          C.c_uint64(width), C.c_uint64(stride), _ptr(encoded), _ptr(status), _stream())
    return selected, weights


def moe_prepare_scored(scores, bias, topk, normalize, scaling, status, worklist: Worklist,
                       values=None, encoded=None):
    """moe_prepare over scores published by matvec_f32_rows_scored."""
    rows, experts = scores.shape
    selected = torch.empty((rows, topk), dtype=torch.int64, device=scores.device)
    weights = torch.empty((rows, topk), dtype=torch.float32, device=scores.device)
    width = 0 if values is None else values.shape[1]
    stride = 0 if values is None else values.stride(0)
    wl = worklist
    _call("yvex_hip_moe_prepare_scored", _ptr(scores), _ptr(bias), C.c_uint64(rows), C.c_uint64(experts),
          C.c_uint64(topk), C.c_int(int(normalize)), C.c_double(scaling), _ptr(selected),
          _ptr(weights), _ptr(wl.order), _ptr(wl.expert_ids), _ptr(wl.bucket_offsets),
          _ptr(wl.bucket_populations), _ptr(wl.sweep_offsets), _ptr(wl.counts), _ptr(values),
          C.c_uint64(width), C.c_uint64(stride), _ptr(encoded), _ptr(status), _stream())
    return selected, weights


def expert_weights(gate, up, down, qtypes, hidden, intermediate) -> ExpertWeights:
    w = ExpertWeights()
    w.gate, w.up, w.down = gate.data_ptr(), up.data_ptr(), down.data_ptr()
    w.gate_qtype, w.up_qtype, w.down_qtype = qtypes
    w.hidden, w.intermediate = hidden, intermediate
    w.gate_row_bytes = row_bytes(qtypes[0], hidden)
    w.up_row_bytes = row_bytes(qtypes[1], hidden)
    w.down_row_bytes = row_bytes(qtypes[2], intermediate)
    w.gate_expert_bytes = w.gate_row_bytes * intermediate
    w.up_expert_bytes = w.up_row_bytes * intermediate
    w.down_expert_bytes = w.down_row_bytes * hidden
    w._keep = (gate, up, down)
    return w


def iq2_sweep_image(canonical):
    """The sweep image of canonical IQ2_XXS bytes (a uint8 tensor of whole superblocks)."""
    blocks = canonical.numel() // 66
    image = torch.empty(blocks * 72, dtype=torch.uint8, device=canonical.device)
    _call("yvex_hip_iq2_sweep_image_build", _ptr(canonical), C.c_uint64(blocks), _ptr(image), _stream())
    return image


def expert_weights_image(w: ExpertWeights, hidden, intermediate) -> ExpertWeights:
    """The same IQ2_XXS experts with all three matrices as sweep images."""
    gate, up, down = (iq2_sweep_image(t) for t in w._keep)
    out = ExpertWeights()
    out.gate, out.up, out.down = gate.data_ptr(), up.data_ptr(), down.data_ptr()
    out.gate_qtype, out.up_qtype, out.down_qtype = w.gate_qtype, w.up_qtype, w.down_qtype
    out.hidden, out.intermediate = hidden, intermediate
    out.gate_row_bytes = out.up_row_bytes = hidden // 256 * 72
    out.down_row_bytes = intermediate // 256 * 72
    out.gate_expert_bytes = out.up_expert_bytes = out.gate_row_bytes * intermediate
    out.down_expert_bytes = out.down_row_bytes * hidden
    out.gate_up_image = out.down_image = 1
    out._keep = (gate, up, down)
    return out


def _wl_ptrs(wl):
    if wl is None:
        return [C.c_void_p(0)] * 6
    return [_ptr(wl.order), _ptr(wl.expert_ids), _ptr(wl.bucket_offsets),
            _ptr(wl.bucket_populations), _ptr(wl.sweep_offsets), _ptr(wl.counts)]


def moe_up(w: ExpertWeights, activations, act_q8, route_weights, wl, pairs, topk, experts, limit,
           intermediate, status, shared: ExpertWeights | None = None, shared_rows=0,
           shared_intermediate=None):
    _call("yvex_hip_moe_up", C.byref(w), _ptr(activations), C.c_int(int(act_q8)),
          _ptr(route_weights), *_wl_ptrs(wl), C.c_uint64(pairs), C.c_uint64(topk),
          C.c_uint64(experts), C.c_double(limit), _ptr(intermediate),
          C.byref(shared) if shared is not None else C.c_void_p(0), C.c_uint64(shared_rows),
          _ptr(shared_intermediate), _ptr(status), _stream())


def moe_down(w: ExpertWeights, intermediate, act_q8, wl, pairs, experts, pair_outputs, status,
             shared: ExpertWeights | None = None, shared_rows=0, shared_intermediate=None,
             shared_outputs=None):
    _call("yvex_hip_moe_down", C.byref(w), _ptr(intermediate), C.c_int(int(act_q8)),
          *_wl_ptrs(wl), C.c_uint64(pairs), C.c_uint64(experts), _ptr(pair_outputs),
          C.byref(shared) if shared is not None else C.c_void_p(0), C.c_uint64(shared_rows),
          _ptr(shared_intermediate), _ptr(shared_outputs), _ptr(status), _stream())


def moe_up_rows(w: ExpertWeights, act_q8k, route_weights, wl, pairs, topk, experts, limit,
                intermediate, status):
    """Matrix-core form of moe_up; wl None is the single-bucket (shared expert) form."""
    ptrs = [C.c_void_p(0)] * 5 if wl is None else [
        _ptr(wl.order), _ptr(wl.expert_ids), _ptr(wl.bucket_offsets), _ptr(wl.bucket_populations),
        _ptr(wl.counts)]
    _call("yvex_hip_moe_up_rows", C.byref(w), _ptr(act_q8k), _ptr(route_weights), *ptrs,
          C.c_uint64(pairs), C.c_uint64(topk), C.c_uint64(experts), C.c_double(limit),
          _ptr(intermediate), _ptr(status), _stream())


def moe_down_rows(w: ExpertWeights, intermediate_q8k, wl, pairs, experts, pair_outputs, status):
    ptrs = [C.c_void_p(0)] * 5 if wl is None else [
        _ptr(wl.order), _ptr(wl.expert_ids), _ptr(wl.bucket_offsets), _ptr(wl.bucket_populations),
        _ptr(wl.counts)]
    _call("yvex_hip_moe_down_rows", C.byref(w), _ptr(intermediate_q8k), *ptrs, C.c_uint64(pairs),
          C.c_uint64(experts), _ptr(pair_outputs), _ptr(status), _stream())


def moe_reduce_combine(pair_outputs, rows, topk, hidden, shared, routed, combined, status):
    _call("yvex_hip_moe_reduce_combine", _ptr(pair_outputs), C.c_uint64(rows), C.c_uint64(topk),
          C.c_uint64(hidden), _ptr(shared), _ptr(routed), _ptr(combined), _ptr(status), _stream())
