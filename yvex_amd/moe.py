"""Launch sequence of one MoE layer over a row batch, driven from Python through the C ABI.

This is the same sequence the C11 host layer's ``execute_rows`` enqueues
(src/backend/cuda/moe.c:1619 in the reference): quantize activations -> route -> worklist ->
grouped up (+SwiGLU) -> quantize intermediate -> grouped down -> rank-ordered reduce -> shared
expert -> combine. It exists so tests and the benchmark can reach each stage's buffers; it does
no arithmetic itself.
"""
from __future__ import annotations

import torch

from . import kernels as K


class MoeLayer:
    def __init__(self, *, hidden, intermediate, experts, topk, qtypes, routed, shared=None,
                 bias=None, scoring=K.SQRT_SOFTPLUS, normalize=True, scaling=1.0, limit=10.0,
                 act_q8=True, max_rows=64, device="cuda", matrix_cores=False, sweep_image=False):
        self.hidden, self.intermediate, self.experts, self.topk = hidden, intermediate, experts, topk
        self.qtypes, self.scoring, self.normalize = qtypes, scoring, normalize
        self.scaling, self.limit, self.act_q8 = scaling, limit, act_q8
        self.device = device
        self.routed = K.expert_weights(*routed, qtypes, hidden, intermediate)
        self.shared = K.expert_weights(*shared, qtypes, hidden, intermediate) if shared else None
        if sweep_image:      # IQ2_XXS experts re-packed for the decode sweeps (built on the device)
            self.routed = K.expert_weights_image(self.routed, hidden, intermediate)
            if self.shared is not None:
                self.shared = K.expert_weights_image(self.shared, hidden, intermediate)
        self.bias = bias
        self.max_rows = max_rows
        pairs = max_rows * topk
        f32 = dict(dtype=torch.float32, device=device)
        u8 = dict(dtype=torch.uint8, device=device)
        self.status = K.new_status(device)
        self.act_q8_rows = torch.empty(max_rows * (hidden // 256) * 292, **u8)
        self.worklist = K.Worklist(pairs, experts, device)
        # the shared expert's intermediate rows sit right behind the routed pairs' (see run()), so
        # one launch quantizes both
        self.intermediate_f32 = torch.empty((pairs + max_rows, intermediate), **f32)
        self.intermediate_q8 = torch.empty((pairs + max_rows) * (intermediate // 256) * 292, **u8)
        self.pair_outputs = torch.empty((pairs, hidden), **f32)
        self.shared_mid = torch.empty((max_rows, intermediate), **f32)
        self.shared_mid_q8 = torch.empty(max_rows * (intermediate // 256) * 292, **u8)
        self.shared_out = torch.zeros((max_rows, hidden), **f32)
        self.routed_out = torch.empty((max_rows, hidden), **f32)
        self.combined = torch.empty((max_rows, hidden), **f32)
        self.selected = None
        self.weights = None
        self.merge_shared = True
        # routing, worklist and input quantization in one launch where the batch is small enough
        self.fused_prepare = True
        # row-batch (prefill-width) kernels on the int8 matrix cores instead of the decode sweeps
        self.matrix_cores = matrix_cores
        # when a list, run() appends (name, event) marks around the two expert sweeps so a caller
        # can read their durations inside its own timed steps
        self.marks = None

    def _mark(self, name):
        if self.marks is not None:
            event = torch.cuda.Event(enable_timing=True)
            event.record()
            self.marks.append((name, event))

    def run(self, rows_f32: torch.Tensor, logits: torch.Tensor):
        """Enqueue one batch; returns the combined rows (device tensor, not synchronised)."""
        rows = rows_f32.shape[0]
        assert rows <= self.max_rows
        pairs = rows * self.topk
        st = self.status
        acts = self.act_q8_rows if self.act_q8 else rows_f32
        if self.fused_prepare and K.moe_prepare_supported(rows, self.experts, self.topk):
            self.selected, self.weights = K.moe_prepare(
                logits, self.bias, self.topk, self.scoring, self.normalize, self.scaling, st, self.worklist,
                rows_f32 if self.act_q8 else None, self.act_q8_rows if self.act_q8 else None)
        else:
            if self.act_q8:
                K.q8k_quantize(rows_f32, st, self.act_q8_rows)
            self.selected, self.weights = K.moe_route_rows(
                logits, self.bias, self.topk, self.scoring, self.normalize, self.scaling, st)
            K.worklist_build(self.selected, self.experts, st, self.worklist)
        if self.matrix_cores:
            return self._run_rows(acts, rows, pairs)
        merged = self.shared is not None and self.merge_shared
        row_q8 = (self.intermediate // 256) * 292
        joined = self.shared is not None and self.act_q8 and (pairs * row_q8) % 16 == 0
        shared_mid = self.intermediate_f32[pairs:pairs + rows] if joined else self.shared_mid
        self._mark("up_begin")
        K.moe_up(self.routed, acts, self.act_q8, self.weights, self.worklist, pairs, self.topk,
                 self.experts, self.limit, self.intermediate_f32, st,
                 shared=self.shared if merged else None, shared_rows=rows if merged else 0,
                 shared_intermediate=shared_mid if merged else None)
        self._mark("up_end")
        if self.shared is not None and not merged:
            K.moe_up(self.shared, acts, self.act_q8, None, None, rows, 1, 1, self.limit,
                     shared_mid, st)
        if self.act_q8:
            mid = self.intermediate_q8
            if joined:
                K.q8k_quantize(self.intermediate_f32[:pairs + rows], st, self.intermediate_q8)
                smid = self.intermediate_q8[pairs * row_q8:]
            else:
                K.q8k_quantize(self.intermediate_f32[:pairs], st, self.intermediate_q8)
                if self.shared is not None:
                    K.q8k_quantize(shared_mid[:rows], st, self.shared_mid_q8)
                smid = self.shared_mid_q8
        else:
            mid, smid = self.intermediate_f32, shared_mid
        self.last_shared_mid, self.last_shared_down_input = shared_mid, smid    # for stage-wise callers
        self._mark("down_begin")
        K.moe_down(self.routed, mid, self.act_q8, self.worklist, pairs, self.experts,
                   self.pair_outputs, st, shared=self.shared if merged else None,
                   shared_rows=rows if merged else 0, shared_intermediate=smid if merged else None,
                   shared_outputs=self.shared_out if merged else None)
        self._mark("down_end")
        if self.shared is not None and not merged:
            K.moe_down(self.shared, smid, self.act_q8, None, rows, 1, self.shared_out, st)
        K.moe_reduce_combine(self.pair_outputs, rows, self.topk, self.hidden, self.shared_out,
                             self.routed_out, self.combined, st)
        return self.combined[:rows]

    def _run_rows(self, acts, rows, pairs):
        if not self.act_q8:
            raise ValueError("the matrix-core kernels take Q8_K activations")
        st = self.status
        K.moe_up_rows(self.routed, acts, self.weights, self.worklist, pairs, self.topk, self.experts,
                      self.limit, self.intermediate_f32, st)
        K.q8k_quantize(self.intermediate_f32[:pairs], st, self.intermediate_q8)
        K.moe_down_rows(self.routed, self.intermediate_q8, self.worklist, pairs, self.experts,
                        self.pair_outputs, st)
        if self.shared is not None:
            K.moe_up_rows(self.shared, acts, None, None, rows, 1, 1, self.limit, self.shared_mid, st)
            K.q8k_quantize(self.shared_mid[:rows], st, self.shared_mid_q8)
            K.moe_down_rows(self.shared, self.shared_mid_q8, None, rows, 1, self.shared_out, st)
        K.moe_reduce_combine(self.pair_outputs, rows, self.topk, self.hidden, self.shared_out,
                             self.routed_out, self.combined, st)
        return self.combined[:rows]
