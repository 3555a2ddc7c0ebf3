"""Small conveniences over the C ABI of the backend for Python callers (tests, the benchmark):
open a backend, allocate and fill its tensors, attach a resident arena and a workspace. Every
call goes through ``include/yvex_rocm.h``; nothing here computes."""
import ctypes as C

import numpy as np

from . import abi


class Backend:
    def __init__(self, memory_limit=0, shared_with=None):
        """An owning backend, or (shared_with = an owning Backend) a session that borrows its
        device and resident arena (yvex_rocm_backend_open_shared)."""
        self.lib = abi.library()
        self.handle = C.c_void_p()
        self.err = abi.Error()
        if shared_with is None:
            opts = abi.BackendOptions(abi.KIND_ROCM, None, memory_limit)
            self.open_rc = self.lib.yvex_rocm_backend_open(C.byref(self.handle), C.byref(opts), C.byref(self.err))
        else:
            self.open_rc = self.lib.yvex_rocm_backend_open_shared(C.byref(self.handle), shared_with.handle,
                                                                  memory_limit, C.byref(self.err))
        self.tensors = []

    def attach_shared_arena(self, owner_tensor, host_base, nbytes, generation=1):
        """Attach the arena the owning backend has published: nothing is uploaded again."""
        return self.lib.yvex_rocm_backend_resident_attach(self.handle, C.c_void_p(host_base), nbytes, owner_tensor,
                                                          generation, C.byref(self.err))

    @property
    def ok(self):
        return self.open_rc == 0

    def tensor(self, nbytes, dtype=abi.DTYPE_F32, name=b"t"):
        desc = abi.TensorDesc(name, dtype, 1, (abi.ULL * 4)(nbytes, 0, 0, 0), nbytes)
        out = C.POINTER(abi.DeviceTensor)()
        rc = self.lib.yvex_rocm_backend_tensor_alloc(self.handle, C.byref(desc), C.byref(out), C.byref(self.err))
        if rc == 0:
            self.tensors.append(out)
        return rc, out

    def f32(self, array):
        array = np.ascontiguousarray(array, np.float32)
        rc, t = self.tensor(array.nbytes)
        assert rc == 0, self.err.message
        rc = self.lib.yvex_rocm_backend_tensor_write(self.handle, t, array.ctypes.data, array.nbytes,
                                                C.byref(self.err))
        assert rc == 0, self.err.message
        return t

    def empty_f32(self, count):
        rc, t = self.tensor(count * 4)
        assert rc == 0, self.err.message
        return t

    def read_f32(self, tensor, count):
        out = np.empty(count, np.float32)
        rc = self.lib.yvex_rocm_backend_tensor_read(self.handle, tensor, out.ctypes.data, out.nbytes,
                                               C.byref(self.err))
        assert rc == 0, self.err.message
        return out

    def resident(self, blob: np.ndarray, generation=1):
        """Allocate a resident arena, fill its host shadow, attach (= publish). Returns
        (tensor, host_base_address)."""
        desc = abi.TensorDesc(b"arena", abi.DTYPE_I8, 1, (abi.ULL * 4)(blob.nbytes, 0, 0, 0), blob.nbytes)
        out = C.POINTER(abi.DeviceTensor)()
        host = C.c_void_p()
        rc = self.lib.yvex_rocm_backend_resident_alloc(self.handle, C.byref(desc), C.byref(out),
                                                  C.byref(host), C.byref(self.err))
        assert rc == 0, self.err.message
        self.tensors.append(out)
        C.memmove(host.value, blob.ctypes.data, blob.nbytes)
        rc = self.lib.yvex_rocm_backend_resident_attach(self.handle, host, blob.nbytes, out, generation,
                                                   C.byref(self.err))
        assert rc == 0, self.err.message
        return out, host.value

    def workspace(self, nbytes):
        rc, t = self.tensor(nbytes, abi.DTYPE_I8, b"workspace")
        assert rc == 0, self.err.message
        rc = self.lib.yvex_rocm_backend_workspace_attach(self.handle, t, nbytes, C.byref(self.err))
        assert rc == 0, self.err.message
        return t

    def release_all(self):
        for t in reversed(self.tensors):
            self.lib.yvex_rocm_backend_tensor_release(self.handle, C.byref(t), C.byref(self.err))
        self.tensors = []

    def close(self):
        self.release_all()
        return self.lib.yvex_rocm_backend_close_checked(C.byref(self.handle), C.byref(self.err))


class RowBatchLayer:
    """One MoE layer behind include/yvex_rocm.h: a backend of its own, weight views that
    carry device addresses, backend-owned row tensors and an attached workspace. `step()` is one
    yvex_rocm_backend_moe_operations_get()->execute_rows with deferred completion, `complete()` the
    phase barrier complete_rows (the reference completes all pending layers of a phase with one
    call, src/runtime/moe.c:1567-1576)."""

    def __init__(self, torch, routed, shared, router, x_host, rows, *, hidden, intermediate, experts, topk,
                 qtype=16, sweep_image=False, scoring=abi.SCORING_SIGMOID, scaling=1.0, limit=10.0,
                 envelope=None, down_qtype=None, shared_qtype=None):
        """envelope: None, or the residual-stream weights around the layer as device tensors,
        dict(streams, iterations, function [F32 (streams + 2) * streams x streams * hidden], scale
        [F32 3], base [F32 (streams + 2) * streams], norm [BF16 hidden]); x_host then holds
        streams * hidden values a row and so does the output."""
        HIDDEN, INTERMEDIATE, EXPERTS, TOPK = hidden, intermediate, experts, topk
        self.C, self.abi, self.np, self.rows, self.hidden = C, abi, np, rows, hidden
        self.b = Backend()
        if not self.b.ok:
            raise RuntimeError(f"backend open failed: {self.b.err.message.decode()}")
        self.keep = (routed, shared, router)
        plan = self.plan = abi.LayerPlan()
        plan.schema_version, plan.router_class, plan.scoring = 1, abi.ROUTER_LEARNED, scoring
        plan.hidden_width = plan.expanded_width = HIDDEN
        plan.residual_streams = 1
        streams = envelope["streams"] if envelope else 0
        expanded = streams * HIDDEN if envelope else HIDDEN
        if envelope:
            plan.residual_streams, plan.expanded_width = streams, expanded
            plan.mhc_mixing_rows, plan.mhc_sinkhorn_iterations = (streams + 2) * streams, envelope["iterations"]
            plan.rms_epsilon, plan.mhc_epsilon, plan.mhc_post_multiplier = 1e-6, 1e-6, 2.0
            self.keep += tuple(envelope[k] for k in ("function", "scale", "base", "norm"))
        plan.routed_experts, plan.shared_experts, plan.experts_per_token = EXPERTS, 1, TOPK
        plan.expert_intermediate_width = plan.shared_intermediate_width = INTERMEDIATE
        plan.routed_scaling_factor, plan.activation_limit = scaling, limit
        plan.requires_correction_bias, plan.normalize_topk_probabilities = 0, 1
        job = self.job = abi.LayerJob()
        job.layer = C.pointer(plan)
        # down_qtype: the down projections' format where it differs from the gate and up projections'
        down_qtype = qtype if down_qtype is None else down_qtype
        # shared_qtype: the format of all three matrices of the shared expert where it differs
        block_bytes = {16: 66, 12: 144, 10: 84, 8: 272}
        rb_h, rb_i = HIDDEN // 256 * block_bytes[qtype], INTERMEDIATE // 256 * block_bytes[down_qtype]
        sq_gate = qtype if shared_qtype is None else shared_qtype
        sq_down = down_qtype if shared_qtype is None else shared_qtype
        srb_h, srb_i = HIDDEN // 256 * block_bytes[sq_gate], INTERMEDIATE // 256 * block_bytes[sq_down]

        self.images = []

        def view(slot, tensor, qtype, width, count, row_bytes, activation, consumer=None):
            v = job.weights[slot]
            v.qtype, v.layout, v.activation = qtype, abi.LAYOUT_EXPERT_MAJOR, activation
            v.kernel_family = abi.FAMILY_GFX950
            v.device_address = tensor.data_ptr()
            v.encoded_bytes = v.storage_bytes = tensor.numel() * tensor.element_size()
            v.row_bytes, v.row_width, v.row_count = row_bytes, width, count
            if sweep_image and consumer is not None and qtype == 16:     # (only IQ2_XXS tensors have an image)
                # the residency step of a caller that keeps its experts as the decode sweeps' image:
                # plan, allocate, build on the device from the resident canonical bytes
                d = abi.ExecutionDecision()
                d.expert_count = 1 if consumer == abi.CONSUMER_SHARED_EXPERT else EXPERTS
                d.canonical_qtype, d.canonical_row_width, d.canonical_row_count = qtype, width, count
                d.encoded_bytes = v.encoded_bytes
                d.consumer, d.layout, d.derived_asset_required = consumer, abi.LAYOUT_DERIVED, 1
                d.kernel_family = abi.FAMILY_GFX950
                storage, err = abi.ULL(), abi.Error()
                if self.b.lib.yvex_rocm_moe_derived_layout_plan(C.byref(d), C.byref(storage), C.byref(err)) != 0:
                    raise RuntimeError(err.message.decode())
                image = torch.empty(storage.value, dtype=torch.uint8, device=tensor.device)
                if self.b.lib.yvex_rocm_moe_sweep_image_build_resident(
                        self.b.handle, C.byref(d), tensor.data_ptr(), image.data_ptr(), storage.value,
                        C.byref(err)) != 0:
                    raise RuntimeError(err.message.decode())
                self.images.append(image)
                v.layout, v.device_address, v.storage_bytes = abi.LAYOUT_DERIVED, image.data_ptr(), storage.value

        enc = abi.ACT_DEVICE_ENCODED
        view(abi.W_ROUTER, router, 0, HIDDEN, EXPERTS, HIDDEN * 4, abi.ACT_DEVICE_F32)
        gate_up, down_c, shared_c = abi.CONSUMER_ROUTED_GATE_UP, abi.CONSUMER_ROUTED_DOWN, abi.CONSUMER_SHARED_EXPERT
        view(abi.W_ROUTED_GATE, routed[0], qtype, HIDDEN, EXPERTS * INTERMEDIATE, rb_h, enc, gate_up)
        view(abi.W_ROUTED_UP, routed[1], qtype, HIDDEN, EXPERTS * INTERMEDIATE, rb_h, enc, gate_up)
        view(abi.W_ROUTED_DOWN, routed[2], down_qtype, INTERMEDIATE, EXPERTS * HIDDEN, rb_i, enc, down_c)
        view(abi.W_SHARED_GATE, shared[0], sq_gate, HIDDEN, INTERMEDIATE, srb_h, enc, shared_c)
        view(abi.W_SHARED_UP, shared[1], sq_gate, HIDDEN, INTERMEDIATE, srb_h, enc, shared_c)
        view(abi.W_SHARED_DOWN, shared[2], sq_down, INTERMEDIATE, HIDDEN, srb_i, enc, shared_c)
        if envelope:
            mixing = (streams + 2) * streams
            f32 = abi.ACT_DEVICE_F32
            view(abi.W_MHC_FUNCTION, envelope["function"], 0, expanded, mixing, expanded * 4, f32)
            view(abi.W_MHC_SCALE, envelope["scale"], 0, 3, 1, 12, f32)
            view(abi.W_MHC_BASE, envelope["base"], 0, mixing, 1, mixing * 4, f32)
            view(abi.W_FFN_NORM, envelope["norm"], 30, HIDDEN, 1, HIDDEN * 2, f32)
        self.ops = self.b.lib.yvex_rocm_backend_moe_operations_get(self.b.handle).contents
        need, err = abi.ULL(), abi.Error()
        if self.ops.workspace_required(C.byref(plan), rows, C.byref(need), C.byref(err)) != 0:
            raise RuntimeError(err.message.decode())
        self.b.workspace(need.value)
        self.width = expanded
        self.rows_in, self.rows_out = self.b.f32(x_host), self.b.empty_f32(rows * expanded)
        batch = self.batch = abi.RowBatch()
        batch.schema_version, batch.row_count, batch.row_width, batch.row_stride = 1, rows, expanded, expanded
        batch.device_rows, batch.device_outputs = self.rows_in, self.rows_out
        batch.provenance, batch.execution_class = abi.BATCH_MULTI_SESSION, 1
        self.out = abi.RowBatchOutput()
        self.result, self.done, self.err = abi.RowBatchResult(), abi.RowBatchResult(), abi.Error()
        self.deferred = abi.DeviceCompletion(1, None)

    def step(self, defer=True, eager=False):
        C = self.C
        self.job.eager_execution = int(eager)
        self.job.device_completion = C.pointer(self.deferred) if defer else None
        rc = self.ops.execute_rows(self.b.handle, C.byref(self.job), C.byref(self.batch), C.byref(self.out),
                                   C.byref(self.result), C.byref(self.err))
        if rc != 0:
            raise RuntimeError(f"execute_rows: {self.err.message.decode()}")

    def complete(self):
        C = self.C
        if self.ops.complete_rows(self.b.handle, 0, C.byref(self.done), C.byref(self.err)) != 0:
            raise RuntimeError(f"complete_rows: {self.err.message.decode()}")

    def timed(self, steps, warmup, *, defer=True, eager=False):
        """Wall-clock ms per step of `steps` execute_rows calls, the backend idle before the
        first and after the last (complete_rows is the closing synchronisation)."""
        for _ in range(warmup):
            self.step(defer, eager)
        self.complete()
        import time
        t0 = time.perf_counter()
        for _ in range(steps):
            self.step(defer, eager)
        self.complete()
        return (time.perf_counter() - t0) * 1e3 / steps

    def output(self):
        return self.b.read_f32(self.rows_out, self.rows * self.width).reshape(self.rows, self.width)

    def close(self):
        self.b.close()
