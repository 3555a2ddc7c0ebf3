"""Host-side contract of the C ABI, exercised without a GPU.

Mirrors what the reference asserts on its own backend: status vocabulary, fail-closed qtype
admission (tests/unit/qtype_support.c:54-56, tests/unit/quant_numeric.c:461-500), qtype geometry
(tests/unit/gguf_qtype_abi.c:35-38,251), refusal order of the encoded matvec
(tests/unit/cuda/quant_qtype.c:273-517) and the no-kernel-bundle state
(tests/test_cuda_failclosed.sh:61-82), here reached through the YVEX_TEST_ROCM_NO_DEVICE seam.
"""
import ctypes as C

import numpy as np
import pytest

from yvex_amd import abi


@pytest.fixture(scope="module")
def lib():
    return abi.library()


@pytest.fixture
def seam(monkeypatch):
    monkeypatch.setenv("YVEX_TEST_ROCM_NO_DEVICE", "1")
    from backend_helpers import Backend
    b = Backend()
    assert b.ok, b.err.message
    yield b
    assert b.close() == 0


def test_library_exports_every_declared_symbol(lib):
    for name in abi.EXPORTS + abi.KERNEL_EXPORTS:
        assert hasattr(lib, name), name


def test_header_and_binding_agree_on_symbols():
    import os
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    declared = set()
    for header in ("yvex_rocm.h", "yvex_rocm_kernels.h"):
        text = open(os.path.join(root, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)          # comments cite reference names
        declared |= set(re.findall(r"\b(yvex_[a-z0-9_]+)\s*\(", text))
    assert declared == set(abi.EXPORTS + abi.KERNEL_EXPORTS)


def test_library_exports_nothing_else():
    """Only the declared entry points leave the library, all under its own prefixes: no name of
    the reference's libyvex (yvex_backend_open, yvex_gguf_*, yvex_error_* ...) is defined, so
    the two can be linked or loaded together without one interposing on the other."""
    import subprocess
    from yvex_amd import LIB_PATH
    listing = subprocess.run(["nm", "-D", "--defined-only", LIB_PATH], capture_output=True, text=True,
                             check=True).stdout
    exported = {line.split()[-1].split("@")[0] for line in listing.splitlines() if line.strip()}
    assert exported == set(abi.EXPORTS + abi.KERNEL_EXPORTS)
    assert all(name.startswith(("yvex_rocm_", "yvex_hip_")) for name in exported)


def test_status_names(lib):
    names = {0: b"ok", -4: b"format", -5: b"unsupported", -6: b"backend", -7: b"bounds",
             -10: b"invalid-arg", -9: b"cancelled", -2: b"nomem", -8: b"state"}
    for code, name in names.items():
        assert lib.yvex_rocm_status_name(code) == name


def test_qtype_geometry_abi(lib):
    expect = {0: (1, 4), 1: (1, 2), 8: (32, 34), 10: (256, 84), 12: (256, 144), 15: (256, 292),
              16: (256, 66), 26: (1, 4), 30: (1, 2), 39: (32, 17)}
    for qtype, (block, nbytes) in expect.items():
        g = lib.yvex_rocm_gguf_qtype_geometry_find(qtype).contents
        assert (g.qtype, g.block_size, g.bytes_per_block) == (qtype, block, nbytes)
    assert lib.yvex_rocm_gguf_qtype_geometry_find(4).contents.identity == 1      # removed
    assert lib.yvex_rocm_gguf_qtype_geometry_find(41).contents.identity == 3     # outside baseline
    assert not lib.yvex_rocm_gguf_qtype_geometry_find(43)


def test_capability_registry_is_total_and_fail_closed(lib, oracle):
    reference_compute = {0, 1, 8, 10, 16, 26, 30, 39}   # src/gguf/quant_registry.c:50-103
    for qtype in range(43):
        cap = lib.yvex_rocm_quant_numeric_capability_at(qtype).contents
        assert cap.qtype == qtype and cap.known == 1
        assert bool(cap.dedicated_cpu_compute_available) == (qtype in reference_compute or qtype == 12)
        assert bool(oracle.lib().yvo_qtype_reference_cpu_compute(qtype)) == (qtype in reference_compute)
        if qtype == 12:
            assert cap.extension_of_reference == 1 and cap.device_compute_available == 1
        elif qtype == 39:
            assert cap.device_compute_available == 0     # admitted, but no kernel here yet
        else:
            assert cap.extension_of_reference == 0
            assert bool(cap.device_compute_available) == (qtype in reference_compute)
    for removed in (4, 5, 31, 32, 33, 36, 37, 38):
        assert lib.yvex_rocm_quant_numeric_capability_at(removed).contents.refusal == 2
    for outside in (40, 41, 42):
        assert lib.yvex_rocm_quant_numeric_capability_at(outside).contents.refusal == 3
    assert not lib.yvex_rocm_quant_numeric_capability_at(43)


def test_open_refuses_other_kinds_and_missing_device(lib, monkeypatch):
    monkeypatch.delenv("YVEX_TEST_ROCM_NO_DEVICE", raising=False)
    handle, err = C.c_void_p(), abi.Error()
    opts = abi.BackendOptions(abi.KIND_CUDA, None, 0)
    assert lib.yvex_rocm_backend_open(C.byref(handle), C.byref(opts), C.byref(err)) == abi.UNSUPPORTED
    assert not handle.value
    import torch
    if not torch.cuda.is_available():
        opts = abi.BackendOptions(abi.KIND_ROCM, None, 0)
        assert lib.yvex_rocm_backend_open(C.byref(handle), C.byref(opts), C.byref(err)) == abi.BACKEND
        assert b"device-unavailable" in err.message and not handle.value
    opts = abi.BackendOptions(abi.KIND_ROCM, b"gpu0", 0)
    assert lib.yvex_rocm_backend_open(C.byref(handle), C.byref(opts), C.byref(err)) == abi.INVALID_ARG


def test_seam_backend_keeps_tensors_and_refuses_compute(seam):
    lib = seam.lib
    assert lib.yvex_rocm_backend_kind_of(seam.handle) == abi.KIND_ROCM
    assert lib.yvex_rocm_backend_status_of(seam.handle) == abi.STATUS_CONTEXT_READY
    x = np.arange(16, dtype=np.float32)
    t = seam.f32(x)
    assert np.array_equal(seam.read_f32(t, 16), x)
    cap = abi.CapabilityResult()
    assert lib.yvex_rocm_backend_query_capability(seam.handle, abi.VARIANT_TENSOR_ALLOC, C.byref(cap), None) == 0
    assert cap.state == abi.CAP_SUPPORTED
    for variant in (abi.VARIANT_ATTENTION_ENCODED, abi.VARIANT_QTYPE_ROW_DOT):
        assert lib.yvex_rocm_backend_query_capability(seam.handle, variant, C.byref(cap), None) == 0
        assert cap.state == abi.CAP_UNSUPPORTED and cap.reason == abi.REASON_KERNEL_BUNDLE_ABSENT
        assert cap.kernel_bundle_available == 0 and cap.context_available == 1
    assert lib.yvex_rocm_backend_query_capability(seam.handle, 9, C.byref(cap), None) == 0
    assert cap.state == abi.CAP_UNSUPPORTED and cap.reason == abi.REASON_VARIANT_UNSUPPORTED
    assert not lib.yvex_rocm_backend_moe_operations_get(seam.handle)


def test_token_local_operation_without_kernels(seam):
    """Argument refusals come first (src/backend/cuda/moe.c:523-540), then the missing kernel
    bundle (moe.c:563-567); close is safe on an execution that never began."""
    lib = seam.lib
    plan, job, result, err = abi.LayerPlan(), abi.LayerJob(), abi.LayerResult(), abi.Error()
    handle = C.c_void_p()
    job.layer = C.pointer(plan)
    assert lib.yvex_rocm_backend_moe_begin(C.byref(handle), seam.handle, C.byref(job), C.byref(result),
                                      C.byref(err)) == abi.INVALID_ARG
    plan.hidden_width, plan.residual_streams, plan.expanded_width = 256, 2, 512
    plan.mhc_mixing_rows, plan.mhc_sinkhorn_iterations = 8, 2
    plan.rms_epsilon = plan.mhc_epsilon = 1e-6
    plan.mhc_post_multiplier, plan.activation_limit, plan.routed_scaling_factor = 2.0, 10.0, 1.0
    plan.routed_experts, plan.experts_per_token, plan.shared_experts = 8, 2, 1
    plan.expert_intermediate_width = plan.shared_intermediate_width = 256
    plan.router_class = abi.ROUTER_LEARNED
    row = np.zeros(512, np.float32)
    out = [np.zeros(n, np.float32) for n in (256, 256, 256, 2, 4)]
    job.expanded_input = row.ctypes.data
    result.combined_output, result.routed_output, result.shared_output = (a.ctypes.data for a in out[:3])
    result.combined_capacity = result.routed_capacity = result.shared_capacity = 256
    result.post, result.post_capacity = out[3].ctypes.data, 2
    result.combination, result.combination_capacity = out[4].ctypes.data, 4
    assert lib.yvex_rocm_backend_moe_begin(C.byref(handle), seam.handle, C.byref(job), C.byref(result),
                                      C.byref(err)) == abi.UNSUPPORTED
    assert not handle.value and b"kernel" in err.message
    plan.mhc_mixing_rows = 7
    assert lib.yvex_rocm_backend_moe_begin(C.byref(handle), seam.handle, C.byref(job), C.byref(result),
                                      C.byref(err)) == abi.BOUNDS
    assert lib.yvex_rocm_backend_moe_close(C.byref(handle), C.byref(err)) == 0
    assert lib.yvex_rocm_backend_moe_finish(None, C.byref(result), C.byref(err)) == abi.INVALID_ARG


def test_tensor_ownership_and_limits(monkeypatch):
    monkeypatch.setenv("YVEX_TEST_ROCM_NO_DEVICE", "1")
    from backend_helpers import Backend
    a, b = Backend(memory_limit=1024), Backend()
    rc, _ = a.tensor(2048)
    assert rc == abi.NOMEM
    ta = a.f32(np.ones(8, np.float32))
    out = np.empty(8, np.float32)
    assert b.lib.yvex_rocm_backend_tensor_read(b.handle, ta, out.ctypes.data, 32, C.byref(b.err)) == abi.FORMAT
    assert a.lib.yvex_rocm_backend_tensor_read(a.handle, ta, out.ctypes.data, 64, C.byref(a.err)) == abi.BOUNDS
    rc, unwritten = a.tensor(32)
    assert a.lib.yvex_rocm_backend_tensor_read(a.handle, unwritten, out.ctypes.data, 32, C.byref(a.err)) == abi.STATE
    assert a.lib.yvex_rocm_backend_close_checked(C.byref(a.handle), C.byref(a.err)) == abi.STATE   # live tensors
    assert a.handle.value
    stats = abi.MemoryStats()
    assert a.lib.yvex_rocm_backend_get_memory_stats(a.handle, C.byref(stats), None) == 0
    assert stats.allocated_bytes == 64 and stats.allocation_count == 2 and stats.h2d_bytes == 32
    assert a.close() == 0 and not a.handle.value
    assert b.close() == 0


def test_cleanup_failure_keeps_the_owner_for_retry(monkeypatch):
    monkeypatch.setenv("YVEX_TEST_ROCM_NO_DEVICE", "1")
    from backend_helpers import Backend
    b = Backend()
    monkeypatch.setenv("YVEX_TEST_ROCM_CLEANUP_FAILURE", "1")
    assert b.lib.yvex_rocm_backend_close_checked(C.byref(b.handle), C.byref(b.err)) == abi.BACKEND
    assert b.handle.value and b.lib.yvex_rocm_backend_status_of(b.handle) == abi.STATUS_FAILED
    monkeypatch.delenv("YVEX_TEST_ROCM_CLEANUP_FAILURE")
    assert b.lib.yvex_rocm_backend_close_checked(C.byref(b.handle), C.byref(b.err)) == 0
    assert not b.handle.value


def test_resident_resolve_semantics(seam):
    lib = seam.lib
    blob = np.arange(4096, dtype=np.uint8)
    arena, host = seam.resident(blob)
    addr = abi.ULL()
    assert lib.yvex_rocm_backend_resident_resolve(seam.handle, host + 100, 50, C.byref(addr)) == abi.RESIDENT_HIT
    assert addr.value == arena.contents.data + 100
    assert lib.yvex_rocm_backend_resident_resolve(seam.handle, host + 4000, 200, C.byref(addr)) == abi.RESIDENT_MISS
    assert lib.yvex_rocm_backend_resident_resolve(seam.handle, host - 1, 4, C.byref(addr)) == abi.RESIDENT_MISS
    assert lib.yvex_rocm_backend_resident_detach(seam.handle, None) == 0
    assert lib.yvex_rocm_backend_resident_resolve(seam.handle, host, 4, C.byref(addr)) == abi.RESIDENT_MISS


def test_workspace_bump_allocation(seam):
    lib = seam.lib
    ws = seam.workspace(4096)
    a, b = abi.ULL(), abi.ULL()
    assert lib.yvex_rocm_backend_workspace_acquire(seam.handle, 100, 256, C.byref(a)) == 1
    assert lib.yvex_rocm_backend_workspace_acquire(seam.handle, 100, 256, C.byref(b)) == 1
    assert a.value % 256 == 0 and b.value % 256 == 0 and b.value >= a.value + 100
    assert lib.yvex_rocm_backend_workspace_acquire(seam.handle, 8192, 256, C.byref(b)) == 0
    assert lib.yvex_rocm_backend_workspace_acquire(seam.handle, 16, 3, C.byref(b)) == 0     # not a power of two
    lib.yvex_rocm_backend_workspace_detach(seam.handle)
    assert lib.yvex_rocm_backend_workspace_acquire(seam.handle, 16, 16, C.byref(b)) == 0
    del ws


def matvec(seam, host, nbytes, qtype, rows, width, row_bytes, x, out, additive=None, q8=0, in_rows=1):
    facts, err = abi.OperationFacts(), abi.Error()
    rc = seam.lib.yvex_rocm_encoded_matvec(
        seam.handle, host, nbytes, qtype, rows, width, row_bytes, in_rows, x, None, 0, additive, out,
        q8, C.byref(facts), C.byref(err))
    return rc, facts, err


def test_encoded_matvec_refusal_order(seam, oracle):
    rows, width = 8, 512
    g = oracle.Generator(1, "host.matvec")
    w = g.weights(oracle.IQ2_XXS, rows, width)
    rb = oracle.row_bytes(oracle.IQ2_XXS, width)
    _, host = seam.resident(w)
    x = seam.f32(g.normal(width))
    out = seam.empty_f32(rows)
    add = seam.f32(np.zeros(rows, np.float32))
    base = dict(seam=seam, host=host, nbytes=w.nbytes, qtype=16, rows=rows, width=width, row_bytes=rb,
                x=x, out=out)
    rc, _, err = matvec(**{**base, "q8": 2})
    assert rc == abi.INVALID_ARG and b"explicitly disabled or enabled" in err.message
    for bad_qtype in (4, 40, 13, 39, 99):          # removed, outside, no codec, no kernel, unknown
        rc, _, _ = matvec(**{**base, "qtype": bad_qtype})
        assert rc == abi.UNSUPPORTED
    rc, _, _ = matvec(**{**base, "width": 500})
    assert rc == abi.BOUNDS
    rc, _, _ = matvec(**{**base, "row_bytes": rb + 2})
    assert rc == abi.BOUNDS
    rc, _, _ = matvec(**{**base, "nbytes": w.nbytes - rb})       # byte count != rows * row_bytes
    assert rc == abi.FORMAT
    unwritten = seam.empty_f32(width)
    rc, _, _ = matvec(**{**base, "x": unwritten})
    assert rc == abi.FORMAT
    rc, _, _ = matvec(**{**base, "additive": out})                # additive aliases the output
    assert rc == abi.FORMAT
    rc, _, _ = matvec(**{**base, "host": host + w.nbytes})        # outside the arena: MISS is an error
    assert rc == abi.FORMAT
    small = seam.empty_f32(rows - 1)
    rc, _, _ = matvec(**{**base, "out": small})
    assert rc == abi.FORMAT
    # a fully valid call reaches the capability gate and stops there, output left unpublished
    rc, facts, err = matvec(**{**base, "additive": add})
    assert rc == abi.UNSUPPORTED and b"kernel-bundle-absent" in err.message
    assert out.contents.is_written == 0 and facts.kernel_launches == 0


def test_encoded_gather_refusals(seam, oracle):
    rows, width = 8, 256
    w = oracle.Generator(2, "host.gather").weights(oracle.Q4_K, rows, width)
    _, host = seam.resident(w)
    out = seam.empty_f32(2 * width)
    facts, err = abi.OperationFacts(), abi.Error()
    ids = (C.c_uint * 2)(1, 9)
    call = lambda qt, ids_: seam.lib.yvex_rocm_encoded_gather(
        seam.handle, host, w.nbytes, qt, rows, width, 144, ids_, 2, out, C.byref(facts), C.byref(err))
    assert call(12, ids) == abi.BOUNDS                # row 9 of 8
    assert call(14, (C.c_uint * 2)(1, 2)) == abi.UNSUPPORTED
    assert call(12, (C.c_uint * 2)(1, 2)) == abi.UNSUPPORTED and b"kernel-bundle-absent" in err.message


def test_host_worklist_matches_oracle_and_refuses(lib, oracle):
    rng = np.random.default_rng(5)
    rows, topk, experts = 11, 3, 16
    sel = np.stack([rng.choice(experts, topk, replace=False) for _ in range(rows)]).astype(np.uint64)
    w = rng.random((rows, topk), dtype=np.float32)
    pairs = rows * topk
    arrays = {n: np.zeros(experts + 1 if n == "bucket_offsets" else max(pairs, experts), np.uint64)
              for n in ("expert_ids", "bucket_offsets", "bucket_populations", "source_pairs",
                        "source_rows", "destination_rows")}
    rw = np.zeros(pairs, np.float32)
    storage = abi.WorklistStorage(*(arrays[n].ctypes.data for n in (
        "expert_ids", "bucket_offsets", "bucket_populations", "source_pairs", "source_rows",
        "destination_rows")), rw.ctypes.data, experts, pairs)
    obs, err = abi.WorklistObservation(), abi.Error()
    rc = lib.yvex_rocm_expert_worklist_build(sel.ctypes.data, w.ctypes.data, pairs, topk, experts,
                                        C.byref(storage), C.byref(obs), C.byref(err))
    assert rc == 0
    orc, want = oracle.worklist_build(sel, w, topk, experts)
    n = len(want["expert_ids"])
    assert orc == 0 and obs.bucket_count == n and obs.pair_count == pairs
    assert obs.maximum_bucket_population == int(want["bucket_populations"].max())
    assert np.array_equal(arrays["expert_ids"][:n], want["expert_ids"])
    assert np.array_equal(arrays["bucket_offsets"][:n + 1], want["bucket_offsets"])
    assert np.array_equal(arrays["source_pairs"][:pairs], want["source_pairs"])
    assert np.array_equal(arrays["source_rows"][:pairs], want["source_rows"])
    assert np.array_equal(arrays["destination_rows"][:pairs], want["destination_rows"])
    assert np.array_equal(rw, want["route_weights"])
    # stable: inside a bucket the source pairs ascend; populations sum to the pair count
    for b in range(n):
        s = arrays["source_pairs"][int(want["bucket_offsets"][b]):int(want["bucket_offsets"][b + 1])]
        assert np.all(np.diff(s.astype(np.int64)) > 0)
    assert sum(obs.population_histogram) == n
    bad = sel.copy()
    bad[0, 0] = experts
    assert lib.yvex_rocm_expert_worklist_build(bad.ctypes.data, w.ctypes.data, pairs, topk, experts,
                                          C.byref(storage), C.byref(obs), C.byref(err)) == abi.FORMAT
    w2 = w.copy()
    w2[1, 1] = np.inf
    assert lib.yvex_rocm_expert_worklist_build(sel.ctypes.data, w2.ctypes.data, pairs, topk, experts,
                                          C.byref(storage), C.byref(obs), C.byref(err)) == abi.FORMAT
    storage.pair_capacity = pairs - 1
    assert lib.yvex_rocm_expert_worklist_build(sel.ctypes.data, w.ctypes.data, pairs, topk, experts,
                                          C.byref(storage), C.byref(obs), C.byref(err)) == abi.INVALID_ARG



def test_shared_sessions_borrow_the_owner(monkeypatch):
    """yvex_backend_open_shared_cuda's contract (src/backend/cuda/backend.c:1913-2000,
    src/backend/residency.c:47-57, src/backend/core.c:251-343) on the host-only backend: a child
    needs an owning backend, attaches the arena its owner published (same base and generation,
    the owner's device address, no copy), keeps tensors and a workspace of its own, and the
    owner does not close while a child is open."""
    monkeypatch.setenv("YVEX_TEST_ROCM_NO_DEVICE", "1")
    from yvex_amd.host import Backend
    owner = Backend()
    assert owner.ok
    blob = np.arange(4096, dtype=np.uint8)
    arena, host = owner.resident(blob, generation=5)
    child = Backend(shared_with=owner, memory_limit=1 << 20)
    assert child.ok and child.lib.yvex_rocm_backend_kind_of(child.handle) == abi.KIND_ROCM
    assert Backend(shared_with=child).open_rc == abi.INVALID_ARG
    # the owner's arena: wrong generation, wrong base, then the matching attach
    assert child.attach_shared_arena(arena, host, blob.nbytes, generation=4) == abi.STATE
    assert child.attach_shared_arena(arena, host + 256, blob.nbytes - 256, generation=5) == abi.STATE
    assert child.attach_shared_arena(arena, host, blob.nbytes, generation=5) == 0, child.err.message
    assert child.attach_shared_arena(arena, host, blob.nbytes, generation=5) == abi.STATE      # already attached
    mine, theirs = abi.ULL(), abi.ULL()
    for b, out in ((owner, theirs), (child, mine)):
        assert b.lib.yvex_rocm_backend_resident_resolve(b.handle, C.c_void_p(host + 100), 50, C.byref(out)) == abi.RESIDENT_HIT
    assert mine.value == theirs.value
    # tensors belong to the session that allocated them, under its own limit
    rc, t = child.tensor(1024)
    assert rc == 0 and t.contents.owner == child.handle.value
    assert child.tensor(2 << 20)[0] == abi.NOMEM
    assert owner.lib.yvex_rocm_backend_tensor_write(owner.handle, t, blob.ctypes.data, 1024, C.byref(owner.err)) != 0
    # the owner waits for its sessions
    assert owner.close() == abi.STATE and owner.handle.value
    assert child.close() == 0, child.err.message
    assert owner.close() == 0, owner.err.message
