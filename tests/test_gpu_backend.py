"""The drop-in boundary on a real MI355X: every call goes through include/yvex_rocm.h.

Scenarios follow tests/unit/cuda/quant_qtype.c:273-517 (encoded matvec: F32 and Q8 activation
paths, additive fusion, refusals, memory facts) and tests/unit/cuda/info.c:316-822 (width-N MoE:
selection equal to the CPU router, weights <= 1e-6, refusal before mutation for an unsupported
width, FORMAT for mixed gate/up activations).
"""
import ctypes as C

import numpy as np
import pytest

from yvex_amd import abi

pytestmark = pytest.mark.gpu


@pytest.fixture
def backend(gpu):
    from backend_helpers import Backend
    b = Backend()
    assert b.ok, b.err.message
    assert b.lib.yvex_rocm_backend_status_of(b.handle) == abi.STATUS_READY
    yield b
    assert b.close() == 0


def same_as_cpu(got, want):
    """North star: final fp32 outputs within 1e-3 relative / 1e-5 absolute of the CPU path. The
    kernels form every row dot as the CPU path does (the same float terms, added in double), so
    they are held to more: the CPU path's values bit for bit."""
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert np.all(err <= 1e-5 + 1e-3 * np.abs(want)), f"{int((err > 1e-5 + 1e-3 * np.abs(want)).sum())} outside tolerance"
    assert np.array_equal(got, want), f"{int((got != want).sum())} of {got.size} values differ"


def close_to(got, want, rel=1e-3, abs_=1e-5):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return np.all(np.abs(got - want) <= abs_ + rel * np.abs(want))


def run_matvec(b, host, w, qt, rows, width, x_tensor, out, in_rows, q8, additive=None):
    facts, err = abi.OperationFacts(), abi.Error()
    rc = b.lib.yvex_rocm_encoded_matvec(
        b.handle, host, w.nbytes, qt, rows, width, w.nbytes // rows, in_rows, x_tensor, None, 0,
        additive, out, q8, C.byref(facts), C.byref(err))
    return rc, facts, err


@pytest.mark.parametrize("qtype,rows,width,in_rows", [
    ("Q8_0", 64, 4096, 1), ("IQ2_XXS", 96, 2048, 1), ("IQ2_XXS", 24, 7168, 3),
    ("Q4_K", 40, 7168, 1), ("Q4_K", 16, 2048, 16), ("Q2_K", 20, 512, 2)])
def test_encoded_matvec_both_activation_paths(backend, oracle, qtype, rows, width, in_rows):
    b = backend
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"backend.matvec.{qtype}.{rows}.{width}")
    w = g.weights(qt, rows, width)
    x = g.normal(in_rows * width).reshape(in_rows, width)
    _, host = b.resident(w)
    b.workspace(1 << 20)
    xt, out = b.f32(x), b.empty_f32(in_rows * rows)
    rc, facts, err = run_matvec(b, host, w, qt, rows, width, xt, out, in_rows, 0)
    assert rc == 0, err.message
    assert out.contents.is_written == 1
    got = b.read_f32(out, in_rows * rows).reshape(in_rows, rows)
    assert close_to(got, oracle.matvec(qt, w, rows, width, x))
    assert facts.active_weight_bytes == w.nbytes and facts.compulsory_memory_facts_available == 1
    assert facts.activation_bytes == x.nbytes + got.nbytes and facts.d2h_bytes == 4
    # Q8_K activations: exact against the integer oracle path, and within the reference's own
    # bound of the CPU path fed with the dequantised activations
    rc, facts, err = run_matvec(b, host, w, qt, rows, width, xt, out, in_rows, 1)
    assert rc == 0, err.message
    got8 = b.read_f32(out, in_rows * rows).reshape(in_rows, rows)
    act = oracle.q8k_quantize(x)
    want8 = oracle.q8_matvec(qt, w, rows, width, act, in_rows)
    if qtype == "Q8_0":
        assert close_to(got8, want8, rel=1e-5, abs_=1e-5)
    else:
        assert np.array_equal(got8.view(np.uint32), want8.view(np.uint32))
    deq = oracle.q8k_dequantize(act).reshape(in_rows, width)
    want = oracle.matvec(qt, w, rows, width, deq)
    assert np.all(np.abs(got8 - want) <= 1e-5 * (1 + np.abs(want)) * 10)
    assert facts.temporary_bytes == 4 + in_rows * (width // 256) * 292


def test_encoded_matvec_additive_and_refusals_on_device(backend, oracle):
    b = backend
    rows, width = 32, 2048
    g = oracle.Generator(3, "backend.additive")
    w = g.weights(oracle.IQ2_XXS, rows, width)
    x, add = g.normal(width), g.normal(rows)
    _, host = b.resident(w)
    xt, at, out = b.f32(x), b.f32(add), b.empty_f32(rows)
    rc, _, err = run_matvec(b, host, w, 16, rows, width, xt, out, 1, 0, additive=at)
    assert rc == 0, err.message
    want = oracle.matvec(16, w, rows, width, x)[0] + add
    assert close_to(b.read_f32(out, rows), want)
    # Q8 path without a workspace is refused, the output stays unpublished
    rc, _, err = run_matvec(b, host, w, 16, rows, width, xt, out, 1, 1)
    assert rc == abi.NOMEM and out.contents.is_written == 0
    # aliasing and unwritten inputs
    assert run_matvec(b, host, w, 16, rows, width, xt, out, 1, 0, additive=out)[0] == abi.FORMAT
    assert run_matvec(b, host, w, 16, rows, width, b.empty_f32(width), out, 1, 0)[0] == abi.FORMAT
    # non-finite activations surface as FORMAT through the device status word
    bad = x.copy()
    bad[5] = np.inf
    rc, _, err = run_matvec(b, host, w, 16, rows, width, b.f32(bad), out, 1, 0)
    assert rc == abi.FORMAT and b"invalid numerics" in err.message and out.contents.is_written == 0
    # and the backend keeps working afterwards
    assert run_matvec(b, host, w, 16, rows, width, xt, out, 1, 0)[0] == 0


@pytest.mark.parametrize("qtype,elements", [("Q8_0", 4096), ("IQ2_XXS", 2048), ("Q4_K", 1024), ("Q2_K", 512),
                                            ("F32", 333), ("BF16", 77)])
def test_quant_row_dot_probe(backend, oracle, qtype, elements):
    """The serial device row dot against the CPU row dot: the reference's bar is
    1e-6 * (1 + |cpu|) (tests/unit/cuda/quant_qtype.c:118-120); the same order and arithmetic
    give the same bits here."""
    qt = {"BF16": 30}.get(qtype) or getattr(oracle, qtype)
    g = oracle.Generator(4, f"probe.{qtype}")
    if qtype == "BF16":
        row = (g.normal(elements).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
        decoded = (row.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    else:
        row = g.weights(qt, 1, elements)
    x = g.normal(elements)
    out, err = C.c_float(), abi.Error()
    rc = backend.lib.yvex_rocm_quant_row_dot(backend.handle, qt, row.ctypes.data, row.nbytes, x.ctypes.data,
                                             elements, C.byref(out), None, C.byref(err))
    assert rc == 0, err.message
    if qtype == "BF16":
        want = np.float32(np.sum(decoded.astype(np.float64) * x.astype(np.float64)))
        assert abs(out.value - want) <= 1e-6 * (1 + abs(want))
    elif qtype == "Q4_K":       # outside the reference's CPU path: the oracle's float decode, double sum
        want = np.float32(np.sum(oracle.decode_rows(qt, row, elements)[0].astype(np.float64) * x.astype(np.float64)))
        assert abs(out.value - want) <= 1e-6 * (1 + abs(want))
    else:
        rc, want = oracle.cpu_dot(qt, row, x)
        assert rc == 0 and np.float32(out.value).view(np.uint32) == np.float32(want).view(np.uint32)
    lib, h = backend.lib, backend.handle
    assert lib.yvex_rocm_quant_row_dot(h, 2, row.ctypes.data, row.nbytes, x.ctypes.data, elements, C.byref(out),
                                       None, C.byref(err)) == abi.UNSUPPORTED
    assert lib.yvex_rocm_quant_row_dot(h, qt, row.ctypes.data, row.nbytes + 2, x.ctypes.data, elements,
                                       C.byref(out), None, C.byref(err)) == abi.BOUNDS
    assert lib.yvex_rocm_quant_row_dot(h, qt, None, row.nbytes, x.ctypes.data, elements, C.byref(out), None,
                                       C.byref(err)) == abi.INVALID_ARG


def test_encoded_matvec_split_input(backend, oracle):
    """The reference's split projection (speculation: src/backend/cuda/qtype.c:256-281,
    kernels.cu:736-782): a row is head ++ tail, every value rounded to bf16, F32 activations even
    when the Q8 policy is asked for."""
    b = backend
    rows, width, head_width, in_rows = 48, 1024, 384, 3
    g = oracle.Generator(8, "backend.split")
    w = g.weights(oracle.Q8_0, rows, width)
    _, host = b.resident(w)
    x = g.normal(in_rows * width).reshape(in_rows, width)
    head, tail = b.f32(x[:, :head_width]), b.f32(x[:, head_width:])
    out = b.empty_f32(in_rows * rows)
    facts, err = abi.OperationFacts(), abi.Error()

    def run(tail_tensor, head_w, q8=0):
        return b.lib.yvex_rocm_encoded_matvec(
            b.handle, host, w.nbytes, oracle.Q8_0, rows, width, w.nbytes // rows, in_rows, head, tail_tensor,
            head_w, None, out, q8, C.byref(facts), C.byref(err))

    assert run(tail, head_width) == abi.NOMEM                   # needs the workspace for the joined rows
    b.workspace(in_rows * width * 4 + 256)
    bits = x.view(np.uint32)
    rounded = ((bits + 0x7fff + ((bits >> 16) & 1)) & 0xffff0000).view(np.float32)
    want = oracle.matvec(oracle.Q8_0, w, rows, width, rounded)
    for q8 in (0, 1):
        assert run(tail, head_width, q8) == 0, err.message
        got = b.read_f32(out, in_rows * rows).reshape(in_rows, rows)
        assert close_to(got, want) and facts.kernel_launches == 3
    assert run(tail, 0) == abi.FORMAT and run(None, head_width) == abi.FORMAT
    assert run(tail, width) == abi.FORMAT and run(out, head_width) == abi.FORMAT


def test_launch_and_sync_failure_seams(backend, oracle, monkeypatch):
    b = backend
    rows, width = 8, 256
    w = oracle.Generator(4, "backend.seams").weights(oracle.Q8_0, rows, width)
    _, host = b.resident(w)
    xt, out = b.f32(np.ones(width, np.float32)), b.empty_f32(rows)
    monkeypatch.setenv("YVEX_TEST_ROCM_LAUNCH_FAILURE", "1")
    rc, _, err = run_matvec(b, host, w, 8, rows, width, xt, out, 1, 0)
    assert rc == abi.BACKEND and out.contents.is_written == 0
    monkeypatch.delenv("YVEX_TEST_ROCM_LAUNCH_FAILURE")
    monkeypatch.setenv("YVEX_TEST_ROCM_SYNC_FAILURE", "1")
    rc, _, err = run_matvec(b, host, w, 8, rows, width, xt, out, 1, 0)
    assert rc == abi.BACKEND and out.contents.is_written == 0
    monkeypatch.delenv("YVEX_TEST_ROCM_SYNC_FAILURE")
    assert run_matvec(b, host, w, 8, rows, width, xt, out, 1, 0)[0] == 0


def test_bundle_failure_seam_is_fail_closed(gpu, monkeypatch):
    monkeypatch.setenv("YVEX_TEST_ROCM_BUNDLE_FAILURE", "1")
    from backend_helpers import Backend
    b = Backend()
    assert b.ok and b.lib.yvex_rocm_backend_status_of(b.handle) == abi.STATUS_CONTEXT_READY
    t = b.f32(np.arange(4, dtype=np.float32))
    assert np.array_equal(b.read_f32(t, 4), np.arange(4, dtype=np.float32))
    cap = abi.CapabilityResult()
    b.lib.yvex_rocm_backend_query_capability(b.handle, abi.VARIANT_ATTENTION_ENCODED, C.byref(cap), None)
    assert cap.state == abi.CAP_UNSUPPORTED and cap.reason == abi.REASON_KERNEL_BUNDLE_ABSENT
    assert not b.lib.yvex_rocm_backend_moe_operations_get(b.handle)
    assert b.close() == 0


def test_bandwidth_probe_publishes_sustainable_rates(backend):
    """include/yvex/internal/backend.h:174-185: five timed samples of streaming reads and of
    device-to-device copies; the published rates are the working set over the median sample."""
    evidence, err = abi.BandwidthEvidence(), abi.Error()
    rc = backend.lib.yvex_rocm_backend_bandwidth_probe(backend.handle, C.byref(evidence), C.byref(err))
    assert rc == 0, err.message
    assert evidence.schema_version == 1 and evidence.sample_count == 5 and evidence.working_set_bytes == 1 << 30
    reads, copies = sorted(evidence.stream_elapsed_ns), sorted(evidence.copy_elapsed_ns)
    assert reads[0] > 0 and copies[0] > 0
    moved = evidence.working_set_bytes * evidence.iterations
    assert abs(evidence.sustainable_read_bytes_per_second - moved * 1e9 / reads[2]) <= 2
    assert abs(evidence.sustainable_copy_bytes_per_second - moved * 1e9 / copies[2]) <= 2
    # an HBM3E part: terabytes a second, and below the 8 TB/s peak
    assert 1e12 < evidence.sustainable_read_bytes_per_second < 8e12
    assert 0.5e12 < evidence.sustainable_copy_bytes_per_second < 8e12
    assert list(evidence.coherent_host_elapsed_ns) == [0] * 5
    print(f"read {evidence.sustainable_read_bytes_per_second / 1e12:.2f} TB/s, "
          f"copy {evidence.sustainable_copy_bytes_per_second / 1e12:.2f} TB/s")
    assert backend.lib.yvex_rocm_backend_bandwidth_probe(backend.handle, None, C.byref(err)) == abi.INVALID_ARG


def test_encoded_gather(backend, oracle):
    b = backend
    rows, width = 40, 512
    w = oracle.Generator(6, "backend.gather").weights(oracle.IQ2_XXS, rows, width)
    _, host = b.resident(w)
    b.workspace(4096)
    ids = np.array([39, 0, 7, 7], np.uint32)
    out = b.empty_f32(ids.size * width)
    facts, err = abi.OperationFacts(), abi.Error()
    rc = b.lib.yvex_rocm_encoded_gather(b.handle, host, w.nbytes, 16, rows, width, 132,
                                                ids.ctypes.data, ids.size, out, C.byref(facts),
                                                C.byref(err))
    assert rc == 0, err.message
    got = b.read_f32(out, ids.size * width).reshape(ids.size, width)
    want = oracle.decode_rows(16, w, width, ids)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert facts.active_weight_bytes == ids.size * 132


def run_greedy(b, logits, rows, width):
    tokens, best, ties = np.full(rows, 7, np.uint32), np.full(rows, 7, np.float32), np.full(rows, 7, np.uint64)
    facts, err = abi.OperationFacts(), abi.Error()
    rc = b.lib.yvex_rocm_select_greedy_rows(b.handle, logits, rows, width, tokens.ctypes.data,
                                                    best.ctypes.data, ties.ctypes.data, C.byref(facts),
                                                    C.byref(err))
    return rc, tokens, best, ties, facts, err


def test_select_greedy_rows(backend, oracle):
    """The sampling table's greedy entry (sampling.c:284-392): results, facts, refusals."""
    b = backend
    rows, width = 3, 5000
    rng = np.random.default_rng(11)
    values = rng.standard_normal((rows, width)).astype(np.float32)
    values[1, 4999] = values[1, 12] = 9.0
    logits = b.f32(values)
    # no workspace attached: nowhere to put the device results
    rc, tokens, best, ties, facts, err = run_greedy(b, logits, rows, width)
    assert rc == abi.NOMEM and not tokens.any() and not ties.any()
    b.workspace(4096)
    rc, tokens, best, ties, facts, err = run_greedy(b, logits, rows, width)
    assert rc == 0, err.message
    _, want_tokens, want_best, want_ties = oracle.argmax_f32(values)
    assert np.array_equal(tokens, want_tokens) and np.array_equal(best, want_best)
    assert np.array_equal(ties, want_ties) and ties[1] == 2 and tokens[1] == 12
    assert facts.kernel_launches == 1 and facts.download_count == 4
    assert facts.d2h_bytes == rows * 16 + 4 and facts.activation_bytes == values.nbytes
    # refusals: rows past the tensor, an unwritten tensor, a non-finite logit (outputs zeroed)
    assert run_greedy(b, logits, rows + 1, width)[0] == abi.FORMAT
    assert run_greedy(b, b.empty_f32(width), 1, width)[0] == abi.FORMAT
    values[2, 77] = np.nan
    rc, tokens, best, ties, facts, err = run_greedy(b, b.f32(values), rows, width)
    assert rc == abi.FORMAT and not tokens.any() and not best.any() and not ties.any()
    assert facts.kernel_launches == 0
    # a vocabulary-sized row: shared among workgroups through the workspace (two launches)
    b.workspace(1 << 16)
    wide = rng.standard_normal((1, 129280)).astype(np.float32)
    rc, tokens, best, ties, facts, err = run_greedy(b, b.f32(wide), 1, 129280)
    assert rc == 0, err.message
    assert tokens[0] == np.argmax(wide[0]) and best[0] == wide[0].max() and ties[0] == 1
    assert facts.kernel_launches == 2


def sweep_image_decision(experts, rows, width, consumer):
    """The decision that asks derived_layout_plan/build for the expert sweeps' image."""
    d = abi.ExecutionDecision()
    d.expert_count, d.canonical_qtype = experts, 16
    d.canonical_row_width, d.canonical_row_count = width, rows
    d.encoded_bytes = rows * (width // 256) * 66
    d.consumer, d.layout, d.derived_asset_required = consumer, abi.LAYOUT_DERIVED, 1
    d.kernel_family = abi.FAMILY_GFX950
    return d


class MoeCase:
    """One synthetic layer resident on the backend plus everything execute_rows needs."""

    def __init__(self, b, oracle, *, qtype="IQ2_XXS", hidden=512, intermediate=256, experts=8, topk=2,
                 rows=5, act=abi.ACT_DEVICE_ENCODED, scoring=abi.SCORING_SQRT_SOFTPLUS, bias=True,
                 shared=True, family=abi.FAMILY_GFX950, seed=42, streams=0, iterations=20, hash_vocab=0,
                 down_qtype=None, sweep_image=(), arena_from=None, norm_qtype="BF16", bias_qtype="F32",
                 shared_qtype=None):
        """arena_from: a MoeCase of the same layer on the owning backend of `b` (a shared session):
        its published arena is attached instead of another copy being made resident."""
        self.b, self.oracle = b, oracle
        self.streams, self.iterations = streams, iterations
        expanded = hidden * max(streams, 1)
        mixing = (streams + 2) * streams
        qt = getattr(oracle, qtype)
        self.qt, self.rows, self.hidden, self.experts, self.topk = qt, rows, hidden, experts, topk
        qt_down = getattr(oracle, down_qtype) if down_qtype else qt
        self.qtypes = (qt, qt, qt_down)
        # the shared expert's three matrices in a format of their own (the reference's model file
        # keeps it in Q8_0)
        qs = getattr(oracle, shared_qtype) if shared_qtype else None
        self.shared_qtypes = (qs, qs, qs) if shared_qtype else self.qtypes
        self.intermediate, self.scoring = intermediate, scoring
        g = oracle.Generator(seed, f"backend.moe.{qtype}.{hidden}.{experts}")
        parts = {
            "router": g.normal(experts * hidden, 0.05).view(np.uint8),
            "bias": (g.normal(experts) * 0.05).astype(np.float32).view(np.uint8),
            "gate": g.weights(qt, experts * intermediate, hidden),
            "up": g.weights(qt, experts * intermediate, hidden),
            "down": g.weights(qt_down, experts * hidden, intermediate),
            "sgate": g.weights(self.shared_qtypes[0], intermediate, hidden),
            "sup": g.weights(self.shared_qtypes[1], intermediate, hidden),
            "sdown": g.weights(self.shared_qtypes[2], hidden, intermediate),
        }
        # the correction bias as F32 values (read where they lie) or as BF16 values (decoded into
        # the workspace first)
        self.bias_qt = getattr(oracle, bias_qtype)
        self.bias_values = parts["bias"].view(np.float32)
        if bias_qtype == "BF16":
            parts["bias"] = (self.bias_values.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
            self.bias_values = (parts["bias"].view(np.uint16).astype(np.uint32) << 16).view(np.float32)
        self.hash_vocab = hash_vocab
        if hash_vocab:  # hash router: an I32 table of expert ordinals per token id
            rng = np.random.default_rng(seed)
            self.table = np.stack([rng.permutation(experts)[:topk] for _ in range(hash_vocab)]).astype(np.int32)
            self.tokens = rng.integers(0, hash_vocab, rows).astype(np.uint32)
            parts["table"] = self.table.view(np.uint8).ravel()
        if streams:     # residual-stream envelope: mixing function, scale, base (F32) and BF16 norm weights
            parts["function"] = g.normal(mixing * expanded, 0.05).view(np.uint8)
            parts["scale"] = g.normal(3, 0.7).view(np.uint8)
            parts["base"] = g.normal(mixing, 0.5).view(np.uint8)
            # norm weights as BF16 or F32 values (the ingress decodes them itself) or as I32 values
            # (a decode launch in front of it)
            self.norm_qt = getattr(oracle, norm_qtype)
            values = (1.0 + g.normal(hidden, 0.2)).astype(np.float32)
            if norm_qtype == "BF16":
                parts["norm"] = (values.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
            elif norm_qtype == "F32":
                parts["norm"] = values.view(np.uint8)
            else:
                parts["norm"] = np.rint(values * 2.0).astype(np.int32).view(np.uint8)
        # experts held as the sweeps' image: built by the library's host builder, resident beside
        # the canonical bytes
        self.decisions = {}
        for group, names in (("routed", ("gate", "up", "down")), ("shared", ("sgate", "sup", "sdown"))):
            if group not in sweep_image:
                continue
            for name in names:
                down = name.endswith("down")
                if down and qt_down != oracle.IQ2_XXS:
                    continue        # (down rows of another format are read as they lie)
                decision = sweep_image_decision(
                    1 if group == "shared" else experts, (hidden if down else intermediate) * (1 if group == "shared" else experts),
                    intermediate if down else hidden,
                    abi.CONSUMER_SHARED_EXPERT if group == "shared" else
                    abi.CONSUMER_ROUTED_DOWN if down else abi.CONSUMER_ROUTED_GATE_UP)
                storage, err = abi.ULL(), abi.Error()
                assert b.lib.yvex_rocm_moe_derived_layout_plan(C.byref(decision), C.byref(storage), C.byref(err)) == 0, err.message
                image = np.full(storage.value, 0xA5, np.uint8)
                assert b.lib.yvex_rocm_moe_derived_layout_build(
                    C.byref(decision), parts[name].ctypes.data, parts[name].nbytes, image.ctypes.data,
                    image.nbytes, C.byref(err)) == 0, err.message
                parts[name + ".image"] = image
                self.decisions[name] = decision
        self.parts = parts
        offsets, cursor = {}, 0
        for name, blob in parts.items():
            offsets[name] = cursor
            cursor += (blob.nbytes + 255) // 256 * 256
        arena = np.zeros(cursor, np.uint8)
        for name, blob in parts.items():
            arena[offsets[name]:offsets[name] + blob.nbytes] = blob
        if arena_from is None:
            arena_tensor, host = b.resident(arena)
        else:
            arena_tensor, host = arena_from.arena_tensor, arena_from.host
            assert b.attach_shared_arena(arena_tensor, host, arena.nbytes) == 0, b.err.message
        self.host, self.offsets, self.arena_tensor, self.arena_bytes = host, offsets, arena_tensor, arena.nbytes
        self.x = g.normal(rows * expanded).reshape(rows, expanded)
        if streams:
            bits = self.x.view(np.uint32)       # bf16 values, as the CPU path expects of its input
            self.x = ((bits + 0x7fff + ((bits >> 16) & 1)) & 0xffff0000).view(np.float32)
        self.plan = abi.LayerPlan()
        p = self.plan
        p.schema_version, p.router_class, p.scoring = 1, abi.ROUTER_LEARNED, scoring
        p.hidden_width, p.expanded_width = hidden, expanded
        p.residual_streams = max(streams, 1)
        if streams:
            p.mhc_mixing_rows, p.mhc_sinkhorn_iterations = mixing, iterations
            p.rms_epsilon, p.mhc_epsilon, p.mhc_post_multiplier = 1e-6, 1e-6, 2.0
        p.routed_experts, p.shared_experts, p.experts_per_token = experts, int(shared), topk
        p.expert_intermediate_width = p.shared_intermediate_width = intermediate
        p.routed_scaling_factor, p.activation_limit = 1.5, 10.0
        p.requires_correction_bias, p.normalize_topk_probabilities = int(bias), 1
        if hash_vocab:
            p.router_class, p.hash_table_rows, p.hash_table_columns = abi.ROUTER_HASH, hash_vocab, topk
        self.job = abi.LayerJob()
        self.job.layer = C.pointer(self.plan)
        rb_h, rb_i = oracle.row_bytes(qt, hidden), oracle.row_bytes(qt_down, intermediate)

        def view(slot, name, q, width, count, row_bytes, activation=act):
            v = self.job.weights[slot]
            v.qtype, v.layout, v.activation, v.kernel_family = q, abi.LAYOUT_EXPERT_MAJOR, activation, family
            v.encoded, v.encoded_bytes = host + offsets[name], parts[name].nbytes
            v.storage_bytes = parts[name].nbytes
            v.row_bytes, v.row_width, v.row_count = row_bytes, width, count
            if name + ".image" in parts:
                v.layout = abi.LAYOUT_DERIVED
                v.encoded, v.storage_bytes = host + offsets[name + ".image"], parts[name + ".image"].nbytes

        view(abi.W_ROUTER, "router", 0, hidden, experts, hidden * 4, abi.ACT_DEVICE_F32)
        view(abi.W_ROUTER_BIAS, "bias", self.bias_qt, experts, 1, oracle.row_bytes(self.bias_qt, experts),
             abi.ACT_DEVICE_F32)
        view(abi.W_ROUTED_GATE, "gate", qt, hidden, experts * intermediate, rb_h)
        view(abi.W_ROUTED_UP, "up", qt, hidden, experts * intermediate, rb_h)
        view(abi.W_ROUTED_DOWN, "down", qt_down, intermediate, experts * hidden, rb_i)
        sq = self.shared_qtypes
        view(abi.W_SHARED_GATE, "sgate", sq[0], hidden, intermediate, oracle.row_bytes(sq[0], hidden))
        view(abi.W_SHARED_UP, "sup", sq[1], hidden, intermediate, oracle.row_bytes(sq[1], hidden))
        view(abi.W_SHARED_DOWN, "sdown", sq[2], intermediate, hidden, oracle.row_bytes(sq[2], intermediate))
        if hash_vocab:
            view(abi.W_ROUTER_TABLE, "table", 26, topk, hash_vocab, topk * 4, abi.ACT_DEVICE_F32)
        if streams:
            view(abi.W_MHC_FUNCTION, "function", 0, expanded, mixing, expanded * 4, abi.ACT_DEVICE_F32)
            view(abi.W_MHC_SCALE, "scale", 0, 3, 1, 12, abi.ACT_DEVICE_F32)
            view(abi.W_MHC_BASE, "base", 0, mixing, 1, mixing * 4, abi.ACT_DEVICE_F32)
            view(abi.W_FFN_NORM, "norm", self.norm_qt, hidden, 1, oracle.row_bytes(self.norm_qt, hidden),
                 abi.ACT_DEVICE_F32)
        self.ops = b.lib.yvex_rocm_backend_moe_operations_get(b.handle).contents
        need, err = abi.ULL(), abi.Error()
        assert self.ops.workspace_required(C.byref(self.plan), rows, C.byref(need), C.byref(err)) == 0
        self.workspace_bytes = need.value
        self.rows_in, self.rows_out = b.f32(self.x), b.empty_f32(rows * expanded)
        self.batch = abi.RowBatch()
        bt = self.batch
        bt.schema_version, bt.row_count, bt.row_width, bt.row_stride = 1, rows, expanded, expanded
        bt.device_rows, bt.device_outputs = self.rows_in, self.rows_out
        bt.provenance, bt.execution_class = abi.BATCH_MULTI_SESSION, 1
        if hash_vocab:
            bt.token_ids, bt.token_ids_present = self.tokens.ctypes.data, 1
        self.sel = np.zeros(rows * topk, np.uint64)
        self.wts = np.zeros(rows * topk, np.float32)
        self.combined = np.zeros((rows, hidden), np.float32)
        self.out = abi.RowBatchOutput()
        self.out.combined_rows, self.out.combined_capacity = self.combined.ctypes.data, rows * hidden
        self.out.selected_experts, self.out.selected_weights = self.sel.ctypes.data, self.wts.ctypes.data
        self.out.selection_capacity = rows * topk
        if streams:
            self.post = np.zeros((rows, streams), np.float32)
            self.comb = np.zeros((rows, streams, streams), np.float32)
            self.out.post_rows, self.out.post_capacity = self.post.ctypes.data, self.post.size
            self.out.combination_rows, self.out.combination_capacity = self.comb.ctypes.data, self.comb.size
        self.result, self.err = abi.RowBatchResult(), abi.Error()

    def execute(self):
        return self.ops.execute_rows(self.b.handle, C.byref(self.job), C.byref(self.batch),
                                     C.byref(self.out), C.byref(self.result), C.byref(self.err))

    def oracle_layer(self, act_q8):
        o, p = self.oracle, self.parts
        x, ingress = self.x, None
        if self.streams:      # src/graph/moe.c:446-495 in front, numeric.c:828-877 behind
            norm = o.decode_rows(self.norm_qt, p["norm"], self.hidden)[0]
            rc, x, post, comb = o.moe_ffn_prepare(
                o.F32, p["function"], self.x, p["scale"].view(np.float32), p["base"].view(np.float32), norm,
                streams=self.streams, width=self.hidden, iterations=self.iterations, rms_epsilon=1e-6,
                mhc_epsilon=1e-6, post_multiplier=2.0)
            assert rc == 0
            ingress = (x, post, comb)
        router = p["router"].view(np.float32).reshape(self.experts, self.hidden)
        logits = o.matvec(o.F32, p["router"], self.experts, self.hidden, x)
        assert np.allclose(logits, x @ router.T, rtol=1e-4, atol=1e-5)
        bias = self.bias_values if self.plan.requires_correction_bias else None
        shared = (p["sgate"], p["sup"], p["sdown"]) if self.plan.shared_experts else None
        own_format = shared is not None and self.shared_qtypes != self.qtypes
        want = o.moe_layer(hidden=self.hidden, intermediate=self.intermediate, experts=self.experts,
                           topk=self.topk, qtypes=self.qtypes, routed=(p["gate"], p["up"], p["down"]),
                           shared=None if own_format else shared, inputs=x, logits=logits, bias=bias,
                           scoring=self.scoring, normalize=True, scaling=1.5, act_q8=act_q8, threads=8,
                           hash_selected=self.table[self.tokens] if self.hash_vocab else None)
        if own_format:
            # the layer's own composition (src/runtime/moe.c:596-632) with the shared expert run in
            # its format: route weight one, combined = bf16(routed + shared)
            rows = np.ascontiguousarray(x, np.float32).reshape(-1, self.hidden)
            outs = []
            for row in rows:
                rc, out, _, _ = o.moe_expert(self.shared_qtypes, *shared, self.hidden, self.intermediate, row, 1.0,
                                             act_q8=act_q8)
                assert rc == 0
                outs.append(out)
            want["shared"] = np.stack(outs)
            bits = (want["routed"] + want["shared"]).astype(np.float32).view(np.uint32)
            want["combined"] = ((bits + 0x7fff + ((bits >> 16) & 1)) & 0xffff0000).view(np.float32)
        if ingress:
            want["normalized"], want["post"], want["combination"] = ingress
            rc, want["envelope"] = o.mhc_post(want["combined"], self.x, ingress[1], ingress[2],
                                              streams=self.streams, width=self.hidden)
            assert rc == 0
        return want


@pytest.mark.parametrize("qtype,act,scoring,shared,bias_qtype", [
    ("IQ2_XXS", abi.ACT_DEVICE_ENCODED, abi.SCORING_SQRT_SOFTPLUS, True, "F32"),
    ("IQ2_XXS", abi.ACT_DEVICE_F32, abi.SCORING_SIGMOID, True, "F32"),
    ("Q4_K", abi.ACT_DEVICE_ENCODED, abi.SCORING_SIGMOID, False, "BF16"),
    ("Q8_0", abi.ACT_DEVICE_ENCODED, abi.SCORING_SQRT_SOFTPLUS, True, "F32")])
def test_execute_rows_matches_cpu_layer(backend, oracle, qtype, act, scoring, shared, bias_qtype):
    case = MoeCase(backend, oracle, qtype=qtype, act=act, scoring=scoring, shared=shared, bias_qtype=bias_qtype)
    backend.workspace(case.workspace_bytes)
    rc = case.execute()
    assert rc == 0, case.err.message
    res = case.result
    want = case.oracle_layer(act_q8=act == abi.ACT_DEVICE_ENCODED)
    assert np.array_equal(case.sel.reshape(case.rows, case.topk), want["selected"])     # identical routing
    assert np.array_equal(case.wts.reshape(case.rows, case.topk), want["weights"])
    got = backend.read_f32(case.rows_out, case.rows * case.hidden).reshape(case.rows, case.hidden)
    assert np.array_equal(got, case.combined) and case.rows_out.contents.is_written == 1
    same_as_cpu(got, want["combined"])
    uniq = len(np.unique(want["selected"]))
    assert res.completed == 1 and res.row_count == case.rows and res.unique_experts == uniq
    assert res.row_expert_pairs == case.rows * case.topk and res.worklists.bucket_count == uniq
    assert res.worklists.pair_count == case.rows * case.topk and res.stream_synchronizations == 1
    per_expert = sum(case.parts[n].nbytes for n in ("gate", "up", "down")) // case.experts
    assert res.active_weight_per_unique_expert_bytes == per_expert
    assert res.encoded_bytes_read == res.active_weight_base_bytes + per_expert * uniq
    assert res.kernel_launches >= 6 and res.memory.complete == 1


@pytest.mark.parametrize("qtype,streams,rows,hidden,iterations,norm_qtype", [
    ("IQ2_XXS", 4, 5, 512, 20, "BF16"), ("IQ2_XXS", 1, 3, 512, 1, "F32"), ("Q8_0", 2, 7, 256, 3, "I32"),
    ("IQ2_XXS", 4, 12, 512, 20, "BF16")])
def test_execute_rows_with_residual_streams(backend, oracle, qtype, streams, rows, hidden, iterations,
                                            norm_qtype):
    """The layer as the reference's row-batch operation runs it (src/backend/cuda/moe.c:1210-1254,
    1533-1541): ingress over the expanded rows, weighted norm, routing and experts on the
    normalised row, egress back onto the streams. The mixes come from the F32-accumulating
    projection, which like the CPU forms products and sums in double, so gates and the mixing
    matrix differ from the CPU's only by what two maths libraries' double exp differ (1e-6), the
    normalised row, the routing and the layer's combined rows are the CPU path's."""
    case = MoeCase(backend, oracle, qtype=qtype, hidden=hidden, rows=rows, streams=streams,
                   iterations=iterations, norm_qtype=norm_qtype)
    backend.workspace(case.workspace_bytes)
    assert case.execute() == 0, case.err.message
    want = case.oracle_layer(act_q8=True)
    assert np.array_equal(case.sel.reshape(rows, case.topk), want["selected"])
    assert np.array_equal(case.wts.reshape(rows, case.topk), want["weights"])
    assert np.max(np.abs(case.post - want["post"])) <= 1e-6
    assert np.max(np.abs(case.comb - want["combination"])) <= 1e-6
    same_as_cpu(case.combined, want["combined"])
    expanded = streams * hidden
    got = backend.read_f32(case.rows_out, rows * expanded).reshape(rows, expanded)
    assert case.rows_out.contents.is_written == 1
    assert np.array_equal(got.view(np.uint32) & 0xffff, np.zeros_like(got.view(np.uint32)))
    # the egress applied to the device's own combined rows is exact
    rc, replay = oracle.mhc_post(case.combined, case.x, case.post, case.comb, streams=streams, width=hidden)
    assert rc == 0 and np.array_equal(got.view(np.uint32), replay.view(np.uint32))
    scale = np.abs(want["envelope"]) + np.abs(want["combined"]).max()
    assert np.all(np.abs(got - want["envelope"]) <= 2.0 ** -6 * scale)
    # mixing projection, ingress (which decodes scale, base and norm itself) and egress on top of
    # the layer's own launches
    assert case.result.completed == 1 and case.result.kernel_launches >= 11


@pytest.mark.parametrize("streams", [0, 4])
def test_execute_rows_hash_router(backend, oracle, streams):
    """Hash-routed layers (the reference's first layers route by token id, src/graph/moe.c:539-559):
    the selection is the token's table row, the rest of the layer is unchanged."""
    case = MoeCase(backend, oracle, hidden=512, rows=6, streams=streams, iterations=4, hash_vocab=40)
    backend.workspace(case.workspace_bytes)
    assert case.execute() == 0, case.err.message
    want = case.oracle_layer(act_q8=True)
    assert np.array_equal(case.sel.reshape(6, case.topk), case.table[case.tokens])
    assert np.array_equal(case.sel.reshape(6, case.topk), want["selected"])
    assert np.array_equal(case.wts.reshape(6, case.topk), want["weights"])
    same_as_cpu(case.combined, want["combined"])
    # a token outside the table refuses before anything runs; a repeated ordinal is caught on the device
    case.tokens[2] = 40
    assert case.execute() == abi.BOUNDS
    case.tokens[2] = 1


@pytest.mark.parametrize("qtype,hidden,intermediate,experts,topk,rows,image", [
    ("IQ2_XXS", 2048, 2048, 16, 4, 20, ()),    # four rows an iteration, buckets past four pairs (two sweeps)
    ("IQ2_XXS", 4096, 3072, 4, 2, 5, ()),      # 24 lanes a row: one row an iteration
    ("Q4_K", 2048, 4096, 5, 2, 3, ()),         # 32 lanes a row: two rows an iteration
    ("IQ2_XXS", 7168, 2048, 12, 4, 6, ()),     # the benchmark layer's widths
    # gate and up rows as the sweeps' image beside canonical Q2_K down rows, which have no image:
    # the one pairing of layouts that need not agree; decode width and matrix-core width
    ("IQ2_XXS", 2048, 2048, 16, 4, 20, ("routed", "shared")),
    ("IQ2_XXS", 2048, 2048, 4, 2, 60, ("routed", "shared"))])
@pytest.mark.parametrize("shared_qtype", [None, "Q8_0"])
def test_execute_rows_with_q2k_down_experts(backend, oracle, qtype, hidden, intermediate, experts, topk, rows,
                                            image, shared_qtype):
    """The pairing of the reference's model file, IQ2_XXS gate and up experts with Q2_K down
    experts (src/backend/cuda/tensorcore.cu:563-564, 660), at decode width: the down projection
    runs the specialised sweeps over Q2_K rows, and the result is the CPU layer's bit for bit."""
    if shared_qtype:        # (a Q8_0 shared expert, the model file's: dense projections from 16 rows on)
        image = tuple(group for group in image if group != "shared")
    case = MoeCase(backend, oracle, qtype=qtype, down_qtype="Q2_K", hidden=hidden, intermediate=intermediate,
                   experts=experts, topk=topk, rows=rows, scoring=abi.SCORING_SIGMOID, sweep_image=image,
                   shared_qtype=shared_qtype)
    backend.workspace(case.workspace_bytes)
    rc = case.execute()
    assert rc == 0, case.err.message
    want = case.oracle_layer(act_q8=True)
    assert np.array_equal(case.sel.reshape(case.rows, case.topk), want["selected"])
    got = backend.read_f32(case.rows_out, case.rows * case.hidden).reshape(case.rows, case.hidden)
    same_as_cpu(got, want["combined"])
    assert case.result.completed == 1 and (case.result.tensor_core_launches > 0) == (rows == 60)


@pytest.mark.parametrize("qtype,down_qtype", [("IQ2_XXS", None), ("Q4_K", None), ("IQ2_XXS", "Q2_K"),
                                              ("Q4_K", "Q2_K"), ("IQ2_XXS", "Q4_K")])
def test_execute_rows_large_batch_takes_matrix_core_kernels(backend, oracle, qtype, down_qtype):
    """Row batches whose buckets average six pairs or more run the int8 matrix-core kernels
    (routed and shared expert); the result is the CPU layer's, bit for bit. IQ2_XXS gate and up
    rows with Q2_K down rows is the pairing the reference's tensor-core kernels serve
    (src/backend/cuda/tensorcore.cu:563-564, 660)."""
    case = MoeCase(backend, oracle, qtype=qtype, down_qtype=down_qtype, hidden=768, intermediate=512, experts=4,
                   topk=2, rows=200, scoring=abi.SCORING_SIGMOID)
    backend.workspace(case.workspace_bytes)
    rc = case.execute()
    assert rc == 0, case.err.message
    assert case.result.tensor_core_launches > 0
    want = case.oracle_layer(act_q8=True)
    assert np.array_equal(case.sel.reshape(case.rows, case.topk), want["selected"])
    got = backend.read_f32(case.rows_out, case.rows * case.hidden).reshape(case.rows, case.hidden)
    same_as_cpu(got, want["combined"])
    assert case.result.row_expert_pairs == 400 and case.result.completed == 1


def sealed_policy(case, minimum):
    """An execution batch and a worklist policy as the runtime seals them for a row batch
    (src/runtime/moe.c:101-193), the policy with the given tensor-core minimum."""
    batch, policy = abi.ExecutionBatch(), abi.WorklistPolicy()
    batch.schema_version, batch.row_count = 1, case.rows
    batch.provenance, batch.phase = case.batch.provenance, case.batch.phase
    policy.schema_version = 1
    policy.supported_width_mask = ((1 << 62) - 1) << 1
    policy.narrow_kernel_family = abi.FAMILY_GFX950
    policy.tensor_core_minimum = minimum
    policy.tensor_core_kernel_family = abi.FAMILY_GFX950_MATRIX_CORE if minimum else b""
    return batch, policy


@pytest.mark.parametrize("minimum,matrix", [(None, True), (0, False), (8, True), (40, False)])
def test_worklist_policy_decides_the_matrix_core_regime(backend, oracle, minimum, matrix):
    """src/backend/cuda/moe.c:1341-1361: the tensor-core kernels run only when the sealed policy
    names a minimum and the batch has that many rows. 36 rows over four experts would take the
    matrix cores by this backend's own threshold: a policy with minimum 0 keeps them off, one with
    a minimum above the batch does too, and the published facts say what ran. The rows are the
    same bits either way."""
    case = MoeCase(backend, oracle, hidden=512, intermediate=256, experts=4, topk=2, rows=36,
                   scoring=abi.SCORING_SIGMOID)
    backend.workspace(case.workspace_bytes)
    if minimum is not None:
        batch, policy = sealed_policy(case, minimum)
        case.job.execution_batch, case.job.worklist_policy = C.pointer(batch), C.pointer(policy)
    assert case.execute() == 0, case.err.message
    res = case.result
    pairs = case.rows * case.topk
    assert (res.tensor_core_launches > 0) == matrix
    assert res.worklists.tensor_core_eligible_pairs == (pairs if matrix else 0)
    assert res.worklists.tensor_core_executed_pairs == (pairs if matrix else 0)
    assert res.worklists.narrow_pairs == (0 if matrix else pairs)
    got = backend.read_f32(case.rows_out, case.rows * case.hidden).reshape(case.rows, case.hidden)
    same_as_cpu(got, case.oracle_layer(act_q8=True)["combined"])


def test_shared_sessions_run_row_batches_against_one_arena(backend, oracle):
    """Sessions that share one set of resident weights (yvex_backend_open_shared_cuda,
    include/yvex/internal/backend.h:254-255; the runtime opens one per session and attaches the
    model-owned arena, src/runtime/residency.c:1463-1469): two children of one owning backend
    attach its arena without another upload and issue row batches in turn, each on its own
    stream, workspace and launch graphs. Their rows are bit for bit the owner's own."""
    from yvex_amd.host import Backend
    owner_case = MoeCase(backend, oracle, rows=7, scoring=abi.SCORING_SIGMOID)
    backend.workspace(owner_case.workspace_bytes)
    assert owner_case.execute() == 0, owner_case.err.message
    want = backend.read_f32(owner_case.rows_out, 7 * owner_case.hidden).reshape(7, owner_case.hidden).copy()
    same_as_cpu(want, owner_case.oracle_layer(act_q8=True)["combined"])
    children = [Backend(shared_with=backend), Backend(shared_with=backend)]
    try:
        assert all(c.ok for c in children)
        # a shared session is not an owner, and the arena must be the one the owner attached
        grandchild = Backend(shared_with=children[0])
        assert grandchild.open_rc == abi.INVALID_ARG and not grandchild.handle.value
        assert children[0].attach_shared_arena(owner_case.arena_tensor, owner_case.host, owner_case.arena_bytes,
                                               generation=2) == abi.STATE
        cases = [MoeCase(children[0], oracle, rows=7, scoring=abi.SCORING_SIGMOID, arena_from=owner_case),
                 MoeCase(children[1], oracle, rows=5, scoring=abi.SCORING_SIGMOID, arena_from=owner_case)]
        for child, case in zip(children, cases):
            child.workspace(case.workspace_bytes)
            stats = abi.MemoryStats()
            assert child.lib.yvex_rocm_backend_get_memory_stats(child.handle, C.byref(stats), C.byref(child.err)) == 0
            assert stats.h2d_bytes < owner_case.arena_bytes        # rows only: the arena was not uploaded again
        for turn in range(4):       # first sight, recording, two replays, interleaved
            for case in cases:
                assert case.execute() == 0, case.err.message
                got = case.b.read_f32(case.rows_out, case.rows * case.hidden).reshape(case.rows, case.hidden)
                assert np.array_equal(got.view(np.uint32), want[:case.rows].view(np.uint32)), turn
        assert cases[0].result.graph_replays == 1 and cases[1].result.graph_replays == 1
        # the owner keeps working beside them
        assert owner_case.execute() == 0, owner_case.err.message
        again = backend.read_f32(owner_case.rows_out, 7 * owner_case.hidden).reshape(7, owner_case.hidden)
        assert np.array_equal(again.view(np.uint32), want.view(np.uint32))
    finally:
        for child in children:
            if child.handle.value:
                assert child.close() == 0, child.err.message


def test_execute_rows_refusals(backend, oracle):
    b = backend
    case = MoeCase(b, oracle)
    # workspace not preflighted
    assert case.execute() == abi.NOMEM and case.rows_out.contents.is_written == 0
    b.workspace(case.workspace_bytes)
    # width outside the sealed mask: UNSUPPORTED before anything is touched
    policy = abi.WorklistPolicy()
    policy.schema_version, policy.supported_width_mask = 1, (1 << 1) | (1 << 4)
    policy.narrow_kernel_family = abi.FAMILY_GFX950
    case.job.worklist_policy = C.pointer(policy)
    batch = abi.ExecutionBatch()
    batch.schema_version, batch.row_count = 1, case.rows
    batch.provenance, batch.phase = case.batch.provenance, case.batch.phase
    case.job.execution_batch = C.pointer(batch)
    sentinel = np.full(case.rows * case.hidden, 7.0, np.float32)
    b.lib.yvex_rocm_backend_tensor_write(b.handle, case.rows_out, sentinel.ctypes.data, sentinel.nbytes, None)
    assert case.execute() == abi.UNSUPPORTED
    assert np.array_equal(b.read_f32(case.rows_out, sentinel.size), sentinel)
    policy.supported_width_mask |= 1 << case.rows
    assert case.execute() == 0, case.err.message
    # src/backend/cuda/moe.c:1845-1852: the batch must describe the rows it comes with
    for field, wrong in (("row_count", case.rows + 1), ("provenance", abi.BATCH_PREFILL), ("phase", 1),
                         ("schema_version", 2)):
        keep = getattr(batch, field)
        setattr(batch, field, wrong)
        assert case.execute() == abi.INVALID_ARG, field
        setattr(batch, field, keep)
    # src/graph/worklist.c:252-272: width 1 admitted, width 0 and bit 63 not, families consistent
    good = policy.supported_width_mask
    for mask in (good & ~2, good | 1, good | (1 << 63)):
        policy.supported_width_mask = mask
        assert case.execute() == abi.INVALID_ARG, hex(mask)
    policy.supported_width_mask = good
    policy.narrow_kernel_family = b""
    assert case.execute() == abi.INVALID_ARG
    policy.narrow_kernel_family = abi.FAMILY_GFX950
    policy.tensor_core_minimum = 4                      # a minimum needs a family of its own
    assert case.execute() == abi.INVALID_ARG
    policy.tensor_core_kernel_family = abi.FAMILY_GFX950
    assert case.execute() == abi.INVALID_ARG            # ... that differs from the narrow one
    policy.tensor_core_kernel_family = b"sm121-int8-tensorcore-expert"
    assert case.execute() == abi.UNSUPPORTED            # ... and be this backend's (src/backend/cuda/moe.c:937-951)
    policy.tensor_core_kernel_family = abi.FAMILY_GFX950_MATRIX_CORE
    assert case.execute() == 0, case.err.message
    policy.tensor_core_minimum = 3                      # ... and must be an admitted width
    assert case.execute() == abi.INVALID_ARG
    policy.tensor_core_minimum, policy.tensor_core_kernel_family = 0, b""
    # a profile identity names a compiled batch: without batch and policy it is refused
    case.job.execution_batch, case.job.worklist_policy = None, None
    case.batch.execution_profile_identity = b"0" * 64
    assert case.execute() == abi.INVALID_ARG
    case.batch.execution_profile_identity = None
    case.job.execution_batch, case.job.worklist_policy = C.pointer(batch), C.pointer(policy)
    # execution batch and worklist policy must come together
    case.job.execution_batch = None
    assert case.execute() == abi.INVALID_ARG
    case.job.worklist_policy = None
    # mixed gate/up activation classes
    case.job.weights[abi.W_ROUTED_UP].activation = abi.ACT_DEVICE_F32
    assert case.execute() == abi.FORMAT
    case.job.weights[abi.W_ROUTED_UP].activation = abi.ACT_DEVICE_ENCODED
    # gate/up kernel families disagree
    case.job.weights[abi.W_ROUTED_UP].kernel_family = abi.FAMILY_PORTABLE_EXPERT_ROW
    assert case.execute() == abi.FORMAT
    # unknown kernel family
    for slot in (abi.W_ROUTED_GATE, abi.W_ROUTED_UP):
        case.job.weights[slot].kernel_family = b"sm121-int8-tensorcore-expert"
    assert case.execute() == abi.UNSUPPORTED
    for slot in (abi.W_ROUTED_GATE, abi.W_ROUTED_UP):
        case.job.weights[slot].kernel_family = abi.FAMILY_GFX950
    # layouts: gate/up must agree and down must be derived exactly when they are (FORMAT); a derived
    # image is refused by the row-batch path (UNSUPPORTED), src/backend/cuda/moe.c:933-958
    case.job.weights[abi.W_ROUTED_UP].layout = abi.LAYOUT_CANONICAL_ROW
    assert case.execute() == abi.FORMAT
    case.job.weights[abi.W_ROUTED_UP].layout = abi.LAYOUT_EXPERT_MAJOR
    case.job.weights[abi.W_ROUTED_DOWN].layout = abi.LAYOUT_DERIVED
    assert case.execute() == abi.FORMAT
    for slot in (abi.W_ROUTED_GATE, abi.W_ROUTED_UP):
        case.job.weights[slot].layout = abi.LAYOUT_DERIVED
    # ... except the expert sweeps' own image (IQ2_XXS, encoded activations, the sweep family on
    # all three views), whose storage is 72 bytes a superblock: these views still hold canonical bytes
    assert case.execute() == abi.FORMAT
    assert b"image" in case.err.message
    for slot in (abi.W_ROUTED_GATE, abi.W_ROUTED_UP, abi.W_ROUTED_DOWN):
        case.job.weights[slot].kernel_family = abi.FAMILY_PORTABLE_EXPERT_ROW
    assert case.execute() == abi.UNSUPPORTED
    for slot in (abi.W_ROUTED_GATE, abi.W_ROUTED_UP, abi.W_ROUTED_DOWN):
        case.job.weights[slot].layout = abi.LAYOUT_EXPERT_MAJOR
        case.job.weights[slot].kernel_family = abi.FAMILY_GFX950
    # the layout entries of the table answer like the exported functions
    decision = abi.ExecutionDecision()
    decision.expert_count, decision.canonical_qtype = 4, 16
    decision.canonical_row_width, decision.canonical_row_count, decision.encoded_bytes = 512, 8, 8 * 2 * 66
    decision.consumer, decision.layout, decision.derived_asset_required = (
        abi.CONSUMER_ROUTED_DOWN, abi.LAYOUT_DERIVED, 1)
    storage = abi.ULL()
    assert case.ops.derived_layout_plan(C.byref(decision), C.byref(storage), C.byref(case.err)) == 0
    assert storage.value == 64 + 16 * 64
    # mixing rows that disagree with the stream count; expanded rows without mixing rows; hash router
    case.plan.mhc_mixing_rows = 24
    assert case.execute() == abi.BOUNDS
    case.plan.mhc_mixing_rows = 0
    case.plan.expanded_width = 2 * case.hidden
    assert case.execute() in (abi.UNSUPPORTED, abi.INVALID_ARG)
    case.plan.expanded_width = case.hidden
    case.plan.router_class = abi.ROUTER_HASH          # no token ids, no table
    assert case.execute() == abi.BOUNDS
    case.plan.router_class = 7
    assert case.execute() == abi.UNSUPPORTED
    case.plan.router_class = abi.ROUTER_LEARNED
    # cancellation is polled before launch
    case.job.cancel_requested = abi.CANCEL_FN(lambda ctx: 1)
    assert case.execute() == abi.CANCELLED
    case.job.cancel_requested = abi.CANCEL_FN(0)
    # a weight view outside the resident arena
    saved = case.job.weights[abi.W_ROUTED_DOWN].encoded
    case.job.weights[abi.W_ROUTED_DOWN].encoded = saved + (1 << 30)
    assert case.execute() == abi.FORMAT
    case.job.weights[abi.W_ROUTED_DOWN].encoded = saved
    assert case.execute() == 0, case.err.message


def test_execute_rows_deferred_completion(backend, oracle):
    case = MoeCase(backend, oracle, rows=3)
    backend.workspace(case.workspace_bytes)
    completion = abi.DeviceCompletion(1, None)
    case.job.device_completion = C.pointer(completion)
    assert case.execute() == 0, case.err.message
    assert case.result.device_completion_pending == 1 and case.result.completed == 0
    done, err = abi.RowBatchResult(), abi.Error()
    assert case.ops.complete_rows(backend.handle, 0, C.byref(done), C.byref(err)) == 0
    assert done.completed == 1 and done.stream_synchronizations == 1
    got = backend.read_f32(case.rows_out, case.rows * case.hidden).reshape(case.rows, case.hidden)
    want = case.oracle_layer(act_q8=True)["combined"]
    same_as_cpu(got, want)


def test_deferred_batches_keep_what_an_earlier_one_raised(backend, oracle):
    """Two batches behind one barrier (src/runtime/moe.c:1567-1576 completes a phase's layers with
    one call): the first is fed a non-finite row and raises the kernels' status, the second is
    clean; the barrier still reports the failure, and the phase after it starts clean."""
    case = MoeCase(backend, oracle, rows=3)
    backend.workspace(case.workspace_bytes)
    completion = abi.DeviceCompletion(1, None)
    case.job.device_completion = C.pointer(completion)
    clean = case.rows_in
    bad = case.x.copy()
    bad[1, 7] = np.inf
    case.batch.device_rows = backend.f32(bad)
    assert case.execute() == 0, case.err.message
    case.batch.device_rows = clean
    assert case.execute() == 0, case.err.message
    done, err = abi.RowBatchResult(), abi.Error()
    assert case.ops.complete_rows(backend.handle, 0, C.byref(done), C.byref(err)) == abi.FORMAT
    assert case.execute() == 0, case.err.message
    assert case.ops.complete_rows(backend.handle, 0, C.byref(done), C.byref(err)) == 0, err.message
    assert done.completed == 1


def test_deferred_hash_routed_batches_keep_their_own_token_ids(backend, oracle):
    """Two hash-routed batches behind one barrier, the caller's token buffer rewritten as soon as
    each call returns: the ids travel through the backend's pinned memory, so each batch routes by
    the ids it was given although neither call waited for the stream."""
    case = MoeCase(backend, oracle, hidden=512, rows=6, iterations=4, hash_vocab=40)
    backend.workspace(case.workspace_bytes)
    completion = abi.DeviceCompletion(1, None)
    case.job.device_completion = C.pointer(completion)
    first = case.tokens.copy()
    second = ((first + 7) % 40).astype(np.uint32)
    outputs = [case.rows_out, backend.empty_f32(case.rows * case.hidden)]
    for ids, out in zip((first, second), outputs):
        case.tokens[:] = ids
        case.batch.device_outputs = out
        assert case.execute() == 0, case.err.message
        assert case.result.device_completion_pending == 1
        case.tokens[:] = 39 - ids          # the caller reuses its buffer at once
    done, err = abi.RowBatchResult(), abi.Error()
    assert case.ops.complete_rows(backend.handle, 0, C.byref(done), C.byref(err)) == 0, err.message
    for ids, out in zip((first, second), outputs):
        case.tokens[:] = ids
        got = backend.read_f32(out, case.rows * case.hidden).reshape(case.rows, case.hidden)
        same_as_cpu(got, case.oracle_layer(act_q8=True)["combined"])


@pytest.mark.parametrize("hidden,intermediate,rows", [(3072, 2048, 5), (2048, 4096, 6), (4096, 3072, 3)])
def test_sweep_image_at_other_widths(backend, oracle, hidden, intermediate, rows):
    """Image sweeps at widths where a wavefront holds one row and lanes are left over (3072: 24
    of 64 lanes hold columns), two rows (4096) or four (2048), in both projections: the CPU
    layer's bits, and the canonical views' bits."""
    results = []
    for image in ((), ("routed", "shared")):
        case = MoeCase(backend, oracle, hidden=hidden, intermediate=intermediate, experts=8, rows=rows,
                       sweep_image=image)
        backend.workspace(case.workspace_bytes)
        assert case.execute() == 0, case.err.message
        results.append(case.combined.copy())
        if image:
            same_as_cpu(case.combined, case.oracle_layer(act_q8=True)["combined"])
        backend.release_all()
    assert np.array_equal(results[0].view(np.uint32), results[1].view(np.uint32))


@pytest.mark.parametrize("imaged,rows,experts", [
    (("routed", "shared"), 5, 8), (("routed",), 7, 8), (("shared",), 6, 8), (("routed", "shared"), 40, 4)])
def test_execute_rows_runs_the_sweep_image(backend, oracle, imaged, rows, experts):
    """Experts resident as the decode sweeps' image (DERIVED_BACKEND views of the gfx950 sweep
    family, built by derived_layout_build) give bit for bit what canonical views give on the
    sweeps, and on the matrix-core kernels when the batch is wide enough for them (the last case).
    No counterpart in the reference, whose row-batch path refuses derived views
    (src/backend/cuda/moe.c:939-958)."""
    results = []
    for image in ((), imaged):
        case = MoeCase(backend, oracle, hidden=2048, intermediate=2048, experts=experts, rows=rows,
                       sweep_image=image)
        backend.workspace(case.workspace_bytes)
        assert case.execute() == 0, case.err.message
        results.append((case.combined.copy(), case.sel.copy(), case.wts.copy()))
        backend.release_all()
    assert np.array_equal(results[0][1], results[1][1]) and np.array_equal(results[0][2], results[1][2])
    assert np.array_equal(results[0][0].view(np.uint32), results[1][0].view(np.uint32))


def test_sweep_image_built_on_the_device_equals_the_host_builder(backend, oracle):
    """yvex_rocm_moe_sweep_image_build_resident against derived_layout_build on the same tensor,
    and its refusals."""
    case = MoeCase(backend, oracle, hidden=2048, intermediate=2048, experts=4, rows=3, sweep_image=("routed",))
    lib, decision = backend.lib, case.decisions["down"]
    want = case.parts["down.image"]
    base = case.arena_tensor.contents.data
    rc, target = backend.tensor(want.nbytes, abi.DTYPE_I8, b"image")
    assert rc == 0
    err = abi.Error()
    build = lib.yvex_rocm_moe_sweep_image_build_resident
    canonical = base + case.offsets["down"]
    assert build(backend.handle, C.byref(decision), canonical, target.contents.data, want.nbytes,
                 C.byref(err)) == 0, err.message
    target.contents.is_written = 1          # written through its address, not through tensor_write
    got = backend.read_f32(target, want.nbytes // 4).view(np.uint8)
    assert np.array_equal(got, want)
    # wrong size, overlapping ranges, a decision for the reference's own image
    assert build(backend.handle, C.byref(decision), canonical, target.contents.data, want.nbytes - 72,
                 C.byref(err)) == abi.INVALID_ARG
    assert build(backend.handle, C.byref(decision), canonical, canonical + 64, want.nbytes,
                 C.byref(err)) == abi.INVALID_ARG
    decision.kernel_family = b""
    assert build(backend.handle, C.byref(decision), canonical, target.contents.data, want.nbytes,
                 C.byref(err)) == abi.UNSUPPORTED
    backend.release_all()


def test_sweep_image_views_are_checked(backend, oracle):
    case = MoeCase(backend, oracle, hidden=2048, intermediate=2048, experts=4, rows=3,
                   sweep_image=("routed", "shared"))
    backend.workspace(case.workspace_bytes)
    assert case.execute() == 0, case.err.message
    routed = (abi.W_ROUTED_GATE, abi.W_ROUTED_UP, abi.W_ROUTED_DOWN)
    # F32 activations, another qtype, another family: only canonical rows serve those
    for slot in routed:
        case.job.weights[slot].activation = abi.ACT_DEVICE_F32
    assert case.execute() == abi.UNSUPPORTED
    for slot in routed:
        case.job.weights[slot].activation = abi.ACT_DEVICE_ENCODED
        case.job.weights[slot].kernel_family = abi.FAMILY_PORTABLE_EXPERT_ROW
    assert case.execute() == abi.UNSUPPORTED
    for slot in routed:
        case.job.weights[slot].kernel_family = abi.FAMILY_GFX950
    case.job.weights[abi.W_ROUTED_DOWN].qtype = 12
    assert case.execute() == abi.UNSUPPORTED
    case.job.weights[abi.W_ROUTED_DOWN].qtype = 16
    # storage that is not 72 bytes a superblock, an image outside the arena
    case.job.weights[abi.W_SHARED_UP].storage_bytes -= 72
    assert case.execute() == abi.FORMAT
    case.job.weights[abi.W_SHARED_UP].storage_bytes += 72
    keep = case.job.weights[abi.W_ROUTED_GATE].encoded
    outside = np.zeros(case.job.weights[abi.W_ROUTED_GATE].storage_bytes, np.uint8)
    case.job.weights[abi.W_ROUTED_GATE].encoded = outside.ctypes.data
    assert case.execute() == abi.FORMAT
    case.job.weights[abi.W_ROUTED_GATE].encoded = keep
    assert case.execute() == 0, case.err.message
    backend.release_all()


@pytest.mark.parametrize("kwargs", [
    dict(rows=5),                                                                # decode sweeps
    dict(rows=3, qtype="Q4_K", shared=False, scoring=abi.SCORING_SIGMOID),       # generic sweeps
    dict(rows=4, streams=4, hidden=512, iterations=5),                           # residual streams
    dict(rows=3, hash_vocab=50),                                                 # hash router
    dict(rows=200, hidden=768, intermediate=512, experts=4, scoring=abi.SCORING_SIGMOID),  # matrix cores
    # the model file's formats: Q2_K down sweeps, the Q8_0 shared expert as dense projections
    dict(rows=7, hidden=2048, intermediate=2048, experts=8, down_qtype="Q2_K", shared_qtype="Q8_0"),
], ids=["sweep", "generic", "streams", "hash", "matrix", "model-file-formats"])
def test_execute_rows_graph_replays_equal_eager(backend, oracle, kwargs):
    """src/backend/cuda/moe.c:1650-1681: a job that does not ask for eager execution runs as a
    launch graph keyed on its topology. Here the key's first use runs eagerly, the second is
    captured, later ones are replayed; every one of them must give the eager bits, also for rows
    written between replays and with other eager work on the stream in between."""
    b = backend
    case = MoeCase(b, oracle, **kwargs)
    b.workspace(case.workspace_bytes)
    width = case.x.shape[1]
    rng = np.random.default_rng(7)

    def run(rows_now, eager):
        rc = b.lib.yvex_rocm_backend_tensor_write(b.handle, case.rows_in, rows_now.ctypes.data, rows_now.nbytes,
                                             C.byref(b.err))
        assert rc == 0, b.err.message
        case.job.eager_execution = int(eager)
        assert case.execute() == 0, case.err.message
        facts = (case.result.graph_launches, case.result.graph_captures, case.result.graph_replays)
        return (b.read_f32(case.rows_out, case.rows * width).copy(), case.combined.copy(),
                case.sel.copy(), case.wts.copy(), facts, case.result.kernel_launches)

    batches = [case.x] + [np.ascontiguousarray(case.x * s + rng.standard_normal(case.x.shape) * 0.05,
                                               np.float32) for s in (0.5, -1.0, 2.0, 1.0, 0.25)]
    if case.streams:      # the CPU path feeds bf16 values; keep the later batches of that kind too
        batches = [((x.view(np.uint32) + 0x8000) & 0xffff0000).view(np.float32) for x in batches]
    want = [run(x, eager=True) for x in batches]
    assert all(w[4] == (0, 0, 0) for w in want)
    expected_facts = [(0, 0, 0), (1, 1, 0)] + [(1, 0, 1)] * (len(batches) - 2)
    for step, x in enumerate(batches):
        got = run(x, eager=False)
        assert got[4] == expected_facts[step], (step, got[4])
        assert got[5] == want[step][5]
        for name, g, w in zip(("rows", "combined", "selected", "weights"), got[:4], want[step][:4]):
            assert np.array_equal(g.view(np.uint8), w.view(np.uint8)), (step, name)
        # other work between replays: an eager batch on the same stream
        run(batches[(step + 1) % len(batches)], eager=True)


def test_execute_rows_graph_key_follows_addresses(backend, oracle):
    """Rows handed over in another tensor are another key: the graph recorded for the first
    tensor must not be replayed against it."""
    b = backend
    case = MoeCase(b, oracle, rows=5)
    b.workspace(case.workspace_bytes)
    for _ in range(3):
        assert case.execute() == 0, case.err.message
    assert case.result.graph_replays == 1
    first = b.read_f32(case.rows_out, case.rows * case.hidden).copy()
    other_in, other_out = b.f32(case.x * 0.5), b.empty_f32(case.rows * case.hidden)
    case.batch.device_rows, case.batch.device_outputs = other_in, other_out
    assert case.execute() == 0, case.err.message
    assert case.result.graph_launches == 0            # first sight of the new key
    assert case.execute() == 0 and case.result.graph_captures == 1
    got = b.read_f32(other_out, case.rows * case.hidden)
    case.job.eager_execution = 1
    assert case.execute() == 0 and case.result.graph_launches == 0
    assert np.array_equal(got, b.read_f32(other_out, case.rows * case.hidden))
    assert np.array_equal(first, b.read_f32(case.rows_out, case.rows * case.hidden))
    assert not np.array_equal(first, got)


# ---- token-local operation: src/backend/cuda/moe.c:516-842 --------------------------------------

class TokenLocal:
    """begin / add_expert / finish / close over one row of a MoeCase with residual streams."""

    def __init__(self, case, row=0, device=False, evidence=0):
        self.case, self.b = case, case.b
        hidden, streams = case.hidden, case.streams
        self.row = np.ascontiguousarray(case.x[row])
        self.combined, self.routed = np.zeros(hidden, np.float32), np.zeros(hidden, np.float32)
        self.shared = np.zeros(hidden, np.float32)
        self.post, self.comb = np.zeros(streams, np.float32), np.zeros(streams * streams, np.float32)
        r = self.result = abi.LayerResult()
        r.combined_output, r.combined_capacity = self.combined.ctypes.data, hidden
        r.routed_output, r.routed_capacity = self.routed.ctypes.data, hidden
        r.shared_output, r.shared_capacity = self.shared.ctypes.data, hidden
        r.post, r.post_capacity = self.post.ctypes.data, streams
        r.combination, r.combination_capacity = self.comb.ctypes.data, streams * streams
        self.job = case.job
        self.job.expanded_input = self.row.ctypes.data
        self.job.evidence_level = evidence
        self.device_in = self.device_out = None
        if device:
            self.device_in, self.device_out = self.b.f32(self.row), self.b.empty_f32(self.row.size)
            self.job.device_input = C.cast(self.device_in, C.c_void_p)
            self.job.device_output = C.cast(self.device_out, C.c_void_p)
        self.handle, self.err = C.c_void_p(), abi.Error()

    def begin(self):
        return self.b.lib.yvex_rocm_backend_moe_begin(C.byref(self.handle), self.b.handle, C.byref(self.job),
                                                 C.byref(self.result), C.byref(self.err))

    def expert_views(self, expert=None, outside=False):
        """Weight views of one routed expert (a slice of the expert-major matrices) or of the
        shared expert; outside=True points them at a private host copy, away from the arena."""
        case, keep = self.case, []
        names = ("gate", "up", "down") if expert is not None else ("sgate", "sup", "sdown")
        slots = (abi.W_ROUTED_GATE, abi.W_ROUTED_UP, abi.W_ROUTED_DOWN) if expert is not None else \
            (abi.W_SHARED_GATE, abi.W_SHARED_UP, abi.W_SHARED_DOWN)
        views = []
        for name, slot, rows in zip(names, slots, (case.intermediate, case.intermediate, case.hidden)):
            whole = case.job.weights[slot]
            v = abi.WeightView()
            C.memmove(C.byref(v), C.byref(whole), C.sizeof(v))
            nbytes = whole.row_bytes * rows
            start = (expert or 0) * nbytes
            v.row_count, v.encoded_bytes, v.storage_bytes = rows, nbytes, nbytes
            if outside:
                copy = np.ascontiguousarray(case.parts[name][start:start + nbytes])
                keep.append(copy)
                v.encoded = copy.ctypes.data
            else:
                v.encoded = case.host + case.offsets[name] + start
            views.append(v)
        return views, keep

    def add(self, views, weight, shared):
        return self.b.lib.yvex_rocm_backend_moe_add_expert(self.handle, C.byref(views[0]), C.byref(views[1]),
                                                      C.byref(views[2]), C.c_float(weight), int(shared),
                                                      C.byref(self.err))

    def finish(self):
        return self.b.lib.yvex_rocm_backend_moe_finish(self.handle, C.byref(self.result), C.byref(self.err))

    def close(self):
        return self.b.lib.yvex_rocm_backend_moe_close(C.byref(self.handle), C.byref(self.err))


def token_oracle(case, row):
    """CPU path for one row: ingress, routing, experts on F32 activations in rank order, shared
    expert, bf16(routed + shared), egress (src/runtime/moe.c:596-645)."""
    o, p = case.oracle, case.parts
    norm = o.decode_rows(case.norm_qt, p["norm"], case.hidden)[0]
    rc, x, post, comb = o.moe_ffn_prepare(
        o.F32, p["function"], case.x[row], p["scale"].view(np.float32), p["base"].view(np.float32), norm,
        streams=case.streams, width=case.hidden, iterations=case.iterations, rms_epsilon=1e-6,
        mhc_epsilon=1e-6, post_multiplier=2.0)
    assert rc == 0
    logits = o.matvec(o.F32, p["router"], case.experts, case.hidden, x)
    want = o.moe_layer(hidden=case.hidden, intermediate=case.intermediate, experts=case.experts,
                       topk=case.topk, qtypes=case.qtypes, routed=(p["gate"], p["up"], p["down"]),
                       shared=(p["sgate"], p["sup"], p["sdown"]), inputs=x, logits=logits,
                       bias=case.bias_values, scoring=case.scoring, normalize=True, scaling=1.5,
                       act_q8=False, threads=1)
    rc, want["envelope"] = o.mhc_post(want["combined"], case.x[row], post, comb, streams=case.streams,
                                      width=case.hidden)
    assert rc == 0
    want.update(logits=logits.ravel(), post=post.ravel(), combination=comb.ravel())
    return want


def to_bf16(values):
    bits = np.ascontiguousarray(values, np.float32).view(np.uint32)
    return ((bits + 0x7fff + ((bits >> 16) & 1)) & 0xffff0000).view(np.float32)


def rows_close(got, ref, steps=2):
    same_as_cpu(got, ref)
    return True


@pytest.mark.parametrize("qtype,outside", [("IQ2_XXS", False), ("Q8_0", True)])
def test_token_local_host_publication(backend, oracle, qtype, outside):
    """The caller's loop of src/runtime/moe.c:647-720: begin publishes logits, scores and the
    routing; each selected expert is added with its route weight, then the shared expert; finish
    publishes routed, shared, combined, post and combination. With outside=True the expert views
    point at host memory outside the arena and travel through the staging range."""
    case = MoeCase(backend, oracle, qtype=qtype, hidden=512, rows=2, streams=4, iterations=20,
                   act=abi.ACT_DEVICE_F32)
    t = TokenLocal(case, row=1)
    assert t.begin() == 0, t.err.message
    want = token_oracle(case, 1)
    router = t.result.router
    assert router.selected_count == case.topk
    assert list(router.selected_experts)[:case.topk] == list(want["selected"][0])
    weights = np.array(list(router.selected_weights)[:case.topk], np.float32)
    assert np.array_equal(weights, want["weights"][0])
    logits = np.array(list(router.router_logits)[:case.experts], np.float32)
    assert np.array_equal(logits, want["logits"])
    rc, _, _, scores = oracle.moe_route(logits, None, case.topk, case.scoring, True, 1.0)
    assert np.allclose(np.array(list(router.router_scores)[:case.experts], np.float32), scores, rtol=1e-6)
    keep = []
    for rank in range(case.topk):
        views, held = t.expert_views(int(router.selected_experts[rank]), outside=outside)
        keep.append(held)
        assert t.add(views, float(weights[rank]), False) == 0, t.err.message
    views, held = t.expert_views(None, outside=outside)
    assert t.add(views, 0.0, True) == 0, t.err.message
    assert t.finish() == 0, t.err.message
    assert np.max(np.abs(t.post - want["post"])) <= 1e-6
    assert np.max(np.abs(t.comb - want["combination"])) <= 1e-6
    assert rows_close(t.routed, want["routed"][0], 4) and rows_close(t.shared, want["shared"][0])
    assert rows_close(t.combined, want["combined"][0], 4)
    assert np.array_equal(t.combined, to_bf16(t.routed + t.shared))      # the combine itself is exact
    r = t.result
    assert r.expert_subviews_accessed == 3 * case.topk and r.kernel_launches >= 12
    assert (r.upload_count > 0) == outside and r.stream_synchronizations == 2
    # a finished execution takes no more experts and does not finish twice
    assert t.add(views, 0.0, True) == abi.INVALID_ARG and t.finish() == abi.INVALID_ARG
    assert t.close() == 0 and not t.handle.value and t.close() == 0


@pytest.mark.parametrize("workspace", [False, True])
def test_token_local_stages_mixed_qtypes(backend, oracle, workspace):
    """The reference's own mix of an IQ2_XXS gate/up with a Q2_K down (src/runtime/moe.c:647-720
    with views outside the arena, staged as src/backend/cuda/moe.c:205-245 does): the down matrix
    of an expert is larger than its gate, and every projection has a staging range of its own
    size. With a workspace attached the execution's block comes from it instead of an allocation."""
    case = MoeCase(backend, oracle, qtype="IQ2_XXS", down_qtype="Q2_K", hidden=512, rows=2, streams=4,
                   iterations=20, act=abi.ACT_DEVICE_F32)
    gate, down = case.job.weights[abi.W_ROUTED_GATE], case.job.weights[abi.W_ROUTED_DOWN]
    assert down.encoded_bytes > gate.encoded_bytes
    if workspace:
        backend.workspace(8 << 20)
    t = TokenLocal(case, row=0)
    assert t.begin() == 0, t.err.message
    want = token_oracle(case, 0)
    router, keep = t.result.router, []
    weights = np.array(list(router.selected_weights)[:case.topk], np.float32)
    for rank in range(case.topk):
        views, held = t.expert_views(int(router.selected_experts[rank]), outside=True)
        keep.append(held)
        assert t.add(views, float(weights[rank]), False) == 0, t.err.message
    views, held = t.expert_views(None, outside=True)
    assert t.add(views, 0.0, True) == 0, t.err.message
    assert t.finish() == 0, t.err.message
    assert rows_close(t.routed, want["routed"][0], 4) and rows_close(t.shared, want["shared"][0])
    assert rows_close(t.combined, want["combined"][0], 4)
    assert t.result.upload_count == 3 * (case.topk + 1)
    # a view larger than the range planned for its projection is refused, not spilled into the next
    big = abi.WeightView()
    C.memmove(C.byref(big), C.byref(views[0]), C.sizeof(big))
    assert t.close() == 0
    t2 = TokenLocal(case, row=1)
    assert t2.begin() == 0, t2.err.message
    wide = np.zeros(case.job.weights[abi.W_SHARED_GATE].encoded_bytes * 2, np.uint8)
    big.encoded, big.row_count = wide.ctypes.data, views[0].row_count * 2
    big.encoded_bytes = big.storage_bytes = wide.nbytes
    up2 = abi.WeightView()
    C.memmove(C.byref(up2), C.byref(big), C.sizeof(big))
    down2 = abi.WeightView()
    C.memmove(C.byref(down2), C.byref(views[2]), C.sizeof(down2))
    assert t2.add([big, up2, down2], 0.0, True) in (abi.BOUNDS, abi.INVALID_ARG)
    assert t2.close() == 0


def test_token_local_device_output_runs_selected_experts(backend, oracle):
    """With a device output, evidence below FULL and resident routed matrices, begin runs the
    selected experts on the device (moe.c:584-672); the caller adds the shared expert only and
    finish writes the egress into the device output."""
    case = MoeCase(backend, oracle, qtype="IQ2_XXS", hidden=512, rows=3, streams=4, iterations=20,
                   act=abi.ACT_DEVICE_F32)
    for slot, name in ((abi.W_ROUTED_GATE, "gate"), (abi.W_ROUTED_UP, "up"), (abi.W_ROUTED_DOWN, "down")):
        case.job.weights[slot].device_address = case.arena_tensor.contents.data + case.offsets[name]
    t = TokenLocal(case, row=2, device=True)
    assert t.begin() == 0, t.err.message
    views, _ = t.expert_views(None)
    assert t.add(views, 0.0, True) == 0, t.err.message
    assert t.finish() == 0, t.err.message
    want = token_oracle(case, 2)
    router = t.result.router
    assert list(router.selected_experts)[:case.topk] == list(want["selected"][0])
    got = backend.read_f32(t.device_out, case.streams * case.hidden)
    assert t.device_out.contents.is_written == 1
    scale = np.abs(want["envelope"][0]) + np.abs(want["combined"]).max()
    assert np.all(np.abs(got - want["envelope"][0]) <= 2.0 ** -6 * scale)
    assert np.array_equal(got.view(np.uint32) & 0xffff, np.zeros(got.size, np.uint32))
    assert not t.combined.any()            # host copies are evidence, not published on this path
    assert t.result.expert_subviews_accessed == 3 * case.topk and t.result.device_to_device_bytes > 0
    assert t.close() == 0
    # without device addresses on the routed views the caller adds the experts itself (the rule of
    # src/runtime/moe.c:654-660), and the routing is published at begin
    for slot in (abi.W_ROUTED_GATE, abi.W_ROUTED_UP, abi.W_ROUTED_DOWN):
        case.job.weights[slot].device_address = 0
    u = TokenLocal(case, row=2, device=True)
    assert u.begin() == 0, u.err.message
    assert list(u.result.router.selected_experts)[:case.topk] == list(want["selected"][0])
    for rank in range(case.topk):
        views, _ = u.expert_views(int(u.result.router.selected_experts[rank]))
        assert u.add(views, float(u.result.router.selected_weights[rank]), False) == 0, u.err.message
    views, _ = u.expert_views(None)
    assert u.add(views, 0.0, True) == 0 and u.finish() == 0, u.err.message
    again = backend.read_f32(u.device_out, case.streams * case.hidden)
    assert np.all(np.abs(again - got) <= 2.0 ** -6 * scale)
    assert u.close() == 0


def test_token_local_hash_router(backend, oracle):
    case = MoeCase(backend, oracle, hidden=512, rows=3, streams=2, iterations=3, act=abi.ACT_DEVICE_F32,
                   hash_vocab=16)
    t = TokenLocal(case, row=1)
    t.job.token_id, t.job.token_id_present = int(case.tokens[1]), 1
    assert t.begin() == 0, t.err.message
    assert list(t.result.router.selected_experts)[:case.topk] == list(case.table[case.tokens[1]])
    rc, _, want_w, _ = oracle.moe_route_hash(
        np.array(list(t.result.router.router_logits)[:case.experts], np.float32), case.table,
        int(case.tokens[1]), case.topk, case.scoring, True, 1.5)
    assert rc == 0 and np.max(np.abs(np.array(list(t.result.router.selected_weights)[:case.topk]) - want_w)) <= 1e-6
    assert t.close() == 0
    t.job.token_id = 16
    assert t.begin() == abi.BOUNDS


def test_token_local_refusals(backend, oracle):
    case = MoeCase(backend, oracle, hidden=512, rows=2, streams=2, iterations=2, act=abi.ACT_DEVICE_F32)
    t = TokenLocal(case)
    t.result.post_capacity = 1
    assert t.begin() == abi.INVALID_ARG and not t.handle.value
    t.result.post_capacity = 2
    case.plan.mhc_mixing_rows = 9
    assert t.begin() == abi.BOUNDS
    case.plan.mhc_mixing_rows = 8
    case.plan.router_class = abi.ROUTER_HASH          # no token id
    assert t.begin() == abi.BOUNDS
    case.plan.router_class = 7
    assert t.begin() == abi.UNSUPPORTED
    case.plan.router_class = abi.ROUTER_LEARNED
    bad = t.row.copy()
    bad[3] = np.inf
    t.job.expanded_input = bad.ctypes.data
    assert t.begin() == abi.BACKEND and not t.handle.value      # kernels flag non-finite input
    t.job.expanded_input = t.row.ctypes.data
    assert t.begin() == 0, t.err.message
    views, _ = t.expert_views(0)
    views[2].row_count = case.hidden - 1
    assert t.add(views, 0.5, False) == abi.INVALID_ARG
    views, _ = t.expert_views(0)
    views[0].qtype = 2                                           # Q4_0: no device compute
    assert t.add(views, 0.5, False) == abi.UNSUPPORTED
    t.result.routed_capacity = 1
    assert t.finish() == abi.INVALID_ARG
    t.result.routed_capacity = case.hidden
    assert t.finish() == 0 and t.close() == 0
