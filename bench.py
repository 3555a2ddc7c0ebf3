#!/usr/bin/env python3
"""Benchmark of the quantized-weight matmul path on one MI355X.

A "step" is one pass of the decode MoE layer (BASELINE.json config 3: hidden 7168, 256 routed
experts + 1 shared, top-8 sigmoid routing, expert width 2048, IQ2_XXS weights, 32 concurrent
single-token rows, Q8_K device activations) over synthetic inputs already resident in HBM.
`value` is the algorithmic expert-weight bytes the step must read, (U + 1) * 11 354 112 with U
the distinct routed experts hit, divided by the step time.

Prints ONE JSON line. `roofline` covers the dominant kernel (the routed gate/up sweep), timed
with events on the launch stream; `cpu_baseline` is the reference's own CPU expert path
(compiled from its sources; the C restatement beside it) timed on the host cores over a bounded
sample of the same workload. `prefill` holds BASELINE config 4 (2048 rows on the int8 matrix
cores), `prefill_q4k` and `decode_q4k` the same batches with Q4_K experts, `model_file_layer` both
batches with the formats of the reference's model file (IQ2_XXS gate/up and Q2_K down routed experts,
a Q8_0 shared expert), `decode_envelope` the
headline step with four residual streams around the layer, `decode_small_batches` the headline
layer at 1 to 16 rows, and `dense` configs
0-2 and an output head as single matvec launches; the prefill legs and the dense configs carry a
CPU baseline of their own (the same sample extrapolated per row; the reference's row dot over
the whole matrix).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_INT8_PEAK_TOPS = 5000.0
HIDDEN, INTERMEDIATE, EXPERTS, TOPK, ROWS = 7168, 2048, 256, 8, 32
EXPERT_BYTES = 3 * 3_784_704   # gate + up + down of one IQ2_XXS expert
# iq2_sweep_kernel<fused gate/up>, 159 distinct routed experts + the shared one: FETCH_SIZE
# 616 664 x 2.000 KiB + WRITE_SIZE 15 776 x 1.000 KiB per launch (counter units scaled by a 1 GiB
# read kernel and a 256 MiB fill kernel in the same runs)
GATE_UP_TRAFFIC_BYTES = int((616_664 * 2.0 + 15_776) * 1024)
GATE_UP_TRAFFIC_EXPERTS = 159
GATE_UP_IMAGE_TRAFFIC_BYTES = int((664_027 * 2.0 + 18_176) * 1024)   # the same launch over the sweep image


def synth_iq2xxs(torch, blocks: int, device, seed: int):
    """Random IQ2_XXS superblocks: uniform grid/sign/scale bytes, positive fp16 block scale."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    raw = torch.randint(0, 256, (blocks, 66), dtype=torch.uint8, device=device, generator=gen)
    d = (torch.rand(blocks, device=device, generator=gen) * 3.5e-4 + 1.0e-4).to(torch.float16)
    raw[:, :2] = d.view(torch.uint8).reshape(blocks, 2)
    return raw.reshape(-1)


def synth_q4k(torch, blocks: int, device, seed: int):
    """Random Q4_K superblocks: uniform scale, minimum and nibble bytes, small positive fp16 d and dmin."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    raw = torch.randint(0, 256, (blocks, 144), dtype=torch.uint8, device=device, generator=gen)
    d = (torch.rand(blocks, device=device, generator=gen) * 1.0e-4 + 2.0e-5).to(torch.float16)
    raw[:, 0:2] = d.view(torch.uint8).reshape(blocks, 2)
    raw[:, 2:4] = raw[:, 0:2]
    return raw.reshape(-1)


def event_ms(torch, fn, repeats: int) -> float:
    """Average duration of fn() in ms, measured with events on the current (launch) stream."""
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(repeats):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / repeats


def device_clock(torch, dev):
    """Clock of the matrix cores under full load, from a launch of known length in cycles
    (every SIMD runs back-to-back 32-cycle matrix instructions on four accumulators), next to the clock the
    device properties name. Fractions of the matrix-core peak are quoted against the published
    peak, which assumes the peak engine clock (2.4 GHz): the measured clock says how much of a
    gap is frequency."""
    import ctypes as C
    from yvex_amd import load_library
    lib = load_library()
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    chain = 100_000

    def once():
        lib.yvex_hip_clock_probe(C.c_uint64(chain), C.c_void_p(sink.data_ptr()), stream)
    once()
    torch.cuda.synchronize()
    ms = event_ms(torch, once, 3)
    engine, memory = C.c_int(0), C.c_int(0)
    lib.yvex_hip_device_clocks(0, C.byref(engine), C.byref(memory))
    return {"matrix_load_ghz": round(chain * 32 / (ms * 1e6), 3),
            "device_peak_engine_mhz": round(engine.value / 1e3, 1),
            "device_peak_memory_mhz": round(memory.value / 1e3, 1),
            "probe": f"{chain} back-to-back V_MFMA_I32_32X32X32_I8 per SIMD on every compute unit, "
                     f"32 cycles each, {round(ms, 3)} ms"}


def cpu_baseline(sample_rows: int, threads: int):
    """Time the CPU oracle (reference algorithm: decode to float, double accumulate) on
    `sample_rows` rows of the same layer shape; weights for the experts those rows hit only."""
    import numpy as np
    import oracle
    g = oracle.Generator(42, "bench.cpu")
    experts = 16   # the rows below route among 16 experts: enough for top-8, small enough to build
    gate = g.iq2xxs(experts * INTERMEDIATE * HIDDEN // 256)
    up = g.iq2xxs(experts * INTERMEDIATE * HIDDEN // 256)
    down = g.iq2xxs(experts * HIDDEN * INTERMEDIATE // 256)
    shared = tuple(g.iq2xxs(INTERMEDIATE * HIDDEN // 256) for _ in range(3))
    x = g.normal(sample_rows * HIDDEN).reshape(sample_rows, HIDDEN)
    logits = g.normal(sample_rows * experts).reshape(sample_rows, experts)
    t0 = time.perf_counter()
    oracle.moe_layer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=experts, topk=TOPK,
                     qtypes=(oracle.IQ2_XXS,) * 3, routed=(gate, up, down), shared=shared,
                     inputs=x, logits=logits, scoring=oracle.SIGMOID, normalize=True, scaling=1.0,
                     act_q8=False, threads=threads)
    seconds = time.perf_counter() - t0
    touched = sample_rows * (TOPK + 1) * EXPERT_BYTES   # the CPU path re-reads an expert per row
    return {"value": touched / seconds / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{sample_rows} rows x (top-8 + shared) expert FFNs of the same layer shape, "
                      f"scalar C restatement of yvex_quant_cpu_dot/yvex_moe_expert_cpu",
            "tokens_per_s": sample_rows / seconds, "seconds": seconds}


def cpu_baseline_reference(sample_rows: int):
    """The same sample through the reference's own yvex_moe_expert_cpu, compiled from its sources
    into oracle/_ref (single thread, as the reference runs it). None where that library is absent."""
    import ctypes as C
    import numpy as np
    import oracle
    from yvex_amd import abi
    ref = oracle.ref_lib()
    if ref is None:
        return None
    g = oracle.Generator(42, "bench.cpu")
    experts = 16
    gate = g.iq2xxs(experts * INTERMEDIATE * HIDDEN // 256)
    up = g.iq2xxs(experts * INTERMEDIATE * HIDDEN // 256)
    down = g.iq2xxs(experts * HIDDEN * INTERMEDIATE // 256)
    shared = tuple(g.iq2xxs(INTERMEDIATE * HIDDEN // 256) for _ in range(3))
    x = g.normal(sample_rows * HIDDEN).reshape(sample_rows, HIDDEN)
    logits = g.normal(sample_rows * experts).reshape(sample_rows, experts)
    plan = abi.LayerPlan()
    plan.hidden_width, plan.activation_limit = HIDDEN, 10.0

    def views(blobs, expert):
        out = []
        for blob, width, rows in zip(blobs, (HIDDEN, HIDDEN, INTERMEDIATE), (INTERMEDIATE, INTERMEDIATE, HIDDEN)):
            v = abi.WeightView()
            row_bytes = width // 256 * 66
            v.qtype, v.row_width, v.row_count, v.row_bytes = oracle.IQ2_XXS, width, rows, row_bytes
            v.encoded, v.encoded_bytes = blob.ctypes.data + expert * rows * row_bytes, rows * row_bytes
            out.append(v)
        return out

    ref.yvex_moe_expert_cpu.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_float, C.c_void_p, C.c_void_p]
    y, err = np.zeros(HIDDEN, np.float32), abi.Error()
    t0 = time.perf_counter()
    for row in range(sample_rows):
        rc, selected, weights, _ = oracle.moe_route(logits[row], None, TOPK, oracle.SIGMOID, True, 1.0)
        work = [(views((gate, up, down), int(e)), float(w)) for e, w in zip(selected, weights)]
        work.append((views(shared, 0), 1.0))
        for v, weight in work:
            rc = ref.yvex_moe_expert_cpu(C.byref(plan), C.byref(v[0]), C.byref(v[1]), C.byref(v[2]),
                                         x[row].ctypes.data, C.c_float(weight), y.ctypes.data, C.byref(err))
            if rc != 0:
                return None
    seconds = time.perf_counter() - t0
    touched = sample_rows * (TOPK + 1) * EXPERT_BYTES
    return {"value": touched / seconds / 1e9, "unit": "GB/s", "cores": 1, "kind": "reference",
            "sample": f"{sample_rows} rows x (top-8 + shared) expert FFNs of the same layer shape through "
                      f"yvex_moe_expert_cpu of the reference, compiled from its own sources",
            "tokens_per_s": sample_rows / seconds, "seconds": seconds}


def cpu_baseline_dense():
    """BASELINE configs 0-2 on the host: one pass of the whole matrix against one F32 input row
    through the reference's own yvex_quant_cpu_dot (compiled from its sources into oracle/_ref;
    one core, row by row, as src/graph/core.c:1131-1166 calls it), or through the C restatement
    where the reference has no codec (Q4_K) or its library is absent. A batch of b rows costs b
    such passes on the CPU path: it has no batched form."""
    import ctypes as C
    import numpy as np
    import oracle
    ref = oracle.ref_lib()
    if ref is not None:
        ref.yvex_quant_cpu_dot.argtypes = [C.c_uint, C.c_void_p, C.c_size_t, C.c_void_p, C.c_ulonglong,
                                           C.c_void_p, C.c_void_p, C.c_void_p]
    out = {}
    g = oracle.Generator(42, "bench.cpu.dense")
    for name, qt, rows, width in (("cfg0_q8_0_4096x4096", oracle.Q8_0, 4096, 4096),
                                  ("cfg1_q4_k_2048x7168", oracle.Q4_K, 2048, 7168),
                                  ("cfg2_iq2_xxs_7168x2048", oracle.IQ2_XXS, 7168, 2048)):
        w = g.weights(qt, rows, width)
        x = g.normal(width)
        row_bytes = oracle.row_bytes(qt, width)
        use_ref = ref is not None and qt != oracle.Q4_K
        t0 = time.perf_counter()
        if use_ref:
            y, failure, err = C.c_float(), (C.c_ubyte * 512)(), (C.c_ubyte * 512)()
            base = w.ctypes.data
            for r in range(rows):
                if ref.yvex_quant_cpu_dot(qt, base + r * row_bytes, row_bytes, x.ctypes.data, width, C.byref(y),
                                          failure, err) != 0:
                    use_ref = False
                    break
        if not use_ref:
            t0 = time.perf_counter()
            oracle.matvec(qt, w, rows, width, x)
        seconds = time.perf_counter() - t0
        out[name] = {"ms": round(seconds * 1e3, 3), "GB_per_s": round(w.nbytes / seconds / 1e9, 4),
                     "cores": 1, "kind": "reference" if use_ref else "port",
                     "sample": "the whole matrix against one F32 input row"
                               + ("" if use_ref or qt != oracle.Q4_K else " (the reference refuses Q4_K: C restatement)")}
    return out


def AbiLayer(torch, routed, shared, router, x_host, rows, qtype=16, sweep_image=False):
    """The benchmark layer behind include/yvex_rocm.h (yvex_amd.host.RowBatchLayer at this
    benchmark's shape)."""
    from yvex_amd.host import RowBatchLayer
    return RowBatchLayer(torch, routed, shared, router, x_host, rows, hidden=HIDDEN, intermediate=INTERMEDIATE,
                         experts=EXPERTS, topk=TOPK, qtype=qtype, sweep_image=sweep_image)


def dense_leg(torch, K, dev, repeats: int):
    """BASELINE configs 0-2 and an output head as single matvec launches: random packed bytes with
    small positive fp16 block scales, at least 32 distinct weight copies and more than 320 MB of
    them walked in turn (2 for the head) so that no launch finds its weights in a cache. Bytes
    counted: the encoded matrix. Batches of 16 rows and more run on the int8 matrix cores."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(7)
    out = {}

    def eager_and_graph(once, calls):
        """Average time of once(): launched eagerly (ms) and replayed from a captured graph of
        `calls` launches (us; None if capture is refused). The graph figure leaves out the host's
        time per call, which is what a launch of a few microseconds is otherwise measured by."""
        for _ in range(calls):
            once()
        torch.cuda.synchronize()
        ms = event_ms(torch, once, repeats)
        graph_us = None
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                with torch.cuda.graph(graph, stream=side):
                    for _ in range(calls):
                        once()
                graph.replay()
                side.synchronize()
                replays = max(1, repeats // calls)
                start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record(side)
                for _ in range(replays):
                    graph.replay()
                stop.record(side)
                stop.synchronize()
                graph_us = start.elapsed_time(stop) / (replays * calls) * 1e3
            torch.cuda.current_stream().wait_stream(side)
        except Exception as error:   # capture refused: keep the eager figure
            graph_us = None
            print(f"dense leg: graph capture unavailable ({error})", file=sys.stderr)
        return ms, graph_us

    def run(name, qt, rows, width, inputs, q8, copies=None):
        total = rows * K.row_bytes(qt, width)
        # enough distinct copies that a launch cannot find its matrix in the 256 MB last-level cache
        copies = copies or max(32, -(-320_000_000 // total))
        if qt == K.IQ2_XXS:
            w = synth_iq2xxs(torch, copies * rows * width // 256, dev, 5)
        else:
            w = torch.randint(0, 256, (copies * total,), dtype=torch.uint8, device=dev, generator=gen)
            blocks = w.view(-1, 34 if qt == K.Q8_0 else 144)
            d = (torch.rand(blocks.shape[0], device=dev, generator=gen) * 1e-3 + 1e-4).to(torch.float16)
            blocks[:, 0:2] = d.view(torch.uint8).reshape(-1, 2)
            if qt == K.Q4_K:
                blocks[:, 2:4] = blocks[:, 0:2]
        x = torch.randn((inputs, width), device=dev, generator=gen)
        status = K.new_status(dev)
        act = K.q8k_quantize(x, status) if q8 else x
        result = torch.empty((inputs, rows), dtype=torch.float32, device=dev)
        turn = [0]

        def once():
            i = turn[0] % copies
            turn[0] += 1
            K.matvec(w[i * total:(i + 1) * total], qt, rows, width, act, input_q8=q8, input_rows=inputs,
                     status=status, out=result)
        ms, graph_us = eager_and_graph(once, copies)
        best_ms = min(ms, graph_us * 1e-3) if graph_us else ms
        out[name] = {"us": round(ms * 1e3, 2), "graph_us": round(graph_us, 2) if graph_us else None,
                     "GB_per_s": round(total / (best_ms * 1e-3) / 1e9, 1),
                     "hbm_peak_frac": round(total / (best_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "matrix_bytes": total, "copies": copies, "status": int(status.item())}
        if inputs >= 16:
            out[name]["int8_TOPs"] = round(2.0 * rows * width * inputs / (best_ms * 1e-3) / 1e12, 1)
        del w

    run("cfg0_q8_0_4096x4096_f32_b1", K.Q8_0, 4096, 4096, 1, False)
    run("cfg0_q8_0_4096x4096_q8k_b1", K.Q8_0, 4096, 4096, 1, True)
    run("cfg0_q8_0_4096x4096_q8k_b16", K.Q8_0, 4096, 4096, 16, True)
    run("cfg0_q8_0_4096x4096_q8k_b2048", K.Q8_0, 4096, 4096, 2048, True)
    run("cfg1_q4_k_2048x7168_q8k_b1", K.Q4_K, 2048, 7168, 1, True)
    run("cfg1_q4_k_2048x7168_q8k_b16", K.Q4_K, 2048, 7168, 16, True)
    run("cfg1_q4_k_2048x7168_q8k_b256", K.Q4_K, 2048, 7168, 256, True)
    run("cfg1_q4_k_2048x7168_q8k_b2048", K.Q4_K, 2048, 7168, 2048, True)
    run("cfg2_iq2_xxs_7168x2048_q8k_b2048", K.IQ2_XXS, 7168, 2048, 2048, True)
    run("cfg2_iq2_xxs_7168x2048_f32_b1", K.IQ2_XXS, 7168, 2048, 1, False)
    run("cfg2_iq2_xxs_7168x2048_q8k_b1", K.IQ2_XXS, 7168, 2048, 1, True)
    run("head_q8_0_129280x7168_q8k_b1", K.Q8_0, 129280, 7168, 1, True, copies=2)
    run("head_q8_0_129280x7168_q8k_b32", K.Q8_0, 129280, 7168, 32, True, copies=2)
    # greedy selection over one 129 280-entry logits row, left on the device by the head
    logits = torch.randn((1, 129280), device=dev, generator=gen)
    status = K.new_status(dev)
    picked = K.argmax_f32(logits, status)
    torch.cuda.synchronize()
    ms, graph_us = eager_and_graph(lambda: K.argmax_f32(logits, status, out=picked), 16)
    out["greedy_selection_1x129280"] = {"us": round(ms * 1e3, 2),
                                        "graph_us": round(graph_us, 2) if graph_us else None,
                                        "status": int(status.item())}
    # residual-stream ingress and egress around a layer: 4 streams of 7168, decode and prefill rows
    streams, width, mixing = 4, 7168, 24
    for rows in (32, 2048):
        x = torch.randn((rows, streams * width), device=dev, generator=gen)
        mixes = torch.randn((rows, mixing), device=dev, generator=gen)
        scale = torch.tensor([0.5, -0.25, 0.75], device=dev)
        base = torch.randn(mixing, device=dev, generator=gen) * 0.5
        norm = 1.0 + 0.2 * torch.randn(width, device=dev, generator=gen)
        kw = dict(streams=streams, width=width, iterations=20, rms_epsilon=1e-6, mhc_epsilon=1e-6,
                  post_multiplier=2.0)
        status = K.new_status(dev)
        held = K.mhc_ingress(x, mixes, scale, base, norm, status=status, **kw)
        ms, graph_us = eager_and_graph(
            lambda: K.mhc_ingress(x, mixes, scale, base, norm, status=status, out=held, **kw), 8)
        best_ms = min(ms, graph_us * 1e-3) if graph_us else ms
        moved = rows * (streams * width + width) * 4
        out[f"stream_ingress_{rows}x4x7168"] = {
            "us": round(ms * 1e3, 2), "graph_us": round(graph_us, 2) if graph_us else None,
            "GB_per_s": round(moved / (best_ms * 1e-3) / 1e9, 1), "bytes": moved, "status": int(status.item())}
        spread = K.mhc_egress(held[0], x, held[1], held[2], streams=streams, width=width, status=status)
        ms, graph_us = eager_and_graph(
            lambda: K.mhc_egress(held[0], x, held[1], held[2], streams=streams, width=width, status=status,
                                 out=spread), 8)
        best_ms = min(ms, graph_us * 1e-3) if graph_us else ms
        moved = rows * (2 * streams * width + width) * 4
        out[f"stream_egress_{rows}x4x7168"] = {
            "us": round(ms * 1e3, 2), "graph_us": round(graph_us, 2) if graph_us else None,
            "GB_per_s": round(moved / (best_ms * 1e-3) / 1e9, 1), "bytes": moved, "status": int(status.item())}
    return out


def tile_classes(populations):
    """Token tiles of the row-batch kernels: full 64-pair tiles, and the partial tile a bucket
    ends with, by whether it runs with two 32-token blocks or one."""
    out = {"64": 0, "33-63": 0, "1-32": 0}
    for n in populations:
        full, rest = divmod(int(n), 64)
        out["64"] += full
        if rest:
            out["33-63" if rest > 32 else "1-32"] += 1
    return out


def prefill_leg(torch, K, MoeLayer, weights, shared, dev, steps: int, warmup: int, qt=16):
    """BASELINE config 4: the same layer over 2048 rows whose top-8 experts follow a Zipf(1.1)
    popularity (Gumbel top-k over log-popularity logits), row-batch kernels on the int8 matrix
    cores. Ops counted: 2 * (2*I*H + H*I) per (row, expert) pair, routed and shared."""
    rows = 2048
    gen = torch.Generator(device=dev)
    gen.manual_seed(4242)
    rank = torch.randperm(EXPERTS, device=dev, generator=gen).float() + 1.0
    popularity = rank.pow(-1.1)
    uniform = torch.rand((rows, EXPERTS), device=dev, generator=gen).clamp_(1e-9, 1.0 - 1e-9)
    wanted = popularity.log()[None, :] - (-uniform.log()).log()
    x = torch.randn((rows, HIDDEN), device=dev, generator=gen)
    # router weights whose projection of x gives those logits: the minimum-norm solution of
    # x . router^T = wanted (2048 equations per expert, 7168 unknowns), solved in double
    xd = x.double()
    router = (xd.T @ torch.linalg.solve(xd @ xd.T, wanted.double())).T.float().contiguous()
    logits = K.matvec(router.view(torch.uint8).reshape(-1), K.F32, EXPERTS, HIDDEN, x,
                      status=K.new_status(dev))
    layer = MoeLayer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK,
                     qtypes=(qt, qt, qt), routed=weights, shared=shared, bias=None,
                     scoring=K.SIGMOID, normalize=True, scaling=1.0, limit=10.0, act_q8=True,
                     max_rows=rows, device=dev, matrix_cores=True)
    for _ in range(warmup):
        layer.run(x, logits)
    torch.cuda.synchronize()
    if int(layer.status.item()) != 0:
        return {"error": f"device status {int(layer.status.item())}"}
    step_ms = event_ms(torch, lambda: layer.run(x, logits), steps)
    pairs = rows * TOPK
    acts = layer.act_q8_rows
    up_ms = event_ms(torch, lambda: K.moe_up_rows(
        layer.routed, acts, layer.weights, layer.worklist, pairs, TOPK, EXPERTS, layer.limit,
        layer.intermediate_f32, layer.status), steps)
    down_ms = event_ms(torch, lambda: K.moe_down_rows(
        layer.routed, layer.intermediate_q8, layer.worklist, pairs, EXPERTS, layer.pair_outputs,
        layer.status), steps)
    # the same step through include/yvex_rocm.h (router projection included)
    stage_rows = layer.run(x, logits).clone()
    torch.cuda.synchronize()
    abi_layer = AbiLayer(torch, weights, shared, router, x.cpu().numpy(), rows, qtype=qt)
    abi_layer.step(defer=False)
    abi_same = bool((torch.from_numpy(abi_layer.output()) == stage_rows.cpu()).all().item())
    abi_unique = int(abi_layer.result.unique_experts)
    abi_eager_ms = abi_layer.timed(steps, warmup, eager=True)
    abi_graph_ms = abi_layer.timed(steps, max(warmup, 2))
    abi_layer.close()
    harness_ms = step_ms
    step_ms = min(abi_graph_ms, abi_eager_ms)
    residency = "canonical bytes"
    # IQ2_XXS experts resident as the sweep image only: the matrix-core kernels read it as well
    image = None
    if qt == 16:
        image_layer = AbiLayer(torch, weights, shared, router, x.cpu().numpy(), rows, qtype=qt, sweep_image=True)
        image_layer.step(defer=False)
        image_same = bool((torch.from_numpy(image_layer.output()) == stage_rows.cpu()).all().item())
        image_ms = image_layer.timed(steps, max(warmup, 2))
        image_layer.close()
        del image_layer
        torch.cuda.empty_cache()
        image = {"graph_ms_per_step": round(image_ms, 4), "rows_identical_to_canonical": image_same}
        if not image_same:
            return {"error": "the sweep image and the canonical rows disagree on the matrix-core kernels"}
        # as for the decode step, the faster residency is the leg's figure (same rows bit for bit;
        # the operations counted do not depend on it)
        if image_ms < step_ms:
            step_ms, residency = image_ms, "sweep image"

    pair_ops = 2 * (2 * INTERMEDIATE * HIDDEN + HIDDEN * INTERMEDIATE)
    routed_ops, shared_ops = pair_ops * pairs, pair_ops * rows
    up_ops = 2 * 2 * INTERMEDIATE * HIDDEN * pairs
    populations = layer.worklist.bucket_populations[: int(layer.worklist.counts[0].item())]
    return {
        "workload": f"moe_prefill_{'iq2xxs' if qt == 16 else 'q4k'}: 2048 rows, Zipf(1.1) top-8 of 256 experts + shared, "
                    "Q8_K activations",
        "ms_per_step": round(step_ms, 4), "tokens_per_s": round(rows / (step_ms * 1e-3), 1),
        "residency": residency,
        "c_abi": {"entry": "yvex_rocm_backend_moe_operations_get()->execute_rows + complete_rows",
                  "graph_ms_per_step": round(abi_graph_ms, 4), "eager_ms_per_step": round(abi_eager_ms, 4),
                  "rows_identical_to_stage_harness": abi_same,
                  "distinct_routed_experts": abi_unique},
        "c_abi_sweep_image": image,
        "stage_harness_ms_per_step": round(harness_ms, 4),
        "int8_TOPs": round((routed_ops + shared_ops) / (step_ms * 1e-3) / 1e12, 2),
        "mfma_peak_frac": round((routed_ops + shared_ops) / (step_ms * 1e-3) / 1e12 / MFMA_INT8_PEAK_TOPS, 4),
        "distinct_routed_experts": int(populations.numel()),
        "token_tiles": tile_classes(populations.cpu().tolist()),
        "max_bucket_population": int(populations.max().item()),
        "roofline": {"bound": "mfma",
                     "kernel": "mfma_iq2_kernel<fused gate/up>" if qt == 16 else "rows_q4k_kernel<fused gate/up>",
                     "achieved": round(up_ops / (up_ms * 1e-3) / 1e12, 2), "peak": MFMA_INT8_PEAK_TOPS,
                     "unit": "TOP/s", "frac": round(up_ops / (up_ms * 1e-3) / 1e12 / MFMA_INT8_PEAK_TOPS, 4),
                     "launch_ms": round(up_ms, 4)},
        "kernels_ms": {"gate_up_rows": round(up_ms, 4), "down_rows": round(down_ms, 4)},
        "clock_after": device_clock(torch, dev),
    }


def decode_q4k_leg(torch, K, weights, shared, dev, steps: int, warmup: int):
    """The headline batch (32 rows, top-8 of 256 + shared) with Q4_K experts, through the C ABI:
    the decode-width sweeps read Q4_K rows too. Bytes counted: the canonical bytes of the distinct
    experts hit."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(77)
    x = torch.randn((ROWS, HIDDEN), device=dev, generator=gen)
    router = (torch.randn((EXPERTS, HIDDEN), device=dev, generator=gen) / HIDDEN ** 0.5).contiguous()
    layer = AbiLayer(torch, weights, shared, router, x.cpu().numpy(), ROWS, qtype=K.Q4_K)
    layer.step(defer=False)
    unique = int(layer.result.unique_experts)
    eager_ms = layer.timed(steps, warmup, eager=True)
    graph_ms = layer.timed(steps, max(warmup, 2))
    layer.close()
    step_ms = min(graph_ms, eager_ms)
    expert_bytes = 3 * INTERMEDIATE * HIDDEN // 256 * 144
    read = (unique + 1) * expert_bytes
    return {"workload": "moe_decode_q4k: 32 rows, top-8 of 256 Q4_K experts + shared, Q8_K activations",
            "ms_per_step": round(step_ms, 4), "graph_ms_per_step": round(graph_ms, 4),
            "eager_ms_per_step": round(eager_ms, 4), "distinct_routed_experts": unique,
            "GB_per_s": round(read / (step_ms * 1e-3) / 1e9, 1),
            "hbm_peak_frac": round(read / (step_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}


def synth_q2k(torch, blocks: int, device, seed: int):
    """Q2_K superblocks (84 bytes): random scale/minimum bytes and 2-bit codes, small positive fp16
    d and dmin behind them."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    raw = torch.randint(0, 256, (blocks, 84), dtype=torch.uint8, device=device, generator=gen)
    scales = (torch.rand((blocks, 2), device=device, generator=gen) * 1e-3 + 1e-4).to(torch.float16)
    raw[:, 80:84] = scales.view(torch.uint8).reshape(-1, 4)
    return raw.reshape(-1)


def synth_q8_0(torch, blocks: int, device, seed: int):
    """Q8_0 blocks (34 bytes): a small positive fp16 scale, then 32 random int8 codes."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    raw = torch.randint(0, 256, (blocks, 34), dtype=torch.uint8, device=device, generator=gen)
    scales = (torch.rand(blocks, device=device, generator=gen) * 1e-3 + 1e-4).to(torch.float16)
    raw[:, 0:2] = scales.view(torch.uint8).reshape(-1, 2)
    return raw.reshape(-1)


def model_file_layer_leg(torch, gate, up, dev, steps: int, warmup: int):
    """The formats of the reference's model file (src/graph/families/deepseek_v4.c:1550-1575: routed
    experts with IQ2_XXS gate and up and Q2_K down matrices, everything else Q8_0, the shared
    expert with it) through the C ABI, the routed gate and up experts resident as the sweeps'
    image and the rest as canonical rows: the headline batch of 32 rows (decode sweeps, the shared
    expert as dense projections) and 2048 rows (matrix cores). Bytes counted: the canonical bytes
    of the distinct experts hit and of the shared expert."""
    from yvex_amd.host import RowBatchLayer
    blocks = INTERMEDIATE * HIDDEN // 256
    down = synth_q2k(torch, EXPERTS * blocks, dev, 41)
    shared = tuple(synth_q8_0(torch, blocks * 8, dev, 42 + i) for i in range(3))
    gen = torch.Generator(device=dev)
    gen.manual_seed(78)
    router = (torch.randn((EXPERTS, HIDDEN), device=dev, generator=gen) / HIDDEN ** 0.5).contiguous()
    out = {"workload": "routed experts IQ2_XXS gate/up (sweep image) + Q2_K down, Q8_0 shared expert, top-8 of 256, "
                       "Q8_K activations"}
    for rows, count in ((ROWS, steps), (2048, max(3, steps // 10))):
        x = torch.randn((rows, HIDDEN), device=dev, generator=gen)
        layer = RowBatchLayer(torch, (gate, up, down), shared, router, x.cpu().numpy(),
                              rows, hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK,
                              qtype=16, down_qtype=10, shared_qtype=8, sweep_image=True)
        layer.step(defer=False)
        unique = int(layer.result.unique_experts)
        matrix = int(layer.result.tensor_core_launches)
        ms = min(layer.timed(count, max(warmup, 2)), layer.timed(count, warmup, eager=True))
        layer.close()
        read = unique * blocks * (2 * 66 + 84) + 3 * blocks * 8 * 34
        leg = {"ms_per_step": round(ms, 4), "distinct_routed_experts": unique, "matrix_core_launches": matrix,
               "GB_per_s": round(read / (ms * 1e-3) / 1e9, 1)}
        if rows > ROWS:
            ops = 2 * 3 * INTERMEDIATE * HIDDEN * rows * (TOPK + 1)
            leg["int8_TOPs"] = round(ops / (ms * 1e-3) / 1e12, 2)
            leg["tokens_per_s"] = round(rows / (ms * 1e-3), 1)
        out[f"rows_{rows}"] = leg
    return out


def envelope_leg(torch, routed, shared, router, dev, steps: int, warmup: int):
    """The headline step for a layer with residual streams around it (four streams of 7168, 24
    mixing rows, 20 Sinkhorn iterations; src/backend/cuda/moe.c:1210-1254, 1533-1541), through the
    same execute_rows over the sweep image: mixing projection, ingress with the weighted norm,
    the layer, egress."""
    from yvex_amd.host import RowBatchLayer
    gen = torch.Generator(device=dev)
    gen.manual_seed(43)
    streams, mixing = 4, 24
    x = torch.randn((ROWS, streams * HIDDEN), device=dev, generator=gen)
    envelope = dict(streams=streams, iterations=20,
                    function=torch.randn((mixing, streams * HIDDEN), device=dev, generator=gen) / (streams * HIDDEN) ** 0.5,
                    scale=torch.tensor([0.5, -0.25, 0.75], device=dev),
                    base=torch.randn(mixing, device=dev, generator=gen) * 0.5,
                    norm=(1.0 + 0.2 * torch.randn(HIDDEN, device=dev, generator=gen)).to(torch.bfloat16))
    layer = RowBatchLayer(torch, routed, shared, router, x.cpu().numpy(), ROWS, hidden=HIDDEN,
                          intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK, sweep_image=True,
                          envelope=envelope)
    layer.step(defer=False)
    launches = int(layer.result.kernel_launches)
    eager_ms = layer.timed(steps, warmup, eager=True)
    graph_ms = layer.timed(steps, max(warmup, 2))
    layer.close()
    return {"workload": "the decode step with 4 residual streams of 7168 around the layer (24 mixing rows, "
                        "20 Sinkhorn iterations), sweep image",
            "ms_per_step": round(min(graph_ms, eager_ms), 4), "graph_ms_per_step": round(graph_ms, 4),
            "eager_ms_per_step": round(eager_ms, 4), "kernel_launches": launches}


def small_batches_leg(torch, routed, shared, router, dev, steps: int, warmup: int):
    """The headline layer at other decode widths (1, 4, 8 and 16 rows) through the same
    execute_rows over the sweep image: step time and GB/s of the distinct experts' canonical bytes."""
    from yvex_amd.host import RowBatchLayer
    gen = torch.Generator(device=dev)
    gen.manual_seed(44)
    out = {}
    for rows in (1, 4, 8, 16):
        x = torch.randn((rows, HIDDEN), device=dev, generator=gen)
        layer = RowBatchLayer(torch, routed, shared, router, x.cpu().numpy(), rows, hidden=HIDDEN,
                              intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK, sweep_image=True)
        layer.step(defer=False)
        unique = int(layer.result.unique_experts)
        layer.timed(steps, warmup)
        ms = min(layer.timed(steps, max(warmup, 2)), layer.timed(steps, warmup, eager=True))
        layer.close()
        out[f"rows_{rows}"] = {"us_per_step": round(ms * 1e3, 1), "distinct_routed_experts": unique,
                               "GB_per_s": round((unique + 1) * EXPERT_BYTES / (ms * 1e-3) / 1e9, 1)}
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--act", choices=["q8k", "f32"], default="q8k")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=4)
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-dense", action="store_true")
    ap.add_argument("--separate-prepare", action="store_true",
                    help="launch routing, worklist and input quantization one by one instead of fused")
    ap.add_argument("--alone", action="store_true",
                    help="also time the two expert sweeps launched alone, back to back")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch a plain 1 GiB read kernel and a 256 MiB fill kernel, so a "
                         "counter run of this command holds kernels of known HBM traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (run with --gpus 1)",
              file=sys.stderr)
        return 2

    import torch
    from yvex_amd import kernels as K
    from yvex_amd.moe import MoeLayer

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    qt = K.IQ2_XXS
    up_blocks = EXPERTS * INTERMEDIATE * HIDDEN // 256
    gate = synth_iq2xxs(torch, up_blocks, dev, 1)
    up = synth_iq2xxs(torch, up_blocks, dev, 2)
    down = synth_iq2xxs(torch, up_blocks, dev, 3)
    shared = tuple(synth_iq2xxs(torch, INTERMEDIATE * HIDDEN // 256, dev, 10 + i) for i in range(3))
    gen = torch.Generator(device=dev)
    gen.manual_seed(42)
    x = torch.randn((ROWS, HIDDEN), device=dev, generator=gen)
    # router weights (F32, as the model stores them): logits = router . row, unit variance
    router = torch.randn((EXPERTS, HIDDEN), device=dev, generator=gen) / HIDDEN ** 0.5
    logits = K.matvec_f32_rows(router, x, K.new_status(dev))     # as execute_rows projects them
    layer = MoeLayer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK,
                     qtypes=(qt, qt, qt), routed=(gate, up, down), shared=shared, bias=None,
                     scoring=K.SIGMOID, normalize=True, scaling=1.0, limit=10.0,
                     act_q8=args.act == "q8k", max_rows=ROWS, device=dev)
    layer.fused_prepare = not args.separate_prepare

    for _ in range(args.warmup):
        layer.run(x, logits)
    torch.cuda.synchronize()
    if int(layer.status.item()) != 0:
        print(f"device status {int(layer.status.item())}", file=sys.stderr)
        return 1
    unique = int(layer.worklist.counts[0].item())
    max_pop = int(layer.worklist.counts[1].item())
    sweeps = int(layer.worklist.counts[3].item())

    def stage_timing(stage_layer):
        """Event and wall-clock ms per eager step of the stage harness, and the launch durations of
        its two expert sweeps inside those steps (events before and after each launch on the
        launch stream): (step by events, step by wall clock, {name: (mean, median)})."""
        torch.cuda.synchronize()
        stage_layer.marks = []          # events around the two expert sweeps of every timed step
        t0 = time.perf_counter()
        by_events = event_ms(torch, lambda: stage_layer.run(x, logits), args.steps)
        torch.cuda.synchronize()
        by_wall = (time.perf_counter() - t0) * 1e3 / args.steps
        marks, stage_layer.marks = stage_layer.marks, None

        def in_step_ms(begin, end):
            starts = [e for n, e in marks if n == begin]
            stops = [e for n, e in marks if n == end]
            spans = sorted(a.elapsed_time(b) for a, b in zip(starts, stops))
            return sum(spans) / len(spans), spans[len(spans) // 2]
        return by_events, by_wall, {"up": in_step_ms("up_begin", "up_end"),
                                    "down": in_step_ms("down_begin", "down_end")}

    step_ms_events, wall_ms, sweeps_ms = stage_timing(layer)
    canonical_sweeps_ms = sweeps_ms
    eager_ms = max(step_ms_events, wall_ms)
    step_ms, launch_mode = eager_ms, "eager launches"
    # The step is eight short launches; replaying them from a captured graph takes the host's
    # per-launch time out of the gaps between kernels. The replay is only used if it reproduces
    # the eager result bit for bit on several replays with eager work in between.
    graph_ms = None
    try:
        want = layer.run(x, logits).clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                captured = layer.run(x, logits)
        torch.cuda.current_stream().wait_stream(side)
        same = True
        for _ in range(3):
            layer.run(x * 0.5, logits)            # eager work between replays
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            same = same and torch.equal(captured, want) and int(layer.status.item()) == 0
        if same:
            for _ in range(args.warmup):
                graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
            if graph_ms < step_ms:
                step_ms, launch_mode = graph_ms, "hip graph replay"
        else:
            print("decode step: graph replay did not reproduce the eager result; eager timing kept",
                  file=sys.stderr)
    except Exception as error:       # capture refused: the eager figure stands
        print(f"decode step: graph capture unavailable ({error})", file=sys.stderr)
    harness_ms, harness_mode = step_ms, launch_mode
    # The step a caller of include/yvex_rocm.h gets: execute_rows on the backend's own stream
    # (router projection included), completion deferred to one complete_rows per phase. Its
    # launch graph is built by the library. This is the headline; the stage harness above only
    # serves the per-kernel timings.
    stage_rows = layer.run(x, logits).clone()
    torch.cuda.synchronize()
    abi_layer = AbiLayer(torch, (gate, up, down), shared, router, x.cpu().numpy(), ROWS)
    abi_layer.step(defer=False)
    abi_unique = int(abi_layer.result.unique_experts)
    abi_same = bool((torch.from_numpy(abi_layer.output()) == stage_rows.cpu()).all().item())
    abi_eager_ms = abi_layer.timed(args.steps, args.warmup, eager=True)
    abi_graph_ms = abi_layer.timed(args.steps, max(args.warmup, 2))
    graph_facts = (int(abi_layer.result.graph_launches), int(abi_layer.result.graph_replays))
    abi_sync_ms = abi_layer.timed(args.steps, args.warmup, defer=False)
    abi_launches = int(abi_layer.result.kernel_launches)
    abi_layer.close()
    if abi_unique != unique or not abi_same:
        print(f"decode step: execute_rows and the stage harness disagree (distinct experts {abi_unique} "
              f"vs {unique}, identical rows {abi_same})", file=sys.stderr)
        return 1
    step_ms = min(abi_graph_ms, abi_eager_ms)
    launch_mode = ("execute_rows, library launch graph, completion deferred to the phase barrier"
                   if abi_graph_ms <= abi_eager_ms else
                   "execute_rows, eager launches, completion deferred to the phase barrier")
    # The same step with the experts resident as the decode sweeps' image: a caller's residency
    # step plans it (derived_layout_plan, 72 bytes a superblock instead of 66) and builds it on the
    # device from the canonical bytes; execute_rows takes DERIVED_BACKEND views of it. The rows
    # must equal the canonical run's bit for bit. The faster of the two residencies is the
    # headline; the weight bytes counted are the canonical GGUF bytes either way.
    image = None
    if args.act == "q8k":
        image_layer = AbiLayer(torch, (gate, up, down), shared, router, x.cpu().numpy(), ROWS, sweep_image=True)
        image_layer.step(defer=False)
        image_same = bool((torch.from_numpy(image_layer.output()) == stage_rows.cpu()).all().item())
        image_eager_ms = image_layer.timed(args.steps, args.warmup, eager=True)
        image_graph_ms = image_layer.timed(args.steps, max(args.warmup, 2))
        image_bytes = sum(t.numel() for t in image_layer.images)
        image_layer.close()
        del image_layer
        if not image_same:
            print("decode step: the sweep image and the canonical rows disagree", file=sys.stderr)
            return 1
        stage_image = MoeLayer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK,
                               qtypes=(qt, qt, qt), routed=(gate, up, down), shared=shared, bias=None,
                               scoring=K.SIGMOID, normalize=True, scaling=1.0, limit=10.0, act_q8=True,
                               max_rows=ROWS, device=dev, sweep_image=True)
        stage_image.fused_prepare = layer.fused_prepare
        for _ in range(args.warmup):
            stage_image.run(x, logits)
        _, _, image_sweeps_ms = stage_timing(stage_image)
        del stage_image
        torch.cuda.empty_cache()
        image = {"entry": "the same execute_rows over DERIVED_BACKEND views built by "
                          "yvex_rocm_moe_derived_layout_plan + yvex_rocm_moe_sweep_image_build_resident",
                 "graph_ms_per_step": round(image_graph_ms, 4), "eager_ms_per_step": round(image_eager_ms, 4),
                 "image_bytes": image_bytes, "canonical_bytes": (EXPERTS + 1) * EXPERT_BYTES,
                 "rows_identical_to_canonical": image_same,
                 "gate_up_sweep_ms": round(image_sweeps_ms["up"][0], 4),
                 "down_sweep_ms": round(image_sweeps_ms["down"][0], 4)}
        if min(image_graph_ms, image_eager_ms) < step_ms:
            step_ms = min(image_graph_ms, image_eager_ms)
            launch_mode = ("execute_rows over the sweep image, " +
                           ("library launch graph" if image_graph_ms <= image_eager_ms else "eager launches") +
                           ", completion deferred to the phase barrier")
            sweeps_ms = image_sweeps_ms
    weight_bytes = (unique + 1) * EXPERT_BYTES
    value = weight_bytes / (step_ms * 1e-3) / 1e9

    # dominant kernel alone, launched exactly as in the step: the gate/up sweep over the routed
    # experts hit plus the shared expert (2/3 of the step's weight bytes)
    pairs = ROWS * TOPK
    acts = layer.act_q8_rows if layer.act_q8 else x

    def up_only():
        K.moe_up(layer.routed, acts, layer.act_q8, layer.weights, layer.worklist, pairs, TOPK,
                 EXPERTS, layer.limit, layer.intermediate_f32, layer.status, shared=layer.shared,
                 shared_rows=ROWS, shared_intermediate=layer.last_shared_mid)

    def down_only():
        mid = layer.intermediate_q8 if layer.act_q8 else layer.intermediate_f32
        smid = layer.last_shared_down_input
        K.moe_down(layer.routed, mid, layer.act_q8, layer.worklist, pairs, EXPERTS,
                   layer.pair_outputs, layer.status, shared=layer.shared, shared_rows=ROWS,
                   shared_intermediate=smid, shared_outputs=layer.shared_out)

    # Launch durations of the two sweeps: inside the timed steps (events before and after the
    # launch on the launch stream; the first completes when the kernel before it has finished),
    # and launched alone back to back for comparison.
    up_ms, up_median_ms = sweeps_ms["up"]
    down_ms, down_median_ms = sweeps_ms["down"]
    up_alone_ms = event_ms(torch, up_only, max(10, args.steps)) if args.alone else None
    down_alone_ms = event_ms(torch, down_only, max(10, args.steps)) if args.alone else None
    up_bytes = (unique + 1) * 2 * 3_784_704   # gate + up of every distinct routed expert and the shared one
    achieved = up_bytes / (up_ms * 1e-3) / 1e9

    if args.calibrate:
        import ctypes as C
        span = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        sink = torch.zeros(1, dtype=torch.int32, device=dev)
        stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        from yvex_amd import load_library
        lib = load_library()
        for _ in range(3):
            lib.yvex_hip_stream_read(C.c_void_p(span.data_ptr()), C.c_uint64(span.numel()),
                                     C.c_void_p(sink.data_ptr()), stream)
            lib.yvex_hip_fill_u32(C.c_void_p(span.data_ptr()), C.c_uint32(7), C.c_uint64(1 << 26), stream)
        torch.cuda.synchronize()

    out = {
        "metric": "IQ2_XXS MoE decode weight GB/s", "value": round(value, 2), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "i8" if layer.act_q8 else "f32",
        "data": "synthetic",
        "config": {"workload": "moe_decode_iq2xxs: hidden 7168, 256 routed + 1 shared experts, "
                               "top-8 sigmoid, expert width 2048, 32 rows",
                   "activations": args.act, "distinct_routed_experts": unique,
                   "max_bucket_population": max_pop, "routed_sweeps": sweeps, "weight_bytes_per_step": weight_bytes},
        "hbm_peak_frac": round(value / HBM_PEAK_GBS, 4),
        "tokens_per_s": round(ROWS / (step_ms * 1e-3), 1),
        "launch": launch_mode,
        "c_abi": {"entry": "yvex_rocm_backend_moe_operations_get()->execute_rows + complete_rows",
                  "graph_ms_per_step": round(abi_graph_ms, 4), "eager_ms_per_step": round(abi_eager_ms, 4),
                  "completed_every_step_ms": round(abi_sync_ms, 4), "kernel_launches": abi_launches,
                  "graph_launches_replays_last_step": graph_facts,
                  "rows_identical_to_stage_harness": abi_same},
        "stage_harness": {"launch": harness_mode, "ms_per_step": round(harness_ms, 4),
                          "eager_ms_per_step": round(eager_ms, 4),
                          "graph_ms_per_step": round(graph_ms, 4) if graph_ms else None,
                          "note": "the same launches from Python with given logits (no router "
                                  "projection); used for the per-kernel timings only"},
        "c_abi_sweep_image": image,
        "roofline": {"bound": "hbm", "kernel": "iq2_sweep_kernel<fused gate/up" +
                                               (", sweep image" if sweeps_ms is not canonical_sweeps_ms else "") +
                                               "> (routed + shared)",
                     "achieved": round(achieved, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     # HBM bytes per launch of this kernel on this workload from the FETCH_SIZE and
                     # WRITE_SIZE counter runs summarised under profiles/ (scaled by the plain
                     # copy kernels of known size in the same runs); null for other settings
                     "traffic": (None if args.act != "q8k" or unique != GATE_UP_TRAFFIC_EXPERTS else
                                 GATE_UP_TRAFFIC_BYTES if sweeps_ms is canonical_sweeps_ms else
                                 GATE_UP_IMAGE_TRAFFIC_BYTES),
                     "launch_ms": round(up_ms, 4), "algorithmic_bytes": up_bytes},
        "kernels_ms": {"gate_up_sweep": round(up_ms, 4), "down_sweep": round(down_ms, 4),
                       "gate_up_sweep_canonical": round(canonical_sweeps_ms["up"][0], 4),
                       "down_sweep_canonical": round(canonical_sweeps_ms["down"][0], 4),
                       "gate_up_sweep_median": round(up_median_ms, 4), "down_sweep_median": round(down_median_ms, 4),
                       "gate_up_sweep_alone": round(up_alone_ms, 4) if up_alone_ms else None,
                       "down_sweep_alone": round(down_alone_ms, 4) if down_alone_ms else None},
    }
    out["clock"] = device_clock(torch, dev)
    if not args.no_dense:
        out["decode_envelope"] = envelope_leg(torch, (gate, up, down), shared, router, dev, args.steps, args.warmup)
        out["decode_small_batches"] = small_batches_leg(torch, (gate, up, down), shared, router, dev,
                                                        args.steps, args.warmup)
    if not args.no_prefill:
        out["prefill"] = prefill_leg(torch, K, MoeLayer, (gate, up, down), shared, dev,
                                     max(3, args.steps // 10), 2)
        out["model_file_layer"] = model_file_layer_leg(torch, gate, up, dev, args.steps, args.warmup)
    if not args.no_prefill:
        # config 4's second weight format: the same layer with Q4_K experts (6.3 GB of them)
        del layer, gate, up, down, shared
        torch.cuda.empty_cache()
        q4_blocks = EXPERTS * INTERMEDIATE * HIDDEN // 256
        q4_routed = tuple(synth_q4k(torch, q4_blocks, dev, 21 + i) for i in range(3))
        q4_shared = tuple(synth_q4k(torch, INTERMEDIATE * HIDDEN // 256, dev, 31 + i) for i in range(3))
        out["prefill_q4k"] = prefill_leg(torch, K, MoeLayer, q4_routed, q4_shared, dev,
                                         max(3, args.steps // 10), 2, qt=K.Q4_K)
        out["decode_q4k"] = decode_q4k_leg(torch, K, q4_routed, q4_shared, dev, args.steps, args.warmup)
        del q4_routed, q4_shared
        torch.cuda.empty_cache()
        layer = gate = up = down = shared = None
    if not args.no_dense:
        del layer, gate, up, down, shared
        torch.cuda.empty_cache()
        out["dense"] = dense_leg(torch, K, dev, 64)
    if not args.no_cpu:
        port = cpu_baseline(args.cpu_rows, 1)
        reference = cpu_baseline_reference(args.cpu_rows)
        out["cpu_baseline"] = reference or port
        if reference:
            out["cpu_baseline_port"] = port
        out["cpu_baseline_all_cores"] = cpu_baseline(max(args.cpu_rows, 8), min(16, os.cpu_count() or 1))
        # The CPU path runs a prefill row exactly as a decode row (top-8 + shared expert FFNs, an
        # expert's bytes decoded again for every row: src/runtime/moe.c:596-632 has no batched
        # form), so the sample above is a sample of the prefill batch too, extrapolated linearly.
        base = out["cpu_baseline"]
        pair_ops = 2 * (2 * INTERMEDIATE * HIDDEN + HIDDEN * INTERMEDIATE)
        for leg in ("prefill", "prefill_q4k"):
            if isinstance(out.get(leg), dict) and "error" not in out[leg]:
                out[leg]["cpu_baseline"] = {
                    "value": round(pair_ops * (TOPK + 1) * base["tokens_per_s"] / 1e12, 6), "unit": "TOP/s",
                    "tokens_per_s": round(base["tokens_per_s"], 4), "cores": base["cores"], "kind": base["kind"],
                    "sample": base["sample"] + " (IQ2_XXS experts); a 2048-row batch is 2048 such rows, "
                              "extrapolated linearly",
                    "extrapolated_step_seconds": round(2048 / base["tokens_per_s"], 1)}
        if isinstance(out.get("dense"), dict):
            out["dense"]["cpu_baseline"] = cpu_baseline_dense()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
