#!/usr/bin/env python3
"""Write tests/golden/reference_vectors.npz from the library compiled out of the reference's own
C sources (oracle/_ref/libyvex_ref.so, built by oracle/Makefile where /root/reference exists).

The fixture holds inputs and the reference's outputs only: random packed blocks with their decoded
floats, encoded rows with their CPU row dots, router logits with selections and weights, and small
expert FFNs with their outputs. tests/test_oracle_pinning.py replays them against the restatement,
so the oracle stays pinned on machines where the reference tree (and so oracle/_ref) is absent.

    python tests/golden/make_golden.py
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from yvex_amd import abi  # noqa: E402  (structure layouts follow the reference's headers)


class RouterResult(C.Structure):
    _fields_ = [("selected_count", abi.ULL), ("selected_experts", abi.ULL * 16),
                ("router_logits", C.c_float * 256), ("router_scores", C.c_float * 256),
                ("selected_weights", C.c_float * 16)]


def ref_decode(ref, qtype, blob, block_bytes, block_size):
    blocks = blob.size // block_bytes
    out = np.zeros((blocks, block_size), np.float32)
    failure, err = (C.c_ubyte * 512)(), abi.Error()
    ref.yvex_quant_decode_block.argtypes = [C.c_uint, C.c_void_p, C.c_size_t, C.c_void_p, abi.ULL,
                                            C.c_void_p, C.c_void_p]
    for b in range(blocks):
        rc = ref.yvex_quant_decode_block(qtype, blob.ctypes.data + b * block_bytes, block_bytes,
                                         out[b].ctypes.data, block_size, failure, C.byref(err))
        assert rc == 0, (qtype, b, err.message)
    return out


def ref_dot(ref, qtype, row, x):
    out, failure, err = C.c_float(), (C.c_ubyte * 512)(), abi.Error()
    ref.yvex_quant_cpu_dot.argtypes = [C.c_uint, C.c_void_p, C.c_size_t, C.c_void_p, abi.ULL,
                                       C.c_void_p, C.c_void_p, C.c_void_p]
    rc = ref.yvex_quant_cpu_dot(qtype, row.ctypes.data, row.size, x.ctypes.data, x.size,
                                C.byref(out), failure, C.byref(err))
    assert rc == 0, err.message
    return out.value


def weight_view(blob, qtype, width, rows):
    v = abi.WeightView()
    v.qtype = qtype
    v.encoded, v.encoded_bytes = blob.ctypes.data, blob.nbytes
    v.row_width, v.row_count, v.row_bytes = width, rows, blob.nbytes // rows
    return v


def main():
    oracle.build()
    ref = oracle.ref_lib()
    if ref is None:
        sys.exit("oracle/_ref/libyvex_ref.so is not available: the reference tree is absent")
    out = {}
    # scalar conversions
    ref.yvex_quant_f16_decode.restype = C.c_float
    ref.yvex_quant_f16_decode.argtypes = [C.c_ushort]
    ref.yvex_quant_f16_encode.restype = C.c_ushort
    ref.yvex_quant_f16_encode.argtypes = [C.c_float]
    ref.yvex_quant_bf16_encode.restype = C.c_ushort
    ref.yvex_quant_bf16_encode.argtypes = [C.c_float]
    # every 7th binary16 code plus all subnormals and specials (the full table compresses badly)
    codes = np.unique(np.concatenate([np.arange(0, 65536, 7), np.arange(0, 1100),
                                      np.arange(0x7bf0, 0x7c10), np.arange(0x8000, 0x8410),
                                      np.arange(0xfbf0, 0xfc10)])).astype(np.uint16)
    out["f16_codes"] = codes
    out["f16_decode_bits"] = np.array([ref.yvex_quant_f16_decode(int(b)) for b in codes],
                                      np.float32).view(np.uint32)
    g = oracle.Generator(42, "golden.scalars")
    samples = np.concatenate([g.normal(3000, 1.0), g.normal(500, 1e-6), g.normal(500, 3e4),
                              np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6.1e-5, 5.96e-8,
                                        1.00048828125, 1.00146484375], np.float32)]).astype(np.float32)
    out["scalar_samples"] = samples
    out["f16_encode"] = np.array([ref.yvex_quant_f16_encode(float(v)) for v in samples], np.uint16)
    out["bf16_encode"] = np.array([ref.yvex_quant_bf16_encode(float(v)) for v in samples], np.uint16)
    # block decoders and row dots
    for name, qtype in (("q8_0", oracle.Q8_0), ("q2_k", oracle.Q2_K), ("iq2_xxs", oracle.IQ2_XXS)):
        block, nbytes = oracle.geometry(qtype)
        gen = oracle.Generator(42, f"golden.{name}")
        width = 512
        rows = 4
        blob = gen.weights(qtype, rows, width)
        x = gen.normal(width)
        out[f"{name}_blob"] = blob
        out[f"{name}_decoded_bits"] = ref_decode(ref, qtype, blob, nbytes, block).view(np.uint32)
        out[f"{name}_x"] = x
        rb = width // block * nbytes
        out[f"{name}_dots_bits"] = np.array(
            [ref_dot(ref, qtype, blob[r * rb:(r + 1) * rb], x) for r in range(rows)],
            np.float32).view(np.uint32)
    # router (sqrt-softplus is the reference's only policy)
    gen = oracle.Generator(42, "golden.router")
    experts, hidden, topk = 64, 32, 6
    router = gen.normal(experts * hidden, 0.3)
    bias = (gen.normal(experts) * 0.2).astype(np.float32)
    xs = gen.normal(5 * hidden).reshape(5, hidden)
    plan = abi.LayerPlan()
    plan.hidden_width, plan.routed_experts, plan.experts_per_token = hidden, experts, topk
    plan.routed_scaling_factor, plan.normalize_topk_probabilities = 1.5, 1
    plan.router_class = abi.ROUTER_LEARNED
    job = abi.LayerJob()
    job.layer = C.pointer(plan)
    job.weights[abi.W_ROUTER] = weight_view(router.view(np.uint8), 0, hidden, experts)
    job.weights[abi.W_ROUTER_BIAS] = weight_view(bias.view(np.uint8), 0, experts, 1)
    ref.yvex_moe_route_cpu.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    sel, wts, logits = [], [], []
    for row in xs:
        result, err = RouterResult(), abi.Error()
        assert ref.yvex_moe_route_cpu(C.byref(job), row.ctypes.data, C.byref(result), C.byref(err)) == 0
        sel.append(list(result.selected_experts)[:topk])
        wts.append(list(result.selected_weights)[:topk])
        logits.append(list(result.router_logits)[:experts])
    out["route_logits"] = np.array(logits, np.float32)
    out["route_bias"] = bias
    out["route_selected"] = np.array(sel, np.uint64)
    out["route_weights_bits"] = np.array(wts, np.float32).view(np.uint32)
    # hash router: the token's row of an I32 table names the experts (same job, same logits)
    table = np.stack([np.random.default_rng(t).permutation(experts)[:topk] for t in range(8)]).astype(np.int32)
    plan.router_class, plan.hash_table_rows, plan.hash_table_columns = abi.ROUTER_HASH, 8, topk
    job.weights[abi.W_ROUTER_TABLE] = weight_view(table.view(np.uint8), 26, topk, 8)
    job.token_id_present = 1
    hash_sel, hash_wts = [], []
    for row, token in zip(xs, (3, 7, 0, 5, 2)):
        result, err = RouterResult(), abi.Error()
        job.token_id = token
        assert ref.yvex_moe_route_cpu(C.byref(job), row.ctypes.data, C.byref(result), C.byref(err)) == 0
        hash_sel.append(list(result.selected_experts)[:topk])
        hash_wts.append(list(result.selected_weights)[:topk])
    out["route_hash_table"] = table
    out["route_hash_tokens"] = np.array([3, 7, 0, 5, 2], np.uint32)
    out["route_hash_selected"] = np.array(hash_sel, np.uint64)
    out["route_hash_weights_bits"] = np.array(hash_wts, np.float32).view(np.uint32)
    plan.router_class = abi.ROUTER_LEARNED
    # expert FFN on IQ2_XXS and Q8_0 weights
    ref.yvex_moe_expert_cpu.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_float, C.c_void_p, C.c_void_p]
    for name, qtype in (("iq2_xxs", oracle.IQ2_XXS), ("q8_0", oracle.Q8_0)):
        gen = oracle.Generator(42, f"golden.expert.{name}")
        hidden, inter = (256, 256) if name == "iq2_xxs" else (128, 64)
        gate, up = gen.weights(qtype, inter, hidden), gen.weights(qtype, inter, hidden)
        down = gen.weights(qtype, hidden, inter)
        x = gen.normal(hidden)
        if name == "iq2_xxs":
            x *= 40.0     # drive some gate/up values past the activation limit
        plan = abi.LayerPlan()
        plan.hidden_width, plan.activation_limit = hidden, 10.0
        views = [weight_view(gate, qtype, hidden, inter), weight_view(up, qtype, hidden, inter),
                 weight_view(down, qtype, inter, hidden)]
        y, err = np.zeros(hidden, np.float32), abi.Error()
        rc = ref.yvex_moe_expert_cpu(C.byref(plan), C.byref(views[0]), C.byref(views[1]),
                                     C.byref(views[2]), x.ctypes.data, C.c_float(0.25),
                                     y.ctypes.data, C.byref(err))
        assert rc == 0, err.message
        out[f"expert_{name}_gate"], out[f"expert_{name}_up"] = gate, up
        out[f"expert_{name}_down"], out[f"expert_{name}_x"] = down, x
        out[f"expert_{name}_out_bits"] = y.view(np.uint32)
    # residual-stream ingress in front of the experts: mixes, Sinkhorn, weighted RMS norm
    ref.yvex_moe_ffn_prepare_cpu.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
    for name, streams, width, iterations, tokens in (("wide", 4, 64, 20, 3), ("single", 1, 32, 1, 2)):
        gen = oracle.Generator(42, f"golden.ingress.{name}")
        mixing, expanded = (streams + 2) * streams, streams * width
        function = gen.normal(mixing * expanded, 0.2)
        scale = gen.normal(3, 0.7)
        base = gen.normal(mixing, 0.5)
        norm_bits = ((1.0 + gen.normal(width, 0.2)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        rows = np.round(gen.normal(tokens * expanded) * 64.0) / 64.0     # multiples of 1/64
        rows = rows.astype(np.float32).reshape(tokens, expanded)
        plan = abi.LayerPlan()
        plan.hidden_width, plan.residual_streams, plan.expanded_width = width, streams, expanded
        plan.mhc_mixing_rows, plan.mhc_sinkhorn_iterations = mixing, iterations
        plan.rms_epsilon, plan.mhc_epsilon, plan.mhc_post_multiplier = 1e-6, 1e-6, 2.0
        job = abi.LayerJob()
        job.layer = C.pointer(plan)
        job.weights[abi.W_MHC_FUNCTION] = weight_view(function.view(np.uint8), 0, expanded, mixing)
        job.weights[abi.W_MHC_SCALE] = weight_view(scale.view(np.uint8), 0, 3, 1)
        job.weights[abi.W_MHC_BASE] = weight_view(base.view(np.uint8), 0, mixing, 1)
        job.weights[abi.W_FFN_NORM] = weight_view(norm_bits.view(np.uint8), 30, width, 1)
        normalized = np.zeros((tokens, width), np.float32)
        post = np.zeros((tokens, streams), np.float32)
        comb = np.zeros((tokens, streams * streams), np.float32)
        for t in range(tokens):
            err = abi.Error()
            job.expanded_input = rows[t].ctypes.data
            rc = ref.yvex_moe_ffn_prepare_cpu(C.byref(job), normalized[t].ctypes.data, post[t].ctypes.data,
                                              comb[t].ctypes.data, C.byref(err))
            assert rc == 0, err.message
        out[f"ingress_{name}_function"], out[f"ingress_{name}_scale"] = function, scale
        out[f"ingress_{name}_base"], out[f"ingress_{name}_norm_bf16"] = base, norm_bits
        out[f"ingress_{name}_rows"] = rows
        out[f"ingress_{name}_normalized_bits"] = normalized.view(np.uint32)
        out[f"ingress_{name}_post_bits"] = post.view(np.uint32)
        out[f"ingress_{name}_combination_bits"] = comb.view(np.uint32)
    # ---- derived expert storage: src/backend/cuda/layout.c:95-167 --------------------------------
    ref.yvex_cuda_moe_derived_layout_plan.argtypes = [C.c_void_p, C.POINTER(abi.ULL), C.c_void_p]
    ref.yvex_cuda_moe_derived_layout_build.argtypes = [C.c_void_p, C.c_void_p, abi.ULL, C.c_void_p, abi.ULL,
                                                       C.c_void_p]
    for name, qtype, block_bytes, experts, rows_per_expert, width in (
            ("iq2_xxs", oracle.IQ2_XXS, 66, 3, 5, 512), ("q2_k", oracle.Q2_K, 84, 2, 6, 768)):
        rows = experts * rows_per_expert
        canonical = oracle.Generator(42, f"golden.layout.{name}").bytes(rows * (width // 256) * block_bytes)
        decision = abi.ExecutionDecision()
        decision.expert_count, decision.canonical_qtype = experts, qtype
        decision.canonical_row_width, decision.canonical_row_count = width, rows
        decision.encoded_bytes, decision.consumer = canonical.size, abi.CONSUMER_ROUTED_GATE_UP
        decision.layout, decision.derived_asset_required = abi.LAYOUT_DERIVED, 1
        storage, err = abi.ULL(), abi.Error()
        assert ref.yvex_cuda_moe_derived_layout_plan(C.byref(decision), C.byref(storage), C.byref(err)) == 0
        derived = np.full(storage.value, 0xA5, np.uint8)
        rc = ref.yvex_cuda_moe_derived_layout_build(C.byref(decision), canonical.ctypes.data, canonical.size,
                                                    derived.ctypes.data, derived.size, C.byref(err))
        assert rc == 0, err.message
        out[f"layout_{name}_shape"] = np.array([qtype, experts, rows, width], np.uint64)
        out[f"layout_{name}_canonical"], out[f"layout_{name}_derived"] = canonical, derived
    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
