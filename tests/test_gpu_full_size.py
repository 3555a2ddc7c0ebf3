"""The decode layer at its full size (hidden 7168, 256 routed + 1 shared IQ2_XXS experts of width
2048, top-8 sigmoid routing, 32 rows, Q8_K activations): properties that do not need the CPU path
over the whole batch, and the CPU oracle on two of the rows.

  * the same batch twice gives the same bits;
  * a row's result does not depend on the batch it arrives in (halves of the batch and a single
    row against the full batch, bit for bit): the sweeps group pairs by expert, four to a sweep,
    so the grouping changes with the batch while every pair's arithmetic must not;
  * routing equals the oracle's for every row, and eight rows' outputs equal the oracle's
    (src/graph/moe.c:497-622, src/runtime/moe.c:596-645) bit for bit, stage by stage and end to
    end: the kernels form the same float term per superblock as the CPU path and add a row's
    terms in double in block order, so every bfloat16 rounding sees the same value.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

HIDDEN, INTERMEDIATE, EXPERTS, TOPK, ROWS = 7168, 2048, 256, 8, 32


def synthetic_iq2xxs(blocks, device, seed):
    """Uniform grid / sign / scale bytes with a small positive fp16 block scale."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    raw = torch.randint(0, 256, (blocks, 66), dtype=torch.uint8, device=device, generator=gen)
    d = (torch.rand(blocks, device=device, generator=gen) * 3.5e-4 + 1.0e-4).to(torch.float16)
    raw[:, :2] = d.view(torch.uint8).reshape(blocks, 2)
    return raw.reshape(-1)


@pytest.fixture(scope="module")
def layer_weights(gpu):
    blocks = EXPERTS * INTERMEDIATE * HIDDEN // 256
    routed = tuple(synthetic_iq2xxs(blocks, gpu, 1 + i) for i in range(3))
    shared = tuple(synthetic_iq2xxs(INTERMEDIATE * HIDDEN // 256, gpu, 10 + i) for i in range(3))
    return routed, shared


def stage_by_stage(oracle, layer, routed, x, picked, label, qt=None):
    """The picked rows' pairs stage by stage: SwiGLU products against the oracle's, expert outputs
    against the oracle fed with the device's own products. Every value must equal the CPU path's."""
    qt = oracle.IQ2_XXS if qt is None else qt
    gate, up, down = (t.cpu().numpy() for t in routed)
    gb = oracle.row_bytes(qt, HIDDEN) * INTERMEDIATE
    db = oracle.row_bytes(qt, INTERMEDIATE) * HIDDEN
    sel = layer.selected.cpu().numpy().reshape(-1)
    wts = layer.weights.cpu().numpy().reshape(-1)
    order = layer.worklist.order.cpu().numpy()[:sel.size]
    position_of = np.empty_like(order)
    position_of[order] = np.arange(order.size)
    mid_bad = mid_all = out_bad = out_all = 0
    for row in picked:
        for rank in range(TOPK):
            source = row * TOPK + rank
            e = int(sel[source])
            mid = layer.intermediate_f32[int(position_of[source])].cpu().numpy()
            rc, _, want_mid, _ = oracle.moe_expert((qt, qt, qt), gate[e * gb:(e + 1) * gb], up[e * gb:(e + 1) * gb],
                                                   down[e * db:(e + 1) * db], HIDDEN, INTERMEDIATE,
                                                   x[row].cpu().numpy(), float(wts[source]), act_q8=True)
            assert rc == 0
            mid_bad += int((mid != want_mid).sum())
            mid_all += mid.size
            raw = oracle.q8_matvec(qt, down[e * db:(e + 1) * db], HIDDEN, INTERMEDIATE, oracle.q8k_quantize(mid), 1)[0]
            want_out = np.array([oracle.lib().yvo_bf16_round(np.float32(v)) for v in raw], np.float32)
            got_out = layer.pair_outputs[source].cpu().numpy()
            out_bad += int((got_out != want_out).sum())
            out_all += got_out.size
    print(f"{label}: {mid_bad} of {mid_all} SwiGLU products and {out_bad} of {out_all} expert outputs "
          f"differ from the oracle's")
    assert mid_bad == 0 and out_bad == 0


def equal_to_oracle(got, want, label):
    """North star: final fp32 outputs within 1e-3 relative / 1e-5 absolute of the CPU path; the
    kernels are held to more, every output the CPU path's bit for bit."""
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    outside = err > 1e-5 + 1e-3 * np.abs(want)
    print(f"{label}: {int(outside.sum())} of {outside.size} outputs beyond 1e-3 / 1e-5, "
          f"bit-identical {np.mean(got == want):.6f}")
    assert np.all(err <= 1e-5 + 1e-3 * np.abs(want))
    assert np.array_equal(got, want)


def test_decode_layer_at_full_size(gpu, oracle, layer_weights):
    from yvex_amd import kernels as K
    from yvex_amd.moe import MoeLayer
    routed, shared = layer_weights
    gen = torch.Generator(device=gpu)
    gen.manual_seed(42)
    x = torch.randn((ROWS, HIDDEN), device=gpu, generator=gen)
    logits = torch.randn((ROWS, EXPERTS), device=gpu, generator=gen)
    qt = K.IQ2_XXS
    layer = MoeLayer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK, qtypes=(qt, qt, qt),
                     routed=routed, shared=shared, scoring=K.SIGMOID, normalize=True, scaling=1.0, limit=10.0,
                     act_q8=True, max_rows=ROWS, device=gpu)

    def run(rows_from, rows_to):
        out = layer.run(x[rows_from:rows_to].contiguous(), logits[rows_from:rows_to].contiguous())
        torch.cuda.synchronize()
        assert int(layer.status.item()) == 0
        return out[:rows_to - rows_from].clone(), layer.selected.clone(), layer.weights.clone()

    full, selected, weights = run(0, ROWS)
    again, _, _ = run(0, ROWS)
    assert torch.equal(full.view(torch.int32), again.view(torch.int32))
    assert torch.isfinite(full).all() and float(full.abs().max()) > 0.0
    for lo, hi in ((0, 16), (16, 32), (5, 6), (29, 32)):
        part, part_selected, _ = run(lo, hi)
        assert torch.equal(part_selected, selected[lo:hi])
        assert torch.equal(part.view(torch.int32), full[lo:hi].view(torch.int32)), (lo, hi)

    # routing of every row against the oracle
    host_logits = logits.cpu().numpy()
    for r in range(ROWS):
        rc, want_selected, want_weights, _ = oracle.moe_route(host_logits[r], None, TOPK, oracle.SIGMOID, True, 1.0)
        assert rc == 0
        assert np.array_equal(selected[r].cpu().numpy().astype(np.uint64), want_selected)
        assert np.array_equal(weights[r].cpu().numpy(), want_weights)

    # eight rows through the CPU oracle with the same weights
    picked = [0, 4, 9, 13, 17, 22, 26, 31]
    want = oracle.moe_layer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK,
                            qtypes=(oracle.IQ2_XXS,) * 3, routed=[t.cpu().numpy() for t in routed],
                            shared=[t.cpu().numpy() for t in shared], inputs=x[picked].cpu().numpy(),
                            logits=host_logits[picked], scoring=oracle.SIGMOID, normalize=True, scaling=1.0,
                            limit=10.0, act_q8=True, threads=16)
    got = full[picked].cpu().numpy()
    assert np.array_equal(selected[picked].cpu().numpy().astype(np.uint64), want["selected"])
    equal_to_oracle(got, want["combined"], "decode layer, 8 rows against the oracle")
    full_again, _, _ = run(0, ROWS)     # leaves the whole batch's stage buffers in place
    stage_by_stage(oracle, layer, routed, x, picked, "decode layer, 8 rows stage by stage")


def synthetic_q4k(blocks, device, seed):
    """Uniform scale, minimum and nibble bytes with small positive fp16 d and dmin."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    raw = torch.randint(0, 256, (blocks, 144), dtype=torch.uint8, device=device, generator=gen)
    d = (torch.rand(blocks, device=device, generator=gen) * 1.0e-4 + 2.0e-5).to(torch.float16)
    raw[:, 0:2] = d.view(torch.uint8).reshape(blocks, 2)
    raw[:, 2:4] = raw[:, 0:2]
    return raw.reshape(-1)


@pytest.mark.parametrize("qtype", ["IQ2_XXS", "Q4_K"])
def test_prefill_layer_at_full_size(gpu, oracle, layer_weights, qtype):
    """2048 rows whose experts follow a Zipf(1.1) popularity (buckets from a handful of pairs to
    more than a thousand) through the matrix-core kernels, with IQ2_XXS and with Q4_K experts: the
    same bits twice, the first 32 rows against the decode sweeps' result for them (bit for bit:
    both add a row's terms as the CPU path does), four rows against the oracle, stage by stage
    and end to end, for equality."""
    from yvex_amd import kernels as K
    from yvex_amd.moe import MoeLayer
    if qtype == "IQ2_XXS":
        routed, shared = layer_weights
    else:
        blocks = EXPERTS * INTERMEDIATE * HIDDEN // 256
        routed = tuple(synthetic_q4k(blocks, gpu, 21 + i) for i in range(3))
        shared = tuple(synthetic_q4k(INTERMEDIATE * HIDDEN // 256, gpu, 31 + i) for i in range(3))
    rows = 2048
    gen = torch.Generator(device=gpu)
    gen.manual_seed(7)
    x = torch.randn((rows, HIDDEN), device=gpu, generator=gen)
    rank = torch.randperm(EXPERTS, device=gpu, generator=gen).float() + 1.0
    uniform = torch.rand((rows, EXPERTS), device=gpu, generator=gen).clamp_(1e-9, 1.0 - 1e-9)
    logits = rank.pow(-1.1).log()[None, :] - (-uniform.log()).log()      # Gumbel top-k over log-popularity
    qt = getattr(K, qtype)
    common = dict(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK, qtypes=(qt, qt, qt),
                  routed=routed, shared=shared, scoring=K.SIGMOID, normalize=True, scaling=1.0, limit=10.0,
                  act_q8=True, device=gpu)
    wide = MoeLayer(max_rows=rows, matrix_cores=True, **common)
    first = wide.run(x, logits)[:rows].clone()
    torch.cuda.synchronize()
    assert int(wide.status.item()) == 0
    second = wide.run(x, logits)[:rows].clone()
    torch.cuda.synchronize()
    assert torch.equal(first.view(torch.int32), second.view(torch.int32))
    assert torch.isfinite(first).all()
    selected = wide.selected.clone()
    picked = [5, 700, 1000, 1900]
    stage_by_stage(oracle, wide, routed, x, picked, f"prefill layer ({qtype}), 4 rows stage by stage",
                   getattr(oracle, qtype))
    keep = list(range(32)) + picked
    populations = torch.bincount(selected.reshape(-1).long(), minlength=EXPERTS).cpu().numpy()
    assert populations.max() > 1000 and (populations[populations > 0] < 32).any()
    print("bucket populations of the experts of the rows checked against the oracle:",
          [sorted(populations[selected[r].cpu().numpy().astype(np.int64)].tolist()) for r in picked])
    wide_pairs = wide.pair_outputs.view(rows, TOPK, HIDDEN)[keep].cpu().numpy()    # [row, rank, column]
    wide_shared = wide.shared_out[keep].cpu().numpy()
    del wide

    narrow = MoeLayer(max_rows=32, **common)
    sweeps = narrow.run(x[:32].contiguous(), logits[:32].contiguous())[:32].clone()
    torch.cuda.synchronize()
    assert int(narrow.status.item()) == 0 and torch.equal(narrow.selected, selected[:32])
    # expert by expert, then the combined rows: the two kernel families agree bit for bit
    mine = wide_pairs[:32].reshape(32 * TOPK, HIDDEN)
    assert np.array_equal(mine, narrow.pair_outputs[:32 * TOPK].cpu().numpy())
    assert np.array_equal(wide_shared[:32], narrow.shared_out[:32].cpu().numpy())
    assert np.array_equal(first[:32].cpu().numpy(), sweeps.cpu().numpy())
    want = oracle.moe_layer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK,
                            qtypes=(getattr(oracle, qtype),) * 3, routed=[t.cpu().numpy() for t in routed],
                            shared=[t.cpu().numpy() for t in shared], inputs=x[picked].cpu().numpy(),
                            logits=logits[picked].cpu().numpy(), scoring=oracle.SIGMOID, normalize=True,
                            scaling=1.0, limit=10.0, act_q8=True, threads=16)
    assert np.array_equal(selected[picked].cpu().numpy().astype(np.uint64), want["selected"])
    equal_to_oracle(first[picked].cpu().numpy(), want["combined"],
                    f"prefill layer ({qtype}), 4 rows against the oracle")


# ---- the same comparisons on the product entry: execute_rows + complete_rows ----------------------

def router_weights(device, seed):
    """F32 router rows whose projection of N(0, 1) rows gives logits of unit size."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    return torch.randn((EXPERTS, HIDDEN), device=device, generator=gen) * HIDDEN ** -0.5


def synthetic_q2k(blocks, device, seed):
    """Q2_K superblocks (84 bytes): random scale | minimum << 4 bytes and 2-bit codes, small positive
    fp16 d and dmin behind them."""
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    raw = torch.randint(0, 256, (blocks, 84), dtype=torch.uint8, device=device, generator=gen)
    scales = (torch.rand((blocks, 2), device=device, generator=gen) * 1e-3 + 1e-4).to(torch.float16)
    raw[:, 80:84] = scales.view(torch.uint8).reshape(-1, 4)
    return raw.reshape(-1)


@pytest.mark.parametrize("rows,qtype,sweep_image", [(32, "IQ2_XXS", False), (32, "IQ2_XXS", True),
                                                    (2048, "IQ2_XXS", False), (2048, "Q4_K", False),
                                                    # the pairing of the reference's model file: Q2_K down experts
                                                    (32, "IQ2_XXS+Q2_K", True), (2048, "IQ2_XXS+Q2_K", False)])
def test_execute_rows_at_full_size_equals_the_cpu_layer(gpu, oracle, layer_weights, rows, qtype, sweep_image):
    """BASELINE configs 3 and 4 through yvex_rocm_backend_moe_operations_get()->execute_rows and
    complete_rows (the reference's row-batch entry, src/backend/cuda/moe.c:1826-1958), router
    projection included: 32 rows take the decode sweeps (over canonical bytes and over the sweep
    image), 2048 rows the matrix-core kernels (IQ2_XXS and Q4_K experts). Picked rows are the CPU
    layer's bit for bit: router logits from the CPU row dot, then src/graph/moe.c:497-622 and
    src/runtime/moe.c:596-632 on Q8_K activations. A second call gives the same bits, and the
    facts say which kernels ran."""
    from yvex_amd import abi
    from yvex_amd import kernels as K
    from yvex_amd.host import RowBatchLayer
    down_qtype = None
    if qtype == "IQ2_XXS":
        routed, shared = layer_weights
    elif qtype == "IQ2_XXS+Q2_K":
        qtype, down_qtype = "IQ2_XXS", "Q2_K"
        routed, shared = layer_weights
        routed = routed[:2] + (synthetic_q2k(EXPERTS * INTERMEDIATE * HIDDEN // 256, gpu, 41),)
        shared = shared[:2] + (synthetic_q2k(INTERMEDIATE * HIDDEN // 256, gpu, 42),)
    else:
        blocks = EXPERTS * INTERMEDIATE * HIDDEN // 256
        routed = tuple(synthetic_q4k(blocks, gpu, 21 + i) for i in range(3))
        shared = tuple(synthetic_q4k(INTERMEDIATE * HIDDEN // 256, gpu, 31 + i) for i in range(3))
    gen = torch.Generator(device=gpu)
    gen.manual_seed(rows)
    x = torch.randn((rows, HIDDEN), device=gpu, generator=gen)
    router = router_weights(gpu, 5)
    qt = getattr(K, qtype)
    layer = RowBatchLayer(torch, routed, shared, router, x.cpu().numpy(), rows, hidden=HIDDEN,
                          intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK, qtype=qt, sweep_image=sweep_image,
                          down_qtype=getattr(K, down_qtype) if down_qtype else None)
    try:
        layer.step(defer=True)
        layer.complete()
        assert layer.done.completed == 1
        first = layer.output().copy()
        layer.step(defer=False)
        assert layer.result.completed == 1 and layer.result.row_expert_pairs == rows * TOPK
        assert np.array_equal(first.view(np.uint32), layer.output().view(np.uint32))
        matrix_cores = layer.result.tensor_core_launches > 0
        assert matrix_cores == (rows == 2048)
    finally:
        layer.close()
    assert np.isfinite(first).all() and np.abs(first).max() > 0.0
    picked = [0, 4, 9, 13, 17, 22, 26, 31] if rows == 32 else [5, 700, 1000, 1900]
    host_x = x[picked].cpu().numpy()
    logits = oracle.matvec(oracle.F32, router.cpu().numpy().view(np.uint8).reshape(-1), EXPERTS, HIDDEN, host_x)
    want = oracle.moe_layer(hidden=HIDDEN, intermediate=INTERMEDIATE, experts=EXPERTS, topk=TOPK,
                            qtypes=(getattr(oracle, qtype),) * 2 + (getattr(oracle, down_qtype or qtype),),
                            routed=[t.cpu().numpy() for t in routed],
                            shared=[t.cpu().numpy() for t in shared], inputs=host_x, logits=logits,
                            scoring=oracle.SIGMOID, normalize=True, scaling=1.0, limit=10.0, act_q8=True,
                            threads=16)
    equal_to_oracle(first[picked], want["combined"],
                    f"execute_rows, {rows} rows, {qtype}{' + Q2_K down' if down_qtype else ''}"
                    f"{' (sweep image)' if sweep_image else ''}: picked rows against the oracle")
