"""Stage-by-stage parity of the decode-width MoE layer against the CPU oracle."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

BF16_ULP = 2.0 ** -7   # spacing relative to the value's binade is at most this


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def bf16_flip_report(got, want):
    """Elements that differ are either inside the path's fp32 tolerance (1e-3 rel / 1e-5 abs:
    sums that cancel to almost nothing) or exactly one bf16 step away, which happens when the
    unrounded value sits on a rounding boundary. Returns the fraction of one-step elements."""
    got = np.asarray(got, np.float32)
    want = np.asarray(want, np.float32)
    err = np.abs(got.astype(np.float64) - want)
    outside = err > 1e-5 + 1e-3 * np.abs(want)
    if outside.any():
        step = err[outside] / np.abs(want[outside]).astype(np.float64)
        assert np.all(step <= BF16_ULP * 1.001), f"worst relative step {step.max()}"
    return outside.mean()


def make_layer(oracle, gpu, *, hidden, intermediate, experts, topk, rows, qtype, act_q8, scoring,
               seed=42, shared=True, matrix_cores=False, sweep_image=False):
    from yvex_amd.moe import MoeLayer
    qt = getattr(oracle, qtype)
    g = oracle.Generator(seed, f"moe.{qtype}.{hidden}.{intermediate}.{experts}")
    gate = g.weights(qt, experts * intermediate, hidden)
    up = g.weights(qt, experts * intermediate, hidden)
    down = g.weights(qt, experts * hidden, intermediate)
    sh = None
    if shared:
        sh = (g.weights(qt, intermediate, hidden), g.weights(qt, intermediate, hidden),
              g.weights(qt, hidden, intermediate))
    x = g.normal(rows * hidden).reshape(rows, hidden)
    logits = g.normal(rows * experts).reshape(rows, experts)
    bias = (g.normal(experts) * 0.05).astype(np.float32)
    layer = MoeLayer(hidden=hidden, intermediate=intermediate, experts=experts, topk=topk,
                     qtypes=(qt, qt, qt), routed=tuple(dev(t, gpu) for t in (gate, up, down)),
                     shared=tuple(dev(t, gpu) for t in sh) if sh else None, bias=dev(bias, gpu),
                     scoring=scoring, normalize=True, scaling=1.5, limit=10.0, act_q8=act_q8,
                     max_rows=rows, device=gpu, matrix_cores=matrix_cores, sweep_image=sweep_image)
    host = dict(qt=qt, gate=gate, up=up, down=down, shared=sh, x=x, logits=logits, bias=bias)
    return layer, host


@pytest.mark.parametrize("qtype,hidden,intermediate,experts,topk,rows,act_q8,scoring,matrix_cores", [
    ("IQ2_XXS", 512, 256, 8, 2, 7, True, 0, False),
    ("IQ2_XXS", 1024, 512, 16, 4, 9, False, 1, False),
    ("Q4_K", 512, 512, 8, 3, 6, True, 1, False),
    ("Q8_0", 512, 256, 6, 2, 5, True, 0, False),
    ("Q2_K", 768, 256, 6, 2, 5, True, 0, False),
    ("IQ2_XXS", 7168, 2048, 12, 4, 6, True, 1, False),
    # specialised IQ2_XXS sweeps: four rows per iteration with buckets past four pairs; two rows
    # per iteration over a down projection whose rows end inside a 16-lane group
    ("IQ2_XXS", 2048, 2048, 6, 4, 20, True, 1, False),
    ("IQ2_XXS", 4096, 3072, 4, 2, 5, True, 0, False),
    # Q4_K rows through the specialised sweeps: four rows per iteration with buckets past four
    # pairs, real widths (56 lanes a row), two rows per iteration
    ("Q4_K", 2048, 2048, 6, 4, 20, True, 1, False),
    ("Q4_K", 7168, 2048, 12, 4, 6, True, 0, False),
    ("Q4_K", 4096, 3072, 4, 2, 5, True, 0, False),
    # Q2_K rows: the down projection through the specialised sweeps (gate and up rows of this
    # format take the generic kernel), buckets past four pairs, one and four rows an iteration
    ("Q2_K", 2048, 2048, 6, 4, 20, True, 1, False),
    ("Q2_K", 4096, 3072, 4, 2, 5, True, 0, False),
    # many buckets: more sweeps than one wavefront lists (the class list is built by several)
    ("IQ2_XXS", 2048, 2048, 200, 8, 40, True, 1, False),
    # row-batch kernels on the matrix cores: tiny buckets, buckets past one 128-pair tile, real widths
    ("IQ2_XXS", 512, 256, 8, 2, 7, True, 0, True),
    ("IQ2_XXS", 768, 512, 4, 2, 300, True, 1, True),
    ("IQ2_XXS", 7168, 2048, 12, 4, 10, True, 1, True),
    # five superblocks per row (steps past the end of a row, rows that start on 2-byte boundaries)
    # with 32-pair tiles; three superblocks with 64-pair tiles
    ("IQ2_XXS", 1280, 256, 4, 2, 40, True, 1, True),
    ("IQ2_XXS", 768, 768, 4, 2, 100, True, 0, True),
    # Q4_K experts on the matrix cores: tiny buckets, buckets of several 32-pair tiles, real
    # widths, five superblocks a row (the four waves of a tile get two, one, one, one)
    ("Q4_K", 512, 512, 8, 3, 6, True, 1, True),
    ("Q4_K", 768, 512, 4, 2, 300, True, 0, True),
    ("Q4_K", 7168, 2048, 12, 4, 10, True, 1, True),
    ("Q4_K", 1280, 256, 4, 2, 40, True, 1, True),
])
def test_moe_layer_stagewise(gpu, oracle, qtype, hidden, intermediate, experts, topk, rows, act_q8,
                             scoring, matrix_cores):
    layer, h = make_layer(oracle, gpu, hidden=hidden, intermediate=intermediate, experts=experts,
                          topk=topk, rows=rows, qtype=qtype, act_q8=act_q8, scoring=scoring,
                          matrix_cores=matrix_cores)
    qt = h["qt"]
    combined = layer.run(dev(h["x"], gpu), dev(h["logits"], gpu)).cpu().numpy()
    torch.cuda.synchronize()
    assert int(layer.status.item()) == 0
    pairs = rows * topk
    sel = layer.selected.cpu().numpy().astype(np.uint64)
    wts = layer.weights.cpu().numpy()
    order = layer.worklist.order.cpu().numpy()[:pairs]
    mid = layer.intermediate_f32.cpu().numpy()[:pairs]
    pair_out = layer.pair_outputs.cpu().numpy()[:pairs]
    gb = oracle.row_bytes(qt, hidden) * intermediate
    db = oracle.row_bytes(qt, intermediate) * hidden

    # Decode sweeps and matrix-core kernels alike: every row sum is the CPU path's (Q8_K
    # activations: the same float term per superblock, added in double in block order; F32
    # activations: the decoder's float weights, products and sums in double), so every stage is
    # compared for equality
    exact = True

    # routing: identical selection and weights (scores and normalisation run in double on both sides)
    for r in range(rows):
        rc, s, w, _ = oracle.moe_route(h["logits"][r], h["bias"], topk, scoring, True, 1.5)
        assert rc == 0 and np.array_equal(sel[r], s)
        assert np.array_equal(wts[r], w)

    # up + SwiGLU, then down, each against the oracle fed with the GPU's own stage input
    flips_mid = flips_out = 0.0
    for position in range(pairs):
        source = int(order[position])
        row, e = source // topk, int(sel.reshape(-1)[source])
        rc, _, want_mid, _ = oracle.moe_expert(
            (qt, qt, qt), h["gate"][e * gb:(e + 1) * gb], h["up"][e * gb:(e + 1) * gb],
            h["down"][e * db:(e + 1) * db], hidden, intermediate, h["x"][row],
            float(wts.reshape(-1)[source]), act_q8=act_q8)
        assert rc == 0
        if exact:
            assert np.array_equal(mid[position], want_mid), f"SwiGLU products of pair {position}"
        flips_mid += bf16_flip_report(mid[position], want_mid)
        if act_q8:
            q = oracle.q8k_quantize(mid[position])
            raw = oracle.q8_matvec(qt, h["down"][e * db:(e + 1) * db], hidden, intermediate, q, 1)[0]
        else:
            raw = oracle.matvec(qt, h["down"][e * db:(e + 1) * db], hidden, intermediate,
                                mid[position])[0]
        want_out = np.array([oracle.lib().yvo_bf16_round(np.float32(v)) for v in raw], np.float32)
        if exact:
            assert np.array_equal(pair_out[source], want_out), f"expert outputs of pair {position}"
        flips_out += bf16_flip_report(pair_out[source], want_out)
    assert flips_mid / pairs < 5e-3 and flips_out / pairs < 5e-3

    # rank-ordered reduce and combine are exact given the pair outputs
    routed = np.zeros((rows, hidden), np.float32)
    for rank in range(topk):
        routed += pair_out.reshape(rows, topk, hidden)[:, rank]
    assert np.array_equal(layer.routed_out.cpu().numpy()[:rows], routed)
    shared = layer.shared_out.cpu().numpy()[:rows]
    want = np.array([oracle.lib().yvo_bf16_round(np.float32(v)) for v in (routed + shared).ravel()],
                    np.float32).reshape(rows, hidden)
    assert np.array_equal(combined, want)

    # whole layer against the oracle's own end-to-end run
    full = oracle.moe_layer(hidden=hidden, intermediate=intermediate, experts=experts, topk=topk,
                            qtypes=(qt, qt, qt), routed=(h["gate"], h["up"], h["down"]),
                            shared=h["shared"], inputs=h["x"], logits=h["logits"], bias=h["bias"],
                            scoring=scoring, normalize=True, scaling=1.5, act_q8=act_q8, threads=8)
    assert np.array_equal(full["selected"], sel)
    if exact:
        assert np.array_equal(combined, full["combined"])
    err = np.abs(combined.astype(np.float64) - full["combined"])
    bound = 1e-5 + 1e-3 * np.abs(full["combined"])
    outside = err > bound
    # beyond the stated tolerance only where a bf16 rounding boundary was crossed upstream: a
    # one-step flip of any of the summed terms, measured against the terms' own magnitude
    assert outside.mean() < 2e-2
    terms = np.abs(pair_out.reshape(rows, topk, hidden)).sum(axis=1) + np.abs(shared)
    assert np.all(err[outside] <= 2 * BF16_ULP * terms[outside] + 1e-4)


def test_sweep_image_is_the_documented_repacking(gpu, oracle):
    """The image the device builds from canonical IQ2_XXS bytes, against a numpy statement of the
    format: per superblock two records of nine dwords {f16 d | four group scales << 16, then per
    group the codebook bytes and the 7-bit sign fields one to a byte}."""
    from yvex_amd import kernels as K
    g = oracle.Generator(5, "sweep.image")
    blocks = 300
    canonical = g.iq2xxs(blocks)
    image = K.iq2_sweep_image(dev(canonical, gpu)).cpu().numpy().view(np.uint32).reshape(blocks, 2, 9)
    raw = canonical.reshape(blocks, 66)
    d = raw[:, 0].astype(np.uint32) | (raw[:, 1].astype(np.uint32) << 8)
    groups = raw[:, 2:].reshape(blocks, 8, 8)
    grids = groups[:, :, :4].copy().view(np.uint32).reshape(blocks, 8)
    aux = groups[:, :, 4:].copy().view(np.uint32).reshape(blocks, 8)
    for half in range(2):
        scales = np.zeros(blocks, np.uint32)
        for j in range(4):
            a = aux[:, 4 * half + j]
            assert np.array_equal(image[:, half, 1 + 2 * j], grids[:, 4 * half + j])
            signs = (a & 127) | (((a >> 7) & 127) << 8) | (((a >> 14) & 127) << 16) | (((a >> 21) & 127) << 24)
            assert np.array_equal(image[:, half, 2 + 2 * j], signs)
            scales |= (a >> 28) << (4 * j)
        assert np.array_equal(image[:, half, 0], d | (scales << 16))


@pytest.mark.parametrize("hidden,intermediate,experts,topk,rows,matrix_cores", [
    (7168, 2048, 12, 4, 6, False), (2048, 2048, 6, 4, 20, False), (4096, 3072, 4, 2, 5, False),
    (2048, 2048, 200, 8, 40, False), (2048, 2048, 6, 4, 150, True), (7168, 768, 3, 2, 70, True),
    (512, 2048, 5, 3, 33, True)])
def test_kernels_give_the_same_bits_from_the_image(gpu, oracle, hidden, intermediate, experts, topk, rows,
                                                   matrix_cores):
    """The decode sweeps (one, two, three, four pairs a sweep, shared expert merged into the
    launches) and the matrix-core row-batch kernels (token tiles of both sizes, ragged row tiles)
    over the sweep image of the experts publish bit for bit what they publish from canonical
    bytes: same integer sums, same scaling, same order."""
    layers = []
    for image in (False, True):
        layer, h = make_layer(oracle, gpu, hidden=hidden, intermediate=intermediate, experts=experts,
                              topk=topk, rows=rows, qtype="IQ2_XXS", act_q8=True, scoring=1,
                              sweep_image=image, matrix_cores=matrix_cores)
        combined = layer.run(dev(h["x"], gpu), dev(h["logits"], gpu)).clone()
        torch.cuda.synchronize()
        assert int(layer.status.item()) == 0
        pairs = rows * topk
        mids = pairs if matrix_cores else pairs + rows      # the sweeps lay the shared expert's products behind the routed ones
        layers.append((combined.cpu().numpy(), layer.intermediate_f32[:mids].cpu().numpy().copy(),
                       layer.pair_outputs[:pairs].cpu().numpy().copy(), layer.shared_out[:rows].cpu().numpy().copy()))
    for a, b in zip(*layers):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("matrix_cores", [False, True])
@pytest.mark.parametrize("block", [0, 5])
def test_expert_kernels_single_superblock_is_bit_exact(gpu, oracle, matrix_cores, block):
    """With activations that are zero outside one 256-column superblock every output is a single
    term ((0.125 d_w) d_a) T, so there is no summation order left: the expert kernels (decode
    sweeps and matrix-core row batches) must equal the CPU path bit for bit, which pins their
    exact int32 superblock sums T through the real hot path."""
    from yvex_amd import kernels as K
    hidden, intermediate, experts, topk, rows = 2048, 2048, 6, 4, 20
    layer, h = make_layer(oracle, gpu, hidden=hidden, intermediate=intermediate, experts=experts,
                          topk=topk, rows=rows, qtype="IQ2_XXS", act_q8=True, scoring=1,
                          matrix_cores=matrix_cores)
    qt = h["qt"]
    x = np.zeros_like(h["x"])
    x[:, 256 * block:256 * (block + 1)] = h["x"][:, 256 * block:256 * (block + 1)]
    layer.run(dev(x, gpu), dev(h["logits"], gpu))
    torch.cuda.synchronize()
    assert int(layer.status.item()) == 0
    pairs = rows * topk
    sel = layer.selected.cpu().numpy().reshape(-1)
    wts = layer.weights.cpu().numpy().reshape(-1)
    order = layer.worklist.order.cpu().numpy()[:pairs]
    mid = layer.intermediate_f32.cpu().numpy()[:pairs]
    gb = oracle.row_bytes(qt, hidden) * intermediate
    db = oracle.row_bytes(qt, intermediate) * hidden
    for position in range(pairs):
        source = int(order[position])
        row, e = source // topk, int(sel[source])
        rc, _, want_mid, _ = oracle.moe_expert(
            (qt, qt, qt), h["gate"][e * gb:(e + 1) * gb], h["up"][e * gb:(e + 1) * gb],
            h["down"][e * db:(e + 1) * db], hidden, intermediate, x[row], float(wts[source]),
            act_q8=True)
        assert rc == 0
        assert np.array_equal(mid[position], want_mid), f"pair {position}"

    # the down projection on an intermediate with one live superblock per pair
    crafted = np.zeros((pairs, intermediate), np.float32)
    crafted[:, 256 * block:256 * (block + 1)] = oracle.Generator(7, "crafted").normal(pairs * 256).reshape(pairs, 256)
    st = layer.status
    q = K.q8k_quantize(dev(crafted, gpu), st)
    if matrix_cores:
        K.moe_down_rows(layer.routed, q, layer.worklist, pairs, experts, layer.pair_outputs, st)
    else:
        K.moe_down(layer.routed, q, True, layer.worklist, pairs, experts, layer.pair_outputs, st)
    torch.cuda.synchronize()
    assert int(st.item()) == 0
    pair_out = layer.pair_outputs.cpu().numpy()[:pairs]
    q_host = q.cpu().numpy().reshape(pairs, -1)
    for position in range(pairs):
        source = int(order[position])
        e = int(sel[source])
        raw = oracle.q8_matvec(qt, h["down"][e * db:(e + 1) * db], hidden, intermediate,
                               q_host[position], 1)[0]
        want = np.array([oracle.lib().yvo_bf16_round(np.float32(v)) for v in raw], np.float32)
        assert np.array_equal(pair_out[source], want), f"pair {position}"
