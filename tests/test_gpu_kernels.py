"""Parity of the launch-level HIP kernels against the CPU oracle (through the C ABI)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

REL, ABS = 1e-3, 1e-5   # the path's stated fp32 tolerance


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def assert_close(got, want, rel=REL, abs_=ABS):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    bound = abs_ + rel * np.abs(want)
    worst = np.argmax(err - bound)
    assert np.all(err <= bound), (
        f"max violation at {worst}: got {got.flat[worst]} want {want.flat[worst]}")


def assert_q8_product(got, want, qtype):
    """Q8_K activations: every format publishes the oracle's bits (exact integer sums, the
    primitive's float term per superblock, for Q8_0 its chain of eight fused terms, and the
    superblocks' terms added in double)."""
    assert np.array_equal(np.asarray(got).view(np.uint32), np.asarray(want).view(np.uint32))


def status_ok(status):
    torch.cuda.synchronize()
    assert int(status.item()) == 0


def test_q8k_quantize_bit_exact(gpu, oracle):
    from yvex_amd import kernels as K
    g = oracle.Generator(42, "q8k.rows")
    x = g.normal(6 * 1024).reshape(6, 1024)
    x[1, :256] = 0.0                       # all-zero block: d = 0, q = 0
    x[2, 256:512] = 0.0
    x[2, 300] = -3.5                       # single spike maps to -127 * sign
    x[3, 10] = 7.25                        # exact |tie|, opposite signs: lowest index wins
    x[3, 200] = -7.25
    x[4] *= 1e-30
    status = K.new_status(gpu)
    got = K.q8k_quantize(dev(x, gpu), status).cpu().numpy()
    status_ok(status)
    want = oracle.q8k_quantize(x)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    ("IQ2_XXS", 37, 2048, 3), ("IQ2_XXS", 5, 7168, 1), ("Q4_K", 19, 1024, 2),
    ("Q4_K", 6, 7168, 1), ("Q8_0", 23, 4096, 2), ("Q2_K", 11, 512, 3)])
def test_integer_block_dots_bit_exact(gpu, oracle, qtype, rows, width, inputs):
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"blockdots.{qtype}.{rows}.{width}")
    w = g.weights(qt, rows, width)
    act = oracle.q8k_quantize(g.normal(inputs * width).reshape(inputs, width))
    status = K.new_status(gpu)
    got = K.block_dots_i32(dev(w, gpu), qt, rows, width, dev(act, gpu), inputs, status).cpu().numpy()
    status_ok(status)
    want = oracle.block_dots_i32(qt, w, rows, width, act, inputs)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    ("IQ2_XXS", 67, 2048, 1), ("IQ2_XXS", 9, 7168, 5), ("Q4_K", 33, 2048, 1),
    ("Q4_K", 10, 7168, 16), ("Q8_0", 64, 4096, 1), ("Q8_0", 13, 96, 3), ("Q2_K", 21, 768, 2),
    ("F32", 17, 100, 3),
    # Q8_0 rows against eight and more F32 rows: the double-precision matrix cores (16 x 16 tiles,
    # sixteen and four waves a tile, staged blocks); a width they do not take stays lane-strided
    ("Q8_0", 70, 512, 9), ("Q8_0", 33, 1024, 300), ("Q8_0", 2100, 256, 1000), ("Q8_0", 20, 96, 30)])
def test_matvec_f32_activations(gpu, oracle, qtype, rows, width, inputs):
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"matvec.{qtype}.{rows}.{width}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    status = K.new_status(gpu)
    got = K.matvec(dev(w, gpu), qt, rows, width, dev(x, gpu), status=status).cpu().numpy()
    status_ok(status)
    want = oracle.matvec(qt, w, rows, width, x)
    assert_close(got, want)


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    ("F16", 300, 4096, 1), ("BF16", 70, 7168, 1), ("F16", 33, 1000, 2), ("BF16", 9, 264, 5), ("F16", 5, 8, 7),
    ("F16", 4100, 264, 1), ("BF16", 4097, 136, 3),      # many rows: a wave a row
    ("BF16", 40, 100, 3),       # rows that are not whole 16-byte pieces: the lane-strided kernel
    # eight input rows and more: the double-precision matrix cores (sixteen waves a tile, four
    # waves a tile from 256 input rows, staged blocks once there is one a compute unit); a row
    # width they do not take stays on the kernel above
    ("F16", 12, 512, 9), ("BF16", 40, 1024, 70), ("BF16", 70, 512, 300), ("F16", 1030, 256, 520),
    ("BF16", 2100, 128, 1000), ("F16", 20, 264, 30)])
def test_matvec_sixteen_bit_weights(gpu, oracle, qtype, rows, width, inputs):
    """F16 and BF16 weight rows against F32 input rows (projections and output heads kept in
    16-bit floats; src/gguf/quant_compute.c:152-172 forms double products and a double sum):
    the CPU path's float, which is the float of the exact double-precision product up to the
    order of the additions."""
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"matvec16.{qtype}.{rows}.{width}.{inputs}")
    values = g.normal(rows * width).reshape(rows, width).astype(np.float32)
    if qtype == "F16":
        encoded = values.astype(np.float16)
        decoded = encoded.astype(np.float32)
    else:
        encoded = (values.view(np.uint32) >> 16).astype(np.uint16)
        decoded = (encoded.astype(np.uint32) << 16).view(np.float32)
    w = np.ascontiguousarray(encoded).view(np.uint8).ravel()
    x = g.normal(inputs * width).reshape(inputs, width)
    status = K.new_status(gpu)
    got = K.matvec(dev(w, gpu), qt, rows, width, dev(x, gpu), status=status).cpu().numpy()
    status_ok(status)
    assert_close(got, oracle.matvec(qt, w, rows, width, x))
    exact = (x.astype(np.float64) @ decoded.astype(np.float64).T).astype(np.float32)
    assert np.mean(got.view(np.uint32) != exact.view(np.uint32)) < 1e-3      # (sums that sit on a rounding boundary)
    assert np.allclose(got, exact, rtol=1e-6, atol=1e-6)
    # a weight that is not finite is reported
    if rows > 1:
        poisoned = encoded.copy()
        poisoned.view(np.uint16).reshape(-1)[width + 3] = 0x7c00 if qtype == "F16" else 0x7f80
        K.matvec(dev(np.ascontiguousarray(poisoned).view(np.uint8).ravel(), gpu), qt, rows, width, dev(x, gpu),
                 status=status)
        torch.cuda.synchronize()
        assert int(status.item()) == 1


@pytest.mark.parametrize("rows,width,inputs", [(256, 7168, 64), (50, 512, 45), (24, 28672, 33), (1, 32, 32),
                                               (256, 7168, 300), (40, 96, 260), (256, 7168, 8), (3, 256, 9),
                                               (45, 448, 257), (32, 64, 256),
                                               # fewer than eight input rows: a workgroup a weight row
                                               (256, 7168, 1), (24, 28672, 5), (7, 100, 3), (9, 4096, 2), (5, 30, 2),
                                               (4100, 132, 2),
                                               # enough (32 rows x 64 input rows) blocks for the device and
                                               # 128-column chunks: the kernel with operands staged in LDS,
                                               # ragged on both sides
                                               (250, 256, 1570), (256, 384, 2048)])
def test_matvec_f32_weights_over_a_row_batch(gpu, oracle, rows, width, inputs):
    """F32 weight rows against 8 or more F32 input rows (a router or mixing projection over a
    row batch) run on the double-precision matrix cores; ragged edges, the additive operand and the bf16
    output behave as in the lane-strided kernel (kernels.cu:560-640)."""
    from yvex_amd import kernels as K
    g = oracle.Generator(42, f"matvec.f32.batch.{rows}.{width}.{inputs}")
    w = g.weights(oracle.F32, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    status = K.new_status(gpu)
    got = K.matvec(dev(w, gpu), oracle.F32, rows, width, dev(x, gpu), status=status).cpu().numpy()
    status_ok(status)
    want = oracle.matvec(oracle.F32, w, rows, width, x)
    assert_close(got, want)
    # against the double-precision product too: a transposed or mis-split operand cannot pass
    exact = x.astype(np.float64) @ w.view(np.float32).reshape(rows, width).astype(np.float64).T
    assert np.allclose(got, exact, rtol=1e-4, atol=1e-4)
    # the same projection with scratch memory (split between workgroups where the shape allows)
    w_rows = dev(w.view(np.float32).reshape(rows, width), gpu)
    split = K.matvec_f32_rows(w_rows, dev(x, gpu), status).cpu().numpy()
    status_ok(status)
    assert_close(split, want)
    assert np.allclose(split, exact, rtol=1e-4, atol=1e-4)
    again = K.matvec_f32_rows(w_rows, dev(x, gpu), status).cpu().numpy()
    assert np.array_equal(split, again)                # partial sums are added in a fixed order
    add = g.normal(inputs * rows).reshape(inputs, rows)
    got = K.matvec(dev(w, gpu), oracle.F32, rows, width, dev(x, gpu), additive=dev(add, gpu),
                   output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    assert np.all((got.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(got - (want + add)) <= np.abs(want + add) * 2.0 ** -8 + 1e-4)
    # a non-finite weight is reported, as by the other kernels
    if rows > 1:
        poisoned = w.copy()
        poisoned.view(np.float32)[width + 5] = np.inf
        K.matvec(dev(poisoned, gpu), oracle.F32, rows, width, dev(x, gpu), status=status)
        assert int(status.item()) == 1


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    ("IQ2_XXS", 67, 2048, 1), ("IQ2_XXS", 9, 7168, 6), ("Q4_K", 33, 7168, 1),
    ("Q4_K", 12, 2048, 16), ("Q8_0", 40, 4096, 2), ("Q2_K", 21, 768, 3)])
def test_matvec_q8k_activations(gpu, oracle, qtype, rows, width, inputs):
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"matvecq8.{qtype}.{rows}.{width}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                   status=status).cpu().numpy()
    status_ok(status)
    act_host = oracle.q8k_quantize(x)
    assert np.array_equal(act.cpu().numpy(), act_host)
    want = oracle.q8_matvec(qt, w, rows, width, act_host, inputs)
    assert_q8_product(got, want, qtype)
    # and against the reference CPU path fed the dequantised activations (its own test's form)
    deq = oracle.q8k_dequantize(act_host).reshape(inputs, width)
    assert_close(got, oracle.matvec(qt, w, rows, width, deq))


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    # lanes a row: 8 (and fewer superblocks than lanes), 16, 32, 64; row counts that leave lanes
    # and waves without a row; a row of more than 8192 columns (several passes of the wave)
    ("IQ2_XXS", 67, 512, 1), ("IQ2_XXS", 7168, 2048, 1), ("IQ2_XXS", 41, 4096, 1), ("IQ2_XXS", 2048, 7168, 1),
    ("IQ2_XXS", 5, 16384, 1), ("Q4_K", 2048, 7168, 1), ("Q4_K", 19, 1024, 1), ("Q4_K", 3, 24576, 1),
    ("Q2_K", 77, 2048, 1), ("Q2_K", 9, 7168, 1),
    # a few input rows over weights decoded once
    ("IQ2_XXS", 7168, 2048, 2), ("IQ2_XXS", 35, 2048, 31), ("IQ2_XXS", 130, 7168, 12), ("IQ2_XXS", 10, 768, 5),
    ("Q4_K", 2048, 7168, 3), ("Q4_K", 21, 512, 2), ("Q2_K", 33, 4096, 7)])
def test_matvec_q8k_one_round_trip_kernels(gpu, oracle, qtype, rows, width, inputs):
    """One (or a few) Q8_K input rows against superblock-format rows run through the kernels
    that ask for all of a lane's bytes at once: the oracle's Q8_K product bit for bit, with the
    additive rows and the bf16 rounding of the other kernels, and the same bits from weights on
    a 2-byte boundary, which take the general kernel."""
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(43, f"matvec.row.{qtype}.{rows}.{width}.{inputs}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    add = g.normal(inputs * rows).reshape(inputs, rows)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                   status=status).cpu().numpy()
    status_ok(status)
    want = oracle.q8_matvec(qt, w, rows, width, oracle.q8k_quantize(x), inputs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    summed = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                      additive=dev(add, gpu), output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    assert np.all((summed.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(summed - (got + add)) <= np.abs(got + add) * 2.0 ** -8 + 1e-30)
    shifted = torch.zeros(w.size + 2, dtype=torch.uint8, device=gpu)
    shifted[2:] = dev(w, gpu)
    moved = K.matvec(shifted[2:], qt, rows, width, act, input_q8=True, input_rows=inputs,
                     status=status).cpu().numpy()
    status_ok(status)
    assert np.array_equal(moved.view(np.uint32), got.view(np.uint32))


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    ("IQ2_XXS", 516, 2048, 32), ("IQ2_XXS", 260, 7168, 70), ("IQ2_XXS", 7168, 2048, 33),
    ("IQ2_XXS", 50, 2304, 40), ("IQ2_XXS", 7, 256, 33),
    # more work items (33 token tiles x 8 row tiles) than workgroups: a workgroup hands over from
    # one item to the next, whose first weight windows come with the last copies of the one before
    ("IQ2_XXS", 2048, 1024, 2112),
    ("Q4_K", 516, 2048, 16), ("Q4_K", 132, 7168, 70), ("Q4_K", 2048, 7168, 16), ("Q4_K", 36, 512, 200),
    ("Q4_K", 50, 2304, 17), ("Q4_K", 24, 7168, 32), ("Q4_K", 7, 256, 31),
    # Q4_K tile shapes by the number of workgroups: 16 x 32 tiles in several token tiles (the
    # cases of 70 and 200 rows above), 32 x 32 tiles, 32 x 64 tiles
    ("Q4_K", 2048, 512, 70), ("Q4_K", 2048, 256, 200)])
def test_matvec_q8k_row_batch_runs_on_matrix_cores(gpu, oracle, qtype, rows, width, inputs):
    """From 2 (Q4_K) or 32 (IQ2_XXS) Q8_K input rows on, projections run on the int8 matrix cores
    (src/backend/cuda/private.h:461-464 turns the tensor-core kernels on at 16). Results are the
    oracle's Q8_K product bit for bit, bf16 output rounds them, and smaller input-row counts
    (other kernels or tile shapes) give the same bits."""
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"matvec.rows.{qtype}.{rows}.{width}.{inputs}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                   status=status).cpu().numpy()
    status_ok(status)
    act_host = oracle.q8k_quantize(x)
    want = oracle.q8_matvec(qt, w, rows, width, act_host, inputs)
    assert_q8_product(got, want, qtype)
    deq = oracle.q8k_dequantize(act_host).reshape(inputs, width)
    assert_close(got, oracle.matvec(qt, w, rows, width, deq, threads=8))
    rounded = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                       output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    assert np.all((rounded.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(rounded - got) <= np.abs(got) * 2.0 ** -8 + 1e-30)
    # fewer rows at a time (the sweep kernel, or another tile shape): the same bits
    for count in (15, 1):
        few = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=count,
                       status=status).cpu().numpy()
        status_ok(status)
        assert np.array_equal(few.view(np.uint32), got[:count].view(np.uint32))


@pytest.mark.parametrize("rows,width,inputs", [(516, 4096, 16), (40, 256, 33), (4096, 4096, 70), (33, 2304, 64),
                                               (7, 512, 200),
                                               # a 256-row tile for every compute unit and up to 32 input rows:
                                               # the 256 x 32 staged shape (ragged last tile, two superblocks)
                                               (65700, 512, 20), (65536, 256, 32)])
def test_matvec_q8_0_row_batch_runs_on_matrix_cores(gpu, oracle, rows, width, inputs):
    """Q8_0 rows against 16 or more Q8_K input rows (the reference's tensor-core threshold,
    src/backend/cuda/private.h:461-464): the oracle's Q8_K product bit for bit (the chain of eight
    fused terms a superblock, superblocks added in double), ragged on both sides, with the additive
    operand and the bf16 rounding; the smaller batches' lane-strided kernel gives the same bits."""
    from yvex_amd import kernels as K
    qt = oracle.Q8_0
    g = oracle.Generator(42, f"matvec.q8_0.rows.{rows}.{width}.{inputs}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    add = g.normal(inputs * rows).reshape(inputs, rows)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                   status=status).cpu().numpy()
    status_ok(status)
    act_host = oracle.q8k_quantize(x)
    want = oracle.q8_matvec(qt, w, rows, width, act_host, inputs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    deq = oracle.q8k_dequantize(act_host).reshape(inputs, width)
    assert_close(got, oracle.matvec(qt, w, rows, width, deq, threads=8))
    summed = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                      additive=dev(add, gpu), output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    assert np.all((summed.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(summed - (got + add)) <= np.abs(got + add) * 2.0 ** -8 + 1e-30)
    few = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=15,
                   status=status).cpu().numpy()          # below the threshold: the lane-strided kernel
    status_ok(status)
    assert_q8_product(few, want[:15], "Q8_0")
    assert np.array_equal(few.view(np.uint32), got[:15].view(np.uint32))


@pytest.mark.parametrize("rows,width,inputs", [(130, 512, 1), (33, 2304, 5), (2048, 7168, 3), (40, 256, 15),
                                               (65700, 256, 3)])
def test_matvec_q8_0_exact_at_few_rows(gpu, oracle, rows, width, inputs):
    """Q8_0 rows below 16 Q8_K input rows (a shared expert run as dense projections at decode
    width): the oracle's product bit for bit from the lane-strided kernel too, which chains a
    superblock's eight terms across the lanes that hold them; additive rows and the bf16 rounding
    on top."""
    from yvex_amd import kernels as K
    qt = oracle.Q8_0
    g = oracle.Generator(42, f"matvec.q8_0.exact.{rows}.{width}.{inputs}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    add = g.normal(inputs * rows).reshape(inputs, rows)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs, status=status).cpu().numpy()
    status_ok(status)
    want = oracle.q8_matvec(qt, w, rows, width, oracle.q8k_quantize(x), inputs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    summed = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs, additive=dev(add, gpu),
                      output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    assert np.all((summed.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(summed - (got + add)) <= np.abs(got + add) * 2.0 ** -8 + 1e-30)


@pytest.mark.parametrize("rows,width,inputs", [(2001, 1280, 1030), (4100, 512, 250)])
def test_matvec_q8_0_large_batch_stages_operands_in_lds(gpu, oracle, rows, width, inputs):
    """A Q8_0 projection with more unstaged tiles than one round of workgroups takes the kernel
    whose operands pass through LDS, on tiles of 128 weight rows (the first case) or 64 (the
    second): ragged row count (the last tile repeats a row), a ragged last tile of input rows,
    several superblocks a row (both LDS buffers), additive rows and bf16 outputs; the oracle's
    product bit for bit, from the unstaged tiles and the lane-strided kernel as well."""
    from yvex_amd import kernels as K
    qt = oracle.Q8_0
    assert (rows + 31) // 32 * ((inputs + 63) // 64) > 256
    g = oracle.Generator(42, f"matvec.rows.staged.q8_0.{rows}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    bias = g.normal(inputs * rows).reshape(inputs, rows)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                   status=status).cpu().numpy()
    status_ok(status)
    act_host = oracle.q8k_quantize(x)
    want = oracle.q8_matvec(qt, w, rows, width, act_host, inputs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    summed = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                      additive=dev(bias, gpu), status=status).cpu().numpy()
    status_ok(status)
    assert np.array_equal(summed, got + bias)
    rounded = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                       output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    assert np.all((rounded.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(rounded - got) <= np.abs(got) * 2.0 ** -8 + 1e-30)
    for count in (70, 16, 3):       # the unstaged tiles, the lane-strided kernel
        few = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=count,
                       status=status).cpu().numpy()
        status_ok(status)
        assert np.array_equal(few.view(np.uint32), got[:count].view(np.uint32))


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    ("Q8_0", 130, 512, 3), ("Q8_0", 130, 512, 20), ("Q8_0", 1030, 256, 70), ("Q8_0", 2001, 256, 1030),
    ("Q4_K", 130, 512, 3), ("Q4_K", 130, 512, 20), ("Q4_K", 2048, 256, 70), ("Q4_K", 2048, 256, 200),
    ("Q4_K", 2001, 256, 1030), ("IQ2_XXS", 132, 512, 3), ("IQ2_XXS", 132, 512, 40), ("F32", 50, 256, 9)])
def test_matvec_writes_rows_of_a_wider_output(gpu, oracle, qtype, rows, width, inputs):
    """Every kernel behind yvex_hip_matvec honours the output stride (the additive operand shares
    it): results land in the first `rows` columns of a wider buffer, bit for bit what the dense
    output holds, and the columns behind them keep what they held."""
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"matvec.stride.{qtype}.{rows}.{inputs}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    add = g.normal(inputs * (rows + 12)).reshape(inputs, rows + 12)
    status = K.new_status(gpu)
    q8 = qtype != "F32"
    act = K.q8k_quantize(dev(x, gpu), status) if q8 else dev(x, gpu)
    wide_add = dev(add, gpu)
    dense_add = wide_add[:, :rows].contiguous()
    for additive in (None, (dense_add, wide_add)):
        dense = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=q8, input_rows=inputs,
                         additive=additive[0] if additive else None, status=status)
        wide = torch.full((inputs, rows + 12), -7.25, dtype=torch.float32, device=gpu)
        K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=q8, input_rows=inputs,
                 additive=additive[1] if additive else None, status=status, out=wide)
        status_ok(status)
        assert torch.equal(wide[:, :rows].contiguous().view(torch.int32), dense.view(torch.int32))
        assert bool((wide[:, rows:] == -7.25).all())


@pytest.mark.parametrize("qtype,rows,width,inputs", [
    ("Q8_0", 130, 512, 20), ("Q8_0", 1030, 256, 70), ("Q8_0", 2001, 256, 1030),
    ("Q4_K", 130, 512, 20), ("Q4_K", 2048, 256, 70), ("Q4_K", 2048, 256, 200), ("Q4_K", 2001, 256, 1030),
    ("IQ2_XXS", 132, 512, 40)])
def test_matvec_row_batch_flags_non_finite(gpu, oracle, qtype, rows, width, inputs):
    """A block scale that is infinite makes every sum of its weight row non-finite: the
    matrix-core kernels raise the numeric status, publish no value that is not finite (a kernel
    may hold back the stores that share an instruction with one: the row's neighbours in its
    32-row tile) and leave the other tiles' results what they are with clean weights."""
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"matvec.poison.{qtype}.{rows}.{inputs}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    clean = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs, status=status)
    status_ok(status)
    row_bytes = oracle.row_bytes(qt, width)
    bad_row = rows - 3
    poisoned = w.copy()
    poisoned[bad_row * row_bytes:bad_row * row_bytes + 2] = (0x00, 0x7c)         # the first block's fp16 scale
    out = torch.full((inputs, rows), -7.25, dtype=torch.float32, device=gpu)
    K.matvec(dev(poisoned, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs, status=status, out=out)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    keep = torch.ones(rows, dtype=torch.bool, device=gpu)
    keep[bad_row // 32 * 32:bad_row // 32 * 32 + 32] = False
    assert torch.equal(out[:, keep].contiguous().view(torch.int32), clean[:, keep].contiguous().view(torch.int32))
    assert bool((out[:, bad_row] == -7.25).all())
    assert bool(torch.isfinite(out).all())


def test_matvec_q4k_large_batch_stages_operands_in_lds(gpu, oracle):
    """A Q4_K projection with at least one (128 rows x 64 tokens) tile per compute unit takes the
    kernel whose operands are staged through LDS: ragged row count (the last tile repeats a row),
    a last token tile of six rows (one 32-token block), additive rows and bf16 outputs; the
    oracle's bits like the other tile shapes, and the smaller batches' bits."""
    from yvex_amd import kernels as K
    qt, rows, width, inputs = oracle.Q4_K, 2001, 768, 1030
    assert (rows + 127) // 128 * ((inputs + 63) // 64) >= 256
    g = oracle.Generator(42, "matvec.rows.staged.q4k")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    bias = g.normal(inputs * rows).reshape(inputs, rows)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                   status=status).cpu().numpy()
    status_ok(status)
    act_host = oracle.q8k_quantize(x)
    want = oracle.q8_matvec(qt, w, rows, width, act_host, inputs)
    assert_q8_product(got, want, "Q4_K")
    summed = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                      additive=dev(bias, gpu), status=status).cpu().numpy()
    status_ok(status)
    assert np.array_equal(summed, got + bias)
    rounded = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs,
                       output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    assert np.all((rounded.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(rounded - got) <= np.abs(got) * 2.0 ** -8 + 1e-30)
    for count in (70, 16):          # the unstaged 32 x 32 tiles, the 16 x 16 tiles
        few = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=count,
                       status=status).cpu().numpy()
        status_ok(status)
        assert np.array_equal(few.view(np.uint32), got[:count].view(np.uint32))


@pytest.mark.parametrize("qtype,rows,width", [("Q8_0", 9600, 7168), ("IQ2_XXS", 37000, 7168)])
def test_matvec_output_head_variant(gpu, oracle, qtype, rows, width):
    """One Q8_K activation row against a matrix of 64 MB or more takes the variant with four
    chunks of a row in flight (the output-head shape): every 97th row against the oracle's
    integer path, exactly as the small shapes are checked."""
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"matvec.head.{qtype}")
    sample = np.arange(0, rows, 97)
    distinct = g.weights(qt, len(sample) + 3, width).reshape(len(sample) + 3, -1)
    row_bytes = distinct.shape[1]
    assert rows * row_bytes >= 64 << 20
    w = np.empty((rows, row_bytes), np.uint8)
    w[:] = distinct[np.arange(rows) % 3 + len(sample)]       # filler rows
    w[sample] = distinct[:len(sample)]
    x = g.normal(width).reshape(1, width)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w.ravel(), gpu), qt, rows, width, act, input_q8=True, input_rows=1,
                   status=status).cpu().numpy()
    status_ok(status)
    act_host = oracle.q8k_quantize(x)
    want = oracle.q8_matvec(qt, np.ascontiguousarray(w[sample]).ravel(), len(sample), width, act_host, 1)
    assert_q8_product(np.ascontiguousarray(got[:, sample]), want, qtype)
    # filler rows repeat with period three: equal weights give equal bits
    filler = np.setdiff1d(np.arange(rows), sample)
    for k in range(3):
        same = got[0, filler[filler % 3 == k]]
        assert np.all(same.view(np.uint32) == same.view(np.uint32)[0])
    if qtype == "Q8_0":
        # a few rows against a Q8_0 matrix this large go to the matrix cores (the lane-strided
        # kernel would read the matrix once per input row): the oracle's bits
        few = g.normal(5 * width).reshape(5, width)
        act = K.q8k_quantize(dev(few, gpu), status)
        got = K.matvec(dev(w.ravel(), gpu), qt, rows, width, act, input_q8=True, input_rows=5,
                       status=status).cpu().numpy()
        status_ok(status)
        want = oracle.q8_matvec(qt, np.ascontiguousarray(w[sample]).ravel(), len(sample), width,
                                oracle.q8k_quantize(few), 5)
        assert np.array_equal(np.ascontiguousarray(got[:, sample]).view(np.uint32), want.view(np.uint32))


def test_matvec_additive_and_bf16(gpu, oracle):
    from yvex_amd import kernels as K
    g = oracle.Generator(7, "matvec.additive")
    rows, width = 33, 2048
    w = g.weights(oracle.IQ2_XXS, rows, width)
    x = g.normal(2 * width).reshape(2, width)
    add = g.normal(2 * rows).reshape(2, rows)
    status = K.new_status(gpu)
    got = K.matvec(dev(w, gpu), oracle.IQ2_XXS, rows, width, dev(x, gpu), additive=dev(add, gpu),
                   output_bf16=True, status=status).cpu().numpy()
    status_ok(status)
    base = oracle.matvec(oracle.IQ2_XXS, w, rows, width, x)
    want = (base + add).astype(np.float32)
    # a bf16 output differs from the unrounded sum by at most half a bf16 ulp
    assert np.all((got.view(np.uint32) & 0xffff) == 0)
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-5)


@pytest.mark.parametrize("qtype,width", [("IQ2_XXS", 512), ("Q4_K", 512), ("Q8_0", 96),
                                         ("Q2_K", 256), ("F32", 40)])
def test_gather_bit_exact(gpu, oracle, qtype, width):
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(11, f"gather.{qtype}")
    rows = 29
    w = g.weights(qt, rows, width)
    ids = np.array([28, 0, 3, 3, 17], np.uint32)
    status = K.new_status(gpu)
    got = K.gather(dev(w, gpu), qt, rows, width, dev(ids, gpu), status).cpu().numpy()
    status_ok(status)
    want = oracle.decode_rows(qt, w, width, ids)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("scoring", [0, 1])
def test_route_rows(gpu, oracle, scoring):
    from yvex_amd import kernels as K
    g = oracle.Generator(42, f"route.{scoring}")
    rows, experts, topk = 32, 256, 8
    logits = g.normal(rows * experts).reshape(rows, experts)
    logits[3, 10] = logits[3, 200]          # exact tie: lowest ordinal first
    bias = (g.normal(experts) * 0.1).astype(np.float32)
    status = K.new_status(gpu)
    sel, w = K.moe_route_rows(dev(logits, gpu), dev(bias, gpu), topk, scoring, True, 2.5, status)
    status_ok(status)
    sel, w = sel.cpu().numpy(), w.cpu().numpy()
    for r in range(rows):
        rc, s, ww, _ = oracle.moe_route(logits[r], bias, topk, scoring, True, 2.5)
        assert rc == 0
        assert np.array_equal(sel[r].astype(np.uint64), s)
        assert np.max(np.abs(w[r] - ww)) <= 1e-6


@pytest.mark.parametrize("scoring", [0, 1])
def test_route_hash_rows(gpu, oracle, scoring):
    """Hash router against the oracle (src/graph/moe.c:539-582): identical selection, weights to
    1e-6; a repeated ordinal, an ordinal outside the experts and a token outside the table raise
    the contract status."""
    from yvex_amd import kernels as K
    g = oracle.Generator(9, f"route.hash.{scoring}")
    rows, experts, topk, vocab = 37, 256, 6, 50
    logits = g.normal(rows * experts).reshape(rows, experts) * 2.0
    rng = np.random.default_rng(2)
    table = np.stack([rng.permutation(experts)[:8] for _ in range(vocab)]).astype(np.int32)   # 8 columns, 6 used
    tokens = rng.integers(0, vocab, rows).astype(np.int32)
    status = K.new_status(gpu)
    sel, w = K.moe_route_hash_rows(dev(logits, gpu), dev(table, gpu), dev(tokens, gpu), topk, scoring, True, 1.5, status)
    status_ok(status)
    sel, w = sel.cpu().numpy(), w.cpu().numpy()
    for r in range(rows):
        rc, want_sel, want_w, _ = oracle.moe_route_hash(logits[r], table, int(tokens[r]), topk, scoring, True, 1.5)
        assert rc == 0 and np.array_equal(sel[r], want_sel.astype(np.int64))
        assert np.max(np.abs(w[r] - want_w)) <= 1e-6
    # one row for every token
    status = K.new_status(gpu)
    sel1, _ = K.moe_route_hash_rows(dev(logits, gpu), dev(table[7:8], gpu), dev(tokens, gpu), topk, scoring, True,
                                    1.5, status, table_rows=vocab)
    status_ok(status)
    assert np.all(sel1.cpu().numpy() == table[7, :topk])
    for poison in ("repeat", "range", "token"):
        t, ids = table.copy(), tokens.copy()
        if poison == "repeat":
            t[ids[5], 3] = t[ids[5], 1]
        elif poison == "range":
            t[ids[5], 2] = experts
        else:
            ids[5] = vocab
        status = K.new_status(gpu)
        K.moe_route_hash_rows(dev(logits, gpu), dev(t, gpu), dev(ids, gpu), topk, scoring, True, 1.5, status)
        torch.cuda.synchronize()
        assert int(status.item()) == 2, poison


@pytest.mark.parametrize("rows,topk,experts", [(32, 8, 256), (1, 6, 256), (61, 6, 256),
                                               (2048, 8, 256), (5, 2, 4), (4096, 3, 256)])
def test_worklist_matches_stable_sort(gpu, oracle, rows, topk, experts):
    from yvex_amd import kernels as K
    rng = np.random.default_rng(rows * 131 + topk)
    # skewed popularity so some experts stay empty and some buckets are large
    p = 1.0 / np.arange(1, experts + 1) ** 1.1
    p /= p.sum()
    sel = np.stack([rng.choice(experts, topk, replace=False, p=p) for _ in range(rows)])
    w = rng.random((rows, topk), dtype=np.float32)
    status = K.new_status(gpu)
    wl = K.worklist_build(dev(sel.astype(np.int64), gpu), experts, status)
    status_ok(status)
    rc, want = oracle.worklist_build(sel, w, topk, experts)
    assert rc == 0
    n = int(wl.counts[0].item())
    assert n == len(want["expert_ids"])
    assert int(wl.counts[2].item()) == rows * topk
    assert int(wl.counts[1].item()) == int(want["bucket_populations"].max())
    assert np.array_equal(wl.expert_ids.cpu().numpy()[:n].astype(np.uint64), want["expert_ids"])
    assert np.array_equal(wl.bucket_offsets.cpu().numpy()[:n + 1].astype(np.uint64),
                          want["bucket_offsets"])
    assert np.array_equal(wl.bucket_populations.cpu().numpy()[:n].astype(np.uint64),
                          want["bucket_populations"])
    assert np.array_equal(wl.order.cpu().numpy().astype(np.uint64), want["source_pairs"])


@pytest.mark.parametrize("rows,experts,topk,width,scoring", [
    (32, 256, 8, 7168, 1), (1, 256, 8, 7168, 0), (128, 64, 6, 512, 0), (17, 200, 16, 1024, 1), (5, 16, 4, 0, 0)])
def test_fused_preparation_equals_the_three_launches(gpu, oracle, rows, experts, topk, width, scoring):
    """Routing + worklist + input quantization in one launch: every output bit for bit what the
    separate launches write, and the oracle's selection."""
    from yvex_amd import kernels as K
    g = oracle.Generator(5, f"prepare.{rows}.{experts}.{topk}")
    logits = dev(g.normal(rows * experts).reshape(rows, experts) * 1.5, gpu)
    bias = dev((g.normal(experts) * 0.05).astype(np.float32), gpu)
    values = dev(g.normal(rows * width).reshape(rows, width), gpu) if width else None
    assert K.moe_prepare_supported(rows, experts, topk)
    assert not K.moe_prepare_supported(129, experts, topk) and not K.moe_prepare_supported(rows, 257, topk)
    status = K.new_status(gpu)
    sel, w = K.moe_route_rows(logits, bias, topk, scoring, True, 2.5, status)
    wl = K.worklist_build(sel, experts, status)
    q8 = K.q8k_quantize(values, status) if width else None
    status_ok(status)
    fused_wl = K.Worklist(rows * topk, experts, gpu)
    fused_q8 = torch.zeros_like(q8) if width else None
    fsel, fw = K.moe_prepare(logits, bias, topk, scoring, True, 2.5, status, fused_wl, values, fused_q8)
    status_ok(status)
    assert torch.equal(fsel, sel) and torch.equal(fw.view(torch.int32), w.view(torch.int32))
    n = int(wl.counts[0].item())
    assert torch.equal(fused_wl.counts, wl.counts)
    assert torch.equal(fused_wl.order, wl.order)
    assert torch.equal(fused_wl.expert_ids[:n], wl.expert_ids[:n])
    assert torch.equal(fused_wl.bucket_populations[:n], wl.bucket_populations[:n])
    assert torch.equal(fused_wl.bucket_offsets[:n + 1], wl.bucket_offsets[:n + 1])
    assert torch.equal(fused_wl.sweep_offsets[:n + 1], wl.sweep_offsets[:n + 1])
    if width:
        assert torch.equal(fused_q8, q8)
    rc, want_sel, _, _ = oracle.moe_route(logits[rows - 1].cpu().numpy(), bias.cpu().numpy(), topk, scoring, True, 2.5)
    assert rc == 0 and np.array_equal(fsel[rows - 1].cpu().numpy().astype(np.uint64), want_sel)
    # a non-finite logit raises the numeric status from inside the fused launch as well
    bad = logits.clone()
    bad[0, 1] = float("nan")
    status = K.new_status(gpu)
    K.moe_prepare(bad, bias, topk, scoring, True, 2.5, status, fused_wl, values, fused_q8)
    torch.cuda.synchronize()
    assert int(status.item()) != 0


@pytest.mark.parametrize("rows,experts,topk,width,scoring", [
    (32, 256, 8, 7168, 1), (32, 256, 8, 7168, 0), (8, 64, 6, 1024, 0), (100, 200, 16, 2048, 1)])
def test_scored_projection_and_preparation_equal_the_plain_pair(gpu, oracle, rows, experts, topk, width,
                                                                scoring):
    """The router projection that publishes the scores beside the logits, and the preparation
    that starts from them: logits, selection, route weights, worklist and quantized input bit
    for bit what the projection and the preparation over logits write; the scores are the
    oracle's (src/graph/moe.c:497-537)."""
    from yvex_amd import kernels as K
    g = oracle.Generator(9, f"scored.{rows}.{experts}.{topk}.{scoring}")
    router = dev(g.normal(experts * width).reshape(experts, width) * 0.05, gpu)
    values = dev(g.normal(rows * width).reshape(rows, width), gpu)
    bias = dev((g.normal(experts) * 0.05).astype(np.float32), gpu)
    status = K.new_status(gpu)
    logits = K.matvec_f32_rows(router, values, status)
    wl = K.Worklist(rows * topk, experts, gpu)
    q8 = torch.zeros(rows * (width // 256) * 292, dtype=torch.uint8, device=gpu)
    sel, w = K.moe_prepare(logits, bias, topk, scoring, True, 2.5, status, wl, values, q8)
    status_ok(status)
    got_logits, scores = K.matvec_f32_rows_scored(router, values, scoring, status)
    got_wl = K.Worklist(rows * topk, experts, gpu)
    got_q8 = torch.zeros_like(q8)
    got_sel, got_w = K.moe_prepare_scored(scores, bias, topk, True, 2.5, status, got_wl, values, got_q8)
    status_ok(status)
    assert torch.equal(got_logits.view(torch.int32), logits.view(torch.int32))
    assert torch.equal(got_sel, sel) and torch.equal(got_w.view(torch.int32), w.view(torch.int32))
    n = int(wl.counts[0].item())
    assert torch.equal(got_wl.counts, wl.counts) and torch.equal(got_wl.order, wl.order)
    assert torch.equal(got_wl.expert_ids[:n], wl.expert_ids[:n])
    assert torch.equal(got_wl.bucket_offsets[:n + 1], wl.bucket_offsets[:n + 1])
    assert torch.equal(got_wl.bucket_populations[:n], wl.bucket_populations[:n])
    assert torch.equal(got_wl.sweep_offsets[:n + 1], wl.sweep_offsets[:n + 1])
    assert torch.equal(got_q8, q8)
    for row in (0, rows - 1):
        rc, want_sel, want_w, want_scores = oracle.moe_route(logits[row].cpu().numpy(), bias.cpu().numpy(), topk,
                                                             scoring, True, 2.5)
        assert rc == 0 and np.array_equal(got_sel[row].cpu().numpy().astype(np.uint64), want_sel)
        np.testing.assert_allclose(scores[row].cpu().numpy(), want_scores, rtol=2e-7, atol=0)
        np.testing.assert_allclose(got_w[row].cpu().numpy(), want_w, rtol=1e-6, atol=0)
    # a shape the projection does not split is refused, not run some other way
    with pytest.raises(K.KernelError):
        K.matvec_f32_rows_scored(router[:, :256].contiguous(), values[:, :256].contiguous(), scoring, status)
    # an input that makes a logit non-finite raises the numeric status from the join
    bad = values.clone()
    bad[0, 3] = float("inf")
    status = K.new_status(gpu)
    K.matvec_f32_rows_scored(router, bad, scoring, status)
    torch.cuda.synchronize()
    assert int(status.item()) != 0


@pytest.mark.parametrize("rows,topk,hidden,offset", [(5, 3, 8, 0), (32, 8, 7168, 0), (3, 6, 10, 0), (4, 5, 64, 1),
                                                     (7, 1, 4, 0)])
def test_reduce_combine_sums_in_rank_order(gpu, oracle, rows, topk, hidden, offset):
    """routed = the ranks' rows added one after another in fp32 (src/runtime/moe.c:596-632),
    combined = bf16(routed + shared): exact, for widths and addresses that take the 16-byte path
    and for those that do not (offset shifts the buffers off 16-byte alignment)."""
    from yvex_amd import kernels as K
    g = oracle.Generator(3, f"reduce.{rows}.{topk}.{hidden}")
    pairs = (g.normal(rows * topk * hidden) * 3.0).astype(np.float32).reshape(rows * topk, hidden)
    shared = g.normal(rows * hidden).astype(np.float32).reshape(rows, hidden)

    def shifted(a):       # a view that starts `offset` floats into a larger allocation
        t = torch.empty(a.size + offset, dtype=torch.float32, device=gpu)
        v = t[offset:].view(a.shape)
        v.copy_(torch.from_numpy(a))
        return v
    d_pairs, d_shared = shifted(pairs), shifted(shared)
    routed, combined = shifted(np.zeros_like(shared)), shifted(np.zeros_like(shared))
    status = K.new_status(gpu)
    K.moe_reduce_combine(d_pairs, rows, topk, hidden, d_shared, routed, combined, status)
    status_ok(status)
    want = np.zeros((rows, hidden), np.float32)
    for rank in range(topk):
        want = (want + pairs.reshape(rows, topk, hidden)[:, rank]).astype(np.float32)
    assert np.array_equal(routed.cpu().numpy(), want)
    total = (want + shared).astype(np.float32)
    want_combined = np.array([oracle.lib().yvo_bf16_round(float(v)) for v in total.ravel()], np.float32)
    assert np.array_equal(combined.cpu().numpy().ravel(), want_combined)
    # a non-finite sum raises the numeric status and publishes nothing for that element
    d_pairs[0, 0] = float("inf")
    status = K.new_status(gpu)
    K.moe_reduce_combine(d_pairs, rows, topk, hidden, d_shared, routed, combined, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1


def test_worklist_flags_duplicate_expert(gpu):
    from yvex_amd import kernels as K
    sel = np.array([[1, 2], [3, 3]], np.int64)
    status = K.new_status(gpu)
    K.worklist_build(dev(sel, gpu), 4, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 2


@pytest.mark.parametrize("rows,width", [(1, 129280), (5, 1001), (3, 7), (32, 4096), (2, 1), (3, 20001)])
def test_greedy_selection_matches_oracle(gpu, oracle, rows, width):
    """Largest value, lowest index holding it, tie count: exact (kernels.cu:59-110)."""
    from yvex_amd import kernels as K
    rng = np.random.default_rng(rows * 1000 + width)
    values = rng.standard_normal((rows, width)).astype(np.float32)
    if width > 4:
        values[0, width - 1] = values[0, 1] = values[0].max() + 1.0   # a tie at both ends of row 0
        values[rows - 1] = np.round(values[rows - 1] * 2.0) / 2.0     # many ties in the last row
    rc, want_tokens, want_best, want_ties = oracle.argmax_f32(values)
    assert rc == 0
    for scratch in (None, False):     # rows split over workgroups (when long), one workgroup per row
        status = K.new_status(gpu)
        tokens, best, ties = K.argmax_f32(dev(values, gpu), status, scratch=scratch)
        status_ok(status)
        assert np.array_equal(tokens.cpu().numpy().astype(np.uint32), want_tokens)
        assert np.array_equal(best.cpu().numpy(), want_best)
        assert np.array_equal(ties.cpu().numpy().astype(np.uint64), want_ties)


def test_greedy_selection_flags_non_finite(gpu, oracle):
    from yvex_amd import kernels as K
    values = np.zeros((3, 515), np.float32)
    values[0, 17] = 2.0
    values[1, 300] = np.inf
    values[2, 2] = values[2, 514] = 1.5
    status = K.new_status(gpu)
    tokens, best, ties = K.argmax_f32(dev(values, gpu), status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    rc, want_tokens, want_best, want_ties = oracle.argmax_f32(values)
    assert rc == 1
    for row in (0, 2):      # the rows without the bad value publish; the bad row stays as it was
        assert int(tokens[row]) == want_tokens[row] and float(best[row]) == want_best[row]
        assert int(ties[row]) == want_ties[row]
    assert int(ties[1]) == 0
    # long rows shared among workgroups: the status is raised and only the bad row stays silent
    values = np.ones((2, 30000), np.float32)
    values[1, 29999] = np.nan
    status = K.new_status(gpu)
    tokens, best, ties = K.argmax_f32(dev(values, gpu), status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1 and int(ties[1]) == 0
    assert int(ties[0]) == 30000 and int(tokens[0]) == 0 and float(best[0]) == 1.0
    # a status another operation left on the shared word does not silence clean rows
    values[1, 29999] = 3.0
    status.fill_(2)
    tokens, best, ties = K.argmax_f32(dev(values, gpu), status)
    torch.cuda.synchronize()
    assert int(status.item()) == 2 and int(tokens[1]) == 29999 and int(ties[0]) == 30000


def envelope_inputs(oracle, tokens, streams, width, name):
    g = oracle.Generator(42, f"envelope.{name}.{streams}.{width}")
    mixing = (streams + 2) * streams
    rows = g.normal(tokens * streams * width).reshape(tokens, streams * width)     # not bf16 values
    rounded = ((rows.view(np.uint32) + 0x7fff + ((rows.view(np.uint32) >> 16) & 1)) & 0xffff0000).view(np.float32)
    mixes = g.normal(tokens * mixing).reshape(tokens, mixing) * 3.0
    scale = np.array([0.5, -0.25, 0.75], np.float32)
    base = g.normal(mixing, 0.5)
    norm = (1.0 + g.normal(width, 0.2)).astype(np.float32)
    return rows, rounded, mixes, scale, base, norm


@pytest.mark.parametrize("tokens,streams,width,iterations", [
    (5, 4, 7168, 20), (3, 1, 512, 1), (2, 7, 200, 3), (33, 4, 256, 20), (1, 2, 16384, 2), (4, 3, 203, 5),
    (2, 4, 1028, 4)])
def test_envelope_ingress_matches_oracle(gpu, oracle, tokens, streams, width, iterations):
    """Ingress + weighted RMS norm against numeric.c's order of operations. The kernel rounds the
    residual to bf16 as the reference's device kernel does, so the oracle is fed the rounded
    rows. Gates and the mixing matrix come from double-precision exp, whose last bit may differ
    between the two maths libraries: 1e-6 as the reference's own envelope test allows
    (tests/unit/deepseek_attention.c:2326-2337); the published row is bf16, so a value on a
    rounding boundary may move by one bf16 step."""
    from yvex_amd import kernels as K
    rows, rounded, mixes, scale, base, norm = envelope_inputs(oracle, tokens, streams, width, "in")
    kw = dict(streams=streams, width=width, iterations=iterations, rms_epsilon=1e-6, mhc_epsilon=1e-6,
              post_multiplier=2.0)
    status = K.new_status(gpu)
    normalized, post, comb = K.mhc_ingress(dev(rows, gpu), dev(mixes, gpu), dev(scale, gpu), dev(base, gpu),
                                           dev(norm, gpu), status=status, **kw)
    status_ok(status)
    rc, collapsed, want_post, want_comb = oracle.mhc_pre(rounded, mixes, scale, base, **kw)
    assert rc == 0
    want = np.zeros_like(collapsed)
    for t in range(tokens):
        rc, want[t] = oracle.rms_norm(collapsed[t], norm, 1e-6)
        assert rc == 0
    want = ((want.view(np.uint32) + 0x7fff + ((want.view(np.uint32) >> 16) & 1)) & 0xffff0000).view(np.float32)
    assert_close(post.cpu().numpy(), want_post, rel=1e-6, abs_=1e-6)
    assert_close(comb.cpu().numpy(), want_comb, rel=1e-6, abs_=1e-6)
    got = normalized.cpu().numpy()
    assert np.array_equal(got.view(np.uint32) & 0xffff, np.zeros_like(got.view(np.uint32)))
    differ = got != want
    assert differ.mean() < 1e-3
    assert np.all(np.abs(got[differ] - want[differ]) <= 2.0 ** -7 * np.abs(want[differ]))


@pytest.mark.parametrize("tokens,streams,width", [(5, 4, 7168), (3, 1, 512), (2, 7, 200), (64, 4, 300),
                                                  (3, 5, 203)])
def test_envelope_egress_bit_exact(gpu, oracle, tokens, streams, width):
    """Egress is double-precision multiply-adds in a fixed order and one bf16 rounding: bit-exact."""
    from yvex_amd import kernels as K
    rows, rounded, _, _, _, _ = envelope_inputs(oracle, tokens, streams, width, "out")
    g = oracle.Generator(7, f"envelope.core.{streams}.{width}")
    core = g.normal(tokens * width).reshape(tokens, width)
    post = np.abs(g.normal(tokens * streams)).reshape(tokens, streams).astype(np.float32)
    comb = np.abs(g.normal(tokens * streams * streams)).reshape(tokens, streams, streams).astype(np.float32)
    status = K.new_status(gpu)
    got = K.mhc_egress(dev(core, gpu), dev(rows, gpu), dev(post, gpu), dev(comb, gpu), streams=streams,
                       width=width, status=status).cpu().numpy()
    status_ok(status)
    rc, want = oracle.mhc_post(core, rounded, post, comb, streams=streams, width=width)
    assert rc == 0 and np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_envelope_flags_non_finite(gpu, oracle):
    from yvex_amd import kernels as K
    rows, _, mixes, scale, base, norm = envelope_inputs(oracle, 3, 2, 256, "bad")
    kw = dict(streams=2, width=256, iterations=2, rms_epsilon=1e-6, mhc_epsilon=1e-6, post_multiplier=2.0)
    for poison in ("rows", "base", "norm"):
        r, b, n = rows.copy(), base.copy(), norm.copy()
        {"rows": r, "base": b, "norm": n}[poison].flat[5] = np.inf
        status = K.new_status(gpu)
        K.mhc_ingress(dev(r, gpu), dev(mixes, gpu), dev(scale, gpu), dev(b, gpu), dev(n, gpu), status=status, **kw)
        torch.cuda.synchronize()
        assert int(status.item()) == 1, poison
    core = np.ones((3, 256), np.float32)
    core[1, 7] = np.nan
    status = K.new_status(gpu)
    K.mhc_egress(dev(core, gpu), dev(rows, gpu), dev(np.ones((3, 2), np.float32), gpu),
                 dev(np.ones((3, 2, 2), np.float32), gpu), streams=2, width=256, status=status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1
    with pytest.raises(K.KernelError):     # eight streams would need 80 mixing rows
        K.mhc_egress(dev(core, gpu), dev(rows, gpu), dev(np.ones((3, 8), np.float32), gpu),
                     dev(np.ones((3, 8, 8), np.float32), gpu), streams=8, width=32, status=status)
