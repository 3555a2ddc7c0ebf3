"""The dense BASELINE configurations at their stated sizes and seeded generators, every output
against the CPU oracle (reference: yvex_quant_cpu_dot, src/gguf/quant_compute.c:116-181, for F32
activations; the integer block dots of src/backend/cuda/kernel_primitives.h:287-359 for Q8_K
activations).

  config 0: Q8_0 4096 x 4096, w ~ N(0, 0.02^2) encoded as the reference's encoder does
            (d = f16(max|w| / 127), q = roundf(w / d)), x ~ N(0, 1), one input row, seed 42;
  config 1: Q4_K 2048 rows x 7168 columns, uniform sub-scales / sub-mins / nibbles, Q8_K
            activations, 1 and 16 input rows;
  config 2: IQ2_XXS 7168 rows x 2048 columns, uniform grid / sign / scale bytes, one input row.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

REL, ABS = 1e-3, 1e-5   # the path's stated fp32 tolerance


def dev(a, device):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def assert_close(got, want, rel, abs_):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    err = np.abs(got - want)
    bound = abs_ + rel * np.abs(want)
    worst = np.argmax(err - bound)
    assert np.all(err <= bound), f"max violation at {worst}: got {got.flat[worst]} want {want.flat[worst]}"


@pytest.mark.parametrize("name,qtype,rows,width,inputs", [
    ("config0", "Q8_0", 4096, 4096, 1),
    ("config1", "Q4_K", 2048, 7168, 1),
    ("config1", "Q4_K", 2048, 7168, 16),
    ("config2", "IQ2_XXS", 7168, 2048, 1),
])
def test_dense_config_at_full_size(gpu, oracle, name, qtype, rows, width, inputs):
    from yvex_amd import kernels as K
    qt = getattr(oracle, qtype)
    g = oracle.Generator(42, f"{name}.{qtype}")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    d_w = dev(w, gpu)
    status = K.new_status(gpu)

    # F32 activations: the CPU row dot (decode to float, double accumulation) on every row
    got = K.matvec(d_w, qt, rows, width, dev(x, gpu), status=status).cpu().numpy()
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    assert_close(got, oracle.matvec(qt, w, rows, width, x, threads=8), REL, ABS)

    # Q8_K activations: identical quantized rows, then the integer path on every row
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(d_w, qt, rows, width, act, input_q8=True, input_rows=inputs, status=status).cpu().numpy()
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    act_host = oracle.q8k_quantize(x)
    assert np.array_equal(act.cpu().numpy(), act_host)
    want = oracle.q8_matvec(qt, w, rows, width, act_host, inputs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))      # every format: the oracle's bits
    # and the reference CPU path fed the dequantised activations (the form of its own test,
    # tests/unit/cuda/quant_qtype.c:402-421)
    deq = oracle.q8k_dequantize(act_host).reshape(inputs, width)
    assert_close(got, oracle.matvec(qt, w, rows, width, deq, threads=8), REL, ABS)


def test_q4k_sixteen_q8k_rows_at_width_7168(gpu, oracle):
    """32 Q4_K rows of 7168 columns against 16 Q8_K input rows: the batch the reference would send
    to its row kernels (input_rows >= 16, src/backend/cuda/private.h:462-464)."""
    from yvex_amd import kernels as K
    qt, rows, width, inputs = oracle.Q4_K, 32, 7168, 16
    g = oracle.Generator(7, "q4k.b16.7168")
    w = g.weights(qt, rows, width)
    x = g.normal(inputs * width).reshape(inputs, width)
    status = K.new_status(gpu)
    act = K.q8k_quantize(dev(x, gpu), status)
    got = K.matvec(dev(w, gpu), qt, rows, width, act, input_q8=True, input_rows=inputs, status=status).cpu().numpy()
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    act_host = oracle.q8k_quantize(x)
    assert np.array_equal(act.cpu().numpy(), act_host)
    want = oracle.q8_matvec(qt, w, rows, width, act_host, inputs)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    sums = K.block_dots_i32(dev(w, gpu), qt, rows, width, act, inputs, status).cpu().numpy()
    torch.cuda.synchronize()
    assert int(status.item()) == 0
    assert np.array_equal(sums, oracle.block_dots_i32(qt, w, rows, width, act_host, inputs))
