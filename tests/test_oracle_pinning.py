"""What pins the CPU oracle: the reference's golden vectors and known-answer tests, fixtures
written by the library compiled from the reference's own sources, that library itself where it
can be built, and closed forms / brute force for what those leave open (Q4_K, sigmoid scoring,
the Q8_K quantizer, the integer block dots).
"""
import ctypes as C
import math
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz")


@pytest.fixture(scope="module")
def golden():
    return np.load(GOLDEN)


@pytest.fixture(scope="module")
def L(oracle):
    return oracle.lib()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


# ---- scalar rules: tests/unit/quant_numeric.c:188-259 ---------------------------------------

def test_f16_exhaustive_round_trip(L):
    for code in range(65536):
        value = L.yvo_f16_decode(code)
        exponent, mantissa = (code >> 10) & 31, code & 1023
        encoded = L.yvo_f16_encode(value)
        if exponent == 31 and mantissa:
            assert math.isnan(value) and (encoded & 0x7c00) == 0x7c00 and (encoded & 0x3ff)
        else:
            assert encoded == code
    # against numpy's IEEE binary16 (an independent implementation) for every finite code
    codes = np.arange(65536, dtype=np.uint16)
    want = codes.view(np.float16).astype(np.float32)
    got = np.array([L.yvo_f16_decode(int(c)) for c in codes], np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(bits(got[finite]), bits(want[finite]))
    assert L.yvo_f16_encode(1.00048828125) == 0x3c00 and L.yvo_f16_encode(1.00146484375) == 0x3c02
    assert L.yvo_f16_decode(0x0001) == 2.0 ** -24 and L.yvo_f16_decode(0x7bff) == 65504.0
    assert math.copysign(1.0, L.yvo_f16_decode(0x8000)) == -1.0
    assert math.isinf(L.yvo_f16_decode(0x7c00)) and L.yvo_f16_encode(3.4e38) == 0x7c00


def test_bf16_exhaustive_round_trip(L):
    for code in range(65536):
        value = L.yvo_bf16_decode(code)
        exponent, mantissa = (code >> 7) & 255, code & 127
        encoded = L.yvo_bf16_encode(value)
        if exponent == 255 and mantissa:
            assert math.isnan(value) and (encoded & 0x7f80) == 0x7f80 and (encoded & 0x7f)
        else:
            assert encoded == code
    halfway = np.array([0x3f808000, 0x3f818000], np.uint32).view(np.float32)
    assert L.yvo_bf16_encode(float(halfway[0])) == 0x3f80 and L.yvo_bf16_encode(float(halfway[1])) == 0x3f82


def test_scalar_rules_match_reference_fixture(L, golden):
    got = np.array([L.yvo_f16_decode(int(c)) for c in golden["f16_codes"]], np.float32)
    want = golden["f16_decode_bits"]
    nan = np.isnan(got)
    assert np.array_equal(bits(got)[~nan], want[~nan])
    assert np.all(np.isnan(want[nan].view(np.float32)))
    samples = golden["scalar_samples"]
    assert np.array_equal(np.array([L.yvo_f16_encode(float(v)) for v in samples], np.uint16), golden["f16_encode"])
    assert np.array_equal(np.array([L.yvo_bf16_encode(float(v)) for v in samples], np.uint16), golden["bf16_encode"])


# ---- block codecs: tests/unit/quant_numeric.c:502-609 -----------------------------------------

def test_golden_block_bytes(L, oracle):
    src = np.zeros(32, np.float32)
    src[:4] = [127.0, -127.0, 0.5, -0.5]
    enc = np.zeros(34, np.uint8)
    assert L.yvo_q8_0_encode_block(src.ctypes.data_as(C.c_void_p), enc.ctypes.data_as(C.c_void_p)) == 1
    assert list(enc[:6]) == [0x00, 0x3c, 0x7f, 0x81, 0x01, 0xff]          # halfway codes round away
    q2 = np.zeros(84, np.uint8)
    q2[:16] = 0x01
    q2[16:80] = 0xe4
    q2[80:82] = [0x00, 0x3c]
    dec = oracle.decode_rows(oracle.Q2_K, q2, 256)[0]
    assert np.array_equal(dec, ((np.arange(256) % 128) // 32).astype(np.float32))
    mx = np.zeros(17, np.uint8)
    mx[0], mx[1:] = 127, 0x21
    out = np.zeros(32, np.float32)
    assert L.yvo_decode_block(oracle.MXFP4, mx.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p)) == 0
    assert np.all(out[:16] == 0.5) and np.all(out[16:] == 1.0)
    # refusals: non-finite or negative scales (quant_block.c:819-833, :856-881)
    bad = np.zeros(34, np.uint8)
    bad[1] = 0x7c
    assert L.yvo_decode_block(oracle.Q8_0, bad.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p)) == oracle.ERR_FORMAT
    bad2 = np.zeros(84, np.uint8)
    bad2[81] = 0x7c
    big = np.zeros(256, np.float32)
    assert L.yvo_decode_block(oracle.Q2_K, bad2.ctypes.data_as(C.c_void_p), big.ctypes.data_as(C.c_void_p)) == oracle.ERR_FORMAT
    neg = np.zeros(66, np.uint8)
    neg[1] = 0xbc
    assert L.yvo_decode_block(oracle.IQ2_XXS, neg.ctypes.data_as(C.c_void_p), big.ctypes.data_as(C.c_void_p)) == oracle.ERR_FORMAT


@pytest.mark.parametrize("name,qtype", [("q8_0", 8), ("q2_k", 10), ("iq2_xxs", 16)])
def test_decode_and_row_dot_match_reference_fixture(oracle, golden, name, qtype):
    blob, x = golden[f"{name}_blob"], golden[f"{name}_x"]
    block, nbytes = oracle.geometry(qtype)
    decoded = oracle.decode_rows(qtype, blob, 512)
    assert np.array_equal(bits(decoded).reshape(-1), golden[f"{name}_decoded_bits"].reshape(-1))
    rb = 512 // block * nbytes
    dots = [oracle.cpu_dot(qtype, blob[r * rb:(r + 1) * rb], x) for r in range(blob.size // rb)]
    assert all(rc == 0 for rc, _ in dots)
    assert np.array_equal(bits(np.array([v for _, v in dots], np.float32)), golden[f"{name}_dots_bits"])
    # float64 brute force of the same definition
    brute = (decoded.astype(np.float64) * x.astype(np.float64)).sum(axis=1)
    assert np.allclose([v for _, v in dots], brute, rtol=1e-6, atol=1e-7)


def test_iq2_grid_is_the_public_codebook(L, oracle):
    # first and last entries of ggml's iq2xxs_grid and structural facts of the table
    one = np.zeros(66, np.uint8)
    one[0:2] = [0x00, 0x3c]                                     # d = 1
    out = np.zeros(256, np.float32)

    def magnitudes(index):
        one[2:6] = [index, 0, 0, 0]
        one[6:10] = [0, 0, 0, 0]
        L.yvo_decode_block(oracle.IQ2_XXS, one.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
        return [int(round(v * 8)) for v in out[:8]]            # gs = 1 * 0.5 * 0.25

    assert magnitudes(0) == [8] * 8
    assert magnitudes(1) == [43, 8, 8, 8, 8, 8, 8, 8]           # 0x080808080808082b
    assert magnitudes(2) == [25, 25, 8, 8, 8, 8, 8, 8]          # 0x0808080808081919
    seen = {tuple(magnitudes(i)) for i in range(256)}
    assert len(seen) == 256 and all(set(m) <= {8, 25, 43} for m in seen)
    # sign rule: seven stored bits plus an even-parity eighth
    one[2:6] = 0
    one[6:10] = np.array([0b0000011], np.uint32).view(np.uint8)
    L.yvo_decode_block(oracle.IQ2_XXS, one.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    assert list(np.sign(out[:8])) == [-1, -1, 1, 1, 1, 1, 1, 1]
    one[6:10] = np.array([0b0000001], np.uint32).view(np.uint8)
    L.yvo_decode_block(oracle.IQ2_XXS, one.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    assert list(np.sign(out[:8])) == [-1, 1, 1, 1, 1, 1, 1, -1]
    # group scale (0.5 + s) / 4 from the top nibble
    one[6:10] = np.array([7 << 28], np.uint32).view(np.uint8)
    L.yvo_decode_block(oracle.IQ2_XXS, one.ctypes.data_as(C.c_void_p), out.ctypes.data_as(C.c_void_p))
    assert out[0] == 8 * 7.5 * 0.25 and out[32] == 8 * 0.5 * 0.25


def test_live_reference_library_agrees(oracle):
    """Where oracle/_ref can be built, replay fresh random data through both."""
    ref = oracle.ref_lib()
    if ref is None:
        pytest.skip("reference tree absent: the committed fixture stands in")
    import sys
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    import make_golden
    for qtype in (oracle.Q8_0, oracle.Q2_K, oracle.IQ2_XXS, oracle.F32):
        block, nbytes = oracle.geometry(qtype)
        g = oracle.Generator(7, f"live.{qtype}")
        width = 1024 if block > 1 else 96
        blob, x = g.weights(qtype, 3, width), g.normal(width)
        rb = width // block * nbytes
        if block > 1:
            want = make_golden.ref_decode(ref, qtype, blob, nbytes, block)
            assert np.array_equal(bits(oracle.decode_rows(qtype, blob, width)).reshape(-1), bits(want).reshape(-1))
        for r in range(3):
            rc, got = oracle.cpu_dot(qtype, blob[r * rb:(r + 1) * rb], x)
            assert rc == 0 and np.float32(got).view(np.uint32) == np.float32(
                make_golden.ref_dot(ref, qtype, blob[r * rb:(r + 1) * rb], x)).view(np.uint32)
    # the reference refuses Q4_K on its CPU path (src/gguf/quant_compute.c:131-136)
    out, failure, err = C.c_float(), (C.c_ubyte * 512)(), (C.c_ubyte * 512)()
    q4 = oracle.Generator(1, "live.q4k").weights(oracle.Q4_K, 1, 256)
    x = np.ones(256, np.float32)
    ref.yvex_quant_cpu_dot.argtypes = [C.c_uint, C.c_void_p, C.c_size_t, C.c_void_p, C.c_ulonglong,
                                       C.c_void_p, C.c_void_p, C.c_void_p]
    assert ref.yvex_quant_cpu_dot(12, q4.ctypes.data, q4.size, x.ctypes.data, 256, C.byref(out),
                                  failure, err) == oracle.ERR_UNSUPPORTED


def test_cpu_dot_refusals(oracle):
    g = oracle.Generator(3, "refusals")
    row, x = g.weights(oracle.IQ2_XXS, 1, 512), g.normal(512)
    assert oracle.cpu_dot(oracle.IQ2_XXS, row, x[:511])[0] == oracle.ERR_BOUNDS       # not block divisible
    assert oracle.cpu_dot(oracle.IQ2_XXS, row[:-2], x)[0] == oracle.ERR_BOUNDS        # byte count
    assert oracle.cpu_dot(13, row, x)[0] == oracle.ERR_UNSUPPORTED                    # Q5_K: no codec
    bad = x.copy()
    bad[3] = np.inf
    assert oracle.cpu_dot(oracle.IQ2_XXS, row, bad)[0] == oracle.ERR_FORMAT


# ---- Q4_K: not in the reference, pinned by the public format's structure ---------------------

def q4k_pack_scales(sc, mn):
    """The public ggml packer (quantize_row_q4_K): the inverse direction of get_scale_min_k4."""
    scales = np.zeros(12, np.uint8)
    for j in range(8):
        if j < 4:
            scales[j] |= sc[j]
            scales[j + 4] |= mn[j]
        else:
            scales[j + 4] = (sc[j] & 0xF) | ((mn[j] & 0xF) << 4)
            scales[j - 4] |= (sc[j] >> 4) << 6
            scales[j] |= (mn[j] >> 4) << 6
    return scales


def q4k_block(d, dmin, sc, mn, values):
    """values[256] in 0..15, element order as the format stores them."""
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([d], np.float16).view(np.uint8)
    blk[2:4] = np.array([dmin], np.float16).view(np.uint8)
    blk[4:16] = q4k_pack_scales(sc, mn)
    v = np.asarray(values, np.uint8).reshape(4, 2, 32)          # chunk, low/high nibble, lane
    blk[16:] = (v[:, 0, :] | (v[:, 1, :] << 4)).reshape(-1)
    return blk


def test_q4k_closed_forms(oracle):
    rng = np.random.default_rng(0)
    values = rng.integers(0, 16, 256)
    # equal scales, zero mins: a plain 4-bit affine code in element order
    dec = oracle.decode_rows(oracle.Q4_K, q4k_block(0.5, 0.0, [3] * 8, [0] * 8, values), 256)[0]
    assert np.array_equal(dec, (1.5 * values).astype(np.float32))
    # all nibbles zero: every value is -dmin * m of its sub-block
    mn = [1, 5, 9, 13, 17, 33, 49, 63]
    dec = oracle.decode_rows(oracle.Q4_K, q4k_block(1.0, 0.25, [7] * 8, mn, np.zeros(256)), 256)[0]
    assert np.array_equal(dec.reshape(8, 32), np.repeat(-0.25 * np.array(mn, np.float32), 32).reshape(8, 32))
    # 6-bit scales above 15 exercise the split high bits; sub-block j scales only its 32 values
    sc = [1, 17, 33, 63, 16, 31, 47, 62]
    dec = oracle.decode_rows(oracle.Q4_K, q4k_block(1.0, 0.0, sc, [0] * 8, np.ones(256)), 256)[0]
    assert np.array_equal(dec.reshape(8, 32)[:, 0], np.array(sc, np.float32))
    # general case against float arithmetic spelt from the format description
    sc, mn = rng.integers(0, 64, 8), rng.integers(0, 64, 8)
    d, dmin = np.float32(np.float16(0.0123)), np.float32(np.float16(0.0071))
    dec = oracle.decode_rows(oracle.Q4_K, q4k_block(d, dmin, sc, mn, values), 256)[0]
    want = (d * sc.astype(np.float32)).repeat(32) * values.astype(np.float32) - \
           (dmin * mn.astype(np.float32)).repeat(32)
    assert np.array_equal(dec, want.astype(np.float32))
    rc, dot = oracle.cpu_dot(oracle.Q4_K, q4k_block(d, dmin, sc, mn, values), np.ones(256, np.float32))
    assert rc == 0 and abs(dot - want.astype(np.float64).sum()) < 1e-4


# ---- Q8_K quantizer: closed forms (kernels.cu:436-489) ------------------------------------------

def test_q8k_quantizer_closed_forms(oracle):
    x = np.zeros((1, 512), np.float32)
    x[0, 300] = -3.5
    q = oracle.q8k_quantize(x).reshape(2, 292)
    assert np.all(q[0] == 0)                                                # zero block: d = 0, q = 0
    d = q[1, :4].view(np.float32)[0]
    codes = q[1, 4:260].view(np.int8)
    assert codes[300 - 256] == -127 and np.count_nonzero(codes) == 1       # the spike maps to -127
    assert np.isclose(d * -127.0, -3.5, rtol=1e-6)
    assert list(q[1, 260:].view(np.int16)) == [0, 0, -127] + [0] * 13
    # exact |tie| with opposite signs: the first one sets the sign, d*q is the same either way
    y = np.zeros((1, 256), np.float32)
    y[0, 10], y[0, 200] = 7.25, -7.25
    q = oracle.q8k_quantize(y)
    assert q[4:260].view(np.int8)[10] == -127 and q[4:260].view(np.int8)[200] == 127
    z = y.copy()
    z[0, 10], z[0, 200] = -7.25, 7.25
    assert np.array_equal(oracle.q8k_dequantize(q), -oracle.q8k_dequantize(oracle.q8k_quantize(z)))
    # round to nearest even and the 16-wide sums on random data
    g = oracle.Generator(9, "q8k")
    r = g.normal(4 * 1024).reshape(4, 1024)
    q = oracle.q8k_quantize(r).reshape(-1, 292)
    for b, block in enumerate(r.reshape(-1, 256)):
        d = q[b, :4].view(np.float32)[0]
        m = block[np.argmax(np.abs(block))]
        inv = np.float32(-127.0) / m
        assert d == np.float32(1.0) / inv
        want = np.clip(np.rint(inv * block), -128, 127).astype(np.int8)
        assert np.array_equal(q[b, 4:260].view(np.int8), want)
        assert np.array_equal(q[b, 260:].view(np.int16), want.reshape(16, 16).sum(axis=1, dtype=np.int16))
    with pytest.raises(RuntimeError):
        oracle.q8k_quantize(np.full((1, 256), np.nan, np.float32))


# ---- integer block dots against the (reference-pinned) float decoders ---------------------------

@pytest.mark.parametrize("qtype", ["IQ2_XXS", "Q8_0", "Q4_K", "Q2_K"])
def test_integer_block_dots_from_decoded_values(oracle, qtype):
    qt = getattr(oracle, qtype)
    g = oracle.Generator(21, f"intdots.{qtype}")
    rows, width = 3, 1024
    w = g.weights(qt, rows, width)
    act = oracle.q8k_quantize(g.normal(2 * width).reshape(2, width))
    sums = oracle.block_dots_i32(qt, w, rows, width, act, 2)
    a = act.reshape(2, -1, 292)[:, :, 4:260].view(np.int8).astype(np.int64)       # [in, block, 256]
    da = act.reshape(2, -1, 292)[:, :, :4].copy().view(np.float32)[..., 0].astype(np.float64)
    decoded = oracle.decode_rows(qt, w, width).astype(np.float64).reshape(rows, -1, 256)
    if qtype == "IQ2_XXS":
        d = np.array([oracle.lib().yvo_f16_decode(int(v)) for v in
                      w.reshape(-1, 66)[:, :2].copy().view(np.uint16).ravel()]).reshape(rows, -1)
        ints = np.rint(decoded / (0.125 * d[..., None])).astype(np.int64)   # (2s+1) * level * sign
        want = np.einsum("rbk,ibk->irb", ints, a)
        assert np.array_equal(sums[..., 0], want) and np.all(sums[..., 1] == 0)
    elif qtype == "Q8_0":
        q = w.reshape(rows, -1, 34)[:, :, 2:].view(np.int8).astype(np.int64)          # [rows, unit, 32]
        want = np.einsum("ruk,iuk->iru", q, a.reshape(2, -1, 32))
        assert np.array_equal(sums, want)
    else:
        # dot and min are not separable from one decode, but their float combination is
        head = 0 if qtype == "Q4_K" else 80
        nb = 144 if qtype == "Q4_K" else 84
        dd = w.reshape(rows, -1, nb)[:, :, head:head + 4].copy().view(np.uint16)
        f = np.vectorize(lambda v: oracle.lib().yvo_f16_decode(int(v)))
        d, dmin = f(dd[..., 0]).astype(np.float64), f(dd[..., 1]).astype(np.float64)
        got = da[:, None, :] * (d[None] * sums[..., 0] - dmin[None] * sums[..., 1])
        want = np.einsum("rbk,ibk->irb", decoded, a * da[..., None])
        assert np.allclose(got, want, rtol=1e-6, atol=1e-6)


# ---- routing and expert: tests/unit/runtime_moe.c:105-212 ----------------------------------------

def score(v):
    return math.sqrt(v + math.log1p(math.exp(-v)) if v > 0 else math.log1p(math.exp(v)))


def test_router_reference_expectations(oracle):
    logits = np.array([1.0, 2.0, 2.0, 0.0], np.float32)      # router rows dotted with input [1,0,0,0]
    rc, sel, w, _ = oracle.moe_route(logits, [5.0, 0.0, 0.0, 0.0], 2, oracle.SQRT_SOFTPLUS, True, 1.5)
    assert rc == 0 and list(sel) == [0, 1]                   # bias picks 0, the tie goes to ordinal 1
    a, b = score(1.0), score(2.0)
    assert abs(w[0] - a / (a + b) * 1.5) < 1e-6 and abs(w[1] - b / (a + b) * 1.5) < 1e-6
    rc, sel, _, _ = oracle.moe_route(logits, [0.0] * 4, 2, oracle.SQRT_SOFTPLUS, True, 1.5)
    assert list(sel) == [1, 2]


def test_router_matches_reference_fixture(oracle, golden):
    for r in range(golden["route_logits"].shape[0]):
        rc, sel, w, _ = oracle.moe_route(golden["route_logits"][r], golden["route_bias"], 6,
                                         oracle.SQRT_SOFTPLUS, True, 1.5)
        assert rc == 0 and np.array_equal(sel, golden["route_selected"][r])
        assert np.array_equal(bits(w), golden["route_weights_bits"][r])


def test_hash_router_reference_expectations_and_fixture(oracle, golden):
    """tests/unit/runtime_moe.c:152-170: the token's table row is the selection, a repeated
    ordinal refuses with FORMAT, a token outside the table with BOUNDS; then the fixture from the
    compiled reference's yvex_moe_route_cpu, bit for bit."""
    logits = np.array([1, 2, 2, 0], np.float32)
    rc, sel, w, _ = oracle.moe_route_hash(logits, np.array([[3, 1]], np.int32), 0, 2, oracle.SQRT_SOFTPLUS, True, 1.5)
    score = lambda v: math.sqrt(math.log1p(math.exp(v)) if v <= 0 else v + math.log1p(math.exp(-v)))
    assert rc == 0 and list(sel) == [3, 1]
    assert abs(w[0] - score(0.0) / (score(0.0) + score(2.0)) * 1.5) < 1e-6
    assert oracle.moe_route_hash(logits, np.array([[3, 3]], np.int32), 0, 2, 0, True, 1.5)[0] == oracle.ERR_FORMAT
    assert oracle.moe_route_hash(logits, np.array([[3, 4]], np.int32), 0, 2, 0, True, 1.5)[0] == oracle.ERR_FORMAT
    assert oracle.moe_route_hash(logits, np.array([[-1, 2]], np.int32), 0, 2, 0, True, 1.5)[0] == oracle.ERR_FORMAT
    assert oracle.moe_route_hash(logits, np.array([[3, 1]], np.int32), 1, 2, 0, True, 1.5)[0] == oracle.ERR_BOUNDS
    for r, token in enumerate(golden["route_hash_tokens"]):
        rc, sel, w, _ = oracle.moe_route_hash(golden["route_logits"][r], golden["route_hash_table"], int(token), 6,
                                              oracle.SQRT_SOFTPLUS, True, 1.5)
        assert rc == 0 and np.array_equal(sel, golden["route_hash_selected"][r])
        assert np.array_equal(bits(w), golden["route_hash_weights_bits"][r])


def test_sigmoid_scoring_closed_form(oracle):
    g = oracle.Generator(5, "sigmoid")
    logits = g.normal(256)
    rc, sel, w, scores = oracle.moe_route(logits, None, 8, oracle.SIGMOID, True, 2.5)
    assert rc == 0
    assert np.allclose(scores, 1.0 / (1.0 + np.exp(-logits.astype(np.float64))), rtol=1e-6)
    assert list(sel) == list(np.argsort(-logits, kind="stable")[:8])      # monotone: order of logits
    assert abs(float(w.sum()) - 2.5) < 1e-6 and np.all(np.diff(w) <= 0)
    rc, _, w, _ = oracle.moe_route(np.zeros(4, np.float32), None, 2, oracle.SIGMOID, False, 1.0)
    assert list(w) == [0.5, 0.5]


def bf16(oracle, v):
    return oracle.lib().yvo_bf16_round(np.float32(v))


def test_expert_exact_equality_case(oracle):
    gate = np.array([1.0, 2.0, -1.0, 1.0], np.float32)
    up = np.array([2.0, 0.0, 1.0, 3.0], np.float32)
    down = np.array([1.0, 0.5, -0.25, 2.0], np.float32)
    x = np.array([1.0, 2.0], np.float32)
    mid = []
    for r in range(2):
        gv = float(gate[2 * r]) * 1.0 + float(gate[2 * r + 1]) * 2.0
        uv = float(up[2 * r]) * 1.0 + float(up[2 * r + 1]) * 2.0
        mid.append(bf16(oracle, np.float32((gv / (1.0 + math.exp(-gv))) * uv * 0.25)))
    want = [bf16(oracle, down[0] * mid[0] + down[1] * mid[1]), bf16(oracle, down[2] * mid[0] + down[3] * mid[1])]
    rc, out, got_mid, _ = oracle.moe_expert((0, 0, 0), gate.view(np.uint8), up.view(np.uint8),
                                            down.view(np.uint8), 2, 2, x, 0.25)
    assert rc == 0 and list(out) == want and list(got_mid) == mid


@pytest.mark.parametrize("name,qtype,hidden,inter", [("iq2_xxs", 16, 256, 256), ("q8_0", 8, 128, 64)])
def test_expert_matches_reference_fixture(oracle, golden, name, qtype, hidden, inter):
    rc, out, mid, _ = oracle.moe_expert(
        (qtype,) * 3, golden[f"expert_{name}_gate"], golden[f"expert_{name}_up"],
        golden[f"expert_{name}_down"], hidden, inter, golden[f"expert_{name}_x"], 0.25)
    assert rc == 0 and np.array_equal(bits(out), golden[f"expert_{name}_out_bits"])
    if name == "iq2_xxs":
        # the fixture drives gate/up beyond +-10: the clamp must have been active somewhere
        g = oracle.matvec(qtype, golden[f"expert_{name}_gate"], inter, hidden, golden[f"expert_{name}_x"])[0]
        assert np.any(np.abs(g) > 10.0)
    assert np.all((bits(mid) & 0xffff) == 0) and np.all((bits(out) & 0xffff) == 0)


def test_worklist_properties(oracle):
    rng = np.random.default_rng(2)
    rows, topk, experts = 40, 6, 64
    sel = np.stack([rng.choice(experts, topk, replace=False) for _ in range(rows)])
    w = rng.random((rows, topk), dtype=np.float32)
    rc, wl = oracle.worklist_build(sel, w, topk, experts)
    assert rc == 0
    flat = sel.reshape(-1)
    order = wl["source_pairs"].astype(np.int64)
    assert np.array_equal(order, np.argsort(flat, kind="stable"))           # stable sort by expert
    assert int(wl["bucket_populations"].sum()) == rows * topk
    assert np.array_equal(wl["expert_ids"], np.unique(flat))
    assert np.array_equal(wl["source_rows"], order // topk) and np.array_equal(wl["destination_rows"], order)
    assert np.array_equal(wl["route_weights"], w.reshape(-1)[order])
    bad = sel.copy()
    bad[0, 0] = experts
    assert oracle.worklist_build(bad, w, topk, experts)[0] == oracle.ERR_FORMAT


def test_greedy_selection_against_brute_force(oracle):
    """The serial restatement of the selection kernel (kernels.cu:59-110) against an independent
    formulation: the maximum, the first position that holds it, the number of positions that
    hold it. Rows are drawn from a few values so ties are common."""
    rng = np.random.default_rng(7)
    for width in (1, 2, 7, 64, 129, 1000):
        values = rng.integers(-3, 4, size=(9, width)).astype(np.float32) * 0.5
        values[3] = -3.402823466e+38          # the starting value itself: first index, all tied
        values[4, width // 2] = 11.0          # a single winner
        rc, tokens, best, ties = oracle.argmax_f32(values)
        assert rc == 0
        for row in range(values.shape[0]):
            top = values[row].max()
            where = np.flatnonzero(values[row] == top)
            assert best[row] == top and tokens[row] == where[0] and ties[row] == where.size
    # a non-finite value: status 1, that row untouched, the others published
    values = np.array([[1.0, 2.0, 2.0], [0.0, np.inf, 1.0], [5.0, np.nan, 5.0], [4.0, 1.0, 0.0]], np.float32)
    rc, tokens, best, ties = oracle.argmax_f32(values)
    assert rc == 1
    assert (tokens[0], best[0], ties[0]) == (1, 2.0, 2) and (tokens[3], best[3], ties[3]) == (0, 4.0, 1)
    assert ties[1] == 0 and ties[2] == 0


# ---- residual-stream envelope: tests/unit/deepseek_attention.c:2255-2340 ----------------------

def test_envelope_egress_reference_vectors(oracle):
    """The reference's own known answers for the egress: combination rows are sources and columns
    are targets (deepseek_attention.c:2263-2266,2302-2309) and the external conformance vector
    (tests/reference/deepseek_attention.c:2725-2730)."""
    rc, out = oracle.mhc_post([0.5, -0.25], [1, 2, 3, 4], [0, 0], [1, 2, 3, 4], streams=2, width=2)
    assert rc == 0 and out.ravel().tolist() == [10.0, 14.0, 14.0, 20.0]
    rc, out = oracle.mhc_post([0.5, -0.25], [1, 2, 3, 4], [2, 1], [1, 2, 3, 4], streams=2, width=2)
    assert rc == 0 and out.ravel().tolist() == [11.0, 13.5, 14.5, 19.75]


def test_envelope_egress_against_einsum(oracle):
    rng = np.random.default_rng(3)
    tokens, streams, width = 5, 4, 48
    core = rng.standard_normal((tokens, width)).astype(np.float32)
    res = rng.standard_normal((tokens, streams, width)).astype(np.float32)
    post = rng.random((tokens, streams)).astype(np.float32)
    comb = rng.random((tokens, streams, streams)).astype(np.float32)
    rc, out = oracle.mhc_post(core, res, post, comb, streams=streams, width=width)
    want = np.einsum("bt,bl->btl", post.astype(np.float64), core.astype(np.float64)) + \
        np.einsum("bst,bsl->btl", comb.astype(np.float64), res.astype(np.float64))
    got = out.reshape(tokens, streams, width)
    assert rc == 0 and np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-30)   # one bf16 rounding
    assert np.array_equal(bits(got) & 0xffff, np.zeros_like(bits(got)))                 # bf16 values
    bad = core.copy()
    bad[2, 5] = np.inf
    assert oracle.mhc_post(bad, res, post, comb, streams=streams, width=width)[0] == oracle.ERR_FORMAT


def test_envelope_ingress_closed_forms(oracle):
    """Ingress against what the mathematics fixes: sigmoid gates from an independent float64
    formula, a combination matrix whose rows and columns sum to one after enough Sinkhorn turns,
    collapsed rows as the gate-weighted sum of the streams, and the unit test's refusal of
    non-finite coefficients."""
    rng = np.random.default_rng(11)
    tokens, streams, width = 4, 4, 40
    mixing = (streams + 2) * streams
    res = (np.round(rng.standard_normal((tokens, streams * width)) * 32) / 32).astype(np.float32)
    mix = rng.standard_normal((tokens, mixing)).astype(np.float32)
    scale = np.array([0.5, -0.25, 0.75], np.float32)
    base = (rng.standard_normal(mixing) * 0.3).astype(np.float32)
    rc, collapsed, post, comb = oracle.mhc_pre(res, mix, scale, base, streams=streams, width=width,
                                               iterations=20, rms_epsilon=1e-6, mhc_epsilon=1e-6,
                                               post_multiplier=2.0)
    assert rc == 0
    r64, m64 = res.astype(np.float64), mix.astype(np.float64)
    inverse = 1.0 / np.sqrt((r64 ** 2).mean(axis=1) + 1e-6)
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    pre = sig(m64[:, :streams] * inverse[:, None] * 0.5 + base[:streams]) + 1e-6
    want_post = 2.0 * sig(m64[:, streams:2 * streams] * inverse[:, None] * -0.25 + base[streams:2 * streams])
    assert np.allclose(post, want_post, rtol=1e-6, atol=0)
    want = np.einsum("bs,bsl->bl", pre, r64.reshape(tokens, streams, width))
    assert np.all(np.abs(collapsed - want) <= 2.0 ** -8 * np.abs(want) + 1e-6)
    assert np.allclose(comb.sum(axis=1), 1.0, atol=1e-4) and np.allclose(comb.sum(axis=2), 1.0, atol=1e-4)
    assert np.all(comb > 0)
    # one Sinkhorn turn is the row softmax followed by one column normalisation
    rc, _, _, once = oracle.mhc_pre(res, mix, scale, base, streams=streams, width=width, iterations=1,
                                    rms_epsilon=1e-6, mhc_epsilon=1e-6, post_multiplier=2.0)
    raw = m64[:, 2 * streams:].reshape(tokens, streams, streams) * inverse[:, None, None] * 0.75 + \
        base[2 * streams:].astype(np.float64).reshape(streams, streams)
    soft = np.exp(raw - raw.max(axis=2, keepdims=True))
    soft = soft / soft.sum(axis=2, keepdims=True) + 1e-6
    soft = soft / (soft.sum(axis=1, keepdims=True) + 1e-6)
    assert rc == 0 and np.allclose(once, soft, rtol=1e-5, atol=1e-7)
    bad = base.copy()
    bad[3] = np.nan
    assert oracle.mhc_pre(res, mix, scale, bad, streams=streams, width=width, iterations=1, rms_epsilon=1e-6,
                          mhc_epsilon=1e-6, post_multiplier=2.0)[0] == oracle.ERR_FORMAT


def test_weighted_rms_norm_closed_form(oracle):
    rng = np.random.default_rng(5)
    v = rng.standard_normal(300).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(300)).astype(np.float32)
    rc, out = oracle.rms_norm(v, w, 1e-6)
    want = v.astype(np.float64) / np.sqrt((v.astype(np.float64) ** 2).mean() + 1e-6) * w
    assert rc == 0 and np.array_equal(out, want.astype(np.float32))
    rc, ones = oracle.rms_norm(np.full(8, 3.0, np.float32), np.ones(8, np.float32), 1e-12)
    assert rc == 0 and np.allclose(ones, 1.0, atol=1e-6)


@pytest.mark.parametrize("name,streams,width,iterations", [("wide", 4, 64, 20), ("single", 1, 32, 1)])
def test_ffn_ingress_matches_reference_fixture(oracle, golden, name, streams, width, iterations):
    """Bit-for-bit against yvex_moe_ffn_prepare_cpu of the compiled reference (moe.c:446-495):
    mixes through the CPU row dot, ingress, BF16 norm weights, weighted RMS norm, bf16 round."""
    norm = (golden[f"ingress_{name}_norm_bf16"].astype(np.uint32) << 16).view(np.float32)
    rc, normalized, post, comb = oracle.moe_ffn_prepare(
        oracle.F32, golden[f"ingress_{name}_function"].view(np.uint8), golden[f"ingress_{name}_rows"],
        golden[f"ingress_{name}_scale"], golden[f"ingress_{name}_base"], norm, streams=streams, width=width,
        iterations=iterations, rms_epsilon=1e-6, mhc_epsilon=1e-6, post_multiplier=2.0)
    assert rc == 0
    assert np.array_equal(bits(normalized), golden[f"ingress_{name}_normalized_bits"])
    assert np.array_equal(bits(post), golden[f"ingress_{name}_post_bits"])
    assert np.array_equal(bits(comb).reshape(comb.shape[0], -1), golden[f"ingress_{name}_combination_bits"])


# ---- the Q8_K-activation path: block floats, row dot, expert, layer ------------------------------
#
# The integer block sums are pinned above. What follows pins how they become floats
# (src/backend/cuda/kernel_primitives.h:312, :336-340, :353-357), how a row's block terms are
# added (double, block order: the CPU row dot's accumulation, src/gguf/quant_compute.c:152-172),
# and how route, expert and layer compose (src/graph/moe.c:587-622, src/runtime/moe.c:596-632).

F32 = np.float32


def f16_of(oracle, raw16):
    return F32(oracle.lib().yvo_f16_decode(int(raw16)))


def fma32(a, b, c):
    """float32 fused multiply-add from exact rational arithmetic, correctly rounded once."""
    from fractions import Fraction
    exact = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
    if exact == 0:
        return F32(0.0)
    # round the exact value to 24 significant bits, ties to even
    sign = -1 if exact < 0 else 1
    mag = abs(exact)
    e = mag.numerator.bit_length() - mag.denominator.bit_length()
    if Fraction(2) ** e > mag:
        e -= 1
    scaled = mag / Fraction(2) ** (e - 23)          # in [2^23, 2^24)
    whole = scaled.numerator // scaled.denominator
    rest = scaled - whole
    if rest > Fraction(1, 2) or (rest == Fraction(1, 2) and whole & 1):
        whole += 1
    return F32(sign * float(Fraction(whole) * Fraction(2) ** (e - 23)))


def block_float(oracle, qt, w_block, a_block):
    return F32(oracle.lib().yvo_block_dot_float(C.c_uint(qt), C.c_void_p(w_block.ctypes.data),
                                                C.c_void_p(a_block.ctypes.data)))


def test_fma32_helper_is_a_fused_multiply_add():
    # 1 + 2^-24 times itself: the exact product needs 49 bits; rounding the product to float first
    # loses the term the fused form keeps
    a = F32(1.0 + 2.0 ** -12)
    assert fma32(a, a, F32(-1.0)) == F32(2.0 ** -11 + 2.0 ** -24)
    assert F32(F32(a * a) + F32(-1.0)) != fma32(a, a, F32(-1.0))


@pytest.mark.parametrize("qtype", ["IQ2_XXS", "Q4_K", "Q2_K", "Q8_0"])
def test_block_float_is_the_primitives_order_of_float_operations(oracle, qtype):
    """One weight superblock against one Q8_K block: the float value is the device primitive's
    expression evaluated in float32 in its written order. Other plausible orders (scales
    multiplied first in another grouping, one rounding at the end, 0.25 for 0.125, a product in
    place of a fused multiply-add) are shown to give different bits on these inputs."""
    qt = getattr(oracle, qtype)
    g = oracle.Generator(77, f"blockfloat.{qtype}")
    wb = {"IQ2_XXS": 66, "Q4_K": 144, "Q2_K": 84, "Q8_0": 272}[qtype]
    orders_seen = set()
    for trial in range(40):
        w = g.weights(qt, 1, 256)
        assert w.size == wb
        act = oracle.q8k_quantize(g.normal(256) * (1.0 + trial))
        da = act[:4].copy().view(np.float32)[0]
        got = block_float(oracle, qt, w, act)
        sums = oracle.block_dots_i32(qt, w, 1, 256, act, 1)
        if qtype == "IQ2_XXS":
            dw = f16_of(oracle, w[:2].copy().view(np.uint16)[0])
            t = F32(int(sums[0, 0, 0, 0]))
            want = F32(F32(F32(F32(0.125) * dw) * da) * t)
            others = [F32(F32(0.125) * F32(dw * F32(da * t))), F32(0.125 * float(dw) * float(da) * float(t)),
                      F32(F32(F32(F32(0.25) * dw) * da) * t)]
        elif qtype == "Q8_0":
            want = F32(0.0)
            loose = F32(0.0)
            for b in range(8):
                d = f16_of(oracle, w[34 * b:34 * b + 2].copy().view(np.uint16)[0])
                dot = F32(int(sums[0, 0, b]))
                want = fma32(F32(d * da), dot, want)
                loose = F32(loose + F32(F32(d * da) * dot))
            others = [loose]
        else:
            head = 0 if qtype == "Q4_K" else 80
            d = f16_of(oracle, w[head:head + 2].copy().view(np.uint16)[0])
            dmin = f16_of(oracle, w[head + 2:head + 4].copy().view(np.uint16)[0])
            dot, minimum = F32(int(sums[0, 0, 0, 0])), F32(int(sums[0, 0, 0, 1]))
            want = F32(F32(F32(da * d) * dot) - F32(F32(da * dmin) * minimum))
            others = [F32(float(da) * float(d) * float(dot) - float(da) * float(dmin) * float(minimum)),
                      F32(da * F32(F32(d * dot) - F32(dmin * minimum)))]
        assert bits(got) == bits(want), (trial, got, want)
        for k, other in enumerate(others):
            if bits(other) != bits(want):
                orders_seen.add(k)
    assert orders_seen == set(range(len(others)))      # every alternative was told apart at least once


@pytest.mark.parametrize("qtype,width", [("IQ2_XXS", 7168), ("Q4_K", 2048), ("Q2_K", 1024), ("Q8_0", 2048)])
def test_q8_row_dot_adds_block_floats_in_double_in_block_order(oracle, qtype, width):
    qt = getattr(oracle, qtype)
    g = oracle.Generator(78, f"rowdot.{qtype}")
    rows, inputs = 24, 2
    w = g.weights(qt, rows, width)
    act = oracle.q8k_quantize(g.normal(inputs * width).reshape(inputs, width))
    got = oracle.q8_matvec(qt, w, rows, width, act, inputs)
    blocks = width // 256
    wb = w.size // (rows * blocks)
    differs_from_float_sum = 0
    for i in range(inputs):
        for r in range(rows):
            terms = [block_float(oracle, qt, w[(r * blocks + b) * wb:(r * blocks + b + 1) * wb],
                                 act[(i * blocks + b) * 292:(i * blocks + b + 1) * 292]) for b in range(blocks)]
            total = 0.0
            single = F32(0.0)
            for t in terms:
                total += float(t)               # Python floats are doubles: one rounded add per block
                single = F32(single + t)
            assert bits(got[i, r]).item() == bits(F32(total)).item()
            differs_from_float_sum += int(bits(single).item() != bits(F32(total)).item())
    assert differs_from_float_sum > 0          # a float accumulator would have been told apart


@pytest.mark.parametrize("qtype", ["IQ2_XXS", "Q8_0", "Q4_K", "Q2_K"])
def test_q8_matvec_against_the_float_path_on_dequantised_activations(oracle, qtype):
    """The reference's own bound for its Q8_K-activation kernels (tests/unit/cuda/quant_qtype.c:402,
    419-421): within 1e-5 (1 + |expected|) of the CPU row dot fed with the dequantised activations.
    A wrong constant, a dropped minimum term or a transposed operand is orders of magnitude outside."""
    qt = getattr(oracle, qtype)
    g = oracle.Generator(79, f"q8matvec.{qtype}")
    rows, width, inputs = 16, 2048, 3
    w = g.weights(qt, rows, width)
    act = oracle.q8k_quantize(g.normal(inputs * width).reshape(inputs, width))
    got = oracle.q8_matvec(qt, w, rows, width, act, inputs)
    want = oracle.matvec(qt, w, rows, width, oracle.q8k_dequantize(act).reshape(inputs, width))
    assert got.shape == want.shape == (inputs, rows)
    assert np.all(np.abs(got.astype(np.float64) - want) <= 1e-5 * (1.0 + np.abs(want)))
    assert np.abs(want).max() > 1e-3


def swiglu_reference(oracle, g, u, weight, limit):
    """src/graph/moe.c:605-611 in Python doubles."""
    out = np.empty(g.size, np.float32)
    for i in range(g.size):
        gv = min(float(g[i]), limit)
        uv = max(-limit, min(float(u[i]), limit))
        silu = gv / (1.0 + math.exp(-gv)) if gv >= 0.0 else gv * math.exp(gv) / (1.0 + math.exp(gv))
        out[i] = oracle.lib().yvo_bf16_round(F32(silu * uv * float(weight)))
    return out


def bf16_rounded(oracle, values):
    return np.array([oracle.lib().yvo_bf16_round(F32(v)) for v in np.ravel(values)], np.float32).reshape(np.shape(values))


def expert_from_pinned_pieces(oracle, qt, gate, up, down, hidden, inter, x, weight, limit):
    q = oracle.q8k_quantize(x)
    g = oracle.q8_matvec(qt, gate, inter, hidden, q, 1)[0]
    u = oracle.q8_matvec(qt, up, inter, hidden, q, 1)[0]
    h = swiglu_reference(oracle, g, u, weight, limit)
    out = oracle.q8_matvec(qt, down, hidden, inter, oracle.q8k_quantize(h), 1)[0]
    return h, bf16_rounded(oracle, out), out


@pytest.mark.parametrize("qtype", ["IQ2_XXS", "Q8_0"])
def test_expert_with_q8k_activations_is_the_composition_of_pinned_pieces(oracle, qtype):
    """yvo_moe_expert(act_q8) against quantize -> gate, up -> clamped SwiGLU with the route weight
    inside the rounding -> quantize -> down -> bfloat16 built from functions pinned above. The
    limit is low enough to clamp; a route weight applied after the down projection, an
    unclamped gate or a float SwiGLU would not give these bits."""
    qt = getattr(oracle, qtype)
    hidden, inter = 512, 256
    g = oracle.Generator(80, f"expert.q8.{qtype}")
    gate, up = g.weights(qt, inter, hidden), g.weights(qt, inter, hidden)
    down = g.weights(qt, hidden, inter)
    x = (g.normal(hidden) * 40.0).astype(np.float32)
    weight, limit = 0.37, 0.75
    rc, out, mid, raw = oracle.moe_expert((qt, qt, qt), gate, up, down, hidden, inter, x, weight, limit=limit,
                                          act_q8=True)
    assert rc == 0
    h, want, want_raw = expert_from_pinned_pieces(oracle, qt, gate, up, down, hidden, inter, x, weight, limit)
    q = oracle.q8k_quantize(x)
    clamped = np.abs(oracle.q8_matvec(qt, up, inter, hidden, q, 1)[0]) > limit
    assert clamped.any() and not clamped.all()
    assert np.array_equal(bits(mid), bits(h))
    assert np.array_equal(bits(out), bits(want))
    # the alternatives are different numbers here
    late = bf16_rounded(oracle, oracle.q8_matvec(
        qt, down, hidden, inter, oracle.q8k_quantize(swiglu_reference(oracle, *(
            oracle.q8_matvec(qt, m, inter, hidden, q, 1)[0] for m in (gate, up)), 1.0, limit)), 1)[0] * F32(weight))
    assert not np.array_equal(bits(late), bits(want))


def test_layer_is_route_then_experts_in_rank_order_then_shared(oracle):
    """yvo_moe_layer against the composition src/runtime/moe.c:596-632 writes: route, one expert per
    rank added to a float row, the shared expert with weight 1, bfloat16 of the float sum routed +
    shared. (The experts' outputs are bfloat16 values, a handful of which add exactly in float, so
    the order of the ranks is not observable on such data.) Plausible slips give other bits here
    and the test shows that they do: the routed sum rounded to bfloat16 before the shared expert
    is added, the shared expert weighted like a routed one, the last rounding left out."""
    qt = oracle.IQ2_XXS
    hidden, inter, experts, topk, rows = 512, 256, 8, 4, 3
    g = oracle.Generator(81, "layer.q8")
    gate, up = g.weights(qt, experts * inter, hidden), g.weights(qt, experts * inter, hidden)
    down = g.weights(qt, experts * hidden, inter)
    shared = (g.weights(qt, inter, hidden), g.weights(qt, inter, hidden), g.weights(qt, hidden, inter))
    x = g.normal(rows * hidden).reshape(rows, hidden)
    logits = g.normal(rows * experts).reshape(rows, experts)
    bias = (g.normal(experts) * 0.05).astype(np.float32)
    got = oracle.moe_layer(hidden=hidden, intermediate=inter, experts=experts, topk=topk, qtypes=(qt, qt, qt),
                           routed=(gate, up, down), shared=shared, inputs=x, logits=logits, bias=bias,
                           scoring=oracle.SIGMOID, normalize=True, scaling=1.5, limit=10.0, act_q8=True)
    gb, db = oracle.row_bytes(qt, hidden) * inter, oracle.row_bytes(qt, inter) * hidden
    order_matters = 0
    for r in range(rows):
        rc, sel, w, _ = oracle.moe_route(logits[r], bias, topk, oracle.SIGMOID, True, 1.5)
        assert rc == 0 and np.array_equal(sel, got["selected"][r]) and np.array_equal(bits(w), bits(got["weights"][r]))
        outs = []
        for rank in range(topk):
            e = int(sel[rank])
            _, out, _ = expert_from_pinned_pieces(oracle, qt, gate[e * gb:(e + 1) * gb], up[e * gb:(e + 1) * gb],
                                                  down[e * db:(e + 1) * db], hidden, inter, x[r], w[rank], 10.0)
            outs.append(out)
        routed = np.zeros(hidden, np.float32)
        for out in outs:
            routed = (routed + out).astype(np.float32)
        _, shared_out, _ = expert_from_pinned_pieces(oracle, qt, *shared, hidden, inter, x[r], 1.0, 10.0)
        assert np.array_equal(bits(got["routed"][r]), bits(routed))
        assert np.array_equal(bits(got["shared"][r]), bits(shared_out))
        assert np.array_equal(bits(got["combined"][r]), bits(bf16_rounded(oracle, (routed + shared_out).astype(np.float32))))
        early = (bf16_rounded(oracle, routed) + shared_out).astype(np.float32)
        _, weighted_shared, _ = expert_from_pinned_pieces(oracle, qt, *shared, hidden, inter, x[r], w[0], 10.0)
        order_matters += int(not np.array_equal(bits(bf16_rounded(oracle, early)), bits(got["combined"][r])))
        order_matters += int(not np.array_equal(bits(weighted_shared), bits(got["shared"][r])))
        order_matters += int(not np.array_equal(bits((routed + shared_out).astype(np.float32)), bits(got["combined"][r])))
    assert order_matters == 3 * rows
