"""ctypes binding of the CPU oracle (test infrastructure only).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` import this
package, and only to check or to time the CPU path. The shipped library never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libyvex_oracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libyvex_ref.so")
REF_BACKEND_PATH = os.path.join(HERE, "_ref", "libyvex_ref_backend.so")

OK, ERR_FORMAT, ERR_UNSUPPORTED, ERR_BOUNDS, ERR_INVALID_ARG = 0, -4, -5, -7, -10
F32, F16, Q8_0, Q2_K, Q4_K, Q8_K, IQ2_XXS, I32, BF16, MXFP4 = 0, 1, 8, 10, 12, 15, 16, 26, 30, 39
SQRT_SOFTPLUS, SIGMOID = 0, 1

u8p = C.POINTER(C.c_uint8)
f32p = C.POINTER(C.c_float)
u64p = C.POINTER(C.c_uint64)
u32p = C.POINTER(C.c_uint32)
i32p = C.POINTER(C.c_int32)


def build(force: bool = False) -> None:
    """Compile the restatement (and oracle/_ref when the reference tree is present)."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.run(["make", "-C", HERE, "oracle"], check=True, capture_output=True)
    if os.path.isdir("/root/reference/src/gguf") and (force or not os.path.exists(REF_PATH)):
        subprocess.run(["make", "-C", HERE, "ref"], check=True, capture_output=True)
    rocm_lib = os.path.join(os.path.dirname(HERE), "yvex_amd", "libyvex_rocm.so")
    if os.path.isdir("/root/reference/src/backend") and os.path.exists(rocm_lib) and (
            force or not os.path.exists(REF_BACKEND_PATH) or
            os.path.getmtime(REF_BACKEND_PATH) < os.path.getmtime(rocm_lib)):
        subprocess.run(["make", "-C", HERE, "ref_backend"], check=True, capture_output=True)


class MoeLayerArgs(C.Structure):
    _fields_ = [
        ("hidden", C.c_uint64), ("intermediate", C.c_uint64), ("experts", C.c_uint64),
        ("topk", C.c_uint64), ("rows", C.c_uint64),
        ("gate_qtype", C.c_uint), ("up_qtype", C.c_uint), ("down_qtype", C.c_uint),
        ("routed_gate", C.c_void_p), ("routed_up", C.c_void_p), ("routed_down", C.c_void_p),
        ("shared_gate", C.c_void_p), ("shared_up", C.c_void_p), ("shared_down", C.c_void_p),
        ("router_bias", C.c_void_p),
        ("scoring", C.c_int), ("normalize", C.c_int), ("act_q8", C.c_int),
        ("scaling", C.c_double), ("activation_limit", C.c_double),
        ("threads", C.c_uint), ("hash_selected", C.c_void_p),
    ]


class Rng(C.Structure):
    _fields_ = [("s", C.c_uint64 * 4)]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.yvo_f16_decode.restype = C.c_float
        L.yvo_f16_decode.argtypes = [C.c_uint16]
        L.yvo_f16_encode.restype = C.c_uint16
        L.yvo_f16_encode.argtypes = [C.c_float]
        L.yvo_bf16_decode.restype = C.c_float
        L.yvo_bf16_decode.argtypes = [C.c_uint16]
        L.yvo_bf16_encode.restype = C.c_uint16
        L.yvo_bf16_encode.argtypes = [C.c_float]
        L.yvo_bf16_round.restype = C.c_float
        L.yvo_bf16_round.argtypes = [C.c_float]
        L.yvo_block_dot_iq2xxs_q8k.restype = C.c_int32
        L.yvo_block_dot_float.restype = C.c_float
        L.yvo_block_dot_float.argtypes = [C.c_uint, C.c_void_p, C.c_void_p]
        L.yvo_rng_uniform.restype = C.c_double
        L.yvo_rng_next.restype = C.c_uint64
        for name in ("yvo_rng_normal_f32",):
            getattr(L, name).argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_double]
        L.yvo_fill_iq2xxs.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_double]
        L.yvo_fill_q4k.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_double]
        L.yvo_fill_q8_0_from_normal.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_double]
        L.yvo_rng_bytes.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64]
        L.yvo_rng_seed.argtypes = [C.c_void_p, C.c_uint64, C.c_char_p]
        _lib = L
    return _lib


def ref_backend_lib():
    """The reference's generic backend code (src/backend/core.c, residency.c) linked with the ROCm
    adapter and libyvex_rocm.so, or None where it cannot exist. Load torch first in a process
    that will use the GPU (it carries its own copy of the HIP runtime)."""
    if not os.path.exists(REF_BACKEND_PATH):
        if os.path.isdir("/root/reference/src/backend"):
            build()
        if not os.path.exists(REF_BACKEND_PATH):
            return None
    return C.CDLL(REF_BACKEND_PATH)


def ref_lib():
    """The library compiled from the reference's own sources, or None where it cannot exist."""
    if not os.path.exists(REF_PATH):
        if os.path.isdir("/root/reference/src/gguf"):
            build()
        if not os.path.exists(REF_PATH):
            return None
    return C.CDLL(REF_PATH)


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def geometry(qtype: int):
    b, n = C.c_uint(), C.c_uint()
    if not lib().yvo_qtype_geometry(C.c_uint(qtype), C.byref(b), C.byref(n)):
        return None
    return b.value, n.value


def row_bytes(qtype: int, width: int) -> int:
    block, nbytes = geometry(qtype)
    assert width % block == 0
    return width // block * nbytes


# ---- synthetic data -------------------------------------------------------------------------

class Generator:
    """splitmix64-seeded xoshiro256**; one sub-stream per tensor name."""

    def __init__(self, seed: int, name: str):
        self.state = Rng()
        lib().yvo_rng_seed(C.byref(self.state), C.c_uint64(seed), name.encode())

    def normal(self, count: int, sigma: float = 1.0) -> np.ndarray:
        out = np.empty(count, np.float32)
        lib().yvo_rng_normal_f32(C.byref(self.state), _p(out), count, sigma)
        return out

    def bytes(self, count: int) -> np.ndarray:
        out = np.empty(count, np.uint8)
        lib().yvo_rng_bytes(C.byref(self.state), _p(out), count)
        return out

    def iq2xxs(self, blocks: int, scale_sigma: float = 3.5e-4) -> np.ndarray:
        out = np.empty(blocks * 66, np.uint8)
        lib().yvo_fill_iq2xxs(C.byref(self.state), _p(out), blocks, scale_sigma)
        return out

    def q4k(self, blocks: int, scale_sigma: float = 1.0e-4) -> np.ndarray:
        out = np.empty(blocks * 144, np.uint8)
        lib().yvo_fill_q4k(C.byref(self.state), _p(out), blocks, scale_sigma)
        return out

    def q8_0(self, blocks: int, sigma: float = 0.02) -> np.ndarray:
        out = np.empty(blocks * 34, np.uint8)
        lib().yvo_fill_q8_0_from_normal(C.byref(self.state), _p(out), blocks, sigma)
        return out

    def weights(self, qtype: int, rows: int, width: int) -> np.ndarray:
        block, _ = geometry(qtype)
        blocks = rows * width // block
        if qtype == IQ2_XXS:
            return self.iq2xxs(blocks)
        if qtype == Q4_K:
            return self.q4k(blocks)
        if qtype == Q8_0:
            return self.q8_0(blocks)
        if qtype == F32:
            return self.normal(rows * width, 0.02).view(np.uint8)
        if qtype == Q2_K:
            out = self.bytes(blocks * 84)
            v = out.reshape(blocks, 84)
            for b in range(blocks):
                for off in (80, 82):
                    bits = int(lib().yvo_f16_encode(C.c_float((0.004 + 0.002 * ((b + off) % 7)) * (1.0 if off == 80 else 1.5))))
                    v[b, off] = bits & 255
                    v[b, off + 1] = bits >> 8
            return out
        raise ValueError(qtype)


# ---- numerical entry points ------------------------------------------------------------------

def decode_rows(qtype: int, encoded: np.ndarray, width: int, row_ids=None) -> np.ndarray:
    rb = row_bytes(qtype, width)
    if row_ids is None:
        count = encoded.size // rb
        ids = None
    else:
        ids = np.ascontiguousarray(row_ids, np.uint32)
        count = ids.size
    out = np.empty((count, width), np.float32)
    rc = lib().yvo_decode_rows(C.c_uint(qtype), _p(encoded), C.c_uint64(width),
                               _p(ids) if ids is not None else None, C.c_uint64(count), _p(out))
    if rc:
        raise RuntimeError(f"yvo_decode_rows rc={rc}")
    return out


def cpu_dot(qtype: int, encoded: np.ndarray, vector: np.ndarray):
    out = C.c_float()
    rc = lib().yvo_cpu_dot(C.c_uint(qtype), _p(encoded), C.c_size_t(encoded.size),
                           _p(vector), C.c_uint64(vector.size), C.byref(out))
    return rc, out.value


def matvec(qtype: int, encoded: np.ndarray, rows: int, width: int, inputs: np.ndarray,
           threads: int = 1) -> np.ndarray:
    inputs = np.ascontiguousarray(inputs, np.float32).reshape(-1, width)
    out = np.empty((inputs.shape[0], rows), np.float32)
    rc = lib().yvo_matvec_threads(C.c_uint(qtype), _p(encoded), C.c_uint64(rows),
                                  C.c_uint64(width), _p(inputs), C.c_uint64(inputs.shape[0]),
                                  _p(out), C.c_uint(threads))
    if rc:
        raise RuntimeError(f"yvo_matvec rc={rc}")
    return out


def q8k_quantize(values: np.ndarray) -> np.ndarray:
    values = np.ascontiguousarray(values, np.float32)
    rows, width = (1, values.size) if values.ndim == 1 else values.shape
    out = np.empty(rows * (width // 256) * 292, np.uint8)
    rc = lib().yvo_q8k_quantize(_p(values), C.c_uint64(rows), C.c_uint64(width), _p(out))
    if rc:
        raise RuntimeError(f"yvo_q8k_quantize rc={rc}")
    return out


def q8k_dequantize(encoded: np.ndarray) -> np.ndarray:
    blocks = encoded.size // 292
    out = np.empty(blocks * 256, np.float32)
    lib().yvo_q8k_dequantize(_p(encoded), C.c_uint64(blocks), _p(out))
    return out


def q8_matvec(qtype: int, encoded: np.ndarray, rows: int, width: int, act: np.ndarray,
              input_rows: int) -> np.ndarray:
    out = np.empty((input_rows, rows), np.float32)
    rc = lib().yvo_q8_matvec(C.c_uint(qtype), _p(encoded), C.c_uint64(rows), C.c_uint64(width),
                             _p(act), C.c_uint64(input_rows), _p(out))
    if rc:
        raise RuntimeError(f"yvo_q8_matvec rc={rc}")
    return out


def block_dots_i32(qtype: int, encoded: np.ndarray, rows: int, width: int, act: np.ndarray,
                   input_rows: int) -> np.ndarray:
    """int32 block sums [input_rows, rows, blocks, 2]; slot 1 is the min-sum (0 where unused).

    For Q8_0 the eight 32-value sums of one 256 block are returned as [.., blocks*8] in slot 0
    of an array with last dimension 1.
    """
    L = lib()
    blocks = width // 256
    wb = {IQ2_XXS: 66, Q4_K: 144, Q2_K: 84, Q8_0: 272}[qtype]
    if qtype == Q8_0:
        out = np.zeros((input_rows, rows, blocks * 8), np.int32)
    else:
        out = np.zeros((input_rows, rows, blocks, 2), np.int32)
    base_w = encoded.ctypes.data
    base_a = act.ctypes.data
    for i in range(input_rows):
        for r in range(rows):
            for b in range(blocks):
                w = C.c_void_p(base_w + (r * blocks + b) * wb)
                a = C.c_void_p(base_a + (i * blocks + b) * 292)
                if qtype == IQ2_XXS:
                    out[i, r, b, 0] = L.yvo_block_dot_iq2xxs_q8k(w, a)
                elif qtype == Q8_0:
                    d = (C.c_int32 * 8)()
                    L.yvo_block_dot_q8_0_q8k(w, a, d)
                    out[i, r, 8 * b:8 * b + 8] = list(d)
                else:
                    d, m = C.c_int32(), C.c_int32()
                    fn = L.yvo_block_dot_q4k_q8k if qtype == Q4_K else L.yvo_block_dot_q2k_q8k
                    fn(w, a, C.byref(d), C.byref(m))
                    out[i, r, b] = (d.value, m.value)
    return out


def moe_route(logits: np.ndarray, bias, topk: int, scoring: int, normalize: bool, scaling: float):
    logits = np.ascontiguousarray(logits, np.float32)
    experts = logits.size
    sel = np.empty(topk, np.uint64)
    w = np.empty(topk, np.float32)
    scores = np.empty(experts, np.float32)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    rc = lib().yvo_moe_route(_p(logits), _p(b) if b is not None else None, C.c_uint64(experts),
                             C.c_uint64(topk), C.c_int(scoring), C.c_int(int(normalize)),
                             C.c_double(scaling), _p(scores), _p(sel), _p(w))
    return rc, sel, w, scores


def moe_route_hash(logits: np.ndarray, table: np.ndarray, token: int, topk: int, scoring: int,
                   normalize: bool, scaling: float):
    """Hash router: table is [rows, columns] int32 (columns >= topk)."""
    logits = np.ascontiguousarray(logits, np.float32)
    table = np.ascontiguousarray(table, np.int32).reshape(-1, np.asarray(table).shape[-1])
    sel, w = np.zeros(topk, np.uint64), np.zeros(topk, np.float32)
    scores = np.empty(logits.size, np.float32)
    rc = lib().yvo_moe_route_hash(_p(logits), _p(table), C.c_uint64(table.shape[0]),
                                  C.c_uint64(table.shape[1] * 4), C.c_uint64(token), C.c_uint64(logits.size),
                                  C.c_uint64(topk), C.c_int(scoring), C.c_int(int(normalize)),
                                  C.c_double(scaling), _p(scores), _p(sel), _p(w))
    return rc, sel, w, scores


def moe_expert(qtypes, gate, up, down, hidden, intermediate, x, route_weight, limit=10.0,
               act_q8=False):
    gq, uq, dq = qtypes
    out = np.empty(hidden, np.float32)
    mid = np.empty(intermediate, np.float32)
    raw = np.empty(hidden, np.float32)
    x = np.ascontiguousarray(x, np.float32)
    rc = lib().yvo_moe_expert(C.c_uint(gq), _p(gate), C.c_uint(uq), _p(up), C.c_uint(dq), _p(down),
                              C.c_uint64(hidden), C.c_uint64(intermediate), _p(x),
                              C.c_float(route_weight), C.c_double(limit), C.c_int(int(act_q8)),
                              _p(out), _p(mid), _p(raw))
    return rc, out, mid, raw


def argmax_f32(values: np.ndarray):
    """Per row of a [rows, width] float32 array: status (1 if a row held a non-finite value),
    tokens u32, values f32, tie counts u64 (kernels.cu:59-110)."""
    values = np.ascontiguousarray(values, np.float32)
    rows, width = values.shape
    tokens = np.zeros(rows, np.uint32)
    best = np.zeros(rows, np.float32)
    ties = np.zeros(rows, np.uint64)
    rc = lib().yvo_argmax_f32(_p(values), C.c_uint64(rows), C.c_uint64(width), _p(tokens), _p(best), _p(ties))
    return rc, tokens, best, ties


def worklist_build(selected: np.ndarray, weights: np.ndarray, topk: int, experts: int):
    selected = np.ascontiguousarray(selected, np.uint64).ravel()
    weights = np.ascontiguousarray(weights, np.float32).ravel()
    pairs = selected.size
    ids = np.zeros(experts, np.uint64)
    off = np.zeros(experts + 1, np.uint64)
    pop = np.zeros(experts, np.uint64)
    sp = np.zeros(pairs, np.uint64)
    sr = np.zeros(pairs, np.uint64)
    dr = np.zeros(pairs, np.uint64)
    ow = np.zeros(pairs, np.float32)
    n = C.c_uint64()
    rc = lib().yvo_worklist_build(_p(selected), _p(weights), C.c_uint64(pairs), C.c_uint64(topk),
                                  C.c_uint64(experts), _p(ids), _p(off), _p(pop), _p(sp), _p(sr),
                                  _p(dr), _p(ow), C.byref(n))
    k = n.value
    return rc, dict(expert_ids=ids[:k], bucket_offsets=off[:k + 1], bucket_populations=pop[:k],
                    source_pairs=sp, source_rows=sr, destination_rows=dr, route_weights=ow)


def rms_norm(values: np.ndarray, weights: np.ndarray, epsilon: float):
    """numeric.c:630-666 on one vector; returns (rc, normalised copy)."""
    out = np.array(values, np.float32).ravel()
    weights = np.ascontiguousarray(weights, np.float32).ravel()
    rc = lib().yvo_rms_norm(_p(out), C.c_uint64(out.size), _p(weights), C.c_double(epsilon))
    return rc, out


def mhc_pre(residual, mixes, scale, base, *, streams, width, iterations, rms_epsilon, mhc_epsilon,
            post_multiplier):
    """numeric.c:752-826: (rc, collapsed [t, width], post [t, streams], combination [t, s, s])."""
    residual = np.ascontiguousarray(residual, np.float32).reshape(-1, streams * width)
    tokens = residual.shape[0]
    mixes = np.ascontiguousarray(mixes, np.float32).reshape(tokens, (streams + 2) * streams)
    scale = np.ascontiguousarray(scale, np.float32).ravel()
    base = np.ascontiguousarray(base, np.float32).ravel()
    collapsed = np.zeros((tokens, width), np.float32)
    post = np.zeros((tokens, streams), np.float32)
    comb = np.zeros((tokens, streams, streams), np.float32)
    rc = lib().yvo_mhc_pre(_p(residual), _p(mixes), _p(scale), _p(base), C.c_uint64(tokens),
                           C.c_uint64(streams), C.c_uint64(width), C.c_uint64(iterations),
                           C.c_double(rms_epsilon), C.c_double(mhc_epsilon),
                           C.c_double(post_multiplier), _p(collapsed), _p(post), _p(comb))
    return rc, collapsed, post, comb


def mhc_post(core, residual, post, combination, *, streams, width):
    """numeric.c:828-877: (rc, envelope output [t, streams * width])."""
    core = np.ascontiguousarray(core, np.float32).reshape(-1, width)
    tokens = core.shape[0]
    residual = np.ascontiguousarray(residual, np.float32).reshape(tokens, streams * width)
    post = np.ascontiguousarray(post, np.float32).reshape(tokens, streams)
    combination = np.ascontiguousarray(combination, np.float32).reshape(tokens, streams * streams)
    out = np.zeros((tokens, streams * width), np.float32)
    rc = lib().yvo_mhc_post(_p(core), _p(residual), _p(post), _p(combination), C.c_uint64(tokens),
                            C.c_uint64(streams), C.c_uint64(width), _p(out))
    return rc, out


def moe_ffn_prepare(function_qtype, function, expanded, scale, base, norm, *, streams, width,
                    iterations, rms_epsilon, mhc_epsilon, post_multiplier):
    """moe.c:446-495: (rc, normalized [t, width], post [t, streams], combination [t, s, s])."""
    function = np.ascontiguousarray(function, np.uint8)
    expanded = np.ascontiguousarray(expanded, np.float32).reshape(-1, streams * width)
    tokens = expanded.shape[0]
    scale = np.ascontiguousarray(scale, np.float32).ravel()
    base = np.ascontiguousarray(base, np.float32).ravel()
    norm = np.ascontiguousarray(norm, np.float32).ravel()
    normalized = np.zeros((tokens, width), np.float32)
    post = np.zeros((tokens, streams), np.float32)
    comb = np.zeros((tokens, streams, streams), np.float32)
    rc = lib().yvo_moe_ffn_prepare(C.c_uint(function_qtype), _p(function), _p(expanded), _p(scale),
                                   _p(base), _p(norm), C.c_uint64(tokens), C.c_uint64(streams),
                                   C.c_uint64(width), C.c_uint64(iterations), C.c_double(rms_epsilon),
                                   C.c_double(mhc_epsilon), C.c_double(post_multiplier),
                                   _p(normalized), _p(post), _p(comb))
    return rc, normalized, post, comb


def moe_layer(*, hidden, intermediate, experts, topk, qtypes, routed, shared, inputs, logits,
              bias=None, scoring=SQRT_SOFTPLUS, normalize=True, scaling=1.0, limit=10.0,
              act_q8=False, threads=1, hash_selected=None):
    inputs = np.ascontiguousarray(inputs, np.float32).reshape(-1, hidden)
    logits = np.ascontiguousarray(logits, np.float32).reshape(-1, experts)
    rows = inputs.shape[0]
    a = MoeLayerArgs()
    a.hidden, a.intermediate, a.experts, a.topk, a.rows = hidden, intermediate, experts, topk, rows
    a.gate_qtype, a.up_qtype, a.down_qtype = qtypes
    keep = [np.ascontiguousarray(t, np.uint8) for t in routed]
    a.routed_gate, a.routed_up, a.routed_down = (t.ctypes.data for t in keep)
    if shared is not None:
        keep_s = [np.ascontiguousarray(t, np.uint8) for t in shared]
        a.shared_gate, a.shared_up, a.shared_down = (t.ctypes.data for t in keep_s)
    b = None if bias is None else np.ascontiguousarray(bias, np.float32)
    a.router_bias = b.ctypes.data if b is not None else None
    a.scoring, a.normalize, a.act_q8 = scoring, int(normalize), int(act_q8)
    a.scaling, a.activation_limit, a.threads = scaling, limit, threads
    forced = None if hash_selected is None else np.ascontiguousarray(hash_selected, np.int32).reshape(rows, topk)
    a.hash_selected = forced.ctypes.data if forced is not None else None
    sel = np.empty((rows, topk), np.uint64)
    w = np.empty((rows, topk), np.float32)
    routed_out = np.empty((rows, hidden), np.float32)
    shared_out = np.empty((rows, hidden), np.float32)
    combined = np.empty((rows, hidden), np.float32)
    rc = lib().yvo_moe_layer(C.byref(a), _p(inputs), _p(logits), _p(sel), _p(w), _p(routed_out),
                             _p(shared_out), _p(combined))
    if rc:
        raise RuntimeError(f"yvo_moe_layer rc={rc}")
    return dict(selected=sel, weights=w, routed=routed_out, shared=shared_out, combined=combined)


def _align64(n: int) -> int:
    return (n + 63) & ~63


def derived_layout_plan(qtype: int, row_count: int, row_width: int, expert_count: int) -> int:
    """Bytes of the derived image of one routed expert tensor (src/backend/cuda/layout.c:23-93).

    numpy restatement; raises ValueError where the reference refuses the geometry."""
    if expert_count <= 1 or row_count % expert_count or row_width % 256:
        raise ValueError("incomplete decision")
    blocks = row_count * (row_width // 256)
    if qtype == IQ2_XXS:
        return _align64(2 * blocks) + 64 * blocks
    if qtype == Q2_K:
        if (row_count // expert_count) % 2:
            raise ValueError("odd rows per expert")
        units = blocks // 2
        return _align64(_align64(8 * units) + 32 * units) + 128 * units
    raise ValueError("qtype not admitted")


def derived_layout_build(qtype: int, canonical, row_count: int, row_width: int, expert_count: int) -> np.ndarray:
    """The derived image itself (src/backend/cuda/layout.c:112-167), by reshapes and transposes.

    IQ2_XXS: column 0:2 of the [blocks, 66] byte matrix, then (64-aligned) columns 2:66.
    Q2_K: [row pair, parity, block, 84] -> per (pair, block): bytes 80:84 of both rows; scale bytes
    as [half, parity, 8]; code bytes as [word, parity, 4]."""
    canonical = np.ascontiguousarray(canonical, np.uint8).ravel()
    total = derived_layout_plan(qtype, row_count, row_width, expert_count)
    per_row = row_width // 256
    out = np.zeros(total, np.uint8)
    if qtype == IQ2_XXS:
        blocks = canonical.reshape(row_count * per_row, 66)
        out[:2 * len(blocks)] = blocks[:, :2].ravel()
        start = _align64(2 * len(blocks))
        out[start:] = blocks[:, 2:].ravel()
        return out
    blocks = canonical.reshape(row_count // 2, 2, per_row, 84)          # [pair, parity, block, byte]
    units = (row_count // 2) * per_row
    factors = blocks[..., 80:84].transpose(0, 2, 1, 3)                  # [pair, block, parity, 4]
    scales = blocks[..., 0:16].reshape(row_count // 2, 2, per_row, 2, 8).transpose(0, 2, 3, 1, 4)
    codes = blocks[..., 16:80].reshape(row_count // 2, 2, per_row, 16, 4).transpose(0, 2, 3, 1, 4)
    out[:8 * units] = factors.ravel()
    second = _align64(8 * units)
    out[second:second + 32 * units] = scales.ravel()
    third = _align64(second + 32 * units)
    out[third:] = codes.ravel()
    return out
