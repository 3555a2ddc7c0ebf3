"""GGUF tensor directory reader and resident loading (yvex_rocm_gguf_open_path,
yvex_rocm_gguf_resident_load, yvex_rocm_gguf_weight_view) against the reference's
structural rules (src/gguf/core.c:850-1250) — live against the reader compiled from the
reference's sources where oracle/_ref exists, and against the outcomes written down here from it."""
import ctypes as C
import os

import numpy as np
import pytest

import gguf_writer as W
from yvex_amd import abi

IQ2_XXS, Q8_0, F32, BF16 = 16, 8, 0, 30


def sample(oracle, alignment=64):
    g = oracle.Generator(42, "gguf.sample")
    gate = g.weights(oracle.IQ2_XXS, 4 * 256, 512)          # [512, 256, 4]: expert-major rows
    down = g.weights(oracle.IQ2_XXS, 4 * 512, 256)          # [256, 512, 4]
    head = g.weights(oracle.Q8_0, 300, 512)                 # [512, 300]
    norm = g.normal(512)
    meta = [("general.architecture", W.STRING, "deepseek4"), ("general.alignment", W.U32, alignment),
            ("deepseek4.expert_count", W.U32, 4), ("deepseek4.rope.scale", W.F32, 0.25),
            ("deepseek4.flag", W.BOOL, 1), ("deepseek4.big", W.U64, 1 << 40),
            ("deepseek4.negative", W.I32, -3),
            ("tokenizer.ggml.tokens", W.ARRAY, (W.STRING, ["a", "bc", ""])),
            ("tokenizer.ggml.scores", W.ARRAY, (W.F32, [0.5, 1.5])),
            ("tokenizer.nested", W.ARRAY, (W.ARRAY, [(W.U8, [1, 2]), (W.U8, [])]))]
    tensors = [("blk.3.ffn_gate_exps.weight", [512, 256, 4], IQ2_XXS, gate.tobytes()),
               ("blk.3.ffn_down_exps.weight", [256, 512, 4], IQ2_XXS, down.tobytes()),
               ("output.weight", [512, 300], Q8_0, head.tobytes()),
               ("blk.3.ffn_norm.weight", [512], F32, norm.tobytes())]
    return meta, tensors, dict(gate=gate, down=down, head=head, norm=norm)


def write(tmp_path, name, data):
    path = os.path.join(str(tmp_path), name)
    with open(path, "wb") as f:
        f.write(data)
    return path.encode()


def open_ours(lib, path):
    handle, err = C.c_void_p(), abi.Error()
    rc = lib.yvex_rocm_gguf_open_path(C.byref(handle), path, C.byref(err))
    return rc, handle, err


def open_reference(ref, path):
    class Options(C.Structure):
        _fields_ = [("path", C.c_char_p), ("readonly", C.c_int), ("map", C.c_int)]
    artifact, handle, err = C.c_void_p(), C.c_void_p(), abi.Error()
    options = Options(path, 1, 0)
    ref.yvex_artifact_open.argtypes = [C.POINTER(C.c_void_p), C.POINTER(Options), C.c_void_p]
    assert ref.yvex_artifact_open(C.byref(artifact), C.byref(options), C.byref(err)) == 0
    ref.yvex_gguf_open.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p]
    rc = ref.yvex_gguf_open(C.byref(handle), artifact, C.byref(err))
    return rc, handle, artifact


def directory(lib, handle, prefix="yvex_rocm_gguf_"):
    """The tensor directory through one library's reader: ours (yvex_rocm_gguf_*) or the
    reference's own (yvex_gguf_*), whose accessors have the same signatures."""
    count, at = getattr(lib, prefix + "tensor_count"), getattr(lib, prefix + "tensor_at")
    data_offset, alignment = getattr(lib, prefix + "tensor_data_offset"), getattr(lib, prefix + "alignment")
    count.restype, count.argtypes = abi.ULL, [C.c_void_p]
    at.restype, at.argtypes = C.POINTER(abi.GgufTensorInfo), [C.c_void_p, abi.ULL]
    data_offset.restype, data_offset.argtypes = abi.ULL, [C.c_void_p]
    alignment.restype, alignment.argtypes = C.c_uint, [C.c_void_p]
    rows = []
    for i in range(count(handle)):
        t = at(handle, i).contents
        rows.append((t.name, t.rank, tuple(t.dims[:t.rank]), t.ggml_type, t.relative_offset,
                     t.absolute_offset, t.storage_bytes, t.absolute_end_offset, t.range_addressable))
    return rows, data_offset(handle), alignment(handle)


@pytest.fixture
def lib():
    return abi.library()


def test_directory_of_a_well_formed_file(lib, oracle, tmp_path):
    meta, tensors, _ = sample(oracle)
    data, relative, start = W.build(meta, tensors, alignment=64)
    path = write(tmp_path, "ok.gguf", data)
    rc, handle, err = open_ours(lib, path)
    assert rc == 0, err.message
    rows, data_offset, alignment = directory(lib, handle)
    assert alignment == 64 and data_offset == start and start % 64 == 0
    assert lib.yvex_rocm_gguf_file_size(handle) == len(data) and lib.yvex_rocm_gguf_metadata_count(handle) == len(meta)
    for row, (name, dims, qtype, blob), offset in zip(rows, tensors, relative):
        assert row == (name.encode(), len(dims), tuple(dims), qtype, offset, start + offset, len(blob),
                       start + offset + len(blob), 1)
    found = lib.yvex_rocm_gguf_tensor_find(handle, b"output.weight")
    assert found and found.contents.ggml_type == Q8_0 and found.contents.ggml_type_name == b"Q8_0"
    assert not lib.yvex_rocm_gguf_tensor_find(handle, b"output.bias")
    value, real, text, length = abi.ULL(), C.c_double(), C.c_char_p(), abi.ULL()
    assert lib.yvex_rocm_gguf_metadata_u64(handle, b"deepseek4.expert_count", C.byref(value)) == 0 and value.value == 4
    assert lib.yvex_rocm_gguf_metadata_u64(handle, b"deepseek4.big", C.byref(value)) == 0 and value.value == 1 << 40
    assert lib.yvex_rocm_gguf_metadata_u64(handle, b"deepseek4.flag", C.byref(value)) == 0 and value.value == 1
    assert lib.yvex_rocm_gguf_metadata_u64(handle, b"deepseek4.negative", C.byref(value)) == abi.BOUNDS
    assert lib.yvex_rocm_gguf_metadata_u64(handle, b"general.architecture", C.byref(value)) == abi.FORMAT
    assert lib.yvex_rocm_gguf_metadata_f64(handle, b"deepseek4.rope.scale", C.byref(real)) == 0 and real.value == 0.25
    assert lib.yvex_rocm_gguf_metadata_string(handle, b"general.architecture", C.byref(text), C.byref(length)) == 0
    assert text.value == b"deepseek4" and length.value == 9
    assert lib.yvex_rocm_gguf_metadata_string(handle, b"missing.key", C.byref(text), None) == abi.FORMAT
    ref = oracle.ref_lib()
    if ref is not None:      # the reference's own reader sees the same directory
        rc, theirs, artifact = open_reference(ref, path)
        assert rc == 0
        assert directory(ref, theirs, "yvex_gguf_") == (rows, data_offset, alignment)
        ref.yvex_gguf_close(C.c_void_p(theirs.value))
        ref.yvex_artifact_close(C.c_void_p(artifact.value))
    lib.yvex_rocm_gguf_close(handle)


# (case, expected status): outcomes of the reference's reader (src/gguf/core.c:52-79 maps them)
def refusal_cases(oracle):
    meta, tensors, _ = sample(oracle, alignment=32)
    ok, relative, start = W.build(meta, tensors)
    swap = lambda i, t: tensors[:i] + [t] + tensors[i + 1:]
    name, dims, qtype, blob = tensors[3]
    return [
        ("magic", W.build(meta, tensors, magic=0x46554746)[0], abi.FORMAT),
        ("version-2", W.build(meta, tensors, version=2)[0], abi.UNSUPPORTED),
        ("short-header", ok[:20], abi.BOUNDS),
        ("truncated-directory", ok[:start - 40], abi.BOUNDS),
        ("misaligned-offset", W.build(meta, tensors, offsets=[r + 8 for r in relative])[0], abi.FORMAT),
        ("duplicate-name", W.build(meta, swap(3, (tensors[2][0], dims, qtype, blob)))[0], abi.FORMAT),
        ("empty-name", W.build(meta, swap(3, ("", dims, qtype, blob)))[0], abi.FORMAT),
        ("zero-dimension", W.build(meta, swap(3, (name, [0], qtype, blob)))[0], abi.FORMAT),
        ("rank-5", W.build(meta, swap(3, (name, [2, 2, 2, 2, 32], qtype, blob)))[0], abi.FORMAT),
        ("unknown-qtype", W.build(meta, swap(3, (name, dims, 77, blob)))[0], abi.UNSUPPORTED),
        ("removed-qtype", W.build(meta, swap(3, (name, dims, 4, blob)))[0], abi.UNSUPPORTED),
        ("alignment-zero", W.build([("general.alignment", W.U32, 0)] + meta[2:], tensors)[0], abi.FORMAT),
        ("alignment-u64", W.build([("general.alignment", W.U64, 32)] + meta[2:], tensors)[0], abi.FORMAT),
        ("bad-key", W.build(meta + [("General.Name", W.U32, 1)], tensors)[0], abi.FORMAT),
        ("duplicate-key", W.build(meta + [("deepseek4.flag", W.U32, 1)], tensors)[0], abi.FORMAT),
        ("metadata-type", W.build(meta, tensors)[0].replace(
            b"deepseek4.flag" + (7).to_bytes(4, "little"), b"deepseek4.flag" + (13).to_bytes(4, "little")),
         abi.UNSUPPORTED),
    ]


def test_refusals_match_the_reference_reader(lib, oracle, tmp_path):
    ref, mismatches = oracle.ref_lib(), []
    for name, data, expected in refusal_cases(oracle):
        path = write(tmp_path, name + ".gguf", data)
        rc, handle, err = open_ours(lib, path)
        assert rc == expected and not handle.value, (name, rc, err.message)
        if ref is not None:
            theirs_rc, theirs, artifact = open_reference(ref, path)
            mismatches += [(name, theirs_rc, expected)] if theirs_rc != expected else []
            ref.yvex_artifact_close(C.c_void_p(artifact.value))
    assert not mismatches
    rc, handle, err = open_ours(lib, os.path.join(str(tmp_path), "absent.gguf").encode())
    assert rc == abi.IO and not handle.value
    assert lib.yvex_rocm_gguf_open_path(None, b"x", None) == abi.INVALID_ARG
    lib.yvex_rocm_gguf_close(None)


def test_tensor_beyond_the_file_is_marked_and_not_loadable(lib, oracle, tmp_path):
    meta, tensors, _ = sample(oracle, alignment=32)
    data, relative, start = W.build(meta, tensors)
    path = write(tmp_path, "cut.gguf", data[:-100])         # the last tensor loses its tail
    rc, handle, err = open_ours(lib, path)
    assert rc == 0, err.message
    rows, _, _ = directory(lib, handle)
    assert [r[-1] for r in rows] == [1, 1, 1, 0]
    ref = oracle.ref_lib()
    if ref is not None:
        theirs_rc, theirs, artifact = open_reference(ref, path)
        assert theirs_rc == 0 and directory(ref, theirs, "yvex_gguf_")[0] == rows
        ref.yvex_gguf_close(C.c_void_p(theirs.value))
        ref.yvex_artifact_close(C.c_void_p(artifact.value))
    view, verr = abi.WeightView(), abi.Error()
    host = (C.c_ubyte * 16)()
    assert lib.yvex_rocm_gguf_weight_view(handle, host, b"blk.3.ffn_norm.weight", C.byref(view),
                                                  C.byref(verr)) == abi.BOUNDS
    assert lib.yvex_rocm_gguf_weight_view(handle, host, b"nope", C.byref(view), C.byref(verr)) == abi.FORMAT
    lib.yvex_rocm_gguf_close(handle)


@pytest.mark.gpu
def test_tensors_loaded_from_a_file_run_through_the_kernels(gpu, oracle, tmp_path):
    """File -> resident arena -> weight views -> dense projection and a gather, against the
    oracle on the bytes that were written."""
    from backend_helpers import Backend
    b = Backend()
    assert b.ok, (b.open_rc, b.err.where, b.err.message)
    lib = b.lib
    meta, tensors, parts = sample(oracle)
    data, relative, start = W.build(meta, tensors, alignment=64, pad_tail=7)
    path = write(tmp_path, "model.gguf", data)
    rc, handle, err = open_ours(lib, path)
    assert rc == 0, err.message
    arena, host, lerr = C.POINTER(abi.DeviceTensor)(), C.c_void_p(), abi.Error()
    assert lib.yvex_rocm_gguf_resident_load(b.handle, handle, 1, C.byref(arena), C.byref(host),
                                                    C.byref(lerr)) == 0, lerr.message
    b.tensors.append(arena)
    assert arena.contents.bytes == len(data) - start
    view = abi.WeightView()
    assert lib.yvex_rocm_gguf_weight_view(handle, host, b"blk.3.ffn_gate_exps.weight", C.byref(view),
                                                  C.byref(lerr)) == 0
    assert (view.qtype, view.row_width, view.row_count, view.row_bytes) == (IQ2_XXS, 512, 1024, 132)
    assert view.layout == abi.LAYOUT_EXPERT_MAJOR and view.encoded == host.value + relative[0]
    assert view.encoded_bytes == parts["gate"].nbytes
    head = abi.WeightView()
    assert lib.yvex_rocm_gguf_weight_view(handle, host, b"output.weight", C.byref(head), C.byref(lerr)) == 0
    assert (head.qtype, head.row_width, head.row_count, head.row_bytes) == (Q8_0, 512, 300, 544)
    g = oracle.Generator(3, "gguf.x")
    x = g.normal(2 * 512).reshape(2, 512)
    xin, out = b.f32(x), b.empty_f32(2 * 300)
    facts = abi.OperationFacts()
    rc = lib.yvex_rocm_encoded_matvec(
        b.handle, C.c_void_p(head.encoded), abi.ULL(head.encoded_bytes), C.c_uint(head.qtype),
        abi.ULL(head.row_count), abi.ULL(head.row_width), abi.ULL(head.row_bytes), abi.ULL(2), xin, None,
        abi.ULL(0), None, out, 0, C.byref(facts), C.byref(lerr))
    assert rc == 0, lerr.message
    want = oracle.matvec(oracle.Q8_0, parts["head"], 300, 512, x)
    got = b.read_f32(out, 600).reshape(2, 300)
    assert np.all(np.abs(got - want) <= 1e-5 + 1e-3 * np.abs(want))
    # rows of the third expert of the gate tensor, decoded on the device
    ids = np.array([2 * 256, 2 * 256 + 255], np.uint32)
    decoded = b.empty_f32(2 * 512)
    b.workspace(4096)       # the gather stages its row identifiers there
    rc = lib.yvex_rocm_encoded_gather(
        b.handle, C.c_void_p(view.encoded), abi.ULL(view.encoded_bytes), C.c_uint(view.qtype),
        abi.ULL(view.row_count), abi.ULL(view.row_width), abi.ULL(view.row_bytes), ids.ctypes.data, abi.ULL(2),
        decoded, C.byref(facts), C.byref(lerr))
    assert rc == 0, lerr.message
    rows = oracle.decode_rows(oracle.IQ2_XXS, parts["gate"], 512, ids)
    assert np.array_equal(b.read_f32(decoded, 1024).reshape(2, 512), rows)
    lib.yvex_rocm_gguf_close(handle)
    assert b.close() == 0
