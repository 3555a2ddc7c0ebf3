"""Derived expert storage (plan + build): the library's host functions against the reference's
own builder (golden images written from it, and the compiled reference where it is present),
against hand-placed bytes, and against the numpy restatement in the oracle.

Reference: src/backend/cuda/layout.c:23-167; the row-batch path refuses a derived view
(src/backend/cuda/moe.c:933-958), which tests/test_gpu_backend.py covers on the device.
"""
import ctypes as C
import os

import numpy as np
import pytest

import oracle
from yvex_amd import abi

GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))
BLOCK_BYTES = {oracle.IQ2_XXS: 66, oracle.Q2_K: 84}


def decision_for(qtype, experts, rows, width, *, consumer=abi.CONSUMER_ROUTED_GATE_UP,
                 layout=abi.LAYOUT_DERIVED, required=1, encoded_bytes=None):
    d = abi.ExecutionDecision()
    d.expert_count, d.canonical_qtype = experts, qtype
    d.canonical_row_width, d.canonical_row_count = width, rows
    bytes_ = rows * (width // 256) * BLOCK_BYTES.get(qtype, 66)
    d.encoded_bytes = bytes_ if encoded_bytes is None else encoded_bytes
    d.consumer, d.layout, d.derived_asset_required = consumer, layout, required
    return d


def plan(lib, decision):
    storage, err = abi.ULL(0xDEAD), abi.Error()
    rc = lib.yvex_rocm_moe_derived_layout_plan(C.byref(decision), C.byref(storage), C.byref(err))
    return rc, storage.value, err


def build(lib, decision, canonical, storage):
    derived = np.full(storage, 0xA5, np.uint8)      # the builder has to clear the padding itself
    err = abi.Error()
    rc = lib.yvex_rocm_moe_derived_layout_build(C.byref(decision), canonical.ctypes.data, canonical.size,
                                                derived.ctypes.data, derived.size, C.byref(err))
    return rc, derived, err


@pytest.fixture(scope="module")
def lib():
    return abi.library()


@pytest.mark.parametrize("name", ["iq2_xxs", "q2_k"])
def test_golden_images_of_the_reference_builder(lib, name):
    qtype, experts, rows, width = (int(v) for v in GOLDEN[f"layout_{name}_shape"])
    canonical, expected = GOLDEN[f"layout_{name}_canonical"], GOLDEN[f"layout_{name}_derived"]
    d = decision_for(qtype, experts, rows, width)
    rc, storage, _ = plan(lib, d)
    assert (rc, storage) == (0, expected.size)
    rc, derived, _ = build(lib, d, canonical, storage)
    assert rc == 0 and np.array_equal(derived, expected)
    assert oracle.derived_layout_plan(qtype, rows, width, experts) == expected.size
    assert np.array_equal(oracle.derived_layout_build(qtype, canonical, rows, width, experts), expected)


def test_hand_placed_bytes_iq2_xxs(lib):
    """Three superblocks: scales fill 6 bytes, the codes start at 64."""
    canonical = np.arange(3 * 66, dtype=np.uint32).astype(np.uint8)   # byte = its own offset (mod 256)
    d = decision_for(oracle.IQ2_XXS, 3, 3, 256)
    rc, storage, _ = plan(lib, d)
    assert (rc, storage) == (0, 64 + 3 * 64)
    rc, derived, _ = build(lib, d, canonical, storage)
    assert rc == 0
    assert derived[2] == canonical[66] and derived[3] == canonical[67]        # scale of block 1
    assert derived[64 + 128 + 3] == canonical[2 * 66 + 5]                     # code byte 3 of block 2
    assert not derived[6:64].any()
    assert np.array_equal(derived, oracle.derived_layout_build(oracle.IQ2_XXS, canonical, 3, 256, 3))


def test_hand_placed_bytes_q2_k(lib):
    """Two experts of two rows, one block a row: 2 units -> factors 16 B, scales at 64, codes at 128."""
    canonical = (np.arange(4 * 84, dtype=np.uint32) * 7 + 3).astype(np.uint8)
    d = decision_for(oracle.Q2_K, 2, 4, 256)
    rc, storage, _ = plan(lib, d)
    assert (rc, storage) == (0, 128 + 2 * 128)
    rc, derived, _ = build(lib, d, canonical, storage)
    assert rc == 0
    odd = 84                                  # expert 0, odd row
    assert np.array_equal(derived[4:8], canonical[odd + 80:odd + 84])          # its d, dmin
    assert derived[64 + 16 + 8 + 1] == canonical[odd + 9]                      # scale byte 9: second half
    assert derived[128 + 3 * 8 + 4 + 2] == canonical[odd + 16 + 4 * 3 + 2]     # word 3, byte 2
    assert derived[128 + 128] == canonical[2 * 84 + 16]                        # expert 1's even row opens unit 1
    assert not derived[16:64].any()
    assert np.array_equal(derived, oracle.derived_layout_build(oracle.Q2_K, canonical, 4, 256, 2))


@pytest.mark.parametrize("qtype,experts,rows_per_expert,width", [
    (oracle.IQ2_XXS, 2, 1, 256), (oracle.IQ2_XXS, 4, 33, 1792), (oracle.IQ2_XXS, 256, 8, 512),
    (oracle.Q2_K, 2, 2, 256), (oracle.Q2_K, 3, 10, 1280), (oracle.Q2_K, 16, 64, 512)])
def test_every_canonical_byte_lands_once(lib, qtype, experts, rows_per_expert, width):
    """The image is a permutation of the canonical bytes plus zero padding: checked by packing the
    bytes of a position counter (three planes) and reading the positions back."""
    rows = experts * rows_per_expert
    size = rows * (width // 256) * BLOCK_BYTES[qtype]
    position = np.arange(1, size + 1, dtype=np.uint32)
    d = decision_for(qtype, experts, rows, width)
    rc, storage, _ = plan(lib, d)
    assert rc == 0 and storage == oracle.derived_layout_plan(qtype, rows, width, experts)
    planes = []
    for shift in (0, 8, 16):
        canonical = ((position >> shift) & 0xFF).astype(np.uint8)
        rc, derived, _ = build(lib, d, canonical, storage)
        assert rc == 0
        assert np.array_equal(derived, oracle.derived_layout_build(qtype, canonical, rows, width, experts))
        planes.append(derived.astype(np.uint32) << shift)
    landed = planes[0] | planes[1] | planes[2]
    assert np.array_equal(np.sort(landed[landed != 0]), position)
    assert np.count_nonzero(landed == 0) == storage - size


@pytest.mark.skipif(not os.path.exists(oracle.REF_PATH), reason="compiled reference absent")
@pytest.mark.parametrize("qtype,experts,rows_per_expert,width", [
    (oracle.IQ2_XXS, 5, 7, 768), (oracle.Q2_K, 4, 6, 1024), (oracle.IQ2_XXS, 2, 31, 256)])
def test_against_the_compiled_reference(lib, qtype, experts, rows_per_expert, width):
    ref = C.CDLL(oracle.REF_PATH)
    rows = experts * rows_per_expert
    canonical = oracle.Generator(7, f"layout.{qtype}.{rows}.{width}").bytes(
        rows * (width // 256) * BLOCK_BYTES[qtype])
    d = decision_for(qtype, experts, rows, width, consumer=abi.CONSUMER_ROUTED_DOWN)
    theirs, err = abi.ULL(), abi.Error()
    assert ref.yvex_cuda_moe_derived_layout_plan(C.byref(d), C.byref(theirs), C.byref(err)) == 0
    rc, storage, _ = plan(lib, d)
    assert (rc, storage) == (0, theirs.value)
    expected = np.full(storage, 0x5A, np.uint8)
    assert ref.yvex_cuda_moe_derived_layout_build(
        C.byref(d), C.c_void_p(canonical.ctypes.data), abi.ULL(canonical.size),
        C.c_void_p(expected.ctypes.data), abi.ULL(expected.size), C.byref(err)) == 0
    rc, derived, _ = build(lib, d, canonical, storage)
    assert rc == 0 and np.array_equal(derived, expected)


def sweep_image_of(canonical):
    """numpy statement of the expert sweeps' image: per superblock two records of nine dwords."""
    blocks = canonical.size // 66
    raw = canonical.reshape(blocks, 66)
    d = raw[:, 0].astype(np.uint32) | (raw[:, 1].astype(np.uint32) << 8)
    groups = raw[:, 2:].reshape(blocks, 8, 8)
    grids = groups[:, :, :4].copy().view(np.uint32).reshape(blocks, 8)
    aux = groups[:, :, 4:].copy().view(np.uint32).reshape(blocks, 8)
    image = np.zeros((blocks, 2, 9), np.uint32)
    for half in range(2):
        scales = np.zeros(blocks, np.uint32)
        for j in range(4):
            a = aux[:, 4 * half + j]
            image[:, half, 1 + 2 * j] = grids[:, 4 * half + j]
            image[:, half, 2 + 2 * j] = ((a & 127) | (((a >> 7) & 127) << 8) | (((a >> 14) & 127) << 16)
                                         | (((a >> 21) & 127) << 24))
            scales |= (a >> 28) << (4 * j)
        image[:, half, 0] = d | (scales << 16)
    return image.view(np.uint8).ravel()


@pytest.mark.parametrize("experts,rows,width,consumer", [
    (4, 8, 512, abi.CONSUMER_ROUTED_GATE_UP), (3, 9, 768, abi.CONSUMER_ROUTED_DOWN),
    (1, 5, 256, abi.CONSUMER_SHARED_EXPERT)])
def test_sweep_image_of_the_gfx950_family(lib, experts, rows, width, consumer):
    """A decision of the gfx950 sweep family gets this backend's own image of an IQ2_XXS tensor
    (72 bytes a superblock; the shared expert admitted), not the reference's two sections."""
    d = decision_for(oracle.IQ2_XXS, experts, rows, width, consumer=consumer)
    d.kernel_family = abi.FAMILY_GFX950
    rc, storage, err = plan(lib, d)
    assert rc == 0, err.message
    assert storage == rows * (width // 256) * 72
    canonical = oracle.Generator(9, f"layout.sweep.{rows}.{width}").iq2xxs(rows * (width // 256))
    rc, derived, err = build(lib, d, canonical, storage)
    assert rc == 0, err.message
    assert np.array_equal(derived, sweep_image_of(canonical))
    # and the image decodes to the same weights: scales, code bytes and sign fields are all there
    records = derived.view(np.uint32).reshape(-1, 2, 9)
    raw = canonical.reshape(-1, 66)
    assert np.array_equal(records[:, :, 0] & 0xffff, np.repeat(raw[:, :2].copy().view(np.uint16), 2, 1))
    # other qtypes have no sweep image; without the family the shared expert has no derived storage
    q2 = decision_for(oracle.Q2_K, 2, 8, 512)
    q2.kernel_family = abi.FAMILY_GFX950
    assert plan(lib, q2)[0] == abi.UNSUPPORTED
    if consumer == abi.CONSUMER_SHARED_EXPERT:
        d.kernel_family = b""
        assert plan(lib, d)[0] == abi.FORMAT


def test_refusals(lib):
    good = dict(qtype=oracle.IQ2_XXS, experts=4, rows=8, width=512)
    cases = [
        (decision_for(**good, layout=abi.LAYOUT_EXPERT_MAJOR), oracle.ERR_FORMAT),
        (decision_for(**good, required=0), oracle.ERR_FORMAT),
        (decision_for(**good, consumer=abi.CONSUMER_SHARED_EXPERT), oracle.ERR_FORMAT),
        (decision_for(oracle.IQ2_XXS, 1, 8, 512), oracle.ERR_FORMAT),            # one expert
        (decision_for(oracle.IQ2_XXS, 3, 8, 512), oracle.ERR_FORMAT),            # rows not a multiple
        (decision_for(oracle.IQ2_XXS, 4, 8, 384, encoded_bytes=8 * 99), oracle.ERR_FORMAT),
        (decision_for(**good, encoded_bytes=8 * 2 * 66 - 1), oracle.ERR_FORMAT),  # bytes differ
        (decision_for(oracle.Q8_0, 4, 8, 512), oracle.ERR_UNSUPPORTED),
        (decision_for(oracle.Q2_K, 4, 12, 512), oracle.ERR_BOUNDS),              # odd rows per expert
        (decision_for(oracle.IQ2_XXS, 2, 1 << 63, 1 << 12, encoded_bytes=1), oracle.ERR_BOUNDS),
    ]
    ref = C.CDLL(oracle.REF_PATH) if os.path.exists(oracle.REF_PATH) else None
    for decision, status in cases:
        if ref is not None:      # the reference's own answer for the same decision
            theirs = abi.ULL(1)
            assert ref.yvex_cuda_moe_derived_layout_plan(C.byref(decision), C.byref(theirs), None) == status
        rc, storage, err = plan(lib, decision)
        assert (rc, storage) == (status, 0), (decision.canonical_qtype, decision.expert_count, err.message)
        assert err.code == status
    err = abi.Error()
    assert lib.yvex_rocm_moe_derived_layout_plan(C.byref(decision_for(**good)), None,
                                                 C.byref(err)) == oracle.ERR_INVALID_ARG
    storage = abi.ULL(5)
    assert lib.yvex_rocm_moe_derived_layout_plan(None, C.byref(storage), C.byref(err)) == oracle.ERR_FORMAT
    assert storage.value == 0
    # build: exact, separate storage only
    d = decision_for(**good)
    rc, size, _ = plan(lib, d)
    canonical = np.zeros(d.encoded_bytes, np.uint8)
    derived = np.zeros(size + 64, np.uint8)
    args = lambda c, cb, o, ob: lib.yvex_rocm_moe_derived_layout_build(   # noqa: E731
        C.byref(d), c, cb, o, ob, C.byref(err))
    assert args(canonical.ctypes.data, canonical.size, derived.ctypes.data, size + 64) == oracle.ERR_INVALID_ARG
    assert args(canonical.ctypes.data, canonical.size - 1, derived.ctypes.data, size) == oracle.ERR_INVALID_ARG
    assert args(None, canonical.size, derived.ctypes.data, size) == oracle.ERR_INVALID_ARG
    assert args(canonical.ctypes.data, canonical.size, None, size) == oracle.ERR_INVALID_ARG
    assert args(derived.ctypes.data, canonical.size, derived.ctypes.data, size) == oracle.ERR_INVALID_ARG
    assert args(canonical.ctypes.data, canonical.size, derived.ctypes.data, size) == 0


def test_operations_table_carries_the_layout_entries(lib):
    """The two table entries are the exported functions (the table itself needs an open backend,
    which the device tests take; here the symbols and their signatures are what is checked)."""
    fields = dict(abi.MoeOperations._fields_)
    assert "derived_layout_plan" in fields and "derived_layout_build" in fields
    assert hasattr(lib, "yvex_rocm_moe_derived_layout_plan")
