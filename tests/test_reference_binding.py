"""The reference-side binding, executed.

`yvex_amd/csrc/reference_binding/rocm_adapter.c` is the file a maintainer adds to the reference
tree. Here it is compiled together with the reference's own generic backend code
(src/backend/core.c: vtable dispatch, ownership and lifecycle checks, workspace; src/backend/
residency.c: resident-arena attach / detach / resolve) where those sources lie, linked against
the built libyvex_rocm.so (oracle/Makefile, target ref_backend), and driven through the
reference's `yvex_backend_*` entry points with the call sequence of its own device test
(tests/unit/cuda/quant_qtype.c:560-574): resident alloc -> memcpy -> resident attach -> tensors ->
encoded matvec. Without a GPU the library's backend is host-only, so the projection ends in the
fail-closed refusal (kernel bundle absent) after every check that depends on the binding has
passed; with a GPU it computes and is compared with the oracle.

The reference's residency code admits only the CUDA kind at its two attach functions
(src/backend/residency.c:32,206); the build applies the edit a maintainer would make there
(oracle/ref_backend_rocm.sed) while compiling the file from where it lies. The reference sources
stay where they are: the compiled library lives under oracle/_ref/ and the test is skipped where
it cannot be built.
"""
import ctypes as C

import numpy as np
import pytest

from yvex_amd import abi


@pytest.fixture(scope="module")
def binding(oracle):
    lib = oracle.ref_backend_lib()
    if lib is None:
        pytest.skip("the reference tree is not here and oracle/_ref/libyvex_ref_backend.so was not shipped")
    P, ULL = C.c_void_p, C.c_ulonglong
    lib.yvex_backend_open_rocm_impl.argtypes = [C.POINTER(P), C.c_char_p, ULL, P]
    lib.yvex_backend_open_shared_rocm.argtypes = [C.POINTER(P), P, ULL, P]
    lib.yvex_backend_close_checked.argtypes = [C.POINTER(P), P]
    lib.yvex_backend_kind_of.argtypes = [P]
    lib.yvex_backend_status_of.argtypes = [P]
    lib.yvex_backend_tensor_alloc.argtypes = [P, P, C.POINTER(C.POINTER(abi.DeviceTensor)), P]
    lib.yvex_backend_tensor_write.argtypes = [P, C.POINTER(abi.DeviceTensor), P, ULL, P]
    lib.yvex_backend_tensor_read.argtypes = [P, C.POINTER(abi.DeviceTensor), P, ULL, P]
    lib.yvex_backend_tensor_release.argtypes = [P, C.POINTER(C.POINTER(abi.DeviceTensor)), P]
    lib.yvex_backend_tensor_owned_by.argtypes = [P, C.POINTER(abi.DeviceTensor)]
    lib.yvex_backend_resident_alloc.argtypes = [P, P, C.POINTER(C.POINTER(abi.DeviceTensor)), C.POINTER(P), P]
    lib.yvex_backend_resident_attach.argtypes = [P, P, ULL, C.POINTER(abi.DeviceTensor), ULL, P]
    lib.yvex_backend_resident_detach.argtypes = [P, P]
    lib.yvex_backend_resident_resolve.argtypes = [P, P, ULL, C.POINTER(ULL)]
    lib.yvex_backend_workspace_attach.argtypes = [P, C.POINTER(abi.DeviceTensor), ULL, P]
    lib.yvex_backend_workspace_detach.argtypes = [P]
    lib.yvex_backend_workspace_detach.restype = None
    lib.yvex_backend_query_capability.argtypes = [P, C.c_int, P, P]
    lib.yvex_backend_rocm_moe_operations_get.argtypes = [P]
    lib.yvex_backend_rocm_moe_operations_get.restype = P
    lib.yvex_backend_rocm_encoded_matvec.argtypes = [
        P, P, ULL, C.c_uint, ULL, ULL, ULL, ULL, C.POINTER(abi.DeviceTensor), C.POINTER(abi.DeviceTensor), ULL,
        C.POINTER(abi.DeviceTensor), C.POINTER(abi.DeviceTensor), C.c_int, P, P]
    return lib


class Reference:
    """A backend opened by the adapter, used through the reference's generic entry points."""

    def __init__(self, lib, shared_with=None):
        self.lib, self.handle, self.err = lib, C.c_void_p(), abi.Error()
        if shared_with is None:
            rc = lib.yvex_backend_open_rocm_impl(C.byref(self.handle), None, 0, C.byref(self.err))
        else:
            rc = lib.yvex_backend_open_shared_rocm(C.byref(self.handle), shared_with.handle, 0, C.byref(self.err))
        assert rc == 0, self.err.message
        assert lib.yvex_backend_kind_of(self.handle) == abi.KIND_ROCM

    def e(self):
        return C.byref(self.err)

    def desc(self, name, dtype, nbytes, elements):
        return abi.TensorDesc(name, dtype, 1, (abi.ULL * 4)(elements, 0, 0, 0), nbytes)

    def tensor(self, name, dtype, nbytes, elements):
        out = C.POINTER(abi.DeviceTensor)()
        d = self.desc(name, dtype, nbytes, elements)
        assert self.lib.yvex_backend_tensor_alloc(self.handle, C.byref(d), C.byref(out), self.e()) == 0, self.err.message
        return out

    def close(self):
        assert self.lib.yvex_backend_close_checked(C.byref(self.handle), self.e()) == 0, self.err.message
        assert not self.handle.value


def run_sequence(lib, oracle, with_gpu):
    ROWS, WIDTH = 12, 512
    qt = oracle.Q8_0
    g = oracle.Generator(91, "binding")
    encoded = g.weights(qt, ROWS, WIDTH)
    row_bytes = oracle.row_bytes(qt, WIDTH)
    x = g.normal(WIDTH)
    ref = Reference(lib)
    space = None
    if True:
        # tensors carry the reference's object as their owner: its own ownership check holds
        inp = ref.tensor(b"input", abi.DTYPE_F32, WIDTH * 4, WIDTH)
        out = ref.tensor(b"output", abi.DTYPE_F32, ROWS * 4, ROWS)
        assert lib.yvex_backend_tensor_owned_by(ref.handle, inp) == 1
        assert inp.contents.owner == ref.handle.value
        assert lib.yvex_backend_tensor_write(ref.handle, inp, x.ctypes.data, x.nbytes, ref.e()) == 0, ref.err.message
        back = np.empty_like(x)
        assert lib.yvex_backend_tensor_read(ref.handle, inp, back.ctypes.data, back.nbytes, ref.e()) == 0
        assert np.array_equal(back, x) and inp.contents.is_written == 1

        # tests/unit/cuda/quant_qtype.c:555-574: resident alloc, memcpy into the mapping, attach
        resident, mapped = C.POINTER(abi.DeviceTensor)(), C.c_void_p()
        d = ref.desc(b"encoded", abi.DTYPE_I8, encoded.nbytes, encoded.nbytes)
        assert lib.yvex_backend_resident_alloc(ref.handle, C.byref(d), C.byref(resident), C.byref(mapped),
                                               ref.e()) == 0, ref.err.message
        assert mapped.value and lib.yvex_backend_tensor_owned_by(ref.handle, resident) == 1
        C.memmove(mapped.value, encoded.ctypes.data, encoded.nbytes)
        facts = abi.OperationFacts()

        def matvec(pointer, q8=0):
            return lib.yvex_backend_rocm_encoded_matvec(
                ref.handle, pointer, encoded.nbytes, qt, ROWS, WIDTH, row_bytes, 1, inp, None, 0, None, out, q8,
                C.byref(facts), ref.e())

        # before the attach the arena resolves nowhere, on either side
        device = abi.ULL()
        assert lib.yvex_backend_resident_resolve(ref.handle, mapped, encoded.nbytes, C.byref(device)) == abi.RESIDENT_MISS
        assert matvec(mapped) == abi.FORMAT and out.contents.is_written == 0
        assert lib.yvex_backend_resident_attach(ref.handle, mapped, encoded.nbytes, resident, 17, ref.e()) == 0, ref.err.message
        # src/backend/residency.c:89-112: a pointer inside maps to device base + offset
        assert lib.yvex_backend_resident_resolve(ref.handle, mapped, encoded.nbytes, C.byref(device)) == abi.RESIDENT_HIT
        base = device.value
        inner = C.c_void_p(mapped.value + 3 * row_bytes)
        assert lib.yvex_backend_resident_resolve(ref.handle, inner, row_bytes, C.byref(device)) == abi.RESIDENT_HIT
        assert device.value == base + 3 * row_bytes
        assert lib.yvex_backend_resident_resolve(ref.handle, inner, encoded.nbytes, C.byref(device)) == abi.RESIDENT_MISS

        # the projection: the adapter carries the attachment over to the library before it runs
        rc = matvec(mapped)
        if with_gpu:
            assert rc == 0, ref.err.message
            got = np.empty(ROWS, np.float32)
            assert lib.yvex_backend_tensor_read(ref.handle, out, got.ctypes.data, got.nbytes, ref.e()) == 0
            want = oracle.matvec(qt, encoded, ROWS, WIDTH, x)[0]
            assert np.all(np.abs(got - want) <= 1e-5 + 1e-3 * np.abs(want))
            assert facts.active_weight_bytes == encoded.nbytes and facts.kernel_launches >= 2
            assert lib.yvex_backend_rocm_moe_operations_get(ref.handle)
            # Q8_K activations need the workspace the reference attaches on its own object
            assert matvec(mapped, 1) == abi.NOMEM
            space = ref.tensor(b"workspace", abi.DTYPE_I8, 1 << 16, 1 << 16)
            assert lib.yvex_backend_workspace_attach(ref.handle, space, 3, ref.e()) == 0, ref.err.message    # (generation 3)
            assert matvec(mapped, 1) == 0, ref.err.message
            assert lib.yvex_backend_tensor_read(ref.handle, out, got.ctypes.data, got.nbytes, ref.e()) == 0
            q = oracle.q8k_quantize(x)
            want_q8 = oracle.q8_matvec(qt, encoded, ROWS, WIDTH, q, 1)[0]
            assert np.all(np.abs(got - want_q8) <= 1e-5 * (1.0 + np.abs(want_q8)))
            lib.yvex_backend_workspace_detach(ref.handle)
            assert matvec(mapped, 1) == abi.NOMEM
        else:
            # host-only library: every check that needs the binding has passed (owners, written
            # input, residency); what refuses is the absent kernel bundle, fail-closed
            assert rc == abi.UNSUPPORTED and b"kernel" in ref.err.message.lower()
            assert out.contents.is_written == 0
            assert not lib.yvex_backend_rocm_moe_operations_get(ref.handle)
        # a shared session (yvex_backend_open_shared_cuda's counterpart in the adapter): the
        # reference's generic attach gives it the owner's arena (src/backend/residency.c:47-57),
        # the adapter carries that over, and the owner cannot close under it
        session = Reference(lib, shared_with=ref)
        assert lib.yvex_backend_resident_attach(session.handle, mapped, encoded.nbytes, resident, 17,
                                                session.e()) == 0, session.err.message
        assert lib.yvex_backend_resident_resolve(session.handle, inner, row_bytes, C.byref(device)) == abi.RESIDENT_HIT
        assert device.value == base + 3 * row_bytes
        s_in = session.tensor(b"session-input", abi.DTYPE_F32, WIDTH * 4, WIDTH)
        s_out = session.tensor(b"session-output", abi.DTYPE_F32, ROWS * 4, ROWS)
        assert lib.yvex_backend_tensor_write(session.handle, s_in, x.ctypes.data, x.nbytes, session.e()) == 0
        rc = lib.yvex_backend_rocm_encoded_matvec(session.handle, mapped, encoded.nbytes, qt, ROWS, WIDTH, row_bytes,
                                                  1, s_in, None, 0, None, s_out, 0, C.byref(facts), session.e())
        if with_gpu:
            assert rc == 0, session.err.message
            got = np.empty(ROWS, np.float32)
            assert lib.yvex_backend_tensor_read(session.handle, s_out, got.ctypes.data, got.nbytes, session.e()) == 0
            want = oracle.matvec(qt, encoded, ROWS, WIDTH, x)[0]
            assert np.all(np.abs(got - want) <= 1e-5 + 1e-3 * np.abs(want))
        else:
            assert rc == abi.UNSUPPORTED
        # the owner's input belongs to the owner, not to the session
        assert lib.yvex_backend_rocm_encoded_matvec(session.handle, mapped, encoded.nbytes, qt, ROWS, WIDTH, row_bytes,
                                                    1, inp, None, 0, None, s_out, 0, C.byref(facts),
                                                    session.e()) == abi.FORMAT
        for t in (s_in, s_out):
            assert lib.yvex_backend_tensor_release(session.handle, C.byref(t), session.e()) == 0
        # src/backend/core.c:610-634: while a session is open the owner releases nothing it may borrow
        assert lib.yvex_backend_tensor_release(ref.handle, C.byref(resident), ref.e()) == abi.STATE and resident
        session.close()
        # a tensor of another backend is refused by the ownership check behind the adapter
        other = Reference(lib)
        foreign = other.tensor(b"foreign", abi.DTYPE_F32, WIDTH * 4, WIDTH)
        other.lib.yvex_backend_tensor_write(other.handle, foreign, x.ctypes.data, x.nbytes, other.e())
        assert lib.yvex_backend_rocm_encoded_matvec(
            ref.handle, mapped, encoded.nbytes, qt, ROWS, WIDTH, row_bytes, 1, foreign, None, 0, None, out, 0,
            C.byref(facts), ref.e()) == abi.FORMAT
        assert lib.yvex_backend_tensor_release(other.handle, C.byref(foreign), other.e()) == 0
        other.close()
        # detach on the reference's object is carried over too: the arena stops resolving
        assert lib.yvex_backend_resident_detach(ref.handle, ref.e()) == 0, ref.err.message
        assert matvec(mapped) == abi.FORMAT
        # capability query through the vtable
        cap = abi.CapabilityResult()
        assert lib.yvex_backend_query_capability(ref.handle, abi.VARIANT_QTYPE_ROW_DOT, C.byref(cap), ref.e()) == 0
        assert cap.backend_kind == abi.KIND_ROCM
        assert cap.state == (abi.CAP_SUPPORTED if with_gpu else abi.CAP_UNSUPPORTED)
        if not with_gpu:
            assert cap.reason == abi.REASON_KERNEL_BUNDLE_ABSENT
        for t in (resident, out, inp) + ((space,) if space is not None else ()):
            assert lib.yvex_backend_tensor_release(ref.handle, C.byref(t), ref.e()) == 0, ref.err.message
        ref.close()


def test_reference_backend_code_drives_the_library_without_a_device(binding, oracle, monkeypatch):
    """The no-device seam: the library opens host-only (tensors in host memory, no kernels)."""
    monkeypatch.setenv("YVEX_TEST_ROCM_NO_DEVICE", "1")
    run_sequence(binding, oracle, with_gpu=False)


@pytest.mark.gpu
def test_reference_backend_code_drives_the_library_on_the_device(binding, oracle, gpu):
    run_sequence(binding, oracle, with_gpu=True)
