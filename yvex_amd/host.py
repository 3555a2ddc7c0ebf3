"""Small conveniences over the C ABI of the backend for Python callers (tests, the benchmark):
open a backend, allocate and fill its tensors, attach a resident arena and a workspace. Every
call goes through ``include/yvex_rocm.h``; nothing here computes."""
import ctypes as C

import numpy as np

from . import abi


class Backend:
    def __init__(self, memory_limit=0):
        self.lib = abi.library()
        self.handle = C.c_void_p()
        self.err = abi.Error()
        opts = abi.BackendOptions(abi.KIND_ROCM, None, memory_limit)
        self.open_rc = self.lib.yvex_rocm_backend_open(C.byref(self.handle), C.byref(opts), C.byref(self.err))
        self.tensors = []

    @property
    def ok(self):
        return self.open_rc == 0

    def tensor(self, nbytes, dtype=abi.DTYPE_F32, name=b"t"):
        desc = abi.TensorDesc(name, dtype, 1, (abi.ULL * 4)(nbytes, 0, 0, 0), nbytes)
        out = C.POINTER(abi.DeviceTensor)()
        rc = self.lib.yvex_rocm_backend_tensor_alloc(self.handle, C.byref(desc), C.byref(out), C.byref(self.err))
        if rc == 0:
            self.tensors.append(out)
        return rc, out

    def f32(self, array):
        array = np.ascontiguousarray(array, np.float32)
        rc, t = self.tensor(array.nbytes)
        assert rc == 0, self.err.message
        rc = self.lib.yvex_rocm_backend_tensor_write(self.handle, t, array.ctypes.data, array.nbytes,
                                                C.byref(self.err))
        assert rc == 0, self.err.message
        return t

    def empty_f32(self, count):
        rc, t = self.tensor(count * 4)
        assert rc == 0, self.err.message
        return t

    def read_f32(self, tensor, count):
        out = np.empty(count, np.float32)
        rc = self.lib.yvex_rocm_backend_tensor_read(self.handle, tensor, out.ctypes.data, out.nbytes,
                                               C.byref(self.err))
        assert rc == 0, self.err.message
        return out

    def resident(self, blob: np.ndarray, generation=1):
        """Allocate a resident arena, fill its host shadow, attach (= publish). Returns
        (tensor, host_base_address)."""
        desc = abi.TensorDesc(b"arena", abi.DTYPE_I8, 1, (abi.ULL * 4)(blob.nbytes, 0, 0, 0), blob.nbytes)
        out = C.POINTER(abi.DeviceTensor)()
        host = C.c_void_p()
        rc = self.lib.yvex_rocm_backend_resident_alloc(self.handle, C.byref(desc), C.byref(out),
                                                  C.byref(host), C.byref(self.err))
        assert rc == 0, self.err.message
        self.tensors.append(out)
        C.memmove(host.value, blob.ctypes.data, blob.nbytes)
        rc = self.lib.yvex_rocm_backend_resident_attach(self.handle, host, blob.nbytes, out, generation,
                                                   C.byref(self.err))
        assert rc == 0, self.err.message
        return out, host.value

    def workspace(self, nbytes):
        rc, t = self.tensor(nbytes, abi.DTYPE_I8, b"workspace")
        assert rc == 0, self.err.message
        rc = self.lib.yvex_rocm_backend_workspace_attach(self.handle, t, nbytes, C.byref(self.err))
        assert rc == 0, self.err.message
        return t

    def release_all(self):
        for t in reversed(self.tensors):
            self.lib.yvex_rocm_backend_tensor_release(self.handle, C.byref(t), C.byref(self.err))
        self.tensors = []

    def close(self):
        self.release_all()
        return self.lib.yvex_rocm_backend_close_checked(C.byref(self.handle), C.byref(self.err))
