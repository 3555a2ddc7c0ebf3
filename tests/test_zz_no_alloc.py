"""yvex_hip_argmax_f32_static: greedy selection that allocates nothing, against
yvex_hip_argmax_f32 given a workspace, through the C ABI."""
import ctypes as C

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def select(lib, name, values, scratch=None):
    """Call one of the two entry points on the current stream; returns (tokens, best, ties, status, rc)."""
    rows, width = values.shape
    dev = values.device
    tokens = torch.full((rows,), -1, dtype=torch.int32, device=dev)
    best = torch.full((rows,), -7.0, dtype=torch.float32, device=dev)
    ties = torch.zeros(rows, dtype=torch.int64, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    args = [C.c_void_p(values.data_ptr()), C.c_uint64(rows), C.c_uint64(width), C.c_void_p(tokens.data_ptr()),
            C.c_void_p(best.data_ptr()), C.c_void_p(ties.data_ptr())]
    if scratch is not None:
        args += [C.c_void_p(scratch.data_ptr()), C.c_uint64(scratch.numel())]
    args += [C.c_void_p(status.data_ptr()), C.c_void_p(torch.cuda.current_stream().cuda_stream)]
    rc = getattr(lib, name)(*args)
    torch.cuda.synchronize()
    return tokens.cpu().numpy(), best.cpu().numpy(), ties.cpu().numpy(), int(status.item()), rc


def test_static_scratch_selection_equals_workspace_selection(gpu, oracle):
    from yvex_amd import load_library
    lib = load_library()
    lib.yvex_hip_argmax_scratch_bytes.restype = C.c_uint64
    lib.yvex_hip_argmax_static_capacity.restype = C.c_uint64
    lib.yvex_hip_last_error.restype = C.c_char_p
    capacity = lib.yvex_hip_argmax_static_capacity()
    assert capacity == 16384 * 16
    rng = np.random.default_rng(11)
    # two calls in a row, the second smaller: 32 rows of a 129 280-token vocabulary (16 spans a
    # row), then 3 rows of 20 001 values (3 spans a row) that must not see the first call's spans
    for rows, width in ((32, 129280), (3, 20001), (2, 100)):
        values = rng.standard_normal((rows, width)).astype(np.float32)
        values[0, width - 1] = values[0, 1] = values[0].max() + 1.0     # a tie at both ends of row 0
        values[rows - 1] = np.round(values[rows - 1] * 2.0) / 2.0       # many ties in the last row
        on_device = torch.from_numpy(values).to(gpu)
        need = lib.yvex_hip_argmax_scratch_bytes(C.c_uint64(rows), C.c_uint64(width))
        assert need <= capacity
        workspace = torch.empty(max(need, 8), dtype=torch.uint8, device=gpu)
        want = select(lib, "yvex_hip_argmax_f32", on_device, workspace)
        got = select(lib, "yvex_hip_argmax_f32_static", on_device)
        assert want[4] == 0 and got[4] == 0 and want[3] == 0 and got[3] == 0
        for g, w in zip(got[:3], want[:3]):
            assert np.array_equal(g, w)
        rc, tokens, best, ties = oracle.argmax_f32(values)
        assert rc == 0 and np.array_equal(got[0].astype(np.uint32), tokens)
        assert np.array_equal(got[1], best) and np.array_equal(got[2].astype(np.uint64), ties)
    # a batch beyond the array is refused with a reason, and launches nothing
    rows, width = 17, 8192 * 1000
    assert lib.yvex_hip_argmax_scratch_bytes(C.c_uint64(rows), C.c_uint64(width)) > capacity
    fake = torch.zeros((1, 8), dtype=torch.float32, device=gpu)

    class Shape:                   # a [rows, width] view nobody reads: the call must refuse first
        shape = (rows, width)
        device = gpu

        @staticmethod
        def data_ptr():
            return fake.data_ptr()
    rc = select(lib, "yvex_hip_argmax_f32_static", Shape)[4]
    assert rc == -7 and b"static scratch" in lib.yvex_hip_last_error()
