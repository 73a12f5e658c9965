"""The entry point that allocates nothing (`kipp_argmax_static`, csrc/no_alloc.h), called
through ctypes the way a caller that cannot allocate would, against `kipp_argmax`, which
takes its scratch buffer from the caller: two calls in a row, the second with a smaller
input, so that what the first call left in the library's own array would show."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _library():
    from kipp_amd.csrc import build
    lib = build.library("sampling")
    ptr, i32 = ctypes.c_void_p, ctypes.c_int
    lib.kipp_argmax_static.argtypes = [ptr, ptr, i32, i32, ptr]
    lib.kipp_argmax_static.restype = i32
    lib.kipp_argmax.argtypes = [ptr, ptr, i32, i32, ptr, ptr]
    lib.kipp_argmax.restype = i32
    lib.kipp_argmax_static_max_rows.restype = i32
    lib.kipp_argmax_scratch_floats.argtypes = [i32]
    lib.kipp_argmax_scratch_floats.restype = i32
    return lib


def test_argmax_without_allocation_matches_the_one_with_a_workspace():
    import torch
    assert torch.cuda.is_available(), "needs a GPU"
    lib = _library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(5)
    most = lib.kipp_argmax_static_max_rows()
    assert most == 256
    for rows, vocab in ((48, 151936), (5, 40007)):       # large enough for the two-stage form; the second call is smaller
        print(f"kipp_argmax_static rows {rows} vocab {vocab}", flush=True)
        values = rng.standard_normal((rows, vocab)).astype(np.float32)
        values[0, vocab - 1] = 9.0                       # the last column of the last stretch
        values[rows - 1, 0] = values[rows - 1, 1] = 8.0  # equal values: the lowest index wins
        logits = torch.from_numpy(values).to(dev)
        got = torch.full((rows + 1,), -7, dtype=torch.int32, device=dev)
        want = torch.full((rows,), -7, dtype=torch.int32, device=dev)
        workspace = torch.empty(lib.kipp_argmax_scratch_floats(rows), dtype=torch.float32, device=dev)
        torch.cuda.synchronize()
        assert lib.kipp_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream) == 0
        assert lib.kipp_argmax(logits.data_ptr(), want.data_ptr(), rows, vocab, workspace.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        got, want = got.cpu().numpy(), want.cpu().numpy()
        assert got[rows] == -7, "wrote past its rows"
        assert np.array_equal(got[:rows], want)
        assert np.array_equal(got[:rows], values.argmax(axis=1))
    # more rows than the array holds: refused before anything is launched
    logits = torch.zeros((most + 1, 16384), dtype=torch.float32, device=dev)
    out = torch.full((most + 1,), -7, dtype=torch.int32, device=dev)
    assert lib.kipp_argmax_static(logits.data_ptr(), out.data_ptr(), most + 1, 16384, stream) == -2
    torch.cuda.synchronize()
    assert (out.cpu().numpy() == -7).all()
