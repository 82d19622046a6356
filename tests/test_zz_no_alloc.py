"""The entry point that allocates nothing (csrc/no_alloc.h): ``tp_argmax_static`` against ``tp_argmax``, called
through ctypes on two inputs in a row, the second smaller than the first (the library's scratch array keeps
the first call's partial results)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _lib():
    from tempura_amd.csrc.build import ensure_built
    lib = ctypes.CDLL(ensure_built())
    lib.tp_last_error.restype = ctypes.c_char_p
    lib.tp_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.tp_argmax.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    lib.tp_argmax_static_init.argtypes = []
    return lib


def test_argmax_static_matches_argmax_on_two_calls_in_a_row():
    lib = _lib()
    torch.cuda.set_device(0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(3)
    # inputs, outputs and the workspace of the existing entry point are made first: nothing is allocated between
    # the calls that are compared
    cases = []
    for rows, vocab in ((64, 128256), (5, 20011)):
        lg = torch.randn(rows, vocab, generator=g)
        lg[1 % rows, 7] = lg[1 % rows, vocab - 3] = 50.0          # an exact tie: the last maximum wins
        lg = lg.to(DEV)
        cases.append((rows, vocab, lg, torch.full((rows,), -1, dtype=torch.int32, device=DEV),
                      torch.full((rows,), -2, dtype=torch.int32, device=DEV),
                      torch.empty(rows * 128, dtype=torch.float32, device=DEV)))
    torch.cuda.synchronize()
    assert lib.tp_argmax_static_init() == 0, lib.tp_last_error().decode()
    # free memory as the driver counts it: a hipMalloc inside the entry point would lower it, whoever made it
    # (the caching allocator's own counter only sees what goes through PyTorch)
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    for rows, vocab, lg, got, want, part in cases:
        rc = lib.tp_argmax_static(lg.data_ptr(), got.data_ptr(), rows, vocab, stream)
        assert rc == 0, lib.tp_last_error().decode()
        rc = lib.tp_argmax(lg.data_ptr(), want.data_ptr(), rows, vocab, part.data_ptr(), stream)
        assert rc == 0, lib.tp_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed during the calls"
    for rows, vocab, lg, got, want, part in cases:
        assert torch.equal(got, want)
        assert got.tolist() == [int(torch.nonzero(row == row.max()).max()) for row in lg.cpu()]
    assert cases[0][3][1] == 128256 - 3 and cases[1][3][1] == 20011 - 3


def test_argmax_static_refuses_more_rows_than_its_array_holds():
    lib = _lib()
    lg = torch.zeros(513, 8, device=DEV)
    out = torch.zeros(513, dtype=torch.int32, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.tp_argmax_static(lg.data_ptr(), out.data_ptr(), 513, 8, stream) != 0
    assert b"513 rows" in lib.tp_last_error()
    assert lib.tp_argmax_static(lg.data_ptr(), out.data_ptr(), 512, 8, stream) == 0
    torch.cuda.synchronize()
    assert out[:512].tolist() == [7] * 512
