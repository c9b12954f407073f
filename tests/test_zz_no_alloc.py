"""The entry point that allocates nothing (``nnis_argmax_static``), called
through ``ctypes`` as a caller outside this library would: two calls in a row,
the second with a smaller input, each against ``nnis_argmax`` with scratch of
the caller's; what it refuses; and that it leaves the allocator alone."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from nnis_amd.kernels import lib

    library = ctypes.CDLL(lib.find_built("core") or lib.build_module("core"))
    library.nnis_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    library.nnis_argmax_static.restype = ctypes.c_int
    library.nnis_argmax.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    library.nnis_argmax.restype = ctypes.c_int
    library.nnis_argmax_scratch.argtypes = [ctypes.c_int, ctypes.c_int]
    library.nnis_argmax_scratch.restype = ctypes.c_int
    library.nnis_last_error.restype = ctypes.c_char_p
    return library


def test_two_calls_in_a_row_the_second_smaller():
    library = _library()
    torch.manual_seed(3)
    stream = torch.cuda.current_stream().cuda_stream
    first = True
    for rows, vocab in ((64, 49152), (5, 1000)):  # the second call uses a part of what the first left in the array
        logits = torch.randn(rows, vocab, device="cuda")
        logits[0, vocab - 1] = 9.0
        logits[rows - 1, 7] = logits[rows - 1, 3] = 11.0  # a tie: the lower index wins
        got = torch.full((rows,), -5, dtype=torch.int32, device="cuda")
        want = torch.full((rows,), -6, dtype=torch.int32, device="cuda")
        scratch = torch.empty(library.nnis_argmax_scratch(rows, vocab), dtype=torch.float32, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        free_before = torch.cuda.mem_get_info()[0]
        status = library.nnis_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream)
        assert status == 0, library.nnis_last_error().decode()
        assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # torch's allocator was not asked for anything
        torch.cuda.synchronize()
        if not first:  # (a module's first launch may load its code)
            assert torch.cuda.mem_get_info()[0] == free_before  # nor the driver
        first = False
        assert library.nnis_argmax(logits.data_ptr(), want.data_ptr(), rows, vocab, scratch.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        assert torch.equal(got.cpu().long(), logits.cpu().argmax(dim=1))
        assert got[0].item() == vocab - 1 and got[rows - 1].item() == 3


def test_sizes_beyond_the_array_are_refused():
    library = _library()
    stream = torch.cuda.current_stream().cuda_stream
    logits = torch.zeros(4, 8, device="cuda")
    out = torch.full((4,), -5, dtype=torch.int32, device="cuda")
    # 2 * 2,049 rows * 16 chunks = 65,568 words: 32 more than the array holds (the pointers are never followed)
    assert library.nnis_argmax_static(logits.data_ptr(), out.data_ptr(), 2049, 65536, stream) != 0
    message = library.nnis_last_error().decode()
    assert "65568" in message and "65536" in message
    assert library.nnis_argmax_static(logits.data_ptr(), out.data_ptr(), 4, 0, stream) != 0
    assert library.nnis_argmax_static(None, out.data_ptr(), 4, 8, stream) != 0
    torch.cuda.synchronize()
    assert bool((out == -5).all())  # nothing was launched
    assert library.nnis_argmax_static(logits.data_ptr(), out.data_ptr(), 0, 8, stream) == 0  # no rows: nothing to do
    # the largest size it takes: 2,048 rows of 65,536 columns
    big = torch.randn(2048, 65536, device="cuda")
    result = torch.empty(2048, dtype=torch.int32, device="cuda")
    assert library.nnis_argmax_static(big.data_ptr(), result.data_ptr(), 2048, 65536, stream) == 0
    torch.cuda.synchronize()
    assert torch.equal(result.cpu().long(), big.cpu().argmax(dim=1))


def test_the_library_s_own_wrapper():
    from nnis_amd.errors import KernelError
    from nnis_amd.kernels import ops

    logits = torch.randn(8, 3001, device="cuda")
    out = torch.empty(8, dtype=torch.int32, device="cuda")
    assert torch.equal(ops.argmax_no_alloc(logits, out).cpu().long(), logits.cpu().argmax(dim=1))
    with pytest.raises(KernelError, match="fixed array"):
        ops.argmax_no_alloc(torch.zeros(40000, 4, device="cuda"), torch.empty(40000, dtype=torch.int32, device="cuda"))
