"""The entry point that allocates nothing, called through ctypes as a caller outside this package would: its tokens
against those of the entry point that takes scratch from the caller, on two calls in a row, the second with a
smaller input (so that what the first left in the static scratch lies behind the second's)."""
import ctypes
from ctypes import c_int, c_long, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def entry_points():
    from geneinfer_amd.kernels import library
    lib = library.load()
    lib.gi_argmax.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_long, c_void_p]
    lib.gi_argmax_no_alloc.argtypes = [c_void_p, c_void_p, c_int, c_int, c_long, c_void_p]
    lib.gi_no_alloc_prepare.argtypes = []
    lib.gi_argmax_chunks.argtypes = [c_int]
    for fn in (lib.gi_argmax, lib.gi_argmax_no_alloc, lib.gi_no_alloc_prepare, lib.gi_argmax_chunks):
        fn.restype = c_int
    lib.gi_last_error.restype = ctypes.c_char_p
    return lib


def test_arg_max_without_allocation_gives_the_tokens_of_the_one_with_scratch():
    lib = entry_points()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.gi_no_alloc_prepare() == 0, lib.gi_last_error().decode()
    gen = torch.Generator().manual_seed(12)
    for rows, vocab, pad in ((37, 128256, 0), (5, 9001, 7)):                       # the second call is smaller, and its rows are strided
        logits = torch.randn(rows, vocab + pad, generator=gen).to(dev)
        logits[1, 17] = logits[1, vocab - 1] = 50.0                                # equal maxima: the lowest index wins
        logits[:, vocab:] = 99.0                                                   # beyond the row's end: never looked at
        view = logits[:, :vocab]
        chunks = lib.gi_argmax_chunks(vocab)
        part_v = torch.empty(rows * chunks, dtype=torch.float32, device=dev)
        part_i = torch.empty(rows * chunks, dtype=torch.int32, device=dev)
        want = torch.full((rows,), -1, dtype=torch.int32, device=dev)
        got = torch.full((rows,), -2, dtype=torch.int32, device=dev)
        assert lib.gi_argmax(view.data_ptr(), want.data_ptr(), part_v.data_ptr(), part_i.data_ptr(), rows, vocab, view.stride(0), stream) == 0
        # Nothing is allocated: the driver's own count of free device memory (which sees a hipMalloc that torch's allocator would
        # not) stands still over a call made after the scratch's address is known; torch's count beside it.
        assert lib.gi_argmax_no_alloc(view.data_ptr(), got.data_ptr(), rows, vocab, view.stride(0), stream) == 0, lib.gi_last_error().decode()
        torch.cuda.synchronize()
        got.fill_(-2)
        torch.cuda.synchronize()
        free_before, held_before = torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_allocated(dev)
        assert lib.gi_argmax_no_alloc(view.data_ptr(), got.data_ptr(), rows, vocab, view.stride(0), stream) == 0, lib.gi_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(dev)[0] == free_before and torch.cuda.memory_allocated(dev) == held_before
        assert torch.equal(got, want) and torch.equal(got.cpu().long(), view.cpu().argmax(dim=-1))
        assert int(got[1]) == 17


def test_arg_max_without_allocation_refuses_what_its_scratch_cannot_hold():
    lib = entry_points()
    x = torch.zeros(8, device="cuda:0")
    out = torch.zeros(8, dtype=torch.int32, device="cuda:0")
    assert lib.gi_argmax_no_alloc(x.data_ptr(), out.data_ptr(), 4097, 65536, 65536, None) != 0           # 4097 x 16 runs > 65536
    assert "static scratch holds 65536" in lib.gi_last_error().decode()
    assert lib.gi_argmax_no_alloc(None, out.data_ptr(), 1, 8, 8, None) != 0
    assert lib.gi_argmax_no_alloc(x.data_ptr(), out.data_ptr(), 1, 8, 8, None) == 0                      # the limit itself is fine
    torch.cuda.synchronize()
    assert int(out[0]) == 0
