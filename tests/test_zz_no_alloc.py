"""The argmax entry point that allocates nothing (``mll_argmax_static``), called through ``ctypes`` as a caller
that cannot allocate would: its output must equal ``mll_argmax``'s, whose scratch the caller brings, on two calls
in a row, the second with a smaller input (the static scratch then still holds the first call's slices)."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"
MAX_PARTS = 65536   # MLL_ARGMAX_STATIC_MAX_PARTS of csrc/microllm_hip.h


def load():
    from microllm_rocm_amd.ops import library
    lib = library.load()
    lib.mll_last_error.restype = ctypes.c_char_p
    lib.mll_argmax_static.restype = ctypes.c_int
    lib.mll_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.mll_argmax.restype = ctypes.c_int
    lib.mll_argmax.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    return lib


def both(lib, logits):
    """(static entry point's result, existing entry point's result) for float32 logits on the GPU."""
    rows, vocab = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    got = torch.full((rows,), -7, dtype=torch.int32, device=DEVICE)
    expected = torch.full((rows,), -7, dtype=torch.int32, device=DEVICE)
    parts = torch.empty((rows, lib.mll_argmax_slices(vocab), 4), dtype=torch.int32, device=DEVICE)
    # The first call on a GPU asks for the static array's address; from then on a call must leave the device's
    # free memory as it found it. ``mem_get_info`` is the driver's own count, so it also sees what a library
    # would take or give back behind torch's allocator (which ``memory_allocated`` does not).
    status = lib.mll_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream)
    assert status == 0, lib.mll_last_error().decode()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    allocated_before = torch.cuda.memory_allocated()
    got.fill_(-7)
    status = lib.mll_argmax_static(logits.data_ptr(), got.data_ptr(), rows, vocab, stream)
    assert status == 0, lib.mll_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_allocated() == allocated_before
    status = lib.mll_argmax(logits.data_ptr(), expected.data_ptr(), parts.data_ptr(), rows, vocab, stream)
    assert status == 0, lib.mll_last_error().decode()
    torch.cuda.synchronize()
    return got.cpu().numpy(), expected.cpu().numpy()


def test_static_argmax_matches_argmax_on_two_calls_the_second_smaller():
    lib = load()
    torch.cuda.set_device(DEVICE)
    generator = torch.Generator(device="cpu").manual_seed(5)
    # First call: many rows of a large vocabulary that is no power of two (64 slices a row).
    first = torch.randn((48, 152_064), generator=generator, dtype=torch.float32)
    first[3, 151_999] = 9.0                       # a maximum in the last slice
    first[4, 7] = first[4, 70_000] = 11.0         # a tie: the first wins
    first[5, 100] = float("nan")                  # a non-finite value gives -1
    got, expected = both(lib, first.to(DEVICE))
    np.testing.assert_array_equal(got, expected)
    np.testing.assert_array_equal(got[[3, 4, 5]], [151_999, 7, -1])
    np.testing.assert_array_equal(np.delete(got, 5), np.delete(first.numpy(), 5, axis=0).argmax(axis=1))
    # Second call: fewer rows and fewer slices, so most of the static scratch holds the first call's results.
    second = torch.randn((5, 5_000), generator=generator, dtype=torch.float32)
    second[2, 4_999] = 8.0
    got, expected = both(lib, second.to(DEVICE))
    np.testing.assert_array_equal(got, expected)
    np.testing.assert_array_equal(got, second.numpy().argmax(axis=1))
    # And a larger one again.
    third = torch.randn((17, 40_003), generator=generator, dtype=torch.float32)
    got, expected = both(lib, third.to(DEVICE))
    np.testing.assert_array_equal(got, expected)
    np.testing.assert_array_equal(got, third.numpy().argmax(axis=1))


def test_static_argmax_refuses_what_its_scratch_cannot_hold():
    lib = load()
    torch.cuda.set_device(DEVICE)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    vocab = 2048 * 64 + 1                          # 64 slices a row
    rows = MAX_PARTS // 64 + 1
    logits = torch.zeros((1, vocab), dtype=torch.float32, device=DEVICE)   # never read: the call must refuse first
    out = torch.full((1,), -7, dtype=torch.int32, device=DEVICE)
    assert lib.mll_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, stream) != 0
    assert "beyond the static scratch" in lib.mll_last_error().decode()
    assert lib.mll_argmax_static(None, out.data_ptr(), 1, vocab, stream) != 0
    torch.cuda.synchronize()
    assert out.item() == -7
    # The most it takes: rows x slices == the scratch's entries.
    rows = MAX_PARTS // 4
    logits = torch.randn((rows, 8_000), dtype=torch.float32, device=DEVICE)   # 4 slices a row
    got, expected = both(lib, logits)
    np.testing.assert_array_equal(got, expected)
