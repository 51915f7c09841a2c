"""The entry point that allocates nothing (``ms_argmax_static``), called through ctypes as a caller that cannot
allocate would: its result against ``ms_argmax``'s on two calls in a row, the second with a smaller input (what
the first call left in the library's static array must not show), and its refusal of sizes beyond its limits."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _lib():
    from llm_infrence_engine_amd.kernels import build

    lib = build.load()
    c_int, c_ll, c_ptr = ctypes.c_int, ctypes.c_longlong, ctypes.c_void_p
    lib.ms_argmax.argtypes = [c_ptr, c_ll, c_int, c_int, c_ptr, c_ptr, c_int, c_ptr, c_ptr]
    lib.ms_argmax.restype = c_int
    lib.ms_argmax_static.argtypes = [c_ptr, c_ll, c_int, c_int, c_int, c_ptr, c_ptr]
    lib.ms_argmax_static.restype = c_int
    lib.ms_argmax_static_init.argtypes = []
    lib.ms_argmax_static_init.restype = c_int
    lib.ms_argmax_static_limits.argtypes = [ctypes.POINTER(c_int), ctypes.POINTER(c_int)]
    lib.ms_argmax_static_limits.restype = None
    return lib


def test_argmax_without_allocation_equals_argmax_twice_in_a_row():
    lib = _lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.ms_argmax_static_init() == 0
    max_rows, max_chunks = ctypes.c_int(), ctypes.c_int()
    lib.ms_argmax_static_limits(ctypes.byref(max_rows), ctypes.byref(max_chunks))
    assert (max_rows.value, max_chunks.value) == (256, 128)
    g = torch.Generator(device=dev).manual_seed(0)
    for rows, vocab, chunks in ((64, 151936, 128), (5, 4099, 4)):       # the second call is smaller in every size
        logits = torch.randn(rows, vocab, generator=g, device=dev)
        logits[1, vocab - 1] = 50.0                                      # a maximum in the last chunk
        logits[2, 7] = logits[2, vocab // 2] = 60.0                      # a tie: the first index wins
        val = torch.empty(rows, chunks, device=dev)
        idx = torch.empty(rows, chunks, dtype=torch.int32, device=dev)
        want = torch.full((rows,), -1, dtype=torch.int32, device=dev)
        got = torch.full((rows,), -2, dtype=torch.int32, device=dev)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated(dev)
        assert lib.ms_argmax(logits.data_ptr(), vocab, rows, vocab, val.data_ptr(), idx.data_ptr(), chunks,
                             want.data_ptr(), stream) == 0
        assert lib.ms_argmax_static(logits.data_ptr(), vocab, rows, vocab, chunks, got.data_ptr(), stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == held
        assert torch.equal(got, want)
        assert torch.equal(got.long(), logits.argmax(dim=1))
        assert got[1].item() == vocab - 1 and got[2].item() == 7
    # beyond the limits: refused with the "unsupported size" code, nothing launched, the output untouched
    small = torch.randn(2, 300, device=dev)
    out = torch.full((2,), -7, dtype=torch.int32, device=dev)
    assert lib.ms_argmax_static(small.data_ptr(), 300, 2, 300, max_chunks.value + 1, out.data_ptr(), stream) == 2
    assert lib.ms_argmax_static(small.data_ptr(), 300, max_rows.value + 1, 300, 4, out.data_ptr(), stream) == 2
    torch.cuda.synchronize()
    assert out.tolist() == [-7, -7]
