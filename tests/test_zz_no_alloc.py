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


def test_argmax_without_allocation_under_graph_capture():
    """The use its header names: captured into a HIP graph (the address of the static array looked up before the
    capture starts), replayed several times with other logits in the same buffer, with eager work and
    synchronisations between the replays; the device's free memory is the same before and after the calls."""
    lib = _lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    assert lib.ms_argmax_static_init() == 0
    rows, vocab, chunks = 8, 151936, 128
    g = torch.Generator(device=dev).manual_seed(1)
    logits = torch.randn(rows, vocab, generator=g, device=dev)
    got = torch.full((rows,), -1, dtype=torch.int32, device=dev)
    fresh = [torch.randn(rows, vocab, generator=g, device=dev) for _ in range(3)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):      # once eagerly, so that nothing is loaded for the first time while capturing
        assert lib.ms_argmax_static(logits.data_ptr(), vocab, rows, vocab, chunks, got.data_ptr(), side.cuda_stream) == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    # (inference mode, as the engine captures its own graphs: torch registers the state of its random generator
    # with a graph at the first capture of a process and updates it in place at every later one)
    with torch.inference_mode(), torch.cuda.graph(graph):
        rc = lib.ms_argmax_static(logits.data_ptr(), vocab, rows, vocab, chunks, got.data_ptr(),
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    small = torch.randn(3, 777, generator=g, device=dev)
    out = torch.empty(3, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream

    def free_bytes():
        torch.cuda.synchronize()
        return torch.cuda.mem_get_info(dev)[0]

    for i, other in enumerate(fresh):
        logits.copy_(other)
        logits[i, 1000 + i] = 99.0
        before = free_bytes()
        graph.replay()
        if i > 0:                      # (the first launch of a graph may upload it)
            assert free_bytes() == before
        torch.cuda.synchronize()
        assert torch.equal(got.long(), logits.argmax(dim=1)) and got[i].item() == 1000 + i
        # eager work of the same entry point between the replays shares the static array and leaves it usable;
        # nothing but the call lies between the two readings of the device's free memory
        before = free_bytes()
        assert lib.ms_argmax_static(small.data_ptr(), 777, 3, 777, 2, out.data_ptr(), stream) == 0
        assert free_bytes() == before
        assert torch.equal(out.long(), small.argmax(dim=1))
