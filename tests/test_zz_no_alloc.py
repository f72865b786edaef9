"""The argmax entry point that allocates nothing, called through ctypes as a caller that cannot allocate
would call it: checked against the entry point with a workspace argument on two calls in a row, the
second with a smaller input (the fixed array then still holds what the first call left)."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from leone_amd.ops.library import library
    lib = library()
    lib.leone_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.leone_argmax_static.restype = ctypes.c_int
    lib.leone_argmax_static_max_entries.argtypes = []
    lib.leone_argmax_static_max_entries.restype = ctypes.c_int
    return lib


def test_argmax_without_allocation_equals_argmax_with_a_workspace():
    from leone_amd import ops
    lib = _library()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    generator = torch.Generator().manual_seed(5)
    for rows, vocab in ((37, 151_936), (5, 3_001)):                       # the second call is the smaller one
        logits = torch.randn(rows, vocab, generator=generator).to(device)
        logits[0, 17] = float("nan")
        logits[rows - 1, vocab - 1] = 50.0                                 # the last place of the last chunk
        if vocab > 4096:
            logits[1, 4095] = logits[1, 4096] = 60.0                       # a tie across a chunk edge: the lower id
        out = torch.full((rows,), -7, dtype=torch.int32, device=device)   # output memory is the caller's
        stream = torch.cuda.current_stream().cuda_stream
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        status = lib.leone_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, stream)
        assert status == 0, lib.leone_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        # torch's figure covers torch's allocator only: the driver's count of free bytes would show a hipMalloc or
        # hipFree inside the entry point (the first call has resolved the array's address, so this one is plain)
        free_before, _ = torch.cuda.mem_get_info(device)
        out.fill_(-7)
        assert lib.leone_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(device)[0] == free_before
        want = ops.argmax(logits)
        assert torch.equal(out, want)
        assert int(out[rows - 1]) == vocab - 1
        if vocab > 4096:
            assert int(out[1]) == 4095


def test_argmax_without_allocation_refuses_what_its_array_cannot_hold():
    lib = _library()
    device = torch.device("cuda:0")
    limit = lib.leone_argmax_static_max_entries()
    rows, vocab = limit // 2 + 1, 8192                                     # two chunks a row: one entry too many
    logits = torch.zeros(1, device=device)                                 # never read: the call is refused first
    out = torch.zeros(rows, dtype=torch.int32, device=device)
    status = lib.leone_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab,
                                     torch.cuda.current_stream().cuda_stream)
    assert status != 0
    assert "scratch array holds" in lib.leone_last_error().decode()


def test_argmax_without_allocation_can_be_recorded_into_a_graph():
    """Under stream capture an allocation is an error: the entry point records, and every replay (with eager
    work between) gives the argmax of what the input buffer then holds."""
    from leone_amd import ops
    lib = _library()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    rows, vocab = 6, 40_000
    logits = torch.randn(rows, vocab, device=device)
    out = torch.full((rows,), -7, dtype=torch.int32, device=device)
    assert lib.leone_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, torch.cuda.current_stream().cuda_stream) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = lib.leone_argmax_static(logits.data_ptr(), out.data_ptr(), rows, vocab, torch.cuda.current_stream().cuda_stream)
    assert status == 0, lib.leone_last_error().decode()
    for replay in range(3):
        logits.copy_(torch.randn(rows, vocab, device=device))
        out.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ops.argmax(logits)), replay
