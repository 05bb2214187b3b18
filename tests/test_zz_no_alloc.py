"""The greedy choice that allocates nothing (fmsamd_argmax_static), called through ctypes as a caller outside
this package would, against the entry point with a caller's workspace (fmsamd_argmax) and against torch:
two calls in a row, the second with a smaller input, so that what the first call left in the library's own
scratch array would show if the second read it."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fms_amd  # noqa: F401
    from fms_amd.kernels.build import ensure_built

    handle = ctypes.CDLL(ensure_built(verbose=False))
    handle.fmsamd_last_error.restype = ctypes.c_char_p
    handle.fmsamd_argmax_workspace.restype = ctypes.c_long
    handle.fmsamd_argmax_workspace.argtypes = [ctypes.c_int, ctypes.c_int]
    handle.fmsamd_argmax.restype = ctypes.c_int
    handle.fmsamd_argmax.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_long,
                                     ctypes.c_void_p, ctypes.c_void_p]
    handle.fmsamd_argmax_static.restype = ctypes.c_int
    handle.fmsamd_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_long, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    return handle


def both(lib, logits):
    """Tokens of the entry point with a workspace and of the one without, for float32 logits on the GPU."""
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.fmsamd_argmax_workspace(rows, vocab)
    workspace = torch.empty(nbytes // 4, dtype=torch.float32, device="cuda")
    with_workspace = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    without = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    code = lib.fmsamd_argmax(logits.data_ptr(), logits.stride(0), rows, vocab, workspace.data_ptr(), nbytes,
                             with_workspace.data_ptr(), stream)
    assert code == 0, lib.fmsamd_last_error().decode()
    # Free device memory as the driver reports it (torch's own counters see torch's allocator only, and the entry
    # point is called past it): nothing may be taken or given back between the two readings.
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    code = lib.fmsamd_argmax_static(logits.data_ptr(), logits.stride(0), rows, vocab, without.data_ptr(), stream)
    assert code == 0, lib.fmsamd_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    return with_workspace.cpu(), without.cpu()


def test_two_calls_in_a_row_the_second_smaller(lib):
    torch.manual_seed(3)
    large = torch.randn(48, 128256, device="cuda")
    large[5, 100000] = large[5, 777] = 40.0  # equal maxima: the lowest index wins
    large[7] = -1e30  # a row whose maximum is everywhere
    small = torch.randn(3, 5000, device="cuda") - 100.0  # every value below the first call's: stale partial results would win
    small[1, 4999] = -50.0
    for logits in (large, small, large[:2, :300].contiguous(), large):
        a, b = both(lib, logits)
        want = logits.argmax(-1).cpu().int()
        if logits is large:
            want[5], want[7] = 777, 0
        assert a.tolist() == want.tolist()
        assert b.tolist() == want.tolist()
    # a view with a row stride of its own
    wide = torch.randn(4, 9000, device="cuda")
    a, b = both(lib, wide[:, 1000:7000])
    assert a.tolist() == b.tolist() == wide[:, 1000:7000].argmax(-1).cpu().tolist()


def test_the_call_can_be_captured_into_a_graph(lib):
    """A stream that is capturing refuses every allocation on the host, without touching the GPU: after one call
    that has looked the array's address up, the entry point records into a graph, and the replays (with the
    program's own work between them) give what the eager call gives."""
    torch.manual_seed(4)
    logits = torch.randn(5, 40000, device="cuda")
    out = torch.full((5,), -1, dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert lib.fmsamd_argmax_static(logits.data_ptr(), logits.stride(0), 5, 40000, out.data_ptr(), side.cuda_stream) == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert out.tolist() == logits.argmax(-1).tolist()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        code = lib.fmsamd_argmax_static(logits.data_ptr(), logits.stride(0), 5, 40000, out.data_ptr(),
                                        torch.cuda.current_stream().cuda_stream)
    assert code == 0, lib.fmsamd_last_error().decode()
    for replay in range(3):
        logits.copy_(torch.randn(5, 40000, device="cuda"))
        logits[replay, 123 + replay] = 30.0
        out.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert out.tolist() == logits.argmax(-1).tolist() and out[replay] == 123 + replay


def test_sizes_beyond_the_scratch_array_are_refused(lib):
    stream = torch.cuda.current_stream().cuda_stream
    out = torch.zeros(1024, dtype=torch.int32, device="cuda")
    logits = torch.zeros(1024, 2048 * 33, device="cuda")  # 1024 x 33 partial results: more than 32768
    assert lib.fmsamd_argmax_static(logits.data_ptr(), logits.stride(0), 1024, 2048 * 33, out.data_ptr(), stream) != 0
    message = lib.fmsamd_last_error().decode()
    assert "array holds" in message and "fmsamd_argmax" in message
    assert lib.fmsamd_argmax_static(logits.data_ptr(), logits.stride(0), 1024, 2048 * 32, out.data_ptr(), stream) == 0
    torch.cuda.synchronize()
    assert out.tolist() == [0] * 1024
    assert lib.fmsamd_argmax_static(logits.data_ptr(), 10, 4, 2048, out.data_ptr(), stream) != 0  # a row stride below the row
    assert lib.fmsamd_argmax_static(None, 2048, 4, 2048, out.data_ptr(), stream) != 0
