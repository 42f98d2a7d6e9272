"""The entry point that allocates nothing (`ei_argmax_static`), called through ctypes and
compared with `ei_argmax`, which takes its partial results in a buffer from the caller."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def sampling():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from edge_infer_amd.csrc import build
    handle = ctypes.CDLL(str(build.build_library("sampling")))
    handle.ei_argmax_static.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    handle.ei_argmax_static.restype = ctypes.c_int
    handle.ei_argmax_static_prepare.argtypes = []
    handle.ei_argmax_static_prepare.restype = ctypes.c_int
    handle.ei_argmax.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                 ctypes.c_void_p, ctypes.c_void_p, ctypes.c_longlong,
                                 ctypes.c_void_p]
    handle.ei_argmax.restype = ctypes.c_int
    handle.ei_argmax_partial_size.argtypes = [ctypes.c_int, ctypes.c_int]
    handle.ei_argmax_partial_size.restype = ctypes.c_int
    handle.ei_last_error.restype = ctypes.c_char_p
    # the array's address is looked up once per device, outside any capture and before the
    # driver's free memory is read below (the lookup may load the library's code)
    assert handle.ei_argmax_static_prepare() == 0, handle.ei_last_error()
    return handle


def _logits(rows, vocab, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    logits = torch.randn((rows, vocab), generator=g, device="cuda", dtype=torch.float32)
    # ties across chunks (the lowest index wins), a NaN, and a row whose best is its last element
    logits[0, 5000] = logits[0, vocab - 3] = 50.0
    if rows > 1:
        logits[1, 7] = float("nan")
        logits[1, vocab - 1] = 60.0
    return logits


def _both(sampling, logits):
    rows, vocab = logits.shape
    stream = torch.cuda.current_stream().cuda_stream
    need = sampling.ei_argmax_partial_size(rows, vocab)
    partial = torch.empty(max(1, 2 * need), dtype=torch.float32, device="cuda")
    want = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    want_p = torch.zeros(rows, dtype=torch.float32, device="cuda")
    status = sampling.ei_argmax(logits.data_ptr(), rows, vocab, want.data_ptr(), want_p.data_ptr(),
                                partial.data_ptr() if need else None, need, stream)
    assert status == 0, sampling.ei_last_error()
    got = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    got_p = torch.zeros(rows, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    # the driver's own count of free bytes: it sees an allocation by anyone in the process,
    # which torch's statistics (its own allocator's only) would not
    free_before, _ = torch.cuda.mem_get_info()
    torch_before = torch.cuda.memory_stats()["allocation.all.allocated"]
    status = sampling.ei_argmax_static(logits.data_ptr(), rows, vocab, got.data_ptr(),
                                       got_p.data_ptr(), stream)
    assert status == 0, sampling.ei_last_error()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after >= free_before, f"{free_before - free_after} bytes were allocated"
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == torch_before
    return got.tolist(), want.tolist(), got_p.tolist(), want_p.tolist()


def test_two_calls_in_a_row_the_second_smaller(sampling):
    large = _logits(9, 151936, seed=1)
    small = _logits(3, 20000, seed=2)       # fewer rows and chunks: stale partial results remain
    for logits in (large, small, large):
        got, want, got_p, want_p = _both(sampling, logits)
        assert got == want == logits.nan_to_num(nan=float("-inf")).argmax(dim=1).tolist()
        assert got_p == want_p
    assert _both(sampling, large)[0][0] == 5000     # the tie went to the lower index


def test_narrow_vocabulary_needs_no_partial_results(sampling):
    logits = _logits(4, 8192, seed=3)
    got, want, _, _ = _both(sampling, logits)
    assert got == want == logits.nan_to_num(nan=float("-inf")).argmax(dim=1).tolist()


def test_sizes_beyond_the_static_buffer_are_refused(sampling):
    rows, vocab = 300, 1_000_000          # 300 * 245 chunks > 65536
    logits = torch.empty((1,), dtype=torch.float32, device="cuda")   # never read: refused first
    tokens = torch.empty((rows,), dtype=torch.int32, device="cuda")
    status = sampling.ei_argmax_static(logits.data_ptr(), rows, vocab, tokens.data_ptr(), None,
                                       torch.cuda.current_stream().cuda_stream)
    assert status != 0
    assert b"65536" in sampling.ei_last_error()
    assert sampling.ei_argmax_static(logits.data_ptr(), 0, vocab, tokens.data_ptr(), None, None) != 0


def test_captured_in_a_graph_and_replayed(sampling):
    """The call inside a stream capture (after the address was looked up outside one), then
    replayed over changing logits, with eager work of the program between the replays; every
    replay against the eager entry point."""
    rows, vocab = 5, 151936
    logits = _logits(rows, vocab, seed=4)
    tokens = torch.full((rows,), -7, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        status = sampling.ei_argmax_static(logits.data_ptr(), rows, vocab, tokens.data_ptr(), None,
                                           torch.cuda.current_stream().cuda_stream)
    assert status == 0, sampling.ei_last_error()
    for seed in (5, 6, 7, 8):
        logits.copy_(_logits(rows, vocab, seed=seed))
        tokens.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        got = tokens.tolist()
        # eager work between the replays: the same search through the other entry point,
        # and a smaller call of this one that leaves stale partial results behind
        assert got == _both(sampling, logits)[0]
        _both(sampling, _logits(2, 20000, seed=seed + 10))
        assert got == logits.nan_to_num(nan=float("-inf")).argmax(dim=1).tolist()
