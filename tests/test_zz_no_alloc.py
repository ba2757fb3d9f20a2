"""The sampling entry point that allocates nothing, called through ctypes: its tokens are those
of the entry point that takes a workspace, on two calls in a row, the second smaller; the
device's free memory does not move across its calls; and a call captured in a graph (after a
first call outside it) gives the same tokens on every replay."""

import ctypes

import pytest
import torch

from qwen3_from_scratch_amd.ops import library

pytestmark = pytest.mark.gpu
UNSUPPORTED = 10002


def _operands(rows, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    logits = (torch.randn((rows, vocab), generator=g) * 3.0).cuda()
    temperature = torch.tensor([0.0 if r % 3 == 0 else 0.5 + 0.25 * (r % 4) for r in range(rows)],
                               dtype=torch.float32).cuda()
    top_k = torch.tensor([0 if r % 2 else 5 + r for r in range(rows)], dtype=torch.int32).cuda()
    seeds = torch.tensor([1000 + 7 * r for r in range(rows)], dtype=torch.int64).cuda()
    counters = torch.tensor([r % 5 for r in range(rows)], dtype=torch.int32).cuda()
    return logits, temperature, top_k, seeds, counters


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, rows, vocab, seed):
    logits, temperature, top_k, seeds, counters = _operands(rows, vocab, seed)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    lib.q3_sample_workspace.restype = ctypes.c_long
    workspace = torch.empty((lib.q3_sample_workspace(rows, vocab) + 7) // 8, dtype=torch.int64, device="cuda")
    want = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    got = torch.full((rows,), -2, dtype=torch.int32, device="cuda")
    assert lib.q3_sample(_p(logits), _p(temperature), _p(top_k), _p(seeds), _p(counters), _p(want), rows, vocab, 1,
                         _p(workspace), stream) == 0
    assert lib.q3_sample_static(_p(logits), _p(temperature), _p(top_k), _p(seeds), _p(counters), _p(got), rows,
                                vocab, 1, stream) == 0
    torch.cuda.synchronize()
    assert got.tolist() == want.tolist()
    assert 0 <= min(got.tolist()) and max(got.tolist()) < vocab
    # greedy rows are the arg-max
    greedy = [r for r in range(rows) if r % 3 == 0]
    assert [got[r].item() for r in greedy] == logits.argmax(dim=1)[greedy].tolist()


def test_two_calls_in_a_row_the_second_smaller():
    lib = library("sampling")
    _both(lib, 24, 5000, 1)
    _both(lib, 3, 777, 2)           # fewer rows, fewer chunks: what the first call left behind is not read
    _both(lib, 24, 5000, 3)


def test_sizes_beyond_the_array_are_refused():
    lib = library("sampling")
    lib.q3_sample_workspace.restype = ctypes.c_long
    rows, vocab = 300, 151936
    assert lib.q3_sample_workspace(rows, vocab) > 320 * 1024
    logits, temperature, top_k, seeds, counters = _operands(2, 16, 0)      # never read: the call launches nothing
    out = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.q3_sample_static(_p(logits), _p(temperature), _p(top_k), _p(seeds), _p(counters), _p(out), rows,
                                vocab, 1, stream) == UNSUPPORTED
    torch.cuda.synchronize()
    assert out.tolist() == [-7, -7]
    # the largest size it is made for
    assert lib.q3_sample_workspace(256, vocab) <= 320 * 1024


def _static(lib, operands, out):
    logits, temperature, top_k, seeds, counters = operands
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return lib.q3_sample_static(_p(logits), _p(temperature), _p(top_k), _p(seeds), _p(counters), _p(out),
                                logits.shape[0], logits.shape[1], 1, stream)


def test_no_device_memory_is_taken_across_calls():
    lib = library("sampling")
    small, large = _operands(3, 777, 4), _operands(24, 5000, 5)
    out = torch.empty((24,), dtype=torch.int32, device="cuda")
    assert _static(lib, large, out) == 0          # the first call on the device: the array's address is asked for
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(20):
        assert _static(lib, small, out) == 0 and _static(lib, large, out) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before and torch.cuda.memory_reserved() == reserved_before


def test_a_captured_call_replays_to_the_same_tokens():
    """Under stream capture nothing may allocate. The call is captured after a first call outside
    the capture, replayed with other work and synchronisations in between and with new logits
    in the captured buffers each time, and every replay is held against q3_sample."""
    lib = library("sampling")
    rows, vocab = 16, 4000
    operands = list(_operands(rows, vocab, 6))
    out = torch.full((rows,), -1, dtype=torch.int32, device="cuda")
    assert _static(lib, operands, out) == 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert _static(lib, operands, out) == 0
    lib.q3_sample_workspace.restype = ctypes.c_long
    workspace = torch.empty((lib.q3_sample_workspace(rows, vocab) + 7) // 8, dtype=torch.int64, device="cuda")
    want = torch.empty((rows,), dtype=torch.int32, device="cuda")
    for replay in range(4):
        operands[0].copy_(_operands(rows, vocab, 10 + replay)[0])        # new logits, same addresses
        operands[4].add_(1)                                              # the requests' next token
        out.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.q3_sample(_p(operands[0]), _p(operands[1]), _p(operands[2]), _p(operands[3]), _p(operands[4]),
                             _p(want), rows, vocab, 1, _p(workspace), stream) == 0
        _both(lib, 5, 900, 20 + replay)                                  # the array is used by others in between
        torch.cuda.synchronize()
        assert out.tolist() == want.tolist(), replay
