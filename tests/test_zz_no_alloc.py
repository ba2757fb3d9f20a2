"""The sampling entry point that allocates nothing, called through ctypes: its tokens are those
of the entry point that takes a workspace, on two calls in a row, the second smaller."""

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
