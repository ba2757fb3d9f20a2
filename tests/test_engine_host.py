"""The engine's host logic (model assembly, cache, step function) on the CPU,
with the plain PyTorch twins standing in for the kernels, against the plain
implementation. These tests find faults of the cache and the batch; the kernels
themselves are tested on the GPU."""

import pytest
import torch

import plain_qwen3
from helpers import (TINY, max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions,
                     trace_tail_decoded, trace_whole)
from qwen3_from_scratch_amd.engine import load_runner


def _requests(name, lengths, seed=5):
    vocab = TINY[name]["config"]["vocab_size"]
    return {"r%d" % i: random_tokens(n, vocab, seed + i) for i, n in enumerate(lengths)}


def _plain(folder, requests):
    cfg, w = plain_qwen3.read_model_folder(folder)
    return {rid: plain_qwen3.logits_of_sequence(cfg, w, toks) for rid, toks in requests.items()}


def _compare(got, want, tol):
    worst = 0.0
    for rid, logits in want.items():
        for p in range(logits.shape[0]):
            assert (rid, p) in got, "no logits for %s at %d" % (rid, p)
            worst = max(worst, float((got[(rid, p)] - logits[p]).abs().max()))
    assert worst <= tol, "largest difference %g" % worst


@pytest.mark.parametrize("name,lengths", [("A", [5, 17, 33]), ("B", [1, 9, 64, 130]), ("C", [40, 70]), ("D", [33, 70])])
@pytest.mark.parametrize("family", ["whole", "tail", "portions", "mixed"])
def test_every_cutting_matches_plain(cpu_ops, model_folders, name, lengths, family):
    requests = _requests(name, lengths)
    want = _plain(model_folders[name], requests)
    steps = {"whole": trace_whole, "tail": trace_tail_decoded, "portions": trace_portions,
             "mixed": trace_mixed}[family](requests)
    page = TINY[name]["page_size"]
    tokens = max_live_tokens(steps, page=page)
    runner = load_runner(model_folders[name], dtype="float32", device="cpu", page_size=page,
                         max_tokens=tokens, max_requests=4)
    got = run_trace(runner, steps)
    _compare(got, want, 2e-5)
    assert runner.manager.num_free() == runner.manager.num_pages()
