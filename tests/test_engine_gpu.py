"""The engine on the GPU against the plain implementation, in float32 and in
bfloat16: every request alone and whole; most of it in one step and the last 32
tokens one by one; portions of changing size; mixed batches with so few pages
that they are used again; long decoding; the first tokens of a sequence."""

import random

import pytest
import torch

import plain_qwen3
from helpers import (TINY, max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions,
                     trace_tail_decoded, trace_whole)
from qwen3_from_scratch_amd.engine import load_runner

pytestmark = pytest.mark.gpu

# float32: the engine and the plain implementation differ by rounding order only.
# bfloat16: activations are rounded to 8 bits of mantissa between kernels; a row's logits may
# be off by a fiftieth of the row's own spread (largest minus smallest logit), which is what a
# handful of such roundings come to and far less than a key, a tile or a page left out.
TOL = {"float32": 2e-4, "bfloat16": 2e-2}

_plain_cache = {}


def _requests(name, lengths, seed=5):
    vocab = TINY[name]["config"]["vocab_size"]
    return {"r%d" % i: random_tokens(n, vocab, seed + i) for i, n in enumerate(lengths)}


def _plain(folder, name, requests):
    out = {}
    cfg, w = None, None
    for rid, toks in requests.items():
        key = (name, tuple(toks))
        if key not in _plain_cache:
            if cfg is None:
                cfg, w = plain_qwen3.read_model_folder(folder)
            _plain_cache[key] = plain_qwen3.logits_of_sequence(cfg, w, toks)
        out[rid] = _plain_cache[key]
    return out


def _compare(got, want, dtype):
    worst, where = 0.0, None
    for rid, logits in want.items():
        for p in range(logits.shape[0]):
            assert (rid, p) in got, "no logits for %s at %d" % (rid, p)
            diff = float((got[(rid, p)] - logits[p]).abs().max())
            if dtype == "float32":
                unit = max(1.0, float(logits[p].abs().max()))
            else:
                unit = float(logits[p].max() - logits[p].min())
            if diff / unit > worst:
                worst, where = diff / unit, (rid, p, diff, unit)
    assert worst <= TOL[dtype], "largest difference %g of its unit at %s (bound %g)" % (worst, where, TOL[dtype])
    return worst


CASES = [("A", [5, 17, 33, 80]), ("B", [1, 9, 64, 130]), ("C", [40, 70, 3, 201]),
         ("D", [33, 1, 150, 64, 300]), ("E", [129, 31, 260]),
         ("DS", [33, 1, 150, 64, 300]), ("ES", [129, 31, 260]), ("DP", [200, 17, 330, 64]), ("EP", [129, 300, 70]),
         ("F", [70, 100, 128, 230])]
FAMILIES = {"whole": trace_whole, "tail": trace_tail_decoded, "portions": trace_portions, "mixed": trace_mixed}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,lengths", CASES)
@pytest.mark.parametrize("family", list(FAMILIES))
def test_every_cutting_matches_plain(model_folders, dtype, name, lengths, family):
    requests = _requests(name, lengths)
    want = _plain(model_folders[name], name, requests)
    steps = FAMILIES[family](requests)
    page = TINY[name]["page_size"]
    runner = load_runner(model_folders[name], dtype=dtype, device="cuda", page_size=page,
                         max_tokens=max_live_tokens(steps, page=page), max_requests=4)
    got = run_trace(runner, steps)
    _compare(got, want, dtype)
    assert runner.manager.num_free() == runner.manager.num_pages()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("family", ["portions", "mixed"])
def test_steps_of_65_to_128_rows(model_folders, dtype, family):
    """Configuration F (width 128, inner sizes 192 and 256) in steps of 65 to 128 rows: in bfloat16
    those take the tiled matrix-core product with the residual addition and the norms in its
    epilogues, which no other tiny configuration reaches (their widths are no multiple of 64).
    Portions of 70, 100 and 128 tokens of one request, and portions of 40 to 60 tokens of two or
    three requests side by side."""
    from qwen3_from_scratch_amd import ops

    name = "F"
    requests = _requests(name, [298, 170, 230, 129])
    want = _plain(model_folders[name], name, requests)
    if family == "portions":
        steps = trace_portions(requests, sizes=(70, 100, 128))
    else:
        steps, at, live = [], {rid: 0 for rid in requests}, ["r0", "r1"]
        waiting = ["r2", "r3"]
        k = 0
        while live:
            entries, ends = [], []
            for rid in list(live):
                n = min((40, 47, 60, 33)[k % 4], len(requests[rid]) - at[rid])
                k += 1
                entries.append((rid, requests[rid][at[rid]:at[rid] + n], list(range(n))))
                at[rid] += n
                if at[rid] == len(requests[rid]):
                    ends.append(rid)
                    live.remove(rid)
                    if waiting:
                        live.append(waiting.pop(0))
            steps.append((entries, ends))
    rows = [sum(len(t) for _, t, _ in entries) for entries, _ in steps]
    assert sum(64 < r <= 128 for r in rows) >= 6
    runner = load_runner(model_folders[name], dtype=dtype, device="cuda", page_size=16,
                         max_tokens=max_live_tokens(steps, page=16), max_requests=4)
    if dtype == "bfloat16":          # the sizes are the tiled kernel's: the test would say nothing otherwise
        mixer = runner.model.layers[0].mixer
        assert ops.fused_rows_take(mixer.qkv.weight, 100) and ops.few_rows_limit(mixer.qkv.weight) == 64
    _compare(run_trace(runner, steps), want, dtype)
    assert runner.manager.num_free() == runner.manager.num_pages()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,lengths,page", [("DS", [33, 1, 150, 64, 300], 64), ("EP", [129, 300, 70], 256),
                                               ("B", [1, 9, 64, 130], 128)])
def test_large_pages(model_folders, dtype, name, lengths, page):
    """Pages of 64 to 256 tokens (a page holds several of the kernels' key tiles): portions and
    single tokens mixed, with so few pages that they are used again."""
    requests = _requests(name, lengths)
    want = _plain(model_folders[name], name, requests)
    steps = trace_mixed(requests)
    runner = load_runner(model_folders[name], dtype=dtype, device="cuda", page_size=page,
                         max_tokens=max_live_tokens(steps, page=page), max_requests=4)
    _compare(run_trace(runner, steps), want, dtype)
    assert runner.manager.num_free() == runner.manager.num_pages()


@pytest.mark.parametrize("name,lengths", [("DS", [33, 1, 150, 64, 300]), ("EP", [129, 300, 70]), ("B", [1, 9, 64, 130])])
def test_matrices_held_once(model_folders, name, lengths):
    """Without the tile-ordered copy of the matrices (half the weights' memory) steps of few rows
    take the row-major product kernels and the norms' own kernels: the same bounds hold."""
    requests = _requests(name, lengths)
    want = _plain(model_folders[name], name, requests)
    steps = trace_mixed(requests)
    page = TINY[name]["page_size"]
    runner = load_runner(model_folders[name], dtype="bfloat16", device="cuda", page_size=page,
                         max_tokens=max_live_tokens(steps, page=page), max_requests=4, tiled_weights=False)
    assert all(getattr(part, "tiled", None) is None for layer in runner.model.layers
               for part in (layer.mixer.qkv, layer.mixer.out, layer.feed_forward.gate_up, layer.feed_forward.down))
    _compare(run_trace(runner, steps), want, "bfloat16")


@pytest.mark.parametrize("name,lengths", [("ES", [129, 31, 260]), ("D", [33, 1, 150, 64, 300])])
def test_two_engines_give_the_same_bits(model_folders, name, lengths):
    """Nothing on the path is chosen by a stopwatch: two engines built one after the other give
    bit-equal bfloat16 logits for the same steps (prompt portions of 17 to 128 rows and more,
    single tokens, graph replays), whatever was run between them."""
    from qwen3_from_scratch_amd import ops

    requests = _requests(name, lengths)
    steps = trace_mixed(requests, seed=11)
    page = TINY[name]["page_size"]
    kw = dict(dtype="bfloat16", device="cuda", page_size=page, max_tokens=max_live_tokens(steps, page=page),
              max_requests=4)
    first = run_trace(load_runner(model_folders[name], **kw), steps)
    # other sizes and other products in between
    x = torch.randn(300, 256, device="cuda").to(torch.bfloat16)
    ops.linear(x, torch.randn(512, 256, device="cuda").to(torch.bfloat16))
    second = run_trace(load_runner(model_folders[name], **kw), steps)
    assert first.keys() == second.keys()
    assert all(torch.equal(first[k], second[k]) for k in first)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_folders, dtype):
    """A short prompt and then hundreds of tokens one by one, across many pages."""
    name = "B"
    toks = random_tokens(400, TINY[name]["config"]["vocab_size"], 77)
    requests = {"long": toks}
    want = _plain(model_folders[name], name, requests)
    steps = trace_tail_decoded(requests, tail=390)
    runner = load_runner(model_folders[name], dtype=dtype, device="cuda", page_size=8, max_tokens=448,
                         max_requests=2)
    _compare(run_trace(runner, steps), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens(model_folders, dtype):
    """Positions 0, 1, 2 of a sequence, each fed alone: one key, two keys, three."""
    for name in ("A", "B"):
        toks = random_tokens(3, TINY[name]["config"]["vocab_size"], 3)
        requests = {"f": toks}
        want = _plain(model_folders[name], name, requests)
        steps = [([("f", [t], [0])], ["f"] if i == 2 else []) for i, t in enumerate(toks)]
        runner = load_runner(model_folders[name], dtype=dtype, device="cuda",
                             page_size=TINY[name]["page_size"], max_tokens=64, max_requests=2)
        _compare(run_trace(runner, steps), want, dtype)


def test_graph_replay_equals_eager_steps(model_folders):
    """Single-token steps replay a captured graph; the same steps run eagerly give the same
    logits up to the order of the splits' sums."""
    name = "D"
    requests = _requests(name, [70, 33, 150])
    steps = trace_mixed(requests, seed=7, decode_tail=40)
    kw = dict(dtype="bfloat16", device="cuda", page_size=16, max_tokens=max_live_tokens(steps, page=16),
              max_requests=4)
    a = run_trace(load_runner(model_folders[name], use_graphs=True, **kw), steps)
    b = run_trace(load_runner(model_folders[name], use_graphs=False, **kw), steps)
    assert a.keys() == b.keys()
    worst = max(float((a[k] - b[k]).abs().max()) for k in a)
    assert worst < 2e-2, worst


def test_batches_of_nearby_sizes_share_a_graph(model_folders):
    """Decoding batches of 11, 9, 10, 5, 7 and 6 requests replay graphs captured for 12, 6 and 8
    rows; the rows that fill a batch up change no request's logits and leave no trace in the
    cache, and steps in between that leave requests out go on correctly."""
    name = "D"
    vocab = TINY[name]["config"]["vocab_size"]
    requests = {"r%d" % i: random_tokens(20 + 3 * i, vocab, 60 + i) for i in range(11)}
    steps = [([(rid, toks[:-8], [])], []) for rid, toks in requests.items()]       # prompts, one a step
    fed = {rid: len(toks) - 8 for rid, toks in requests.items()}
    for size, seed in [(11, 0), (9, 1), (10, 2), (5, 3), (7, 4), (6, 5), (11, 6), (6, 7)]:
        chosen = random.Random(seed).sample(sorted(requests), size)
        entries = []
        for rid in chosen:
            entries.append((rid, [requests[rid][fed[rid]]], [0]))
            fed[rid] += 1
        steps.append((entries, []))
    steps.append(([], list(requests)))
    kw = dict(dtype="bfloat16", device="cuda", page_size=16, max_tokens=max_live_tokens(steps, page=16),
              max_requests=12)
    with_graphs = load_runner(model_folders[name], use_graphs=True, **kw)
    a = run_trace(with_graphs, steps)
    b = run_trace(load_runner(model_folders[name], use_graphs=False, **kw), steps)
    assert a.keys() == b.keys() and len(a) == 11 + 9 + 10 + 5 + 7 + 6 + 11 + 6
    worst = max(float((a[k] - b[k]).abs().max()) for k in a)
    assert worst < 2e-2, worst
    assert sorted(rows for rows, _ in with_graphs._graphs) == [6, 8, 12]
    with_graphs.manager.audit()
    assert all(g.pool.num_free == g.pool.num_pages for g in with_graphs.manager.groups)

