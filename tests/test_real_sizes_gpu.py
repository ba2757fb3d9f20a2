"""Layers of the Qwen3-8B configuration's sizes (hidden 4096, 32 query and 8 key
heads of 128, feed-forward 12288, vocabulary 151936) with random weights, two of
them instead of 36 so that the plain implementation finishes on the CPU: the
sizes at which the matrix-core kernels, the weight-streaming GEMM and the
vocabulary-wide head actually run. Every comparison takes its truth from the
plain implementation, never from another run of the engine."""

import pytest
import torch

import plain_qwen3
from helpers import (max_live_tokens, nearly_the_best, off_by, random_tokens, run_trace, trace_mixed,
                     trace_portions, trace_tail_decoded, trace_whole)
from qwen3_from_scratch_amd.config import ModelConfig
from qwen3_from_scratch_amd.engine import StepEntry, load_runner
from qwen3_from_scratch_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

VOCAB = 151936
CONFIG = dict(architectures=["Qwen3ForCausalLM"], vocab_size=VOCAB, hidden_size=4096, hidden_act="silu",
              num_hidden_layers=2, max_position_embeddings=40960, num_attention_heads=32,
              num_key_value_heads=8, head_dim=128, intermediate_size=12288, rms_norm_eps=1e-6,
              rope_theta=1000000.0, tie_word_embeddings=False)
BOUND = {"float32": 1.5, "bfloat16": 1.0}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("real") / "two_layers")
    write_random_model(path, ModelConfig.from_dict(CONFIG), seed=5, std=0.02, norm_jitter=0.1)
    return path


@pytest.fixture(scope="module")
def plain(folder):
    """The plain implementation's logits of a sequence at some places, each sequence once."""
    cfg, w = plain_qwen3.read_model_folder(folder)
    known = {}

    def logits(tokens, places):
        key = (tuple(tokens), tuple(places))
        if key not in known:
            known[key] = plain_qwen3.logits_of_sequence(cfg, w, list(tokens), rows=list(places))
        return known[key]

    return logits


@pytest.fixture(scope="module")
def truth(plain):
    requests = {"a": random_tokens(150, VOCAB, 1), "b": random_tokens(70, VOCAB, 2), "c": random_tokens(33, VOCAB, 3)}
    rows = {rid: sorted({0, 1, len(t) // 2, len(t) - 2, len(t) - 1}) for rid, t in requests.items()}
    want = {rid: plain(toks, rows[rid]) for rid, toks in requests.items()}
    return requests, rows, want


FAMILIES = {"whole": trace_whole, "tail": lambda r: trace_tail_decoded(r, tail=32), "portions": trace_portions,
            "mixed": lambda r: trace_mixed(r, seed=2)}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("family", list(FAMILIES))
def test_real_layer_sizes_match_plain(folder, truth, dtype, family):
    requests, rows, want = truth
    steps = FAMILIES[family](requests)
    runner = load_runner(folder, dtype=dtype, page_size=16, max_tokens=max_live_tokens(steps, page=16),
                         max_requests=4)
    got = run_trace(runner, steps)
    for rid, logits in want.items():
        for i, p in enumerate(rows[rid]):
            assert off_by(got[(rid, p)], logits[i], dtype) <= BOUND[dtype], (rid, p)


def test_tight_pages_and_preemption_at_real_sizes(folder, plain):
    """Sixteen requests through the engine twice, once with room for everything and once with
    small portions, few sequences per step and so few pages that requests are preempted. In
    float32 every kernel sums a row's numbers in an order that does not depend on the batch, so
    the two runs give the same greedy tokens to the last one; and given the tokens before it,
    every one of them is the plain implementation's best (or level with it to a part in ten
    thousand of the row's spread, which is what two float32 summation orders may differ by)."""
    from qwen3_from_scratch_amd.engine import SyncEngine

    g = torch.Generator().manual_seed(9)
    lengths = torch.randint(64, 600, (16,), generator=g).tolist()
    news = torch.randint(8, 40, (16,), generator=g).tolist()
    prompts = [random_tokens(n, VOCAB, 100 + i) for i, n in enumerate(lengths)]

    def run(**kw):
        engine = SyncEngine(path=folder, dtype="float32", block_size=16, **kw)
        requests = [engine.add_request(p, engine.default_params(n, temperature=0.0, ignore_eos=True))
                    for p, n in zip(prompts, news)]
        while engine.scheduler.has_work():
            engine.step()
            engine.runner.manager.audit()
        assert engine.runner.manager.num_free() == engine.runner.manager.num_pages()
        return [r.generated for r in requests], sum(r.preemptions for r in requests)

    roomy, _ = run(num_blocks=16 * 48, max_num_seqs=16, max_num_tokens=4096, chunked_prefill_size=512)
    tight, preemptions = run(num_blocks=120, max_num_seqs=5, max_num_tokens=300, chunked_prefill_size=96)
    assert [len(t) for t in roomy] == news
    assert preemptions > 0
    assert tight == roomy
    for prompt, new in zip(prompts, tight):
        places = [len(prompt) - 1 + i for i in range(len(new))]
        logits = plain(prompt + new, places)
        for i, token in enumerate(new):
            assert nearly_the_best(logits[i], token, share=1e-4), (len(prompt), i)


LONG_PLACES = [0, 1499, 2559, 2998, 2999]


@pytest.fixture(scope="module")
def long_prompt(plain):
    tokens = random_tokens(3000, VOCAB, 7)
    return tokens, plain(tokens, LONG_PLACES)


@pytest.mark.parametrize("dtype,portion", [("bfloat16", 3000), ("bfloat16", 512), ("bfloat16", 300),
                                           ("float32", 3000), ("float32", 700)])
def test_long_prompt_in_portions_at_real_sizes(folder, long_prompt, dtype, portion):
    """A prompt of 3,000 tokens whole and in portions of 700, 512 and 300: the later portions run
    over thousands of cached keys, where the prompt kernel shares a row tile's keys out over
    several blocks and a further kernel joins their results."""
    tokens, want = long_prompt
    runner = load_runner(folder, dtype=dtype, page_size=16, max_tokens=3008, max_requests=2)
    got, at = {}, 0
    while at < len(tokens):
        part = tokens[at:at + portion]
        here = [p for p in LONG_PLACES if at <= p < at + len(part)]
        logits = runner.step([StepEntry("long", part, [p - at for p in here])])
        for row, p in enumerate(here):
            got[p] = logits[row].float().cpu()
        at += len(part)
    runner.finish("long")
    assert runner.manager.num_free() == runner.manager.num_pages()
    for i, p in enumerate(LONG_PLACES):
        assert off_by(got[p], want[i], dtype) <= BOUND[dtype], (portion, p)


COUNT = 40


@pytest.fixture(scope="module")
def forty(plain):
    """Forty requests: prompts of 20 to 59 tokens and six more tokens each, with the plain
    implementation's logits at the prompt's last place and at the six."""
    prompts = [random_tokens(20 + i, VOCAB, 300 + i) for i in range(COUNT)]
    tails = [random_tokens(6, VOCAB, 400 + i) for i in range(COUNT)]
    want = {}
    for i, (p, t) in enumerate(zip(prompts, tails)):
        places = list(range(len(p) - 1, len(p) + 6))
        for place, row in zip(places, plain(p + t, places)):
            want[("r%d" % i, place)] = row
    return prompts, tails, want


@pytest.mark.parametrize("which", ["both", "library", "own"])
def test_some_tens_of_rows_at_real_sizes(folder, forty, which):
    """Steps of 17 to 128 rows, where the tiled matrix-core kernel carries the residual addition
    and the norms: prompts of 20 to 59 tokens one at a time, then forty requests that decode
    together. "library": every such product goes the other way, the library's product with the
    division behind it, and every writer leaves its size to the plain product and the norm's own
    kernel; "own": the tiled kernel wherever it takes the size."""
    from qwen3_from_scratch_amd import ops

    prompts, tails, want = forty
    steps = [([("r%d" % i, p, [len(p) - 1])], []) for i, p in enumerate(prompts)]
    for t in range(6):
        steps.append(([("r%d" % i, [tails[i][t]], [0]) for i in range(COUNT)], []))
    steps[-1] = (steps[-1][0], ["r%d" % i for i in range(COUNT)])
    ops.matmul_kernels(which)
    try:
        runner = load_runner(folder, dtype="bfloat16", page_size=16, max_tokens=max_live_tokens(steps, page=16),
                             max_requests=COUNT)
        got = run_trace(runner, steps)
    finally:
        ops.matmul_kernels("both")
    assert set(want) == set(got) and len(got) == COUNT * 7
    for key, logits in want.items():
        assert off_by(got[key], logits, "bfloat16") <= 1.0, (which, key)


@pytest.mark.parametrize("max_num_seqs", [COUNT, 4])
def test_generation_at_some_tens_of_rows(folder, forty, plain, max_num_seqs):
    """Greedy generation of forty requests together (graph replays of 40 rows: the tiled kernel's
    fusions) and four at a time (the few-row kernels' fusions). bfloat16 rounds differently along
    the two paths and a near tie between two tokens may fall either way: given the tokens before
    it, every token is the plain implementation's best or within a fiftieth of the row's spread."""
    from qwen3_from_scratch_amd.engine import SyncEngine

    prompts = forty[0]
    engine = SyncEngine(path=folder, dtype="bfloat16", block_size=16, num_blocks=COUNT * 8,
                        max_num_seqs=max_num_seqs, max_num_tokens=4096, chunked_prefill_size=512,
                        enable_prefix_cache=False)
    tokens = engine.generate_ids(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True)
    for prompt, new in zip(prompts, tokens):
        assert len(new) == 12
        places = [len(prompt) - 1 + i for i in range(len(new))]
        logits = plain(prompt + new, places)
        for i, token in enumerate(new):
            assert nearly_the_best(logits[i], token), (len(prompt), i)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_behind_shared_pages_at_real_sizes(folder, plain, dtype):
    """A request whose first 96 tokens are another request's: it takes over that one's pages from
    the prefix index and computes only what follows them, in one portion and then token by token.
    Its logits are the plain implementation's for its whole sequence."""
    stem = random_tokens(100, VOCAB, 21)
    first = stem + random_tokens(30, VOCAB, 22)
    second = stem + random_tokens(45, VOCAB, 23)
    model_runner = load_runner(folder, dtype=dtype, page_size=16, max_tokens=512, max_requests=4, prefix_cache=True)
    manager = model_runner.manager
    model_runner.step([StepEntry("first", first, [])])
    manager.register_prefix("first", first)
    manager.admit("second")
    held = manager.share_prefix("second", second)
    assert held == 96
    places = [96, 97, 120, 139, 140, 144]
    want = plain(second, places)
    got = {}
    logits = model_runner.step([StepEntry("second", second[held:140], [p - held for p in places if p < 140])])
    for row, p in enumerate(p for p in places if p < 140):
        got[p] = logits[row].float().cpu()
    for p in range(140, len(second)):
        logits = model_runner.step([StepEntry("second", [second[p]], [0]), StepEntry("first", [first[0]], [])])
        if p in places:
            got[p] = logits[0].float().cpu()
    manager.audit()
    for i, p in enumerate(places):
        assert off_by(got[p], want[i], dtype) <= BOUND[dtype], p
    model_runner.finish("first")
    model_runner.finish("second")
    manager.forget_prefixes()
    assert manager.num_free() == manager.num_pages()
