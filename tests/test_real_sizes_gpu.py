"""Layers of the Qwen3-8B configuration's sizes (hidden 4096, 32 query and 8 key
heads of 128, feed-forward 12288, vocabulary 151936) with random weights, two of
them instead of 36 so that the plain implementation finishes on the CPU: the
sizes at which the matrix-core kernels, the weight-streaming GEMM and the
vocabulary-wide head actually run."""

import pytest
import torch

import plain_qwen3
from helpers import (max_live_tokens, nearly_the_best, off_by, random_tokens, run_trace, trace_mixed,
                     trace_tail_decoded)
from qwen3_from_scratch_amd.config import ModelConfig
from qwen3_from_scratch_amd.engine import StepEntry, load_runner
from qwen3_from_scratch_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

CONFIG = dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096, hidden_act="silu",
              num_hidden_layers=2, max_position_embeddings=40960, num_attention_heads=32,
              num_key_value_heads=8, head_dim=128, intermediate_size=12288, rms_norm_eps=1e-6,
              rope_theta=1000000.0, tie_word_embeddings=False)


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("real") / "two_layers")
    write_random_model(path, ModelConfig.from_dict(CONFIG), seed=5, std=0.02, norm_jitter=0.1)
    return path


@pytest.fixture(scope="module")
def truth(folder):
    cfg, w = plain_qwen3.read_model_folder(folder)
    requests = {"a": random_tokens(150, 151936, 1), "b": random_tokens(70, 151936, 2),
                "c": random_tokens(33, 151936, 3)}
    rows = {rid: sorted({0, 1, len(t) // 2, len(t) - 2, len(t) - 1}) for rid, t in requests.items()}
    want = {rid: plain_qwen3.logits_of_sequence(cfg, w, toks, rows=rows[rid]) for rid, toks in requests.items()}
    return requests, rows, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("family", ["tail", "mixed"])
def test_real_layer_sizes_match_plain(folder, truth, dtype, family):
    requests, rows, want = truth
    steps = (trace_tail_decoded(requests, tail=32) if family == "tail" else trace_mixed(requests, seed=2))
    runner = load_runner(folder, dtype=dtype, page_size=16, max_tokens=max_live_tokens(steps, page=16),
                         max_requests=4)
    got = run_trace(runner, steps)
    for rid, logits in want.items():
        for i, p in enumerate(rows[rid]):
            assert off_by(got[(rid, p)], logits[i], dtype) <= (1.5 if dtype == "float32" else 1.0), (rid, p)


def test_schedules_agree_at_real_sizes(folder):
    """Sixteen requests through the engine twice, once with room for everything and once with
    small portions, few sequences per step and so few pages that requests are preempted. In
    float32 every kernel sums a row's numbers in an order that does not depend on the batch, so
    the greedy tokens must be the same to the last one."""
    from qwen3_from_scratch_amd.engine import SyncEngine

    g = torch.Generator().manual_seed(9)
    lengths = torch.randint(64, 600, (16,), generator=g).tolist()
    news = torch.randint(8, 40, (16,), generator=g).tolist()
    prompts = [random_tokens(n, 151936, 100 + i) for i, n in enumerate(lengths)]

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


def test_long_prompt_in_portions_at_real_sizes(folder):
    """A prompt of 3,000 tokens whole, in portions of 512 and in portions of 300: the later
    portions run over thousands of cached keys, where the prompt kernel shares a row tile's keys
    out over several blocks. bfloat16 against the float32 engine at a few places."""
    tokens = random_tokens(3000, 151936, 7)
    places = [0, 1499, 2559, 2998, 2999]

    def run(dtype, portion):
        runner = load_runner(folder, dtype=dtype, page_size=16, max_tokens=3008, max_requests=2)
        got, at = {}, 0
        while at < len(tokens):
            part = tokens[at:at + portion]
            want = [p - at for p in places if at <= p < at + len(part)]
            logits = runner.step([StepEntry("long", part, want)])
            for row, p in enumerate(p for p in places if at <= p < at + len(part)):
                got[p] = logits[row].float().cpu()
            at += len(part)
        runner.finish("long")
        assert runner.manager.num_free() == runner.manager.num_pages()
        return got

    truth = run("float32", 3000)
    for portion in (3000, 512, 300):
        got = run("bfloat16", portion)
        for p in places:
            assert off_by(got[p], truth[p], "bfloat16") <= 1.0, (portion, p)
    again = run("float32", 700)
    for p in places:
        assert off_by(again[p], truth[p], "float32") <= 1.5, p


def test_some_tens_of_rows_at_real_sizes(folder):
    """Steps of 17 to 128 rows, where the tiled matrix-core kernel carries the residual addition
    and the norms: prompts of 20 to 60 tokens one at a time, then 40 requests that decode
    together (as eager steps and, in the engine's graphs, the same), against the float32 engine
    on the same steps; and the tokens of greedy generation at that batch size against the same
    requests served four at a time, where the few-row kernels carry the same fusions."""
    from qwen3_from_scratch_amd.engine import SyncEngine

    count = 40
    prompts = [random_tokens(20 + i, 151936, 300 + i) for i in range(count)]
    tails = [random_tokens(6, 151936, 400 + i) for i in range(count)]
    steps = [([("r%d" % i, p, [len(p) - 1])], []) for i, p in enumerate(prompts)]
    for t in range(6):
        steps.append(([("r%d" % i, [tails[i][t]], [0]) for i in range(count)], []))
    steps[-1] = (steps[-1][0], ["r%d" % i for i in range(count)])

    def run(dtype):
        runner = load_runner(folder, dtype=dtype, page_size=16, max_tokens=max_live_tokens(steps, page=16),
                             max_requests=count)
        return run_trace(runner, steps)

    from qwen3_from_scratch_amd import ops

    want = run("float32")
    # "library": every such product goes the other way, the contest's product with the division behind it,
    # and every writer leaves its size to the plain product and the norm's own kernel
    for which in ("both", "library"):
        ops.matmul_kernels(which)
        try:
            got = run("bfloat16")
        finally:
            ops.matmul_kernels("both")
        assert set(want) == set(got) and len(got) == count * 7
        for key, logits in want.items():
            assert off_by(got[key], logits, "bfloat16") <= 1.0, (which, key)

    def generate(max_num_seqs):
        engine = SyncEngine(path=folder, dtype="bfloat16", block_size=16, num_blocks=count * 8,
                            max_num_seqs=max_num_seqs, max_num_tokens=4096, chunked_prefill_size=512,
                            enable_prefix_cache=False)
        return engine.generate_ids(prompts, max_new_tokens=12, temperature=0.0, ignore_eos=True)

    together, few = generate(count), generate(4)
    # bfloat16 rounds differently along the two paths and a near tie between two tokens may fall
    # either way: every token of either run is the float32 engine's best, or within a fiftieth of
    # the row's spread of it, given the tokens before it
    judge = load_runner(folder, dtype="float32", page_size=16, max_tokens=128, max_requests=1)
    for run_tokens in (together, few):
        for prompt, new in zip(prompts, run_tokens):
            places = [len(prompt) - 1 + i for i in range(len(new))]
            logits = judge.step([StepEntry("judge", prompt + new, places)]).float().cpu()
            judge.finish("judge")
            for i, token in enumerate(new):
                assert nearly_the_best(logits[i], token), (len(prompt), i)
