"""Generation through the entry point on the CPU (plain twins in place of the
kernels): greedy tokens equal the plain implementation's, whatever the batching,
the portions, and the preemptions."""

import pytest
import torch

import plain_qwen3
from helpers import TINY, arrivals_scenario, random_tokens
from qwen3_from_scratch_amd.engine import SyncEngine


def _plain_greedy(folder, prompts, n):
    cfg, w = plain_qwen3.read_model_folder(folder)
    return [plain_qwen3.greedy_generate(cfg, w, p, n) for p in prompts]


def test_greedy_generation_matches_plain_a(cpu_ops, model_folders):
    # the workload of the first tiny configuration: prompts of 5, 17 and 33 tokens, 16 greedy tokens each
    vocab = TINY["A"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 40 + n) for n in (5, 17, 33)]
    want = _plain_greedy(model_folders["A"], prompts, 16)
    engine = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", block_size=16, num_blocks=12,
                        max_num_seqs=4)
    got = engine.generate_ids(prompts, max_new_tokens=16, temperature=0.0, ignore_eos=True)
    assert got == want
    assert engine.runner.manager.num_free() == 12


def test_chunked_mixed_generation_matches_plain_b(cpu_ops, model_folders):
    # the second: prompts of 1, 9, 64 and 130 tokens in portions of 24 beside decoding requests
    vocab = TINY["B"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 50 + n) for n in (1, 9, 64, 130)]
    want = _plain_greedy(model_folders["B"], prompts, 6)
    engine = SyncEngine(path=model_folders["B"], dtype="float32", device="cpu", block_size=8, num_blocks=40,
                        max_num_seqs=4, max_num_tokens=30, chunked_prefill_size=24)
    got = engine.generate_ids(prompts, max_new_tokens=6, temperature=0.0, ignore_eos=True)
    assert got == want


def test_preemption_changes_no_token(cpu_ops, model_folders):
    vocab = TINY["B"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 60 + n) for n in (30, 28, 17)]
    want = _plain_greedy(model_folders["B"], prompts, 12)
    # 11 pages of 8: the three requests need 6 + 5 + 4 pages at their ends
    engine = SyncEngine(path=model_folders["B"], dtype="float32", device="cpu", block_size=8, num_blocks=11,
                        max_num_seqs=3, chunked_prefill_size=16)
    requests = [engine.add_request(p, engine.default_params(12, temperature=0.0, ignore_eos=True))
                for p in prompts]
    while engine.scheduler.has_work():
        engine.step()
        engine.runner.manager.audit()
    assert [r.generated for r in requests] == want
    assert sum(r.preemptions for r in requests) > 0
    assert engine.runner.manager.num_free() == 11


def test_stream_and_metrics(cpu_ops, model_folders):
    engine = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", num_blocks=8, max_num_seqs=2)
    engine.warmup()
    chunks = list(engine.generate_stream([3, 1, 4, 1, 5], max_new_tokens=4, temperature=0.0, ignore_eos=True))
    assert len(chunks) == 4 and chunks[-1].metrics.token_count == 4
    assert chunks[0].metrics.tps == 0.0 and chunks[-1].metrics.total_elapsed >= chunks[0].metrics.ttft
    assert chunks[0].prompt_tokens == 5
    texts, batch = engine.batch_generate([[1, 2, 3], [4, 5]], max_new_tokens=3, ignore_eos=True, temperature=0.0)
    assert batch.num_requests == 2 and batch.total_tokens == 6 and len(batch.per_request) == 2
    assert len(texts[0].split()) == 3
    with pytest.raises(ValueError):
        engine.generate("text needs a tokenizer", 2)


def test_sampling_is_reproducible_per_request(cpu_ops, model_folders):
    vocab = TINY["B"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 70 + n) for n in (9, 20)]
    kw = dict(path=model_folders["B"], dtype="float32", device="cpu", block_size=8, num_blocks=40)
    alone = SyncEngine(max_num_seqs=1, **kw).generate_ids([prompts[0]], 8, temperature=0.8, seed=5,
                                                          ignore_eos=True)[0]
    both = SyncEngine(max_num_seqs=2, **kw).generate_ids(prompts, 8, temperature=0.8, seed=5, ignore_eos=True)
    assert both[0] == alone
    other = SyncEngine(max_num_seqs=1, **kw).generate_ids([prompts[0]], 8, temperature=0.8, seed=6,
                                                          ignore_eos=True)[0]
    assert other != alone


@pytest.mark.parametrize("num_blocks", [40, 10])
def test_a_step_ahead_changes_no_token(cpu_ops, model_folders, num_blocks):
    plain, preempted, none_ahead = arrivals_scenario(model_folders["B"], False, num_blocks)
    ahead, preempted_ahead, steps_ahead = arrivals_scenario(model_folders["B"], True, num_blocks)
    assert none_ahead == 0 and steps_ahead > 10
    assert ahead == plain
    assert [len(g) for g in plain][:2] == [40, 25] and len(plain[2]) < 30         # the third ends early, by a token
    if num_blocks == 10:
        assert sum(preempted) > 0 and sum(preempted_ahead) > 0


def test_abort_while_a_step_is_ahead(cpu_ops, model_folders):
    vocab = TINY["A"]["config"]["vocab_size"]
    engine = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", num_blocks=16, max_num_seqs=2)
    engine.lookahead = True
    a = engine.add_request(random_tokens(6, vocab, 1), engine.default_params(30, temperature=0.0, ignore_eos=True))
    b = engine.add_request(random_tokens(9, vocab, 2), engine.default_params(30, temperature=0.0, ignore_eos=True))
    for _ in range(5):
        engine.step()
    assert engine._ahead is not None
    engine.abort(a)                                   # its row of the step ahead is dropped
    before = len(b.generated)
    plan = engine.step()
    assert [s.request for s in plan] == [b] and len(b.generated) == before + 1 and len(a.generated) < 30
    while engine.scheduler.has_work():
        engine.step()
    assert len(b.generated) == 30 and engine.runner.manager.num_free() == 16
    solo = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", num_blocks=16, max_num_seqs=2)
    assert solo.generate_ids([b.prompt], 30, temperature=0.0, ignore_eos=True)[0] == b.generated


@pytest.mark.parametrize("seed", range(6))
def test_a_step_ahead_under_random_arrivals(cpu_ops, model_folders, seed):
    """Random prompts, counts, sampling options, arrival steps, end-of-sequence sets, page
    budgets and aborts: the engine that looks a step ahead produces what the one that does not
    produces, request by request, and gives every page back."""
    import random

    rng = random.Random(seed)
    vocab = TINY["A"]["config"]["vocab_size"]
    num_blocks = rng.choice([8, 12, 30])
    eos = tuple(rng.sample(range(vocab), rng.choice([0, 8, 40])))
    plan = []
    for i in range(rng.randint(3, 7)):
        n, new = rng.randint(1, 40), rng.randint(1, 30)
        if n + new > 16 * num_blocks:
            continue
        sampling = rng.choice([dict(temperature=0.0), dict(temperature=0.8, seed=rng.randint(0, 99)),
                               dict(temperature=1.1, top_k=rng.randint(1, 9), seed=rng.randint(0, 99))])
        plan.append(dict(at=rng.randint(0, 25), prompt=random_tokens(n, vocab, 1000 * seed + i), new=new,
                         ignore=rng.random() < 0.5, sampling=sampling,
                         abort_after=rng.choice([None, None, None, rng.randint(1, 10)])))

    def run(lookahead):
        engine = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", block_size=16,
                            num_blocks=num_blocks, max_num_seqs=3, chunked_prefill_size=rng.choice([8, 64]))
        engine.lookahead = lookahead
        engine.eos_ids = eos
        live, out = {}, {}
        step = 0
        while step < 600 and (engine.scheduler.has_work() or step <= 25):
            for i, item in enumerate(plan):
                if item["at"] == step:
                    params = engine.default_params(item["new"], ignore_eos=item["ignore"], **item["sampling"])
                    live[i] = engine.add_request(item["prompt"], params)
            for i, request in list(live.items()):
                limit = plan[i]["abort_after"]
                if limit is not None and len(request.generated) >= limit and request.status.name != "FINISHED":
                    engine.abort(request)
            engine.step()
            engine.runner.manager.audit()
            step += 1
        assert not engine.scheduler.has_work()
        assert engine.runner.manager.num_free() == num_blocks
        for i, request in live.items():
            limit = plan[i]["abort_after"]
            out[i] = request.generated if limit is None else request.generated[:limit]   # an abort lands a step later when ahead
        return out

    state = rng.getstate()
    plain = run(False)
    rng.setstate(state)
    assert run(True) == plain


def test_shared_prefixes_change_no_token(cpu_ops, model_folders):
    """Requests that begin alike take over each other's cached blocks (at once, later, and after
    a preemption) and generate what the plain implementation generates; the index saves prompt
    tokens and loses no page."""
    vocab = TINY["B"]["config"]["vocab_size"]
    stem = random_tokens(50, vocab, 90)
    prompts = [stem + random_tokens(n, vocab, 91 + n) for n in (3, 11, 1)] + [stem[:33], random_tokens(20, vocab, 99)]
    want = _plain_greedy(model_folders["B"], prompts, 8)
    kw = dict(path=model_folders["B"], dtype="float32", device="cpu", block_size=8, max_num_seqs=3,
              max_num_tokens=40, chunked_prefill_size=24)
    for num_blocks in (60, 14):                  # room for all; so little that requests are preempted
        engine = SyncEngine(num_blocks=num_blocks, **kw)
        manager = engine.runner.manager
        assert manager.prefix_cache
        requests = [engine.add_request(p, engine.default_params(8, temperature=0.0, ignore_eos=True)) for p in prompts]
        steps = 0
        while engine.scheduler.has_work():
            engine.step()
            manager.audit()
            steps += 1
        assert [r.generated for r in requests] == want, num_blocks
        assert manager.prefix_hits >= 48 + 32                      # at least two requests found the stem
        assert manager.num_free() == num_blocks
        if num_blocks == 14:
            assert sum(r.preemptions for r in requests) > 0
        # a later request finds what the ended ones left
        before = manager.prefix_hits
        again = engine.generate_ids([prompts[1]], max_new_tokens=8, temperature=0.0, ignore_eos=True)
        assert again == [want[1]]
        if num_blocks == 60:
            assert manager.prefix_hits - before == 56              # 61 tokens: seven full blocks of eight
    # with the index off the same tokens, and nothing is taken over
    engine = SyncEngine(num_blocks=60, enable_prefix_cache=False, **kw)
    assert engine.generate_ids(prompts, max_new_tokens=8, temperature=0.0, ignore_eos=True) == want
    assert engine.runner.manager.prefix_hits == 0 and not engine.runner.manager.prefix_cache
