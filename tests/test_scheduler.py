"""The scheduler's decisions, on the host, with a stub in place of the model.
Vectors are those of the reference's test/inference/test_scheduler.py where the
policy is the same; where it differs on purpose the test says so."""

import random

import pytest

from qwen3_from_scratch_amd.cache import CacheManager
from qwen3_from_scratch_amd.engine import Request, RequestStatus, Scheduler
from qwen3_from_scratch_amd.parts.attention import keys_and_values
from qwen3_from_scratch_amd.sampling import SamplingParams


def make(num_pages, page=16, max_num_seqs=32, max_num_tokens=3000, chunk=512):
    m = CacheManager([keys_and_values(2, 16)], page_size=page, num_pages=num_pages, max_requests=max(max_num_seqs, 1))
    return m, Scheduler(m, max_num_seqs, max_num_tokens, chunk)


def req(rid, n, max_new=10, **kw):
    return Request(rid, list(range(n)), SamplingParams(max_new_tokens=max_new, **kw))


def run_step(m, s, token=7):
    """What the engine does around the model: take pages, commit, book-keep."""
    plan = s.schedule()
    for e in plan:
        rid = e.request.request_id
        if not m.has(rid):
            m.admit(rid)
        m.reserve(rid, e.num_tokens)
    for e in plan:
        m.commit(e.request.request_id, e.num_tokens)
    s.after_step(plan, [token for e in plan if e.samples])
    m.audit()
    return plan


def test_token_budget_cuts_prompts_into_portions():
    # test_scheduler.py:105-122: budget 5, prompts of 2 -> 2, 2, 1; budget 3, prompt 5 -> 3 then 2
    m, s = make(64, max_num_tokens=5)
    for i in range(4):
        s.add(req(i, 2))
    assert [e.num_tokens for e in s.schedule()] == [2, 2, 1]
    m, s = make(64, max_num_tokens=3)
    s.add(req("a", 5))
    plan = run_step(m, s)
    assert [(e.num_tokens, e.samples) for e in plan] == [(3, False)]
    plan = run_step(m, s)
    assert [(e.num_tokens, e.samples) for e in plan] == [(2, True)]
    assert plan[0].request.generated == [7]


def test_sequence_budget_and_decode_first():
    # :124-144 and :33-50: 100 waiting, max_num_seqs 2 -> 2 then the same 2 decoding
    m, s = make(4096, max_num_seqs=2)
    for i in range(100):
        s.add(req(i, 3))
    first = run_step(m, s)
    assert [e.request.request_id for e in first] == [0, 1]
    second = run_step(m, s)
    assert [(e.request.request_id, e.num_tokens) for e in second] == [(0, 1), (1, 1)]
    # decodes come before portions of prompts in the plan
    m, s = make(4096, max_num_seqs=3, max_num_tokens=50)
    s.add(req("old", 4))
    run_step(m, s)
    s.add(req("new", 30))
    plan = s.schedule()
    assert [(e.request.request_id, e.num_tokens) for e in plan] == [("old", 1), ("new", 30)]


def test_decode_budgets_rotate():
    # :161-187: 9 decoders, token budget 7 -> 7; sequence cap 5 -> 5; the skipped go first next time
    m, s = make(4096, max_num_seqs=9, max_num_tokens=3000)
    for i in range(9):
        s.add(req(i, 2, max_new=50))
    run_step(m, s)
    s.max_num_tokens = 7
    a = run_step(m, s)
    assert len(a) == 7 and all(e.num_tokens == 1 for e in a)
    b = run_step(m, s)
    assert [e.request.request_id for e in b][:2] == [7, 8]
    s.max_num_tokens, s.max_num_seqs = 3000, 5
    assert len(run_step(m, s)) == 5


def test_a_request_that_can_never_fit_is_refused():
    # :52-58: 100 + 61 > 10 * 16
    m, s = make(10)
    with pytest.raises(ValueError):
        s.add(req("big", 100, max_new=61))
    s.add(req("ok", 100, max_new=60))
    with pytest.raises(ValueError):
        s.add(Request("empty", []))


def test_pages_run_out_while_decoding_the_newest_is_preempted_and_keeps_its_tokens():
    # :229-280: 4 pages, two 32-token prompts. The reference drops the victim's tokens and
    # restarts it from its prompt; here it keeps them and goes through prompt + tokens again.
    m, s = make(4, max_num_seqs=4)
    s.add(req("first", 32, max_new=8))
    s.add(req("second", 32, max_new=8))
    plan = run_step(m, s, token=5)
    assert [(e.request.request_id, e.num_tokens, e.samples) for e in plan] == [("first", 32, True),
                                                                                ("second", 32, True)]
    assert m.num_free() == 0
    first, second = plan[0].request, plan[1].request
    plan = run_step(m, s, token=6)               # each decode needs a third page: none is free
    assert [e.request.request_id for e in plan] == ["first"]
    assert second.status == RequestStatus.WAITING and second.computed == 0 and second.generated == [5]
    assert second.preemptions == 1 and not m.has("second") and s.waiting[0] is second
    while first.status != RequestStatus.FINISHED:
        plan = run_step(m, s, token=6)
    assert first.generated == [5] + [6] * 7
    # the victim comes back: 33 tokens in one portion, then it decodes on
    plan = run_step(m, s, token=9)
    assert [(e.request.request_id, e.num_tokens, e.samples) for e in plan] == [("second", 33, True)]
    while second.status != RequestStatus.FINISHED:
        run_step(m, s, token=9)
    assert second.generated == [5] + [9] * 7     # no token was produced twice
    assert m.num_free() == 4 and not s.has_work()


def test_the_last_decoder_preempts_itself_and_prompts_in_progress_cannot_deadlock():
    m, s = make(3, page=4, max_num_seqs=4, chunk=4)
    s.add(req("a", 7, max_new=5))
    s.add(req("b", 7, max_new=5))
    seen = 0
    while s.has_work():
        plan = run_step(m, s)
        assert plan, "a step must always be possible"
        seen += 1
        assert seen < 100
    assert m.num_free() == 3


def test_waiting_requests_do_not_overtake():
    m, s = make(4, page=4, max_num_seqs=4)
    s.add(req("big", 12, max_new=4))
    s.add(req("small", 2, max_new=2))
    s.add(req("tiny", 1, max_new=1))
    plan = run_step(m, s)
    # big takes 3 of 4 pages; small fits the last; tiny must wait behind nobody it could pass
    assert [e.request.request_id for e in plan] == ["big", "small"]
    assert [r.request_id for r in s.waiting] == ["tiny"]


def test_abort_gives_everything_back():
    m, s = make(8, page=4)
    a, b = req("a", 9, max_new=5), req("b", 5, max_new=5)
    s.add(a)
    s.add(b)
    run_step(m, s)
    s.abort(a)
    assert a.status == RequestStatus.FINISHED and not m.has("a")
    while s.has_work():
        run_step(m, s)
    assert m.num_free() == 8 and len(b.generated) == 5


def test_eos_and_ignore_eos():
    m, s = make(64)
    a = Request("a", [1, 2], SamplingParams(max_new_tokens=5), eos_ids=(7,))
    b = Request("b", [1, 2], SamplingParams(max_new_tokens=3, ignore_eos=True), eos_ids=(7,))
    s.add(a)
    s.add(b)
    run_step(m, s, token=7)
    assert a.status == RequestStatus.FINISHED and a.generated == [7]
    assert b.status == RequestStatus.RUNNING
    run_step(m, s, token=7)
    run_step(m, s, token=7)
    assert b.status == RequestStatus.FINISHED and b.generated == [7, 7, 7]
    assert m.num_free() == 64


@pytest.mark.parametrize("seed", range(5))
def test_every_request_finishes_within_budgets_under_random_load(seed):
    rng = random.Random(seed)
    page = rng.choice([4, 8, 16])
    m, s = make(rng.randint(8, 24), page=page, max_num_seqs=rng.randint(1, 5),
                max_num_tokens=rng.randint(4, 40), chunk=rng.randint(2, 16))
    cap = m.capacity_tokens()
    todo = []
    for i in range(25):
        n = rng.randint(1, max(1, cap // 2))
        todo.append(req(i, n, max_new=rng.randint(1, max(1, min(20, cap - n)))))
    done_order, steps = [], 0
    while todo or s.has_work():
        for _ in range(rng.randint(0, 3)):
            if todo:
                s.add(todo.pop(0))
        if not s.has_work():
            continue
        plan = run_step(m, s, token=rng.randint(0, 9))
        steps += 1
        assert steps < 5000
        assert len(plan) <= s.max_num_seqs and sum(e.num_tokens for e in plan) <= s.max_num_tokens
        ids = [e.request.request_id for e in plan]
        assert len(set(ids)) == len(ids)
    assert m.num_free() == m.num_pages()


def test_a_request_starts_behind_the_blocks_the_prefix_index_holds():
    """The reference's share_prefix (scheduler.py:121-135; test_scheduler.py's prefix cases): a
    request whose first blocks are cached is scheduled from behind them; a whole hit keeps its
    last block to compute; one that cannot get its remaining pages gives back what it took over
    and waits."""
    m = CacheManager([keys_and_values(2, 16)], page_size=4, num_pages=8, max_requests=4, prefix_cache=True)
    s = Scheduler(m, 4, 100, 100)
    s.add(Request("a", list(range(10)), SamplingParams(max_new_tokens=1)))
    plan = run_step(m, s)
    assert [(e.num_tokens, e.samples) for e in plan] == [(10, True)] and not s.has_work()
    assert m.num_free() == 8 and m.groups[0].pool.num_free == 6       # two nodes keep their pages
    s.add(Request("b", list(range(8)) + [50, 51, 52], SamplingParams(max_new_tokens=2)))
    s.add(Request("c", list(range(8)), SamplingParams(max_new_tokens=2)))
    plan = s.schedule()
    assert [(e.request.request_id, e.request.computed, e.num_tokens) for e in plan] == [("b", 8, 3), ("c", 4, 4)]
    for e in plan:
        m.reserve(e.request.request_id, e.num_tokens)
        m.commit(e.request.request_id, e.num_tokens)
    s.after_step(plan, [7, 7])
    m.audit()
    assert m.prefix_hits == 12
    # five pages are in use (two nodes, b's third block, c's second, which stays its own); d's whole
    # prompt is cached, but the four more pages that its remaining tokens and d2 ask for are not there
    s.add(Request("d", list(range(8)) + [50, 51, 52] + list(range(60, 72)), SamplingParams(max_new_tokens=1)))
    before = m.prefix_hits
    plan = s.schedule()
    assert [e.request.request_id for e in plan] == ["b", "c"] and s.waiting[0].computed == 0
    assert not m.has("d") and m.prefix_hits == before
    m.audit()


def test_portions_end_at_multiples_that_a_part_asks_for():
    """A part may ask that every portion of a prompt but the last be a multiple of N tokens
    (`Part.portion_multiple`; the reference has no counterpart). Cuts are counted from the
    request's first token, so a request that was preempted is cut at the same places again, and
    whatever room decoding requests leave in the budget is rounded down, not overrun."""
    m = CacheManager([keys_and_values(2, 16)], page_size=16, num_pages=64, max_requests=8)
    s = Scheduler(m, max_num_seqs=8, max_num_tokens=100, chunked_prefill_size=50, portion_multiple=8)
    a, b = req("a", 131, max_new=3), req("b", 45, max_new=3)
    s.add(a)
    s.add(b)
    seen = {"a": [], "b": []}
    for _ in range(20):
        if not s.has_work():
            break
        for e in run_step(m, s):
            if e.num_tokens > 1 or e.request.is_prefill:
                seen[e.request.request_id].append(e.num_tokens)
    assert not s.has_work()
    # a: 48 (of 50), b: 45 whole (it fits in the 52 left); then a beside b's decoding: 48, then the last 35
    assert seen["a"] == [48, 48, 35] and seen["b"] == [45]
    for cuts in seen.values():
        at = 0
        for n in cuts[:-1]:
            at += n
            assert at % 8 == 0
    # a budget that cannot hold one multiple is refused when the scheduler is made
    with pytest.raises(ValueError):
        Scheduler(m, max_num_seqs=8, max_num_tokens=100, chunked_prefill_size=6, portion_multiple=8)
    # room smaller than a multiple beside decoding requests: the prompt waits a step, nothing is cut to less
    m2 = CacheManager([keys_and_values(2, 16)], page_size=16, num_pages=64, max_requests=8)
    s2 = Scheduler(m2, max_num_seqs=8, max_num_tokens=10, chunked_prefill_size=10, portion_multiple=8)
    for i in range(3):
        s2.add(req("d%d" % i, 2, max_new=30))
    run_step(m2, s2)
    s2.add(req("long", 30, max_new=2))
    portions = []
    for _ in range(40):
        if not s2.has_work():
            break
        portions += [e.num_tokens for e in run_step(m2, s2) if e.request.request_id == "long" and e.request.computed <= 30
                     and e.num_tokens > 1]
    assert portions and all(n % 8 == 0 for n in portions[:-1]) and sum(portions) == 30
