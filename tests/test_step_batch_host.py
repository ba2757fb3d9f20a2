"""The packed description of a step: the reference's own vectors, the description that a graph
keeps between replays against a fresh packing, and the collector's pause around a capture."""

import gc
import random

import numpy as np
import pytest
import torch

from qwen3_from_scratch_amd.cache import CacheManager
from qwen3_from_scratch_amd.engine import StepEntry, pack_step
from qwen3_from_scratch_amd.engine.batch import packed_layout
from qwen3_from_scratch_amd.engine.runner import DecodeDescription, collector_paused, padded_batch
from qwen3_from_scratch_amd.parts import CacheNeed
from qwen3_from_scratch_amd.parts.attention import keys_and_values


def _pack(entries, lengths, tables=None):
    tables = tables or [[[i] for i in range(len(entries))]]
    batch, _ = pack_step(entries, lengths, list(range(len(entries))), tables, "cpu")
    return batch


def test_decoded_tokens_sit_at_the_last_index():
    # test/inference/test_model_worker.py:15-33: two requests of 5 and 3 cached tokens decode one each
    batch = _pack([StepEntry("a", [100], [0]), StepEntry("b", [100], [0])], [5, 3])
    assert batch.positions.tolist() == [5, 3]
    assert batch.kv_lens.tolist() == [6, 4]


def test_a_portion_starts_where_the_cache_ends():
    # test/inference/test_model_worker.py:36-47: 2 tokens cached, tokens 2 and 3 come now
    batch = _pack([StepEntry("a", [2, 3], [1])], [2])
    assert batch.positions.tolist() == [2, 3]
    assert batch.cu_seqlens_q.tolist() == [0, 2]
    assert batch.kv_lens.tolist() == [4]
    assert batch.logits_rows.tolist() == [1]


def test_a_decoded_token_beside_a_portion():
    # test/inference/test_model_worker.py:50-69
    batch = _pack([StepEntry("d", [100], [0]), StepEntry("p", [3, 4, 5], [2])], [5, 3])
    assert batch.positions.tolist() == [5, 3, 4, 5]
    assert batch.cu_seqlens_q.tolist() == [0, 1, 4]
    assert batch.kv_lens.tolist() == [6, 6]            # the reference's cumulative [0, 6, 12]
    assert batch.seq_index.tolist() == [0, 1, 1, 1]
    assert batch.logits_rows.tolist() == [0, 3]
    assert (batch.max_q_len, batch.min_q_len, batch.max_kv_len, batch.max_kv_len_portions) == (3, 1, 6, 6)


def test_the_last_prompt_token_alone():
    # test/inference/test_model_worker.py:72-88: everything but the last prompt token is cached
    batch = _pack([StepEntry("a", [4], [0])], [4])
    assert batch.positions.tolist() == [4]
    assert batch.cu_seqlens_q.tolist() == [0, 1]
    assert batch.kv_lens.tolist() == [5]


def test_tables_are_padded_and_wanted_places_checked():
    batch, tables = pack_step([StepEntry("a", [1, 2], [0, 1]), StepEntry("b", [3], [])], [30, 0], [4, 1],
                              [[[7, 8, 9], [2]], [[-1, -1, 5], [0]]], "cpu", fixed_widths=[4, 3])
    assert tables[0].tolist() == [[7, 8, 9, -1], [2, -1, -1, -1]]
    assert tables[1].tolist() == [[-1, -1, 5], [0, -1, -1]]
    assert batch.state_slots.tolist() == [4, 1]
    with pytest.raises(ValueError):
        pack_step([StepEntry("a", [1, 2], [2])], [0], [0], [[[0]]], "cpu")
    with pytest.raises(ValueError):
        pack_step([StepEntry("a", [1], [0])], [40], [0], [[[0, 1, 2]]], "cpu", fixed_widths=[2])


def test_the_layout_has_no_gap_and_no_overlap():
    lay = packed_layout(3, 7, 2, [4, 5])
    parts = [lay.tokens, lay.positions, lay.seq_index, lay.cu_seqlens_q, lay.kv_lens, lay.state_slots,
             lay.logits_rows] + [sl for sl, _ in lay.tables]
    assert parts[0].start == 0 and parts[-1].stop == lay.total
    assert all(a.stop == b.start for a, b in zip(parts, parts[1:]))
    assert [p.stop - p.start for p in parts] == [7, 7, 7, 4, 3, 3, 2, 12, 15]


class _Decoding:
    """A cache manager and a set of requests that decode through `DecodeDescription`s, one per
    padded batch size as the runner keeps them, each step compared with a fresh packing."""

    def __init__(self, needs, page_size, num_pages, max_requests, max_tokens):
        self.m = CacheManager(needs, page_size, num_pages, max_requests)
        self.widths = [-(-max_tokens // page_size)] * len(self.m.groups)
        self.spare_pages = [g.pool.num_pages for g in self.m.groups]
        self.descriptions = {}
        self.patched = self.packed = 0

    def prompt(self, rid, n):
        self.m.admit(rid)
        self.m.reserve(rid, n)
        self.m.commit(rid, n)

    def step(self, rids, rng):
        m = self.m
        entries = [StepEntry(r, [rng.randrange(1000)], [0]) for r in rids]
        for r in rids:
            m.reserve(r, 1)
        lengths = [m.length(r) for r in rids]
        slots = [m.slot(r) for r in rids]
        tables = [[m.block_table(r, g) for r in rids] for g in range(len(m.groups))]
        ids = [(r, m.admission(r)) for r in rids]
        B = padded_batch(len(rids))
        d = self.descriptions.get(B)
        if d is None:
            lay = packed_layout(B, B, B, self.widths)
            d = self.descriptions[B] = DecodeDescription(
                B, self.widths, torch.zeros(lay.total, dtype=torch.int32), self.spare_pages, m.max_requests,
                [g.window > 0 for g in m.groups])
        fresh = d.fill(entries, ids, lengths, slots, tables, "cpu", None)
        self.patched += fresh is None
        self.packed += fresh is not None
        fill = B - len(rids)
        want = np.zeros(d.layout.total, dtype=np.int32)
        pack_step(entries + [StepEntry(None, [0])] * fill, lengths + [0] * fill, slots + [m.max_requests] * fill,
                  [group + [[self.spare_pages[g]]] * fill for g, group in enumerate(tables)], "cpu",
                  fixed_widths=self.widths, buffers=(torch.from_numpy(want), None), all_rows=True)
        got = d.host.numpy()[:d.layout.total]
        assert np.array_equal(got, want), (rids, np.nonzero(got != want)[0].tolist())
        # what the kernels index with: pages inside the pool (or the spare one), slots inside theirs,
        # a table entry for every key that is visible, positions below the lengths
        lay = d.layout
        kv = got[lay.kv_lens]
        assert np.array_equal(got[lay.positions], np.maximum(kv - 1, 0)) and (kv >= 1).all()
        assert (got[lay.state_slots] >= 0).all() and (got[lay.state_slots] <= m.max_requests).all()
        for g, (sl, w) in enumerate(lay.tables):
            table = got[sl].reshape(B, w)
            assert (table >= -1).all() and (table <= self.spare_pages[g]).all()
            for i in range(B):
                assert kv[i] <= w * m.page_size
                assert table[i, (kv[i] - 1) // m.page_size] >= 0          # the page the new key is written to
        for r in rids:
            m.commit(r, 1)
        m.audit()


def test_a_patched_description_equals_a_fresh_one():
    """Growth across page ends, a windowed group whose entries turn -1, requests that leave a
    step out or end and come back under the same name, and batch sizes that share a row count."""
    rng = random.Random(3)
    needs = [keys_and_values(2, 8), keys_and_values(2, 8, window=12), keys_and_values(2, 8)]
    d = _Decoding(needs, page_size=4, num_pages=200, max_requests=8, max_tokens=160)
    for i, n in enumerate([3, 9, 16, 1, 30, 7]):
        d.prompt("r%d" % i, n)
    live = ["r%d" % i for i in range(6)]
    for step in range(120):
        if step % 17 == 5:                             # one leaves for a step: 5 rows, padded to 6 as well
            rids = live[:2] + live[3:]
        elif step % 29 == 11:                          # one ends and comes back under its old name
            d.m.release(live[1])
            d.prompt(live[1], 1 + step % 5)
            rids = list(live)
        elif step == 60:
            live = live[:4]
            rids = list(live)
        else:
            rids = list(live)
        d.step(rids, rng)
    assert d.patched > 80 and d.packed >= 8


def test_the_scenario_of_arrivals_keeps_its_descriptions_right(cpu_ops, model_folders, monkeypatch):
    """Every single-token step of the arrivals scenario (requests that come, end by count or
    token, and preempt one another), run through the descriptions a graph would keep."""
    from helpers import TINY, arrivals_scenario
    from qwen3_from_scratch_amd.engine import runner as runner_module

    checked = [0]
    real_step = runner_module.ModelRunner.step
    trackers = {}

    def step(self, entries, device_tokens=None):
        single = entries and all(len(e.tokens) == 1 for e in entries)
        if single:
            m = self.manager
            t = trackers.setdefault(id(self), {})
            B = padded_batch(len(entries))
            widths = [-(-self.max_request_tokens // m.page_size)] * len(m.groups)
            if B not in t:
                lay = packed_layout(B, B, B, widths)
                t[B] = DecodeDescription(B, widths, torch.zeros(lay.total, dtype=torch.int32),
                                         [g.pool.num_pages for g in m.groups], m.max_requests,
                                         [g.window > 0 for g in m.groups])
            # as ModelRunner.step does before it packs
            admitted = [e.request_id for e in entries if not m.has(e.request_id)]
            assert not admitted
            held = {e.request_id: m.length(e.request_id) for e in entries}
            lengths = [held[e.request_id] for e in entries]
            slots = [m.slot(e.request_id) for e in entries]
            ids = [(e.request_id, m.admission(e.request_id)) for e in entries]
        logits = real_step(self, entries, device_tokens)
        if single:
            tables = [[m.block_table(e.request_id, g) for e in entries] for g in range(len(m.groups))]
            d = t[B]
            d.fill(entries, ids, lengths, slots, tables, "cpu", None)
            fill = B - len(entries)
            want = np.zeros(d.layout.total, dtype=np.int32)
            pack_step(list(entries) + [StepEntry(None, [0])] * fill, lengths + [0] * fill,
                      slots + [m.max_requests] * fill,
                      [group + [[m.groups[g].pool.num_pages]] * fill for g, group in enumerate(tables)], "cpu",
                      fixed_widths=widths, buffers=(torch.from_numpy(want), None), all_rows=True)
            assert np.array_equal(d.host.numpy()[:d.layout.total], want)
            checked[0] += 1
        return logits

    monkeypatch.setattr(runner_module.ModelRunner, "step", step)
    for name, block_size, num_blocks in (("E", 16, 40), ("E", 16, 5), ("B", 8, 10), ("D", 16, 6)):
        arrivals_scenario(model_folders[name], False, num_blocks, name=name, block_size=block_size)
    assert checked[0] > 100


class _Owner:
    """Stands for an engine that owns captured graphs: its finalizer must not run inside a capture."""

    def __init__(self, log):
        self.log = log
        self.me = self                     # a cycle: only the collector finds it once it is dropped

    def __del__(self):
        self.log.append("finalized")


def _churn():
    return [[i] for i in range(200000)]     # container allocations enough for several automatic collections


def test_the_collector_finds_a_dead_owner_in_the_middle_of_any_code():
    """What went wrong without the pause: a dead cycle is finalized wherever the collector happens to run."""
    gc.collect()
    log = []
    _Owner(log)
    log.append("capture begins")
    keep = _churn()
    log.append("capture ends")
    assert log == ["capture begins", "finalized", "capture ends"] and keep


def test_nothing_is_finalized_inside_a_paused_block():
    gc.collect()
    log = []
    _Owner(log)
    with collector_paused():
        log.append("capture begins")
        keep = _churn()
        _Owner(log)                        # dies inside the block: waits for its end
        more = _churn()
        log.append("capture ends")
    assert log[:3] == ["finalized", "capture begins", "capture ends"] and keep and more
    assert gc.isenabled()
    gc.collect()
    assert log == ["finalized", "capture begins", "capture ends", "finalized"]


def test_the_pause_leaves_a_disabled_collector_disabled():
    gc.disable()
    try:
        with collector_paused():
            assert not gc.isenabled()
        assert not gc.isenabled()
    finally:
        gc.enable()
