"""Tiny configurations, model folders and trace builders shared by the tests."""

import os

import torch

from qwen3_from_scratch_amd.config import ModelConfig
from qwen3_from_scratch_amd.weights import write_random_model

# Two configurations that differ in every size and option; neither has a size
# that is a power of two throughout. A third exercises odd head counts.
TINY = {
    "A": dict(
        config=dict(architectures=["Qwen3ForCausalLM"], vocab_size=256, hidden_size=64, hidden_act="silu",
                    num_hidden_layers=2, max_position_embeddings=256, num_attention_heads=4,
                    num_key_value_heads=2, head_dim=16, intermediate_size=128, rms_norm_eps=1e-6,
                    rope_theta=10000.0, tie_word_embeddings=True),
        seed=11, std=0.02, norm_jitter=0.1, page_size=16),
    "B": dict(
        config=dict(architectures=["Qwen3ForCausalLM"], vocab_size=384, hidden_size=96, hidden_act="silu",
                    num_hidden_layers=3, max_position_embeddings=512, num_attention_heads=8,
                    num_key_value_heads=2, head_dim=32, intermediate_size=224, rms_norm_eps=1e-5,
                    rope_theta=1000000.0, tie_word_embeddings=False),
        seed=23, std=0.03, norm_jitter=0.2, page_size=8),
    "C": dict(
        config=dict(architectures=["Qwen3ForCausalLM"], vocab_size=331, hidden_size=72, hidden_act="silu",
                    num_hidden_layers=2, max_position_embeddings=640, num_attention_heads=6,
                    num_key_value_heads=3, head_dim=48, intermediate_size=200, rms_norm_eps=3e-6,
                    rope_theta=50000.0, tie_word_embeddings=False),
        seed=37, std=0.05, norm_jitter=0.3, page_size=16),
    # head sizes and page sizes that the matrix-core attention kernels take
    "D": dict(
        config=dict(architectures=["Qwen3ForCausalLM"], vocab_size=300, hidden_size=80, hidden_act="silu",
                    num_hidden_layers=2, max_position_embeddings=1024, num_attention_heads=4,
                    num_key_value_heads=2, head_dim=64, intermediate_size=144, rms_norm_eps=1e-6,
                    rope_theta=10000.0, tie_word_embeddings=True),
        seed=41, std=0.04, norm_jitter=0.2, page_size=16),
    "E": dict(
        config=dict(architectures=["Qwen3ForCausalLM"], vocab_size=270, hidden_size=96, hidden_act="silu",
                    num_hidden_layers=2, max_position_embeddings=2048, num_attention_heads=6,
                    num_key_value_heads=1, head_dim=128, intermediate_size=160, rms_norm_eps=1e-5,
                    rope_theta=500000.0, tie_word_embeddings=False),
        seed=43, std=0.04, norm_jitter=0.2, page_size=32),
    # a width and inner sizes in steps of 64, so that steps of 65 to 128 rows take the tiled
    # matrix-core product with the norms in its epilogues; weights so large that logits span tens
    "F": dict(
        config=dict(architectures=["Qwen3ForCausalLM"], vocab_size=520, hidden_size=128, hidden_act="silu",
                    num_hidden_layers=2, max_position_embeddings=1024, num_attention_heads=4,
                    num_key_value_heads=2, head_dim=64, intermediate_size=192, rms_norm_eps=1e-6,
                    rope_theta=10000.0, tie_word_embeddings=False),
        seed=53, std=0.2, norm_jitter=0.2, page_size=16),
}
# D and E with weights so large that logits span ten units or more, where a rounding of bfloat16
# is small beside a fault; and with query norms twice as large, so that every query's
# softmax stands on a few keys, most of them far back: a key or a tile left out then shows in
# the logits of the rows that stood on it
TINY["DS"] = dict(TINY["D"], seed=45, std=0.2)
TINY["ES"] = dict(TINY["E"], seed=47, std=0.2)
TINY["DP"] = dict(TINY["D"], seed=49, std=0.2, peak=2.0)
TINY["EP"] = dict(TINY["E"], seed=51, std=0.2, peak=2.0)


def tiny_config(name):
    return ModelConfig.from_dict(TINY[name]["config"])


def make_folder(folder, name):
    t = TINY[name]
    write_random_model(folder, tiny_config(name), seed=t["seed"], std=t["std"], norm_jitter=t["norm_jitter"])
    if t.get("peak"):
        from safetensors.torch import load_file, save_file

        path = os.path.join(folder, "model.safetensors")
        tensors = load_file(path)
        for key in tensors:
            if key.endswith("q_norm.weight"):
                tensors[key] = (tensors[key].float() * t["peak"]).to(tensors[key].dtype)
        save_file(tensors, path, metadata={"format": "pt"})
    return folder


def random_tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# ---- traces: lists of steps; a step is (entries, ends); an entry is (id, tokens, want) ----

def trace_whole(requests):
    """Each request alone and whole, all places wanted."""
    steps = []
    for rid, toks in requests.items():
        steps.append(([(rid, toks, list(range(len(toks))))], [rid]))
    return steps


def trace_tail_decoded(requests, tail=32):
    """Most of each request in one step, its last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(len(toks) - tail, 1)
        steps.append(([(rid, toks[:head], list(range(head)))], []))
        for i in range(head, len(toks)):
            steps.append(([(rid, [toks[i]], [0])], [rid] if i == len(toks) - 1 else []))
        if head == len(toks):
            steps[-1] = (steps[-1][0], [rid])
    return steps


def trace_portions(requests, sizes=(24, 7, 2, 16, 3, 2, 33, 5, 2, 9)):
    """Each request alone, cut into portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            last = at + n == len(toks)
            steps.append(([(rid, toks[at:at + n], list(range(n)))], [rid] if last else []))
            at += n
    return steps


def trace_mixed(requests, max_live=4, seed=0, decode_tail=12):
    """Up to `max_live` requests at a time; each goes through its prompt in
    portions of random size and through its last `decode_tail` tokens one at a
    time, so that portions of some sit beside single tokens of others; a
    request may sit a step out. New requests start as earlier ones end."""
    g = torch.Generator().manual_seed(seed)

    def rnd(n):
        return int(torch.randint(0, n, (1,), generator=g))

    waiting = list(requests.items())
    live = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, ends = [], []
        for rid in list(live):
            toks, at = live[rid]
            if len(live) > 1 and rnd(5) == 0:
                continue                                   # sits this step out
            left = len(toks) - at
            if left <= decode_tail:
                n = 1
            else:
                n = min(left - decode_tail, 2 + rnd(30))
            entries.append((rid, toks[at:at + n], list(range(n))))
            live[rid][1] = at + n
            if at + n == len(toks):
                ends.append(rid)
                del live[rid]
        if entries:
            steps.append((entries, ends))
    return steps


def run_trace(runner, steps):
    """Drive a ModelRunner through a trace; returns {(id, position): logits row}."""
    from qwen3_from_scratch_amd.engine import StepEntry

    got = {}
    for entries, ends in steps:
        where = []
        for rid, toks, want in entries:
            base = runner.length(rid)
            where += [(rid, base + w) for w in want]
        logits = runner.step([StepEntry(rid, toks, want) for rid, toks, want in entries])
        logits = logits.float().cpu()
        for key, row in zip(where, logits):
            got[key] = row
        for rid in ends:
            runner.finish(rid)
        runner.manager.audit()
    return got


def max_live_tokens(steps, page=64):
    """The most tokens live requests hold at any time, each rounded up to `page`."""
    held, worst = {}, 0
    for entries, ends in steps:
        for rid, toks, _ in entries:
            held[rid] = held.get(rid, 0) + len(toks)
        worst = max(worst, sum(-(-n // page) * page for n in held.values()))
        for rid in ends:
            held.pop(rid, None)
    return worst


def arrivals_scenario(folder, lookahead, num_blocks, name="B", device="cpu", dtype="float32", block_size=8):
    """Requests that arrive over time, end by count or by an end-of-sequence token, sample with
    seeds or greedily, and (with few pages) preempt one another. Returns what was generated
    and how many steps were put on the GPU ahead of their tokens."""
    from qwen3_from_scratch_amd.engine import SyncEngine

    vocab = TINY[name]["config"]["vocab_size"]
    engine = SyncEngine(path=folder, dtype=dtype, device=device, block_size=block_size, num_blocks=num_blocks,
                        max_num_seqs=4, chunked_prefill_size=16)
    engine.lookahead = lookahead
    engine.eos_ids = tuple(range(0, vocab, 9))            # every ninth token ends a request that honours it
    ahead = [0]
    launch_ahead = engine._launch_ahead

    def counting(current):
        got = launch_ahead(current)
        ahead[0] += got is not None
        return got

    engine._launch_ahead = counting
    arrivals = {0: [(21, dict(temperature=0.9, seed=3), 40, True), (9, dict(temperature=0.0), 25, True)],
                7: [(33, dict(temperature=0.7, top_k=5, seed=11), 30, False)],
                30: [(5, dict(temperature=0.0), 12, False)]}
    requests = []
    step = 0
    while step < 400 and (engine.scheduler.has_work() or step <= max(arrivals)):
        for n, sampling, new, ignore in arrivals.get(step, []):
            params = engine.default_params(new, ignore_eos=ignore, **sampling)
            requests.append(engine.add_request(random_tokens(n, vocab, 90 + n), params))
        plan = engine.step()
        for s in plan:
            assert s.request.status.name in ("RUNNING", "FINISHED")
        engine.runner.manager.audit()
        step += 1
    assert not engine.scheduler.has_work()
    assert engine.runner.manager.num_free() == num_blocks
    return [list(r.generated) for r in requests], [r.preemptions for r in requests], ahead[0]


# ---- how far logits may be off ----
# float32: rounding order only, 2e-4 of the row's largest magnitude (at least 1). bfloat16: a
# fiftieth of the row's spread (largest minus smallest logit): a handful of 8-bit roundings, far
# less than what a key, a tile or a page left out does to a row.
BF16_SHARE = 2e-2


def off_by(got_row, want_row, dtype):
    """The largest difference between two rows of logits, in units of what `dtype` may be off by
    (1.0 = at the bound)."""
    diff = float((got_row.float() - want_row.float()).abs().max())
    if dtype == "float32":
        return diff / (2e-4 * max(1.0, float(want_row.abs().max())))
    return diff / (BF16_SHARE * float(want_row.max() - want_row.min()))


def nearly_the_best(logits_row, token, share=BF16_SHARE):
    """Whether `token` is the row's largest logit or within `share` of the row's spread of it:
    what a greedy choice made from logits that are off by that much may be."""
    spread = float(logits_row.max() - logits_row.min())
    return float(logits_row[token]) >= float(logits_row.max()) - share * spread
