"""Greedy generation through the entry point on the GPU, and the replay program
as a user runs it."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_qwen3
from helpers import (TINY, arrivals_scenario, max_live_tokens, nearly_the_best, off_by, random_tokens, trace_mixed,
                     trace_portions)
from qwen3_from_scratch_amd.engine import SyncEngine

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _plain_greedy(folder, prompts, n):
    cfg, w = plain_qwen3.read_model_folder(folder)
    return [plain_qwen3.greedy_generate(cfg, w, p, n) for p in prompts]


def test_greedy_generation_float32_equals_plain(model_folders):
    vocab = TINY["A"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 40 + n) for n in (5, 17, 33)]
    want = _plain_greedy(model_folders["A"], prompts, 16)
    engine = SyncEngine(path=model_folders["A"], dtype="float32", block_size=16, num_blocks=12, max_num_seqs=4)
    assert engine.generate_ids(prompts, max_new_tokens=16, temperature=0.0, ignore_eos=True) == want


def test_chunked_generation_with_preemption_equals_plain(model_folders):
    vocab = TINY["B"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 60 + n) for n in (30, 28, 17)]
    want = _plain_greedy(model_folders["B"], prompts, 12)
    engine = SyncEngine(path=model_folders["B"], dtype="float32", block_size=8, num_blocks=11, max_num_seqs=3,
                        chunked_prefill_size=16)
    requests = [engine.add_request(p, engine.default_params(12, temperature=0.0, ignore_eos=True))
                for p in prompts]
    while engine.scheduler.has_work():
        engine.step()
    assert [r.generated for r in requests] == want
    assert sum(r.preemptions for r in requests) > 0


@pytest.mark.parametrize("name,block_size,num_blocks", [("B", 8, 60), ("B", 8, 14), ("D", 16, 30)])
def test_shared_prefixes_change_no_token(model_folders, name, block_size, num_blocks):
    """Requests that begin alike take over each other's cached blocks, at once, later and after
    a preemption, through prompt steps and graph replays; float32 tokens are the plain
    implementation's."""
    vocab = TINY[name]["config"]["vocab_size"]
    stem = random_tokens(50, vocab, 90)
    prompts = [stem + random_tokens(n, vocab, 91 + n) for n in (3, 11, 1)] + [stem[:33], random_tokens(20, vocab, 99)]
    want = _plain_greedy(model_folders[name], prompts, 8)
    engine = SyncEngine(path=model_folders[name], dtype="float32", block_size=block_size, num_blocks=num_blocks,
                        max_num_seqs=3, max_num_tokens=40, chunked_prefill_size=24)
    manager = engine.runner.manager
    requests = [engine.add_request(p, engine.default_params(8, temperature=0.0, ignore_eos=True)) for p in prompts]
    while engine.scheduler.has_work():
        engine.step()
        manager.audit()
    assert [r.generated for r in requests] == want
    assert manager.prefix_hits >= 48 + 32 and manager.num_free() == num_blocks      # at least two requests found the stem
    if num_blocks == 14:
        assert sum(r.preemptions for r in requests) > 0
    before = manager.prefix_hits
    assert engine.generate_ids([prompts[1]], max_new_tokens=8, temperature=0.0, ignore_eos=True) == [want[1]]
    assert manager.prefix_hits > before


def test_bfloat16_generation_and_seeded_sampling(model_folders):
    vocab = TINY["B"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 50 + n) for n in (1, 9, 64, 130)]
    kw = dict(path=model_folders["B"], dtype="bfloat16", block_size=8, num_blocks=64, max_num_tokens=30,
              chunked_prefill_size=24)
    got = SyncEngine(max_num_seqs=4, **kw).generate_ids(prompts, 6, temperature=0.0, ignore_eos=True)
    # bfloat16 may flip a near-tie: every token is the plain implementation's best or within a
    # fiftieth of the row's spread of it, given the tokens before it
    cfg, w = plain_qwen3.read_model_folder(model_folders["B"])
    for prompt, new in zip(prompts, got):
        logits = plain_qwen3.logits_of_sequence(cfg, w, prompt + new)
        for i, token in enumerate(new):
            assert nearly_the_best(logits[len(prompt) + i - 1], token), (len(prompt), i)
    a = SyncEngine(max_num_seqs=4, **kw).generate_ids(prompts, 6, temperature=0.8, top_k=20, seed=3, ignore_eos=True)
    b = SyncEngine(max_num_seqs=1, **kw).generate_ids(prompts[2:3], 6, temperature=0.8, top_k=20, seed=3,
                                                      ignore_eos=True)
    assert a[2] == b[0]                       # a request's draws do not depend on its batch


@pytest.mark.parametrize("name,dtype,block_size,num_blocks", [("E", "bfloat16", 16, 40), ("E", "bfloat16", 16, 5),
                                                              ("B", "float32", 8, 10), ("D", "bfloat16", 16, 6)])
def test_a_step_ahead_changes_no_token(model_folders, name, dtype, block_size, num_blocks):
    """Decode steps launched before the last step's tokens are on the host (graph replays fed
    from the device) give the tokens of the step-by-step engine, through arrivals, ends by
    count and by token, seeded sampling, and preemption."""
    kw = dict(name=name, device="cuda", dtype=dtype, block_size=block_size)
    plain, preempted, none_ahead = arrivals_scenario(model_folders[name], False, num_blocks, **kw)
    ahead, preempted_ahead, steps_ahead = arrivals_scenario(model_folders[name], True, num_blocks, **kw)
    assert none_ahead == 0 and steps_ahead > (10 if num_blocks >= 20 else 0)
    assert ahead == plain and preempted_ahead == preempted
    if num_blocks < 20:
        assert sum(preempted) > 0


def test_a_dropped_engine_in_a_cycle_is_freed_before_the_next_capture(model_folders):
    """An engine that is dropped while something points back at it is only found by the cyclic
    collector, which must not finalize its captured graphs while another capture is open
    (destroying a graph synchronizes the device): the capture collects what is dead first and
    keeps the collector off until it ends."""
    import gc
    import weakref

    kw = dict(path=model_folders["D"], dtype="bfloat16", block_size=16, num_blocks=12, max_num_seqs=2)

    def first():
        engine = SyncEngine(**kw)
        engine.myself = engine                       # the cycle
        tokens = engine.generate_ids([[1, 2, 3]], 6, temperature=0.0, ignore_eos=True)
        assert engine.runner._graphs
        return weakref.ref(engine.runner), tokens

    gc.collect()
    gc.disable()                                     # only the capture's own collection can find it
    try:
        gone, tokens = first()
        assert gone() is not None
        second = SyncEngine(**kw)
        assert second.generate_ids([[1, 2, 3]], 6, temperature=0.0, ignore_eos=True) == tokens
        assert gone() is None
        assert not gc.isenabled()
    finally:
        gc.enable()


def test_more_graphs_than_are_kept(model_folders):
    """With room for two graphs, batches of one to four requests and a step ahead: the graph used
    longest ago goes each time a new one comes, after the work that still reads it has ended;
    tokens are those of an engine that keeps them all."""
    vocab = TINY["D"]["config"]["vocab_size"]
    prompts = [random_tokens(n, vocab, 70 + n) for n in (5, 9, 13, 17)]
    kw = dict(path=model_folders["D"], dtype="bfloat16", block_size=16, num_blocks=40, max_num_seqs=4)

    def run(max_graphs):
        engine = SyncEngine(**kw)
        engine.runner.max_graphs = max_graphs
        out = []
        for count in (1, 2, 3, 4, 2, 1, 4, 3):
            out.append(engine.generate_ids(prompts[:count], 5, temperature=0.7, top_k=8, seed=5, ignore_eos=True))
            assert len(engine.runner._graphs) <= max_graphs
        return out

    assert run(2) == run(32)


def _replay(folder, dtype, steps, out, max_tokens):
    lines = []
    for i, (entries, ends) in enumerate(steps):
        lines.append(json.dumps({"step": i, "entries": [{"id": r, "tokens": t, "want": w} for r, t, w in entries],
                                 "end": ends}))
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", out, "--max-tokens", str(max_tokens)],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l] == ["done %d" % i for i in range(len(steps))]
    got, lengths = {}, {}
    for i, (entries, ends) in enumerate(steps):
        wanted = [(r, lengths.get(r, 0) + w) for r, t, ws in entries for w in ws]
        for r, t, _ in entries:
            lengths[r] = lengths.get(r, 0) + len(t)
        if wanted:
            data = np.fromfile(os.path.join(out, "%d.f32" % i), dtype="<f4")
            data = data.reshape(len(wanted), -1)
            for key, row in zip(wanted, data):
                got[key] = torch.from_numpy(row.copy())
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(model_folders, tmp_path, dtype):
    name = "C"
    vocab = TINY[name]["config"]["vocab_size"]
    requests = {"q%d" % i: random_tokens(n, vocab, 80 + i) for i, n in enumerate([50, 90, 7, 130, 64, 33])}
    cfg, w = plain_qwen3.read_model_folder(model_folders[name])
    want = {rid: plain_qwen3.logits_of_sequence(cfg, w, toks) for rid, toks in requests.items()}
    for label, steps in (("mixed", trace_mixed(requests, seed=4)), ("portions", trace_portions(requests))):
        got = _replay(model_folders[name], dtype, steps, str(tmp_path / (label + dtype)),
                      max_live_tokens(steps, page=64))
        for rid, logits in want.items():
            for p in range(logits.shape[0]):
                assert off_by(got[(rid, p)], logits[p], dtype) <= 1.0, (label, rid, p)


def test_trace_run_answers_step_by_step(model_folders, tmp_path):
    """The program reads a step, runs it, writes its file and prints `done <step>` before the
    next step is sent; it exits with 0 when its input ends."""
    out = str(tmp_path / "out")
    proc = subprocess.Popen(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_folders["D"], "--dtype", "bfloat16",
         "--out", out, "--max-tokens", "256"], stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for step in range(4):
            record = {"step": step, "entries": [{"id": "a", "tokens": [5, 2, 3] if step == 0 else [step], "want": [0]}],
                      "end": ["a"] if step == 3 else []}
            proc.stdin.write(json.dumps(record) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == "done %d" % step
            assert os.path.getsize(os.path.join(out, "%d.f32" % step)) == 4 * TINY["D"]["config"]["vocab_size"]
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


def _run(arguments, timeout=300):
    proc = subprocess.run([sys.executable] + arguments, capture_output=True, text=True, timeout=timeout, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return proc.stdout


def test_the_command_line_and_the_examples_as_a_user_runs_them(tmp_path):
    """`python -m qwen3_from_scratch_amd` writes a random-weights folder and generates from it,
    and the two example scripts run on that folder, each as a process of its own on the GPU;
    with float32 and temperature 0 the ids they print are the plain implementation's."""
    config = tmp_path / "config.json"
    config.write_text(json.dumps(TINY["D"]["config"]))
    folder = str(tmp_path / "model")
    module = ["-m", "qwen3_from_scratch_amd"]
    assert "wrote" in _run(module + ["--write_random", folder, "--from_config", str(config), "--seed", "3",
                                     "--std", "0.05"])
    cfg, w = plain_qwen3.read_model_folder(folder)

    def plain(prompt, n):
        return plain_qwen3.greedy_generate(cfg, w, prompt, n)

    greedy = ["--dtype", "float32", "--temperature", "0"]
    out = _run(module + ["--path", folder, "--prompt_ids", "5,17,3", "--max_new_tokens", "8", "--ignore_eos"] + greedy)
    want = plain([5, 17, 3], 8)
    assert [int(t) for t in out.split()] == want
    # a stop token on the command line: generation ends with its first occurrence
    out = _run(module + ["--path", folder, "--prompt_ids", "5,17,3", "--max_new_tokens", "8", "--eos_id", str(want[3])]
               + greedy)
    assert [int(t) for t in out.split()] == want[:want.index(want[3]) + 1]
    out = _run(module + ["--path", folder, "--prompt_ids", "5,17,3", "--prompt_ids", "9,9", "--max_new_tokens", "5",
                         "--ignore_eos"] + greedy)
    assert [[int(t) for t in line.split()] for line in out.strip().split("\n")] == [plain([5, 17, 3], 5), plain([9, 9], 5)]

    out = _run([os.path.join(ROOT, "examples", "sync_engine_example.py"), "--path", folder, "--max_new_tokens", "6"]
               + greedy)
    lines = out.split("\n")
    streamed = lines[lines.index("=== one request, streamed ===") + 1]
    assert [int(t) for t in streamed.split()] == plain([5, 17, 3, 9], 6)
    whole = lines[lines.index("=== one request, whole ===") + 1]
    assert [int(t) for t in whole.split()] == plain([2, 4, 6], 6)
    batch = [l[2:] for l in lines if l.startswith("- ")]
    assert [[int(t) for t in l.split()] for l in batch] == [plain(p, 6) for p in ([5, 17, 3], [2, 4, 6, 8], [9])]
    assert any(l.startswith("requests: 3 | tokens: 18") for l in lines)

    out = _run([os.path.join(ROOT, "examples", "llm_runner.py"), "--path", folder, "--max_new_tokens", "6"] + greedy)
    for tag, prompt in (("req0", [5, 17, 3, 9]), ("req1", [2, 4, 6])):
        ids = [int(l.split("]")[1]) for l in out.split("\n") if l.startswith("[%s]" % tag)]
        assert ids == plain(prompt, 6), tag
    # the default precision and sampling run too
    assert len(_run(module + ["--path", folder, "--prompt_ids", "5,17,3", "--max_new_tokens", "8", "--seed", "2",
                              "--ignore_eos"]).split()) == 8
