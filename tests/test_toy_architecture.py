"""An architecture defined in tests/toy_architecture.py, with config.json keys of its own, a
mixer that keeps a state per request and, in its second example, a norm and a block arrangement
of its own, goes through the framework's model folder writer, loader,
cache manager, step function, engine and replay program without a change to the framework."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
from safetensors.torch import load_file

import toy_architecture as toy
from helpers import max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions, trace_tail_decoded
from qwen3_from_scratch_amd.config import architectures, load_model_config
from qwen3_from_scratch_amd.engine import SyncEngine, load_runner
from qwen3_from_scratch_amd.weights import write_random_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


EXAMPLES = {"sequential": toy.EXAMPLE, "parallel": toy.EXAMPLE_PARALLEL}


@pytest.fixture(scope="module", params=sorted(EXAMPLES))
def folder(request, tmp_path_factory):
    config = toy.ToyHybridConfig.from_dict(EXAMPLES[request.param])
    return write_random_model(str(tmp_path_factory.mktemp("hybrid")), config, seed=9, std=0.08, norm_jitter=0.2)


def _plain(folder, requests):
    config = load_model_config(folder)
    w = {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, w, {rid: toy.plain_logits(config, w, toks) for rid, toks in requests.items()}


def _requests(folder):
    vocab = load_model_config(folder).vocab
    return {"h%d" % i: random_tokens(n, vocab, 60 + i) for i, n in enumerate([70, 9, 41, 130, 25])}


def _worst(got, want):
    return max(float((got[(rid, p)] - logits[p]).abs().max()) for rid, logits in want.items()
               for p in range(logits.shape[0]))


def test_folder_is_read_by_its_architectures_own_keys(folder):
    assert toy.NAME in architectures()
    config = load_model_config(folder)
    example = EXAMPLES[config.arrangement]
    assert isinstance(config, toy.ToyHybridConfig) and config == toy.ToyHybridConfig.from_dict(example)
    with open(os.path.join(folder, "config.json")) as fh:
        assert set(json.load(fh)) == set(example)
    names = set(load_file(os.path.join(folder, "model.safetensors")))
    mean_layer, attention_layer = config.pattern.index("s"), config.pattern.index("a")
    assert "hybrid.layers.%d.self_attn.mix.weight" % mean_layer in names
    assert "hybrid.layers.%d.self_attn.q_proj.weight" % attention_layer in names
    assert ("hybrid.norm.bias" in names) == (config.norm == "centred")
    if config.norm == "centred":
        # the parts say what their tensors are: a scale is drawn around one, a bias around zero
        tensors = load_file(os.path.join(folder, "model.safetensors"))
        assert abs(float(tensors["hybrid.norm.weight"].float().mean()) - 1.0) < 0.1
        assert abs(float(tensors["hybrid.norm.bias"].float().mean())) < 0.05
        assert float(tensors["hybrid.norm.bias"].float().abs().max()) < 0.5


def test_a_layer_with_a_position_part_of_its_own(folder):
    """Layers `b` name a rotation of their own (half of each head, another base); the model
    keeps it beside its own, once, however many layers name it."""
    from qwen3_from_scratch_amd.config import lookup_architecture

    config = load_model_config(folder)
    spec = lookup_architecture(toy.NAME)[1](config)
    own = [ls.position for ls in spec.layers if ls.position is not None]
    assert len(own) == config.pattern.count("b") >= 1 and len(set(own)) == 1
    assert own[0].get("rotary_dim") == config.head_size // 2 and own[0] != spec.position


def test_every_cutting_and_generation_on_the_host(cpu_ops, folder):
    requests = _requests(folder)
    config, w, want = _plain(folder, requests)
    for make in (trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype="float32", device="cpu", page_size=8,
                             max_tokens=max_live_tokens(steps, page=8), max_requests=4)
        assert len(runner.manager.state_groups) == 1            # the mixer's slots
        assert _worst(run_trace(runner, steps), want) <= 2e-4, make.__name__
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)
    # greedy generation through the engine, prompts in portions beside decoding requests
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=256, block_size=8, num_blocks=40,
                        max_num_seqs=3, max_num_tokens=24, chunked_prefill_size=16)
    prompts = [toks[:n] for toks, n in zip(requests.values(), (30, 9, 41))]
    got = engine.generate_ids(prompts, max_new_tokens=6, temperature=0.0, ignore_eos=True)
    for prompt, new in zip(prompts, got):
        seq = list(prompt)
        for _ in range(6):
            seq.append(int(torch.argmax(toy.plain_logits(config, w, seq)[-1])))
        assert new == seq[len(prompt):]


def test_cache_sizing_counts_the_states(cpu_ops, folder):
    """Sized from memory, the cache leaves room for every request's fixed-size states."""
    kw = dict(path=folder, dtype="float32", device="cpu", max_len=256, block_size=8, max_num_tokens=24,
              gpu_utilization=3e-4)                       # of the gigabyte a host engine pretends to have
    few, many = SyncEngine(max_num_seqs=2, **kw), SyncEngine(max_num_seqs=40, **kw)
    needs = few.model.plane_needs
    per_page = sum(2 * n.kv_heads * n.head_dim * 4 for n in needs if n is not None and n.paged) * 8
    per_request = sum(4 * int(np.prod(n.state_shape)) for n in needs if n is not None and n.has_state)
    assert per_request > 0
    budget = int((1 << 30) * 3e-4)
    whole = -(-min(256, few.model.config.max_position_embeddings) // 8)      # pages of one request of full length
    assert few.runner.manager.num_pages() == min((budget - 3 * per_request) // per_page, 2 * whole)
    assert many.runner.manager.num_pages() == (budget - 41 * per_request) // per_page < 40 * whole
    assert (budget - 41 * per_request) // per_page < (budget - 3 * per_request) // per_page


def _replay(folder, dtype, steps, out, max_tokens, plugins):
    lines = [json.dumps({"step": i, "entries": [{"id": r, "tokens": t, "want": ws} for r, t, ws in entries],
                         "end": ends}) for i, (entries, ends) in enumerate(steps)]
    env = dict(os.environ, PYTHONPATH=os.path.join(ROOT, "tests") + os.pathsep + os.environ.get("PYTHONPATH", ""))
    env.pop("QWEN3_FROM_SCRATCH_AMD_PLUGINS", None)
    if plugins:
        env["QWEN3_FROM_SCRATCH_AMD_PLUGINS"] = plugins
    return subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
         "--max-tokens", str(max_tokens), "--page-size", "16"],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600, env=env)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 5e-4), ("bfloat16", 0.25)])
def test_replay_program_takes_the_architecture_as_a_plugin(folder, tmp_path, dtype, tol):
    requests = _requests(folder)
    _, _, want = _plain(folder, requests)
    steps = trace_mixed(requests, seed=2)
    out = str(tmp_path / dtype)
    proc = _replay(folder, dtype, steps, out, max_live_tokens(steps, page=64), "toy_architecture")
    assert proc.returncode == 0, proc.stderr[-2000:]
    got, lengths = {}, {}
    for i, (entries, _) in enumerate(steps):
        wanted = [(r, lengths.get(r, 0) + p) for r, t, ws in entries for p in ws]
        for r, t, _ in entries:
            lengths[r] = lengths.get(r, 0) + len(t)
        if wanted:
            data = np.fromfile(os.path.join(out, "%d.f32" % i), dtype="<f4").reshape(len(wanted), -1)
            for key, row in zip(wanted, data):
                got[key] = torch.from_numpy(row.copy())
    assert _worst(got, want) <= tol
    # without the plugin the program says which architectures it knows
    proc = _replay(folder, dtype, steps[:1], out + "_none", 256, "")
    assert proc.returncode != 0 and "is not registered" in proc.stderr
