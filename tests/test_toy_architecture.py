"""An architecture defined in tests/toy_architecture.py, with config.json keys of its own, a
mixer that keeps a state per request, in its second example a norm and a block arrangement
of its own, and in its third a block with four norms, a mixer that pages one tensor of a width
of its own and a layer without a feed-forward, goes through the framework's model folder writer, loader,
cache manager, step function, engine and replay program without a change to the framework."""

import dataclasses
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


EXAMPLES = {"sequential": toy.EXAMPLE, "parallel": toy.EXAMPLE_PARALLEL, "sandwich": toy.EXAMPLE_SANDWICH}


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


def test_a_block_with_four_norms_a_paged_tensor_of_its_own_and_a_layer_without_feed_forward(cpu_ops, tmp_path):
    """The third example's parts are declarations only: the layer says which parts its block
    gets, the mixer says what it pages (one float32 tensor of 24 numbers a token, the last twelve
    tokens kept), and the cache storage builds exactly that."""
    config = toy.ToyHybridConfig.from_dict(toy.EXAMPLE_SANDWICH)
    folder = write_random_model(str(tmp_path / "m"), config, seed=9, std=0.08, norm_jitter=0.2)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=256, max_requests=4)
    layers = runner.model.layers
    kinds = dict(zip(config.pattern, layers))
    assert set(kinds["p"].named) == {"mixer", "feed_forward", "mixer_norm", "mixer_out_norm", "feed_forward_norm",
                                     "feed_forward_out_norm"}
    assert set(kinds["n"].named) == {"mixer", "mixer_norm"}
    names = set(load_file(os.path.join(folder, "model.safetensors")))
    n_at = config.pattern.index("n")
    assert "hybrid.layers.%d.post_mlp_norm.weight" % config.pattern.index("p") in names
    assert not any(name.startswith("hybrid.layers.%d.mlp" % n_at) for name in names)
    groups = runner.manager.groups
    mine = [g for g in groups if [t.name for t in g.tensors] == ["memory"]]
    assert len(mine) == 1 and mine[0].window == toy.LAG + 1 and len(mine[0].planes) == 2     # layers p and n
    stored = runner.storage.paged[groups.index(mine[0])]["memory"]
    assert stored.dtype == torch.float32 and stored.shape[2:] == (8, toy.MEMORY)
    attention = [g for g in groups if [t.name for t in g.tensors] == ["keys", "values"]]
    assert sorted(g.window for g in attention) == [0, config.window]
    # pages behind the mixer's window go back while the request lives
    from qwen3_from_scratch_amd.engine import StepEntry

    tokens = random_tokens(100, config.vocab, 3)
    for at in range(0, 100, 10):
        runner.step([StepEntry("r", tokens[at:at + 10], [])])
    table = runner.manager.block_table("r", groups.index(mine[0]))
    assert table[:10] == [-1] * 10 and min(table[11:]) >= 0
    # the storage is sized by what the parts declare
    per_token = sum(n.bytes_per_token(torch.float32) for n in runner.model.plane_needs if n is not None)
    assert per_token == 2 * (4 * toy.MEMORY) + 2 * (2 * 4 * config.kv_heads * config.head_size)


def test_a_layers_own_position_table_bounds_a_request(cpu_ops, tmp_path):
    """A position beyond a rotation table would go without its rotation; the step function bounds
    a request by the shortest table among the model's and the layers' own, and the operation
    itself refuses a step that passes the table it is given."""
    from qwen3_from_scratch_amd.config import register_architecture
    from qwen3_from_scratch_amd.engine import StepEntry

    def short_table(c):
        spec = toy.toy_hybrid_spec(c)
        layers = tuple(dataclasses.replace(ls, position=ls.position.with_params(max_positions=40))
                       if ls.position is not None else ls for ls in spec.layers)
        return dataclasses.replace(spec, layers=layers)

    register_architecture("ToyShortTableForCausalLM", toy.ToyHybridConfig, short_table)
    config = toy.ToyHybridConfig.from_dict(dict(toy.EXAMPLE, architectures=["ToyShortTableForCausalLM"]))
    folder = write_random_model(str(tmp_path / "m"), config, seed=9, std=0.08, norm_jitter=0.2)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=256, max_requests=2)
    assert runner.max_positions == 40 and runner.max_request_tokens == 40
    runner.step([StepEntry("r", random_tokens(40, config.vocab, 1), [39])])
    with pytest.raises(ValueError, match="position 39"):
        runner.step([StepEntry("r", [5], [0])])
    # the operation on its own: a table of 40 positions and a step that reaches position 40
    D, table = 16, cpu_ops.rope_table(torch.ones(8), 40)
    qkv = torch.zeros(3, 3 * D)
    positions, seq = torch.tensor([38, 39, 40], dtype=torch.int32), torch.zeros(3, dtype=torch.int32)
    with pytest.raises(ValueError, match="rotation table ends at 39"):
        cpu_ops.qk_norm_rope_store(qkv, 1, 1, D, positions, seq, table=table, max_kv_len=41)


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
    per_page = sum(n.bytes_per_token(torch.float32) for n in needs if n is not None) * 8
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
