"""Configuration, registry, weight loading errors and the random-weights mode."""

import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY, tiny_config
from qwen3_from_scratch_amd import architectures, load_model_config
from qwen3_from_scratch_amd.config import ConfigError, EngineConfig, ModelConfig, lookup_part
from qwen3_from_scratch_amd.models import build_model, expected_tensors
from qwen3_from_scratch_amd.models.qwen3 import qwen3_spec
from qwen3_from_scratch_amd.parts import Precision
from qwen3_from_scratch_amd.weights import Checkpoint, WeightError, check_tensors


def test_config_reads_the_architectures_own_keys(model_folders):
    cfg = load_model_config(model_folders["B"])
    raw = TINY["B"]["config"]
    assert isinstance(cfg, ModelConfig) and cfg.architecture == "Qwen3ForCausalLM"
    for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                "head_dim", "intermediate_size", "rms_norm_eps", "rope_theta", "max_position_embeddings"):
        assert getattr(cfg, key) == raw[key]
    assert cfg.tie_word_embeddings is False
    assert "Qwen3ForCausalLM" in architectures()


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "hidden_act", "num_hidden_layers",
                                 "max_position_embeddings", "num_key_value_heads", "num_attention_heads",
                                 "head_dim", "intermediate_size", "rms_norm_eps", "rope_theta"])
def test_no_size_has_a_default(key):
    # the reference's reader raises KeyError for the same keys (factory/config.py:111-124)
    raw = dict(TINY["A"]["config"])
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        ModelConfig.from_dict(raw)


def test_config_refusals(tmp_path):
    raw = dict(TINY["A"]["config"])
    for change, match in [
        (dict(num_attention_heads=5), "multiple"), (dict(hidden_act="gelu"), "hidden_act"),
        (dict(head_dim=15), "even"), (dict(attention_bias=True), "attention_bias"),
        (dict(use_sliding_window=True), "sliding"), (dict(architectures=["NoSuchModel"]), "not registered"),
        (dict(vocab_size="many"), "vocab_size"),
    ]:
        bad = dict(raw, **change)
        folder = tmp_path / ("bad_%s" % list(change)[0])
        folder.mkdir()
        (folder / "config.json").write_text(json.dumps(bad))
        with pytest.raises(ConfigError, match=match):
            load_model_config(str(folder))
    # rope_theta may also sit under rope_parameters
    alt = dict(raw)
    alt["rope_parameters"] = {"rope_theta": alt.pop("rope_theta"), "rope_type": "default"}
    assert ModelConfig.from_dict(alt).rope_theta == 10000.0
    # tie_word_embeddings defaults to false
    del alt["tie_word_embeddings"]
    assert ModelConfig.from_dict(alt).tie_word_embeddings is False


def test_spec_is_data_and_sizes_come_from_the_config():
    cfg = tiny_config("B")
    spec = qwen3_spec(cfg)
    assert len(spec.layers) == cfg.num_hidden_layers and [s.layer for s in spec.order] == [0, 1, 2]
    mixer = spec.layers[1].slot("mixer").part
    assert mixer.get("num_heads") == 8 and mixer.get("num_kv_heads") == 2 and mixer.get("head_dim") == 32
    assert spec.layers[0].slot("mixer_norm").part.get("eps") == 1e-5 and spec.position.get("theta") == 1e6
    names = expected_tensors(spec)
    assert names["model.layers.2.self_attn.q_proj.weight"] == (256, 96)
    assert names["model.layers.0.self_attn.k_norm.weight"] == (32,)
    assert names["lm_head.weight"] == (384, 96)
    assert "lm_head.weight" not in expected_tensors(qwen3_spec(tiny_config("A")))
    with pytest.raises(ConfigError, match="no mixer part named"):
        lookup_part("mixer", "nonesuch")


def test_a_head_size_no_kernel_takes_is_refused_when_the_model_is_built():
    raw = dict(TINY["A"]["config"], head_dim=24)
    with pytest.raises(ValueError, match="steps of 16"):
        build_model(ModelConfig.from_dict(raw), Precision(torch.float32), "cpu")


def _rewrite(folder, out, change):
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    change(tensors)
    os.makedirs(out, exist_ok=True)
    save_file(tensors, os.path.join(out, "model.safetensors"))
    with open(os.path.join(folder, "config.json")) as fh, open(os.path.join(out, "config.json"), "w") as oh:
        oh.write(fh.read())
    return out


def test_one_error_lists_missing_unexpected_and_wrong_shapes(model_folders, tmp_path):
    def change(t):
        del t["model.layers.1.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.7.extra.weight"] = torch.zeros(3)
        t["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(33, dtype=torch.bfloat16)

    bad = _rewrite(model_folders["B"], str(tmp_path / "bad"), change)
    model = build_model(load_model_config(bad), Precision(torch.float32), "cpu")
    with pytest.raises(WeightError) as err:
        model.load(Checkpoint(bad))
    e = err.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.7.extra.weight"]
    assert e.wrong_shape == [("model.layers.0.self_attn.q_norm.weight", (32,), (33,))]
    text = str(e)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "expected [32], found [33]"):
        assert piece in text


def test_stored_dtypes_are_kept(model_folders, tmp_path):
    def change(t):
        t["model.norm.weight"] = t["model.norm.weight"].float()             # 32-bit stays 32-bit
    folder = _rewrite(model_folders["A"], str(tmp_path / "f32norm"), change)
    ck = Checkpoint(folder)
    assert ck.get("model.norm.weight", "cpu").dtype == torch.float32
    assert ck.get("model.embed_tokens.weight", "cpu").dtype == torch.bfloat16

    def change16(t):
        t["model.norm.weight"] = t["model.norm.weight"].to(torch.float16)
    folder = _rewrite(model_folders["A"], str(tmp_path / "f16norm"), change16)
    # a float16 tensor is read as float32, which holds every float16 number
    got = Checkpoint(folder).get("model.norm.weight", "cpu")
    assert got.dtype == torch.float32
    assert torch.equal(got, Checkpoint(model_folders["A"]).get("model.norm.weight", "cpu").to(torch.float16).float())
    from qwen3_from_scratch_amd.weights.checkpoint import stored_to_kept
    assert stored_to_kept(torch.arange(4, dtype=torch.int64)).dtype == torch.int32
    with pytest.raises(ValueError, match="float8"):
        stored_to_kept(torch.zeros(4).to(torch.float8_e4m3fn), "w")


def test_a_float16_checkpoint_loads_and_runs(cpu_ops, model_folders, tmp_path):
    """All tensors stored in float16 (the reference keeps any stored dtype): the engine reads them
    as float32, brings them to its compute dtype, and gives the plain implementation's logits
    for the same file."""
    import plain_qwen3
    from helpers import random_tokens
    from qwen3_from_scratch_amd.engine import StepEntry, load_runner

    def halve(t):
        for name in list(t):
            t[name] = t[name].to(torch.float16)
    folder = _rewrite(model_folders["A"], str(tmp_path / "f16"), halve)
    cfg, w = plain_qwen3.read_model_folder(folder)
    toks = random_tokens(20, cfg["vocab_size"], 4)
    want = plain_qwen3.logits_of_sequence(cfg, w, toks)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=16, max_tokens=64, max_requests=1)
    got = runner.step([StepEntry("a", toks, list(range(20)))])
    torch.testing.assert_close(got, want, rtol=2e-5, atol=2e-5)


def test_random_weights_are_seeded_by_name_not_by_order(model_folders, tmp_path):
    from qwen3_from_scratch_amd.weights import RandomWeights, write_random_model

    names = expected_tensors(qwen3_spec(tiny_config("A")))
    a = RandomWeights(names, seed=11, std=0.02, norm_jitter=0.1)
    stored = load_file(os.path.join(model_folders["A"], "model.safetensors"))
    assert set(stored) == set(names)
    for name in reversed(sorted(names)):
        assert torch.equal(a.get(name, "cpu"), stored[name])
        assert stored[name].dtype == torch.bfloat16
    norm = stored["model.layers.0.input_layernorm.weight"].float()
    assert 0.89 <= float(norm.min()) and float(norm.max()) <= 1.11 and float(norm.std()) > 0.01
    assert abs(float(stored["model.embed_tokens.weight"].float().std()) - 0.02) < 0.003
    other = write_random_model(str(tmp_path / "other"), tiny_config("A"), seed=12)
    assert not torch.equal(load_file(os.path.join(other, "model.safetensors"))["model.norm.weight"],
                           stored["model.norm.weight"])
    check_tensors(Checkpoint(other), names)


def test_tied_checkpoint_may_carry_an_unused_head(cpu_ops, model_folders, tmp_path):
    def change(t):
        t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    folder = _rewrite(model_folders["A"], str(tmp_path / "tied"), change)
    build_model(load_model_config(folder), Precision(torch.float32), "cpu").load(Checkpoint(folder))


def test_engine_config_from_the_references_yaml(model_folders, tmp_path):
    text = """
generation:
  temperature: 0.85
  top_k: 40
  max_new_tokens: 512
models:
  - name: "tiny"
    path: "%s"
    dtype: "bf16"
    components:
      self_attn: "paged_attn"
    generation:
      temperature: 0.7
scheduler:
  max_num_seqs: 8
  chunked_prefill_size: 24
  enable_prefix_cache: false
kv_cache_dtype: bfloat16
""" % model_folders["B"]
    path = tmp_path / "engine.yaml"
    path.write_text(text)
    cfg = EngineConfig.from_yaml(str(path), "tiny", device="cpu")
    assert cfg.dtype == "bfloat16" and cfg.max_num_seqs == 8 and cfg.chunked_prefill_size == 24
    assert cfg.max_num_tokens == 3000 and cfg.block_size == 16 and cfg.gpu_utilization == 0.5
    assert cfg.generation.temperature == 0.7 and cfg.generation.top_k == 40
    assert cfg.generation.max_new_tokens == 512 and cfg.max_len == 2048
    assert cfg.enable_prefix_cache is False and EngineConfig().enable_prefix_cache is True
    assert cfg.components == {"self_attn": "paged_attn"} and cfg.kv_cache_dtype == "bfloat16"
    with pytest.raises(KeyError):
        EngineConfig.from_yaml(str(path), "other")
    with pytest.raises(ConfigError):
        EngineConfig(dtype="float16")
    # what the engine cannot honour is an error, not silence
    for wrong, word in (("self_attn: \"paged_attn\"", "self_attn: \"my_op\""),
                        ("self_attn: \"paged_attn\"", "sefl_attn: \"paged_attn\""),
                        ("kv_cache_dtype: bfloat16", "kv_cache_dtype: float32")):
        path.write_text(text.replace(wrong, word))
        with pytest.raises(ConfigError) as caught:
            EngineConfig.from_yaml(str(path), "tiny", device="cpu")
        assert word.split(":")[0] in str(caught.value) or "my_op" in str(caught.value)


def test_components_name_registered_parts_or_fail(cpu_ops, model_folders):
    """`components` swaps in another registered implementation of a kind of part, under this
    package's kind names or the reference's slot names; an unknown slot or name is an error
    that lists what there is (src/qwen3_from_scratch/inference/model_loader.py:24-35)."""
    from qwen3_from_scratch_amd.config import register_part
    from qwen3_from_scratch_amd.config.registry import resolve_components
    from qwen3_from_scratch_amd.engine import SyncEngine, load_model
    from qwen3_from_scratch_amd.parts.norm import RMSNorm

    @register_part("norm", "counted_rms")
    class CountedNorm(RMSNorm):
        calls = 0

        def __init__(self, *args, bonus=0, **kw):
            super().__init__(*args, **kw)
            self.bonus = bonus

        def forward(self, *args, **kw):
            CountedNorm.calls += 1
            return super().forward(*args, **kw)

    assert resolve_components({"mlp": "base", "norm": {"name": "counted_rms", "kwargs": {"bonus": 2}}}) == {
        "feed_forward": (None, {}), "norm": ("counted_rms", {"bonus": 2})}
    model = load_model(model_folders["A"], "float32", "cpu", components={"norm": {"name": "counted_rms",
                                                                                  "kwargs": {"bonus": 2}}})
    norms = [model.final_norm] + [n for layer in model.layers for n in (layer.mixer_norm, layer.feed_forward_norm)]
    assert all(type(n) is CountedNorm and n.bonus == 2 for n in norms)
    plain = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", num_blocks=8)
    swapped = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", num_blocks=8,
                         components={"norm": "counted_rms", "decoder_layer": "base"})
    before = CountedNorm.calls
    ids = swapped.generate_ids([[5, 17, 3]], 4, temperature=0.0, ignore_eos=True)
    assert CountedNorm.calls > before
    assert ids == plain.generate_ids([[5, 17, 3]], 4, temperature=0.0, ignore_eos=True)
    for wrong, word in (({"norm": "layer_norm_of_nowhere"}, "layer_norm_of_nowhere"), ({"norms": "rms"}, "norms"),
                        ({"attn": "flash"}, "attn"), ({"mlp": {"kwargs": {}}}, "name"), ({"mlp": 3}, "mlp"),
                        ({"mlp": "swiglu", "feed_forward": "swiglu"}, "twice")):
        with pytest.raises(ConfigError) as caught:
            EngineConfig(components=wrong)
        assert word in str(caught.value)
    with pytest.raises(ConfigError):
        EngineConfig(dtype="bfloat16", kv_cache_dtype="fp32")
    assert EngineConfig(dtype="float32", kv_cache_dtype="fp32").kv_cache_dtype == "float32"
