"""Sizes at the edges of what the configuration allows, through the replay path against the
plain implementation: one head of 16, head sizes 80, 96, 112 and 256 (the general attention
kernel), groups of 1, 2, 6 and 20 query heads per key head, widths and vocabularies that are
no multiple of 8, the full vocabulary of 151,936 on a narrow model."""

import pytest
import torch

import plain_qwen3
from helpers import max_live_tokens, off_by, random_tokens, run_trace, trace_mixed, trace_portions
from qwen3_from_scratch_amd.config import ModelConfig
from qwen3_from_scratch_amd.engine import load_runner
from qwen3_from_scratch_amd.weights import write_random_model

pytestmark = pytest.mark.gpu


def _config(V, H, L, Hq, Hkv, D, I, eps=1e-6, theta=1e6, tie=False, maxpos=1024):
    return dict(architectures=["Qwen3ForCausalLM"], vocab_size=V, hidden_size=H, hidden_act="silu",
                num_hidden_layers=L, max_position_embeddings=maxpos, num_attention_heads=Hq,
                num_key_value_heads=Hkv, head_dim=D, intermediate_size=I, rms_norm_eps=eps, rope_theta=theta,
                tie_word_embeddings=tie)


CONFIGS = {
    "one_head_of_16": _config(101, 24, 1, 1, 1, 16, 40),
    "head_80_groups_of_2": _config(1001, 200, 2, 10, 5, 80, 504, tie=True, eps=1e-5, theta=1e4),
    "head_96_groups_of_6": _config(5003, 264, 2, 12, 2, 96, 700),
    "head_112_no_groups": _config(777, 104, 2, 7, 7, 112, 300, theta=5e5),
    "head_256_groups_of_4": _config(999, 136, 2, 4, 1, 256, 384),
    "head_128_groups_of_20": _config(1500, 320, 2, 40, 2, 128, 800),
    "odd_width": _config(333, 90, 2, 3, 1, 16, 150, tie=True),
    "full_vocabulary": _config(151936, 1024, 1, 16, 8, 128, 3072, tie=True, maxpos=2048),
}


# configurations whose query norms are doubled after the weights are drawn: every query's softmax
# then stands on a few keys, most of them far back, and a key that the general attention kernel
# dropped would move the rows that stood on it by many times the bound
PEAKED = {"head_96_groups_of_6", "head_128_groups_of_20"}
CASES = sorted(CONFIGS) + sorted(name + "+peaked" for name in PEAKED)


def _double_query_norms(folder):
    import os

    from safetensors.torch import load_file, save_file

    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for key in tensors:
        if key.endswith("q_norm.weight"):
            tensors[key] = (tensors[key].float() * 2.0).to(tensors[key].dtype)
    save_file(tensors, path, metadata={"format": "pt"})


@pytest.mark.parametrize("case", CASES)
def test_edge_sizes_match_plain(case, tmp_path):
    """Weights of standard deviation 0.2, so that logits span tens of units and a rounding of
    bfloat16 is small beside a fault; a row may be off by 2e-4 of its largest magnitude in
    float32 and by a fiftieth of its own spread in bfloat16 (`helpers.off_by`)."""
    name = case.split("+")[0]
    config = CONFIGS[name]
    folder = str(tmp_path / name)
    write_random_model(folder, ModelConfig.from_dict(config), seed=5, std=0.2, norm_jitter=0.2)
    if case.endswith("+peaked"):
        _double_query_norms(folder)
    plain_config, weights = plain_qwen3.read_model_folder(folder)
    requests = {"r%d" % i: random_tokens(n, config["vocab_size"], 50 + i) for i, n in enumerate([70, 300, 9, 41])}
    want = {rid: plain_qwen3.logits_of_sequence(plain_config, weights, toks) for rid, toks in requests.items()}
    for dtype in ("float32", "bfloat16"):
        for make in (trace_portions, trace_mixed):
            steps = make(requests)
            runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=max_live_tokens(steps),
                                 max_requests=8)
            got = run_trace(runner, steps)
            for rid, logits in want.items():
                worst = max(off_by(got[(rid, p)], logits[p], dtype) for p in range(logits.shape[0]))
                assert worst <= 1.0, (dtype, make.__name__, rid, worst)
            assert runner.manager.num_free() == runner.manager.num_pages()
