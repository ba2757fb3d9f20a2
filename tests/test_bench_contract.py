"""What bench.py promises without a GPU: more than one GPU is refused in one line with exit
code 2, and the pieces of its record that are arithmetic (bytes of a decode step, flops of a
prompt) agree with sums written out by hand."""

import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_in_one_line():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                          text=True, timeout=300)
    assert proc.returncode == 2
    lines = [ln for ln in (proc.stdout + proc.stderr).splitlines() if ln.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_bytes_and_flops_by_hand():
    sys.path.insert(0, ROOT)
    try:
        import bench
    finally:
        sys.path.remove(ROOT)
    from qwen3_from_scratch_amd.config import ModelConfig

    c = ModelConfig.from_dict(dict(
        architectures=["Qwen3ForCausalLM"], vocab_size=1000, hidden_size=64, hidden_act="silu", num_hidden_layers=3,
        max_position_embeddings=512, num_attention_heads=4, num_key_value_heads=2, head_dim=32, intermediate_size=96,
        rms_norm_eps=1e-6, rope_theta=1e4, tie_word_embeddings=False))
    per_layer = (4 + 2 * 2) * 32 * 64 + 64 * 4 * 32 + 3 * 64 * 96          # q/k/v, output, gate/up/down
    weights = 3 * per_layer + 1000 * 64                                       # and the vocabulary projection
    kv_per_token = 3 * 2 * 2 * 32                                             # layers x (k, v) x heads x head size
    need = bench.decode_bytes(c, [10, 30], 2)
    assert abs(need - 2 * (weights + 40 * kv_per_token)) <= 0.01 * need       # norms' weights and the like aside
    T = 128
    flops = bench.prefill_flops(c, T)
    # products of every token; the vocabulary's for the one row whose logits the step returns; scores and
    # values under the causal mask
    by_hand = 2 * T * 3 * per_layer + 2 * 1000 * 64 + 3 * (2 * 2 * 4 * 32 * T * (T + 1) / 2)
    assert abs(flops - by_hand) <= 0.02 * by_hand
