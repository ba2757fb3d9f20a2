"""A plain, slow Qwen3 dense decoder: whole sequences, no cache, one function per part.

It is written from the formulas of the reference repository (paths below are
relative to its root) and shares no code with the engine under
``qwen3_from_scratch_amd``: it reads ``config.json`` and ``model.safetensors``
with the json and safetensors libraries directly, and evaluates every part with
elementary tensor operations in one dtype (float32, or float64 as a tighter
yardstick).
"""

import json
import math
import os

import torch
from safetensors import safe_open


def read_model_folder(folder, dtype=torch.float32):
    """config.json as a dict and every tensor of model.safetensors in `dtype`.

    Names consumed are those of src/qwen3_from_scratch/models/qwen3.py:36-42,67-74.
    """
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as fh:
        for name in fh.keys():
            tensors[name] = fh.get_tensor(name).to(dtype)
    return cfg, tensors


def rms_norm(x, weight, eps):
    """y = x * rsqrt(mean(x^2) + eps) * w, eps inside the root, plain weight.

    src/qwen3_from_scratch/models/norm.py:51-53 (explicit form) and :18-22.
    """
    mean_sq = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(mean_sq + eps) * weight


def rotary_angles(positions, head_dim, theta, dtype):
    """angle[p, i] = p * theta^(-2i/D), i = 0 .. D/2-1.

    src/qwen3_from_scratch/models/rotary.py:36-42. The inverse frequencies are
    formed in float32 as the reference does, so that a float64 run uses the
    same angles' definition.
    """
    exponent = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    inv_freq = (1.0 / (theta ** exponent)).to(dtype)
    return positions.to(dtype)[:, None] * inv_freq[None, :]


def apply_rotary(x, angles):
    """NeoX rotation, pairs (i, i + D/2): y1 = x1 cos - x2 sin, y2 = x2 cos + x1 sin.

    x: (T, heads, D); angles: (T, D/2).
    src/qwen3_from_scratch/models/rotary.py:19-22, models/self_attn.py:328-336.
    """
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    cos = torch.cos(angles)[:, None, :]
    sin = torch.sin(angles)[:, None, :]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def causal_attention(q, k, v, scale, window=None):
    """Softmax attention over one whole sequence with grouped heads.

    q: (T, Hq, D), k and v: (T, Hkv, D). Query head h reads key head h // G
    (src/qwen3_from_scratch/models/attn.py:412-414), scores are scaled by
    `scale` = D^-0.5 (:407), key j is visible to query i iff j <= i (:476-480),
    and, if `window` is given, iff i - j < window.
    """
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    out = torch.empty_like(q)
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    hidden = j > i
    if window is not None:
        hidden = hidden | (i - j >= window)
    for h in range(Hq):
        g = h // G
        s = (q[:, h, :] @ k[:, g, :].T) * scale
        s = s.masked_fill(hidden, float("-inf"))
        s = s - s.max(dim=-1, keepdim=True).values
        p = torch.exp(s)
        p = p / p.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ v[:, g, :]
    return out


def self_attention(x, w, prefix, cfg, positions):
    """qkv projections, per-head q/k RMSNorm, rotation, attention, output projection.

    src/qwen3_from_scratch/models/self_attn.py:310-342: norm before rotation,
    v untouched, no biases; heads are consecutive blocks of D columns (:319-322).
    """
    T = x.shape[0]
    Hq, Hkv, D = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps = cfg["rms_norm_eps"]
    q = (x @ w[prefix + ".q_proj.weight"].T).view(T, Hq, D)
    k = (x @ w[prefix + ".k_proj.weight"].T).view(T, Hkv, D)
    v = (x @ w[prefix + ".v_proj.weight"].T).view(T, Hkv, D)
    q = rms_norm(q, w[prefix + ".q_norm.weight"], eps)
    k = rms_norm(k, w[prefix + ".k_norm.weight"], eps)
    angles = rotary_angles(positions, D, cfg["rope_theta"], x.dtype)
    q = apply_rotary(q, angles)
    k = apply_rotary(k, angles)
    o = causal_attention(q, k, v, 1.0 / math.sqrt(D), cfg.get("_window"))
    return o.reshape(T, Hq * D) @ w[prefix + ".o_proj.weight"].T


def swiglu_mlp(x, w, prefix):
    """down(up(x) * silu(gate(x))), silu(g) = g * sigmoid(g), no biases.

    src/qwen3_from_scratch/models/feedback.py:28-34.
    """
    up = x @ w[prefix + ".up_proj.weight"].T
    gate = x @ w[prefix + ".gate_proj.weight"].T
    act = gate / (1.0 + torch.exp(-gate))
    return (up * act) @ w[prefix + ".down_proj.weight"].T


def decoder_layer(x, w, i, cfg, positions):
    """Pre-norm block with the residual added outside each sub-module.

    src/qwen3_from_scratch/models/transformer_block.py:38-46.
    """
    p = "model.layers.%d" % i
    eps = cfg["rms_norm_eps"]
    h = rms_norm(x, w[p + ".input_layernorm.weight"], eps)
    x = x + self_attention(h, w, p + ".self_attn", cfg, positions)
    h = rms_norm(x, w[p + ".post_attention_layernorm.weight"], eps)
    return x + swiglu_mlp(h, w, p + ".mlp")


def logits_of_sequence(cfg, w, token_ids, first_position=0, rows=None):
    """Logits (T, V) at every position of one whole sequence (or at `rows` only).

    Embedding gather without scaling, the layers, the final norm, the output
    matrix, which is the embedding itself when tie_word_embeddings is set
    (src/qwen3_from_scratch/models/qwen3.py:44-50,67-74,83-84).
    `first_position` shifts all positions; only distances count for rotation.
    """
    emb = w["model.embed_tokens.weight"]
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    x = emb[ids]
    positions = torch.arange(first_position, first_position + len(token_ids))
    for i in range(cfg["num_hidden_layers"]):
        x = decoder_layer(x, w, i, cfg, positions)
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long)]
    x = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    head = emb if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return x @ head.T


def greedy_generate(cfg, w, prompt, n_new):
    """n_new tokens by repeated argmax of the last position's logits.

    src/qwen3_from_scratch/inference/sampler.py:17-21.
    """
    ids = list(prompt)
    for _ in range(n_new):
        logits = logits_of_sequence(cfg, w, ids)
        ids.append(int(torch.argmax(logits[-1])))
    return ids[len(prompt):]
