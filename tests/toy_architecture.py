"""A whole architecture that lives outside the framework: its own config.json keys, its
own configuration class, a function from that configuration to a ModelSpec, and one
`register_architecture` call. Layers follow a pattern string: `a` is the framework's
attention (with a window), `s` the running-mean mixer of test_toy_parts.py, which keeps a
state of fixed size per request. It is no model of anyone's; it shows that the loader, the
random-weights writer, the cache manager, the step function, the engine and the replay
program take an architecture they have never heard of.

The programs that take only a model folder find it when this module is named in
$QWEN3_FROM_SCRATCH_AMD_PLUGINS and is importable.
"""

import dataclasses
import math

import torch

import plain_qwen3 as plain
import test_toy_parts  # registers the mixer "toy_running_mean"  # noqa: F401
from qwen3_from_scratch_amd.config import register_architecture
from qwen3_from_scratch_amd.config.model_config import ConfigError
from qwen3_from_scratch_amd.models import LayerSpec, ModelSpec, RunStep
from qwen3_from_scratch_amd.parts import PartSpec

NAME = "ToyHybridForCausalLM"
KEYS = (("vocab", int), ("width", int), ("inner", int), ("heads", int), ("kv_heads", int), ("head_size", int),
        ("pattern", str), ("window", int), ("eps", float), ("theta", float), ("max_position_embeddings", int))


@dataclasses.dataclass(frozen=True)
class ToyHybridConfig:
    architecture: str
    vocab: int
    width: int
    inner: int
    heads: int
    kv_heads: int
    head_size: int
    pattern: str
    window: int
    eps: float
    theta: float
    max_position_embeddings: int
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, data):
        missing = [k for k, _ in KEYS if k not in data]
        if missing:
            raise ConfigError("config.json of %s lacks %s" % (NAME, ", ".join(missing)))
        if not data["pattern"] or set(data["pattern"]) - set("as"):
            raise ConfigError("pattern must be a string of 'a' and 's'")
        return cls(architecture=data["architectures"][0], **{k: kind(data[k]) for k, kind in KEYS})

    def to_dict(self):
        data = dataclasses.asdict(self)
        data["architectures"] = [data.pop("architecture")]
        data.pop("eos_token_ids")
        return data


def toy_hybrid_spec(c):
    norm = PartSpec.of("norm", "rms", size=c.width, eps=c.eps)
    attention = PartSpec.of("mixer", "attention", hidden_size=c.width, num_heads=c.heads, num_kv_heads=c.kv_heads,
                            head_dim=c.head_size, qk_norm=False, qk_norm_eps=c.eps, window=c.window)
    mean = PartSpec.of("mixer", "toy_running_mean", hidden_size=c.width)
    ff = PartSpec.of("feed_forward", "swiglu", hidden_size=c.width, intermediate_size=c.inner)
    layers = tuple(LayerSpec(prefix="hybrid.layers.%d" % i, mixer=attention if kind == "a" else mean, feed_forward=ff,
                             mixer_norm=norm, feed_forward_norm=norm) for i, kind in enumerate(c.pattern))
    return ModelSpec(
        hidden_size=c.width, vocab_size=c.vocab,
        embedding=PartSpec.of("embedding", "token", vocab_size=c.vocab, hidden_size=c.width),
        embedding_prefix="hybrid.embed",
        position=PartSpec.of("position", "rotary", rotary_dim=c.head_size, theta=c.theta,
                             max_positions=c.max_position_embeddings),
        layers=layers, order=tuple(RunStep(i) for i in range(len(layers))),
        final_norm=norm, final_norm_prefix="hybrid.norm",
        head=PartSpec.of("head", "linear", hidden_size=c.width, vocab_size=c.vocab, weight_name="hybrid.embed.weight"))


register_architecture(NAME, ToyHybridConfig, toy_hybrid_spec)

EXAMPLE = dict(architectures=[NAME], vocab=211, width=40, inner=72, heads=6, kv_heads=2, head_size=16, pattern="asa",
               window=21, eps=1e-5, theta=10000.0, max_position_embeddings=512)


def plain_logits(c, w, tokens):
    """The architecture on one whole sequence with elementary operations; `w` maps tensor names
    to float32 tensors."""
    T = len(tokens)
    pos = torch.arange(T)
    x = w["hybrid.embed.weight"][torch.tensor(tokens)]
    for i, kind in enumerate(c.pattern):
        p = "hybrid.layers.%d" % i
        h = plain.rms_norm(x, w[p + ".input_layernorm.weight"], c.eps)
        if kind == "s":
            mean = torch.cumsum(h, dim=0) / torch.arange(1, T + 1)[:, None]
            x = x + mean @ w[p + ".self_attn.mix.weight"].T
        else:
            a = p + ".self_attn"
            ang = plain.rotary_angles(pos, c.head_size, c.theta, torch.float32)
            q = plain.apply_rotary((h @ w[a + ".q_proj.weight"].T).view(T, c.heads, c.head_size), ang)
            k = plain.apply_rotary((h @ w[a + ".k_proj.weight"].T).view(T, c.kv_heads, c.head_size), ang)
            v = (h @ w[a + ".v_proj.weight"].T).view(T, c.kv_heads, c.head_size)
            o = plain.causal_attention(q, k, v, 1.0 / math.sqrt(c.head_size), c.window or None)
            x = x + o.reshape(T, c.heads * c.head_size) @ w[a + ".o_proj.weight"].T
        h = plain.rms_norm(x, w[p + ".post_attention_layernorm.weight"], c.eps)
        x = x + plain.swiglu_mlp(h, w, p + ".mlp")
    return plain.rms_norm(x, w["hybrid.norm.weight"], c.eps) @ w["hybrid.embed.weight"].T
