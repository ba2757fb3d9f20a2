"""A whole architecture that lives outside the framework: its own config.json keys, its
own configuration class, a function from that configuration to a ModelSpec, and one
`register_architecture` call. Layers follow a pattern string: `a` is the framework's
attention (with a window), `b` the same attention without a window and with a position part of
its own (a rotation over the first half of each head only, by another base), `s` the
running-mean mixer of test_toy_parts.py, which keeps a state of fixed size per request, `p` a
mixer defined here that pages one tensor of a width of its own (a float32 vector per token, of
which it reads the one `LAG` tokens back) and `n` a layer of that mixer alone, without a
feed-forward. Two more keys choose between the framework's RMS norm and a
mean-subtracting norm with a bias defined here, and between the framework's sequential block,
a block defined here whose mixer and feed-forward read the same stream, and one with four norms
(each part's result is normalised too before it is added). It is no model of anyone's; it shows that the loader, the
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
from qwen3_from_scratch_amd.config import register_architecture, register_part
from qwen3_from_scratch_amd.config.model_config import ConfigError
from qwen3_from_scratch_amd.models import LayerSpec, ModelSpec, RunStep, Slot, pre_norm_layer
from qwen3_from_scratch_amd.parts import CacheNeed, PagedTensor, Part, PartSpec, TensorShape

NAME = "ToyHybridForCausalLM"
OTHER_BASE = 7.0     # a `b` layer rotates by theta / 7
LAG = 11             # a `p` or `n` layer multiplies a token's vector with the one of the token 11 back
MEMORY = 24          # the width of that vector
KEYS = (("vocab", int), ("width", int), ("inner", int), ("heads", int), ("kv_heads", int), ("head_size", int),
        ("pattern", str), ("window", int), ("eps", float), ("theta", float), ("max_position_embeddings", int),
        ("norm", str), ("arrangement", str))


@register_part("norm", "toy_centred")
class CentredNorm(Part):
    """y = (x - mean(x)) * rsqrt(var(x) + eps) * weight + bias over the last dimension, in
    float32, rounded once. The contract of a norm: it reads the float32 stream, and with
    `delta` adds it into the stream first (in place, unless `rows` selects a subset)."""

    def __init__(self, prefix, precision, device, size, eps):
        super().__init__(prefix, precision, device)
        self.size, self.eps = size, float(eps)
        self.weight = self.bias = None

    def tensors(self):
        return {self._name("weight"): TensorShape((self.size,), "scale"),
                self._name("bias"): TensorShape((self.size,), "bias")}

    def load(self, fetch):
        self.weight = fetch(self._name("weight"), torch.float32)
        self.bias = fetch(self._name("bias"), torch.float32)

    def forward(self, x, delta=None, rows=None):
        if rows is not None:
            picked = x[rows.long()]
            if delta is not None:
                picked = picked + delta[rows.long()].float()
        else:
            if delta is not None:
                x.add_(delta.float())
            picked = x
        centred = picked - picked.mean(dim=-1, keepdim=True)
        y = centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + self.eps)
        return (y * self.weight + self.bias).to(self.precision.act)


@register_part("block", "toy_parallel")
class ParallelBlock(Part):
    """x = x + mixer(norm_1(x)) + feed_forward(norm_2(x)): both branches read the stream as it
    entered the block. The contract of a block: the float32 stream and an addend it still lacks
    come in, the stream and the next such addend go out."""

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)

    def attach(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.mixer_norm, self.feed_forward_norm = mixer_norm, feed_forward_norm

    def forward(self, x, pending, batch, cache, next_norm=None):
        h1 = self.mixer_norm.forward(x, delta=pending)          # the stream is whole from here on
        h2 = self.feed_forward_norm.forward(x)
        mixed = self.mixer.forward(h1, batch, cache)
        return x, mixed.float() + self.feed_forward.forward(h2, batch).float()


@register_part("block", "toy_sandwich")
class SandwichBlock(Part):
    """x = x + norm_2(mixer(norm_1(x))); x = x + norm_4(feed_forward(norm_3(x))): four norms a
    layer, two of them on what the parts return."""

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)

    def attach(self, mixer, feed_forward, mixer_norm, mixer_out_norm, feed_forward_norm, feed_forward_out_norm):
        self.mixer, self.feed_forward = mixer, feed_forward
        self.norms = (mixer_norm, mixer_out_norm, feed_forward_norm, feed_forward_out_norm)

    def forward(self, x, pending, batch, cache, next_norm=None):
        n1, n2, n3, n4 = self.norms
        mixed = self.mixer.forward(n1.forward(x, delta=pending), batch, cache)
        fed = self.feed_forward.forward(n3.forward(x, delta=n2.forward(mixed.float())), batch)
        return x, n4.forward(fed.float())


@register_part("block", "toy_mixer_only")
class MixerOnlyBlock(Part):
    """x = x + mixer(norm(x)): a layer without a feed-forward."""

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)

    def attach(self, mixer, mixer_norm):
        self.mixer, self.mixer_norm = mixer, mixer_norm

    def forward(self, x, pending, batch, cache, next_norm=None):
        return x, self.mixer.forward(self.mixer_norm.forward(x, delta=pending), batch, cache)


@register_part("mixer", "toy_lookback")
class Lookback(Part):
    """y_t = W_out (m_t * m_{t - lag}) with m_t = W_in x_t, a vector of `memory` numbers, and
    m_{t - lag} = 0 before the sequence's start. Every token's m goes to the request's pages: one
    paged tensor, float32 whatever the engine's precision, a token's numbers side by side; only
    the last lag + 1 tokens are kept, so pages behind that go back while the request lives."""

    graph_safe = False          # reads lengths and block tables on the host

    def __init__(self, prefix, precision, device, hidden_size, memory, lag):
        super().__init__(prefix, precision, device)
        self.hidden_size, self.memory, self.lag = hidden_size, memory, lag
        self.w_in = self.w_out = None

    def cache_need(self):
        return CacheNeed(paged=(PagedTensor("memory", (self.memory,), token_axis=0, dtype=torch.float32),),
                         window=self.lag + 1)

    def tensors(self):
        return {self._name("in.weight"): (self.memory, self.hidden_size),
                self._name("out.weight"): (self.hidden_size, self.memory)}

    def load(self, fetch):
        self.w_in = fetch(self._name("in.weight"), torch.float32)
        self.w_out = fetch(self._name("out.weight"), torch.float32)

    def forward(self, x, batch, cache):
        pages = cache.paged["memory"]                      # (pages, page_size, memory)
        size = pages.shape[1]
        m = x.float() @ self.w_in.T
        table = cache.block_table.tolist()
        out = torch.empty_like(x)
        at = 0
        for b, (n, kv) in enumerate(zip(batch.q_lens, batch.kv_lens_host)):
            for i in range(n):
                pos = kv - n + i
                if cache.writes:
                    pages[table[b][pos // size], pos % size] = m[at + i]
                back = pos - self.lag
                if back < 0:
                    old = torch.zeros_like(m[at + i])
                else:
                    page = table[b][back // size]
                    assert page >= 0, "the page of a position inside the window was given back"
                    old = pages[page, back % size]
                out[at + i] = ((m[at + i] * old) @ self.w_out.T).to(x.dtype)
            at += n
        return out


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
    norm: str
    arrangement: str
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, data):
        missing = [k for k, _ in KEYS if k not in data]
        if missing:
            raise ConfigError("config.json of %s lacks %s" % (NAME, ", ".join(missing)))
        if not data["pattern"] or set(data["pattern"]) - set("abspn"):
            raise ConfigError("pattern must be a string of 'a', 'b', 's', 'p' and 'n'")
        if data["norm"] not in ("rms", "centred") or data["arrangement"] not in ("sequential", "parallel", "sandwich"):
            raise ConfigError("norm is rms or centred, arrangement sequential, parallel or sandwich")
        return cls(architecture=data["architectures"][0], **{k: kind(data[k]) for k, kind in KEYS})

    def to_dict(self):
        data = dataclasses.asdict(self)
        data["architectures"] = [data.pop("architecture")]
        data.pop("eos_token_ids")
        return data


def toy_hybrid_spec(c):
    norm = PartSpec.of("norm", "rms" if c.norm == "rms" else "toy_centred", size=c.width, eps=c.eps)
    block = PartSpec.of("block", {"sequential": "pre_norm", "parallel": "toy_parallel",
                                  "sandwich": "toy_sandwich"}[c.arrangement])
    attention = PartSpec.of("mixer", "attention", hidden_size=c.width, num_heads=c.heads, num_kv_heads=c.kv_heads,
                            head_dim=c.head_size, qk_norm=False, qk_norm_eps=c.eps, window=c.window)
    everything = attention.with_params(window=0)
    half_rotation = PartSpec.of("position", "rotary", rotary_dim=c.head_size // 2, theta=c.theta / OTHER_BASE,
                                max_positions=c.max_position_embeddings)
    mean = PartSpec.of("mixer", "toy_running_mean", hidden_size=c.width)
    ff = PartSpec.of("feed_forward", "swiglu", hidden_size=c.width, intermediate_size=c.inner)
    lookback = PartSpec.of("mixer", "toy_lookback", hidden_size=c.width, memory=MEMORY, lag=LAG)
    mixers = {"a": attention, "b": everything, "s": mean, "p": lookback, "n": lookback}

    def layer(i, kind):
        prefix = "hybrid.layers.%d" % i
        if kind == "n":                 # a mixer behind its norm and nothing else
            return LayerSpec(prefix=prefix, block=PartSpec.of("block", "toy_mixer_only"), slots=(
                Slot("mixer", lookback, "self_attn"), Slot("mixer_norm", norm, "input_layernorm")))
        usual = pre_norm_layer(prefix, mixer=mixers[kind], feed_forward=ff, mixer_norm=norm, feed_forward_norm=norm,
                               block=block, position=half_rotation if kind == "b" else None)
        if c.arrangement != "sandwich":
            return usual
        return dataclasses.replace(usual, slots=usual.slots + (
            Slot("mixer_out_norm", norm, "post_mixer_norm"), Slot("feed_forward_out_norm", norm, "post_mlp_norm")))

    layers = tuple(layer(i, kind) for i, kind in enumerate(c.pattern))
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

EXAMPLE = dict(architectures=[NAME], vocab=211, width=40, inner=72, heads=6, kv_heads=2, head_size=16, pattern="asab",
               window=21, eps=1e-5, theta=10000.0, max_position_embeddings=512, norm="rms", arrangement="sequential")
# every size and option differs; the norm and the block are the ones defined above
EXAMPLE_PARALLEL = dict(architectures=[NAME], vocab=157, width=56, inner=100, heads=4, kv_heads=4, head_size=32,
                        pattern="sbas", window=0, eps=1e-6, theta=500000.0, max_position_embeddings=300,
                        norm="centred", arrangement="parallel")
# a block with four norms, a mixer that pages one tensor of its own width, a layer without a feed-forward
EXAMPLE_SANDWICH = dict(architectures=[NAME], vocab=173, width=48, inner=88, heads=3, kv_heads=1, head_size=16,
                        pattern="pasnb", window=17, eps=1e-5, theta=20000.0, max_position_embeddings=400,
                        norm="rms", arrangement="sandwich")


def _norm(c, x, w, name):
    if c.norm == "rms":
        return plain.rms_norm(x, w[name + ".weight"], c.eps)
    centred = x - x.mean(dim=-1, keepdim=True)
    return centred * torch.rsqrt(centred.pow(2).mean(dim=-1, keepdim=True) + c.eps) * w[name + ".weight"] + w[name + ".bias"]


def plain_logits(c, w, tokens):
    """The architecture on one whole sequence with elementary operations; `w` maps tensor names
    to float32 tensors."""
    T = len(tokens)
    pos = torch.arange(T)
    x = w["hybrid.embed.weight"][torch.tensor(tokens)]
    for i, kind in enumerate(c.pattern):
        p = "hybrid.layers.%d" % i
        h = _norm(c, x, w, p + ".input_layernorm")
        if kind == "s":
            mean = torch.cumsum(h, dim=0) / torch.arange(1, T + 1)[:, None]
            mixed = mean @ w[p + ".self_attn.mix.weight"].T
        elif kind in "pn":
            m = h @ w[p + ".self_attn.in.weight"].T
            old = torch.cat((torch.zeros(min(LAG, T), m.shape[1]), m[:max(T - LAG, 0)]), dim=0)
            mixed = (m * old) @ w[p + ".self_attn.out.weight"].T
        else:
            a = p + ".self_attn"
            q = (h @ w[a + ".q_proj.weight"].T).view(T, c.heads, c.head_size)
            k = (h @ w[a + ".k_proj.weight"].T).view(T, c.kv_heads, c.head_size)
            if kind == "a":
                ang = plain.rotary_angles(pos, c.head_size, c.theta, torch.float32)
                q, k = plain.apply_rotary(q, ang), plain.apply_rotary(k, ang)
            else:       # the first half of each head rotates, by another base; the second half stays
                R = c.head_size // 2
                ang = plain.rotary_angles(pos, R, c.theta / OTHER_BASE, torch.float32)
                q = torch.cat((plain.apply_rotary(q[..., :R], ang), q[..., R:]), dim=-1)
                k = torch.cat((plain.apply_rotary(k[..., :R], ang), k[..., R:]), dim=-1)
            v = (h @ w[a + ".v_proj.weight"].T).view(T, c.kv_heads, c.head_size)
            o = plain.causal_attention(q, k, v, 1.0 / math.sqrt(c.head_size),
                                       (c.window or None) if kind == "a" else None)
            mixed = o.reshape(T, c.heads * c.head_size) @ w[a + ".o_proj.weight"].T
        if kind == "n":
            x = x + mixed
        elif c.arrangement == "sandwich":
            x = x + _norm(c, mixed, w, p + ".post_mixer_norm")
            fed = plain.swiglu_mlp(_norm(c, x, w, p + ".post_attention_layernorm"), w, p + ".mlp")
            x = x + _norm(c, fed, w, p + ".post_mlp_norm")
        elif c.arrangement == "parallel":
            x = x + mixed + plain.swiglu_mlp(_norm(c, x, w, p + ".post_attention_layernorm"), w, p + ".mlp")
        else:
            x = x + mixed
            x = x + plain.swiglu_mlp(_norm(c, x, w, p + ".post_attention_layernorm"), w, p + ".mlp")
    return _norm(c, x, w, "hybrid.norm") @ w["hybrid.embed.weight"].T
