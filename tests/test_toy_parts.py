"""Parts defined here, outside the framework, are registered, built into a model
with the framework's own parts, and stepped: a mixer with a state of fixed size
per request, a feed-forward whose router gives most experts no weight, a
position encoding added to the embeddings, an attention layer with a window, a
layer that runs twice, and a layer that reads another layer's cache. Nothing under qwen3_from_scratch_amd changes for them. They never
become a model of anyone's: they exist to show what the interfaces carry.

The same test runs on the CPU (plain twins in place of the kernels) and, marked
gpu, on the GPU in float32 and bfloat16.
"""

import math

import pytest
import torch

import plain_qwen3 as plain
from helpers import max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions, trace_tail_decoded, trace_whole
from qwen3_from_scratch_amd.config import register_part
from qwen3_from_scratch_amd.engine import ModelRunner
from qwen3_from_scratch_amd.models import DecoderModel, ModelSpec, RunStep, pre_norm_layer
from qwen3_from_scratch_amd.parts import CacheNeed, Part, PartSpec, Precision
from qwen3_from_scratch_amd.weights import RandomWeights

V, HQ, HKV, I = 97, 4, 2, 80
EXPERTS, EXPERT_I = 4, 24
EPS, THETA, WINDOW, MAXPOS = 1e-5, 10000.0, 19, 512
H, D = 48, 16                 # the default sizes; `sizes()` swaps in others for one test


@register_part("mixer", "toy_running_mean")
class RunningMean(Part):
    """y_t = W . mean(x_0 .. x_t): needs, per request, the sum so far and the
    count, H + 1 numbers, whatever the request's length. The state lives in
    the slot the cache manager gave the request."""

    graph_safe = False          # reads slots and lengths on the host

    def __init__(self, prefix, precision, device, hidden_size):
        super().__init__(prefix, precision, device)
        self.hidden_size = hidden_size
        self.weight = None

    def cache_need(self):
        return CacheNeed(state_shape=(self.hidden_size + 1,), state_dtype=torch.float32)

    def tensors(self):
        return {self._name("mix.weight"): (self.hidden_size, self.hidden_size)}

    def load(self, fetch):
        self.weight = fetch(self._name("mix.weight"), torch.float32)

    def forward(self, x, batch, cache):
        out = torch.empty_like(x)
        slots = batch.state_slots.tolist()
        at = 0
        for b, n in enumerate(batch.q_lens):
            state = cache.state[slots[b]]
            sums = state[:-1] + torch.cumsum(x[at:at + n].float(), dim=0)
            counts = state[-1] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
            out[at:at + n] = ((sums / counts[:, None]) @ self.weight.T).to(x.dtype)
            state[:-1] = sums[-1]
            state[-1] = counts[-1]
            at += n
        return out


@register_part("position", "toy_learned")
class LearnedPosition(Part):
    """A table of position vectors added to the embeddings; no rotation."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, max_positions):
        super().__init__(prefix, precision, device)
        self.hidden_size, self.max_positions = hidden_size, max_positions
        self.table = None

    def tensors(self):
        return {"toy.positions.weight": (self.max_positions, self.hidden_size)}

    def load(self, fetch):
        self.table = fetch("toy.positions.weight", torch.float32)

    def on_embeddings(self, x, batch):
        return x + self.table[batch.positions.long()]

    def rotation_table(self):
        return None


def routing_weights(probabilities):
    """An expert counts by how far its probability lies above the uniform one,
    and not at all below it; the weights sum to one. Unlike a top-k choice this
    is continuous in the router's logits, so that rounding moves the result a
    little and never to another expert's."""
    above = torch.relu(probabilities - 1.0 / probabilities.shape[-1])
    return above / above.sum(dim=-1, keepdim=True).clamp_min(1e-6)


@register_part("feed_forward", "toy_routed")
class RoutedFeedForward(Part):
    """sum_e g_e(x) . down_e(relu(up_e(x))), the router in float32. All experts
    are computed for all rows and weighted (g_e is zero for most), which keeps
    the part free of host decisions and so fit for graph replays."""

    graph_safe = True

    def __init__(self, prefix, precision, device, hidden_size, intermediate_size, num_experts):
        super().__init__(prefix, precision, device)
        self.hidden_size, self.intermediate_size, self.num_experts = hidden_size, intermediate_size, num_experts
        self.router = self.up = self.down = None

    def tensors(self):
        names = {self._name("router.weight"): (self.num_experts, self.hidden_size)}
        for e in range(self.num_experts):
            names[self._name("experts.%d.up.weight" % e)] = (self.intermediate_size, self.hidden_size)
            names[self._name("experts.%d.down.weight" % e)] = (self.hidden_size, self.intermediate_size)
        return names

    def load(self, fetch):
        act = self.precision.act
        self.router = fetch(self._name("router.weight"), torch.float32)
        self.up = [fetch(self._name("experts.%d.up.weight" % e), act) for e in range(self.num_experts)]
        self.down = [fetch(self._name("experts.%d.down.weight" % e), act) for e in range(self.num_experts)]

    def forward(self, x, batch=None):
        g = routing_weights(torch.softmax(x.float() @ self.router.T, dim=-1))
        out = torch.zeros(x.shape, dtype=torch.float32, device=x.device)
        for e in range(self.num_experts):
            out += g[:, e:e + 1] * (torch.relu(x @ self.up[e].T) @ self.down[e].T).float()
        return out.to(x.dtype)


def toy_spec(position, with_state=True):
    norm = PartSpec.of("norm", "rms", size=H, eps=EPS)
    attn = dict(hidden_size=H, num_heads=HQ, num_kv_heads=HKV, head_dim=D, qk_norm=True, qk_norm_eps=EPS)
    ff = PartSpec.of("feed_forward", "swiglu", hidden_size=H, intermediate_size=I)

    routed = PartSpec.of("feed_forward", "toy_routed", hidden_size=H, intermediate_size=EXPERT_I, num_experts=EXPERTS)

    def layer(i, mixer):
        return pre_norm_layer("toy.layers.%d" % i, mixer=mixer, feed_forward=routed if i == 2 else ff,
                              mixer_norm=norm, feed_forward_norm=norm)

    layers = (
        layer(0, PartSpec.of("mixer", "attention", window=0, **attn)),
        layer(1, PartSpec.of("mixer", "toy_running_mean", hidden_size=H) if with_state
              else PartSpec.of("mixer", "attention", window=0, **dict(attn, qk_norm=False))),
        layer(2, PartSpec.of("mixer", "attention", window=WINDOW, **attn)),
        layer(3, PartSpec.of("mixer", "attention", window=0, **dict(attn, qk_norm=False))),
    )
    # layer 0 runs twice (weights shared, a cache each); the last entry reads the first entry's cache
    order = (RunStep(0), RunStep(1), RunStep(2), RunStep(0), RunStep(3, reads_cache_of=0))
    if position == "rotary":
        pos = PartSpec.of("position", "rotary", rotary_dim=D, theta=THETA, max_positions=MAXPOS)
    else:
        pos = PartSpec.of("position", "toy_learned", hidden_size=H, max_positions=MAXPOS)
    return ModelSpec(hidden_size=H, vocab_size=V,
                     embedding=PartSpec.of("embedding", "token", vocab_size=V, hidden_size=H),
                     embedding_prefix="toy.embed", position=pos, layers=layers, order=order,
                     final_norm=norm, final_norm_prefix="toy.norm",
                     head=PartSpec.of("head", "linear", hidden_size=H, vocab_size=V, weight_name="toy.head.weight"))


def plain_toy_logits(w, spec, position, tokens):
    """The toy model on one whole sequence with elementary operations."""
    T = len(tokens)
    pos = torch.arange(T)
    x = w["toy.embed.weight"][torch.tensor(tokens)]
    if position != "rotary":
        x = x + w["toy.positions.weight"][pos]
    kept = {}
    for step_index, step in enumerate(spec.order):
        i = step.layer
        p = "toy.layers.%d" % i
        h = plain.rms_norm(x, w[p + ".input_layernorm.weight"], EPS)
        mixer = spec.layers[i].slot("mixer").part
        if mixer.name == "toy_running_mean":
            mean = torch.cumsum(h, dim=0) / torch.arange(1, T + 1)[:, None]
            d = mean @ w[p + ".self_attn.mix.weight"].T
        else:
            a = p + ".self_attn"
            q = (h @ w[a + ".q_proj.weight"].T).view(T, HQ, D)
            k = (h @ w[a + ".k_proj.weight"].T).view(T, HKV, D)
            v = (h @ w[a + ".v_proj.weight"].T).view(T, HKV, D)
            if mixer.get("qk_norm"):
                q = plain.rms_norm(q, w[a + ".q_norm.weight"], EPS)
                k = plain.rms_norm(k, w[a + ".k_norm.weight"], EPS)
            if position == "rotary":
                ang = plain.rotary_angles(pos, D, THETA, torch.float32)
                q, k = plain.apply_rotary(q, ang), plain.apply_rotary(k, ang)
            if step.reads_cache_of is None:
                kept[step_index] = (k, v)
            else:
                k, v = kept[step.reads_cache_of]
            o = plain.causal_attention(q, k, v, 1.0 / math.sqrt(D), mixer.get("window") or None)
            d = o.reshape(T, HQ * D) @ w[a + ".o_proj.weight"].T
        x = x + d
        h = plain.rms_norm(x, w[p + ".post_attention_layernorm.weight"], EPS)
        if spec.layers[i].slot("feed_forward").part.name == "toy_routed":
            g = routing_weights(torch.softmax(h @ w[p + ".mlp.router.weight"].T, dim=-1))
            for e in range(EXPERTS):
                up, down = w[p + ".mlp.experts.%d.up.weight" % e], w[p + ".mlp.experts.%d.down.weight" % e]
                x = x + g[:, e:e + 1] * (torch.relu(h @ up.T) @ down.T)
        else:
            x = x + plain.swiglu_mlp(h, w, p + ".mlp")
    return plain.rms_norm(x, w["toy.norm.weight"], EPS) @ w["toy.head.weight"].T


def build(position, dtype, device, with_state=True):
    spec = toy_spec(position, with_state)
    model = DecoderModel(spec, Precision.named(dtype), device)
    source = RandomWeights(model.tensors(), seed=3, std=0.08, norm_jitter=0.2)
    model.load(source)
    weights = {name: source.get(name, "cpu").float() for name in source.names()}
    return spec, model, weights


def check(position, dtype, device, tol, with_state=True, page=8):
    spec, model, weights = build(position, dtype, device, with_state)
    needs = model.plane_needs
    if with_state:
        assert not model.graph_safe()                   # the toy mixer says it is not: it runs without graphs
        assert [n.window for n in needs if n.paged] == [0, WINDOW, 0] and needs[1].has_state
    else:
        assert model.graph_safe() and [n.window for n in needs if n.paged] == [0, 0, WINDOW, 0]
    requests = {"t%d" % i: random_tokens(n, V, 30 + i) for i, n in enumerate([70, 9, 41, 130, 25])}
    want = {rid: plain_toy_logits(weights, spec, position, toks) for rid, toks in requests.items()}
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = ModelRunner(model, page_size=page, num_pages=max_live_tokens(steps, page=page) // page, max_requests=4)
        assert len(runner.manager.groups) == 2 and len(runner.manager.state_groups) == (1 if with_state else 0)
        got = run_trace(runner, steps)
        worst = max(float((got[(rid, p)] - logits[p]).abs().max())
                    for rid, logits in want.items() for p in range(logits.shape[0]))
        assert worst <= tol, (make.__name__, worst)
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)


@pytest.mark.parametrize("position", ["rotary", "toy_learned"])
def test_toy_model_on_the_host(cpu_ops, position):
    check(position, "float32", "cpu", 2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("position", ["rotary", "toy_learned"])
@pytest.mark.parametrize("dtype,tol", [("float32", 5e-4), ("bfloat16", 0.25)])
def test_toy_model_on_the_gpu(position, dtype, tol):
    check(position, dtype, "cuda", tol)


@pytest.fixture
def graph_sizes(monkeypatch):
    """Sizes the matrix-core and few-row kernels take (head 64, width 64), so that a model of
    built-in parts alone goes through graph replays, the fused decoding kernel and the norm
    fusion, with a window and a layer that reads another's cache in play."""
    import sys
    module = sys.modules[__name__]
    monkeypatch.setattr(module, "H", 64)
    monkeypatch.setattr(module, "D", 64)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 5e-4), ("bfloat16", 0.25)])
def test_windows_and_shared_caches_through_graph_replays(graph_sizes, dtype, tol):
    check("rotary", dtype, "cuda", tol, with_state=False, page=16)


def test_a_window_frees_pages_while_the_request_lives(cpu_ops):
    spec, model, _ = build("rotary", "float32", "cpu")
    runner = ModelRunner(model, page_size=8, num_pages=40, max_requests=2)
    steps = trace_portions({"w": random_tokens(200, V, 1)}, sizes=(16,))
    from qwen3_from_scratch_amd.engine import StepEntry
    windowed = [g for g, grp in enumerate(runner.manager.groups) if grp.window][0]
    for entries, _ in steps:
        runner.step([StepEntry(r, t, []) for r, t, _ in entries])
        held = sum(p >= 0 for p in runner.manager.block_table("w", windowed))
        assert held <= (WINDOW + 8 - 1) // 8 + 2       # about a window's worth, however long the request
    assert sum(p >= 0 for p in runner.manager.block_table("w", 1 - windowed)) == 25
    runner.finish("w")
    runner.manager.audit()
