"""Each part alone on the GPU against the plain implementation's function for it,
at sizes of its own (not a model's)."""

import math

import pytest
import torch

import plain_qwen3 as plain
from qwen3_from_scratch_amd.cache import CacheManager, CacheStorage
from qwen3_from_scratch_amd.engine.batch import StepEntry, pack_step
from qwen3_from_scratch_amd.parts import PartSpec, Precision, build_part

pytestmark = pytest.mark.gpu
MODES = [("float32", 1e-5, 1e-5), ("bfloat16", 2e-2, 2e-2)]


def _weights(part, seed, std=0.1):
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in part.tensors().items():
        t = torch.randn(shape, generator=g) * std
        if len(shape) == 1:
            t = 1 + t
        w[name] = t.to(torch.bfloat16)
    return w


def _load(part, w):
    def fetch(name, dtype=None, keep=True):
        t = w[name].cuda()
        return t.to(dtype) if dtype is not None else t
    part.load(fetch)
    return {k: v.float() for k, v in w.items()}


def _build(kind, name, prefix, dtype, **params):
    return build_part(PartSpec.of(kind, name, **params), prefix, Precision.named(dtype), "cuda")


@pytest.mark.parametrize("dtype,rtol,atol", MODES)
def test_rms_norm_part(dtype, rtol, atol):
    part = _build("norm", "rms", "n", dtype, size=200, eps=1e-4)
    w = _load(part, _weights(part, 1))
    x = torch.randn(9, 200).cuda()
    d = torch.randn(9, 200).to(part.precision.act).cuda()
    x0 = x.clone()
    got = part.forward(x, delta=d)
    want = plain.rms_norm(x0.cpu() + d.float().cpu(), w["n.weight"], 1e-4)
    torch.testing.assert_close(got.float().cpu(), want, rtol=rtol, atol=atol)
    torch.testing.assert_close(x.cpu(), x0.cpu() + d.float().cpu())       # the stream took the delta


def test_rotary_position_part():
    part = _build("position", "rotary", "", "float32", rotary_dim=48, theta=50000.0, max_positions=300)
    part.load(None)
    table = part.rotation_table().cpu()
    ang = plain.rotary_angles(torch.arange(300), 48, 50000.0, torch.float32)
    torch.testing.assert_close(table[:, :24], ang.cos(), rtol=0, atol=2e-6)
    torch.testing.assert_close(table[:, 24:], ang.sin(), rtol=0, atol=2e-6)


@pytest.mark.parametrize("dtype,rtol,atol", MODES)
def test_embedding_and_head_parts(dtype, rtol, atol):
    emb = _build("embedding", "token", "e", dtype, vocab_size=77, hidden_size=40)
    w = _load(emb, _weights(emb, 2))
    ids = torch.tensor([0, 76, 5, 5], dtype=torch.int32).cuda()
    assert torch.equal(emb.forward(ids).cpu(), w["e.weight"][ids.cpu().long()])
    head = _build("head", "linear", "", dtype, hidden_size=40, vocab_size=77, weight_name="e.weight")
    _load(head, {"e.weight": (w["e.weight"]).to(torch.bfloat16)})
    h = torch.randn(3, 40).to(head.precision.act).cuda()
    logits = head.forward(h)
    assert logits.dtype == torch.float32
    torch.testing.assert_close(logits.cpu(), h.float().cpu() @ w["e.weight"].T, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("dtype,rtol,atol", MODES)
def test_swiglu_part(dtype, rtol, atol):
    part = _build("feed_forward", "swiglu", "m", dtype, hidden_size=72, intermediate_size=136)
    w = _load(part, _weights(part, 3))
    x = torch.randn(11, 72).to(part.precision.act).cuda()
    got = part.forward(x)
    want = plain.swiglu_mlp(x.float().cpu(), w, "m")
    torch.testing.assert_close(got.float().cpu(), want, rtol=rtol, atol=atol)


@pytest.mark.parametrize("dtype,rtol,atol", [("float32", 1e-4, 1e-5), ("bfloat16", 3e-2, 3e-2)])
@pytest.mark.parametrize("Hq,Hkv,D,page", [(6, 2, 32, 8), (4, 1, 64, 16)])
def test_attention_part_over_a_cache(dtype, rtol, atol, Hq, Hkv, D, page):
    """The mixer alone: a prompt in two portions, then two single tokens, against
    the plain attention over the whole sequence."""
    Hd, T = 56, 45
    pos = _build("position", "rotary", "", dtype, rotary_dim=D, theta=1e4, max_positions=128)
    pos.load(None)
    part = _build("mixer", "attention", "a", dtype, hidden_size=Hd, num_heads=Hq, num_kv_heads=Hkv, head_dim=D,
                  qk_norm=True, qk_norm_eps=1e-5)
    part.attach_position(pos)
    w = _load(part, _weights(part, 4))
    manager = CacheManager([part.cache_need()], page, 16, 2)
    storage = CacheStorage(manager, part.precision.act, "cuda")
    x = torch.randn(T, Hd).to(part.precision.act)
    cfg = dict(num_attention_heads=Hq, num_key_value_heads=Hkv, head_dim=D, rms_norm_eps=1e-5, rope_theta=1e4)
    want = plain.self_attention(x.float(), w, "a", cfg, torch.arange(T))
    manager.admit("r")
    at, outs = 0, []
    for n in (30, 13, 1, 1):
        manager.reserve("r", n)
        batch, tables = pack_step([StepEntry("r", [0] * n, [])], [at], [0], [[manager.block_table("r", 0)]], "cuda")
        storage.bind(tables)
        outs.append(part.forward(x[at:at + n].cuda(), batch, storage.view(0)))
        manager.commit("r", n)
        at += n
    torch.testing.assert_close(torch.cat(outs).float().cpu(), want, rtol=rtol, atol=atol)


def test_block_part_defers_its_second_addition():
    dtype = "float32"
    prec = Precision.named(dtype)
    norm = PartSpec.of("norm", "rms", size=32, eps=1e-6)
    block = build_part(PartSpec("block", "pre_norm"), "b", prec, "cuda")

    class Doubler:                      # stands for a mixer and for a feed-forward
        def forward(self, h, batch, cache=None):
            return 2 * h
    n1 = build_part(norm, "b.n1", prec, "cuda")
    n2 = build_part(norm, "b.n2", prec, "cuda")
    for n in (n1, n2):
        n.load(lambda name, dtype=None, keep=True: torch.ones(32, device="cuda"))
    block.attach(Doubler(), Doubler(), n1, n2)
    x = torch.randn(5, 32).cuda()
    pending = torch.randn(5, 32).cuda()
    x0 = (x + pending).cpu()
    out, delta = block.forward(x, pending, None, None)
    h1 = plain.rms_norm(x0, torch.ones(32), 1e-6)
    x1 = x0 + 2 * h1
    torch.testing.assert_close(out.cpu(), x1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(delta.cpu(), 2 * plain.rms_norm(x1, torch.ones(32), 1e-6), rtol=1e-5, atol=1e-5)
