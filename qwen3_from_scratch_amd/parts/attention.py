"""Softmax attention over the paged cache, with grouped heads."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import CacheNeed, PagedTensor, Part, TensorShape
from .linear import LinearWeight


def keys_and_values(kv_heads, head_dim, window=0):
    """What softmax attention keeps in pages, as its kernels read it: a page of keys is
    (kv_heads, page, head_dim), one head's keys contiguous, so a workgroup that serves one key
    head streams page * head_dim elements at a time; a page of values is (kv_heads, head_dim,
    page), transposed within the page, so that the values a matrix-core lane multiplies
    together lie side by side in memory and need no transposition on the way to the registers."""
    return CacheNeed(paged=(PagedTensor("keys", (kv_heads, head_dim), token_axis=1),
                            PagedTensor("values", (kv_heads, head_dim), token_axis=2)), window=int(window))


@register_part("mixer", "paged_attn")        # the reference's name for this component (models/self_attn.py:300)
@register_part("mixer", "attention")
class PagedAttention(Part):
    """q, k, v projections (no bias), optional per-head RMSNorm of q and k before
    rotation, rotation by the position part's table, cache write, causal
    attention over everything the cache holds for the request, output
    projection (src/qwen3_from_scratch/models/self_attn.py:310-342). The
    three projections are one matrix [q | k | v]. This step's keys and values
    are written first and attention then reads old and new alike from the
    cache (self_attn.py:382-384), which is what makes portions of prompts and
    single decoded tokens uniform.

    Parameters: hidden_size, num_heads, num_kv_heads, head_dim, qk_norm (bool),
    qk_norm_eps, window (0 = all keys), scale (None = head_dim ** -0.5).
    """

    graph_safe = True
    feeds_sink = True

    def __init__(self, prefix, precision, device, hidden_size, num_heads, num_kv_heads, head_dim,
                 qk_norm=True, qk_norm_eps=1e-6, window=0, scale=None):
        super().__init__(prefix, precision, device)
        if num_heads % num_kv_heads:
            raise ValueError("num_heads (%d) must be a multiple of num_kv_heads (%d)"
                             % (num_heads, num_kv_heads))
        if head_dim % 16 or not 16 <= head_dim <= 256:
            raise ValueError("the attention kernels take head sizes in steps of 16 from 16 to 256, not %d"
                             % head_dim)
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.qk_norm = bool(qk_norm)
        self.qk_norm_eps = float(qk_norm_eps)
        self.window = int(window)
        self.scale = float(scale) if scale is not None else head_dim ** -0.5
        self.position = None
        self.qkv = self.out = self.q_weight = self.k_weight = None

    def attach_position(self, position):
        self.position = position

    def cache_need(self):
        return keys_and_values(self.num_kv_heads, self.head_dim, self.window)

    def tensors(self):
        H, Hq, Hkv, D = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        names = {
            self._name("q_proj.weight"): (Hq * D, H),
            self._name("k_proj.weight"): (Hkv * D, H),
            self._name("v_proj.weight"): (Hkv * D, H),
            self._name("o_proj.weight"): (H, Hq * D),
        }
        if self.qk_norm:
            names[self._name("q_norm.weight")] = TensorShape((D,), "scale")
            names[self._name("k_norm.weight")] = TensorShape((D,), "scale")
        return names

    def load(self, fetch):
        act = self.precision.act
        Hq, Hkv, D = self.num_heads, self.num_kv_heads, self.head_dim
        qkv = torch.empty(((Hq + 2 * Hkv) * D, self.hidden_size), dtype=act, device=self.device)
        qkv[: Hq * D].copy_(fetch(self._name("q_proj.weight"), act, keep=False))
        qkv[Hq * D: (Hq + Hkv) * D].copy_(fetch(self._name("k_proj.weight"), act, keep=False))
        qkv[(Hq + Hkv) * D:].copy_(fetch(self._name("v_proj.weight"), act, keep=False))
        self.qkv = LinearWeight(qkv, self.precision)
        self.out = LinearWeight(fetch(self._name("o_proj.weight"), act), self.precision)
        if self.qk_norm:
            self.q_weight = fetch(self._name("q_norm.weight"))
            self.k_weight = fetch(self._name("k_norm.weight"))

    @property
    def takes_unscaled(self):
        return self.qkv is not None and self.qkv.fuses

    def forward(self, x, batch, cache, sink=None):
        Hq, Hkv, D = self.num_heads, self.num_kv_heads, self.head_dim
        qkv = self.qkv.forward(x)
        keys, values = cache.paged["keys"], cache.paged["values"]
        table = self.position.rotation_table() if self.position is not None else None
        if batch.max_q_len == 1 and qkv.shape[0] == batch.kv_lens.shape[0] and ops.decode_attention_takes(
                Hq, Hkv, D, keys.shape[2], qkv.dtype, 0 if table is None else table.shape[1]):
            # every sequence brings one token: preparation, cache write and attention are one kernel
            o = ops.decode_attention(
                qkv, Hq, Hkv, D, keys, values, cache.block_table, batch.cu_seqlens_q, batch.kv_lens,
                batch.max_kv_len, self.scale, window=self.window, q_weight=self.q_weight, k_weight=self.k_weight,
                eps=self.qk_norm_eps, table=table, store=cache.writes)
            return self.out.forward(o) if sink is None else self.out.forward_into(o, sink)
        ops.qk_norm_rope_store(
            qkv, Hq, Hkv, D, batch.positions, batch.seq_index,
            q_weight=self.q_weight, k_weight=self.k_weight, eps=self.qk_norm_eps, table=table,
            block_table=cache.block_table if cache.writes else None,
            k_cache=keys if cache.writes else None,
            v_cache=values if cache.writes else None,
            cu_seqlens_q=batch.cu_seqlens_q, kv_lens=batch.kv_lens, max_q_len=batch.max_q_len,
            max_kv_len=batch.max_kv_len,
        )
        q = qkv[:, : Hq * D].unflatten(1, (Hq, D))
        o = ops.paged_attention(
            q, Hq, keys, values, cache.block_table, batch.cu_seqlens_q, batch.kv_lens,
            batch.max_q_len, batch.max_kv_len, self.scale, window=self.window,
            min_q_len=batch.min_q_len, max_kv_len_of_many=getattr(batch, "max_kv_len_portions", None),
        )
        return self.out.forward(o) if sink is None else self.out.forward_into(o, sink)
