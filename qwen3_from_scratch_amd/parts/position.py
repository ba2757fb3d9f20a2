"""Position encodings.

A position part may act at two places: on the embeddings (`on_embeddings`,
for encodings that are added to the input) and inside a mixer, which asks it
for a rotation table (`rotation_table`) and applies it to queries and keys in
its own fused kernel. Either hook may be a no-op.
"""

import torch

from .. import ops
from ..config.registry import register_part
from .base import Part


@register_part("position", "none")
class NoPosition(Part):
    graph_safe = True

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)

    def on_embeddings(self, x, batch):
        return x

    def rotation_table(self):
        return None


@register_part("position", "rotary")
class RotaryPosition(NoPosition):
    """Rotate-half (NeoX) rotary encoding over `rotary_dim` leading elements of
    each head. angle[p, i] = p * theta^(-2i / rotary_dim); the table holds
    [cos | sin] per position in float32
    (src/qwen3_from_scratch/models/rotary.py:36-45). Inverse frequencies are
    formed on the host exactly as the reference forms them; angles, cosines
    and sines are computed on the GPU in float32."""

    def __init__(self, prefix, precision, device, rotary_dim, theta, max_positions):
        super().__init__(prefix, precision, device)
        if rotary_dim % 2:
            raise ValueError("rotary_dim must be even, found %d" % rotary_dim)
        self.rotary_dim = rotary_dim
        self.theta = float(theta)
        self.max_positions = max_positions
        self._table = None

    def load(self, fetch):
        exponent = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        inv_freq = (1.0 / (self.theta ** exponent)).to(self.device)
        self._table = ops.rope_table(inv_freq, self.max_positions)

    def rotation_table(self):
        return self._table
