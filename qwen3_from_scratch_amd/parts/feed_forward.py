"""Feed-forward parts."""

import torch

from .. import ops
from ..config.registry import register_part
from .base import Part
from .linear import LinearWeight


@register_part("feed_forward", "swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)), no biases
    (src/qwen3_from_scratch/models/feedback.py:28-34). gate and up are kept as
    one matrix with their rows interleaved (row 2i gate's, row 2i + 1 up's), so
    that one product feeds the activation, which for few rows is the product
    kernel's epilogue (the reference's fused variant concatenates them,
    feedback.py:52-54)."""

    graph_safe = True
    feeds_sink = True

    def __init__(self, prefix, precision, device, hidden_size, intermediate_size):
        super().__init__(prefix, precision, device)
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.gate_up = None
        self.down = None

    def tensors(self):
        H, I = self.hidden_size, self.intermediate_size
        return {
            self._name("gate_proj.weight"): (I, H),
            self._name("up_proj.weight"): (I, H),
            self._name("down_proj.weight"): (H, I),
        }

    def load(self, fetch):
        act = self.precision.act
        I, H = self.intermediate_size, self.hidden_size
        gate_up = torch.empty((2 * I, H), dtype=act, device=self.device)
        gate_up[0::2].copy_(fetch(self._name("gate_proj.weight"), act, keep=False))
        gate_up[1::2].copy_(fetch(self._name("up_proj.weight"), act, keep=False))
        self.gate_up = LinearWeight(gate_up, self.precision)
        self.down = LinearWeight(fetch(self._name("down_proj.weight"), act), self.precision)

    @property
    def takes_unscaled(self):
        return self.gate_up is not None and self.gate_up.fuses

    def forward(self, x, batch=None, sink=None):
        h = self.gate_up.forward_swiglu(x)
        return self.down.forward(h) if sink is None else self.down.forward_into(h, sink)
