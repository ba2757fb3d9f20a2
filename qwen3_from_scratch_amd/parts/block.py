"""How a layer's parts are arranged around the residual stream."""

from ..config.registry import register_part
from .base import Part


@register_part("block", "pre_norm")
class PreNormBlock(Part):
    """x = x + mixer(norm_1(x)); x = x + feed_forward(norm_2(x))
    (src/qwen3_from_scratch/models/transformer_block.py:38-46).

    The residual stream x is float32. The second addition is handed to whoever
    normalises next, so that each addition is fused with the norm that follows
    it: `forward` takes the stream and a pending delta and returns the same
    pair.
    """

    graph_safe = True

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)
        self.mixer = self.feed_forward = self.mixer_norm = self.feed_forward_norm = None

    def attach(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def forward(self, x, pending, batch, cache):
        h = self.mixer_norm.forward(x, delta=pending)
        d = self.mixer.forward(h, batch, cache)
        h = self.feed_forward_norm.forward(x, delta=d)
        return x, self.feed_forward.forward(h, batch)
