"""How a layer's parts are arranged around the residual stream."""

from ..config.registry import register_part
from .base import Part, UnscaledRows


def _says(part, what):
    return bool(getattr(part, what, False))


@register_part("block", "pre_norm")
class PreNormBlock(Part):
    """x = x + mixer(norm_1(x)); x = x + feed_forward(norm_2(x))
    (src/qwen3_from_scratch/models/transformer_block.py:38-46).

    The residual stream x is float32. The second addition is handed to whoever
    normalises next, so that each addition is fused with the norm that follows
    it: `forward` takes the stream and a pending delta and returns the same
    pair. In steps of few rows the addition and the norm move further, into
    the products on either side (NormSink, UnscaledRows), where the parts on
    both sides say they can; the stand-alone norm kernel serves all other cases.
    """

    graph_safe = True

    def __init__(self, prefix, precision, device):
        super().__init__(prefix, precision, device)
        self.mixer = self.feed_forward = self.mixer_norm = self.feed_forward_norm = None

    def attach(self, mixer, feed_forward, mixer_norm, feed_forward_norm):
        """The layer's parts, under the names its LayerSpec gave them: a block's `attach` names
        the parts it arranges as its keywords, and a layer that brings others does not build."""
        self.mixer = mixer
        self.feed_forward = feed_forward
        self.mixer_norm = mixer_norm
        self.feed_forward_norm = feed_forward_norm

    def entry_norm(self):
        """The norm a preceding block may fuse into its last product (see
        NormSink), or None if this block's mixer wants finished rows."""
        return self.mixer_norm if _says(self.mixer, "takes_unscaled") and hasattr(self.mixer_norm, "sink_for") else None

    def forward(self, x, pending, batch, cache, next_norm=None):
        """`pending`: None, the addend the stream still lacks, or UnscaledRows
        (then the addition is done and `mixer_norm` all but applied).
        `next_norm`: the norm that reads the stream after this block, if its
        reader takes UnscaledRows. Returns the stream and the next `pending`."""
        h = pending if isinstance(pending, UnscaledRows) else self.mixer_norm.forward(x, delta=pending)
        sink = None
        if (_says(self.mixer, "feeds_sink") and _says(self.feed_forward, "takes_unscaled")
                and hasattr(self.feed_forward_norm, "sink_for")):
            sink = self.feed_forward_norm.sink_for(x)
        d = self.mixer.forward(h, batch, cache, sink=sink) if sink is not None else self.mixer.forward(h, batch, cache)
        h = d if isinstance(d, UnscaledRows) else self.feed_forward_norm.forward(x, delta=d)
        sink = next_norm.sink_for(x) if next_norm is not None and _says(self.feed_forward, "feeds_sink") else None
        if sink is not None:
            return x, self.feed_forward.forward(h, batch, sink=sink)
        return x, self.feed_forward.forward(h, batch)
