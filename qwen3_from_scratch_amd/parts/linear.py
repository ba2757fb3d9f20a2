"""A weight matrix as the parts hold it: row-major, and for bfloat16 a second copy
in the order the few-row product kernel streams it."""

import torch

from .. import ops
from .base import UnscaledRows


class LinearWeight:
    """y = x @ W^T, no bias. W (N, K) is kept row-major for products with many
    rows (the vendor library's) and for float32; when the precision asks for
    it, a tile-ordered bfloat16 copy serves steps with few rows (16, or 32 or 64
    for a small weight), where every weight is read once and the order in memory
    decides the bandwidth. The copy doubles the weight's memory."""

    def __init__(self, weight, precision):
        self.weight = weight
        self.tiled = ops.tile_weight(weight) if precision.tiled else None
        if weight.is_cuda and weight.dtype == torch.bfloat16:
            ops.matmul_init()          # the many-row products' buffers: now, not inside a step

    def forward(self, x, out_dtype=None):
        """x @ W^T; x may be UnscaledRows (see `fuses`)."""
        if isinstance(x, UnscaledRows):
            return ops.linear(x.values, self.weight, out_dtype=out_dtype, tiled=self.tiled, unscaled=x.scale_args())
        return ops.linear(x, self.weight, out_dtype=out_dtype, tiled=self.tiled)

    def forward_swiglu(self, x):
        """swiglu(x @ W^T) for a W whose rows interleave gate and up."""
        if isinstance(x, UnscaledRows):
            return ops.linear_swiglu(x.values, self.weight, tiled=self.tiled, unscaled=x.scale_args())
        return ops.linear_swiglu(x, self.weight, tiled=self.tiled)

    @property
    def fuses(self):
        """Whether steps of few rows go through kernels whose epilogues carry the
        norm fusion, UnscaledRows in, a NormSink out: up to 16 rows (32 or 64 for a
        small weight) the few-row kernel on the tiled copy, up to 128 the tiled
        matrix-core kernel. A
        reader of UnscaledRows must have output rows in steps of 4."""
        return self.tiled is not None and self.weight.shape[0] % 4 == 0

    def forward_into(self, x, sink):
        """x @ W^T added into the sink's residual and prepared for its norm, as
        UnscaledRows; or, where the kernels do not take the case, returned."""
        rows = x.shape[0]
        if self.tiled is None or not (self.weight.shape[0] % 16 == 0 if rows <= ops.few_rows_limit(self.weight)
                                      else ops.fused_rows_take(self.weight, rows)):
            return self.forward(x)
        fused = ops.linear_residual_norm(x, self.weight, self.tiled, sink.residual, sink.weight)
        if fused is None:                       # the kernel leaves this size to the plain product
            return self.forward(x)
        return UnscaledRows(fused[0], fused[1], sink.eps, sink.width)
