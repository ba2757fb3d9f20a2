"""What every part is: a named, parameterised piece with tensors of its own.

A part is described by a `PartSpec` (kind, registered name, parameters) and
built by `build_part`. It declares the checkpoint tensors it needs
(`tensors()`), receives them (`load()`), and computes (`forward` with the
signature of its kind, see each module). Parameters carry every size and
constant; a part never looks at a model configuration and does not know which
model it is in.
"""

from dataclasses import dataclass, field

import torch

from ..config.registry import lookup_part


@dataclass(frozen=True)
class Precision:
    """Compute dtypes of one engine instance. Activations, matrices and the
    cache share `act`; the residual stream and logits are float32. `tiled`:
    keep a second, tile-ordered copy of every bfloat16 matrix for the few-row
    product kernel (decoding); it costs the matrices' memory once more."""

    act: torch.dtype
    tiled: bool = True

    @classmethod
    def named(cls, name, tiled=True):
        name = str(name).replace("torch.", "")
        if name in ("bfloat16", "bf16"):
            return cls(torch.bfloat16, tiled=bool(tiled))
        if name in ("float32", "fp32"):
            return cls(torch.float32, tiled=bool(tiled))
        raise ValueError("dtype must be bfloat16 or float32, found %r" % (name,))

    @property
    def name(self):
        return "bfloat16" if self.act == torch.bfloat16 else "float32"


@dataclass(frozen=True)
class PartSpec:
    kind: str
    name: str
    params: tuple = ()

    @classmethod
    def of(cls, kind, name, **params):
        return cls(kind, name, tuple(sorted(params.items())))

    def get(self, key, default=None):
        return dict(self.params).get(key, default)

    def with_params(self, **more):
        merged = dict(self.params)
        merged.update(more)
        return PartSpec(self.kind, self.name, tuple(sorted(merged.items())))


class TensorShape(tuple):
    """A tensor's shape, with a word on what the tensor is for whoever has to make
    one up (the random-weights mode): "matrix" (products and tables: small values
    around zero), "scale" (a norm's multiplier: values around one) or "bias"
    (an addend: small values around zero). A plain tuple stands for a matrix."""

    kind = "matrix"

    def __new__(cls, shape, kind="matrix"):
        if kind not in ("matrix", "scale", "bias"):
            raise ValueError("a tensor is a matrix, a scale or a bias, not %r" % (kind,))
        self = super().__new__(cls, tuple(shape))
        self.kind = kind
        return self


class Part:
    """Base class. `prefix` is the checkpoint name prefix of the part's tensors."""

    # whether forward() may be captured in a HIP graph: it launches kernels only,
    # never synchronises with the host, and sizes nothing by a tensor's values.
    # A model with a part that does not declare this is run without graphs.
    graph_safe = False
    # the norm fusion of steps with few rows (see NormSink, UnscaledRows): whether forward()
    # takes `sink=`, and whether it takes UnscaledRows for its input
    feeds_sink = False
    takes_unscaled = False
    # a part that works on a request's tokens in runs of fixed length (a mixer that keeps its
    # state per run of N tokens, say) sets N here: the scheduler then cuts every portion of a
    # prompt except its last to a multiple of N. The step function itself takes any cut.
    portion_multiple = 1

    def __init__(self, prefix, precision, device):
        self.prefix = prefix
        self.precision = precision
        self.device = torch.device(device)

    def tensors(self):
        """{checkpoint tensor name: shape} of everything this part loads; a
        shape is a tuple, or a `TensorShape` that also says what the tensor is."""
        return {}

    def load(self, fetch):
        """`fetch(name, dtype=None)` returns the tensor on the device, in its
        stored dtype or converted to `dtype`; equal requests share one tensor."""

    def _name(self, leaf):
        return self.prefix + "." + leaf if self.prefix else leaf


@dataclass
class NormSink:
    """Where a part's last product may go instead of being returned: added into
    `residual` (float32 (T, width), in place) and prepared for the root-mean-square
    norm that reads the residual next, which is given by its numbers alone:
    `weight` (width,), `eps`, `width`. A part whose class sets `feeds_sink` takes
    it as `forward(..., sink=...)` and then returns `UnscaledRows`; it may also
    ignore the sink and return its result as always. A norm of another form (a
    bias, a mean taken out) offers no sink and is applied by its own kernel."""

    residual: torch.Tensor
    weight: torch.Tensor
    eps: float
    width: int


@dataclass
class UnscaledRows:
    """A norm's output before the division by the root mean square: `values`
    (T, width) hold residual * weight in the activation dtype, `sums` (P, T
    rounded up to 16) float32 hold the rows' sums of squares in P partial
    sums (row t in column t). A part whose `takes_unscaled` is true accepts this in place of its
    input tensor and applies rsqrt(sum / width + eps) to its first product."""

    values: torch.Tensor
    sums: torch.Tensor
    eps: float
    width: int

    def scale_args(self):
        return (self.sums, self.eps, self.width)


def build_part(spec, prefix, precision, device):
    cls = lookup_part(spec.kind, spec.name)
    return cls(prefix=prefix, precision=precision, device=device, **dict(spec.params))


@dataclass(frozen=True)
class PagedTensor:
    """One tensor that a mixer keeps in pages: every token adds one element of `shape` to it.

    A page of it holds `page_size` tokens and is shaped shape[:token_axis] + (page_size,) +
    shape[token_axis:], so the mixer says where in a page the tokens' axis stands: 0 puts a
    token's numbers side by side, the last place puts the same number of consecutive tokens
    side by side. `dtype`: None for the engine's activation dtype. The mixer finds the tensor
    under `name` in its view of the cache (`LayerCacheView.paged[name]`, shaped (pages, *page))."""

    name: str
    shape: tuple
    token_axis: int = 0
    dtype: object = None

    def __post_init__(self):
        object.__setattr__(self, "shape", tuple(int(n) for n in self.shape))
        if not self.shape or min(self.shape) <= 0:
            raise ValueError("paged tensor %r: a token's shape needs positive sizes, found %r" % (self.name, self.shape))
        if not 0 <= self.token_axis <= len(self.shape):
            raise ValueError("paged tensor %r: token_axis %d is outside 0..%d"
                             % (self.name, self.token_axis, len(self.shape)))

    def page_shape(self, page_size):
        return self.shape[:self.token_axis] + (int(page_size),) + self.shape[self.token_axis:]

    def numbers_per_token(self):
        n = 1
        for size in self.shape:
            n *= size
        return n


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer keeps per request between steps.

    paged: the tensors that grow by one element per token (`PagedTensor`s: for softmax
    attention a request's keys and values; another mixer may page one tensor, or tensors of
    different widths), all tokens kept (window == 0) or the last `window`. state: a tensor of
    fixed `state_shape` and `state_dtype` per request. A mixer may need neither, either or
    both. Mixers whose needs are equal share page numbers: one block table serves them all.
    """

    paged: tuple = ()
    window: int = 0
    state_shape: tuple = ()
    state_dtype: torch.dtype = torch.float32

    def __post_init__(self):
        object.__setattr__(self, "paged", tuple(self.paged))
        object.__setattr__(self, "state_shape", tuple(self.state_shape))
        names = [t.name for t in self.paged]
        if len(set(names)) != len(names):
            raise ValueError("paged tensors of one mixer need different names, found %r" % (names,))

    @property
    def has_state(self):
        return len(self.state_shape) > 0

    def bytes_per_token(self, act_dtype):
        """Bytes that one token adds to one layer's pages."""
        total = 0
        for t in self.paged:
            total += t.numbers_per_token() * torch.empty((), dtype=t.dtype or act_dtype).element_size()
        return total

    def bytes_of_state(self):
        if not self.has_state:
            return 0
        n = torch.empty((), dtype=self.state_dtype).element_size()
        for size in self.state_shape:
            n *= size
        return n
