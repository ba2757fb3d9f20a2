"""A decoder put together from a ModelSpec: embedding, position encoding, the
layers in their run order, final norm, head. It knows parts only through their
interfaces, never by architecture."""

import torch

from ..parts.base import build_part
from ..weights.checkpoint import check_tensors


class _Layer:
    """A layer's block and the parts it arranges, built from a LayerSpec. The parts are also
    reachable by the names the spec gave them (`layer.mixer`, `layer.feed_forward_norm`, ...)."""

    def __init__(self, spec, precision, device, position):
        self.block = build_part(spec.block, spec.prefix, precision, device)
        self.named = {slot.name: build_part(slot.part, spec.prefix + "." + slot.prefix, precision, device)
                      for slot in spec.slots}
        keepers = [name for name, part in self.named.items() if hasattr(part, "cache_need")]
        if len(keepers) > 1:
            raise ValueError("layer %s: more than one part keeps a cache (%s)" % (spec.prefix, ", ".join(keepers)))
        self.cache_owner = self.named[keepers[0]] if keepers else None
        for part in self.named.values():
            if hasattr(part, "attach_position"):
                part.attach_position(position)
        self.block.attach(**self.named)

    def __getattr__(self, name):
        named = self.__dict__.get("named", {})
        if name in named:
            return named[name]
        raise AttributeError(name)

    def parts(self):
        return (self.block,) + tuple(self.named.values())


class DecoderModel:
    def __init__(self, spec, precision, device):
        self.spec = spec
        self.precision = precision
        self.device = torch.device(device)
        self.embedding = build_part(spec.embedding, spec.embedding_prefix, precision, device)
        self.position = build_part(spec.position, "", precision, device)
        self.layer_positions = {}            # position parts that layers name for themselves, one per distinct spec
        for ls in spec.layers:
            if ls.position is not None and ls.position not in self.layer_positions:
                self.layer_positions[ls.position] = build_part(ls.position, "", precision, device)
        self.layers = [_Layer(ls, precision, device,
                              self.position if ls.position is None else self.layer_positions[ls.position])
                       for ls in spec.layers]
        self.final_norm = build_part(spec.final_norm, spec.final_norm_prefix, precision, device)
        self.head = build_part(spec.head, spec.head_prefix, precision, device)
        # each run-order entry that owns a cache gets a plane; readers point at the owner's
        self.plane_of_step = []
        self.plane_needs = []
        for i, step in enumerate(spec.order):
            if step.reads_cache_of is None:
                owner = self.layers[step.layer].cache_owner
                need = owner.cache_need() if owner is not None else None
                self.plane_of_step.append(len(self.plane_needs))
                self.plane_needs.append(need)
            else:
                self.plane_of_step.append(self.plane_of_step[step.reads_cache_of])

    def parts(self):
        yield self.embedding
        yield self.position
        yield from self.layer_positions.values()
        for layer in self.layers:
            yield from layer.parts()
        yield self.final_norm
        yield self.head

    def portion_multiple(self):
        """The number of tokens that every portion of a prompt except its last must be a
        multiple of: the least common multiple of what the parts say (`Part.portion_multiple`)."""
        import math

        multiple = 1
        for part in self.parts():
            n = int(getattr(part, "portion_multiple", 1) or 1)
            if n < 1:
                raise ValueError("%s: portion_multiple must be positive" % type(part).__name__)
            multiple = multiple * n // math.gcd(multiple, n)
        return multiple

    def graph_safe(self):
        """Whether every part's forward may be captured in a HIP graph (no
        host synchronisation, no shapes that depend on values). Parts say so
        with a class attribute `graph_safe`; one that does not is taken not to be."""
        return all(getattr(part, "graph_safe", False) for part in self.parts())

    def tensors(self):
        names = {}
        for part in self.parts():
            for name, shape in part.tensors().items():
                if name in names and tuple(names[name]) != tuple(shape):
                    raise ValueError("tensor %s is wanted with shapes %s and %s" % (name, names[name], shape))
                if name not in names or not hasattr(names[name], "kind"):
                    names[name] = shape if hasattr(shape, "kind") else tuple(shape)
        return names

    def load(self, source):
        """Check the source's names and shapes against the model, then load."""
        check_tensors(source, self.tensors(), ignorable=self.spec.ignorable_tensors)
        kept = {}

        def fetch(name, dtype=None, keep=True):
            key = (name, dtype)
            if key in kept:
                return kept[key]
            tensor = source.get(name, self.device)
            if dtype is not None and tensor.dtype != dtype:
                if not tensor.dtype.is_floating_point:
                    raise ValueError("%s is an integer table and cannot become %s" % (name, dtype))
                tensor = tensor.to(dtype)
            if keep:
                kept[key] = tensor
            return tensor

        with torch.no_grad():
            for part in self.parts():
                part.load(fetch)
        return self

    @torch.no_grad()
    def forward(self, batch, cache):
        """Logits (R, V) float32 at batch.logits_rows, from batch.token_ids and
        what `cache` holds. `cache.view(plane, writes)` gives a mixer its view."""
        x = self.embedding.forward(batch.token_ids)
        x = self.position.on_embeddings(x, batch)
        pending = None
        order = self.spec.order
        for i, step in enumerate(order):
            view = cache.view(self.plane_of_step[i], writes=step.reads_cache_of is None)
            # the norm at the next block's entry, if that block can take over its division
            entry = getattr(self.layers[order[i + 1].layer].block, "entry_norm", None) if i + 1 < len(order) else None
            x, pending = self.layers[step.layer].block.forward(x, pending, batch, view,
                                                               next_norm=entry() if entry else None)
        h = self.final_norm.forward(x, delta=pending, rows=batch.logits_rows)
        return self.head.forward(h)


def expected_tensors(spec):
    """{name: shape} of every tensor a model of this spec loads."""
    from ..parts.base import Precision

    return DecoderModel(spec, Precision(torch.bfloat16), "cpu").tensors()


def build_model(config, precision, device, components=None):
    """The model of `config`'s architecture, unloaded. `components`: a user's choice of other
    registered implementations for some kinds of parts (`resolve_components`)."""
    from ..config.registry import lookup_architecture, resolve_components
    from .spec import with_components

    _, build_spec = lookup_architecture(config.architecture)
    return DecoderModel(with_components(build_spec(config), resolve_components(components)), precision, device)
