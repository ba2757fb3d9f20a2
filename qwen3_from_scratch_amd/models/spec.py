"""A model as data: which parts make each layer, and in which order layers run."""

from dataclasses import dataclass

from ..parts.base import PartSpec


@dataclass(frozen=True)
class LayerSpec:
    """One layer's parts. `prefix` is the layer's checkpoint name prefix; the
    `*_prefix` fields are the sub-prefixes of its parts under it. `position`:
    the position part this layer's mixer asks for its rotation table, if it is
    not the model's (layers that rotate by another base or over another part of
    the head, or not at all); layers that name equal parts share one."""

    prefix: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    block: PartSpec = PartSpec("block", "pre_norm")
    position: PartSpec = None
    mixer_prefix: str = "self_attn"
    feed_forward_prefix: str = "mlp"
    mixer_norm_prefix: str = "input_layernorm"
    feed_forward_norm_prefix: str = "post_attention_layernorm"


@dataclass(frozen=True)
class RunStep:
    """One entry of the run order. `layer` indexes ModelSpec.layers (a layer
    may be named by several entries: its weights are shared, each entry has a
    cache of its own). `reads_cache_of` names an earlier entry of the run order
    whose cache this entry's mixer reads without writing; None = its own."""

    layer: int
    reads_cache_of: int = None


@dataclass(frozen=True)
class ModelSpec:
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    embedding_prefix: str
    position: PartSpec
    layers: tuple
    order: tuple
    final_norm: PartSpec
    final_norm_prefix: str
    head: PartSpec
    head_prefix: str = ""
    ignorable_tensors: tuple = ()

    def __post_init__(self):
        for i, step in enumerate(self.order):
            if not (0 <= step.layer < len(self.layers)):
                raise ValueError("run order entry %d names layer %d of %d" % (i, step.layer, len(self.layers)))
            if step.reads_cache_of is not None:
                j = step.reads_cache_of
                if not (0 <= j < i) or self.order[j].reads_cache_of is not None:
                    raise ValueError(
                        "run order entry %d must read the cache of an earlier entry that owns one" % i)


def with_components(spec, resolved):
    """`spec` with every part of a kind that `resolved` names (see
    `config.registry.resolve_components`) replaced by the named implementation. The replacement
    stands where the other stood: it is built with the same parameters (the sizes and constants
    the architecture gave that place) plus the user's `kwargs`, so it must take them."""
    if not resolved:
        return spec
    import dataclasses

    def swap(part):
        if part is None or part.kind not in resolved:
            return part
        name, kwargs = resolved[part.kind]
        return PartSpec(part.kind, name or part.name, part.params).with_params(**kwargs)

    layers = tuple(dataclasses.replace(
        ls, mixer=swap(ls.mixer), feed_forward=swap(ls.feed_forward), mixer_norm=swap(ls.mixer_norm),
        feed_forward_norm=swap(ls.feed_forward_norm), block=swap(ls.block), position=swap(ls.position))
        for ls in spec.layers)
    return dataclasses.replace(spec, embedding=swap(spec.embedding), position=swap(spec.position), layers=layers,
                               final_norm=swap(spec.final_norm), head=swap(spec.head))
