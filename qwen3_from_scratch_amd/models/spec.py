"""A model as data: which parts make each layer, and in which order layers run."""

from dataclasses import dataclass

from ..parts.base import PartSpec


@dataclass(frozen=True)
class Slot:
    """One part of a layer: `name` is what the layer's block calls it (the keyword under which
    the block receives it), `part` what it is, `prefix` the sub-prefix of its tensors under the
    layer's checkpoint prefix."""

    name: str
    part: PartSpec
    prefix: str


@dataclass(frozen=True)
class LayerSpec:
    """One layer: a block arrangement and the parts it arranges, by name. Which parts a layer
    has is between the architecture and its block: two norms, a mixer and a feed-forward for the
    pre-norm block, four norms for a block that also normalises what its parts return, no
    feed-forward at all for a block that has none. `prefix` is the layer's checkpoint name
    prefix. At most one part of a layer keeps a cache (the one whose class has `cache_need`).
    `position`: the position part this layer's mixer asks for its rotation table, if it is not
    the model's (layers that rotate by another base or over another part of the head, or not at
    all); layers that name equal parts share one."""

    prefix: str
    slots: tuple
    block: PartSpec = PartSpec("block", "pre_norm")
    position: PartSpec = None

    def __post_init__(self):
        object.__setattr__(self, "slots", tuple(self.slots))
        names = [slot.name for slot in self.slots]
        if len(set(names)) != len(names):
            raise ValueError("layer %s names a part twice: %r" % (self.prefix, names))

    def slot(self, name):
        for slot in self.slots:
            if slot.name == name:
                return slot
        raise KeyError("layer %s has no part called %r" % (self.prefix, name))


def pre_norm_layer(prefix, mixer, feed_forward, mixer_norm, feed_forward_norm,
                   block=PartSpec("block", "pre_norm"), position=None, mixer_prefix="self_attn",
                   feed_forward_prefix="mlp", mixer_norm_prefix="input_layernorm",
                   feed_forward_norm_prefix="post_attention_layernorm"):
    """The usual layer: a mixer and a feed-forward, each behind a norm of its own; the tensor
    prefixes default to the names that Qwen3's checkpoints use."""
    return LayerSpec(prefix=prefix, block=block, position=position, slots=(
        Slot("mixer", mixer, mixer_prefix), Slot("feed_forward", feed_forward, feed_forward_prefix),
        Slot("mixer_norm", mixer_norm, mixer_norm_prefix),
        Slot("feed_forward_norm", feed_forward_norm, feed_forward_norm_prefix)))


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
        ls, slots=tuple(dataclasses.replace(slot, part=swap(slot.part)) for slot in ls.slots),
        block=swap(ls.block), position=swap(ls.position))
        for ls in spec.layers)
    return dataclasses.replace(spec, embedding=swap(spec.embedding), position=swap(spec.position), layers=layers,
                               final_norm=swap(spec.final_norm), head=swap(spec.head))
