"""The parts a model is put together from. Importing registers them."""

from .base import CacheNeed, NormSink, PagedTensor, Part, PartSpec, Precision, TensorShape, UnscaledRows, build_part
from . import attention, block, embedding, feed_forward, head, norm, position  # noqa: F401

__all__ = ["CacheNeed", "NormSink", "PagedTensor", "Part", "PartSpec", "Precision", "TensorShape", "UnscaledRows", "build_part"]
