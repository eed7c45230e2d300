"""The parts a model is put together from. Importing registers them."""

from .base import (CacheNeed, HyperAddend, NormSink, PagedTensor, Part, PartSpec, Precision, StreamAddend, TensorShape, UnscaledRows,
                   build_part)
from . import (attention, block, embedding, feed_forward, head, latent_attention, mamba2, norm, parallel, position,  # noqa: F401
               retention, rglru, routed_experts, softcap_attention)

__all__ = ["CacheNeed", "HyperAddend", "NormSink", "PagedTensor", "Part", "PartSpec", "Precision", "StreamAddend", "TensorShape", "UnscaledRows", "build_part"]
