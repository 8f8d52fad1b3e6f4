"""The parts a model is put together from. Importing registers them."""

from .base import (AnySize, BiasedRows, CacheNeed, HyperAddend, NormSink, PagedTensor, Part, PartSpec, Precision, StreamAddend, TensorShape, UnscaledRows,
                   build_part)
from . import (attention, block, channel_delta, embedding, feed_forward, head, latent_attention, mamba2, norm,  # noqa: F401
               parallel, position, retention, rglru, routed_experts, sink_attention, softcap_attention)

__all__ = ["AnySize", "BiasedRows", "CacheNeed", "HyperAddend", "NormSink", "PagedTensor", "Part", "PartSpec", "Precision", "StreamAddend", "TensorShape", "UnscaledRows", "build_part"]
