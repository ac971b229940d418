"""MI355X-native streaming paged-KV attention for LingBot-Map's global blocks.

``HipPagedKVCacheManager`` stands in for the reference's ``FlashInferKVCacheManager``
(lingbot_map/layers/flashinfer_cache.py:55); ``HipPagedBlock`` for its ``FlashInferBlock``
(lingbot_map/layers/block.py:151); ``HipAggregatorStream`` for its ``AggregatorStream``
(lingbot_map/aggregator/stream.py:37).  Importing this package loads the HIP library and raises
if it has not been built: there is no CPU path.
"""
from . import _native  # noqa: F401  (loads the library, fails loudly when missing)
from .aggregator import GraphedAggregator, HipAggregatorStream, PatchConv, PatchTrunk, PipelinedAggregator
from .block import (HipPagedAttention, HipPagedBlock, PositionGetter, RotaryPositionEmbedding2D,
                    RotaryPositionEmbedding3D, WanRotaryPosEmbed, keyframe_flags, set_skip_append)
from .dense import dense_attention
from .graph import GraphedFrame, GraphedStream
from .manager import HipPagedKVCacheManager

__all__ = ["HipAggregatorStream", "PatchConv", "PatchTrunk", "HipPagedKVCacheManager", "HipPagedAttention", "HipPagedBlock", "RotaryPositionEmbedding2D",
           "RotaryPositionEmbedding3D", "WanRotaryPosEmbed", "PositionGetter",
           "dense_attention", "GraphedFrame", "GraphedStream", "GraphedAggregator", "PipelinedAggregator", "keyframe_flags", "set_skip_append"]
