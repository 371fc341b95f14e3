"""torchgt_amd — MI355X (gfx950) implementation of TorchGT's topology-aware
sparse attention behind the reference's ``CoreAttention`` module API.

The compute lives in ``libtorchgt_hip.so`` (sources in ``csrc/``, C ABI in
``include/torchgt_hip.h``); this package is the thin host side.
"""
from .core_attention import (CoreAttention, SparseAttentionFunction, DenseAttentionFunction, sparse_attention,
                             dense_attention, gather_dense_bias)
from .plan import GraphPlan, get_plan, clear_plan_cache, set_plan_cache_bytes
from .multi_head_attention import MultiHeadAttention, LinearFunction, fused_linear
from .encoder import FeedForwardNetwork, EncoderLayer, Graphormer, nll_loss
from .graph_bias import GraphAttnBias, floyd_warshall, gen_edge_input
from .graph_level import GraphNodeFeature, Graphormer as GraphLevelGraphormer
from .gt import GT, GraphLevelGT, MLPReadout
from .block_attention import BlockAttentionFunction, TileSet, block_attention, expand_tiles

__all__ = ["CoreAttention", "SparseAttentionFunction", "DenseAttentionFunction", "sparse_attention",
           "dense_attention", "gather_dense_bias",
           "GraphPlan", "get_plan", "clear_plan_cache", "set_plan_cache_bytes", "BlockAttentionFunction", "TileSet", "block_attention",
           "expand_tiles", "MultiHeadAttention", "LinearFunction", "fused_linear",
           "FeedForwardNetwork", "EncoderLayer", "Graphormer", "nll_loss", "GraphAttnBias", "floyd_warshall", "gen_edge_input",
           "GraphNodeFeature", "GraphLevelGraphormer", "GT", "GraphLevelGT", "MLPReadout"]
