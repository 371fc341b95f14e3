"""Oracle: the graph-level Graphormer forward (test infrastructure, CPU, torch float64 so that
autograd gives the reference gradients).

Restates, op for op, ``GraphNodeFeature.forward`` (models/graphormer_graph_level.py:38-60),
``EncoderLayer.forward`` (:283-306) with dropout rate 0 and ``Graphormer.forward`` (:368-389) on top of
``oracle.dense_attention`` (the attention and both ``GraphAttnBias`` branches).  LayerNorm and GELU
are written out (biased variance with eps inside the root; ``0.5 x (1 + erf(x / sqrt 2))``).

Pinned in ``tests/test_oracle_graph_level.py``: ``graph_node_feature`` against
``torch.nn.functional.embedding`` and a hand-computed answer; the model against the same network
assembled from torch's own ``layer_norm`` / ``linear`` / ``gelu`` / ``softmax`` routines, the closed form
of a model without layers (output = head of the normalised graph token), invariance under a
relabelling of the nodes of a graph and under extra padding.
"""
import math

import torch

from . import dense_attention as _da


def graph_node_feature(x, in_degree, out_degree, atom_table, in_table, out_table, graph_token):
    """x [b, s, Fx] int64, in_degree / out_degree [b, s] int64, tables [num, C], graph_token [1, C].
    Returns [b, s + 1, C], the graph token first."""
    n_graph = x.shape[0]
    node_feature = atom_table[x].sum(dim=-2)                                           # :45
    node_feature = node_feature + in_table[in_degree] + out_table[out_degree]          # :46-50
    graph_token_feature = graph_token.unsqueeze(0).repeat(n_graph, 1, 1)               # :52
    return torch.cat([graph_token_feature, node_feature], dim=1)                       # :56


def layer_norm(x, gamma, beta, eps=1e-5):
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * gamma + beta


def gelu(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def _linear(x, p, name):
    return x @ p[name + ".weight"].t() + p[name + ".bias"]


def encoder_layer(x, p, prefix, attn_bias, num_heads):
    """x [b, S, hidden]; p: the model's parameters by ``state_dict`` key (float64 tensors)."""
    b, S, hidden = x.shape
    d = hidden // num_heads
    y = layer_norm(x, p[prefix + "self_attention_norm.weight"], p[prefix + "self_attention_norm.bias"])      # :287
    q = _linear(y, p, prefix + "self_attention.linear_q").view(b, S, num_heads, d)                          # :244-246
    k = _linear(y, p, prefix + "self_attention.linear_k").view(b, S, num_heads, d)
    v = _linear(y, p, prefix + "self_attention.linear_v").view(b, S, num_heads, d)
    y = _da.dense_attention(q, k, v, attn_bias)                                                             # :253
    y = _linear(y, p, prefix + "self_attention.output_layer")                                               # :260
    x = x + y                                                                                               # :290
    y = layer_norm(x, p[prefix + "ffn_norm.weight"], p[prefix + "ffn_norm.bias"])                            # :296
    y = _linear(gelu(_linear(y, p, prefix + "ffn.layer1")), p, prefix + "ffn.layer2")                        # :172-175
    return x + y                                                                                            # :299


def graphormer_forward(p, batch, n_layers, num_heads, edge_type, multi_hop_max_dist, head="downstream_out_proj"):
    """``Graphormer.forward`` (:368-389).  ``batch``: dict with x, in_degree, out_degree, attn_bias,
    spatial_pos and attn_edge_type or edge_input.  Returns [b, output_dim]."""
    x = graph_node_feature(batch["x"], batch["in_degree"], batch["out_degree"], p["graph_node_feature.atom_encoder.weight"],
                           p["graph_node_feature.in_degree_encoder.weight"], p["graph_node_feature.out_degree_encoder.weight"],
                           p["graph_node_feature.graph_token.weight"])                                       # :369
    g = "graph_attn_bias."
    if edge_type == "multi_hop":                                                                            # :370
        bias = _da.graph_attn_bias_multi_hop(batch["attn_bias"], batch["spatial_pos"], batch["edge_input"],
                                             p[g + "spatial_pos_encoder.weight"], p[g + "edge_encoder.weight"],
                                             p[g + "edge_dis_encoder.weight"], p[g + "graph_token_virtual_distance.weight"],
                                             multi_hop_max_dist)
    else:
        bias = _da.graph_attn_bias(batch["attn_bias"], batch["spatial_pos"], batch["attn_edge_type"],
                                   p[g + "spatial_pos_encoder.weight"], p[g + "edge_encoder.weight"],
                                   p[g + "graph_token_virtual_distance.weight"])
    out = x
    for l in range(n_layers):                                                                               # :375-380
        out = encoder_layer(out, p, f"layers.{l}.", bias, num_heads)
    out = layer_norm(out, p["final_ln.weight"], p["final_ln.bias"])                                          # :381
    return _linear(out[:, 0, :], p, head)                                                                   # :387
