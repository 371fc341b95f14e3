"""Oracle: the node-level GT model forward (test infrastructure, CPU, torch float64 so that autograd gives
the reference gradients).

Restates, op for op, ``EncoderLayer.forward`` (models/gt_dist_node_level.py:238-261), ``MLPReadout.forward``
(:278-286) and ``GT.forward`` (:321-341) with dropout rate 0 on top of ``oracle.sparse_attention``.  Kept
quirks: the feed-forward block reads the attention branch (after ``O``), not the normalised sum; LayerNorm
follows each residual add; ``self_attention_norm`` and ``downstream_out_proj`` take no part.

Pinned in ``tests/test_oracle_gt.py``: the same network from torch's own ``layer_norm`` / ``linear`` / ``relu`` /
``softmax`` routines on a complete graph (where the sparse attention without clamping is a dense softmax), the
closed form of a model without layers, invariance under a relabelling of the nodes.
"""
import torch

from . import sparse_attention as _sa


def layer_norm(x, gamma, beta, eps=1e-5):
    mean = x.mean(dim=-1, keepdim=True)
    var = ((x - mean) ** 2).mean(dim=-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * gamma + beta


def relu(x):
    return torch.where(x > 0, x, torch.zeros_like(x))


def _linear(x, p, name):
    return x @ p[name + ".weight"].t() + p[name + ".bias"]


def encoder_layer(x, p, prefix, edge_index, num_heads):
    """x [1, S, hidden]; p: parameters by ``state_dict`` key (float64 tensors)."""
    b, S, hidden = x.shape
    d = hidden // num_heads
    q = _linear(x, p, prefix + "self_attention.linear_q").view(b, S, num_heads, d)        # :197-199
    k = _linear(x, p, prefix + "self_attention.linear_k").view(b, S, num_heads, d)
    v = _linear(x, p, prefix + "self_attention.linear_v").view(b, S, num_heads, d)
    y, _ = _sa.sparse_attention(q, k, v, edge_index)                                      # :208
    y = y.reshape(b, S, hidden)
    y = _linear(y, p, prefix + "O")                                                       # :246
    x = layer_norm(x + y, p[prefix + "layer_norm1.weight"], p[prefix + "layer_norm1.bias"])   # :247-248
    y = _linear(y, p, prefix + "FFN_layer1")                                              # :254  (reads y)
    y = relu(y)                                                                           # :255
    y = _linear(y, p, prefix + "FFN_layer2")                                              # :257
    return layer_norm(x + y, p[prefix + "layer_norm2.weight"], p[prefix + "layer_norm2.bias"])  # :258-259


def mlp_readout(x, p, prefix="MLP_layer.", L=2):
    y = x
    for l in range(L):
        y = relu(_linear(y, p, f"{prefix}FC_layers.{l}"))                                 # :281-283
    return _linear(y, p, f"{prefix}FC_layers.{L}")                                        # :284


def gt_forward(p, x, edge_index, n_layers, num_heads):
    """``GT.forward`` (:321-341).  x [S, input_dim].  Returns log-probabilities [S, output_dim]."""
    out = _linear(x.unsqueeze(0), p, "node_encoder")                                      # :323-327
    for l in range(n_layers):                                                             # :332-337
        out = encoder_layer(out, p, f"layers.{l}.", edge_index, num_heads)
    out = mlp_readout(out[0], p)                                                          # :340
    return torch.log_softmax(out, dim=1)                                                  # :341


def gt_graph_level_forward(p, x_ids, edge_index, n_layers, num_heads):
    """``GT.forward`` of models/gt_graph_level.py:333-363 (one sequence per graph).  x_ids int64 [b, s, Fx];
    edge_index over the flattened b * s axis.  Returns [b, output_dim].  Pinned in tests/test_oracle_gt.py by
    the closed form without layers and by the independence of the graphs of a batch."""
    out = p["embedding_h.weight"][x_ids].sum(dim=-2)                                      # :334
    for l in range(n_layers):                                                             # :344-349
        out = encoder_layer(out, p, f"layers.{l}.", edge_index, num_heads)
    out = out.mean(dim=1)                                                                 # :357
    return mlp_readout(out, p)                                                            # :360
