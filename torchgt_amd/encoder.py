"""The encoder layer and the node-level Graphormer around ``MultiHeadAttention``.

Mirrors of ``FeedForwardNetwork``, ``EncoderLayer`` and ``Graphormer`` of
models/graphormer_dist_node_level.py (:27-39, :276-314, :316-392): same
constructors, same parameter names (a reference ``state_dict`` loads; the
parameter counts 111 913 / 110 576 of README.md:70,114 are reproduced), same
``forward`` signatures.  Every residual add is folded into the LayerNorm that
follows it (``tgt_add_layer_norm_fwd``), GELU and all linears run on the
library's kernels; torch only keeps the autograd graph.

Dropout: the fused path covers rate 0 and eval mode (what the attention
supports); with a positive rate in training mode torch's dropout is applied at
the reference's places, with torch's random stream.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _ext, _lib
from .multi_head_attention import MultiHeadAttention, fused_linear, _DT
from .plan import GraphPlan, get_plan


def nll_loss(log_probs, target, ignore_index=-100):
    """``F.nll_loss(log_probs, target)`` of the training and evaluation loops (main_sp_sparse_node_level.py:200,
    gt_sp/evaluate.py:52): mean over the rows whose target is not ``ignore_index``, no class weights.
    ``torch.ops.torchgt.nll_loss``: one row per lane and a fixed-order sum (torch's kernel walks the rows with a
    single workgroup, ~95 + 60 us forward + backward for 64 K rows against ~5 + 3 here).  A target outside
    [0, C) other than ``ignore_index`` counts as ignored - torch raises there: check labels that may be corrupt
    before they reach the loss."""
    return _ext.ops().nll_loss(log_probs, target, int(ignore_index))


def init_params(module, n_layers):
    """models/graphormer_dist_node_level.py:18-24."""
    if isinstance(module, nn.Linear):
        module.weight.data.normal_(mean=0.0, std=0.02 / math.sqrt(n_layers))
        if module.bias is not None:
            module.bias.data.zero_()
    if isinstance(module, nn.Embedding):
        module.weight.data.normal_(mean=0.0, std=0.02)


class FeedForwardNetwork(nn.Module):
    def __init__(self, hidden_size, ffn_size, dropout_rate):
        super().__init__()
        self.layer1 = nn.Linear(hidden_size, ffn_size)
        self.gelu = nn.GELU()            # kept for the reference's module tree; the library kernel computes it
        self.layer2 = nn.Linear(ffn_size, hidden_size)

    def forward(self, x):
        l1, l2 = self.layer1, self.layer2
        ve = 4 if x.dtype == torch.float32 else 8
        if x.is_cuda and l1.bias is not None and l2.bias is not None and not (l1.in_features % ve or l1.out_features % ve or l2.out_features % ve):
            # one operator: GELU in the epilogue of layer1 (64 -> 64) and in the input gradient of layer2
            return _ext.ops().ffn(x, l1.weight, l1.bias, l2.weight, l2.bias)
        (u,) = fused_linear(x, l1)
        h = _ext.ops().gelu(u)
        (y,) = fused_linear(h, l2)
        return y


class EncoderLayer(nn.Module):
    def __init__(self, hidden_size, ffn_size, dropout_rate, attention_dropout_rate, num_heads, attn_bias_dim):
        super().__init__()
        self.self_attention_norm = nn.LayerNorm(hidden_size)
        self.self_attention = MultiHeadAttention(hidden_size, attention_dropout_rate, num_heads, attn_bias_dim)
        self.self_attention_dropout = nn.Dropout(dropout_rate)
        self.ffn_norm = nn.LayerNorm(hidden_size)
        self.ffn = FeedForwardNetwork(hidden_size, ffn_size, dropout_rate)
        self.ffn_dropout = nn.Dropout(dropout_rate)

    one_operator = True      # False: always run the layer operator by operator

    def _one_operator(self, x, attn_bias, edge_index, attn_type):
        """Whether ``torch.ops.torchgt.encoder_layer`` covers this call: sparse attention without a bias, no dropout at
        work, feature widths the kernels read without padding."""
        if not self.one_operator or attn_type != "sparse" or attn_bias is not None or edge_index is None or not x.is_cuda:
            return False
        if self.training and (self.self_attention_dropout.p > 0 or self.ffn_dropout.p > 0):
            return False
        att = self.self_attention
        if att.output_layer is None or x.dtype not in _DT:
            return False
        ve = 4 if x.dtype == torch.float32 else 8
        widths = (x.shape[-1], self.ffn.layer1.out_features, att.num_heads * att.att_size)
        return all(w % ve == 0 for w in widths) and att.num_heads * att.att_size == x.shape[-1] and all(
            lin.bias is not None for lin in (att.linear_q, att.linear_k, att.linear_v, att.output_layer, self.ffn.layer1, self.ffn.layer2))

    def forward(self, x, attn_bias=None, edge_index=None, attn_type=None, residual=None, defer_residual=False):
        """``residual``: a tensor still to be added to x (the previous layer's FFN output when it was
        called with ``defer_residual=True``); the add rides on this layer's first LayerNorm.
        ``defer_residual=True`` returns (x, ffn_output) instead of their sum."""
        n1, n2 = self.self_attention_norm, self.ffn_norm
        if self._one_operator(x, attn_bias, edge_index, attn_type):
            # the whole layer as one operator and one autograd node: the same kernels in the same order, without the
            # per-operator cost of dispatcher and autograd between the launches
            att = self.self_attention
            plan = edge_index if isinstance(edge_index, GraphPlan) else get_plan(edge_index, x.numel() // x.shape[-1])
            params = [n1.weight, n1.bias, att.linear_q.weight, att.linear_q.bias, att.linear_k.weight, att.linear_k.bias,
                      att.linear_v.weight, att.linear_v.bias, att.output_layer.weight, att.output_layer.bias, n2.weight, n2.bias,
                      self.ffn.layer1.weight, self.ffn.layer1.bias, self.ffn.layer2.weight, self.ffn.layer2.bias]
            plan.handle      # raises if the plan was closed
            x, y = _ext.ops().encoder_layer(x, residual, params, plan.holder, plan.workspace(att.num_heads, att.att_size),
                                            att.num_heads, n1.eps, n2.eps)
            return (x, y) if defer_residual else _ext.ops().add(x, y)
        x, y = _ext.ops().add_layer_norm(x, residual, n1.weight, n1.bias, float(n1.eps))
        y = self.self_attention(y, attn_bias, edge_index, attn_type=attn_type)
        y = self.self_attention_dropout(y)
        x, y = _ext.ops().add_layer_norm(x, y, n2.weight, n2.bias, float(n2.eps))
        y = self.ffn(y)
        y = self.ffn_dropout(y)
        if defer_residual:
            return x, y
        return _ext.ops().add(x, y)


class Graphormer(nn.Module):
    """Graphormer for node-level tasks, global token at index 0
    (models/graphormer_dist_node_level.py:316-392)."""

    def __init__(self, n_layers, num_heads, input_dim, hidden_dim, output_dim, attn_bias_dim, dropout_rate,
                 input_dropout_rate, attention_dropout_rate, ffn_dim, num_global_node):
        super().__init__()
        self.num_heads = num_heads
        self.node_encoder = nn.Linear(input_dim, hidden_dim)
        self.input_dropout = nn.Dropout(input_dropout_rate)
        self.layers = nn.ModuleList([EncoderLayer(hidden_dim, ffn_dim, dropout_rate, attention_dropout_rate, num_heads,
                                                  attn_bias_dim) for _ in range(n_layers)])
        self.n_layers = n_layers
        self.final_ln = nn.LayerNorm(hidden_dim)
        self.downstream_out_proj = nn.Linear(hidden_dim, output_dim)
        self.hidden_dim = hidden_dim
        self.num_global_node = num_global_node
        self.graph_token = nn.Embedding(self.num_global_node, hidden_dim)
        self.graph_token_virtual_distance = nn.Embedding(self.num_global_node, attn_bias_dim)
        self.apply(lambda module: init_params(module, n_layers=n_layers))

    def forward(self, x, attn_bias, edge_index, perturb=None, attn_type=None):
        x = x.unsqueeze(0)
        n_graph = x.shape[0]
        (node_feature,) = fused_linear(x, self.node_encoder)
        if perturb is not None:
            node_feature = node_feature + perturb
        global_node_feature = self.graph_token.weight.unsqueeze(0).expand(n_graph, -1, -1)      # a view: cat makes the copy
        node_feature = torch.cat([global_node_feature, node_feature], dim=1)
        output = self.input_dropout(node_feature)
        if attn_bias is not None:
            # the dense bias of the reference (:363-376); only practical for short sequences
            attn_bias = attn_bias.unsqueeze(0)
            n_graph, subseq_len, seq_len = attn_bias.size()[:3]
            vd = self.graph_token_virtual_distance.weight
            graph_attn_bias = torch.cat([vd.unsqueeze(0).unsqueeze(2).repeat(n_graph, 1, seq_len, 1), attn_bias.clone()], dim=1)
            graph_attn_bias = torch.cat([vd.unsqueeze(0).unsqueeze(0).repeat(n_graph, subseq_len + self.num_global_node, 1, 1),
                                         graph_attn_bias], dim=2)
            graph_attn_bias = graph_attn_bias.repeat(1, 1, 1, self.num_heads)
        else:
            graph_attn_bias = None
        pending = None
        for enc_layer in self.layers:
            output, pending = enc_layer(output, attn_bias=graph_attn_bias, edge_index=edge_index, attn_type=attn_type,
                                        residual=pending, defer_residual=True)
        fl = self.final_ln
        _, output = _ext.ops().add_layer_norm(output, pending, fl.weight, fl.bias, float(fl.eps))
        # rows 1.. of graph 0 (:391 `output[0, 1:, :]`); through a view, so that autograd pads the gradient once, not twice
        (output,) = fused_linear(output.reshape(-1, self.hidden_dim)[1:output.shape[1]], self.downstream_out_proj)
        return F.log_softmax(output, dim=1)
