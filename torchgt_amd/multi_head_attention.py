"""``MultiHeadAttention`` with the projections on the library's kernels.

Mirror of the reference module of the same name
(models/graphormer_dist_node_level.py:224-273, models/gt_dist_node_level.py:169-216,
models/graphormer_dist_graph_level.py): same constructor, same parameter names
(``linear_q``, ``linear_k``, ``linear_v``, ``output_layer``, so a reference
``state_dict`` loads), same ``forward(x, attn_bias, edge_index, attn_type)``.
The three input projections run as ONE kernel that reads ``x`` once and writes q, k
and v in the ``[N, H, d]`` layout the attention kernels read; their backward is
one pass over the three output gradients for ``dx`` and all weight and bias
gradients (64 -> 64 features; two kernels for other widths) plus a small
fixed-order sum of per-workgroup partials.  With sparse attention and no bias
the whole module is one operator (``torch.ops.torchgt.multi_head_attention``).  At sequence-parallel size 1 the reference's
``DistributedAttentionNoMerge`` (gt_sp/layer.py:502-550) hands q, k, v to the local
attention unchanged, which is what ``dist_attn`` does here.
"""
import torch
import torch.nn as nn

from . import _ext, _lib
from .core_attention import CoreAttention
from .plan import GraphPlan, get_plan

_DT = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16}


class LinearFunction:
    """``(x W_0^T + b_0, ..., x W_{n-1}^T + b_{n-1})`` for n <= 3 weights of one shape:
    ``torch.ops.torchgt.linear`` (a C++ autograd function over ``tgt_linear_fwd`` / ``_bwd``).

    ``apply(x, W_0, b_0, W_1, b_1, ...)``; x ``[..., in]``, W_j ``[out, in]``, b_j
    ``[out]`` or None.  Returns a tuple of ``[..., out]`` tensors."""

    @staticmethod
    def apply(x, *wb):
        Ws, bs = list(wb[0::2]), list(wb[1::2])
        if not 1 <= len(Ws) <= 3 or len(bs) != len(Ws):
            raise ValueError("LinearFunction takes 1 to 3 (weight, bias) pairs")
        return tuple(_ext.ops().linear(x, Ws, bs))


def fused_linear(x, *layers):
    """Applies 1 to 3 ``nn.Linear`` layers of one shape to the same input in one pass.

    The kernels read rows in 16-byte pieces (feature widths that are multiples of 4 in fp32, 8 in
    bf16).  Other widths (47 classes, 100-d features in bf16) are zero-padded here with torch ops on
    the weights (and on x when its width does not fit) and the outputs sliced back; autograd sees
    the padding."""
    ve = 4 if x.dtype == torch.float32 else 8
    out_f, in_f = layers[0].weight.shape
    pad_in, pad_out = (-in_f) % ve, (-out_f) % ve
    if pad_in:
        x = torch.nn.functional.pad(x, (0, pad_in))
    args = []
    for layer in layers:
        W, b = layer.weight, layer.bias
        if pad_in or pad_out:
            W = torch.nn.functional.pad(W, (0, pad_in, 0, pad_out))
            b = None if b is None else torch.nn.functional.pad(b, (0, pad_out))
        args += [W, b]
    ys = LinearFunction.apply(x, *args)
    if pad_out:
        ys = tuple(y[..., :out_f] for y in ys)
    return ys


class _LocalAttention(nn.Module):
    """Stands where the reference puts ``DistributedAttentionNoMerge`` (one rank: identity)."""

    def __init__(self, local_attention):
        super().__init__()
        self.local_attn = local_attention

    def forward(self, query, key, value, attn_bias, edge_index, attn_type, *args):
        return self.local_attn(query, key, value, attn_bias, edge_index, attn_type, *args)


class MultiHeadAttention(nn.Module):
    """``MultiHeadAttention(hidden_size, attention_dropout_rate, num_heads, attn_bias_dim)``:
    the Graphormer flavour with an output layer (graphormer_dist_node_level.py:228-241).
    Without ``attn_bias_dim`` it is the GT flavour, which has none
    (gt_dist_node_level.py:173-184)."""

    def __init__(self, hidden_size, attention_dropout_rate, num_heads, attn_bias_dim=None):
        super().__init__()
        self.num_heads = num_heads
        self.att_size = att_size = hidden_size // num_heads
        self.linear_q = nn.Linear(hidden_size, num_heads * att_size)
        self.linear_k = nn.Linear(hidden_size, num_heads * att_size)
        self.linear_v = nn.Linear(hidden_size, num_heads * att_size)
        if attn_bias_dim is not None:
            local_attn = CoreAttention(hidden_size, attention_dropout_rate, num_heads, attn_bias_dim)
            self.output_layer = nn.Linear(num_heads * att_size, hidden_size)
        else:
            local_attn = CoreAttention(hidden_size, attention_dropout_rate, num_heads)
            self.output_layer = None
        self.dist_attn = _LocalAttention(local_attn)

    one_operator = True      # False: always run projections and attention operator by operator

    def _one_operator(self, x, attn_bias, edge_index, attn_type):
        """Whether ``torch.ops.torchgt.multi_head_attention`` covers this call: sparse attention without a bias, feature
        widths the kernels read without padding, every layer with its bias."""
        if not self.one_operator or attn_type != "sparse" or attn_bias is not None or edge_index is None or not x.is_cuda:
            return False
        ve = 4 if x.dtype == torch.float32 else 8
        layers = [self.linear_q, self.linear_k, self.linear_v] + ([] if self.output_layer is None else [self.output_layer])
        return all(l.bias is not None and l.in_features % ve == 0 and l.out_features % ve == 0 for l in layers)

    def forward(self, x, attn_bias=None, edge_index=None, attn_type=None):
        if self._one_operator(x, attn_bias, edge_index, attn_type):
            # projections, attention and output layer as one operator and one autograd node: the same kernels and
            # numbers, without the per-operator cost of dispatcher and autograd between the launches
            plan = edge_index if isinstance(edge_index, GraphPlan) else get_plan(edge_index, x.numel() // x.shape[-1])
            params = [self.linear_q.weight, self.linear_q.bias, self.linear_k.weight, self.linear_k.bias, self.linear_v.weight,
                      self.linear_v.bias]
            if self.output_layer is not None:
                params += [self.output_layer.weight, self.output_layer.bias]
            plan.handle      # raises if the plan was closed
            return _ext.ops().multi_head_attention(x, params, plan.holder, plan.workspace(self.num_heads, self.att_size), self.num_heads)
        batch_size = x.size(0)
        q, k, v = fused_linear(x, self.linear_q, self.linear_k, self.linear_v)
        q = q.view(batch_size, -1, self.num_heads, self.att_size)
        k = k.view(batch_size, -1, self.num_heads, self.att_size)
        v = v.view(batch_size, -1, self.num_heads, self.att_size)
        x = self.dist_attn(q, k, v, attn_bias, edge_index, attn_type)
        if self.output_layer is not None:
            (x,) = fused_linear(x, self.output_layer)
        return x
