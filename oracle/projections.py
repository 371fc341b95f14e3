"""Oracle: the projections of ``MultiHeadAttention`` and the module's forward
(test infrastructure, CPU, numpy float64 + the sparse-attention oracle).

Restates, for the one-GPU case (sequence-parallel size 1, where
``DistributedAttentionNoMerge.forward`` hands q, k, v to the local attention
unchanged: ``gt_sp/layer.py:514-550`` with an all-to-all over one rank):

* ``nn.Linear`` as used by ``linear_q / linear_k / linear_v / output_layer``
  (``models/graphormer_dist_node_level.py:233-241``): ``y = x W^T + b`` with
  ``W`` of shape ``[out_features, in_features]``;
* its autograd backward: ``dx = dy W``, ``dW = dy^T x``, ``db = sum_rows dy``;
* ``MultiHeadAttention.forward`` (``:246-273``): q, k, v = three linears of the
  same x viewed ``[b, S, H, d]``, sparse attention, output linear.

Pinned in ``tests/test_oracle_projections.py`` against
``torch.nn.functional.linear`` + autograd (an independent library routine) and
against a closed form of the whole module (zero query weights make every edge
weigh the same, so each node's output is the output projection of the mean of
its neighbours' value rows).
"""
import numpy as np
import torch

from . import sparse_attention as _sa


def linear_forward(x, W, b=None):
    """x [N, in], W [out, in], b [out] -> [N, out]  (float64)."""
    y = np.einsum("ni,oi->no", np.asarray(x, np.float64), np.asarray(W, np.float64))
    if b is not None:
        y = y + np.asarray(b, np.float64)[None, :]
    return y


def linear_backward(x, W, dy):
    """Gradients of ``linear_forward`` for the upstream gradient dy [N, out]:
    (dx [N, in], dW [out, in], db [out])."""
    x = np.asarray(x, np.float64)
    W = np.asarray(W, np.float64)
    dy = np.asarray(dy, np.float64)
    dx = np.einsum("no,oi->ni", dy, W)
    dW = np.einsum("no,ni->oi", dy, x)
    db = dy.sum(axis=0)
    return dx, dW, db


def multi_head_attention_forward(x, params, edge_index, num_heads, edge_bias=None):
    """``MultiHeadAttention.forward`` with ``attn_type='sparse'``.

    x: [b, S, hidden] array; params: dict with ``linear_q.weight`` ... as in the
    module's ``state_dict`` (``output_layer.*`` optional: the GT flavour,
    ``models/gt_dist_node_level.py:173-184``, has none); edge_index [2, E] over the
    flattened b*S axis.  Returns [b, S, hidden] float64.
    """
    x = np.asarray(x, np.float64)
    b, S, hidden = x.shape
    x2 = x.reshape(b * S, hidden)
    d = params["linear_q.weight"].shape[0] // num_heads

    def proj(name):
        y = linear_forward(x2, params[name + ".weight"], params.get(name + ".bias"))
        return torch.from_numpy(y).view(b, S, num_heads, d)          # :255-257

    q, k, v = proj("linear_q"), proj("linear_k"), proj("linear_v")
    eb = None if edge_bias is None else torch.as_tensor(np.asarray(edge_bias, np.float64))
    out, _ = _sa.sparse_attention(q, k, v, torch.as_tensor(np.asarray(edge_index)), eb)
    y = out.reshape(b * S, num_heads * d).numpy()
    if "output_layer.weight" in params:                              # :271
        y = linear_forward(y, params["output_layer.weight"], params.get("output_layer.bias"))
    return y.reshape(b, S, -1)
