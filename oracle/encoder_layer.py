"""Oracle: the encoder layer and the node-level Graphormer forward (test
infrastructure, CPU, float64).

Restates, in plain numpy on top of ``oracle.projections`` and
``oracle.sparse_attention``:

* ``nn.LayerNorm`` (biased variance over the last axis, eps inside the root);
* ``nn.GELU()`` exact form ``0.5 x (1 + erf(x / sqrt 2))``
  (``FeedForwardNetwork``, models/graphormer_dist_node_level.py:27-39);
* ``EncoderLayer.forward`` (:296-314) with dropout rate 0:
  ``x = x + MHA(LN1(x)); x = x + FFN(LN2(x))``;
* ``Graphormer.forward`` (:355-392) without a dense bias: node encoder, global
  token row 0, the layers, final LayerNorm, output projection of rows 1.., and
  ``log_softmax``.

* ``F.nll_loss`` of the training loop (main_sp_sparse_node_level.py:200), reduction 'mean' with ``ignore_index``.

Pinned in ``tests/test_oracle_encoder.py`` against ``torch.nn.functional.layer_norm``
and ``gelu`` (independent library routines), closed forms (constant rows, the GELU
reflection identity ``gelu(x) - gelu(-x) = x``, a layer with zero attention/FFN
output weights is the identity) and the parameter counts of README.md:70,114; ``nll_loss`` against torch's CPU
``F.nll_loss`` and the closed form log C of a uniform prediction.
"""
import math

import numpy as np

from . import projections as _proj


def layer_norm(x, gamma, beta, eps=1e-5):
    x = np.asarray(x, np.float64)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * np.asarray(gamma, np.float64) + np.asarray(beta, np.float64)


_erf = np.vectorize(math.erf, otypes=[np.float64])


def gelu(x):
    x = np.asarray(x, np.float64)
    return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))


def ffn_forward(x, params, prefix="ffn."):
    u = _proj.linear_forward(x, params[prefix + "layer1.weight"], params[prefix + "layer1.bias"])
    return _proj.linear_forward(gelu(u), params[prefix + "layer2.weight"], params[prefix + "layer2.bias"])


def _sub(params, prefix):
    return {k[len(prefix):]: v for k, v in params.items() if k.startswith(prefix)}


def encoder_layer_forward(x, params, edge_index, num_heads, edge_bias=None):
    """x: [b, S, hidden]; params: the layer's ``state_dict`` as float arrays."""
    x = np.asarray(x, np.float64)
    b, S, hidden = x.shape
    y = layer_norm(x, params["self_attention_norm.weight"], params["self_attention_norm.bias"])      # :302
    y = _proj.multi_head_attention_forward(y, _sub(params, "self_attention."), edge_index, num_heads, edge_bias)
    x = x + y                                                                                        # :305
    y = layer_norm(x, params["ffn_norm.weight"], params["ffn_norm.bias"])                            # :311
    y = ffn_forward(y.reshape(b * S, hidden), params).reshape(b, S, hidden)
    return x + y                                                                                     # :314


def graphormer_forward(x, params, edge_index, n_layers, num_heads):
    """x: [S, input_dim] -> log-probabilities [S, output_dim] (attn_bias=None, perturb=None)."""
    h = _proj.linear_forward(x, params["node_encoder.weight"], params["node_encoder.bias"])          # :361
    h = np.concatenate([np.asarray(params["graph_token.weight"], np.float64), h], axis=0)[None]      # :367-369
    for i in range(n_layers):
        h = encoder_layer_forward(h, _sub(params, f"layers.{i}."), edge_index, num_heads)
    h = layer_norm(h, params["final_ln.weight"], params["final_ln.bias"])
    out = _proj.linear_forward(h[0, 1:, :], params["downstream_out_proj.weight"], params["downstream_out_proj.bias"])
    out = out - out.max(axis=1, keepdims=True)
    return out - np.log(np.exp(out).sum(axis=1, keepdims=True))                                      # log_softmax


def nll_loss(log_probs, target, ignore_index=-100):
    """``F.nll_loss(log_probs, target)`` (main_sp_sparse_node_level.py:200): minus the mean, over the rows whose
    target is not ``ignore_index``, of the log-probability of the target class.  Returns (loss, d loss / d log_probs)."""
    lp = np.asarray(log_probs, np.float64)
    t = np.asarray(target, np.int64)
    rows = np.nonzero(t != ignore_index)[0]
    grad = np.zeros_like(lp)
    if rows.size == 0:
        return float("nan"), grad
    loss = -lp[rows, t[rows]].sum() / rows.size
    grad[rows, t[rows]] = -1.0 / rows.size
    return float(loss), grad
