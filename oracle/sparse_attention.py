"""Oracle: topology-aware sparse attention (test infrastructure, CPU, plain torch).

Op-for-op restatement of the reference's ``CoreAttention.sparse_attention`` /
``sparse_attention_bias``:

* ``attn_module.py:133-189``                        (canonical, no bias in shipped runs)
* ``models/graphormer_dist_graph_level.py:238-292`` (the shape-correct bias add)
* ``models/graphormer_dist_node_level.py:69-127``   (k-first argument order)

``torch_scatter.scatter(src, index, dim=0, out=out, reduce='add')``
(``attn_module.py:180,185``; torch-scatter 2.1.1, absent here) is
``out.index_add_(0, index, src)``; that is the only third-party arithmetic on
the path.

The gradients are those of torch autograd through this restatement, which is
what the reference uses.  ``sparse_attention_backward_analytic`` states the
closed-form gradients the HIP kernels implement; tests check it against
autograd in fp64.
"""
import math

import torch

EPS = 1e-6       # attn_module.py:187
CLAMP = 5.0      # attn_module.py:155


def sparse_attention(q, k, v, edge_index, edge_bias=None):
    """q, k, v: [b, S, H, d] (or [b*S, H, d]); edge_index int64 [2, E] with
    row 0 = source (key/value node) and row 1 = destination (query node) over
    the flattened b*S axis; edge_bias: None, [E, H] or [E] / [E, 1] (one scalar
    per edge broadcast over heads, the ``repeat(1,1,1,num_heads)`` of
    ``graphormer_dist_node_level.py:384``).

    Returns (out [b*S, H, d], Z [b*S, H]).
    """
    H, d = q.shape[-2], q.shape[-1]
    scale = math.sqrt(d)                                  # attn_module.py:94
    q = q.reshape(-1, H, d)                               # :141-143
    k = k.reshape(-1, H, d)
    v = v.reshape(-1, H, d)
    src_idx = edge_index[0].to(torch.long)
    dst_idx = edge_index[1].to(torch.long)
    src = k[src_idx]                                      # :146
    dest = q[dst_idx]                                     # :147
    score = torch.mul(src, dest)                          # :148
    score = score / scale                                 # :151  (divide BEFORE the sum)
    score = score.sum(-1, keepdim=True).clamp(-CLAMP, CLAMP)   # :155
    if edge_bias is not None:                             # graphormer_dist_graph_level.py:262-267
        eb = edge_bias
        if eb.dim() == 1:
            eb = eb.unsqueeze(1)
        if eb.shape[1] == 1:
            eb = eb.expand(-1, H)
        score = score + eb.unsqueeze(2)                   # bias is added AFTER the clamp
    score = torch.exp(score)                              # :168 (no max subtraction)
    msg = v[src_idx] * score                              # :173
    wV = torch.zeros_like(v)                              # :179
    wV.index_add_(0, dst_idx, msg)                        # :180
    Z = score.new_zeros(v.size(0), H, 1)                  # :184
    Z.index_add_(0, dst_idx, score)                       # :185
    x = wV / (Z + EPS)                                    # :187
    return x, Z.squeeze(-1)


def dense_bias_to_edge_bias(attn_bias, edge_index, layout="bhss"):
    """The reference passes a dense bias and gathers it per edge as
    ``bias[src, dst, h]`` (``graphormer_dist_graph_level.py:262-267``: permute
    [b,H,S,S] -> [b,S,S,H], tile over the batch, view [b*S, b*S, H], index
    [edge_index[0], edge_index[1]]).  Flattened node id n = g*S + s; the tiling
    ``unsqueeze(2).repeat(1,1,b,1,1)`` makes entry [g*S+s, g2*S+t] equal to
    bias[g, s, t] for every g2.

    layout "bhss": attn_bias [b, H, S, S] (graph-level); "bssh": [b, S, S, H]
    (node-level, ``graphormer_dist_node_level.py:100-106``).
    Returns [E, H].
    """
    if layout == "bhss":
        attn_bias = attn_bias.permute(0, 2, 3, 1)
    b, S = attn_bias.shape[0], attn_bias.shape[1]
    src = edge_index[0].to(torch.long)
    dst = edge_index[1].to(torch.long)
    g, s = src // S, src % S
    t = dst % S
    return attn_bias[g, s, t, :]


def sparse_attention_module_forward(q, k, v, attn_bias=None, edge_index=None, layout="bhss"):
    """``CoreAttention.forward(..., attn_type='sparse')``
    (``models/graphormer_dist_node_level.py:199-221``): output viewed as
    [b, S, H*d]."""
    b, S = q.shape[0], q.shape[1]
    eb = None
    if attn_bias is not None:
        eb = attn_bias if attn_bias.dim() <= 2 else dense_bias_to_edge_bias(attn_bias, edge_index, layout)
    x, _ = sparse_attention(q, k, v, edge_index, eb)
    return x.view(b, S, -1)


def sparse_attention_backward_analytic(q, k, v, edge_index, edge_bias, out, Z, dout):
    """Closed-form gradients of ``sparse_attention`` (what the HIP backward
    computes).  With g = dout, Ze = Z + EPS, D_i[h] = sum_c g_i[h,c] out_i[h,c]:

        w_e   = exp(clamp(raw_e) + bias_e),  raw_e = sum_c k_src q_dst / sqrt(d)
        dV_j  = sum_{e: src=j} w_e g_dst / Ze_dst
        dS_e  = w_e (g_dst . v_src - D_dst) / Ze_dst          (= dBias_e)
        m_e   = 1[-5 <= raw_e <= 5]                            (torch clamp backward)
        dQ_i  = sum_{e: dst=i} m_e dS_e k_src / sqrt(d)
        dK_j  = sum_{e: src=j} m_e dS_e q_dst / sqrt(d)

    Returns (dq, dk, dv, dbias [E, H]).
    """
    H, d = q.shape[-2], q.shape[-1]
    scale = math.sqrt(d)
    q = q.reshape(-1, H, d)
    k = k.reshape(-1, H, d)
    v = v.reshape(-1, H, d)
    g = dout.reshape(-1, H, d)
    o = out.reshape(-1, H, d)
    src = edge_index[0].to(torch.long)
    dst = edge_index[1].to(torch.long)
    raw = (k[src] * q[dst] / scale).sum(-1)                       # [E, H]
    s = raw.clamp(-CLAMP, CLAMP)
    if edge_bias is not None:
        eb = edge_bias if edge_bias.dim() == 2 else edge_bias.unsqueeze(1)
        s = s + eb
    w = torch.exp(s)
    rZ = 1.0 / (Z.reshape(-1, H) + EPS)
    D = (g * o).sum(-1)                                           # [N, H]
    p = w * rZ[dst]
    dv = torch.zeros_like(v).index_add_(0, src, p.unsqueeze(-1) * g[dst])
    dS = p * ((g[dst] * v[src]).sum(-1) - D[dst])
    m = ((raw >= -CLAMP) & (raw <= CLAMP)).to(dS.dtype)
    mdS = (m * dS).unsqueeze(-1)
    dq = torch.zeros_like(q).index_add_(0, dst, mdS * k[src] / scale)
    dk = torch.zeros_like(k).index_add_(0, src, mdS * q[dst] / scale)
    return dq, dk, dv, dS


def sparse_attention_bruteforce(q, k, v, edge_index, edge_bias=None):
    """Per-destination Python loops in fp64 straight from the definition
    (exp-weighted average of neighbour values).  Used only to pin
    ``sparse_attention`` on tiny graphs."""
    H, d = q.shape[-2], q.shape[-1]
    q = q.reshape(-1, H, d).double()
    k = k.reshape(-1, H, d).double()
    v = v.reshape(-1, H, d).double()
    N = q.shape[0]
    out = torch.zeros(N, H, d, dtype=torch.float64)
    E = edge_index.shape[1]
    for i in range(N):
        for h in range(H):
            num = torch.zeros(d, dtype=torch.float64)
            den = 0.0
            for e in range(E):
                if int(edge_index[1, e]) != i:
                    continue
                j = int(edge_index[0, e])
                raw = float((k[j, h] * q[i, h]).sum()) / math.sqrt(d)
                raw = max(-CLAMP, min(CLAMP, raw))
                if edge_bias is not None:
                    eb = edge_bias[e]
                    raw = raw + float(eb[h] if eb.dim() > 0 and eb.numel() > 1 else eb)
                w = math.exp(raw) if raw != float("-inf") else 0.0
                num += w * v[j, h]
                den += w
            out[i, h] = num / (den + EPS)
    return out
