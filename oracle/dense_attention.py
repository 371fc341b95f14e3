"""Oracle: dense biased attention for graph-level batches (test infrastructure).

Restates ``CoreAttention.forward`` of ``models/graphormer_graph_level.py:186-214``
(same body: ``attn_module.py:99-127``, ``graphormer_dist_graph_level.py:211-235``)
and the bias producer ``GraphAttnBias.forward``
(``models/graphormer_graph_level.py:94-156``, both edge-type branches).
"""
import math

import torch


def dense_attention(q, k, v, attn_bias=None, mask=None, drop_keep=None, p_drop=0.0):
    """q, k, v: [b, S, H, d]; attn_bias [b, H, S, S] (additive, -inf on padded
    keys); mask [b, S, S] bool or None.  NOTE the reference MULTIPLIES q by
    sqrt(d) (graphormer_graph_level.py:198).  ``att_dropout`` (:208) is the identity
    (eval / p = 0) unless ``drop_keep`` [b, H, S, S] (1 = kept) is given: torch's Dropout
    with that mask, i.e. kept probabilities times 1 / (1 - p_drop).  Returns [b, S, H*d]."""
    b, S, H, d = q.shape
    scale = math.sqrt(d)
    qt = q.transpose(1, 2)                      # :192  [b, H, S, d]
    vt = v.transpose(1, 2)                      # :193
    kt = k.transpose(1, 2).transpose(2, 3)      # :194  [b, H, d, S]
    qt = qt * scale                             # :198
    x = torch.matmul(qt, kt)                    # :199
    if attn_bias is not None:
        x = x + attn_bias                       # :202
    if mask is not None:
        x = x.masked_fill(mask.unsqueeze(1), 0)  # :204-205
    x = torch.softmax(x, dim=3)                 # :207
    if drop_keep is not None:
        x = x * drop_keep.to(x.dtype) / (1.0 - p_drop)   # :208 with the mask made explicit
    x = x.matmul(vt)                            # :209
    x = x.transpose(1, 2).contiguous()          # :211
    return x.view(b, S, -1)                     # :212


def graph_attn_bias(attn_bias, spatial_pos, attn_edge_type, spatial_table, edge_table, virtual_dist):
    """``GraphAttnBias.forward`` (graphormer_graph_level.py:94-156), simple
    edge-type branch (:150).

    attn_bias       [b, S+1, S+1] float (0 / -inf from the collator)
    spatial_pos     [b, S, S] int64   (shortest-path distance + 1, 0 = pad)
    attn_edge_type  [b, S, S, F] int64 (edge feature ids + 1, 0 = none)
    spatial_table   [num_spatial, H]  (row 0 = padding_idx, zeros)
    edge_table      [num_edges, H]    (row 0 = padding_idx, zeros)
    virtual_dist    [1, H]
    Returns [b, H, S+1, S+1].
    """
    H = spatial_table.shape[1]
    g = attn_bias.clone().unsqueeze(1).repeat(1, H, 1, 1)             # :104-107
    sp = spatial_table[spatial_pos].permute(0, 3, 1, 2)               # :110
    g[:, :, 1:, 1:] = g[:, :, 1:, 1:] + sp                            # :111
    t = virtual_dist.view(1, H, 1)                                    # :115
    g[:, :, 1:, 0] = g[:, :, 1:, 0] + t                               # :116
    g[:, :, 0, :] = g[:, :, 0, :] + t                                 # :117
    ei = edge_table[attn_edge_type].mean(-2).permute(0, 3, 1, 2)      # :150
    g[:, :, 1:, 1:] = g[:, :, 1:, 1:] + ei                            # :152
    g = g + attn_bias.unsqueeze(1)                                    # :153
    return g


def graph_attn_bias_multi_hop(attn_bias, spatial_pos, edge_input, spatial_table, edge_table, edge_dis_weight, virtual_dist,
                              multi_hop_max_dist):
    """``GraphAttnBias.forward`` (graphormer_graph_level.py:94-156), edge_type == 'multi_hop'
    (:119-147), op for op.

    edge_input       [b, S, S, D0, F] int64 (features of the edges on the shortest path + 1, 0 = none)
    edge_dis_weight  [num_edge_dis * H * H, 1] (the weight of ``edge_dis_encoder``)
    the other arguments as in ``graph_attn_bias``.  Returns [b, H, S+1, S+1].
    """
    H = spatial_table.shape[1]
    n_graph, n_node = spatial_pos.shape[:2]
    g = attn_bias.clone().unsqueeze(1).repeat(1, H, 1, 1)             # :104-107
    sp = spatial_table[spatial_pos].permute(0, 3, 1, 2)               # :110
    g[:, :, 1:, 1:] = g[:, :, 1:, 1:] + sp                            # :111
    t = virtual_dist.view(1, H, 1)                                    # :115
    g[:, :, 1:, 0] = g[:, :, 1:, 0] + t                               # :116
    g[:, :, 0, :] = g[:, :, 0, :] + t                                 # :117
    sp_ = spatial_pos.clone()                                         # :121
    sp_[sp_ == 0] = 1                                                 # :122
    sp_ = torch.where(sp_ > 1, sp_ - 1, sp_)                          # :124
    if multi_hop_max_dist > 0:
        sp_ = sp_.clamp(0, multi_hop_max_dist)                        # :126
        edge_input = edge_input[:, :, :, :multi_hop_max_dist, :]      # :127
    e = edge_table[edge_input].mean(-2)                               # :129  [b, S, S, D, H]
    max_dist = e.size(-2)
    flat = e.permute(3, 0, 1, 2, 4).reshape(max_dist, -1, H)          # :131-133
    flat = torch.bmm(flat, edge_dis_weight.reshape(-1, H, H)[:max_dist, :, :])     # :134-139
    e = flat.reshape(max_dist, n_graph, n_node, n_node, H).permute(1, 2, 3, 0, 4)  # :141-143
    e = (e.sum(-2) / (sp_.to(e.dtype).unsqueeze(-1))).permute(0, 3, 1, 2)          # :145-147
    g[:, :, 1:, 1:] = g[:, :, 1:, 1:] + e                             # :152
    g = g + attn_bias.unsqueeze(1)                                    # :153
    return g


def dense_attention_bruteforce(q, k, v, attn_bias=None):
    """fp64 loops from the definition; pins ``dense_attention`` on tiny inputs."""
    b, S, H, d = q.shape
    q, k, v = q.double(), k.double(), v.double()
    out = torch.zeros(b, S, H * d, dtype=torch.float64)
    for g in range(b):
        for h in range(H):
            for i in range(S):
                sc = torch.empty(S, dtype=torch.float64)
                for j in range(S):
                    sc[j] = (q[g, i, h] * math.sqrt(d) * k[g, j, h]).sum()
                    if attn_bias is not None:
                        sc[j] = sc[j] + float(attn_bias[g, h, i, j])
                m = sc.max()
                w = torch.exp(sc - m)
                out[g, i, h * d:(h + 1) * d] = (w.unsqueeze(1) * v[g, :, h]).sum(0) / w.sum()
    return out
