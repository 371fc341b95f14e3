"""``GraphAttnBias`` and ``floyd_warshall`` on the library's kernels.

Mirrors of models/graphormer_graph_level.py:63-156 (``GraphAttnBias``: same
constructor, same embedding parameter names, ``forward(batched_data)``) and of
data/algos.pyx:9-54 (``floyd_warshall``).  The bias is built by one kernel from
the id tensors and the three embedding tables; its backward reduces the bias
gradient into the tables.  ``edge_type='multi_hop'`` (the path-encoding branch,
:119-147) is not built and raises.
"""
import numpy as np
import torch
import torch.nn as nn

from . import _lib

_DT = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16}


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


class GraphAttnBiasFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, attn_bias, spatial_pos, attn_edge_type, spatial_table, edge_table, virtual_dist):
        if not attn_bias.is_cuda:
            raise RuntimeError("GraphAttnBias runs on the GPU only (no CPU fallback)")
        dt = spatial_table.dtype
        if dt not in _DT:
            raise TypeError(f"unsupported dtype {dt}")
        b, S1 = attn_bias.shape[0], attn_bias.shape[1]
        s, H, F = S1 - 1, spatial_table.shape[1], attn_edge_type.shape[-1]
        ab = attn_bias.to(dt).contiguous()
        sp = spatial_pos.to(torch.int64).contiguous()
        et = attn_edge_type.to(torch.int64).contiguous()
        st_, e_, v_ = spatial_table.contiguous(), edge_table.contiguous(), virtual_dist.reshape(-1).contiguous()
        out = torch.empty((b, H, S1, S1), dtype=dt, device=ab.device)
        with torch.cuda.device(ab.device):
            _lib.check(_lib.lib().tgt_graph_attn_bias_fwd(ab.data_ptr(), sp.data_ptr(), et.data_ptr(), F, st_.data_ptr(),
                                                          st_.shape[0], e_.data_ptr(), e_.shape[0], v_.data_ptr(), b, s, H,
                                                          _DT[dt], out.data_ptr(), _stream(ab)))
        ctx.save_for_backward(sp, et)
        ctx.dims = (b, s, H, F, st_.shape[0], e_.shape[0], dt, virtual_dist.shape)
        return out

    @staticmethod
    def backward(ctx, dout):
        sp, et = ctx.saved_tensors
        b, s, H, F, ns, ne, dt, vshape = ctx.dims
        L = _lib.lib()
        dout = dout.to(dt).contiguous()
        d_sp = torch.empty((ns, H), dtype=dt, device=dout.device)
        d_e = torch.empty((ne, H), dtype=dt, device=dout.device)
        d_v = torch.empty(H, dtype=dt, device=dout.device)
        nbytes = L.tgt_graph_attn_bias_bwd_workspace_bytes(ns, ne, H)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dout.device)
        with torch.cuda.device(dout.device):
            _lib.check(L.tgt_graph_attn_bias_bwd(dout.data_ptr(), sp.data_ptr(), et.data_ptr(), F, ns, ne, b, s, H, _DT[dt],
                                                 d_sp.data_ptr(), d_e.data_ptr(), d_v.data_ptr(), ws.data_ptr(), nbytes,
                                                 _stream(dout)))
        return None, None, None, d_sp, d_e, d_v.view(vshape)


class GraphAttnBias(nn.Module):
    """Attention bias for each head, global token at index 0 (graphormer_graph_level.py:63-156)."""

    def __init__(self, num_heads, num_atoms, num_edges, num_spatial, num_edge_dis, hidden_dim, edge_type,
                 multi_hop_max_dist):
        super().__init__()
        self.num_heads = num_heads
        self.multi_hop_max_dist = multi_hop_max_dist
        self.edge_type = edge_type
        self.edge_encoder = nn.Embedding(num_edges, num_heads, padding_idx=0)
        if self.edge_type == "multi_hop":
            self.edge_dis_encoder = nn.Embedding(num_edge_dis * num_heads * num_heads, 1)
        self.spatial_pos_encoder = nn.Embedding(num_spatial, num_heads, padding_idx=0)
        self.graph_token_virtual_distance = nn.Embedding(1, num_heads)

    def forward(self, batched_data):
        if self.edge_type == "multi_hop":
            raise NotImplementedError("the multi_hop edge encoding (graphormer_graph_level.py:119-147) is not built")
        return GraphAttnBiasFunction.apply(batched_data.attn_bias, batched_data.spatial_pos, batched_data.attn_edge_type,
                                           self.spatial_pos_encoder.weight, self.edge_encoder.weight,
                                           self.graph_token_virtual_distance.weight)


def floyd_warshall(adjacency_matrix, n_nodes=None):
    """``floyd_warshall`` of data/algos.pyx:9-54 on the GPU.

    ``adjacency_matrix``: [n, n] (one graph, as in the reference) or [B, n_max, n_max] (a padded batch with
    ``n_nodes`` [B]); numpy array or tensor, entries = edge weights 0..255, 0 = no edge.  Returns
    ``(dist, path)`` as int64 arrays / tensors of the input's kind and shape (padding entries are 0)."""
    is_np = isinstance(adjacency_matrix, np.ndarray)
    adj = torch.as_tensor(adjacency_matrix)
    single = adj.dim() == 2
    if single:
        adj = adj.unsqueeze(0)
    if not torch.cuda.is_available():
        raise RuntimeError("floyd_warshall runs on the GPU only (no CPU fallback)")
    dev = adj.device if adj.is_cuda else torch.device("cuda:0")
    a8 = adj.to(device=dev, dtype=torch.uint8).contiguous()
    B, n_max = a8.shape[0], a8.shape[1]
    nn_ = None if n_nodes is None else torch.as_tensor(n_nodes).to(device=dev, dtype=torch.int32).contiguous()
    dist = torch.zeros((B, n_max, n_max), dtype=torch.int32, device=dev)
    path = torch.zeros((B, n_max, n_max), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().tgt_floyd_warshall(a8.data_ptr(), None if nn_ is None else nn_.data_ptr(), B, n_max,
                                                 dist.data_ptr(), path.data_ptr(), torch.cuda.current_stream(dev).cuda_stream))
    dist, path = dist.long(), path.long()
    if single:
        dist, path = dist[0], path[0]
    if is_np:
        return dist.cpu().numpy(), path.cpu().numpy()
    return dist, path
