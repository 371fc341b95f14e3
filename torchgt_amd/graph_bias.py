"""``GraphAttnBias``, ``floyd_warshall`` and ``gen_edge_input`` on the library's kernels.

Mirrors of models/graphormer_graph_level.py:63-156 (``GraphAttnBias``: same
constructor, same embedding parameter names, ``forward(batched_data)``) and of
data/algos.pyx:9-54 (``floyd_warshall``) and :64-92 (``gen_edge_input``).  The
bias is built by one kernel from the id tensors and the embedding tables; its
backward reduces the bias gradient into the tables.  Both edge-type branches are
built: the plain one (mean of the edge-type embeddings, :148-150) and
``edge_type='multi_hop'`` (embeddings of the edges along the shortest path, one
H x H matrix per hop, :119-147).
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


class GraphAttnBiasMultiHopFunction(torch.autograd.Function):
    """The 'multi_hop' branch (graphormer_graph_level.py:119-147) with gradients for the four parameter tensors."""

    @staticmethod
    def forward(ctx, attn_bias, spatial_pos, edge_input, spatial_table, edge_table, edge_dis_weight, virtual_dist,
                multi_hop_max_dist):
        if not attn_bias.is_cuda:
            raise RuntimeError("GraphAttnBias runs on the GPU only (no CPU fallback)")
        dt = spatial_table.dtype
        if dt not in _DT:
            raise TypeError(f"unsupported dtype {dt}")
        b, S1 = attn_bias.shape[0], attn_bias.shape[1]
        s, H = S1 - 1, spatial_table.shape[1]
        D0, F = edge_input.shape[-2], edge_input.shape[-1]
        mhd = int(multi_hop_max_dist)
        ab = attn_bias.to(dt).contiguous()
        sp = spatial_pos.to(torch.int64).contiguous()
        ei = edge_input.to(torch.int64).contiguous()
        st_, e_, v_ = spatial_table.contiguous(), edge_table.contiguous(), virtual_dist.reshape(-1).contiguous()
        w_ = edge_dis_weight.to(dt).reshape(-1).contiguous()
        n_dis = w_.numel() // (H * H)
        out = torch.empty((b, H, S1, S1), dtype=dt, device=ab.device)
        with torch.cuda.device(ab.device):
            _lib.check(_lib.lib().tgt_graph_attn_bias_multi_hop_fwd(
                ab.data_ptr(), sp.data_ptr(), ei.data_ptr(), D0, F, st_.data_ptr(), st_.shape[0], e_.data_ptr(), e_.shape[0],
                w_.data_ptr(), n_dis, v_.data_ptr(), mhd, b, s, H, _DT[dt], out.data_ptr(), _stream(ab)))
        ctx.save_for_backward(sp, ei, e_, w_)
        ctx.dims = (b, s, H, F, D0, st_.shape[0], e_.shape[0], n_dis, mhd, dt, virtual_dist.shape, edge_dis_weight.shape)
        return out

    @staticmethod
    def backward(ctx, dout):
        sp, ei, e_, w_ = ctx.saved_tensors
        b, s, H, F, D0, ns, ne, n_dis, mhd, dt, vshape, wshape = ctx.dims
        L = _lib.lib()
        dout = dout.to(dt).contiguous()
        dev = dout.device
        d_sp = torch.empty((ns, H), dtype=dt, device=dev)
        d_e = torch.empty((ne, H), dtype=dt, device=dev)
        d_w = torch.empty(n_dis * H * H, dtype=dt, device=dev)
        d_v = torch.empty(H, dtype=dt, device=dev)
        D = min(D0, mhd) if mhd > 0 else D0
        nbytes = L.tgt_graph_attn_bias_multi_hop_bwd_workspace_bytes(ns, ne, H, D)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            _lib.check(L.tgt_graph_attn_bias_multi_hop_bwd(
                dout.data_ptr(), sp.data_ptr(), ei.data_ptr(), D0, F, e_.data_ptr(), ns, ne, w_.data_ptr(), n_dis, mhd, b, s, H,
                _DT[dt], d_sp.data_ptr(), d_e.data_ptr(), d_w.data_ptr(), d_v.data_ptr(), ws.data_ptr(), nbytes, _stream(dout)))
        return None, None, None, d_sp, d_e, d_w.view(wshape), d_v.view(vshape), None


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

    def forward(self, batched_data, as_ids=False):
        """The [b, H, S, S] bias; with ``as_ids=True`` (plain edge-type branch only) a ``GraphBiasIds`` that the dense
        attention takes in its place and that builds the tensor only if a layer needs it."""
        if as_ids and self.edge_type != "multi_hop":
            from . import _ext
            from .core_attention import GraphBiasIds
            sp_w, e_w, vd_w = self.spatial_pos_encoder.weight, self.edge_encoder.weight, self.graph_token_virtual_distance.weight
            if not batched_data.attn_bias.is_cuda:
                raise RuntimeError("GraphAttnBias runs on the GPU only (no CPU fallback)")
            sp16, et16 = _ext.ops().dense_ids_pack(batched_data.spatial_pos, batched_data.attn_edge_type, sp_w.shape[0], e_w.shape[0])
            build = lambda: GraphAttnBiasFunction.apply(batched_data.attn_bias, batched_data.spatial_pos,
                                                        batched_data.attn_edge_type, sp_w, e_w, vd_w)
            return GraphBiasIds(batched_data.attn_bias, sp16, et16, sp_w, e_w, vd_w, build)
        if self.edge_type == "multi_hop":
            return GraphAttnBiasMultiHopFunction.apply(batched_data.attn_bias, batched_data.spatial_pos, batched_data.edge_input,
                                                       self.spatial_pos_encoder.weight, self.edge_encoder.weight,
                                                       self.edge_dis_encoder.weight, self.graph_token_virtual_distance.weight,
                                                       self.multi_hop_max_dist)
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


def gen_edge_input(max_dist, path, edge_feat, n_nodes=None):
    """``gen_edge_input`` of data/algos.pyx:64-92 on the GPU.

    ``path``: [n, n] (one graph, as in the reference) or [B, n_max, n_max] with ``n_nodes`` [B], as
    ``floyd_warshall`` returns it; ``edge_feat``: [n, n, F] / [B, n_max, n_max, F] integer features of the
    direct edges; numpy arrays or tensors.  Returns int64 [..., max_dist, F] of the input's kind: the
    features of the edges along the recorded shortest path of every pair, -1 where there is none."""
    is_np = isinstance(path, np.ndarray)
    pt = torch.as_tensor(path)
    ft = torch.as_tensor(edge_feat)
    single = pt.dim() == 2
    if single:
        pt, ft = pt.unsqueeze(0), ft.unsqueeze(0)
    if not torch.cuda.is_available():
        raise RuntimeError("gen_edge_input runs on the GPU only (no CPU fallback)")
    dev = pt.device if pt.is_cuda else torch.device("cuda:0")
    B, n_max = pt.shape[0], pt.shape[1]
    if ft.shape[:3] != (B, n_max, n_max):
        raise ValueError(f"edge_feat {tuple(ft.shape)} does not match path {tuple(pt.shape)}")
    F = ft.shape[3]
    p32 = pt.to(device=dev, dtype=torch.int32).contiguous()
    f64 = ft.to(device=dev, dtype=torch.int64).contiguous()
    nn_ = None if n_nodes is None else torch.as_tensor(n_nodes).to(device=dev, dtype=torch.int32).contiguous()
    max_dist = int(max_dist)
    out = torch.empty((B, n_max, n_max, max_dist, F), dtype=torch.int64, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().tgt_gen_edge_input(p32.data_ptr(), f64.data_ptr(), 1, F, None if nn_ is None else nn_.data_ptr(),
                                                 B, n_max, max_dist, out.data_ptr(),
                                                 torch.cuda.current_stream(dev).cuda_stream))
    if single:
        out = out[0]
    return out.cpu().numpy() if is_np else out
