"""Host-side mirror of the reference's edge construction helpers, backed by the
GPU kernels of csrc/graph_prep.hip (no CPU implementation).

  fix_edge_index(x, num_node)                       gt_sp/utils.py:34-50
  gen_sub_edge_index(edge_index, idx_batch, N)      gt_sp/utils.py:202-215
  prepare_batch(...)                                gt_sp/utils.py:409-520 at sequence-parallel size 1
  adjust_edge_index_nomerge(edge_index, L)          gt_sp/utils.py:53-58
  reformat_graph(edge_index, k, block_size, ...)    gt_sp/utils.py:319-359
"""
import ctypes

import torch

from . import _lib


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


def fix_edge_index(x, num_node):
    """Add the global node 0 and its 2*num_node edges.  x: int64 [2, E0] CUDA tensor."""
    if not x.is_cuda:
        raise RuntimeError("fix_edge_index needs a GPU tensor (no CPU implementation)")
    x = x.to(torch.int64).contiguous()
    out = torch.empty((2, x.size(1) + 2 * num_node), dtype=torch.int64, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().tgt_fix_edge_index(x.data_ptr() if x.numel() else None, x.size(1), num_node,
                                                 out.data_ptr(), _stream(x.device)))
    return out


def gen_sub_edge_index(edge_index, idx_batch, N):
    """Edges among the nodes of ``idx_batch`` (int64 [S]), renamed to batch positions, with the
    self-loops of the input dropped and one self-loop per batch node appended - the result of the
    reference's remove_self_loops / add_self_loops / subgraph(relabel_nodes=True) chain, in the
    same order.  edge_index: int64 [2, E] CUDA tensor over nodes 0..N-1."""
    if not edge_index.is_cuda:
        raise RuntimeError("gen_sub_edge_index needs GPU tensors (no CPU implementation)")
    dev = edge_index.device
    ei = edge_index.to(torch.int64).contiguous()
    idx = idx_batch.to(device=dev, dtype=torch.int64).contiguous()
    E, S = ei.size(1), idx.numel()
    cap = E + min(S, N)
    out = torch.empty((2, cap), dtype=torch.int64, device=dev)
    n = ctypes.c_int64()
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().tgt_sub_edge_index(ei.data_ptr() if E else None, E, N, idx.data_ptr() if S else None, S,
                                                 out.data_ptr() if cap else None, cap, ctypes.byref(n), _stream(dev)))
    return out[:, :n.value].contiguous()


def adjust_edge_index_nomerge(edge_index, sub_seq_len):
    """idx + (idx-1)//L for idx > 0: the shift that leaves room for every rank's copy of the
    global token; the identity at sequence-parallel size 1 (every idx <= L)."""
    shift = torch.div(edge_index - 1, sub_seq_len, rounding_mode="floor")
    return torch.where(edge_index > 0, edge_index + shift, edge_index)


def reformat_graph(edge_index, k, block_size, beta_coeffi="1", partition_ids=None, blockize=True,
                   return_tiles=False):
    """Relabel nodes by partition, (optionally) replace the edges of every partition pair by
    random dense blocks, and stably sort the edges by source.  Same return value as the
    reference: (sorted_edge_index [2, E'], sorted_indices [N]).

    The reference obtains ``partition_ids`` from dgl's METIS binding, which does not exist
    here; they must be passed in (int64 [N], values in [0, k)).  ``beta_coeffi`` is accepted
    and ignored, as in the reference (p is overwritten with 1, gt_sp/utils.py:344).

    ``return_tiles=True`` additionally returns the emitted blocks as a tile list (numpy int32
    [T, 2], first source / first destination in new ids) and the edges that were kept as they
    are (int64 [2, E_raw]), the inputs of ``torchgt_amd.block_attention``."""
    if partition_ids is None:
        raise ValueError("reformat_graph: partition_ids must be given (METIS is not available)")
    if not edge_index.is_cuda:
        raise RuntimeError("reformat_graph needs GPU tensors (no CPU implementation)")
    dev = edge_index.device
    ei = edge_index.to(torch.int64).contiguous()
    part = partition_ids.to(device=dev, dtype=torch.int64).contiguous()
    N, E = part.numel(), ei.size(1)
    L = _lib.lib()
    handle = ctypes.c_void_p()
    with torch.cuda.device(dev):
        st = _stream(dev)
        _lib.check(L.tgt_reformat_create(ei[0].data_ptr() if E else None, ei[1].data_ptr() if E else None, E, N,
                                         part.data_ptr(), int(k), int(block_size), 1 if blockize else 0, st,
                                         ctypes.byref(handle)))
        try:
            E_out = L.tgt_reformat_num_edges(handle)
            out = torch.empty((2, E_out), dtype=torch.int64, device=dev)
            sorted_indices = torch.empty(N, dtype=torch.int64, device=dev)
            _lib.check(L.tgt_reformat_export(handle, out.data_ptr() if E_out else None,
                                             sorted_indices.data_ptr(), st))
            tiles = raw = None
            if return_tiles:
                import numpy as np
                T, E_raw = L.tgt_reformat_num_tiles(handle), L.tgt_reformat_num_raw_edges(handle)
                tiles = np.empty((T, 2), dtype=np.int32)
                raw = torch.empty((2, E_raw), dtype=torch.int64, device=dev)
                _lib.check(L.tgt_reformat_export_tiles(handle, tiles.ctypes.data_as(ctypes.c_void_p) if T else None,
                                                       raw.data_ptr() if E_raw else None, st))
            torch.cuda.current_stream(dev).synchronize()
        finally:
            L.tgt_reformat_destroy(handle)
    if return_tiles:
        return out, sorted_indices, tiles, raw
    return out, sorted_indices


def prepare_batch(x, y, idx_batch, edge_index, N, k, block_size, partition, model="graphormer", reorder=True,
                  blockize=True, return_tiles=False):
    """``get_batch_reorder_blockize`` (gt_sp/utils.py:409-520) for one rank: features and labels
    of the batch nodes, their sub-graph (``gen_sub_edge_index``), the global node for
    ``model='graphormer'`` (``fix_edge_index``), the cluster reordering (``reformat_graph``) with
    x and y permuted to match (:463-472), and ``adjust_edge_index_nomerge`` (the identity on one
    rank).  Everything stays on the GPU.

    ``partition``: int64 [n_sub] cluster ids of the sub-graph's nodes, or a callable
    ``partition(edge_index_sub, n_sub, k) -> ids`` (the reference calls METIS on every batch's
    sub-graph, :326).  Returns (x_i, y_i, edge_index_i, attn_bias=None) like the reference, plus
    (tiles, raw_edge_index) when ``return_tiles``."""
    idx_batch = idx_batch.to(edge_index.device)
    x_i, y_i = x[idx_batch], y[idx_batch]
    S = idx_batch.shape[0]
    ei = gen_sub_edge_index(edge_index, idx_batch, N)
    n_sub = S
    if model == "graphormer":
        ei = fix_edge_index(ei, S)
        n_sub = S + 1
    extra = ()
    if reorder:
        part = partition(ei, n_sub, k) if callable(partition) else partition
        if part.numel() != n_sub:
            raise ValueError(f"partition ids for {part.numel()} nodes, the sub-graph has {n_sub}")
        res = reformat_graph(ei, k, block_size, partition_ids=part, blockize=blockize, return_tiles=return_tiles)
        ei, sorted_indices = res[0], res[1]
        extra = tuple(res[2:])
        if model == "graphormer":
            sorted_indices = sorted_indices[sorted_indices != 0] - 1      # drop the global node, back to batch positions
        x_i = torch.index_select(x_i, 0, sorted_indices)
        y_i = torch.index_select(y_i, 0, sorted_indices)
    if model == "graphormer":
        ei = adjust_edge_index_nomerge(ei, S)
    return (x_i, y_i, ei, None) + extra
