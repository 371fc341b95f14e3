"""Host-side mirror of the reference's edge construction helpers, backed by the
GPU kernels of csrc/graph_prep.hip (no CPU implementation).

  fix_edge_index(x, num_node)                       gt_sp/utils.py:34-50
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
