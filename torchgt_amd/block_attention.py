"""Block path: attention over dense 16 x 16 tiles plus remaining edges (one softmax per node).

A tile ``(r0, c0)`` stands for the 256 edges ``a -> b``, ``a in [r0, r0+16)``,
``b in [c0, c0+16)`` that the reference's cluster reordering emits as an expanded edge list
(gt_sp/utils.py:284-299) before calling ``sparse_attention`` (attn_module.py:133-189).  The
result equals sparse attention over the expanded tiles plus the remaining edges.
"""
import ctypes

import numpy as np
import torch

from . import _lib
from .core_attention import _DTYPES, _ptr
from .plan import GraphPlan


class TileSet:
    """Handle on ``tgt_tiles_t``: the tile list grouped by destination block and by source block."""

    def __init__(self, tiles, num_nodes, device, block_size=16):
        t = np.ascontiguousarray(np.asarray(tiles.cpu() if isinstance(tiles, torch.Tensor) else tiles), dtype=np.int32)
        if t.ndim != 2 or (t.size and t.shape[1] != 2):
            raise ValueError("tiles must be [T, 2] = (first source, first destination)")
        self.num_tiles = int(t.shape[0])
        self.num_nodes = int(num_nodes)
        self.device = torch.device(device)
        self._handle = ctypes.c_void_p()
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            _lib.check(_lib.lib().tgt_tiles_create(t.ctypes.data_as(ctypes.c_void_p) if t.size else None,
                                                   self.num_tiles, block_size, self.num_nodes, stream,
                                                   ctypes.byref(self._handle)))
        self._ws = {}

    @property
    def handle(self):
        if not self._handle:
            raise RuntimeError("tile set was destroyed")
        return self._handle

    def close(self):
        if getattr(self, "_handle", None):
            _lib.lib().tgt_tiles_destroy(self._handle)
            self._handle = ctypes.c_void_p()
            self._ws = {}

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def workspace(self, plan, H, d):
        key = (id(plan), H, d)
        ws = self._ws.get(key)
        if ws is None:
            n = _lib.lib().tgt_block_attn_workspace_bytes(self.handle, plan.handle, H, d)
            if n < 0:
                raise ValueError("bad H / d")
            ws = torch.zeros(max(int(n), 256), dtype=torch.uint8, device=self.device)   # counters start at 0
            self._ws[key] = (ws, plan)
            return ws
        return ws[0]


class BlockAttentionFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, edge_bias, tiles, plan):
        if not (q.is_cuda and k.is_cuda and v.is_cuda):
            raise RuntimeError("block attention needs GPU tensors (no CPU implementation)")
        if q.dtype not in _DTYPES or k.dtype != q.dtype or v.dtype != q.dtype:
            raise TypeError("q/k/v must share dtype float32 or bfloat16")
        if q.dim() != 3 or q.shape != k.shape or q.shape != v.shape:
            raise ValueError("q, k, v must be [N, H, d] with equal shapes")
        N, H, d = q.shape
        if N != plan.num_nodes or N != tiles.num_nodes:
            raise ValueError("q, the tile set and the plan disagree on the number of nodes")
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        mode = _lib.BIAS_NONE
        if edge_bias is not None:
            if edge_bias.dtype != q.dtype:
                raise TypeError("edge bias must have the dtype of q")
            edge_bias = edge_bias.contiguous()
            E = plan.num_edges
            if edge_bias.dim() == 2 and edge_bias.shape == (E, H) and H != 1:
                mode = _lib.BIAS_EDGE_HEAD
            elif edge_bias.numel() == E:
                mode = _lib.BIAS_EDGE
            else:
                raise ValueError("edge bias must be [E] or [E, H] over the remaining edges")
        out = torch.empty_like(q)
        Z = torch.empty((N, H), dtype=torch.float32, device=q.device)
        ws = tiles.workspace(plan, H, d)
        with torch.cuda.device(q.device):
            stream = torch.cuda.current_stream(q.device).cuda_stream
            _lib.check(_lib.lib().tgt_block_attn_fwd(
                tiles.handle, plan.handle, _ptr(q), _ptr(k), _ptr(v), _ptr(edge_bias), mode, H, d,
                _DTYPES[q.dtype], _ptr(out), _ptr(Z), _ptr(ws), ws.numel(), stream))
        ctx.tiles, ctx.plan, ctx.mode = tiles, plan, mode
        ctx.has_bias = edge_bias is not None
        ctx.save_for_backward(q, k, v, edge_bias, out, Z)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, edge_bias, out, Z = ctx.saved_tensors
        N, H, d = q.shape
        dout = dout.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dbias = torch.empty_like(edge_bias) if (ctx.has_bias and ctx.needs_input_grad[3]) else None
        ws = ctx.tiles.workspace(ctx.plan, H, d)
        with torch.cuda.device(q.device):
            stream = torch.cuda.current_stream(q.device).cuda_stream
            _lib.check(_lib.lib().tgt_block_attn_bwd(
                ctx.tiles.handle, ctx.plan.handle, _ptr(q), _ptr(k), _ptr(v), _ptr(edge_bias), ctx.mode, H, d,
                _DTYPES[q.dtype], _ptr(out), _ptr(Z), _ptr(dout), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(dbias),
                _ptr(ws), ws.numel(), stream))
        return dq, dk, dv, dbias, None, None


def block_attention(q, k, v, tiles, edge_index=None, edge_bias=None, plan=None):
    """q, k, v: [N, H, d]; ``tiles``: a TileSet or a [T, 2] array of (first source, first
    destination); ``edge_index`` int64 [2, E]: the edges outside the tiles (may be None);
    ``edge_bias``: [E] / [E, H] over those edges.  Returns [N, H, d]."""
    H, d = q.shape[-2], q.shape[-1]
    q3, k3, v3 = q.reshape(-1, H, d), k.reshape(-1, H, d), v.reshape(-1, H, d)
    N = q3.shape[0]
    if not isinstance(tiles, TileSet):
        tiles = TileSet(tiles, N, q.device)
    if plan is None:
        if edge_index is None:
            edge_index = torch.zeros((2, 0), dtype=torch.int64, device=q.device)
        plan = GraphPlan(edge_index, N, rows_with_edges_only=True)
    if edge_bias is not None:
        edge_bias = edge_bias.to(q3.dtype)
    return BlockAttentionFunction.apply(q3, k3, v3, edge_bias, tiles, plan)


def expand_tiles(tiles, block_size=16):
    """The edge list a tile list stands for, in the reference's emission order (create_pairs,
    gt_sp/utils.py:218-220): for each tile, pairs (a, b) row-major.  int64 [2, T*bs*bs] numpy."""
    t = np.asarray(tiles, dtype=np.int64).reshape(-1, 2)
    a = (t[:, :1] + np.repeat(np.arange(block_size), block_size)[None, :]).reshape(-1)
    b = (t[:, 1:] + np.tile(np.arange(block_size), block_size)[None, :]).reshape(-1)
    return np.stack([a, b])
