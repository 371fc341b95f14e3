"""Graph plan: Python handle on ``tgt_plan_t`` (include/torchgt_hip.h).

The reference re-gathers ``k[edge_index[0]]`` / ``q[edge_index[1]]`` and
scatter-adds over ``edge_index[1]`` on every attention call of every layer
(attn_module.py:146-147,180,185) although ``edge_index`` is shared by all layers
of a step and by all steps of a pre-packed batch
(main_sp_sparse_node_level.py:155-161).  A plan is the sorted form of one
``edge_index``; it is built once and reused.
"""
import collections
import ctypes

import numpy as np
import torch

from . import _ext, _lib


class GraphPlan:
    """Stable CSR-by-destination / CSC-by-source views of ``edge_index`` plus the
    row schedule, resident on the GPU."""

    def __init__(self, edge_index, num_nodes):
        if not isinstance(edge_index, torch.Tensor) or edge_index.dim() != 2 or edge_index.size(0) != 2:
            raise ValueError("edge_index must be a [2, E] tensor")
        if not edge_index.is_cuda:
            raise RuntimeError("GraphPlan needs edge_index on the GPU (there is no CPU implementation)")
        ei = edge_index.to(torch.int64).contiguous()
        self.num_nodes = int(num_nodes)
        self.num_edges = int(ei.size(1))
        self.device = ei.device
        self._handle = ctypes.c_void_p()
        self._workspaces = {}
        L = _lib.lib()
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            src_ptr = ei[0].data_ptr() if self.num_edges else None
            dst_ptr = ei[1].data_ptr() if self.num_edges else None
            _lib.check(L.tgt_plan_create(src_ptr, dst_ptr, self.num_edges, self.num_nodes, stream,
                                         ctypes.byref(self._handle)))
        # the owner of the C plan: shared with every autograd node that needs the plan in its backward, so that
        # the plan outlives this object if a backward is still pending
        _ext.ops()
        self.holder = torch.classes.torchgt.PlanHolder(self._handle.value)

    @property
    def handle(self):
        if not self._handle:
            raise RuntimeError("plan was destroyed")
        return self._handle

    def close(self):
        """Lets go of the plan; its device memory is freed when the last pending backward that uses it has run."""
        if getattr(self, "_handle", None):
            if getattr(self, "holder", None) is None:
                _lib.lib().tgt_plan_destroy(self._handle)        # creation failed half-way: nobody else owns it
            self.holder = None
            self._handle = ctypes.c_void_p()
            self._workspaces = {}

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def info(self):
        arr = (ctypes.c_int64 * 16)()
        _lib.check(_lib.lib().tgt_plan_info(self.handle, arr))
        keys = ["N", "E", "items_dst", "split_rows_dst", "segments_dst", "items_src", "split_rows_src",
                "segments_src", "segment_len", "wave_row_max", "block_items_dst", "block_items_src"]
        return {k: int(arr[i]) for i, k in enumerate(keys)}

    def export(self, which):
        """Copy one plan array to host as int32 numpy (tests compare it with the oracle)."""
        L = _lib.lib()
        n = L.tgt_plan_array_len(self.handle, which)
        if n < 0:
            raise ValueError(f"bad plan array id {which}")
        out = np.empty(n, dtype=np.int32)
        _lib.check(L.tgt_plan_export(self.handle, which, out.ctypes.data_as(ctypes.c_void_p), n))
        return out

    def edge_order(self):
        """int64 [E] on the GPU: the caller's index of every edge in the plan's destination-sorted (stable)
        order.  ``bias[plan.edge_order()]`` is a bias in plan order (see ``sort_bias``).  Also builds, once,
        the map the walk by source needs for a bias that is given in that order only."""
        if getattr(self, "_edge_order", None) is None:
            L = _lib.lib()
            out = torch.empty(self.num_edges, dtype=torch.int64, device=self.device)
            with torch.cuda.device(self.device):
                stream = torch.cuda.current_stream(self.device).cuda_stream
                _lib.check(L.tgt_plan_enable_bias_order(self.handle, stream))
                _lib.check(L.tgt_plan_edge_order(self.handle, out.data_ptr() if self.num_edges else None, stream))
            self._edge_order = out
        return self._edge_order

    def edge_order_src(self):
        """The same for the source-sorted order (the walk by source of the backward)."""
        if getattr(self, "_edge_order_src", None) is None:
            out = torch.empty(self.num_edges, dtype=torch.int64, device=self.device)
            with torch.cuda.device(self.device):
                _lib.check(_lib.lib().tgt_plan_edge_order_src(self.handle, out.data_ptr() if self.num_edges else None,
                                                              torch.cuda.current_stream(self.device).cuda_stream))
            self._edge_order_src = out
        return self._edge_order_src

    def sort_bias(self, edge_bias, both_orders=True):
        """A per-edge bias ([E] or [E, H], caller's edge order) in plan order, for
        ``sparse_attention(..., bias_in_plan_order=True)``.  With ``both_orders`` the result has 2 E rows: the
        destination-sorted copy, then the source-sorted one, so that no walk has to gather the bias.
        Differentiable: the gradient comes back in the caller's order.  Permute a bias that several layers share
        once and pass the result to all of them."""
        return _SortRows.apply(edge_bias, self, both_orders)

    def _permute(self, t, direction, out=None):
        """direction 0: caller's -> destination-sorted; 1: back; 2: caller's -> source-sorted."""
        if direction != 2:
            self.edge_order()
        t = t.contiguous()
        if t.shape[0] != self.num_edges:
            raise ValueError(f"expected {self.num_edges} rows, got {t.shape[0]}")
        if out is None:
            out = torch.empty_like(t)
        if self.num_edges:
            row_bytes = t.element_size() * (t.numel() // self.num_edges)
            with torch.cuda.device(self.device):
                _lib.check(_lib.lib().tgt_plan_sort_rows(self.handle, t.data_ptr(), row_bytes, out.data_ptr(), int(direction),
                                                         torch.cuda.current_stream(self.device).cuda_stream))
        return out

    def workspace(self, H, d):
        """Device scratch for the attention calls on this plan (cached per (H, d)).
        Calls that share it must be ordered on one stream."""
        key = (H, d)
        ws = self._workspaces.get(key)
        if ws is None:
            nbytes = _lib.lib().tgt_sparse_attn_workspace_bytes(self.handle, H, d)
            if nbytes < 0:
                raise ValueError("bad H / d")
            ws = torch.zeros(max(int(nbytes), 256), dtype=torch.uint8, device=self.device)   # counters start at 0
            self._workspaces[key] = ws
        return ws


class _SortRows(torch.autograd.Function):
    """bias in plan order (one or both copies); the gradient is carried back to the caller's order."""

    @staticmethod
    def forward(ctx, t, plan, both):
        ctx.plan = plan
        E = plan.num_edges
        if not both:
            return plan._permute(t, 0)
        t = t.contiguous()
        out = torch.empty((2 * E,) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
        plan._permute(t, 0, out=out[:E])
        plan._permute(t, 2, out=out[E:])
        return out

    @staticmethod
    def backward(ctx, g):
        E = ctx.plan.num_edges
        return ctx.plan._permute(g[:E], 1), None, None     # only the destination-sorted rows carry a gradient


_CACHE = collections.OrderedDict()
_CACHE_BYTES = 1 << 30        # device memory the cached plans (and the edge_index tensors they were built from) may hold


def set_plan_cache_bytes(nbytes):
    """Bound on the device memory held by ``get_plan``'s cache (default 1 GiB).  The plan asked for last is
    always kept, whatever its size."""
    global _CACHE_BYTES
    _CACHE_BYTES = int(nbytes)
    _evict()


def _plan_bytes(plan, edge_index):
    # two sorted views (rowptr, col, eid), items, wave records of one shape, and the edge_index kept alive
    return 56 * plan.num_edges + 450 * plan.num_nodes + edge_index.numel() * edge_index.element_size()


def _evict():
    total = sum(v[2] for v in _CACHE.values())
    while len(_CACHE) > 1 and total > _CACHE_BYTES:
        _, (_, _, nbytes) = _CACHE.popitem(last=False)      # freed when its last user (a pending backward) lets go
        total -= nbytes


def get_plan(edge_index, num_nodes):
    """Plan for ``edge_index``, cached on (storage address, shape, version, N) so
    that the layers of a model and the iterations over a pre-packed batch share
    one plan.  The cache keeps the tensor alive, so the address cannot be reused; it is bounded by bytes
    (``set_plan_cache_bytes``), least recently used plans go first.  A driver that moves a fresh edge_index
    to the GPU for every iteration therefore holds one large plan at a time, not sixteen.  Build plans before
    capturing a HIP graph: building one allocates and synchronises."""
    key = (edge_index.data_ptr(), tuple(edge_index.shape), edge_index._version, edge_index.dtype,
           str(edge_index.device), int(num_nodes))
    hit = _CACHE.get(key)
    if hit is not None:
        _CACHE.move_to_end(key)
        return hit[0]
    plan = GraphPlan(edge_index, num_nodes)
    _CACHE[key] = (plan, edge_index, _plan_bytes(plan, edge_index))
    _evict()
    return plan


def clear_plan_cache():
    _CACHE.clear()
    from . import core_attention
    core_attention._BIAS_CACHE.clear()
