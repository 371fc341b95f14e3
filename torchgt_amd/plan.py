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
import weakref

import numpy as np
import torch

from . import _ext, _lib


class GraphPlan:
    """Stable CSR-by-destination / CSC-by-source views of ``edge_index`` plus the
    row schedule, resident on the GPU.  ``rows_with_edges_only``: a plan of the edges beside a tile set
    (``block_attention``): rows without edges are left out of the schedule and written by the tile kernels;
    ``sparse_attention`` refuses such a plan."""

    def __init__(self, edge_index, num_nodes, rows_with_edges_only=False):
        if not isinstance(edge_index, torch.Tensor) or edge_index.dim() != 2 or edge_index.size(0) != 2:
            raise ValueError("edge_index must be a [2, E] tensor")
        if not edge_index.is_cuda:
            raise RuntimeError("GraphPlan needs edge_index on the GPU (there is no CPU implementation)")
        ei = edge_index.to(torch.int64).contiguous()
        self.num_nodes = int(num_nodes)
        self.num_edges = int(ei.size(1))
        self.device = ei.device
        self.rows_with_edges_only = bool(rows_with_edges_only)
        self._handle = ctypes.c_void_p()
        self._workspaces = {}
        _ext.ops()                       # registers torch's caching allocator with the library: no hipMalloc per plan
        L = _lib.lib()
        with torch.cuda.device(self.device):
            stream = torch.cuda.current_stream(self.device).cuda_stream
            src_ptr = ei[0].data_ptr() if self.num_edges else None
            dst_ptr = ei[1].data_ptr() if self.num_edges else None
            create = L.tgt_plan_create_remaining if rows_with_edges_only else L.tgt_plan_create
            _lib.check(create(src_ptr, dst_ptr, self.num_edges, self.num_nodes, stream, ctypes.byref(self._handle)))
        # the owner of the C plan: shared with every autograd node that needs the plan in its backward, so that
        # the plan outlives this object if a backward is still pending
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


_CACHE = collections.OrderedDict()      # content key -> (plan, bytes)
_BY_TENSOR = {}                          # id(tensor) -> (weak reference, version, plan): the layers of one step
_CACHE_BYTES = 1 << 30                   # device memory the cached plans may hold
_STATS = {"builds": 0, "content_hits": 0, "tensor_hits": 0}


def set_plan_cache_bytes(nbytes):
    """Bound on the device memory held by ``get_plan``'s cache (default 1 GiB).  The plan asked for last is
    always kept, whatever its size."""
    global _CACHE_BYTES
    _CACHE_BYTES = int(nbytes)
    _evict()


def plan_cache_stats():
    """Counters since the last ``clear_plan_cache``: plans built, look-ups answered by the content key, look-ups
    answered by the tensor itself."""
    return dict(_STATS)


def _plan_bytes(plan):
    # two sorted views (rowptr, col, eid), items, wave records of one shape
    return 56 * plan.num_edges + 450 * plan.num_nodes


def _evict():
    total = sum(v[1] for v in _CACHE.values())
    while len(_CACHE) > 1 and total > _CACHE_BYTES:
        _, (gone, nbytes) = _CACHE.popitem(last=False)      # freed when its last user (a pending backward) lets go
        total -= nbytes
        for tid in [t for t, ent in _BY_TENSOR.items() if ent[2] is gone]:
            del _BY_TENSOR[tid]


def edge_index_key(edge_index):
    """128-bit content key of ``edge_index`` (values and positions), computed on the GPU."""
    ei = edge_index if (edge_index.dtype == torch.int64 and edge_index.is_contiguous()) else edge_index.to(torch.int64).contiguous()
    E = int(ei.size(1))
    key = (ctypes.c_uint64 * 2)()
    with torch.cuda.device(ei.device):
        _ext.ops()
        _lib.check(_lib.lib().tgt_edge_index_hash(ei[0].data_ptr() if E else None, ei[1].data_ptr() if E else None, E,
                                                  torch.cuda.current_stream(ei.device).cuda_stream, key))
    return int(key[0]), int(key[1])


def get_plan(edge_index, num_nodes):
    """Plan for ``edge_index``, shared by the layers of a model and by the iterations over a pre-packed batch.

    The cache is keyed on the CONTENT of ``edge_index`` (a 128-bit key computed by two small kernels and one
    16-byte read-back), so a driver that moves the same CPU-resident edge list to the GPU in every iteration -
    the reference's loops do (main_sp_sparse_node_level.py:178-183, gt_sp/utils.py:455-458) - gets the plan it
    built the first time.  The tensor object itself is remembered through a weak reference (no hashing for the
    second and later layers of a step; the tensor is not kept alive).  The cache is bounded by bytes
    (``set_plan_cache_bytes``), least recently used plans go first.  Build plans before capturing a HIP graph:
    the look-up synchronises the stream, building allocates."""
    ent = _BY_TENSOR.get(id(edge_index))
    if ent is not None:
        ref, version, plan, n = ent
        if ref() is edge_index and version == edge_index._version and n == int(num_nodes) and plan._handle:
            _STATS["tensor_hits"] += 1
            return plan
    if not edge_index.is_cuda:
        raise RuntimeError("get_plan needs edge_index on the GPU (there is no CPU implementation)")
    key = (edge_index_key(edge_index), tuple(edge_index.shape), str(edge_index.device), int(num_nodes))
    hit = _CACHE.get(key)
    if hit is not None and hit[0]._handle:
        _CACHE.move_to_end(key)
        plan = hit[0]
        _STATS["content_hits"] += 1
    else:
        plan = GraphPlan(edge_index, num_nodes)
        _STATS["builds"] += 1
        _CACHE[key] = (plan, _plan_bytes(plan))
        _evict()
    _remember(edge_index, plan, int(num_nodes))
    return plan


def _remember(edge_index, plan, n):
    tid = id(edge_index)

    def forget(_ref, tid=tid):
        ent = _BY_TENSOR.get(tid)
        if ent is not None and ent[0] is _ref:
            del _BY_TENSOR[tid]

    _BY_TENSOR[tid] = (weakref.ref(edge_index, forget), edge_index._version, plan, n)


def clear_plan_cache():
    _CACHE.clear()
    _BY_TENSOR.clear()
    for k in _STATS:
        _STATS[k] = 0
    from . import core_attention
    core_attention._BIAS_CACHE.clear()
