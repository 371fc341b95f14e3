"""Drop-in ``CoreAttention`` for TorchGT's node-level models, backed by the
gfx950 library.

Mirrors the reference classes
  * ``models/graphormer_dist_node_level.py:42-221``  (4-argument constructor,
    ``sparse_attention_bias(k, q, v, edge_index, attn_bias)``, forward dispatch)
  * ``models/gt_dist_node_level.py:30-166`` / ``graphormer_dist_graph_level.py``
    (3-argument constructor)
  * ``attn_module.py:87-229`` (``(hidden, dropout, heads, device)`` constructor,
    ``forward(q, k, v, edge_index, flash_attn=False, full=False, mask=None)``)
with sequence-parallel size 1 (``num_attention_heads_per_partition == num_heads``).

There is no CPU or eager fallback: tensors must live on the GPU and the HIP
library must be built, otherwise an exception is raised.
"""
import math
import weakref

import torch
import torch.nn as nn

from . import _ext, _lib
from .plan import GraphPlan, get_plan

_DTYPES = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16}


def _ptr(t):
    return t.data_ptr() if t is not None else None


class SparseAttentionFunction:
    """out[N,H,d], Z[N,H] = sparse_attention(q, k, v, plan, edge_bias): ``torch.ops.torchgt.sparse_attention`` (a C++
    autograd function over ``tgt_sparse_attn_fwd`` / ``_bwd``; the reference relies on autograd through ATen /
    torch_scatter ops, attn_module.py:146-187).  ``apply`` keeps the call convention of an autograd function."""

    @staticmethod
    def apply(q, k, v, edge_bias, plan, bias_in_plan_order=False):
        if not (q.is_cuda and k.is_cuda and v.is_cuda):
            raise RuntimeError("sparse attention needs GPU tensors (no CPU implementation)")
        if q.dtype not in _DTYPES or k.dtype != q.dtype or v.dtype != q.dtype:
            raise TypeError(f"q/k/v must share dtype float32 or bfloat16, got {q.dtype}/{k.dtype}/{v.dtype}")
        if q.dim() != 3 or q.shape != k.shape or q.shape != v.shape:
            raise ValueError("q, k, v must be [N, H, d] with equal shapes")
        N, H, d = q.shape
        if N != plan.num_nodes:
            raise ValueError(f"q has {N} rows but the plan was built for {plan.num_nodes} nodes")
        mode = _lib.BIAS_NONE
        if edge_bias is not None:
            if edge_bias.dtype != q.dtype:
                raise TypeError("edge bias must have the dtype of q (convert it outside, where autograd sees it)")
            E = plan.num_edges
            both = bias_in_plan_order and edge_bias.shape[0] == 2 * E and E > 0
            rows = 2 * E if both else E
            if edge_bias.dim() == 2 and edge_bias.shape == (rows, H) and H != 1:
                mode = _lib.BIAS_EDGE_HEAD
            elif edge_bias.numel() == rows:
                mode = _lib.BIAS_EDGE
            else:
                raise ValueError(f"edge bias must be [E] or [E, H] with E={E}, H={H}; got {tuple(edge_bias.shape)}")
            if bias_in_plan_order:
                mode |= _lib.BIAS_PLAN_ORDER
                if both:
                    mode |= _lib.BIAS_BOTH_ORDERS      # [2E, ...]: destination-sorted rows, then source-sorted rows
                else:
                    plan.edge_order()                  # makes sure the plan holds the map for this mode
        plan.handle      # raises if the plan was closed
        return _ext.ops().sparse_attention(q, k, v, edge_bias, plan.holder, mode, plan.workspace(H, d))


class DenseAttentionFunction:
    """out[b,S,H*d] = dropout(softmax((q*sqrt(d)) k^T + bias)) v, the dense ``CoreAttention.forward`` of
    models/graphormer_graph_level.py:186-214: ``torch.ops.torchgt.dense_attention``.  bfloat16 tensors run on the
    matrix cores (bf16 products, fp32 accumulation and softmax); float32 tensors run in float32 arithmetic like the
    reference, unless ``bf16_products`` asks for the matrix cores (about 2e-2 instead of 1e-5).  ``p_drop`` / ``seed``:
    attention dropout regenerated in the backward from the same pair, no mask is stored."""

    @staticmethod
    def apply(q, k, v, bias, p_drop=0.0, seed=0, bf16_products=False):
        return _ext.ops().dense_attention(q, k, v, bias, float(p_drop), int(seed), bool(bf16_products))


def dense_dropout_mask(b, S, H, p_drop, seed, device):
    """uint8 [b, H, S, S]: 1 where the dense kernels keep a probability for (p_drop, seed) - the mask torch's
    Dropout would hold."""
    keep = torch.empty((b, H, S, S), dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        _lib.check(_lib.lib().tgt_dense_attn_dropout_mask(b, S, H, float(p_drop), int(seed), keep.data_ptr(),
                                                          torch.cuda.current_stream(device).cuda_stream))
    return keep


class GraphBiasIds:
    """The graph-level attention bias in unbuilt form: what ``GraphAttnBias`` (models/graphormer_graph_level.py:94-156,
    plain edge-type branch) would turn into a [b, H, S, S] tensor, kept as 16-bit ids over the padded [b, S, S] index
    space (``torch.ops.torchgt.dense_ids_pack``), the [b, S, S] ``attn_bias`` of the batch and the three embedding
    tables.  ``dense_attention`` accepts it in place of the bias tensor: the kernels then form the bias on chip and
    return the table gradients directly (bf16 matrix-product kernels only).  ``materialize()`` builds the tensor the
    reference would pass, once, for the float32-arithmetic kernels and for shapes whose bias does not fit the LDS."""

    def __init__(self, attn_bias, sp16, et16, spatial_table, edge_table, virtual_dist, build):
        self.attn_bias, self.sp16, self.et16 = attn_bias, sp16, et16
        self.spatial_table, self.edge_table, self.virtual_dist = spatial_table, edge_table, virtual_dist
        self._build = build            # () -> [b, H, S, S] tensor with autograd to the tables
        self._tensor = None
        self.fits = True               # cleared when the kernels report that this shape needs the tensor

    def materialize(self):
        if self._tensor is None:
            self._tensor = self._build()
        return self._tensor


def dense_attention(q, k, v, attn_bias=None, p_drop=0.0, seed=None, bf16_products=False):
    """Functional form of the dense path: q, k, v [b, S, H, d], attn_bias [b, H, S, S] or None;
    returns [b, S, H*d].  A bias of another float dtype or with a broadcast head axis
    ([b, 1, S, S]) is converted / expanded here, where autograd sees it.  ``p_drop`` > 0 applies attention
    dropout; ``seed`` (default: drawn from torch's CPU generator, so ``torch.manual_seed`` governs it) names
    the mask.  ``attn_bias`` may be a ``GraphBiasIds``."""
    if p_drop > 0 and seed is None:
        seed = int(torch.randint(0, 2 ** 62, (1,)).item())
    if isinstance(attn_bias, GraphBiasIds):
        ids = attn_bias
        if ids.fits and (q.dtype == torch.bfloat16 or bf16_products):
            ab = None if ids.attn_bias is None else ids.attn_bias.to(q.dtype)
            try:
                return _ext.ops().dense_attention_ids(q, k, v, ab, ids.sp16, ids.et16, ids.spatial_table.to(q.dtype),
                                                      ids.edge_table.to(q.dtype), ids.virtual_dist.to(q.dtype), float(p_drop),
                                                      int(seed or 0), bool(bf16_products))
            except RuntimeError as exc:
                if "bytes of LDS" not in str(exc):
                    raise
                ids.fits = False       # this shape needs the bias tensor: build it once, below
        attn_bias = ids.materialize()
    if attn_bias is not None:
        b, S, H = q.shape[0], q.shape[1], q.shape[2]
        if attn_bias.dim() == 4 and attn_bias.shape[1] == 1 and H != 1:
            attn_bias = attn_bias.expand(b, H, S, S)
        elif attn_bias.dim() == 4 and tuple(attn_bias.shape) == (b, S, S, H) and S != H:
            # the node-level models hand over [b, S, S, H] and the reference REINTERPRETS that memory as [b, H, S, S]
            # (`attn_bias.view(*output_size)`, models/graphormer_dist_node_level.py:160 - a view, not a permute)
            attn_bias = attn_bias.contiguous().view(b, H, S, S)
        attn_bias = attn_bias.to(q.dtype)
    return DenseAttentionFunction.apply(q, k, v, attn_bias, p_drop, seed or 0, bf16_products)


def sparse_attention(q, k, v, edge_index=None, edge_bias=None, plan=None, return_z=False, bias_in_plan_order=False):
    """Functional form.  q, k, v: [N, H, d] (or [b, S, H, d], flattened over b*S
    as in attn_module.py:141-143); ``edge_index`` int64 [2, E] (row 0 = source /
    key node, row 1 = destination / query node) or a prebuilt ``plan``;
    ``edge_bias``: None, [E] or [E, H] in the order of ``edge_index`` - or, with
    ``bias_in_plan_order=True``, already permuted with ``plan.sort_bias(bias)``
    (worth it when several layers share one bias: see ``GraphPlan.sort_bias``)."""
    H, d = q.shape[-2], q.shape[-1]
    q3, k3, v3 = q.reshape(-1, H, d), k.reshape(-1, H, d), v.reshape(-1, H, d)
    if plan is None:
        if edge_index is None:
            raise ValueError("need edge_index or plan")
        plan = get_plan(edge_index, q3.shape[0])
    if edge_bias is not None:
        edge_bias = edge_bias.to(q3.dtype)
    out, Z = SparseAttentionFunction.apply(q3, k3, v3, edge_bias, plan, bias_in_plan_order)
    return (out, Z) if return_z else out


def gather_dense_bias(attn_bias, edge_index, layout):
    """Per-edge view ``bias[src, dst, :]`` of a dense bias, the indexing of
    models/graphormer_dist_graph_level.py:262-267.  layout 'bhss' = [b, H, S, S]
    (graph-level), 'bssh' = [b, S, S, H'] (node-level,
    graphormer_dist_node_level.py:100-106).  The dense [b*S, b*S, H] tensor the
    reference builds is never materialised.  Differentiable (torch indexing)."""
    if layout == "bhss":
        attn_bias = attn_bias.permute(0, 2, 3, 1)
    S = attn_bias.shape[1]
    src, dst = edge_index[0].long(), edge_index[1].long()
    return attn_bias[src // S, src % S, dst % S, :]


def _drop_bias_cache(_grad):
    _BIAS_CACHE.clear()


_BIAS_CACHE = {}      # at most one entry: the per-edge bias in plan order of the bias tensor seen last


def _plan_order_bias(module, attn_bias, edge_index, plan, dtype):
    """Per-edge bias in the plan's sorted orders for a dense or per-edge ``attn_bias``.  The layers of one
    forward pass get one and the same bias tensor: the first brings it into plan order, the others reuse the
    result.  The entry is tied to the tensor (held weakly), its version, the plan, the dtype and the autograd
    state it was made under - a result made under ``no_grad`` carries no graph and is not handed to a pass that
    needs one - and it is dropped when the backward of any layer that used it begins, so neither the bias nor its 2E-row copy
    outlives the step.  Differentiable."""
    key = (id(attn_bias), attn_bias._version, id(plan), dtype, module.dense_bias_layout,
           torch.is_grad_enabled(), attn_bias.requires_grad)
    hit = _BIAS_CACHE.get("entry")
    if hit is not None and hit[0] == key and hit[1]() is attn_bias and hit[2] is plan:
        return hit[3]
    if attn_bias.dim() <= 2:
        eb = plan.sort_bias(attn_bias.to(dtype))
    else:
        if isinstance(edge_index, GraphPlan):
            raise ValueError("a dense attn_bias needs the edge_index tensor (not a prebuilt plan)")
        both = torch.cat([plan.edge_order(), plan.edge_order_src()])       # destination-sorted rows, then source-sorted
        eb = gather_dense_bias(attn_bias, edge_index.index_select(1, both), module.dense_bias_layout)
        if eb.shape[-1] == 1:
            eb = eb.squeeze(-1)
        eb = eb.to(dtype)
    _BIAS_CACHE["entry"] = (key, weakref.ref(attn_bias), plan, eb)
    return eb


class CoreAttention(nn.Module):
    """Same constructor and call conventions as the reference's ``CoreAttention``
    classes (see the module docstring for the three flavours)."""

    def __init__(self, hidden_size, attention_dropout_rate, num_heads, *extra, **kw):
        super().__init__()
        self.hidden_size_per_partition = hidden_size
        self.hidden_size_per_attention_head = hidden_size // num_heads
        self.num_attention_heads_per_partition = num_heads      # sequence-parallel size 1
        self.scale = math.sqrt(self.hidden_size_per_attention_head)
        self.num_heads = num_heads
        self.att_dropout = nn.Dropout(attention_dropout_rate)
        self.attention_dropout_rate = attention_dropout_rate
        self.drop_out_rate = attention_dropout_rate
        # 4th positional argument: attn_bias_dim (node-level Graphormer) or a device (attn_module.py)
        fourth = extra[0] if extra else kw.get("attn_bias_dim", kw.get("device"))
        self.attn_bias_dim = fourth if isinstance(fourth, int) else None
        self.dense_bias_layout = "bssh" if self.attn_bias_dim is not None else "bhss"
        # float32 dense attention runs in float32 arithmetic like the reference; True moves its products to the
        # bf16 matrix cores (faster, about 2e-2 instead of 1e-5)
        self.dense_bf16_products = False

    # -- helpers ---------------------------------------------------------
    def _edge_bias(self, attn_bias, edge_index):
        if attn_bias is None:
            return None
        if attn_bias.dim() <= 2:
            return attn_bias                       # already per edge: [E], [E, 1] or [E, H]
        eb = gather_dense_bias(attn_bias, edge_index, self.dense_bias_layout)
        if eb.shape[-1] == 1:
            eb = eb.squeeze(-1)
        return eb

    def _sparse(self, q, k, v, edge_index, attn_bias):
        H, d = self.num_heads, self.hidden_size_per_attention_head
        q3 = q.reshape(-1, H, d)
        k3 = k.reshape(-1, H, d)
        v3 = v.reshape(-1, H, d)
        plan = edge_index if isinstance(edge_index, GraphPlan) else get_plan(edge_index, q3.shape[0])
        if attn_bias is None:
            out, _ = SparseAttentionFunction.apply(q3, k3, v3, None, plan)
            return out
        # The layers of a model get one and the same bias tensor: it is brought into the plan's edge order once
        # (by the first layer that sees it) and every layer then streams it.
        eb = _plan_order_bias(self, attn_bias, edge_index, plan, q3.dtype)
        out, _ = SparseAttentionFunction.apply(q3, k3, v3, eb, plan, True)
        if out.requires_grad:
            out.register_hook(_drop_bias_cache)     # the backward has begun: the step's forward passes are over
        return out

    # -- reference method names -------------------------------------------
    def sparse_attention_bias(self, k, q, v, edge_index, attn_bias):
        """models/graphormer_dist_node_level.py:69-127 — note the (k, q, v) order.
        Returns [b*S, H, d]."""
        return self._sparse(q, k, v, edge_index, attn_bias)

    def sparse_attention(self, q, k, v, edge_index, attn_bias=None):
        """attn_module.py:133-189.  Returns [b, S, H*d]."""
        b, S = k.size(0), k.size(1)
        return self._sparse(q, k, v, edge_index, attn_bias).view(b, S, -1)

    def full_attention(self, q, k, v, attn_bias=None, mask=None):
        """attn_module.py:99-127 / graphormer_graph_level.py:186-214: dense attention with an
        additive [b, H, S, S] bias.  Returns [b, S, H*d]."""
        if mask is not None:
            raise NotImplementedError("the reference never passes `mask` (graphormer_graph_level.py:380); "
                                      "it is not supported")
        # the reference applies att_dropout to the softmax output (graphormer_graph_level.py:207-209); here the
        # kernels do, in training mode
        p = float(self.attention_dropout_rate) if self.training else 0.0
        return dense_attention(q, k, v, attn_bias, p_drop=p, bf16_products=self.dense_bf16_products)

    def forward(self, q, k, v, attn_bias=None, edge_index=None, attn_type=None, mask=None,
                flash_attn=False, full=False):
        """Node-level convention (graphormer_dist_node_level.py:199-221):
        ``forward(q, k, v, attn_bias, edge_index, attn_type)`` with q, k, v
        [b, S, H, d]; returns [b, S, H*d].  The benchmark convention of
        attn_module.py:221-229, ``forward(q, k, v, edge_index)``, is recognised
        by an integer [2, E] fourth argument; the graph-level convention of
        graphormer_graph_level.py:186, ``forward(q, k, v, attn_bias, mask)``, by
        the absence of both edge_index and attn_type."""
        if (edge_index is None and isinstance(attn_bias, torch.Tensor) and attn_bias.dim() == 2
                and attn_bias.size(0) == 2 and not attn_bias.is_floating_point()):
            edge_index, attn_bias = attn_bias, None
            if attn_type is None:
                attn_type = "full" if full else ("flash" if flash_attn else "sparse")
        if attn_type is None and edge_index is None:
            attn_type = "full"        # graph-level convention: forward(q, k, v, attn_bias, mask)
        b, S = q.size(0), q.size(1)
        if attn_type == "sparse":
            x = self._sparse(q, k, v, edge_index, attn_bias)
        elif attn_type == "full":
            x = self.full_attention(q, k, v, attn_bias, mask)
        elif attn_type == "flash":
            raise NotImplementedError(
                "attn_type='flash' calls the CUDA-only flash_attn package in the reference "
                "(graphormer_dist_node_level.py:211-216); it has no counterpart here")
        else:
            raise ValueError(f"unknown attn_type {attn_type!r}")
        return x.view(b, S, -1)
