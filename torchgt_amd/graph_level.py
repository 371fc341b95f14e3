"""The graph-level Graphormer on the library's kernels.

Mirrors of models/graphormer_graph_level.py: ``GraphNodeFeature`` (:18-60), ``EncoderLayer``
(:267-306) and ``Graphormer`` (:309-389) with the reference's constructors, ``forward(batched_data)``
and ``state_dict`` keys.  One sequence per graph, virtual node at index 0; the attention is the dense
biased kernel (``CoreAttention`` with ``attn_type='full'``), the bias comes from ``GraphAttnBias`` once
per step and is shared by all layers, the input rows from one gather kernel.
"""
import torch
import torch.nn as nn

from . import _ext, _lib
from .core_attention import GraphBiasIds
from .encoder import FeedForwardNetwork, init_params
from .graph_bias import GraphAttnBias
from .multi_head_attention import MultiHeadAttention, fused_linear

_DT = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16}


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


class GraphNodeFeatureFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, in_degree, out_degree, atom_table, in_table, out_table, graph_token):
        if not x.is_cuda:
            raise RuntimeError("GraphNodeFeature runs on the GPU only (no CPU fallback)")
        dt = atom_table.dtype
        if dt not in _DT:
            raise TypeError(f"unsupported dtype {dt}")
        b, s, Fx = x.shape
        C = atom_table.shape[1]
        x = x.to(torch.int64).contiguous()
        ind = in_degree.to(torch.int64).contiguous()
        outd = out_degree.to(torch.int64).contiguous()
        ta, ti, to, tk = (t.contiguous() for t in (atom_table, in_table, out_table, graph_token))
        out = torch.empty((b, s + 1, C), dtype=dt, device=x.device)
        with torch.cuda.device(x.device):
            _lib.check(_lib.lib().tgt_graph_node_feature_fwd(x.data_ptr(), ind.data_ptr(), outd.data_ptr(), Fx, ta.data_ptr(),
                                                             ta.shape[0], ti.data_ptr(), ti.shape[0], to.data_ptr(), to.shape[0],
                                                             tk.data_ptr(), b, s, C, _DT[dt], out.data_ptr(), _stream(x)))
        ctx.save_for_backward(x, ind, outd)
        ctx.dims = (b, s, Fx, C, ta.shape[0], ti.shape[0], to.shape[0], dt, graph_token.shape)
        return out

    @staticmethod
    def backward(ctx, dout):
        x, ind, outd = ctx.saved_tensors
        b, s, Fx, C, na, ni, no, dt, tshape = ctx.dims
        L = _lib.lib()
        dout = dout.to(dt).contiguous()
        dev = dout.device
        d_a = torch.empty((na, C), dtype=dt, device=dev)
        d_i = torch.empty((ni, C), dtype=dt, device=dev)
        d_o = torch.empty((no, C), dtype=dt, device=dev)
        d_t = torch.empty(C, dtype=dt, device=dev)
        nbytes = L.tgt_graph_node_feature_bwd_workspace_bytes(na, ni, no, C)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            _lib.check(L.tgt_graph_node_feature_bwd(dout.data_ptr(), x.data_ptr(), ind.data_ptr(), outd.data_ptr(), Fx, na, ni, no,
                                                    b, s, C, _DT[dt], d_a.data_ptr(), d_i.data_ptr(), d_o.data_ptr(),
                                                    d_t.data_ptr(), ws.data_ptr(), nbytes, _stream(dout)))
        return None, None, None, d_a, d_i, d_o, d_t.view(tshape)


class GraphNodeFeature(nn.Module):
    """Node features of every node of the batch, global token at index 0 (graphormer_graph_level.py:18-60)."""

    def __init__(self, num_heads, num_atoms, num_in_degree, num_out_degree, hidden_dim):
        super().__init__()
        self.num_heads = num_heads
        self.num_atoms = num_atoms
        self.atom_encoder = nn.Embedding(num_atoms, hidden_dim, padding_idx=0)
        self.in_degree_encoder = nn.Embedding(num_in_degree, hidden_dim, padding_idx=0)
        self.out_degree_encoder = nn.Embedding(num_out_degree, hidden_dim, padding_idx=0)
        self.graph_token = nn.Embedding(1, hidden_dim)

    def forward(self, batched_data):
        return GraphNodeFeatureFunction.apply(batched_data.x, batched_data.in_degree, batched_data.out_degree,
                                              self.atom_encoder.weight, self.in_degree_encoder.weight,
                                              self.out_degree_encoder.weight, self.graph_token.weight)


class EncoderLayer(nn.Module):
    """graphormer_graph_level.py:267-306: pre-norm attention and feed-forward blocks with residuals.
    ``residual`` / ``defer_residual`` as in the node-level layer: the last add of a layer rides on the
    first LayerNorm of the next."""

    def __init__(self, hidden_size, ffn_size, dropout_rate, attention_dropout_rate, num_heads):
        super().__init__()
        self.self_attention_norm = nn.LayerNorm(hidden_size)
        self.self_attention = MultiHeadAttention(hidden_size, attention_dropout_rate, num_heads, num_heads)
        self.self_attention_dropout = nn.Dropout(dropout_rate)
        self.ffn_norm = nn.LayerNorm(hidden_size)
        self.ffn = FeedForwardNetwork(hidden_size, ffn_size, dropout_rate)
        self.ffn_dropout = nn.Dropout(dropout_rate)

    one_operator = True      # False: always run the layer operator by operator

    def _one_operator(self, x, attn_bias):
        """``(extra, attn_bias[b,S,S], sp16, et16)`` for ``torch.ops.torchgt.dense_encoder_layer`` when it covers this call
        (no torch dropout at work, widths the kernels read without padding, a bias it can take as it is), else None."""
        if not self.one_operator or not x.is_cuda or x.dim() != 3 or x.dtype not in (torch.float32, torch.bfloat16):
            return None
        if self.training and (self.self_attention_dropout.p > 0 or self.ffn_dropout.p > 0):
            return None
        att = self.self_attention
        core = att.dist_attn.local_attn
        ve = 4 if x.dtype == torch.float32 else 8
        if att.output_layer is None or any(w % ve for w in (x.shape[-1], self.ffn.layer1.out_features)) or \
                att.num_heads * att.att_size != x.shape[-1]:
            return None
        b, S, H = x.shape[0], x.shape[1], att.num_heads
        if attn_bias is None:
            return [], None, None, None
        if isinstance(attn_bias, GraphBiasIds):
            ids = attn_bias
            if ids.fits and (x.dtype == torch.bfloat16 or core.dense_bf16_products) and all(
                    t.dtype == x.dtype for t in (ids.spatial_table, ids.edge_table, ids.virtual_dist)):
                ab = None if ids.attn_bias is None else ids.attn_bias.to(x.dtype)
                return [ids.spatial_table, ids.edge_table, ids.virtual_dist], ab, ids.sp16, ids.et16
            attn_bias = ids.materialize()
        if isinstance(attn_bias, torch.Tensor) and tuple(attn_bias.shape) == (b, H, S, S) and attn_bias.dtype == x.dtype:
            return [attn_bias], None, None, None
        return None

    def forward(self, x, attn_bias=None, mask=None, residual=None, defer_residual=False):
        if mask is not None:
            raise NotImplementedError("the reference never passes `mask` (graphormer_graph_level.py:380)")
        n1, n2 = self.self_attention_norm, self.ffn_norm
        fused = self._one_operator(x, attn_bias)
        if fused is not None:
            # the whole layer as one operator and one autograd node (same kernels, same order, same numbers)
            extra, ab, sp16, et16 = fused
            att = self.self_attention
            core = att.dist_attn.local_attn
            p = float(core.attention_dropout_rate) if self.training else 0.0
            seed = int(torch.randint(0, 2 ** 62, (1,)).item()) if p > 0 else 0
            params = [n1.weight, n1.bias, att.linear_q.weight, att.linear_q.bias, att.linear_k.weight, att.linear_k.bias,
                      att.linear_v.weight, att.linear_v.bias, att.output_layer.weight, att.output_layer.bias, n2.weight, n2.bias,
                      self.ffn.layer1.weight, self.ffn.layer1.bias, self.ffn.layer2.weight, self.ffn.layer2.bias]
            try:
                x2, y = _ext.ops().dense_encoder_layer(x, residual, params, extra, ab, sp16, et16, att.num_heads, n1.eps, n2.eps, p,
                                                       seed, bool(core.dense_bf16_products))
                return (x2, y) if defer_residual else _ext.ops().add(x2, y)
            except RuntimeError as exc:
                if sp16 is None or "bytes of LDS" not in str(exc):
                    raise
                attn_bias.fits = False       # this shape needs the bias tensor: the attention below builds it once
        x, y = _ext.ops().add_layer_norm(x, residual, n1.weight, n1.bias, float(n1.eps))
        y = self.self_attention(y, attn_bias, None, attn_type="full")
        y = self.self_attention_dropout(y)
        x, y = _ext.ops().add_layer_norm(x, y, n2.weight, n2.bias, float(n2.eps))
        y = self.ffn(y)
        y = self.ffn_dropout(y)
        if defer_residual:
            return x, y
        return _ext.ops().add(x, y)


class Graphormer(nn.Module):
    """Graphormer for graph-level tasks: one graph, one sequence (graphormer_graph_level.py:309-389)."""

    def __init__(self, n_layers, num_heads, hidden_dim, dropout_rate, intput_dropout_rate, ffn_dim, dataset_name, edge_type,
                 multi_hop_max_dist, attention_dropout_rate, output_dim):
        super().__init__()
        if dataset_name == "ZINC":                      # :325-339
            num_atoms, num_edges, num_edge_dis, num_spatial, num_in_degree, num_out_degree = 64, 64, 40, 40, 64, 64
        else:
            num_atoms, num_edges, num_edge_dis, num_spatial = 512 * 9 + 1, 512 * 3 + 1, 128, 512
            num_in_degree = num_out_degree = 512
        self.graph_node_feature = GraphNodeFeature(num_heads=num_heads, num_atoms=num_atoms, num_in_degree=num_in_degree,
                                                   num_out_degree=num_out_degree, hidden_dim=hidden_dim)
        self.graph_attn_bias = GraphAttnBias(num_heads=num_heads, num_atoms=num_atoms, num_edges=num_edges,
                                             num_spatial=num_spatial, num_edge_dis=num_edge_dis, edge_type=edge_type,
                                             multi_hop_max_dist=multi_hop_max_dist, hidden_dim=hidden_dim)
        self.input_dropout = nn.Dropout(intput_dropout_rate)
        self.layers = nn.ModuleList([EncoderLayer(hidden_dim, ffn_dim, dropout_rate, attention_dropout_rate, num_heads)
                                     for _ in range(n_layers)])
        self.final_ln = nn.LayerNorm(hidden_dim)
        if dataset_name == "PCQM4M-LSC":
            self.out_proj = nn.Linear(hidden_dim, 1)
        else:
            self.downstream_out_proj = nn.Linear(hidden_dim, output_dim)
        self.apply(lambda module: init_params(module, n_layers=n_layers))
        # True: the layers get the bias as ids + tables and the bf16 attention kernels form it on chip (the [b, H, S, S]
        # tensor is built only for layers that cannot: float32 arithmetic, the multi-hop branch, very long sequences).
        # It saves the bias tensor and one bias-gradient tensor per layer (68 MB each for 256 graphs of 129 nodes in bf16)
        # and costs GPU time: every attention launch rebuilds the bias of its (graph, head) pairs and every backward runs
        # the id histogram the tensor form runs once per step (1.85 against 2.30 ms per training step on that batch).
        self.bias_from_ids = False

    def forward(self, batched_data, perturb=None):
        x = self.graph_node_feature(batched_data)            # [b, s + 1, h]
        attn_bias = self.graph_attn_bias(batched_data, as_ids=self.bias_from_ids)       # [b, H, s + 1, s + 1], or its ids
        output = self.input_dropout(x)
        pending = None
        for enc_layer in self.layers:
            output, pending = enc_layer(output, attn_bias, mask=None, residual=pending, defer_residual=True)
        fl = self.final_ln
        _, output = _ext.ops().add_layer_norm(output, pending, fl.weight, fl.bias, float(fl.eps))
        head = self.out_proj if hasattr(self, "out_proj") else self.downstream_out_proj
        (output,) = fused_linear(output[:, 0, :].contiguous(), head)      # the virtual node's row (:387)
        return output
