"""The graph-level Graphormer on the library's kernels.

Mirrors of models/graphormer_graph_level.py: ``GraphNodeFeature`` (:18-60), ``EncoderLayer``
(:267-306) and ``Graphormer`` (:309-389) with the reference's constructors, ``forward(batched_data)``
and ``state_dict`` keys.  One sequence per graph, virtual node at index 0; the attention is the dense
biased kernel (``CoreAttention`` with ``attn_type='full'``), the bias comes from ``GraphAttnBias`` once
per step and is shared by all layers, the input rows from one gather kernel.
"""
import torch
import torch.nn as nn

from . import _lib
from .encoder import AddFunction, AddLayerNormFunction, FeedForwardNetwork, init_params
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

    def forward(self, x, attn_bias=None, mask=None, residual=None, defer_residual=False):
        if mask is not None:
            raise NotImplementedError("the reference never passes `mask` (graphormer_graph_level.py:380)")
        n1, n2 = self.self_attention_norm, self.ffn_norm
        x, y = AddLayerNormFunction.apply(x, residual, n1.weight, n1.bias, n1.eps)
        y = self.self_attention(y, attn_bias, None, attn_type="full")
        y = self.self_attention_dropout(y)
        x, y = AddLayerNormFunction.apply(x, y, n2.weight, n2.bias, n2.eps)
        y = self.ffn(y)
        y = self.ffn_dropout(y)
        if defer_residual:
            return x, y
        return AddFunction.apply(x, y)


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
        # tensor is built only for layers that cannot: float32 arithmetic, the multi-hop branch, very long sequences)
        self.bias_from_ids = True

    def forward(self, batched_data, perturb=None):
        x = self.graph_node_feature(batched_data)            # [b, s + 1, h]
        attn_bias = self.graph_attn_bias(batched_data, as_ids=self.bias_from_ids)       # [b, H, s + 1, s + 1], or its ids
        output = self.input_dropout(x)
        pending = None
        for enc_layer in self.layers:
            output, pending = enc_layer(output, attn_bias, mask=None, residual=pending, defer_residual=True)
        fl = self.final_ln
        _, output = AddLayerNormFunction.apply(output, pending, fl.weight, fl.bias, fl.eps)
        head = self.out_proj if hasattr(self, "out_proj") else self.downstream_out_proj
        (output,) = fused_linear(output[:, 0, :].contiguous(), head)      # the virtual node's row (:387)
        return output
