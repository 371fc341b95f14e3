"""The node-level GT model on the library's kernels.

Mirrors of models/gt_dist_node_level.py: ``EncoderLayer`` (:218-267), ``MLPReadout`` (:270-286) and ``GT``
(:290-341) with the reference's constructors, ``forward`` signatures and ``state_dict`` keys.  No global token;
the attention is the sparse kernel without an output layer inside ``MultiHeadAttention`` (the layer's ``O``
follows it), LayerNorm comes after each residual add, the activations are ReLU.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _ext, _lib
from .encoder import init_params
from .multi_head_attention import MultiHeadAttention, fused_linear

_DT = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16}


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


class ReluFunction:
    """``torch.ops.torchgt.relu`` (C++ autograd function over ``tgt_relu_fwd`` / ``_bwd``)."""

    @staticmethod
    def apply(u):
        return _ext.ops().relu(u)


class EncoderLayer(nn.Module):
    """gt_dist_node_level.py:218-267.  As in the reference, ``self_attention_norm`` is constructed but not used,
    ``ffn_size`` is ignored (the feed-forward width is twice the hidden size) and the feed-forward block reads
    the attention branch ``y`` (after ``O``), not the normalised sum."""

    def __init__(self, hidden_size, ffn_size, dropout_rate, attention_dropout_rate, num_heads):
        super().__init__()
        self.self_attention_norm = nn.LayerNorm(hidden_size)
        self.self_attention = MultiHeadAttention(hidden_size, attention_dropout_rate, num_heads)
        self.self_attention_dropout = nn.Dropout(dropout_rate)
        self.O = nn.Linear(hidden_size, hidden_size)
        self.layer_norm1 = nn.LayerNorm(hidden_size)
        self.FFN_layer1 = nn.Linear(hidden_size, hidden_size * 2)
        self.FFN_layer2 = nn.Linear(hidden_size * 2, hidden_size)
        self.layer_norm2 = nn.LayerNorm(hidden_size)

    def forward(self, x, attn_bias=None, edge_index=None, attn_type=None):
        n1, n2 = self.layer_norm1, self.layer_norm2
        y = self.self_attention(x, attn_bias, edge_index=edge_index, attn_type=attn_type)      # :244
        y = self.self_attention_dropout(y)
        (y,) = fused_linear(y, self.O)                                                         # :246
        _, x = _ext.ops().add_layer_norm(x, y, n1.weight, n1.bias, float(n1.eps))                    # :247-248
        (y,) = fused_linear(y, self.FFN_layer1)                                                # :254
        y = ReluFunction.apply(y)
        y = self.self_attention_dropout(y)
        (y,) = fused_linear(y, self.FFN_layer2)
        _, x = _ext.ops().add_layer_norm(x, y, n2.weight, n2.bias, float(n2.eps))                    # :258-259
        return x


class MLPReadout(nn.Module):
    """gt_dist_node_level.py:270-286: L halving layers with ReLU, then the output layer."""

    def __init__(self, input_dim, output_dim, L=2):
        super().__init__()
        layers = [nn.Linear(input_dim // 2 ** l, input_dim // 2 ** (l + 1), bias=True) for l in range(L)]
        layers.append(nn.Linear(input_dim // 2 ** L, output_dim, bias=True))
        self.FC_layers = nn.ModuleList(layers)
        self.L = L

    def forward(self, x):
        y = x
        for l in range(self.L):
            (y,) = fused_linear(y, self.FC_layers[l])
            y = ReluFunction.apply(y)
        (y,) = fused_linear(y, self.FC_layers[self.L])
        return y


class GT(nn.Module):
    """GT for node-level tasks, no global token (gt_dist_node_level.py:290-341)."""

    def __init__(self, n_layers, num_heads, input_dim, hidden_dim, output_dim, attn_bias_dim, dropout_rate,
                 input_dropout_rate, attention_dropout_rate, ffn_dim, num_global_node):
        super().__init__()
        self.node_encoder = nn.Linear(input_dim, hidden_dim)
        self.input_dropout = nn.Dropout(input_dropout_rate)
        self.layers = nn.ModuleList([EncoderLayer(hidden_dim, ffn_dim, dropout_rate, attention_dropout_rate, num_heads)
                                     for _ in range(n_layers)])
        self.MLP_layer = MLPReadout(hidden_dim, output_dim)
        self.downstream_out_proj = nn.Linear(hidden_dim, output_dim)      # constructed, not used (:321)
        self.apply(lambda module: init_params(module, n_layers=n_layers))

    def forward(self, x, attn_bias, edge_index, perturb=None, attn_type=None):
        x = x.unsqueeze(0)
        (node_feature,) = fused_linear(x, self.node_encoder)
        output = self.input_dropout(node_feature)
        for enc_layer in self.layers:
            output = enc_layer(output, edge_index=edge_index, attn_type=attn_type)
        output = self.MLP_layer(output[0, :, :])
        return F.log_softmax(output, dim=1)


class EmbeddingSumFunction(torch.autograd.Function):
    """``embedding(x).sum(dim=-2)`` for integer features x [b, s, Fx] and a table without padding index."""

    @staticmethod
    def forward(ctx, x, table):
        if not x.is_cuda:
            raise RuntimeError("torchgt_amd kernels run on the GPU only (no CPU fallback)")
        dt = table.dtype
        if dt not in _DT:
            raise TypeError(f"unsupported dtype {dt}")
        b, s, Fx = x.shape
        x = x.to(torch.int64).contiguous()
        tab = table.contiguous()
        out = torch.empty((b, s, tab.shape[1]), dtype=dt, device=x.device)
        with torch.cuda.device(x.device):
            _lib.check(_lib.lib().tgt_embedding_sum_fwd(x.data_ptr(), Fx, tab.data_ptr(), tab.shape[0], b, s, tab.shape[1], _DT[dt],
                                                        out.data_ptr(), _stream(x)))
        ctx.save_for_backward(x)
        ctx.dims = (b, s, Fx, tab.shape[0], tab.shape[1], dt)
        return out

    @staticmethod
    def backward(ctx, dout):
        (x,) = ctx.saved_tensors
        b, s, Fx, rows, C, dt = ctx.dims
        L = _lib.lib()
        dout = dout.to(dt).contiguous()
        d_tab = torch.empty((rows, C), dtype=dt, device=dout.device)
        nbytes = L.tgt_embedding_sum_bwd_workspace_bytes(rows, C)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dout.device)
        with torch.cuda.device(dout.device):
            _lib.check(L.tgt_embedding_sum_bwd(dout.data_ptr(), x.data_ptr(), Fx, rows, b, s, C, _DT[dt], d_tab.data_ptr(),
                                               ws.data_ptr(), nbytes, _stream(dout)))
        return None, d_tab


class GraphLevelEncoderLayer(EncoderLayer):
    """models/gt_graph_level.py:210-254: the same layer with the reference's unused ``mask`` argument."""

    def forward(self, x, attn_bias=None, mask=None, edge_index=None, attn_type=None):
        if mask is not None:
            raise NotImplementedError("the reference never passes `mask` (gt_graph_level.py:344-348)")
        return super().forward(x, attn_bias, edge_index=edge_index, attn_type=attn_type)


class GraphLevelGT(nn.Module):
    """GT for graph-level tasks, one sequence per graph (models/gt_graph_level.py:276-363; class ``GT`` there).
    The node rows are the summed embeddings of the integer features, the edges of all graphs of the batch
    index the flattened [b * s] axis, the graph representation is the mean over all s rows (padding included,
    as in the reference) and the readout is ``MLPReadout``.  ``graph_token`` is constructed and not used."""

    def __init__(self, n_layers, num_heads, hidden_dim, dropout_rate, intput_dropout_rate, ffn_dim, dataset_name, edge_type,
                 multi_hop_max_dist, attention_dropout_rate, output_dim):
        super().__init__()
        num_atoms = {"ZINC": 64, "MalNet": 560000}.get(dataset_name, 7000)          # :294-315
        self.embedding_h = nn.Embedding(num_atoms, hidden_dim)
        self.graph_token = nn.Embedding(1, hidden_dim)
        self.input_dropout = nn.Dropout(intput_dropout_rate)
        self.layers = nn.ModuleList([GraphLevelEncoderLayer(hidden_dim, ffn_dim, dropout_rate, attention_dropout_rate, num_heads)
                                     for _ in range(n_layers)])
        self.MLP_layer = MLPReadout(hidden_dim, output_dim)
        self.apply(lambda module: init_params(module, n_layers=n_layers))

    def forward(self, batched_data, perturb=None, attn_type=None):
        x = EmbeddingSumFunction.apply(batched_data.x, self.embedding_h.weight)     # :334
        output = self.input_dropout(x)
        edge_index = batched_data.edge_index
        for enc_layer in self.layers:
            output = enc_layer(output, edge_index=edge_index, attn_type=attn_type)
        output = output.mean(dim=1)                                                 # :357
        return self.MLP_layer(output)
