"""Host-side checks of the model mirrors that need no GPU: module trees and parameter counts follow from the
reference's constructors (models/graphormer_graph_level.py:309-366, models/gt_dist_node_level.py:290-319,
models/gt_graph_level.py:276-330), and every forward refuses CPU tensors instead of falling back."""
import types

import pytest
import torch

from torchgt_amd import GT, GraphLevelGT, GraphLevelGraphormer, GraphAttnBias
from torchgt_amd.graph_level import GraphNodeFeature


def count(m):
    return sum(p.numel() for p in m.parameters())


def test_graph_level_graphormer_parameter_count_and_keys():
    L, H, hid, ffn, out = 4, 8, 64, 64, 1
    m = GraphLevelGraphormer(L, H, hid, 0.0, 0.0, ffn, "ZINC", "multi_hop", 5, 0.0, out)
    # ZINC tables (:325-331): 64 atoms, 64 in / out degrees, 64 edge types, 40 spatial ids, 40 hop matrices
    tables = (64 + 64 + 64 + 1) * hid + (64 + 40 + 1) * H + 40 * H * H
    layer = 2 * 2 * hid + 4 * (hid * hid + hid) + (hid * ffn + ffn) + (ffn * hid + hid)
    assert count(m) == tables + L * layer + 2 * hid + (hid * out + out)
    single = GraphLevelGraphormer(L, H, hid, 0.0, 0.0, ffn, "ZINC", "single_hop", 5, 0.0, out)
    assert count(m) - count(single) == 40 * H * H == 2560 and count(single) == 114249
    # the other datasets (:332-338): 512 * 9 + 1 atom rows, 512 * 3 + 1 edge rows, 512 spatial ids and degrees
    big = GraphLevelGraphormer(1, H, hid, 0.0, 0.0, ffn, "ogbg-molhiv", "single_hop", 5, 0.0, out)
    assert big.graph_node_feature.atom_encoder.weight.shape == (4609, hid)
    assert big.graph_attn_bias.edge_encoder.weight.shape == (1537, H)
    assert big.graph_attn_bias.spatial_pos_encoder.weight.shape == (512, H)
    pcq = GraphLevelGraphormer(1, H, hid, 0.0, 0.0, ffn, "PCQM4M-LSC", "single_hop", 5, 0.0, 7)
    assert "out_proj.weight" in pcq.state_dict() and pcq.out_proj.weight.shape == (1, hid)        # (:363-364)
    # the reference's init (:9-15): embeddings N(0, 0.02), linear biases zero, LayerNorm untouched
    assert float(m.layers[0].ffn.layer1.bias.detach().abs().max()) == 0 and float(m.final_ln.weight.detach().min()) == 1
    assert 0.01 < float(m.graph_node_feature.atom_encoder.weight.detach().std()) < 0.03


def test_gt_parameter_counts_and_keys():
    L, H, inp, hid, out = 4, 8, 128, 64, 40
    m = GT(L, H, inp, hid, out, 1, 0.0, 0.0, 0.0, 64, 0)
    layer = 3 * 2 * hid + 3 * (hid * hid + hid) + (hid * hid + hid) + (hid * 2 * hid + 2 * hid) + (2 * hid * hid + hid)
    readout = (hid * hid // 2 + hid // 2) + (hid // 2 * hid // 4 + hid // 4) + (hid // 4 * out + out)
    assert count(m) == (inp * hid + hid) + L * layer + readout + (hid * out + out)
    assert not any("output_layer" in k for k in m.state_dict())
    g = GraphLevelGT(L, H, hid, 0.0, 0.0, 64, "ZINC", "single_hop", 5, 0.0, 1)
    readout1 = (hid * hid // 2 + hid // 2) + (hid // 2 * hid // 4 + hid // 4) + (hid // 4 + 1)
    assert count(g) == 64 * hid + hid + L * layer + readout1
    assert GraphLevelGT(1, H, hid, 0.0, 0.0, 64, "MalNet", "x", 5, 0.0, 1).embedding_h.weight.shape == (560000, hid)
    assert GraphLevelGT(1, H, hid, 0.0, 0.0, 64, "other", "x", 5, 0.0, 1).embedding_h.weight.shape == (7000, hid)


def test_models_refuse_cpu_tensors():
    b, s = 2, 3
    batch = types.SimpleNamespace(x=torch.ones(b, s, 1, dtype=torch.long), in_degree=torch.ones(b, s, dtype=torch.long),
                                  out_degree=torch.ones(b, s, dtype=torch.long), attn_bias=torch.zeros(b, s + 1, s + 1),
                                  spatial_pos=torch.ones(b, s, s, dtype=torch.long),
                                  attn_edge_type=torch.zeros(b, s, s, 1, dtype=torch.long),
                                  edge_input=torch.zeros(b, s, s, 2, 1, dtype=torch.long),
                                  edge_index=torch.zeros(2, 4, dtype=torch.long))
    with pytest.raises(RuntimeError, match="GPU only"):
        GraphNodeFeature(8, 64, 64, 64, 64)(batch)
    for et in ("single_hop", "multi_hop"):
        with pytest.raises(RuntimeError, match="GPU only"):
            GraphAttnBias(8, 64, 64, 40, 40, 64, et, 5)(batch)
    with pytest.raises(RuntimeError, match="GPU only"):
        GraphLevelGraphormer(1, 8, 64, 0.0, 0.0, 64, "ZINC", "single_hop", 5, 0.0, 1)(batch)
    with pytest.raises(RuntimeError, match="GPU only"):
        GraphLevelGT(1, 8, 64, 0.0, 0.0, 64, "ZINC", "single_hop", 5, 0.0, 1)(batch, attn_type="sparse")
    with pytest.raises(RuntimeError):
        GT(1, 8, 16, 64, 4, 1, 0.0, 0.0, 0.0, 64, 0)(torch.zeros(5, 16), None, torch.zeros(2, 4, dtype=torch.long), attn_type="sparse")
