"""GPU parity of the graph-level model with the oracle: the GraphNodeFeature kernel (a gather and a sum: float32
1e-5, bf16 2e-2 on max|a-b| / max|b|, forward and table gradients) and the whole Graphormer of
models/graphormer_graph_level.py (forward output and the gradient of every parameter; the dense attention
runs on bf16 matrix instructions whatever the tensor type, so the bar is the bf16 one, 3x for the whole
module as for the node-level model).
"""
import types

import numpy as np
import pytest
import torch

from oracle import graph_level as ogl
from oracle import graph_prep as ogp
from torchgt_amd import _lib, workloads
from torchgt_amd.graph_level import GraphNodeFeature, Graphormer

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    assert a.shape == b.shape, (a.shape, b.shape)
    denom = b.abs().max().item()
    return (a - b).abs().max().item() / (denom if denom > 0 else 1.0)


def node_inputs(data, num_atoms, num_deg, Fx, seed):
    """Atom ids and degrees of the padded batch in the collator's conventions (ids + 1, 0 = padding)."""
    rng = np.random.default_rng(seed)
    sizes = data["n_nodes"]
    b, s = len(sizes), data["spatial_pos"].shape[1]
    x = np.zeros((b, s, Fx), np.int64)
    deg = np.zeros((b, s), np.int64)
    for g in range(b):
        n = int(sizes[g])
        x[g, :n] = rng.integers(1, num_atoms, size=(n, Fx))
        x[g, :n, Fx - 1] *= rng.random(n) < 0.7                               # some features are the padding id
        deg[g, :n] = np.minimum((data["spatial_pos"][g][:n, :n] == 2).sum(1) + 1, num_deg - 1)
    return torch.from_numpy(x), torch.from_numpy(deg)


# tables of 64 rows are summed in LDS by the backward, the molecule-sized ones (4 609 atom types, 512 degrees) with
# memory atomics
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,Fx,num_atoms,num_deg", [(64, 1, 64, 64), (64, 3, 64, 64), (40, 2, 64, 64), (64, 3, 4609, 512)])
def test_graph_node_feature_matches_oracle(cuda, dtype, C, Fx, num_atoms, num_deg):
    print(f"graph_node_feature case: C={C} Fx={Fx} tables {num_atoms}/{num_deg} {dtype}", flush=True)
    data = workloads.erdos_renyi_batch(batch=12, seed=11)
    x, deg = node_inputs(data, num_atoms, num_deg, Fx, 1)
    g = torch.Generator().manual_seed(2)
    m = GraphNodeFeature(8, num_atoms, num_deg, num_deg, C)
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(0, 0.5, generator=g)
    m = m.to(dtype)
    tabs = [p.detach().double().requires_grad_(True) for p in (m.atom_encoder.weight, m.in_degree_encoder.weight,
                                                               m.out_degree_encoder.weight, m.graph_token.weight)]
    want = ogl.graph_node_feature(x, deg, deg.flip(1) * (deg > 0), *tabs)
    mc = m.to(cuda)
    batch = types.SimpleNamespace(x=x.to(cuda), in_degree=deg.to(cuda), out_degree=(deg.flip(1) * (deg > 0)).to(cuda))
    got = mc(batch)
    assert got.shape == want.shape and got.dtype == dtype
    assert err(got, want) <= TOL[dtype], err(got, want)
    dout = torch.randn(want.shape, generator=g).to(dtype)
    ref = [r.clone() for r in torch.autograd.grad(want, tabs, dout.double())]
    for r in ref[:3]:
        assert r[0].abs().max() > 0 or r is ref[0]
        r[0] = 0                                           # nn.Embedding(padding_idx=0): row 0 gets no gradient
    got_g = torch.autograd.grad(got, [mc.atom_encoder.weight, mc.in_degree_encoder.weight, mc.out_degree_encoder.weight,
                                      mc.graph_token.weight], dout.to(cuda))
    for nm, a, r in zip(("atom", "in_degree", "out_degree", "graph_token"), got_g, ref):
        assert err(a, r) <= TOL[dtype], f"d{nm} err {err(a, r)}"
        if nm != "graph_token":
            assert not a[0].any()


def test_graph_node_feature_empty_batch_and_bad_arguments(cuda):
    m = GraphNodeFeature(8, 64, 64, 64, 64).to(cuda)
    out = m(types.SimpleNamespace(x=torch.zeros(0, 5, 1, dtype=torch.long, device=cuda),
                                  in_degree=torch.zeros(0, 5, dtype=torch.long, device=cuda),
                                  out_degree=torch.zeros(0, 5, dtype=torch.long, device=cuda)))
    assert out.shape == (0, 6, 64)
    L = _lib.lib()
    assert L.tgt_graph_node_feature_fwd(None, None, None, 0, None, 1, None, 1, None, 1, None, 1, 1, 8, 0, None, None) \
        == _lib.ERR_INVALID_ARG
    with pytest.raises(RuntimeError):
        GraphNodeFeature(8, 64, 64, 64, 64)(types.SimpleNamespace(x=torch.zeros(1, 5, 1, dtype=torch.long),
                                                                  in_degree=torch.zeros(1, 5, dtype=torch.long),
                                                                  out_degree=torch.zeros(1, 5, dtype=torch.long)))


def _edge_input(data, D0):
    sizes = data["n_nodes"]
    b, s = len(sizes), data["spatial_pos"].shape[1]
    out = np.zeros((b, s, s, D0, 1), np.int64)
    for g in range(b):
        n = int(sizes[g])
        adj = (data["spatial_pos"][g][:n, :n] == 2).astype(np.int64)
        _, path = ogp.floyd_warshall(adj)
        out[g, :n, :n] = ogp.gen_edge_input(D0, path, (data["edge_type"][g][:n, :n] * adj)[:, :, None]) + 1
    return torch.from_numpy(out)


@pytest.mark.parametrize("edge_type,dtype,from_ids", [("single_hop", torch.float32, False), ("multi_hop", torch.float32, False),
                                                      ("single_hop", torch.bfloat16, False), ("single_hop", torch.bfloat16, True)])
def test_graph_level_graphormer_matches_oracle(cuda, edge_type, dtype, from_ids):
    """Graphormer-Slim shape of the graph-level scripts (hidden 64, ffn 64, 8 heads), 3 layers, ZINC tables,
    on 12 padded ER graphs: output [b, 1] and the gradient of every parameter against float64 autograd."""
    print(f"graph-level model case: {edge_type} {dtype}", flush=True)
    n_layers, H, mhd = 3, 8, 4
    data = workloads.erdos_renyi_batch(batch=12, seed=21)
    x, deg = node_inputs(data, 64, 64, 1, 3)
    torch.manual_seed(5)
    m = Graphormer(n_layers, H, 64, 0.0, 0.0, 64, "ZINC", edge_type, mhd, 0.0, 1)
    m.bias_from_ids = from_ids          # the attention kernels form the bias from ids + tables (no [b, H, S, S] tensor)
    assert sorted(k for k in m.state_dict() if not k.startswith("layers.")) == sorted(
        ["graph_node_feature.atom_encoder.weight", "graph_node_feature.in_degree_encoder.weight",
         "graph_node_feature.out_degree_encoder.weight", "graph_node_feature.graph_token.weight",
         "graph_attn_bias.edge_encoder.weight", "graph_attn_bias.spatial_pos_encoder.weight",
         "graph_attn_bias.graph_token_virtual_distance.weight", "final_ln.weight", "final_ln.bias",
         "downstream_out_proj.weight", "downstream_out_proj.bias"]
        + (["graph_attn_bias.edge_dis_encoder.weight"] if edge_type == "multi_hop" else []))
    assert sorted(k[len("layers.0."):] for k in m.state_dict() if k.startswith("layers.0.")) == sorted(
        f"{a}.{w}" for a in ("self_attention_norm", "ffn_norm", "self_attention.linear_q", "self_attention.linear_k",
                             "self_attention.linear_v", "self_attention.output_layer", "ffn.layer1", "ffn.layer2")
        for w in ("weight", "bias"))
    # the reference's init (std 0.02) leaves the attention flat: larger weights, but queries and keys small enough that
    # the scores (the reference multiplies q by sqrt(d)) stay within a few units, where bf16 products mean something
    with torch.no_grad():
        for k, p in m.named_parameters():
            if p.dim() == 2:
                p.normal_(0, 0.3 if "graph_attn_bias" in k else (0.05 if "linear_q" in k or "linear_k" in k else 0.15))
        m.graph_node_feature.atom_encoder.weight[0] = 0
        m.graph_attn_bias.spatial_pos_encoder.weight[0] = 0
        m.graph_attn_bias.edge_encoder.weight[0] = 0
    m = m.to(dtype)
    names = [k for k, _ in m.named_parameters()]
    pd = {k: v.detach().double().requires_grad_(True) for k, v in m.named_parameters()}
    batch = {"x": x, "in_degree": deg, "out_degree": deg, "attn_bias": torch.from_numpy(data["attn_bias"]).double(),
             "spatial_pos": torch.from_numpy(data["spatial_pos"]).long(),
             "attn_edge_type": torch.from_numpy(data["edge_type"]).long().unsqueeze(-1), "edge_input": _edge_input(data, 5)}
    want = ogl.graphormer_forward(pd, batch, n_layers, H, edge_type, mhd)
    target = torch.randn(want.shape, generator=torch.Generator().manual_seed(6)).double()
    ref = torch.autograd.grad(((want - target) ** 2).mean(), [pd[k] for k in names], allow_unused=True)
    mc = m.to(cuda)
    cb = types.SimpleNamespace(**{k: v.to(cuda) for k, v in batch.items()})
    cb.attn_bias = cb.attn_bias.to(dtype)
    got = mc(cb)
    assert got.shape == want.shape == (12, 1) and got.dtype == dtype
    tol = 3 * TOL[torch.bfloat16]
    assert err(got, want) <= tol, err(got, want)
    loss = ((got.double() - target.to(cuda)) ** 2).mean()
    got_g = torch.autograd.grad(loss, [p for _, p in mc.named_parameters()], allow_unused=True)
    scale = max(r.abs().max().item() for r in ref if r is not None)
    checked, errs = 0, {}
    for k, a, r in zip(names, got_g, ref):
        assert (a is None) == (r is None), k
        if r is None:
            continue
        r = r.clone()
        if k.endswith(("atom_encoder.weight", "in_degree_encoder.weight", "out_degree_encoder.weight", "spatial_pos_encoder.weight",
                       "edge_encoder.weight")):
            r[0] = 0                               # padding index rows
        if r.abs().max().item() < 1e-3 * scale:
            # e.g. the key bias: a constant added to every key shifts all scores of a row alike and the softmax
            # cancels it; the float64 gradient is rounding noise there, so only the size is checked
            assert a.detach().double().abs().max().item() <= 2e-2 * scale, k
            continue
        errs[k] = err(a, r)
        checked += 1
    print("forward err", err(got, want), "gradient errs", {k: round(v, 4) for k, v in errs.items()}, flush=True)
    bad = {k: v for k, v in errs.items() if v > tol}
    assert not bad, bad
    assert checked >= len(names) - n_layers - 2


def test_graph_level_graphormer_with_molecule_sized_tables(cuda):
    """The table sizes of the reference's molecule datasets (4 609 atom types, 1 537 edge types, 512 spatial ids and
    degrees): two layers (with one, only the virtual node's query row reaches the loss and the inner bias tables get
    no gradient), forward against the oracle, and a backward that reaches every table."""
    data = workloads.erdos_renyi_batch(batch=6, seed=23)
    x, deg = node_inputs(data, 4609, 512, 3, 4)
    torch.manual_seed(8)
    m = Graphormer(2, 8, 64, 0.0, 0.0, 64, "ogbg-molhiv", "single_hop", 5, 0.0, 2)
    with torch.no_grad():
        for k, p in m.named_parameters():
            if p.dim() == 2:
                p.normal_(0, 0.3 if "graph_attn_bias" in k else (0.05 if "linear_q" in k or "linear_k" in k else 0.15))
    pd = {k: v.detach().double() for k, v in m.named_parameters()}
    batch = {"x": x, "in_degree": deg, "out_degree": deg, "attn_bias": torch.from_numpy(data["attn_bias"]).double(),
             "spatial_pos": torch.from_numpy(data["spatial_pos"]).long() * 20,
             "attn_edge_type": torch.from_numpy(data["edge_type"]).long().unsqueeze(-1) * 300}
    want = ogl.graphormer_forward(pd, batch, 2, 8, "single_hop", 5)
    mc = m.to(cuda)
    cb = types.SimpleNamespace(**{k: v.to(cuda) for k, v in batch.items()}, edge_input=None)
    cb.attn_bias = cb.attn_bias.float()
    got = mc(cb)
    assert got.shape == (6, 2) and err(got, want) <= 3 * TOL[torch.bfloat16], err(got, want)
    got.square().sum().backward()
    for k, p in mc.named_parameters():
        assert p.grad is not None and p.grad.shape == p.shape and torch.isfinite(p.grad).all(), k
    assert mc.graph_node_feature.atom_encoder.weight.grad[1:].any()
    assert mc.graph_attn_bias.edge_encoder.weight.grad[300].any() and mc.graph_attn_bias.spatial_pos_encoder.weight.grad[40].any()


@pytest.mark.parametrize("dtype,from_ids", [(torch.bfloat16, True), (torch.bfloat16, False), (torch.float32, False)])
def test_dense_layer_as_one_operator_equals_layer_op_by_op(cuda, dtype, from_ids):
    """``torch.ops.torchgt.dense_encoder_layer`` launches the kernels the modules launch one by one: the model's output
    and every parameter gradient agree bit for bit between the two ways of running the layers (bias tensor and bias
    from ids; the id form's table gradients are integer sums, the weight gradients have a fixed order)."""
    import types
    from torchgt_amd import workloads
    from torchgt_amd.graph_level import Graphormer
    data = workloads.erdos_renyi_batch(batch=6, seed=9)
    b, S = 6, data["S"]
    rng = np.random.default_rng(1)
    torch.manual_seed(4)
    m = Graphormer(2, 8, 64, 0.0, 0.0, 64, "ZINC", "single_hop", 5, 0.0, 1)
    with torch.no_grad():
        for p_ in m.parameters():
            if p_.dim() == 2 and p_.shape[0] > 1:
                p_.normal_(0, 0.1)
    m = m.to(cuda, dtype)
    m.bias_from_ids = from_ids
    batch = types.SimpleNamespace(
        x=torch.from_numpy(rng.integers(1, 60, size=(b, S - 1, 1))).to(cuda), in_degree=torch.from_numpy(rng.integers(1, 60, size=(b, S - 1))).to(cuda),
        out_degree=torch.from_numpy(rng.integers(1, 60, size=(b, S - 1))).to(cuda), attn_bias=torch.from_numpy(data["attn_bias"]).to(cuda, dtype),
        spatial_pos=torch.from_numpy(data["spatial_pos"]).long().to(cuda),
        attn_edge_type=torch.from_numpy(data["edge_type"]).long().unsqueeze(-1).contiguous().to(cuda), edge_input=None)
    results = []
    for fused in (False, True):
        for layer in m.layers:
            layer.one_operator = fused
        out = m(batch)
        named = list(m.named_parameters())
        grads = torch.autograd.grad(out.float().sum(), [p_ for _, p_ in named], allow_unused=True)
        results.append([("out", out.detach())] + [(n_, g_) for (n_, _), g_ in zip(named, grads) if g_ is not None])
    assert len(results[0]) == len(results[1]) and len(results[0]) > 20
    for (name, a), (_, r) in zip(*results):
        if name.startswith("graph_node_feature.") or (name.startswith("graph_attn_bias.") and not from_ids):
            # the node-feature and bias-builder backward kernels sum with floating-point atomics: equal to rounding from run to run
            assert (a.double() - r.double()).abs().max().item() <= 1e-5 * max(r.double().abs().max().item(), 1e-30), name
        else:
            assert torch.equal(a, r), name
