"""Pins of oracle.graph_level (CPU): library routines, closed forms and invariances."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import graph_level as ogl

H, HID, FFN, OUT = 4, 16, 24, 3
NUM = dict(atoms=11, edges=6, spatial=9, in_deg=7, out_deg=7, edge_dis=5)


def make_params(n_layers, seed=0, multi_hop=False):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * 0.3
    p = {"graph_node_feature.atom_encoder.weight": r(NUM["atoms"], HID),
         "graph_node_feature.in_degree_encoder.weight": r(NUM["in_deg"], HID),
         "graph_node_feature.out_degree_encoder.weight": r(NUM["out_deg"], HID),
         "graph_node_feature.graph_token.weight": r(1, HID),
         "graph_attn_bias.spatial_pos_encoder.weight": r(NUM["spatial"], H),
         "graph_attn_bias.edge_encoder.weight": r(NUM["edges"], H),
         "graph_attn_bias.graph_token_virtual_distance.weight": r(1, H),
         "final_ln.weight": 1 + r(HID), "final_ln.bias": r(HID),
         "downstream_out_proj.weight": r(OUT, HID), "downstream_out_proj.bias": r(OUT)}
    if multi_hop:
        p["graph_attn_bias.edge_dis_encoder.weight"] = r(NUM["edge_dis"] * H * H, 1)
    for l in range(n_layers):
        pre = f"layers.{l}."
        for nm in ("self_attention_norm", "ffn_norm"):
            p[pre + nm + ".weight"], p[pre + nm + ".bias"] = 1 + r(HID), r(HID)
        for nm in ("linear_q", "linear_k", "linear_v", "output_layer"):
            p[pre + "self_attention." + nm + ".weight"], p[pre + "self_attention." + nm + ".bias"] = r(HID, HID), r(HID)
        p[pre + "ffn.layer1.weight"], p[pre + "ffn.layer1.bias"] = r(FFN, HID), r(FFN)
        p[pre + "ffn.layer2.weight"], p[pre + "ffn.layer2.bias"] = r(HID, FFN), r(HID)
    return p


def make_batch(sizes, s, seed=1, Fx=2, Fe=1, D0=3):
    """Random small graphs padded to s nodes in the collator's conventions (data/collator.py:50-76): ids + 1 with
    0 = padding, -inf bias on padded key columns."""
    rng = np.random.default_rng(seed)
    b = len(sizes)
    x = np.zeros((b, s, Fx), np.int64)
    ind = np.zeros((b, s), np.int64)
    outd = np.zeros((b, s), np.int64)
    sp = np.zeros((b, s, s), np.int64)
    et = np.zeros((b, s, s, Fe), np.int64)
    ei = np.zeros((b, s, s, D0, Fe), np.int64)
    ab = np.zeros((b, s + 1, s + 1))
    for g, n in enumerate(sizes):
        x[g, :n] = rng.integers(1, NUM["atoms"], size=(n, Fx))
        ind[g, :n] = rng.integers(1, NUM["in_deg"], size=n)
        outd[g, :n] = rng.integers(1, NUM["out_deg"], size=n)
        sp[g, :n, :n] = rng.integers(1, NUM["spatial"], size=(n, n))
        et[g, :n, :n] = rng.integers(0, NUM["edges"], size=(n, n, Fe))
        ei[g, :n, :n] = rng.integers(0, NUM["edges"], size=(n, n, D0, Fe))
        ab[g, :, n + 1:] = -np.inf
    t = torch.from_numpy
    return {"x": t(x), "in_degree": t(ind), "out_degree": t(outd), "spatial_pos": t(sp), "attn_edge_type": t(et),
            "edge_input": t(ei), "attn_bias": t(ab)}


def test_graph_node_feature_against_embedding_and_known_answer():
    p = make_params(0)
    batch = make_batch([3, 5], 5)
    got = ogl.graph_node_feature(batch["x"], batch["in_degree"], batch["out_degree"], p["graph_node_feature.atom_encoder.weight"],
                                 p["graph_node_feature.in_degree_encoder.weight"], p["graph_node_feature.out_degree_encoder.weight"],
                                 p["graph_node_feature.graph_token.weight"])
    want = F.embedding(batch["x"], p["graph_node_feature.atom_encoder.weight"]).sum(-2) \
        + F.embedding(batch["in_degree"], p["graph_node_feature.in_degree_encoder.weight"]) \
        + F.embedding(batch["out_degree"], p["graph_node_feature.out_degree_encoder.weight"])
    assert got.shape == (2, 6, HID)
    torch.testing.assert_close(got[:, 1:], want, rtol=0, atol=1e-14)
    torch.testing.assert_close(got[:, 0], p["graph_node_feature.graph_token.weight"].expand(2, HID), rtol=0, atol=0)
    # hand-computed: tables whose row r is the constant r (times 1, 10, 100); token 7
    a = torch.arange(4, dtype=torch.float64).unsqueeze(1).repeat(1, 2)
    out = ogl.graph_node_feature(torch.tensor([[[1, 3], [2, 0]]]), torch.tensor([[2, 1]]), torch.tensor([[3, 0]]),
                                 a, 10 * a, 100 * a, torch.full((1, 2), 7.0))
    assert out.tolist() == [[[7.0, 7.0], [324.0, 324.0], [12.0, 12.0]]]


def _library_model(p, batch, n_layers, edge_type, mhd):
    """The same network from torch's own routines (layer_norm, linear, gelu, softmax, embedding)."""
    x = torch.cat([p["graph_node_feature.graph_token.weight"].unsqueeze(0).expand(batch["x"].shape[0], 1, HID),
                   F.embedding(batch["x"], p["graph_node_feature.atom_encoder.weight"]).sum(-2)
                   + F.embedding(batch["in_degree"], p["graph_node_feature.in_degree_encoder.weight"])
                   + F.embedding(batch["out_degree"], p["graph_node_feature.out_degree_encoder.weight"])], 1)
    b, S = x.shape[:2]
    ab = batch["attn_bias"]
    bias = (2 * ab).unsqueeze(1).repeat(1, H, 1, 1)
    t = p["graph_attn_bias.graph_token_virtual_distance.weight"].view(1, H, 1)
    bias[:, :, 1:, 0] += t
    bias[:, :, 0, :] += t
    inner = F.embedding(batch["spatial_pos"], p["graph_attn_bias.spatial_pos_encoder.weight"])            # [b, s, s, H]
    if edge_type == "multi_hop":
        ei = batch["edge_input"][:, :, :, :mhd] if mhd > 0 else batch["edge_input"]
        m = F.embedding(ei, p["graph_attn_bias.edge_encoder.weight"]).mean(-2)                            # [b, s, s, D, H]
        W = p["graph_attn_bias.edge_dis_encoder.weight"].reshape(-1, H, H)[:m.shape[3]]
        hops = batch["spatial_pos"].clone()
        hops[hops == 0] = 1
        hops = torch.where(hops > 1, hops - 1, hops)
        if mhd > 0:
            hops = hops.clamp(0, mhd)
        inner = inner + torch.einsum("bijdk,dkh->bijh", m, W) / hops.unsqueeze(-1)
    else:
        inner = inner + F.embedding(batch["attn_edge_type"], p["graph_attn_bias.edge_encoder.weight"]).mean(-2)
    bias[:, :, 1:, 1:] += inner.permute(0, 3, 1, 2)
    lin = lambda v, n: F.linear(v, p[n + ".weight"], p[n + ".bias"])
    for l in range(n_layers):
        pre = f"layers.{l}."
        y = F.layer_norm(x, (HID,), p[pre + "self_attention_norm.weight"], p[pre + "self_attention_norm.bias"])
        q, k, v = (lin(y, pre + "self_attention." + n).view(b, S, H, HID // H).transpose(1, 2) for n in ("linear_q", "linear_k", "linear_v"))
        a = torch.softmax(q @ k.transpose(2, 3) * (HID // H) ** 0.5 + bias, dim=-1) @ v                  # q * sqrt(d): the reference's scale
        x = x + lin(a.transpose(1, 2).reshape(b, S, HID), pre + "self_attention.output_layer")
        y = F.layer_norm(x, (HID,), p[pre + "ffn_norm.weight"], p[pre + "ffn_norm.bias"])
        x = x + lin(F.gelu(lin(y, pre + "ffn.layer1")), pre + "ffn.layer2")
    x = F.layer_norm(x, (HID,), p["final_ln.weight"], p["final_ln.bias"])
    return lin(x[:, 0], "downstream_out_proj")


def test_model_against_library_routines():
    for edge_type, mhd in (("single_hop", 0), ("multi_hop", 2), ("multi_hop", 0)):
        p = make_params(2, seed=3, multi_hop=edge_type == "multi_hop")
        batch = make_batch([4, 6, 2], 6, seed=4)
        got = ogl.graphormer_forward(p, batch, 2, H, edge_type, mhd)
        want = _library_model(p, batch, 2, edge_type, mhd)
        assert got.shape == (3, OUT) and torch.isfinite(got).all()
        torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-12)


def test_model_without_layers_is_the_head_of_the_normalised_token():
    p = make_params(0, seed=5)
    batch = make_batch([3, 1], 4, seed=6)
    got = ogl.graphormer_forward(p, batch, 0, H, "single_hop", 0)
    tok = p["graph_node_feature.graph_token.weight"][0]
    z = (tok - tok.mean()) / torch.sqrt(tok.var(unbiased=False) + 1e-5) * p["final_ln.weight"] + p["final_ln.bias"]
    want = p["downstream_out_proj.weight"] @ z + p["downstream_out_proj.bias"]
    torch.testing.assert_close(got, want.expand(2, OUT), rtol=1e-12, atol=1e-13)


def test_model_is_invariant_to_node_relabelling_and_padding():
    p = make_params(2, seed=7)
    batch = make_batch([5, 3], 5, seed=8)
    base = ogl.graphormer_forward(p, batch, 2, H, "single_hop", 0)
    # relabel the nodes of graph 0
    perm = torch.tensor([3, 0, 4, 1, 2])
    pb = {k: v.clone() for k, v in batch.items()}
    for k in ("x", "in_degree", "out_degree"):
        pb[k][0] = batch[k][0][perm]
    for k in ("spatial_pos", "attn_edge_type", "edge_input"):
        pb[k][0] = batch[k][0][perm][:, perm]
    torch.testing.assert_close(ogl.graphormer_forward(p, pb, 2, H, "single_hop", 0), base, rtol=1e-10, atol=1e-12)
    # two more padding nodes per graph
    def pad(v, dims):
        shape = list(v.shape)
        for d in dims:
            shape[d] += 2
        out = torch.zeros(shape, dtype=v.dtype)
        out[tuple(slice(0, n) for n in v.shape)] = v
        return out
    wb = {"x": pad(batch["x"], [1]), "in_degree": pad(batch["in_degree"], [1]), "out_degree": pad(batch["out_degree"], [1]),
          "spatial_pos": pad(batch["spatial_pos"], [1, 2]), "attn_edge_type": pad(batch["attn_edge_type"], [1, 2]),
          "edge_input": pad(batch["edge_input"], [1, 2])}
    ab = torch.zeros(2, 8, 8, dtype=torch.float64)
    ab[:, :6, :6] = batch["attn_bias"]
    ab[:, :, 6:] = float("-inf")
    wb["attn_bias"] = ab
    torch.testing.assert_close(ogl.graphormer_forward(p, wb, 2, H, "single_hop", 0), base, rtol=1e-10, atol=1e-12)
