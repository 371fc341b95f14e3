"""Pins of oracle.gt (CPU): library routines on a complete graph, a closed form and an invariance."""
import torch
import torch.nn.functional as F

from oracle import gt as ogt

H, HID, IN, OUT = 2, 8, 5, 3


def make_params(n_layers, seed=0, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64) * scale
    p = {"node_encoder.weight": r(HID, IN), "node_encoder.bias": r(HID)}
    for l in range(n_layers):
        pre = f"layers.{l}."
        for nm in ("linear_q", "linear_k", "linear_v"):
            p[pre + "self_attention." + nm + ".weight"], p[pre + "self_attention." + nm + ".bias"] = r(HID, HID), r(HID)
        p[pre + "O.weight"], p[pre + "O.bias"] = r(HID, HID), r(HID)
        p[pre + "FFN_layer1.weight"], p[pre + "FFN_layer1.bias"] = r(2 * HID, HID), r(2 * HID)
        p[pre + "FFN_layer2.weight"], p[pre + "FFN_layer2.bias"] = r(HID, 2 * HID), r(HID)
        for nm in ("layer_norm1", "layer_norm2"):
            p[pre + nm + ".weight"], p[pre + nm + ".bias"] = 1 + r(HID), r(HID)
    dims = [HID, HID // 2, HID // 4, OUT]
    for l in range(3):
        p[f"MLP_layer.FC_layers.{l}.weight"], p[f"MLP_layer.FC_layers.{l}.bias"] = r(dims[l + 1], dims[l]), r(dims[l + 1])
    return p


def complete_graph(S):
    src, dst = torch.meshgrid(torch.arange(S), torch.arange(S), indexing="ij")
    return torch.stack([src.reshape(-1), dst.reshape(-1)])


def _library_model(p, x, n_layers):
    """Complete graph, scores inside the clamp: the sparse attention is softmax(q k^T / sqrt(d)) v up to the
    1e-6 in the denominator."""
    lin = lambda v, n: F.linear(v, p[n + ".weight"], p[n + ".bias"])
    S, d = x.shape[0], HID // H
    h = lin(x, "node_encoder")
    for l in range(n_layers):
        pre = f"layers.{l}."
        q, k, v = (lin(h, pre + "self_attention." + n).view(S, H, d).transpose(0, 1) for n in ("linear_q", "linear_k", "linear_v"))
        s = q @ k.transpose(1, 2) / d ** 0.5
        assert s.abs().max() < 5                         # the clamp of the sparse path is inactive
        a = (torch.softmax(s, -1) @ v).transpose(0, 1).reshape(S, HID)
        y = lin(a, pre + "O")
        h = F.layer_norm(h + y, (HID,), p[pre + "layer_norm1.weight"], p[pre + "layer_norm1.bias"])
        y = lin(F.relu(lin(y, pre + "FFN_layer1")), pre + "FFN_layer2")
        h = F.layer_norm(h + y, (HID,), p[pre + "layer_norm2.weight"], p[pre + "layer_norm2.bias"])
    y = h
    for l in range(2):
        y = F.relu(lin(y, f"MLP_layer.FC_layers.{l}"))
    return torch.log_softmax(lin(y, "MLP_layer.FC_layers.2"), 1)


def test_gt_against_library_routines_on_a_complete_graph():
    p = make_params(2, seed=1)
    x = torch.randn(7, IN, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    got = ogt.gt_forward(p, x, complete_graph(7), 2, H)
    want = _library_model(p, x, 2)
    assert got.shape == (7, OUT)
    # the sparse path divides by Z + 1e-6 where softmax divides by Z: relative 1e-6 / Z
    torch.testing.assert_close(got, want, rtol=0, atol=2e-6)
    torch.testing.assert_close(got.exp().sum(1), torch.ones(7, dtype=torch.float64), rtol=0, atol=1e-12)


def test_gt_without_layers_is_the_readout_of_the_encoded_features():
    p = make_params(0, seed=3)
    x = torch.randn(4, IN, generator=torch.Generator().manual_seed(4), dtype=torch.float64)
    got = ogt.gt_forward(p, x, complete_graph(4), 0, H)
    h = x @ p["node_encoder.weight"].t() + p["node_encoder.bias"]
    for l in range(2):
        h = (h @ p[f"MLP_layer.FC_layers.{l}.weight"].t() + p[f"MLP_layer.FC_layers.{l}.bias"]).clamp(min=0)
    z = h @ p["MLP_layer.FC_layers.2.weight"].t() + p["MLP_layer.FC_layers.2.bias"]
    want = z - torch.logsumexp(z, 1, keepdim=True)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-13)


def test_gt_commutes_with_node_relabelling():
    p = make_params(2, seed=5)
    g = torch.Generator().manual_seed(6)
    S = 9
    x = torch.randn(S, IN, generator=g, dtype=torch.float64)
    e = torch.randint(0, S, (2, 30), generator=g)
    e = torch.cat([e, torch.arange(S).repeat(2, 1)], 1)            # self-loops: no empty rows
    base = ogt.gt_forward(p, x, e, 2, H)
    perm = torch.randperm(S, generator=g)                          # new id of old node i is perm[i]
    xp = torch.empty_like(x)
    xp[perm] = x
    got = ogt.gt_forward(p, xp, perm[e], 2, H)
    torch.testing.assert_close(got[perm], base, rtol=1e-10, atol=1e-12)


def test_graph_level_gt_closed_form_and_batch_independence():
    g = torch.Generator().manual_seed(8)
    p = make_params(2, seed=7)
    p["embedding_h.weight"] = torch.randn(11, HID, generator=g, dtype=torch.float64) * 0.3
    b, s = 3, 5
    x = torch.randint(0, 11, (b, s, 2), generator=g)
    # without layers: readout of the mean of the summed embeddings
    got = ogt.gt_graph_level_forward(p, x, torch.zeros(2, 0, dtype=torch.long), 0, H)
    h = torch.stack([sum(p["embedding_h.weight"][int(x[gi, i, f])] for i in range(s) for f in range(2)) / s for gi in range(b)])
    want = ogt.mlp_readout(h, p)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-13)
    # edges inside the graphs only: every graph's output is what it gets alone
    edges = []
    for gi in range(b):
        e = torch.randint(0, s, (2, 8), generator=g)
        e = torch.cat([e, torch.arange(s).repeat(2, 1)], 1)
        edges.append(e + gi * s)
    full = ogt.gt_graph_level_forward(p, x, torch.cat(edges, 1), 2, H)
    for gi in range(b):
        alone = ogt.gt_graph_level_forward(p, x[gi:gi + 1], edges[gi] - gi * s, 2, H)
        torch.testing.assert_close(full[gi:gi + 1], alone, rtol=1e-10, atol=1e-12)
