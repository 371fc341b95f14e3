"""Pins oracle/encoder_layer.py and the module mirrors' parameter counts (no GPU)."""
import numpy as np
import torch

from oracle import encoder_layer as E


def test_layer_norm_matches_torch_and_closed_forms():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((7, 24)) * 3 + 1
    g, b = rng.standard_normal(24), rng.standard_normal(24)
    want = torch.nn.functional.layer_norm(torch.tensor(x), (24,), torch.tensor(g), torch.tensor(b), 1e-5).numpy()
    np.testing.assert_allclose(E.layer_norm(x, g, b), want, rtol=1e-12, atol=1e-12)
    # a constant row has zero variance: the output is beta
    np.testing.assert_allclose(E.layer_norm(np.full((2, 24), 3.7), g, b), np.tile(b, (2, 1)), atol=1e-12)
    # two values +-a: xhat = +-a / sqrt(a^2 + eps)
    a = 0.01
    y = E.layer_norm(np.array([[a, -a]]), np.ones(2), np.zeros(2))
    np.testing.assert_allclose(y, [[a / np.sqrt(a * a + 1e-5), -a / np.sqrt(a * a + 1e-5)]], rtol=1e-12)


def test_gelu_matches_torch_and_reflection_identity():
    x = np.linspace(-6, 6, 101)
    np.testing.assert_allclose(E.gelu(x), torch.nn.functional.gelu(torch.tensor(x)).numpy(), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(E.gelu(x) - E.gelu(-x), x, atol=1e-12)       # Phi(x) + Phi(-x) = 1
    assert E.gelu(np.array([0.0]))[0] == 0.0


def _params(m):
    return {k: v.detach().double().numpy() for k, v in m.state_dict().items()}


def test_encoder_layer_is_identity_when_both_blocks_output_zero():
    from torchgt_amd import EncoderLayer
    torch.manual_seed(0)
    m = EncoderLayer(16, 16, 0.0, 0.0, 4, 1)
    with torch.no_grad():
        for lin in (m.self_attention.output_layer, m.ffn.layer2):
            lin.weight.zero_(); lin.bias.zero_()
    x = np.random.default_rng(1).standard_normal((1, 6, 16))
    ei = np.array([[0, 1, 2, 3, 4, 5, 0], [1, 2, 3, 4, 5, 0, 0]])
    np.testing.assert_allclose(E.encoder_layer_forward(x, _params(m), ei, 4), x, atol=1e-14)


def test_encoder_layer_matches_torch_functional_composition():
    """The numpy restatement against the same layer written with torch.nn.functional pieces
    (layer_norm, linear, gelu) around the sparse-attention oracle."""
    from oracle import sparse_attention as osa
    from torchgt_amd import EncoderLayer
    torch.manual_seed(3)
    hidden, H, S = 16, 4, 9
    m = EncoderLayer(hidden, 24, 0.0, 0.0, H, 1).double()
    p = dict(m.state_dict())
    rng = np.random.default_rng(4)
    x = torch.tensor(rng.standard_normal((1, S, hidden)))
    ei = torch.tensor(np.stack([rng.integers(0, S, 30), rng.integers(0, S, 30)]))
    lin, F = torch.nn.functional.linear, torch.nn.functional
    y = F.layer_norm(x, (hidden,), p["self_attention_norm.weight"], p["self_attention_norm.bias"])
    q, k, v = (lin(y, p[f"self_attention.linear_{c}.weight"], p[f"self_attention.linear_{c}.bias"]).view(1, S, H, hidden // H)
               for c in "qkv")
    o, _ = osa.sparse_attention(q, k, v, ei)
    x1 = x + lin(o.reshape(1, S, hidden), p["self_attention.output_layer.weight"], p["self_attention.output_layer.bias"])
    y = F.layer_norm(x1, (hidden,), p["ffn_norm.weight"], p["ffn_norm.bias"])
    want = x1 + lin(F.gelu(lin(y, p["ffn.layer1.weight"], p["ffn.layer1.bias"])), p["ffn.layer2.weight"], p["ffn.layer2.bias"])
    got = E.encoder_layer_forward(x.numpy(), _params(m), ei.numpy(), H)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-11, atol=1e-12)


def test_graphormer_parameter_counts_and_names():
    """README.md:70,114: 111 913 parameters (128-d input, 40 classes), 110 576 (100-d, 47 classes),
    4 layers, hidden 64, ffn 64, 8 heads, one global node."""
    from torchgt_amd import Graphormer
    m = Graphormer(4, 8, 128, 64, 40, 1, 0.0, 0.0, 0.0, 64, 1)
    assert sum(p.numel() for p in m.parameters()) == 111913
    assert sum(p.numel() for p in Graphormer(4, 8, 100, 64, 47, 1, 0.0, 0.0, 0.0, 64, 1).parameters()) == 110576
    names = set(m.state_dict())
    for n in ("node_encoder.weight", "graph_token.weight", "graph_token_virtual_distance.weight", "final_ln.bias",
              "downstream_out_proj.weight", "layers.3.self_attention.linear_q.weight", "layers.0.self_attention_norm.weight",
              "layers.2.self_attention.output_layer.bias", "layers.1.ffn.layer1.weight", "layers.1.ffn_norm.weight"):
        assert n in names, n


def test_graphormer_forward_rows_are_log_probabilities():
    from torchgt_amd import Graphormer
    torch.manual_seed(0)
    m = Graphormer(2, 4, 12, 16, 5, 1, 0.0, 0.0, 0.0, 16, 1)
    rng = np.random.default_rng(2)
    S = 7
    x = rng.standard_normal((S, 12))
    from oracle import graph_prep as gp
    ei = gp.fix_edge_index(np.stack([rng.integers(0, S, 20), rng.integers(0, S, 20)]), S)
    out = E.graphormer_forward(x, _params(m), ei, 2, 4)
    assert out.shape == (S, 5)
    np.testing.assert_allclose(np.exp(out).sum(axis=1), 1.0, rtol=1e-12)


def test_nll_loss_matches_torch_and_the_uniform_closed_form():
    rng = np.random.default_rng(5)
    N, C = 37, 7
    lp = np.log(rng.dirichlet(np.ones(C), size=N))
    t = rng.integers(0, C, size=N)
    t[[3, 11, 30]] = -100
    loss, grad = E.nll_loss(lp, t)
    x = torch.tensor(lp, requires_grad=True)
    want = torch.nn.functional.nll_loss(x, torch.tensor(t))
    want.backward()
    assert abs(loss - want.item()) < 1e-12
    assert np.abs(grad - x.grad.numpy()).max() < 1e-15
    # a uniform prediction costs log C whatever the targets; a dropped sign or a division by N instead of the count shows here
    loss_u, grad_u = E.nll_loss(np.full((N, C), -np.log(C)), t)
    assert abs(loss_u - np.log(C)) < 1e-12
    assert abs(grad_u.sum() + 1.0) < 1e-12 and (grad_u[[3, 11, 30]] == 0).all()
    assert np.isnan(E.nll_loss(lp, np.full(N, -100))[0])
