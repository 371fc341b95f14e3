"""GPU parity of the encoder-layer kernels (residual add + LayerNorm, GELU) and of the
EncoderLayer / Graphormer modules with the oracle.

Error measure: max|a - b| / max|b| against float64 on the same inputs.  Bars:
float32 1e-5; bf16 2e-2 for single kernels, 3x that for whole modules (every
intermediate tensor is rounded to bf16 between kernels).
"""
import numpy as np
import pytest
import torch

from oracle import encoder_layer as E
from oracle import graph_prep as ogp
from oracle import sparse_attention as osa
from torchgt_amd import EncoderLayer, FeedForwardNetwork, Graphormer, _lib, fused_linear, nll_loss, workloads
from torchgt_amd import _ext

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def err(a, b):
    a = a.detach().double().cpu().numpy()
    b = b.detach().double().cpu().numpy() if isinstance(b, torch.Tensor) else np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    denom = np.abs(b).max()
    return np.abs(a - b).max() / (denom if denom > 0 else 1.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C", [64, 16, 128, 256])
def test_add_layer_norm_forward_backward(cuda, dtype, C):
    for N, with_r in ((1000, True), (37, False), (1, True)):
        print(f"add_layer_norm case: N={N} C={C} {dtype} residual={with_r}", flush=True)
        g = torch.Generator().manual_seed(N + C)
        x = (torch.randn(N, C, generator=g) * 2 + 0.5).to(dtype)
        r = torch.randn(N, C, generator=g).to(dtype) if with_r else None
        gamma, beta = (torch.randn(C, generator=g) + 1).to(dtype), torch.randn(C, generator=g).to(dtype)
        ds_out, dy = torch.randn(N, C, generator=g).to(dtype), torch.randn(N, C, generator=g).to(dtype)
        # float64 with torch's own layer_norm + autograd
        leaves = [t.double().requires_grad_(True) for t in ([x, r] if with_r else [x]) + [gamma, beta]]
        s_ref = leaves[0] + leaves[1] if with_r else leaves[0] * 1.0
        y_ref = torch.nn.functional.layer_norm(s_ref, (C,), leaves[-2], leaves[-1], 1e-5)
        g_ref = torch.autograd.grad([s_ref, y_ref], leaves, [ds_out.double(), dy.double()])
        cl = [t.to(cuda).requires_grad_(True) for t in ([x, r] if with_r else [x]) + [gamma, beta]]
        s, y = _ext.ops().add_layer_norm(cl[0], cl[1] if with_r else None, cl[-2], cl[-1], float(1e-5))
        g_got = torch.autograd.grad([s, y], cl, [ds_out.to(cuda), dy.to(cuda)])
        tol = TOL[dtype]
        assert err(s, s_ref) <= tol and err(y, y_ref) <= tol, (err(s, s_ref), err(y, y_ref))
        for nm, a, b in zip(["x"] + (["r"] if with_r else []) + ["gamma", "beta"], g_got, g_ref):
            assert err(a, b) <= tol, f"d{nm} err {err(a, b)}"


def test_layer_norm_rejects_unsupported_width(cuda):
    x = torch.zeros(4, 24, device=cuda)
    w = torch.ones(24, device=cuda)
    with pytest.raises(RuntimeError, match="unsupported"):
        _ext.ops().add_layer_norm(x, None, w, w, float(1e-5))          # 24 / 4 = 6 lanes: not a power of two
    with pytest.raises(RuntimeError):
        _ext.ops().gelu(torch.zeros(8))                        # CPU tensor: no fallback


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu_and_add(cuda, dtype):
    g = torch.Generator().manual_seed(0)
    u = (torch.randn(3001, 64, generator=g) * 3).to(dtype)
    dh = torch.randn(3001, 64, generator=g).to(dtype)
    ud = u.double().requires_grad_(True)
    h_ref = torch.nn.functional.gelu(ud)
    (du_ref,) = torch.autograd.grad(h_ref, ud, dh.double())
    uc = u.to(cuda).requires_grad_(True)
    h = _ext.ops().gelu(uc)
    (du,) = torch.autograd.grad(h, uc, dh.to(cuda))
    np.testing.assert_allclose(h.detach().double().cpu().numpy(), E.gelu(u.double().numpy()), rtol=0, atol=TOL[dtype] * 10)
    assert err(h, h_ref) <= TOL[dtype] and err(du, du_ref) <= TOL[dtype]
    s = _ext.ops().add(uc, dh.to(cuda))
    assert torch.equal(s.detach().cpu(), u + dh)        # one rounding of the exact sum, in either dtype


def _ref_layer(p, x, ei, H, prefix=""):
    """The layer with torch.nn.functional pieces in float64 (differentiable)."""
    F, lin = torch.nn.functional, torch.nn.functional.linear
    b, S, hidden = x.shape
    g = lambda n: p[prefix + n]
    y = F.layer_norm(x, (hidden,), g("self_attention_norm.weight"), g("self_attention_norm.bias"))
    q, k, v = (lin(y, g(f"self_attention.linear_{c}.weight"), g(f"self_attention.linear_{c}.bias")).view(b, S, H, hidden // H)
               for c in "qkv")
    o, _ = osa.sparse_attention(q, k, v, ei)
    x1 = x + lin(o.reshape(b, S, hidden), g("self_attention.output_layer.weight"), g("self_attention.output_layer.bias"))
    y = F.layer_norm(x1, (hidden,), g("ffn_norm.weight"), g("ffn_norm.bias"))
    return x1 + lin(F.gelu(lin(y, g("ffn.layer1.weight"), g("ffn.layer1.bias"))), g("ffn.layer2.weight"), g("ffn.layer2.bias"))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,ffn", [(64, 64), (64, 128), (40, 24)])
def test_ffn_operator_matches_oracle_and_the_separate_operators(cuda, dtype, hidden, ffn):
    """FeedForwardNetwork.forward as one operator (torch.ops.torchgt.ffn): against the oracle (layer2(gelu(layer1 x)),
    float32 1e-5 / bf16 2e-2) and bit for bit against linear -> gelu -> linear through the separate operators."""
    print(f"ffn case: hidden={hidden} ffn={ffn} {dtype}", flush=True)
    torch.manual_seed(hidden + ffn)
    m = FeedForwardNetwork(hidden, ffn, 0.0)
    with torch.no_grad():
        for p in m.parameters():
            p.normal_(0, 0.3)
    m = m.to(dtype)
    x = torch.randn(3, 333, hidden).to(dtype)
    dy = torch.randn(3, 333, hidden).to(dtype)
    pd = {k: v.detach().double().numpy() for k, v in m.named_parameters()}
    want = E.gelu(x.double().numpy() @ pd["layer1.weight"].T + pd["layer1.bias"]) @ pd["layer2.weight"].T + pd["layer2.bias"]
    mc = m.to(cuda)
    xc = x.to(cuda).requires_grad_(True)
    got = mc(xc)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert np.abs(got.detach().double().cpu().numpy() - want).max() <= tol * np.abs(want).max()
    grads = torch.autograd.grad(got, [xc] + list(mc.parameters()), dy.to(cuda))
    xs = x.to(cuda).requires_grad_(True)
    (u,) = fused_linear(xs, mc.layer1)
    (ys,) = fused_linear(_ext.ops().gelu(u), mc.layer2)
    assert torch.equal(got, ys)
    for a, b in zip(grads, torch.autograd.grad(ys, [xs] + list(mc.parameters()), dy.to(cuda))):
        assert torch.equal(a, b)
    # gradients against torch autograd of the same composition in float64 on the CPU
    md = FeedForwardNetwork(hidden, ffn, 0.0).double()
    md.load_state_dict({k: v.double() for k, v in m.state_dict().items()})
    xd = x.double().requires_grad_(True)
    yd = torch.nn.functional.linear(torch.nn.functional.gelu(torch.nn.functional.linear(xd, md.layer1.weight, md.layer1.bias)),
                                    md.layer2.weight, md.layer2.bias)
    for a, b in zip(grads, torch.autograd.grad(yd, [xd] + list(md.parameters()), dy.double())):
        assert (a.double().cpu() - b).abs().max() <= tol * b.abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("N,C", [(64000, 40), (1000, 47), (5, 3), (1, 1)])
def test_nll_loss_matches_oracle(cuda, dtype, N, C):
    """loss and its gradient against the oracle; float32 1e-6 (one fp32 sum of N terms in a tree), bf16: the loss is
    rounded to bf16 once (4e-3), the gradient likewise."""
    print(f"nll_loss case: N={N} C={C} {dtype}", flush=True)
    g = torch.Generator().manual_seed(N + C)
    lp = torch.log_softmax(torch.randn(N, C, generator=g), 1).to(dtype)
    t = torch.randint(0, C, (N,), generator=g)
    if N > 3:
        t[torch.randperm(N, generator=g)[: N // 10]] = -100
    want, want_grad = E.nll_loss(lp.double().numpy(), t.numpy())
    x = lp.to(cuda).requires_grad_(True)
    loss = nll_loss(x, t.to(cuda))
    assert loss.dtype == dtype and loss.dim() == 0
    (gx,) = torch.autograd.grad(loss, x, torch.tensor(2.0, dtype=dtype, device=cuda))
    tol = 1e-6 if dtype == torch.float32 else 4e-3
    assert abs(loss.item() - want) <= tol * abs(want)
    assert np.abs(gx.double().cpu().numpy() - 2.0 * want_grad).max() <= tol * np.abs(2.0 * want_grad).max()
    assert ((gx != 0).sum(1) <= 1).all()
    # the same bits from call to call, and another ignore_index
    assert torch.equal(loss, nll_loss(x, t.to(cuda)))
    if N > 3:
        t2 = torch.where(t == -100, torch.tensor(1 % C), t)
        want2, _ = E.nll_loss(lp.double().numpy(), t2.numpy(), ignore_index=0)
        got2 = nll_loss(x, t2.to(cuda), ignore_index=0).item()
        assert abs(got2 - want2) <= tol * abs(want2)


def test_nll_loss_edge_cases(cuda):
    x = torch.log_softmax(torch.randn(6, 4), 1).to(cuda).requires_grad_(True)
    every_row_ignored = nll_loss(x, torch.full((6,), -100, device=cuda))
    assert torch.isnan(every_row_ignored)                      # 0 / 0 like torch
    empty = nll_loss(torch.zeros(0, 4, device=cuda), torch.zeros(0, dtype=torch.int64, device=cuda))
    assert torch.isnan(empty)
    with pytest.raises(RuntimeError):
        nll_loss(torch.zeros(4, 3), torch.zeros(4, dtype=torch.int64))              # CPU tensors: no fallback
    with pytest.raises(RuntimeError):
        nll_loss(x, torch.zeros(6, dtype=torch.int32, device=cuda))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_encoder_layer_matches_oracle(cuda, dtype):
    torch.manual_seed(0)
    e, n_nodes = workloads.barabasi_albert()
    ei = torch.as_tensor(e)
    hidden, H = 64, 8
    m = EncoderLayer(hidden, 64, 0.0, 0.0, H, 1)
    with torch.no_grad():
        # weights large enough for the attention and the FFN to matter, small enough that scores stay inside the
        # clamp (a score within rounding distance of +-5 flips the clamp mask and with it whole gradient terms)
        for p in m.parameters():
            if p.dim() == 2:
                p.normal_(0, 0.1)
    x = torch.randn(1, n_nodes, hidden)
    if dtype == torch.bfloat16:
        x, m = x.bfloat16(), m.bfloat16()
    params = {k: v.detach().double().numpy() for k, v in m.state_dict().items()}
    want = E.encoder_layer_forward(x.double().numpy(), params, e, H)
    mc = m.to(cuda)
    xc = x.to(cuda).requires_grad_(True)
    got = mc(xc, None, ei.to(cuda), "sparse")
    tol = TOL[dtype] * (3 if dtype == torch.bfloat16 else 1)
    assert got.shape == (1, n_nodes, hidden) and got.dtype == dtype
    assert err(got, want) <= tol, err(got, want)
    # gradients against autograd through the float64 composition
    pd = {k: torch.tensor(v, requires_grad=True) for k, v in params.items()}
    xd = x.double().requires_grad_(True)
    gy = torch.randn(1, n_nodes, hidden, generator=torch.Generator().manual_seed(5)).to(dtype)
    names = sorted(pd)
    ref = torch.autograd.grad(_ref_layer(pd, xd, ei, H), [xd] + [pd[n] for n in names], gy.double())
    got_g = torch.autograd.grad(got, [xc] + [dict(mc.named_parameters())[n] for n in names], gy.to(cuda))
    ref_by = dict(zip(["x"] + names, ref))
    for nm, a, r in zip(["x"] + names, got_g, ref):
        if nm == "self_attention.linear_k.bias":       # cancels to ~0 (see test_gpu_projections): scale by the q-bias gradient
            ev = (a.detach().double().cpu() - r).abs().max().item() / ref_by["self_attention.linear_q.bias"].abs().max().item()
            # in bf16 it is the sum of 4 097 rows of dk, each rounded to bf16, whose exact sum cancels:
            # the rounding noise does not cancel, so this one quantity gets twice the module bar
            ev = ev / 2 if dtype == torch.bfloat16 else ev
        else:
            ev = err(a, r)
        assert ev <= tol, f"d{nm} err {ev}"


def test_graphormer_forward_backward_matches_oracle(cuda):
    """Graphormer-Slim of the benchmark (4 layers, hidden 64, ffn 64, 8 heads; 128-d input, 40 classes) on a
    2 000-node batch with the global node: log-probabilities against the oracle, input gradient against autograd
    through the float64 composition."""
    torch.manual_seed(1)
    rng = np.random.default_rng(3)
    S = 2000
    e, _ = workloads.power_law_graph(n=S, directed_edges=20000)        # already holds the global node 0: S + 1 nodes
    m = Graphormer(4, 8, 128, 64, 40, 1, 0.0, 0.0, 0.0, 64, 1)
    with torch.no_grad():
        for p in m.parameters():
            if p.dim() == 2 and p.shape[0] > 1:
                p.normal_(0, 0.15)
    x = torch.randn(S, 128)
    params = {k: v.detach().double().numpy() for k, v in m.state_dict().items()}
    want = E.graphormer_forward(x.double().numpy(), params, e, 4, 8)
    mc = m.to(cuda)
    xc = x.to(cuda).requires_grad_(True)
    got = mc(xc, None, torch.as_tensor(e).to(cuda), attn_type="sparse")
    assert got.shape == (S, 40)
    assert err(got, torch.as_tensor(want)) <= 1e-5, err(got, torch.as_tensor(want))
    # loss = nll of random labels, as the training loop computes it (main_sp_node_level.py); gradient of the input
    y = torch.as_tensor(rng.integers(0, 40, S))
    (gx,) = torch.autograd.grad(torch.nn.functional.nll_loss(got, y.to(cuda)), xc)
    pd = {k: torch.tensor(v) for k, v in params.items()}
    xd = x.double().requires_grad_(True)
    lin = torch.nn.functional.linear
    h = torch.cat([pd["graph_token.weight"], lin(xd, pd["node_encoder.weight"], pd["node_encoder.bias"])], 0)[None]
    for i in range(4):
        h = _ref_layer(pd, h, torch.as_tensor(e), 8, prefix=f"layers.{i}.")
    h = torch.nn.functional.layer_norm(h, (64,), pd["final_ln.weight"], pd["final_ln.bias"])
    out = torch.log_softmax(lin(h[0, 1:, :], pd["downstream_out_proj.weight"], pd["downstream_out_proj.bias"]), 1)
    (gx_ref,) = torch.autograd.grad(torch.nn.functional.nll_loss(out, y), xd)
    assert err(gx, gx_ref) <= 1e-5, err(gx, gx_ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_as_one_operator_equals_layer_op_by_op(cuda, dtype):
    """``torch.ops.torchgt.encoder_layer`` launches the kernels the modules launch one by one, in the same order on the
    same inputs: outputs and every gradient agree bit for bit (the attention is reproducible, the weight-gradient sums
    have a fixed order)."""
    torch.manual_seed(3)
    e, n_nodes = workloads.barabasi_albert()
    ei = torch.as_tensor(e).to(cuda)
    m = EncoderLayer(64, 96, 0.0, 0.0, 8, 1)
    with torch.no_grad():
        for p in m.parameters():
            if p.dim() == 2:
                p.normal_(0, 0.1)
    m = m.to(cuda, dtype)
    x = torch.randn(1, n_nodes, 64).to(cuda, dtype)
    r = torch.randn(1, n_nodes, 64).to(cuda, dtype)
    gy = torch.randn(1, n_nodes, 64).to(cuda, dtype)
    results = []
    for fused in (False, True):
        m.one_operator = fused
        for residual, defer in ((None, False), (r, True)):
            xc = x.clone().requires_grad_(True)
            rc = None if residual is None else residual.clone().requires_grad_(True)
            out = m(xc, None, ei, "sparse", residual=rc, defer_residual=defer)
            outs = list(out) if defer else [out]
            leaves = [xc] + ([rc] if rc is not None else []) + list(m.parameters())
            grads = torch.autograd.grad(outs, leaves, [gy] * len(outs))
            results.append([o.detach() for o in outs] + list(grads))
    half = len(results) // 2
    for a_case, b_case in zip(results[:half], results[half:]):
        assert len(a_case) == len(b_case)
        for a, b in zip(a_case, b_case):
            assert torch.equal(a, b)
    # in training mode with a positive dropout rate the layer runs operator by operator (torch's dropout)
    m.one_operator = True
    m.ffn_dropout.p = 0.5
    m.train()
    assert not m._one_operator(x, None, ei, "sparse")
    m.eval()
    assert m._one_operator(x, None, ei, "sparse")
