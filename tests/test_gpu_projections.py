"""GPU parity of the projections (tgt_linear_fwd / tgt_linear_bwd) and of the
MultiHeadAttention module with the oracle.

Error measure: max|a - b| / max|b| against the oracle in float64 on the same
inputs.  Bars: float32 1e-5 (fp32 matrix instructions, exact products, fp32
accumulation), bf16 2e-2 (bf16 inputs and outputs, fp32 accumulation).
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import projections as P
from torchgt_amd import MultiHeadAttention, _lib, fused_linear, get_plan, workloads
from torchgt_amd.multi_head_attention import LinearFunction

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def err(a, b):
    a = a.detach().double().cpu().numpy()
    b = np.asarray(b, np.float64)
    assert a.shape == b.shape, (a.shape, b.shape)
    denom = np.abs(b).max()
    return np.abs(a - b).max() / (denom if denom > 0 else 1.0)


def run_linear(name, N, in_f, out_f, n, dtype, cuda, seed, bias=True):
    print(f"linear case {name}: N={N} in={in_f} out={out_f} n={n} {dtype} bias={bias} seed={seed}", flush=True)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(N, in_f, generator=g).to(dtype)
    Ws = [(torch.randn(out_f, in_f, generator=g) / in_f ** 0.5).to(dtype) for _ in range(n)]
    bs = [torch.randn(out_f, generator=g).to(dtype) if bias else None for _ in range(n)]
    dys = [torch.randn(N, out_f, generator=g).to(dtype) for _ in range(n)]
    xc = x.to(cuda).requires_grad_(True)
    Wc = [W.to(cuda).requires_grad_(True) for W in Ws]
    bc = [None if b is None else b.to(cuda).requires_grad_(True) for b in bs]
    args = []
    for W, b in zip(Wc, bc):
        args += [W, b]
    ys = LinearFunction.apply(xc, *args)
    leaves = [xc] + Wc + [b for b in bc if b is not None]
    grads = torch.autograd.grad(ys, leaves, [dy.to(cuda) for dy in dys])
    tol = TOL[dtype]
    dx_ref = 0
    for j in range(n):
        y_ref = P.linear_forward(x.double().numpy(), Ws[j].double().numpy(), None if bs[j] is None else bs[j].double().numpy())
        assert ys[j].dtype == dtype
        assert err(ys[j], y_ref) <= tol, f"y{j} err {err(ys[j], y_ref)}"
        dx_j, dW_j, db_j = P.linear_backward(x.double().numpy(), Ws[j].double().numpy(), dys[j].double().numpy())
        dx_ref = dx_ref + dx_j
        assert err(grads[1 + j], dW_j) <= tol, f"dW{j} err {err(grads[1 + j], dW_j)}"
        if bias:
            assert err(grads[1 + n + j], db_j) <= tol, f"db{j} err {err(grads[1 + n + j], db_j)}"
    assert err(grads[0], dx_ref) <= tol, f"dx err {err(grads[0], dx_ref)}"
    return ys, grads


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_shapes(cuda, dtype):
    run_linear("qkv-64", 1000, 64, 64, 3, dtype, cuda, 1)
    run_linear("out-64", 777, 64, 64, 1, dtype, cuda, 2)
    run_linear("ragged-panel", 129, 64, 64, 3, dtype, cuda, 3)        # one row past a 128-row panel
    run_linear("tiny", 5, 8, 8, 2, dtype, cuda, 4)                     # narrower than one tile
    run_linear("wide", 300, 128, 192, 3, dtype, cuda, 5)               # several contraction chunks and column tiles
    run_linear("odd-tiles", 201, 72, 40, 1, dtype, cuda, 6, bias=False)  # partial chunks both ways, no bias
    run_linear("gt-128", 513, 128, 128, 3, dtype, cuda, 7)
    if dtype == torch.float32:
        run_linear("in-100-out-44", 333, 100, 44, 1, dtype, cuda, 8)     # multiples of 4 only (100-d node features)


def test_linear_weight_gradient_is_reproducible(cuda):
    """The weight gradients are summed in a fixed order: two runs give the same bits."""
    a = run_linear("repro-a", 20000, 64, 64, 3, torch.float32, cuda, 9)[1]
    b = run_linear("repro-b", 20000, 64, 64, 3, torch.float32, cuda, 9)[1]
    for ga, gb in zip(a, b):
        assert torch.equal(ga, gb)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_deferred_sums_in_one_launch_equal_the_plain_entry_points(cuda, dtype):
    """tgt_linear_bwd_deferred (two projections, one of them the 64-wide one-pass form) and tgt_layer_norm_bwd_deferred
    followed by ONE tgt_reduce_partials give the bits of tgt_linear_bwd / tgt_layer_norm_bwd."""
    L = _lib.lib()
    code = 0 if dtype == torch.float32 else 1
    g = torch.Generator().manual_seed(21)
    vp3 = ctypes.c_void_p * 3
    descs = (_lib.ReduceDesc * 3)()
    keep, pairs = [], []

    def linear(idx, N, in_f, out_f, n):
        print(f"deferred linear: N={N} in={in_f} out={out_f} n={n} {dtype}", flush=True)
        x = torch.randn(N, in_f, generator=g).to(dtype).to(cuda)
        Ws = [torch.randn(out_f, in_f, generator=g).to(dtype).to(cuda) for _ in range(n)]
        dys = [torch.randn(N, out_f, generator=g).to(dtype).to(cuda) for _ in range(n)]
        nbytes = L.tgt_linear_bwd_workspace_bytes(n, in_f, out_f)
        outs = []
        for deferred in (False, True):
            dx = torch.empty_like(x)
            dW = [torch.full_like(W, 7.0) for W in Ws]
            db = [torch.full((out_f,), 7.0, dtype=dtype, device=cuda) for _ in range(n)]
            ws = torch.empty(nbytes, dtype=torch.uint8, device=cuda)
            a = (x.data_ptr(), vp3(*[W.data_ptr() for W in Ws]), vp3(*[d.data_ptr() for d in dys]), n, N, in_f, out_f, code,
                 dx.data_ptr(), vp3(*[t.data_ptr() for t in dW]), vp3(*[t.data_ptr() for t in db]), ws.data_ptr(), nbytes, None)
            if deferred:
                _lib.check(L.tgt_linear_bwd_deferred(*a, ctypes.byref(descs[idx])))
            else:
                _lib.check(L.tgt_linear_bwd(*a))
            outs.append([dx] + dW + db)
            keep.append((ws, x, Ws, dys))
        pairs.append(outs)

    linear(0, 3000, 64, 64, 3)
    linear(1, 1111, 128, 72, 1)
    N, C = 2500, 64
    print(f"deferred LayerNorm backward: N={N} C={C} {dtype}", flush=True)
    s_ = torch.randn(N, C, generator=g).to(dtype).to(cuda)
    gam = torch.randn(C, generator=g).to(dtype).to(cuda)
    dy = torch.randn(N, C, generator=g).to(dtype).to(cuda)
    mean = s_.float().mean(1).contiguous()
    rstd = (s_.float().var(1, unbiased=False) + 1e-5).rsqrt().contiguous()
    nbytes = L.tgt_layer_norm_bwd_workspace_bytes(C)
    outs = []
    for deferred in (False, True):
        ds, dg, dbt = torch.empty_like(s_), torch.full_like(gam, 7.0), torch.full_like(gam, 7.0)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=cuda)
        a = (s_.data_ptr(), gam.data_ptr(), mean.data_ptr(), rstd.data_ptr(), dy.data_ptr(), None, N, C, code, ds.data_ptr(),
             dg.data_ptr(), dbt.data_ptr(), ws.data_ptr(), nbytes, None)
        if deferred:
            _lib.check(L.tgt_layer_norm_bwd_deferred(*a, ctypes.byref(descs[2])))
        else:
            _lib.check(L.tgt_layer_norm_bwd(*a))
        outs.append([ds, dg, dbt])
        keep.append(ws)
    pairs.append(outs)
    assert [d.n for d in descs] == [3 * (64 * 64 + 64), 128 * 72 + 72, 2 * C]
    _lib.check(L.tgt_reduce_partials(descs, 3, code, None))
    torch.cuda.synchronize()
    for plain, later in pairs:
        for a, b in zip(plain, later):
            assert torch.equal(a, b)
    assert L.tgt_reduce_partials(descs, 9, code, None) == _lib.ERR_INVALID_ARG
    assert L.tgt_reduce_partials((_lib.ReduceDesc * 1)(), 1, code, None) == _lib.ERR_INVALID_ARG      # not filled in
    assert L.tgt_linear_bwd_deferred(None, None, None, 1, 0, 64, 64, code, None, None, None, None, 0, None, None) == _lib.ERR_INVALID_ARG


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("act", ["gelu", "relu"])
@pytest.mark.parametrize("N,in_f,out_f", [(3000, 64, 64), (70, 64, 64), (257, 64, 128), (100, 128, 64)])
def test_linear_with_activation_equals_linear_then_activation(cuda, dtype, act, N, in_f, out_f):
    """tgt_linear_act_fwd / tgt_linear_act_bwd (the activation in the epilogue of the 64 -> 64 kernels; two launches for
    other shapes) give the bits of tgt_linear_fwd + tgt_gelu_fwd and of tgt_linear_bwd + tgt_gelu_bwd, which the
    other tests hold against the oracle."""
    print(f"linear+activation case: N={N} in={in_f} out={out_f} {act} {dtype}", flush=True)
    L = _lib.lib()
    code = 0 if dtype == torch.float32 else 1
    a = 1 if act == "gelu" else 2
    fwd_act, bwd_act = (L.tgt_gelu_fwd, L.tgt_gelu_bwd) if act == "gelu" else (L.tgt_relu_fwd, L.tgt_relu_bwd)
    g = torch.Generator().manual_seed(N + out_f)
    vp3 = ctypes.c_void_p * 3
    x = torch.randn(N, in_f, generator=g).to(dtype).to(cuda)
    W1 = (torch.randn(out_f, in_f, generator=g) / in_f ** 0.5).to(dtype).to(cuda)
    b1 = torch.randn(out_f, generator=g).to(dtype).to(cuda)
    # forward
    u0, h0, u1, h1 = (torch.empty(N, out_f, dtype=dtype, device=cuda) for _ in range(4))
    _lib.check(L.tgt_linear_fwd(x.data_ptr(), vp3(W1.data_ptr()), vp3(b1.data_ptr()), vp3(u0.data_ptr()), 1, N, in_f, out_f, code, None))
    _lib.check(fwd_act(u0.data_ptr(), N * out_f, code, h0.data_ptr(), None))
    _lib.check(L.tgt_linear_act_fwd(x.data_ptr(), W1.data_ptr(), b1.data_ptr(), N, in_f, out_f, code, a, u1.data_ptr(), h1.data_ptr(), None))
    assert torch.equal(u0, u1) and torch.equal(h0, h1)
    # backward of the next layer: its input is h = act(u), [N, out_f] -> [N, in_f]
    W2 = (torch.randn(in_f, out_f, generator=g) / out_f ** 0.5).to(dtype).to(cuda)
    dy = torch.randn(N, in_f, generator=g).to(dtype).to(cuda)
    nbytes = L.tgt_linear_bwd_workspace_bytes(1, out_f, in_f)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=cuda)
    dh, du0, du1 = (torch.empty(N, out_f, dtype=dtype, device=cuda) for _ in range(3))
    dW0, dW1 = torch.empty_like(W2), torch.empty_like(W2)
    db0, db1 = (torch.empty(in_f, dtype=dtype, device=cuda) for _ in range(2))
    _lib.check(L.tgt_linear_bwd(h0.data_ptr(), vp3(W2.data_ptr()), vp3(dy.data_ptr()), 1, N, out_f, in_f, code, dh.data_ptr(),
                                vp3(dW0.data_ptr()), vp3(db0.data_ptr()), ws.data_ptr(), nbytes, None))
    _lib.check(bwd_act(u0.data_ptr(), dh.data_ptr(), N * out_f, code, du0.data_ptr(), None))
    _lib.check(L.tgt_linear_act_bwd(h0.data_ptr(), W2.data_ptr(), dy.data_ptr(), u0.data_ptr(), N, out_f, in_f, code, a, du1.data_ptr(),
                                    dW1.data_ptr(), db1.data_ptr(), ws.data_ptr(), nbytes, None, None))
    torch.cuda.synchronize()
    assert torch.equal(du0, du1) and torch.equal(dW0, dW1) and torch.equal(db0, db1)
    assert L.tgt_linear_act_fwd(x.data_ptr(), W1.data_ptr(), None, N, in_f, out_f, code, 3, u1.data_ptr(), h1.data_ptr(), None) == _lib.ERR_INVALID_ARG


def test_linear_empty_input(cuda):
    x = torch.zeros(0, 64, device=cuda, requires_grad=True)
    W = torch.randn(64, 64, device=cuda, requires_grad=True)
    b = torch.randn(64, device=cuda, requires_grad=True)
    (y,) = LinearFunction.apply(x, W, b)
    assert y.shape == (0, 64)
    dx, dW, db = torch.autograd.grad(y, [x, W, b], torch.zeros(0, 64, device=cuda))
    assert dx.shape == (0, 64) and not dW.any() and not db.any()


def test_linear_rejects_bad_arguments(cuda):
    L = _lib.lib()
    arr = (ctypes.c_void_p * 3)()
    x = torch.zeros(16, 10, device=cuda)
    W = torch.zeros(8, 10, device=cuda)
    y = torch.zeros(16, 8, device=cuda)
    arr_w = (ctypes.c_void_p * 3)(W.data_ptr())
    arr_y = (ctypes.c_void_p * 3)(y.data_ptr())
    assert L.tgt_linear_fwd(x.data_ptr(), arr_w, arr, arr_y, 1, 16, 10, 8, 0, None) == _lib.ERR_UNSUPPORTED   # 10 % 4
    assert L.tgt_linear_fwd(x.data_ptr(), arr_w, arr, arr_y, 4, 16, 16, 8, 0, None) == _lib.ERR_INVALID_ARG   # n_out
    assert L.tgt_linear_fwd(x.data_ptr(), arr, arr, arr_y, 1, 16, 16, 8, 0, None) == _lib.ERR_INVALID_ARG     # null weight
    assert L.tgt_linear_bwd(x.data_ptr(), arr_w, arr_y, 1, 16, 16, 8, 0, None, arr_w, None, None, 0, None) == _lib.ERR_WORKSPACE
    with pytest.raises(RuntimeError):
        LinearFunction.apply(torch.zeros(4, 8), torch.zeros(8, 8), None)          # CPU tensors: no fallback


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_module_matches_oracle_and_reference_state_dict(cuda, dtype):
    """MultiHeadAttention(hidden 64, 8 heads) on the 4 097-node configuration-1 graph:
    forward against the oracle's module forward; parameter names are the reference's."""
    torch.manual_seed(0)
    e, n_nodes = workloads.barabasi_albert()
    ei = torch.as_tensor(e)
    hidden, H = 64, 8
    m = MultiHeadAttention(hidden, 0.0, H, 1)
    assert sorted(m.state_dict()) == sorted(
        f"{l}.{p}" for l in ("linear_q", "linear_k", "linear_v", "output_layer") for p in ("weight", "bias"))
    x = torch.randn(1, n_nodes, hidden)
    if dtype == torch.bfloat16:      # the oracle sees the rounded values
        x = x.bfloat16()
        m = m.bfloat16()
    params = {k: v.detach().double().numpy() for k, v in m.state_dict().items()}
    want = P.multi_head_attention_forward(x.double().numpy(), params, ei.numpy(), H)
    mc = m.to(cuda)
    xc = x.to(cuda).requires_grad_(True)
    got = mc(xc, None, ei.to(cuda), "sparse")
    assert got.shape == (1, n_nodes, hidden) and got.dtype == dtype
    assert err(got, want) <= TOL[dtype], err(got, want)
    # backward against torch autograd through the oracle's pieces in float64
    from oracle import sparse_attention as osa
    xd = x.double().requires_grad_(True)
    pd = {k: torch.tensor(v, requires_grad=True) for k, v in params.items()}
    lin = torch.nn.functional.linear
    q, k, v = (lin(xd[0], pd[f"linear_{c}.weight"], pd[f"linear_{c}.bias"]).view(1, n_nodes, H, hidden // H) for c in "qkv")
    o, _ = osa.sparse_attention(q, k, v, ei)
    y = lin(o.reshape(n_nodes, hidden), pd["output_layer.weight"], pd["output_layer.bias"])
    gy = torch.randn(n_nodes, hidden, generator=torch.Generator().manual_seed(5)).to(dtype)
    names = sorted(pd)
    ref = torch.autograd.grad(y, [xd] + [pd[n] for n in names], gy.double())
    got_g = torch.autograd.grad(got, [xc] + [dict(mc.named_parameters())[n] for n in names], gy.to(cuda).view(1, n_nodes, hidden))
    # the bf16 module rounds q, k, v, the attention output and every gradient to bf16 between its four kernels
    tol = TOL[dtype] * (3 if dtype == torch.bfloat16 else 1)
    ref_by_name = dict(zip(["x"] + names, ref))
    for nm, a, r in zip(["x"] + names, got_g, ref):
        if nm == "linear_k.bias":
            # shifting every key by one vector shifts all scores of a destination alike, which the
            # normalisation cancels: this gradient is a sum of terms that cancel to ~0, so it is
            # measured against the size of the query-bias gradient (same terms, no cancellation)
            scale = ref_by_name["linear_q.bias"].abs().max().item()
            e = (a.detach().double().cpu() - r).abs().max().item() / scale
        else:
            e = err(a, r.numpy())
        assert e <= tol, f"d{nm} err {e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("with_output_layer", [True, False])
def test_module_as_one_operator_equals_operator_by_operator(cuda, dtype, with_output_layer):
    """torch.ops.torchgt.multi_head_attention (projections, sparse attention, output layer: one operator, one autograd
    node, one launch for the weight-gradient sums) gives the bits of the three operators one after the other."""
    torch.manual_seed(3)
    e, n_nodes = workloads.barabasi_albert()
    ei = torch.as_tensor(e).to(cuda)
    m = (MultiHeadAttention(64, 0.0, 8, 1) if with_output_layer else MultiHeadAttention(64, 0.0, 8)).to(cuda, dtype)
    x = torch.randn(1, n_nodes, 64, device=cuda).to(dtype)
    gy = torch.randn(1, n_nodes, 64, device=cuda).to(dtype)
    results = []
    for one in (True, False):
        m.one_operator = one
        xc = x.clone().requires_grad_(True)
        y = m(xc, None, ei, "sparse")
        results.append([y] + list(torch.autograd.grad(y, [xc] + list(m.parameters()), gy)))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    # rows that do not match the plan are refused before any kernel runs
    m.one_operator = True
    with pytest.raises(RuntimeError, match="plan was built for"):
        m(x[:, :-1], None, get_plan(ei, n_nodes), "sparse")


def test_module_without_output_layer(cuda):
    """GT flavour (no attn_bias_dim): no output layer, output = attention output."""
    m = MultiHeadAttention(64, 0.0, 8).to(cuda)
    assert m.output_layer is None
    e, n_nodes = workloads.barabasi_albert()
    ei = torch.as_tensor(e)
    x = torch.randn(1, n_nodes, 64, generator=torch.Generator().manual_seed(1))
    params = {k: v.detach().double().cpu().numpy() for k, v in m.state_dict().items()}
    want = P.multi_head_attention_forward(x.double().numpy(), params, ei.numpy(), 8)
    got = m(x.to(cuda), None, ei.to(cuda), "sparse")
    assert err(got, want) <= 1e-5


def test_fused_linear_pads_widths_that_do_not_fit(cuda):
    """47 classes / 100-d bf16 features: the module-level helper pads to the vector width and slices back."""
    for dtype, in_f, out_f in ((torch.float32, 64, 47), (torch.bfloat16, 100, 47)):
        torch.manual_seed(0)
        lin = torch.nn.Linear(in_f, out_f).to(dtype)
        x = torch.randn(301, in_f).to(dtype)
        dy = torch.randn(301, out_f).to(dtype)
        xd = x.double().requires_grad_(True)
        Wd, bd = lin.weight.detach().double().requires_grad_(True), lin.bias.detach().double().requires_grad_(True)
        ref = torch.autograd.grad(torch.nn.functional.linear(xd, Wd, bd), [xd, Wd, bd], dy.double())
        lc = lin.to(cuda)
        xc = x.to(cuda).requires_grad_(True)
        (y,) = fused_linear(xc, lc)
        assert y.shape == (301, out_f)
        got = torch.autograd.grad(y, [xc, lc.weight, lc.bias], dy.to(cuda))
        assert err(y, torch.nn.functional.linear(xd, Wd, bd).detach().numpy()) <= TOL[dtype]
        for a, r in zip(got, ref):
            assert a.shape == r.shape and err(a, r.numpy()) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_at_the_row_count_of_the_largest_configuration(cuda, dtype):
    """870 001 rows (configs[2]), q/k/v shape: the float64 oracle is out of reach at this size, so the outputs and the
    input gradient are held against float64 products on a sample of rows, and the weight gradients - sums over all
    rows - against torch's float64 matmul on the GPU (an independent library routine)."""
    N, n = 870001, 3
    print(f"linear at N={N} x{n} {dtype}", flush=True)
    g = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(N, 64, device=cuda, generator=g).to(dtype).requires_grad_(True)
    Ws = [(torch.randn(64, 64, device=cuda, generator=g) / 8).to(dtype).requires_grad_(True) for _ in range(n)]
    bs = [torch.randn(64, device=cuda, generator=g).to(dtype).requires_grad_(True) for _ in range(n)]
    dys = [torch.randn(N, 64, device=cuda, generator=g).to(dtype) for _ in range(n)]
    args = []
    for W, b in zip(Ws, bs):
        args += [W, b]
    ys = LinearFunction.apply(x, *args)
    grads = torch.autograd.grad(ys, [x] + Ws + bs, dys)
    tol = TOL[dtype]
    rows = torch.cat([torch.arange(0, 70, device=cuda), torch.randint(0, N, (2000,), device=cuda, generator=g),
                      torch.arange(N - 70, N, device=cuda)])
    xd = x.detach().double()
    dx_ref = 0
    for j in range(n):
        Wd, dyd = Ws[j].detach().double(), dys[j].double()
        y_ref = xd[rows] @ Wd.T + bs[j].detach().double()
        assert ((ys[j][rows].double() - y_ref).abs().max() / y_ref.abs().max()).item() <= tol
        dx_ref = dx_ref + dyd[rows] @ Wd
        dW_ref = dyd.T @ xd
        assert ((grads[1 + j].double() - dW_ref).abs().max() / dW_ref.abs().max()).item() <= tol
        db_ref = dyd.sum(0)
        assert ((grads[1 + n + j].double() - db_ref).abs().max() / db_ref.abs().max()).item() <= tol
    assert ((grads[0][rows].double() - dx_ref).abs().max() / dx_ref.abs().max()).item() <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_module_as_one_operator_on_the_benchmark_graph(cuda, dtype):
    """The same equality at the size the benchmark runs (configs[1]: 64 001 nodes, ~530 K edges, 1001 panels of rows,
    256 partial sums per weight): one operator and three operators give the same bits, and the output is finite."""
    e, n_nodes = workloads.power_law_graph(n=64000, exponent=2.1, directed_edges=530_000, seed=42)
    print(f"module at N={n_nodes} E={e.shape[1]} {dtype}", flush=True)
    torch.manual_seed(4)
    ei = torch.as_tensor(e).to(cuda)
    m = MultiHeadAttention(64, 0.0, 8, 1).to(cuda, dtype)
    x = torch.randn(1, n_nodes, 64, device=cuda).to(dtype)
    gy = torch.randn(1, n_nodes, 64, device=cuda).to(dtype)
    results = []
    for one in (True, False):
        m.one_operator = one
        xc = x.clone().requires_grad_(True)
        y = m(xc, None, ei, "sparse")
        results.append([y] + list(torch.autograd.grad(y, [xc] + list(m.parameters()), gy)))
    for a, b in zip(*results):
        assert torch.isfinite(a).all()
        assert torch.equal(a, b)
