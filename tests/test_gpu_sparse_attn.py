"""GPU parity of the HIP sparse attention (forward and gradients) with the oracle.

Error measure: err(a, b) = max|a - b| / max|b| against the oracle evaluated in
float64 on the same (dtype-rounded) inputs.  Bars (from the task statement):
fp32 <= 1e-5, bf16 I/O with fp32 accumulation <= 2e-2, on outputs AND gradients.
"""
import math

import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa
from torchgt_amd import CoreAttention, GraphPlan, _lib, sparse_attention, workloads

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    denom = b.abs().max().item()
    return (a - b).abs().max().item() / (denom if denom > 0 else 1.0)


def make_inputs(N, E, H, d, dtype, bias_kind, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(N, H, d, generator=g) * scale for _ in range(3))
    bias = {"none": None, "edge": torch.randn(E, generator=g) * 0.5,
            "edge_head": torch.randn(E, H, generator=g) * 0.5}[bias_kind]
    dout = torch.randn(N, H, d, generator=g)
    cast = lambda t: None if t is None else t.to(dtype)
    return cast(q), cast(k), cast(v), cast(bias), cast(dout)


def oracle_fwd_bwd(q, k, v, bias, ei, dout):
    """float64 oracle on the dtype-rounded inputs (autograd of the restatement)."""
    t = [x.detach().double().cpu().requires_grad_(True) for x in (q, k, v)]
    b = None if bias is None else bias.detach().double().cpu().requires_grad_(True)
    out, Z = osa.sparse_attention(t[0], t[1], t[2], ei.cpu(), b)
    grads = torch.autograd.grad(out, t + ([b] if b is not None else []), dout.double().cpu())
    return out, Z, grads


def hip_fwd_bwd(q, k, v, bias, ei, dout, cuda):
    t = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    b = None if bias is None else bias.to(cuda).requires_grad_(True)
    out, Z = sparse_attention(t[0], t[1], t[2], ei.to(cuda), b, return_z=True)
    grads = torch.autograd.grad(out, t + ([b] if b is not None else []), dout.to(cuda))
    return out, Z, grads


def run_case(name, N, ei, H, d, dtype, bias_kind, seed, cuda, scale=1.0):
    print(f"case {name}: N={N} E={ei.shape[1]} H={H} d={d} {dtype} bias={bias_kind} seed={seed}", flush=True)
    q, k, v, bias, dout = make_inputs(N, ei.shape[1], H, d, dtype, bias_kind, seed, scale)
    o_ref, Z_ref, g_ref = oracle_fwd_bwd(q, k, v, bias, ei, dout)
    o, Z, g = hip_fwd_bwd(q, k, v, bias, ei, dout, cuda)
    tol = TOL[dtype]
    assert o.dtype == dtype and Z.dtype == torch.float32
    assert err(o, o_ref) <= tol, f"out err {err(o, o_ref)}"
    assert err(Z, Z_ref) <= (1e-5 if dtype == torch.float32 else 2e-2), f"Z err {err(Z, Z_ref)}"
    for name_g, a, b in zip(("dq", "dk", "dv", "dbias"), g, g_ref):
        assert a.dtype == dtype
        assert not torch.isnan(a).any()
        assert err(a, b) <= tol, f"{name_g} err {err(a, b)}"


def rand_graph(N, E, seed):
    return torch.randint(0, N, (2, E), generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("bias_kind", ["none", "edge", "edge_head"])
def test_config1_barabasi_albert(cuda, dtype, bias_kind):
    e, n = workloads.barabasi_albert()
    run_case("config1", n, torch.from_numpy(e), 8, 8, dtype, bias_kind, 42, cuda)


def test_config1_with_learned_spd_table(cuda):
    # benchmark config 1: per-edge scalar bias = table[spd id], table ~ N(0, 0.02), grads reach the table
    e, n = workloads.barabasi_albert()
    ids = torch.from_numpy(workloads.spd_edge_ids(e))
    ei = torch.from_numpy(e)
    g = torch.Generator().manual_seed(42)
    q, k, v = (torch.randn(1, n, 8, 8, generator=g) for _ in range(3))
    table = torch.randn(7, generator=g) * 0.02
    target = torch.randn(1, n, 64, generator=g)

    def loss_of(fn, dev, dt):
        qq, kk, vv, tt = (x.to(dev, dt).requires_grad_(True) for x in (q, k, v, table))
        out = fn(qq, kk, vv, tt[ids.to(dev)], ei.to(dev))
        loss = torch.nn.functional.mse_loss(out.reshape(1, n, 64), target.to(dev, dt))   # attn_module.py:401-407
        return (loss,) + torch.autograd.grad(loss, (qq, kk, vv, tt))

    ref = loss_of(lambda a, b, c, eb, ei_: osa.sparse_attention(a, b, c, ei_, eb)[0], "cpu", torch.float64)
    mod = CoreAttention(64, 0.0, 8, 1)
    got = loss_of(lambda a, b, c, eb, ei_: mod(a, b, c, eb, ei_, "sparse"), cuda, torch.float32)
    for a, b in zip(got, ref):
        assert err(a, b) <= 1e-5


SHAPES = [(8, 8), (4, 16), (8, 16), (16, 8), (4, 8), (2, 8), (1, 8), (2, 16), (1, 16), (4, 32), (2, 32), (1, 32)]


@pytest.mark.parametrize("H,d", SHAPES)
def test_head_shapes(cuda, H, d):
    N, E = 777, 6000
    ei = rand_graph(N, E, H * 100 + d)
    ei[1, :1500] = 3           # one split row on the destination side
    ei[0, 1500:2600] = 9       # and on the source side
    for dtype, bias_kind in ((torch.float32, "edge_head"), (torch.bfloat16, "edge"), (torch.float32, "none")):
        run_case(f"shape{H}x{d}", N, ei, H, d, dtype, bias_kind, 7, cuda)


def test_all_length_classes_and_ragged_rows(cuda):
    # rows of in-degree 0..70 (every slot width), 255..1024 (one wave / one workgroup) and 1025, 2500 (split rows)
    degs = list(range(0, 71)) + [300, 1000, 0, 0, 257, 256, 255, 1024, 1025, 2500]
    N = len(degs)
    rng = np.random.default_rng(5)
    src = np.concatenate([rng.integers(0, N, dg) for dg in degs]).astype(np.int64)
    dst = np.repeat(np.arange(N), degs).astype(np.int64)
    perm = rng.permutation(src.shape[0])
    ei = torch.from_numpy(np.stack([src[perm], dst[perm]]))
    for dtype in (torch.float32, torch.bfloat16):
        run_case("ragged", N, ei, 8, 8, dtype, "edge_head", 11, cuda)
    run_case("ragged-T", N, ei.flip(0).contiguous(), 8, 8, torch.float32, "edge", 12, cuda)


def test_large_scores_hit_the_clamp(cuda):
    N, E = 500, 5000
    ei = rand_graph(N, E, 21)
    run_case("clamp", N, ei, 8, 8, torch.float32, "edge_head", 22, cuda, scale=2.5)


def test_empty_graph_and_isolated_rows(cuda):
    N, H, d = 10, 8, 8
    q, k, v, _, dout = make_inputs(N, 0, H, d, torch.float32, "none", 1)
    ei = torch.zeros(2, 0, dtype=torch.int64)
    o, Z, g = hip_fwd_bwd(q, k, v, None, ei, dout, cuda)
    assert torch.count_nonzero(o) == 0 and torch.count_nonzero(Z) == 0
    for a in g:
        assert torch.count_nonzero(a) == 0
    # one edge 3 -> 1: only row 1 receives
    ei = torch.tensor([[3], [1]])
    o, Z, g = hip_fwd_bwd(q, k, v, None, ei, dout, cuda)
    w = math.exp(max(-5.0, min(5.0, float((k[3] * q[1]).sum(-1)[0] / math.sqrt(d)))))
    assert torch.count_nonzero(o[[0, 2, 3, 4, 5, 6, 7, 8, 9]]) == 0
    assert Z[1, 0].item() == pytest.approx(w, rel=1e-6)
    torch.testing.assert_close(o[1, 0].cpu(), v[3, 0] * (w / (w + 1e-6)), rtol=1e-6, atol=1e-7)


def test_neg_inf_bias_gives_zero_weight_and_finite_grads(cuda):
    N, E, H, d = 60, 500, 8, 8
    ei = rand_graph(N, E, 31)
    q, k, v, bias, dout = make_inputs(N, E, H, d, torch.float32, "edge_head", 32)
    bias[::3] = float("-inf")
    bias[ei[1] == 5] = float("-inf")        # a row whose every edge is masked -> exact zeros
    o_ref, Z_ref, g_ref = oracle_fwd_bwd(q, k, v, bias, ei, dout)
    o, Z, g = hip_fwd_bwd(q, k, v, bias, ei, dout, cuda)
    assert torch.count_nonzero(o[5]) == 0
    assert err(o, o_ref) <= 1e-5
    for a, b in zip(g, g_ref):
        assert not torch.isnan(a).any() and not torch.isinf(a).any()
        assert err(a, b) <= 1e-5
    assert torch.count_nonzero(g[3][::3]) == 0


def test_duplicate_edges_count_twice(cuda):
    N, H, d = 20, 8, 8
    q, k, v, _, dout = make_inputs(N, 0, H, d, torch.float32, "none", 41)
    ei = torch.tensor([[1, 1, 2, 1], [0, 0, 0, 0]])
    o, _, _ = hip_fwd_bwd(q, k, v, None, ei, dout, cuda)
    ei1 = torch.tensor([[1, 2], [0, 0]])
    b1 = torch.tensor([math.log(3.0), 0.0])
    o1, _, _ = hip_fwd_bwd(q, k, v, b1, ei1, dout, cuda)
    assert err(o, o1) <= 1e-6


def test_clamp_mask_inclusive_at_exactly_five(cuda):
    # d = 16 (scale 4): q.k = 20 -> raw == 5.0 exactly, gradient must flow; raw slightly above -> blocked
    N, H, d = 3, 1, 16
    q = torch.zeros(N, H, d)
    k = torch.zeros(N, H, d)
    v = torch.randn(N, H, d, generator=torch.Generator().manual_seed(51))
    q[0, 0, 0] = 4.0
    k[1, 0, 0] = 5.0          # raw = 5.0 exactly
    k[2, 0, 0] = 5.0000005    # raw just above 5 -> masked
    k[0, 0, 0] = -5.0         # raw = -5.0 exactly (self loop)
    ei = torch.tensor([[1, 2, 0], [0, 0, 0]])
    dout = torch.ones(N, H, d)
    o_ref, _, g_ref = oracle_fwd_bwd(q, k, v, None, ei, dout)
    o, _, g = hip_fwd_bwd(q, k, v, None, ei, dout, cuda)
    assert err(o, o_ref) <= 1e-5
    for a, b in zip(g, g_ref):
        assert err(a, b) <= 1e-5
    assert g[1][1, 0, 0].abs() > 0 and g[1][0, 0, 0].abs() > 0     # dk of the edges at exactly +-5
    assert g[1][2, 0, 0] == 0                                       # dk of the edge beyond the clamp


def test_bitwise_reproducible(cuda):
    e, n = workloads.barabasi_albert()
    ei = torch.from_numpy(e)
    q, k, v, bias, dout = make_inputs(n, e.shape[1], 8, 8, torch.float32, "edge_head", 61)
    a = hip_fwd_bwd(q, k, v, bias, ei, dout, cuda)
    b = hip_fwd_bwd(q, k, v, bias, ei, dout, cuda)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    for x, y in zip(a[2], b[2]):
        assert torch.equal(x, y)


def test_split_rows_fresh_inputs_every_call(cuda):
    """Rows long enough to be split over several workgroups (in both views), called again and
    again on ONE plan and workspace with new operands: a partial sum left over from an earlier
    call, or read before it was published, would show against the oracle."""
    N = 600
    g = torch.Generator().manual_seed(71)
    hubs = torch.arange(0, 24)
    parts = []
    for h in hubs:   # every hub receives from and sends to 1500..4500 random nodes
        deg = int(torch.randint(1500, 4500, (1,), generator=g))
        other = torch.randint(0, N, (deg,), generator=g)
        parts.append(torch.stack([other, torch.full((deg,), int(h))]))
        parts.append(torch.stack([torch.full((deg,), int(h)), other]))
    parts.append(rand_graph(N, 3000, 72))
    ei = torch.cat(parts, dim=1)
    ei = ei[:, torch.randperm(ei.shape[1], generator=g)]
    ei = ei.to(cuda)          # one tensor: the plan (and its workspace) is cached on it
    plan = GraphPlan(ei, N)
    info = plan.info()
    assert info["segments_dst"] >= 48 and info["segments_src"] >= 48
    plan.close()
    for call in range(6):
        for dtype in (torch.float32, torch.bfloat16):
            run_case(f"split rows call {call}", N, ei, 8, 8, dtype, "edge_head", 700 + call, cuda, scale=0.5)


def test_module_api_matches_reference_conventions(cuda):
    # forward(q,k,v,attn_bias,edge_index,'sparse') with [b,S,H,d] and a dense [b,H,S,S] bias,
    # sparse_attention_bias(k,q,v,...) with the k-first order, and the attn_module.py convention
    b, S, H, d = 2, 40, 8, 8
    g = torch.Generator().manual_seed(71)
    q, k, v = (torch.randn(b, S, H, d, generator=g) for _ in range(3))
    bias = torch.randn(b, H, S, S, generator=g) * 0.3
    ei = torch.cat([torch.randint(0, S, (2, 300), generator=g), torch.randint(0, S, (2, 200), generator=g) + S], 1)
    ref = osa.sparse_attention_module_forward(q.double(), k.double(), v.double(), bias.double(), ei, "bhss")
    mod = CoreAttention(H * d, 0.1, H).to(cuda)
    out = mod(q.to(cuda), k.to(cuda), v.to(cuda), bias.to(cuda), ei.to(cuda), "sparse")
    assert out.shape == (b, S, H * d)
    assert err(out, ref) <= 1e-5
    out2 = mod.sparse_attention_bias(k.to(cuda), q.to(cuda), v.to(cuda), ei.to(cuda), bias.to(cuda))
    assert out2.shape == (b * S, H, d)
    assert torch.equal(out2.reshape(b, S, -1), out)
    bench_mod = CoreAttention(H * d, 0.1, H, cuda)
    out3 = bench_mod(q.to(cuda), k.to(cuda), v.to(cuda), ei.to(cuda))
    ref3 = osa.sparse_attention_module_forward(q.double(), k.double(), v.double(), None, ei)
    assert err(out3, ref3) <= 1e-5
    # node-level layout [b, S, S, 1] broadcast over heads (graphormer_dist_node_level.py:384)
    nl = CoreAttention(H * d, 0.1, H, 1)
    bias1 = torch.randn(1, S, S, 1, generator=g) * 0.3
    ei1 = torch.randint(0, S, (2, 300), generator=g)
    ref4 = osa.sparse_attention_module_forward(q[:1].double(), k[:1].double(), v[:1].double(),
                                               bias1.double().expand(-1, -1, -1, H), ei1, "bssh")
    out4 = nl(q[:1].to(cuda), k[:1].to(cuda), v[:1].to(cuda), bias1.to(cuda), ei1.to(cuda), "sparse")
    assert err(out4, ref4) <= 1e-5


def test_loud_failures(cuda):
    q = torch.randn(10, 8, 4, device=cuda)        # d = 4: no kernel
    ei = torch.tensor([[0, 1], [1, 2]], device=cuda)
    with pytest.raises(RuntimeError, match="unsupported"):     # the C entry point's error, through the torch operator
        sparse_attention(q, q, q, ei)
    qc = torch.randn(10, 8, 8)
    with pytest.raises(RuntimeError):
        sparse_attention(qc, qc, qc, ei.cpu())     # CPU tensors: no fallback
    qh = torch.randn(10, 8, 8, device=cuda, dtype=torch.float16)
    with pytest.raises(TypeError):
        sparse_attention(qh, qh, qh, ei)
    with pytest.raises(ValueError):
        sparse_attention(torch.randn(10, 8, 8, device=cuda), q.new_zeros(10, 8, 8), q.new_zeros(10, 8, 8),
                         ei, torch.zeros(5, device=cuda))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_config2_full_size_against_oracle(cuda, dtype):
    # 64 001 nodes, ~530 K edges, H = 8, d = 8, bias [E, 8] with gradient
    e, n = workloads.power_law_graph()
    run_case("config2", n, torch.from_numpy(e), 8, 8, dtype, "edge_head", 42, cuda)


def test_config2_size_independent_properties(cuda):
    e, n = workloads.power_law_graph()
    ei = torch.from_numpy(e)
    E = e.shape[1]
    q, k, v, bias, dout = make_inputs(n, E, 8, 8, torch.float32, "edge_head", 43)
    base = hip_fwd_bwd(q, k, v, bias, ei, dout, cuda)
    # edge-order permutation invariance (a different plan, same mathematics)
    perm = torch.randperm(E, generator=torch.Generator().manual_seed(44))
    p = hip_fwd_bwd(q, k, v, bias[perm], ei[:, perm], dout, cuda)
    assert err(p[0], base[0]) <= 1e-5
    for i in range(3):
        assert err(p[2][i], base[2][i]) <= 1e-5
    assert err(p[2][3], base[2][3][perm]) <= 1e-5
    # node relabelling equivariance
    pi = torch.randperm(n, generator=torch.Generator().manual_seed(45))
    inv = torch.argsort(pi)
    r = hip_fwd_bwd(q[inv], k[inv], v[inv], bias, pi[ei], dout[inv], cuda)
    assert err(r[0][pi.to(cuda)], base[0]) <= 1e-5
    assert err(r[2][1][pi.to(cuda)], base[2][1]) <= 1e-5
    # head independence: heads 0..3 computed alone equal the same heads computed together
    h = hip_fwd_bwd(q[:, :4].contiguous(), k[:, :4].contiguous(), v[:, :4].contiguous(),
                    bias[:, :4].contiguous(), ei, dout[:, :4].contiguous(), cuda)
    assert err(h[0], base[0][:, :4]) <= 1e-6
    assert err(h[2][0], base[2][0][:, :4]) <= 1e-6
    # weights are a convex combination: out lies within the range of v over the row's sources
    assert torch.isfinite(base[0]).all()
    assert base[0].abs().max() <= v.abs().max() + 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("per_head", [True, False])
def test_bias_in_plan_order_is_the_same_computation(cuda, dtype, per_head):
    """TGT_BIAS_PLAN_ORDER: the bias permuted into the plan's destination-sorted order gives bit-identical
    outputs and gradients, and the bias gradient comes back in the caller's order (graphs with split rows,
    workgroup rows and all wave classes)."""
    from torchgt_amd import get_plan, sparse_attention
    for name, (e, n) in (("config1", workloads.barabasi_albert()),
                         ("power-law", workloads.power_law_graph(n=20000, directed_edges=200000))):
        print(f"plan-order bias case: {name} {dtype} per_head={per_head}", flush=True)
        ei = torch.from_numpy(e).to(cuda)
        E, H, d = e.shape[1], 8, 8
        g = torch.Generator().manual_seed(3)
        q, k, v, dout = (torch.randn(n, H, d, generator=g).to(cuda, dtype) for _ in range(4))
        bias = (torch.randn(E, H, generator=g) if per_head else torch.randn(E, generator=g)).to(cuda, dtype)
        plan = get_plan(ei, n)
        order = plan.edge_order()
        # the permutation is the stable sort of the destinations
        want_order = torch.sort(ei[1], stable=True).indices
        assert torch.equal(order, want_order)
        assert torch.equal(plan.edge_order_src(), torch.sort(ei[0], stable=True).indices)
        outs = []
        for sorted_mode in (None, "dst", "both"):
            t = [x.clone().requires_grad_(True) for x in (q, k, v)]
            b = bias.clone().requires_grad_(True)
            bb = b if sorted_mode is None else plan.sort_bias(b, both_orders=(sorted_mode == "both"))
            assert bb.shape[0] == (2 * E if sorted_mode == "both" else E)
            o = sparse_attention(t[0], t[1], t[2], plan=plan, edge_bias=bb, bias_in_plan_order=sorted_mode is not None)
            outs.append((o, torch.autograd.grad(o, t + [b], dout)))
        (o0, g0) = outs[0]
        for o1, g1 in outs[1:]:
            assert torch.equal(o0, o1)
            for nm, a, b_ in zip(("dq", "dk", "dv", "dbias"), g0, g1):
                assert torch.equal(a, b_), nm


def test_module_bias_cache_respects_autograd_state(cuda):
    """A leaf per-edge bias first seen under no_grad (an evaluation pass) must still get its gradient in the
    training pass that follows, and a second training step over the same bias object must not walk a freed
    graph: the module's plan-order copy of the bias is tied to the autograd state and dropped at backward."""
    e, n = workloads.barabasi_albert(n=512, m=3, seed=5)
    ei = torch.from_numpy(e).to(cuda)
    H, d = 8, 8
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(1, n, H, d, generator=g).to(cuda).requires_grad_(True) for _ in range(3))
    bias = (torch.randn(e.shape[1], H, generator=g) * 0.3).to(cuda).requires_grad_(True)
    layers = [CoreAttention(H * d, 0.0, H).to(cuda) for _ in range(2)]
    with torch.no_grad():
        ref = sum(m(q, k, v, bias, ei, "sparse") for m in layers)
    for step in range(2):
        out = sum(m(q, k, v, bias, ei, "sparse") for m in layers)
        assert torch.equal(out, ref)
        bias.grad = None
        out.square().sum().backward()
        assert bias.grad is not None and torch.isfinite(bias.grad).all() and bias.grad.abs().max() > 0
    # the gradient equals the one of the functional path
    b2 = bias.detach().clone().requires_grad_(True)
    out2 = 2 * sparse_attention(q.detach()[0], k.detach()[0], v.detach()[0], ei, b2).view(1, n, -1)
    out2.square().sum().backward()
    assert err(bias.grad, b2.grad) <= 1e-5
    from torchgt_amd import core_attention
    assert not core_attention._BIAS_CACHE      # nothing outlives the step


def test_plan_cache_is_bounded_by_bytes(cuda):
    from torchgt_amd import plan as plan_mod, get_plan, set_plan_cache_bytes, clear_plan_cache
    clear_plan_cache()
    rng = np.random.default_rng(0)
    keep = [torch.from_numpy(rng.integers(0, 1000, (2, 5000))).to(cuda) for _ in range(6)]
    try:
        set_plan_cache_bytes(3 * (56 * 5000 + 450 * 1000 + 16 * 5000))     # room for three such plans
        plans = [get_plan(t, 1000) for t in keep]
        assert len(plan_mod._CACHE) == 3
        assert get_plan(keep[-1], 1000) is plans[-1]                         # still cached
        assert get_plan(keep[0], 1000) is not plans[0]                       # evicted and rebuilt
        set_plan_cache_bytes(1)
        assert len(plan_mod._CACHE) == 1                                     # the last one always stays
    finally:
        set_plan_cache_bytes(1 << 30)
        clear_plan_cache()


def test_plan_survives_a_fresh_copy_of_edge_index(cuda):
    """The reference's training loops move the CPU-resident edge_index of a pre-packed batch to the GPU in every
    iteration (main_sp_sparse_node_level.py:178-183): the second copy, at whatever address, must find the plan
    of the first (one build), and the results are bit-identical.  A different edge list of the same shape gets
    its own plan."""
    from torchgt_amd import plan as plan_mod, get_plan, clear_plan_cache
    clear_plan_cache()
    e, n = workloads.barabasi_albert(n=2048, m=4, seed=11)
    ei_cpu = torch.from_numpy(e)
    H, d = 8, 8
    g = torch.Generator().manual_seed(21)
    q, k, v, dout = (torch.randn(n, H, d, generator=g).to(cuda) for _ in range(4))
    bias = (torch.randn(e.shape[1], H, generator=g) * 0.1).to(cuda)
    layer = CoreAttention(H * d, 0.0, H).to(cuda)
    results, plans, held = [], [], []
    for it in range(3):
        ei = ei_cpu.to(cuda)                      # a new tensor every iteration
        held.append(ei)                           # kept alive: the copies sit at different addresses
        t = [x.clone().requires_grad_(True) for x in (q, k, v, bias)]
        out = layer(t[0][None], t[1][None], t[2][None], t[3], ei, "sparse")
        out2 = layer(t[0][None], t[1][None], t[2][None], t[3], ei, "sparse")          # second layer of the step
        results.append((out,) + torch.autograd.grad(out + out2, t, dout.view(1, n, -1)))
        plans.append(get_plan(ei, n))
    stats = plan_mod.plan_cache_stats()
    assert stats["builds"] == 1 and stats["content_hits"] == 2, stats
    assert stats["tensor_hits"] >= 3            # the second layer and the explicit look-up never hash
    assert plans[0] is plans[1] is plans[2]
    for r in results[1:]:
        for a, b in zip(results[0], r):
            assert torch.equal(a, b)
    # same shape, other content: a plan of its own; the key looks at positions too
    e2 = np.ascontiguousarray(e[:, ::-1])          # the same edges in another order
    assert get_plan(torch.from_numpy(e2).to(cuda), n) is not plans[0]
    e3 = e.copy()
    e3[0, 5] = (e3[0, 5] + 1) % n
    assert get_plan(torch.from_numpy(e3).to(cuda), n) is not plans[0]
    assert plan_mod.plan_cache_stats()["builds"] == 3
    # the key itself: equal for equal content, whatever the address
    assert plan_mod.edge_index_key(held[0]) == plan_mod.edge_index_key(held[1])
    assert plan_mod.edge_index_key(held[0]) != plan_mod.edge_index_key(torch.from_numpy(e3).to(cuda))
    clear_plan_cache()


def test_plan_order_needs_the_map(cuda):
    e, n = workloads.barabasi_albert()
    ei = torch.from_numpy(e).to(cuda)
    plan = GraphPlan(ei, n)
    L = _lib.lib()
    H = d = 8
    q = torch.zeros(n, H, d, device=cuda)
    b = torch.zeros(e.shape[1], H, device=cuda)
    Z = torch.zeros(n, H, device=cuda)
    ws = plan.workspace(H, d)
    rc = L.tgt_sparse_attn_fwd(plan.handle, q.data_ptr(), q.data_ptr(), q.data_ptr(), b.data_ptr(),
                               _lib.BIAS_EDGE_HEAD | _lib.BIAS_PLAN_ORDER, H, d, _lib.DTYPE_F32, q.data_ptr(), Z.data_ptr(),
                               ws.data_ptr(), ws.numel(), None)
    assert rc == _lib.ERR_INVALID_ARG and b"tgt_plan_enable_bias_order" in L.tgt_last_error()
    assert L.tgt_sparse_attn_fwd(plan.handle, q.data_ptr(), q.data_ptr(), q.data_ptr(), b.data_ptr(), 0x23, H, d,
                                 _lib.DTYPE_F32, q.data_ptr(), Z.data_ptr(), ws.data_ptr(), ws.numel(), None) == _lib.ERR_INVALID_ARG
    plan.close()
