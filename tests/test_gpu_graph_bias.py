"""GPU parity of GraphAttnBias (both edge-type branches, forward and parameter gradients), of the
Floyd-Warshall kernel and of gen_edge_input with the oracle.  Floyd-Warshall and gen_edge_input are
integer work: bit-exact.  The bias is a sum of
table entries: float32 1e-5 / bf16 2e-2 on max|a-b| / max|b| (finite entries; -inf stays -inf).
"""
import types

import numpy as np
import pytest
import torch

from oracle import dense_attention as oda
from oracle import graph_prep as ogp
from torchgt_amd import GraphAttnBias, _lib, floyd_warshall, gen_edge_input, workloads

pytestmark = pytest.mark.gpu
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


def err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    fin = torch.isfinite(b)
    assert torch.equal(torch.isfinite(a), fin)
    assert torch.equal(a[~fin], b[~fin])
    denom = b[fin].abs().max().item()
    return (a[fin] - b[fin]).abs().max().item() / (denom if denom > 0 else 1.0)


def test_floyd_warshall_matches_oracle_bit_for_bit(cuda):
    rng = np.random.default_rng(0)
    # single graphs, the reference's call shape
    for n, p in ((1, 0.0), (5, 0.5), (23, 0.12), (64, 0.05), (128, 0.03), (129, 0.03), (222, 0.012), (256, 0.02)):
        print(f"floyd_warshall case: n={n} p={p}", flush=True)
        a = (rng.random((n, n)) < p).astype(np.int64)
        a = np.maximum(a, a.T)
        M, path = floyd_warshall(a)
        M_ref, path_ref = ogp.floyd_warshall(a) if n <= 128 else ogp.floyd_warshall_by_steps(a)
        assert M.dtype == np.int64 and path.dtype == np.int64
        np.testing.assert_array_equal(M, M_ref)
        np.testing.assert_array_equal(path, path_ref)
    # directed, weighted, with self-loops in the input (the diagonal is reset to 0)
    a = rng.integers(0, 4, size=(17, 17)) * (rng.random((17, 17)) < 0.2)
    M, path = floyd_warshall(a)
    M_ref, path_ref = ogp.floyd_warshall(a)
    np.testing.assert_array_equal(M, M_ref)
    np.testing.assert_array_equal(path, path_ref)
    # a padded batch of graphs of different sizes: the configuration-4 generator
    data = workloads.erdos_renyi_batch(batch=12, seed=3)
    sizes = data["n_nodes"]
    n_max = int(sizes.max())
    adj = np.zeros((12, n_max, n_max), dtype=np.uint8)
    for g in range(12):
        n = int(sizes[g])
        sp = data["spatial_pos"][g][:n, :n]
        adj[g, :n, :n] = (sp == 2)                # spatial_pos = distance + 1: direct neighbours
    dist, path = floyd_warshall(torch.from_numpy(adj), sizes)
    for g in range(12):
        n = int(sizes[g])
        M_ref, path_ref = ogp.floyd_warshall(adj[g, :n, :n])
        np.testing.assert_array_equal(dist[g, :n, :n].cpu().numpy(), M_ref)
        np.testing.assert_array_equal(path[g, :n, :n].cpu().numpy(), path_ref)
        assert not dist[g, n:, :].any() and not dist[g, :, n:].any()
    # a padded batch with graphs of more than 128 nodes (intermediate nodes kept in the output array), one of them
    # a ring: the longest shortest paths a graph of that size can have
    sizes = np.array([130, 222, 17, 200], dtype=np.int64)
    adj = np.zeros((4, 222, 222), dtype=np.uint8)
    for g, n in enumerate(sizes):
        if g == 3:
            idx = np.arange(n)
            adj[g, idx, (idx + 1) % n] = 1
            adj[g, (idx + 1) % n, idx] = 1
        else:
            a = rng.random((n, n)) < 2.5 / n
            adj[g, :n, :n] = np.maximum(a, a.T)
    dist, path = floyd_warshall(torch.from_numpy(adj), sizes)
    for g, n in enumerate(sizes):
        M_ref, path_ref = ogp.floyd_warshall_by_steps(adj[g, :n, :n])
        np.testing.assert_array_equal(dist[g, :n, :n].cpu().numpy(), M_ref)
        np.testing.assert_array_equal(path[g, :n, :n].cpu().numpy(), path_ref)


def test_floyd_warshall_rejects_large_graphs(cuda):
    with pytest.raises(_lib.TorchGTHipError) as ei:
        floyd_warshall(np.zeros((257, 257), dtype=np.int64))
    assert ei.value.code == _lib.ERR_UNSUPPORTED


# (heads, edge features): every kernel variant -- eight heads with one feature, with up to four, with more (several
# passes over the features); more than eight heads (several passes over the heads); fewer than eight
@pytest.mark.parametrize("H,F", [(8, 3), (8, 1), (8, 6), (16, 2), (4, 1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_graph_attn_bias_matches_oracle(cuda, dtype, H, F):
    print(f"graph_attn_bias case: H={H} F={F} {dtype}", flush=True)
    data = workloads.erdos_renyi_batch(batch=16, seed=42)
    g = torch.Generator().manual_seed(1)
    m = GraphAttnBias(H, 512, 5, 22, 128, 64, "single_hop", 5)
    with torch.no_grad():
        m.spatial_pos_encoder.weight.normal_(0, 0.5, generator=g); m.spatial_pos_encoder.weight[0] = 0
        m.edge_encoder.weight.normal_(0, 0.5, generator=g); m.edge_encoder.weight[0] = 0
        m.graph_token_virtual_distance.weight.normal_(0, 0.5, generator=g)
    assert sorted(n for n, _ in m.named_parameters()) == ["edge_encoder.weight", "graph_token_virtual_distance.weight",
                                                          "spatial_pos_encoder.weight"]
    m = m.to(dtype)
    attn_bias = torch.from_numpy(data["attn_bias"])                       # 0 / -inf, [b, S1, S1]
    spatial_pos = torch.from_numpy(data["spatial_pos"]).long()
    et1 = torch.from_numpy(data["edge_type"]).long()
    # F edge features per pair; from the third on, every other one is the padding id
    edge_type = torch.stack([(et1 * (f + 1)) % 5 if f < 2 or f % 2 else torch.zeros_like(et1) for f in range(F)], -1)
    assert int(spatial_pos.max()) > 6                 # ids beyond the ones the backward keeps in registers occur
    st, et, vd = (p.detach().double() for p in (m.spatial_pos_encoder.weight, m.edge_encoder.weight, m.graph_token_virtual_distance.weight))
    st.requires_grad_(True); et.requires_grad_(True); vd.requires_grad_(True)
    want = oda.graph_attn_bias(attn_bias.double(), spatial_pos, edge_type, st, et, vd)
    mc = m.to(cuda)
    batch = types.SimpleNamespace(attn_bias=attn_bias.to(cuda), spatial_pos=spatial_pos.to(cuda), attn_edge_type=edge_type.to(cuda),
                                  edge_input=None)
    got = mc(batch)
    assert got.shape == want.shape and got.dtype == dtype
    assert err(got, want) <= TOL[dtype], err(got, want)
    # table gradients; the upstream gradient is zero on the masked (-inf) entries, as the attention's is
    dout = torch.randn(want.shape, generator=g)
    dout[~torch.isfinite(want)] = 0
    dout = dout.to(dtype)
    finite = torch.where(torch.isfinite(want), want, torch.zeros_like(want))
    ref = [r.clone() for r in torch.autograd.grad((finite * dout.double()).sum(), [st, et, vd])]
    # the oracle indexes plain tensors; the module's tables are nn.Embedding(padding_idx=0), whose row 0 gets no
    # gradient (checked here on torch's own embedding), although padded query rows do look it up
    w = torch.ones(3, 2, requires_grad=True)
    torch.nn.functional.embedding(torch.tensor([0, 0, 1]), w, padding_idx=0).sum().backward()
    assert w.grad[0].abs().sum() == 0 and w.grad[1].sum() == 2
    assert ref[0][0].abs().max() > 0          # the case is exercised
    ref[0][0] = 0
    ref[1][0] = 0
    got_g = torch.autograd.grad(got, [mc.spatial_pos_encoder.weight, mc.edge_encoder.weight, mc.graph_token_virtual_distance.weight],
                                dout.to(cuda))
    for nm, a, r in zip(("spatial", "edge", "virtual"), got_g, ref):
        assert err(a, r) <= TOL[dtype], f"d{nm} err {err(a, r)}"
    assert not got_g[0][0].any() and not got_g[1][0].any()              # padding index rows get no gradient


def _edge_input_of_batch(data, F, max_dist):
    """Shortest-path edge features of the configuration-4 style batch through the oracle's Floyd-Warshall and
    gen_edge_input, in the collator's conventions (features + 1, 0 = padding; data/collator.py:59-66)."""
    sizes = data["n_nodes"]
    b, s = len(sizes), data["spatial_pos"].shape[1]
    et1 = data["edge_type"].astype(np.int64)                              # [b, s, s], 0 = no edge
    edge_input = np.zeros((b, s, s, max_dist, F), dtype=np.int64)
    for g in range(b):
        n = int(sizes[g])
        adj = (data["spatial_pos"][g][:n, :n] == 2).astype(np.int64)
        feat = np.stack([(et1[g, :n, :n] * (f + 1)) % 4 for f in range(F)], -1) * adj[:, :, None]    # 0..3, ids 1..4
        _, path = ogp.floyd_warshall(adj)
        edge_input[g, :n, :n] = ogp.gen_edge_input(max_dist, path, feat) + 1
    return edge_input


# (heads, edge features, hops held by the input, hop limit): eight heads, fewer, sixteen and thirty-two (the wider
# head tiles); a limit below, at and above the hops the input holds, and no limit
@pytest.mark.parametrize("H,F,D0,mhd", [(8, 1, 5, 5), (8, 3, 6, 4), (4, 2, 3, 0), (16, 1, 4, 6), (32, 1, 3, 2), (8, 2, 10, 0)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_graph_attn_bias_multi_hop_matches_oracle(cuda, dtype, H, F, D0, mhd):
    print(f"multi_hop bias case: H={H} F={F} D0={D0} multi_hop_max_dist={mhd} {dtype}", flush=True)
    data = workloads.erdos_renyi_batch(batch=8, seed=7)
    g = torch.Generator().manual_seed(2)
    n_dis = 12
    m = GraphAttnBias(H, 512, 5, 22, n_dis, 64, "multi_hop", mhd)
    with torch.no_grad():
        m.spatial_pos_encoder.weight.normal_(0, 0.5, generator=g); m.spatial_pos_encoder.weight[0] = 0
        m.edge_encoder.weight.normal_(0, 0.5, generator=g); m.edge_encoder.weight[0] = 0
        m.edge_dis_encoder.weight.normal_(0, 0.5, generator=g)
        m.graph_token_virtual_distance.weight.normal_(0, 0.5, generator=g)
    assert sorted(n for n, _ in m.named_parameters()) == ["edge_dis_encoder.weight", "edge_encoder.weight",
                                                          "graph_token_virtual_distance.weight", "spatial_pos_encoder.weight"]
    assert m.edge_dis_encoder.weight.shape == (n_dis * H * H, 1)
    m = m.to(dtype)
    attn_bias = torch.from_numpy(data["attn_bias"])
    spatial_pos = torch.from_numpy(data["spatial_pos"]).long()
    edge_input = torch.from_numpy(_edge_input_of_batch(data, F, D0))
    assert int(edge_input.max()) > 0 and int(spatial_pos.max()) > 4           # paths of several hops occur
    params = [p.detach().double().requires_grad_(True) for p in (m.spatial_pos_encoder.weight, m.edge_encoder.weight,
                                                                 m.edge_dis_encoder.weight, m.graph_token_virtual_distance.weight)]
    st, et, wd, vd = params
    want = oda.graph_attn_bias_multi_hop(attn_bias.double(), spatial_pos, edge_input, st, et, wd, vd, mhd)
    mc = m.to(cuda)
    batch = types.SimpleNamespace(attn_bias=attn_bias.to(cuda), spatial_pos=spatial_pos.to(cuda), edge_input=edge_input.to(cuda),
                                  attn_edge_type=None)
    got = mc(batch)
    assert got.shape == want.shape and got.dtype == dtype
    assert err(got, want) <= TOL[dtype], err(got, want)
    dout = torch.randn(want.shape, generator=g)
    dout[~torch.isfinite(want)] = 0
    dout = dout.to(dtype)
    finite = torch.where(torch.isfinite(want), want, torch.zeros_like(want))
    ref = [r.clone() for r in torch.autograd.grad((finite * dout.double()).sum(), params)]
    ref[0][0] = 0                                  # nn.Embedding(padding_idx=0): row 0 gets no gradient
    ref[1][0] = 0
    got_g = torch.autograd.grad(got, [mc.spatial_pos_encoder.weight, mc.edge_encoder.weight, mc.edge_dis_encoder.weight,
                                      mc.graph_token_virtual_distance.weight], dout.to(cuda))
    for nm, a, r in zip(("spatial", "edge", "hop matrices", "virtual"), got_g, ref):
        assert a.shape == r.shape
        assert err(a, r) <= TOL[dtype], f"d{nm} err {err(a, r)}"
    assert not got_g[0][0].any() and not got_g[1][0].any()
    D = min(D0, mhd) if mhd > 0 else D0
    assert not got_g[2].reshape(n_dis, H, H)[D:].any() and got_g[2].reshape(n_dis, H, H)[:D].any()


@pytest.mark.parametrize("edge_type", ["single_hop", "multi_hop"])
def test_graph_attn_bias_with_molecule_sized_tables(cuda, edge_type):
    """The tables of the reference's molecule datasets (models/graphormer_graph_level.py:332-338: 512 spatial ids,
    1 537 edge types, 128 hop matrices) with ids spread over them: the tables no longer fit next to the hop matrices
    in LDS (the kernels read them from memory) and the gradient sums take 66 KB of LDS per workgroup."""
    print(f"molecule-sized tables: {edge_type}", flush=True)
    H, F, D0, mhd = 8, 1, 4, 4
    data = workloads.erdos_renyi_batch(batch=6, seed=17)
    g = torch.Generator().manual_seed(3)
    m = GraphAttnBias(H, 512 * 9 + 1, 512 * 3 + 1, 512, 128, 64, edge_type, mhd)
    with torch.no_grad():
        m.spatial_pos_encoder.weight.normal_(0, 0.5, generator=g); m.spatial_pos_encoder.weight[0] = 0
        m.edge_encoder.weight.normal_(0, 0.5, generator=g); m.edge_encoder.weight[0] = 0
        m.graph_token_virtual_distance.weight.normal_(0, 0.5, generator=g)
        if edge_type == "multi_hop":
            m.edge_dis_encoder.weight.normal_(0, 0.5, generator=g)
    attn_bias = torch.from_numpy(data["attn_bias"])
    spatial_pos = torch.from_numpy(data["spatial_pos"]).long() * 20          # 0 stays the padding id, up to 420
    et = torch.from_numpy(data["edge_type"]).long().unsqueeze(-1) * 300       # up to 1 200
    edge_input = torch.from_numpy(_edge_input_of_batch(data, F, D0))
    edge_input = torch.where(edge_input > 0, (edge_input - 1) * 300 + 1, edge_input)
    names = ["spatial_pos_encoder", "edge_encoder"] + (["edge_dis_encoder"] if edge_type == "multi_hop" else []) \
        + ["graph_token_virtual_distance"]
    params = [getattr(m, n).weight.detach().double().requires_grad_(True) for n in names]
    if edge_type == "multi_hop":
        # the oracle's path length comes from spatial_pos itself; keep the ids, scale only the table rows they select
        want = oda.graph_attn_bias_multi_hop(attn_bias.double(), spatial_pos, edge_input, params[0], params[1], params[2], params[3], mhd)
    else:
        want = oda.graph_attn_bias(attn_bias.double(), spatial_pos, et, params[0], params[1], params[2])
    mc = m.to(cuda)
    got = mc(types.SimpleNamespace(attn_bias=attn_bias.to(cuda), spatial_pos=spatial_pos.to(cuda), attn_edge_type=et.to(cuda),
                                   edge_input=edge_input.to(cuda)))
    assert err(got, want) <= 1e-5, err(got, want)
    dout = torch.randn(want.shape, generator=g)
    dout[~torch.isfinite(want)] = 0
    finite = torch.where(torch.isfinite(want), want, torch.zeros_like(want))
    ref = [r.clone() for r in torch.autograd.grad((finite * dout.double()).sum(), params)]
    ref[0][0] = 0
    ref[1][0] = 0
    got_g = torch.autograd.grad(got, [getattr(mc, n).weight for n in names], dout.to(cuda))
    for n, a, r in zip(names, got_g, ref):
        assert err(a, r) <= 1e-5, f"d{n} err {err(a, r)}"
    assert got_g[0][420].any() and got_g[1][300 if edge_type == "single_hop" else 301].any()


def test_graph_attn_bias_multi_hop_without_hops_is_the_spatial_and_virtual_part(cuda):
    # an edge_input that holds no hops (the reference's reshape raises on it): the edge term vanishes, forward and
    # gradients still come out; the single-hop oracle with an all-zero edge table is the same sum
    data = workloads.erdos_renyi_batch(batch=4, seed=9)
    H = 8
    m = GraphAttnBias(H, 512, 5, 22, 3, 64, "multi_hop", 5)
    with torch.no_grad():
        m.spatial_pos_encoder.weight.normal_(0, 0.5); m.spatial_pos_encoder.weight[0] = 0
        m.graph_token_virtual_distance.weight.normal_(0, 0.5)
    attn_bias = torch.from_numpy(data["attn_bias"])
    spatial_pos = torch.from_numpy(data["spatial_pos"]).long()
    b, s = spatial_pos.shape[:2]
    edge_input = torch.zeros(b, s, s, 0, 1, dtype=torch.long)
    params = [p.detach().double().requires_grad_(True) for p in (m.spatial_pos_encoder.weight, m.edge_encoder.weight,
                                                                 m.edge_dis_encoder.weight, m.graph_token_virtual_distance.weight)]
    want = oda.graph_attn_bias(attn_bias.double(), spatial_pos, torch.zeros(b, s, s, 1, dtype=torch.long), params[0],
                               torch.zeros(5, H, dtype=torch.float64), params[3])
    mc = m.to(cuda)
    got = mc(types.SimpleNamespace(attn_bias=attn_bias.to(cuda), spatial_pos=spatial_pos.to(cuda), edge_input=edge_input.to(cuda)))
    assert err(got, want) <= 1e-5
    dout = torch.randn(want.shape, generator=torch.Generator().manual_seed(1))
    dout[~torch.isfinite(want)] = 0
    finite = torch.where(torch.isfinite(want), want, torch.zeros_like(want))
    ref = torch.autograd.grad((finite * dout.double()).sum(), [params[0], params[3]])
    ref[0][0] = 0
    g = torch.autograd.grad(got, [mc.spatial_pos_encoder.weight, mc.edge_encoder.weight, mc.edge_dis_encoder.weight,
                                  mc.graph_token_virtual_distance.weight], dout.to(cuda))
    assert err(g[0], ref[0]) <= 1e-5 and err(g[3], ref[1]) <= 1e-5
    assert not g[1].any() and not g[2].any()


def test_graph_attn_bias_multi_hop_on_graphs_without_nodes(cuda):
    # s = 0: only the virtual node; every entry is 2 * attn_bias + the virtual distance, the id tensors are empty
    H = 8
    m = GraphAttnBias(H, 512, 5, 22, 5, 64, "multi_hop", 5).to(cuda)
    with torch.no_grad():
        m.graph_token_virtual_distance.weight.normal_(0, 0.5)
    ab = torch.randn(3, 1, 1, device=cuda)
    batch = types.SimpleNamespace(attn_bias=ab, spatial_pos=torch.zeros(3, 0, 0, dtype=torch.long, device=cuda),
                                  edge_input=torch.zeros(3, 0, 0, 4, 1, dtype=torch.long, device=cuda))
    got = m(batch)
    want = 2 * ab.unsqueeze(1) + m.graph_token_virtual_distance.weight.view(1, H, 1, 1)
    assert got.shape == (3, H, 1, 1) and err(got, want) <= 1e-6
    dout = torch.randn(3, H, 1, 1, device=cuda)
    g = torch.autograd.grad(got, [m.spatial_pos_encoder.weight, m.edge_encoder.weight, m.edge_dis_encoder.weight,
                                  m.graph_token_virtual_distance.weight], dout)
    assert not g[0].any() and not g[1].any() and not g[2].any()
    assert err(g[3], dout.sum(0).view(1, H)) <= 1e-6


def test_graph_attn_bias_multi_hop_rejects_more_hops_than_matrices(cuda):
    m = GraphAttnBias(8, 512, 5, 22, 2, 64, "multi_hop", 0).to(cuda)       # two hop matrices, three hops of input
    batch = types.SimpleNamespace(attn_bias=torch.zeros(1, 4, 4, device=cuda), spatial_pos=torch.ones(1, 3, 3, dtype=torch.long, device=cuda),
                                  edge_input=torch.zeros(1, 3, 3, 3, 1, dtype=torch.long, device=cuda))
    with pytest.raises(_lib.TorchGTHipError) as ei:
        m(batch)
    assert ei.value.code == _lib.ERR_INVALID_ARG


def test_gen_edge_input_matches_oracle_bit_for_bit(cuda):
    rng = np.random.default_rng(4)
    # single graphs, the reference's call shape (max_dist = the longest distance, 510 when a pair is unreachable:
    # data/wrapper.py passes np.amax of the distance matrix)
    for n, p, F in ((1, 0.0, 1), (6, 0.4, 2), (23, 0.12, 3), (64, 0.06, 1), (128, 0.03, 2), (222, 0.012, 1)):
        a = (rng.random((n, n)) < p).astype(np.int64)
        a = np.maximum(a, a.T)
        np.fill_diagonal(a, 0)
        feat = rng.integers(1, 9, size=(n, n, F)) * a[:, :, None]
        M, path = ogp.floyd_warshall(a) if n <= 128 else ogp.floyd_warshall_by_steps(a)
        reach = M[M < 510]
        for max_dist in sorted({int(reach.max()) if reach.size else 0, 2, 5}):
            print(f"gen_edge_input case: n={n} p={p} F={F} max_dist={max_dist}", flush=True)
            want = ogp.gen_edge_input(max_dist, path, feat)
            got = gen_edge_input(max_dist, path, feat)
            assert got.dtype == np.int64 and got.shape == want.shape
            np.testing.assert_array_equal(got, want)
    # a ring of 200 nodes: paths of up to 100 hops
    idx = np.arange(200)
    a = np.zeros((200, 200), dtype=np.int64)
    a[idx, (idx + 1) % 200] = 1
    a[(idx + 1) % 200, idx] = 1
    feat = rng.integers(1, 9, size=(200, 200, 1)) * a[:, :, None]
    M, path = ogp.floyd_warshall_by_steps(a)
    np.testing.assert_array_equal(gen_edge_input(100, path, feat), ogp.gen_edge_input(100, path, feat))
    # directed graph: paths and features are not symmetric
    a = (rng.random((40, 40)) < 0.08).astype(np.int64)
    np.fill_diagonal(a, 0)
    feat = rng.integers(1, 100, size=(40, 40, 2)) * a[:, :, None]
    M, path = ogp.floyd_warshall(a)
    np.testing.assert_array_equal(gen_edge_input(7, path, feat), ogp.gen_edge_input(7, path, feat))
    # the GPU chain: Floyd-Warshall then gen_edge_input on a padded batch
    data = workloads.erdos_renyi_batch(batch=10, seed=5)
    sizes = data["n_nodes"]
    n_max = int(sizes.max())
    adj = np.zeros((10, n_max, n_max), dtype=np.uint8)
    feat = np.zeros((10, n_max, n_max, 1), dtype=np.int64)
    for g in range(10):
        n = int(sizes[g])
        adj[g, :n, :n] = data["spatial_pos"][g][:n, :n] == 2
        feat[g, :n, :n, 0] = data["edge_type"][g][:n, :n] * adj[g, :n, :n]
    dist, path = floyd_warshall(torch.from_numpy(adj), sizes)
    got = gen_edge_input(6, path, torch.from_numpy(feat).to(path.device), sizes)
    assert got.is_cuda and got.shape == (10, n_max, n_max, 6, 1)
    for g in range(10):
        n = int(sizes[g])
        _, path_ref = ogp.floyd_warshall(adj[g, :n, :n])
        np.testing.assert_array_equal(got[g, :n, :n].cpu().numpy(), ogp.gen_edge_input(6, path_ref, feat[g, :n, :n]))
        assert (got[g, n:] == -1).all() and (got[g, :, n:] == -1).all()


def test_gen_edge_input_rejects_large_graphs(cuda):
    with pytest.raises(_lib.TorchGTHipError) as ei:
        gen_edge_input(3, np.zeros((257, 257), dtype=np.int64), np.zeros((257, 257, 1), dtype=np.int64))
    assert ei.value.code == _lib.ERR_UNSUPPORTED
