"""GPU parity of the block path (dense 16 x 16 tiles on the matrix cores + remaining edges on the
sparse kernels, one softmax per node) with the oracle evaluated on the EXPANDED edge list.

Tile products use bf16 matrix instructions with fp32 accumulation, so the bar is 2e-2
(max|a-b| / max|b| against the float64 oracle on the same bf16-rounded inputs) for both dtypes.
"""
import numpy as np
import pytest
import torch

from oracle import graph_prep as ogp
from oracle import sparse_attention as osa
from torchgt_amd import GraphPlan, _lib, block_attention, expand_tiles, graph_prep, sparse_attention, workloads

pytestmark = pytest.mark.gpu
TOL = 2e-2


def err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    denom = b.abs().max().item()
    return (a - b).abs().max().item() / (denom if denom > 0 else 1.0)


def run_case(name, N, tiles, rest, H, d, dtype, bias_kind, seed, cuda):
    print(f"block case {name}: N={N} T={len(tiles)} E_rest={rest.shape[1]} H={H} d={d} {dtype} bias={bias_kind}", flush=True)
    g = torch.Generator().manual_seed(seed)
    q, k, v, dout = (torch.randn(N, H, d, generator=g).to(torch.bfloat16).to(dtype) for _ in range(4))
    E_rest = rest.shape[1]
    bias = {"none": None, "edge": torch.randn(E_rest, generator=g) * 0.5,
            "edge_head": torch.randn(E_rest, H, generator=g) * 0.5}[bias_kind]
    if bias is not None:
        bias = bias.to(torch.bfloat16).to(dtype)
    # oracle: expanded tiles (bias 0) followed by the remaining edges
    ex = torch.from_numpy(expand_tiles(tiles))
    ei_all = torch.cat([ex, rest], 1)
    t = [x.double().requires_grad_(True) for x in (q, k, v)]
    bb = None
    if bias is not None:
        bb = bias.double().requires_grad_(True)
        full_bias = torch.cat([torch.zeros((ex.shape[1],) + tuple(bb.shape[1:]), dtype=torch.float64), bb])
    else:
        full_bias = None
    o_ref, _ = osa.sparse_attention(t[0], t[1], t[2], ei_all, full_bias)
    g_ref = torch.autograd.grad(o_ref, t + ([bb] if bb is not None else []), dout.double())
    tc = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    bc = bias.to(cuda).requires_grad_(True) if bias is not None else None
    o = block_attention(tc[0], tc[1], tc[2], tiles, rest.to(cuda), bc)
    g_got = torch.autograd.grad(o, tc + ([bc] if bc is not None else []), dout.to(cuda))
    assert o.dtype == dtype and o.shape == (N, H, d)
    assert err(o, o_ref) <= TOL, f"out err {err(o, o_ref)}"
    for nm, a, r in zip(("dq", "dk", "dv", "dbias"), g_got, g_ref):
        assert not torch.isnan(a).any()
        assert err(a, r) <= TOL, f"{nm} err {err(a, r)}"


def _random_tiles(rng, N, T, align=0):
    nb = (N - align) // 16
    return np.stack([rng.integers(0, nb, T) * 16 + align, rng.integers(0, nb, T) * 16 + align], 1).astype(np.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_tiles_only_and_tiles_plus_edges(cuda, dtype):
    rng = np.random.default_rng(0)
    N = 400
    tiles = _random_tiles(rng, N, 60)
    none = torch.zeros(2, 0, dtype=torch.int64)
    run_case("tiles-only", N, tiles, none, 8, 8, dtype, "none", 1, cuda)
    rest = torch.from_numpy(rng.integers(0, N, (2, 3000)))
    run_case("tiles+edges", N, tiles, rest, 8, 8, dtype, "edge_head", 2, cuda)
    run_case("tiles+edges scalar bias", N, tiles, rest, 8, 8, dtype, "edge", 3, cuda)
    # duplicate tiles count twice, like duplicate edges; offset block grid; a hub row among the rest
    tiles2 = np.concatenate([_random_tiles(rng, N, 20, align=5), _random_tiles(rng, N, 10, align=5)[:5].repeat(2, 0)])
    rest2 = rest.clone()
    rest2[1, :1500] = 7
    run_case("dup+offset+hub", N, tiles2, rest2, 8, 8, dtype, "edge_head", 4, cuda)


def test_other_shapes(cuda):
    rng = np.random.default_rng(1)
    N = 300
    tiles = _random_tiles(rng, N, 40)
    rest = torch.from_numpy(rng.integers(0, N, (2, 1000)))
    run_case("H4d16", N, tiles, rest, 4, 16, torch.bfloat16, "edge_head", 5, cuda)
    run_case("H8d16", N, tiles, rest, 8, 16, torch.bfloat16, "none", 6, cuda)
    run_case("H2d8", N, tiles, rest, 2, 8, torch.bfloat16, "edge", 7, cuda)
    # no remaining edges: the tile kernels write the final rows (and zeros on rows without tiles)
    none = torch.zeros(2, 0, dtype=torch.int64)
    run_case("H4d16 tiles-only", N, tiles, none, 4, 16, torch.bfloat16, "none", 8, cuda)
    run_case("H8d16 tiles-only", N, tiles, none, 8, 16, torch.float32, "none", 9, cuda)
    run_case("H2d8 tiles-only", N, tiles, none, 2, 8, torch.bfloat16, "none", 10, cuda)


def test_reference_pipeline_blockize_then_attention(cuda):
    # the reference's flow: reformat_graph (relabel + blockize + sort) then sparse attention on the new edge
    # list.  Here: the same reordering, the blocks kept as tiles, the block path; and the sparse path on the
    # expanded list as a second witness.
    rng = np.random.default_rng(2)
    N, k = 2048, 8
    part = np.repeat(np.arange(k), N // k)
    ei = np.concatenate([rng.integers(0, N // k, (2, 9000)) + rng.integers(0, k, 9000) * (N // k),
                         rng.integers(0, N, (2, 800))], 1)
    ref_edges, ref_sorted = ogp.reformat_graph(ei, part, k, 16)
    new_e, sorted_idx, tiles, raw = graph_prep.reformat_graph(
        torch.from_numpy(ei).to(cuda), k, 16, partition_ids=torch.from_numpy(part), return_tiles=True)
    np.testing.assert_array_equal(new_e.cpu().numpy(), ref_edges)
    assert raw.shape[1] == 0 and tiles.shape[0] * 256 == ref_edges.shape[1]
    # the tile list expands to the same multiset of edges
    ex = expand_tiles(tiles)
    key = lambda e: np.sort(e[0] * N + e[1])
    np.testing.assert_array_equal(key(ex), key(ref_edges))
    g = torch.Generator().manual_seed(8)
    q, k_, v, dout = (torch.randn(N, 8, 8, generator=g).to(torch.bfloat16) for _ in range(4))
    t = [x.double().requires_grad_(True) for x in (q, k_, v)]
    o_ref, _ = osa.sparse_attention(t[0], t[1], t[2], torch.from_numpy(ref_edges))
    g_ref = torch.autograd.grad(o_ref, t, dout.double())
    tc = [x.to(cuda).requires_grad_(True) for x in (q, k_, v)]
    o_blk = block_attention(tc[0], tc[1], tc[2], tiles)
    g_blk = torch.autograd.grad(o_blk, tc, dout.to(cuda))
    o_sp = sparse_attention(tc[0], tc[1], tc[2], new_e)
    assert err(o_blk, o_ref) <= TOL and err(o_sp, o_ref) <= TOL
    for a, r in zip(g_blk, g_ref):
        assert err(a, r) <= TOL


def test_config5_blockized_full_size(cuda):
    # configs[4]: SBM 64 x 4096, cluster-ordered; the reference's reordering with the clusters as partitions
    e, n, cluster = workloads.stochastic_block_model()
    new_e, _, tiles, raw = graph_prep.reformat_graph(torch.from_numpy(e).to(cuda), 64, 16,
                                                     partition_ids=torch.from_numpy(cluster), return_tiles=True)
    print(f"config5 blockized: T={tiles.shape[0]} E'={new_e.shape[1]} raw={raw.shape[1]}", flush=True)
    assert tiles.shape[0] * 256 == new_e.shape[1]
    run_case("config5-blockized", n, tiles, raw.cpu(), 8, 8, torch.bfloat16, "none", 9, cuda)


def test_config5_hybrid_full_size(cuda):
    # configs[4] as the benchmark words it: the intra-cluster edges of the 64 clusters as dense 16 x 16 tiles on the
    # matrix cores, the ~5 % inter-cluster edges raw on the sparse kernels (with a per-edge bias), one softmax per
    # node - against the float64 oracle on the expanded edge list, outputs and all gradients, at full size
    e, n, cluster = workloads.stochastic_block_model()
    tiles, raw, expanded = workloads.hybrid_tiles(e, cluster, 64, 16, seed=42)
    print(f"config5 hybrid: T={tiles.shape[0]} raw={raw.shape[1]} expanded={expanded.shape[1]}", flush=True)
    assert n == 262144 and 0.03 < raw.shape[1] / e.shape[1] < 0.07
    assert expanded.shape[1] == 256 * tiles.shape[0] + raw.shape[1]
    run_case("config5-hybrid", n, tiles, torch.from_numpy(raw), 8, 8, torch.bfloat16, "edge_head", 10, cuda)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_plan_of_the_remaining_edges_schedules_only_rows_with_edges(cuda, dtype):
    # few remaining edges: most rows have none - some under tiles (finished by the tile kernels), some under
    # nothing (zeros from the tile launches), a few with edges only (sparse kernels), a few with both
    rng = np.random.default_rng(5)
    N = 1000
    tiles = _random_tiles(rng, 640, 50)                      # nodes 640.. have no tiles
    rest = torch.from_numpy(np.concatenate([rng.integers(0, N, (2, 150)), rng.integers(700, 720, (2, 60))], 1))
    run_case("few remaining edges", N, tiles, rest, 8, 8, dtype, "edge_head", 11, cuda)
    run_case("few remaining edges, no tiles", N, np.zeros((0, 2), np.int32), rest, 8, 8, dtype, "edge", 12, cuda)
    # the same numbers whichever kind of plan holds the remaining edges
    g = torch.Generator().manual_seed(13)
    q, k, v, dout = (torch.randn(N, 8, 8, generator=g).to(cuda, dtype) for _ in range(4))
    bias = (torch.randn(rest.shape[1], 8, generator=g) * 0.5).to(cuda, dtype)
    res = []
    for only in (False, True):
        plan = GraphPlan(rest.to(cuda), N, rows_with_edges_only=only)
        tc = [x.clone().requires_grad_(True) for x in (q, k, v, bias)]
        o = block_attention(tc[0], tc[1], tc[2], tiles, edge_bias=tc[3], plan=plan)
        res.append([o] + list(torch.autograd.grad(o, tc, dout)))
        info = plan.info()
        assert info["items_dst"] == (len(np.unique(rest[1].numpy())) if only else N)
    for a, b in zip(*res):
        assert torch.equal(a, b)
    # on their own the sparse kernels would leave the other rows unwritten: refused
    with pytest.raises(RuntimeError, match="tgt_block_attn"):
        sparse_attention(q, k, v, rest.to(cuda), plan=plan)


def test_block_loud_failures(cuda):
    q = torch.randn(100, 8, 8, device=cuda, dtype=torch.bfloat16)
    with pytest.raises(_lib.TorchGTHipError) as exc:
        block_attention(q, q, q, np.array([[0, 0], [0, 8]], dtype=np.int32))      # destination blocks overlap partially
    assert exc.value.code == _lib.ERR_INVALID_ARG
    with pytest.raises(_lib.TorchGTHipError) as exc:
        block_attention(q, q, q, np.array([[90, 0]], dtype=np.int32))             # leaves [0, N)
    assert exc.value.code == _lib.ERR_INDEX_RANGE
    q32 = torch.randn(100, 2, 32, device=cuda, dtype=torch.bfloat16)
    with pytest.raises(_lib.TorchGTHipError) as exc:
        block_attention(q32, q32, q32, np.array([[0, 0]], dtype=np.int32))        # head dim 32
    assert exc.value.code == _lib.ERR_UNSUPPORTED
