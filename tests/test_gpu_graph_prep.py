"""GPU: fix_edge_index / reformat_graph are bit-exact with the numpy oracle."""
import numpy as np
import pytest
import torch

from oracle import graph_prep as ogp
from torchgt_amd import _lib, graph_prep, workloads

pytestmark = pytest.mark.gpu


def test_fix_edge_index(cuda):
    rng = np.random.default_rng(0)
    for n, e0 in ((3, 1), (5, 0), (1000, 7000), (64000, 300000)):
        x = rng.integers(0, n, (2, e0))
        got = graph_prep.fix_edge_index(torch.from_numpy(x).to(cuda), n).cpu().numpy()
        np.testing.assert_array_equal(got, ogp.fix_edge_index(x, n))
    np.testing.assert_array_equal(
        graph_prep.fix_edge_index(torch.tensor([[0], [1]], device=cuda), 3).cpu().numpy(),
        [[1, 1, 2, 3, 0, 0, 0], [2, 0, 0, 0, 1, 2, 3]])
    # the workload builder's closed form agrees
    np.testing.assert_array_equal(workloads.add_global_node(np.array([[0], [1]]), 3),
                                  ogp.fix_edge_index(np.array([[0], [1]]), 3))


def test_adjust_edge_index_nomerge(cuda):
    e = np.array([[0, 1, 5, 8], [8, 4, 0, 1]])
    for L in (8, 4, 3):
        got = graph_prep.adjust_edge_index_nomerge(torch.from_numpy(e).to(cuda), L).cpu().numpy()
        np.testing.assert_array_equal(got, ogp.adjust_edge_index_nomerge(e, L))


def _check_reformat(ei, part, k, bs, blockize, cuda):
    print(f"reformat case N={len(part)} E={ei.shape[1]} k={k} bs={bs} blockize={blockize}", flush=True)
    got_e, got_s = graph_prep.reformat_graph(torch.from_numpy(ei).to(cuda), k, bs,
                                             partition_ids=torch.from_numpy(part), blockize=blockize)
    if blockize:
        ref_e, ref_s = ogp.reformat_graph(ei, part, k, bs)
    else:
        ref_e, ref_s = ogp.relabel_and_sort(ei, part, k)
    np.testing.assert_array_equal(got_s.cpu().numpy(), ref_s)
    np.testing.assert_array_equal(got_e.cpu().numpy(), ref_e)


def test_reformat_blockize_matches_oracle(cuda):
    rng = np.random.default_rng(1)
    # reference shape: k = 8 parts, block 16
    N, k = 4000, 8
    part = rng.integers(0, k, N)
    ei = rng.integers(0, N, (2, 30000))
    _check_reformat(ei, part, k, 16, True, cuda)
    # contiguous clusters, heavier intra-cluster traffic
    part2 = np.repeat(np.arange(k), N // k)
    intra = rng.integers(0, N // k, (2, 20000)) + (rng.integers(0, k, 20000) * (N // k))
    _check_reformat(np.concatenate([intra, ei[:, :3000]], 1), part2, k, 16, True, cuda)
    # single partition known answer (k = 1, N = 32)
    _check_reformat(np.array([[0, 3, 7, 20, 31], [1, 9, 2, 5, 30]]), np.zeros(32, dtype=np.int64), 1, 16, True, cuda)
    # an empty partition pair: the compact-count quirk of the reference is reproduced
    part3 = np.repeat([0, 1, 2], 40)
    e3 = np.concatenate([rng.integers(0, 40, (2, 500)), rng.integers(40, 80, (2, 300)),
                         rng.integers(80, 120, (2, 700)), np.stack([rng.integers(0, 40, 50), rng.integers(80, 120, 50)])], 1)
    _check_reformat(e3, part3, 3, 16, True, cuda)


def test_reformat_raw_branch_when_duplicates_exceed_capacity(cuda):
    # a partition pair with more edges than n_i*n_j (duplicates): sparsity > 1 keeps the raw edges,
    # taken from the list sorted by ((part_src, part_dst), (src, dst))
    rng = np.random.default_rng(2)
    part = np.repeat([0, 1], [4, 60])
    dense = rng.integers(0, 4, (2, 40))                 # 40 edges in a 4x4 pair -> sparsity 2.5
    rest = np.stack([rng.integers(4, 64, 300), rng.integers(0, 64, 300)])
    rest2 = np.stack([rng.integers(0, 4, 30), rng.integers(4, 64, 30)])
    _check_reformat(np.concatenate([rest, dense, rest2], 1), part, 2, 2, True, cuda)


def test_reformat_hand_computed_compact_counts_and_raw_branch(cuda):
    # the hand-computed example of tests/test_oracle_graph_prep.py (compact edge counts read at the wrong
    # pair, raw-edge branch, duplicate blocks): 7 nodes in parts of 2, 3, 2, block size 2, no random draw matters
    part = np.array([0, 0, 1, 1, 1, 2, 2])
    pairs = [(1, 0), (0, 1), (0, 1), (1, 1), (0, 0), (1, 6), (0, 5), (0, 5), (1, 5), (0, 6), (1, 6), (0, 5),
             (4, 0), (2, 0), (3, 1), (2, 5), (6, 6), (5, 5), (5, 6), (6, 5), (5, 5)]
    blk = lambda r0, c0: [(r0, c0), (r0, c0 + 1), (r0 + 1, c0), (r0 + 1, c0 + 1)]
    emitted = ([(0, 0), (0, 1), (0, 1), (1, 0), (1, 1)] + [(0, 5), (0, 5), (0, 5), (0, 6), (1, 5), (1, 6), (1, 6)]
               + blk(0, 5) + blk(2, 0) + blk(2, 2) + blk(2, 2) + blk(2, 5) + blk(5, 0) + blk(5, 2) + blk(5, 5))
    emitted = np.array(emitted).T
    want = emitted[:, np.argsort(emitted[0], kind="stable")]
    got_e, got_s = graph_prep.reformat_graph(torch.tensor(pairs).t().contiguous().to(cuda), 3, 2,
                                             partition_ids=torch.from_numpy(part))
    np.testing.assert_array_equal(got_e.cpu().numpy(), want)
    np.testing.assert_array_equal(got_s.cpu().numpy(), np.arange(7))


def test_relabel_and_sort_without_blockize(cuda):
    rng = np.random.default_rng(3)
    N, k = 70000, 8
    part = rng.integers(0, k, N)
    ei = rng.integers(0, N, (2, 250000))
    _check_reformat(ei, part, k, 16, False, cuda)


def test_reformat_errors(cuda):
    ei = torch.tensor([[0, 1], [1, 2]], device=cuda)
    with pytest.raises(_lib.TorchGTHipError) as exc:
        graph_prep.reformat_graph(ei, 2, 16, partition_ids=torch.tensor([0, 1, 5]))
    assert exc.value.code == _lib.ERR_INDEX_RANGE
    with pytest.raises(_lib.TorchGTHipError) as exc:       # part 1 empty: the reference divides by zero
        graph_prep.reformat_graph(ei, 2, 16, partition_ids=torch.tensor([0, 0, 0]))
    assert exc.value.code == _lib.ERR_INVALID_ARG
    with pytest.raises(ValueError):
        graph_prep.reformat_graph(ei, 2, 16)


def _check_sub(e, idx, N, cuda):
    print(f"sub_edge_index case: N={N} E={e.shape[1]} S={len(idx)}", flush=True)
    want = ogp.gen_sub_edge_index(e, idx, N)
    got = graph_prep.gen_sub_edge_index(torch.as_tensor(e, dtype=torch.int64).to(cuda), torch.as_tensor(np.asarray(idx), dtype=torch.int64), N)
    assert got.dtype == torch.int64 and got.is_contiguous()
    np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_gen_sub_edge_index_matches_oracle(cuda):
    rng = np.random.default_rng(0)
    _check_sub(np.array([[0, 1, 2, 3, 4, 1, 5, 2], [1, 1, 3, 2, 5, 0, 5, 0]]), [3, 0, 2], 6, cuda)      # known answer
    _check_sub(rng.integers(0, 50, size=(2, 400)), rng.permutation(50)[:17], 50, cuda)
    _check_sub(rng.integers(0, 50, size=(2, 400)), rng.integers(0, 50, size=23), 50, cuda)              # repeated nodes
    _check_sub(np.zeros((2, 0), dtype=np.int64), [2, 1], 4, cuda)                                       # no edges
    _check_sub(np.array([[0, 1], [1, 0]]), [], 3, cuda)                                                 # empty batch
    _check_sub(rng.integers(0, 5000, size=(2, 70001)), rng.permutation(5000)[:1025], 5000, cuda)        # ragged tiles
    e, n = workloads.power_law_graph()                       # 64 K nodes, 530 K edges; a 16 K-node batch
    _check_sub(e, rng.permutation(n)[:16384], n, cuda)
    _check_sub(e, np.arange(n), n, cuda)                     # the whole graph: every edge survives


def test_gen_sub_edge_index_errors(cuda):
    e = torch.tensor([[0, 1], [1, 7]], device=cuda)
    with pytest.raises(_lib.TorchGTHipError) as ei:
        graph_prep.gen_sub_edge_index(e, torch.tensor([0, 1]), 4)          # endpoint 7 outside [0, 4)
    assert ei.value.code == _lib.ERR_INDEX_RANGE
    with pytest.raises(_lib.TorchGTHipError) as ei:
        graph_prep.gen_sub_edge_index(torch.tensor([[0], [1]], device=cuda), torch.tensor([0, 9]), 4)
    assert ei.value.code == _lib.ERR_INDEX_RANGE
    with pytest.raises(RuntimeError):
        graph_prep.gen_sub_edge_index(torch.tensor([[0], [1]]), torch.tensor([0]), 4)      # CPU tensor


def test_prepare_batch_composes_the_reference_steps(cuda):
    """prepare_batch = the oracle's gen_sub_edge_index -> fix_edge_index -> reformat_graph ->
    adjust_edge_index_nomerge, with x and y permuted by the sorted indices (gt_sp/utils.py:409-520, one rank)."""
    rng = np.random.default_rng(5)
    e, n = workloads.power_law_graph(n=4000, directed_edges=40000)
    S, k, bs = 1024, 4, 16
    idx = rng.permutation(n)[:S]
    x = torch.randn(n, 12, generator=torch.Generator().manual_seed(0))
    y = torch.randint(0, 40, (n,), generator=torch.Generator().manual_seed(1))
    part = rng.integers(0, k, size=S + 1)
    sub = ogp.fix_edge_index(ogp.gen_sub_edge_index(e, idx, n), S)
    want_ei, want_sorted = ogp.reformat_graph(sub, part, k, bs)
    want_ei = ogp.adjust_edge_index_nomerge(want_ei, S)
    order = want_sorted[want_sorted != 0] - 1
    x_i, y_i, ei, bias = graph_prep.prepare_batch(x.to(cuda), y.to(cuda), torch.as_tensor(idx), torch.as_tensor(e).to(cuda), n, k, bs,
                                                  torch.as_tensor(part))
    assert bias is None
    np.testing.assert_array_equal(ei.cpu().numpy(), want_ei)
    assert torch.equal(x_i.cpu(), x[idx][order]) and torch.equal(y_i.cpu(), y[idx][order])
    # a callable partitioner sees the sub-graph
    seen = {}
    def partition(ei_sub, n_sub, kk):
        seen["args"] = (tuple(ei_sub.shape), n_sub, kk)
        return torch.as_tensor(part)
    out2 = graph_prep.prepare_batch(x.to(cuda), y.to(cuda), torch.as_tensor(idx), torch.as_tensor(e).to(cuda), n, k, bs, partition)
    assert seen["args"] == ((2, sub.shape[1]), S + 1, k) and torch.equal(out2[2], ei)
