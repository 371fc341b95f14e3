"""Pins of the graph-preparation oracle (CPU only): hand-computed known answers
and structural invariants for fix_edge_index / relabel / blockize / sort / CSR."""
import numpy as np
import pytest

from oracle import graph_prep as gp


def test_fix_edge_index_known_answer():
    # N = 3 real nodes, one edge 0 -> 1 (gt_sp/utils.py:34-50 worked by hand)
    out = gp.fix_edge_index(np.array([[0], [1]]), 3)
    expect = np.array([[1, 1, 2, 3, 0, 0, 0],
                       [2, 0, 0, 0, 1, 2, 3]])
    np.testing.assert_array_equal(out, expect)
    assert out.dtype == np.int64


def test_fix_edge_index_no_self_loop_on_virtual_node():
    e = gp.fix_edge_index(np.zeros((2, 0), dtype=np.int64), 5)
    assert e.shape == (2, 10)
    assert not np.any((e[0] == 0) & (e[1] == 0))
    np.testing.assert_array_equal(np.bincount(e[1], minlength=6), [5, 1, 1, 1, 1, 1])


def test_adjust_edge_index_nomerge_identity_at_p1_and_shift_at_p2():
    e = np.array([[0, 1, 5, 8], [8, 4, 0, 1]])
    np.testing.assert_array_equal(gp.adjust_edge_index_nomerge(e, 8), e)       # every idx <= L
    # L = 4: idx 5..8 belong to the second rank and shift by one slot (its global-token copy)
    np.testing.assert_array_equal(gp.adjust_edge_index_nomerge(e, 4), [[0, 1, 6, 9], [9, 4, 0, 1]])


def test_relabel_known_answer():
    # parts: node0->1, node1->0, node2->1, node3->0  => part 0 = {1,3} -> ids 0,1 ; part 1 = {0,2} -> 2,3
    m = gp.relabel_by_partition(np.array([1, 0, 1, 0]), 2)
    np.testing.assert_array_equal(m, [2, 0, 3, 1])


def test_blockize_known_answer_single_partition():
    # k = 1, N = 32, block 16: 5 edges -> sparsity 5/1024 <= 1 -> int(5/256)+1 = 1 random block,
    # drawn exactly as the reference does: np.random.seed(0); randint(0, 2); randint(0, 2)
    N, bs = 32, 16
    part = np.zeros(N, dtype=np.int64)
    ei = np.array([[0, 3, 7, 20, 31], [1, 9, 2, 5, 30]])
    mapping = gp.relabel_by_partition(part, 1)
    np.testing.assert_array_equal(mapping, np.arange(N))
    out = gp.blockize(ei, 1, part, 1, bs, mapping)
    np.random.seed(0)
    br = np.random.randint(0, N // bs)
    bc = np.random.randint(0, N // bs)
    a = np.repeat(np.arange(br * bs, br * bs + bs), bs)
    b = np.tile(np.arange(bc * bs, bc * bs + bs), bs)
    np.testing.assert_array_equal(out, np.stack([a, b]))
    assert out.shape == (2, 256)


def test_blockize_counts_and_offsets_two_partitions():
    # k = 2 with 32 nodes each and every partition pair non-empty (so the compact-count quirk is
    # inactive): pair (i,j) with c edges emits int(c/256)+1 blocks inside [off_i, off_i+32) x [off_j, off_j+32)
    rng = np.random.default_rng(0)
    N, k, bs = 64, 2, 16
    part = np.repeat([0, 1], 32)
    counts = {(0, 0): 300, (0, 1): 10, (1, 0): 257, (1, 1): 600}
    src, dst = [], []
    for (i, j), c in counts.items():
        src.append(rng.integers(0, 32, c) + 32 * i)
        dst.append(rng.integers(0, 32, c) + 32 * j)
    ei = np.stack([np.concatenate(src), np.concatenate(dst)])
    mapping = gp.relabel_by_partition(part, k)
    out = gp.blockize(ei, k, part, 1, bs, mapping)
    pos = 0
    for (i, j), c in counts.items():
        nblk = c // 256 + 1
        blk = out[:, pos:pos + nblk * 256]
        assert blk[0].min() >= 32 * i and blk[0].max() < 32 * (i + 1)
        assert blk[1].min() >= 32 * j and blk[1].max() < 32 * (j + 1)
        for t in range(nblk):
            one = blk[:, t * 256:(t + 1) * 256]
            r0, c0 = one[0, 0], one[1, 0]
            assert r0 % bs == 0 and c0 % bs == 0
            np.testing.assert_array_equal(one[0], np.repeat(np.arange(r0, r0 + bs), bs))
            np.testing.assert_array_equal(one[1], np.tile(np.arange(c0, c0 + bs), bs))
        pos += nblk * 256
    assert pos == out.shape[1]


def test_blockize_compact_counts_and_raw_edge_branch_by_hand():
    """Hand-computed answer for the two branches nothing else pins (gt_sp/utils.py:237-246, 270-283).
    7 nodes in 3 parts of 2, 3, 2 nodes (already in part order, so the relabelling is the identity), block
    size 2: every part holds exactly one block row, so every randint(0, 1) is 0 and no random stream enters.
    Non-empty partition pairs in sorted order: (0,0) 5 edges, (0,2) 7, (1,0) 3, (1,2) 1, (2,2) 5.  The reference
    stores these counts compactly, [5, 7, 3, 1, 5, 0, 0, 0, 0], and reads entry i*3+j for pair (i, j):
      (0,0) reads 5 > 2*2      -> raw branch: the 5 sorted edges of slice [0, 5)
      (0,1) reads 7 > 2*3      -> raw branch: slice [5, 12), which holds the edges of pair (0,2)
      (0,2) reads 3 <= 4       -> int(3/4)+1 = 1 block on rows {0,1} x columns {5,6}
      (1,0) reads 1            -> 1 block rows {2,3} x columns {0,1}
      (1,1) reads 5 <= 9       -> int(5/4)+1 = 2 (identical) blocks rows {2,3} x columns {2,3}
      (1,2), (2,0), (2,1), (2,2) read 0 -> 1 block each."""
    part = np.array([0, 0, 1, 1, 1, 2, 2])
    pairs = [(1, 0), (0, 1), (0, 1), (1, 1), (0, 0),                          # (0,0), unsorted on purpose
             (1, 6), (0, 5), (0, 5), (1, 5), (0, 6), (1, 6), (0, 5),          # (0,2)
             (4, 0), (2, 0), (3, 1),                                          # (1,0)
             (2, 5),                                                          # (1,2)
             (6, 6), (5, 5), (5, 6), (6, 5), (5, 5)]                          # (2,2)
    ei = np.array(pairs).T
    mapping = gp.relabel_by_partition(part, 3)
    np.testing.assert_array_equal(mapping, np.arange(7))
    out = gp.blockize(ei, 3, part, 1, 2, mapping)

    def block(r0, c0):
        return [(r0, c0), (r0, c0 + 1), (r0 + 1, c0), (r0 + 1, c0 + 1)]
    want = ([(0, 0), (0, 1), (0, 1), (1, 0), (1, 1)]
            + [(0, 5), (0, 5), (0, 5), (0, 6), (1, 5), (1, 6), (1, 6)]
            + block(0, 5) + block(2, 0) + block(2, 2) + block(2, 2) + block(2, 5)
            + block(5, 0) + block(5, 2) + block(5, 5))
    np.testing.assert_array_equal(out, np.array(want).T)


def test_reformat_graph_sorted_by_source_stably():
    rng = np.random.default_rng(1)
    N, k = 96, 3
    part = rng.integers(0, k, N)
    part[:48] = np.repeat([0, 1, 2], 16)           # every part has >= 16 nodes
    ei = rng.integers(0, N, (2, 400))
    edges, sorted_indices = gp.reformat_graph(ei, part, k, 16)
    assert np.all(np.diff(edges[0]) >= 0)
    mapping = gp.relabel_by_partition(part, k)
    np.testing.assert_array_equal(mapping[sorted_indices], np.arange(N))   # new -> old inverse
    raw = gp.blockize(ei, k, part, 1, 16, mapping)
    # stable: among equal sources the emission order is kept
    for s in np.unique(raw[0])[:10]:
        np.testing.assert_array_equal(edges[1][edges[0] == s], raw[1][raw[0] == s])


@pytest.mark.parametrize("by", ["dst", "src"])
def test_build_csr_invariants(by):
    rng = np.random.default_rng(2)
    N, E = 50, 600
    ei = rng.integers(0, N, (2, E))
    ei[:, :100] = ei[:, 100:200]                    # duplicates
    rowptr, col, eid = gp.build_csr(ei, N, by)
    key, other = (ei[1], ei[0]) if by == "dst" else (ei[0], ei[1])
    assert rowptr[0] == 0 and rowptr[-1] == E and np.all(np.diff(rowptr) >= 0)
    np.testing.assert_array_equal(np.sort(eid), np.arange(E))
    np.testing.assert_array_equal(np.diff(rowptr), np.bincount(key, minlength=N))
    for r in range(N):
        seg = eid[rowptr[r]:rowptr[r + 1]]
        assert np.all(key[seg] == r)
        assert np.all(np.diff(seg) > 0)             # stable: caller's order inside a row
    np.testing.assert_array_equal(col, other[eid])


def test_gen_sub_edge_index_known_answer():
    # N = 6; batch [3, 0, 2] renames 3 -> 0, 0 -> 1, 2 -> 2.  Input self-loops (1,1), (5,5) are dropped;
    # kept, in input order: (2,3) (3,2) (2,0); then the batch nodes' self-loops in ascending ORIGINAL id 0, 2, 3.
    e = np.array([[0, 1, 2, 3, 4, 1, 5, 2],
                  [1, 1, 3, 2, 5, 0, 5, 0]])
    got = gp.gen_sub_edge_index(e, [3, 0, 2], 6)
    want = np.array([[2, 0, 2, 1, 2, 0],
                     [0, 2, 1, 1, 2, 0]])
    np.testing.assert_array_equal(got, want)


def _sub_edge_index_bruteforce(e, idx, N):
    """Independent statement: Python loops and a dict."""
    pos = {}
    for p, v in enumerate(idx):
        pos[int(v)] = p                      # the last position of a repeated node wins
    out = []
    for s, d in zip(e[0].tolist(), e[1].tolist()):
        if s != d and s in pos and d in pos:
            out.append((pos[s], pos[d]))
    for v in range(N):
        if v in pos:
            out.append((pos[v], pos[v]))
    return np.array(out, dtype=np.int64).reshape(-1, 2).T


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_gen_sub_edge_index_matches_bruteforce(seed):
    rng = np.random.default_rng(seed)
    N, E = 50, 400
    e = rng.integers(0, N, size=(2, E))
    idx = rng.permutation(N)[:17] if seed < 2 else rng.integers(0, N, size=23)     # seed 2: repeated nodes
    got = gp.gen_sub_edge_index(e, idx, N)
    np.testing.assert_array_equal(got, _sub_edge_index_bruteforce(e, idx, N))
    # every kept edge maps back to an input edge or to a self-loop of a batch node
    back = np.asarray(idx)[got]
    pairs = set(zip(e[0].tolist(), e[1].tolist()))
    for s, d in zip(back[0].tolist(), back[1].tolist()):
        assert s == d or (s, d) in pairs
    assert (got[0] == got[1]).sum() == len(set(np.asarray(idx).tolist()))


def test_gen_sub_edge_index_empty_batch_and_no_edges():
    e = np.zeros((2, 0), dtype=np.int64)
    np.testing.assert_array_equal(gp.gen_sub_edge_index(e, [2, 1], 4), np.array([[1, 0], [1, 0]]))
    assert gp.gen_sub_edge_index(np.array([[0, 1], [1, 0]]), [], 3).shape == (2, 0)


def test_floyd_warshall_known_answer_and_scipy():
    # path graph 0-1-2-3 plus an isolated node 4
    adj = np.zeros((5, 5), dtype=np.int64)
    for a, b in ((0, 1), (1, 2), (2, 3)):
        adj[a, b] = adj[b, a] = 1
    M, path = gp.floyd_warshall(adj)
    want = np.array([[0, 1, 2, 3, 510], [1, 0, 1, 2, 510], [2, 1, 0, 1, 510], [3, 2, 1, 0, 510], [510] * 4 + [0]])
    np.testing.assert_array_equal(M, want)
    assert path[0, 1] == -1 and path[0, 2] == 1 and path[0, 4] == 510 and path[4, 4] == -1
    assert path[0, 3] == 2        # the improvement through k = 2 comes last (k = 1 gave 0-1-..-3 only after 1-3 was known)
    # distances against scipy's shortest paths on random graphs
    from scipy.sparse.csgraph import shortest_path
    rng = np.random.default_rng(0)
    for n in (7, 20):
        a = (rng.random((n, n)) < 0.15).astype(np.int64)
        a = np.maximum(a, a.T)
        np.fill_diagonal(a, 0)
        M, path = gp.floyd_warshall(a)
        d = shortest_path(a, method="D", unweighted=True)
        d[np.isinf(d)] = 510
        np.testing.assert_array_equal(M, d.astype(np.int64))
        # every recorded intermediate node splits the distance exactly
        for i in range(n):
            for j in range(n):
                k = path[i, j]
                if 0 <= k < 510:
                    assert M[i, j] == M[i, k] + M[k, j]
                elif k == -1:
                    assert i == j or a[i, j] == 1


def test_floyd_warshall_by_steps_is_the_loop():
    """The one-array-operation-per-k form used for graphs of more than 128 nodes gives the loop's matrices
    (distances and recorded intermediate nodes), on undirected, directed and weighted graphs."""
    rng = np.random.default_rng(3)
    for n, p, directed, wmax in ((1, 0.0, False, 1), (9, 0.3, False, 1), (33, 0.08, False, 1), (40, 0.06, True, 1),
                                 (25, 0.15, True, 4), (30, 0.02, False, 1)):
        a = (rng.random((n, n)) < p) * rng.integers(1, wmax + 1, size=(n, n))
        if not directed:
            a = np.maximum(a, a.T)
        M0, P0 = gp.floyd_warshall(a)
        M1, P1 = gp.floyd_warshall_by_steps(a)
        np.testing.assert_array_equal(M0, M1)
        np.testing.assert_array_equal(P0, P1)
    # and against scipy's distances at a size the loop is too slow for
    from scipy.sparse.csgraph import shortest_path
    a = (rng.random((200, 200)) < 0.012).astype(np.int64)
    a = np.maximum(a, a.T)
    np.fill_diagonal(a, 0)
    M, _ = gp.floyd_warshall_by_steps(a)
    d = shortest_path(a, method="D", unweighted=True)
    d[np.isinf(d)] = 510
    np.testing.assert_array_equal(M, d.astype(np.int64))


def test_gen_edge_input_known_answer_and_walk_property():
    # path graph 0-1-2-3 plus an isolated node 4; the feature of edge (a, b) is (10 a + b, 7)
    n = 5
    adj = np.zeros((n, n), dtype=np.int64)
    for a, b in ((0, 1), (1, 2), (2, 3)):
        adj[a, b] = adj[b, a] = 1
    feat = np.zeros((n, n, 2), dtype=np.int64)
    for a in range(n):
        for b in range(n):
            if adj[a, b]:
                feat[a, b] = (10 * a + b, 7)
    M, path = gp.floyd_warshall(adj)
    out = gp.gen_edge_input(3, path, feat)
    assert out.shape == (n, n, 3, 2) and out.dtype == np.int64
    np.testing.assert_array_equal(out[0, 3], [[1, 7], [12, 7], [23, 7]])      # 0-1, 1-2, 2-3
    np.testing.assert_array_equal(out[3, 0], [[32, 7], [21, 7], [10, 7]])     # 3-2, 2-1, 1-0
    np.testing.assert_array_equal(out[1, 2], [[12, 7], [-1, -1], [-1, -1]])
    assert (out[2, 2] == -1).all() and (out[0, 4] == -1).all() and (out[4, 1] == -1).all()
    # a smaller max_dist keeps the first hops
    np.testing.assert_array_equal(gp.gen_edge_input(2, path, feat)[0, 3], [[1, 7], [12, 7]])
    # random graphs: the hops of (i, j) form a walk of existing edges from i to j of the shortest length
    rng = np.random.default_rng(1)
    for n in (9, 24):
        a = (rng.random((n, n)) < 0.15).astype(np.int64)
        a = np.maximum(a, a.T)
        np.fill_diagonal(a, 0)
        M, path = gp.floyd_warshall(a)
        code = np.zeros((n, n, 1), dtype=np.int64)             # the feature names the edge: a * n + b
        code[:, :, 0] = np.arange(n)[:, None] * n + np.arange(n)[None, :]
        md = int(M[M < 510].max())
        out = gp.gen_edge_input(md, path, code)
        for i in range(n):
            for j in range(n):
                hops = out[i, j, :, 0]
                real = hops[hops >= 0]
                if i == j or M[i, j] == 510:
                    assert real.size == 0
                    continue
                assert real.size == M[i, j] and (hops[:real.size] >= 0).all()
                cur = i
                for h in real:
                    s_, t_ = divmod(int(h), n)
                    assert s_ == cur and a[s_, t_] == 1
                    cur = t_
                assert cur == j
