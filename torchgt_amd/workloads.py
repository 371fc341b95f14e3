"""Seeded synthetic graphs for the benchmark configurations (host side, numpy).

No dataset can be downloaded, so every workload is generated.  Each builder
returns ``edge_index`` as int64 ``[2, E]`` (row 0 = source / key node, row 1 =
destination / query node) in the layout the reference feeds its attention:
real nodes shifted by +1, a global node at index 0 linked to and from every
real node (``gt_sp/utils.py:34-50``), and a self-loop on every real node
(``gt_sp/utils.py:211-212``).
"""
import hashlib

import numpy as np


def add_global_node(edge_index, num_node):
    """Closed form of ``fix_edge_index`` (gt_sp/utils.py:34-50)."""
    ar = np.arange(1, num_node + 1, dtype=np.int64)
    z = np.zeros(num_node, dtype=np.int64)
    return np.concatenate(
        [np.asarray(edge_index, dtype=np.int64) + 1, np.stack([ar, z]), np.stack([z, ar])], axis=1)


def _symmetrize_with_self_loops(und, n):
    """und: [M, 2] undirected simple edges -> directed both ways + self-loops."""
    a, b = und[:, 0], und[:, 1]
    loops = np.arange(n, dtype=np.int64)
    src = np.concatenate([a, b, loops])
    dst = np.concatenate([b, a, loops])
    return np.stack([src, dst])


def _simple_pairs(a, b, n):
    """Drop self-pairs and duplicate unordered pairs, keep first occurrence order."""
    keep = a != b
    a, b = a[keep], b[keep]
    lo, hi = np.minimum(a, b), np.maximum(a, b)
    key = lo * np.int64(n) + hi
    _, first = np.unique(key, return_index=True)
    first.sort()
    return np.stack([lo[first], hi[first]], axis=1)


def barabasi_albert(n=4096, m=4, seed=42):
    """Config 1: Barabasi-Albert (networkx generator), bidirectional, self-loops,
    global node.  N = n + 1."""
    import networkx as nx
    g = nx.barabasi_albert_graph(n, m, seed=seed)
    und = np.asarray(list(g.edges()), dtype=np.int64).reshape(-1, 2)
    e = _symmetrize_with_self_loops(und, n)
    return add_global_node(e, n), n + 1


def power_law_degrees(n, exponent, target_sum, kmax, rng):
    """Pareto-tailed integer degrees >= 1 with P(k) ~ k^-exponent, scaled by
    bisection on x_min so that sum(deg) ~= target_sum; capped at kmax."""
    u = rng.random(n)
    base = u ** (-1.0 / (exponent - 1.0))
    lo, hi = 0.05, 64.0
    for _ in range(60):
        mid = 0.5 * (lo + hi)
        deg = np.minimum(np.maximum(np.floor(mid * base), 1), kmax)
        if deg.sum() < target_sum:
            lo = mid
        else:
            hi = mid
    deg = np.minimum(np.maximum(np.floor(hi * base), 1), kmax).astype(np.int64)
    return deg


def configuration_model(n, exponent, mean_degree, kmax, seed, oversample=1.0):
    """Erased configuration model: random stub matching, self-pairs and
    multi-edges dropped.  Returns undirected simple edges [M, 2]."""
    rng = np.random.default_rng(seed)
    target = int(n * mean_degree * oversample)
    deg = power_law_degrees(n, exponent, target, kmax, rng)
    if deg.sum() % 2:
        deg[int(np.argmax(deg))] += 1
    stubs = np.repeat(np.arange(n, dtype=np.int64), deg)
    rng.shuffle(stubs)
    half = stubs.shape[0] // 2
    return _simple_pairs(stubs[:half], stubs[half:2 * half], n)


def power_law_graph(n=64000, exponent=2.1, directed_edges=530_000, kmax=None, seed=42):
    """Configs 2 and 3: power-law simple graph sized so that
    2*M + n (self-loops) + 2*n (global edges) ~= directed_edges.  N = n + 1."""
    m_target = (directed_edges - 3 * n) // 2
    if kmax is None:
        kmax = int(np.sqrt(2.0 * m_target))        # structural cutoff of a simple graph
    mean_deg = 2.0 * m_target / n
    und = configuration_model(n, exponent, mean_deg, kmax, seed, oversample=1.0)
    # the erased model loses a few percent of stubs; one corrective pass
    loss = m_target / max(1, und.shape[0])
    if abs(loss - 1.0) > 0.01:
        und = configuration_model(n, exponent, mean_deg, kmax, seed, oversample=loss)
    e = _symmetrize_with_self_loops(und, n)
    return add_global_node(e, n), n + 1


def spd_edge_ids(edge_index, clamp=5):
    """Per-edge bias id for config 1: shortest-path distance between the two
    endpoints on the real graph clamped to ``clamp`` (0 for a self-loop, 1 for
    an edge) and a separate id ``clamp + 1`` for edges touching the global
    node 0."""
    src, dst = edge_index
    ids = np.where(src == dst, 0, 1).astype(np.int64)
    ids = np.minimum(ids, clamp)
    ids[(src == 0) | (dst == 0)] = clamp + 1
    return ids


def stochastic_block_model(n_clusters=64, cluster_size=4096, p_intra=0.004, inter_fraction=0.05, seed=42):
    """Config 5: nodes ordered contiguously by cluster.  Every UNORDERED intra-cluster pair is
    sampled with probability p_intra and becomes ONE directed edge with a random direction;
    inter-cluster edges (random ordered pairs of different clusters) make up ``inter_fraction``
    of the total.  No global node, no self-loops.  Returns (edge_index, N, cluster_of_node)."""
    rng = np.random.default_rng(seed)
    n = n_clusters * cluster_size
    srcs, dsts = [], []
    pairs = cluster_size * (cluster_size - 1) // 2
    for c in range(n_clusters):
        m = rng.binomial(pairs, p_intra)
        # sample m distinct unordered pairs by rejection on ordered draws
        a = rng.integers(0, cluster_size, size=int(m * 1.05) + 16, dtype=np.int64)
        b = rng.integers(0, cluster_size, size=a.shape[0], dtype=np.int64)
        keep = a != b
        lo, hi = np.minimum(a[keep], b[keep]), np.maximum(a[keep], b[keep])
        _, first = np.unique(lo * cluster_size + hi, return_index=True)
        first = np.sort(first)[:m]
        lo, hi = lo[first], hi[first]
        flip = rng.random(lo.shape[0]) < 0.5
        srcs.append(np.where(flip, hi, lo) + c * cluster_size)
        dsts.append(np.where(flip, lo, hi) + c * cluster_size)
    intra = sum(x.shape[0] for x in srcs)
    m_inter = int(intra * inter_fraction / (1.0 - inter_fraction))
    a = rng.integers(0, n, size=int(m_inter * 1.03), dtype=np.int64)
    b = rng.integers(0, n, size=a.shape[0], dtype=np.int64)
    keep = (a // cluster_size) != (b // cluster_size)
    srcs.append(a[keep][:m_inter])
    dsts.append(b[keep][:m_inter])
    e = np.stack([np.concatenate(srcs), np.concatenate(dsts)])
    key = np.unique(e[0] * np.int64(n) + e[1])
    e = np.stack([key // n, key % n])
    e = e[:, rng.permutation(e.shape[1])]
    return e, n, np.repeat(np.arange(n_clusters, dtype=np.int64), cluster_size)


def hybrid_tiles(edge_index, cluster, n_clusters, block_size, seed=42):
    """Config 5 as a hybrid: every cluster's intra-cluster edges are replaced by int(count / bs^2) + 1 random
    dense bs x bs tiles inside the cluster (the recipe of generate_new_edges_optimized for one partition pair,
    gt_sp/utils.py:284-299, applied to the diagonal pairs only, with this module's own seeded generator); the
    inter-cluster edges stay as they are.  Nodes must be ordered contiguously by cluster.  Returns (tiles int32
    [T, 2] = first source / first destination, raw inter-cluster edges int64 [2, E_raw], the equivalent
    expanded edge list int64 [2, T * bs^2 + E_raw])."""
    rng = np.random.default_rng(seed)
    src, dst = np.asarray(edge_index[0]), np.asarray(edge_index[1])
    cs, cd = cluster[src], cluster[dst]
    intra = cs == cd
    counts = np.bincount(cs[intra], minlength=n_clusters)
    sizes = np.bincount(cluster, minlength=n_clusters)
    offs = np.concatenate([[0], np.cumsum(sizes)[:-1]])
    tiles = []
    for c in range(n_clusters):
        nb = sizes[c] // block_size
        if nb == 0:
            continue
        t = counts[c] // (block_size * block_size) + 1
        tiles.append(np.stack([rng.integers(0, nb, t) * block_size + offs[c],
                               rng.integers(0, nb, t) * block_size + offs[c]], 1))
    tiles = np.concatenate(tiles).astype(np.int32)
    raw = np.ascontiguousarray(np.stack([src[~intra], dst[~intra]]).astype(np.int64))
    ar = np.arange(block_size)
    a = (tiles[:, 0:1, None] + ar[None, :, None] + 0 * ar[None, None, :]).reshape(-1)
    b = (tiles[:, 1:2, None] + 0 * ar[None, :, None] + ar[None, None, :]).reshape(-1)
    expanded = np.concatenate([np.stack([a, b]).astype(np.int64), raw], axis=1)
    return tiles, raw, np.ascontiguousarray(expanded)


def clustered_power_law_graph(n=870_000, exponent=2.0, directed_edges=44_000_000, n_clusters=64,
                              intra_fraction=0.8, seed=42, oversample=None):
    """Config 3: power-law graph (mean degree ~50) whose nodes are grouped into contiguous
    clusters, the order a cluster / degree reordering leaves behind: a fraction
    ``intra_fraction`` of every node's stubs is matched inside its cluster, the rest globally.
    Bidirectional, self-loops, global node 0.  N = n + 1."""
    rng = np.random.default_rng(seed)
    m_target = (directed_edges - 3 * n) // 2
    kmax = int(np.sqrt(2.0 * m_target))
    first_pass = oversample is None
    deg = power_law_degrees(n, exponent, int(2 * m_target * (oversample or 1.0)), kmax, rng)
    csize = (n + n_clusters - 1) // n_clusters
    intra = rng.binomial(deg, intra_fraction)
    pairs = []
    for c in range(n_clusters):
        lo, hi = c * csize, min(n, (c + 1) * csize)
        stubs = np.repeat(np.arange(lo, hi, dtype=np.int64), intra[lo:hi])
        rng.shuffle(stubs)
        h = stubs.shape[0] // 2
        pairs.append(np.stack([stubs[:h], stubs[h:2 * h]], axis=1))
    stubs = np.repeat(np.arange(n, dtype=np.int64), deg - intra)
    rng.shuffle(stubs)
    h = stubs.shape[0] // 2
    pairs.append(np.stack([stubs[:h], stubs[h:2 * h]], axis=1))
    allp = np.concatenate(pairs)
    und = _simple_pairs(allp[:, 0], allp[:, 1], n)
    loss = m_target / max(1, und.shape[0])
    if first_pass and abs(loss - 1.0) > 0.02:      # the erased model drops multi-edges: one corrective pass
        return clustered_power_law_graph(n, exponent, directed_edges, n_clusters, intra_fraction, seed,
                                         oversample=loss)
    e = _symmetrize_with_self_loops(und, n)
    return add_global_node(e, n), n + 1


def erdos_renyi_batch(batch=256, n_min=16, n_max=128, p=0.1, n_edge_types=4, spd_clamp=20, seed=42):
    """Config 4: batch of G(n, p) graphs padded to n_max plus a virtual node 0
    (S = n_max + 1).  Returns a dict of numpy arrays in the collator's
    conventions (data/collator.py:50-76,248-251): ``spatial_pos`` = SPD + 1
    (0 = padding; unreachable pairs clamp to spd_clamp), ``edge_type`` in
    1..n_edge_types on edges (0 = none), ``attn_bias`` [b, S, S] with -inf on
    padded key columns, ``n_nodes`` [b]."""
    from scipy.sparse import csr_matrix
    from scipy.sparse.csgraph import shortest_path
    rng = np.random.default_rng(seed)
    S = n_max + 1
    spatial = np.zeros((batch, n_max, n_max), dtype=np.uint8)
    etype = np.zeros((batch, n_max, n_max), dtype=np.uint8)
    bias = np.zeros((batch, S, S), dtype=np.float32)
    sizes = rng.integers(n_min, n_max + 1, size=batch)
    for g in range(batch):
        n = int(sizes[g])
        upper = np.triu(rng.random((n, n)) < p, 1)
        adj = upper | upper.T
        dist = shortest_path(csr_matrix(adj.astype(np.int8)), method="D", unweighted=True)
        dist[~np.isfinite(dist)] = spd_clamp
        dist = np.minimum(dist, spd_clamp).astype(np.uint8)
        spatial[g, :n, :n] = dist + 1
        t = np.triu(rng.integers(1, n_edge_types + 1, size=(n, n)), 1)
        t = (t + t.T) * adj
        etype[g, :n, :n] = t.astype(np.uint8)
        bias[g, :, n + 1:] = -np.inf
    return {"spatial_pos": spatial, "edge_type": etype, "attn_bias": bias, "n_nodes": sizes.astype(np.int64), "S": S}


def describe(edge_index, num_nodes):
    """Exact N, E, max in/out degree and a sha256 of edge_index (for logs)."""
    e = np.ascontiguousarray(edge_index, dtype=np.int64)
    indeg = np.bincount(e[1], minlength=num_nodes)
    outdeg = np.bincount(e[0], minlength=num_nodes)
    return {
        "N": int(num_nodes), "E": int(e.shape[1]),
        "max_in_degree": int(indeg.max()), "max_out_degree": int(outdeg.max()),
        "sha256": hashlib.sha256(e.tobytes()).hexdigest()[:16],
    }
