"""Pins of the sparse-attention oracle (CPU only).

The reference has no tests or fixtures for this path, so the restatement in
``oracle/sparse_attention.py`` is pinned by what the mathematics fixes:
library softmax on a complete graph, fp64 brute-force loops from the
definition, closed-form special cases and invariants.  A dropped term, wrong
sign, swapped src/dst or transposed bias fails at least one of these.
"""
import math

import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa


def _rand_graph(N, E, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, N, (2, E), generator=g)


def _qkv(N, H, d, seed, scale=1.0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(N, H, d, generator=g, dtype=dtype) * scale for _ in range(3))


def test_dense_softmax_equivalence():
    # complete directed graph incl. self-loops, small scores (no clamp active):
    # out = softmax(Q K^T / sqrt(d) + B^T) V * Z / (Z + eps)   with B indexed [src, dst]
    N, H, d = 12, 3, 8
    q, k, v = _qkv(N, H, d, 0, scale=0.5)
    src, dst = torch.meshgrid(torch.arange(N), torch.arange(N), indexing="ij")
    ei = torch.stack([src.reshape(-1), dst.reshape(-1)])
    B = torch.randn(N, N, H, dtype=torch.float64, generator=torch.Generator().manual_seed(1))  # [src, dst, h]
    eb = B[ei[0], ei[1]]
    out, Z = osa.sparse_attention(q, k, v, ei, eb)
    scores = torch.einsum("ihc,jhc->hij", q, k) / math.sqrt(d)      # [h, dst i, src j]
    assert scores.abs().max() < 5
    scores = scores + B.permute(2, 1, 0)                              # B[src j, dst i] -> [h, i, j]
    P = torch.softmax(scores, dim=-1)
    dense = torch.einsum("hij,jhc->ihc", P, v)
    Zd = torch.exp(scores).sum(-1).t()                                # [i, h]
    torch.testing.assert_close(Z, Zd, rtol=1e-12, atol=0)
    torch.testing.assert_close(out, dense * (Zd / (Zd + 1e-6)).unsqueeze(-1), rtol=1e-12, atol=1e-14)


def test_src_dst_roles_not_swapped():
    # a single edge j -> i: only row i receives, and it receives v[j]
    N, H, d = 5, 2, 8
    q, k, v = _qkv(N, H, d, 2)
    ei = torch.tensor([[3], [1]])
    out, Z = osa.sparse_attention(q, k, v, ei)
    raw = ((k[3] * q[1]).sum(-1) / math.sqrt(d)).clamp(-5, 5)
    w = torch.exp(raw)
    torch.testing.assert_close(out[1], v[3] * (w / (w + 1e-6)).unsqueeze(-1))
    assert torch.count_nonzero(out[[0, 2, 3, 4]]) == 0          # zero in-degree -> exactly 0
    torch.testing.assert_close(Z[1], w)


@pytest.mark.parametrize("bias_kind", ["none", "edge", "edge_head"])
def test_bruteforce(bias_kind):
    N, H, d, E = 9, 2, 8, 40
    q, k, v = _qkv(N, H, d, 3, scale=1.5)
    ei = _rand_graph(N, E, 4)
    g = torch.Generator().manual_seed(5)
    eb = {"none": None, "edge": torch.randn(E, generator=g, dtype=torch.float64),
          "edge_head": torch.randn(E, H, generator=g, dtype=torch.float64)}[bias_kind]
    out, _ = osa.sparse_attention(q, k, v, ei, eb)
    ref = osa.sparse_attention_bruteforce(q, k, v, ei, eb)
    torch.testing.assert_close(out, ref, rtol=1e-11, atol=1e-13)


def test_clamp_before_bias_and_saturation():
    # scores far beyond +-5 saturate to exp(+-5); the bias is added after the clamp
    N, H, d = 3, 1, 8
    q = torch.zeros(N, H, d, dtype=torch.float64)
    k = torch.zeros(N, H, d, dtype=torch.float64)
    v = torch.randn(N, H, d, dtype=torch.float64, generator=torch.Generator().manual_seed(6))
    q[0] = 10.0
    k[1] = 10.0      # raw = 8*100/sqrt(8) >> 5
    k[2] = -10.0     # raw << -5
    ei = torch.tensor([[1, 2], [0, 0]])
    eb = torch.tensor([0.25, -0.5], dtype=torch.float64)
    out, Z = osa.sparse_attention(q, k, v, ei, eb)
    w1, w2 = math.exp(5 + 0.25), math.exp(-5 - 0.5)
    assert Z[0, 0].item() == pytest.approx(w1 + w2, rel=1e-14)
    torch.testing.assert_close(out[0], (w1 * v[1] + w2 * v[2]) / (w1 + w2 + 1e-6))


def test_duplicate_edge_counts_twice_and_neg_inf_bias():
    N, H, d = 4, 2, 8
    q, k, v = _qkv(N, H, d, 7)
    ei = torch.tensor([[1, 1, 2], [0, 0, 0]])
    out, Z = osa.sparse_attention(q, k, v, ei)
    ei1 = torch.tensor([[1, 2], [0, 0]])
    eb1 = torch.tensor([math.log(2.0), 0.0], dtype=torch.float64)   # doubling the weight
    out1, Z1 = osa.sparse_attention(q, k, v, ei1, eb1)
    torch.testing.assert_close(out, out1)
    torch.testing.assert_close(Z, Z1)
    # -inf bias removes the edge; all -inf -> exact zeros, no NaN
    eb = torch.full((3,), float("-inf"), dtype=torch.float64)
    out2, Z2 = osa.sparse_attention(q, k, v, ei, eb)
    assert torch.count_nonzero(out2) == 0 and torch.count_nonzero(Z2) == 0
    assert not torch.isnan(out2).any()


def test_invariants_permutation_relabel_heads_batch():
    N, H, d, E = 20, 4, 8, 90
    q, k, v = _qkv(N, H, d, 8)
    ei = _rand_graph(N, E, 9)
    eb = torch.randn(E, H, dtype=torch.float64, generator=torch.Generator().manual_seed(10))
    out, Z = osa.sparse_attention(q, k, v, ei, eb)
    # edge-order permutation
    perm = torch.randperm(E, generator=torch.Generator().manual_seed(11))
    out_p, _ = osa.sparse_attention(q, k, v, ei[:, perm], eb[perm])
    torch.testing.assert_close(out, out_p, rtol=1e-12, atol=1e-14)
    # node relabelling equivariance
    pi = torch.randperm(N, generator=torch.Generator().manual_seed(12))     # new id of old node
    inv = torch.argsort(pi)
    out_r, _ = osa.sparse_attention(q[inv], k[inv], v[inv], pi[ei], eb)
    torch.testing.assert_close(out_r[pi], out, rtol=1e-12, atol=1e-14)
    # head independence (what head-sharded sequence parallelism relies on)
    for h in range(H):
        o_h, _ = osa.sparse_attention(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], ei, eb[:, h:h + 1])
        torch.testing.assert_close(o_h[:, 0], out[:, h], rtol=1e-12, atol=1e-14)
    # two graphs in one batch with disjoint index ranges are independent
    q2, k2, v2 = _qkv(N, H, d, 13)
    ei2 = _rand_graph(N, 50, 14)
    ob, _ = osa.sparse_attention(torch.stack([q, q2]), torch.stack([k, k2]), torch.stack([v, v2]),
                                 torch.cat([ei, ei2 + N], 1))
    oa, _ = osa.sparse_attention(q, k, v, ei)
    oc, _ = osa.sparse_attention(q2, k2, v2, ei2)
    torch.testing.assert_close(ob, torch.cat([oa, oc]), rtol=1e-12, atol=1e-14)


def test_analytic_backward_matches_autograd():
    N, H, d, E = 15, 2, 8, 70
    q, k, v = _qkv(N, H, d, 15, scale=2.0)     # some scores beyond +-5 -> clamp mask exercised
    ei = _rand_graph(N, E, 16)
    eb = torch.randn(E, H, dtype=torch.float64, generator=torch.Generator().manual_seed(17))
    for t in (q, k, v, eb):
        t.requires_grad_(True)
    out, Z = osa.sparse_attention(q, k, v, ei, eb)
    g = torch.randn(out.shape, dtype=torch.float64, generator=torch.Generator().manual_seed(18))
    dq, dk, dv, db = torch.autograd.grad(out, (q, k, v, eb), g)
    raw = (k[ei[0]] * q[ei[1]] / math.sqrt(d)).sum(-1)
    assert (raw.abs() > 5).any() and (raw.abs() < 5).any()
    aq, ak, av, ab = osa.sparse_attention_backward_analytic(
        q.detach(), k.detach(), v.detach(), ei, eb.detach(), out.detach(), Z.detach(), g)
    for a, b in ((aq, dq), (ak, dk), (av, dv), (ab, db)):
        torch.testing.assert_close(a, b, rtol=1e-10, atol=1e-12)


def test_gradcheck_of_restatement():
    N, H, d, E = 6, 1, 8, 14
    q, k, v = _qkv(N, H, d, 19, scale=0.7)
    ei = _rand_graph(N, E, 20)
    eb = torch.randn(E, dtype=torch.float64, generator=torch.Generator().manual_seed(21))
    for t in (q, k, v, eb):
        t.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b, c, e: osa.sparse_attention(a, b, c, ei, e)[0], (q, k, v, eb))


def test_clamp_mask_inclusive_at_exactly_five():
    # d = 16 -> scale 4; q.k = 20 exactly -> raw = 5.0 exactly: gradient flows (torch clamp backward)
    N, H, d = 2, 1, 16
    q = torch.zeros(N, H, d, dtype=torch.float32)
    k = torch.zeros(N, H, d, dtype=torch.float32)
    v = torch.randn(N, H, d, generator=torch.Generator().manual_seed(22))
    q[0, 0, 0] = 4.0
    k[1, 0, 0] = 5.0
    k[0, 0, 0] = 0.5
    ei = torch.tensor([[1, 0], [0, 0]])
    q.requires_grad_(True)
    out, Z = osa.sparse_attention(q, k, v, ei)
    raw = (k[ei[0]] * q[ei[1]] / 4.0).sum(-1)
    assert raw[0, 0].item() == 5.0
    g = torch.ones_like(out)
    (dq,) = torch.autograd.grad(out, (q,), g)
    aq, _, _, _ = osa.sparse_attention_backward_analytic(q.detach(), k, v, ei, None, out.detach(), Z.detach(), g)
    torch.testing.assert_close(aq, dq)
    # and the edge at exactly 5 does contribute: compare with the mask forced off
    w = torch.exp(raw[:, 0].detach())
    assert dq[0, 0, 0].abs() > 0 and w[0] == pytest.approx(math.exp(5.0))


def test_dense_bias_gather_matches_loops():
    b, S, H = 2, 5, 3
    bias = torch.randn(b, H, S, S, dtype=torch.float64, generator=torch.Generator().manual_seed(23))
    ei = torch.tensor([[0, 4, 6, 9, 7], [1, 0, 8, 5, 7]])     # edges inside each graph
    eb = osa.dense_bias_to_edge_bias(bias, ei, "bhss")
    for e in range(ei.shape[1]):
        s, t = int(ei[0, e]), int(ei[1, e])
        g = s // S
        torch.testing.assert_close(eb[e], bias[g, :, s % S, t % S])
    eb2 = osa.dense_bias_to_edge_bias(bias.permute(0, 2, 3, 1).contiguous(), ei, "bssh")
    torch.testing.assert_close(eb, eb2)
