"""Pins of the dense-attention oracle (CPU only): brute-force loops from the
definition (with the reference's q*sqrt(d) quirk), -inf key padding, and the
bias producer against explicit loops."""
import math

import torch

from oracle import dense_attention as oda


def test_dense_matches_bruteforce_with_bias_and_padding():
    g = torch.Generator().manual_seed(0)
    b, S, H, d = 2, 7, 3, 8
    q, k, v = (torch.randn(b, S, H, d, generator=g, dtype=torch.float64) * 0.5 for _ in range(3))
    bias = torch.randn(b, H, S, S, generator=g, dtype=torch.float64)
    bias[1, :, :, 5:] = float("-inf")            # graph 1 has 5 real nodes: padded keys masked
    out = oda.dense_attention(q, k, v, bias)
    ref = oda.dense_attention_bruteforce(q, k, v, bias)
    torch.testing.assert_close(out, ref, rtol=1e-11, atol=1e-13)
    assert out.shape == (b, S, H * d)


def test_q_is_multiplied_by_sqrt_d_not_divided():
    g = torch.Generator().manual_seed(1)
    b, S, H, d = 1, 5, 1, 16
    q, k, v = (torch.randn(b, S, H, d, generator=g, dtype=torch.float64) * 0.3 for _ in range(3))
    out = oda.dense_attention(q, k, v)
    scores = torch.einsum("bqhd,bkhd->bhqk", q, k) * math.sqrt(d)        # graphormer_graph_level.py:198
    expect = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(scores, -1), v).reshape(b, S, -1)
    torch.testing.assert_close(out, expect)
    wrong = torch.einsum("bhqk,bkhd->bqhd", torch.softmax(scores / d, -1), v).reshape(b, S, -1)
    assert (out - wrong).abs().max() > 1e-3


def test_graph_attn_bias_against_loops():
    g = torch.Generator().manual_seed(2)
    b, S, H, F = 2, 4, 3, 2
    attn_bias = torch.zeros(b, S + 1, S + 1, dtype=torch.float64)
    attn_bias[1, :, 4:] = float("-inf")
    spatial = torch.randint(0, 6, (b, S, S), generator=g)
    etype = torch.randint(0, 4, (b, S, S, F), generator=g)
    st = torch.randn(6, H, generator=g, dtype=torch.float64); st[0] = 0
    et = torch.randn(4, H, generator=g, dtype=torch.float64); et[0] = 0
    vd = torch.randn(1, H, generator=g, dtype=torch.float64)
    out = oda.graph_attn_bias(attn_bias, spatial, etype, st, et, vd)
    for gi in range(b):
        for h in range(H):
            for i in range(S + 1):
                for j in range(S + 1):
                    x = 2 * attn_bias[gi, i, j]                       # :104 clone + :153 "reset" add
                    if i >= 1 and j >= 1:
                        x = x + st[spatial[gi, i - 1, j - 1], h] + et[etype[gi, i - 1, j - 1], h].mean()
                    if i == 0 or j == 0:
                        x = x + vd[0, h]
                    got = out[gi, h, i, j]
                    assert (torch.isinf(x) and torch.isinf(got)) or abs(float(got - x)) < 1e-12


def _multi_hop_case(seed, b=2, S=5, H=3, D0=4, F=2, ne=6, nsp=9):
    g = torch.Generator().manual_seed(seed)
    attn_bias = torch.zeros(b, S + 1, S + 1, dtype=torch.float64)
    attn_bias[1, :, S:] = float("-inf")
    spatial_pos = torch.randint(0, nsp, (b, S, S), generator=g)
    edge_input = torch.randint(0, ne, (b, S, S, D0, F), generator=g)
    st = torch.randn(nsp, H, generator=g, dtype=torch.float64)
    et = torch.randn(ne, H, generator=g, dtype=torch.float64)
    w = torch.randn(7 * H * H, 1, generator=g, dtype=torch.float64)
    vd = torch.randn(1, H, generator=g, dtype=torch.float64)
    return attn_bias, spatial_pos, edge_input, st, et, w, vd


def test_multi_hop_bias_matches_loops_from_the_definition():
    for mhd in (3, 0, 6):       # fewer hops than the input holds, no limit, more
        attn_bias, sp, ei, st, et, w, vd = _multi_hop_case(mhd)
        got = oda.graph_attn_bias_multi_hop(attn_bias, sp, ei, st, et, w, vd, mhd)
        b, S = sp.shape[:2]
        H, D0, F = st.shape[1], ei.shape[3], ei.shape[4]
        D = min(D0, mhd) if mhd > 0 else D0
        W = w.reshape(-1, H, H)
        want = torch.zeros(b, H, S + 1, S + 1, dtype=torch.float64)
        for g in range(b):
            for h in range(H):
                for i in range(S + 1):
                    for j in range(S + 1):
                        x = 2 * attn_bias[g, i, j]
                        if i == 0 or j == 0:
                            x = x + vd[0, h]
                        else:
                            p = int(sp[g, i - 1, j - 1])
                            x = x + st[p, h]
                            hops = 1 if p <= 1 else p - 1            # pad -> 1, distance + 1 -> distance, self -> 1
                            if mhd > 0:
                                hops = min(hops, mhd)
                            acc = 0.0
                            for dd in range(D):
                                for h0 in range(H):
                                    mean = sum(et[int(ei[g, i - 1, j - 1, dd, f]), h0] for f in range(F)) / F
                                    acc = acc + mean * W[dd, h0, h]
                            x = x + acc / hops
                        want[g, h, i, j] = x
        fin = torch.isfinite(want)
        assert torch.equal(torch.isfinite(got), fin)
        torch.testing.assert_close(got[fin], want[fin], rtol=1e-11, atol=1e-12)


def test_multi_hop_bias_reduces_to_the_single_hop_branch():
    # one hop, identity hop matrix, every pair adjacent (or self / pad): the path encoding is the edge encoding
    attn_bias, sp, ei, st, et, w, vd = _multi_hop_case(5)
    H = st.shape[1]
    sp = sp.clamp(0, 2)
    w = torch.eye(H, dtype=torch.float64).repeat(7, 1, 1).reshape(-1, 1)
    got = oda.graph_attn_bias_multi_hop(attn_bias, sp, ei, st, et, w, vd, 1)
    want = oda.graph_attn_bias(attn_bias, sp, ei[:, :, :, 0, :], st, et, vd)
    fin = torch.isfinite(want)
    torch.testing.assert_close(got[fin], want[fin], rtol=1e-12, atol=1e-13)
    # twice the distance halves the edge term: spatial_pos 3 (two hops) against 2 (one hop), zero spatial table
    z = torch.zeros_like(st)
    a1 = oda.graph_attn_bias_multi_hop(torch.zeros_like(attn_bias), torch.full_like(sp, 2), ei, z, et, w, vd * 0, 0)
    a2 = oda.graph_attn_bias_multi_hop(torch.zeros_like(attn_bias), torch.full_like(sp, 3), ei, z, et, w, vd * 0, 0)
    torch.testing.assert_close(a1[:, :, 1:, 1:], 2 * a2[:, :, 1:, 1:], rtol=1e-12, atol=1e-13)


def test_dropout_mask_is_dropout_of_the_softmax_output():
    """``att_dropout`` with an explicit mask: the oracle equals softmax -> torch's dropout arithmetic (zero the
    dropped entries, scale the kept ones by 1 / (1 - p)) -> times v, written out with loops; an all-ones mask with
    p = 0 is the plain forward."""
    import math
    g = torch.Generator().manual_seed(3)
    b, S, H, d, p = 2, 5, 2, 4, 0.25
    q, k, v = (torch.randn(b, S, H, d, generator=g, dtype=torch.float64) for _ in range(3))
    bias = torch.randn(b, H, S, S, generator=g, dtype=torch.float64)
    keep = (torch.rand(b, H, S, S, generator=g) > p)
    got = oda.dense_attention(q, k, v, bias, drop_keep=keep, p_drop=p)
    want = torch.zeros(b, S, H * d, dtype=torch.float64)
    for gi in range(b):
        for h in range(H):
            for i in range(S):
                sc = torch.stack([(q[gi, i, h] * math.sqrt(d) * k[gi, j, h]).sum() + bias[gi, h, i, j] for j in range(S)])
                w = torch.softmax(sc, 0) * keep[gi, h, i].double() / (1 - p)
                want[gi, i, h * d:(h + 1) * d] = (w.unsqueeze(1) * v[gi, :, h]).sum(0)
    assert (got - want).abs().max() < 1e-12
    ones = torch.ones(b, H, S, S)
    assert torch.equal(oda.dense_attention(q, k, v, bias, drop_keep=ones, p_drop=0.0), oda.dense_attention(q, k, v, bias))
