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
