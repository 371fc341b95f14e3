"""GPU parity of the dense attention that forms the graph-level bias on chip from packed ids and the three embedding
tables (``torch.ops.torchgt.dense_attention_ids`` over ``tgt_dense_attn_ids_fwd`` / ``_bwd``) with the oracle:
``oracle.dense_attention(q, k, v, oracle.graph_attn_bias(...))`` in float64, outputs, dq / dk / dv and the gradients of
the spatial, edge and virtual-distance tables (autograd through the oracle).  Error measure max|a - b| / max|b|; bar
2e-2 (bf16 matrix products, bf16 bias on chip), as for the dense kernels with a bias tensor; 3e-2 for the table
gradients, each a sum of thousands of signed dS terms of that accuracy whose exact sum partly cancels.  The id packing
is integer work: bit-exact against numpy.
"""
import types

import numpy as np
import pytest
import torch

from oracle import dense_attention as oda
from torchgt_amd import _ext, workloads
from torchgt_amd.core_attention import GraphBiasIds, dense_attention, dense_dropout_mask
from torchgt_amd.graph_bias import GraphAttnBias

pytestmark = pytest.mark.gpu
TOL = 2e-2
TOL_TABLE = 2e-2


def err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    assert a.shape == b.shape, (a.shape, b.shape)
    denom = b.abs().max().item()
    return (a - b).abs().max().item() / (denom if denom > 0 else 1.0)


def make_batch(b, s, F, ns, ne, seed):
    """A padded batch in the collator's conventions (data/collator.py:44-108): graph g has n_g <= s nodes, ids of padded
    pairs are 0, attn_bias is -inf on padded keys.  Some ids lie beyond their table (the kernels clamp them)."""
    rng = np.random.default_rng(seed)
    n = rng.integers(max(1, s // 4), s + 1, size=b)
    n[0] = s                                                   # one graph without padding
    sp = np.zeros((b, s, s), np.int64)
    et = np.zeros((b, s, s, F), np.int64)
    ab = np.zeros((b, s + 1, s + 1), np.float32)
    for g in range(b):
        m = int(n[g])
        sp[g, :m, :m] = rng.integers(1, ns + 3, size=(m, m)) * (rng.random((m, m)) < 0.9) + (rng.random((m, m)) < 0.02) * 40
        edge = rng.random((m, m)) < 0.15
        for f in range(F):
            et[g, :m, :m, f] = rng.integers(1, ne + 2, size=(m, m)) * edge * (rng.random((m, m)) < 0.8)
        ab[g, :, m + 1:] = -np.inf
    return n, torch.from_numpy(sp), torch.from_numpy(et), torch.from_numpy(ab)


def test_ids_pack_bit_exact(cuda):
    for (b, s, F, ns, ne) in ((3, 7, 1, 5, 4), (4, 32, 3, 40, 64), (2, 128, 2, 512, 1537)):
        _, sp, et, _ = make_batch(b, s, F, ns, ne, seed=s)
        sp[0, 0, 0] = -3                                       # negative ids clamp to 0
        sp16, et16 = _ext.ops().dense_ids_pack(sp.to(cuda), et.to(cuda), ns, ne)
        want_sp = np.full((b, s + 1, s + 1), ns, np.int64)
        want_sp[:, 1:, 1:] = np.clip(sp.numpy(), 0, ns - 1)
        want_et = np.full((b, s + 1, s + 1, F), ne, np.int64)
        want_et[:, 1:, 1:] = np.clip(et.numpy(), 0, ne - 1)
        assert sp16.dtype == torch.int16 and sp16.shape == (b, s + 1, s + 1) and et16.shape == (b, s + 1, s + 1, F)
        np.testing.assert_array_equal(sp16.cpu().numpy().astype(np.uint16).astype(np.int64), want_sp)
        np.testing.assert_array_equal(et16.cpu().numpy().astype(np.uint16).astype(np.int64), want_et)


def _tables(H, ns, ne, seed, scale=0.5):
    g = torch.Generator().manual_seed(seed)
    st = torch.randn(ns, H, generator=g) * scale; st[0] = 0
    et = torch.randn(ne, H, generator=g) * scale; et[0] = 0
    vd = torch.randn(1, H, generator=g) * scale
    return st, et, vd


def _oracle(q, k, v, ab, sp, et_ids, st, et, vd, dout, keep=None, p=0.0):
    """float64 outputs and gradients; the tables' padding row 0 gets no gradient (nn.Embedding(padding_idx=0))."""
    t = [x.double().requires_grad_(True) for x in (q, k, v)]
    tabs = [x.double().requires_grad_(True) for x in (st, et, vd)]
    ns, ne = st.shape[0], et.shape[0]
    bias = oda.graph_attn_bias(ab.double(), sp.clamp(0, ns - 1), et_ids.clamp(0, ne - 1), *tabs)
    o = oda.dense_attention(t[0], t[1], t[2], bias, drop_keep=keep, p_drop=p)
    grads = [g_.clone() for g_ in torch.autograd.grad(o, t + tabs, dout.reshape(o.shape).double())]
    grads[3][0] = 0
    grads[4][0] = 0
    return o, grads


# (graphs, s, heads, head dim, edge features, spatial rows, edge rows): the benchmark shape (128 + virtual node = 129:
# four full tiles and a one-row last tile), one tile, a ragged last tile, several features, the molecule tables, 16 heads
CASES = [(9, 128, 8, 8, 1, 22, 5), (5, 31, 8, 8, 1, 22, 5), (10, 49, 4, 16, 3, 40, 64), (3, 96, 8, 8, 2, 512, 1537),
         (17, 19, 16, 8, 1, 7, 3), (4, 66, 2, 32, 1, 22, 5),
         # S = 4 (no whole group of sixteen keys), S = 16 (exactly one), S = 33 (a one-row last tile behind one full tile)
         (3, 3, 2, 8, 1, 5, 4), (2, 15, 8, 8, 2, 22, 5), (3, 32, 8, 8, 1, 22, 5),
         # one edge id in all four features of every edge position: the edge accumulator collects F dS per position
         (4, 40, 8, 8, 4, 5, 2)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%d-s%d-H%d-d%d-F%d-ns%d-ne%d" % c)
def test_dense_from_ids_matches_oracle(cuda, dtype, case):
    b, s, H, d, F, ns, ne = case
    print(f"dense_from_ids case: {case} {dtype}", flush=True)
    S = s + 1
    _, sp, et_ids, ab = make_batch(b, s, F, ns, ne, seed=11 * s + H)
    st, et, vd = _tables(H, ns, ne, seed=s)
    g = torch.Generator().manual_seed(5)
    # scores (q sqrt(d)) . k of standard deviation 3 whatever the head dim, like a trained model's
    q, k, v, dout = (torch.randn(b, S, H, d, generator=g) * f for f in ((3 / d) ** 0.5, (3 / d) ** 0.5, 0.5, 0.5))
    if dtype == torch.bfloat16:
        q, k, v, dout, st, et, vd = (x.to(dtype) for x in (q, k, v, dout, st, et, vd))
    o_ref, g_ref = _oracle(q, k, v, ab, sp, et_ids, st, et, vd, dout)
    sp16, et16 = _ext.ops().dense_ids_pack(sp.to(cuda), et_ids.to(cuda), ns, ne)
    tc = [x.to(cuda).requires_grad_(True) for x in (q, k, v, st, et, vd)]
    o = _ext.ops().dense_attention_ids(tc[0], tc[1], tc[2], ab.to(cuda, dtype), sp16, et16, tc[3], tc[4], tc[5], 0.0, 0,
                                       dtype == torch.float32)
    assert o.shape == (b, S, H * d) and o.dtype == dtype
    assert err(o, o_ref) <= TOL, err(o, o_ref)
    g_got = torch.autograd.grad(o, tc, dout.reshape(b, S, -1).to(cuda))
    for nm, a, r in zip(("q", "k", "v", "spatial", "edge", "virtual"), g_got, g_ref):
        assert err(a, r) <= (TOL if len(nm) == 1 else TOL_TABLE), f"d{nm} err {err(a, r)}"
    assert not g_got[3][0].any() and not g_got[4][0].any()      # padding index rows
    # integer accumulators and fixed-order sums: a second run gives the same bits
    g_again = torch.autograd.grad(_ext.ops().dense_attention_ids(tc[0], tc[1], tc[2], ab.to(cuda, dtype), sp16, et16, tc[3], tc[4], tc[5],
                                                                 0.0, 0, dtype == torch.float32), tc, dout.reshape(b, S, -1).to(cuda))
    for a, r in zip(g_again, g_got):
        assert torch.equal(a, r)
    # the same numbers through the bias tensor (the library's other form): both round the bias to bf16 in bf16 runs
    if dtype == torch.bfloat16:
        bias = oda.graph_attn_bias(ab, sp.clamp(0, ns - 1), et_ids.clamp(0, ne - 1), st.float(), et.float(), vd.float()).to(dtype)
        o2 = dense_attention(tc[0].detach(), tc[1].detach(), tc[2].detach(), bias.to(cuda))
        assert err(o, o2) <= 1e-2, err(o, o2)
    # gradients of q, k, v alone (no table partials are written)
    tq = [x.detach().requires_grad_(True) for x in tc[:3]]
    o3 = _ext.ops().dense_attention_ids(tq[0], tq[1], tq[2], ab.to(cuda, dtype), sp16, et16, tc[3].detach(), tc[4].detach(),
                                        tc[5].detach(), 0.0, 0, dtype == torch.float32)
    g3 = torch.autograd.grad(o3, tq, dout.reshape(b, S, -1).to(cuda))
    for a, r in zip(g3, g_got[:3]):
        assert torch.equal(a, r)


def test_dense_from_ids_without_attn_bias_and_with_dropout(cuda):
    b, s, H, d, F, ns, ne = 6, 128, 8, 8, 1, 22, 5
    S = s + 1
    _, sp, et_ids, ab = make_batch(b, s, F, ns, ne, seed=3)
    st, et, vd = (x.to(torch.bfloat16) for x in _tables(H, ns, ne, seed=9))
    g = torch.Generator().manual_seed(8)
    q, k, v, dout = (torch.randn(b, S, H, d, generator=g).to(torch.bfloat16) for _ in range(4))
    sp16, et16 = _ext.ops().dense_ids_pack(sp.to(cuda), et_ids.to(cuda), ns, ne)
    for with_ab, p, seed in ((False, 0.0, 0), (True, 0.25, 1234), (False, 0.5, 77)):
        print(f"dense_from_ids case: attn_bias={with_ab} p={p}", flush=True)
        keep = dense_dropout_mask(b, S, H, p, seed, cuda).cpu().bool() if p > 0 else None
        o_ref, g_ref = _oracle(q, k, v, ab if with_ab else torch.zeros_like(ab), sp, et_ids, st, et, vd, dout, keep, p)
        tc = [x.to(cuda).requires_grad_(True) for x in (q, k, v, st, et, vd)]
        o = _ext.ops().dense_attention_ids(tc[0], tc[1], tc[2], ab.to(cuda, torch.bfloat16) if with_ab else None, sp16, et16,
                                           tc[3], tc[4], tc[5], p, seed, False)
        assert err(o, o_ref) <= TOL, err(o, o_ref)
        g_got = torch.autograd.grad(o, tc, dout.reshape(b, S, -1).to(cuda))
        for nm, a, r in zip(("q", "k", "v", "spatial", "edge", "virtual"), g_got, g_ref):
            assert err(a, r) <= (TOL if len(nm) == 1 else TOL_TABLE), f"d{nm} err {err(a, r)} (attn_bias={with_ab}, p={p})"


def test_module_passes_ids_and_falls_back(cuda):
    """GraphAttnBias(as_ids=True) -> dense_attention: bf16 runs form the bias on chip; float32 arithmetic and shapes
    whose bias does not fit the LDS build the tensor once and give the numbers of the tensor path."""
    data = workloads.erdos_renyi_batch(batch=8, seed=5)
    H, d, b, S = 8, 8, 8, data["S"]
    m = GraphAttnBias(H, 512, 5, 22, 128, 64, "single_hop", 5)
    g = torch.Generator().manual_seed(2)
    with torch.no_grad():
        m.spatial_pos_encoder.weight.normal_(0, 0.5, generator=g); m.spatial_pos_encoder.weight[0] = 0
        m.edge_encoder.weight.normal_(0, 0.5, generator=g); m.edge_encoder.weight[0] = 0
        m.graph_token_virtual_distance.weight.normal_(0, 0.5, generator=g)
    q, k, v, dout = (torch.randn(b, S, H, d, generator=g) for _ in range(4))
    for dtype in (torch.bfloat16, torch.float32):
        mc = m.to(cuda, dtype)
        batch = types.SimpleNamespace(attn_bias=torch.from_numpy(data["attn_bias"]).to(cuda, dtype),
                                      spatial_pos=torch.from_numpy(data["spatial_pos"]).long().to(cuda),
                                      attn_edge_type=torch.from_numpy(data["edge_type"]).long().unsqueeze(-1).to(cuda), edge_input=None)
        ids = mc(batch, as_ids=True)
        assert isinstance(ids, GraphBiasIds)
        tc = [x.to(cuda, dtype).requires_grad_(True) for x in (q, k, v)]
        o = dense_attention(tc[0], tc[1], tc[2], ids)
        params = [mc.spatial_pos_encoder.weight, mc.edge_encoder.weight, mc.graph_token_virtual_distance.weight]
        got = torch.autograd.grad(o, tc + params, dout.reshape(b, S, -1).to(cuda, dtype))
        assert (ids._tensor is None) == (dtype == torch.bfloat16)          # float32 arithmetic built the tensor
        bias = mc(batch)                                                   # the tensor path
        tc2 = [x.detach().requires_grad_(True) for x in tc]
        o2 = dense_attention(tc2[0], tc2[1], tc2[2], bias)
        want = torch.autograd.grad(o2, tc2 + params, dout.reshape(b, S, -1).to(cuda, dtype))
        tol = 2e-2 if dtype == torch.bfloat16 else 0.0
        assert err(o, o2) <= tol
        for a, r in zip(got, want):
            # float32: the same kernels ran twice; the table sums are formed with atomics and agree to rounding
            assert err(a, r) <= (3e-2 if dtype == torch.bfloat16 else 1e-6), err(a, r)
    # a bias that does not fit next to the tables: S = 250 with 30 000 table rows
    b, s = 2, 249
    _, sp, et_ids, ab = make_batch(b, s, 1, 20000, 10000, seed=1)
    st, et, vd = (x.to(cuda, torch.bfloat16) for x in _tables(H, 20000, 10000, seed=4))
    sp16, et16 = _ext.ops().dense_ids_pack(sp.to(cuda), et_ids.to(cuda), 20000, 10000)
    q = torch.randn(b, s + 1, H, d, generator=g).to(cuda, torch.bfloat16)
    with pytest.raises(RuntimeError, match="bytes of LDS"):
        _ext.ops().dense_attention_ids(q, q, q, None, sp16, et16, st, et, vd, 0.0, 0, False)
    built = []
    ids = GraphBiasIds(None, sp16, et16, st, et, vd, lambda: built.append(1) or torch.zeros(b, H, s + 1, s + 1, device=cuda))
    o = dense_attention(q, q, q, ids)
    assert built == [1] and not ids.fits and torch.isfinite(o).all()
    # float32 tensors without the bf16-products flag are refused by the operator itself
    with pytest.raises(RuntimeError, match="bf16"):
        _ext.ops().dense_attention_ids(q.float(), q.float(), q.float(), None, sp16, et16, st.float(), et.float(), vd.float(), 0.0, 0, False)


def test_a_shape_the_forward_accepts_can_be_trained(cuda):
    """The id form keeps the bias of a (graph, head) pair and the table columns in LDS and its backward needs more of it
    than its forward: the forward applies the backward's limit, so that a training step never passes the forward and
    dies inside autograd.  Swept over the sizes around the limit with the molecule tables (512 + 1537 rows)."""
    H, d, b, ns, ne = 8, 8, 2, 512, 1537
    g = torch.Generator().manual_seed(4)
    st, et, vd = (x.to(cuda, torch.bfloat16) for x in _tables(H, ns, ne, seed=2))
    accepted = refused = 0
    for s in (128, 160, 192, 208, 224, 232, 240, 248, 255):
        print(f"id-form limit case: S={s + 1}", flush=True)
        _, sp, et_ids, _ = make_batch(b, s, 1, ns, ne, seed=s)
        sp16, et16 = _ext.ops().dense_ids_pack(sp.to(cuda), et_ids.to(cuda), ns, ne)
        q, k, v = (torch.randn(b, s + 1, H, d, generator=g).to(cuda, torch.bfloat16).requires_grad_(True) for _ in range(3))
        tabs = [t.clone().requires_grad_(True) for t in (st, et, vd)]
        try:
            o = _ext.ops().dense_attention_ids(q, k, v, None, sp16, et16, tabs[0], tabs[1], tabs[2], 0.0, 0, False)
        except RuntimeError as exc:
            assert "bytes of LDS" in str(exc)
            refused += 1
            continue
        accepted += 1
        grads = torch.autograd.grad(o, [q, k, v] + tabs, torch.ones_like(o))          # must not raise
        assert all(torch.isfinite(x).all() for x in grads)
    assert accepted >= 1 and refused >= 1, (accepted, refused)       # the sweep straddles the limit
