"""GPU parity of the dense biased attention with the oracle.

Error measure: max|a - b| / max|b| against the oracle in float64 on the same inputs, outputs and
gradients.  bfloat16 tensors (bf16 matrix instructions, fp32 accumulation and softmax): bar 2e-2.
float32 tensors run in float32 arithmetic: bar 1e-5 on inputs that are NOT rounded to bf16.  float32
tensors with ``bf16_products=True`` (the matrix cores, by request): 2e-2 on bf16-rounded inputs, and the
error on unrounded inputs is measured and printed.
"""
import numpy as np
import pytest
import torch

from oracle import dense_attention as oda
from torchgt_amd import CoreAttention, _lib, dense_attention, workloads
from torchgt_amd.core_attention import dense_dropout_mask

pytestmark = pytest.mark.gpu
TOL = 2e-2
TOL_F32 = 1e-5


def err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    fin = torch.isfinite(b)
    assert torch.equal(torch.isfinite(a), fin)
    denom = b[fin].abs().max().item()
    return (a[fin] - b[fin]).abs().max().item() / (denom if denom > 0 else 1.0)


def run_case(name, b, S, H, d, dtype, with_bias, n_real, seed, cuda, bias_grad=True, bf16_products=False, p_drop=0.0,
             round_inputs=None, tol=None):
    """float32 without bf16_products: unrounded inputs, 1e-5.  Everything else: bf16-rounded inputs, 2e-2."""
    exact = dtype == torch.float32 and not bf16_products
    if round_inputs is None:
        round_inputs = not exact
    if tol is None:
        tol = TOL_F32 if exact else TOL
    print(f"dense case {name}: b={b} S={S} H={H} d={d} {dtype} bias={with_bias} seed={seed} bf16_products={bf16_products} "
          f"p_drop={p_drop} rounded={round_inputs}", flush=True)
    g = torch.Generator().manual_seed(seed)
    rnd = (lambda t: t.to(torch.bfloat16).to(dtype)) if round_inputs else (lambda t: t.to(dtype))
    q, k, v, dout = (rnd(torch.randn(b, S, H, d, generator=g)) for _ in range(4))
    dout = dout.reshape(b, S, H * d)
    bias = None
    if with_bias:
        bias = rnd(torch.randn(b, H, S, S, generator=g) * 0.5)
        if n_real is not None:
            for gi in range(b):
                bias[gi, :, :, n_real[gi]:] = float("-inf")       # padded keys (data/collator.py:50-57)
    # oracle in float64
    t = [x.double().requires_grad_(True) for x in (q, k, v)]
    bb = bias.double().requires_grad_(True) if with_bias else None
    keep = None
    drop_seed = 1000 + seed
    if p_drop > 0:      # the mask the kernels will use, handed to the oracle: softmax -> mask / (1 - p) -> . v
        keep = dense_dropout_mask(b, S, H, p_drop, drop_seed, cuda).cpu()
    o_ref = oda.dense_attention(t[0], t[1], t[2], bb, drop_keep=keep, p_drop=p_drop)
    g_ref = torch.autograd.grad(o_ref, t + ([bb] if with_bias and bias_grad else []), dout.double())
    # library
    tc = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    bc = bias.to(cuda).requires_grad_(bias_grad) if with_bias else None
    o = dense_attention(tc[0], tc[1], tc[2], bc, p_drop=p_drop, seed=drop_seed, bf16_products=bf16_products)
    g_got = torch.autograd.grad(o, tc + ([bc] if with_bias and bias_grad else []), dout.to(cuda))
    assert o.shape == (b, S, H * d) and o.dtype == dtype
    errs = {"out": err(o, o_ref)}
    for nm, a, r in zip(("dq", "dk", "dv", "dbias"), g_got, g_ref):
        assert not torch.isnan(a).any(), nm
        errs[nm] = err(a, r)
    print("   errors", {kk: f"{vv:.2e}" for kk, vv in errs.items()}, flush=True)
    bad = {kk: vv for kk, vv in errs.items() if vv > tol}
    assert not bad, f"{name}: {bad} above {tol}"
    return errs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_small_shapes(cuda, dtype):
    run_case("s7", 2, 7, 3, 8, dtype, True, None, 1, cuda)
    run_case("s32", 3, 32, 8, 8, dtype, True, None, 2, cuda)
    run_case("s33-nobias", 2, 33, 4, 8, dtype, False, None, 3, cuda)
    run_case("s129", 4, 129, 8, 8, dtype, True, [129, 17, 64, 100], 4, cuda)


# 1, 4, 34, 65, 100, 131, 161: a last tile of one to four rows (a virtual node behind a multiple of 32), which the
# kernels treat apart from full tiles; 36 and 69: one row more than that.  (Sequences of two or three rows are left
# out: with a graph of one real key every dS cancels to zero, and the rounding of the stored bf16 output alone --
# the same arithmetic in float64 with the kernel's rounding points -- puts dk 3 % off in this error measure.)
@pytest.mark.parametrize("S", [1, 4, 31, 34, 36, 64, 65, 69, 96, 100, 131, 160, 161, 200, 256])
def test_every_tile_count(cuda, S):
    run_case(f"S{S}", 2, S, 2, 8, torch.bfloat16, True, [S, max(1, S // 2)], 10 + S, cuda)


def test_float32_is_float32_accurate_and_bf16_products_are_opt_in(cuda):
    # float32 callers get float32 arithmetic (1e-5 on unrounded inputs: checked by run_case's default bars)
    run_case("f32-exact", 3, 129, 8, 8, torch.float32, True, [129, 40, 77], 50, cuda)
    run_case("f32-exact-d16", 2, 70, 4, 16, torch.float32, True, [70, 33], 51, cuda)
    run_case("f32-exact-long", 1, 300, 2, 8, torch.float32, True, None, 52, cuda)          # beyond the matrix path's 256
    # the matrix cores for float32 tensors, by request: 2e-2 on bf16-rounded inputs
    run_case("f32-bf16mm", 3, 129, 8, 8, torch.float32, True, [129, 40, 77], 53, cuda, bf16_products=True)
    # ... and what that costs on inputs that are not rounded first (the reference multiplies q by sqrt(d), so
    # the logits are large and 2^-8 on them moves the probabilities): measured, bar 1.5e-1
    e = run_case("f32-bf16mm-unrounded", 3, 129, 8, 8, torch.float32, True, [129, 40, 77], 53, cuda, bf16_products=True,
                 round_inputs=False, tol=1.5e-1)
    print("bf16 products on unrounded float32 inputs: errors", e, flush=True)


@pytest.mark.parametrize("dtype,p", [(torch.bfloat16, 0.1), (torch.float32, 0.5), (torch.bfloat16, 0.5)])
def test_attention_dropout_matches_oracle_with_the_exported_mask(cuda, dtype, p):
    # every tile shape of the matrix kernels (full tiles, a row that ends inside a tile, a last tile of one row)
    run_case("drop-s129", 3, 129, 8, 8, dtype, True, [129, 40, 77], 60, cuda, p_drop=p)
    run_case("drop-s70", 2, 70, 4, 8, dtype, True, [70, 33], 61, cuda, p_drop=p)
    run_case("drop-s32-nobias", 2, 32, 2, 16, dtype, False, None, 62, cuda, p_drop=p)
    if dtype == torch.float32:
        run_case("drop-f32-bf16mm", 2, 100, 4, 8, dtype, True, None, 63, cuda, p_drop=p, bf16_products=True)

# Keep mask of seed 2024, p = 0.5 for b = 2, H = 2, S = 4, listed by hand: [graph][head][query][key].  It comes from
# the documented generator evaluated with pencil-and-paper integer arithmetic (32-bit multiply / xor-shift rounds on
# (seed, graph * H + head, query, key)), not from the library.
HAND_MASK = [[[[1, 1, 1, 1], [1, 1, 1, 1], [0, 0, 0, 1], [0, 0, 1, 1]],
              [[1, 1, 1, 1], [1, 1, 0, 0], [1, 0, 0, 0], [0, 1, 0, 0]]],
             [[[1, 0, 0, 1], [1, 0, 1, 0], [1, 1, 0, 1], [1, 0, 1, 0]],
              [[0, 1, 0, 1], [0, 1, 1, 1], [1, 0, 0, 0], [1, 0, 0, 0]]]]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dropout_mask_indexing_read_off_the_kernels(cuda, dtype):
    """Which (graph, head, query, key) the kernels drop, read off their outputs and compared with the hand-listed
    mask - the exported mask plays no part.  With q = k = 0 and no bias every probability is 1/4; values that are
    unit vectors (v[key] = e_key) make out[g, q, h, c] = keep[g, h, q, c] / (4 (1 - p)), and an upstream gradient
    of unit vectors (dout[q] = e_q) makes dv[g, k, h, c] = keep[g, h, c, k] / (4 (1 - p)): the forward's mask and
    the backward's, position by position."""
    b, S, H, d, p = 2, 4, 2, 8, 0.5
    want = torch.tensor(HAND_MASK, dtype=torch.bool)                     # [b, H, q, k]
    q = torch.zeros(b, S, H, d, dtype=dtype, device=cuda)
    v = torch.zeros(b, S, H, d, dtype=dtype)
    for key in range(S):
        v[:, key, :, key] = 1.0
    v = v.to(cuda).requires_grad_(True)
    out = dense_attention(q, q.clone(), v, None, p_drop=p, seed=2024)
    o = out.view(b, S, H, d).float().cpu()                               # [g, q, h, c]
    assert torch.equal(o[..., S:], torch.zeros(b, S, H, d - S))
    shown = o[..., :S].permute(0, 2, 1, 3)                               # [g, h, q, key]
    assert torch.equal(shown, want.float() * 0.5), shown                 # 1/4 * 1/(1 - p), exact in bf16 as well
    dout = torch.zeros(b, S, H, d, dtype=dtype)
    for qq in range(S):
        dout[:, qq, :, qq] = 1.0
    dv, = torch.autograd.grad(out, v, dout.reshape(b, S, H * d).to(cuda))
    shown_b = dv.float().cpu()[..., :S].permute(0, 2, 3, 1)              # dv[g, k, h, c=q] -> [g, h, q, k]
    assert torch.equal(shown_b, want.float() * 0.5), shown_b
    # and the exported mask is the same one
    assert torch.equal(dense_dropout_mask(b, S, H, p, 2024, cuda).cpu().bool(), want)


def test_dropout_mask_statistics_and_module(cuda):
    b, S, H = 4, 129, 8
    for p in (0.1, 0.5):
        keep = dense_dropout_mask(b, S, H, p, 12345, cuda).float()
        n = keep.numel()
        sigma = (p * (1 - p) / n) ** 0.5
        assert abs(keep.mean().item() - (1 - p)) <= 3 * sigma, (p, keep.mean().item())
        # rows and heads are not copies of each other, and another seed gives another mask
        assert not torch.equal(keep[0, 0], keep[0, 1]) and not torch.equal(keep[0, 0, 0], keep[0, 0, 1])
        assert not torch.equal(keep, dense_dropout_mask(b, S, H, p, 12346, cuda).float())
        # per-row keep rates are binomial too (no stripes): the spread of row means is what independence gives
        row_sigma = (p * (1 - p) / S) ** 0.5
        assert abs(keep.mean(-1).std().item() - row_sigma) <= 0.2 * row_sigma
    # the module applies dropout in training mode with the reference's constructor arguments, not in eval mode
    mod = CoreAttention(64, 0.5, 8).to(cuda)
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(2, 40, 8, 8, generator=g).to(cuda) for _ in range(3))
    mod.eval()
    base = mod(q, k, v)
    assert torch.equal(base, mod(q, k, v))
    mod.train()
    torch.manual_seed(5)
    a = mod(q, k, v)
    torch.manual_seed(5)
    a2 = mod(q, k, v)
    c = mod(q, k, v)
    assert torch.equal(a, a2) and not torch.equal(a, c) and not torch.equal(a, base)
    # expectation over masks is the undropped output
    acc = torch.zeros_like(base)
    for i in range(200):
        acc += dense_attention(q, k, v, None, p_drop=0.5, seed=i)
    assert (acc / 200 - base).abs().max().item() <= 0.25 * base.abs().max().item()


@pytest.mark.parametrize("d", [16, 32])
def test_other_head_dims(cuda, d):
    run_case(f"d{d}", 2, 70, 4, d, torch.bfloat16, True, [70, 33], 20 + d, cuda)
    run_case(f"d{d}-f32", 1, 129, 2, d, torch.float32, True, None, 30 + d, cuda, bias_grad=False)
    run_case(f"d{d}-s67", 2, 67, 2, d, torch.bfloat16, True, [67, 40], 40 + d, cuda)        # three rows in the last tile


def test_config4_batch_with_bias_from_tables(cuda):
    # benchmark config 4 (reduced batch for the fp64 oracle): ER graphs padded to 128 + virtual node,
    # bias built by the reference's GraphAttnBias recipe from SPD / edge-type ids and N(0, 0.02) tables
    data = workloads.erdos_renyi_batch(batch=16, seed=42)
    S, H, d, b = data["S"], 8, 8, 16
    g = torch.Generator().manual_seed(42)
    st = torch.randn(22, H, generator=g) * 0.02; st[0] = 0
    et = torch.randn(5, H, generator=g) * 0.02; et[0] = 0
    vd = torch.randn(1, H, generator=g) * 0.02
    bias = oda.graph_attn_bias(torch.from_numpy(data["attn_bias"]), torch.from_numpy(data["spatial_pos"]).long(),
                               torch.from_numpy(data["edge_type"]).long().unsqueeze(-1), st, et, vd)
    bias = bias.to(torch.bfloat16)
    q, k, v, dout = (torch.randn(b, S, H, d, generator=g).to(torch.bfloat16) for _ in range(4))
    t = [x.double().requires_grad_(True) for x in (q, k, v)]
    bb = bias.double().requires_grad_(True)
    o_ref = oda.dense_attention(t[0], t[1], t[2], bb)
    g_ref = torch.autograd.grad(o_ref, t + [bb], dout.reshape(b, S, -1).double())
    mod = CoreAttention(H * d, 0.0, H).to(cuda)
    tc = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    bc = bias.to(cuda).requires_grad_(True)
    o = mod(tc[0], tc[1], tc[2], bc)                         # graph-level call convention
    g_got = torch.autograd.grad(o, tc + [bc], dout.reshape(b, S, -1).to(cuda))
    assert err(o, o_ref) <= TOL
    for a, r in zip(g_got, g_ref):
        assert err(a, r) <= TOL
    # padded keys get exactly zero probability: dbias there is exactly 0
    n0 = int(data["n_nodes"][0])
    assert torch.count_nonzero(g_got[3][0, :, :, n0 + 1:]) == 0
    # attn_type='full' spelling and full_attention() give the same tensor
    o2 = mod(tc[0], tc[1], tc[2], bc, None, "full")
    assert torch.equal(o2, o)


def test_rows_sum_to_one_property_full_size(cuda):
    # size-independent property at the full config-4 batch: with v = 1 the output is exactly the row sum
    # of the probabilities = 1, for every graph, head and query (padding included)
    data = workloads.erdos_renyi_batch(batch=256, seed=42)
    S, H, d, b = data["S"], 8, 8, 256
    g = torch.Generator().manual_seed(7)
    q, k = (torch.randn(b, S, H, d, generator=g).to(torch.bfloat16).to(cuda) for _ in range(2))
    v = torch.ones(b, S, H, d, dtype=torch.bfloat16, device=cuda)
    bias = torch.from_numpy(data["attn_bias"]).to(torch.bfloat16).unsqueeze(1).expand(b, H, S, S).contiguous().to(cuda)
    o = dense_attention(q, k, v, bias)
    assert torch.isfinite(o).all()
    assert (o.float() - 1.0).abs().max().item() <= 1e-2
    # linearity in v
    v2 = torch.randn(b, S, H, d, generator=g).to(torch.bfloat16).to(cuda)
    o_a = dense_attention(q, k, v2, bias).float()
    o_b = dense_attention(q, k, (2 * v2), bias).float()
    assert (o_b - 2 * o_a).abs().max().item() <= 2e-2 * o_a.abs().max().item()


def test_dense_loud_failures(cuda):
    q = torch.randn(2, 300, 2, 8, device=cuda, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="exceeds 256"):
        dense_attention(q, q, q)                            # S > 256 on the matrix path
    q = torch.randn(2, 10, 2, 12, device=cuda, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="head dim"):
        dense_attention(q, q, q)                            # head dim 12
    q = torch.randn(2, 10, 8, 8, device=cuda)
    with pytest.raises(RuntimeError, match="dropout rate"):
        dense_attention(q, q, q, p_drop=1.0, seed=1)        # rate outside [0, 1)
    with pytest.raises(RuntimeError):
        dense_attention(q.cpu(), q.cpu(), q.cpu())


def test_node_level_bias_layout_is_reinterpreted_like_the_reference(cuda):
    """models/graphormer_dist_node_level.py:157-161: the node-level 'full' path receives [b, S, S, H] and views that
    memory as [b, H, S, S] (no permute).  The module does the same."""
    b, S, H, d = 1, 40, 4, 8
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(b, S, H, d, generator=g).to(torch.bfloat16).to(cuda) for _ in range(3))
    bias = torch.randn(b, S, S, H, generator=g).to(torch.bfloat16).to(cuda)
    mod = CoreAttention(H * d, 0.0, H, 1).to(cuda)
    got = mod(q, k, v, bias, None, "full")
    want = dense_attention(q, k, v, bias.contiguous().view(b, H, S, S))
    assert torch.equal(got, want)
    o_ref = oda.dense_attention(q.double().cpu(), k.double().cpu(), v.double().cpu(), bias.double().cpu().contiguous().view(b, H, S, S))
    assert err(got, o_ref) <= TOL
