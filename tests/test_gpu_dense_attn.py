"""GPU parity of the dense biased attention (bf16 MFMA, fp32 softmax) with the oracle.

Error measure: max|a - b| / max|b| against the oracle in float64 on the same
bf16-rounded inputs; bar 2e-2 (bf16 matrix instructions with fp32 accumulation),
outputs and gradients.  float32 tensors go through the same bf16 instructions, so
their inputs are rounded to bf16 first and the same bar applies.
"""
import numpy as np
import pytest
import torch

from oracle import dense_attention as oda
from torchgt_amd import CoreAttention, _lib, dense_attention, workloads

pytestmark = pytest.mark.gpu
TOL = 2e-2


def err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    fin = torch.isfinite(b)
    assert torch.equal(torch.isfinite(a), fin)
    denom = b[fin].abs().max().item()
    return (a[fin] - b[fin]).abs().max().item() / (denom if denom > 0 else 1.0)


def run_case(name, b, S, H, d, dtype, with_bias, n_real, seed, cuda, bias_grad=True):
    print(f"dense case {name}: b={b} S={S} H={H} d={d} {dtype} bias={with_bias} seed={seed}", flush=True)
    g = torch.Generator().manual_seed(seed)
    q, k, v, dout = (torch.randn(b, S, H, d, generator=g).to(torch.bfloat16).to(dtype) for _ in range(4))
    dout = dout.reshape(b, S, H * d)
    bias = None
    if with_bias:
        bias = (torch.randn(b, H, S, S, generator=g) * 0.5).to(torch.bfloat16).to(dtype)
        if n_real is not None:
            for gi in range(b):
                bias[gi, :, :, n_real[gi]:] = float("-inf")       # padded keys (data/collator.py:50-57)
    # oracle in float64
    t = [x.double().requires_grad_(True) for x in (q, k, v)]
    bb = bias.double().requires_grad_(True) if with_bias else None
    o_ref = oda.dense_attention(t[0], t[1], t[2], bb)
    g_ref = torch.autograd.grad(o_ref, t + ([bb] if with_bias and bias_grad else []), dout.double())
    # library
    tc = [x.to(cuda).requires_grad_(True) for x in (q, k, v)]
    bc = bias.to(cuda).requires_grad_(bias_grad) if with_bias else None
    o = dense_attention(tc[0], tc[1], tc[2], bc)
    g_got = torch.autograd.grad(o, tc + ([bc] if with_bias and bias_grad else []), dout.to(cuda))
    assert o.shape == (b, S, H * d) and o.dtype == dtype
    assert err(o, o_ref) <= TOL, f"out err {err(o, o_ref)}"
    for nm, a, r in zip(("dq", "dk", "dv", "dbias"), g_got, g_ref):
        assert not torch.isnan(a).any(), nm
        assert err(a, r) <= TOL, f"{nm} err {err(a, r)}"


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
    with pytest.raises(_lib.TorchGTHipError) as exc:
        dense_attention(q, q, q)
    assert exc.value.code == _lib.ERR_UNSUPPORTED          # S > 256
    q = torch.randn(2, 10, 2, 12, device=cuda, dtype=torch.bfloat16)
    with pytest.raises(_lib.TorchGTHipError):
        dense_attention(q, q, q)                            # head dim 12
    mod = CoreAttention(64, 0.1, 8)
    mod.train()
    q = torch.randn(2, 10, 8, 8, device=cuda)
    with pytest.raises(NotImplementedError):
        mod(q, q, q)                                        # dropout inside the dense kernel
    with pytest.raises(RuntimeError):
        dense_attention(q.cpu(), q.cpu(), q.cpu())
