"""GPU: tgt_sparse_attn_fwd_noalloc (the forward that allocates nothing: the partial sums and arrival
counters of split rows live in a fixed array inside the library) gives the bits of tgt_sparse_attn_fwd,
through the C ABI, on two calls in a row, the second on a smaller graph; and also agrees with the oracle."""
import numpy as np
import pytest
import torch

from oracle import sparse_attention as osa
from torchgt_amd import GraphPlan, _lib, workloads

pytestmark = pytest.mark.gpu


def _graph(n_real, extra_hub_edges, seed):
    """Power-law-free test graph with a global node (a split row with many segments), one more hub row and
    self-loops; node 0 is the global node."""
    rng = np.random.default_rng(seed)
    und = rng.integers(0, n_real, (2, 3 * n_real))
    hub = np.stack([rng.integers(0, n_real, extra_hub_edges), np.full(extra_hub_edges, 7)])
    loops = np.stack([np.arange(n_real), np.arange(n_real)])
    e = np.concatenate([und, und[::-1], hub, loops], axis=1)
    return workloads.add_global_node(e, n_real), n_real + 1


def _fwd_both(e, n, H, d, dtype, seed, cuda):
    print(f"no-alloc case N={n} E={e.shape[1]} H={H} d={d} {dtype} seed={seed}", flush=True)
    L = _lib.lib()
    ei = torch.from_numpy(e).to(cuda)
    plan = GraphPlan(ei, n)
    info = plan.info()
    assert info["split_rows_dst"] >= 1, "the test graph must have split rows, or no scratch is used"
    _lib.check(L.tgt_plan_prepare(plan.handle, H, d, None))
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(n, H, d, generator=g).to(cuda, dtype) for _ in range(3))
    bias = (torch.randn(e.shape[1], H, generator=g) * 0.5).to(cuda, dtype)
    code = _lib.DTYPE_BF16 if dtype == torch.bfloat16 else _lib.DTYPE_F32
    stream = torch.cuda.current_stream(cuda).cuda_stream
    P = lambda t: t.data_ptr()
    ws = plan.workspace(H, d)
    out_a, out_b = torch.empty_like(q), torch.full_like(q, float("nan"))
    Z_a, Z_b = torch.empty(n, H, device=cuda), torch.full((n, H), float("nan"), device=cuda)
    _lib.check(L.tgt_sparse_attn_fwd(plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d, code, P(out_a),
                                     P(Z_a), P(ws), ws.numel(), stream))
    # with kernel timing switched on (the workspace forward then takes events from a pool that grows on demand):
    # the call neither creates events nor moves the device's free memory
    torch.cuda.synchronize()
    L.tgt_timing_enable(1)
    free_before = torch.cuda.mem_get_info(cuda)[0]
    _lib.check(L.tgt_sparse_attn_fwd_noalloc(plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d, code,
                                             P(out_b), P(Z_b), stream))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(cuda)[0] == free_before
    L.tgt_timing_enable(0)
    assert torch.equal(out_a, out_b) and torch.equal(Z_a, Z_b)
    ref, _ = osa.sparse_attention(q.double().cpu(), k.double().cpu(), v.double().cpu(), ei.cpu(), bias.double().cpu())
    rel = (out_b.double().cpu() - ref).abs().max().item() / ref.abs().max().item()
    assert rel <= (2e-2 if dtype == torch.bfloat16 else 1e-5), rel
    plan.close()
    return rel


def test_no_alloc_forward_matches_workspace_forward_twice(cuda):
    # two calls in a row on one GPU, the second on a smaller graph: the array keeps the first call's contents
    big, n_big = _graph(9000, 3000, seed=1)       # global row: 71 segments, combined in two levels
    small, n_small = _graph(1500, 700, seed=2)
    _fwd_both(big, n_big, 8, 8, torch.float32, 11, cuda)
    _fwd_both(small, n_small, 8, 8, torch.float32, 12, cuda)
    _fwd_both(small, n_small, 4, 16, torch.bfloat16, 13, cuda)


def test_no_alloc_forward_refuses_what_it_cannot_hold(cuda):
    L = _lib.lib()
    e, n = _graph(1500, 700, seed=3)
    ei = torch.from_numpy(e).to(cuda)
    plan = GraphPlan(ei, n)
    q = torch.randn(n, 2, 16, device=cuda)
    out, Z = torch.empty_like(q), torch.empty(n, 2, device=cuda)
    P = lambda t: t.data_ptr()
    # H * d = 32 was neither prepared nor used: making its launch descriptors would allocate
    rc = L.tgt_sparse_attn_fwd_noalloc(plan.handle, P(q), P(q), P(q), None, _lib.BIAS_NONE, 2, 16, _lib.DTYPE_F32,
                                       P(out), P(Z), None)
    assert rc == _lib.ERR_INVALID_ARG and b"tgt_plan_prepare" in L.tgt_last_error()
    plan.close()
    # a graph whose split rows need more than the fixed array: 7500 rows of two segments each
    rng = np.random.default_rng(4)
    hubs = 7500
    src = rng.integers(0, 20000, hubs * 1100)
    dst = np.repeat(np.arange(hubs), 1100)
    ei = torch.from_numpy(np.stack([src, dst])).to(cuda)
    plan = GraphPlan(ei, 20000)
    q = torch.randn(20000, 8, 8, device=cuda)
    out, Z = torch.empty_like(q), torch.empty(20000, 8, device=cuda)
    rc = L.tgt_sparse_attn_fwd_noalloc(plan.handle, P(q), P(q), P(q), None, _lib.BIAS_NONE, 8, 8, _lib.DTYPE_F32,
                                       P(out), P(Z), None)
    assert rc == _lib.ERR_WORKSPACE and b"scratch" in L.tgt_last_error()
    plan.close()
