"""The C-ABI calls launch kernels only (no allocation, no synchronisation, no memset), so a
forward + backward step can be captured into a HIP graph and replayed.  Every replay is checked
against the eager result, with the program's own eager work and synchronisations in between."""
import pytest
import torch

import numpy as np

from torchgt_amd import GraphPlan, TileSet, _lib, workloads

pytestmark = pytest.mark.gpu


def _buffers(n, E, H, d, dtype, dev, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v, dout = (torch.randn(n, H, d, generator=g).to(dev, dtype) for _ in range(4))
    bias = (torch.randn(E, H, generator=g) * 0.1).to(dev, dtype)
    return q, k, v, dout, bias


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sparse_step_replays_from_a_graph(cuda, dtype):
    e, n = workloads.barabasi_albert()          # config 1: launch-bound size, has split rows (the global node)
    ei = torch.from_numpy(e).to(cuda)
    E, H, d = e.shape[1], 8, 8
    plan = GraphPlan(ei, n)
    ws = plan.workspace(H, d)
    L = _lib.lib()
    code = _lib.DTYPE_F32 if dtype == torch.float32 else _lib.DTYPE_BF16
    q, k, v, dout, bias = _buffers(n, E, H, d, dtype, cuda, 0)
    out = torch.empty_like(q)
    Z = torch.empty(n, H, device=cuda)
    dq, dk, dv, db = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q), torch.empty_like(bias)
    P = lambda t: t.data_ptr()

    def step(stream):
        _lib.check(L.tgt_sparse_attn_fwd(plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d, code,
                                         P(out), P(Z), P(ws), ws.numel(), stream))
        _lib.check(L.tgt_sparse_attn_bwd(plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d, code,
                                         P(out), P(Z), P(dout), P(dq), P(dk), P(dv), P(db), P(ws), ws.numel(), stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(side.cuda_stream)                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(torch.cuda.current_stream().cuda_stream)
    for replay in range(4):
        nq, nk, nv, ndout, nbias = _buffers(n, E, H, d, dtype, cuda, 10 + replay)
        for dst_t, src_t in ((q, nq), (k, nk), (v, nv), (dout, ndout), (bias, nbias)):
            dst_t.copy_(src_t)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (out, Z, dq, dk, dv, db)]
        step(torch.cuda.current_stream().cuda_stream)      # eager, same buffers
        torch.cuda.synchronize()
        for a, b in zip(got, (out, Z, dq, dk, dv, db)):
            assert torch.equal(a, b), f"replay {replay} differs from the eager step"
    plan.close()


def test_block_step_replays_from_a_graph(cuda):
    """The block path (tile kernels, the per-node side, the sparse kernels on the remaining edges with their plan
    of rows that have edges) is kernel launches only as well: captured once, replayed on fresh inputs."""
    rng = np.random.default_rng(3)
    n, H, d = 2048, 8, 8
    nb = n // 16
    tiles = np.stack([rng.integers(0, nb, 300) * 16, rng.integers(0, nb, 300) * 16], 1).astype(np.int32)
    rest = torch.from_numpy(rng.integers(0, n, (2, 1500))).to(cuda)
    E = rest.shape[1]
    ts = TileSet(tiles, n, cuda)
    plan = GraphPlan(rest, n, rows_with_edges_only=True)
    ws = ts.workspace(plan, H, d)
    L = _lib.lib()
    dtype, code = torch.bfloat16, _lib.DTYPE_BF16
    q, k, v, dout, bias = _buffers(n, E, H, d, dtype, cuda, 0)
    out = torch.empty_like(q)
    Z = torch.empty(n, H, device=cuda)
    dq, dk, dv, db = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q), torch.empty_like(bias)
    P = lambda t: t.data_ptr()

    def step(stream):
        _lib.check(L.tgt_block_attn_fwd(ts.handle, plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d, code,
                                        P(out), P(Z), P(ws), ws.numel(), stream))
        _lib.check(L.tgt_block_attn_bwd(ts.handle, plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d, code,
                                        P(out), P(Z), P(dout), P(dq), P(dk), P(dv), P(db), P(ws), ws.numel(), stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(side.cuda_stream)                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        nq, nk, nv, ndout, nbias = _buffers(n, E, H, d, dtype, cuda, 20 + replay)
        for dst_t, src_t in ((q, nq), (k, nk), (v, nv), (dout, ndout), (bias, nbias)):
            dst_t.copy_(src_t)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (out, Z, dq, dk, dv, db)]
        step(torch.cuda.current_stream().cuda_stream)      # eager, same buffers
        torch.cuda.synchronize()
        for a, b in zip(got, (out, Z, dq, dk, dv, db)):
            assert torch.equal(a, b), f"replay {replay} differs from the eager step"
    plan.close()
    ts.close()


def test_model_training_step_replays_from_a_graph(cuda):
    """A whole training step of the Graphormer mirror (forward, nll loss, backward, AdamW) captured once and
    replayed on fresh inputs: every replay gives the loss of the eager step bit for bit, with eager work and
    synchronisations between the replays, and the weights end up identical."""
    from torchgt_amd import Graphormer
    e, n = workloads.power_law_graph(n=3000, directed_edges=30000)
    ei = torch.from_numpy(e).to(cuda)
    g = torch.Generator().manual_seed(0)
    xs = [torch.randn(n - 1, 32, generator=g).to(cuda) for _ in range(4)]
    y = torch.randint(0, 10, (n - 1,), generator=g).to(cuda)

    def make():
        torch.manual_seed(7)
        m = Graphormer(2, 8, 32, 64, 10, 1, 0.0, 0.0, 0.0, 64, 1).to(cuda)
        return m, torch.optim.AdamW(m.parameters(), lr=1e-2, capturable=True)

    def step(m, opt, x):
        opt.zero_grad(set_to_none=True)
        loss = torch.nn.functional.nll_loss(m(x, None, ei, attn_type="sparse"), y)
        loss.backward()
        opt.step()
        return loss

    m, opt = make()
    for _ in range(3):
        step(m, opt, xs[0])
    eager = [step(m, opt, xs[i]).item() for i in range(1, 4)]
    w_eager = [p.detach().clone() for p in m.parameters()]

    m, opt = make()
    static_x = xs[0].clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(m, opt, static_x)
    torch.cuda.current_stream().wait_stream(side)
    gr = torch.cuda.CUDAGraph()
    opt.zero_grad(set_to_none=True)
    with torch.cuda.graph(gr):
        static_loss = torch.nn.functional.nll_loss(m(static_x, None, ei, attn_type="sparse"), y)
        static_loss.backward()
        opt.step()
    for i in range(1, 4):
        static_x.copy_(xs[i])
        gr.replay()
        torch.cuda.synchronize()
        assert static_loss.item() == eager[i - 1], (i, static_loss.item(), eager[i - 1])
        assert torch.isfinite(torch.randn(1000, device=cuda).sum()).item()        # eager work between replays
    for a, b in zip(w_eager, m.parameters()):
        assert torch.equal(a, b.detach())


def test_graph_level_training_step_replays_from_a_graph(cuda):
    """A training step of the graph-level Graphormer mirror (node features, bias builder, dense attention, encoder
    kernels, L1 loss, backward, SGD) captured once and replayed on other batches' targets and features, with eager
    work between the replays.  The table gradients are summed with atomics, whose order changes from run to run: the
    losses and the final weights agree with the eager sequence within the spread that two eager runs show (times 20; at least
    1e-3 of the loss and of the largest weight: the dense attention rounds its operands to bf16, so a last-bit difference
    in a sum can move a rounded operand by 2^-9 of its value) with the eager sequence, not bit for
    bit; SGD keeps that noise proportional (an Adam step would turn a rounding-sized gradient into a full-sized update)."""
    import types
    import numpy as np
    from torchgt_amd.graph_level import Graphormer
    data = workloads.erdos_renyi_batch(batch=8, seed=13)
    sizes, s = data["n_nodes"], data["spatial_pos"].shape[1]
    rng = np.random.default_rng(1)
    deg = np.zeros((8, s), np.int64)
    xs = []
    for g in range(8):
        n = int(sizes[g])
        deg[g, :n] = np.minimum((data["spatial_pos"][g][:n, :n] == 2).sum(1) + 1, 63)
    for _ in range(4):
        x = np.zeros((8, s, 1), np.int64)
        for g in range(8):
            x[g, :int(sizes[g]), 0] = rng.integers(1, 64, size=int(sizes[g]))
        xs.append(torch.from_numpy(x).to(cuda))
    ys = [torch.randn(8, generator=torch.Generator().manual_seed(i)).to(cuda) for i in range(4)]
    batch = types.SimpleNamespace(
        x=xs[0].clone(), in_degree=torch.from_numpy(deg).to(cuda), out_degree=torch.from_numpy(deg).to(cuda),
        attn_bias=torch.from_numpy(data["attn_bias"]).float().to(cuda), spatial_pos=torch.from_numpy(data["spatial_pos"]).long().to(cuda),
        attn_edge_type=torch.from_numpy(data["edge_type"]).long().unsqueeze(-1).contiguous().to(cuda), edge_input=None)
    static_y = ys[0].clone()

    def make():
        torch.manual_seed(3)
        m = Graphormer(2, 8, 64, 0.0, 0.0, 64, "ZINC", "single_hop", 5, 0.0, 1).to(cuda)
        with torch.no_grad():
            for p in m.parameters():
                if p.dim() == 2:
                    p.mul_(5.0)                       # away from the flat attention of the reference's init
        return m, torch.optim.SGD(m.parameters(), lr=0.05)

    def step(m, opt):
        opt.zero_grad(set_to_none=True)
        loss = torch.nn.functional.l1_loss(m(batch).view(-1), static_y)
        loss.backward()
        opt.step()
        return loss

    def load(i):
        batch.x.copy_(xs[i])
        static_y.copy_(ys[i])

    m, opt = make()
    load(0)
    for _ in range(2):
        step(m, opt)
    eager = []
    for i in range(1, 4):
        load(i)
        eager.append(step(m, opt).item())
    w_eager = [p.detach().clone() for p in m.parameters()]

    # the run-to-run spread of the eager sequence itself: the yardstick for the replays
    m, opt = make()
    load(0)
    for _ in range(2):
        step(m, opt)
    eager2 = []
    for i in range(1, 4):
        load(i)
        eager2.append(step(m, opt).item())
    wmax = max(p.abs().max().item() for p in w_eager)
    spread_w = max((a - b.detach()).abs().max().item() for a, b in zip(w_eager, m.parameters()))
    spread_l = max(abs(a - b) for a, b in zip(eager, eager2))
    print(f"eager run-to-run spread: loss {spread_l:.3e}, weights {spread_w:.3e} (largest weight {wmax:.3f})", flush=True)
    tol_l, tol_w = max(1e-3, 20 * spread_l), max(1e-3 * wmax, 20 * spread_w)

    m, opt = make()
    load(0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(m, opt)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    gr = torch.cuda.CUDAGraph()
    opt.zero_grad(set_to_none=True)
    with torch.cuda.graph(gr):
        static_loss = torch.nn.functional.l1_loss(m(batch).view(-1), static_y)
        static_loss.backward()
        opt.step()
    for i in range(1, 4):
        load(i)
        gr.replay()
        torch.cuda.synchronize()
        assert abs(static_loss.item() - eager[i - 1]) <= tol_l, (i, static_loss.item(), eager[i - 1], tol_l)
        assert torch.isfinite(torch.randn(1000, device=cuda).sum()).item()        # eager work between replays
    got_w = max((a - b.detach()).abs().max().item() for a, b in zip(w_eager, m.parameters()))
    print(f"graph replays against eager: weights {got_w:.3e} (bar {tol_w:.3e})", flush=True)
    assert got_w <= tol_w
