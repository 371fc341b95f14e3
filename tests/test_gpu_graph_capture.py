"""The C-ABI calls launch kernels only (no allocation, no synchronisation, no memset), so a
forward + backward step can be captured into a HIP graph and replayed.  Every replay is checked
against the eager result, with the program's own eager work and synchronisations in between."""
import pytest
import torch

from torchgt_amd import GraphPlan, _lib, workloads

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
