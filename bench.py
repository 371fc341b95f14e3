#!/usr/bin/env python3
"""Benchmark of the sparse-attention hot path on one MI355X.

A step is one forward + backward of one layer's sparse attention (the C-ABI calls
tgt_sparse_attn_fwd + tgt_sparse_attn_bwd) on the 64 K-node power-law graph of
the benchmark configuration "configs[1]": N = 64 001, E ~ 530 K, H = 8, d = 8, per-edge bias
[E, 8] with gradient, inputs resident in HBM, plan prebuilt (its build time is
reported separately).  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--dtype f32|bf16] [--no-cpu-baseline]
                    [--workload config1|config2|config2-mha|config2-model|config2-gt-model|config3|config4|config4-bias|
                               config4-bias-multihop|config4-model|config5|config5-blockized]

config3 / config5: larger sparse workloads (bf16); config4: dense biased attention of a graph-level
batch; config4-bias: the bias builder in front of it (GraphAttnBias forward + table gradients); config4-bias-multihop:
the same with the path-encoding ('multi_hop') edge term; config4-model: a training step of the graph-level Graphormer
on that batch; config5-blockized: the block path on the reordered config5 graph; config2-mha: one whole
MultiHeadAttention layer (projections + sparse attention) on the config2 graph; config2-model: a training
step of the 4-layer Graphormer-Slim on that graph; config2-gt-model: the same for the node-level GT.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0     # MI355X HBM3E, published


def alg_bytes(N, E, H, d, esize, bias_bytes_per_edge, bias_grad):
    """Compulsory bytes of one fwd+bwd (every operand once per pass, gathers cache-served),
    and the share of each pass.  R = H*d*esize."""
    R = H * d * esize
    fwd = 3 * N * R + N * R + 4 * N * H + 4 * (N + 1) + 4 * E + E * bias_bytes_per_edge
    bwd = (5 * N * R + 3 * N * R + 4 * N * H + 2 * (4 * (N + 1) + 4 * E) + 4 * E
           + E * bias_bytes_per_edge * (2 if bias_grad else 1))
    return fwd, bwd


def kernel_alg_bytes(name, N, E, H, d, esize, bpe):
    """Compulsory bytes of ONE launch of a named kernel (what it must read and write once)."""
    R = H * d * esize
    csr = 4 * (N + 1) + 4 * E + 4 * E      # rowptr, col, edge ids (bias is addressed through them)
    table = {
        # q,k,v in, out + Z out, one sorted view, bias
        "attn_fwd": 3 * N * R + N * R + 4 * N * H + csr + E * bpe,
        "bwd_node_side": 2 * N * R + 4 * N * H + 8 * N * H,
        # q,k,v,dout + nd in, dq,dk,dv out, both sorted views, bias in (once), dbias out
        "attn_bwd": 4 * N * R + 8 * N * H + 3 * N * R + 2 * csr + 2 * E * bpe,
    }
    return table.get(name)


# HBM-side bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, each
# scaled by the reading of a copy kernel of known size: FETCH x2.000, WRITE x1.000); the summary is
# profiles/sparse_attn_config2_hbm_traffic_pmc.txt.  Counters cannot be read from inside this process,
# so the figures are carried here, reported only for the workload / dtype they were measured on, and the
# bench line says when and on which commit of the kernels they were taken (a kernel change after that
# commit makes them stale: measure again).
MEASURED_TRAFFIC = {
    ("config2", "f32"): {"attn_fwd": 237.2e6, "bwd_node_side": 38.9e6, "attn_bwd": 546.6e6},
    ("config2", "bf16"): {"attn_fwd": 131.1e6, "bwd_node_side": 22.5e6, "attn_bwd": 318.7e6},
}
MEASURED_TRAFFIC_AT = {"date": "2026-11-26", "kernels_as_of_commit": "95a5294",
                       "summary": "profiles/sparse_attn_config2_hbm_traffic_pmc.txt"}


def build_workload(name):
    import numpy as np
    from torchgt_amd import workloads
    if name == "config2":
        e, n = workloads.power_law_graph(n=64000, exponent=2.1, directed_edges=530_000, seed=42)
        label = "configs[1]: power-law (exp 2.1) 64000 nodes + 1 global node"
    elif name == "config1":
        e, n = workloads.barabasi_albert(n=4096, m=4, seed=42)
        label = "configs[0]: Barabasi-Albert 4096 nodes m=4 + 1 global node"
    elif name == "config3":
        e, n = workloads.clustered_power_law_graph(n=870_000, exponent=2.0, directed_edges=44_000_000, seed=42)
        label = "configs[2]: clustered power-law (exp 2.0) 870000 nodes + 1 global node, cluster-ordered"
    elif name == "config5":
        e, n, _ = workloads.stochastic_block_model(seed=42)
        label = "configs[4]: SBM 64 x 4096 nodes, p_intra 0.004, 5% inter-cluster, cluster-ordered"
    else:
        raise SystemExit(f"unknown workload {name}")
    return e, n, label, workloads.describe(e, n)


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(e, n, H, d, seconds_budget=30.0):
    """The oracle (op-for-op restatement of the reference's PyTorch path, fp32,
    autograd backward) timed on this host's cores with the same seeded inputs."""
    import torch
    from oracle import sparse_attention as osa
    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(42)
    ei = torch.from_numpy(e)
    E = e.shape[1]
    q, k, v = (torch.randn(n, H, d, generator=g).requires_grad_(True) for _ in range(3))
    bias = (torch.randn(E, H, generator=g) * 0.02).requires_grad_(True)
    dout = torch.randn(n, H, d, generator=g)

    def step():
        out, _ = osa.sparse_attention(q, k, v, ei, bias)
        torch.autograd.grad(out, (q, k, v, bias), dout)

    times = []
    t_start = time.perf_counter()
    for _ in range(3):                           # warm-up
        step()
    while len(times) < 10 and (len(times) < 3 or (time.perf_counter() - t_start) < seconds_budget):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {"value": E / med, "unit": "edges/s", "cores": cores, "cpu_model": cpu_model(), "kind": "port",
            "sample": f"full workload (E={E}), fp32, {len(times)} fwd+bwd iterations after 3 warm-ups, median",
            "ms_per_step": med * 1e3}


def reference_ops_on_gpu(ei, q, k, v, bias, dout, steps=20):
    """The reference's formulation on this GPU: its chain of stock PyTorch-ROCm ops (gathers,
    elementwise ops, index_add_ scatter-adds, autograd backward; attn_module.py:146-187), fp32, same
    inputs.  A datapoint beside the HIP path, not a checker: nothing is compared with it."""
    import torch
    H, d = q.shape[1], q.shape[2]
    src, dst = ei[0], ei[1]
    qf, kf, vf, bf = (t.detach().float().requires_grad_(True) for t in (q, k, v, bias))
    g = dout.float()

    def step():
        s = (kf[src] * qf[dst] / (d ** 0.5)).sum(-1).clamp(-5, 5) + bf
        w = torch.exp(s)
        wv = torch.zeros_like(qf).index_add_(0, dst, w.unsqueeze(-1) * vf[src])
        z = torch.zeros(qf.shape[0], H, device=qf.device).index_add_(0, dst, w)
        out = wv / (z.unsqueeze(-1) + 1e-6)
        torch.autograd.grad(out, (qf, kf, vf, bf), g)

    for _ in range(3):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    return {"ms_per_step": ms, "edges_per_s": ei.shape[1] / (ms * 1e-3), "dtype": "f32",
            "what": "reference op chain with stock PyTorch-ROCm kernels (index gathers + index_add_, autograd)"}


def bench_dense(args):
    """Benchmark configuration configs[3]: dense biased attention on a batch of 256 padded ER graphs (S = 129,
    H = 8, d = 8, bf16, bias [b,H,S,S] with gradient).  A step = tgt_dense_attn_fwd + _bwd."""
    import torch
    from torchgt_amd import _lib, workloads
    dev = torch.device("cuda:0")
    b, H, d = 256, 8, 8
    data = workloads.erdos_renyi_batch(batch=b, seed=42)
    S = data["S"]
    tdt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    esize = 2 if args.dtype == "bf16" else 4
    g = torch.Generator().manual_seed(42)
    q, k, v, dout = (torch.randn(b, S, H, d, generator=g).to(dev, tdt) for _ in range(4))
    bias = (torch.randn(b, H, S, S, generator=g) * 0.02 + torch.from_numpy(data["attn_bias"]).unsqueeze(1)).to(dev, tdt)
    out = torch.empty(b, S, H * d, device=dev, dtype=tdt)
    lse = torch.empty(b, H, S, device=dev)
    dq, dk, dv, dbias = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q), torch.empty_like(bias)
    L = _lib.lib()
    dt_code = _lib.DTYPE_BF16 if args.dtype == "bf16" else _lib.DTYPE_F32
    stream = torch.cuda.current_stream(dev).cuda_stream
    P = lambda t: t.data_ptr()

    def step():
        _lib.check(L.tgt_dense_attn_fwd(P(q), P(k), P(v), P(bias), b, S, H, d, dt_code, P(out), P(lse), stream))
        _lib.check(L.tgt_dense_attn_bwd(P(q), P(k), P(v), P(bias), b, S, H, d, dt_code, P(out), P(lse), P(dout),
                                        P(dq), P(dk), P(dv), P(dbias), stream))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    L.tgt_timing_reset()
    L.tgt_timing_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    L.tgt_timing_enable(0)
    kernels = {n: {"avg_us": t / c * 1e3, "launches": c} for n, (t, c) in _lib.kernel_timings().items() if c}
    node_b = b * S * H * d * esize
    bias_b = b * H * S * S * esize
    alg = {"dense_fwd": 4 * node_b + bias_b + 4 * b * H * S, "dense_bwd": 8 * node_b + 2 * bias_b + 4 * b * H * S}
    flops = {"dense_fwd": 4 * b * H * S * S * d, "dense_bwd": 10 * b * H * S * S * d}
    # The same attention with the bias formed on chip from 16-bit ids and the three tables of the graph-level model
    # (tgt_dense_attn_ids_fwd / _bwd, table gradients included): no [b, H, S, S] tensor in either direction.
    from_ids = None
    if args.dtype == "bf16":
        n_sp, n_e, F = 40, 64, 1                                   # the ZINC tables of models/graphormer_graph_level.py:325-339
        sp = torch.from_numpy(data["spatial_pos"]).long().to(dev)
        et = torch.from_numpy(data["edge_type"]).long().unsqueeze(-1).contiguous().to(dev)
        sp16 = torch.empty(b, S, S, dtype=torch.int16, device=dev)
        et16 = torch.empty(b, S, S, F, dtype=torch.int16, device=dev)
        _lib.check(L.tgt_dense_ids_pack(P(sp), P(et), b, S - 1, F, n_sp, n_e, P(sp16), P(et16), stream))
        ab = torch.from_numpy(data["attn_bias"]).to(dev, tdt)
        t_sp, t_e, t_v = ((torch.randn(n, H, generator=g) * 0.02).to(dev, tdt) for n in (n_sp, n_e, 1))
        d_sp, d_e, d_v = torch.empty_like(t_sp), torch.empty_like(t_e), torch.empty_like(t_v)
        code = dt_code
        nbytes = L.tgt_dense_attn_ids_bwd_workspace_bytes(b, H, n_sp, n_e)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)

        def step_ids():
            _lib.check(L.tgt_dense_attn_ids_fwd(P(q), P(k), P(v), P(ab), P(sp16), P(et16), F, P(t_sp), n_sp, P(t_e), n_e, P(t_v),
                                                b, S, H, d, code, 0.0, 0, P(out), P(lse), stream))
            _lib.check(L.tgt_dense_attn_ids_bwd(P(q), P(k), P(v), P(ab), P(sp16), P(et16), F, P(t_sp), n_sp, P(t_e), n_e, P(t_v),
                                                b, S, H, d, code, 0.0, 0, P(out), P(lse), P(dout), P(dq), P(dk), P(dv),
                                                P(d_sp), P(d_e), P(d_v), P(ws), nbytes, stream))

        for _ in range(args.warmup):
            step_ids()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step_ids()
        torch.cuda.synchronize()
        ms_ids = (time.perf_counter() - t0) / args.steps * 1e3
        L.tgt_timing_reset()
        L.tgt_timing_enable(1)
        for _ in range(args.steps):
            step_ids()
        torch.cuda.synchronize()
        L.tgt_timing_enable(0)
        k_ids = {n: {"avg_us": t / c * 1e3, "launches": c} for n, (t, c) in _lib.kernel_timings().items() if c}
        ids_b = b * S * S * (2 + 2 * F + esize)
        alg_ids = {"dense_fwd": 4 * node_b + ids_b + 4 * b * H * S, "dense_bwd": 8 * node_b + ids_b + 4 * b * H * S}
        from_ids = {"ms_per_step": ms_ids, "graphs_per_s": b / (ms_ids * 1e-3), "tables": [n_sp, n_e, 1], "edge_features": F,
                    "step": "tgt_dense_attn_ids_fwd + tgt_dense_attn_ids_bwd (dq, dk, dv and the three table gradients)",
                    "kernels": {n: dict(v, alg_bytes=alg_ids[n], hbm_frac=alg_ids[n] / (v["avg_us"] * 1e-6) / 1e9 / HBM_PEAK_GBS,
                                        alg_tflops=flops[n] / (v["avg_us"] * 1e-6) / 1e12) for n, v in k_ids.items() if n in alg_ids},
                    "bias_tensor_bytes_avoided": 3 * bias_b}
    dom = max(kernels, key=lambda n: kernels[n]["avg_us"])
    gbs = alg[dom] / (kernels[dom]["avg_us"] * 1e-6) / 1e9
    result = {
        "metric": "fwd+bwd dense biased attention (graph-level batch); % HBM roofline",
        "value": b / (ms * 1e-3), "unit": "graphs/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "configs[3]: 256 ER graphs n~U[16,128] p=0.1 padded to 128 + virtual node",
                   "b": b, "S": S, "H": H, "d": d, "bias": "[b,H,S,S] with gradient, -inf on padded keys",
                   "step": "tgt_dense_attn_fwd + tgt_dense_attn_bwd", "parallelism": "1 GPU"},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS,
                     # rocprofv3 FETCH_SIZE x2.000 + WRITE_SIZE x1.000, profiles/dense_attn_config4_bf16.txt
                     "traffic": {"dense_fwd": 107.6e6, "dense_bwd": 219.8e6}.get(dom) if args.dtype == "bf16" else None,
                     "alg_bytes": alg[dom],
                     "avg_us": kernels[dom]["avg_us"]},
        "mfma": {n: {"alg_tflops": flops[n] / (kernels[n]["avg_us"] * 1e-6) / 1e12, "peak_tflops": 2500.0}
                 for n in kernels},
        "kernels": kernels,
        "from_ids": from_ids,
    }
    return result


def bench_graph_bias(args):
    """The bias builder in front of configs[3]: GraphAttnBias forward and the gradients of its three tables for
    the batch of 256 padded ER graphs (S = 129, H = 8, one edge feature, tables [22, 8] and [5, 8]).
    A step = tgt_graph_attn_bias_fwd + tgt_graph_attn_bias_bwd."""
    import torch
    from torchgt_amd import _lib, workloads
    dev = torch.device("cuda:0")
    b, H, F, n_sp, n_e = 256, 8, 1, 22, 5
    data = workloads.erdos_renyi_batch(batch=b, seed=42)
    S1 = data["S"]
    s = S1 - 1
    tdt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    esize = 2 if args.dtype == "bf16" else 4
    g = torch.Generator().manual_seed(42)
    attn_bias = torch.from_numpy(data["attn_bias"]).to(dev, tdt)
    spatial_pos = torch.from_numpy(data["spatial_pos"]).long().to(dev)
    edge_type = torch.from_numpy(data["edge_type"]).long().unsqueeze(-1).contiguous().to(dev)
    t_sp, t_e, t_v = ((torch.randn(n, H, generator=g) * 0.02).to(dev, tdt) for n in (n_sp, n_e, 1))
    out = torch.empty(b, H, S1, S1, device=dev, dtype=tdt)
    dout = torch.randn(b, H, S1, S1, generator=g).to(dev, tdt)
    dout[~torch.isfinite(attn_bias).unsqueeze(1).expand_as(dout)] = 0       # masked entries carry no gradient
    d_sp, d_e, d_v = torch.empty_like(t_sp), torch.empty_like(t_e), torch.empty_like(t_v)
    L = _lib.lib()
    dt_code = _lib.DTYPE_BF16 if args.dtype == "bf16" else _lib.DTYPE_F32
    nbytes = L.tgt_graph_attn_bias_bwd_workspace_bytes(n_sp, n_e, H)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    P = lambda t: t.data_ptr()
    multi_hop = args.workload == "config4-bias-multihop"
    prep_ms = None
    if multi_hop:
        # the path-encoding branch: edge_input [b, s, s, D, F] from the library's own Floyd-Warshall and gen_edge_input
        from torchgt_amd import floyd_warshall, gen_edge_input
        D, n_dis = 5, 128                  # multi_hop_max_dist and num_edge_dis of the reference's graph-level scripts
        sizes = torch.from_numpy(data["n_nodes"]).to(dev)
        adj = (spatial_pos == 2).to(torch.uint8)
        feat = edge_type * adj.unsqueeze(-1).long()

        def prep():
            _, path = floyd_warshall(adj, sizes)
            return gen_edge_input(D, path, feat, sizes) + 1        # collator: features + 1, 0 = padding
        edge_input = prep()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            edge_input = prep()
        torch.cuda.synchronize()
        prep_ms = (time.perf_counter() - t0) / 5 * 1e3
        edge_input = edge_input.contiguous()
        t_w = (torch.randn(n_dis * H * H, generator=g) * 0.02).to(dev, tdt)
        d_w = torch.empty_like(t_w)
        nbytes_mh = L.tgt_graph_attn_bias_multi_hop_bwd_workspace_bytes(n_sp, n_e, H, D)
        ws_mh = torch.empty(nbytes_mh, dtype=torch.uint8, device=dev)

    def step():
        if multi_hop:
            _lib.check(L.tgt_graph_attn_bias_multi_hop_fwd(P(attn_bias), P(spatial_pos), P(edge_input), D, F, P(t_sp), n_sp,
                                                           P(t_e), n_e, P(t_w), n_dis, P(t_v), D, b, s, H, dt_code, P(out),
                                                           stream))
            _lib.check(L.tgt_graph_attn_bias_multi_hop_bwd(P(dout), P(spatial_pos), P(edge_input), D, F, P(t_e), n_sp, n_e,
                                                           P(t_w), n_dis, D, b, s, H, dt_code, P(d_sp), P(d_e), P(d_w),
                                                           P(d_v), P(ws_mh), nbytes_mh, stream))
            return
        _lib.check(L.tgt_graph_attn_bias_fwd(P(attn_bias), P(spatial_pos), P(edge_type), F, P(t_sp), n_sp, P(t_e), n_e, P(t_v),
                                             b, s, H, dt_code, P(out), stream))
        _lib.check(L.tgt_graph_attn_bias_bwd(P(dout), P(spatial_pos), P(edge_type), F, n_sp, n_e, b, s, H, dt_code,
                                             P(d_sp), P(d_e), P(d_v), P(ws), nbytes, stream))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    L.tgt_timing_reset()
    L.tgt_timing_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    L.tgt_timing_enable(0)
    kernels = {n: {"avg_us": t / c * 1e3, "launches": c} for n, (t, c) in _lib.kernel_timings().items() if c}
    ids_b = b * s * s * 8 * (1 + (D if multi_hop else 1) * F)      # int64 spatial_pos and edge_type / edge_input
    bias_b = b * H * S1 * S1 * esize
    alg = {"graph_bias_fwd": b * S1 * S1 * esize + ids_b + bias_b, "graph_bias_bwd": bias_b + ids_b}
    dom = max(kernels, key=lambda n: kernels[n]["avg_us"])
    gbs = alg[dom] / (kernels[dom]["avg_us"] * 1e-6) / 1e9
    result = {
        "metric": "GraphAttnBias forward + table gradients (graph-level batch); % HBM roofline",
        "value": b / (ms * 1e-3), "unit": "graphs/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "bias builder of configs[3]: 256 ER graphs n~U[16,128] p=0.1 padded to 128 + virtual node",
                   "b": b, "S": S1, "H": H, "edge_features": F, "tables": [[n_sp, H], [n_e, H], [1, H]],
                   "step": ("tgt_graph_attn_bias_multi_hop_fwd + _bwd (5 hops, 128 hop matrices)" if multi_hop
                            else "tgt_graph_attn_bias_fwd + tgt_graph_attn_bias_bwd"), "parallelism": "1 GPU"},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": gbs / HBM_PEAK_GBS, "traffic": None, "alg_bytes": alg[dom], "avg_us": kernels[dom]["avg_us"]},
        "alg_bytes": alg,
        "kernels": kernels,
    }
    if prep_ms is not None:
        result["floyd_warshall_plus_gen_edge_input_ms"] = prep_ms
    return result


def bench_block(args):
    """Benchmark configuration configs[4] through the reference's pipeline: SBM 64 x 4096, the reference's
    cluster reordering with the clusters as partitions (every partition pair's edges become
    dense 16 x 16 blocks), then attention.  A step = tgt_block_attn_fwd + _bwd on the tile list;
    the same edges through the sparse kernels (expanded list) are timed next to it."""
    import numpy as np
    import torch
    from torchgt_amd import _lib, graph_prep, workloads
    from torchgt_amd.block_attention import TileSet
    from torchgt_amd.plan import GraphPlan
    dev = torch.device("cuda:0")
    H, d = 8, 8
    tdt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    e, n, cluster = workloads.stochastic_block_model(seed=42)
    hybrid = args.workload == "config5-hybrid"
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if hybrid:
        tiles, raw, new_e = workloads.hybrid_tiles(e, cluster, 64, 16, seed=42)
        raw, new_e = torch.from_numpy(raw).to(dev), torch.from_numpy(new_e).to(dev)
    else:
        new_e, _, tiles, raw = graph_prep.reformat_graph(torch.from_numpy(e).to(dev), 64, 16,
                                                         partition_ids=torch.from_numpy(cluster), return_tiles=True)
    torch.cuda.synchronize()
    reorder_ms = (time.perf_counter() - t0) * 1e3
    E = int(new_e.shape[1])
    ts = TileSet(tiles, n, dev)
    plan_rest = GraphPlan(raw, n, rows_with_edges_only=True)
    plan_full = GraphPlan(new_e, n)
    g = torch.Generator().manual_seed(42)
    q, k, v, dout = (torch.randn(n, H, d, generator=g).to(dev, tdt) for _ in range(4))
    out = torch.empty_like(q)
    Z = torch.empty(n, H, device=dev)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    L = _lib.lib()
    code = _lib.DTYPE_BF16 if args.dtype == "bf16" else _lib.DTYPE_F32
    stream = torch.cuda.current_stream(dev).cuda_stream
    P = lambda t: t.data_ptr()
    wsb = ts.workspace(plan_rest, H, d)
    wss = plan_full.workspace(H, d)

    def step_block():
        _lib.check(L.tgt_block_attn_fwd(ts.handle, plan_rest.handle, P(q), P(k), P(v), None, 0, H, d, code, P(out),
                                        P(Z), P(wsb), wsb.numel(), stream))
        _lib.check(L.tgt_block_attn_bwd(ts.handle, plan_rest.handle, P(q), P(k), P(v), None, 0, H, d, code, P(out),
                                        P(Z), P(dout), P(dq), P(dk), P(dv), None, P(wsb), wsb.numel(), stream))

    def step_sparse():
        _lib.check(L.tgt_sparse_attn_fwd(plan_full.handle, P(q), P(k), P(v), None, 0, H, d, code, P(out), P(Z),
                                         P(wss), wss.numel(), stream))
        _lib.check(L.tgt_sparse_attn_bwd(plan_full.handle, P(q), P(k), P(v), None, 0, H, d, code, P(out), P(Z),
                                         P(dout), P(dq), P(dk), P(dv), None, P(wss), wss.numel(), stream))

    def timed(fn):
        for _ in range(args.warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    ms_block = timed(step_block)
    L.tgt_timing_reset()
    L.tgt_timing_enable(1)
    for _ in range(args.steps):
        step_block()
    torch.cuda.synchronize()
    L.tgt_timing_enable(0)
    kernels = {nm: {"avg_us": t / c * 1e3, "launches": c} for nm, (t, c) in _lib.kernel_timings().items() if c}
    ms_sparse = timed(step_sparse)
    esize = 2 if args.dtype == "bf16" else 4
    R = H * d * esize
    # compulsory bytes: every node row once per pass (12 N R), Z written and read (8 N H), a tile is 8 bytes and
    # is read by the forward and by both walks of the backward, 16 bytes of sorted views per remaining edge.  The
    # fp32 tile sums the hybrid mode passes between its kernels are the implementation's own traffic: not counted.
    alg = 12 * n * R + 8 * n * H + 3 * 8 * len(tiles) + 16 * int(raw.shape[1])
    result = {
        "metric": "fwd+bwd block attention (16x16 tiles on MFMA + sparse remainder) edges/sec; ms/layer",
        "value": E / (ms_block * 1e-3), "unit": "edges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_block, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": ("configs[4]: SBM 64 x 4096, hybrid: intra-cluster edges as 16x16 tiles, inter-cluster edges raw, one softmax"
                                if hybrid else
                                "configs[4]: SBM 64 x 4096 reordered by the reference's blockize (k=64, 16x16 blocks)"),
                   "N": n, "tiles": int(len(tiles)), "E_expanded": E, "E_remainder": int(raw.shape[1]), "H": H, "d": d,
                   "step": "tgt_block_attn_fwd + tgt_block_attn_bwd", "parallelism": "1 GPU"},
        "roofline": {"bound": "hbm", "kernel": "whole step", "achieved": alg / (ms_block * 1e-3) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": alg / (ms_block * 1e-3) / 1e9 / HBM_PEAK_GBS,
                     "traffic": None, "alg_bytes": alg},
        "kernels": kernels,
        "sparse_path_same_edges_ms": ms_sparse,
        "reorder_ms": reorder_ms,
    }
    return result


def bench_mha(args):
    """One MultiHeadAttention layer of configs[1] (hidden 64, 8 heads, N = 64 001, E ~ 530 K, no bias as in the
    shipped node-level runs): q/k/v projections, sparse attention, output projection, forward + backward with all
    parameter gradients.  A step = tgt_linear_fwd(3) + tgt_sparse_attn_fwd + tgt_linear_fwd(1) and their backwards,
    driven through the module (torch autograd bookkeeping included in the wall time)."""
    import torch
    from torchgt_amd import MultiHeadAttention, _lib
    dev = torch.device("cuda:0")
    hidden, H = 64, 8
    e, n, label, desc = build_workload("config2")
    tdt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    esize = 2 if args.dtype == "bf16" else 4
    torch.manual_seed(42)
    m = MultiHeadAttention(hidden, 0.0, H, 1).to(dev, tdt)
    ei = torch.from_numpy(e).to(dev)
    x = torch.randn(1, n, hidden, device=dev).to(tdt).requires_grad_(True)
    gy = torch.randn(1, n, hidden, device=dev).to(tdt)
    params = list(m.parameters())

    def step():
        y = m(x, None, ei, "sparse")
        torch.autograd.grad(y, [x] + params, gy)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    L = _lib.lib()
    L.tgt_timing_reset()
    L.tgt_timing_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    L.tgt_timing_enable(0)
    # per step: linear_fwd runs twice (q/k/v and output), linear_dx and linear_dw twice
    kernels = {k: {"avg_us": t / c * 1e3, "launches_per_step": c / args.steps} for k, (t, c) in _lib.kernel_timings().items() if c}
    gpu_us = sum(v["avg_us"] * v["launches_per_step"] for v in kernels.values())
    row = n * hidden * esize
    # projections, every operand once: forward reads x and writes q, k, v (4 rows), output layer 2 rows;
    # input gradients read 3 + 1 and write 1 + 1 rows; weight gradients read 4 + 2 rows
    lin_bytes = (4 + 2 + 4 + 2 + 4 + 2) * row
    lin_us = sum(kernels[k]["avg_us"] * kernels[k]["launches_per_step"] for k in kernels if k.startswith("linear"))
    lin_flops = 2 * n * hidden * hidden * 4 * 3       # four 64 x 64 weights, forward + two backward products
    result = {
        "metric": "fwd+bwd of one MultiHeadAttention layer (projections + sparse attention)",
        "value": e.shape[1] / (ms * 1e-3), "unit": "edges/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "configs[1] graph, MultiHeadAttention(hidden 64, 8 heads) layer, no bias", "N": n,
                   "E": int(e.shape[1]), "step": "module forward + autograd backward (x and all parameters)",
                   "parallelism": "1 GPU"},
        "gpu_kernel_us_per_step": gpu_us,
        "projections": {"us_per_step": lin_us, "alg_bytes": lin_bytes,
                        "hbm_frac": lin_bytes / (lin_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                        "alg_tflops": lin_flops / (lin_us * 1e-6) / 1e12,
                        "mfma_peak_tflops": 157.3 if args.dtype == "f32" else 2500.0},
        "kernels": kernels,
    }
    return result


def bench_model(args):
    """One training step of the Graphormer-Slim of configs[1] (4 layers, hidden 64, ffn 64, 8 heads, 128-d input,
    40 classes; 111 913 parameters) on the whole 64 K-node graph as one sequence: forward, nll loss, backward,
    AdamW step (torch's optimizer, as in the reference's training loop)."""
    import torch
    from torchgt_amd import GT, Graphormer as NodeGraphormer, _lib, nll_loss as lib_nll_loss
    nll_loss = torch.nn.functional.nll_loss if args.torch_loss else lib_nll_loss
    dev = torch.device("cuda:0")
    e, n, label, desc = build_workload("config2")
    tdt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    gt = args.workload == "config2-gt-model"
    # the GT of models/gt_dist_node_level.py has no global token: node 0 of the graph is an ordinary node there
    Graphormer = (lambda *a: GT(*a[:-1], 0)) if gt else NodeGraphormer
    n_rows = n if gt else n - 1
    torch.manual_seed(42)
    m = Graphormer(4, 8, 128, 64, 40, 1, 0.0, 0.0, 0.0, 64, 1).to(dev, tdt)
    opt = torch.optim.AdamW(m.parameters(), lr=1e-3, weight_decay=0.01, fused=not args.foreach_adamw)
    ei = torch.from_numpy(e).to(dev)
    x = torch.randn(n_rows, 128, device=dev).to(tdt)
    y = torch.randint(0, 40, (n_rows,), device=dev)

    def step():
        opt.zero_grad(set_to_none=True)
        out = m(x, None, ei, attn_type="sparse")
        loss = nll_loss(out.float(), y)
        loss.backward()
        opt.step()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    # The reference's loop moves the CPU-resident edge_index of a pre-packed batch to the GPU in every iteration
    # (main_sp_sparse_node_level.py:178-183): the same step with a fresh copy each time.  The first such step
    # finds the plan by its content key; no step builds one.
    from torchgt_amd import plan as plan_mod
    ei_cpu = torch.from_numpy(e).pin_memory()
    builds_before = plan_mod.plan_cache_stats()["builds"]

    def fresh_step():
        opt.zero_grad(set_to_none=True)
        out = m(x, None, ei_cpu.to(dev, non_blocking=True), attn_type="sparse")
        loss = nll_loss(out.float(), y)
        loss.backward()
        opt.step()

    for _ in range(3):
        fresh_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fresh_step()
    torch.cuda.synchronize()
    fresh_ms = (time.perf_counter() - t0) / args.steps * 1e3
    fresh_builds = plan_mod.plan_cache_stats()["builds"] - builds_before
    # what of that is the copy itself (the reference's loop pays it too) and what the look-up by content costs
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fresh = ei_cpu.to(dev, non_blocking=True)
        torch.cuda.synchronize()
    copy_ms = (time.perf_counter() - t0) / args.steps * 1e3
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fresh = ei_cpu.to(dev, non_blocking=True)
        plan_mod.get_plan(fresh, n)
        torch.cuda.synchronize()
    lookup_ms = (time.perf_counter() - t0) / args.steps * 1e3 - copy_ms
    L = _lib.lib()
    L.tgt_timing_reset()
    L.tgt_timing_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    L.tgt_timing_enable(0)
    kernels = {k: {"avg_us": t / c * 1e3, "launches_per_step": c / args.steps} for k, (t, c) in _lib.kernel_timings().items() if c}
    lib_us = sum(v["avg_us"] * v["launches_per_step"] for v in kernels.values())
    loss_value = float(loss.detach())
    # The same step captured once into a HIP graph (the library calls only launch kernels) and replayed.  A fresh
    # model and optimizer are used, warmed up on a side stream: autograd nodes that earlier eager steps created on
    # the default stream (kept alive by their loss tensor) must not take part in a capture.
    graph_ms = None
    if args.hip_graph:
        del loss
        torch.manual_seed(42)
        gm = Graphormer(4, 8, 128, 64, 40, 1, 0.0, 0.0, 0.0, 64, 1).to(dev, tdt)
        gopt = torch.optim.AdamW(gm.parameters(), lr=1e-3, weight_decay=0.01, capturable=True)

        def gstep():
            gloss = nll_loss(gm(x, None, ei, attn_type="sparse").float(), y)
            gloss.backward()
            gopt.step()
            return gloss

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                gopt.zero_grad(set_to_none=True)
                gstep()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        gopt.zero_grad(set_to_none=True)
        with torch.cuda.graph(gr):
            gstep()
        for _ in range(args.warmup):
            gr.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            gr.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) / args.steps * 1e3
    groups = {"attention": ("attn_fwd", "bwd_node_side", "attn_bwd"), "projections and ffn linears": ("linear_fwd", "linear_dx", "linear_dw"),
              "layer norm + residual": ("layer_norm_fwd", "layer_norm_bwd"), "gelu": ("gelu",), "nll loss": ("nll_loss",)}
    result = {
        "metric": "training step of the 4-layer " + ("GT" if gt else "Graphormer-Slim") + " on one 64 K-node sequence",
        "value": 1e3 / ms, "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "configs[1] graph as one sequence, " + ("GT 4 x (hidden 64, ffn 128, 8 heads, MLP readout), " if gt else
                               "Graphormer-Slim 4 x (hidden 64, ffn 64, 8 heads), ") +
                               "128-d features, 40 classes, no bias, dropout 0", "N": n, "E": int(e.shape[1]),
                   "parameters": sum(p.numel() for p in m.parameters()),
                   "step": "forward + nll_loss (" + ("torch's" if args.torch_loss else "the library's") + ") + backward + torch AdamW (" + ("foreach" if args.foreach_adamw else "fused") + ")",
                   "parallelism": "1 GPU"},
        "loss": loss_value,
        "step_with_fresh_edge_index_ms": fresh_ms,
        "plans_built_by_the_fresh_edge_index_steps": fresh_builds,
        "edge_index_host_to_device_copy_ms": copy_ms,
        "plan_lookup_by_content_ms": lookup_ms,
        "ms_per_step_hip_graph": graph_ms,
        "library_kernel_us_per_step": lib_us,
        "kernel_groups_us": {g: sum(kernels[k]["avg_us"] * kernels[k]["launches_per_step"] for k in ks if k in kernels)
                             for g, ks in groups.items()},
        "kernels": kernels,
    }
    return result


def bench_graph_model(args):
    """One training step of the graph-level Graphormer (models/graphormer_graph_level.py; 4 layers, hidden 64, ffn 64,
    8 heads, ZINC tables, one regression target) on the batch of configs[3]: forward, L1 loss as the graph-level
    script computes it, backward, AdamW step (torch's optimizer)."""
    import numpy as np
    import torch
    import types
    from torchgt_amd import _lib, workloads
    from torchgt_amd.graph_level import Graphormer
    dev = torch.device("cuda:0")
    tdt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    b = 256
    data = workloads.erdos_renyi_batch(batch=b, seed=42)
    rng = np.random.default_rng(42)
    sizes = data["n_nodes"]
    s = data["spatial_pos"].shape[1]
    x = np.zeros((b, s, 1), np.int64)
    deg = np.zeros((b, s), np.int64)
    for g in range(b):
        n = int(sizes[g])
        x[g, :n, 0] = rng.integers(1, 64, size=n)
        deg[g, :n] = np.minimum((data["spatial_pos"][g][:n, :n] == 2).sum(1) + 1, 63)
    batch = types.SimpleNamespace(
        x=torch.from_numpy(x).to(dev), in_degree=torch.from_numpy(deg).to(dev), out_degree=torch.from_numpy(deg).to(dev),
        attn_bias=torch.from_numpy(data["attn_bias"]).to(dev, tdt), spatial_pos=torch.from_numpy(data["spatial_pos"]).long().to(dev),
        attn_edge_type=torch.from_numpy(data["edge_type"]).long().unsqueeze(-1).contiguous().to(dev), edge_input=None)
    torch.manual_seed(42)
    m = Graphormer(4, 8, 64, 0.0, 0.0, 64, "ZINC", "single_hop", 5, 0.0, 1).to(dev, tdt)
    m.bias_from_ids = bool(args.bias_from_ids)
    opt = torch.optim.AdamW(m.parameters(), lr=1e-3, weight_decay=0.01, fused=not args.foreach_adamw)
    y = torch.randn(b, device=dev)

    def step():
        opt.zero_grad(set_to_none=True)
        out = m(batch)
        loss = torch.nn.functional.l1_loss(out.float().view(-1), y)
        loss.backward()
        opt.step()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    L = _lib.lib()
    L.tgt_timing_reset()
    L.tgt_timing_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    L.tgt_timing_enable(0)
    kernels = {k: {"avg_us": t / c * 1e3, "launches_per_step": c / args.steps} for k, (t, c) in _lib.kernel_timings().items() if c}
    lib_us = sum(v["avg_us"] * v["launches_per_step"] for v in kernels.values())
    # The same step captured once into a HIP graph and replayed (the library calls only launch kernels); a fresh model
    # and optimizer, warmed up on a side stream, as for the node-level model.
    graph_ms = None
    if args.hip_graph:
        loss_value = float(loss.detach())
        del loss
        torch.manual_seed(42)
        gm = Graphormer(4, 8, 64, 0.0, 0.0, 64, "ZINC", "single_hop", 5, 0.0, 1).to(dev, tdt)
        gm.bias_from_ids = bool(args.bias_from_ids)
        gopt = torch.optim.AdamW(gm.parameters(), lr=1e-3, weight_decay=0.01, capturable=True)

        def gstep():
            gloss = torch.nn.functional.l1_loss(gm(batch).float().view(-1), y)
            gloss.backward()
            gopt.step()
            return gloss

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                gopt.zero_grad(set_to_none=True)
                gstep()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        gr = torch.cuda.CUDAGraph()
        gopt.zero_grad(set_to_none=True)
        with torch.cuda.graph(gr):
            gstep()
        for _ in range(args.warmup):
            gr.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            gr.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) / args.steps * 1e3
    else:
        loss_value = float(loss.detach())
    groups = {"dense attention": ("dense_fwd", "dense_bwd"), "bias builder": ("graph_bias_fwd", "graph_bias_bwd"),
              "projections and ffn linears": ("linear_fwd", "linear_dx", "linear_dw"),
              "layer norm + residual": ("layer_norm_fwd", "layer_norm_bwd"), "gelu": ("gelu",)}
    result = {
        "metric": "training step of the 4-layer graph-level Graphormer on a batch of 256 padded graphs",
        "value": b / (ms * 1e-3), "unit": "graphs/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "configs[3] batch (256 ER graphs n~U[16,128] p=0.1 padded to 128 + virtual node), graph-level "
                               "Graphormer 4 x (hidden 64, ffn 64, 8 heads), ZINC tables, dropout 0", "b": b, "S": s + 1,
                   "parameters": sum(p.numel() for p in m.parameters()),
                   "step": "forward + l1_loss + backward + torch AdamW (" + ("foreach" if args.foreach_adamw else "fused") + ")", "parallelism": "1 GPU"},
        "loss": loss_value,
        "ms_per_step_hip_graph": graph_ms,
        "library_kernel_us_per_step": lib_us,
        "kernel_groups_us": {g: sum(kernels[k]["avg_us"] * kernels[k]["launches_per_step"] for k in ks if k in kernels)
                             for g, ks in groups.items()},
        "kernels": kernels,
    }
    return result


def bench_sparse(args):
    """Sparse attention fwd+bwd of one layer through the C ABI on the graph of args.workload (config1, config2,
    config3, config5): the headline measurement for config2."""
    import torch
    from torchgt_amd import _lib
    from torchgt_amd.plan import GraphPlan
    dev = torch.device("cuda:0")
    H, d = 8, 8
    tdt = torch.float32 if args.dtype == "f32" else torch.bfloat16
    esize = 4 if args.dtype == "f32" else 2
    e, n, label, desc = build_workload(args.workload)
    E = e.shape[1]

    ei = torch.from_numpy(e).to(dev)

    def build_plan():
        # everything a first attention call on a new edge list pays for: sorted views, schedule, wave records
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        p = GraphPlan(ei, n)
        _lib.check(_lib.lib().tgt_plan_prepare(p.handle, H, d, torch.cuda.current_stream(dev).cuda_stream))
        torch.cuda.synchronize()
        return p, (time.perf_counter() - t0) * 1e3

    plan, plan_first_ms = build_plan()
    samples = []
    for _ in range(5):          # later builds find their memory in torch's caching allocator
        p2, ms = build_plan()
        p2.close()
        del p2
        samples.append(ms)
    plan_ms = sorted(samples)[len(samples) // 2]

    g = torch.Generator().manual_seed(42)
    q, k, v = (torch.randn(n, H, d, generator=g).to(dev, tdt) for _ in range(3))
    bias = (torch.randn(E, H, generator=g) * 0.02).to(dev, tdt)
    dout = torch.randn(n, H, d, generator=g).to(dev, tdt)
    out = torch.empty_like(q)
    Z = torch.empty(n, H, dtype=torch.float32, device=dev)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    dbias = torch.empty_like(bias)
    ws = plan.workspace(H, d)
    L = _lib.lib()
    dt_code = _lib.DTYPE_F32 if args.dtype == "f32" else _lib.DTYPE_BF16
    stream = torch.cuda.current_stream(dev).cuda_stream
    P = lambda t: t.data_ptr()

    def step():
        _lib.check(L.tgt_sparse_attn_fwd(plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d,
                                         dt_code, P(out), P(Z), P(ws), ws.numel(), stream))
        _lib.check(L.tgt_sparse_attn_bwd(plan.handle, P(q), P(k), P(v), P(bias), _lib.BIAS_EDGE_HEAD, H, d,
                                         dt_code, P(out), P(Z), P(dout), P(dq), P(dk), P(dv), P(dbias),
                                         P(ws), ws.numel(), stream))

    if args.calibration_copy:
        # reads 256 MiB and writes 256 MiB in one elementwise kernel (name contains "elementwise")
        b = torch.ones(64 << 20, dtype=torch.float32, device=dev)
        a = torch.empty_like(b)
        torch.cuda.synchronize()
        torch.neg(b, out=a)
        torch.cuda.synchronize()
        del a, b
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    sec = time.perf_counter() - t0
    ms_per_step = sec / args.steps * 1e3

    # per-kernel durations: HIP events on the launch stream around every kernel, same K steps
    L.tgt_timing_reset()
    L.tgt_timing_enable(1)
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    L.tgt_timing_enable(0)
    timings = _lib.kernel_timings()
    kernels = {name: {"avg_us": ms / cnt * 1e3, "launches": cnt} for name, (ms, cnt) in timings.items() if cnt}

    # Second datapoint, not the headline: the same step with the bias already in the plan's destination-sorted
    # order (TGT_BIAS_PLAN_ORDER; a bias shared by the layers of a model is permuted once per step), plus what
    # the permutation of the bias and of its gradient costs.
    def plan_order_point():
        order_mode = _lib.BIAS_EDGE_HEAD | _lib.BIAS_PLAN_ORDER | _lib.BIAS_BOTH_ORDERS
        bias2 = torch.empty((2 * E, H), dtype=bias.dtype, device=dev)     # destination-sorted rows, then source-sorted
        dbias2 = torch.empty_like(bias2)

        def permute():
            plan._permute(bias, 0, out=bias2[:E])
            plan._permute(bias, 2, out=bias2[E:])

        permute()

        def ostep():
            _lib.check(L.tgt_sparse_attn_fwd(plan.handle, P(q), P(k), P(v), P(bias2), order_mode, H, d,
                                             dt_code, P(out), P(Z), P(ws), ws.numel(), stream))
            _lib.check(L.tgt_sparse_attn_bwd(plan.handle, P(q), P(k), P(v), P(bias2), order_mode, H, d,
                                             dt_code, P(out), P(Z), P(dout), P(dq), P(dk), P(dv), P(dbias2),
                                             P(ws), ws.numel(), stream))

        n_it = max(5, args.steps // 4)
        for _ in range(3):
            ostep()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_it):
            ostep()
        torch.cuda.synchronize()
        step_us = (time.perf_counter() - t0) / n_it * 1e6
        t0 = time.perf_counter()
        for _ in range(n_it):
            permute()
            plan._permute(dbias2[:E], 1, out=dbias)
        torch.cuda.synchronize()
        perm_us = (time.perf_counter() - t0) / n_it * 1e6
        return {"step_us": step_us, "edges_per_s": E / (step_us * 1e-6),
                "permute_bias_and_gradient_us_once_per_model_step": perm_us,
                "mode": "TGT_BIAS_PLAN_ORDER | TGT_BIAS_BOTH_ORDERS"}

    plan_order = plan_order_point()
    bpe = H * esize
    dom = max((kk for kk in kernels if kernel_alg_bytes(kk, n, E, H, d, esize, bpe)),
              key=lambda kk: kernels[kk]["avg_us"])
    dom_bytes = kernel_alg_bytes(dom, n, E, H, d, esize, bpe)
    dom_gbs = dom_bytes / (kernels[dom]["avg_us"] * 1e-6) / 1e9
    fwd_b, bwd_b = alg_bytes(n, E, H, d, esize, bpe, True)
    step_gbs = (fwd_b + bwd_b) / (ms_per_step * 1e-3) / 1e9

    result = {
        "metric": "fwd+bwd sparse-attn edges/sec at 64K nodes; % HBM roofline; ms/layer",
        "value": E / (ms_per_step * 1e-3),
        "unit": "edges/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": label, "N": n, "E": E, "H": H, "d": d, "bias": "[E,H] with gradient",
                   "max_in_degree": desc["max_in_degree"], "edge_index_sha256": desc["sha256"],
                   "step": "tgt_sparse_attn_fwd + tgt_sparse_attn_bwd (one layer)", "parallelism": "1 GPU, SP=1"},
        "hbm_roofline_frac_step": step_gbs / HBM_PEAK_GBS,
        "alg_bytes_step": fwd_b + bwd_b,
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": dom_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": dom_gbs / HBM_PEAK_GBS,
                     "traffic": MEASURED_TRAFFIC.get((args.workload, args.dtype), {}).get(dom),
                     "traffic_measured_at": MEASURED_TRAFFIC_AT if (args.workload, args.dtype) in MEASURED_TRAFFIC else None,
                     "alg_bytes": dom_bytes,
                     "avg_us": kernels[dom]["avg_us"]},
        "kernels": kernels,
        "bias_in_plan_order": plan_order,
        "plan_build_ms": plan_ms, "plan_build_first_ms": plan_first_ms,
    }
    if E <= 4_000_000 and not args.no_reference_ops:      # the op chain materialises several [E,H,d] fp32 tensors
        result["reference_ops_on_gpu"] = reference_ops_on_gpu(ei, q, k, v, bias, dout)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(e, n, H, d)
    plan.close()
    return result


DISPATCH = {"config4": bench_dense, "config4-bias": bench_graph_bias, "config4-bias-multihop": bench_graph_bias,
            "config4-model": bench_graph_model, "config5-blockized": bench_block, "config5-hybrid": bench_block,
            "config2-mha": bench_mha, "config2-model": bench_model, "config2-gt-model": bench_model}
BF16_BY_DEFAULT = ("config3", "config4", "config4-bias", "config4-bias-multihop", "config4-model", "config5",
                   "config5-blockized", "config5-hybrid")


def run_workload(args):
    fn = DISPATCH.get(args.workload)
    if fn is not None:
        return fn(args)
    if args.workload in ("config3", "config5"):
        args.no_cpu_baseline = True      # the CPU restatement needs minutes per step at this size
    return bench_sparse(args)


def other_configs(args):
    """The other benchmark configurations, each timed by its own workload function inside this run (so that
    they sit under the same clock as the headline): step time, algorithmic bytes, fraction of the 8 TB/s roofline."""
    import copy
    import gc
    import torch
    out = {}
    todo = [("configs[1] bf16", "config2", "bf16", 100, 10), ("configs[2] bf16", "config3", "bf16", 10, 3),
            ("configs[3] bf16 dense", "config4", "bf16", 100, 10), ("configs[4] bf16 sparse path", "config5", "bf16", 50, 5),
            ("configs[4] bf16 hybrid (tiles + remaining edges)", "config5-hybrid", "bf16", 50, 5),
            ("configs[4] bf16 blockized by the reference's reordering", "config5-blockized", "bf16", 50, 5),
            ("configs[1] f32 model step (4-layer Graphormer-Slim)", "config2-model", "f32", 30, 5)]
    for tag, workload, dtype, steps, warmup in todo:
        a = copy.copy(args)
        a.workload, a.dtype, a.steps, a.warmup = workload, dtype, steps, warmup
        a.no_cpu_baseline = a.no_reference_ops = a.brief = True
        a.calibration_copy = False
        t0 = time.perf_counter()
        try:
            r = run_workload(a)
        except Exception as exc:                       # one configuration must not take the headline line down
            out[tag] = {"error": f"{type(exc).__name__}: {exc}"}
            continue
        roof = r.get("roofline", {})
        entry = {"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "value": r["value"], "unit": r["unit"],
                 "steps": steps, "alg_bytes_step": r.get("alg_bytes_step", roof.get("alg_bytes")),
                 "hbm_roofline_frac_step": r.get("hbm_roofline_frac_step"),
                 "roofline": {kk: roof.get(kk) for kk in ("kernel", "frac", "alg_bytes", "avg_us")},
                 "kernels_avg_us": {kk: round(vv["avg_us"], 2) for kk, vv in r.get("kernels", {}).items()},
                 "seconds_spent": None}
        for extra in ("bias_in_plan_order", "mfma", "sparse_path_same_edges_ms", "ids_and_tables", "plan_build_ms",
                      "step_with_fresh_edge_index_ms", "plans_built_by_the_fresh_edge_index_steps",
                      "edge_index_host_to_device_copy_ms", "plan_lookup_by_content_ms"):
            if extra in r:
                entry[extra] = r[extra]
        entry["seconds_spent"] = round(time.perf_counter() - t0, 1)
        out[tag] = entry
        del r
        gc.collect()
        torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--dtype", default="f32", choices=["f32", "bf16"])
    ap.add_argument("--workload", default="config2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-reference-ops", action="store_true",
                    help="skip the datapoint that runs the reference's op chain with stock torch kernels (profiling runs)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="config2 / f32 only: skip the other benchmark configurations (they are timed in the default run)")
    ap.add_argument("--bias-from-ids", action="store_true",
                    help="config4-model: the attention kernels form the bias from ids and tables instead of reading a [b,H,S,S] tensor")
    ap.add_argument("--foreach-adamw", action="store_true",
                    help="model workloads: torch.optim.AdamW's default multi-tensor implementation instead of fused=True "
                         "(the same update from one kernel; the default one issues a dozen launches per step from Python)")
    ap.add_argument("--torch-loss", action="store_true",
                    help="config2-model / config2-gt-model: torch's F.nll_loss instead of the library's kernel")
    ap.add_argument("--hip-graph", action="store_true",
                    help="config2-model: also time the step captured into a HIP graph and replayed")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one 256 MiB device copy (a kernel of known traffic, for scaling rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    args.brief = False
    if args.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU (sequence-parallel size 1); "
                         "--gpus N with N > 1 is not supported")

    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    if args.workload in BF16_BY_DEFAULT and "--dtype" not in sys.argv:
        args.dtype = "bf16"              # the dtype those configurations are quoted on
    headline = args.workload == "config2" and args.dtype == "f32"
    result = run_workload(args)
    if headline and not args.no_other_configs:
        result["other_configs"] = other_configs(args)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
