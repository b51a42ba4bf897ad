#!/usr/bin/env python3
"""Benchmark of the structure2vec mean-field forward on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-spmm]

A step is one forward (input + L levels + readout) over one synthetic batch of
configuration 2 (256 graphs, hidden 64, 4 levels) with every input already
resident in HBM.  Prints ONE JSON line: graphs/s as `value`, plus
  roofline      the CSR SpMM kernel on configuration 3 (1M rows, 10M entries,
                width 128): algorithmic bytes / HIP-event time vs 8 TB/s
  cpu_baseline  the CPU restatement (oracle/) timed on this host's cores
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, published

# HBM bytes per launch of the SpMM kernel on configuration 3, from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs scaled by a copy kernel of known size (factors 2.000 and 1.000).
MEASURED_TRAFFIC_BYTES = {"spmm_cfg3": 5_679_000_000}


def spmm_algorithmic_bytes(m, k, nnz, d):
    return 4 * (m + 1) + 8 * nnz + 4 * k * d + 4 * m * d


def level_algorithmic_bytes(N, E, C):
    return 4 * (N + 1) + 8 * E + 12 * N * C + 4 * C * C


def build_forward_workload(dev):
    import torch
    from graphnn_amd import batching, synth
    batch, w, cfg = synth.make_config(2)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    X = batch.one_hot()
    t = lambda arr: torch.from_numpy(np.ascontiguousarray(arr)).to(dev)
    dev_args = (tuple(map(t, a)), tuple(map(t, s)), t(X), t(w.W_n2l), t(w.W_conv), t(w.W_h1), t(w.W_h2))
    host = dict(batch=batch, w=w, cfg=cfg, a=a, s=s, X=X)
    return dev_args, host


def time_forward(dev_args, cfg, batch, steps, warmup, route):
    """Wall-clock seconds per forward.  route = "graph_resident" (one launch, embeddings in LDS; valid
    because the batch is block diagonal, as GetBatch builds it) or "general" (input + L levels + readout
    launches that accept any CSR)."""
    import torch
    from graphnn_amd import ops
    N, B = batch.num_nodes, batch.num_graphs
    dev = dev_args[2].device
    if route == "graph_resident":
        bufs = ops.BatchedBuffers(N, B, cfg["C"], cfg["H"], cfg["Q"], dev)
        nmax = int(batch.graph_sizes.max())
        run = lambda: ops.s2v_forward_batched(*dev_args, cfg["L"], nmax, bufs=bufs)
    else:
        bufs = ops.ForwardBuffers(N, B, cfg["C"], cfg["H"], cfg["Q"], dev)
        run = lambda: ops.s2v_forward(*dev_args, cfg["L"], bufs=bufs)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    if route == "graph_resident":
        assert int(bufs.status.cpu()[0]) == 0, "graph-resident forward reported a layout violation"
    return (t1 - t0) / steps, bufs


def time_spmm_cfg3(dev, reps=20, warmup=3):
    """HIP-event time of the SpMM kernel alone on configuration 3."""
    import torch
    from graphnn_amd import ops, synth
    n, nnz, d = 1_000_000, 10_000_000, 128
    rp, ci, v = synth.erdos_renyi_csr(synth.config_seed(3), n, nnz)
    t = lambda arr: torch.from_numpy(np.ascontiguousarray(arr)).to(dev)
    rp_d, ci_d, v_d = t(rp), t(ci), t(v)
    gen = torch.Generator(device=dev)
    gen.manual_seed(synth.config_seed(3))
    X = torch.randn((n, d), generator=gen, device=dev, dtype=torch.float32)
    Y = torch.empty((n, d), device=dev, dtype=torch.float32)
    for _ in range(warmup):
        ops.spmm(rp_d, ci_d, v_d, X, n, out=Y)
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for e0, e1 in evs:
        e0.record()
        ops.spmm(rp_d, ci_d, v_d, X, n, out=Y)
        e1.record()
    torch.cuda.synchronize()
    ms = np.array([e0.elapsed_time(e1) for e0, e1 in evs])
    # property check at full size: A * ones = row lengths, exactly
    ones = torch.ones((n, 4), device=dev, dtype=torch.float32)
    deg = ops.spmm(rp_d, ci_d, v_d, ones, n)
    torch.cuda.synchronize()
    assert np.array_equal(deg[:, 0].cpu().numpy(), np.diff(rp).astype(np.float32)), "SpMM row-length check failed"
    return float(ms.mean()), float(ms.min()), spmm_algorithmic_bytes(n, n, nnz, d), (n, nnz, d)


def cpu_baseline(host, budget_s=12.0):
    """The CPU restatement of the reference path on the same batch, timed on this host."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from conftest import Oracle
    orc = Oracle()
    threads = int(orc.lib.orc_num_threads())
    batch, cfg = host["batch"], host["cfg"]
    orc.forward(host["a"], host["s"], host["X"], host["w"], cfg["L"], None)      # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        orc.forward(host["a"], host["s"], host["X"], host["w"], cfg["L"], None)
        reps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or reps >= 100000:
            break
    return dict(value=batch.num_graphs * reps / el, unit="graphs/s", cores=threads, kind="port",
                sample="%d forwards of the same configuration-2 batch in %.1f s (gcc -O3 -mavx2, OpenMP over rows)" % (reps, el))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-spmm", action="store_true", help="skip the configuration-3 SpMM roofline leg")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one element-wise copy kernel of known size (1 GiB read, 1 GiB written) "
                         "so hardware counters collected over this run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a HIP device")
    from graphnn_amd import ops
    ops.init(0)
    dev = torch.device("cuda:0")

    dev_args, host = build_forward_workload(dev)
    batch, cfg = host["batch"], host["cfg"]
    sec_general, bufs_general = time_forward(dev_args, cfg, batch, args.steps, args.warmup, "general")
    sec, bufs = time_forward(dev_args, cfg, batch, args.steps, args.warmup, "graph_resident")
    # the two routes must agree on what they computed
    assert bool((bufs.pred == bufs_general.pred).all()), "routes disagree on predictions"
    assert float((bufs.logits - bufs_general.logits).abs().max()) <= 1e-4 * float(bufs_general.logits.abs().max()), \
        "routes disagree on logits"

    out = {
        "metric": "s2v forward graphs/sec (B=256,h=64,L=4); SpMM achieved HBM GB/s vs peak",
        "value": batch.num_graphs / sec,
        "unit": "graphs/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": sec * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "s2v mean-field forward, configuration 2: 256 graphs, %d nodes, %d directed edges, "
                               "38 label types, hidden 64, 4 levels, MLP 64-32-2, softmax + argmax"
                               % (batch.num_nodes, batch.num_edges),
                   "graphs": batch.num_graphs, "nodes": batch.num_nodes, "edges": batch.num_edges},
        "nodes_per_s": batch.num_nodes / sec,
        "route": "graph-resident forward, one launch (gnnhip_s2v_forward_batched_f32)",
        "general_route": {"graphs_per_s": batch.num_graphs / sec_general, "ms_per_step": sec_general * 1e3,
                          "what": "gnnhip_s2v_forward_f32: input + 4 fused levels + readout, any CSR"},
    }

    if not args.no_spmm:
        mean_ms, min_ms, bytes_alg, (n, nnz, d) = time_spmm_cfg3(dev)
        achieved = bytes_alg / (mean_ms * 1e-3) / 1e9
        out["roofline"] = {
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES["spmm_cfg3"],
            "kernel": "spmm_rowgroup_kernel<4,1>",
            "workload": "configuration 3: CSR SpMM, %d rows, %d entries, width %d" % (n, nnz, d),
            "algorithmic_bytes": bytes_alg, "avg_ms": mean_ms, "min_ms": min_ms,
        }
    else:
        out["roofline"] = None

    if args.calibrate:
        n = 1 << 28
        src = torch.ones(n, device=dev, dtype=torch.float32)
        dst = torch.empty_like(src)
        ops.relu(src, dst)              # map1_kernel<FReLU>: reads 4n bytes, writes 4n bytes
        torch.cuda.synchronize()
        out["calibration"] = {"kernel": "map1_kernel<FReLU>", "bytes_read": 4 * n, "bytes_written": 4 * n}

    out["cpu_baseline"] = None if args.no_cpu else cpu_baseline(host)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
