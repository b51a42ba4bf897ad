"""Checks at the full sizes of the named configurations, through properties that do not need a CPU
run of the whole problem: exact row counts, linearity, independence of the graphs of a batch (a few
graphs recomputed alone by the CPU oracle), segment sums, determinism."""
import numpy as np
import pytest

from conftest import PARITY_TOL, max_rel
from graphnn_amd import batching, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def test_spmm_configuration_3_properties(gpu):
    """1,000,000 rows, 10,000,000 entries, width 128"""
    import torch
    from graphnn_amd import ops
    n, nnz, d = 1_000_000, 10_000_000, 128
    rp, ci, v = synth.erdos_renyi_csr(synth.config_seed(3), n, nnz)
    rp_d, ci_d, v_d = _t(rp, gpu), _t(ci, gpu), _t(v, gpu)
    g = torch.Generator(device=gpu); g.manual_seed(3)
    X = torch.randn((n, d), generator=g, device=gpu)
    Y = torch.randn((n, d), generator=g, device=gpu)
    # A * ones = row lengths, exactly (unit weights: every partial sum is a small integer)
    deg = ops.spmm(rp_d, ci_d, v_d, torch.ones((n, d), device=gpu), n)
    assert torch.equal(deg[:, 0], _t(np.diff(rp).astype(np.float32), gpu)) and torch.equal(deg[:, 0], deg[:, d - 1])
    # linearity: A (2X - 3Y) = 2 AX - 3 AY up to fp32 rounding of sums of ~10 terms
    ax, ay = ops.spmm(rp_d, ci_d, v_d, X, n), ops.spmm(rp_d, ci_d, v_d, Y, n)
    az = ops.spmm(rp_d, ci_d, v_d, 2 * X - 3 * Y, n)
    ref = 2 * ax - 3 * ay
    assert float((az - ref).abs().max()) <= 1e-4 * float(ref.abs().max())
    # against a float64 gather-sum on a sample of rows
    rows = torch.randint(0, n, (2000,), device=gpu, generator=g)
    for r in rows[:200].tolist():
        cols = ci_d[rp[r]:rp[r + 1]].long()
        want = X[cols].double().sum(dim=0)
        assert float((ax[r].double() - want).abs().max()) <= 1e-5 * max(1.0, float(want.abs().max()))
    # same bits on a second run
    assert torch.equal(ax, ops.spmm(rp_d, ci_d, v_d, X, n))


def test_forward_configuration_4_sampled_graphs(gpu, oracle):
    """10,000 graphs, hidden 256, 5 levels: the graphs of a batch do not interact, so a graph recomputed
    alone by the CPU oracle must give the logits the full batch gave it"""
    from graphnn_amd import ops
    batch, w, cfg = synth.make_config(4)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    X = batch.one_hot()
    bufs = ops.s2v_forward(tuple(_t(x, gpu) for x in a), tuple(_t(x, gpu) for x in s), _t(X, gpu), _t(w.W_n2l, gpu),
                           _t(w.W_conv, gpu), _t(w.W_h1, gpu), _t(w.W_h2, gpu), cfg["L"])
    logits = bufs.logits.cpu().numpy()
    pred = bufs.pred.cpu().numpy()
    h_final = (bufs.h_b if bufs.which.value else bufs.h_a).cpu().numpy()
    offs = np.concatenate([[0], np.cumsum(batch.graph_sizes)])
    scale = np.abs(logits).max()
    for gidx in (0, 1, 4999, 7777, batch.num_graphs - 1):
        lo, hi = int(offs[gidx]), int(offs[gidx + 1])
        n = hi - lo
        sel = (batch.edge_x >= lo) & (batch.edge_x < hi)
        assert np.all((batch.edge_y[sel] >= lo) & (batch.edge_y[sel] < hi))
        a1 = batching.node2node_csr(n, batch.edge_x[sel] - lo, batch.edge_y[sel] - lo)
        s1 = batching.subgraph_csr(1, np.zeros(n, np.int32), np.arange(n, dtype=np.int32))
        ref = oracle.forward(a1, s1, X[lo:hi], w, cfg["L"], None)
        assert max_rel(h_final[lo:hi], ref["h"][cfg["L"]]) < PARITY_TOL
        assert np.abs(logits[gidx] - ref["logits"][0]).max() <= PARITY_TOL * scale
        margin = abs(float(ref["logits"][0][0] - ref["logits"][0][1]))
        if margin > 1e-3 * scale:
            assert pred[gidx] == ref["pred"][0]


def test_skewed_configuration_5_properties(gpu):
    """R-MAT scale 22 (4,194,304 rows, 67,108,864 entries) generated on the device; hidden 64"""
    import torch
    from graphnn_amd import ops
    scale, C = 22, 64
    N, E = 1 << scale, 16 << scale
    g = torch.Generator(device=gpu); g.manual_seed(55)
    rows = torch.zeros(E, dtype=torch.int64, device=gpu)
    cols = torch.zeros(E, dtype=torch.int64, device=gpu)
    for _ in range(scale):
        u = torch.rand(E, device=gpu, generator=g)
        rows = (rows << 1) | (u >= 0.76).long()
        cols = (cols << 1) | (((u >= 0.57) & (u < 0.76)) | (u >= 0.95)).long()
        del u
    key, _ = torch.sort(rows * N + cols)
    del rows, cols
    r = key // N
    ci = (key - r * N).int()
    cnt = torch.bincount(r, minlength=N)
    del key, r
    rp = torch.zeros(N + 1, dtype=torch.int32, device=gpu)
    rp[1:] = torch.cumsum(cnt, 0).int()
    val = torch.ones(E, dtype=torch.float32, device=gpu)
    assert int(cnt.max()) > 50_000                                   # the hub rows this configuration is about

    # row lengths, exactly, through the balanced pass over long rows (sums up to 160,000 < 2^24)
    deg = ops.spmm(rp, ci, val, torch.ones((N, 4), device=gpu), N)
    assert torch.equal(deg[:, 0], cnt.float())

    h = torch.rand((N, C), device=gpu, generator=g)
    agg = ops.spmm(rp, ci, val, h, N)
    assert torch.equal(agg, ops.spmm(rp, ci, val, h, N))             # deterministic
    # the three longest rows and 300 others against a float64 gather-sum
    top = torch.topk(cnt, 3).indices
    sample = torch.cat([top, torch.randint(0, N, (300,), device=gpu, generator=g)])
    for row in sample.tolist():
        lo, hi = int(rp[row]), int(rp[row + 1])
        want = h[ci[lo:hi].long()].double().sum(dim=0)
        assert float((agg[row].double() - want).abs().max()) <= 2e-5 * max(1.0, float(want.abs().max()))

    # one level = ReLU(agg W + msg): the device's own SpMM result through a float64 contraction
    W = torch.randn((C, C), device=gpu, generator=g) * 0.1
    msg = torch.randn((N, C), device=gpu, generator=g)
    out = ops.s2v_level(rp, ci, val, h, W, msg)
    idx = sample.long()
    want = torch.relu(agg[idx].double() @ W.double() + msg[idx].double())
    floor = 0.01 * float(want.abs().max())
    rel = (out[idx].double() - want).abs() / torch.clamp(torch.maximum(out[idx].double().abs(), want.abs()), min=floor)
    assert float(rel.max()) < PARITY_TOL

    # jagged softmax over 4096 segments of 1024 scores, and the sum-pool of the same segments
    B = N // 1024
    score = torch.randn((N, 1), device=gpu, generator=g) * 3
    lens = torch.full((B,), 1024, dtype=torch.int32, device=gpu)
    soft = ops.jagged_softmax(score.clone(), lens).view(B, 1024)
    want_soft = torch.softmax(score.view(B, 1024).double(), dim=1)
    assert float((soft.double() - want_soft).abs().max()) < 1e-6
    assert float((soft.double().sum(dim=1) - 1).abs().max()) < 1e-5
    s_rp = (torch.arange(B + 1, device=gpu) * 1024).int()
    pool = ops.spmm(s_rp, torch.arange(N, device=gpu).int(), torch.ones(N, device=gpu), out, B)
    want_pool = out.view(B, 1024, C).double().sum(dim=1)
    assert float((pool.double() - want_pool).abs().max()) <= 1e-4 * float(want_pool.abs().max())


def test_level_past_4_gib_of_activations(gpu):
    """16.8M nodes at hidden 64: each of h_in, msg and h_out spans 4 GiB, past the reach of the 32-bit buffer
    offsets of the streaming level kernel, so the kernel with 64-bit addressing runs.  Ring graph with
    weights (every node sums its two neighbours); sampled rows against float64, the rows at both ends of
    the address range included."""
    import torch
    from graphnn_amd import ops
    n, c = (1 << 24) + 48, 64
    assert n * c * 4 >= 0xFFFF0000
    idx = torch.arange(n, device=gpu, dtype=torch.int64)
    ci = torch.stack(((idx - 1) % n, (idx + 1) % n), dim=1).to(torch.int32).reshape(-1).contiguous()
    rp = (2 * torch.arange(n + 1, device=gpu, dtype=torch.int64)).to(torch.int32)
    g = torch.Generator(device=gpu); g.manual_seed(24)
    val = torch.rand((2 * n,), generator=g, device=gpu) + 0.5
    h = torch.rand((n, c), generator=g, device=gpu)
    msg = torch.randn((n, c), generator=g, device=gpu)
    W = torch.randn((c, c), generator=g, device=gpu) * 0.1
    out = ops.s2v_level(rp, ci, val, h, W, msg)
    rows = torch.cat((torch.arange(0, 40, device=gpu), torch.arange(n - 40, n, device=gpu),
                      torch.randint(0, n, (2000,), device=gpu, generator=g)))
    left, right = (rows - 1) % n, (rows + 1) % n
    agg = val[2 * rows].double()[:, None] * h[left].double() + val[2 * rows + 1].double()[:, None] * h[right].double()
    want = torch.relu(agg @ W.double() + msg[rows].double())
    got = out[rows].double()
    assert float((got - want).abs().max()) <= PARITY_TOL * max(1.0, float(want.abs().max()))


def test_spmm_long_rows_past_4m_rows(gpu):
    """4.3M rows: the planning of the balanced pass over long rows takes its three-launch form (count, scan,
    fill) past 4,096 row blocks.  One entry per row plus long rows in the first, a middle and the last block;
    the long rows and sampled short ones against float64."""
    import torch
    from graphnn_amd import ops
    m, k, n = 4_300_007, 50_000, 16
    g = torch.Generator(device=gpu); g.manual_seed(43)
    lens = torch.ones(m, dtype=torch.int64, device=gpu)
    hubs = {5: 70, 2_222_222: 5_000, m - 1: 3_001, m - 2050: 65}
    for r, l in hubs.items():
        lens[r] = l
    rp = torch.zeros(m + 1, dtype=torch.int64, device=gpu)
    rp[1:] = torch.cumsum(lens, 0)
    nnz = int(rp[-1].item())
    ci = torch.randint(0, k, (nnz,), device=gpu, generator=g, dtype=torch.int64).to(torch.int32)
    val = torch.rand((nnz,), generator=g, device=gpu) - 0.5
    X = torch.randn((k, n), generator=g, device=gpu)
    Y = ops.spmm(rp.to(torch.int32), ci, val, X, m)
    rows = torch.cat((torch.tensor(sorted(hubs), device=gpu), torch.randint(0, m, (3000,), device=gpu, generator=g)))
    for r in rows.tolist():
        a, b = int(rp[r].item()), int(rp[r + 1].item())
        want = (val[a:b].double()[:, None] * X[ci[a:b].long()].double()).sum(0)
        got = Y[r].double()
        assert float((got - want).abs().max()) <= PARITY_TOL * max(1.0, float(want.abs().max())), r
