"""Checks at the full sizes of the named configurations: the whole device outputs of configurations 3, 4 and 5 against
the CPU oracle on the same seeded inputs, and properties that need no CPU run of the whole problem: exact row
counts, linearity, independence of the graphs of a batch (a few graphs recomputed alone by the oracle), determinism."""
import numpy as np
import pytest

from conftest import FLOOR_POOL, FLOOR_PROBS_ABS, PARITY_TOL, Lazy, assert_condition, assert_parity, condition_error, forward_float64, max_rel
from graphnn_amd import batching, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def test_spmm_configuration_3_whole_output_against_the_oracle(gpu, oracle):
    """1,000,000 rows, 10,000,000 entries, width 128; inputs from the SplitMix64 streams of configuration 3 (the matrix
    by synth.erdos_renyi_csr on the host, the dense operand by the torch twin of Stream.normal on the device).  The
    whole device output is compared with the oracle's, and with the float64 product under the condition metric."""
    import torch
    from graphnn_amd import ops
    n, nnz, d = 1_000_000, 10_000_000, 128
    seed = synth.config_seed(3)
    rp, ci, v = synth.erdos_renyi_csr(seed, n, nnz)
    rp_d, ci_d, v_d = _t(rp, gpu), _t(ci, gpu), _t(v, gpu)
    x_seed = synth.Stream(seed).child(2).seed
    X = synth.torch_normal_f32(x_seed, n * d, gpu).view(n, d)
    Xh = X.cpu().numpy()
    # the device-made operand is the numpy stream's: a prefix, element by element (equal or the neighbouring float32)
    head = synth.Stream(x_seed).normal(1 << 16)
    assert np.all(np.abs(Xh.ravel()[:1 << 16] - head) <= np.spacing(np.abs(head))) and np.mean(Xh.ravel()[:1 << 16] == head) > 0.99
    ax = ops.spmm(rp_d, ci_d, v_d, X, n)
    got = ax.cpu().numpy()
    want = oracle.spmm(rp, ci, v, Xh, n)
    model = Lazy(lambda: oracle.spmm_f64(rp, ci, v, Xh, n), Lazy(lambda: oracle.spmm_f64(rp, ci, v, Xh, n, absolute=True)))
    assert_parity("spmm configuration 3", got, want, model)
    # unit weights, rows of at most a few dozen entries added front to back on both sides: the same additions in the
    # same order, so the whole output has the oracle's bits
    assert np.array_equal(got, want)
    del got, want, model
    # A * ones = row lengths, exactly (unit weights: every partial sum is a small integer)
    deg = ops.spmm(rp_d, ci_d, v_d, torch.ones((n, d), device=gpu), n)
    assert torch.equal(deg[:, 0], _t(np.diff(rp).astype(np.float32), gpu)) and torch.equal(deg[:, 0], deg[:, d - 1])
    # linearity: A (2X - 3Y) = 2 AX - 3 AY up to fp32 rounding of sums of ~10 terms
    Y = synth.torch_uniform_f32(synth.Stream(seed).child(3).seed, n * d, gpu, -1.0, 1.0).view(n, d)
    ay = ops.spmm(rp_d, ci_d, v_d, Y, n)
    az = ops.spmm(rp_d, ci_d, v_d, 2 * X - 3 * Y, n)
    ref = 2 * ax - 3 * ay
    assert float((az - ref).abs().max()) <= 1e-4 * float(ref.abs().max())
    # same bits on a second run
    assert torch.equal(ax, ops.spmm(rp_d, ci_d, v_d, X, n))


def test_spmm_configuration_3_regular_variant(gpu, oracle):
    """the other reading of "uniform degree": exactly 10 entries in every row; whole output against the oracle,
    bit for bit (unit weights, rows added front to back on both sides)"""
    from graphnn_amd import ops
    n, nnz, d = 1_000_000, 10_000_000, 128
    seed = synth.config_seed(3)
    rp, ci, v = synth.erdos_renyi_csr(seed, n, nnz, regular=True)
    X = synth.torch_uniform_f32(synth.Stream(seed).child(3).seed, n * d, gpu, -1.0, 1.0).view(n, d)
    Xh = X.cpu().numpy()
    got = ops.spmm(_t(rp, gpu), _t(ci, gpu), _t(v, gpu), X, n).cpu().numpy()
    want = oracle.spmm(rp, ci, v, Xh, n)
    assert_parity("spmm configuration 3, 10 per row", got, want,
                  Lazy(lambda: oracle.spmm_f64(rp, ci, v, Xh, n), Lazy(lambda: oracle.spmm_f64(rp, ci, v, Xh, n, absolute=True))))
    assert np.array_equal(got, want)


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


def test_forward_configuration_4_whole_outputs_against_the_oracle(gpu, oracle):
    """10,000 graphs, 299,536 nodes, hidden 256, 5 levels (the FP32 matrix-core level kernel, the tile readout): every
    output of the whole batch against the CPU oracle's forward on the same seeded inputs (about ten seconds of CPU), with
    the float64 model of the network behind it where two fp32 orders disagree, and its condition bound on every element"""
    from graphnn_amd import ops
    batch, w, cfg = synth.make_config(4)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    X = batch.one_hot()
    L = cfg["L"]
    bufs = ops.s2v_forward(tuple(_t(x, gpu) for x in a), tuple(_t(x, gpu) for x in s), _t(X, gpu), _t(w.W_n2l, gpu),
                           _t(w.W_conv, gpu), _t(w.W_h1, gpu), _t(w.W_h2, gpu), L)
    got = {"msg": bufs.msg, "h_final": bufs.h_b if bufs.which.value else bufs.h_a, "pool": bufs.pool, "hidden": bufs.hidden,
           "logits": bufs.logits, "probs": bufs.probs}
    got = {k: v.cpu().numpy() for k, v in got.items()}
    pred = bufs.pred.cpu().numpy()
    want = oracle.forward(a, s, X, w, L, None)
    f64 = Lazy(lambda: forward_float64(a, s, X, w, L), Lazy(lambda: forward_float64(a, s, X, w, L, magnitudes=True)))
    for key in ("msg", "h_final", "pool", "hidden", "logits", "probs"):
        ref = want["h"][L] if key == "h_final" else want[key]
        ref64 = f64["h"][L] if key == "h_final" else f64[key]
        kw = {"floor_frac": FLOOR_POOL} if key == "pool" else {"floor": FLOOR_PROBS_ABS} if key == "probs" else {}
        assert_parity("%s configuration 4" % key, got[key], ref, ref64, **kw)
    # predictions: identical wherever the two logits are not a near tie
    margin = np.abs(want["logits"][:, 0] - want["logits"][:, 1])
    clear = margin > 1e-3 * np.abs(want["logits"]).max()
    assert clear.mean() > 0.9
    assert np.array_equal(pred[clear], want["pred"][clear])


def test_skewed_configuration_5_whole_outputs_against_the_oracle(gpu, oracle):
    """R-MAT scale 22 (4,194,304 rows, 67,108,864 entries, a = 0.57, b = c = 0.19) from the SplitMix64 streams of
    configuration 5, generated on the device by the torch twin of synth.rmat_csr (bit-identical: a window of the edge
    list is compared with the host generator here, the whole matrix at a small scale in the CPU tests); hidden 64.
    The SpMM, one level, the jagged softmax over 4,096 segments of 1,024 and the sum-pool are each compared, whole
    output, with the oracle on the same inputs copied to the host; rows of more than 256 entries, which the reference
    path adds serially and therefore less accurately than the device does, are held to the float64 result instead."""
    import torch
    from graphnn_amd import ops
    scale, C = 22, 64
    N, E = 1 << scale, 16 << scale
    seed = synth.config_seed(5)
    root = synth.Stream(seed)
    rows_d, cols_d = synth.rmat_edges_torch(seed, scale, E, gpu, lo=E - 70_000, hi=E)
    rows_h, cols_h = synth.rmat_edges_torch(seed, scale, E, "cpu", lo=E - 70_000, hi=E)
    assert torch.equal(rows_d.cpu(), rows_h) and torch.equal(cols_d.cpu(), cols_h)
    del rows_d, cols_d
    rp, ci, val = synth.rmat_csr_torch(seed, scale, E, gpu)
    rp_h, ci_h, val_h = rp.cpu().numpy(), ci.cpu().numpy(), val.cpu().numpy()
    lens = np.diff(rp_h)
    assert rp_h[-1] == E and lens.max() > 50_000                     # the hub rows this configuration is about
    print("configuration 5: longest row %d, %d rows over 256 entries, %d empty rows" % (lens.max(), (lens > 256).sum(), (lens == 0).sum()))

    # row lengths, exactly, through the balanced pass over long rows (sums up to 160,000 < 2^24)
    deg = ops.spmm(rp, ci, val, torch.ones((N, 4), device=gpu), N)
    assert np.array_equal(deg[:, 0].cpu().numpy(), lens.astype(np.float32))
    del deg

    h = synth.torch_uniform_f32(root.child(30).seed, N * C, gpu).view(N, C)          # non-negative, as embeddings are
    hh = h.cpu().numpy()
    agg = ops.spmm(rp, ci, val, h, N)
    assert torch.equal(agg, ops.spmm(rp, ci, val, h, N))             # deterministic
    got = agg.cpu().numpy()
    want = oracle.spmm(rp_h, ci_h, val_h, hh, N)
    agg64 = oracle.spmm_f64(rp_h, ci_h, val_h, hh, N)                # all terms non-negative: its own condition tensor
    short = lens <= 256
    assert_condition("spmm configuration 5, all rows", got, agg64, agg64)
    assert_parity("spmm configuration 5, rows of up to 256 entries", got[short], want[short], Lazy(lambda: agg64[short]))
    worst_ref, _ = condition_error(want, agg64, agg64)
    print("configuration 5: the serial fp32 sums of the reference path are %.2e of a row's terms from float64 at worst" % worst_ref)
    del want, got

    # one level = ReLU((A h) W + msg)
    W = root.child(101).normal(C * C, 0.1).reshape(C, C)
    msg = synth.torch_uniform_f32(root.child(31).seed, N * C, gpu, -1.0, 1.0).view(N, C)
    mh = msg.cpu().numpy()
    out = ops.s2v_level(rp, ci, val, h, _t(W, gpu), msg)
    got = out.cpu().numpy()
    want = oracle.level(rp_h, ci_h, val_h, hh, W, mh)
    z64 = agg64 @ W.astype(np.float64)
    z64 += mh
    np.maximum(z64, 0, out=z64)
    cond = agg64 @ np.abs(W.astype(np.float64))
    cond += np.abs(mh)
    assert_condition("level configuration 5, all rows", got, z64, cond)
    assert_parity("level configuration 5, rows of up to 256 entries", got[short], want[short], Lazy(lambda: z64[short]))
    del want, z64, cond, agg64, mh, hh

    # jagged softmax over 4096 segments of 1024 scores, and the sum-pool of the same segments
    B = N // 1024
    score = synth.torch_uniform_f32(root.child(32).seed, N, gpu, -6.0, 6.0).view(N, 1)
    seg = np.full(B, 1024, np.int32)
    want_soft = oracle.jagged_softmax(score.cpu().numpy(), seg)
    soft = ops.jagged_softmax(score.clone(), _t(seg, gpu)).cpu().numpy()
    assert_parity("jagged softmax configuration 5", soft, want_soft, floor=FLOOR_PROBS_ABS)
    assert np.abs(soft.reshape(B, 1024).astype(np.float64).sum(axis=1) - 1).max() < 1e-5
    s_csr = synth.contiguous_subgraph_csr(N, B)
    pool = ops.spmm(*(_t(x, gpu) for x in s_csr), out, B).cpu().numpy()
    want_pool = oracle.spmm(*s_csr, got, B)
    pool64 = Lazy(lambda: oracle.spmm_f64(*s_csr, got, B), Lazy(lambda: oracle.spmm_f64(*s_csr, got, B, absolute=True)))
    assert_parity("pool configuration 5", pool, want_pool, pool64, floor_frac=FLOOR_POOL)


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
