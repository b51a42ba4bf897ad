"""The kernels that carry one training iteration of the structure2vec path (loss/accuracy tail, readout
backward, gradient gate, batched momentum-SGD update) against the oracle, and the whole iteration composed
from C-ABI calls the way the host layer's fused training plan composes it, against float64 autograd."""
import numpy as np
import pytest

from conftest import PARITY_TOL, assert_parity, max_rel
from graphnn_amd import batching, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _n(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("B,Q", [(256, 2), (1, 3), (5000, 7), (1025, 2), (300, 70)])
def test_loss_and_accuracy_tail(gpu, oracle, B, Q):
    from graphnn_amd import ops
    rng = np.random.default_rng(B + Q)
    logits = (rng.standard_normal((B, Q)) * 3).astype(np.float32)
    logits[::7] = np.round(logits[::7])                            # ties between logits
    if B > 10:
        logits[3] = [200.0] + [-200.0] * (Q - 1)                   # a probability that underflows: the 1e-8 clamp
    y = rng.integers(0, Q, B).astype(np.int32)
    if B > 10:
        y[3] = Q - 1
    lab = (np.arange(B + 1, dtype=np.int32), y, np.ones(B, np.float32))
    loss, acc, probs, loss_rows, hit = ops.loss_acc(_t(logits, gpu), *[_t(a, gpu) for a in lab], want_rows=True)
    w_probs = oracle.row_softmax(logits)
    w_rows = oracle.cross_entropy(w_probs, *lab)
    w_hit = oracle.in_top_k(logits, oracle.csr_row_argmax(*lab), 1)
    assert max_rel(_n(probs), w_probs, floor=1e-6) < PARITY_TOL
    assert np.allclose(_n(loss_rows), w_rows, rtol=1e-4, atol=1e-6)
    assert np.array_equal(_n(hit), w_hit)
    assert abs(float(_n(loss)[0]) - oracle.mean(w_rows)) <= 1e-4 * abs(oracle.mean(w_rows))
    assert abs(float(_n(acc)[0]) - oracle.mean(oracle.cast(w_hit))) <= 1e-6


def test_loss_tail_with_weighted_and_empty_label_rows(gpu, oracle):
    from graphnn_amd import ops
    rng = np.random.default_rng(9)
    B, Q = 40, 5
    logits = rng.standard_normal((B, Q)).astype(np.float32)
    lens = rng.integers(0, 4, B); lens[0] = 0
    rp = np.zeros(B + 1, np.int32); np.cumsum(lens, out=rp[1:])
    ci = rng.integers(0, Q, rp[-1]).astype(np.int32)
    v = rng.random(rp[-1]).astype(np.float32)
    lab = (rp, ci, v)
    loss, acc, probs, loss_rows, hit = ops.loss_acc(_t(logits, gpu), *[_t(a, gpu) for a in lab], want_rows=True)
    w_probs = oracle.row_softmax(logits)
    assert np.allclose(_n(loss_rows), oracle.cross_entropy(w_probs, *lab), rtol=1e-4, atol=1e-6)
    assert np.array_equal(_n(hit), oracle.in_top_k(logits, oracle.csr_row_argmax(*lab), 1))


@pytest.mark.parametrize("C,H,Q,B", [(64, 32, 2, 256), (16, 8, 3, 5), (256, 128, 2, 700), (48, 100, 70, 33),
                                     # from 1,024 graphs: du W_h1^T as one product over all graphs, node rows by a kernel of their own
                                     (256, 128, 2, 1024), (64, 32, 2, 3000), (130, 20, 3, 1100), (600, 16, 2, 1030)])
def test_readout_backward(gpu, oracle, C, H, Q, B):
    from graphnn_amd import ops
    rng = np.random.default_rng(C + H + B)
    batch = synth.molecule_batch(C + B, B, 5, Q, size_mode="uniform", size_lo=1, size_hi=40)
    N = batch.num_nodes
    s = batching.subgraph_csr(B, batch.subg_id, batch.node_idx)
    s = (s[0], s[1], (0.5 + rng.random(N)).astype(np.float32))
    lab = batch.label_csr()
    probs = oracle.row_softmax(rng.standard_normal((B, Q)).astype(np.float32))
    hidden = np.maximum(rng.standard_normal((B, H)), 0).astype(np.float32)
    W1 = (rng.standard_normal((C, H)) * 0.2).astype(np.float32)
    W2 = (rng.standard_normal((H, Q)) * 0.2).astype(np.float32)
    scale = 1.0 / B
    dl, du, gh = ops.readout_backward([_t(a, gpu) for a in s], _t(probs, gpu), [_t(a, gpu) for a in lab], scale,
                                      _t(hidden, gpu), _t(W1, gpu), _t(W2, gpu), N)
    Y = np.zeros((B, Q), np.float32); Y[np.arange(B), batch.graph_label] = 1.0
    w_dl = ((probs - Y) * np.float32(scale)).astype(np.float32)
    w_du = (oracle.gemm(w_dl, W2, transB=True) * (hidden > 0)).astype(np.float32)
    w_dpool = oracle.gemm(w_du, W1, transB=True)
    w_gh = oracle.spmm_T(*s, w_dpool, B, N)
    assert np.array_equal(_n(dl), w_dl)
    f8 = np.float64
    du64 = (w_dl.astype(f8) @ W2.astype(f8).T) * (hidden > 0)
    assert_parity("du", _n(du), w_du, du64)
    gh64 = np.repeat(du64 @ W1.astype(f8).T, batch.graph_sizes, axis=0) * s[2][:, None].astype(f8)
    assert_parity("g_h", _n(gh), w_gh, gh64)


@pytest.mark.parametrize("N,C", [(N, C) for C in (16, 32, 64, 128, 256) for N in (77, 7450, 40_000)] + [(70_001, 128), (70_001, 256), (16_400, 256)])
def test_level_backward(gpu, oracle, C, N):
    """u = A^T dz and g_prev = u W^T in one pass (hidden 16/32/64: the streaming kernel; hidden 128/256: the wide kernel's
    backward variant in passes of 16, 32 and 64 rows, which the row counts select): ragged rows, two long rows (the larger
    matrices send them through the balanced pass at the narrow sizes), signed dz"""
    from graphnn_amd import ops
    rng = np.random.default_rng(C + N)
    lens = rng.integers(0, 7, N); lens[N // 3] = min(N, 3000); lens[N - 1] = 70
    rp = np.zeros(N + 1, np.int32); np.cumsum(lens, out=rp[1:])
    nnz = int(rp[-1])
    ci = rng.integers(0, N, nnz).astype(np.int32)
    v = (rng.random(nnz) * 0.5).astype(np.float32)
    dz = (rng.standard_normal((N, C)) * (rng.random((N, C)) < 0.5)).astype(np.float32)      # about half the gates closed
    W = (rng.standard_normal((C, C)) * 0.1).astype(np.float32)
    u, g = ops.s2v_level_backward(_t(rp, gpu), _t(ci, gpu), _t(v, gpu), _t(dz, gpu), _t(W, gpu))
    w_u = oracle.spmm(rp, ci, v, dz, N)
    w_g = oracle.gemm(w_u, W, transB=True)
    import scipy.sparse as sp
    u64 = sp.csr_matrix((v.astype(np.float64), ci, rp), shape=(N, N)) @ dz.astype(np.float64)
    assert_parity("u", _n(u), w_u, u64)
    assert_parity("g_prev", _n(g), w_g, u64 @ W.astype(np.float64).T)
    # with the ReLU gate of the level below and the running sum of the msg gradient: the stored g_prev is the
    # ungated one with the closed gates zeroed (same bits), and acc grows by exactly what was stored
    h_prev = rng.standard_normal((N, C)).astype(np.float32)
    h_prev[rng.random((N, C)) < 0.1] = 0.0                       # zeros close the gate, like negative values
    acc0 = rng.standard_normal((N, C)).astype(np.float32)
    acc = _t(acc0, gpu)
    u2, g2 = ops.s2v_level_backward(_t(rp, gpu), _t(ci, gpu), _t(v, gpu), _t(dz, gpu), _t(W, gpu), gate_h=_t(h_prev, gpu), acc=acc)
    gated = np.where(h_prev > 0, _n(g), np.float32(0))
    assert np.array_equal(_n(u2), _n(u))
    assert np.array_equal(_n(g2), gated)
    assert np.array_equal(_n(acc), acc0 + gated)
    # the sum alone, without a gate
    acc = _t(acc0, gpu)
    _, g3 = ops.s2v_level_backward(_t(rp, gpu), _t(ci, gpu), _t(v, gpu), _t(dz, gpu), _t(W, gpu), acc=acc)
    assert np.array_equal(_n(g3), _n(g)) and np.array_equal(_n(acc), acc0 + _n(g))


@pytest.mark.parametrize("C", [128, 256])
@pytest.mark.parametrize("nnz", [0, 3, 6])
def test_level_backward_wide_with_hardly_any_entries(gpu, oracle, C, nnz):
    """the wide kernel's backward variant on a transposed adjacency with fewer entries than one index batch (and none)"""
    from graphnn_amd import ops
    rng = np.random.default_rng(C + nnz)
    N = 40
    rows = np.sort(rng.integers(0, N, nnz))
    rp = np.zeros(N + 1, np.int32); np.cumsum(np.bincount(rows, minlength=N), out=rp[1:])
    ci = rng.integers(0, N, nnz).astype(np.int32)
    v = (0.5 + rng.random(nnz)).astype(np.float32)
    dz = rng.standard_normal((N, C)).astype(np.float32)
    W = (rng.standard_normal((C, C)) * 0.1).astype(np.float32)
    h_prev = rng.standard_normal((N, C)).astype(np.float32)
    acc0 = rng.standard_normal((N, C)).astype(np.float32)
    acc = _t(acc0, gpu)
    pad = lambda a, dt: _t(np.concatenate([a, np.zeros(1, dt)]), gpu)[:a.size]      # never a null pointer for an empty array
    u, g = ops.s2v_level_backward(_t(rp, gpu), pad(ci, np.int32), pad(v, np.float32), _t(dz, gpu), _t(W, gpu), gate_h=_t(h_prev, gpu), acc=acc)
    import scipy.sparse as sp
    u64 = sp.csr_matrix((v.astype(np.float64), ci, rp), shape=(N, N)) @ dz.astype(np.float64)
    g64 = (u64 @ W.astype(np.float64).T) * (h_prev > 0)
    w_u = oracle.spmm(rp, ci, v, dz, N)
    w_g = (oracle.gemm(w_u, W, transB=True) * (h_prev > 0)).astype(np.float32)
    assert_parity("u", _n(u), w_u, u64)
    assert_parity("g_prev", _n(g), w_g, g64)
    assert np.array_equal(_n(acc), acc0 + _n(g))


def test_grad_gate_is_exact(gpu):
    import torch
    from graphnn_amd import ops
    rng = np.random.default_rng(3)
    n = 100003
    h = np.maximum(rng.standard_normal(n), 0).astype(np.float32); h[5] = -0.0; h[6] = np.nan
    g = rng.standard_normal(n).astype(np.float32)
    acc0 = rng.standard_normal(n).astype(np.float32)
    dz = torch.empty(n, device=gpu); acc = _t(acc0, gpu)
    ops.grad_gate(_t(h, gpu), _t(g, gpu), dz, acc, accumulate=True)
    want = np.where(h > 0, g, 0).astype(np.float32)
    assert np.array_equal(_n(dz), want) and np.array_equal(_n(acc), acc0 + want)
    gd = _t(g, gpu)
    ops.grad_gate(_t(h, gpu), gd, gd, acc, accumulate=False)            # in place, acc overwritten
    assert np.array_equal(_n(gd), want) and np.array_equal(_n(acc), want)


@pytest.mark.parametrize("momentum", [0.9, 0.0])
def test_momentum_sgd_batch_two_steps(gpu, oracle, momentum):
    from graphnn_amd import ops
    rng = np.random.default_rng(17)
    shapes = [(38, 64), (64, 64), (64, 32), (32, 2), (1,), (100003,)]
    lr, l2 = 0.05, 0.01
    w = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    wd, vd = [_t(a, gpu) for a in w], [_t(a, gpu) for a in v]
    for step in range(2):
        g = [rng.standard_normal(s).astype(np.float32) for s in shapes]
        gd = [_t(a, gpu) for a in g]
        ops.momentum_sgd_batch(wd, gd, vd if momentum > 0 else None, lr, momentum, l2)
        for i in range(len(shapes)):
            w[i], g0, v[i] = oracle.momentum_sgd(w[i], g[i], v[i], lr, momentum, l2)
            assert not _n(gd[i]).any()
            assert np.allclose(_n(wd[i]), w[i], rtol=1e-6, atol=1e-7), (step, i)
            if momentum > 0:
                assert np.allclose(_n(vd[i]), v[i], rtol=1e-6, atol=1e-7), (step, i)


@pytest.mark.parametrize("clip,l2", [(5.0, 0.01), (0.0, 0.0), (1e6, 0.3)])
def test_adam_batch_three_steps(gpu, oracle, clip, l2):
    """AdamOptimizer::Update over a parameter set in two launches (the norm of all gradients, then the update with
    the clipping factor formed on the device), three consecutive steps: gradients that are clipped (their norm is
    far above 5), not clipped (threshold off or out of reach), 18 tensors (more than one table), one of them large"""
    from graphnn_amd import ops
    rng = np.random.default_rng(23)
    shapes = [(38, 64), (64, 64), (64, 32), (32, 2), (1,), (300007,)] + [(5, 3)] * 12
    lr, b1, b2, eps = 0.01, 0.9, 0.999, 1e-8
    w = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    m = [np.zeros(s, np.float32) for s in shapes]
    v = [np.zeros(s, np.float32) for s in shapes]
    wd, md, vd = [_t(a, gpu) for a in w], [_t(a, gpu) for a in m], [_t(a, gpu) for a in v]
    for step in range(1, 4):
        g = [(rng.standard_normal(s) * (0.02 if step == 3 else 1.0)).astype(np.float32) for s in shapes]
        gd = [_t(a, gpu) for a in g]
        ops.adam_batch(wd, gd, md, vd, lr, l2, clip, b1, b2, eps, step)
        scale = oracle.clip_factor(g, clip) if clip > 0 else 1.0
        if clip == 5.0:
            assert (scale < 0.05) == (step < 3)
        for i in range(len(shapes)):
            # where weight decay and the scaled gradient cancel (l2 w = -scale g to four digits) the sum carries the
            # last bits of the clipping factor, which the device forms in double: those elements are left out
            parts = np.abs(l2 * w[i]) + np.abs(scale * g[i])
            steady = np.abs(l2 * w[i] + scale * g[i]) > 1e-3 * parts
            w[i], g0, m[i], v[i] = oracle.adam(w[i], g[i], m[i], v[i], lr, l2, scale, b1, b2, eps, step)
            assert not _n(gd[i]).any()
            assert steady.size < 1000 or steady.mean() > 0.99
            # both sides round b m + (1 - b) g term by term, the device with one fused step: an ulp of the larger term
            assert np.allclose(_n(md[i]), m[i], rtol=2e-6, atol=1e-6), (step, i)
            assert np.allclose(_n(vd[i]), v[i], rtol=4e-6, atol=1e-6), (step, i)
            assert np.allclose(_n(wd[i])[steady], w[i][steady], rtol=1e-6, atol=2e-7), (step, i)
            assert np.allclose(_n(wd[i]), w[i], rtol=0, atol=2.1 * lr), (step, i)
            # the device's own values go on, so that a left-out element does not carry into the next step
            w[i], m[i], v[i] = _n(wd[i]).copy(), _n(md[i]).copy(), _n(vd[i]).copy()


def _dense(csr, rows, cols):
    import scipy.sparse as sp
    return sp.csr_matrix((csr[2].astype(np.float64), csr[1], csr[0]), shape=(rows, cols)).toarray()


@pytest.mark.parametrize("config_id,C", [(1, 64), (2, 64), (1, 128)])
def test_training_iteration_composed_from_the_c_abi(gpu, oracle, config_id, C):
    """forward with every level kept, loss tail, backward (readout backward; per level gate, A^T dz, (.) W^T;
    the weight gradients as four products) and one momentum-SGD update: gradients against float64 autograd
    of the same network at 1e-4, updated weights against the oracle's update of those gradients"""
    import torch
    from graphnn_amd import ops
    batch, w, cfg = synth.make_config(config_id)
    K, H, Q, L = cfg["K"], cfg["H"], cfg["Q"], cfg["L"]
    if C != cfg["C"]:
        w = synth.make_weights(synth.Stream(900 + C), K, C, H, Q)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    lab = batch.label_csr()
    X = batch.one_hot()
    N, B = batch.num_nodes, batch.num_graphs
    a_d, s_d, lab_d = ([_t(x, gpu) for x in m] for m in (a, s, lab))
    Wn, Wc, W1, W2 = (_t(m, gpu) for m in (w.W_n2l, w.W_conv, w.W_h1, w.W_h2))
    X_d = _t(X, gpu)
    # ---- forward, embeddings of all levels stacked
    hs = torch.empty((L + 1, N, C), device=gpu)
    msg, h0 = ops.s2v_input(X_d, Wn)
    hs[0] = h0
    for l in range(L):
        ops.s2v_level(*a_d, hs[l], Wc, msg, out=hs[l + 1])
    pool, hidden, logits, probs, pred = ops.s2v_readout(*s_d, hs[L], W1, W2, B)
    loss, acc, probs2, _, _ = ops.loss_acc(logits, *lab_d)
    # ---- backward
    dl, du, g = ops.readout_backward(s_d, probs2, lab_d, 1.0 / B, hidden, W1, W2, N)
    at = ops.csr_transpose(*a_d, N, N)
    us = torch.empty((L, N, C), device=gpu)
    dmsg = torch.empty((N, C), device=gpu)
    g2 = torch.empty_like(g)
    ops.grad_gate(hs[L], g, g, dmsg, accumulate=False)
    for l in range(L, 0, -1):
        # the gradient comes out past the gate of the level below and is added to the msg gradient on the way
        ops.s2v_level_backward(*at, g, Wc, u=us[l - 1], g_prev=g2, gate_h=hs[l - 1], acc=dmsg)
        g, g2 = g2, g
    gWc = ops.gemm(hs[:L].reshape(L * N, C), us.reshape(L * N, C), transA=True)
    gWn = ops.gemm(X_d, dmsg, transA=True)
    gW1 = ops.gemm(pool, du, transA=True)
    gW2 = ops.gemm(hidden, dl, transA=True)
    # ---- float64 autograd of the same network
    t64 = lambda m: torch.tensor(np.asarray(m, np.float64), requires_grad=True)
    P = [t64(m) for m in (w.W_n2l, w.W_conv, w.W_h1, w.W_h2)]
    A = torch.tensor(_dense(a, N, N)); S = torch.tensor(_dense(s, B, N)); X64 = torch.tensor(X.astype(np.float64))
    m64 = X64 @ P[0]
    h64 = torch.relu(m64)
    for _ in range(L):
        h64 = torch.relu((A @ h64) @ P[1] + m64)
    lg64 = torch.relu((S @ h64) @ P[2]) @ P[3]
    loss64 = torch.nn.functional.cross_entropy(lg64, torch.tensor(batch.graph_label.astype(np.int64)))
    loss64.backward()
    assert abs(float(_n(loss)[0]) - float(loss64)) <= 1e-5 * abs(float(loss64))
    for name, got, p in (("w_n2l", gWn, P[0]), ("w_conv", gWc, P[1]), ("w_h1", gW1, P[2]), ("w_h2", gW2, P[3])):
        err = max_rel(_n(got), p.grad.numpy())
        print("gradient %s: max_rel %.2e against float64" % (name, err))
        assert err < PARITY_TOL, name
    # ---- one update of all four tensors in one launch
    ws = [Wn.clone(), Wc.clone(), W1.clone(), W2.clone()]
    gs = [gWn.clone(), gWc.clone(), gW1.clone(), gW2.clone()]
    vs = [torch.zeros_like(t) for t in ws]
    ops.momentum_sgd_batch(ws, gs, vs, 0.01, 0.9, 1e-4)
    for t, w0, g0 in zip(ws, (w.W_n2l, w.W_conv, w.W_h1, w.W_h2), (gWn, gWc, gW1, gW2)):
        want_w, _, _ = oracle.momentum_sgd(w0, _n(g0), np.zeros_like(w0), 0.01, 0.9, 1e-4)
        assert np.allclose(_n(t), want_w, rtol=1e-6, atol=1e-8)
