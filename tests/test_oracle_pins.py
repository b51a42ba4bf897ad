"""Pins the CPU oracle (oracle/s2v_oracle.c) before anything is compared with it.

Each oracle function is checked against something that does not share its code:
brute force in float64, closed forms, invariants, the reference's own known-answer
matrix, the reference's own GraphStruct container (oracle/_ref, when built) and,
when libmkl_rt can be loaded, Intel MKL called with the argument pattern graphnn's
CPU tensors use (mkl_scsrmm "GLNC", cblas_sgemm row-major).
"""
import ctypes
import json
import os

import numpy as np
import pytest

from conftest import max_rel
from graphnn_amd import batching, synth

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _rng(seed):
    return np.random.default_rng(seed)


# ------------------------------------------------------------------ CSR builders
def _random_graph(rng, N, E, B):
    ex = rng.integers(0, N, E).astype(np.int32)
    ey = rng.integers(0, N, E).astype(np.int32)
    sid = np.sort(rng.integers(0, B, N)).astype(np.int32)
    nid = np.arange(N, dtype=np.int32)
    return ex, ey, sid, nid


def test_csr_node2node_bruteforce(oracle):
    rng = _rng(1)
    for N, E in [(1, 0), (5, 7), (40, 200), (64, 64)]:
        ex, ey, _, _ = _random_graph(rng, N, E, 1)
        rp, ci, v = oracle.csr_node2node(N, ex, ey)
        # invariants
        assert rp[0] == 0 and rp[N] == E and np.all(np.diff(rp) >= 0)
        # brute force: row y holds the sources of edges into y, in edge order
        for y in range(N):
            want = [int(ex[e]) for e in range(E) if ey[e] == y]
            assert list(ci[rp[y]:rp[y + 1]]) == want
        assert np.all(v == 1.0)
        # dense adjacency counts (duplicates accumulate)
        dense = np.zeros((N, N), np.int64)
        for e in range(E):
            dense[ey[e], ex[e]] += 1
        rebuilt = np.zeros((N, N), np.int64)
        for y in range(N):
            for t in range(rp[y], rp[y + 1]):
                rebuilt[y, ci[t]] += 1
        assert np.array_equal(dense, rebuilt)


def test_csr_average_values(oracle):
    rng = _rng(2)
    ex, ey, sid, nid = _random_graph(rng, 30, 90, 4)
    rp, ci, v = oracle.csr_node2node(30, ex, ey, average=True)
    for y in range(30):
        d = rp[y + 1] - rp[y]
        if d:
            assert np.all(v[rp[y]:rp[y + 1]] == np.float32(1.0 / d))
    rp, ci, v = oracle.csr_subgraph(4, sid, nid, average=True)
    for g in range(4):
        d = rp[g + 1] - rp[g]
        if d:
            assert np.all(v[rp[g]:rp[g + 1]] == np.float32(1.0 / d))


def test_csr_subgraph_contiguous(oracle):
    b = synth.molecule_batch(7, 12, 5)
    rp, ci, v = oracle.csr_subgraph(b.num_graphs, b.subg_id, b.node_idx)
    assert np.array_equal(ci, np.arange(b.num_nodes))            # identity permutation
    assert np.array_equal(rp, np.concatenate([[0], np.cumsum(b.graph_sizes)]))
    assert np.all(v == 1.0)


def test_csr_undirected_batch_is_symmetric_and_sorted(oracle):
    b = synth.molecule_batch(11, 20, 7)
    rp, ci, _ = oracle.csr_node2node(b.num_nodes, b.edge_x, b.edge_y)
    assert rp[-1] == b.num_edges
    dense = np.zeros((b.num_nodes, b.num_nodes), np.int32)
    for y in range(b.num_nodes):
        row = ci[rp[y]:rp[y + 1]]
        assert np.all(np.diff(row) > 0)                           # ascending, no duplicates
        dense[y, row] = 1
    assert np.array_equal(dense, dense.T)
    # block diagonal: no edge leaves its graph
    off = np.concatenate([[0], np.cumsum(b.graph_sizes)])
    gid = np.repeat(np.arange(b.num_graphs), b.graph_sizes)
    rows = np.repeat(np.arange(b.num_nodes), np.diff(rp))
    assert np.array_equal(gid[rows], gid[ci])
    assert off[-1] == b.num_nodes


def test_csr_against_reference_graphstruct(oracle, ref_graph):
    if ref_graph is None:
        pytest.skip("oracle/_ref/libref_graph.so not built (reference tree absent)")
    rng = _rng(3)
    for N, E, B in [(1, 0, 1), (9, 20, 3), (200, 1000, 17)]:
        ex, ey, sid, nid = _random_graph(rng, N, E, B)
        # AddNode order need not be sorted by subgraph: shuffle it
        perm = rng.permutation(N)
        sid, nid = sid[perm].copy(), nid[perm].copy()
        P = lambda a: a.ctypes.data_as(ctypes.c_void_p)
        arp = np.zeros(N + 1, np.int32); aci = np.zeros(E, np.int32)
        srp = np.zeros(B + 1, np.int32); sci = np.zeros(N, np.int32)
        rc = ref_graph.ref_graph_to_csr(B, N, E, P(sid), P(nid), P(ex), P(ey), P(arp), P(aci), P(srp), P(sci))
        assert rc == 0
        rp, ci, _ = oracle.csr_node2node(N, ex, ey)
        assert np.array_equal(rp, arp) and np.array_equal(ci, aci)
        rp, ci, _ = oracle.csr_subgraph(B, sid, nid)
        assert np.array_equal(rp, srp) and np.array_equal(ci, sci)


def test_host_batching_matches_oracle(oracle):
    """the product's numpy CSR builders are bit-exact with the oracle (and thereby with GraphStruct)"""
    rng = _rng(4)
    for avg in (False, True):
        for N, E, B in [(1, 0, 1), (50, 300, 6), (1000, 5000, 40)]:
            ex, ey, sid, nid = _random_graph(rng, N, E, B)
            for got, want in zip(batching.node2node_csr(N, ex, ey, avg), oracle.csr_node2node(N, ex, ey, avg)):
                assert got.dtype == want.dtype and np.array_equal(got, want)
            for got, want in zip(batching.subgraph_csr(B, sid, nid, avg), oracle.csr_subgraph(B, sid, nid, avg)):
                assert got.dtype == want.dtype and np.array_equal(got, want)


# ------------------------------------------------------------------ SpMM / GEMM
def _random_csr(rng, m, k, nnz):
    rows = np.sort(rng.integers(0, m, nnz))
    rp = np.zeros(m + 1, np.int32)
    np.cumsum(np.bincount(rows, minlength=m), out=rp[1:])
    ci = rng.integers(0, max(k, 1), nnz).astype(np.int32)
    v = rng.standard_normal(nnz).astype(np.float32)
    return rp, ci, v


def _dense_of(rp, ci, v, m, k):
    A = np.zeros((m, k), np.float64)
    for i in range(m):
        for t in range(rp[i], rp[i + 1]):
            A[i, ci[t]] += float(v[t])
    return A


def test_spmm_known_answer(oracle):
    g = json.load(open(os.path.join(GOLDEN, "sparse_mm_known_answer.json")))
    rp = np.array(g["row_ptr"], np.int32); ci = np.array(g["col_idx"], np.int32); v = np.array(g["val"], np.float32)
    got = oracle.spmm(rp, ci, v, np.array(g["b_for_normal"], np.float32), g["a_rows"])
    assert np.array_equal(got, np.array(g["expected_A_b"], np.float32))
    got_t = oracle.spmm_T(rp, ci, v, np.array(g["b_for_transpose"], np.float32), g["a_rows"], g["a_cols"])
    assert np.array_equal(got_t, np.array(g["expected_At_b"], np.float32))


def test_spmm_bruteforce_identity_duplicates(oracle):
    rng = _rng(5)
    m, k, n = 37, 23, 11
    rp, ci, v = _random_csr(rng, m, k, 300)            # 300 entries over 37x23: duplicates certain
    B = rng.standard_normal((k, n)).astype(np.float32)
    C0 = rng.standard_normal((m, n)).astype(np.float32)
    want = 0.5 * _dense_of(rp, ci, v, m, k) @ B.astype(np.float64) + 2.0 * C0
    got = oracle.spmm(rp, ci, v, B, m, alpha=0.5, beta=2.0, C=C0)
    assert max_rel(got, want, 1.0) < 1e-5
    # identity
    n_id = 19
    rp_i = np.arange(n_id + 1, dtype=np.int32); ci_i = np.arange(n_id, dtype=np.int32); v_i = np.ones(n_id, np.float32)
    X = rng.standard_normal((n_id, 8)).astype(np.float32)
    assert np.array_equal(oracle.spmm(rp_i, ci_i, v_i, X, n_id), X)
    # beta = 0 ignores what was in C, even NaN
    Cn = np.full((m, n), np.nan, np.float32)
    assert np.all(np.isfinite(oracle.spmm(rp, ci, v, B, m, C=Cn)))
    # empty rows give zeros
    rp_e = np.zeros(5, np.int32)
    assert np.array_equal(oracle.spmm(rp_e, ci[:0], v[:0], B, 4), np.zeros((4, n), np.float32))
    # transpose
    Bt = rng.standard_normal((m, n)).astype(np.float32)
    want_t = _dense_of(rp, ci, v, m, k).T @ Bt.astype(np.float64)
    assert max_rel(oracle.spmm_T(rp, ci, v, Bt, m, k), want_t, 1.0) < 1e-5


def test_gemm_bruteforce_all_transposes(oracle):
    rng = _rng(6)
    m, n, k = 13, 9, 21
    for ta in (False, True):
        for tb in (False, True):
            A = rng.standard_normal((k, m) if ta else (m, k)).astype(np.float32)
            B = rng.standard_normal((n, k) if tb else (k, n)).astype(np.float32)
            C0 = rng.standard_normal((m, n)).astype(np.float32)
            opA = A.T if ta else A
            opB = B.T if tb else B
            want = 1.5 * opA.astype(np.float64) @ opB.astype(np.float64) - 0.5 * C0
            got = oracle.gemm(A, B, ta, tb, alpha=1.5, beta=-0.5, C=C0)
            assert max_rel(got, want, 1.0) < 1e-5, (ta, tb)
    # the reference's own GEMM test shape: 10x20 . (30x20)^T, |delta ASum| <= 1e-4 (test/gpu_tensor_test.cpp:131-149)
    A = rng.standard_normal((10, 20)).astype(np.float32); B = rng.standard_normal((30, 20)).astype(np.float32)
    got = oracle.gemm(A, B, False, True)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    assert abs(np.abs(got).sum() - np.abs(want).sum()) <= 1e-4 * 30


# ------------------------------------------------------------------ MKL (the reference's arithmetic dependency)
def _load_mkl():
    os.environ.setdefault("MKL_THREADING_LAYER", "SEQUENTIAL")
    for name in ("libmkl_rt.so.1", "libmkl_rt.so", "/opt/conda/lib/libmkl_rt.so.1", "/opt/conda/lib/libmkl_rt.so"):
        try:
            return ctypes.CDLL(name)
        except OSError:
            continue
    return None


def test_spmm_and_gemm_against_mkl(oracle):
    mkl = _load_mkl()
    if mkl is None:
        pytest.skip("libmkl_rt not loadable on this host")
    rng = _rng(7)
    P = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    ci_t, cf = ctypes.c_int, ctypes.c_float
    # mkl_scsrmm('N', m, n, k, alpha, "GLNC", val, col_idx, row_ptr, row_ptr + 1, B, ldb, beta, C, ldc)
    # as called by DTensor<CPU>::MM(SpTensor...) (src/tensor/cpu_dense_tensor.cpp:221-224)
    m, k, n = 101, 77, 64
    B = rng.standard_normal((k, n)).astype(np.float32)
    for trans, rows_out in ((b"N", m), (b"T", k)):
        rp, ci, v = _random_csr(rng, m, k, 900)
        if trans == b"T":
            # MKL's transposed kernel does not accumulate repeated (row, col) coordinates
            # (observed with oneMKL 2021.4), so the 'T' comparison uses a duplicate-free matrix;
            # the 'N' orientation, the one the forward uses, is compared with duplicates present.
            key = np.unique(np.repeat(np.arange(m), np.diff(rp)).astype(np.int64) * k + ci)
            rows_u, ci = key // k, (key % k).astype(np.int32)
            rp = np.zeros(m + 1, np.int32); np.cumsum(np.bincount(rows_u, minlength=m), out=rp[1:])
            v = v[:len(key)].copy()
        Bm = B if trans == b"N" else rng.standard_normal((m, n)).astype(np.float32)
        C = np.zeros((rows_out, n), np.float32)
        mm, nn, kk, al, be, ld = ci_t(m), ci_t(n), ci_t(k), cf(1.25), cf(0.0), ci_t(n)
        pe = rp[1:]
        mkl.mkl_scsrmm(ctypes.c_char_p(trans), ctypes.byref(mm), ctypes.byref(nn), ctypes.byref(kk), ctypes.byref(al),
                       ctypes.c_char_p(b"GLNC"), P(v), P(ci), P(rp), P(pe), P(Bm), ctypes.byref(ld), ctypes.byref(be),
                       P(C), ctypes.byref(ld))
        got = oracle.spmm(rp, ci, v, Bm, m, alpha=1.25) if trans == b"N" else oracle.spmm_T(rp, ci, v, Bm, m, k, alpha=1.25)
        assert max_rel(got, C, 1.0) < 1e-5, trans
    # cblas_sgemm(CblasRowMajor=101, NoTrans=111 / Trans=112, ...) (cpu_dense_tensor.cpp:206-210)
    for ta in (False, True):
        for tb in (False, True):
            M, N, K = 33, 17, 40
            A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
            Bd = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
            C = np.zeros((M, N), np.float32)
            mkl.cblas_sgemm(101, 112 if ta else 111, 112 if tb else 111, M, N, K, cf(1.0), P(A), A.shape[1],
                            P(Bd), Bd.shape[1], cf(0.0), P(C), N)
            assert max_rel(oracle.gemm(A, Bd, ta, tb), C, 1.0) < 1e-5, (ta, tb)


# ------------------------------------------------------------------ element-wise
def test_unary_closed_forms(oracle):
    x = np.array([-2.5, -0.0, 0.0, 0.3, 1.0, 4.0, np.nan], np.float32)
    relu = oracle.unary(6, x)
    assert np.array_equal(relu[:6], np.array([0.0, -0.0, 0.0, 0.3, 1.0, 4.0], np.float32))
    assert np.signbit(relu[1]) and np.isnan(relu[6])             # -0.0 and NaN pass through
    assert np.array_equal(oracle.unary(0, x, 3.0), np.full(7, 3.0, np.float32))
    assert np.array_equal(oracle.unary(1, x[:6], -1.0, 1.0), np.clip(x[:6], -1.0, 1.0))
    assert np.array_equal(oracle.unary(2, x[:6], 2.0), x[:6] * np.float32(2.0))
    assert np.array_equal(oracle.unary(3, x[:6], 2.0), x[:6] + np.float32(2.0))
    assert np.array_equal(oracle.unary(4, x[:6]), np.abs(x[:6]))
    assert np.array_equal(oracle.unary(12, x[:6]), x[:6] * x[:6])
    pos = np.array([0.25, 1.0, 9.0], np.float32)
    assert np.array_equal(oracle.unary(13, pos), np.array([0.5, 1.0, 3.0], np.float32))
    assert np.array_equal(oracle.unary(5, pos), np.float32(1.0) / pos)
    assert np.allclose(oracle.unary(10, pos), 1.0 / np.sqrt(pos.astype(np.float64)), rtol=1e-6)
    y = np.linspace(-3, 3, 13).astype(np.float32)
    assert np.allclose(oracle.unary(7, y), 1.0 / (1.0 + np.exp(-y.astype(np.float64))), rtol=1e-6)
    assert np.allclose(oracle.unary(8, y), np.tanh(y.astype(np.float64)), rtol=2e-6, atol=1e-7)
    assert np.allclose(oracle.unary(11, y), np.exp(y.astype(np.float64)), rtol=1e-6)
    assert np.allclose(oracle.unary(9, pos), np.log(pos.astype(np.float64)), rtol=1e-6, atol=1e-7)


def test_axpy_axpby_exact(oracle):
    rng = _rng(8)
    x = rng.standard_normal(1001).astype(np.float32); y = rng.standard_normal(1001).astype(np.float32)
    assert np.array_equal(oracle.axpy(1.0, x, y), x + y)         # single rounded add
    assert np.array_equal(oracle.axpy(-1.0, x, y), y - x)
    a, b = np.float32(0.75), np.float32(-1.5)
    assert np.array_equal(oracle.axpby(0.75, x, -1.5, y), a * x + b * y)
    assert np.array_equal(oracle.cast(np.array([-3, 0, 7, 2**24 + 1], np.int32)),
                          np.array([-3, 0, 7, 2**24 + 1], np.int32).astype(np.float32))


# ------------------------------------------------------------------ softmax family
def test_softmax_properties(oracle):
    rng = _rng(9)
    x = rng.standard_normal((20, 200)).astype(np.float32)        # the reference's test shape
    p = oracle.row_softmax(x)
    assert np.allclose(p.sum(axis=1), 1.0, atol=1e-5)
    assert np.all(p > 0)
    assert max_rel(oracle.row_softmax(x + np.float32(5.0)), p, 1e-6) < 1e-4     # shift invariance
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    assert np.abs(p - e / e.sum(axis=1, keepdims=True)).sum() <= 1e-4          # ASum(diff) <= 1e-4
    two = rng.standard_normal((50, 2)).astype(np.float32)
    sig = 1.0 / (1.0 + np.exp(-(two[:, 0].astype(np.float64) - two[:, 1])))
    assert np.allclose(oracle.row_softmax(two)[:, 0], sig, rtol=1e-6)
    big = np.array([[1000.0, 1000.0, -1000.0]], np.float32)                     # no overflow
    assert np.allclose(oracle.row_softmax(big), [[0.5, 0.5, 0.0]])


def test_jagged_softmax_equals_per_segment(oracle):
    rng = _rng(10)
    x = (1.0 + rng.random(10)).astype(np.float32)                 # U(1,2), lens {2,3,5}: the reference's test
    lens = np.array([2, 3, 5], np.int32)
    got = oracle.jagged_softmax(x, lens)
    off = 0
    for ln in lens:
        seg = x[off:off + ln].astype(np.float64)
        e = np.exp(seg - seg.max())
        assert np.abs(got[off:off + ln] - e / e.sum()).sum() <= 1e-5
        assert np.array_equal(got[off:off + ln], oracle.row_softmax(x[off:off + ln][None, :])[0])
        off += ln
    # ragged with empty segments
    lens2 = np.array([0, 4, 0, 1, 5, 0], np.int32)
    g2 = oracle.jagged_softmax(x, lens2)
    assert np.isclose(g2[0:4].sum(), 1.0, atol=1e-6) and g2[4] == 1.0 and np.isclose(g2[5:].sum(), 1.0, atol=1e-6)


# ------------------------------------------------------------------ reductions, arg-max, CE, top-k
def test_jagged_softmax_gradient_is_the_softmax_jacobian(oracle):
    """dst += J^T g with J the Jacobian of softmax, segment by segment: checked against the Jacobian
    written out in float64 (d p_i / d x_j = p_i (delta_ij - p_j)) and against a central difference"""
    rng = _rng(23)
    lens = np.array([1, 4, 0, 7, 2], np.int32)
    x = rng.standard_normal(int(lens.sum())).astype(np.float32)
    g = rng.standard_normal(x.size).astype(np.float32)
    d0 = rng.standard_normal(x.size).astype(np.float32)
    p = oracle.jagged_softmax(x, lens)
    got = oracle.jagged_softmax_deriv(d0, p, g, lens)
    want = d0.astype(np.float64).copy()
    off = 0
    for n in lens:
        pp = p[off:off + n].astype(np.float64)
        J = np.diag(pp) - np.outer(pp, pp)
        want[off:off + n] += J.T @ g[off:off + n].astype(np.float64)
        off += n
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    # central difference of <g, softmax(x)> in float64
    def f(xv):
        tot, o = 0.0, 0
        for n in lens:
            if n:
                e = np.exp(xv[o:o + n] - xv[o:o + n].max())
                tot += float(g[o:o + n].astype(np.float64) @ (e / e.sum()))
            o += n
        return tot
    x64 = x.astype(np.float64)
    num = np.array([(f(x64 + 1e-6 * np.eye(x.size)[i]) - f(x64 - 1e-6 * np.eye(x.size)[i])) / 2e-6 for i in range(x.size)])
    assert np.allclose(got - d0, num, atol=1e-4)


def test_momentum_sgd_two_steps_closed_form(oracle):
    """two consecutive updates with l2 != 0 and momentum 0.9 against the recurrence written out in float64
    (g' = g + l2 w; v' = lr g' + m v; w' = w - v'; src/nn/optimizer.cpp:69-92), the velocity starting at
    zero, and the plain-SGD branch for momentum 0.  (ClipGradients is not part of this optimizer: only
    AdamOptimizer::Update calls it, src/nn/optimizer.cpp:108.)"""
    rng = _rng(31)
    lr, m, l2 = 0.05, 0.9, 0.01
    w0 = rng.standard_normal(1000).astype(np.float32)
    g1 = rng.standard_normal(1000).astype(np.float32)
    g2 = rng.standard_normal(1000).astype(np.float32)
    w, g, v = oracle.momentum_sgd(w0, g1, np.zeros_like(w0), lr, m, l2)
    assert not g.any()
    w, g, v = oracle.momentum_sgd(w, g2, v, lr, m, l2)
    W0, G1, G2 = (a.astype(np.float64) for a in (w0, g1, g2))
    V1 = lr * (G1 + l2 * W0)
    W1 = W0 - V1
    V2 = lr * (G2 + l2 * W1) + m * V1
    W2 = W1 - V2
    assert np.allclose(v, V2, rtol=1e-5, atol=1e-7) and np.allclose(w, W2, rtol=1e-5, atol=1e-6)
    # the step is not a plain SGD step: the second update moves further along g1 than lr alone would
    assert not np.allclose(w, W1 - lr * (G2 + l2 * W1), atol=1e-3)
    w_sgd, g_sgd, _ = oracle.momentum_sgd(w0, g1, np.zeros_like(w0), lr, 0.0, l2)
    assert np.allclose(w_sgd, (1 - lr * l2) * W0 - lr * G1, rtol=1e-5, atol=1e-6) and not g_sgd.any()


def test_adam_first_steps_closed_form(oracle):
    """what the published algorithm fixes: after the first update from zero moments the bias-corrected moments are
    g and g^2, so every weight moves by lr g / (|g| + eps), whatever the size of g; two updates against the
    recurrence written out in float64; weight decay enters the gradient (a zero gradient still moves w by its
    sign); clipping scales the gradient to the threshold norm before anything else (src/nn/optimizer.cpp:16-32,105-160)"""
    rng = _rng(41)
    lr, l2, b1, b2, eps = 0.01, 0.0, 0.9, 0.999, 1e-8
    w0 = rng.standard_normal(500).astype(np.float32)
    g1 = (rng.standard_normal(500) * np.logspace(-3, 3, 500)).astype(np.float32)
    zero = np.zeros_like(w0)
    w1, g, m1, v1 = oracle.adam(w0, g1, zero, zero, lr, l2, 1.0, b1, b2, eps, 1)
    assert not g.any()
    G1 = g1.astype(np.float64)
    assert np.allclose(w1, w0 - lr * G1 / (np.abs(G1) + eps), rtol=1e-5, atol=1e-7)
    # the decay rates as single precision holds them (1 - 0.999f is 1.0000467e-3)
    B1, B2 = float(np.float32(b1)), float(np.float32(b2))
    C1, C2 = float(np.float32(1) - np.float32(b1)), float(np.float32(1) - np.float32(b2))
    assert np.allclose(m1, C1 * G1, rtol=1e-5) and np.allclose(v1, C2 * G1 * G1, rtol=1e-5)
    # second update, with weight decay
    l2 = 0.05
    g2 = rng.standard_normal(500).astype(np.float32)
    w2, _, m2, v2 = oracle.adam(w1, g2, m1, v1, lr, l2, 1.0, b1, b2, eps, 2)
    W1, M1, V1 = (a.astype(np.float64) for a in (w1, m1, v1))
    G2 = g2.astype(np.float64) + l2 * W1
    M2 = B1 * M1 + C1 * G2
    V2 = B2 * V1 + C2 * G2 * G2
    W2 = W1 - lr / (1 - B1 ** 2) * M2 / (np.sqrt(V2 / (1 - B2 ** 2)) + eps)
    assert np.allclose(m2, M2, rtol=1e-5, atol=1e-7) and np.allclose(v2, V2, rtol=1e-5, atol=1e-9)
    assert np.allclose(w2, W2, rtol=1e-5, atol=1e-6)
    # a zero gradient with weight decay: the first step is lr * sign(w)
    w3, _, _, _ = oracle.adam(w0, zero, zero, zero, lr, 0.3, 1.0, b1, b2, eps, 1)
    assert np.allclose(w3, w0 - lr * np.sign(w0), atol=1e-6)
    # clipping: factor = threshold / global norm over all tensors, 1 below the threshold
    ga, gb = rng.standard_normal(300).astype(np.float32), rng.standard_normal((20, 7)).astype(np.float32)
    norm = np.sqrt((ga.astype(np.float64) ** 2).sum() + (gb.astype(np.float64) ** 2).sum())
    assert abs(oracle.clip_factor([ga, gb], 5.0) - 5.0 / norm) <= 1e-6 and oracle.clip_factor([ga, gb], 1e3) == 1.0
    w4, _, m4, _ = oracle.adam(w0[:300], ga, zero[:300], zero[:300], lr, 0.0, 0.25, b1, b2, eps, 1)
    assert np.allclose(m4, C1 * 0.25 * ga.astype(np.float64), rtol=1e-5)


def test_reductions(oracle):
    ints = np.arange(1, 1001, dtype=np.float32)
    assert oracle.sum(ints) == 500500.0 and oracle.mean(ints) == 500.5 and oracle.max(ints) == 1000.0
    rng = _rng(11)
    x = (1.0 + rng.random((20, 200))).astype(np.float32)          # U(1,2) 20x200: reference Mean test, tol 1e-5
    assert abs(oracle.mean(x) - x.astype(np.float64).mean()) <= 1e-5


def test_argmax_rules(oracle):
    x = np.array([[1, 3, 3, 2], [5, 5, 5, 5], [-1, -2, -0.5, -0.5], [0.0, -0.0, 0.0, 0.0]], np.float32)
    assert list(oracle.row_argmax(x)) == [1, 0, 2, 0]             # first index among ties
    rng = _rng(12)
    big = rng.standard_normal((10, 1023)).astype(np.float32)       # reference ArgMax test shape
    assert np.array_equal(oracle.row_argmax(big), big.argmax(axis=1).astype(np.int32))
    withnan = np.array([[np.nan, 9, 1], [1, np.nan, 3], [2, 5, np.nan]], np.float32)
    assert list(oracle.row_argmax(withnan)) == [0, 2, 1]          # strict '>' never selects a later NaN
    # CSR rows: first largest stored value wins, empty row -> 0
    rp = np.array([0, 1, 1, 4, 6], np.int32)
    ci = np.array([2, 0, 3, 1, 4, 0], np.int32)
    v = np.array([1.0, 0.5, 0.9, 0.9, -2.0, -1.0], np.float32)
    assert list(oracle.csr_row_argmax(rp, ci, v)) == [2, 0, 3, 0]


def test_cross_entropy_and_top_k(oracle):
    prob = np.array([[0.25, 0.75], [1.0, 0.0], [0.5, 0.5]], np.float32)
    rp = np.array([0, 1, 2, 3], np.int32); ci = np.array([1, 1, 0], np.int32); v = np.ones(3, np.float32)
    got = oracle.cross_entropy(prob, rp, ci, v)
    want = np.array([-np.log(0.75), -np.log(1e-8), -np.log(0.5)])
    assert np.allclose(got, want, rtol=1e-6)
    # weighted multi-entry label row
    rp2 = np.array([0, 2], np.int32); ci2 = np.array([0, 1], np.int32); v2 = np.array([0.25, 0.75], np.float32)
    got2 = oracle.cross_entropy(prob[:1], rp2, ci2, v2)
    assert np.isclose(got2[0], -(0.25 * np.log(0.25) + 0.75 * np.log(0.75)), rtol=1e-6)
    pred = np.array([[0.1, 0.9, 0.0], [0.3, 0.3, 0.4], [0.2, 0.2, 0.2]], np.float32)
    label = np.array([1, 0, 2], np.int32)
    assert list(oracle.in_top_k(pred, label, 1)) == [1, 0, 1]     # ties do not count against the target
    assert list(oracle.in_top_k(pred, label, 2)) == [1, 1, 1]


# ------------------------------------------------------------------ level and forward compose the pinned ops
def _forward_float64(a_csr, s_csr, X, w, L):
    N = X.shape[0]; B = len(s_csr[0]) - 1
    A = _dense_of(*a_csr, N, N); S = _dense_of(*s_csr, B, N)
    msg = X.astype(np.float64) @ w.W_n2l.astype(np.float64)
    h = np.maximum(msg, 0)
    hs = [h]
    for _ in range(L):
        h = np.maximum(A @ h @ w.W_conv.astype(np.float64) + msg, 0)
        hs.append(h)
    pool = S @ h
    hidden = np.maximum(pool @ w.W_h1.astype(np.float64), 0)
    logits = hidden @ w.W_h2.astype(np.float64)
    e = np.exp(logits - logits.max(axis=1, keepdims=True))
    return dict(msg=msg, h=np.stack(hs), pool=pool, hidden=hidden, logits=logits, probs=e / e.sum(axis=1, keepdims=True))


def test_forward_against_float64_dense_model(oracle):
    batch, w, cfg = synth.make_config(1, B=12)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    X = batch.one_hot()
    got = oracle.forward(a, s, X, w, cfg["L"], batch.label_csr())
    want = _forward_float64(a, s, X, w, cfg["L"])
    for key in ("msg", "h", "pool", "hidden", "logits", "probs"):
        assert max_rel(got[key], want[key]) < 1e-4, key
    assert np.array_equal(got["pred"], want["logits"].argmax(axis=1))
    assert np.array_equal(got["truth"], batch.graph_label)
    assert np.array_equal(got["hit"], (got["pred"] == batch.graph_label).astype(np.int32))
    lp = -np.log(want["probs"][np.arange(batch.num_graphs), batch.graph_label])
    assert np.allclose(got["loss_rows"], lp, rtol=1e-4)
    assert np.isclose(got["scalars"][0], lp.mean(), rtol=1e-4)
    assert np.isclose(got["scalars"][1], got["hit"].mean(), rtol=1e-6)
    # the level with bias: (pool * W + b) + msg, then ReLU
    rng = _rng(13)
    bias = rng.standard_normal(cfg["C"]).astype(np.float32)
    lvl = oracle.level(*a, got["h"][0], w.W_conv, got["msg"], bias)
    A = _dense_of(*a, batch.num_nodes, batch.num_nodes)
    want_lvl = np.maximum(A @ got["h"][0].astype(np.float64) @ w.W_conv.astype(np.float64) + bias + got["msg"], 0)
    assert max_rel(lvl, want_lvl) < 1e-4


def _min_floor(got, ref64, tol=1e-4):
    """smallest floor (as a fraction of max|ref|) under which max_rel(got, ref64) stays below tol"""
    g = np.asarray(got, np.float64)
    d = np.abs(g - ref64)
    den = np.maximum(np.abs(g), np.abs(ref64))
    bad = d > tol * den
    return 0.0 if not bad.any() else float((d[bad] / tol).max() / np.abs(ref64).max())


@pytest.mark.parametrize("config_id,B", [(1, 50), (1, 200), (2, 256), (2, 1000)])
def test_parity_floors_are_the_smallest_the_oracle_itself_survives(oracle, config_id, B):
    """The floors of conftest.max_rel are measured, not picked: against a float64 model of the same network
    the oracle (a correct fp32 evaluation) needs a floor of about 1e-3 of the tensor's scale on embeddings,
    hidden layer and logits to stay within 1e-4, 3e-5 on the pooled features and none on the probabilities.
    The floors in use must cover that with at most a factor of four to spare."""
    from conftest import FLOOR_DEFAULT, FLOOR_POOL, FLOOR_PROBS_ABS, forward_float64
    batch, w, cfg = synth.make_config(config_id, B=B)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    X = batch.one_hot()
    got = oracle.forward(a, s, X, w, cfg["L"], batch.label_csr())
    want = forward_float64(a, s, X, w, cfg["L"])
    need = {k: _min_floor(got[k][1:] if k == "h" else got[k], want[k][1:] if k == "h" else want[k])
            for k in ("h", "pool", "hidden", "logits", "probs")}
    print("configuration %d, %d graphs: smallest floor / max|ref| " % (config_id, B)
          + "  ".join("%s %.2e" % kv for kv in need.items()))
    assert max(need["h"], need["hidden"], need["logits"]) <= FLOOR_DEFAULT
    assert need["pool"] <= FLOOR_POOL
    assert max_rel(got["probs"], want["probs"], floor=FLOOR_PROBS_ABS) < 1e-4
    if config_id == 2:
        # ... and are not generous: a floor four times smaller already fails the oracle itself
        assert max(need["h"], need["hidden"], need["logits"]) > FLOOR_DEFAULT / 4
        assert need["pool"] > FLOOR_POOL / 10


@pytest.mark.parametrize("config_id,B", [(1, 50), (2, 256), (2, 1000)])
def test_condition_metric_holds_for_the_oracle_and_has_no_blind_band(oracle, config_id, B):
    """conftest.assert_condition: |x - float64| <= 1e-4 * (the same network on absolute values), element by element,
    no floor.  A correct fp32 evaluation (the oracle) meets it with a wide margin on every tensor; an error planted on
    an element far below the tensor's scale, which max_rel's floor hides, breaks it."""
    from conftest import FLOOR_DEFAULT, condition_error, forward_float64
    batch, w, cfg = synth.make_config(config_id, B=B)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    X = batch.one_hot()
    got = oracle.forward(a, s, X, w, cfg["L"], batch.label_csr())
    want = forward_float64(a, s, X, w, cfg["L"])
    cond = forward_float64(a, s, X, w, cfg["L"], magnitudes=True)
    worst = {k: condition_error(got[k], want[k], cond[k])[0] for k in ("msg", "h", "pool", "hidden", "logits", "probs")}
    print("configuration %d, %d graphs: oracle, worst |x - float64| / sum|terms|: " % (config_id, B)
          + "  ".join("%s %.2e" % kv for kv in worst.items()))
    assert max(worst.values()) < 2e-5            # an fp32 sum of n terms is within n * 2^-24 in these units
    # the condition tensor dominates the value it belongs to (triangle inequality), so the metric is never laxer than
    # an absolute error of 1e-4 of the element's own magnitude
    for k in ("msg", "h", "pool", "hidden", "logits"):
        assert np.all(cond[k] >= np.abs(want[k]) * (1 - 1e-12))
    # plant an error of 1 % on the smallest non-zero logit: invisible to max_rel at its floor when that logit is
    # far below the scale, caught by the condition metric whenever it exceeds 1e-4 of the element's terms
    lg = got["logits"].copy()
    flat = np.abs(want["logits"]).ravel()
    i = int(np.argmin(np.where(flat > 0, flat, np.inf)))
    lg.ravel()[i] *= 1.5
    planted, at = condition_error(lg, want["logits"], cond["logits"])
    if 0.5 * flat[i] > 1e-4 * cond["logits"].ravel()[i]:
        assert planted > 1e-4 and at == i
    if 0.5 * flat[i] < 1e-4 * FLOOR_DEFAULT * np.abs(want["logits"]).max():
        assert max_rel(lg, got["logits"]) < 1e-4     # the floored metric does not see it


def test_stage_checker_accepts_the_oracle_and_catches_a_planted_error(oracle):
    """conftest.assert_stages on the oracle's own outputs (a correct fp32 evaluation passes every stage), then with one
    embedding element moved by 1e-3 of its terms (the stage that produced it must fail)"""
    from conftest import assert_stages
    batch, w, cfg = synth.make_config(1)
    a = batching.node2node_csr(batch.num_nodes, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(batch.num_graphs, batch.subg_id, batch.node_idx)
    X = batch.one_hot()
    got = oracle.forward(a, s, X, w, cfg["L"], batch.label_csr())
    dev = {k: got[k] for k in ("msg", "h", "pool", "hidden", "logits", "probs")}
    assert_stages("", a, s, X, w, dev, tol=2e-6)
    bad = dict(dev, h=got["h"].copy())
    i = np.unravel_index(np.argmax(got["h"][2]), got["h"][2].shape)
    bad["h"][2][i] *= 1.001
    with pytest.raises(AssertionError, match="h2"):
        assert_stages("", a, s, X, w, bad)


def test_condition_metric_on_products(oracle):
    """the same bound for the oracle's SpMM, GEMM and level on signed random operands (every output a cancelling
    sum), and what it means at its edges: an element whose terms are all zero must be exactly zero"""
    import scipy.sparse as sp
    from conftest import condition_error
    rng = _rng(77)
    m, k, n, nnz = 300, 200, 64, 6000
    rows = np.sort(rng.integers(0, m, nnz))
    rp = np.zeros(m + 1, np.int32); np.cumsum(np.bincount(rows, minlength=m), out=rp[1:])
    ci = rng.integers(0, k, nnz).astype(np.int32); v = rng.standard_normal(nnz).astype(np.float32)
    Bm = rng.standard_normal((k, n)).astype(np.float32)
    A64 = sp.csr_matrix((v.astype(np.float64), ci, rp), shape=(m, k))
    A64_mag = sp.csr_matrix((np.abs(v.astype(np.float64)), ci, rp), shape=(m, k))
    got = oracle.spmm(rp, ci, v, Bm, m)
    worst, _ = condition_error(got, A64 @ Bm.astype(np.float64), A64_mag @ np.abs(Bm.astype(np.float64)))
    assert worst < 1e-5
    Am = rng.standard_normal((150, 333)).astype(np.float32); Bg = rng.standard_normal((333, 40)).astype(np.float32)
    worst, _ = condition_error(oracle.gemm(Am, Bg), Am.astype(np.float64) @ Bg.astype(np.float64),
                               np.abs(Am.astype(np.float64)) @ np.abs(Bg.astype(np.float64)))
    assert worst < 1e-5
    # the oracle's own float64 product (the arbiter at full sizes) against scipy's
    f64 = oracle.spmm_f64(rp, ci, v, Bm, m, alpha=-0.75)
    assert np.allclose(f64, -0.75 * (A64 @ Bm.astype(np.float64)), rtol=1e-13, atol=1e-13)
    assert np.allclose(oracle.spmm_f64(rp, ci, v, Bm, m, alpha=-0.75, absolute=True), 0.75 * (A64_mag @ np.abs(Bm.astype(np.float64))), rtol=1e-13)
    # all-zero terms: zero passes, anything else is infinitely wrong
    assert condition_error(np.zeros(3), np.zeros(3), np.zeros(3))[0] == 0.0
    assert condition_error(np.array([0.0, 1e-30, 0.0]), np.zeros(3), np.zeros(3)) == (np.inf, 1)


def test_edge_based_operands_against_dense_definitions(oracle):
    """Edge2Node / Node2Edge / Edge2Edge (src/nn/msg_pass.cpp:72-152) against matrices written straight
    from their definitions, and the numpy builders against the oracle"""
    from graphnn_amd import batching
    rng = np.random.default_rng(12)
    N, E = 23, 90
    ex = rng.integers(0, N, E); ey = rng.integers(0, N, E)
    ex[5], ey[5] = ey[4], ex[4]                                   # a reverse pair
    ex[7], ey[7] = 3, 3                                           # a self-loop
    def dense(rp, ci, v, rows, cols):
        M = np.zeros((rows, cols))
        for r in range(rows):
            for t in range(rp[r], rp[r + 1]):
                M[r, ci[t]] += v[t]
        return M
    for average in (False, True):
        rp, ci, v = oracle.csr_edge2node(N, ey, average)
        want = np.zeros((N, E))
        for e in range(E):
            want[ey[e], e] = 1.0
        if average:
            want = want / np.maximum(want.sum(axis=1, keepdims=True), 1)
        assert np.allclose(dense(rp, ci, v, N, E), want, atol=1e-7)
        assert all(np.all(np.diff(ci[rp[r]:rp[r + 1]]) > 0) for r in range(N))       # insertion order = ascending e
        for got, w2 in zip(batching.edge2node_csr(N, ey, average), (rp, ci, v)):
            assert np.array_equal(got, w2)
    rp, ci, v = oracle.csr_node2edge(ex)
    assert np.array_equal(rp, np.arange(E + 1)) and np.array_equal(ci, ex) and np.all(v == 1)
    for got, w2 in zip(batching.node2edge_csr(ex), (rp, ci, v)):
        assert np.array_equal(got, w2)
    rp, ci, v = oracle.csr_edge2edge(N, ex, ey)
    want = np.zeros((E, E))
    for e in range(E):
        for o in range(E):
            if ey[o] == ex[e] and ex[o] != ey[e]:
                want[e, o] = 1.0
    assert np.array_equal(dense(rp, ci, v, E, E), want)
    assert all(np.all(np.diff(ci[rp[r]:rp[r + 1]]) > 0) for r in range(E))
    for got, w2 in zip(batching.edge2edge_csr(N, ex, ey), (rp, ci, v)):
        assert np.array_equal(got, w2)
    # no edges at all
    rp, ci, v = oracle.csr_edge2edge(4, np.zeros(0, np.int32), np.zeros(0, np.int32))
    assert np.array_equal(rp, [0]) and ci.size == 0
