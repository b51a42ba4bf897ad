import ctypes
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# --------------------------------------------------------------------------- oracle binding
_ORACLE_PATH = os.path.join(ROOT, "oracle", "liboracle.so")
_REF_PATH = os.path.join(ROOT, "oracle", "_ref", "libref_graph.so")


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


class Oracle:
    """ctypes view of oracle/liboracle.so (the CPU restatement; checker only)."""

    def __init__(self):
        if not os.path.exists(_ORACLE_PATH):
            import subprocess
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "liboracle.so"])
        self.lib = ctypes.CDLL(_ORACLE_PATH)
        self.lib.orc_sum.restype = ctypes.c_float
        self.lib.orc_mean.restype = ctypes.c_float
        self.lib.orc_max.restype = ctypes.c_float

    # ---- CSR builders
    def csr_node2node(self, N, ex, ey, average=False):
        E = len(ex)
        ex = np.ascontiguousarray(ex, dtype=np.int32)
        ey = np.ascontiguousarray(ey, dtype=np.int32)
        rp = np.zeros(N + 1, np.int32); ci = np.zeros(E, np.int32); v = np.zeros(E, np.float32)
        self.lib.orc_csr_node2node(N, E, _ptr(ex), _ptr(ey), int(average), _ptr(rp), _ptr(ci), _ptr(v))
        return rp, ci, v

    def csr_edge2node(self, N, ey, average=False):
        ey = np.ascontiguousarray(ey, np.int32)
        E = ey.size
        rp, ci, v = np.zeros(N + 1, np.int32), np.zeros(E, np.int32), np.zeros(E, np.float32)
        self.lib.orc_csr_edge2node(N, E, _ptr(ey), int(average), _ptr(rp), _ptr(ci), _ptr(v))
        return rp, ci, v

    def csr_node2edge(self, ex):
        ex = np.ascontiguousarray(ex, np.int32)
        E = ex.size
        rp, ci, v = np.zeros(E + 1, np.int32), np.zeros(E, np.int32), np.zeros(E, np.float32)
        self.lib.orc_csr_node2edge(E, _ptr(ex), _ptr(rp), _ptr(ci), _ptr(v))
        return rp, ci, v

    def csr_edge2edge(self, N, ex, ey):
        ex, ey = np.ascontiguousarray(ex, np.int32), np.ascontiguousarray(ey, np.int32)
        E = ex.size
        rp = np.zeros(E + 1, np.int32)
        self.lib.orc_csr_edge2edge.restype = ctypes.c_int
        nnz = self.lib.orc_csr_edge2edge(N, E, _ptr(ex), _ptr(ey), _ptr(rp), None, None)
        ci, v = np.zeros(max(nnz, 1), np.int32), np.zeros(max(nnz, 1), np.float32)
        self.lib.orc_csr_edge2edge(N, E, _ptr(ex), _ptr(ey), _ptr(rp), _ptr(ci), _ptr(v))
        return rp, ci[:nnz], v[:nnz]

    def csr_subgraph(self, B, sid, nid, average=False):
        N = len(sid)
        sid = np.ascontiguousarray(sid, dtype=np.int32)
        nid = np.ascontiguousarray(nid, dtype=np.int32)
        rp = np.zeros(B + 1, np.int32); ci = np.zeros(N, np.int32); v = np.zeros(N, np.float32)
        self.lib.orc_csr_subgraph(B, N, _ptr(sid), _ptr(nid), int(average), _ptr(rp), _ptr(ci), _ptr(v))
        return rp, ci, v

    # ---- tensor ops
    def spmm(self, rp, ci, v, Bm, m, alpha=1.0, beta=0.0, C=None):
        Bm = np.ascontiguousarray(Bm, np.float32)
        n = Bm.shape[1]
        out = np.zeros((m, n), np.float32) if C is None else np.array(C, dtype=np.float32, copy=True)
        self.lib.orc_spmm_csr(m, n, ctypes.c_float(alpha), _ptr(rp), _ptr(ci), _ptr(v), _ptr(Bm), n,
                              ctypes.c_float(beta), _ptr(out), n)
        return out

    def spmm_f64(self, rp, ci, v, Bm, m, alpha=1.0, absolute=False):
        """float64 arbiter: alpha * A * B with products and sums in double (absolute: over magnitudes)"""
        Bm = np.ascontiguousarray(Bm, np.float32)
        n = Bm.shape[1]
        out = np.empty((m, n), np.float64)
        self.lib.orc_spmm_csr_f64(m, n, ctypes.c_float(alpha), _ptr(rp), _ptr(ci), _ptr(v), _ptr(Bm), n, int(absolute), _ptr(out), n)
        return out

    def spmm_T(self, rp, ci, v, Bm, m, k, alpha=1.0, beta=0.0, C=None):
        Bm = np.ascontiguousarray(Bm, np.float32)
        n = Bm.shape[1]
        out = np.zeros((k, n), np.float32) if C is None else np.array(C, dtype=np.float32, copy=True)
        self.lib.orc_spmm_csr_T(m, n, k, ctypes.c_float(alpha), _ptr(rp), _ptr(ci), _ptr(v), _ptr(Bm), n,
                                ctypes.c_float(beta), _ptr(out), n)
        return out

    def gemm(self, A, Bm, transA=False, transB=False, alpha=1.0, beta=0.0, C=None):
        A = np.ascontiguousarray(A, np.float32); Bm = np.ascontiguousarray(Bm, np.float32)
        m = A.shape[1] if transA else A.shape[0]
        k = A.shape[0] if transA else A.shape[1]
        n = Bm.shape[0] if transB else Bm.shape[1]
        out = np.zeros((m, n), np.float32) if C is None else np.array(C, dtype=np.float32, copy=True)
        self.lib.orc_gemm(int(transA), int(transB), m, n, k, ctypes.c_float(alpha), _ptr(A), A.shape[1],
                          _ptr(Bm), Bm.shape[1], ctypes.c_float(beta), _ptr(out), n)
        return out

    def axpy(self, a, x, y):
        y = np.array(y, np.float32, copy=True); x = np.ascontiguousarray(x, np.float32)
        self.lib.orc_axpy(ctypes.c_size_t(x.size), ctypes.c_float(a), _ptr(x), _ptr(y))
        return y

    def axpby(self, a, x, b, y):
        y = np.array(y, np.float32, copy=True); x = np.ascontiguousarray(x, np.float32)
        self.lib.orc_axpby(ctypes.c_size_t(x.size), ctypes.c_float(a), _ptr(x), ctypes.c_float(b), _ptr(y))
        return y

    def unary(self, op, x, a0=0.0, a1=0.0):
        x = np.array(x, np.float32, copy=True)
        self.lib.orc_unary(int(op), _ptr(x), ctypes.c_size_t(x.size), ctypes.c_float(a0), ctypes.c_float(a1))
        return x

    def row_softmax(self, x):
        x = np.array(x, np.float32, copy=True)
        self.lib.orc_row_softmax(_ptr(x), x.shape[0], x.shape[1])
        return x

    def jagged_softmax(self, x, lens):
        x = np.array(x, np.float32, copy=True); lens = np.ascontiguousarray(lens, np.int32)
        self.lib.orc_jagged_softmax(_ptr(x), _ptr(lens), len(lens))
        return x

    def jagged_softmax_deriv(self, dst, out, grad, lens):
        dst = np.array(dst, np.float32, copy=True)
        out = np.ascontiguousarray(out, np.float32); grad = np.ascontiguousarray(grad, np.float32)
        lens = np.ascontiguousarray(lens, np.int32)
        self.lib.orc_jagged_softmax_deriv(_ptr(dst), _ptr(out), _ptr(grad), _ptr(lens), len(lens))
        return dst

    def momentum_sgd(self, w, g, v, lr, momentum, l2):
        """one update; returns the new (w, g, v)"""
        w, g, v = (np.array(a, np.float32, copy=True) for a in (w, g, v))
        self.lib.orc_momentum_sgd(ctypes.c_size_t(w.size), _ptr(w), _ptr(g), _ptr(v), ctypes.c_float(lr),
                                  ctypes.c_float(momentum), ctypes.c_float(l2))
        return w, g, v

    def clip_factor(self, grads, threshold):
        gs = [np.ascontiguousarray(g, np.float32) for g in grads]
        ptrs = (ctypes.c_void_p * len(gs))(*[g.ctypes.data for g in gs])
        counts = (ctypes.c_size_t * len(gs))(*[g.size for g in gs])
        self.lib.orc_clip_factor.restype = ctypes.c_float
        return float(self.lib.orc_clip_factor(len(gs), ptrs, counts, ctypes.c_float(threshold)))

    def adam(self, w, g, m, v, lr, l2, gscale, b1, b2, eps, t):
        """one update of one tensor; returns the new (w, g, m, v)"""
        w, g, m, v = (np.array(a, np.float32, copy=True) for a in (w, g, m, v))
        self.lib.orc_adam(ctypes.c_size_t(w.size), _ptr(w), _ptr(g), _ptr(m), _ptr(v), ctypes.c_float(lr), ctypes.c_float(l2),
                          ctypes.c_float(gscale), ctypes.c_float(b1), ctypes.c_float(b2), ctypes.c_float(eps), ctypes.c_int(t))
        return w, g, m, v

    def sum(self, x):
        x = np.ascontiguousarray(x, np.float32)
        return float(self.lib.orc_sum(_ptr(x), ctypes.c_size_t(x.size)))

    def mean(self, x):
        x = np.ascontiguousarray(x, np.float32)
        return float(self.lib.orc_mean(_ptr(x), ctypes.c_size_t(x.size)))

    def max(self, x):
        x = np.ascontiguousarray(x, np.float32)
        return float(self.lib.orc_max(_ptr(x), ctypes.c_size_t(x.size)))

    def row_argmax(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.zeros(x.shape[0], np.int32)
        self.lib.orc_row_argmax(_ptr(x), x.shape[0], x.shape[1], _ptr(out))
        return out

    def csr_row_argmax(self, rp, ci, v):
        out = np.zeros(len(rp) - 1, np.int32)
        self.lib.orc_csr_row_argmax(_ptr(rp), _ptr(ci), _ptr(v), len(rp) - 1, _ptr(out))
        return out

    def cross_entropy(self, prob, rp, ci, v):
        prob = np.ascontiguousarray(prob, np.float32)
        out = np.zeros(prob.shape[0], np.float32)
        self.lib.orc_cross_entropy(_ptr(prob), prob.shape[0], prob.shape[1], _ptr(rp), _ptr(ci), _ptr(v), _ptr(out))
        return out

    def in_top_k(self, pred, label, k=1):
        pred = np.ascontiguousarray(pred, np.float32); label = np.ascontiguousarray(label, np.int32)
        out = np.zeros(pred.shape[0], np.int32)
        self.lib.orc_in_top_k(_ptr(pred), _ptr(label), pred.shape[0], pred.shape[1], k, _ptr(out))
        return out

    def cast(self, src):
        src = np.ascontiguousarray(src, np.int32)
        dst = np.zeros(src.shape, np.float32)
        self.lib.orc_cast_i32_f32(_ptr(src), _ptr(dst), ctypes.c_size_t(src.size))
        return dst

    def level(self, rp, ci, v, h_in, W, msg=None, bias=None):
        h_in = np.ascontiguousarray(h_in, np.float32); W = np.ascontiguousarray(W, np.float32)
        N, C = h_in.shape
        tmp = np.zeros((N, C), np.float32); out = np.zeros((N, C), np.float32)
        msg_p = _ptr(np.ascontiguousarray(msg, np.float32)) if msg is not None else None
        bias_a = np.ascontiguousarray(bias, np.float32) if bias is not None else None
        self.lib.orc_s2v_level(N, C, _ptr(rp), _ptr(ci), _ptr(v), _ptr(h_in), _ptr(W), msg_p,
                               _ptr(bias_a) if bias_a is not None else None, _ptr(tmp), _ptr(out))
        return out

    def forward(self, a_csr, s_csr, X, w, L, label_csr=None):
        X = np.ascontiguousarray(X, np.float32)
        N, K = X.shape
        C, H, Q = w.W_n2l.shape[1], w.W_h1.shape[1], w.W_h2.shape[1]
        B = len(s_csr[0]) - 1
        f = np.float32
        out = dict(msg=np.zeros((N, C), f), h=np.zeros((L + 1, N, C), f), pool=np.zeros((B, C), f),
                   hidden=np.zeros((B, H), f), logits=np.zeros((B, Q), f), probs=np.zeros((B, Q), f),
                   loss_rows=np.zeros(B, f), pred=np.zeros(B, np.int32), truth=np.zeros(B, np.int32),
                   hit=np.zeros(B, np.int32), scalars=np.zeros(2, f))
        Ws = [np.ascontiguousarray(a, f) for a in (w.W_n2l, w.W_conv, w.W_h1, w.W_h2)]
        lab = [(_ptr(a) if label_csr is not None else None) for a in (label_csr or (None, None, None))]
        self.lib.orc_s2v_forward(N, B, K, C, H, Q, L, _ptr(a_csr[0]), _ptr(a_csr[1]), _ptr(a_csr[2]),
                                 _ptr(s_csr[0]), _ptr(s_csr[1]), _ptr(s_csr[2]), _ptr(X),
                                 _ptr(Ws[0]), _ptr(Ws[1]), _ptr(Ws[2]), _ptr(Ws[3]), lab[0], lab[1], lab[2],
                                 _ptr(out["msg"]), _ptr(out["h"]), _ptr(out["pool"]), _ptr(out["hidden"]),
                                 _ptr(out["logits"]), _ptr(out["probs"]), _ptr(out["loss_rows"]),
                                 _ptr(out["pred"]), _ptr(out["truth"]), _ptr(out["hit"]), _ptr(out["scalars"]))
        return out


@pytest.fixture(scope="session")
def oracle():
    return Oracle()


@pytest.fixture(scope="session")
def ref_graph():
    """The reference's own GraphStruct compiled into oracle/_ref (None when not built)."""
    if not os.path.exists(_REF_PATH):
        return None
    return ctypes.CDLL(_REF_PATH)


PARITY_TOL = 1e-4     # the north-star tolerance for fp32 activations and logits

# Floors of the parity metric, measured (test_oracle_pins.py repeats the sweep on every run): the smallest floor at which
# the oracle itself stays within 1e-4 of a float64 model of the same network on configurations 1 and 2
# (12 to 3,000 graphs) is 1.3e-3 of the tensor's largest magnitude for the embeddings and the hidden layer,
# 4e-5 for the pooled features and zero for the probabilities.  Two correct fp32 summation orders differ
# by the sum of two such errors, hence the values below.
FLOOR_DEFAULT = 2e-3          # fraction of max|ref|: embeddings, hidden layer, general sums
FLOOR_POOL = 1e-4             # fraction of max|ref|: pooled features (sums of non-negative terms)
FLOOR_PROBS_ABS = 1e-6        # absolute: probabilities


def max_rel(a, b, floor=None, floor_frac=FLOOR_DEFAULT):
    """Parity metric for fp32 tensors: max_i |a_i - b_i| / max(|a_i|, |b_i|, floor).

    floor (absolute) defaults to floor_frac times the reference tensor's largest magnitude.  A fixed tiny
    floor is not usable on post-ReLU activations and logits: they are sums with cancellation, so an element
    at 1e-4 of the tensor's scale legitimately differs by parts in 1e-3 between two correct fp32 summation
    orders (the oracle itself fails a 1e-6 floor against a float64 model, see worst_element).
    """
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    if a.size == 0:
        return 0.0
    if floor is None:
        floor = max(floor_frac * float(np.max(np.abs(b))), 1e-30)
    return float(np.max(np.abs(a - b) / np.maximum(np.maximum(np.abs(a), np.abs(b)), floor)))


def worst_element(a, b, floor=1e-6):
    """(relative error, flat index, a_i, b_i) of the worst element under a fixed absolute floor."""
    a = np.asarray(a, np.float64).ravel(); b = np.asarray(b, np.float64).ravel()
    if a.size == 0:
        return 0.0, -1, 0.0, 0.0
    rel = np.abs(a - b) / np.maximum(np.maximum(np.abs(a), np.abs(b)), floor)
    i = int(np.argmax(rel))
    return float(rel[i]), i, float(a[i]), float(b[i])


class Lazy:
    """A value computed on first use (float64 models are only needed when a comparison misses);
    lazy[key] is the lazily indexed value.  cond, when given, is a Lazy of the model's condition
    tensor (the same computation on absolute values), which assert_parity always checks."""

    def __init__(self, fn, cond=None):
        self._fn, self._done, self._val = fn, False, None
        self.cond = cond

    def __call__(self):
        if not self._done:
            self._val, self._done = self._fn(), True
        return self._val

    def __getitem__(self, key):
        return Lazy(lambda: self()[key], None if self.cond is None else Lazy(lambda: self.cond()[key]))


# Two correct fp32 evaluations of one sum are each a few 1e-5 to 1e-4 from float64 on the worst element of a
# large tensor under the floored metric, and which of the two is further is a coin toss (observed device/oracle
# ratios on the tests of this suite: 0.3 to 2.6; the matrix cores do not round partial sums the way a serial fp32
# loop does).  Where the device misses the oracle under the floors, the float64 arbiter accepts it when it is within
# the tolerance of float64, or at most this factor further from float64 than the oracle itself is.  (A fixed ceiling
# on top of that, say twice the tolerance, does not hold: on tensors whose floor is tight the oracle itself is three
# tolerances from float64.)  The arbiter is the weaker of two guards: every comparison that carries a float64 model
# is also held to the condition bound (assert_condition), which has neither floor nor slack, and a wrong index, a
# dropped term or reduced precision is off by orders of magnitude under either.
ARBITER_SLACK = 3.0

# What the run decided how: name -> worst |device - float64| / condition over the run (condition-aware check),
# and the comparisons that the float64 arbiter settled.  Printed at the end of the session.
CONDITION_WORST = {}
ARBITER_DECIDED = []


def condition_error(got, want64, cond):
    """max_i |got_i - want64_i| / cond_i, the error in units of the sum of the magnitudes of the terms that make
    up element i (cond = the same computation carried out on absolute values).  An fp32 evaluation of a sum of n
    terms is within n * 2^-24 of float64 in these units whatever the cancellation, so this metric has no floor and
    no blind band.  An element whose terms are all zero must be zero: any other value gives inf."""
    got = np.asarray(got, np.float64); want64 = np.asarray(want64, np.float64); cond = np.asarray(cond, np.float64)
    assert got.shape == want64.shape == cond.shape, (got.shape, want64.shape, cond.shape)
    if got.size == 0:
        return 0.0, -1
    err = np.abs(got - want64).ravel()
    c = cond.ravel()
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = np.where(err == 0, 0.0, err / c)
    ratio = np.where(np.isnan(ratio), np.inf, ratio)
    i = int(np.argmax(ratio))
    return float(ratio[i]), i


def assert_condition(name, got, want64, cond, tol=PARITY_TOL):
    """|device - float64| <= tol * (sum of |terms|), element by element: no floor, no slack."""
    worst, i = condition_error(got, want64, cond)
    kind = name.split()[0].rstrip(",:")
    CONDITION_WORST[kind] = max(CONDITION_WORST.get(kind, 0.0), worst)
    print("cond   %-10s worst |device - float64| / sum|terms| %.2e at [%d]" % (name, worst, i))
    assert worst <= tol, ("%s: element [%d] is %.3e of the sum of its terms' magnitudes away from float64 (bound %.1e): "
                          "device %.9g float64 %.9g sum|terms| %.9g"
                          % (name, i, worst, tol, np.asarray(got).ravel()[i], np.asarray(want64).ravel()[i],
                             np.asarray(cond).ravel()[i]))
    return worst


def assert_parity(name, got, want, want64=None, tol=PARITY_TOL, floor=None, floor_frac=FLOOR_DEFAULT):
    """got (device) against want (oracle) under max_rel; prints the worst element under the fixed 1e-6 floor.

    With want64 (a float64 model of the same computation, or a callable giving it) a miss is still a pass
    when the device is about as close to float64 as the oracle is (ARBITER_SLACK): both are then correct fp32 evaluations that differ in summation order on an element the
    floor does not cover.  When want64 carries a condition tensor (Lazy.cond), the device result is in addition
    held to |device - float64| <= tol * sum|terms| on every element (assert_condition), which has no floor."""
    cond = getattr(want64, "cond", None)
    if cond is not None:
        assert_condition(name, got, want64(), cond(), tol)
    err = max_rel(got, want, floor, floor_frac)
    rel, i, gi, wi = worst_element(got, want)
    print("parity %-10s max_rel %.2e (floor %s); worst element under the fixed 1e-6 floor: [%d] device %.9g oracle %.9g rel %.2e"
          % (name, err, ("%.1e" % floor) if floor is not None else ("%.0e x max|ref|" % floor_frac), i, gi, wi, rel))
    if err < tol:
        return err
    if want64 is not None:
        if callable(want64):
            want64 = want64()
        e_dev = max_rel(got, want64, floor, floor_frac)
        e_ref = max_rel(want, want64, floor, floor_frac)
        print("       %-10s vs float64: device %.2e, oracle %.2e" % (name, e_dev, e_ref))
        ARBITER_DECIDED.append((os.environ.get("PYTEST_CURRENT_TEST", "?").split(" ")[0], name, err, e_dev, e_ref))
        assert e_dev <= max(ARBITER_SLACK * e_ref, tol), \
            "%s: device %.3e from float64, oracle %.3e (device vs oracle %.3e)" % (name, e_dev, e_ref, err)
        return err
    raise AssertionError("%s differs from the oracle: max_rel %.3e >= %.1e" % (name, err, tol))


def pytest_terminal_summary(terminalreporter):
    if CONDITION_WORST:
        terminalreporter.write_line("condition-aware parity, worst |device - float64| / sum|terms| per tensor kind (bound %.0e):" % PARITY_TOL)
        for k in sorted(CONDITION_WORST):
            terminalreporter.write_line("  %-28s %.2e" % (k, CONDITION_WORST[k]))
    if ARBITER_DECIDED:
        terminalreporter.write_line("comparisons that missed the oracle under the floors and were settled by the float64 arbiter: %d" % len(ARBITER_DECIDED))
        for t, name, err, e_dev, e_ref in ARBITER_DECIDED:
            terminalreporter.write_line("  %s [%s]: device vs oracle %.2e; vs float64: device %.2e, oracle %.2e" % (t, name, err, e_dev, e_ref))


def forward_float64(a_csr, s_csr, X, w, L, magnitudes=False):
    """The network of kernel_mean_field.cpp:31-56 in float64 (scipy CSR products): the arbiter between two
    fp32 evaluations.  magnitudes=True evaluates the same network on absolute values (|A| |h| |W| + |msg|, and so
    on through pooling and the dense layers): element i of each tensor is then the sum of the magnitudes of every
    term that element i of the real tensor is made of, all the way back to the inputs, which bounds how far
    rounding can move it (ReLU is 1-Lipschitz).  For the probabilities the bound is the first-order propagation of
    the logits' bound through the softmax plus the softmax's own rounding: p_i (1 + c_i + sum_j p_j c_j)."""
    import scipy.sparse as sp
    N = X.shape[0]; B = len(s_csr[0]) - 1
    f8 = np.float64
    mag = np.abs if magnitudes else (lambda x: x)
    A = sp.csr_matrix((mag(a_csr[2].astype(f8)), a_csr[1], a_csr[0]), shape=(N, N))
    S = sp.csr_matrix((mag(s_csr[2].astype(f8)), s_csr[1], s_csr[0]), shape=(B, N))
    msg = mag(X.astype(f8)) @ mag(w.W_n2l.astype(f8))
    h = msg if magnitudes else np.maximum(msg, 0)
    hs = [h]
    for _ in range(L):
        z = (A @ h) @ mag(w.W_conv.astype(f8)) + msg
        h = z if magnitudes else np.maximum(z, 0)
        hs.append(h)
    pool = S @ h
    z = pool @ mag(w.W_h1.astype(f8))
    hidden = z if magnitudes else np.maximum(z, 0)
    logits = hidden @ mag(w.W_h2.astype(f8))
    if magnitudes:
        real = forward_float64(a_csr, s_csr, X, w, L)
        p = real["probs"]
        probs = p * (1.0 + logits + (p * logits).sum(axis=1, keepdims=True))
    else:
        e = np.exp(logits - logits.max(axis=1, keepdims=True))
        probs = e / e.sum(axis=1, keepdims=True)
    return dict(msg=msg, h=np.stack(hs), pool=pool, hidden=hidden, logits=logits, probs=probs)


def assert_stages(tag, a_csr, s_csr, X, w, dev, tol=PARITY_TOL):
    """Every stage of the network checked on its own: the stage is recomputed in float64 from the DEVICE's input to
    that stage and the device's output must lie within tol * sum|terms of that stage| of it, element by element
    (assert_condition: no floor).  Rounding carried over from earlier stages is in the input, so the bound is the
    stage's own: a few times 2^-24 per term for a correct fp32 evaluation.
    dev: device arrays by name; any of msg, h (all levels [L+1,N,C]), h_final, pool, hidden, logits, probs; a stage is
    checked when its input and its output are both there."""
    import scipy.sparse as sp
    f8 = np.float64
    d = {k: np.asarray(v, f8) for k, v in dev.items()}
    N = X.shape[0]; B = len(s_csr[0]) - 1
    W = {k: getattr(w, k).astype(f8) for k in ("W_n2l", "W_conv", "W_h1", "W_h2")}
    if "msg" in d:
        assert_condition("msg%s, stage" % tag, d["msg"], X.astype(f8) @ W["W_n2l"], np.abs(X.astype(f8)) @ np.abs(W["W_n2l"]), tol)
    if "h" in d and "msg" in d:
        # (scipy's abs() merges repeated coordinates in place, in the caller's index arrays too: build |A| from the data)
        A = sp.csr_matrix((a_csr[2].astype(f8), a_csr[1], a_csr[0]), shape=(N, N))
        A_mag = sp.csr_matrix((np.abs(a_csr[2].astype(f8)), a_csr[1], a_csr[0]), shape=(N, N))
        assert np.array_equal(d["h"][0], np.maximum(d["msg"], 0)), "h0 is not ReLU(msg)"
        for l in range(1, d["h"].shape[0]):
            z = (A @ d["h"][l - 1]) @ W["W_conv"] + d["msg"]
            c = (A_mag @ np.abs(d["h"][l - 1])) @ np.abs(W["W_conv"]) + np.abs(d["msg"])
            assert_condition("h%d%s, stage" % (l, tag), d["h"][l], np.maximum(z, 0), c, tol)
    h_final = d["h"][-1] if "h" in d else d.get("h_final")
    if h_final is not None and "pool" in d:
        S = sp.csr_matrix((s_csr[2].astype(f8), s_csr[1], s_csr[0]), shape=(B, N))
        S_mag = sp.csr_matrix((np.abs(s_csr[2].astype(f8)), s_csr[1], s_csr[0]), shape=(B, N))
        assert_condition("pool%s, stage" % tag, d["pool"], S @ h_final, S_mag @ np.abs(h_final), tol)
    if "pool" in d and "hidden" in d:
        assert_condition("hidden%s, stage" % tag, d["hidden"], np.maximum(d["pool"] @ W["W_h1"], 0), np.abs(d["pool"]) @ np.abs(W["W_h1"]), tol)
    if "hidden" in d and "logits" in d:
        assert_condition("logits%s, stage" % tag, d["logits"], d["hidden"] @ W["W_h2"], np.abs(d["hidden"]) @ np.abs(W["W_h2"]), tol)
    if "logits" in d and "probs" in d:
        x = d["logits"]
        e = np.exp(x - x.max(axis=1, keepdims=True))
        p = e / e.sum(axis=1, keepdims=True)
        # the shifted arguments carry a rounding error of up to 2^-24 (|x_i| + max|x|), which scales p_i by its exponential
        assert_condition("probs%s, stage" % tag, d["probs"], p, p * (1.0 + 2.0 * np.abs(x).max(axis=1, keepdims=True)), tol)


@pytest.fixture(scope="session")
def gpu():
    """torch CUDA device + initialised gnnhip library; GPU tests fail loudly without either."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a HIP device"
    from graphnn_amd import ops
    ops.init(0)
    return torch.device("cuda:0")
