"""Thin torch-pointer helpers over the C ABI (used by the tests, the smoke check and the bench).

torch supplies device memory and the stream; all arithmetic happens in libgnnhip.so.
Every helper validates dtype / device / contiguity on the host before a pointer
reaches a kernel, and raises GnnHipError on a non-zero status.
"""
import ctypes
import numpy as np

import torch

from ._lib import check, load_library

UNARY = {
    "set": 0, "truncate": 1, "scale": 2, "add": 3, "abs": 4, "inv": 5, "relu": 6, "sigmoid": 7,
    "tanh": 8, "log": 9, "invsqrt": 10, "exp": 11, "square": 12, "sqrt": 13,
}
REDUCE = {"sum": 0, "mean": 1, "max": 2, "sumsq": 3}

_initialised = False


def init(device_id=0):
    global _initialised
    lib = load_library()
    check(lib.gnnhip_init(int(device_id)))
    _initialised = True
    return lib


def _lib():
    if not _initialised:
        init(torch.cuda.current_device())
    return load_library()


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _f32(t, name):
    if t is None:
        return None
    if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous()):
        raise ValueError("%s must be a contiguous float32 CUDA tensor" % name)
    return ctypes.c_void_p(t.data_ptr())


def _i32(t, name):
    if t is None:
        return None
    if not (t.is_cuda and t.dtype == torch.int32 and t.is_contiguous()):
        raise ValueError("%s must be a contiguous int32 CUDA tensor" % name)
    return ctypes.c_void_p(t.data_ptr())


def _check_csr(row_ptr, col_idx, val, rows, name):
    if row_ptr.numel() != rows + 1:
        raise ValueError("%s.row_ptr must have rows+1 = %d entries" % (name, rows + 1))
    if col_idx.numel() != val.numel():
        raise ValueError("%s: col_idx and val differ in length" % name)


def spmm(row_ptr, col_idx, val, B, m, alpha=1.0, beta=0.0, out=None, nnz_hint=None):
    """out[m,n] = alpha * A * B + beta * out, A CSR with m rows and B.shape[0] columns.
    nnz_hint: the host-side entry count handed to the library (default: the arrays' length); it only sizes
    scratch, so any value from 0 up must give the same values."""
    k, n = B.shape
    _check_csr(row_ptr, col_idx, val, m, "A")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=B.device)
    elif tuple(out.shape) != (m, n):
        raise ValueError("out has the wrong shape")
    nnz = int(col_idx.numel()) if nnz_hint is None else int(nnz_hint)
    check(_lib().gnnhip_spmm_csr_f32(m, k, n, nnz, alpha, _i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"),
                                     _f32(val, "val"), _f32(B, "B"), n, beta, _f32(out, "out"), n, _stream()))
    return out


class CsrPlan:
    """gnnhip_csr_plan_create for a CSR matrix [m, k] held in torch tensors, which the plan keeps alive; close() (or
    the end of a `with` block) destroys it.  spmm / level run the planned entry points."""

    def __init__(self, row_ptr, col_idx, val, m, k):
        _check_csr(row_ptr, col_idx, val, m, "A")
        self.m, self.k = int(m), int(k)
        self._keep = (row_ptr, col_idx, val)
        h = ctypes.c_void_p()
        check(_lib().gnnhip_csr_plan_create(self.m, self.k, _i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"), _f32(val, "val"),
                                            _stream(), ctypes.byref(h)))
        self.handle = h

    def bytes(self):
        n = ctypes.c_size_t()
        check(_lib().gnnhip_csr_plan_bytes(self.handle, ctypes.byref(n)))
        return int(n.value)

    def spmm(self, B, alpha=1.0, beta=0.0, out=None):
        k, n = B.shape
        if k != self.k:
            raise ValueError("B must have %d rows" % self.k)
        if out is None:
            out = torch.empty((self.m, n), dtype=torch.float32, device=B.device)
        elif tuple(out.shape) != (self.m, n):
            raise ValueError("out has the wrong shape")
        check(_lib().gnnhip_spmm_csr_planned_f32(self.handle, n, alpha, _f32(B, "B"), n, beta, _f32(out, "out"), n, _stream()))
        return out

    def level(self, h_in, W, msg=None, bias=None, out=None):
        N, C = h_in.shape
        if N != self.m or tuple(W.shape) != (C, C):
            raise ValueError("h_in must be [m,C] and W [C,C]")
        if out is None:
            out = torch.empty_like(h_in)
        check(_lib().gnnhip_s2v_level_planned_f32(self.handle, C, _f32(h_in, "h_in"), _f32(W, "W"), _f32(msg, "msg"),
                                                  _f32(bias, "bias"), _f32(out, "out"), _stream()))
        return out

    def close(self):
        if self.handle is not None:
            check(_lib().gnnhip_csr_plan_destroy(self.handle))
            self.handle = None
            self._keep = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def release_scratch():
    """gives the current stream's library scratch back to the driver"""
    check(_lib().gnnhip_release_scratch(_stream()))


def gemm(A, B, transA=False, transB=False, alpha=1.0, beta=0.0, out=None, cols_a=None, cols_b=None):
    """cols_a / cols_b: use only the first so many columns of the stored A / B (the row stride stays the tensor's)"""
    ca = A.shape[1] if cols_a is None else int(cols_a)
    cb = B.shape[1] if cols_b is None else int(cols_b)
    if not (0 <= ca <= A.shape[1] and 0 <= cb <= B.shape[1]):
        raise ValueError("cols_a / cols_b out of range")
    m = ca if transA else A.shape[0]
    k = A.shape[0] if transA else ca
    kb = cb if transB else B.shape[0]
    n = B.shape[0] if transB else cb
    if k != kb:
        raise ValueError("mat dim doesn't match")
    if out is None:
        out = torch.empty((m, n), dtype=torch.float32, device=A.device)
    elif tuple(out.shape) != (m, n):
        raise ValueError("out has the wrong shape")
    check(_lib().gnnhip_gemm_f32(int(transA), int(transB), m, n, k, alpha, _f32(A, "A"), A.shape[1],
                                 _f32(B, "B"), B.shape[1], beta, _f32(out, "out"), n, _stream()))
    return out


def read_scalars(tensors):
    """the first element of each device tensor, all behind one wait for the stream"""
    n = len(tensors)
    outs = [np.zeros(1, np.float32 if t.dtype == torch.float32 else np.int32) for t in tensors]
    P = ctypes.c_void_p * n
    check(_lib().gnnhip_memcpy_d2h_batch(n, P(*[o.ctypes.data for o in outs]), P(*[t.data_ptr() for t in tensors]),
                                         (ctypes.c_size_t * n)(*[4] * n), _stream()))
    return [o[0] for o in outs]


def row_softmax_deriv(dst, out, grad):
    """dst += out * (grad - <grad, out> per row), in place on dst"""
    rows, cols = out.shape
    check(_lib().gnnhip_row_softmax_deriv_f32(_f32(dst, "dst"), _f32(out, "out"), _f32(grad, "grad"), rows, cols, _stream()))
    return dst


def gemm_tn_batch(products, alpha=1.0, beta=0.0):
    """products: list of (A [k,m], B [k,n], out [m,n]); out = alpha * A^T B + beta * out for all of them in two launches"""
    import ctypes
    count = len(products)
    ints = lambda vals: (ctypes.c_int * count)(*vals)
    ptrs = lambda ts: (ctypes.c_void_p * count)(*[t.data_ptr() for t in ts])
    for A, B, out in products:
        if A.shape[0] != B.shape[0] or tuple(out.shape) != (A.shape[1], B.shape[1]):
            raise ValueError("mat dim doesn't match")
        _f32(A, "A"), _f32(B, "B"), _f32(out, "out")
    As, Bs, Cs = zip(*products) if count else ((), (), ())
    check(_lib().gnnhip_gemm_tn_batch_f32(count, ints([a.shape[1] for a in As]), ints([b.shape[1] for b in Bs]),
                                          ints([a.shape[0] for a in As]), ptrs(As), ints([a.shape[1] for a in As]),
                                          ptrs(Bs), ints([b.shape[1] for b in Bs]), alpha, beta, ptrs(Cs),
                                          ints([c.shape[1] for c in Cs]), _stream()))
    return [c for c in Cs]


def s2v_input(X, W_n2l):
    N, K = X.shape
    if W_n2l.shape[0] != K:
        raise ValueError("X and W_n2l disagree on the label width")
    C = W_n2l.shape[1]
    msg = torch.empty((N, C), dtype=torch.float32, device=X.device)
    h0 = torch.empty_like(msg)
    check(_lib().gnnhip_s2v_input_f32(N, K, C, _f32(X, "X"), _f32(W_n2l, "W_n2l"), _f32(msg, "msg"),
                                      _f32(h0, "h0"), _stream()))
    return msg, h0


def s2v_input_labels(label, W_n2l, status=None):
    """msg = W_n2l[label], h0 = ReLU(msg): the input stage from one int label per node."""
    N = label.numel()
    K, C = W_n2l.shape
    msg = torch.empty((N, C), dtype=torch.float32, device=W_n2l.device)
    h0 = torch.empty_like(msg)
    check(_lib().gnnhip_s2v_input_labels_f32(N, K, C, _i32(label, "label"), _f32(W_n2l, "W_n2l"), _f32(msg, "msg"),
                                             _f32(h0, "h0"), _i32(status, "status"), _stream()))
    return msg, h0


def s2v_level(row_ptr, col_idx, val, h_in, W, msg=None, bias=None, out=None, nnz_hint=None):
    """nnz_hint: the host-side entry count handed to the library (default: the arrays' length); it only
    sizes scratch, so any value from 0 up must give the same result."""
    N, C = h_in.shape
    _check_csr(row_ptr, col_idx, val, N, "A")
    if tuple(W.shape) != (C, C):
        raise ValueError("W must be [C,C]")
    if msg is not None and tuple(msg.shape) != (N, C):
        raise ValueError("msg must be [N,C]")
    if bias is not None and bias.numel() != C:
        raise ValueError("bias must have C entries")
    if out is None:
        out = torch.empty_like(h_in)
    nnz = int(col_idx.numel()) if nnz_hint is None else int(nnz_hint)
    check(_lib().gnnhip_s2v_level_f32(N, C, nnz, _i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"), _f32(val, "val"),
                                      _f32(h_in, "h_in"), _f32(W, "W"), _f32(msg, "msg"), _f32(bias, "bias"),
                                      _f32(out, "out"), _stream()))
    return out


def s2v_readout(s_row_ptr, s_col_idx, s_val, h, W_h1, W_h2, B):
    N, C = h.shape
    H, Q = W_h1.shape[1], W_h2.shape[1]
    _check_csr(s_row_ptr, s_col_idx, s_val, B, "S")
    if W_h1.shape[0] != C or W_h2.shape[0] != H:
        raise ValueError("readout weight shapes do not chain")
    dev = h.device
    pool = torch.empty((B, C), dtype=torch.float32, device=dev)
    hidden = torch.empty((B, H), dtype=torch.float32, device=dev)
    logits = torch.empty((B, Q), dtype=torch.float32, device=dev)
    probs = torch.empty((B, Q), dtype=torch.float32, device=dev)
    pred = torch.empty((B,), dtype=torch.int32, device=dev)
    check(_lib().gnnhip_s2v_readout_f32(B, N, C, H, Q, _i32(s_row_ptr, "s_row_ptr"), _i32(s_col_idx, "s_col_idx"),
                                        _f32(s_val, "s_val"), _f32(h, "h"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
                                        _f32(pool, "pool"), _f32(hidden, "hidden"), _f32(logits, "logits"),
                                        _f32(probs, "probs"), _i32(pred, "pred"), _stream()))
    return pool, hidden, logits, probs, pred


class ForwardBuffers:
    """Caller-owned activations of one forward; allocated once and reused across calls."""

    def __init__(self, N, B, C, H, Q, device):
        f = dict(dtype=torch.float32, device=device)
        self.msg = torch.empty((N, C), **f)
        self.h_a = torch.empty((N, C), **f)
        self.h_b = torch.empty((N, C), **f)
        self.pool = torch.empty((B, C), **f)
        self.hidden = torch.empty((B, H), **f)
        self.logits = torch.empty((B, Q), **f)
        self.probs = torch.empty((B, Q), **f)
        self.pred = torch.empty((B,), dtype=torch.int32, device=device)
        self.which = ctypes.c_int(0)

    @property
    def h_final(self):
        return self.h_a if self.which.value == 0 else self.h_b


def s2v_forward(a_csr, s_csr, X, W_n2l, W_conv, W_h1, W_h2, L, bufs=None):
    """Whole forward.  a_csr / s_csr are (row_ptr, col_idx, val) triples of int32/int32/float32 device tensors."""
    N, K = X.shape
    C, H, Q = W_n2l.shape[1], W_h1.shape[1], W_h2.shape[1]
    B = s_csr[0].numel() - 1
    _check_csr(a_csr[0], a_csr[1], a_csr[2], N, "A")
    _check_csr(s_csr[0], s_csr[1], s_csr[2], B, "S")
    if W_n2l.shape[0] != K or tuple(W_conv.shape) != (C, C) or W_h1.shape[0] != C or W_h2.shape[0] != H:
        raise ValueError("weight shapes do not chain")
    if bufs is None:
        bufs = ForwardBuffers(N, B, C, H, Q, X.device)
    check(_lib().gnnhip_s2v_forward_f32(
        N, B, K, C, H, Q, L, int(a_csr[1].numel()),
        _i32(a_csr[0], "a_row_ptr"), _i32(a_csr[1], "a_col_idx"), _f32(a_csr[2], "a_val"),
        _i32(s_csr[0], "s_row_ptr"), _i32(s_csr[1], "s_col_idx"), _f32(s_csr[2], "s_val"),
        _f32(X, "X"), _f32(W_n2l, "W_n2l"), _f32(W_conv, "W_conv"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
        _f32(bufs.msg, "msg"), _f32(bufs.h_a, "h_a"), _f32(bufs.h_b, "h_b"), _f32(bufs.pool, "pool"),
        _f32(bufs.hidden, "hidden"), _f32(bufs.logits, "logits"), _f32(bufs.probs, "probs"),
        _i32(bufs.pred, "pred"), ctypes.byref(bufs.which), _stream()))
    return bufs


def s2v_forward_planned(plan, s_csr, X, W_n2l, W_conv, W_h1, W_h2, L, bufs=None):
    """Whole forward with a CsrPlan of A (gnnhip_s2v_forward_planned_f32)."""
    N, K = X.shape
    C, H, Q = W_n2l.shape[1], W_h1.shape[1], W_h2.shape[1]
    B = s_csr[0].numel() - 1
    if N != plan.m or plan.m != plan.k:
        raise ValueError("the plan must be of the [N,N] adjacency")
    _check_csr(s_csr[0], s_csr[1], s_csr[2], B, "S")
    if W_n2l.shape[0] != K or tuple(W_conv.shape) != (C, C) or W_h1.shape[0] != C or W_h2.shape[0] != H:
        raise ValueError("weight shapes do not chain")
    if bufs is None:
        bufs = ForwardBuffers(N, B, C, H, Q, X.device)
    check(_lib().gnnhip_s2v_forward_planned_f32(
        plan.handle, B, K, C, H, Q, L,
        _i32(s_csr[0], "s_row_ptr"), _i32(s_csr[1], "s_col_idx"), _f32(s_csr[2], "s_val"),
        _f32(X, "X"), _f32(W_n2l, "W_n2l"), _f32(W_conv, "W_conv"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
        _f32(bufs.msg, "msg"), _f32(bufs.h_a, "h_a"), _f32(bufs.h_b, "h_b"), _f32(bufs.pool, "pool"),
        _f32(bufs.hidden, "hidden"), _f32(bufs.logits, "logits"), _f32(bufs.probs, "probs"),
        _i32(bufs.pred, "pred"), ctypes.byref(bufs.which), _stream()))
    return bufs


class BatchedBuffers:
    """Caller-owned outputs of the graph-resident forward."""

    def __init__(self, N, B, C, H, Q, device):
        f = dict(dtype=torch.float32, device=device)
        self.msg = torch.empty((N, C), **f)
        self.h_final = torch.empty((N, C), **f)
        self.pool = torch.empty((B, C), **f)
        self.hidden = torch.empty((B, H), **f)
        self.logits = torch.empty((B, Q), **f)
        self.probs = torch.empty((B, Q), **f)
        self.pred = torch.empty((B,), dtype=torch.int32, device=device)
        self.status = torch.zeros((1,), dtype=torch.int32, device=device)


def s2v_forward_batched(a_csr, s_csr, X, W_n2l, W_conv, W_h1, W_h2, L, max_graph_nodes, bufs=None):
    """One-launch forward for block-diagonal batches (see gnnhip_s2v_forward_batched_f32)."""
    N, K = X.shape
    C, H, Q = W_n2l.shape[1], W_h1.shape[1], W_h2.shape[1]
    B = s_csr[0].numel() - 1
    _check_csr(a_csr[0], a_csr[1], a_csr[2], N, "A")
    _check_csr(s_csr[0], s_csr[1], s_csr[2], B, "S")
    if s_csr[1].numel() != N:
        raise ValueError("S must list every node exactly once")
    if W_n2l.shape[0] != K or tuple(W_conv.shape) != (C, C) or W_h1.shape[0] != C or W_h2.shape[0] != H:
        raise ValueError("weight shapes do not chain")
    if bufs is None:
        bufs = BatchedBuffers(N, B, C, H, Q, X.device)
    check(_lib().gnnhip_s2v_forward_batched_f32(
        N, B, K, C, H, Q, L, int(max_graph_nodes),
        _i32(a_csr[0], "a_row_ptr"), _i32(a_csr[1], "a_col_idx"), _f32(a_csr[2], "a_val"),
        _i32(s_csr[0], "s_row_ptr"), _i32(s_csr[1], "s_col_idx"), _f32(s_csr[2], "s_val"),
        _f32(X, "X"), _f32(W_n2l, "W_n2l"), _f32(W_conv, "W_conv"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
        _f32(bufs.msg, "msg"), _f32(bufs.h_final, "h_final"), _f32(bufs.pool, "pool"),
        _f32(bufs.hidden, "hidden"), _f32(bufs.logits, "logits"), _f32(bufs.probs, "probs"),
        _i32(bufs.pred, "pred"), _i32(bufs.status, "status"), _stream()))
    return bufs


def s2v_forward_batched_train(a_csr, s_csr, X, W_n2l, W_conv, W_h1, W_h2, L, max_graph_nodes, bufs=None):
    """The one-launch forward that keeps every level: returns (bufs, h_levels [(L + 1), N, C]); bufs.h_final is
    not written (h_levels[L] is that embedding)."""
    N, K = X.shape
    C, H, Q = W_n2l.shape[1], W_h1.shape[1], W_h2.shape[1]
    B = s_csr[0].numel() - 1
    _check_csr(a_csr[0], a_csr[1], a_csr[2], N, "A")
    _check_csr(s_csr[0], s_csr[1], s_csr[2], B, "S")
    if s_csr[1].numel() != N:
        raise ValueError("S must list every node exactly once")
    if W_n2l.shape[0] != K or tuple(W_conv.shape) != (C, C) or W_h1.shape[0] != C or W_h2.shape[0] != H:
        raise ValueError("weight shapes do not chain")
    if bufs is None:
        bufs = BatchedBuffers(N, B, C, H, Q, X.device)
    h_levels = torch.empty((L + 1, N, C), dtype=torch.float32, device=X.device)
    check(_lib().gnnhip_s2v_forward_batched_train_f32(
        N, B, K, C, H, Q, L, int(max_graph_nodes),
        _i32(a_csr[0], "a_row_ptr"), _i32(a_csr[1], "a_col_idx"), _f32(a_csr[2], "a_val"),
        _i32(s_csr[0], "s_row_ptr"), _i32(s_csr[1], "s_col_idx"), _f32(s_csr[2], "s_val"),
        _f32(X, "X"), _f32(W_n2l, "W_n2l"), _f32(W_conv, "W_conv"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
        _f32(bufs.msg, "msg"), _f32(h_levels, "h_levels"), _f32(bufs.pool, "pool"),
        _f32(bufs.hidden, "hidden"), _f32(bufs.logits, "logits"), _f32(bufs.probs, "probs"),
        _i32(bufs.pred, "pred"), _i32(bufs.status, "status"), _stream()))
    return bufs, h_levels


def bind_s2v_forward_batched(a_csr, s_csr, X, W_n2l, W_conv, W_h1, W_h2, L, max_graph_nodes, bufs, stream):
    """The call of s2v_forward_batched with every argument converted once: returns a function that queues one
    forward on `stream` (a torch.cuda.Stream) and raises on a non-zero status code.  For callers that keep several
    batches in flight on several streams, where the per-call argument checks of the helper above would be the
    bottleneck."""
    N, K = X.shape
    C, H, Q = W_n2l.shape[1], W_h1.shape[1], W_h2.shape[1]
    B = s_csr[0].numel() - 1
    _check_csr(a_csr[0], a_csr[1], a_csr[2], N, "A")
    _check_csr(s_csr[0], s_csr[1], s_csr[2], B, "S")
    if s_csr[1].numel() != N:
        raise ValueError("S must list every node exactly once")
    if W_n2l.shape[0] != K or tuple(W_conv.shape) != (C, C) or W_h1.shape[0] != C or W_h2.shape[0] != H:
        raise ValueError("weight shapes do not chain")
    fn = _lib().gnnhip_s2v_forward_batched_f32
    args = (N, B, K, C, H, Q, L, int(max_graph_nodes),
            _i32(a_csr[0], "a_row_ptr"), _i32(a_csr[1], "a_col_idx"), _f32(a_csr[2], "a_val"),
            _i32(s_csr[0], "s_row_ptr"), _i32(s_csr[1], "s_col_idx"), _f32(s_csr[2], "s_val"),
            _f32(X, "X"), _f32(W_n2l, "W_n2l"), _f32(W_conv, "W_conv"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
            _f32(bufs.msg, "msg"), _f32(bufs.h_final, "h_final"), _f32(bufs.pool, "pool"),
            _f32(bufs.hidden, "hidden"), _f32(bufs.logits, "logits"), _f32(bufs.probs, "probs"),
            _i32(bufs.pred, "pred"), _i32(bufs.status, "status"), ctypes.c_void_p(stream.cuda_stream))

    def queue():
        rc = fn(*args)
        if rc:
            check(rc)
    return queue


def s2v_forward_batched_labels(a_csr, s_csr, label, W_n2l, W_conv, W_h1, W_h2, L, max_graph_nodes, bufs=None):
    """One-launch forward from one int label per node (see gnnhip_s2v_forward_batched_labels_f32)."""
    N = label.numel()
    K, C = W_n2l.shape
    H, Q = W_h1.shape[1], W_h2.shape[1]
    B = s_csr[0].numel() - 1
    _check_csr(a_csr[0], a_csr[1], a_csr[2], N, "A")
    _check_csr(s_csr[0], s_csr[1], s_csr[2], B, "S")
    if s_csr[1].numel() != N:
        raise ValueError("S must list every node exactly once")
    if tuple(W_conv.shape) != (C, C) or W_h1.shape[0] != C or W_h2.shape[0] != H:
        raise ValueError("weight shapes do not chain")
    if bufs is None:
        bufs = BatchedBuffers(N, B, C, H, Q, W_n2l.device)
    check(_lib().gnnhip_s2v_forward_batched_labels_f32(
        N, B, K, C, H, Q, L, int(max_graph_nodes),
        _i32(a_csr[0], "a_row_ptr"), _i32(a_csr[1], "a_col_idx"), _f32(a_csr[2], "a_val"),
        _i32(s_csr[0], "s_row_ptr"), _i32(s_csr[1], "s_col_idx"), _f32(s_csr[2], "s_val"),
        _i32(label, "label"), _f32(W_n2l, "W_n2l"), _f32(W_conv, "W_conv"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
        _f32(bufs.msg, "msg"), _f32(bufs.h_final, "h_final"), _f32(bufs.pool, "pool"),
        _f32(bufs.hidden, "hidden"), _f32(bufs.logits, "logits"), _f32(bufs.probs, "probs"),
        _i32(bufs.pred, "pred"), _i32(bufs.status, "status"), _stream()))
    return bufs


def unary(op, x, a0=0.0, a1=0.0):
    check(_lib().gnnhip_unary_f32(UNARY[op], _f32(x, "x"), x.numel(), a0, a1, _stream()))
    return x


def relu(x, out=None):
    if out is None:
        out = torch.empty_like(x)
    check(_lib().gnnhip_relu_f32(_f32(x, "x"), _f32(out, "out"), x.numel(), _stream()))
    return out


def axpy(a, x, y):
    if x.numel() != y.numel():
        raise ValueError("shape doesn't match in Axpy")
    check(_lib().gnnhip_axpy_f32(x.numel(), a, _f32(x, "x"), _f32(y, "y"), _stream()))
    return y


def axpby(a, x, b, y):
    if x.numel() != y.numel():
        raise ValueError("shape doesn't match in Axpby")
    check(_lib().gnnhip_axpby_f32(x.numel(), a, _f32(x, "x"), b, _f32(y, "y"), _stream()))
    return y


def add(a, b, out=None):
    if a.numel() != b.numel():
        raise ValueError("no broadcasting is supported")
    if out is None:
        out = torch.empty_like(a)
    check(_lib().gnnhip_add_f32(a.numel(), _f32(a, "a"), _f32(b, "b"), _f32(out, "out"), _stream()))
    return out


def row_softmax(x):
    rows, cols = x.shape
    check(_lib().gnnhip_row_softmax_f32(_f32(x, "x"), rows, cols, _stream()))
    return x


def jagged_softmax(x, lens):
    check(_lib().gnnhip_jagged_softmax_f32(_f32(x, "x"), _i32(lens, "lens"), lens.numel(), _stream()))
    return x


def jagged_softmax_deriv(dst, out, grad, lens):
    """dst += (grad - <grad, out> per segment) * out"""
    check(_lib().gnnhip_jagged_softmax_deriv_f32(_f32(dst, "dst"), _f32(out, "out"), _f32(grad, "grad"), _i32(lens, "lens"),
                                                 lens.numel(), _stream()))
    return dst


def jagged_softmax_static(x, lens):
    """gnnhip_jagged_softmax_static_f32: the same result, segment offsets in the library's static array."""
    check(_lib().gnnhip_jagged_softmax_static_f32(_f32(x, "x"), _i32(lens, "lens"), lens.numel(), _stream()))
    return x


def reduce(op, x):
    out = torch.empty((1,), dtype=torch.float32, device=x.device)
    check(_lib().gnnhip_reduce_f32(REDUCE[op], _f32(x, "x"), x.numel(), _f32(out, "out"), _stream()))
    return out


def row_argmax(x):
    rows, cols = x.shape
    out = torch.empty((rows,), dtype=torch.int32, device=x.device)
    check(_lib().gnnhip_row_argmax_f32(_f32(x, "x"), rows, cols, _i32(out, "out"), _stream()))
    return out


def csr_row_argmax(row_ptr, col_idx, val):
    rows = row_ptr.numel() - 1
    out = torch.empty((rows,), dtype=torch.int32, device=row_ptr.device)
    check(_lib().gnnhip_csr_row_argmax_f32(_i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"), _f32(val, "val"),
                                           rows, _i32(out, "out"), _stream()))
    return out


def cross_entropy(prob, l_row_ptr, l_col_idx, l_val):
    rows, cols = prob.shape
    _check_csr(l_row_ptr, l_col_idx, l_val, rows, "label")
    out = torch.empty((rows, 1), dtype=torch.float32, device=prob.device)
    check(_lib().gnnhip_cross_entropy_f32(_f32(prob, "prob"), rows, cols, _i32(l_row_ptr, "l_row_ptr"),
                                          _i32(l_col_idx, "l_col_idx"), _f32(l_val, "l_val"), _f32(out, "out"),
                                          _stream()))
    return out


def in_top_k(pred, label, k=1):
    rows, cols = pred.shape
    if label.numel() != rows:
        raise ValueError("# instances doesn't match")
    out = torch.empty((rows,), dtype=torch.int32, device=pred.device)
    check(_lib().gnnhip_in_top_k_f32(_f32(pred, "pred"), _i32(label, "label"), rows, cols, k, _i32(out, "out"),
                                     _stream()))
    return out


def cast_i32_f32(src):
    dst = torch.empty(src.shape, dtype=torch.float32, device=src.device)
    check(_lib().gnnhip_cast_i32_f32(_i32(src, "src"), _f32(dst, "dst"), src.numel(), _stream()))
    return dst


def memset0(t):
    check(_lib().gnnhip_memset0(ctypes.c_void_p(t.data_ptr()), t.numel() * t.element_size(), _stream()))
    return t


def memset0_batch(tensors):
    """zero-fill several device buffers in one launch"""
    n = len(tensors)
    ptrs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in tensors])
    sizes = (ctypes.c_size_t * n)(*[t.numel() * t.element_size() for t in tensors])
    check(_lib().gnnhip_memset0_batch(n, ptrs, sizes, _stream()))
    return tensors


# ---- backward-pass entry points
def spmm_t(row_ptr, col_idx, val, B, m, k, alpha=1.0, beta=0.0, out=None):
    """out[k,n] = alpha * A^T * B + beta * out, A CSR [m,k], B [m,n]"""
    n = B.shape[1]
    _check_csr(row_ptr, col_idx, val, m, "A")
    if B.shape[0] != m:
        raise ValueError("mat dim doesn't match")
    if out is None:
        out = torch.zeros((k, n), dtype=torch.float32, device=B.device)
    check(_lib().gnnhip_spmm_csr_t_f32(m, k, n, alpha, _i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"),
                                       _f32(val, "val"), _f32(B, "B"), n, beta, _f32(out, "out"), n, _stream()))
    return out


def csr_axpy(a, row_ptr, col_idx, val, dense):
    rows, cols = dense.shape
    _check_csr(row_ptr, col_idx, val, rows, "x")
    check(_lib().gnnhip_csr_axpy_f32(rows, cols, a, _i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"), _f32(val, "val"),
                                     _f32(dense, "dense"), _stream()))
    return dense


def relu_deriv(dst, out, grad):
    if not (dst.numel() == out.numel() == grad.numel()):
        raise ValueError("shape mismatch in ReLUDeriv")
    check(_lib().gnnhip_relu_deriv_f32(dst.numel(), _f32(out, "out"), _f32(grad, "grad"), _f32(dst, "dst"), _stream()))
    return dst


def mul(x, y):
    if x.numel() != y.numel():
        raise ValueError("shape mismatch in ElewiseMul")
    check(_lib().gnnhip_mul_f32(x.numel(), _f32(x, "x"), _f32(y, "y"), _stream()))
    return y


def row_scale(scale, y):
    rows, cols = y.shape
    if scale.numel() != rows:
        raise ValueError("one factor per row is needed")
    check(_lib().gnnhip_row_scale_f32(rows, cols, _f32(scale, "scale"), _f32(y, "y"), _stream()))
    return y


# ---- device-side CSR construction
def csr_group(rows, key, payload, average=False, key_stride=1, payload_stride=1, n=None):
    """row i lists payload[e] of the pairs with key[e] == i in input order (device arrays, int32)"""
    if n is None:
        n = key.numel() // key_stride
    dev = key.device
    row_ptr = torch.empty(rows + 1, dtype=torch.int32, device=dev)
    col_idx = torch.empty(n, dtype=torch.int32, device=dev)
    val = torch.empty(n, dtype=torch.float32, device=dev)
    check(_lib().gnnhip_csr_group_i32(rows, n, _i32(key, "key"), key_stride, _i32(payload, "payload"), payload_stride,
                                      int(average), _i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"), _f32(val, "val"), _stream()))
    return row_ptr, col_idx, val


def csr_group_both(rows, x, y, x_stride=1, y_stride=1, n=None):
    """the pairs (x, y) grouped by y (row i lists x) and by x (row i lists y): a matrix and its transpose, values 1"""
    if n is None:
        n = x.numel() // x_stride
    dev = x.device
    out = []
    for _ in range(2):
        out += [torch.empty(rows + 1, dtype=torch.int32, device=dev), torch.empty(n, dtype=torch.int32, device=dev),
                torch.empty(n, dtype=torch.float32, device=dev)]
    check(_lib().gnnhip_csr_group_both_i32(rows, n, _i32(x, "x"), x_stride, _i32(y, "y"), y_stride,
                                           _i32(out[0], "row_ptr"), _i32(out[1], "col_idx"), _f32(out[2], "val"),
                                           _i32(out[3], "t_row_ptr"), _i32(out[4], "t_col_idx"), _f32(out[5], "t_val"), _stream()))
    return tuple(out[:3]), tuple(out[3:])


def csr_consecutive_rows(row_ptr, average=False):
    """col_idx, val of the CSR matrix whose row i lists the columns row_ptr[i] .. row_ptr[i+1]-1 (row_ptr on the device)"""
    rows = row_ptr.numel() - 1
    n = int(row_ptr[-1].item())
    col_idx = torch.empty(n, dtype=torch.int32, device=row_ptr.device)
    val = torch.empty(n, dtype=torch.float32, device=row_ptr.device)
    check(_lib().gnnhip_csr_consecutive_rows_f32(rows, _i32(row_ptr, "row_ptr"), int(average), _i32(col_idx, "col_idx"),
                                                 _f32(val, "val"), _stream()))
    return col_idx, val


def csr_consecutive_rows_host(offsets, device, average=False):
    """(row_ptr, col_idx, val) on the device from the row offsets in a host int32 array"""
    offsets = np.ascontiguousarray(offsets, np.int32)
    rows, n = offsets.size - 1, int(offsets[-1])
    row_ptr = torch.empty(rows + 1, dtype=torch.int32, device=device)
    col_idx = torch.empty(n, dtype=torch.int32, device=device)
    val = torch.empty(n, dtype=torch.float32, device=device)
    check(_lib().gnnhip_csr_consecutive_rows_host_f32(rows, ctypes.c_void_p(offsets.ctypes.data), int(average), _i32(row_ptr, "row_ptr"),
                                                      _i32(col_idx, "col_idx") if n else None, _f32(val, "val") if n else None, _stream()))
    return row_ptr, col_idx, val


def csr_transpose(row_ptr, col_idx, val, m, k):
    nnz = col_idx.numel()
    dev = row_ptr.device
    t_rp = torch.empty(k + 1, dtype=torch.int32, device=dev)
    t_ci = torch.empty(nnz, dtype=torch.int32, device=dev)
    t_v = torch.empty(nnz, dtype=torch.float32, device=dev)
    check(_lib().gnnhip_csr_transpose_f32(m, k, nnz, _i32(row_ptr, "row_ptr"), _i32(col_idx, "col_idx"), _f32(val, "val"),
                                          _i32(t_rp, "t_row_ptr"), _i32(t_ci, "t_col_idx"), _f32(t_v, "t_val"), _stream()))
    return t_rp, t_ci, t_v


# ---------------------------------------------------------------- training iteration
def loss_acc(logits, lrow_ptr, lcol, lval, want_rows=False):
    """mean cross-entropy (softmax inside) and mean top-1 accuracy of a batch in one pass over the logits"""
    B, Q = logits.shape
    dev = logits.device
    probs = torch.empty_like(logits)
    loss = torch.empty((1,), dtype=torch.float32, device=dev)
    acc = torch.empty((1,), dtype=torch.float32, device=dev)
    loss_rows = torch.empty((B,), dtype=torch.float32, device=dev) if want_rows else None
    hit = torch.empty((B,), dtype=torch.int32, device=dev) if want_rows else None
    check(_lib().gnnhip_s2v_loss_acc_f32(B, Q, _f32(logits, "logits"), _i32(lrow_ptr, "lrow_ptr"), _i32(lcol, "lcol"),
                                         _f32(lval, "lval"), _f32(probs, "probs"), _f32(loss_rows, "loss_rows"),
                                         _i32(hit, "hit"), _f32(loss, "loss"), _f32(acc, "acc"), _stream()))
    return loss, acc, probs, loss_rows, hit


def readout_backward(s_csr, probs, label_csr, scale, hidden, W_h1, W_h2, N):
    B, Q = probs.shape
    C, H = W_h1.shape
    dev = probs.device
    dlogits = torch.empty((B, Q), dtype=torch.float32, device=dev)
    du = torch.empty((B, H), dtype=torch.float32, device=dev)
    g_h = torch.empty((N, C), dtype=torch.float32, device=dev)
    check(_lib().gnnhip_s2v_readout_backward_f32(
        B, N, C, H, Q, _i32(s_csr[0], "s_row_ptr"), _i32(s_csr[1], "s_col_idx"), _f32(s_csr[2], "s_val"),
        _f32(probs, "probs"), _i32(label_csr[0], "lrow_ptr"), _i32(label_csr[1], "lcol"), _f32(label_csr[2], "lval"),
        float(scale), _f32(hidden, "hidden"), _f32(W_h1, "W_h1"), _f32(W_h2, "W_h2"),
        _f32(dlogits, "dlogits"), _f32(du, "du"), _f32(g_h, "g_h"), _stream()))
    return dlogits, du, g_h


def s2v_level_backward(t_row_ptr, t_col_idx, t_val, dz, W, u=None, g_prev=None, gate_h=None, acc=None):
    """u = A^T dz, g_prev = u W^T (zeroed where gate_h <= 0 when gate_h is given), acc += g_prev when acc is given;
    the CSR arrays are those of A^T"""
    N, C = dz.shape
    _check_csr(t_row_ptr, t_col_idx, t_val, N, "A^T")
    if u is None:
        u = torch.empty_like(dz)
    if g_prev is None:
        g_prev = torch.empty_like(dz)
    check(_lib().gnnhip_s2v_level_backward_f32(N, C, int(t_col_idx.numel()), _i32(t_row_ptr, "t_row_ptr"), _i32(t_col_idx, "t_col_idx"),
                                               _f32(t_val, "t_val"), _f32(dz, "dz"), _f32(W, "W"), _f32(u, "u"), _f32(g_prev, "g_prev"),
                                               _f32(gate_h, "gate_h"), _f32(acc, "acc"), _stream()))
    return u, g_prev


def grad_gate(h, g, dz=None, acc=None, accumulate=False):
    check(_lib().gnnhip_s2v_grad_gate_f32(h.numel(), _f32(h, "h"), _f32(g, "g"), _f32(dz, "dz"), _f32(acc, "acc"),
                                          1 if accumulate else 0, _stream()))


def momentum_sgd_batch(ws, gs, vs, lr, momentum, l2):
    n = len(ws)
    P = ctypes.c_void_p * n
    Z = ctypes.c_size_t * n
    wp, gp = P(*[t.data_ptr() for t in ws]), P(*[t.data_ptr() for t in gs])
    vp = P(*[t.data_ptr() for t in vs]) if vs is not None else None
    for t in list(ws) + list(gs) + (list(vs) if vs is not None else []):
        _f32(t, "tensor")
    cnt = Z(*[t.numel() for t in ws])
    check(_lib().gnnhip_momentum_sgd_batch_f32(n, wp, gp, vp, cnt, float(lr), float(momentum), float(l2), _stream()))


def adam_batch(ws, gs, ms, vs, lr, l2, clip_threshold, beta1, beta2, eps, t):
    """one AdamOptimizer::Update over the tensors, t = the iteration count after the increment (1 for the first)"""
    n = len(ws)
    P = ctypes.c_void_p * n
    Z = ctypes.c_size_t * n
    for x in list(ws) + list(gs) + list(ms) + list(vs):
        _f32(x, "tensor")
    ptr = lambda ts: P(*[x.data_ptr() for x in ts])
    s1 = np.float32(1.0 / (1 - float(np.float32(beta1)) ** t))
    s2 = np.float32(1.0 / (1 - float(np.float32(beta2)) ** t))
    check(_lib().gnnhip_adam_batch_f32(n, ptr(ws), ptr(gs), ptr(ms), ptr(vs), Z(*[x.numel() for x in ws]), float(lr), float(l2),
                                       float(clip_threshold), float(beta1), float(beta2), float(eps), float(s1), float(s2), _stream()))


def upload_sparse32(host_array, out=None):
    """Host numpy array of 32-bit elements -> device tensor through gnnhip_memcpy_h2d_sparse32 (non-zero words only
    when they are few); the device tensor has the bits of the host array."""
    import numpy as np
    a = np.ascontiguousarray(host_array)
    if a.dtype.itemsize != 4:
        raise ValueError("upload_sparse32 takes 32-bit elements")
    tdt = {"float32": torch.float32, "int32": torch.int32}[a.dtype.name]
    if out is None:
        out = torch.empty(a.shape, dtype=tdt, device="cuda")
    check(_lib().gnnhip_memcpy_h2d_sparse32(ctypes.c_void_p(out.data_ptr()), a.ctypes.data_as(ctypes.c_void_p), a.size, _stream()))
    return out
