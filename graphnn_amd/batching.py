"""Host-side batch assembly: the CSR operands of the mean-field forward.

numpy counterpart of what graphnn does on the host for every batch:
GraphStruct::AddEdge / AddNode collect the lists (src/util/graph_struct.cpp:62-87)
and Node2NodeMsgPass / SubgraphMsgPass::InitCPUWeight flatten them into CSR
(src/nn/msg_pass.cpp:46-67,156-177).  Rows keep insertion order, which makes the
construction a stable counting sort; indices are int32, values fp32.
"""
import numpy as np


def _stable_csr(keys, vals, n_rows, average):
    keys = np.asarray(keys)
    vals = np.asarray(vals)
    if keys.size and (keys.min() < 0 or keys.max() >= n_rows):
        raise ValueError("row key out of range")
    counts = np.bincount(keys, minlength=n_rows).astype(np.int64)
    row_ptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(counts, out=row_ptr[1:])
    if row_ptr[-1] > np.iinfo(np.int32).max:
        raise ValueError("more entries than int32 CSR indices can address")
    order = np.argsort(keys, kind="stable")
    col_idx = vals[order].astype(np.int32)
    if average:
        # 1.0 / list.size() evaluated in double, then narrowed (msg_pass.cpp:59)
        val = (1.0 / counts[keys[order]].astype(np.float64)).astype(np.float32)
    else:
        val = np.ones(keys.size, dtype=np.float32)
    return row_ptr.astype(np.int32), col_idx, val


def node2node_csr(num_nodes, edge_x, edge_y, average=False):
    """A [N,N]: row y lists the sources x of the edges x->y in edge order."""
    return _stable_csr(edge_y, edge_x, num_nodes, average)


def subgraph_csr(num_subgraph, subg_id, node_idx, average=False):
    """S [B,N]: row g lists the nodes added to subgraph g in AddNode order."""
    return _stable_csr(subg_id, node_idx, num_subgraph, average)


def edge2node_csr(num_nodes, edge_y, average=False):
    """[N,E]: row i lists the indices of the edges that end in node i, in edge order
    (Edge2NodeMsgPass, src/nn/msg_pass.cpp:72-94)."""
    edge_y = np.asarray(edge_y)
    return _stable_csr(edge_y, np.arange(edge_y.size, dtype=np.int32), num_nodes, average)


def node2edge_csr(edge_x):
    """[E,N]: row e holds the tail node of edge e (Node2EdgeMsgPass, src/nn/msg_pass.cpp:98-116)."""
    edge_x = np.asarray(edge_x, dtype=np.int32)
    E = edge_x.size
    return np.arange(E + 1, dtype=np.int32), edge_x.copy(), np.ones(E, dtype=np.float32)


def edge2edge_csr(num_nodes, edge_x, edge_y):
    """[E,E]: row e = (x -> y) lists the edges that end in x and do not start in y, in edge order
    (Edge2EdgeMsgPass, src/nn/msg_pass.cpp:120-152)."""
    edge_x = np.asarray(edge_x, dtype=np.int64)
    edge_y = np.asarray(edge_y, dtype=np.int64)
    E = edge_x.size
    in_rp, in_edges, _ = edge2node_csr(num_nodes, edge_y)
    lens = (in_rp[1:] - in_rp[:-1])[edge_x]                      # candidates per row: in-degree of the tail
    row_of = np.repeat(np.arange(E, dtype=np.int64), lens)
    start = np.repeat(in_rp[:-1][edge_x].astype(np.int64), lens)
    within = np.arange(row_of.size, dtype=np.int64) - np.repeat(np.cumsum(lens) - lens, lens)
    cand = in_edges[start + within].astype(np.int64)
    keep = edge_x[cand] != edge_y[row_of]
    counts = np.bincount(row_of[keep], minlength=E)
    row_ptr = np.zeros(E + 1, dtype=np.int32)
    np.cumsum(counts, out=row_ptr[1:])
    col = cand[keep].astype(np.int32)
    return row_ptr, col, np.ones(col.size, dtype=np.float32)
