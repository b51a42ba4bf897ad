"""Host API layer without a GPU: the C++ GraphStruct + message-pass factors, scheduled by FactorGraph,
produce CSR operands bit-identical to the oracle (and thereby to the reference's GraphStruct)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "graphnn_amd", "host", "build", "host_csr_check")


def _run(tmp_path, B, N, E, sid, nid, ex, ey, average):
    if not os.path.exists(EXE):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "graphnn_amd", "host"), "build/host_csr_check"])
    inp, out = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(inp, "wb") as f:
        np.array([B, N, E], np.int32).tofile(f)
        for a in (sid, nid, ex, ey):
            np.ascontiguousarray(a, np.int32).tofile(f)
    r = subprocess.run([EXE, inp, out, "1" if average else "0"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    raw = open(out, "rb").read()
    pos = 0

    def take(n, dt):
        nonlocal pos
        a = np.frombuffer(raw, dtype=dt, count=n, offset=pos)
        pos += 4 * n
        return a

    res = (take(N + 1, np.int32), take(E, np.int32), take(E, np.float32),
           take(B + 1, np.int32), take(N, np.int32), take(N, np.float32), take(3, np.int32))
    e2n = (take(N + 1, np.int32), take(E, np.int32), take(E, np.float32))
    n2e = (take(E + 1, np.int32), take(E, np.int32), take(E, np.float32))
    nnz = int(take(1, np.int32)[0])
    e2e = (take(E + 1, np.int32), take(nnz, np.int32), take(nnz, np.float32))
    assert pos == len(raw)
    _run.edge_operands = (e2n, n2e, e2e)
    return res


@pytest.mark.parametrize("average", [False, True])
def test_cpp_builders_match_oracle_random(oracle, tmp_path, average):
    rng = np.random.default_rng(5)
    B, N, E = 9, 120, 700
    ex = rng.integers(0, N, E); ey = rng.integers(0, N, E)
    perm = rng.permutation(N)
    sid = np.sort(rng.integers(0, B, N))[perm]; nid = np.arange(N)[perm]
    arp, aci, av, srp, sci, sv, flags = _run(tmp_path, B, N, E, sid, nid, ex, ey, average)
    for got, want in zip((arp, aci, av), oracle.csr_node2node(N, ex, ey, average)):
        assert np.array_equal(got, want)
    for got, want in zip((srp, sci, sv), oracle.csr_subgraph(B, sid, nid, average)):
        assert np.array_equal(got, want)
    assert flags[0] == 0 and flags[1] == np.bincount(sid, minlength=B).max() and flags[2] == 0     # edges cross subgraphs
    e2n, n2e, e2e = _run.edge_operands
    for got, want in zip(e2n, oracle.csr_edge2node(N, ey, average)):
        assert np.array_equal(got, want)
    for got, want in zip(n2e, oracle.csr_node2edge(ex)):
        assert np.array_equal(got, want)
    for got, want in zip(e2e, oracle.csr_edge2edge(N, ex, ey)):
        assert np.array_equal(got, want)


def test_cpp_builders_on_a_getbatch_style_batch(oracle, tmp_path):
    from graphnn_amd import synth
    b = synth.molecule_batch(99, 30, 5)
    arp, aci, av, srp, sci, sv, flags = _run(tmp_path, b.num_graphs, b.num_nodes, b.num_edges, b.subg_id, b.node_idx,
                                             b.edge_x, b.edge_y, False)
    for got, want in zip((arp, aci, av), oracle.csr_node2node(b.num_nodes, b.edge_x, b.edge_y)):
        assert np.array_equal(got, want)
    assert np.array_equal(sci, np.arange(b.num_nodes)) and np.all(sv == 1)
    assert flags[0] == 1 and flags[1] == b.graph_sizes.max() and flags[2] == 1      # GetBatch layout recognised
    e2n, n2e, e2e = _run.edge_operands
    for got, want in zip(e2e, oracle.csr_edge2edge(b.num_nodes, b.edge_x, b.edge_y)):
        assert np.array_equal(got, want)
    # undirected graphs stored in both directions: every edge sees the other in-edges of its tail
    indeg = np.bincount(b.edge_y, minlength=b.num_nodes)
    assert e2e[1].size == int((indeg * (indeg - 1)).sum())


def test_folded_level_runs_after_the_producers_of_all_its_operands():
    """inference plan of a graph whose msg comes out of a deeper chain than the fed embedding: the folded level
    must be scheduled where its last factor stood, behind the step that produces msg (no GPU: nothing runs)"""
    exe = os.path.join(ROOT, "graphnn_amd", "host", "build", "host_plan_check")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "graphnn_amd", "host"), "build/host_plan_check"])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "host_plan_check ok" in r.stdout
