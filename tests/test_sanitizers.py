"""Host code under AddressSanitizer / UndefinedBehaviorSanitizer (no GPU involved): the CPU oracle on configuration 1, and
the host API layer's CPU-mode drivers, among them batch assembly with graphnn's write one float past the feature rows,
which has to land in the slack the host allocator leaves for it."""
import os
import subprocess

import numpy as np
import pytest

from graphnn_amd import batching, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")


def _built(path, make_dir, target):
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", make_dir, target])
    return path


def test_oracle_under_sanitizers_gives_the_bits_of_the_regular_build(oracle, tmp_path):
    exe = _built(os.path.join(ROOT, "oracle", "asan_check"), os.path.join(ROOT, "oracle"), "asan")
    batch, w, cfg = synth.make_config(1)
    N, E, B = batch.num_nodes, batch.num_edges, batch.num_graphs
    K, C, H, Q, L = (cfg[k] for k in ("K", "C", "H", "Q", "L"))
    X = batch.one_hot()
    lab = batch.label_csr()
    inp, out = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(inp, "wb") as f:
        np.array([N, E, B, K, C, H, Q, L], np.int32).tofile(f)
        for a in (batch.edge_x, batch.edge_y, batch.subg_id, batch.node_idx):
            np.ascontiguousarray(a, np.int32).tofile(f)
        for a in (X, w.W_n2l, w.W_conv, w.W_h1, w.W_h2):
            np.ascontiguousarray(a, np.float32).tofile(f)
        lab[0].astype(np.int32).tofile(f); lab[1].astype(np.int32).tofile(f); lab[2].astype(np.float32).tofile(f)
    r = subprocess.run([exe, inp, out], capture_output=True, text=True, timeout=120, env=ENV)
    assert r.returncode == 0 and "asan_check ok" in r.stdout, r.stdout + r.stderr
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr
    raw = open(out, "rb").read()
    pos = 0

    def take(n, dt, shape=None):
        nonlocal pos
        a = np.frombuffer(raw, dtype=dt, count=n, offset=pos)
        pos += 4 * n
        return a if shape is None else a.reshape(shape)

    a = batching.node2node_csr(N, batch.edge_x, batch.edge_y)
    s = batching.subgraph_csr(B, batch.subg_id, batch.node_idx)
    want = oracle.forward(a, s, X, w, L, lab)
    for ref in a:
        assert np.array_equal(take(ref.size, ref.dtype), ref)
    for ref in s:
        assert np.array_equal(take(ref.size, ref.dtype), ref)
    f4 = np.float32
    for key, shape in (("msg", (N, C)), ("h", (L + 1, N, C)), ("pool", (B, C)), ("hidden", (B, H)), ("logits", (B, Q)),
                       ("probs", (B, Q)), ("loss_rows", (B,))):
        got = take(int(np.prod(shape)), f4, shape)
        # the same IEEE operations in the same order (-ffp-contract=off in both builds); the vectorised exp / log of the
        # optimised build may differ from the scalar ones in the last place
        assert np.allclose(got, want[key], rtol=1e-6, atol=1e-7), key
        if key in ("msg", "h", "pool", "hidden", "logits"):
            assert np.array_equal(got, want[key]), key
    for key in ("pred", "truth", "hit"):
        assert np.array_equal(take(B, np.int32), want[key]), key
    assert np.allclose(take(2, f4), want["scalars"], rtol=1e-6)
    jag = take(N, f4)
    assert np.allclose(jag, oracle.jagged_softmax(want["h"][L][:, :1].copy(), batch.graph_sizes)[:, 0], rtol=1e-6, atol=1e-7)
    assert pos == len(raw)


def _csr_case_file(tmp_path):
    rng = np.random.default_rng(7)
    B, N, E = 6, 40, 150
    sid = np.sort(rng.integers(0, B, N)).astype(np.int32)
    nid = np.arange(N, dtype=np.int32)
    ex, ey = rng.integers(0, N, E).astype(np.int32), rng.integers(0, N, E).astype(np.int32)
    inp = str(tmp_path / "csr_in.bin")
    with open(inp, "wb") as f:
        np.array([B, N, E], np.int32).tofile(f)
        for a in (sid, nid, ex, ey):
            a.tofile(f)
    return inp, (B, N, E, sid, nid, ex, ey)


def test_host_layer_cpu_mode_under_sanitizers(oracle, tmp_path):
    host = os.path.join(ROOT, "graphnn_amd", "host")
    asan = os.path.join(host, "build", "asan")
    for name in ("host_csr_check", "host_plan_check", "host_batch_check"):
        _built(os.path.join(asan, name), host, "asan")
    # batch assembly as GetBatch does it: the largest tag's write one float past the row stays inside the allocation
    r = subprocess.run([os.path.join(asan, "host_batch_check")], capture_output=True, text=True, timeout=120, env=ENV)
    assert r.returncode == 0 and "host_batch_check ok" in r.stdout, r.stdout + r.stderr
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr
    # execution plans (fusion, fold, ordering): host logic only
    r = subprocess.run([os.path.join(asan, "host_plan_check")], capture_output=True, text=True, timeout=120, env=ENV)
    assert r.returncode == 0 and "host_plan_check ok" in r.stdout, r.stdout + r.stderr
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr
    # the CSR builders and their factors, against the oracle
    inp, (B, N, E, sid, nid, ex, ey) = _csr_case_file(tmp_path)
    out = str(tmp_path / "csr_out.bin")
    r = subprocess.run([os.path.join(asan, "host_csr_check"), inp, out, "1"], capture_output=True, text=True, timeout=120, env=ENV)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "runtime error" not in r.stderr and "AddressSanitizer" not in r.stderr, r.stderr
    raw = np.fromfile(out, dtype=np.int32)
    rp, ci, v = oracle.csr_node2node(N, ex, ey, True)
    assert np.array_equal(raw[:N + 1], rp) and np.array_equal(raw[N + 1:N + 1 + E], ci)
    assert np.array_equal(raw[N + 1 + E:N + 1 + 2 * E].view(np.float32), v)
