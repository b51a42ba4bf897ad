"""Seeded synthetic workloads for the structure2vec forward (numpy, host side).

Random numbers come from SplitMix64 used as a counter-based generator, so every
stream is reproducible on any machine and can be generated vectorised.
Sub-streams are taken in a fixed order per workload: graph sizes, tree parents,
extra edges, node labels, graph labels, then the weight matrices.

Workloads
  molecule_batch   batches of small undirected graphs (random spanning tree plus
                   extra edges, mean degree ~2.2), one-hot node labels
  erdos_renyi_csr  G(n, m) with iid uniform (row, col), duplicates kept
  rmat_csr         R-MAT (a, b, c, d) edge list, duplicates kept, contiguous subgraphs
"""
from dataclasses import dataclass, field

import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_MASK64 = (1 << 64) - 1


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


class Stream:
    """SplitMix64 output sequence of `seed`, addressable by position."""

    def __init__(self, seed):
        self.seed = int(seed) & _MASK64
        self.pos = 0

    def u64(self, n):
        idx = np.arange(self.pos + 1, self.pos + n + 1, dtype=np.uint64)
        self.pos += n
        with np.errstate(over="ignore"):
            z = np.uint64(self.seed) + idx * _GOLDEN
            return _mix(z)

    def uniform(self, n):
        """float64 in [0, 1) with 53 random bits"""
        return (self.u64(n) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)

    def randint(self, n, lo, hi):
        """integers in [lo, hi) (hi - lo far below 2^53, so the float scaling is unbiased enough)"""
        return (lo + np.floor(self.uniform(n) * (hi - lo))).astype(np.int64)

    def normal(self, n, std=1.0, mean=0.0):
        """Box-Muller, cosine branch only: two uniforms per sample"""
        u = self.uniform(2 * n)
        u1, u2 = u[0::2], u[1::2]
        z = np.sqrt(-2.0 * np.log1p(-u1)) * np.cos(2.0 * np.pi * u2)
        return (mean + std * z).astype(np.float32)

    def child(self, k):
        """independent sub-stream number k"""
        with np.errstate(over="ignore"):
            s = _mix(np.array([np.uint64(self.seed) + np.uint64(k + 1) * _GOLDEN], dtype=np.uint64))[0]
        return Stream(int(s))


def config_seed(config_id):
    return 0x5EED0000 + int(config_id)


@dataclass
class Weights:
    W_n2l: np.ndarray   # [K, C]
    W_conv: np.ndarray  # [C, C]
    W_h1: np.ndarray    # [C, H]
    W_h2: np.ndarray    # [H, Q]


def make_weights(stream, K, C, H, Q, std=0.1):
    return Weights(
        W_n2l=stream.child(100).normal(K * C, std).reshape(K, C),
        W_conv=stream.child(101).normal(C * C, std).reshape(C, C),
        W_h1=stream.child(102).normal(C * H, std).reshape(C, H),
        W_h2=stream.child(103).normal(H * Q, std).reshape(H, Q),
    )


@dataclass
class Batch:
    """A batch of graphs in the order graphnn's GetBatch feeds GraphStruct."""
    num_graphs: int
    num_nodes: int
    graph_sizes: np.ndarray          # int32 [B]
    edge_x: np.ndarray               # int32 [E] source node of edge e (AddEdge order)
    edge_y: np.ndarray               # int32 [E] destination node of edge e
    subg_id: np.ndarray              # int32 [N] subgraph of node i (AddNode order)
    node_idx: np.ndarray             # int32 [N] node index passed to AddNode
    node_label: np.ndarray           # int32 [N]
    graph_label: np.ndarray          # int32 [B]
    num_label_types: int
    num_classes: int
    extra: dict = field(default_factory=dict)

    @property
    def num_edges(self):
        return int(self.edge_x.size)

    def one_hot(self):
        X = np.zeros((self.num_nodes, self.num_label_types), dtype=np.float32)
        X[np.arange(self.num_nodes), self.node_label] = 1.0
        return X

    def label_csr(self):
        """one-hot graph labels as the CSR GetBatch builds (one entry per row)"""
        B = self.num_graphs
        return (np.arange(B + 1, dtype=np.int32), self.graph_label.astype(np.int32), np.ones(B, dtype=np.float32))


def _sizes_uniform(stream, B, lo, hi):
    return stream.randint(B, lo, hi + 1)


def _sizes_skewed(stream, B):
    # right-skewed like NCI109: 10 + min(100, floor(-20 ln(1 - u))), mean ~30, max 110
    u = stream.uniform(B)
    return 10 + np.minimum(100, np.floor(-20.0 * np.log1p(-u))).astype(np.int64)


def molecule_batch(seed, B, K, Q=2, size_mode="uniform", size_lo=10, size_hi=28, edge_factor=1.1):
    """B random molecule-like graphs: spanning tree parent(v) ~ U{0..v-1}, plus
    round(edge_factor n) - (n - 1) distinct extra non-tree, non-self pairs (1.1 n undirected
    edges: mean degree 2.2, what the molecule datasets have); every undirected
    edge is stored in both directions and adjacency lists are ascending, which is
    the order the dataset files (and therefore GetBatch) present them in."""
    root = Stream(seed)
    s_sizes, s_tree, s_extra, s_nlab, s_glab = (root.child(i) for i in range(5))
    if size_mode == "uniform":
        sizes = _sizes_uniform(s_sizes, B, size_lo, size_hi)
    elif size_mode == "skewed":
        sizes = _sizes_skewed(s_sizes, B)
    else:
        raise ValueError("size_mode must be 'uniform' or 'skewed'")
    sizes = sizes.astype(np.int64)
    offsets = np.concatenate([[0], np.cumsum(sizes)])
    N = int(offsets[-1])

    # spanning trees, all graphs at once: node v >= 1 of each graph draws a parent in [0, v)
    local = np.arange(N, dtype=np.int64) - np.repeat(offsets[:-1], sizes)
    u = s_tree.uniform(N)
    parent = np.floor(u * np.maximum(local, 1)).astype(np.int64)
    child_mask = local >= 1
    g_off = np.repeat(offsets[:-1], sizes)
    tree_a = (g_off + parent)[child_mask]
    tree_b = (g_off + local)[child_mask]

    # extra edges by rejection, graph by graph (few per graph)
    n_extra = np.maximum(0, np.rint(edge_factor * sizes).astype(np.int64) - (sizes - 1))
    extra_a, extra_b = [], []
    tree_parent_local = parent
    for g in range(B):
        n = int(sizes[g])
        want = int(n_extra[g])
        max_pairs = n * (n - 1) // 2 - (n - 1)
        want = min(want, max_pairs)
        if want <= 0:
            continue
        o = int(offsets[g])
        have = set()
        for v in range(1, n):
            p = int(tree_parent_local[o + v])
            have.add((p, v) if p < v else (v, p))
        got = 0
        while got < want:
            cand = s_extra.randint(2 * max(8, 4 * (want - got)), 0, n).reshape(-1, 2)
            for a, b in cand:
                if a == b:
                    continue
                key = (int(a), int(b)) if a < b else (int(b), int(a))
                if key in have:
                    continue
                have.add(key)
                extra_a.append(o + key[0])
                extra_b.append(o + key[1])
                got += 1
                if got == want:
                    break
    und_a = np.concatenate([tree_a, np.asarray(extra_a, dtype=np.int64)])
    und_b = np.concatenate([tree_b, np.asarray(extra_b, dtype=np.int64)])
    x = np.concatenate([und_a, und_b])
    y = np.concatenate([und_b, und_a])
    order = np.lexsort((y, x))             # GetBatch order: by source node, neighbours ascending
    edge_x = x[order].astype(np.int32)
    edge_y = y[order].astype(np.int32)

    node_label = s_nlab.randint(N, 0, K).astype(np.int32)
    graph_label = s_glab.randint(B, 0, Q).astype(np.int32)
    return Batch(
        num_graphs=B, num_nodes=N, graph_sizes=sizes.astype(np.int32), edge_x=edge_x, edge_y=edge_y,
        subg_id=np.repeat(np.arange(B, dtype=np.int32), sizes), node_idx=np.arange(N, dtype=np.int32),
        node_label=node_label, graph_label=graph_label, num_label_types=K, num_classes=Q,
    )


def _csr_from_sorted_rows(rows, n_rows):
    counts = np.bincount(rows, minlength=n_rows)
    row_ptr = np.zeros(n_rows + 1, dtype=np.int64)
    np.cumsum(counts, out=row_ptr[1:])
    return row_ptr.astype(np.int32)


def erdos_renyi_csr(seed, n, nnz, regular=False):
    """G(n, m): nnz entries with iid uniform (row, col), duplicates and self-loops kept,
    columns ascending inside a row, unit values.  regular=True gives exactly nnz/n per row."""
    root = Stream(seed)
    if regular:
        per = nnz // n
        rows = np.repeat(np.arange(n, dtype=np.int64), per)
        nnz = per * n
    else:
        rows = root.child(0).randint(nnz, 0, n)
    cols = root.child(1).randint(nnz, 0, n)
    order = np.lexsort((cols, rows))
    rows, cols = rows[order], cols[order]
    return _csr_from_sorted_rows(rows, n), cols.astype(np.int32), np.ones(nnz, dtype=np.float32)


def rmat_csr(seed, scale, nnz, a=0.57, b=0.19, c=0.19, chunk=1 << 24):
    """R-MAT: each edge picks one quadrant per bit level with probabilities (a, b, c, d);
    no vertex permutation, duplicates kept, rows ascending and columns ascending inside a row."""
    root = Stream(seed)
    n = 1 << scale
    rows = np.zeros(nnz, dtype=np.int64)
    cols = np.zeros(nnz, dtype=np.int64)
    ab, abc = a + b, a + b + c
    for level in range(scale):
        s = root.child(level)
        for lo in range(0, nnz, chunk):
            hi = min(nnz, lo + chunk)
            s.pos = lo
            u = s.uniform(hi - lo)
            r_bit = (u >= ab).astype(np.int64)                       # quadrants c, d -> lower half of rows
            c_bit = (((u >= a) & (u < ab)) | (u >= abc)).astype(np.int64)   # quadrants b, d
            rows[lo:hi] = (rows[lo:hi] << 1) | r_bit
            cols[lo:hi] = (cols[lo:hi] << 1) | c_bit
    key = rows * n + cols
    key.sort()
    rows = key // n
    cols = (key - rows * n).astype(np.int32)
    return _csr_from_sorted_rows(rows, n), cols, np.ones(nnz, dtype=np.float32)


# ---- the same streams generated by torch (on the GPU for the large configurations) --------------------
# SplitMix64 in two's-complement int64 arithmetic: products wrap exactly as the unsigned ones do, and a logical
# right shift is an arithmetic one with the sign copies masked off, so every value equals the numpy stream's
# bit for bit; tests assert it.
def _i64(x):
    x &= _MASK64
    return x - (1 << 64) if x >= (1 << 63) else x


def _lsr(z, s):
    return (z >> s) & ((1 << (64 - s)) - 1)


def torch_u64(seed, pos, n, device):
    """int64 tensor with the bits of Stream(seed) outputs number pos + 1 .. pos + n"""
    import torch
    idx = torch.arange(pos + 1, pos + n + 1, dtype=torch.int64, device=device)
    z = idx * _i64(int(_GOLDEN)) + _i64(int(seed))
    z = (z ^ _lsr(z, 30)) * _i64(int(_M1))
    z = (z ^ _lsr(z, 27)) * _i64(int(_M2))
    return z ^ _lsr(z, 31)


def torch_uniform(seed, pos, n, device):
    """float64 tensor equal to Stream(seed).uniform at positions pos .. pos + n"""
    return _lsr(torch_u64(seed, pos, n, device), 11).double() * (1.0 / 9007199254740992.0)


def rmat_edges_torch(seed, scale, nnz, device, a=0.57, b=0.19, c=0.19, lo=0, hi=None, chunk=1 << 24):
    """(rows, cols) int64 of edges lo .. hi of rmat_csr's edge list before sorting, generated on `device`"""
    import torch
    hi = nnz if hi is None else hi
    root = Stream(seed)
    seeds = [root.child(level).seed for level in range(scale)]
    rows = torch.zeros(hi - lo, dtype=torch.int64, device=device)
    cols = torch.zeros(hi - lo, dtype=torch.int64, device=device)
    ab, abc = a + b, a + b + c
    for p in range(lo, hi, chunk):
        q = min(hi, p + chunk)
        r = torch.zeros(q - p, dtype=torch.int64, device=device)
        cc = torch.zeros(q - p, dtype=torch.int64, device=device)
        for level in range(scale):
            u = torch_uniform(seeds[level], p, q - p, device)
            r = (r << 1) | (u >= ab).long()
            cc = (cc << 1) | (((u >= a) & (u < ab)) | (u >= abc)).long()
        rows[p - lo:q - lo] = r
        cols[p - lo:q - lo] = cc
    return rows, cols


def rmat_csr_torch(seed, scale, nnz, device, a=0.57, b=0.19, c=0.19):
    """rmat_csr on `device`: (row_ptr int32 [n + 1], col_idx int32 [nnz], val float32 [nnz]) as torch tensors, equal to
    the numpy generator's arrays bit for bit"""
    import torch
    n = 1 << scale
    rows, cols = rmat_edges_torch(seed, scale, nnz, device, a, b, c)
    key = rows * n + cols
    del rows, cols
    key, _ = torch.sort(key)
    r = key >> scale
    col_idx = (key - (r << scale)).int()
    cnt = torch.bincount(r, minlength=n)
    del key, r
    row_ptr = torch.zeros(n + 1, dtype=torch.int32, device=device)
    row_ptr[1:] = torch.cumsum(cnt, 0).int()
    return row_ptr, col_idx, torch.ones(nnz, dtype=torch.float32, device=device)


def torch_uniform_f32(seed, n, device, lo=0.0, hi=1.0, chunk=1 << 25):
    """float32 tensor of n values lo + (hi - lo) u, u the uniforms of Stream(seed) from its start, rounded to float32
    once: equal to (lo + (hi - lo) * Stream(seed).uniform(n)).astype(float32)"""
    import torch
    out = torch.empty(n, dtype=torch.float32, device=device)
    for p in range(0, n, chunk):
        q = min(n, p + chunk)
        out[p:q] = (lo + (hi - lo) * torch_uniform(seed, p, q - p, device)).float()
    return out


def torch_normal_f32(seed, n, device, std=1.0, chunk=1 << 24):
    """float32 tensor of n Box-Muller normals from the uniforms of Stream(seed), as Stream(seed).normal(n, std): the
    uniforms are the numpy stream's bit for bit; log1p / sqrt / cos are the device's float64 routines, whose last bit
    may differ from the host library's, so a value may land on the neighbouring float32 (tests bound that on a prefix)"""
    import math
    import torch
    out = torch.empty(n, dtype=torch.float32, device=device)
    for p in range(0, n, chunk):
        q = min(n, p + chunk)
        u = torch_uniform(seed, 2 * p, 2 * (q - p), device)
        z = torch.sqrt(-2.0 * torch.log1p(-u[0::2])) * torch.cos(2.0 * math.pi * u[1::2])
        out[p:q] = (std * z).float()
    return out


def contiguous_subgraph_csr(num_nodes, num_subgraph):
    """S for subgraphs that are equal contiguous node ranges (row g lists its nodes)"""
    per = num_nodes // num_subgraph
    row_ptr = (np.arange(num_subgraph + 1, dtype=np.int64) * per)
    row_ptr[-1] = num_nodes
    return row_ptr.astype(np.int32), np.arange(num_nodes, dtype=np.int32), np.ones(num_nodes, dtype=np.float32)


# ---- the named configurations -------------------------------------------------
CONFIGS = {
    1: dict(B=50, K=7, C=64, H=32, Q=2, L=3, size_mode="uniform", size_lo=10, size_hi=28),
    2: dict(B=256, K=38, C=64, H=32, Q=2, L=4, size_mode="skewed"),
    4: dict(B=10000, K=64, C=256, H=128, Q=2, L=5, size_mode="uniform", size_lo=20, size_hi=40),
}


def make_config(config_id, B=None, size_mode=None, edge_factor=None):
    """(batch, weights, dims) for the molecule-style configurations 1, 2 and 4.  size_mode="uniform" on configuration 2
    takes its "nodes per graph ~ U[10,110]" literally (mean 60) instead of the right-skewed sizes with mean ~30.
    edge_factor: undirected edges per node (default 1.1, mean degree 2.2; 2.2 reads configuration 4's "~660k undirected
    edges" on ~300k nodes literally)."""
    cfg = dict(CONFIGS[config_id])
    if B is not None:
        cfg["B"] = B
    if size_mode is not None and size_mode != cfg["size_mode"]:
        cfg["size_mode"] = size_mode
        if size_mode == "uniform" and "size_lo" not in cfg:
            cfg["size_lo"], cfg["size_hi"] = 10, 110
    seed = config_seed(config_id)
    kw = {k: cfg[k] for k in ("size_lo", "size_hi") if k in cfg}
    if edge_factor is not None:
        kw["edge_factor"] = edge_factor
    batch = molecule_batch(seed, cfg["B"], cfg["K"], cfg["Q"], size_mode=cfg["size_mode"], **kw)
    weights = make_weights(Stream(seed), cfg["K"], cfg["C"], cfg["H"], cfg["Q"])
    return batch, weights, cfg


def write_graphnn_txt(batch, graph_path, train_idx_path=None, test_idx_path=None, test_fraction=0.2):
    """Write a batch as a dataset in graphnn's txt layout (examples/graph_classification/data/README.md:1-9):
    first line the number of graphs; per graph a line `n label`, then one line per node
    `tag m nbr_1 .. nbr_m` with neighbour indices local to the graph.  Optionally writes index files
    (one graph index per line) splitting the graphs into train / test."""
    offsets = np.concatenate([[0], np.cumsum(batch.graph_sizes)])
    # adjacency of node x = destinations of its out-edges, which are stored grouped by x and ascending
    deg = np.bincount(batch.edge_x, minlength=batch.num_nodes)
    starts = np.concatenate([[0], np.cumsum(deg)])
    lines = [str(batch.num_graphs)]
    for g in range(batch.num_graphs):
        n, o = int(batch.graph_sizes[g]), int(offsets[g])
        lines.append("%d %d" % (n, int(batch.graph_label[g])))
        for j in range(n):
            nb = batch.edge_y[starts[o + j]:starts[o + j + 1]] - o
            lines.append(" ".join([str(int(batch.node_label[o + j])), str(nb.size)] + [str(int(v)) for v in nb]))
    with open(graph_path, "w") as f:
        f.write("\n".join(lines) + "\n")
    if train_idx_path and test_idx_path:
        n_test = max(1, int(round(batch.num_graphs * test_fraction)))
        idx = np.arange(batch.num_graphs)
        with open(test_idx_path, "w") as f:
            f.write("\n".join(str(int(i)) for i in idx[:n_test]) + "\n")
        with open(train_idx_path, "w") as f:
            f.write("\n".join(str(int(i)) for i in idx[n_test:]) + "\n")
