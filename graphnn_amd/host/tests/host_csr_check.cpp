// CPU-only check of the host layer: GraphStruct + the message-pass factors scheduled by
// FactorGraph build the CSR operands of a batch; the arrays are written out for a bit-exact
// comparison with the oracle.  Needs no GPU (mode = CPU end to end).
//
//   host_csr_check <in.bin> <out.bin> <average 0|1>
//   in.bin : int32 B, N, E, then subg_id[N], node_idx[N], edge_x[E], edge_y[E]
//   out.bin: int32 a_row_ptr[N+1], a_col[E], fp32 a_val[E], int32 s_row_ptr[B+1], s_col[N], fp32 s_val[N],
//            int32 flags {contiguous_subgraphs, max_subgraph_nodes, block_diagonal},
//            then the edge-based operands: e2n row_ptr[N+1], col[E], val[E]; n2e row_ptr[E+1], col[E], val[E];
//            int32 nnz of e2e, e2e row_ptr[E+1], col[nnz], val[nnz]
#include <cstdio>
#include <vector>
#include "tensor/tensor_all.h"
#include "nn/nn_all.h"

using namespace gnn;

int main(int argc, char** argv)
{
    ASSERT(argc == 4, "usage: host_csr_check in.bin out.bin average");
    FILE* f = fopen(argv[1], "rb");
    ASSERT(f, "cannot open input");
    int hdr[3];
    ASSERT(fread(hdr, sizeof(int), 3, f) == 3, "short header");
    const int B = hdr[0], N = hdr[1], E = hdr[2];
    std::vector<int> sid(N), nid(N), ex(E), ey(E);
    ASSERT(fread(sid.data(), 4, N, f) == (size_t)N && fread(nid.data(), 4, N, f) == (size_t)N, "short read");
    ASSERT(fread(ex.data(), 4, E, f) == (size_t)E && fread(ey.data(), 4, E, f) == (size_t)E, "short read");
    fclose(f);
    const bool average = atoi(argv[3]) != 0;

    GraphStruct g;
    // a first, larger batch leaves stale capacity behind; the second Resize must not leak it
    g.Resize(B + 3, N + 5);
    for (int i = 0; i < N + 5; ++i) g.AddNode(i % (B + 3), i);
    g.AddEdge(0, N + 4, 0);
    g.Resize(B, N);
    for (int i = 0; i < N; ++i) g.AddNode(sid[i], nid[i]);
    for (int e = 0; e < E; ++e) g.AddEdge(e, ex[e], ey[e]);

    // the per-node and per-subgraph lists, made on demand, hold what graphnn's AddEdge / AddNode would have
    // appended (src/util/graph_struct.cpp:62-75): (edge, other end) per edge in edge order, nodes in AddNode order
    {
        std::vector<size_t> seen_out(N, 0), seen_in(N, 0), seen_sub(B, 0);
        ASSERT(g.out_edges->n == N && g.in_edges->n == N && g.subgraph->n == B, "list counts");
        for (int e = 0; e < E; ++e) {
            auto& o = g.out_edges->head[ex[e]];
            auto& in = g.in_edges->head[ey[e]];
            ASSERT(seen_out[ex[e]] < o.size() && o[seen_out[ex[e]]] == std::make_pair(e, ey[e]), "out_edges differ at edge " << e);
            ASSERT(seen_in[ey[e]] < in.size() && in[seen_in[ey[e]]] == std::make_pair(e, ex[e]), "in_edges differ at edge " << e);
            seen_out[ex[e]]++; seen_in[ey[e]]++;
        }
        for (int i = 0; i < N; ++i) {
            ASSERT(seen_out[i] == g.out_edges->head[i].size() && seen_in[i] == g.in_edges->head[i].size(), "stale list entries at node " << i);
            auto& sg = g.subgraph->head[sid[i]];
            ASSERT(seen_sub[sid[i]] < sg.size() && sg[seen_sub[sid[i]]] == nid[i], "subgraph list differs at node " << i);
            seen_sub[sid[i]]++;
        }
        for (int b = 0; b < B; ++b) ASSERT(seen_sub[b] == g.subgraph->head[b].size(), "stale subgraph entries");
    }

    FactorGraph fg;
    auto gv = add_const<GraphVar>(fg, "graph", true);
    auto a = af< Node2NodeMsgPass<CPU, float> >(fg, {gv}, average);
    auto s = af< SubgraphMsgPass<CPU, float> >(fg, {gv}, average);
    std::map<std::string, void*> feed;
    feed["graph"] = &g;
    fg.FeedForward({a, s}, feed, Phase::TEST);
    ASSERT(fg.LastPlanFactorCount() == 2, "both builders must run");
    // requesting only one target must run only its builder
    fg.FeedForward({s}, feed, Phase::TEST);
    ASSERT(fg.LastPlanFactorCount() == 1, "dependency pruning failed");

    FILE* o = fopen(argv[2], "wb");
    ASSERT(o, "cannot open output");
    auto& ad = *a->value.data;
    auto& sd = *s->value.data;
    ASSERT(ad.nnz == E && ad.len_ptr == N + 1 && sd.nnz == N && sd.len_ptr == B + 1, "unexpected CSR sizes");
    fwrite(ad.row_ptr, 4, N + 1, o); fwrite(ad.col_idx, 4, E, o); fwrite(ad.val, 4, E, o);
    fwrite(sd.row_ptr, 4, B + 1, o); fwrite(sd.col_idx, 4, N, o); fwrite(sd.val, 4, N, o);
    auto* sf = dynamic_cast<SubgraphMsgPass<CPU, float>*>(fg.factor_list[1].get());
    int flags[3] = {sf->layout.contiguous_subgraphs ? 1 : 0, sf->layout.max_subgraph_nodes,
                    fg.factor_list[0]->Layout()->block_diagonal ? 1 : 0};
    fwrite(flags, 4, 3, o);

    // ---- edge-based operands of the loopy-BP embedding
    FactorGraph fg2;
    auto gv2 = add_const<GraphVar>(fg2, "graph", true);
    auto e2n = af< Edge2NodeMsgPass<CPU, float> >(fg2, {gv2}, average);
    auto n2e = af< Node2EdgeMsgPass<CPU, float> >(fg2, {gv2});
    auto e2e = af< Edge2EdgeMsgPass<CPU, float> >(fg2, {gv2});
    fg2.FeedForward({e2n, n2e, e2e}, feed, Phase::TEST);
    auto& d1 = *e2n->value.data;
    auto& d2 = *n2e->value.data;
    auto& d3 = *e2e->value.data;
    ASSERT(d1.nnz == E && d1.len_ptr == N + 1 && d2.nnz == E && d2.len_ptr == E + 1 && d3.len_ptr == E + 1, "unexpected CSR sizes");
    ASSERT(e2n->value.rows() == (size_t)N && e2n->value.cols() == (size_t)E && n2e->value.rows() == (size_t)E &&
           n2e->value.cols() == (size_t)N && e2e->value.rows() == (size_t)E && e2e->value.cols() == (size_t)E, "unexpected shapes");
    fwrite(d1.row_ptr, 4, N + 1, o); fwrite(d1.col_idx, 4, E, o); fwrite(d1.val, 4, E, o);
    fwrite(d2.row_ptr, 4, E + 1, o); fwrite(d2.col_idx, 4, E, o); fwrite(d2.val, 4, E, o);
    int nnz3 = d3.nnz;
    fwrite(&nnz3, 4, 1, o);
    fwrite(d3.row_ptr, 4, E + 1, o); fwrite(d3.col_idx, 4, nnz3, o); fwrite(d3.val, 4, nnz3, o);
    fclose(o);
    return 0;
}
