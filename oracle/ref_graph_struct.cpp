// TEST INFRASTRUCTURE ONLY.  Thin extern "C" driver around the reference's own
// GraphStruct (compiled from /root/reference/src/util/graph_struct.cpp where it
// lies; see oracle/Makefile).  It replays a batch through
// GraphStruct::Resize / AddNode / AddEdge and flattens in_edges / subgraph the
// way the reference's message-pass builders read them (in_edges[i][j].second,
// subgraph[g][j]), so the restated CSR builders in s2v_oracle.c can be checked
// against the real container.  Built only where the reference tree is present.
#include "util/graph_struct.h"

extern "C" int ref_graph_to_csr(int num_subgraph, int num_nodes, int num_edges,
                                const int* subg_id, const int* node_idx,
                                const int* edge_x, const int* edge_y,
                                int* a_row_ptr, int* a_col_idx,
                                int* s_row_ptr, int* s_col_idx)
{
    gnn::GraphStruct g;
    g.Resize((unsigned)num_subgraph, (unsigned)num_nodes);
    for (int i = 0; i < num_nodes; ++i) g.AddNode(subg_id[i], node_idx[i]);
    for (int e = 0; e < num_edges; ++e) g.AddEdge(e, edge_x[e], edge_y[e]);

    int nnz = 0;
    for (unsigned i = 0; i < g.num_nodes; ++i) {
        a_row_ptr[i] = nnz;
        auto& lst = g.in_edges->head[i];
        for (size_t j = 0; j < lst.size(); ++j) a_col_idx[nnz++] = lst[j].second;
    }
    a_row_ptr[g.num_nodes] = nnz;
    if (nnz != (int)g.num_edges) return -1;

    int cnt = 0;
    for (unsigned s = 0; s < g.num_subgraph; ++s) {
        s_row_ptr[s] = cnt;
        auto& lst = g.subgraph->head[s];
        for (size_t j = 0; j < lst.size(); ++j) s_col_idx[cnt++] = lst[j];
    }
    s_row_ptr[g.num_subgraph] = cnt;
    return cnt == num_nodes ? 0 : -2;
}
