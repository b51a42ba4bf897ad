// Batch graph container with graphnn's interface (include/util/graph_struct.h,
// src/util/graph_struct.cpp): per-node in/out edge lists, per-subgraph node lists
// and the flat edge list, filled by AddNode / AddEdge in insertion order.
// Header-only.  Unlike the reference, the lists are made on demand from two flat arrays
// (see LazyTable) and Resize only clears the lists that were in use, not the whole capacity.
#ifndef GRAPH_STRUCT_H
#define GRAPH_STRUCT_H

#include <algorithm>
#include <cassert>
#include <utility>
#include <vector>

namespace gnn
{

template<typename T>
class LinkedTable
{
public:
    LinkedTable() : n(0), ncap(0) {}

    // append `content` to list `head_id`, growing the table when needed
    void AddEntry(int head_id, T content)
    {
        if (head_id >= n) {
            Reserve(head_id + 1);
            n = head_id + 1;
        }
        head[head_id].push_back(content);
    }

    // make the table hold exactly new_n empty lists (capacity is kept)
    void Resize(int new_n)
    {
        const int used = std::max(n, new_n);
        Reserve(new_n);
        for (int i = 0; i < used && i < (int)head.size(); ++i) head[i].clear();
        n = new_n;
    }

    int n;                                   // number of lists in use
    std::vector< std::vector<T> > head;      // the lists

private:
    void Reserve(int want)
    {
        if (want > ncap) {
            ncap = std::max(ncap * 2, want);
            head.resize(ncap);
        }
    }
    int ncap;
};

class GraphStruct;

// graphnn declares in_edges / out_edges / subgraph as pointers to LinkedTable and fills them on every
// AddEdge / AddNode (three heap appends per edge).  Here AddEdge / AddNode only append to two flat arrays;
// the per-node and per-subgraph lists are made from them the first time somebody looks
// (`graph.in_edges->head[i]` reads as it does with the reference).  The message-pass factors build their CSR
// operands from the flat arrays and never ask for the lists.
template<typename T>
class LazyTable
{
public:
    LinkedTable<T>* operator->() { Materialize(); return &table; }
    LinkedTable<T>& operator*() { Materialize(); return table; }

private:
    friend class GraphStruct;
    void Materialize();
    GraphStruct* owner = nullptr;
    int which = 0;                 // 0 out_edges, 1 in_edges, 2 subgraph
    bool valid = true;
    LinkedTable<T> table;
};

class GraphStruct
{
public:
    GraphStruct() : num_nodes(0), num_edges(0), num_subgraph(0)
    {
        out_edges.owner = in_edges.owner = this;
        subgraph.owner = this;
        out_edges.which = 0; in_edges.which = 1; subgraph.which = 2;
    }
    GraphStruct(const GraphStruct&) = delete;
    GraphStruct& operator=(const GraphStruct&) = delete;

    // edge idx: x -> y; indices must arrive as 0, 1, 2, ...
    void AddEdge(int idx, int x, int y)
    {
        assert((unsigned)idx == num_edges);
        (void)idx;
        edge_list.push_back(std::make_pair(x, y));
        out_edges.valid = in_edges.valid = false;
        num_edges++;
    }

    void AddNode(int subg_id, int n_idx)
    {
        node_list.push_back(std::make_pair(subg_id, n_idx));
        subgraph.valid = false;
    }

    void Resize(unsigned _num_subgraph, unsigned _num_nodes = 0)
    {
        num_subgraph = _num_subgraph;
        num_nodes = _num_nodes;
        num_edges = 0;
        edge_list.clear();
        node_list.clear();
        out_edges.valid = in_edges.valid = subgraph.valid = false;
    }

    // Stable grouping of the edges by head node: row y of the result lists, in edge order, the tail
    // (payload_is_edge false) or the index (true) of every edge x -> y.  row_ptr has num_nodes + 1 entries.
    // This is what reading in_edges->head[y] row after row gives (src/nn/msg_pass.cpp:46-94).
    void GroupEdgesByHead(bool payload_is_edge, int* row_ptr, int* payload)
    {
        const int N = (int)num_nodes, E = (int)num_edges;
        cursor.assign((size_t)N + 1, 0);
        for (int e = 0; e < E; ++e) {
            assert(edge_list[e].second >= 0 && edge_list[e].second < N);
            cursor[(size_t)edge_list[e].second + 1]++;
        }
        row_ptr[0] = 0;
        for (int i = 0; i < N; ++i) { row_ptr[i + 1] = row_ptr[i] + cursor[(size_t)i + 1]; cursor[i] = row_ptr[i]; }
        for (int e = 0; e < E; ++e) payload[cursor[edge_list[e].second]++] = payload_is_edge ? e : edge_list[e].first;
    }
    // Stable grouping of the nodes by subgraph, in AddNode order (src/nn/msg_pass.cpp:156-177).
    void GroupNodesBySubgraph(int* row_ptr, int* nodes)
    {
        const int B = (int)num_subgraph, M = (int)node_list.size();
        cursor.assign((size_t)B + 1, 0);
        for (int i = 0; i < M; ++i) {
            assert(node_list[i].first >= 0 && node_list[i].first < B);
            cursor[(size_t)node_list[i].first + 1]++;
        }
        row_ptr[0] = 0;
        for (int g = 0; g < B; ++g) { row_ptr[g + 1] = row_ptr[g] + cursor[(size_t)g + 1]; cursor[g] = row_ptr[g]; }
        for (int i = 0; i < M; ++i) nodes[cursor[node_list[i].first]++] = node_list[i].second;
    }

    LazyTable< std::pair<int, int> > out_edges;      // per node: (edge index, head node)
    LazyTable< std::pair<int, int> > in_edges;       // per node: (edge index, tail node)
    LazyTable<int> subgraph;                          // per subgraph: its nodes
    std::vector< std::pair<int, int> > edge_list;     // edge index -> (x, y)
    std::vector< std::pair<int, int> > node_list;     // AddNode order -> (subgraph, node)
    unsigned num_nodes, num_edges, num_subgraph;

private:
    std::vector<int> cursor;
};

template<typename T>
inline void LazyTable<T>::Materialize()
{
    if (valid) return;
    valid = true;
    fill_table(*owner, which, table);
}

// the lists exactly as the reference's AddEdge / AddNode leave them (src/util/graph_struct.cpp:62-75)
inline void fill_table(GraphStruct& g, int which, LinkedTable< std::pair<int, int> >& t)
{
    t.Resize((int)g.num_nodes);
    for (int e = 0; e < (int)g.edge_list.size(); ++e) {
        const int x = g.edge_list[e].first, y = g.edge_list[e].second;
        if (which == 0) t.AddEntry(x, std::make_pair(e, y));
        else t.AddEntry(y, std::make_pair(e, x));
    }
}
inline void fill_table(GraphStruct& g, int, LinkedTable<int>& t)
{
    t.Resize((int)g.num_subgraph);
    for (const auto& sn : g.node_list) t.AddEntry(sn.first, sn.second);
}

}  // namespace gnn

#endif
