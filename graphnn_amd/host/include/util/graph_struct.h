// Batch graph container with graphnn's interface (include/util/graph_struct.h,
// src/util/graph_struct.cpp): per-node in/out edge lists, per-subgraph node lists
// and the flat edge list, filled by AddNode / AddEdge in insertion order.
// Header-only.  Unlike the reference, Resize only clears the lists that were in
// use, not the whole capacity.
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

class GraphStruct
{
public:
    GraphStruct() : num_nodes(0), num_edges(0), num_subgraph(0)
    {
        out_edges = new LinkedTable< std::pair<int, int> >();
        in_edges = new LinkedTable< std::pair<int, int> >();
        subgraph = new LinkedTable<int>();
    }
    ~GraphStruct()
    {
        delete out_edges;
        delete in_edges;
        delete subgraph;
    }
    GraphStruct(const GraphStruct&) = delete;
    GraphStruct& operator=(const GraphStruct&) = delete;

    // edge idx: x -> y; indices must arrive as 0, 1, 2, ...
    void AddEdge(int idx, int x, int y)
    {
        assert((unsigned)idx == num_edges);
        out_edges->AddEntry(x, std::make_pair(idx, y));
        in_edges->AddEntry(y, std::make_pair(idx, x));
        edge_list.push_back(std::make_pair(x, y));
        num_edges++;
    }

    void AddNode(int subg_id, int n_idx) { subgraph->AddEntry(subg_id, n_idx); }

    void Resize(unsigned _num_subgraph, unsigned _num_nodes = 0)
    {
        num_subgraph = _num_subgraph;
        num_nodes = _num_nodes;
        num_edges = 0;
        edge_list.clear();
        in_edges->Resize((int)num_nodes);
        out_edges->Resize((int)num_nodes);
        subgraph->Resize((int)num_subgraph);
    }

    LinkedTable< std::pair<int, int> >* out_edges;   // per node: (edge index, head node)
    LinkedTable< std::pair<int, int> >* in_edges;    // per node: (edge index, tail node)
    LinkedTable<int>* subgraph;                       // per subgraph: its nodes
    std::vector< std::pair<int, int> > edge_list;     // edge index -> (x, y)
    unsigned num_nodes, num_edges, num_subgraph;
};

}  // namespace gnn

#endif
