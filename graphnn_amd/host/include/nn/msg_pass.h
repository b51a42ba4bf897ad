// Message-passing operands: CSR matrices built from the batch GraphStruct on the host and
// copied to the device (interface of graphnn's include/nn/msg_pass.h; construction rules of
// src/nn/msg_pass.cpp:46-177).  Row i of the node-to-node matrix lists the in-neighbours of
// node i in edge order; row g of the subgraph matrix lists the nodes of graph g in AddNode
// order; values are 1, or 1/row length when `average` is set.  The edge-based operands of the
// loopy-BP embedding: edge-to-node [N,E] (edges that end in node i), node-to-edge [E,N] (the
// tail of edge e) and edge-to-edge [E,E] (edges that end in the tail of edge e, except its own
// reverse).
#ifndef MSG_PASS_H
#define MSG_PASS_H

#include "nn/factor.h"
#include "util/graph_struct.h"

namespace gnn
{

namespace detail
{
// stable CSR transpose on the host (row c of the result lists, in ascending row order, the rows of `a` with an
// entry in column c), handed to the device tensor as its cached transpose; host tensors keep none
template<typename Dtype>
inline void send_transpose(SpTensor<CPU, Dtype>&, SpTensor<CPU, Dtype>&, std::vector<int>&, SpTensor<CPU, Dtype>&) {}
template<typename Dtype>
inline void send_transpose(SpTensor<CPU, Dtype>& a, SpTensor<CPU, Dtype>& t, std::vector<int>& cursor, SpTensor<GPU, Dtype>& out)
{
    const int m = (int)a.rows(), k = (int)a.cols(), nnz = a.data->nnz;
    t.Reshape({(size_t)k, (size_t)m});
    t.ResizeSp(nnz, k + 1);
    cursor.assign((size_t)k + 1, 0);
    const int* rp = a.data->row_ptr;
    const int* ci = a.data->col_idx;
    for (int e = 0; e < nnz; ++e) cursor[(size_t)ci[e] + 1]++;
    int* trp = t.data->row_ptr;
    trp[0] = 0;
    for (int c = 0; c < k; ++c) { trp[c + 1] = trp[c] + cursor[(size_t)c + 1]; cursor[c] = trp[c]; }
    for (int r = 0; r < m; ++r)
        for (int e = rp[r]; e < rp[r + 1]; ++e) {
            const int dst = cursor[ci[e]]++;
            t.data->col_idx[dst] = r;
            t.data->val[dst] = a.data->val[e];
        }
    out.SetTransposed(t);
}
}  // namespace detail

template<typename mode, typename Dtype>
class IMsgPass : public Factor
{
public:
    static std::string StrType() { return "IMsgPass"; }

    IMsgPass(std::string _name, bool _average) : Factor(_name, PropErr::N), average(_average) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase phase) override
    {
        ASSERT(operands.size() == 1, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        auto* gv = dynamic_cast<GraphVar*>(operands[0].get());
        ASSERT(gv && gv->graph, "message passing needs a bound GraphVar");
        auto& out = detail::sparse_var<mode, Dtype>(outputs[0], "IMsgPass").value;
        if (BuildOnDevice(gv->graph, out, phase)) return;
        InitCPUWeight(gv->graph);
        out.CopyFrom(cpu_weight);          // host -> device (or host -> host) copy of the three CSR arrays
        // training multiplies by the transpose in the backward pass: the matrix is on the host right now,
        // so its transpose goes along instead of being sorted out on the device later
        if (phase == Phase::TRAIN && TransposeForBackward()) detail::send_transpose(cpu_weight, cpu_transpose, cursor, out);
    }

    // layout facts about the last batch, gathered while the CSR was built (used to choose kernels)
    virtual const BatchLayout* Layout() const override { return &layout; }
    BatchLayout layout;

protected:
    virtual void InitCPUWeight(GraphStruct* graph) = 0;
    // Operands that are a grouping of the flat edge list can be built on the device from one copy
    // of that list; returns false where the host construction is to be used.
    virtual bool BuildOnDevice(GraphStruct*, SpTensor<mode, Dtype>&, Phase) { return false; }
    virtual bool TransposeForBackward() const { return false; }
    SpTensor<CPU, Dtype> cpu_weight, cpu_transpose;
    std::vector<int> cursor;
    bool average;
};

namespace detail
{
// val = 1, or 1 / row length when average is set (computed as the reference does: 1.0 / (double)size)
template<typename Dtype>
inline void fill_row_weights(const int* row_ptr, int rows, bool average, Dtype* val)
{
    if (!average) {
        std::fill(val, val + row_ptr[rows], (Dtype)1.0);
        return;
    }
    for (int i = 0; i < rows; ++i) {
        const int len = row_ptr[i + 1] - row_ptr[i];
        const Dtype weight = len ? (Dtype)(1.0 / (double)len) : (Dtype)1.0;
        std::fill(val + row_ptr[i], val + row_ptr[i + 1], weight);
    }
}

// CSR [num_rows, num_cols] on the device whose row y lists, in edge order, the tail x (payload_is_edge
// false) or the index (true) of every edge x -> y: one copy of the (x, y) pairs, then a stable
// grouping by y (gnnhip_csr_group_i32).
// with_transpose (node-to-node operand of a training pass, unit values): the same call groups the pairs by x
// as well and the result becomes the cached transpose of `out`.
inline void group_edges_on_device(GraphStruct* graph, bool payload_is_edge, bool average, size_t num_cols,
                                  SpTensor<GPU, float>& out, DTensor<GPU, int>& staging, bool with_transpose = false)
{
    static_assert(sizeof(std::pair<int, int>) == 2 * sizeof(int), "edge list is not a flat (x, y) array");
    const int E = (int)graph->num_edges, N = (int)graph->num_nodes;
    out.Reshape({(size_t)N, num_cols});
    out.ResizeSp(E, N + 1);
    staging.Reshape({(size_t)(payload_is_edge ? 3 : 2) * (size_t)std::max(E, 1)});
    int* pairs = staging.data->ptr;
    if (E > 0) GNN_HIP(gnnhip_memcpy_h2d(pairs, graph->edge_list.data(), sizeof(int) * 2 * (size_t)E, GpuHandle::Stream()));
    const int* payload = pairs;
    int payload_stride = 2;
    if (payload_is_edge) {
        // edge indices 0..E-1 behind the pairs
        DTensor<CPU, int> idx({(size_t)std::max(E, 1)});
        for (int e = 0; e < E; ++e) idx.data->ptr[e] = e;
        if (E > 0) GNN_HIP(gnnhip_memcpy_h2d(pairs + 2 * (size_t)E, idx.data->ptr, sizeof(int) * (size_t)E, GpuHandle::Stream()));
        payload = pairs + 2 * (size_t)E;
        payload_stride = 1;
    }
    if (with_transpose && !payload_is_edge && !average && num_cols == (size_t)N) {
        auto& t = out.AdoptTransposed();
        GNN_HIP(gnnhip_csr_group_both_i32(N, E, pairs, 2, pairs + 1, 2, out.data->row_ptr, out.data->col_idx, out.data->val,
                                          t.row_ptr, t.col_idx, t.val, GpuHandle::Stream()));
        return;
    }
    GNN_HIP(gnnhip_csr_group_i32(N, E, pairs + 1, 2, payload, payload_stride, average ? 1 : 0,
                                 out.data->row_ptr, out.data->col_idx, out.data->val, GpuHandle::Stream()));
}
// CSR [num_subgraph, num_nodes] on the device for nodes that were added subgraph after subgraph, each with the next
// index: the subgraph offsets (the host has just found them) travel, the device writes the entries.
// offsets[q] is set for q <= last; the subgraphs behind the last one that has nodes are empty.
inline void consecutive_rows_on_device(GraphStruct* graph, std::vector<int>& offsets, int last, int nodes, bool average,
                                       SpTensor<GPU, float>& out)
{
    const int B = (int)graph->num_subgraph;
    for (int q = last + 1; q <= B; ++q) offsets[q] = nodes;
    out.Reshape({(size_t)B, (size_t)graph->num_nodes});
    out.ResizeSp(nodes, B + 1);
    GNN_HIP(gnnhip_csr_consecutive_rows_host_f32(B, offsets.data(), average ? 1 : 0, out.data->row_ptr, out.data->col_idx, out.data->val,
                                                 GpuHandle::Stream()));
}
// The device groups a batch in one launch (up to 16 workgroups, each a run of the rows) when a run's counters
// (4 bytes per row) and the slots of all pairs (2.35 bytes each, with the lists and one bitmap) fit 160 KB of
// LDS, and with a radix sort from 65,536 pairs.  What is left to the host loop is what neither covers (fewer
// pairs than that over more than about 40,000 rows), where the dozen launches of the sort cost more than the loop.
constexpr size_t kRadixGroupingPairs = 1u << 16;
inline bool device_grouping_pays(size_t pairs, size_t rows)
{
    return pairs >= kRadixGroupingPairs || rows / 4 + 47 * pairs / 20 + 1024 <= 160 * 1024;
}
template<typename Dtype, typename SpT>
inline bool group_edges_if_gpu(GraphStruct*, bool, bool, size_t, SpT&, DTensor<GPU, int>&, bool = false) { return false; }
template<>
inline bool group_edges_if_gpu<float, SpTensor<GPU, float> >(GraphStruct* graph, bool payload_is_edge, bool average, size_t num_cols,
                                                             SpTensor<GPU, float>& out, DTensor<GPU, int>& staging, bool with_transpose)
{
    if (!device_grouping_pays(graph->num_edges, graph->num_nodes)) return false;
    group_edges_on_device(graph, payload_is_edge, average, num_cols, out, staging, with_transpose);
    return true;
}
template<typename Dtype, typename SpT>
inline bool consecutive_rows_if_gpu(GraphStruct*, std::vector<int>&, int, int, bool, SpT&) { return false; }
template<>
inline bool consecutive_rows_if_gpu<float, SpTensor<GPU, float> >(GraphStruct* graph, std::vector<int>& offsets, int last, int nodes,
                                                                  bool average, SpTensor<GPU, float>& out)
{
    consecutive_rows_on_device(graph, offsets, last, nodes, average, out);
    return true;
}
// Batches of up to this many nodes are examined on the host for edges between subgraphs (the one-launch
// forward needs to know before it is chosen); larger ones take the general kernels either way.
constexpr unsigned kExamineBlocksMaxNodes = 1u << 17;
}  // namespace detail

template<typename mode, typename Dtype>
class Node2NodeMsgPass : public IMsgPass<mode, Dtype>
{
public:
    static std::string StrType() { return "Node2NodeMsgPass"; }
    using OutType = std::shared_ptr< SpTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< SpTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    Node2NodeMsgPass(std::string _name, bool _average = false) : IMsgPass<mode, Dtype>(_name, _average) {}
    virtual const char* FuseKind() const override { return "msg_node2node"; }

protected:
    virtual bool TransposeForBackward() const override { return true; }
    virtual bool BuildOnDevice(GraphStruct* graph, SpTensor<mode, Dtype>& out, Phase phase) override
    {
        if (!detail::group_edges_if_gpu<Dtype>(graph, false, this->average, graph->num_nodes, out, edge_staging, phase == Phase::TRAIN))
            return false;
        this->layout.block_diagonal = graph->num_nodes <= detail::kExamineBlocksMaxNodes && NoEdgeBetweenSubgraphs(graph);
        return true;
    }
    DTensor<GPU, int> edge_staging;

    // does every edge stay inside one subgraph?  (node -> subgraph from the AddNode records: read in place when the
    // records came in node order, as GetBatch writes them, through a table otherwise)
    bool NoEdgeBetweenSubgraphs(GraphStruct* graph)
    {
        static_assert(sizeof(std::pair<int, int>) == 2 * sizeof(int), "node list is not a flat (subgraph, node) array");
        const auto& records = graph->node_list;
        const size_t N = graph->num_nodes;
        bool in_order = records.size() == N;
        for (size_t i = 0; in_order && i < N; ++i) in_order = (size_t)records[i].second == i;
        const int* where;
        size_t stride;
        if (in_order && N > 0) {
            where = &records[0].first;
            stride = 2;
        } else {
            node_subgraph.assign(N, -1);
            for (const auto& sn : records)
                if (sn.second >= 0 && sn.second < (int)N) node_subgraph[sn.second] = sn.first;
            where = node_subgraph.data();
            stride = 1;
        }
        int differ = 0;
        for (const auto& e : graph->edge_list) differ |= where[(size_t)e.first * stride] ^ where[(size_t)e.second * stride];
        return differ == 0;
    }

    virtual void InitCPUWeight(GraphStruct* graph) override
    {
        auto& w = this->cpu_weight;
        w.Reshape({graph->num_nodes, graph->num_nodes});
        w.ResizeSp((int)graph->num_edges, (int)graph->num_nodes + 1);
        int* rp = w.data->row_ptr;
        // rows from the flat edge list (stable by head node): the entries of in_edges->head[i], row after row
        graph->GroupEdgesByHead(false, rp, w.data->col_idx);
        detail::fill_row_weights(rp, (int)graph->num_nodes, this->average, w.data->val);
        this->layout.block_diagonal = NoEdgeBetweenSubgraphs(graph);
    }
    std::vector<int> node_subgraph;
};

template<typename mode, typename Dtype>
class Edge2NodeMsgPass : public IMsgPass<mode, Dtype>
{
public:
    static std::string StrType() { return "Edge2NodeMsgPass"; }
    using OutType = std::shared_ptr< SpTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< SpTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    Edge2NodeMsgPass(std::string _name, bool _average = false) : IMsgPass<mode, Dtype>(_name, _average) {}

protected:
    virtual bool BuildOnDevice(GraphStruct* graph, SpTensor<mode, Dtype>& out, Phase phase) override
    {
        return detail::group_edges_if_gpu<Dtype>(graph, true, this->average, graph->num_edges, out, edge_staging);
    }
    DTensor<GPU, int> edge_staging;

    virtual void InitCPUWeight(GraphStruct* graph) override
    {
        auto& w = this->cpu_weight;
        w.Reshape({graph->num_nodes, graph->num_edges});
        w.ResizeSp((int)graph->num_edges, (int)graph->num_nodes + 1);
        graph->GroupEdgesByHead(true, w.data->row_ptr, w.data->col_idx);
        detail::fill_row_weights(w.data->row_ptr, (int)graph->num_nodes, this->average, w.data->val);
    }
};

template<typename mode, typename Dtype>
class Node2EdgeMsgPass : public IMsgPass<mode, Dtype>
{
public:
    static std::string StrType() { return "Node2EdgeMsgPass"; }
    using OutType = std::shared_ptr< SpTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< SpTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    Node2EdgeMsgPass(std::string _name, bool _average = false) : IMsgPass<mode, Dtype>(_name, _average) {}

protected:
    virtual void InitCPUWeight(GraphStruct* graph) override
    {
        auto& w = this->cpu_weight;
        const int E = (int)graph->num_edges;
        w.Reshape({graph->num_edges, graph->num_nodes});
        w.ResizeSp(E, E + 1);
        for (int e = 0; e < E; ++e) {
            w.data->row_ptr[e] = e;
            w.data->col_idx[e] = graph->edge_list[e].first;
            w.data->val[e] = (Dtype)1.0;
        }
        w.data->row_ptr[E] = E;
    }
};

template<typename mode, typename Dtype>
class Edge2EdgeMsgPass : public IMsgPass<mode, Dtype>
{
public:
    static std::string StrType() { return "Edge2EdgeMsgPass"; }
    using OutType = std::shared_ptr< SpTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< SpTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    Edge2EdgeMsgPass(std::string _name, bool _average = false) : IMsgPass<mode, Dtype>(_name, _average) {}

protected:
    virtual void InitCPUWeight(GraphStruct* graph) override
    {
        auto& w = this->cpu_weight;
        const int E = (int)graph->num_edges;
        // entries: for every edge (x -> y), the edges that end in x and do not start in y
        size_t cnt = 0;
        for (int e = 0; e < E; ++e) {
            const int from = graph->edge_list[e].first, to = graph->edge_list[e].second;
            for (const auto& in : graph->in_edges->head[from]) cnt += (in.second != to);
        }
        w.Reshape({graph->num_edges, graph->num_edges});
        w.ResizeSp((int)cnt, E + 1);
        int nnz = 0;
        for (int e = 0; e < E; ++e) {
            w.data->row_ptr[e] = nnz;
            const int from = graph->edge_list[e].first, to = graph->edge_list[e].second;
            for (const auto& in : graph->in_edges->head[from]) {
                if (in.second == to) continue;           // the same edge in the other direction
                w.data->col_idx[nnz] = in.first;
                w.data->val[nnz] = (Dtype)1.0;
                ++nnz;
            }
        }
        w.data->row_ptr[E] = nnz;
        ASSERT(nnz == (int)cnt, "edge-to-edge entry count changed between the two passes");
    }
};

template<typename mode, typename Dtype>
class SubgraphMsgPass : public IMsgPass<mode, Dtype>
{
public:
    static std::string StrType() { return "SubgraphMsgPass"; }
    using OutType = std::shared_ptr< SpTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< SpTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    SubgraphMsgPass(std::string _name, bool _average = false) : IMsgPass<mode, Dtype>(_name, _average) {}
    virtual const char* FuseKind() const override { return "msg_subgraph"; }

protected:
    // Nodes added subgraph after subgraph, each with the next index (GetBatch does): the matrix is then the
    // identity layout, its facts are known from one pass over the records, and the device groups it.
    virtual bool BuildOnDevice(GraphStruct* graph, SpTensor<mode, Dtype>& out, Phase) override
    {
        const int M = (int)graph->node_list.size(), B = (int)graph->num_subgraph;
        if (M != (int)graph->num_nodes) return false;
        offsets.assign((size_t)B + 1, 0);
        int biggest = 0, prev = 0, start = 0;
        bool ordered = true;
        for (int i = 0; i < M && ordered; ++i) {
            const int g = graph->node_list[i].first;
            ordered = graph->node_list[i].second == i && g >= prev && g < B;
            if (g != prev && ordered) {
                biggest = std::max(biggest, i - start);
                for (int q = prev + 1; q <= g; ++q) offsets[q] = i;
                prev = g;
                start = i;
            }
        }
        if (!ordered || !detail::consecutive_rows_if_gpu<Dtype>(graph, offsets, prev, M, this->average, out)) return false;
        this->layout.contiguous_subgraphs = true;
        this->layout.max_subgraph_nodes = std::max(biggest, M - start);
        return true;
    }
    std::vector<int> offsets;

    virtual void InitCPUWeight(GraphStruct* graph) override
    {
        auto& w = this->cpu_weight;
        w.Reshape({graph->num_subgraph, graph->num_nodes});
        w.ResizeSp((int)graph->num_nodes, (int)graph->num_subgraph + 1);
        ASSERT(graph->node_list.size() == graph->num_nodes, "node count does not match the subgraph lists");
        int* rp = w.data->row_ptr;
        int* ci = w.data->col_idx;
        graph->GroupNodesBySubgraph(rp, ci);
        detail::fill_row_weights(rp, (int)graph->num_subgraph, this->average, w.data->val);
        int biggest = 0;
        bool contiguous = true;
        for (unsigned g = 0; g < graph->num_subgraph; ++g) biggest = std::max(biggest, rp[g + 1] - rp[g]);
        for (int i = 0; i < (int)graph->num_nodes; ++i) contiguous = contiguous && ci[i] == i;
        this->layout.contiguous_subgraphs = contiguous;
        this->layout.max_subgraph_nodes = biggest;
    }
};

}  // namespace gnn
#endif
