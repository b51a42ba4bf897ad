// CPU-only driver for the sanitizer build of the host layer (make -C graphnn_amd/host asan): batch assembly as graphnn's
// GetBatch does it (examples/graph_classification/include/nn_common.h:36-105), several batches of different sizes through
// the same host tensors and the same GraphStruct.  It keeps the example's sizing of the feature rows: the row width is the
// LARGEST TAG (kernel_mean_field.cpp:75-85), so a node that carries that tag sets the float one past its row, and in the
// last row one past the tensor; the host allocator leaves 64 bytes of slack behind every block for exactly this write,
// which must therefore stay inside the allocation under AddressSanitizer.
//
//   host_batch_check        prints "host_batch_check ok" and the checksum of the features it wrote
#include <cstdio>
#include <map>
#include <string>
#include <vector>
#include "tensor/tensor_all.h"
#include "nn/nn_all.h"

using namespace gnn;
typedef float Dtype;

int main()
{
    DTensor<CPU, Dtype> x_cpu;
    SpTensor<CPU, Dtype> y_cpu;
    GraphStruct graph;
    // the operands of a batch, built on the host from the graph's lists by the message-pass factors in CPU mode
    FactorGraph fg;
    auto gv = add_const<GraphVar>(fg, "graph", true);
    auto a_var = af< Node2NodeMsgPass<CPU, Dtype> >(fg, {gv}, false);
    auto s_var = af< SubgraphMsgPass<CPU, Dtype> >(fg, {gv}, true);
    std::map<std::string, void*> feed;
    feed["graph"] = &graph;
    const int node_dim = 7, num_class = 2;             // tags 0..7: the largest one is node_dim itself
    unsigned state = 12345u;
    auto next = [&]() { state = state * 1664525u + 1013904223u; return state >> 8; };
    double checksum = 0;
    for (int round = 0; round < 6; ++round) {
        const unsigned num = 3 + (round * 5) % 11;      // graphs in this batch: up and down, so buffers grow and are reused
        std::vector<unsigned> sizes(num), prefix(num);
        unsigned node_cnt = 0;
        for (unsigned i = 0; i < num; ++i) { sizes[i] = 1 + next() % 9; prefix[i] = node_cnt; node_cnt += sizes[i]; }
        graph.Resize(num, node_cnt);
        x_cpu.Reshape({node_cnt, (uint)node_dim});
        x_cpu.Zeros();
        y_cpu.Reshape({num, (uint)num_class});
        y_cpu.ResizeSp(num, num + 1);
        Dtype* ptr = x_cpu.data->ptr;
        for (unsigned i = 0; i < num; ++i)
            for (unsigned j = 0; j < sizes[i]; ++j) {
                // the last node of the batch always carries the largest tag: the write past the tensor
                const int tag = (i + 1 == num && j + 1 == sizes[i]) ? node_dim : (int)(next() % (node_dim + 1));
                ptr[tag] = 1.0;
                ptr += node_dim;
                graph.AddNode(i, prefix[i] + j);
            }
        int cur_edge = 0;
        for (unsigned i = 0; i < num; ++i)
            for (unsigned j = 1; j < sizes[i]; ++j) {
                const unsigned p = next() % j;
                graph.AddEdge(cur_edge, prefix[i] + j, prefix[i] + p);
                graph.AddEdge(cur_edge + 1, prefix[i] + p, prefix[i] + j);
                cur_edge += 2;
            }
        for (unsigned i = 0; i < num; ++i) {
            y_cpu.data->row_ptr[i] = i;
            y_cpu.data->val[i] = 1.0;
            y_cpu.data->col_idx[i] = next() % num_class;
        }
        y_cpu.data->row_ptr[num] = num;
        fg.FeedForward({a_var, s_var}, feed, Phase::TEST);
        auto& a = a_var->value;
        auto& s = s_var->value;
        ASSERT(a.data->nnz == cur_edge && s.data->nnz == (int)node_cnt, "operand sizes are off");
        for (size_t t = 0; t < (size_t)node_cnt * node_dim; ++t) checksum += x_cpu.data->ptr[t] * (double)(1 + t % 13);
        for (int e = 0; e < a.data->nnz; ++e) checksum += a.data->col_idx[e];
        for (int e = 0; e < s.data->nnz; ++e) checksum += s.data->val[e];
    }
    printf("host_batch_check ok: checksum %.1f\n", checksum);
    return 0;
}
