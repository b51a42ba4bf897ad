// Times what graphnn's example does per test batch (examples/graph_classification/include/nn_common.h:36-105,
// 140-160): build the batch on the host (GraphStruct lists, one-hot node features, label CSR), copy it to
// the device, FactorGraph::FeedForward in the TEST phase, read loss and accuracy back.
//
//   host_forward_bench <dir> K C H Q L reps [train]
//   <dir>/graphs.txt  dataset in graphnn's txt layout (all graphs form the batch); weights are random
// Prints one JSON line with microseconds per batch: whole, host batch build, copies + forward + read-back.
// With "train" every batch runs what the example's training loop runs (nn_common.h:158-171):
// FeedForward in the TRAIN phase, BackPropagate from the loss, one momentum-SGD update; the loss is read
// back once at the end, as the example only reads it on report iterations.
#include <chrono>
#include <cmath>
#include <cstdio>
#include <fstream>
#include <map>
#include <string>
#include <vector>
#include "tensor/tensor_all.h"
#include "nn/nn_all.h"

using namespace gnn;
typedef GPU mode;
typedef float Dtype;
typedef std::chrono::steady_clock Clock;

static double us_since(Clock::time_point t0)
{
    return std::chrono::duration<double, std::micro>(Clock::now() - t0).count();
}

int main(int argc, char** argv)
{
    ASSERT(argc == 8 || argc == 9, "usage: host_forward_bench <dir> K C H Q L reps [train]");
    const bool train = argc == 9 && std::string(argv[8]) == "train";
    const std::string dir = argv[1];
    const size_t K = atoi(argv[2]), C = atoi(argv[3]), H = atoi(argv[4]), Q = atoi(argv[5]);
    const int L = atoi(argv[6]), reps = atoi(argv[7]);
    GpuHandle::Init(0, 1);

    std::ifstream ff(dir + "/graphs.txt");
    ASSERT(ff.good(), "cannot open the graph file");
    int num_graph;
    ff >> num_graph;
    std::vector<int> sizes(num_graph), labels(num_graph);
    std::vector< std::vector<int> > tags(num_graph);
    std::vector< std::vector< std::vector<int> > > nbrs(num_graph);
    size_t N = 0;
    for (int g = 0; g < num_graph; ++g) {
        ff >> sizes[g] >> labels[g];
        tags[g].resize(sizes[g]);
        nbrs[g].resize(sizes[g]);
        for (int j = 0; j < sizes[g]; ++j) {
            int m;
            ff >> tags[g][j] >> m;
            nbrs[g][j].resize(m);
            for (int k = 0; k < m; ++k) ff >> nbrs[g][j][k];
        }
        N += sizes[g];
    }

    FactorGraph fg;
    ParamSet<mode, Dtype> model;
    auto graph_var = add_const<GraphVar>(fg, "graph", true);
    auto a_n2n = af< Node2NodeMsgPass<mode, Dtype> >(fg, {graph_var});
    auto s_pool = af< SubgraphMsgPass<mode, Dtype> >(fg, {graph_var});
    auto w_n2l = add_diff<DTensorVar>(model, "w_n2l", {K, C});
    auto w_conv = add_diff<DTensorVar>(model, "w_conv", {C, C});
    auto w_h1 = add_diff<DTensorVar>(model, "w_h1", {C, H});
    auto w_h2 = add_diff<DTensorVar>(model, "w_h2", {H, Q});
    // (standard deviation 0.1 at hidden 64, scaled down with the width so that the embeddings of wide networks stay finite)
    const float w_std = 0.1f * std::sqrt(64.0f / (float)(C > 64 ? C : 64));
    for (auto& p : {w_n2l, w_conv, w_h1, w_h2}) { p->value.SetRandN(0, w_std); fg.AddParam(p); }
    auto x_var = add_const< DTensorVar<mode, Dtype> >(fg, "data", true);
    auto y_var = add_const< SpTensorVar<mode, Dtype> >(fg, "label", true);
    auto msg = af<MatMul>(fg, {x_var, w_n2l});
    auto h = af<ReLU>(fg, {msg});
    for (int lv = 0; lv < L; ++lv) {
        auto pooled = af<MatMul>(fg, {a_n2n, h});
        auto lin = af<MatMul>(fg, {pooled, w_conv});
        auto merged = af<ElewiseAdd>(fg, {lin, msg});
        h = af<ReLU>(fg, {merged});
    }
    auto y_pot = af<MatMul>(fg, {s_pool, h});
    auto hidden = af<ReLU>(fg, {af<MatMul>(fg, {y_pot, w_h1})});
    auto logits = af<MatMul>(fg, {hidden, w_h2});
    auto ce = af<CrossEntropy>(fg, {logits, y_var}, true);
    auto loss = af<ReduceMean>(fg, {ce});
    auto truth = af<ArgMax>(fg, {y_var});
    auto hit = af< InTopK<mode, Dtype> >(fg, std::make_pair(logits, truth));
    auto acc = af<ReduceMean>(fg, {af< TypeCast<mode, Dtype> >(fg, {hit})});

    GraphStruct graph;
    DTensor<CPU, Dtype> x_cpu;
    SpTensor<CPU, Dtype> y_cpu;
    DTensor<mode, Dtype> input;
    SpTensor<mode, Dtype> label;
    std::map<std::string, void*> feed;
    feed["data"] = &input;
    feed["label"] = &label;
    feed["graph"] = &graph;
    std::vector< std::shared_ptr<Variable> > targets = {loss, acc};
    std::vector< std::shared_ptr<Variable> > objs = {loss};
    MomentumSGDOptimizer<mode, Dtype> learner(&model, 0.001f, 0.9f, 0.0001f);

    double t_build = 0, t_device = 0;
    float checksum = 0;
    const int warm = 5;
    for (int it = 0; it < reps + warm; ++it) {
        const Clock::time_point t0 = Clock::now();
        // ---- the batch, as GetBatch assembles it
        graph.Resize(num_graph, N);
        x_cpu.Reshape({N, K});
        x_cpu.Zeros();
        y_cpu.Reshape({(size_t)num_graph, Q});
        y_cpu.ResizeSp(num_graph, num_graph + 1);
        size_t base = 0;
        int edge = 0;
        for (int g = 0; g < num_graph; ++g) {
            for (int j = 0; j < sizes[g]; ++j) {
                x_cpu.data->ptr[(base + j) * K + tags[g][j]] = 1.0f;
                graph.AddNode(g, (int)(base + j));
            }
            for (int j = 0; j < sizes[g]; ++j)
                for (int nb : nbrs[g][j]) graph.AddEdge(edge++, (int)(base + j), (int)(base + nb));
            y_cpu.data->row_ptr[g] = g;
            y_cpu.data->col_idx[g] = labels[g];
            y_cpu.data->val[g] = 1.0f;
            base += sizes[g];
        }
        y_cpu.data->row_ptr[num_graph] = num_graph;
        const double b = us_since(t0);
        const Clock::time_point t1 = Clock::now();
        input.CopyFrom(x_cpu);
        label.CopyFrom(y_cpu);
        if (train) {
            fg.FeedForward(targets, feed, Phase::TRAIN);
            fg.BackPropagate(objs);
            learner.Update();
            if (it + 1 == reps + warm || it + 1 == warm) checksum += loss->AsScalar();     // drains the stream
        } else {
            fg.FeedForward(targets, feed, Phase::TEST);  // builds the CSR of A and S on the host, copies, runs
            checksum += loss->AsScalar() + acc->AsScalar();
        }
        const double d = us_since(t1);
        if (it >= warm) { t_build += b; t_device += d; }
    }
    GpuHandle::Destroy();
    printf("{\"graphs\": %d, \"nodes\": %zu, \"reps\": %d, \"mode\": \"%s\", \"us_per_batch\": %.2f, \"us_host_batch_build\": %.2f, "
           "\"%s\": %.2f, \"fused_factors\": %d, \"plan_steps\": %d, \"checksum\": %.6f}\n",
           num_graph, N, reps, train ? "train" : "test", (t_build + t_device) / reps, t_build / reps,
           train ? "us_csr_copy_forward_backward_update" : "us_csr_copy_forward_readback", t_device / reps,
           (int)fg.LastPlanFusedCount(), (int)fg.LastPlanFactorCount(), std::isfinite(checksum) ? checksum : -1.0f);
    return 0;
}
