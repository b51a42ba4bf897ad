// Test driver for the host API layer: builds the structure2vec mean-field graph through
// FactorGraph / af<> / add_diff<> exactly as a graphnn user would, runs it on one batch with
// weights read from files, and writes what it computed so the Python test can compare with
// the CPU oracle:  inference pass (fused plan), training pass (folded forward + backward, then factor by
// factor), gradients, two optimizer steps, checkpoint.
//
//   host_forward_check <dir> K C H Q L [bridges]
//   bridges: that many extra undirected edges, node 0 of graph g to node 0 of graph g + 1 for g = 0 .. bridges - 1, added after
//   the graphs' own edges: the batch is then not block diagonal and takes the routes that accept any adjacency
//   <dir>/graphs.txt            dataset in graphnn's txt layout (all graphs form the batch)
//   <dir>/w_n2l.bin w_conv.bin w_h1.bin w_h2.bin   row-major fp32
//   -> <dir>/out.bin            see the write() calls at the bottom
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

static std::vector<float> read_floats(const std::string& path, size_t n)
{
    std::vector<float> v(n);
    FILE* f = fopen(path.c_str(), "rb");
    ASSERT(f, "cannot open " << path);
    ASSERT(fread(v.data(), sizeof(float), n, f) == n, "short read on " << path);
    fclose(f);
    return v;
}

static void upload(DTensor<mode, Dtype>& dst, const std::vector<float>& src, size_t rows, size_t cols)
{
    DTensor<CPU, Dtype> host({rows, cols});
    memcpy(host.data->ptr, src.data(), sizeof(float) * rows * cols);
    dst.CopyFrom(host);
}

static void append(std::vector<float>& out, DTensor<mode, Dtype>& t)
{
    DTensor<CPU, Dtype> host;
    host.CopyFrom(t);
    out.insert(out.end(), host.data->ptr, host.data->ptr + host.shape.Count());
}

int main(int argc, char** argv)
{
    ASSERT(argc == 7 || argc == 8, "usage: host_forward_check <dir> K C H Q L [bridges]");
    const std::string dir = argv[1];
    const size_t K = atoi(argv[2]), C = atoi(argv[3]), H = atoi(argv[4]), Q = atoi(argv[5]);
    const int L = atoi(argv[6]);
    const int bridges = argc == 8 ? atoi(argv[7]) : 0;
    GpuHandle::Init(0, 1);

    // ---- the batch: every graph of the file
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
    GraphStruct graph;
    graph.Resize(num_graph, N);
    DTensor<CPU, Dtype> x_cpu({N, K});
    x_cpu.Zeros();
    SpTensor<CPU, Dtype> y_cpu;
    y_cpu.Reshape({(size_t)num_graph, Q});
    y_cpu.ResizeSp(num_graph, num_graph + 1);
    size_t base = 0;
    int edge = 0;
    for (int g = 0; g < num_graph; ++g) {
        for (int j = 0; j < sizes[g]; ++j) {
            x_cpu.data->ptr[(base + j) * K + tags[g][j]] = 1.0f;
            graph.AddNode(g, (int)(base + j));
        }
        base += sizes[g];
    }
    base = 0;
    for (int g = 0; g < num_graph; ++g) {
        for (int j = 0; j < sizes[g]; ++j)
            for (int nb : nbrs[g][j]) graph.AddEdge(edge++, (int)(base + j), (int)(base + nb));
        y_cpu.data->row_ptr[g] = g;
        y_cpu.data->col_idx[g] = labels[g];
        y_cpu.data->val[g] = 1.0f;
        base += sizes[g];
    }
    y_cpu.data->row_ptr[num_graph] = num_graph;
    {
        std::vector<size_t> first(num_graph + 1, 0);
        for (int g = 0; g < num_graph; ++g) first[g + 1] = first[g] + sizes[g];
        for (int g = 0; g < bridges && g + 1 < num_graph; ++g) {
            graph.AddEdge(edge++, (int)first[g], (int)first[g + 1]);
            graph.AddEdge(edge++, (int)first[g + 1], (int)first[g]);
        }
    }
    DTensor<mode, Dtype> input;
    SpTensor<mode, Dtype> label;
    input.CopyFrom(x_cpu);
    label.CopyFrom(y_cpu);

    // ---- the model, declared through the public API
    FactorGraph fg;
    ParamSet<mode, Dtype> model;
    auto graph_var = add_const<GraphVar>(fg, "graph", true);
    auto a_n2n = af< Node2NodeMsgPass<mode, Dtype> >(fg, {graph_var});
    auto s_pool = af< SubgraphMsgPass<mode, Dtype> >(fg, {graph_var});
    auto w_n2l = add_diff<DTensorVar>(model, "w_n2l", {K, C});
    auto w_conv = add_diff<DTensorVar>(model, "w_conv", {C, C});
    auto w_h1 = add_diff<DTensorVar>(model, "w_h1", {C, H});
    auto w_h2 = add_diff<DTensorVar>(model, "w_h2", {H, Q});
    upload(w_n2l->value, read_floats(dir + "/w_n2l.bin", K * C), K, C);
    upload(w_conv->value, read_floats(dir + "/w_conv.bin", C * C), C, C);
    upload(w_h1->value, read_floats(dir + "/w_h1.bin", C * H), C, H);
    upload(w_h2->value, read_floats(dir + "/w_h2.bin", H * Q), H, Q);
    for (auto& p : {w_n2l, w_conv, w_h1, w_h2}) fg.AddParam(p);

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

    std::map<std::string, void*> feed;
    feed["data"] = &input;
    feed["label"] = &label;
    feed["graph"] = &graph;
    std::vector< std::shared_ptr<Variable> > targets = {loss, acc, logits};

    std::vector<float> out;
    // 1. inference: the plan folds the operator chains into the fused kernels
    fg.FeedForward(targets, feed, Phase::TEST);
    out.push_back((float)fg.LastPlanFactorCount());
    out.push_back((float)fg.LastPlanFusedCount());
    out.push_back(loss->AsScalar());
    out.push_back(acc->AsScalar());
    append(out, logits->value);
    {
        // loss and accuracy were fetched together behind one wait; a tensor written in place afterwards must be read
        // from the device again (graphnn's AsScalar reads the device every time)
        const float l0 = loss->AsScalar();
        loss->value.Scale(2.0f);
        ASSERT(loss->value.AsScalar() == 2.0f * l0, "AsScalar returned a value fetched before the tensor was rewritten");
        loss->value.Scale(0.5f);
        ASSERT(loss->value.AsScalar() == l0, "AsScalar after the second in-place write");
    }
    // 2. training pass: the plan folds the forward (keeping every level for its backward pass) and the loss tail
    fg.FeedForward(targets, feed, Phase::TRAIN);
    out.push_back((float)fg.LastPlanFactorCount());
    out.push_back((float)fg.LastPlanFusedCount());
    out.push_back(loss->AsScalar());
    out.push_back(acc->AsScalar());
    append(out, logits->value);
    // 3. gradients of the loss from the folded backward pass
    fg.BackPropagate({loss});
    for (auto& p : {w_n2l, w_conv, w_h1, w_h2}) {
        auto g = p->grad.Full();
        append(out, g);
    }
    // 3b. the same with every factor on its own (forward and backward as graphnn schedules them)
    fg.EnableFusion(false);
    fg.FeedForward(targets, feed, Phase::TRAIN);
    out.push_back((float)fg.LastPlanFactorCount());
    out.push_back((float)fg.LastPlanFusedCount());
    out.push_back(loss->AsScalar());
    append(out, h->value);
    fg.BackPropagate({loss});
    for (auto& p : {w_n2l, w_conv, w_h1, w_h2}) {
        auto g = p->grad.Full();
        append(out, g);
    }
    fg.EnableFusion(true);
    // 4. two momentum-SGD steps with weight decay (all four tensors in one launch each): weights after the first,
    //    gradients of the second iteration, weights after the second; then the loss
    MomentumSGDOptimizer<mode, Dtype> opt(&model, 0.01f, 0.9f, 0.001f);
    opt.Update();
    for (auto& p : {w_n2l, w_conv, w_h1, w_h2}) append(out, p->value);
    fg.FeedForward(targets, feed, Phase::TRAIN);
    fg.BackPropagate({loss});
    for (auto& p : {w_n2l, w_conv, w_h1, w_h2}) {
        auto g = p->grad.Full();
        append(out, g);
    }
    opt.Update();
    for (auto& p : {w_n2l, w_conv, w_h1, w_h2}) append(out, p->value);
    fg.FeedForward(targets, feed, Phase::TEST);
    out.push_back(loss->AsScalar());
    // 5. checkpoint round trip in graphnn's wire format
    model.Save(dir + "/model.bin");
    w_conv->value.Zeros();
    model.Load(dir + "/model.bin");
    fg.FeedForward(targets, feed, Phase::TEST);
    out.push_back(loss->AsScalar());

    FILE* f = fopen((dir + "/out.bin").c_str(), "wb");
    ASSERT(f, "cannot write out.bin");
    fwrite(out.data(), sizeof(float), out.size(), f);
    fclose(f);
    GpuHandle::Destroy();
    printf("host_forward_check ok: %d graphs, %zu nodes, %d edges\n", num_graph, N, edge);
    return 0;
}
