// Test driver for the operators of the path that graphnn's example does not use itself: FullyConnected
// (the "+ b" of the level), JaggedSoftmax (per-subgraph softmax over node scores) and Reduce, through
// FactorGraph as a graphnn user would write them:
//
//   msg = MatMul(X, w_n2l); h = ReLU(msg)
//   L x: h = ReLU(ElewiseAdd(FullyConnected(MatMul(A, h), fc[C+1, C]), msg))        level with bias row
//   score = MatMul(h, w_score[C,1]); att = JaggedSoftmax(score, lens)               lens = nodes per graph
//   pool = MatMul(S, h)
//   z = MatMul(att^T, h)  [1, C];  obj = Reduce(SUM)(z);  pm = Reduce(MEAN)(pool)
//
//   host_ops_check <dir> K C L
//   <dir>/graphs.txt, w_n2l.bin [K,C], fc.bin [C+1,C], w_score.bin [C,1]  ->  <dir>/out.bin
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

static void upload_file(DTensor<mode, Dtype>& dst, const std::string& path, size_t rows, size_t cols)
{
    DTensor<CPU, Dtype> host({rows, cols});
    FILE* f = fopen(path.c_str(), "rb");
    ASSERT(f, "cannot open " << path);
    ASSERT(fread(host.data->ptr, sizeof(float), rows * cols, f) == rows * cols, "short read on " << path);
    fclose(f);
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
    ASSERT(argc == 5, "usage: host_ops_check <dir> K C L");
    const std::string dir = argv[1];
    const size_t K = atoi(argv[2]), C = atoi(argv[3]);
    const int L = atoi(argv[4]);
    GpuHandle::Init(0, 1);

    std::ifstream ff(dir + "/graphs.txt");
    ASSERT(ff.good(), "cannot open the graph file");
    int num_graph;
    ff >> num_graph;
    std::vector<int> sizes(num_graph);
    std::vector< std::vector<int> > tags(num_graph);
    std::vector< std::vector< std::vector<int> > > nbrs(num_graph);
    size_t N = 0;
    for (int g = 0; g < num_graph; ++g) {
        int label;
        ff >> sizes[g] >> label;
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
    DTensor<CPU, int> lens_cpu({(size_t)num_graph});
    size_t base = 0;
    int edge = 0;
    for (int g = 0; g < num_graph; ++g) {
        lens_cpu.data->ptr[g] = sizes[g];
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
        base += sizes[g];
    }
    DTensor<mode, Dtype> input;
    DTensor<mode, int> lens;
    input.CopyFrom(x_cpu);
    lens.CopyFrom(lens_cpu);

    FactorGraph fg;
    ParamSet<mode, Dtype> model;
    auto graph_var = add_const<GraphVar>(fg, "graph", true);
    auto a_n2n = af< Node2NodeMsgPass<mode, Dtype> >(fg, {graph_var});
    auto s_pool = af< SubgraphMsgPass<mode, Dtype> >(fg, {graph_var});
    auto w_n2l = add_diff<DTensorVar>(model, "w_n2l", {K, C});
    auto fc = add_diff<DTensorVar>(model, "fc", {C + 1, C});
    auto w_score = add_diff<DTensorVar>(model, "w_score", {C, (size_t)1});
    upload_file(w_n2l->value, dir + "/w_n2l.bin", K, C);
    upload_file(fc->value, dir + "/fc.bin", C + 1, C);
    upload_file(w_score->value, dir + "/w_score.bin", C, 1);
    for (auto& p : {w_n2l, fc, w_score}) fg.AddParam(p);

    auto x_var = add_const< DTensorVar<mode, Dtype> >(fg, "data", true);
    auto lens_var = add_const< DTensorVar<mode, int> >(fg, "lens", true);
    auto msg = af<MatMul>(fg, {x_var, w_n2l});
    auto h = af<ReLU>(fg, {msg});
    for (int lv = 0; lv < L; ++lv) {
        auto pooled = af<MatMul>(fg, {a_n2n, h});
        auto lin = af<FullyConnected>(fg, {pooled, fc});
        auto merged = af<ElewiseAdd>(fg, {lin, msg});
        h = af<ReLU>(fg, {merged});
    }
    auto score = af<MatMul>(fg, {h, w_score});
    typedef std::vector< std::shared_ptr<Variable> > Ops;
    auto att = af< JaggedSoftmax<mode, Dtype> >(fg, Ops{score, lens_var});
    auto pool = af<MatMul>(fg, {s_pool, h});
    auto z = af<MatMul>(fg, {att, h}, Trans::T, Trans::N);
    auto obj = af<Reduce>(fg, {z}, ReduceType::SUM);
    auto pm = af<Reduce>(fg, {pool}, ReduceType::MEAN);

    std::map<std::string, void*> feed;
    feed["data"] = &input;
    feed["lens"] = &lens;
    feed["graph"] = &graph;
    std::vector< std::shared_ptr<Variable> > targets = {obj, pm, att, pool};

    std::vector<float> out;
    for (Phase ph : {Phase::TEST, Phase::TRAIN}) {
        fg.FeedForward(targets, feed, ph);
        out.push_back((float)fg.LastPlanFactorCount());
        out.push_back((float)fg.LastPlanFusedCount());
        out.push_back(obj->AsScalar());
        out.push_back(pm->AsScalar());
        append(out, att->value);
        append(out, pool->value);
    }
    fg.BackPropagate({obj});
    for (auto& p : {w_n2l, fc, w_score}) {
        auto g = p->grad.Full();
        append(out, g);
    }
    // one Adam update from those gradients (threshold 0.5: the clipping factor is in play), then the parameters
    AdamOptimizer<mode, Dtype> adam(&model, 0.01f, 0.001f);
    adam.clip_threshold = 0.5f;
    adam.Update();
    for (auto& p : {w_n2l, fc, w_score}) append(out, p->value);
    FILE* f = fopen((dir + "/out.bin").c_str(), "wb");
    ASSERT(f, "cannot write out.bin");
    fwrite(out.data(), sizeof(float), out.size(), f);
    fclose(f);
    GpuHandle::Destroy();
    printf("host_ops_check ok: %d graphs, %zu nodes, %d edges\n", num_graph, N, edge);
    return 0;
}
