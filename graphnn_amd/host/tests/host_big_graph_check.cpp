// Test driver for one large graph with many entries per row (the shape of a power-law graph) through graphnn's API:
// the sparse operand is then large and dense enough for the library to plan its products, and SpTensor<GPU> keeps
// that plan from the first product until the matrix is rebuilt.
//
//   1. tensor level: C1 = A * B, C2 = A * B again (same plan), Ct = A^T * B (the transpose and its plan), then A's values
//      are replaced (CopyFrom: the plans are dropped) and C3 = A' * B;
//   2. FactorGraph (TEST phase): msg = MatMul(X, w_n2l); h = ReLU(msg); L x h = ReLU(ElewiseAdd(MatMul(MatMul(A, h), w), msg))
//      with A from Node2NodeMsgPass over the same edges: every level is one fused step with the plan of A.
//
//   host_big_graph_check <dir> N K C L
//   <dir>/edges.bin (int32 pairs x y, E of them), val.bin [E] (values for step 1, in CSR order), val2.bin [E], b.bin [N,C],
//   x.bin [N,K], w_n2l.bin [K,C], w.bin [C,C]   ->   <dir>/out.bin = C1, C2, Ct, C3, h_L (each [N,C])
#include <cstdio>
#include <map>
#include <string>
#include <vector>
#include "tensor/tensor_all.h"
#include "nn/nn_all.h"

using namespace gnn;
typedef GPU mode;
typedef float Dtype;

template<typename T>
static std::vector<T> read_all(const std::string& path)
{
    FILE* f = fopen(path.c_str(), "rb");
    ASSERT(f, "cannot open " << path);
    fseek(f, 0, SEEK_END);
    const size_t bytes = (size_t)ftell(f);
    fseek(f, 0, SEEK_SET);
    std::vector<T> v(bytes / sizeof(T));
    ASSERT(fread(v.data(), sizeof(T), v.size(), f) == v.size(), "short read on " << path);
    fclose(f);
    return v;
}

static void upload(DTensor<mode, Dtype>& dst, const std::vector<float>& src, size_t rows, size_t cols)
{
    ASSERT(src.size() == rows * cols, "file does not hold " << rows << " x " << cols << " floats");
    DTensor<CPU, Dtype> host({rows, cols});
    std::copy(src.begin(), src.end(), host.data->ptr);
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
    ASSERT(argc == 6, "usage: host_big_graph_check <dir> N K C L");
    const std::string dir = argv[1];
    const size_t N = atoi(argv[2]), K = atoi(argv[3]), C = atoi(argv[4]);
    const int L = atoi(argv[5]);
    GpuHandle::Init(0, 1);
    const std::vector<int> edges = read_all<int>(dir + "/edges.bin");
    const size_t E = edges.size() / 2;
    GraphStruct graph;
    graph.Resize(1, N);
    for (size_t i = 0; i < N; ++i) graph.AddNode(0, (int)i);
    for (size_t e = 0; e < E; ++e) graph.AddEdge((int)e, edges[2 * e], edges[2 * e + 1]);

    // ---- 1. the matrix as Node2NodeMsgPass lists it (row = head y, entries = tails x in insertion order), with values
    SpTensor<CPU, Dtype> a_cpu;
    a_cpu.Reshape({N, N});
    a_cpu.ResizeSp((int)E, (int)N + 1);
    {
        std::vector<int> cnt(N + 1, 0);
        for (size_t e = 0; e < E; ++e) cnt[edges[2 * e + 1] + 1]++;
        for (size_t i = 0; i < N; ++i) cnt[i + 1] += cnt[i];
        std::copy(cnt.begin(), cnt.end(), a_cpu.data->row_ptr);
        std::vector<int> at(cnt.begin(), cnt.end() - 1);
        for (size_t e = 0; e < E; ++e) a_cpu.data->col_idx[at[edges[2 * e + 1]]++] = edges[2 * e];
    }
    const std::vector<float> val = read_all<float>(dir + "/val.bin"), val2 = read_all<float>(dir + "/val2.bin");
    ASSERT(val.size() == E && val2.size() == E, "val files do not hold one value per edge");
    std::copy(val.begin(), val.end(), a_cpu.data->val);
    SpTensor<mode, Dtype> a;
    a.CopyFrom(a_cpu);
    DTensor<mode, Dtype> b, c1, c2, ct, c3;
    upload(b, read_all<float>(dir + "/b.bin"), N, C);
    std::vector<float> out;
    c1.MM(a, b, Trans::N, Trans::N, 1.0f, 0.0f);
    const bool planned = a.Plan() != nullptr;
    c2.MM(a, b, Trans::N, Trans::N, 1.0f, 0.0f);
    ct.MM(a, b, Trans::T, Trans::N, 1.0f, 0.0f);
    const bool t_planned = a.TransposedPlan() != nullptr;
    append(out, c1);
    append(out, c2);
    append(out, ct);
    std::copy(val2.begin(), val2.end(), a_cpu.data->val);
    a.CopyFrom(a_cpu);                                   // new contents: the plans of the old ones must not be used
    c3.MM(a, b, Trans::N, Trans::N, 1.0f, 0.0f);
    append(out, c3);

    // ---- 2. L fused levels over the operand that Node2NodeMsgPass builds (unit values)
    FactorGraph fg;
    ParamSet<mode, Dtype> model;
    auto graph_var = add_const<GraphVar>(fg, "graph", true);
    auto a_n2n = af< Node2NodeMsgPass<mode, Dtype> >(fg, {graph_var});
    auto w_n2l = add_diff<DTensorVar>(model, "w_n2l", {K, C});
    auto w = add_diff<DTensorVar>(model, "w", {C, C});
    upload(w_n2l->value, read_all<float>(dir + "/w_n2l.bin"), K, C);
    upload(w->value, read_all<float>(dir + "/w.bin"), C, C);
    for (auto& p : {w_n2l, w}) fg.AddParam(p);
    DTensor<mode, Dtype> input;
    upload(input, read_all<float>(dir + "/x.bin"), N, K);
    auto x_var = add_const< DTensorVar<mode, Dtype> >(fg, "data", true);
    auto msg = af<MatMul>(fg, {x_var, w_n2l});
    auto h = af<ReLU>(fg, {msg});
    for (int lv = 0; lv < L; ++lv) {
        auto pooled = af<MatMul>(fg, {a_n2n, h});
        auto lin = af<MatMul>(fg, {pooled, w});
        auto merged = af<ElewiseAdd>(fg, {lin, msg});
        h = af<ReLU>(fg, {merged});
    }
    std::map<std::string, void*> feed;
    feed["data"] = &input;
    feed["graph"] = &graph;
    fg.FeedForward({h}, feed, Phase::TEST);
    const int fused = fg.LastPlanFusedCount();
    append(out, h->value);
    FILE* f = fopen((dir + "/out.bin").c_str(), "wb");
    ASSERT(f, "cannot write out.bin");
    fwrite(out.data(), sizeof(float), out.size(), f);
    fclose(f);
    printf("host_big_graph_check ok: %zu nodes, %zu edges, planned %d, transpose planned %d, fused steps %d\n", N, E, (int)planned,
           (int)t_planned, fused);
    GpuHandle::Destroy();
    return 0;
}
