// CPU-only check of FactorGraph's inference plan: a folded chain must run after the producers of ALL of
// its operands.  Builds (and never runs) a graph in which msg comes out of a deeper chain than the fed
// embedding, so the sparse product of the level is ready long before msg is:
//
//   msg = MatMul(ReLU(MatMul(X, W0)), W1)              depth 3
//   out = ReLU(ElewiseAdd(MatMul(MatMul(A, h), W), msg))   with A and h fed
//
// Prints the plan; exits non-zero if the level step precedes the step that produces msg.
#include <cstdio>
#include <map>
#include <string>
#include <vector>
#include "tensor/tensor_all.h"
#include "nn/nn_all.h"

using namespace gnn;
typedef GPU mode;
typedef float Dtype;

static int step_of(const std::vector< std::vector<std::string> >& plan, const std::string& factor)
{
    for (size_t i = 0; i < plan.size(); ++i)
        for (auto& f : plan[i]) if (f == factor) return (int)i;
    return -1;
}

int main()
{
    FactorGraph fg;
    auto x = add_const< DTensorVar<mode, Dtype> >(fg, "x", true);
    auto h = add_const< DTensorVar<mode, Dtype> >(fg, "h", true);
    auto a = add_const< SpTensorVar<mode, Dtype> >(fg, "a", true);
    auto w0 = add_const< DTensorVar<mode, Dtype> >(fg, "w0", false);
    auto w1 = add_const< DTensorVar<mode, Dtype> >(fg, "w1", false);
    auto w = add_const< DTensorVar<mode, Dtype> >(fg, "w", false);

    typedef std::vector< std::shared_ptr<Variable> > Ops;
    typedef MatMul<mode, Dtype> MM;
    // the level's factors are registered FIRST, so Kahn's order reaches the sparse product before msg exists
    auto pooled = af<MM>(fg, Ops{a, h});
    const std::string f_pool = fg.factor_list.back()->name;
    auto lin = af<MM>(fg, Ops{pooled, w});
    auto pre = af<MM>(fg, Ops{x, w0});
    auto act = af< ReLU<mode, Dtype> >(fg, Ops{pre});
    auto msg = af<MM>(fg, Ops{act, w1});
    const std::string f_msg = fg.factor_list.back()->name;
    auto merged = af< ElewiseAdd<mode, Dtype> >(fg, Ops{lin, msg});
    auto out = af< ReLU<mode, Dtype> >(fg, Ops{merged});
    const std::string f_out = fg.factor_list.back()->name;

    std::map<std::string, void*> feed;
    feed["x"] = nullptr; feed["h"] = nullptr; feed["a"] = nullptr;      // PlanSteps runs nothing
    std::vector< std::shared_ptr<Variable> > targets = {out};
    auto plan = fg.PlanSteps(targets, feed, Phase::TEST);
    for (size_t i = 0; i < plan.size(); ++i) {
        printf("step %zu:", i);
        for (auto& f : plan[i]) printf(" %s", f.c_str());
        printf("\n");
    }
    const int s_level = step_of(plan, f_pool), s_msg = step_of(plan, f_msg);
    ASSERT(s_level >= 0 && s_msg >= 0, "factors missing from the plan");
    ASSERT(s_level == step_of(plan, f_out) && plan[s_level].size() == 4, "the level chain was not folded into one step");
    if (s_msg >= s_level) {
        fprintf(stderr, "the folded level (step %d) runs before msg is produced (step %d)\n", s_level, s_msg);
        return 1;
    }
    // operator by operator the same graph keeps the order of factor_graph.cpp's scheduler
    auto plain = fg.PlanSteps(targets, feed, Phase::TRAIN);
    ASSERT(plain.size() == 7, "seven factors must run one by one in the TRAIN phase");
    printf("host_plan_check ok\n");
    return 0;
}
