// Scheduler bodies of FactorGraph and the inference-time fusion of the structure2vec
// operator chains onto libgnnhip's fused kernels:
//
//   MatMul(sparse A, h) -> MatMul(., W) -> ElewiseAdd(., msg) -> ReLU      => gnnhip_s2v_level_f32
//   MatMul(dense X, W)  -> ReLU                                             => gnnhip_s2v_input_f32
//
// (the chains of examples/graph_classification/src/kernel_mean_field.cpp:31-47).  A chain
// is folded only at Phase::TEST and only when its intermediate variables have no other
// reader and are not requested as targets, because the fused kernels do not materialise
// them; training keeps every factor separate so Backward finds the values it needs.
#ifndef S2V_FUSION_H
#define S2V_FUSION_H

#include <algorithm>
#include <cstring>
#include <functional>
#include <queue>

namespace gnn
{

namespace detail
{
struct FusedStep
{
    std::vector<size_t> factors;            // graph factors this step stands for
    std::function<void(Phase)> run;
    bool fused;
};
}  // namespace detail

inline size_t FactorGraph::LastPlanFactorCount() const { return last_plan ? last_plan->steps.size() : 0; }
inline size_t FactorGraph::LastPlanFusedCount() const { return last_plan ? last_plan->n_fused : 0; }

inline FactorGraph::Plan* FactorGraph::GetPlan(const std::vector<VarPtr>& targets,
                                               const std::map<std::string, void*>& feed_dict, Phase phase)
{
    std::vector<size_t> t_idx, f_idx;
    for (auto& p : targets) t_idx.push_back(VarIdx(p));
    for (auto& kv : feed_dict) f_idx.push_back(VarIdx(kv.first));
    for (auto& pl : plans)
        if (pl->version == version && pl->phase == phase && pl->target_idx == t_idx && pl->feed_idx == f_idx) return pl.get();
    // the graph changed or this request is new: drop stale plans, build a fresh one
    plans.erase(std::remove_if(plans.begin(), plans.end(),
                               [&](const std::unique_ptr<Plan>& pl) { return pl->version != version; }), plans.end());
    std::unique_ptr<Plan> plan(new Plan());
    plan->version = version;
    plan->phase = phase;
    plan->target_idx = t_idx;
    plan->feed_idx = f_idx;
    BuildPlan(*plan);
    plans.push_back(std::move(plan));
    return plans.back().get();
}

inline void FactorGraph::BuildPlan(Plan& plan)
{
    const size_t nv = var_list.size(), nf = factor_list.size();
    // which variables the targets depend on (walk producers backwards)
    plan.required.assign(nv, false);
    std::vector<size_t> stack(plan.target_idx.begin(), plan.target_idx.end());
    for (size_t v : stack) plan.required[v] = true;
    while (!stack.empty()) {
        size_t v = stack.back();
        stack.pop_back();
        for (size_t f : var_nodes[v].producers)
            for (size_t u : factor_nodes[f].in)
                if (!plan.required[u]) { plan.required[u] = true; stack.push_back(u); }
    }
    // Kahn's algorithm from the variables that are available up front
    std::vector<bool> ready(nv, false);
    for (size_t v : always_ready) ready[v] = true;
    for (size_t v : plan.feed_idx) ready[v] = true;
    std::vector<size_t> pending(nf);
    for (size_t f = 0; f < nf; ++f) pending[f] = factor_nodes[f].in.size();
    std::queue<size_t> q;
    for (size_t f = 0; f < nf; ++f) if (pending[f] == 0) q.push(f);           // factors without operands
    auto release = [&](size_t v) {
        for (size_t f : var_nodes[v].consumers)
            if (pending[f] && --pending[f] == 0) q.push(f);
    };
    for (size_t v = 0; v < nv; ++v) if (ready[v]) release(v);
    plan.order.clear();
    plan.executed.assign(nf, false);
    while (!q.empty()) {
        size_t f = q.front();
        q.pop();
        bool necessary = false;
        for (size_t v : factor_nodes[f].out) necessary = necessary || plan.required[v];
        if (!necessary) continue;
        plan.order.push_back(f);
        plan.executed[f] = true;
        for (size_t v : factor_nodes[f].out) { ready[v] = true; release(v); }
    }
    for (size_t v : plan.target_idx)
        ASSERT(ready[v], "required variable " << var_list[v]->name << " is not ready");
    BuildFusedSteps(plan);
}

inline void FactorGraph::BuildFusedSteps(Plan& plan)
{
    typedef DTensorVar<GPU, float> DVar;
    typedef SpTensorVar<GPU, float> SVar;
    plan.steps.clear();
    plan.n_fused = 0;
    std::vector<bool> taken(factor_list.size(), false);
    std::vector<bool> is_target(var_list.size(), false);
    for (size_t v : plan.target_idx) is_target[v] = true;

    auto kind = [&](size_t f) { return factor_list[f]->FuseKind(); };
    // the one factor of this plan that reads v, if v is private to it (single reader, not a target)
    auto sole_reader = [&](size_t v, size_t& reader) {
        if (is_target[v]) return false;
        size_t n = 0;
        for (size_t f : var_nodes[v].consumers) if (plan.executed[f]) { reader = f; ++n; }
        // readers outside the plan do not run, so they do not need the value
        return n == 1;
    };
    auto gpu_dense = [&](size_t v) { return dynamic_cast<DVar*>(var_list[v].get()); };
    auto gpu_sparse = [&](size_t v) { return dynamic_cast<SVar*>(var_list[v].get()); };
    auto single_step = [&](size_t f) {
        auto step = std::make_shared<detail::FusedStep>();
        step->factors.push_back(f);
        step->fused = false;
        auto fac = factor_list[f];
        auto ins = std::make_shared<VarList>();
        auto outs = std::make_shared<VarList>();
        for (size_t v : factor_nodes[f].in) ins->push_back(var_list[v]);
        for (size_t v : factor_nodes[f].out) outs->push_back(var_list[v]);
        step->run = [fac, ins, outs](Phase ph) { fac->Forward(*ins, *outs, ph); };
        return step;
    };

    const bool fold = fusion_enabled && plan.phase == Phase::TEST;
    for (size_t f1 : plan.order) {
        if (taken[f1]) continue;
        bool done = false;
        if (fold && !strcmp(kind(f1), "matmul_nn") && factor_nodes[f1].in.size() == 2 && factor_nodes[f1].out.size() == 1) {
            const size_t a = factor_nodes[f1].in[0], b = factor_nodes[f1].in[1], p1 = factor_nodes[f1].out[0];
            size_t f2 = 0, f3 = 0, f4 = 0;
            // ---- level: sparse x dense, then dense x dense, then + msg, then ReLU
            if (gpu_sparse(a) && gpu_dense(b) && gpu_dense(p1) && sole_reader(p1, f2) && !taken[f2] &&
                !strcmp(kind(f2), "matmul_nn") && factor_nodes[f2].in[0] == p1 && gpu_dense(factor_nodes[f2].in[1])) {
                const size_t w = factor_nodes[f2].in[1], p2 = factor_nodes[f2].out[0];
                if (sole_reader(p2, f3) && !taken[f3] && !strcmp(kind(f3), "elewise_add2") && factor_nodes[f3].in.size() == 2) {
                    const size_t other = factor_nodes[f3].in[0] == p2 ? factor_nodes[f3].in[1] : factor_nodes[f3].in[0];
                    const size_t p3 = factor_nodes[f3].out[0];
                    if (other != p2 && gpu_dense(other) && sole_reader(p3, f4) && !taken[f4] && !strcmp(kind(f4), "relu") &&
                        gpu_dense(factor_nodes[f4].out[0])) {
                        SVar* A = gpu_sparse(a);
                        DVar *H = gpu_dense(b), *W = gpu_dense(w), *M = gpu_dense(other), *O = gpu_dense(factor_nodes[f4].out[0]);
                        auto step = std::make_shared<detail::FusedStep>();
                        step->factors = {f1, f2, f3, f4};
                        step->fused = true;
                        step->run = [A, H, W, M, O](Phase) {
                            ASSERT(A->value.cols() == H->value.rows() && H->value.cols() == W->value.rows() &&
                                   W->value.rows() == W->value.cols() && M->value.shape == H->value.shape &&
                                   A->value.rows() == H->value.rows(),
                                   "fused level: operand shapes do not chain");
                            O->value.Reshape(H->value.shape.dims);
                            GNN_HIP(gnnhip_s2v_level_f32((int)H->value.rows(), (int)H->value.cols(), A->value.data->nnz, A->value.data->row_ptr,
                                                         A->value.data->col_idx, A->value.data->val, H->value.data->ptr,
                                                         W->value.data->ptr, M->value.data->ptr, nullptr,
                                                         O->value.data->ptr, GpuHandle::Stream()));
                        };
                        for (size_t f : step->factors) taken[f] = true;
                        plan.steps.push_back(step);
                        plan.n_fused++;
                        done = true;
                    }
                }
            }
            // ---- input: dense x dense followed by a ReLU of the product (the product itself stays available)
            if (!done && gpu_dense(a) && gpu_dense(b) && gpu_dense(p1)) {
                size_t fr = (size_t)-1;
                for (size_t f : var_nodes[p1].consumers)
                    if (plan.executed[f] && !taken[f] && !strcmp(kind(f), "relu") && gpu_dense(factor_nodes[f].out[0])) { fr = f; break; }
                if (fr != (size_t)-1) {
                    DVar *X = gpu_dense(a), *W = gpu_dense(b), *M = gpu_dense(p1), *O = gpu_dense(factor_nodes[fr].out[0]);
                    auto step = std::make_shared<detail::FusedStep>();
                    step->factors = {f1, fr};
                    step->fused = true;
                    step->run = [X, W, M, O](Phase) {
                        ASSERT(X->value.rank() == 2 && W->value.rank() == 2 && X->value.cols() == W->value.rows(), "mat dim doesn't match");
                        M->value.Reshape({X->value.rows(), W->value.cols()});
                        O->value.Reshape({X->value.rows(), W->value.cols()});
                        GNN_HIP(gnnhip_s2v_input_f32((int)X->value.rows(), (int)X->value.cols(), (int)W->value.cols(),
                                                     X->value.data->ptr, W->value.data->ptr, M->value.data->ptr,
                                                     O->value.data->ptr, GpuHandle::Stream()));
                    };
                    for (size_t f : step->factors) taken[f] = true;
                    plan.steps.push_back(step);
                    plan.n_fused++;
                    done = true;
                }
            }
        }
        if (!done) {
            taken[f1] = true;
            plan.steps.push_back(single_step(f1));
        }
    }
}

inline FactorGraph::VarList FactorGraph::FeedForward(std::vector<VarPtr> targets, std::map<std::string, void*> feed_dict,
                                                     Phase phase, uint n_thread)
{
    if (n_thread != 1) throw std::runtime_error("not implemented");
    Plan* plan = GetPlan(targets, feed_dict, phase);
    for (auto& kv : feed_dict) var_dict[kv.first].second->SetRef(kv.second);
    for (auto& step : plan->steps) step->run(phase);
    last_plan = plan;
    return VarList(targets.begin(), targets.end());
}

// Reverse sweep over the factors the last FeedForward executed.  A factor runs its Backward once
// every reader of each of its outputs has contributed, it propagates errors (PropErr::T), at least
// one output carries a gradient and at least one operand is differentiable
// (the rules of src/nn/factor_graph.cpp:182-270).
inline void FactorGraph::BackPropagate(std::vector<VarPtr> targets, uint n_thread)
{
    if (n_thread != 1) throw std::runtime_error("not implemented");
    ASSERT(last_plan && last_plan->version == version, "unexpected change of computation graph in backward stage");
    Plan& plan = *last_plan;
    ASSERT(plan.n_fused == 0, "BackPropagate needs a FeedForward run with Phase::TRAIN (inference plans fuse factors)");
    const size_t nv = var_list.size(), nf = factor_list.size();

    var_has_grad.assign(nv, false);
    for (size_t v = 0; v < nv; ++v)
        if (!isConst[v])
            if (auto* d = dynamic_cast<IDifferentiable*>(var_list[v].get())) d->ZeroGrad();
    for (auto& p : targets) {
        const size_t v = VarIdx(p);
        ASSERT(var_nodes[v].consumers.empty(), "only allow backprop from top variables");
        ASSERT(!isConst[v], "cannot calc grad for const variable");
        if (auto* d = dynamic_cast<IDifferentiable*>(p.get())) { var_has_grad[v] = true; d->OnesGrad(); }
    }

    std::vector<size_t> readers_left(nv, 0), outputs_left(nf, 0);
    for (size_t v = 0; v < nv; ++v)
        for (size_t f : var_nodes[v].consumers) if (plan.executed[f]) readers_left[v]++;
    std::queue<size_t> q;
    for (size_t f = 0; f < nf; ++f) {
        for (size_t v : factor_nodes[f].out)
            if (plan.required[v] && !var_nodes[v].consumers.empty()) outputs_left[f]++;
        if (outputs_left[f] == 0 && plan.executed[f]) q.push(f);
    }

    std::vector<bool> const_flags;
    while (!q.empty()) {
        const size_t f = q.front();
        q.pop();
        auto& node = factor_nodes[f];
        bool run = factor_list[f]->properr == PropErr::T;
        if (run) {
            bool has_grad = false, need_prop = false;
            for (size_t v : node.out) if (!isConst[v]) has_grad = has_grad || var_has_grad[v];
            const_flags.assign(node.in.size(), true);
            if (has_grad)
                for (size_t i = 0; i < node.in.size(); ++i) {
                    const_flags[i] = isConst[node.in[i]];
                    need_prop = need_prop || !const_flags[i];
                }
            run = has_grad && need_prop;
        }
        if (run) {
            VarList ins, outs;
            for (size_t v : node.in) ins.push_back(var_list[v]);
            for (size_t v : node.out) outs.push_back(var_list[v]);
            factor_list[f]->Backward(ins, const_flags, outs);
            for (size_t i = 0; i < node.in.size(); ++i) if (!const_flags[i]) var_has_grad[node.in[i]] = true;
        }
        for (size_t v : node.in) {
            ASSERT(readers_left[v], "variable " + var_list[v]->name + " has more visits than expected");
            if (--readers_left[v]) continue;
            for (size_t p : var_nodes[v].producers)
                if (outputs_left[p] && --outputs_left[p] == 0) q.push(p);
        }
    }
}

}  // namespace gnn
#endif
