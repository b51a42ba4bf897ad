// Scheduler bodies of FactorGraph and the inference-time fusion of the structure2vec
// operator chains onto libgnnhip's fused kernels:
//
//   MatMul(sparse A, h) -> MatMul(., W) -> ElewiseAdd(., msg) -> ReLU      => gnnhip_s2v_level_f32
//   MatMul(dense X, W)  -> ReLU                                             => gnnhip_s2v_input_f32
//   input -> levels -> MatMul(S, h) -> MatMul(., W1) -> ReLU -> MatMul(., W2), when the batch is laid
//   out as GetBatch lays it out (contiguous graphs, no edge between graphs)  => gnnhip_s2v_forward_batched_f32
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
// What the folded forward of a training plan keeps for its backward pass.
struct TrainState
{
    DTensor<GPU, float> hstack;             // [(L + 1) N, C]: the embeddings of every level, h0 first
    DTensor<GPU, float> ustack;             // [L N, C]: A^T dz of every level
    DTensor<GPU, float> g, g2, dmsg, dl, du;   // [N, C] x 3, [B, Q], [B, H]
    DTensor<GPU, float>* probs = nullptr;   // the CrossEntropy factor's probabilities (filled by the loss tail)
    SpTensorVar<GPU, float>* label = nullptr;
    size_t loss_var = (size_t)-1;           // the variable BackPropagate must start from
    bool loss_attached = false;             // a folded loss tail reads this forward's logits
    bool fused_ran = false;                 // the last forward took the folded route (else the factors ran one by one)
};

struct FusedStep
{
    std::vector<size_t> factors;            // graph factors this step stands for
    std::function<void(Phase)> run;
    bool fused;
    enum Tag { SINGLE, INPUT, LEVEL, FORWARD, LOSS } tag = SINGLE;
    std::vector<size_t> vars;               // INPUT: X, W, msg, h0;  LEVEL: A, h_in, W, msg, h_out;  FORWARD: logits
    bool bias_row = false;                  // LEVEL through FullyConnected: W may carry a bias row
    std::shared_ptr<TrainState> train;      // FORWARD of a training plan
    std::function<void()> backward;         // FORWARD of a training plan: gradients of the four weight matrices
};
// Larger batches run the forward as separate kernels.  Inference: the one-launch forward packs the graphs of
// batches past 512 graphs into bins and stays ahead up to about 4,000 graphs of 29 nodes (98 against 124 us at
// 3,000 graphs, 130 against 139 us at 4,000, 165 against 155 us at 5,000).  Training keeps every level and takes
// the graphs one by one: there the separate kernels win from about 20,000 nodes.
constexpr size_t kOneLaunchMaxNodes = 120000;
constexpr size_t kOneLaunchTrainMaxNodes = 20000;
}  // namespace detail

// The factor names of every step of the plan a FeedForward with these arguments would run, in
// execution order (a folded step lists the factors it stands for).  Runs nothing.
inline std::vector< std::vector<std::string> > FactorGraph::PlanSteps(std::vector<VarPtr> targets,
                                                                      std::map<std::string, void*> feed_dict, Phase phase)
{
    Plan* plan = GetPlan(targets, feed_dict, phase);
    std::vector< std::vector<std::string> > out;
    for (auto& step : plan->steps) {
        out.emplace_back();
        for (size_t f : step->factors) out.back().push_back(factor_list[f]->name);
    }
    return out;
}

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

inline std::shared_ptr<detail::FusedStep> FactorGraph::MakeSingleStep(size_t f)
{
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
}

// Inference plans fold whatever chain they recognise.  A training plan folds only what still lets
// BackPropagate work: the loss tail (it leaves behind what the factors' Backward read), and the whole forward
// when the loss tail hangs off its logits (the folded forward then brings its own backward pass).
inline void FactorGraph::BuildFusedSteps(Plan& plan)
{
    if (plan.phase == Phase::TEST) {
        BuildSteps(plan, fusion_enabled);
        if (fusion_enabled) { FoldWholeForward(plan); FoldLossTail(plan); }
        return;
    }
    if (fusion_enabled) {
        BuildSteps(plan, true);
        FoldWholeForward(plan);
        FoldLossTail(plan);
        bool ok = true;
        for (auto& st : plan.steps)
            if (st->fused && st->tag != detail::FusedStep::LOSS &&
                !(st->tag == detail::FusedStep::FORWARD && st->train && st->train->loss_attached)) ok = false;
        if (ok) return;
    }
    BuildSteps(plan, false);
    if (fusion_enabled) FoldLossTail(plan);
}

inline void FactorGraph::BuildSteps(Plan& plan, bool fold)
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
    auto single_step = [&](size_t f) { return MakeSingleStep(f); };

    // A folded chain runs where its LAST factor stood in the order: only there are the operands of all
    // of its factors ready (msg and W enter the level at its second and third factor, and their
    // producers may sit anywhere before those, e.g. behind the sparse product when msg comes out of a
    // deeper chain than h_in does).
    std::vector< std::shared_ptr<detail::FusedStep> > emit_at(factor_list.size());
    for (size_t f1 : plan.order) {
        if (taken[f1]) {
            if (emit_at[f1]) plan.steps.push_back(emit_at[f1]);
            continue;
        }
        bool done = false;
        if (fold && !strcmp(kind(f1), "matmul_nn") && factor_nodes[f1].in.size() == 2 && factor_nodes[f1].out.size() == 1) {
            const size_t a = factor_nodes[f1].in[0], b = factor_nodes[f1].in[1], p1 = factor_nodes[f1].out[0];
            size_t f2 = 0, f3 = 0, f4 = 0;
            // ---- level: sparse x dense, then dense x dense, then + msg, then ReLU
            if (gpu_sparse(a) && gpu_dense(b) && gpu_dense(p1) && sole_reader(p1, f2) && !taken[f2] &&
                (!strcmp(kind(f2), "matmul_nn") || !strcmp(kind(f2), "fully_connected")) && factor_nodes[f2].in.size() == 2 &&
                factor_nodes[f2].in[0] == p1 && gpu_dense(factor_nodes[f2].in[1])) {
                const bool through_fc = !strcmp(kind(f2), "fully_connected");
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
                        step->tag = detail::FusedStep::LEVEL;
                        step->vars = {a, b, w, other, factor_nodes[f4].out[0]};
                        step->bias_row = through_fc;
                        step->run = [A, H, W, M, O, through_fc](Phase) {
                            const size_t C = H->value.cols();
                            // FullyConnected: rows [0, C) of the parameter are the weights, row C (if there) the bias
                            const bool bias = through_fc && W->value.rows() == C + 1;
                            ASSERT(A->value.cols() == H->value.rows() && W->value.cols() == C &&
                                   (W->value.rows() == C || bias) && M->value.shape == H->value.shape &&
                                   A->value.rows() == H->value.rows(),
                                   "fused level: operand shapes do not chain");
                            O->value.Reshape(H->value.shape.dims);
                            // a matrix large and dense enough for the library to plan keeps its plan across the levels
                            if (void* plan = A->value.Plan())
                                GNN_HIP(gnnhip_s2v_level_planned_f32(plan, (int)C, H->value.data->ptr, W->value.data->ptr, M->value.data->ptr,
                                                                     bias ? W->value.data->ptr + C * C : nullptr, O->value.data->ptr,
                                                                     GpuHandle::Stream()));
                            else
                                GNN_HIP(gnnhip_s2v_level_f32((int)H->value.rows(), (int)C, A->value.data->nnz, A->value.data->row_ptr,
                                                             A->value.data->col_idx, A->value.data->val, H->value.data->ptr,
                                                             W->value.data->ptr, M->value.data->ptr,
                                                             bias ? W->value.data->ptr + C * C : nullptr,
                                                             O->value.data->ptr, GpuHandle::Stream()));
                        };
                        for (size_t f : step->factors) taken[f] = true;
                        emit_at[f4] = step;                 // f4 reads f3 reads f2 reads f1: it is the last of the four
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
                    step->tag = detail::FusedStep::INPUT;
                    step->vars = {a, b, p1, factor_nodes[fr].out[0]};
                    step->run = [X, W, M, O](Phase) {
                        ASSERT(X->value.rank() == 2 && W->value.rank() == 2 && X->value.cols() == W->value.rows(), "mat dim doesn't match");
                        M->value.Reshape({X->value.rows(), W->value.cols()});
                        O->value.Reshape({X->value.rows(), W->value.cols()});
                        GNN_HIP(gnnhip_s2v_input_f32((int)X->value.rows(), (int)X->value.cols(), (int)W->value.cols(),
                                                     X->value.data->ptr, W->value.data->ptr, M->value.data->ptr,
                                                     O->value.data->ptr, GpuHandle::Stream()));
                    };
                    for (size_t f : step->factors) taken[f] = true;
                    plan.steps.push_back(step);             // both operands are f1's; other readers of the product may precede the ReLU
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

// Second pass over the steps: input + a chain of levels with one A and one W + the readout
// MatMul(S, h) -> MatMul(., W1) -> ReLU -> MatMul(., W2) become one step that, batch by batch, calls the
// one-launch graph-resident forward when the batch is block diagonal with contiguous graphs (facts the
// message-pass factors record while they build their operands) and the library covers the shape, and
// otherwise runs the steps it replaced.  The one-launch kernel keeps the inner levels' embeddings and
// the pre-activation of the hidden layer in LDS, so those variables must be private to the chain.
inline void FactorGraph::FoldWholeForward(Plan& plan)
{
    typedef DTensorVar<GPU, float> DVar;
    typedef SpTensorVar<GPU, float> SVar;
    typedef detail::FusedStep Step;
    auto& steps = plan.steps;
    std::vector<bool> is_target(var_list.size(), false);
    for (size_t v : plan.target_idx) is_target[v] = true;
    auto dense = [&](size_t v) { return dynamic_cast<DVar*>(var_list[v].get()); };
    auto sparse = [&](size_t v) { return dynamic_cast<SVar*>(var_list[v].get()); };
    auto find_step = [&](std::function<bool(const Step&)> pred) -> int {
        for (size_t i = 0; i < steps.size(); ++i) if (steps[i] && pred(*steps[i])) return (int)i;
        return -1;
    };
    auto single_of_kind = [&](const Step& st, const char* k) {
        return st.tag == Step::SINGLE && st.factors.size() == 1 && !strcmp(factor_list[st.factors[0]]->FuseKind(), k);
    };

    for (size_t si = 0; si < steps.size(); ++si) {
        if (!steps[si] || steps[si]->tag != Step::INPUT) continue;
        const size_t vX = steps[si]->vars[0], vWn = steps[si]->vars[1], vMsg = steps[si]->vars[2], vH0 = steps[si]->vars[3];
        std::vector<int> chain = {(int)si};
        // ---- levels
        size_t cur = vH0, vA = (size_t)-1, vWc = (size_t)-1;
        std::vector<size_t> inner;                       // embeddings the one-launch kernel does not write
        for (;;) {
            const int li = find_step([&](const Step& st) {
                return st.tag == Step::LEVEL && !st.bias_row && st.vars[1] == cur && st.vars[3] == vMsg &&
                       (vA == (size_t)-1 || (st.vars[0] == vA && st.vars[2] == vWc));
            });
            if (li < 0) break;
            vA = steps[li]->vars[0];
            vWc = steps[li]->vars[2];
            inner.push_back(cur);
            cur = steps[li]->vars[4];
            chain.push_back(li);
        }
        const int L = (int)chain.size() - 1;
        if (L < 1) continue;
        // ---- readout
        const int i5 = find_step([&](const Step& st) {
            return single_of_kind(st, "matmul_nn") && sparse(factor_nodes[st.factors[0]].in[0]) && factor_nodes[st.factors[0]].in[1] == cur;
        });
        if (i5 < 0) continue;
        const size_t vS = factor_nodes[steps[i5]->factors[0]].in[0], vPool = factor_nodes[steps[i5]->factors[0]].out[0];
        // the hidden layer: MatMul + ReLU, already folded into one input-style step or still two factors
        size_t vW1, vLin, vHid;
        int i6 = find_step([&](const Step& st) { return st.tag == Step::INPUT && st.vars[0] == vPool; });
        int i7 = -1;
        if (i6 >= 0) {
            vW1 = steps[i6]->vars[1]; vLin = steps[i6]->vars[2]; vHid = steps[i6]->vars[3];
        } else {
            i6 = find_step([&](const Step& st) {
                return single_of_kind(st, "matmul_nn") && factor_nodes[st.factors[0]].in[0] == vPool && dense(factor_nodes[st.factors[0]].in[1]);
            });
            if (i6 < 0) continue;
            vW1 = factor_nodes[steps[i6]->factors[0]].in[1];
            vLin = factor_nodes[steps[i6]->factors[0]].out[0];
            i7 = find_step([&](const Step& st) { return single_of_kind(st, "relu") && factor_nodes[st.factors[0]].in[0] == vLin; });
            if (i7 < 0) continue;
            vHid = factor_nodes[steps[i7]->factors[0]].out[0];
        }
        const int i8 = find_step([&](const Step& st) {
            return single_of_kind(st, "matmul_nn") && factor_nodes[st.factors[0]].in[0] == vHid && dense(factor_nodes[st.factors[0]].in[1]);
        });
        if (i8 < 0) continue;
        const size_t vW2 = factor_nodes[steps[i8]->factors[0]].in[1], vLogits = factor_nodes[steps[i8]->factors[0]].out[0];
        if (!(dense(vX) && dense(vWn) && dense(vWc) && dense(vW1) && dense(vW2) && dense(vPool) && dense(vHid) && dense(vLogits) &&
              dense(vMsg) && dense(cur) && sparse(vA) && sparse(vS))) continue;
        chain.push_back(i5); chain.push_back(i6); if (i7 >= 0) chain.push_back(i7); chain.push_back(i8);

        // ---- everything between X and the logits is read inside the chain only; what the kernel keeps
        //      in LDS is not a target either
        std::vector<bool> in_chain(factor_list.size(), false);
        for (int c : chain) for (size_t f : steps[c]->factors) in_chain[f] = true;
        auto private_to_chain = [&](size_t v) {
            for (size_t f : var_nodes[v].consumers) if (plan.executed[f] && !in_chain[f]) return false;
            return true;
        };
        bool ok = private_to_chain(vMsg) && private_to_chain(cur) && private_to_chain(vPool) && private_to_chain(vLin) &&
                  private_to_chain(vHid) && !is_target[vLin];
        inner.erase(inner.begin());                     // h0 is tested with the other inner embeddings below
        ok = ok && private_to_chain(vH0) && !is_target[vH0];
        for (size_t v : inner) ok = ok && private_to_chain(v) && !is_target[v];
        // the operands must come from the message-pass factors that know the batch layout
        auto producer = [&](size_t v) -> Factor* {
            return var_nodes[v].producers.size() == 1 ? factor_list[var_nodes[v].producers[0]].get() : nullptr;
        };
        Factor* fa = producer(vA);
        Factor* fs = producer(vS);
        if (!ok || !fa || !fs || strcmp(fa->FuseKind(), "msg_node2node") || strcmp(fs->FuseKind(), "msg_subgraph")) continue;
        const BatchLayout* n2n = fa->Layout();
        const BatchLayout* sub = fs->Layout();
        if (!n2n || !sub) continue;

        std::vector< std::shared_ptr<Step> > parts;
        std::sort(chain.begin(), chain.end());
        for (int c : chain) parts.push_back(steps[c]);
        auto step = std::make_shared<Step>();
        step->fused = true;
        step->tag = Step::FORWARD;
        for (auto& p : parts) step->factors.insert(step->factors.end(), p->factors.begin(), p->factors.end());
        DVar *X = dense(vX), *Wn = dense(vWn), *Wc = dense(vWc), *W1 = dense(vW1), *W2 = dense(vW2), *Msg = dense(vMsg),
             *Hl = dense(cur), *Pool = dense(vPool), *Hid = dense(vHid), *Logits = dense(vLogits);
        SVar *A = sparse(vA), *S = sparse(vS);
        DVar* H0 = dense(vH0);                           // h0: the second embedding buffer of the general route
        step->vars = {vLogits};
        if (plan.phase == Phase::TRAIN) {
            // ---- training: every level's embedding is kept (stacked), and the step carries its backward pass.
            // The factors it stands for, one by one and in plan order, are the fallback for batches the folded
            // route does not take; BackPropagate then walks them as usual.
            std::vector<size_t> pos(factor_list.size(), 0);
            for (size_t i = 0; i < plan.order.size(); ++i) pos[plan.order[i]] = i;
            std::vector<size_t> fs_sorted = step->factors;
            std::sort(fs_sorted.begin(), fs_sorted.end(), [&](size_t x, size_t y) { return pos[x] < pos[y]; });
            std::vector< std::shared_ptr<Step> > singles;
            for (size_t f : fs_sorted) singles.push_back(MakeSingleStep(f));
            auto st = std::make_shared<detail::TrainState>();
            step->train = st;
            const bool cWn = isConst[vWn], cWc = isConst[vWc], cW1 = isConst[vW1], cW2 = isConst[vW2];
            step->run = [=](Phase ph) {
                const size_t N = X->value.rows(), K = X->value.cols(), C = Wn->value.cols(), H = W1->value.cols(),
                             Q = W2->value.cols(), B = S->value.rows();
                ASSERT(Wn->value.rows() == K && Wc->value.rows() == C && Wc->value.cols() == C && W1->value.rows() == C &&
                       W2->value.rows() == H && A->value.rows() == N && A->value.cols() == N && S->value.cols() == N,
                       "fused forward: operand shapes do not chain");
                // the folded backward needs S to list every node once and the per-graph LDS of its readout kernel
                st->fused_ran = st->loss_attached && sub->contiguous_subgraphs && (Q + H + C) * 4 <= 64 * 1024;
                if (!st->fused_ran) {
                    for (auto& p : singles) p->run(ph);
                    return;
                }
                void* s = GpuHandle::Stream();
                const size_t NC = N * C;
                st->hstack.Reshape({(size_t)(L + 1) * N, C});
                Msg->value.Reshape({N, C});
                Pool->value.Reshape({B, C});
                Hid->value.Reshape({B, H});
                Logits->value.Reshape({B, Q});
                float* hs = st->hstack.data->ptr;
                // small block-diagonal batches: everything in one launch, the levels stored on the way
                if (n2n->block_diagonal && sub->max_subgraph_nodes > 0 && N <= detail::kOneLaunchTrainMaxNodes) {
                    const int rc = gnnhip_s2v_forward_batched_train_f32(
                        (int)N, (int)B, (int)K, (int)C, (int)H, (int)Q, L, sub->max_subgraph_nodes,
                        A->value.data->row_ptr, A->value.data->col_idx, A->value.data->val,
                        S->value.data->row_ptr, S->value.data->col_idx, S->value.data->val,
                        X->value.data->ptr, Wn->value.data->ptr, Wc->value.data->ptr, W1->value.data->ptr, W2->value.data->ptr,
                        Msg->value.data->ptr, hs, Pool->value.data->ptr, Hid->value.data->ptr, Logits->value.data->ptr,
                        nullptr, nullptr, nullptr, s);
                    if (rc == GNNHIP_OK) return;
                    ASSERT(rc == GNNHIP_EUNSUPPORTED, gnnhip_last_error());
                }
                GNN_HIP(gnnhip_s2v_input_f32((int)N, (int)K, (int)C, X->value.data->ptr, Wn->value.data->ptr, Msg->value.data->ptr, hs, s));
                void* a_plan = A->value.Plan();
                for (int l = 0; l < L; ++l) {
                    if (a_plan)
                        GNN_HIP(gnnhip_s2v_level_planned_f32(a_plan, (int)C, hs + (size_t)l * NC, Wc->value.data->ptr, Msg->value.data->ptr,
                                                             nullptr, hs + (size_t)(l + 1) * NC, s));
                    else
                        GNN_HIP(gnnhip_s2v_level_f32((int)N, (int)C, A->value.data->nnz, A->value.data->row_ptr, A->value.data->col_idx,
                                                     A->value.data->val, hs + (size_t)l * NC, Wc->value.data->ptr, Msg->value.data->ptr,
                                                     nullptr, hs + (size_t)(l + 1) * NC, s));
                }
                GNN_HIP(gnnhip_s2v_readout_f32((int)B, (int)N, (int)C, (int)H, (int)Q, S->value.data->row_ptr, S->value.data->col_idx,
                                               S->value.data->val, hs + (size_t)L * NC, W1->value.data->ptr, W2->value.data->ptr,
                                               Pool->value.data->ptr, Hid->value.data->ptr, Logits->value.data->ptr, nullptr, nullptr, s));
            };
            // Backward of the folded forward (the gradient rules of src/nn/matmul.cpp:35-76, src/nn/relu.cu:18-37,
            // src/nn/elewise_add.cpp:35-52, src/nn/cross_entropy.cpp:52-78 and src/nn/reduce_mean.cpp:44-65 composed):
            //   g_L = S^T ((dlogits W2^T . [hidden > 0]) W1^T),  dlogits = (probs - y) / B
            //   dz_L = g_L . [h_L > 0];  dmsg = dz_L
            //   level l = L..1:  u_l = A^T dz_l;  dz_{l-1} = (u_l W^T) . [h_{l-1} > 0];  dmsg += dz_{l-1}
            //   dW_conv += [h_0; ..; h_{L-1}]^T [u_1; ..; u_L],  dW_n2l += X^T dmsg,  dW_h1 += pool^T du,  dW_h2 += hidden^T dlogits
            // (A^T dz_l serves both the gradient of W, h_{l-1}^T (A^T dz_l) = (A h_{l-1})^T dz_l, and g_{l-1}.)
            step->backward = [=]() {
                ASSERT(st->fused_ran && st->probs && st->label, "folded backward without a folded forward");
                const size_t N = X->value.rows(), K = X->value.cols(), C = Wn->value.cols(), H = W1->value.cols(),
                             Q = W2->value.cols(), B = S->value.rows();
                const size_t NC = N * C;
                void* s = GpuHandle::Stream();
                st->g.Reshape({N, C});
                st->g2.Reshape({N, C});
                st->dmsg.Reshape({N, C});
                st->dl.Reshape({B, Q});
                st->du.Reshape({B, H});
                if (L > 0) st->ustack.Reshape({(size_t)L * N, C});
                auto& lab = st->label->value;
                GNN_HIP(gnnhip_s2v_readout_backward_f32((int)B, (int)N, (int)C, (int)H, (int)Q, S->value.data->row_ptr,
                                                        S->value.data->col_idx, S->value.data->val, st->probs->data->ptr,
                                                        lab.data->row_ptr, lab.data->col_idx, lab.data->val, 1.0f / (float)B,
                                                        Hid->value.data->ptr, W1->value.data->ptr, W2->value.data->ptr,
                                                        st->dl.data->ptr, st->du.data->ptr, st->g.data->ptr, s));
                float* hs = st->hstack.data->ptr;
                float* g = st->g.data->ptr;
                float* dmsg = st->dmsg.data->ptr;
                if (L > 0) {
                    auto& at = A->value.Transposed();
                    float* us = st->ustack.data->ptr;
                    float* g2 = st->g2.data->ptr;
                    GNN_HIP(gnnhip_s2v_grad_gate_f32(NC, hs + (size_t)L * NC, g, g, dmsg, 0, s));
                    for (int l = L; l >= 1; --l) {
                        // g_{l-1} comes out past the gate of h_{l-1} and is added to dmsg in the same pass
                        GNN_HIP(gnnhip_s2v_level_backward_f32((int)N, (int)C, at.nnz, at.row_ptr, at.col_idx, at.val, g,
                                                              Wc->value.data->ptr, us + (size_t)(l - 1) * NC, g2,
                                                              hs + (size_t)(l - 1) * NC, dmsg, s));
                        std::swap(g, g2);
                    }
                } else {
                    GNN_HIP(gnnhip_s2v_grad_gate_f32(NC, hs, g, nullptr, dmsg, 0, s));
                }
                // the weight gradients, x^T dy each and none of them large enough to fill the GPU: one batch
                int gm[4], gn[4], gk[4], glda[4], gldb[4], gldc[4], count = 0;
                const float* ga[4];
                const float* gb[4];
                float* gc[4];
                auto product = [&](const float* x, size_t rows, size_t m, const float* dy, size_t n, float* grad) {
                    ga[count] = x; gb[count] = dy; gc[count] = grad;
                    gm[count] = glda[count] = (int)m; gn[count] = gldb[count] = gldc[count] = (int)n; gk[count] = (int)rows;
                    ++count;
                };
                if (L > 0 && !cWc) product(hs, (size_t)L * N, C, st->ustack.data->ptr, C, Wc->grad.Full().data->ptr);
                if (!cWn) product(X->value.data->ptr, N, K, dmsg, C, Wn->grad.Full().data->ptr);
                if (!cW1) product(Pool->value.data->ptr, B, C, st->du.data->ptr, H, W1->grad.Full().data->ptr);
                if (!cW2) product(Hid->value.data->ptr, B, H, st->dl.data->ptr, Q, W2->grad.Full().data->ptr);
                GNN_HIP(gnnhip_gemm_tn_batch_f32(count, gm, gn, gk, ga, glda, gb, gldb, 1.0f, 1.0f, gc, gldc, s));
            };
        } else
        step->run = [=](Phase ph) {
            bool done = false;
            const size_t N = X->value.rows(), K = X->value.cols(), C = Wn->value.cols(), H = W1->value.cols(),
                         Q = W2->value.cols(), B = S->value.rows();
            ASSERT(Wn->value.rows() == K && Wc->value.rows() == C && Wc->value.cols() == C && W1->value.rows() == C &&
                   W2->value.rows() == H && A->value.rows() == N && A->value.cols() == N && S->value.cols() == N,
                   "fused forward: operand shapes do not chain");
            Msg->value.Reshape({N, C});
            Hl->value.Reshape({N, C});
            Pool->value.Reshape({B, C});
            Hid->value.Reshape({B, H});
            Logits->value.Reshape({B, Q});
            // small and medium block-diagonal batches in one launch (256 graphs of configuration 2: 23 us against 40)
            if (n2n->block_diagonal && sub->contiguous_subgraphs && sub->max_subgraph_nodes > 0 &&
                N <= detail::kOneLaunchMaxNodes) {
                const int rc = gnnhip_s2v_forward_batched_f32(
                    (int)N, (int)B, (int)K, (int)C, (int)H, (int)Q, L, sub->max_subgraph_nodes,
                    A->value.data->row_ptr, A->value.data->col_idx, A->value.data->val,
                    S->value.data->row_ptr, S->value.data->col_idx, S->value.data->val,
                    X->value.data->ptr, Wn->value.data->ptr, Wc->value.data->ptr, W1->value.data->ptr, W2->value.data->ptr,
                    Msg->value.data->ptr, Hl->value.data->ptr, Pool->value.data->ptr, Hid->value.data->ptr,
                    Logits->value.data->ptr, nullptr, nullptr, nullptr, GpuHandle::Stream());
                if (rc == GNNHIP_OK) done = true;
                else ASSERT(rc == GNNHIP_EUNSUPPORTED, gnnhip_last_error());
            }
            if (!done && H0) {
                // any CSR: input, levels and readout in one call; the library picks which of the two embedding
                // buffers ends up with the last level, and the variables swap their storage if it is h0's
                H0->value.Reshape({N, C});
                int which = 0;
                const int rc = gnnhip_s2v_forward_f32(
                    (int)N, (int)B, (int)K, (int)C, (int)H, (int)Q, L, (int)A->value.data->nnz,
                    A->value.data->row_ptr, A->value.data->col_idx, A->value.data->val,
                    S->value.data->row_ptr, S->value.data->col_idx, S->value.data->val,
                    X->value.data->ptr, Wn->value.data->ptr, Wc->value.data->ptr, W1->value.data->ptr, W2->value.data->ptr,
                    Msg->value.data->ptr, Hl->value.data->ptr, H0->value.data->ptr, Pool->value.data->ptr,
                    Hid->value.data->ptr, Logits->value.data->ptr, nullptr, nullptr, &which, GpuHandle::Stream());
                ASSERT(rc == GNNHIP_OK, gnnhip_last_error());
                if (which == 1) std::swap(Hl->value.data, H0->value.data);
                done = true;
            }
            if (!done) for (auto& p : parts) p->run(ph);
        };
        // the new step takes the place of the last part; the others leave the schedule
        const int last = chain.back();
        size_t folded = 0;
        for (int c : chain) { folded += steps[c]->fused ? 1 : 0; steps[c].reset(); }
        steps[last] = step;
        plan.n_fused = plan.n_fused - folded + 1;
    }
    steps.erase(std::remove(steps.begin(), steps.end(), std::shared_ptr<Step>()), steps.end());
}

// The tail that turns logits into the two numbers a training loop looks at,
//   CrossEntropy(logits, y, softmax inside) -> ReduceMean                       (the loss)
//   ArgMax(y) -> InTopK(logits, ., 1) -> TypeCast -> ReduceMean                 (the accuracy; optional)
// (examples/graph_classification/src/kernel_mean_field.cpp:51-56), becomes one call of gnnhip_s2v_loss_acc_f32.
// It leaves behind what the factors' Backward read (the CrossEntropy factor's probabilities, the loss rows), so
// a training plan may fold it as well.
inline void FactorGraph::FoldLossTail(Plan& plan)
{
    typedef DTensorVar<GPU, float> DVar;
    typedef SpTensorVar<GPU, float> SVar;
    typedef detail::FusedStep Step;
    auto& steps = plan.steps;
    std::vector<bool> is_target(var_list.size(), false);
    for (size_t v : plan.target_idx) is_target[v] = true;
    auto dense = [&](size_t v) { return dynamic_cast<DVar*>(var_list[v].get()); };
    auto kind_is = [&](size_t f, const char* k) { return !strcmp(factor_list[f]->FuseKind(), k); };
    // the step that is exactly factor f on its own, or -1
    auto single_step_of = [&](size_t f) -> int {
        for (size_t i = 0; i < steps.size(); ++i)
            if (steps[i] && steps[i]->tag == Step::SINGLE && steps[i]->factors.size() == 1 && steps[i]->factors[0] == f) return (int)i;
        return -1;
    };
    // the one executed reader of v, of the given kind, when v is private to it
    auto sole_reader = [&](size_t v, const char* k, size_t& reader) {
        if (is_target[v]) return false;
        size_t n = 0;
        for (size_t f : var_nodes[v].consumers) if (plan.executed[f]) { reader = f; ++n; }
        return n == 1 && kind_is(reader, k) && single_step_of(reader) >= 0;
    };
    for (size_t f_ce = 0; f_ce < factor_list.size(); ++f_ce) {
        if (!plan.executed[f_ce] || !kind_is(f_ce, "cross_entropy_softmax") || single_step_of(f_ce) < 0) continue;
        if (factor_nodes[f_ce].in.size() != 2) continue;
        const size_t vLogits = factor_nodes[f_ce].in[0], vY = factor_nodes[f_ce].in[1], vCe = factor_nodes[f_ce].out[0];
        DVar *Logits = dense(vLogits), *Ce = dense(vCe);
        SVar* Y = dynamic_cast<SVar*>(var_list[vY].get());
        auto* probs = static_cast<DTensor<GPU, float>*>(factor_list[f_ce]->FusePayload());
        size_t f_m1 = 0;
        if (!Logits || !Ce || !Y || !probs || !sole_reader(vCe, "reduce_mean", f_m1)) continue;
        DVar* Loss = dense(factor_nodes[f_m1].out[0]);
        if (!Loss) continue;
        std::vector<size_t> fs = {f_ce, f_m1};
        // the accuracy chain on the same logits and labels, if there is one
        DVar* Acc = nullptr;
        for (size_t f_am : var_nodes[vY].consumers) {
            if (!plan.executed[f_am] || !kind_is(f_am, "arg_max") || single_step_of(f_am) < 0) continue;
            size_t f_tk = 0, f_tc = 0, f_m2 = 0;
            const size_t vTruth = factor_nodes[f_am].out[0];
            if (!sole_reader(vTruth, "in_top_1", f_tk) || factor_nodes[f_tk].in.size() != 2 || factor_nodes[f_tk].in[0] != vLogits ||
                factor_nodes[f_tk].in[1] != vTruth) continue;
            if (!sole_reader(factor_nodes[f_tk].out[0], "type_cast", f_tc)) continue;
            if (!sole_reader(factor_nodes[f_tc].out[0], "reduce_mean", f_m2)) continue;
            Acc = dense(factor_nodes[f_m2].out[0]);
            if (!Acc) continue;
            fs.insert(fs.end(), {f_am, f_tk, f_tc, f_m2});
            break;
        }
        auto step = std::make_shared<Step>();
        step->fused = true;
        step->tag = Step::LOSS;
        step->factors = fs;
        step->run = [=](Phase) {
            ASSERT(Logits->value.rank() == 2 && Logits->value.rows() == Y->value.rows() && Logits->value.cols() == Y->value.cols(),
                   "loss tail: logits and labels disagree in shape");
            const size_t B = Logits->value.rows(), Q = Logits->value.cols();
            probs->Reshape({B, Q});
            Ce->value.Reshape({B, 1});
            Loss->value.Reshape({1});
            if (Acc) Acc->value.Reshape({1});
            GNN_HIP(gnnhip_s2v_loss_acc_f32((int)B, (int)Q, Logits->value.data->ptr, Y->value.data->row_ptr, Y->value.data->col_idx,
                                            Y->value.data->val, probs->data->ptr, Ce->value.data->ptr, nullptr,
                                            Loss->value.data->ptr, Acc ? Acc->value.data->ptr : nullptr, GpuHandle::Stream()));
            if (Acc) {
                // the caller reads the two numbers one after the other: the first read brings both
                auto both = std::make_shared< detail::ScalarGroup<float> >();
                Loss->value.JoinScalars(both);
                Acc->value.JoinScalars(both);
            }
        };
        int last = -1;
        for (size_t f : fs) { const int i = single_step_of(f); last = std::max(last, i); }
        for (size_t f : fs) steps[single_step_of(f)].reset();
        steps[last] = step;
        plan.n_fused++;
        // a folded training forward that ends in these logits starts its backward pass from this loss
        for (auto& st : steps)
            if (st && st->tag == Step::FORWARD && st->train && !st->vars.empty() && st->vars[0] == vLogits) {
                st->train->probs = probs;
                st->train->label = Y;
                st->train->loss_var = factor_nodes[f_m1].out[0];
                st->train->loss_attached = true;
            }
    }
    steps.erase(std::remove(steps.begin(), steps.end(), std::shared_ptr<Step>()), steps.end());
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
    // A folded step is fine when it left behind what Backward reads (the loss tail), or when it brings its own
    // backward pass (the folded forward of a training plan, if its last run took the folded route).
    detail::FusedStep* folded_forward = nullptr;
    for (auto& st : plan.steps) {
        if (!st->fused || st->tag == detail::FusedStep::LOSS) continue;
        ASSERT(plan.phase == Phase::TRAIN && st->tag == detail::FusedStep::FORWARD && st->train,
               "BackPropagate needs a FeedForward run with Phase::TRAIN (inference plans fuse factors)");
        if (st->train->fused_ran) folded_forward = st.get();
    }
    const size_t nv = var_list.size(), nf = factor_list.size();

    var_has_grad.assign(nv, false);
    // the reference clears the gradients one by one (src/nn/factor_graph.cpp:190-196); device gradients are
    // collected and cleared in one launch
    std::vector<void*> zero_ptr;
    std::vector<size_t> zero_bytes;
    for (size_t v = 0; v < nv; ++v)
        if (!isConst[v])
            if (auto* d = dynamic_cast<IDifferentiable*>(var_list[v].get())) {
                void* p = nullptr;
                size_t bytes = 0;
                if (!d->GradBuffer(&p, &bytes)) d->ZeroGrad();
                else if (bytes) { zero_ptr.push_back(p); zero_bytes.push_back(bytes); }
            }
    if (!zero_ptr.empty())
        GNN_HIP(gnnhip_memset0_batch((int)zero_ptr.size(), zero_ptr.data(), zero_bytes.data(), GpuHandle::Stream()));
    if (folded_forward) {
        // gradients of the weight matrices straight from the folded forward's own backward pass; the variables
        // between them were never materialised, so only the loss the fold was built around can be the start
        ASSERT(targets.size() == 1 && VarIdx(targets[0]) == folded_forward->train->loss_var,
               "after a folded training forward BackPropagate starts from the mean cross-entropy it was built around; "
               "call EnableFusion(false) for other targets");
        folded_forward->backward();
        return;
    }
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
