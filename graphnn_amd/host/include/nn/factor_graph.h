// Computation graph and its scheduler (interface of graphnn's include/nn/factor_graph.h,
// behaviour of src/nn/factor_graph.cpp): variables and factors are registered by name,
// FeedForward runs the factors a set of targets depends on in topological order,
// BackPropagate walks the executed factors in reverse.
//
// Differences in construction, not in behaviour: adjacency is kept by index, and the
// execution order for a given (targets, placeholders) request is computed once and cached,
// so a steady-state FeedForward does no string-keyed lookups per edge.  At inference
// (Phase::TEST) the cached plan also folds the structure2vec operator chains into the
// library's fused kernels (see nn/s2v_fusion.h).
#ifndef FACTOR_GRAPH_H
#define FACTOR_GRAPH_H

#include "util/gnn_macros.h"
#include "nn/variable.h"
#include "nn/factor.h"
#include <array>
#include <initializer_list>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

namespace gnn
{

namespace detail
{
// output bundle of a factor -> flat list of variables (one shared_ptr, or a tuple of them)
template<typename T>
inline void collect_outputs(std::vector< std::shared_ptr<Variable> >& dst, std::shared_ptr<T>& one) { dst.push_back(one); }

template<typename Tuple, size_t... I>
inline void collect_tuple(std::vector< std::shared_ptr<Variable> >& dst, Tuple& t, std::index_sequence<I...>)
{
    int expand[] = {0, (dst.push_back(std::get<I>(t)), 0)...};
    (void)expand;
}
template<typename... Ts>
inline void collect_outputs(std::vector< std::shared_ptr<Variable> >& dst, std::tuple<Ts...>& many)
{
    collect_tuple(dst, many, std::index_sequence_for<Ts...>());
}

struct FusedStep;     // defined in nn/s2v_fusion.h
}  // namespace detail

class FactorGraph
{
public:
    typedef std::shared_ptr<Variable> VarPtr;
    typedef std::vector< std::shared_ptr<Variable> > VarList;
    typedef std::vector< std::shared_ptr<Factor> > FactorList;

    FactorGraph() : version(0), fusion_enabled(true), last_plan(nullptr) {}

    // constants are never differentiated; a placeholder must be fed on every FeedForward
    void AddConst(VarPtr var, bool isPlaceholder)
    {
        size_t idx = AddVar(var);
        isConst[idx] = true;
        if (!isPlaceholder) always_ready.push_back(idx);
    }
    void AddParam(VarPtr var)
    {
        size_t idx = AddVar(var);
        always_ready.push_back(idx);
    }

    template<typename FactorPtr, typename VarPtrList, typename VarOutList>
    void AddFactor(FactorPtr factor, VarPtrList vars_in, VarOutList vars_out)
    {
        ASSERT(factor_dict.count(factor->name) == 0, fmt::sprintf("factor %s is already inserted", factor->name.c_str()));
        FactorNode node;
        for (size_t i = 0; i < vars_in.size(); ++i) {
            ASSERT(var_dict.count(vars_in[i]->name), "the operand " << vars_in[i]->name << " must be registered beforehand");
            node.in.push_back(var_dict[vars_in[i]->name].first);
        }
        const size_t fidx = factor_list.size();
        for (size_t i = 0; i < vars_out.size(); ++i) {
            size_t vidx = AddVar(vars_out[i]);
            if (factor->properr == PropErr::N) isConst[vidx] = true;     // nothing flows back through this factor
            node.out.push_back(vidx);
            var_nodes[vidx].producers.push_back(fidx);
        }
        for (size_t vidx : node.in) var_nodes[vidx].consumers.push_back(fidx);
        factor_dict[factor->name] = std::make_pair(fidx, std::shared_ptr<Factor>(factor));
        factor_list.push_back(factor);
        factor_nodes.push_back(node);
        ++version;
    }

    VarList FeedForward(std::vector<VarPtr> targets, std::map<std::string, void*> feed_dict, Phase phase, uint n_thread = 1);
    void BackPropagate(std::vector<VarPtr> targets, uint n_thread = 1);

    size_t VarIdx(VarPtr var) { return VarIdx(var->name); }
    size_t VarIdx(std::string var_name)
    {
        auto it = var_dict.find(var_name);
        ASSERT(it != var_dict.end(), "variable " << var_name << " is not registered");
        return it->second.first;
    }
    size_t FacIdx(std::shared_ptr<Factor> fac)
    {
        auto it = factor_dict.find(fac->name);
        ASSERT(it != factor_dict.end(), "factor " << fac->name << " is not registered");
        return it->second.first;
    }

    // switch the inference-time kernel fusion off (every factor then runs as written)
    void EnableFusion(bool on) { fusion_enabled = on; ++version; }
    // how the last FeedForward was executed: number of factor launches and of fused steps
    std::vector< std::vector<std::string> > PlanSteps(std::vector<VarPtr> targets, std::map<std::string, void*> feed_dict, Phase phase);
    size_t LastPlanFactorCount() const;
    size_t LastPlanFusedCount() const;

    std::map<std::string, std::pair<size_t, VarPtr> > var_dict;
    std::map<std::string, std::pair<size_t, std::shared_ptr<Factor> > > factor_dict;
    std::vector<VarPtr> var_list;
    std::vector< std::shared_ptr<Factor> > factor_list;

    struct FactorNode { std::vector<size_t> in, out; };
    struct VarNode { std::vector<size_t> producers, consumers; };
    std::vector<FactorNode> factor_nodes;
    std::vector<VarNode> var_nodes;
    std::vector<bool> isConst;

    // one cached execution order
    struct Plan
    {
        size_t version;
        Phase phase;
        std::vector<size_t> target_idx, feed_idx;
        std::vector<bool> required;                 // per variable
        std::vector<size_t> order;                  // factors, topologically sorted
        std::vector<bool> executed;                 // per factor
        std::vector< std::shared_ptr<detail::FusedStep> > steps;   // what actually runs (fused or single factors)
        size_t n_fused;
    };

protected:
    size_t AddVar(VarPtr var)
    {
        ASSERT(var_dict.count(var->name) == 0, fmt::sprintf("variable %s is already inserted", var->name.c_str()));
        const size_t idx = var_list.size();
        var_dict[var->name] = std::make_pair(idx, var);
        var_list.push_back(var);
        var_nodes.push_back(VarNode());
        isConst.push_back(false);
        ++version;
        return idx;
    }

    Plan* GetPlan(const std::vector<VarPtr>& targets, const std::map<std::string, void*>& feed_dict, Phase phase);
    void BuildPlan(Plan& plan);
    void BuildFusedSteps(Plan& plan);      // nn/s2v_fusion.h
    void BuildSteps(Plan& plan, bool fold);
    void FoldWholeForward(Plan& plan);     // nn/s2v_fusion.h
    void FoldLossTail(Plan& plan);         // nn/s2v_fusion.h
    std::shared_ptr<detail::FusedStep> MakeSingleStep(size_t f);

    std::vector<size_t> always_ready;       // params and non-placeholder constants
    std::vector< std::unique_ptr<Plan> > plans;
    size_t version;
    bool fusion_enabled;
    Plan* last_plan;
    std::vector<bool> var_has_grad;
};

template<typename VarType, typename... Args>
std::shared_ptr<VarType> add_const(FactorGraph& g, std::string var_name, bool isPlaceholder, Args&&... args)
{
    auto v = std::make_shared<VarType>(var_name, std::forward<Args>(args)...);
    g.AddConst(v, isPlaceholder);
    return v;
}

// register a factor of type FacType over `operands`; returns its freshly created output variable(s)
template<typename FacType, typename OprList, typename... Args>
typename FacType::OutType af(FactorGraph& g, OprList operands, Args&&... args)
{
    auto fname = fmt::sprintf("%s_%d", FacType::StrType(), (int)g.factor_list.size());
    auto f = std::make_shared<FacType>(fname, std::forward<Args>(args)...);
    auto out_vars = f->CreateOutVar();
    std::vector< std::shared_ptr<Variable> > out_list;
    detail::collect_outputs(out_list, out_vars);
    g.AddFactor(f, operands, out_list);
    return out_vars;
}

template<typename FacType, typename VarPtr, typename... Args>
typename FacType::OutType af(FactorGraph& g, std::initializer_list<VarPtr> op, Args&&... args)
{
    std::vector<VarPtr> op_list(op.begin(), op.end());
    return af<FacType>(g, op_list, std::forward<Args>(args)...);
}

template<typename FacType, typename VarPtr1, typename VarPtr2, typename... Args>
typename FacType::OutType af(FactorGraph& g, std::pair<VarPtr1, VarPtr2> op, Args&&... args)
{
    std::vector< std::shared_ptr<Variable> > op_list(2);
    op_list[0] = op.first;
    op_list[1] = op.second;
    return af<FacType>(g, op_list, std::forward<Args>(args)...);
}

}  // namespace gnn

#include "nn/s2v_fusion.h"
#endif
