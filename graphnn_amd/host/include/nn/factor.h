// Operator base class (interface of graphnn's include/nn/factor.h).
#ifndef FACTOR_H
#define FACTOR_H

#include "nn/variable.h"
#include "util/fmt.h"
#include <memory>
#include <string>

namespace gnn
{

typedef std::vector< std::shared_ptr<Variable> > VarPtrList;

// what a message-pass factor learnt about the layout of the last batch while building its operand
struct BatchLayout
{
    bool block_diagonal = false;           // node-to-node operand: no edge joins two subgraphs
    bool contiguous_subgraphs = false;     // subgraph operand: graph g owns one contiguous, ascending node range
    int max_subgraph_nodes = 0;
};

class Factor
{
public:
    Factor(std::string _name, PropErr _properr = PropErr::T) : name(_name), properr(_properr) {}
    virtual ~Factor() {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs,
                         Phase phase) NOT_IMPLEMENTED
    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands,
                          std::vector< bool >& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) NOT_IMPLEMENTED

    // tag used by the inference-time fusion pass of FactorGraph; "" = never fused
    virtual const char* FuseKind() const { return ""; }
    // a tensor the fused plans fill on the factor's behalf (CrossEntropy: its probabilities), or null
    virtual void* FusePayload() { return nullptr; }
    // layout facts of the last batch, for factors that build batch operands (null otherwise)
    virtual const BatchLayout* Layout() const { return nullptr; }

    std::string name;
    PropErr properr;
};

namespace detail
{
// operand / output accessors shared by the operator bodies
template<typename mode, typename Dtype>
inline DTensorVar<mode, Dtype>& dense_var(std::shared_ptr<Variable>& v, const char* what)
{
    auto* p = dynamic_cast<DTensorVar<mode, Dtype>*>(v.get());
    ASSERT(p, what << ": expected a dense " << (mode::type == MatMode::gpu ? "GPU" : "CPU") << " tensor variable, got " << v->name);
    return *p;
}
template<typename mode, typename Dtype>
inline SpTensorVar<mode, Dtype>& sparse_var(std::shared_ptr<Variable>& v, const char* what)
{
    auto* p = dynamic_cast<SpTensorVar<mode, Dtype>*>(v.get());
    ASSERT(p, what << ": expected a sparse tensor variable, got " << v->name);
    return *p;
}
}  // namespace detail

}  // namespace gnn
#endif
