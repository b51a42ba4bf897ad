// Global mean of a tensor into a one-element tensor (include/nn/reduce_mean.h, src/nn/reduce_mean.cpp:14-65).
#ifndef REDUCE_MEAN_H
#define REDUCE_MEAN_H

#include "nn/factor.h"

namespace gnn
{

template<typename mode, typename Dtype>
class ReduceMean : public Factor
{
public:
    static std::string StrType() { return "ReduceMean"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    ReduceMean(std::string _name, int _axis = -1, bool _keep_dim = false, PropErr _properr = PropErr::T)
        : Factor(_name, _properr), axis(_axis), keep_dim(_keep_dim) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 1 && outputs.size() == 1, "unexpected operand count for " << StrType());
        ASSERT(axis == -1 && keep_dim == false, "currently only support axis=-1 and keep_dim=false in " << StrType());
        detail::dense_var<mode, Dtype>(outputs[0], "ReduceMean").value.Mean(detail::dense_var<mode, Dtype>(operands[0], "ReduceMean").value, axis);
    }
    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        if (isConst[0]) return;
        auto g_out = detail::dense_var<mode, Dtype>(outputs[0], "ReduceMean").grad.Full();
        auto g_in = detail::dense_var<mode, Dtype>(operands[0], "ReduceMean").grad.Full();
        g_in.Add(g_out.AsScalar() / (Dtype)g_in.shape.Count());
    }
    virtual const char* FuseKind() const override { return (axis == -1 && !keep_dim) ? "reduce_mean" : ""; }
    int axis;
    bool keep_dim;
};

}  // namespace gnn
#endif
