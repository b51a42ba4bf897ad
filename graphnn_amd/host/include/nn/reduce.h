// Global sum or mean of a tensor into a one-element tensor (interface of graphnn's include/nn/reduce.h,
// behaviour of src/nn/reduce.cpp:16-85: only axis = -1 without keep_dim is supported there, too).
#ifndef REDUCE_H
#define REDUCE_H

#include "nn/factor.h"

namespace gnn
{

enum class ReduceType
{
    MEAN = 0,
    SUM = 1
};

template<typename mode, typename Dtype>
class Reduce : public Factor
{
public:
    static std::string StrType() { return "Reduce"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    Reduce(std::string _name, ReduceType _r_type, int _axis = -1, bool _keep_dim = false, PropErr _properr = PropErr::T)
        : Factor(_name, _properr), r_type(_r_type), axis(_axis), keep_dim(_keep_dim) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 1, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        ASSERT(axis == -1 && keep_dim == false, "currently only support axis=-1 and keep_dim=false in " << StrType());
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "Reduce").value;
        auto& in = detail::dense_var<mode, Dtype>(operands[0], "Reduce").value;
        if (r_type == ReduceType::MEAN) out.Mean(in, axis);
        else if (r_type == ReduceType::SUM) out.Sum(in, axis);
        else ASSERT(false, "unexpected reduction type");
    }

    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        ASSERT(operands.size() == 1, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        if (isConst[0]) return;
        ASSERT(axis == -1 && keep_dim == false, "currently only support axis=-1 and keep_dim=false in " << StrType());
        auto g_out = detail::dense_var<mode, Dtype>(outputs[0], "Reduce").grad.Full();
        auto g_in = detail::dense_var<mode, Dtype>(operands[0], "Reduce").grad.Full();
        const Dtype g = g_out.AsScalar();
        g_in.Add(r_type == ReduceType::MEAN ? g / (Dtype)g_in.shape.Count() : g);
    }

    ReduceType r_type;
    int axis;
    bool keep_dim;
};

}  // namespace gnn
#endif
