// Per-row arg-max of a dense or sparse tensor (include/nn/arg_max.h, src/nn/arg_max.cpp).
#ifndef ARG_MAX_H
#define ARG_MAX_H

#include "nn/factor.h"

namespace gnn
{

template<typename mode, typename Dtype>
class ArgMax : public Factor
{
public:
    static std::string StrType() { return "ArgMax"; }
    using OutType = std::shared_ptr< DTensorVar<mode, int> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, int> >(fmt::sprintf("%s:out_0", this->name)); }
    ArgMax(std::string _name, uint _axis = 0) : Factor(_name, PropErr::N), axis(_axis) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 1 && outputs.size() == 1, "unexpected operand count for " << StrType());
        auto& out = detail::dense_var<mode, int>(outputs[0], "ArgMax").value;
        auto* in = dynamic_cast<TensorVar<mode, Dtype>*>(operands[0].get());
        ASSERT(in, "ArgMax needs a tensor operand");
        MAT_TYPE_SWITCH(in->GetMatType(), matType, {
            in->template Derived<matType>().value.ArgMax(out, axis);
        });
    }
    virtual const char* FuseKind() const override { return axis == 0 ? "arg_max" : ""; }
    uint axis;
};

}  // namespace gnn
#endif
