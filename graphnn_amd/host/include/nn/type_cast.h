// Element-type conversion of a dense tensor, e.g. int hits -> float for the accuracy mean
// (include/nn/type_cast.h, src/nn/type_cast.cpp:13-29).
#ifndef TYPE_CAST_H
#define TYPE_CAST_H

#include "nn/factor.h"

namespace gnn
{

template<typename mode, typename Dtype>
class TypeCast : public Factor
{
public:
    static std::string StrType() { return "TypeCast"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    TypeCast(std::string _name, PropErr _properr = PropErr::T) : Factor(_name, _properr) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 1 && outputs.size() == 1, "unexpected operand count for " << StrType());
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "TypeCast").value;
        if (auto* src_i = dynamic_cast<DTensorVar<mode, int>*>(operands[0].get())) out.CopyFrom(src_i->value);
        else out.CopyFrom(detail::dense_var<mode, Dtype>(operands[0], "TypeCast").value);
    }
    virtual const char* FuseKind() const override { return "type_cast"; }
    // nothing flows back through a cast from integers
    virtual void Backward(std::vector< std::shared_ptr<Variable> >&, std::vector<bool>&,
                          std::vector< std::shared_ptr<Variable> >&) override {}
};

}  // namespace gnn
#endif
