// Row softmax and jagged (per-segment) softmax as graph operators, forward only
// (include/nn/softmax.h, include/nn/jagged_softmax.h; src/nn/softmax.cpp, src/nn/jagged_softmax.cpp:38-54).
#ifndef SOFTMAX_H
#define SOFTMAX_H

#include "nn/factor.h"

namespace gnn
{

template<typename mode, typename Dtype>
class Softmax : public Factor
{
public:
    static std::string StrType() { return "Softmax"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    Softmax(std::string _name, PropErr _properr = PropErr::T) : Factor(_name, _properr) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 1 && outputs.size() == 1, "unexpected operand count for " << StrType());
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "Softmax").value;
        out.CopyFrom(detail::dense_var<mode, Dtype>(operands[0], "Softmax").value);
        out.Softmax();
    }
};

}  // namespace gnn
#endif
