// out = sum_i coeff_i * operand_i (coefficients default to 1), shapes must agree
// (include/nn/elewise_add.h, src/nn/elewise_add.cpp:13-55).
#ifndef ELEWISE_ADD_H
#define ELEWISE_ADD_H

#include "nn/factor.h"

namespace gnn
{

template<typename mode, typename Dtype>
class ElewiseAdd : public Factor
{
public:
    static std::string StrType() { return "ElewiseAdd"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    ElewiseAdd(std::string _name, std::vector<Dtype> _coeff = std::vector<Dtype>(), PropErr _properr = PropErr::T)
        : Factor(_name, _properr), coeff(_coeff) {}
    virtual const char* FuseKind() const override { return coeff.empty() ? "elewise_add2" : ""; }

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() >= 2, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        ASSERT(coeff.empty() || coeff.size() == operands.size(), "wrong number of coefficients");
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "ElewiseAdd").value;
        out.CopyFrom(detail::dense_var<mode, Dtype>(operands[0], "ElewiseAdd").value);
        if (!coeff.empty()) out.Scale(coeff[0]);
        for (size_t i = 1; i < operands.size(); ++i) {
            auto& x = detail::dense_var<mode, Dtype>(operands[i], "ElewiseAdd").value;
            ASSERT(x.shape == out.shape, "no broadcasting is supported right now");
            out.Axpy(coeff.empty() ? (Dtype)1 : coeff[i], x);
        }
    }
    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        auto g_out = detail::dense_var<mode, Dtype>(outputs[0], "ElewiseAdd").grad.Full();
        for (size_t i = 0; i < operands.size(); ++i) {
            if (isConst[i]) continue;
            auto g_i = detail::dense_var<mode, Dtype>(operands[i], "ElewiseAdd").grad.Full();
            ASSERT(g_i.shape == g_out.shape, "no broadcasting is supported right now");
            g_i.Axpy(coeff.empty() ? (Dtype)1 : coeff[i], g_out);
        }
    }
    std::vector<Dtype> coeff;
};

}  // namespace gnn
#endif
