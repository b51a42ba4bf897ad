// out = in * W (+ b): the parameter has one row per input column and, optionally, one more row that is
// the bias (interface of graphnn's include/nn/fully_connected.h, behaviour of
// src/nn/fully_connected.cpp:13-93).  operands: input (dense or sparse), parameter.
#ifndef FULLY_CONNECTED_H
#define FULLY_CONNECTED_H

#include "nn/factor.h"

namespace gnn
{

template<typename mode, typename Dtype>
class FullyConnected : public Factor
{
public:
    static std::string StrType() { return "FullyConnected"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    FullyConnected(std::string _name, PropErr _properr = PropErr::T) : Factor(_name, _properr) {}

    // the inference plan folds MatMul(A, h) -> FullyConnected -> ElewiseAdd -> ReLU into the level kernel,
    // whose bias argument is this factor's last parameter row
    virtual const char* FuseKind() const override { return "fully_connected"; }

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 2, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "FullyConnected").value;
        auto& param = detail::dense_var<mode, Dtype>(operands[1], "FullyConnected").value;
        auto* lhs = dynamic_cast<TensorVar<mode, Dtype>*>(operands[0].get());
        ASSERT(lhs, "FullyConnected: the input must be a tensor variable");
        MAT_TYPE_SWITCH(lhs->GetMatType(), matType, {
            auto& in = lhs->template Derived<matType>().value;
            ASSERT(param.rows() == in.cols() || param.rows() == in.cols() + 1, "size mismatch");
            auto weight = param.GetRowRef(0, in.cols());
            out.MM(in, weight, Trans::N, Trans::N, 1.0, 0.0);
            if (param.rows() > in.cols()) {
                // + ones[N,1] * bias[1,C]
                auto bias = param.GetRowRef(in.cols(), 1);
                DTensor<mode, Dtype> ones({in.rows(), (size_t)1});
                ones.Fill(1.0);
                out.MM(ones, bias, Trans::N, Trans::N, 1.0, 1.0);
            }
        });
    }

    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        ASSERT(operands.size() == 2, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        auto g_out = detail::dense_var<mode, Dtype>(outputs[0], "FullyConnected").grad.Full();
        auto& rhs = detail::dense_var<mode, Dtype>(operands[1], "FullyConnected");
        auto* lhs = dynamic_cast<TensorVar<mode, Dtype>*>(operands[0].get());
        if (!isConst[1]) {
            auto g_param = rhs.grad.Full();
            MAT_TYPE_SWITCH(lhs->GetMatType(), matType, {
                auto& in = lhs->template Derived<matType>().value;
                auto g_weight = g_param.GetRowRef(0, in.cols());
                g_weight.MM(in, g_out, Trans::T, Trans::N, 1.0, 1.0);
                if (g_param.rows() > in.cols()) {
                    auto g_bias = g_param.GetRowRef(in.cols(), 1);
                    DTensor<mode, Dtype> ones({in.rows(), (size_t)1});
                    ones.Fill(1.0);
                    g_bias.MM(ones, g_out, Trans::T, Trans::N, 1.0, 1.0);
                }
            });
        }
        if (!isConst[0]) {
            ASSERT(lhs->GetMatType() == MatType::dense, "differentiable lhs can't be sparse");
            auto g_in = lhs->template Derived<DENSE>().grad.Full();
            auto weight = rhs.value.GetRowRef(0, g_in.cols());
            g_in.MM(g_out, weight, Trans::N, Trans::T, 1.0, 1.0);
        }
    }
};

}  // namespace gnn
#endif
