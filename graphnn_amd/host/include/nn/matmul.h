// out = op(lhs) * op(rhs) with a sparse or dense lhs (interface of graphnn's include/nn/matmul.h,
// gradient rules of src/nn/matmul.cpp:35-76).
#ifndef MATMUL_H
#define MATMUL_H

#include "nn/factor.h"

namespace gnn
{

template<typename mode, typename Dtype>
class MatMul : public Factor
{
public:
    static std::string StrType() { return "MatMul"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }

    MatMul(std::string _name, Trans _transA = Trans::N, Trans _transB = Trans::N, PropErr _properr = PropErr::T)
        : Factor(_name, _properr), transA(_transA), transB(_transB) {}

    virtual const char* FuseKind() const override
    {
        return (transA == Trans::N && transB == Trans::N) ? "matmul_nn" : "";
    }

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 2, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "MatMul").value;
        auto* rhs = dynamic_cast<TensorVar<mode, Dtype>*>(operands[1].get());
        auto* lhs = dynamic_cast<TensorVar<mode, Dtype>*>(operands[0].get());
        ASSERT(lhs && rhs && rhs->GetMatType() == MatType::dense, "only support [sparse/dense] x [dense]");
        auto& right = rhs->template Derived<DENSE>().value;
        MAT_TYPE_SWITCH(lhs->GetMatType(), matType, {
            auto& left = lhs->template Derived<matType>().value;
            out.MM(left, right, transA, transB, 1.0, 0.0);
        });
    }

    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        ASSERT(operands.size() == 2 && outputs.size() == 1, "unexpected operand count for " << StrType());
        auto g_out = detail::dense_var<mode, Dtype>(outputs[0], "MatMul").grad.Full();
        auto& rhs = detail::dense_var<mode, Dtype>(operands[1], "MatMul");
        auto* lhs = dynamic_cast<TensorVar<mode, Dtype>*>(operands[0].get());
        if (!isConst[1]) {
            // d rhs += op(lhs)^T * g_out   (or g_out^T * op(lhs) when rhs enters transposed)
            auto g_rhs = rhs.grad.Full();
            if (transB == Trans::T) {
                ASSERT(lhs->GetMatType() == MatType::dense, "unsupported backprop in matmul");
                g_rhs.MM(g_out, lhs->template Derived<DENSE>().value, Trans::T, transA, 1.0, 1.0);
            } else {
                const Trans flipped = transA == Trans::N ? Trans::T : Trans::N;
                MAT_TYPE_SWITCH(lhs->GetMatType(), matType, {
                    g_rhs.MM(lhs->template Derived<matType>().value, g_out, flipped, Trans::N, 1.0, 1.0);
                });
            }
        }
        if (!isConst[0]) {
            ASSERT(lhs->GetMatType() == MatType::dense, "differentiable lhs can't be sparse");
            auto g_lhs = lhs->template Derived<DENSE>().grad.Full();
            if (transA == Trans::N)
                g_lhs.MM(g_out, rhs.value, Trans::N, transB == Trans::N ? Trans::T : Trans::N, 1.0, 1.0);
            else
                g_lhs.MM(rhs.value, g_out, transB, Trans::T, 1.0, 1.0);
        }
    }

    Trans transA;
    Trans transB;
};

}  // namespace gnn
#endif
