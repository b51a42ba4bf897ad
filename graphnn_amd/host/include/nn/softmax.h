// Row softmax as a graph operator (include/nn/softmax.h; src/nn/softmax.cpp).
#ifndef SOFTMAX_H
#define SOFTMAX_H

#include "nn/factor.h"

namespace gnn
{

// dst += (cur_grad - <cur_grad, cur_output> per row) * cur_output   (src/nn/softmax.cpp:8-29, src/nn/softmax.cu:10-59)
inline void SoftmaxDeriv(DTensor<GPU, float>& dst, DTensor<GPU, float>& cur_output, DTensor<GPU, float>& cur_grad)
{
    ASSERT(dst.shape == cur_output.shape && dst.shape == cur_grad.shape, "shape mismatch in softmax derivative");
    GNN_HIP(gnnhip_row_softmax_deriv_f32(dst.data->ptr, cur_output.data->ptr, cur_grad.data->ptr, (int)cur_output.rows(),
                                         (int)cur_output.cols(), GpuHandle::Stream()));
}

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

    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        ASSERT(operands.size() == 1 && outputs.size() == 1, "unexpected operand count for " << StrType());
        if (isConst[0]) return;
        auto& out_var = detail::dense_var<mode, Dtype>(outputs[0], "Softmax");
        auto cur_grad = out_var.grad.Full();
        auto prev_grad = detail::dense_var<mode, Dtype>(operands[0], "Softmax").grad.Full();
        SoftmaxDeriv(prev_grad, out_var.value, cur_grad);
    }
};

}  // namespace gnn
#endif
