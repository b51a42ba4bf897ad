// Softmax over consecutive segments of a column vector (interface of graphnn's
// include/nn/jagged_softmax.h, behaviour of src/nn/jagged_softmax.cpp:38-74).
// operands: the column vector and an int tensor with the segment lengths.
#ifndef JAGGED_SOFTMAX_H
#define JAGGED_SOFTMAX_H

#include "nn/factor.h"

namespace gnn
{

// dst += (cur_grad - <cur_grad, cur_output> per segment) * cur_output.  graphnn leaves its GPU overload
// empty (src/nn/jagged_softmax.cu:9-12); this one applies the CPU rule (src/nn/jagged_softmax.cpp:8-31).
inline void JaggedSoftmaxDeriv(DTensor<GPU, float>& dst, DTensor<GPU, float>& cur_output, DTensor<GPU, float>& cur_grad,
                               DTensor<GPU, int>& lens)
{
    ASSERT(dst.shape.Count() == cur_output.shape.Count() && dst.shape.Count() == cur_grad.shape.Count(),
           "length mismatch in jagged softmax");
    GNN_HIP(gnnhip_jagged_softmax_deriv_f32(dst.data->ptr, cur_output.data->ptr, cur_grad.data->ptr, lens.data->ptr,
                                            (int)lens.shape.Count(), GpuHandle::Stream()));
}

template<typename mode, typename Dtype>
class JaggedSoftmax : public Factor
{
public:
    static std::string StrType() { return "JaggedSoftmax"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    JaggedSoftmax(std::string _name, PropErr _properr = PropErr::T) : Factor(_name, _properr) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 2, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "JaggedSoftmax").value;
        out.CopyFrom(detail::dense_var<mode, Dtype>(operands[0], "JaggedSoftmax").value);
        out.JaggedSoftmax(detail::dense_var<mode, int>(operands[1], "JaggedSoftmax").value);
    }

    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        ASSERT(operands.size() == 2, "unexpected input size for " << StrType());
        ASSERT(outputs.size() == 1, "unexpected output size for " << StrType());
        if (isConst[0]) return;
        auto& lens = detail::dense_var<mode, int>(operands[1], "JaggedSoftmax").value;
        auto& out_var = detail::dense_var<mode, Dtype>(outputs[0], "JaggedSoftmax");
        auto cur_grad = out_var.grad.Full();
        auto prev_grad = detail::dense_var<mode, Dtype>(operands[0], "JaggedSoftmax").grad.Full();
        JaggedSoftmaxDeriv(prev_grad, out_var.value, cur_grad, lens);
    }
};

}  // namespace gnn
#endif
