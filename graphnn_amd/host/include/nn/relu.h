// out = max(in, 0) written as graphnn does: `if (x < 0) x = 0` (include/nn/relu.h, src/nn/relu.cu:9-37).
#ifndef RELU_H
#define RELU_H

#include "nn/factor.h"

namespace gnn
{

inline void ReLUAct(DTensor<GPU, float>& in, DTensor<GPU, float>& out)
{
    out.Reshape(in.shape.dims);
    GNN_HIP(gnnhip_relu_f32(in.data->ptr, out.data->ptr, in.shape.Count(), GpuHandle::Stream()));
}
// dst += cur_grad where cur_out > 0
inline void ReLUDeriv(DTensor<GPU, float>& dst, DTensor<GPU, float>& cur_out, DTensor<GPU, float>& cur_grad)
{
    ASSERT(dst.shape == cur_out.shape && dst.shape == cur_grad.shape, "shape mismatch in ReLUDeriv");
    GNN_HIP(gnnhip_relu_deriv_f32(dst.shape.Count(), cur_out.data->ptr, cur_grad.data->ptr, dst.data->ptr, GpuHandle::Stream()));
}

template<typename mode, typename Dtype>
class ReLU : public Factor
{
public:
    static std::string StrType() { return "ReLU"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    ReLU(std::string _name, PropErr _properr = PropErr::T) : Factor(_name, _properr) {}
    virtual const char* FuseKind() const override { return "relu"; }

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 1 && outputs.size() == 1, "unexpected operand count for " << StrType());
        ReLUAct(detail::dense_var<mode, Dtype>(operands[0], "ReLU").value, detail::dense_var<mode, Dtype>(outputs[0], "ReLU").value);
    }
    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        ASSERT(operands.size() == 1 && outputs.size() == 1, "unexpected operand count for " << StrType());
        if (isConst[0]) return;
        auto& out = detail::dense_var<mode, Dtype>(outputs[0], "ReLU");
        auto g_out = out.grad.Full();
        auto g_in = detail::dense_var<mode, Dtype>(operands[0], "ReLU").grad.Full();
        ReLUDeriv(g_in, out.value, g_out);
    }
};

}  // namespace gnn
#endif
