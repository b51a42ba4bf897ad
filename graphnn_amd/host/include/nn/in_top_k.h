// out[r] = 1 when fewer than k entries of row r beat the labelled one (include/nn/in_top_k.h, src/nn/in_top_k.cu:9-51).
#ifndef IN_TOP_H_H
#define IN_TOP_H_H

#include "nn/factor.h"

namespace gnn
{

inline void IsInTopK(DTensor<GPU, float>& pred, DTensor<GPU, int>& label, DTensor<GPU, int>& out, int k)
{
    ASSERT(pred.rank() == 2, "predicted prob(or logits) should be a matrix");
    ASSERT(pred.rows() == label.shape.Count(), "# instances doesn't match");
    out.Reshape(label.shape.dims);
    GNN_HIP(gnnhip_in_top_k_f32(pred.data->ptr, label.data->ptr, (int)pred.rows(), (int)pred.cols(), k, out.data->ptr,
                                GpuHandle::Stream()));
}

template<typename mode, typename Dtype>
class InTopK : public Factor
{
public:
    static std::string StrType() { return "InTopK"; }
    using OutType = std::shared_ptr< DTensorVar<mode, int> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, int> >(fmt::sprintf("%s:out_0", this->name)); }
    InTopK(std::string _name, int _topK = 1) : Factor(_name, PropErr::N), topK(_topK) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 2 && outputs.size() == 1, "unexpected operand count for " << StrType());
        IsInTopK(detail::dense_var<mode, Dtype>(operands[0], "InTopK").value, detail::dense_var<mode, int>(operands[1], "InTopK").value,
                 detail::dense_var<mode, int>(outputs[0], "InTopK").value, topK);
    }
    virtual const char* FuseKind() const override { return topK == 1 ? "in_top_1" : ""; }
    int topK;
};

}  // namespace gnn
#endif
