// Row-wise cross-entropy of (optionally soft-maxed) predictions against a sparse label matrix
// (include/nn/cross_entropy.h, src/nn/cross_entropy.cpp:7-78, src/nn/cross_entropy.cu:9-49).
#ifndef CROSS_ENTROPY_H
#define CROSS_ENTROPY_H

#include "nn/factor.h"

namespace gnn
{

// out[r] = -sum_k log(prob[r, col_k]) * val_k over the label's row r
inline void CalcCrossEntropy(DTensor<GPU, float>& prob, SpTensor<GPU, float>& label, DTensor<GPU, float>& out)
{
    ASSERT(prob.cols() == label.cols(), "# class doesn't match");
    ASSERT(prob.rows() == label.rows(), "# instances doesn't match");
    out.Reshape({prob.rows(), 1});
    GNN_HIP(gnnhip_cross_entropy_f32(prob.data->ptr, (int)prob.rows(), (int)prob.cols(), label.data->row_ptr,
                                     label.data->col_idx, label.data->val, out.data->ptr, GpuHandle::Stream()));
}

template<typename mode, typename Dtype>
class CrossEntropy : public Factor
{
public:
    static std::string StrType() { return "CrossEntropy"; }
    using OutType = std::shared_ptr< DTensorVar<mode, Dtype> >;
    OutType CreateOutVar() { return std::make_shared< DTensorVar<mode, Dtype> >(fmt::sprintf("%s:out_0", this->name)); }
    CrossEntropy(std::string _name, bool _need_softmax, PropErr _properr = PropErr::T)
        : Factor(_name, _properr), need_softmax(_need_softmax) {}

    virtual void Forward(std::vector< std::shared_ptr<Variable> >& operands,
                         std::vector< std::shared_ptr<Variable> >& outputs, Phase) override
    {
        ASSERT(operands.size() == 2 && outputs.size() == 1, "unexpected operand count for " << StrType());
        auto* lhs = dynamic_cast<TensorVar<mode, Dtype>*>(operands[0].get());
        ASSERT(lhs && lhs->GetMatType() == MatType::dense, "[dense prediction] cross_entropy [sparse/dense label]");
        probs.CopyFrom(lhs->template Derived<DENSE>().value);
        if (need_softmax) probs.Softmax();
        CalcCrossEntropy(probs, detail::sparse_var<mode, Dtype>(operands[1], "CrossEntropy").value,
                         detail::dense_var<mode, Dtype>(outputs[0], "CrossEntropy").value);
    }
    // d logits += (softmax - label) * g_out   (or -label / p * g_out without the softmax)
    virtual void Backward(std::vector< std::shared_ptr<Variable> >& operands, std::vector<bool>& isConst,
                          std::vector< std::shared_ptr<Variable> >& outputs) override
    {
        if (isConst[0]) return;
        auto g_out = detail::dense_var<mode, Dtype>(outputs[0], "CrossEntropy").grad.Full();
        auto g_lhs = detail::dense_var<mode, Dtype>(operands[0], "CrossEntropy").grad.Full();
        auto& label = detail::sparse_var<mode, Dtype>(operands[1], "CrossEntropy").value;
        if (need_softmax) {
            probs.Axpy(-1.0, label);
            probs.ElewiseMul(g_out);
        } else {
            DTensor<mode, Dtype> lab_over_p(probs.shape.dims);
            lab_over_p.Zeros();
            lab_over_p.Axpy(1.0, label);
            probs.Inv();
            probs.ElewiseMul(lab_over_p);
            probs.ElewiseMul(g_out);
            probs.Scale(-1.0);
        }
        g_lhs.Axpy(1.0, probs);
    }

    // the inference and training plans fold CrossEntropy(softmax inside) -> ReduceMean into one launch
    virtual const char* FuseKind() const override { return need_softmax ? "cross_entropy_softmax" : ""; }
    // the probabilities of the last forward (Backward reads them); the fused loss tail writes them here
    virtual void* FusePayload() override { return &probs; }

    bool need_softmax;
protected:
    DTensor<mode, Dtype> probs;
};

}  // namespace gnn
#endif
