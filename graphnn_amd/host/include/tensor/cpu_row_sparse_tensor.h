// Host gradient tensor: dense storage with graphnn's RowSpTensor<CPU> method names
// (include/tensor/cpu_row_sparse_tensor.h).  Only what a CPU-resident variable needs to
// exist; host-side training is not part of this layer.
#ifndef CPU_ROW_SPARSE_TENSOR_H
#define CPU_ROW_SPARSE_TENSOR_H

#include "tensor/cpu_dense_tensor.h"

namespace gnn
{

template<typename Dtype>
class TensorTemplate<CPU, ROW_SPARSE, Dtype> : public Tensor
{
public:
    TensorTemplate() : data(std::make_shared< DenseData<CPU, Dtype> >()), is_full(true) {}
    virtual ~TensorTemplate() {}
    virtual void Reshape(std::vector<size_t> l) override
    {
        shape.Reshape(l);
        data->Resize(shape.Count());
        is_full = true;
    }
    virtual MatType GetMatType() override { return MatType::row_sparse; }
    virtual MatMode GetMatMode() override { return MatMode::cpu; }
    DTensor<CPU, Dtype> Full() { return DTensor<CPU, Dtype>(shape, data->ptr); }
    void FullZeros() { is_full = true; Full().Zeros(); }
    void RowSpZeros() { Full().Zeros(); }

    std::shared_ptr< DenseData<CPU, Dtype> > data;
    bool is_full;
};

}  // namespace gnn
#endif
