// Gradient tensor (interface of graphnn's include/tensor/gpu_row_sparse_tensor.h).
// graphnn's device version only works in "full" mode — every row-sparse branch of
// src/tensor/gpu_row_sparse_tensor.cu throws — so this one is a dense buffer with the
// same method names; the mean-field path never asks for anything else.
#ifndef GPU_ROW_SPARSE_TENSOR_H
#define GPU_ROW_SPARSE_TENSOR_H

#include "tensor/gpu_sparse_tensor.h"
#include <cmath>

namespace gnn
{

template<>
class TensorTemplate<GPU, ROW_SPARSE, float> : public Tensor
{
public:
    typedef float Dtype;
    TensorTemplate() : data(std::make_shared< DenseData<GPU, Dtype> >()), is_full(true) {}
    virtual ~TensorTemplate() {}

    virtual void Reshape(std::vector<size_t> l) override
    {
        shape.Reshape(l);
        data->Resize(shape.Count());
        is_full = true;
    }
    virtual MatType GetMatType() override { return MatType::row_sparse; }
    virtual MatMode GetMatMode() override { return MatMode::gpu; }
    void ReshapeLike(RowSpTensor<GPU, Dtype>& src) { Reshape(src.shape.dims); }

    // dense view sharing this tensor's memory
    DTensor<GPU, Dtype> Full() { return DTensor<GPU, Dtype>(shape, data->ptr); }
    void FullZeros() { is_full = true; Full().Zeros(); }
    void RowSpZeros() { Full().Zeros(); }
    void RowSparseFill(Dtype scalar) { Full().Fill(scalar); }
    void Scale(Dtype scalar) { Full().Scale(scalar); }
    void Sqrt() { Full().Sqrt(); }
    void Square() { Full().Square(); }
    void RowSparseAdd(Dtype scalar) { Full().Add(scalar); }
    void RowSparseInv() { Full().Inv(); }
    void RowSparseCopy(DTensor<GPU, Dtype>& src) { Full().CopyFrom(src); }
    void RowSparseAxpy(Dtype a, DTensor<GPU, Dtype>& x) { Full().Axpy(a, x); }
    void RowSparseAxpby(Dtype a, DTensor<GPU, Dtype>& x, Dtype b) { Full().Axpby(a, x, b); }
    void ElewiseMul(DTensor<GPU, Dtype>& src) { Full().ElewiseMul(src); }
    void SparseMM(SpTensor<GPU, Dtype>& a, DTensor<GPU, Dtype>& b, Trans transA, Trans transB, Dtype alpha, Dtype beta)
    {
        Full().MM(a, b, transA, transB, alpha, beta);
    }
    Dtype Norm2()
    {
        DTensor<GPU, Dtype> s({1});
        GNN_HIP(gnnhip_reduce_f32(GNNHIP_REDUCE_SUMSQ, data->ptr, shape.Count(), s.data->ptr, GpuHandle::Stream()));
        return std::sqrt(s.AsScalar());
    }

    std::shared_ptr< DenseData<GPU, Dtype> > data;
    DTensor<GPU, int> row_idxes;     // unused in full mode; kept because optimizers look at it
    bool is_full;
};

template<>
class TensorTemplate<GPU, ROW_SPARSE, int> : public Tensor
{
public:
    TensorTemplate() {}
    virtual ~TensorTemplate() {}
    virtual void Reshape(std::vector<size_t> l) override { shape.Reshape(l); }
    virtual MatType GetMatType() override { return MatType::row_sparse; }
    virtual MatMode GetMatMode() override { return MatMode::gpu; }
    DTensor<GPU, int> Full() { throw std::logic_error(std::string("not implemented")); }
    void RowSpZeros() {}
    void FullZeros() {}
};

// ---- dense methods that take the types above
inline void TensorTemplate<GPU, DENSE, float>::ElewiseMul(DTensor<GPU, float>& src)
{
    Touched();
    if (src.shape == shape) {
        GNN_HIP(gnnhip_mul_f32(shape.Count(), src.data->ptr, data->ptr, GpuHandle::Stream()));
        return;
    }
    // one factor per row, broadcast over the columns: [rows, 1] or [rows] against [rows, cols]
    ASSERT(rank() == 2 && src.shape.Count() == rows() && src.shape[0] == rows(),
           "unsupported broadcast in ElewiseMul: " << shape.toString() << " by " << src.shape.toString());
    GNN_HIP(gnnhip_row_scale_f32((int)rows(), (int)cols(), src.data->ptr, data->ptr, GpuHandle::Stream()));
}

}  // namespace gnn
#endif
