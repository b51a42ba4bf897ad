// Host CSR tensor (interface of graphnn's include/tensor/cpu_sparse_tensor.h):
// a shape plus SparseData that callers fill through data->row_ptr / col_idx / val.
#ifndef CPU_SPARSE_TENSOR_H
#define CPU_SPARSE_TENSOR_H

#include "tensor/t_data.h"

namespace gnn
{

template<typename Dtype>
class TensorTemplate<CPU, CSR_SPARSE, Dtype> : public Tensor
{
public:
    TensorTemplate() : data(std::make_shared< SparseData<CPU, Dtype> >()) {}
    virtual ~TensorTemplate() {}

    virtual void Reshape(std::vector<size_t> l) override
    {
        ASSERT(l.size() == 2, "only support sparse matrix");
        shape.Reshape(l);
    }
    virtual MatType GetMatType() override { return MatType::sparse; }
    virtual MatMode GetMatMode() override { return MatMode::cpu; }

    void ResizeSp(int newNNZ, int newNPtr)
    {
        data->Reserve(newNNZ, newNPtr);
        data->nnz = newNNZ;
        data->len_ptr = newNPtr;
    }
    void CopyFrom(SpTensor<CPU, Dtype>& src)
    {
        shape = src.shape;
        ResizeSp(src.data->nnz, src.data->len_ptr);
        if (data->nnz) {
            memcpy(data->val, src.data->val, sizeof(Dtype) * (size_t)data->nnz);
            memcpy(data->col_idx, src.data->col_idx, sizeof(int) * (size_t)data->nnz);
        }
        if (data->len_ptr) memcpy(data->row_ptr, src.data->row_ptr, sizeof(int) * (size_t)data->len_ptr);
    }
    void CopyFrom(SpTensor<GPU, Dtype>& src);         // defined in gpu_sparse_tensor.h
    void ShallowCopy(SpTensor<CPU, Dtype>& src) { shape = src.shape; data = src.data; }

    // per row, the column of the largest stored value (first one among equals); empty row -> 0
    void ArgMax(DTensor<CPU, int>& dst, uint axis = 0)
    {
        ASSERT(axis == 0, "not supported for axis > 0 in CPU Sparse Tensor");
        dst.Reshape({shape[0]});
        for (size_t i = 0; i < shape[0]; ++i) {
            int best = 0;
            Dtype cur = 0;
            for (int j = data->row_ptr[i]; j < data->row_ptr[i + 1]; ++j)
                if (j == data->row_ptr[i] || data->val[j] > cur) { cur = data->val[j]; best = data->col_idx[j]; }
            dst.data->ptr[i] = best;
        }
    }

    std::shared_ptr< SparseData<CPU, Dtype> > data;
};

}  // namespace gnn
#endif
