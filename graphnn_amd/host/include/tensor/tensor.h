// Tensor base class and the DTensor / SpTensor / RowSpTensor aliases
// (interface of graphnn's include/tensor/tensor.h).
#ifndef TENSOR_H
#define TENSOR_H

#include "util/gnn_macros.h"
#include "tensor/t_shape.h"
#include <cstdio>
#include <memory>
#include <string>
#include <vector>

namespace gnn
{

// result dims of op(lhs) x op(rhs); aborts when the inner dims disagree
inline void GetDims(const size_t& lhs_rows, const size_t& lhs_cols, Trans ltrans,
                    const size_t& rhs_rows, const size_t& rhs_cols, Trans rtrans,
                    size_t& m, size_t& n, size_t& k)
{
    m = ltrans == Trans::N ? lhs_rows : lhs_cols;
    k = ltrans == Trans::N ? lhs_cols : lhs_rows;
    n = rtrans == Trans::N ? rhs_cols : rhs_rows;
    const size_t inner = rtrans == Trans::N ? rhs_rows : rhs_cols;
    ASSERT(inner == k, "mat dim doesn't match");
}

template<typename mode, typename matType, typename Dtype> class TensorTemplate;
template<typename mode, typename Dtype> using DTensor = TensorTemplate<mode, DENSE, Dtype>;
template<typename mode, typename Dtype> using SpTensor = TensorTemplate<mode, CSR_SPARSE, Dtype>;
template<typename mode, typename Dtype> using RowSpTensor = TensorTemplate<mode, ROW_SPARSE, Dtype>;

class Tensor
{
public:
    virtual ~Tensor() {}

    template<typename mode, typename matType, typename Dtype>
    TensorTemplate<mode, matType, Dtype>& Derived()
    {
        auto* p = dynamic_cast<TensorTemplate<mode, matType, Dtype>*>(this);
        ASSERT(p, "wrong derived type of Tensor");
        return *p;
    }

    inline uint rank() { return (uint)shape.dims.size(); }
    inline size_t rows()
    {
        ASSERT(rank() <= 2, "rows is not well defined for rank > 2");
        return shape[0];
    }
    inline size_t cols()
    {
        if (rank() == 1) return 1;          // a vector is a column
        ASSERT(rank() == 2, "cols is not well defined for rank > 2");
        return shape[1];
    }

    virtual void Reshape(std::vector<size_t> l) NOT_IMPLEMENTED
    virtual MatType GetMatType() = 0;
    virtual MatMode GetMatMode() = 0;

    // wire format of graphnn's Tensor::Serialize (src/tensor/tensor.cpp:15-29): rank, then dims, as size_t
    virtual void Serialize(FILE* fid)
    {
        size_t r = shape.dims.size();
        ASSERT(fwrite(&r, sizeof(size_t), 1, fid) == 1, "write failed");
        if (r) ASSERT(fwrite(shape.dims.data(), sizeof(size_t), r, fid) == r, "write failed");
    }
    virtual void Deserialize(FILE* fid)
    {
        size_t r = 0;
        ASSERT(fread(&r, sizeof(size_t), 1, fid) == 1, "read failed");
        std::vector<size_t> d(r);
        if (r) ASSERT(fread(d.data(), sizeof(size_t), r, fid) == r, "read failed");
        Reshape(d);
    }

    TShape shape;
};

template<typename mode, typename matType, typename Dtype>
class TensorTemplate : public Tensor {};

}  // namespace gnn
#endif
