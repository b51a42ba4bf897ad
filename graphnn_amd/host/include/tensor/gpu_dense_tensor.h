// Device dense tensor: the method set of graphnn's DTensor<GPU, Dtype>
// (include/tensor/gpu_dense_tensor.h:21-438) that the structure2vec path touches,
// each method a thin call into libgnnhip's C ABI (no CUDA, no vendor BLAS).
// fp32 only, as the reference example (Dtype = float).
#ifndef GPU_DENSE_TENSOR_H
#define GPU_DENSE_TENSOR_H

#include "tensor/t_data.h"
#include "tensor/cpu_dense_tensor.h"
#include "tensor/gpu_handle.h"

namespace gnn
{

template<typename Dtype> class TensorTemplate<GPU, CSR_SPARSE, Dtype>;
template<typename Dtype> class TensorTemplate<GPU, ROW_SPARSE, Dtype>;

namespace detail
{
// One-element tensors that one launch writes and a caller reads one after the other (the loss and the accuracy):
// the first AsScalar of any of them fetches all, behind one wait for the device.
template<typename Dtype>
struct ScalarGroup
{
    std::vector<const Dtype*> device;
    std::vector<Dtype> host;
    bool fetched = false;
};

// storage shared by the float and int specialisations
template<typename Dtype>
class GpuDenseBase : public Tensor
{
public:
    GpuDenseBase() : data(std::make_shared< DenseData<GPU, Dtype> >()) {}
    virtual void Reshape(std::vector<size_t> l) override
    {
        scalars.reset();                   // whoever writes the tensor next reshapes it first
        shape.Reshape(l);
        if (!data) data = std::make_shared< DenseData<GPU, Dtype> >();
        data->Resize(shape.Count());
    }
    virtual MatType GetMatType() override { return MatType::dense; }
    virtual MatMode GetMatMode() override { return MatMode::gpu; }

    void CopyFrom(DTensor<CPU, Dtype>& src)
    {
        Reshape(src.shape.dims);
        // 32-bit elements: only the non-zero words travel when they are few (one-hot feature matrices)
        static_assert(sizeof(Dtype) == 4, "dense GPU tensors hold 32-bit elements");
        GNN_HIP(gnnhip_memcpy_h2d_sparse32(data->ptr, src.data->ptr, shape.Count(), GpuHandle::Stream()));
    }
    void CopyFrom(DTensor<GPU, Dtype>& src)
    {
        Reshape(src.shape.dims);
        GNN_HIP(gnnhip_memcpy_d2d(data->ptr, src.data->ptr, sizeof(Dtype) * shape.Count(), GpuHandle::Stream()));
    }
    void ShallowCopy(DTensor<GPU, Dtype>& src) { Touched(); shape = src.shape; data = src.data; }
    void Zeros() { Touched(); GNN_HIP(gnnhip_memset0(data->ptr, sizeof(Dtype) * shape.Count(), GpuHandle::Stream())); }
    // every method that writes the tensor in place calls this: a host copy of its value fetched earlier (AsScalar of a
    // grouped scalar) no longer stands for it, and the next AsScalar reads the device again, as graphnn's does every time
    void Touched() { scalars.reset(); }
    // blocking read of a one-element tensor: the forward's only synchronisation point
    Dtype AsScalar()
    {
        ASSERT(shape.Count() == 1, "can only convert trivial tensor to scalar");
        if (scalars && scalar_slot < scalars->device.size() && scalars->device[scalar_slot] == data->ptr) {
            auto& g = *scalars;
            if (!g.fetched) {
                const size_t n = g.device.size();
                g.host.resize(n);
                std::vector<void*> dst(n);
                std::vector<const void*> src(n);
                std::vector<size_t> bytes(n, sizeof(Dtype));
                for (size_t i = 0; i < n; ++i) { dst[i] = &g.host[i]; src[i] = g.device[i]; }
                GNN_HIP(gnnhip_memcpy_d2h_batch((int)n, dst.data(), src.data(), bytes.data(), GpuHandle::Stream()));
                g.fetched = true;
            }
            return g.host[scalar_slot];
        }
        Dtype v;
        GNN_HIP(gnnhip_memcpy_d2h(&v, data->ptr, sizeof(Dtype), GpuHandle::Stream()));
        return v;
    }
    // the tensor joins a group of scalars written together (the writer calls this after its launch)
    void JoinScalars(const std::shared_ptr< ScalarGroup<Dtype> >& group)
    {
        scalar_slot = group->device.size();
        group->device.push_back(data->ptr);
        scalars = group;
    }
    std::shared_ptr< DenseData<GPU, Dtype> > data;
    std::shared_ptr< ScalarGroup<Dtype> > scalars;
    size_t scalar_slot = 0;
};
}  // namespace detail

template<>
class TensorTemplate<GPU, DENSE, int> : public detail::GpuDenseBase<int>
{
public:
    TensorTemplate() {}
    virtual ~TensorTemplate() {}
    void Fill(int scalar)
    {
        if (scalar == 0) { Zeros(); return; }
        DTensor<CPU, int> host(shape.dims);
        host.Fill(scalar);
        CopyFrom(host);
    }
    using detail::GpuDenseBase<int>::CopyFrom;
};

template<>
class TensorTemplate<GPU, DENSE, float> : public detail::GpuDenseBase<float>
{
public:
    typedef float Dtype;
    TensorTemplate() {}
    virtual ~TensorTemplate() {}
    TensorTemplate(std::vector<size_t> l, Dtype* _data = nullptr) : TensorTemplate(TShape(l), _data) {}
    TensorTemplate(TShape s, Dtype* _data = nullptr)
    {
        shape = s;
        if (_data) data = std::make_shared< DenseData<GPU, Dtype> >(_data, 0, shape.Count());
        else data->Resize(shape.Count());
    }

    using detail::GpuDenseBase<float>::CopyFrom;
    // element-type conversion on the device (int -> float is the one the path uses)
    void CopyFrom(DTensor<GPU, int>& src)
    {
        Reshape(src.shape.dims);
        GNN_HIP(gnnhip_cast_i32_f32(src.data->ptr, data->ptr, shape.Count(), GpuHandle::Stream()));
    }

    DTensor<GPU, Dtype> GetRowRef(size_t row_start, size_t row_cnt)
    {
        ASSERT(row_start + row_cnt <= shape[0], "row range out of bounds");
        const size_t stride = rank() > 1 ? shape.Count(1) : 1;
        std::vector<size_t> d = shape.dims;
        d[0] = row_cnt;
        return DTensor<GPU, Dtype>(TShape(d), data->ptr + row_start * stride);
    }

    // weights are drawn on the host and uploaded: the device path has no RNG kernels
    void SetRandN(Dtype mean, Dtype std)
    {
        DTensor<CPU, Dtype> host(shape.dims);
        host.SetRandN(mean, std);
        CopyFrom(host);
    }
    void SetRandU(Dtype lb, Dtype ub)
    {
        DTensor<CPU, Dtype> host(shape.dims);
        host.SetRandU(lb, ub);
        CopyFrom(host);
    }
    void Fill(Dtype scalar)
    {
        if (scalar == 0) { Zeros(); return; }
        Unary(GNNHIP_UNARY_SET, scalar);
    }

    void ArgMax(DTensor<GPU, int>& dst, uint axis = 0)
    {
        ASSERT(axis == 0, "not supported for axis > 0 in GPU DENSE Tensor");
        dst.Reshape({shape[0]});
        GNN_HIP(gnnhip_row_argmax_f32(data->ptr, (int)shape[0], (int)shape.Count(1), dst.data->ptr, GpuHandle::Stream()));
    }

    void MM(DTensor<GPU, Dtype>& a, DTensor<GPU, Dtype>& b, Trans transA, Trans transB, Dtype alpha, Dtype beta)
    {
        ASSERT(a.rank() == 2 && b.rank() == 2, "only support mat x mat now");
        size_t m, n, k;
        GetDims(a.rows(), a.cols(), transA, b.rows(), b.cols(), transB, m, n, k);
        Reshape({m, n});
        GNN_HIP(gnnhip_gemm_f32(transA == Trans::T, transB == Trans::T, (int)m, (int)n, (int)k, alpha,
                                a.data->ptr, (int)a.cols(), b.data->ptr, (int)b.cols(), beta,
                                data->ptr, (int)n, GpuHandle::Stream()));
    }
    void MM(SpTensor<GPU, Dtype>& a, DTensor<GPU, Dtype>& b, Trans transA, Trans transB, Dtype alpha, Dtype beta);

    void Softmax()
    {
        ASSERT(rank() == 2, "Softmax is assumed to exec on matrix");
        Touched();
        GNN_HIP(gnnhip_row_softmax_f32(data->ptr, (int)rows(), (int)cols(), GpuHandle::Stream()));
    }
    void JaggedSoftmax(DTensor<GPU, int>& lens)
    {
        ASSERT(rows() == shape.Count(), "input must be a column vector");
        Touched();
        GNN_HIP(gnnhip_jagged_softmax_f32(data->ptr, lens.data->ptr, (int)lens.shape.Count(), GpuHandle::Stream()));
    }
    void Sum(DTensor<GPU, Dtype>& a, int axis = -1)
    {
        ASSERT(axis == -1, "currently only support global sum");
        Reshape({1});
        GNN_HIP(gnnhip_reduce_f32(GNNHIP_REDUCE_SUM, a.data->ptr, a.shape.Count(), data->ptr, GpuHandle::Stream()));
    }
    void Mean(DTensor<GPU, Dtype>& a, int axis = -1)
    {
        ASSERT(axis == -1, "currently only support global mean");
        Reshape({1});
        GNN_HIP(gnnhip_reduce_f32(GNNHIP_REDUCE_MEAN, a.data->ptr, a.shape.Count(), data->ptr, GpuHandle::Stream()));
    }

    void Add(Dtype scalar) { Unary(GNNHIP_UNARY_ADD, scalar); }
    void Scale(Dtype scalar)
    {
        if (scalar == 0) { Zeros(); return; }
        if (scalar != 1) Unary(GNNHIP_UNARY_SCALE, scalar);
    }
    void Axpy(Dtype a, DTensor<GPU, Dtype>& x)
    {
        ASSERT(shape == x.shape, "shape doesn't match in Axpy");
        Touched();
        GNN_HIP(gnnhip_axpy_f32(shape.Count(), a, x.data->ptr, data->ptr, GpuHandle::Stream()));
    }
    void Axpy(Dtype a, SpTensor<GPU, Dtype>& x);
    void Axpby(Dtype a, DTensor<GPU, Dtype>& x, Dtype b)
    {
        ASSERT(shape == x.shape, "shape doesn't match in Axpby");
        Touched();
        GNN_HIP(gnnhip_axpby_f32(shape.Count(), a, x.data->ptr, b, data->ptr, GpuHandle::Stream()));
    }
    void ElewiseMul(DTensor<GPU, Dtype>& src);

    void Abs() { Unary(GNNHIP_UNARY_ABS); }
    void Inv() { Unary(GNNHIP_UNARY_INV); }
    void Square() { Unary(GNNHIP_UNARY_SQUARE); }
    void Sqrt() { Unary(GNNHIP_UNARY_SQRT); }
    void InvSqrt() { Unary(GNNHIP_UNARY_INVSQRT); }
    void Sigmoid() { Unary(GNNHIP_UNARY_SIGMOID); }
    void Log() { Unary(GNNHIP_UNARY_LOG); }
    void Exp() { Unary(GNNHIP_UNARY_EXP); }
    void Truncate(Dtype lb, Dtype ub) { Unary(GNNHIP_UNARY_TRUNCATE, lb, ub); }

    void Print2Screen()
    {
        DTensor<CPU, Dtype> host;
        host.CopyFrom(*this);
        const size_t c = rank() > 1 ? shape.Count(1) : 1;
        for (size_t i = 0; i < shape.Count(); ++i) std::cerr << host.data->ptr[i] << ((i + 1) % c ? " " : "\n");
    }

    // graphnn's checkpoint layout for a tensor: shape, element count, raw elements
    virtual void Serialize(FILE* fid) override
    {
        DTensor<CPU, Dtype> host;
        host.CopyFrom(*this);
        host.Serialize(fid);
    }
    virtual void Deserialize(FILE* fid) override
    {
        DTensor<CPU, Dtype> host;
        host.Deserialize(fid);
        CopyFrom(host);
    }

private:
    void Unary(int op, Dtype a0 = 0, Dtype a1 = 0)
    {
        Touched();
        GNN_HIP(gnnhip_unary_f32(op, data->ptr, shape.Count(), a0, a1, GpuHandle::Stream()));
    }
};

// ---- host <- device copy declared in cpu_dense_tensor.h
template<typename Dtype>
void TensorTemplate<CPU, DENSE, Dtype>::CopyFrom(DTensor<GPU, Dtype>& src)
{
    Reshape(src.shape.dims);
    GNN_HIP(gnnhip_memcpy_d2h(data->ptr, src.data->ptr, sizeof(Dtype) * shape.Count(), GpuHandle::Stream()));
}

}  // namespace gnn
#endif
