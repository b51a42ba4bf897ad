// Host dense tensor (subset of graphnn's include/tensor/cpu_dense_tensor.h that the
// structure2vec path and its drivers use: storage, views, fills, copies in both
// directions).  Arithmetic on the host is not part of this layer.
#ifndef CPU_DENSE_TENSOR_H
#define CPU_DENSE_TENSOR_H

#include "tensor/t_data.h"
#include <chrono>
#include <random>
#include <thread>
#include <vector>

namespace gnn
{

template<typename Dtype>
class TensorTemplate<CPU, DENSE, Dtype> : public Tensor
{
public:
    TensorTemplate() : data(std::make_shared< DenseData<CPU, Dtype> >()) {}
    TensorTemplate(std::vector<size_t> l, Dtype* _data = nullptr) : TensorTemplate(TShape(l), _data) {}
    TensorTemplate(TShape s, Dtype* _data = nullptr)
    {
        shape = s;
        if (_data) data = std::make_shared< DenseData<CPU, Dtype> >(_data, 0, shape.Count());
        else { data = std::make_shared< DenseData<CPU, Dtype> >(); data->Resize(shape.Count()); }
    }
    virtual ~TensorTemplate() {}

    virtual void Reshape(std::vector<size_t> l) override
    {
        shape.Reshape(l);
        if (!data) data = std::make_shared< DenseData<CPU, Dtype> >();
        data->Resize(shape.Count());
    }
    virtual MatType GetMatType() override { return MatType::dense; }
    virtual MatMode GetMatMode() override { return MatMode::cpu; }

    void CopyFrom(DTensor<CPU, Dtype>& src)
    {
        Reshape(src.shape.dims);
        if (shape.Count()) memcpy(data->ptr, src.data->ptr, sizeof(Dtype) * shape.Count());
    }
    void CopyFrom(DTensor<GPU, Dtype>& src);          // defined in gpu_dense_tensor.h
    void ShallowCopy(DTensor<CPU, Dtype>& src) { shape = src.shape; data = src.data; }
    DTensor<CPU, Dtype> GetRowRef(size_t row_start, size_t row_cnt)
    {
        ASSERT(row_start + row_cnt <= shape[0], "row range out of bounds");
        const size_t stride = rank() > 1 ? shape.Count(1) : 1;
        std::vector<size_t> d = shape.dims;
        d[0] = row_cnt;
        return DTensor<CPU, Dtype>(TShape(d), data->ptr + row_start * stride);
    }

    // (the one-hot feature matrix of a batch of ten thousand graphs is 77 MB, cleared for every batch: from 32 MB on the
    // clearing is shared by a few threads)
    void Zeros()
    {
        const size_t bytes = sizeof(Dtype) * shape.Count();
        if (!bytes) return;
        char* p = reinterpret_cast<char*>(data->ptr);
        const unsigned hw = std::thread::hardware_concurrency();
        const size_t parts = bytes < ((size_t)32 << 20) ? 1 : hw >= 8 ? 4 : hw >= 4 ? 2 : 1;
        if (parts == 1) { memset(p, 0, bytes); return; }
        const size_t per = (bytes / parts + 4095) & ~(size_t)4095;
        std::vector<std::thread> workers;
        for (size_t i = 1; i < parts; ++i) {
            const size_t lo = i * per, hi = lo + per < bytes ? lo + per : bytes;
            if (lo < hi) workers.emplace_back([p, lo, hi] { memset(p + lo, 0, hi - lo); });
        }
        memset(p, 0, per < bytes ? per : bytes);
        for (auto& t : workers) t.join();
    }
    void Fill(Dtype scalar)
    {
        const size_t n = shape.Count();
        for (size_t i = 0; i < n; ++i) data->ptr[i] = scalar;
    }
    Dtype AsScalar()
    {
        ASSERT(shape.Count() == 1, "can only convert trivial tensor to scalar");
        return data->ptr[0];
    }
    // graphnn seeds this from the clock (cpu_unary_functor.h:96-168); so does this one.
    void SetRandN(Dtype mean, Dtype std)
    {
        std::mt19937_64 gen((uint64_t)std::chrono::system_clock::now().time_since_epoch().count());
        std::normal_distribution<double> dist((double)mean, (double)std);
        const size_t n = shape.Count();
        for (size_t i = 0; i < n; ++i) data->ptr[i] = (Dtype)dist(gen);
    }
    void SetRandU(Dtype lb, Dtype ub)
    {
        std::mt19937_64 gen((uint64_t)std::chrono::system_clock::now().time_since_epoch().count());
        std::uniform_real_distribution<double> dist((double)lb, (double)ub);
        const size_t n = shape.Count();
        for (size_t i = 0; i < n; ++i) data->ptr[i] = (Dtype)dist(gen);
    }

    virtual void Serialize(FILE* fid) override
    {
        Tensor::Serialize(fid);
        size_t n = shape.Count();      // graphnn writes mem_size here; equal to the count for a tensor that never shrank
        ASSERT(fwrite(&n, sizeof(size_t), 1, fid) == 1, "write failed");
        if (n) ASSERT(fwrite(data->ptr, sizeof(Dtype), n, fid) == n, "write failed");
    }
    virtual void Deserialize(FILE* fid) override
    {
        Tensor::Deserialize(fid);
        size_t n = 0;
        ASSERT(fread(&n, sizeof(size_t), 1, fid) == 1, "read failed");
        // graphnn stores the buffer's capacity, which can exceed the element count of the shape
        ASSERT(n >= shape.Count(), "stored buffer is smaller than the stored shape");
        data->Resize(n);
        if (n) ASSERT(fread(data->ptr, sizeof(Dtype), n, fid) == n, "read failed");
    }

    std::shared_ptr< DenseData<CPU, Dtype> > data;
};

}  // namespace gnn
#endif
