// Device CSR tensor (interface of graphnn's include/tensor/gpu_sparse_tensor.h) and the
// sparse-operand methods of the dense tensor.
#ifndef GPU_CSR_SPARSE_TENSOR_H
#define GPU_CSR_SPARSE_TENSOR_H

#include "tensor/gpu_dense_tensor.h"
#include "tensor/cpu_sparse_tensor.h"

namespace gnn
{

// The library's plan for the products with one CSR matrix (gnnhip_csr_plan_create): made at the first product after
// the matrix was (re)built when the matrix is large and dense enough for the library to plan at all (the thresholds
// of its column-ordered route), kept for the later products with it (the levels of a forward multiply with the same
// operand), destroyed with the matrix's contents.
struct CsrPlanBox {
    void* handle = nullptr;
    bool tried = false;
    ~CsrPlanBox() { Drop(); }
    void Drop()
    {
        if (handle) (void)gnnhip_csr_plan_destroy(handle);
        handle = nullptr;
        tried = false;
    }
    // null when the matrix is not worth a plan
    void* Get(int rows, int cols, int nnz, const int* row_ptr, const int* col_idx, const float* val)
    {
        if (!tried) {
            tried = true;
            if (rows >= 32768 && (long long)nnz >= 12ll * rows)
                GNN_HIP(gnnhip_csr_plan_create(rows, cols, row_ptr, col_idx, val, GpuHandle::Stream(), &handle));
        }
        return handle;
    }
};

template<typename Dtype>
class TensorTemplate<GPU, CSR_SPARSE, Dtype> : public Tensor
{
public:
    TensorTemplate() : data(std::make_shared< SparseData<GPU, Dtype> >()) {}
    virtual ~TensorTemplate() {}

    virtual void Reshape(std::vector<size_t> l) override
    {
        ASSERT(l.size() == 2, "only support sparse matrix");
        shape.Reshape(l);
    }
    virtual MatType GetMatType() override { return MatType::sparse; }
    virtual MatMode GetMatMode() override { return MatMode::gpu; }

    void ResizeSp(int newNNZ, int newNPtr)
    {
        data->Reserve(newNNZ, newNPtr);
        data->nnz = newNNZ;
        data->len_ptr = newNPtr;
        t_valid = false;                   // every builder resizes first: the cached transpose is stale
        DropPlans();                       // ... and so are the plans of the products with the old contents
    }
    // plan of the products with this matrix / with its transpose (null: the plain entry points are as good)
    void* Plan()
    {
        if (!plan) plan = std::make_shared<CsrPlanBox>();
        return plan->Get((int)shape[0], (int)shape[1], data->nnz, data->row_ptr, data->col_idx, data->val);
    }
    void* TransposedPlan()
    {
        auto& t = Transposed();
        if (!t_plan) t_plan = std::make_shared<CsrPlanBox>();
        return t_plan->Get((int)shape[1], (int)shape[0], t.nnz, t.row_ptr, t.col_idx, t.val);
    }
    void DropPlans()
    {
        if (plan) plan->Drop();
        if (t_plan) t_plan->Drop();
    }
    // CSR of the transpose, built on the device at the first use after the matrix was (re)built and kept
    // for the following ones (the backward pass multiplies by A^T once per level).  The product with it
    // goes through the forward SpMM: no atomics, the same bits on every run.
    SparseData<GPU, Dtype>& Transposed()
    {
        if (!t_valid) {
            if (!t_data) t_data = std::make_shared< SparseData<GPU, Dtype> >();
            t_data->Reserve(data->nnz, (int)shape[1] + 1);
            t_data->nnz = data->nnz;
            t_data->len_ptr = (int)shape[1] + 1;
            GNN_HIP(gnnhip_csr_transpose_f32((int)shape[0], (int)shape[1], data->nnz, data->row_ptr, data->col_idx, data->val,
                                             t_data->row_ptr, t_data->col_idx, t_data->val, GpuHandle::Stream()));
            t_valid = true;
        }
        return *t_data;
    }
    // Storage for a transpose that the builder of the matrix fills on the device in the same launch; what it
    // writes there counts as the transpose from now on (any order of the entries inside a row will do: the
    // products with it sum a row in the order it is stored, the same on every run).
    SparseData<GPU, Dtype>& AdoptTransposed()
    {
        if (!t_data) t_data = std::make_shared< SparseData<GPU, Dtype> >();
        t_data->Reserve(data->nnz, (int)shape[1] + 1);
        t_data->nnz = data->nnz;
        t_data->len_ptr = (int)shape[1] + 1;
        t_valid = true;
        return *t_data;
    }
    // The transpose handed over by a builder that had the matrix on the host anyway (three small copies instead
    // of the dozen launches of the device transposition); t must be the stable transpose of what this tensor
    // holds: row c of t lists the rows of the matrix that have an entry in column c, in ascending row order.
    void SetTransposed(SpTensor<CPU, Dtype>& t)
    {
        ASSERT(t.rows() == shape[1] && t.cols() == shape[0] && t.data->nnz == data->nnz, "not the transpose of this matrix");
        if (!t_data) t_data = std::make_shared< SparseData<GPU, Dtype> >();
        t_data->Reserve(t.data->nnz, t.data->len_ptr);
        t_data->nnz = t.data->nnz;
        t_data->len_ptr = t.data->len_ptr;
        void* dst[3] = {t_data->val, t_data->col_idx, t_data->row_ptr};
        const void* from[3] = {t.data->val, t.data->col_idx, t.data->row_ptr};
        const size_t bytes[3] = {sizeof(Dtype) * (size_t)t.data->nnz, sizeof(int) * (size_t)t.data->nnz, sizeof(int) * (size_t)t.data->len_ptr};
        GNN_HIP(gnnhip_memcpy_h2d_batch(3, dst, from, bytes, GpuHandle::Stream()));
        t_valid = true;
    }
    // the three arrays in one batch of host-to-device copies, ordered on the layer's stream
    void CopyFrom(SpTensor<CPU, Dtype>& src)
    {
        shape = src.shape;
        ResizeSp(src.data->nnz, src.data->len_ptr);
        void* dst[3] = {data->val, data->col_idx, data->row_ptr};
        const void* from[3] = {src.data->val, src.data->col_idx, src.data->row_ptr};
        const size_t bytes[3] = {sizeof(Dtype) * (size_t)data->nnz, sizeof(int) * (size_t)data->nnz, sizeof(int) * (size_t)data->len_ptr};
        GNN_HIP(gnnhip_memcpy_h2d_batch(3, dst, from, bytes, GpuHandle::Stream()));
    }
    void CopyFrom(SpTensor<GPU, Dtype>& src)
    {
        shape = src.shape;
        ResizeSp(src.data->nnz, src.data->len_ptr);
        void* s = GpuHandle::Stream();
        GNN_HIP(gnnhip_memcpy_d2d(data->val, src.data->val, sizeof(Dtype) * (size_t)data->nnz, s));
        GNN_HIP(gnnhip_memcpy_d2d(data->col_idx, src.data->col_idx, sizeof(int) * (size_t)data->nnz, s));
        GNN_HIP(gnnhip_memcpy_d2d(data->row_ptr, src.data->row_ptr, sizeof(int) * (size_t)data->len_ptr, s));
    }
    void ShallowCopy(SpTensor<GPU, Dtype>& src) { shape = src.shape; data = src.data; t_valid = false; plan = src.plan; t_plan.reset(); }

    void ArgMax(DTensor<GPU, int>& dst, uint axis = 0)
    {
        ASSERT(axis == 0, "not supported for axis > 0 in GPU Sparse Tensor");
        dst.Reshape({shape[0]});
        GNN_HIP(gnnhip_csr_row_argmax_f32(data->row_ptr, data->col_idx, data->val, (int)shape[0], dst.data->ptr,
                                          GpuHandle::Stream()));
    }

    std::shared_ptr< SparseData<GPU, Dtype> > data;

private:
    std::shared_ptr< SparseData<GPU, Dtype> > t_data;   // transpose, see Transposed()
    bool t_valid = false;
    std::shared_ptr<CsrPlanBox> plan, t_plan;           // see Plan(); shared with shallow copies, which share the arrays
};

// dense <- alpha * op(sparse) * dense + beta * dense
inline void TensorTemplate<GPU, DENSE, float>::MM(SpTensor<GPU, float>& a, DTensor<GPU, float>& b,
                                                  Trans transA, Trans transB, float alpha, float beta)
{
    ASSERT(transB == Trans::N, "the dense operand of a sparse product cannot be transposed");
    size_t m, n, k;
    GetDims(a.rows(), a.cols(), transA, b.rows(), b.cols(), transB, m, n, k);
    Reshape({m, n});
    if (transA == Trans::N) {
        if (void* plan = a.Plan()) {
            GNN_HIP(gnnhip_spmm_csr_planned_f32(plan, (int)n, alpha, b.data->ptr, (int)b.cols(), beta, data->ptr, (int)n, GpuHandle::Stream()));
            return;
        }
        GNN_HIP(gnnhip_spmm_csr_f32((int)m, (int)k, (int)n, a.data->nnz, alpha, a.data->row_ptr, a.data->col_idx, a.data->val,
                                    b.data->ptr, (int)b.cols(), beta, data->ptr, (int)n, GpuHandle::Stream()));
    } else {
        auto& t = a.Transposed();
        if (void* plan = a.TransposedPlan()) {
            GNN_HIP(gnnhip_spmm_csr_planned_f32(plan, (int)n, alpha, b.data->ptr, (int)b.cols(), beta, data->ptr, (int)n, GpuHandle::Stream()));
            return;
        }
        GNN_HIP(gnnhip_spmm_csr_f32((int)m, (int)k, (int)n, t.nnz, alpha, t.row_ptr, t.col_idx, t.val,
                                    b.data->ptr, (int)b.cols(), beta, data->ptr, (int)n, GpuHandle::Stream()));
    }
}

// dense += a * sparse
inline void TensorTemplate<GPU, DENSE, float>::Axpy(float a, SpTensor<GPU, float>& x)
{
    ASSERT(shape == x.shape, "shape doesn't match in Axpy");
    Touched();
    GNN_HIP(gnnhip_csr_axpy_f32((int)x.rows(), (int)x.cols(), a, x.data->row_ptr, x.data->col_idx, x.data->val,
                                data->ptr, GpuHandle::Stream()));
}

// ---- host <- device CSR copy declared in cpu_sparse_tensor.h
template<typename Dtype>
void TensorTemplate<CPU, CSR_SPARSE, Dtype>::CopyFrom(SpTensor<GPU, Dtype>& src)
{
    shape = src.shape;
    ResizeSp(src.data->nnz, src.data->len_ptr);
    void* s = GpuHandle::Stream();
    GNN_HIP(gnnhip_memcpy_d2h(data->val, src.data->val, sizeof(Dtype) * (size_t)data->nnz, s));
    GNN_HIP(gnnhip_memcpy_d2h(data->col_idx, src.data->col_idx, sizeof(int) * (size_t)data->nnz, s));
    GNN_HIP(gnnhip_memcpy_d2h(data->row_ptr, src.data->row_ptr, sizeof(int) * (size_t)data->len_ptr, s));
}

}  // namespace gnn
#endif
