// Storage behind tensors (interface of graphnn's include/tensor/t_data.h):
// DenseData = one grow-only buffer (or a view into somebody else's),
// SparseData = the three CSR arrays with capacities.  Buffers come from
// MemHolder<mode> and are parked there again when the owner dies, so
// activations keep their device memory from batch to batch.
#ifndef T_DATA_H
#define T_DATA_H

#include "tensor/tensor.h"
#include "util/mem_holder.h"
#include <cstring>

namespace gnn
{

template<typename mode, typename mType, typename Dtype> class TDataTemplate;
template<typename mode, typename Dtype> using DenseData = TDataTemplate<mode, DENSE, Dtype>;
template<typename mode, typename Dtype> using SparseData = TDataTemplate<mode, CSR_SPARSE, Dtype>;

class TData
{
public:
    virtual ~TData() {}
};

namespace detail
{
template<typename mode> struct Zero;
template<> struct Zero<CPU> { static void run(void* p, size_t bytes) { if (bytes) memset(p, 0, bytes); } };
template<> struct Zero<GPU> { static void run(void* p, size_t bytes) { GNN_HIP(gnnhip_memset0(p, bytes, nullptr)); } };
}

template<typename mode, typename Dtype>
class TDataTemplate<mode, DENSE, Dtype> : public TData
{
public:
    TDataTemplate() : ptr(nullptr), mem_size(0), is_referring(false) {}
    // a view of `_msize` elements starting `offset` elements into src_ptr; never frees
    TDataTemplate(Dtype* src_ptr, size_t offset, size_t _msize)
        : ptr(src_ptr + offset), mem_size(_msize), is_referring(true) {}
    virtual ~TDataTemplate()
    {
        if (!is_referring && ptr) MemHolder<mode>::Recycle(ptr);
    }
    TDataTemplate(const TDataTemplate&) = delete;
    TDataTemplate& operator=(const TDataTemplate&) = delete;

    // grow-only; new memory arrives zeroed, old contents are not kept
    void Resize(size_t new_size)
    {
        if (new_size <= mem_size) return;
        ASSERT(!is_referring, "cannot grow a view");
        if (ptr) MemHolder<mode>::Recycle(ptr);
        MemHolder<mode>::MallocArr(ptr, sizeof(Dtype) * new_size);
        detail::Zero<mode>::run(ptr, sizeof(Dtype) * new_size);
        mem_size = new_size;
    }

    Dtype* ptr;
    size_t mem_size;       // capacity in elements
    bool is_referring;
};

template<typename mode, typename Dtype>
class TDataTemplate<mode, CSR_SPARSE, Dtype> : public TData
{
public:
    TDataTemplate() : val(nullptr), col_idx(nullptr), row_ptr(nullptr), nnz(0), len_ptr(0), nzCap(0), ptrCap(0) {}
    TDataTemplate(int newNzCap, int newPtrCap) : TDataTemplate()
    {
        Reserve(newNzCap, newPtrCap);
    }
    virtual ~TDataTemplate()
    {
        if (val) MemHolder<mode>::Recycle(val);
        if (col_idx) MemHolder<mode>::Recycle(col_idx);
        if (row_ptr) MemHolder<mode>::Recycle(row_ptr);
    }
    TDataTemplate(const TDataTemplate&) = delete;
    TDataTemplate& operator=(const TDataTemplate&) = delete;

    // capacity doubling, contents are not kept
    void Reserve(int wantNz, int wantPtr)
    {
        if (wantNz > nzCap) {
            int cap = nzCap * 2 > wantNz ? nzCap * 2 : wantNz;
            if (val) MemHolder<mode>::Recycle(val);
            if (col_idx) MemHolder<mode>::Recycle(col_idx);
            MemHolder<mode>::MallocArr(val, sizeof(Dtype) * (size_t)cap);
            MemHolder<mode>::MallocArr(col_idx, sizeof(int) * (size_t)cap);
            nzCap = cap;
        }
        if (wantPtr > ptrCap) {
            int cap = ptrCap * 2 > wantPtr ? ptrCap * 2 : wantPtr;
            if (row_ptr) MemHolder<mode>::Recycle(row_ptr);
            MemHolder<mode>::MallocArr(row_ptr, sizeof(int) * (size_t)cap);
            ptrCap = cap;
        }
    }

    Dtype* val;
    int* col_idx;
    int* row_ptr;
    int nnz;        // entries in use
    int len_ptr;    // row pointers in use (rows + 1)
    int nzCap;
    int ptrCap;
};

}  // namespace gnn
#endif
