// Pooled allocators behind the tensor storage (interface of graphnn's
// include/util/mem_holder.h).  MemHolder<GPU> forwards to the library's
// size-keyed device pool (gnnhip_malloc / gnnhip_recycle / gnnhip_free);
// MemHolder<CPU> keeps its own size-keyed free list of 64-byte aligned blocks.
#ifndef MEM_HOLDER_H
#define MEM_HOLDER_H

#include "util/gnn_macros.h"
#include "gnnhip.h"
#include <cstdint>
#include <cstdlib>
#include <map>
#include <mutex>

namespace gnn
{

#define GNN_HIP(call) ASSERT((call) == GNNHIP_OK, "gnnhip: " << gnnhip_last_error())

template<typename mode> class MemHolder;

template<>
class MemHolder<CPU>
{
public:
    template<typename T> static void MallocArr(T*& p, size_t nBytes)
    {
        State& s = state();
        std::lock_guard<std::mutex> lock(s.mu);
        auto it = s.parked.lower_bound(nBytes);
        if (it != s.parked.end()) {
            p = static_cast<T*>(it->second);
            s.size_of[p] = it->first;
            s.parked.erase(it);
            return;
        }
        void* q = nullptr;
        // 64 bytes of slack behind every block: graphnn's GetBatch sets ptr[node_label] = 1 on rows of
        // width max(tag) (examples/graph_classification: kernel_mean_field.cpp:81-82, nn_common.h:57),
        // so a node carrying the largest tag in the last row writes one float past the tensor.
        size_t want = (nBytes + 63) / 64 * 64 + 64;
        ASSERT(posix_memalign(&q, 64, want) == 0, "host allocation of " << want << " bytes failed");
        s.size_of[q] = want;
        p = static_cast<T*>(q);
    }
    template<typename T> static void Recycle(T*& p)
    {
        if (!p) return;
        State& s = state();
        std::lock_guard<std::mutex> lock(s.mu);
        auto it = s.size_of.find(p);
        ASSERT(it != s.size_of.end(), "pointer was not handed out by MemHolder<CPU>");
        s.parked.emplace(it->second, (void*)p);
        p = nullptr;
    }
    template<typename T> static void ForceDel(T*& p)
    {
        if (!p) return;
        State& s = state();
        std::lock_guard<std::mutex> lock(s.mu);
        s.size_of.erase(p);
        free(p);
        p = nullptr;
    }
private:
    struct State {
        std::mutex mu;
        std::multimap<size_t, void*> parked;
        std::map<void*, size_t> size_of;
    };
    // never destroyed: tensors with static storage duration hand blocks back during program exit
    static State& state() { static State* s = new State(); return *s; }
};

template<>
class MemHolder<GPU>
{
public:
    template<typename T> static void MallocArr(T*& p, size_t nBytes)
    {
        void* q = nullptr;
        GNN_HIP(gnnhip_malloc(&q, nBytes));
        p = static_cast<T*>(q);
    }
    // Tensors that outlive GpuHandle::Destroy() (globals, as in graphnn's examples) hand their
    // blocks back after the pool is gone; the library reports that state and it is not an error.
    template<typename T> static void Recycle(T*& p)
    {
        if (!p) return;
        const int rc = gnnhip_recycle(p);
        ASSERT(rc == GNNHIP_OK || rc == GNNHIP_ENOTINIT, "gnnhip: " << gnnhip_last_error());
        p = nullptr;
    }
    template<typename T> static void ForceDel(T*& p)
    {
        if (!p) return;
        const int rc = gnnhip_free(p);
        ASSERT(rc == GNNHIP_OK || rc == GNNHIP_ENOTINIT, "gnnhip: " << gnnhip_last_error());
        p = nullptr;
    }
};

}  // namespace gnn
#endif
