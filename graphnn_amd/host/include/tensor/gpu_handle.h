// Device context (interface of graphnn's include/tensor/gpu_handle.h).  There are no
// vendor BLAS/SPARSE handles to pool: Init selects the device and brings up the library,
// Destroy releases the pool.  All work of this layer goes to one stream (the HIP null
// stream), which keeps the ordering the reference gets from its per-thread default stream.
#ifndef GPU_HANDLE_H
#define GPU_HANDLE_H

#include "util/mem_holder.h"

namespace gnn
{

struct GpuHandle
{
    static void Init(int dev_id, unsigned int _streamcnt = 1U)
    {
        (void)_streamcnt;
        GNN_HIP(gnnhip_init(dev_id));
    }
    static void Destroy() { GNN_HIP(gnnhip_shutdown()); }
    static void* Stream() { return nullptr; }
    static void Sync() { GNN_HIP(gnnhip_stream_sync(Stream())); }
};

}  // namespace gnn
#endif
