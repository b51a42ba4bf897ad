// Runtime of the gfx950 backend: device selection, error text, the size-keyed
// device-memory pool and the copy entry points.
//
// The pool follows the policy of graphnn's MemHolder<GPU>
// (src/util/mem_holder.cpp:15-97): recycle parks a block under its byte size,
// malloc hands out the smallest parked block that is large enough, and only
// free() gives memory back to the driver.  Per-level activations therefore stay
// resident in HBM from batch to batch.
#include <immintrin.h>
#include "gnnhip_internal.h"

#include <cstdarg>
#include <cstdio>
#include <atomic>
#include <map>
#include <string.h>
#include <functional>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

namespace gnnhip {

namespace {

thread_local char g_err[512] = "";

// Pinned staging for host-to-device copies: two halves used in turn.  A copy is placed in the current
// half and sent from there asynchronously, so the caller's buffer is free as soon as the call returns
// and nothing waits for the device.  A half is reused only after the event recorded behind its last
// copy has completed.
constexpr size_t kStagingHalf = 2u << 20;
constexpr int kExpandBlock = 256;
constexpr int kExpandTile = 1024;        // sparse uploads: 32-bit words of the destination per workgroup
constexpr size_t kReadbackBytes = 4096;
struct Staging {
    char* base = nullptr;              // 2 * kStagingHalf bytes from hipHostMalloc
    hipEvent_t done[2] = {nullptr, nullptr};
    bool pending[2] = {false, false};
    int half = 0;
    size_t used = 0;
};

// One pinned buffer per stream for the sparse form of a large upload (the positions and values of its non-zero words:
// about half a byte per word of the tensor), sized to the largest one seen; reused once the kernel that read it has run.
struct BigStaging {
    char* base = nullptr;
    size_t bytes = 0;
    hipEvent_t done = nullptr;
    bool pending = false;
};

struct Runtime {
    std::mutex mu;
    bool ready = false;
    int device = -1;
    std::multimap<size_t, void*> parked;           // size -> free block
    std::unordered_map<void*, size_t> live;        // block handed out -> size
    std::unordered_map<void*, size_t> all;         // every driver allocation -> size
    size_t bytes_in_use = 0;
    size_t bytes_parked = 0;
    size_t n_driver_allocs = 0;
    std::map<std::pair<hipStream_t, int>, std::pair<void*, size_t>> scratch;   // library scratch per (stream, slot)
    std::map<hipStream_t, struct Staging> staging;  // pinned upload buffers per stream
    std::map<hipStream_t, void*> readback;          // pinned landing buffer for small device-to-host reads, per stream
    std::map<hipStream_t, struct BigStaging> big_staging;
};

Runtime& rt()
{
    static Runtime r;
    return r;
}

constexpr size_t kAllocGranule = 256;   // keeps every block 256-byte aligned in size as well as address

}  // namespace

int set_error(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

bool runtime_ready() { return rt().ready; }

int require_ready()
{
    if (!rt().ready) return set_error(GNNHIP_ENOTINIT, "gnnhip_init has not been called");
    return GNNHIP_OK;
}

int pool_acquire(void** p, size_t bytes)
{
    if (!p) return set_error(GNNHIP_EINVAL, "null output pointer");
    *p = nullptr;
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (!r.ready) return set_error(GNNHIP_ENOTINIT, "gnnhip_init has not been called");
    if (bytes == 0) bytes = 1;
    size_t want = (bytes + kAllocGranule - 1) / kAllocGranule * kAllocGranule;
    auto it = r.parked.lower_bound(want);
    if (it != r.parked.end()) {
        void* q = it->second;
        size_t sz = it->first;
        r.parked.erase(it);
        r.bytes_parked -= sz;
        r.live[q] = sz;
        r.bytes_in_use += sz;
        *p = q;
        return GNNHIP_OK;
    }
    void* q = nullptr;
    hipError_t e = hipMalloc(&q, want);
    if (e != hipSuccess || q == nullptr) {
        (void)hipGetLastError();
        return set_error(GNNHIP_ENOMEM, "hipMalloc of %zu bytes failed: %s", want, hipGetErrorString(e));
    }
    r.all[q] = want;
    r.live[q] = want;
    r.bytes_in_use += want;
    r.n_driver_allocs += 1;
    *p = q;
    return GNNHIP_OK;
}

// A block of exactly `bytes` (rounded to the granule) straight from the driver, known to the pool (pool_free or
// shutdown returns it): for long-lived blocks of hundreds of megabytes, which must not take a larger parked block.
int pool_acquire_exact(void** p, size_t bytes)
{
    if (!p) return set_error(GNNHIP_EINVAL, "null output pointer");
    *p = nullptr;
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (!r.ready) return set_error(GNNHIP_ENOTINIT, "gnnhip_init has not been called");
    if (bytes == 0) bytes = 1;
    const size_t want = (bytes + kAllocGranule - 1) / kAllocGranule * kAllocGranule;
    void* q = nullptr;
    hipError_t e = hipMalloc(&q, want);
    if (e != hipSuccess || q == nullptr) {
        (void)hipGetLastError();
        return set_error(GNNHIP_ENOMEM, "hipMalloc of %zu bytes failed: %s", want, hipGetErrorString(e));
    }
    r.all[q] = want;
    r.live[q] = want;
    r.bytes_in_use += want;
    r.n_driver_allocs += 1;
    *p = q;
    return GNNHIP_OK;
}

int pool_free(void* p) { return gnnhip_free(p); }

int pool_release(void* p)
{
    if (!p) return GNNHIP_OK;
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    // after gnnhip_shutdown every block is already gone; late owners (static destructors) are told so
    if (!r.ready) return set_error(GNNHIP_ENOTINIT, "gnnhip is shut down; the block was released with the pool");
    auto it = r.live.find(p);
    if (it == r.live.end()) return set_error(GNNHIP_EINVAL, "pointer %p was not handed out by gnnhip_malloc", p);
    size_t sz = it->second;
    r.live.erase(it);
    r.bytes_in_use -= sz;
    r.parked.emplace(sz, p);
    r.bytes_parked += sz;
    return GNNHIP_OK;
}

int stream_scratch(hipStream_t s, size_t bytes, void** p) { return stream_scratch_slot(s, 0, bytes, p); }

// Test hook (exported, not part of the public header): the next request for this scratch slot fails as if the device
// were out of memory, so that the tests can walk the fallback paths that a full device would take.  -1: off.
static std::atomic<int> g_fail_scratch_slot{-1};
extern "C" void gnnhip_test_fail_next_scratch(int slot) { g_fail_scratch_slot.store(slot); }

int stream_scratch_slot(hipStream_t s, int which, size_t bytes, void** p)
{
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (!r.ready) return set_error(GNNHIP_ENOTINIT, "gnnhip_init has not been called");
    if (which < 0 || which >= kScratchSlots) return set_error(GNNHIP_EINVAL, "bad scratch slot %d", which);
    int expected = which;
    if (g_fail_scratch_slot.compare_exchange_strong(expected, -1))
        return set_error(GNNHIP_ENOMEM, "scratch slot %d: allocation failure injected by gnnhip_test_fail_next_scratch", which);
    auto& slot = r.scratch[std::make_pair(s, which)];
    if (slot.second < bytes) {
        size_t want = (bytes + 65535) / 65536 * 65536;
        const bool exact = which >= kExactScratchSlot;
        if (!exact && want < slot.second * 2) want = slot.second * 2;
        if (exact && slot.first) {
            // these slots run to gigabytes: the old block goes before the new one comes, so that the peak is the need
            // (kernels queued earlier on this stream may still read it)
            (void)hipStreamSynchronize(s);
            (void)hipFree(slot.first);
            slot.first = nullptr;
            slot.second = 0;
        }
        void* q = nullptr;
        hipError_t e = hipMalloc(&q, want);
        if (e != hipSuccess || !q) {
            (void)hipGetLastError();
            return set_error(GNNHIP_ENOMEM, "hipMalloc of %zu scratch bytes failed: %s", want, hipGetErrorString(e));
        }
        if (slot.first) {
            // kernels queued earlier on this stream may still read the old buffer
            (void)hipStreamSynchronize(s);
            (void)hipFree(slot.first);
        }
        slot.first = q;
        slot.second = want;
    }
    *p = slot.first;
    return GNNHIP_OK;
}

}  // namespace gnnhip

using namespace gnnhip;

extern "C" {

const char* gnnhip_last_error(void) { return g_err; }

const char* gnnhip_version(void) { return "gnnhip 0.1 (gfx950)"; }

int gnnhip_init(int device_id)
{
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return set_error(GNNHIP_EHIP, "no HIP device visible (%s)", hipGetErrorString(e));
    }
    if (device_id < 0 || device_id >= count)
        return set_error(GNNHIP_EINVAL, "device_id %d out of range [0,%d)", device_id, count);
    if (r.ready && r.device != device_id)
        return set_error(GNNHIP_EINVAL, "already initialised on device %d", r.device);
    GNNHIP_HIP(hipSetDevice(device_id));
    r.device = device_id;
    r.ready = true;
    // resolve this device's copy of the static offsets array now, so the entry point that may not
    // allocate finds it ready (it resolves it itself if the caller moved to another device)
    int* unused = nullptr;
    if (int rc = static_offsets_ptr(&unused)) return rc;
    return GNNHIP_OK;
}

int gnnhip_shutdown(void)
{
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (!r.ready) return GNNHIP_OK;
    (void)hipDeviceSynchronize();
    for (auto& kv : r.all) (void)hipFree(kv.first);
    for (auto& kv : r.scratch) (void)hipFree(kv.second.first);
    r.scratch.clear();
    for (auto& kv : r.staging) {
        if (kv.second.base) (void)hipHostFree(kv.second.base);
        for (hipEvent_t e : kv.second.done) if (e) (void)hipEventDestroy(e);
    }
    r.staging.clear();
    for (auto& kv : r.readback) if (kv.second) (void)hipHostFree(kv.second);
    r.readback.clear();
    for (auto& kv : r.big_staging) {
        if (kv.second.base) (void)hipHostFree(kv.second.base);
        if (kv.second.done) (void)hipEventDestroy(kv.second.done);
    }
    r.big_staging.clear();
    r.all.clear();
    r.live.clear();
    r.parked.clear();
    r.bytes_in_use = r.bytes_parked = 0;
    r.ready = false;
    r.device = -1;
    return GNNHIP_OK;
}

int gnnhip_release_scratch(void* stream)
{
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (!r.ready) return GNNHIP_OK;
    hipStream_t s = as_stream(stream);
    GNNHIP_HIP(hipStreamSynchronize(s));
    for (auto it = r.scratch.begin(); it != r.scratch.end();) {
        if (it->first.first == s) {
            (void)hipFree(it->second.first);
            it = r.scratch.erase(it);
        } else {
            ++it;
        }
    }
    return GNNHIP_OK;
}

int gnnhip_malloc(void** device_ptr, size_t bytes) { return pool_acquire(device_ptr, bytes); }

int gnnhip_recycle(void* device_ptr) { return pool_release(device_ptr); }

int gnnhip_free(void* device_ptr)
{
    if (!device_ptr) return GNNHIP_OK;
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (!r.ready) return set_error(GNNHIP_ENOTINIT, "gnnhip is shut down; the block was released with the pool");
    auto it = r.all.find(device_ptr);
    if (it == r.all.end())
        return set_error(GNNHIP_EINVAL, "pointer %p is not owned by the gnnhip pool", device_ptr);
    size_t sz = it->second;
    auto lv = r.live.find(device_ptr);
    if (lv != r.live.end()) {
        r.live.erase(lv);
        r.bytes_in_use -= sz;
    } else {
        auto range = r.parked.equal_range(sz);
        for (auto p = range.first; p != range.second; ++p) {
            if (p->second == device_ptr) {
                r.parked.erase(p);
                r.bytes_parked -= sz;
                break;
            }
        }
    }
    r.all.erase(it);
    GNNHIP_HIP(hipFree(device_ptr));
    return GNNHIP_OK;
}

int gnnhip_pool_stats(size_t* bytes_in_use, size_t* bytes_parked, size_t* n_driver_allocs)
{
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    if (bytes_in_use) *bytes_in_use = r.bytes_in_use;
    if (bytes_parked) *bytes_parked = r.bytes_parked;
    if (n_driver_allocs) *n_driver_allocs = r.n_driver_allocs;
    return GNNHIP_OK;
}

}  // extern "C"

namespace {

// `bytes` (<= kStagingHalf) of the stream's pinned upload buffer, or null when pinned memory is not to be had.
// The slot stays valid until the stream has run everything queued up to the copy that reads it: a half of
// the buffer is reused only after the event recorded behind its last copy has completed.  Caller holds r.mu.
int staging_slot(Runtime& r, hipStream_t s, size_t bytes, char** out)
{
    *out = nullptr;
    Staging& st = r.staging[s];
    if (!st.base) {
        void* q = nullptr;
        if (hipHostMalloc(&q, 2 * kStagingHalf, hipHostMallocDefault) == hipSuccess && q) {
            st.base = static_cast<char*>(q);
            GNNHIP_HIP(hipEventCreateWithFlags(&st.done[0], hipEventDisableTiming));
            GNNHIP_HIP(hipEventCreateWithFlags(&st.done[1], hipEventDisableTiming));
        } else {
            (void)hipGetLastError();
            return GNNHIP_OK;
        }
    }
    const size_t need = (bytes + 255) & ~(size_t)255;
    if (st.used + need > kStagingHalf) {
        // close this half behind its last copy and move to the other one once the device has left it
        GNNHIP_HIP(hipEventRecord(st.done[st.half], s));
        st.pending[st.half] = true;
        st.half ^= 1;
        st.used = 0;
        if (st.pending[st.half]) {
            GNNHIP_HIP(hipEventSynchronize(st.done[st.half]));
            st.pending[st.half] = false;
        }
    }
    *out = st.base + (size_t)st.half * kStagingHalf + st.used;
    st.used += need;
    return GNNHIP_OK;
}

// Positions and values of the non-zero words of w[from, words), appended at *count; false when there are more than cap.
// starts[t] = how many of them lie ahead of word 1024 t (the tiles the device rebuilds the buffer by).
bool collect_nonzero(const unsigned* w, size_t from, size_t words, size_t cap, unsigned* idx, unsigned* val, size_t* count,
                     unsigned* starts)
{
    size_t c = *count;
    for (size_t i = from; i < words; ++i) {
        if ((i & (kExpandTile - 1)) == 0) starts[i / kExpandTile] = (unsigned)c;     // the tile of 1,024 words that begins here
        if (w[i]) {
            if (c == cap) return false;
            idx[c] = (unsigned)i;
            val[c] = w[i];
            ++c;
        }
    }
    *count = c;
    return true;
}

// The same with 256-bit loads, 32 words at a time: four compares against zero make one 32-bit mask, and only the set
// bits are visited.  (One branch per 32 words instead of one per 8: a one-hot matrix of 283,100 words has a non-zero
// word in every fifth group of 8, a pattern branch predictors lose against: 113 -> 25 us on a desktop-class core, and the whole upload of that matrix
// 25 -> 21 us on the host of the GPU box.)
__attribute__((target("avx2"))) bool collect_nonzero_avx2(const unsigned* w, size_t words, size_t cap, unsigned* idx, unsigned* val,
                                                          size_t* count, unsigned* starts)
{
    size_t c = 0, i = 0;
    const __m256i zero = _mm256_setzero_si256();
#define GNNHIP_ZEROS_OF(at) \
    ((unsigned)_mm256_movemask_ps(_mm256_castsi256_ps(_mm256_cmpeq_epi32(_mm256_loadu_si256(reinterpret_cast<const __m256i*>(w + (at))), zero))))
    for (; i + 32 <= words; i += 32) {
        if ((i & (kExpandTile - 1)) == 0) starts[i / kExpandTile] = (unsigned)c;
        unsigned nz = ~(GNNHIP_ZEROS_OF(i) | (GNNHIP_ZEROS_OF(i + 8) << 8) | (GNNHIP_ZEROS_OF(i + 16) << 16) | (GNNHIP_ZEROS_OF(i + 24) << 24));
        if (!nz) continue;
        if (c + (size_t)__builtin_popcount(nz) > cap) return false;
        while (nz) {
            const unsigned j = (unsigned)__builtin_ctz(nz);
            nz &= nz - 1;
            idx[c] = (unsigned)(i + j);
            val[c] = w[i + j];
            ++c;
        }
    }
#undef GNNHIP_ZEROS_OF
    *count = c;
    return collect_nonzero(w, i, words, cap, idx, val, count, starts);
}

// Words [from, to) only (from a multiple of the tile size), for one of several threads that share a large tensor: positions
// are absolute, *count and the starts are relative to this thread's own idx / val region.
__attribute__((target("avx2"))) bool collect_range_avx2(const unsigned* w, size_t from, size_t to, size_t cap, unsigned* idx, unsigned* val,
                                                        size_t* count, unsigned* starts)
{
    size_t c = 0, i = from;
    const __m256i zero = _mm256_setzero_si256();
#define GNNHIP_ZEROS_OF(at) \
    ((unsigned)_mm256_movemask_ps(_mm256_castsi256_ps(_mm256_cmpeq_epi32(_mm256_loadu_si256(reinterpret_cast<const __m256i*>(w + (at))), zero))))
    for (; i + 32 <= to; i += 32) {
        if ((i & (kExpandTile - 1)) == 0) starts[i / kExpandTile] = (unsigned)c;
        unsigned nz = ~(GNNHIP_ZEROS_OF(i) | (GNNHIP_ZEROS_OF(i + 8) << 8) | (GNNHIP_ZEROS_OF(i + 16) << 16) | (GNNHIP_ZEROS_OF(i + 24) << 24));
        if (!nz) continue;
        if (c + (size_t)__builtin_popcount(nz) > cap) return false;
        while (nz) {
            const unsigned j = (unsigned)__builtin_ctz(nz);
            nz &= nz - 1;
            idx[c] = (unsigned)(i + j);
            val[c] = w[i + j];
            ++c;
        }
    }
#undef GNNHIP_ZEROS_OF
    *count = c;
    return collect_nonzero(w, i, to, cap, idx, val, count, starts);
}

// A staged upload leaves the pinned buffer through a kernel, not through hipMemcpyAsync: the runtime hands copies of
// this size to a DMA engine, and the kernel that consumes the data then waits for that engine's completion signal to
// cross over to the compute queue, 15 to 20 us per copy on an otherwise idle device.  A kernel of the stream's own
// queue reads the pinned memory over the bus just as fast at these sizes (up to 2 MB) and orders itself.
constexpr int kStageBlock = 256;
template <typename T>
__global__ __launch_bounds__(kStageBlock) void stage_copy_kernel(T* __restrict__ dst, const T* __restrict__ src, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * kStageBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kStageBlock) dst[i] = src[i];
}

// dst_device[0, bytes) = pinned[0, bytes) on stream s, in the widest pieces the three of them allow
int stage_copy(void* dst_device, const void* pinned, size_t bytes, hipStream_t s)
{
    const uintptr_t bits = reinterpret_cast<uintptr_t>(dst_device) | reinterpret_cast<uintptr_t>(pinned) | (uintptr_t)bytes;
    auto grid_for = [](size_t n) {
        size_t g = (n + kStageBlock - 1) / kStageBlock;                    // one piece per lane: every read of a small copy in flight at once
        return (unsigned)(g < 1 ? 1 : (g > 2048 ? 2048 : g));
    };
    if ((bits & 15) == 0) {
        const size_t n = bytes / 16;
        hipLaunchKernelGGL(stage_copy_kernel<uint4>, dim3(grid_for(n)), dim3(kStageBlock), 0, s, static_cast<uint4*>(dst_device),
                           static_cast<const uint4*>(pinned), n);
    } else if ((bits & 3) == 0) {
        const size_t n = bytes / 4;
        hipLaunchKernelGGL(stage_copy_kernel<unsigned>, dim3(grid_for(n)), dim3(kStageBlock), 0, s, static_cast<unsigned*>(dst_device),
                           static_cast<const unsigned*>(pinned), n);
    } else {
        hipLaunchKernelGGL(stage_copy_kernel<unsigned char>, dim3(grid_for(bytes)), dim3(kStageBlock), 0, s,
                           static_cast<unsigned char*>(dst_device), static_cast<const unsigned char*>(pinned), bytes);
    }
    GNNHIP_LAUNCH_CHECK("stage_copy");
    return GNNHIP_OK;
}

// several staged pieces leaving in one launch: piece blockIdx.y, 32-bit words
constexpr int kStagePieces = 8;
struct StagePieces {
    unsigned* dst[kStagePieces];
    const unsigned* src[kStagePieces];
    size_t words[kStagePieces];
};
__global__ __launch_bounds__(kStageBlock) void stage_copy_pieces_kernel(StagePieces p)
{
    unsigned* __restrict__ dst = p.dst[blockIdx.y];
    const unsigned* __restrict__ src = p.src[blockIdx.y];
    const size_t n = p.words[blockIdx.y];
    for (size_t i = (size_t)blockIdx.x * kStageBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kStageBlock) dst[i] = src[i];
}


// dst[0..n) = 0 except dst[idx[i]] = val[i], idx ascending: a workgroup builds its tile of the destination in
// LDS (zeros, then the entries that fall into it: numbers starts[tile] .. starts[tile + 1] - 1) and writes it out
// whole.  starts, idx and val are read where the host left them, in pinned memory: two trips over the bus per
// workgroup, no copy ahead of the kernel.
__global__ __launch_bounds__(kExpandBlock) void expand_pairs_kernel(unsigned* __restrict__ dst, size_t n, const unsigned* __restrict__ starts,
                                                                    const unsigned* __restrict__ idx, const unsigned* __restrict__ val)
{
    __shared__ unsigned tile[kExpandTile];
    const size_t base = (size_t)blockIdx.x * kExpandTile;
    const unsigned a = starts[blockIdx.x], b = starts[blockIdx.x + 1];
    for (int i = threadIdx.x; i < kExpandTile; i += kExpandBlock) tile[i] = 0u;
    __syncthreads();
    for (unsigned i = a + threadIdx.x; i < b; i += kExpandBlock) tile[idx[i] - base] = val[i];
    __syncthreads();
    for (int i = threadIdx.x; i < kExpandTile; i += kExpandBlock)
        if (base + i < n) dst[base + i] = tile[i];
}

}  // namespace

namespace gnnhip {

// bytes of host memory placed in the stream's pinned staging buffer, for a kernel of that stream to read in place;
// *pinned stays valid until the stream has run everything queued behind this call's next launch.  *pinned = null
// where that cannot be had (no pinned memory, or more than the buffer takes): the caller copies instead.
int stage_in_pinned(hipStream_t s, const void* src_host, size_t bytes, const void** pinned)
{
    *pinned = nullptr;
    if (bytes == 0 || bytes > kStagingHalf) return GNNHIP_OK;
    Runtime& r = rt();
    std::lock_guard<std::mutex> lock(r.mu);
    char* slot = nullptr;
    if (int rc = staging_slot(r, s, bytes, &slot)) return rc;
    if (!slot) return GNNHIP_OK;
    memcpy(slot, src_host, bytes);
    *pinned = slot;
    return GNNHIP_OK;
}

}  // namespace gnnhip

namespace {

// dst_device[0, words) = w[0, words) for a tensor past the staging halves (the dense one-hot feature matrix of a batch of
// ten thousand graphs is 77 MB): the scan for non-zero words is cut into tile-aligned ranges, one per thread, each
// thread collecting into its own part of the pinned buffer; the parts are then pushed together and one kernel rebuilds
// the tensor.  GNNHIP_EUNSUPPORTED (nothing queued) when more than one word in sixteen of some range is non-zero or no
// pinned memory is to be had: the caller copies the tensor as it is.
int sparse_upload_large(void* dst_device, const unsigned* w, size_t words, hipStream_t s)
{
    const size_t tiles = (words + kExpandTile - 1) / kExpandTile;
    const size_t cap = words / 16;
    const size_t bytes = cap * 8 + (tiles + 1) * 4;
    char* base = nullptr;
    hipEvent_t done = nullptr;
    {
        Runtime& r = rt();
        std::lock_guard<std::mutex> lock(r.mu);
        BigStaging& st = r.big_staging[s];
        if (st.pending) {                          // the kernel of the previous large upload still reads the buffer
            GNNHIP_HIP(hipEventSynchronize(st.done));
            st.pending = false;
        }
        if (st.bytes < bytes) {
            if (st.base) (void)hipHostFree(st.base);
            st.base = nullptr;
            st.bytes = 0;
            void* q = nullptr;
            if (hipHostMalloc(&q, bytes, hipHostMallocDefault) != hipSuccess || !q) {
                (void)hipGetLastError();
                return GNNHIP_EUNSUPPORTED;
            }
            st.base = static_cast<char*>(q);
            st.bytes = bytes;
        }
        if (!st.done) GNNHIP_HIP(hipEventCreateWithFlags(&st.done, hipEventDisableTiming));
        base = st.base;
        done = st.done;
    }
    // one host thread at a time feeds a stream: the buffer is this call's from here on
    unsigned* idx = reinterpret_cast<unsigned*>(base);
    unsigned* val = idx + cap;
    unsigned* starts = val + cap;
    const bool avx2 = __builtin_cpu_supports("avx2");
    unsigned hw = std::thread::hardware_concurrency();
    size_t nthreads = hw >= 16 ? 8 : hw >= 4 ? hw / 2 : 1;
    const size_t per_min = (size_t)1 << 20;        // a thread is worth starting for a million words
    if (nthreads > (words + per_min - 1) / per_min) nthreads = (words + per_min - 1) / per_min;
    if (nthreads < 1) nthreads = 1;
    const size_t tiles_per = (tiles + nthreads - 1) / nthreads;
    struct Part { size_t t0, t1, off, count; bool ok; };
    std::vector<Part> parts;
    for (size_t t0 = 0; t0 < tiles; t0 += tiles_per) {
        const size_t t1 = t0 + tiles_per < tiles ? t0 + tiles_per : tiles;
        parts.push_back(Part{t0, t1, t0 * kExpandTile / 16, 0, true});      // its share of cap starts where its words do, over 16
    }
    auto scan = [&](Part& p) {
        const size_t from = p.t0 * kExpandTile, to = p.t1 * kExpandTile < words ? p.t1 * kExpandTile : words;
        const size_t room = (to - from) / 16;
        p.ok = avx2 ? collect_range_avx2(w, from, to, room, idx + p.off, val + p.off, &p.count, starts)
                    : collect_nonzero(w, from, to, room, idx + p.off, val + p.off, &(p.count = 0), starts);
    };
    {
        std::vector<std::thread> workers;
        for (size_t i = 1; i < parts.size(); ++i) workers.emplace_back(scan, std::ref(parts[i]));
        scan(parts[0]);
        for (auto& t : workers) t.join();
    }
    size_t total = 0;
    for (Part& p : parts) {
        if (!p.ok) return GNNHIP_EUNSUPPORTED;
        if (p.off != total) {                      // push the part up against the one before it (it only ever moves down)
            memmove(idx + total, idx + p.off, p.count * sizeof(unsigned));
            memmove(val + total, val + p.off, p.count * sizeof(unsigned));
        }
        if (total)                                 // the part's tile starts were counted from its own first entry
            for (size_t t = p.t0; t < p.t1; ++t) starts[t] += (unsigned)total;
        total += p.count;
    }
    starts[tiles] = (unsigned)total;
    hipLaunchKernelGGL(expand_pairs_kernel, dim3((unsigned)tiles), dim3(kExpandBlock), 0, s, static_cast<unsigned*>(dst_device), words,
                       starts, idx, val);
    GNNHIP_LAUNCH_CHECK("expand_pairs (large)");
    GNNHIP_HIP(hipEventRecord(done, s));
    {
        Runtime& r = rt();
        std::lock_guard<std::mutex> lock(r.mu);
        r.big_staging[s].pending = true;
    }
    return GNNHIP_OK;
}

}  // namespace

extern "C" {

int gnnhip_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes, void* stream)
{
    if (bytes == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(dst_device && src_host, "null pointer in memcpy_h2d");
    if (int rc = require_ready()) return rc;
    // Ordered after earlier work on the stream; returns once the host buffer has been read, so the
    // caller may overwrite it at once (the reference's blocking cudaMemcpy gives callers the same promise).
    hipStream_t s = as_stream(stream);
    if (bytes <= kStagingHalf) {
        Runtime& r = rt();
        std::lock_guard<std::mutex> lock(r.mu);
        char* slot = nullptr;
        if (int rc = staging_slot(r, s, bytes, &slot)) return rc;
        if (slot) {
            memcpy(slot, src_host, bytes);
            return stage_copy(dst_device, slot, bytes, s);
        }
    }
    GNNHIP_HIP(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, s));
    GNNHIP_HIP(hipStreamSynchronize(s));
    return GNNHIP_OK;
}

// Host-to-device copy of `words` 32-bit words that sends only the non-zero ones when they are few (one-hot
// feature matrices: 1.1 MB of which 30 KB are ones).  Same promise as gnnhip_memcpy_h2d; the device ends up with
// the same bits.
// count host-to-device copies; pieces of whole, aligned 32-bit words that fit the staging buffer together leave in
// one launch (the three arrays of a CSR matrix), anything else piece by piece.  Same promise as gnnhip_memcpy_h2d.
int gnnhip_memcpy_h2d_batch(int count, void* const* dst_device, const void* const* src_host, const size_t* bytes, void* stream)
{
    GNNHIP_REQUIRE(count >= 0 && (count == 0 || (dst_device && src_host && bytes)), "bad arguments in memcpy_h2d_batch");
    if (count == 0) return GNNHIP_OK;
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    size_t total = 0;
    bool together = count <= kStagePieces;
    for (int i = 0; i < count; ++i) {
        GNNHIP_REQUIRE(bytes[i] == 0 || (dst_device[i] && src_host[i]), "null pointer in memcpy_h2d_batch");
        together = together && bytes[i] % 4 == 0 && reinterpret_cast<uintptr_t>(dst_device[i]) % 4 == 0;
        total += (bytes[i] + 255) & ~(size_t)255;
    }
    char* slot = nullptr;
    if (together && total <= kStagingHalf) {
        Runtime& r = rt();
        std::lock_guard<std::mutex> lock(r.mu);
        if (int rc = staging_slot(r, s, total, &slot)) return rc;
    }
    if (!slot) {
        for (int i = 0; i < count; ++i)
            if (int rc = gnnhip_memcpy_h2d(dst_device[i], src_host[i], bytes[i], stream)) return rc;
        return GNNHIP_OK;
    }
    StagePieces p;
    size_t at = 0, largest = 0;
    int k = 0;
    for (int i = 0; i < count; ++i) {
        if (bytes[i] == 0) continue;
        memcpy(slot + at, src_host[i], bytes[i]);
        p.dst[k] = static_cast<unsigned*>(dst_device[i]);
        p.src[k] = reinterpret_cast<const unsigned*>(slot + at);
        p.words[k] = bytes[i] / 4;
        if (p.words[k] > largest) largest = p.words[k];
        at += (bytes[i] + 255) & ~(size_t)255;
        ++k;
    }
    if (k == 0) return GNNHIP_OK;
    size_t gx = (largest + kStageBlock - 1) / kStageBlock;
    if (gx > 1024) gx = 1024;
    hipLaunchKernelGGL(stage_copy_pieces_kernel, dim3((unsigned)gx, (unsigned)k), dim3(kStageBlock), 0, s, p);
    GNNHIP_LAUNCH_CHECK("stage_copy_pieces");
    return GNNHIP_OK;
}

int gnnhip_memcpy_h2d_sparse32(void* dst_device, const void* src_host, size_t words, void* stream)
{
    constexpr size_t kMinWords = 16384;                  // below this the plain copy is one short DMA anyway
    const size_t cap = words / 16;                       // non-zero words beyond this: the plain copy
    const size_t tiles = (words + kExpandTile - 1) / kExpandTile;
    if (words < kMinWords || words >= ((size_t)1 << 32)) return gnnhip_memcpy_h2d(dst_device, src_host, words * 4, stream);
    GNNHIP_REQUIRE(dst_device && src_host, "null pointer in memcpy_h2d_sparse32");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    if (cap * 8 + (tiles + 1) * 4 > kStagingHalf) {
        // too large for the staging halves: a pinned buffer of its own, the scan shared by a few threads
        if (int rc = sparse_upload_large(dst_device, static_cast<const unsigned*>(src_host), words, s); rc != GNNHIP_EUNSUPPORTED) return rc;
        return gnnhip_memcpy_h2d(dst_device, src_host, words * 4, stream);
    }
    char* slot = nullptr;
    {
        Runtime& r = rt();
        std::lock_guard<std::mutex> lock(r.mu);
        if (int rc = staging_slot(r, s, cap * 8 + (tiles + 1) * 4, &slot)) return rc;
    }
    if (!slot) return gnnhip_memcpy_h2d(dst_device, src_host, words * 4, stream);
    // the slot belongs to this call from here on: scan without the lock
    const unsigned* w = static_cast<const unsigned*>(src_host);
    unsigned* idx = reinterpret_cast<unsigned*>(slot);
    unsigned* val = idx + cap;
    unsigned* starts = val + cap;
    size_t count = 0;
    const bool few = __builtin_cpu_supports("avx2") ? collect_nonzero_avx2(w, words, cap, idx, val, &count, starts)
                                                    : collect_nonzero(w, 0, words, cap, idx, val, &count, starts);
    if (!few) return gnnhip_memcpy_h2d(dst_device, src_host, words * 4, stream);
    starts[tiles] = (unsigned)count;
    // the kernel reads the slot in place; the slot is not reused before the stream has run past it
    hipLaunchKernelGGL(expand_pairs_kernel, dim3((unsigned)tiles), dim3(kExpandBlock), 0, s, static_cast<unsigned*>(dst_device), words,
                       starts, idx, val);
    GNNHIP_LAUNCH_CHECK("expand_pairs");
    return GNNHIP_OK;
}

int gnnhip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream)
{
    if (bytes == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(dst_host && src_device, "null pointer in memcpy_d2h");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    if (bytes <= kReadbackBytes) {
        // small reads (scalars such as the loss) land in pinned memory: the copy is then a plain DMA that
        // the stream wait covers, instead of the runtime's staged path for pageable destinations
        Runtime& r = rt();
        void* pin = nullptr;
        {
            std::lock_guard<std::mutex> lock(r.mu);
            void*& slot = r.readback[s];
            if (!slot && (hipHostMalloc(&slot, kReadbackBytes, hipHostMallocDefault) != hipSuccess || !slot)) {
                (void)hipGetLastError();
                slot = nullptr;
            }
            pin = slot;
        }
        if (pin) {
            // one reader per stream at a time (the caller's thread owns the stream while it waits)
            GNNHIP_HIP(hipMemcpyAsync(pin, src_device, bytes, hipMemcpyDeviceToHost, s));
            GNNHIP_HIP(hipStreamSynchronize(s));
            memcpy(dst_host, pin, bytes);
            return GNNHIP_OK;
        }
    }
    GNNHIP_HIP(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, s));
    GNNHIP_HIP(hipStreamSynchronize(s));
    return GNNHIP_OK;
}

int gnnhip_memcpy_d2h_batch(int count, void* const* dst_host, const void* const* src_device, const size_t* bytes, void* stream)
{
    GNNHIP_REQUIRE(count >= 0 && (count == 0 || (dst_host && src_device && bytes)), "bad arguments in memcpy_d2h_batch");
    if (count == 0) return GNNHIP_OK;
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    // every piece at an 8-byte boundary of the pinned landing buffer
    size_t total = 0;
    for (int i = 0; i < count; ++i) {
        GNNHIP_REQUIRE(bytes[i] == 0 || (dst_host[i] && src_device[i]), "null pointer in memcpy_d2h_batch");
        total += (bytes[i] + 7) & ~(size_t)7;
    }
    void* pin = nullptr;
    if (total <= kReadbackBytes) {
        Runtime& r = rt();
        std::lock_guard<std::mutex> lock(r.mu);
        void*& slot = r.readback[s];
        if (!slot && (hipHostMalloc(&slot, kReadbackBytes, hipHostMallocDefault) != hipSuccess || !slot)) {
            (void)hipGetLastError();
            slot = nullptr;
        }
        pin = slot;
    }
    if (!pin) {
        for (int i = 0; i < count; ++i)
            if (int rc = gnnhip_memcpy_d2h(dst_host[i], src_device[i], bytes[i], stream)) return rc;
        return GNNHIP_OK;
    }
    size_t at = 0;
    for (int i = 0; i < count; ++i) {
        if (bytes[i]) GNNHIP_HIP(hipMemcpyAsync(static_cast<char*>(pin) + at, src_device[i], bytes[i], hipMemcpyDeviceToHost, s));
        at += (bytes[i] + 7) & ~(size_t)7;
    }
    GNNHIP_HIP(hipStreamSynchronize(s));
    at = 0;
    for (int i = 0; i < count; ++i) {
        if (bytes[i]) memcpy(dst_host[i], static_cast<char*>(pin) + at, bytes[i]);
        at += (bytes[i] + 7) & ~(size_t)7;
    }
    return GNNHIP_OK;
}

int gnnhip_memcpy_d2d(void* dst_device, const void* src_device, size_t bytes, void* stream)
{
    if (bytes == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(dst_device && src_device, "null pointer in memcpy_d2d");
    if (int rc = require_ready()) return rc;
    GNNHIP_HIP(hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return GNNHIP_OK;
}

int gnnhip_stream_sync(void* stream)
{
    if (int rc = require_ready()) return rc;
    GNNHIP_HIP(hipStreamSynchronize(as_stream(stream)));
    return GNNHIP_OK;
}

}  // extern "C"
