// Internal helpers shared by the gfx950 kernels: status handling, launch
// geometry and wave64 reduction primitives (DPP inside a 16-lane row, then two
// cross-row exchanges).
#ifndef GNNHIP_INTERNAL_H
#define GNNHIP_INTERNAL_H

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include <mutex>

#include "gnnhip.h"

namespace gnnhip {

constexpr int kWave = 64;            // CDNA wavefront width
constexpr int kNumCU = 256;          // MI355X compute units
constexpr int kNumXCD = 8;           // accelerator complex dies, one L2 each

int set_error(int code, const char* fmt, ...);
bool runtime_ready();
int require_ready();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

#define GNNHIP_REQUIRE(cond, ...)                                         \
    do {                                                                  \
        if (!(cond)) return ::gnnhip::set_error(GNNHIP_EINVAL, __VA_ARGS__); \
    } while (0)

#define GNNHIP_HIP(call)                                                            \
    do {                                                                            \
        hipError_t e__ = (call);                                                    \
        if (e__ != hipSuccess)                                                      \
            return ::gnnhip::set_error(GNNHIP_EHIP, "%s failed: %s", #call,         \
                                       hipGetErrorString(e__));                     \
    } while (0)

#define GNNHIP_LAUNCH_CHECK(name)                                                   \
    do {                                                                            \
        hipError_t e__ = hipGetLastError();                                         \
        if (e__ != hipSuccess)                                                      \
            return ::gnnhip::set_error(GNNHIP_EHIP, "launch of %s failed: %s", name, \
                                       hipGetErrorString(e__));                     \
    } while (0)

// Kernels that use more than 64 KB of dynamic LDS have to be allowed to, once per kernel instantiation.
// A function-local `static LdsLimit limit;` per instantiation keeps the largest size granted so far;
// raise() is safe to call from several host threads (the runtime serves one device per process).
struct LdsLimit {
    std::mutex mu;
    size_t granted = 0;
    hipError_t raise(const void* kernel, size_t bytes)
    {
        if (bytes <= 64 * 1024) return hipSuccess;
        std::lock_guard<std::mutex> lock(mu);
        if (bytes <= granted) return hipSuccess;
        hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e == hipSuccess) granted = bytes;
        return e;
    }
};

inline unsigned ceil_div_u(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- wave64 primitives
template <int CTRL>
__device__ __forceinline__ float dpp_mov_f(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_mov_i(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}

// DPP controls: quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror.
// Each is an involution that pairs lanes, so both partners combine the same two
// operands and every lane ends with bit-identical results.
constexpr int kDppXor1 = 0xB1;
constexpr int kDppXor2 = 0x4E;
constexpr int kDppHalfMirror = 0x141;   // lane i <-> 7-i inside each group of 8
constexpr int kDppMirror = 0x140;       // lane i <-> 15-i inside each row of 16

// The wave-wide operations below must be called by a whole wavefront (all 64 lanes active).  After the four
// DPP steps every lane of a row of 16 holds its row's result; the four rows are then combined through
// v_readlane (scalar registers), as (row0 . row1) . (row2 . row3), which costs no trip through LDS.
__device__ __forceinline__ float row_value_f(float v, int row) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16 * row)); }
__device__ __forceinline__ int row_value_i(int v, int row) { return __builtin_amdgcn_readlane(v, 16 * row); }

// Every lane of the wavefront receives the sum over all 64 lanes.
__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_mov_f<kDppXor1>(v);
    v += dpp_mov_f<kDppXor2>(v);
    v += dpp_mov_f<kDppHalfMirror>(v);
    v += dpp_mov_f<kDppMirror>(v);
    return (row_value_f(v, 0) + row_value_f(v, 1)) + (row_value_f(v, 2) + row_value_f(v, 3));
}

__device__ __forceinline__ int wave_sum_i(int v)
{
    v += dpp_mov_i<kDppXor1>(v);
    v += dpp_mov_i<kDppXor2>(v);
    v += dpp_mov_i<kDppHalfMirror>(v);
    v += dpp_mov_i<kDppMirror>(v);
    return (row_value_i(v, 0) + row_value_i(v, 1)) + (row_value_i(v, 2) + row_value_i(v, 3));
}

// max with "a < b ? b : a" so that a NaN in b never replaces a (the reference's
// strict comparison never selects a NaN that is not first in the row).
__device__ __forceinline__ float max_keep(float a, float b) { return a < b ? b : a; }

__device__ __forceinline__ float wave_max(float v)
{
    v = max_keep(v, dpp_mov_f<kDppXor1>(v));
    v = max_keep(v, dpp_mov_f<kDppXor2>(v));
    v = max_keep(v, dpp_mov_f<kDppHalfMirror>(v));
    v = max_keep(v, dpp_mov_f<kDppMirror>(v));
    return max_keep(max_keep(row_value_f(v, 0), row_value_f(v, 1)), max_keep(row_value_f(v, 2), row_value_f(v, 3)));
}

// (value, index) arg-max with the lowest index winning ties.
__device__ __forceinline__ void argmax_combine(float& v, int& i, float ov, int oi)
{
    if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
}

__device__ __forceinline__ void wave_argmax(float& v, int& i)
{
    argmax_combine(v, i, dpp_mov_f<kDppXor1>(v), dpp_mov_i<kDppXor1>(i));
    argmax_combine(v, i, dpp_mov_f<kDppXor2>(v), dpp_mov_i<kDppXor2>(i));
    argmax_combine(v, i, dpp_mov_f<kDppHalfMirror>(v), dpp_mov_i<kDppHalfMirror>(i));
    argmax_combine(v, i, dpp_mov_f<kDppMirror>(v), dpp_mov_i<kDppMirror>(i));
    float v0 = row_value_f(v, 0), v2 = row_value_f(v, 2);
    int i0 = row_value_i(i, 0), i2 = row_value_i(i, 2);
    argmax_combine(v0, i0, row_value_f(v, 1), row_value_i(i, 1));
    argmax_combine(v2, i2, row_value_f(v, 3), row_value_i(i, 3));
    argmax_combine(v0, i0, v2, i2);
    v = v0;
    i = i0;
}

// ---------------------------------------------------------------- small vector helpers
typedef float mfma_f4 __attribute__((ext_vector_type(4)));   // accumulator of v_mfma_f32_16x16x4_f32

__device__ __forceinline__ float4 f4_zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ void f4_fma(float4& a, float s, const float4& x)
{
    a.x += s * x.x; a.y += s * x.y; a.z += s * x.z; a.w += s * x.w;
}
// ReLU exactly as the reference writes it: `if (x < 0) x = 0`, so -0.0 and NaN pass through.
__device__ __forceinline__ float relu_ref(float v) { return v < 0.f ? 0.f : v; }
__device__ __forceinline__ float4 relu_ref4(const float4& v)
{
    return make_float4(relu_ref(v.x), relu_ref(v.y), relu_ref(v.z), relu_ref(v.w));
}

// Device memory from the library's pool (released with pool_release).
int pool_acquire(void** p, size_t bytes);
int pool_release(void* p);
// a block of exactly this size straight from the driver, for long-lived blocks of hundreds of megabytes (pool_free
// gives it back to the driver)
int pool_acquire_exact(void** p, size_t bytes);

// Grow-only scratch owned by the library, one buffer per stream, so that calls
// ordered on one stream reuse it safely and calls on different streams never
// share it.  The pointer stays valid until a later call on the same stream asks
// for more bytes.
int stream_scratch(hipStream_t s, size_t bytes, void** p);
// The same with several independent buffers per stream (slot 0 is stream_scratch's):
// slot 1 holds the hub pre-pass results, which must outlive a consumer that itself
// takes slot 0; slot 2 holds the partial tiles of a GEMM split along k, whose operands
// may sit in slot 0.
constexpr int kScratchSlots = 7;     // 3: plan of the column-ordered SpMM, 4: its partial sums, 5: identity matrix of the wide level, 6: (index, value) pairs of a sparse upload
constexpr int kExactScratchSlot = 3;  // slots from here on hold what one matrix needs (up to gigabytes): sized exactly, the old block freed first
int stream_scratch_slot(hipStream_t s, int slot, size_t bytes, void** p);

// reduce.hip: device address of the statically allocated segment offsets on the current device
// (hipGetSymbolAddress once per device; allocates nothing).
int static_offsets_ptr(int** out);

// ---- high-degree rows (hub.hip)
constexpr int kHubThreshold = 64;      // rows with more entries are summed by the pre-pass
constexpr int kHubChunk = 2048;        // entries per partial sum of the pre-pass
constexpr int kHubMinRows = 32768;     // smaller matrices skip the pre-pass: its launches would cost more than a long row
struct HubPlan {
    const int* row_slot;               // [m], defined for rows longer than the pass's threshold only; -1: not summed
    const float* agg;                  // [slots][ld]
    int ld;
};
// A block of pool memory that holds the plan and the sums of one balanced pass for an owner that keeps it across
// calls (a CSR plan); planned: the planning launches have run in it.
struct HubStore {
    void* base = nullptr;
    size_t bytes = 0;
    bool planned = false;
};
// threshold / chunk_len: rows with more entries than `threshold` are summed, cut into chunks of `chunk_len`
// (the consumer must apply the same threshold when it looks a row up in row_slot); max_hubs >= 0: the caller's
// bound on the number of such rows; store: where the pass keeps its arrays (null: the stream's scratch slot 1)
// reuse_plan: the caller states that the previous call on this stream had the very same matrix: same arrays, same structure
// AND same values (the column-ordered pieces keep a copy of the values), nothing rewritten in between.
int hub_prepass(int m, int n, long long nnz, const int* row_ptr, const int* col_idx, const float* val,
                const float* B, int ldb, hipStream_t s, HubPlan* plan, bool reuse_plan = false, bool relu_in = false,
                int threshold = kHubThreshold, int chunk_len = kHubChunk, long long max_hubs = -1, HubStore* store = nullptr);
// scratch bytes of that call (0 when the pass does not apply)
size_t hub_scratch_bytes(int m, int n, long long nnz, int threshold = kHubThreshold, int chunk_len = kHubChunk, long long max_hubs = -1);
// runtime.hip: host bytes placed in the stream's pinned staging buffer for a kernel to read in place (null: not to be had)
int stage_in_pinned(hipStream_t s, const void* src_host, size_t bytes, const void** pinned);
// pieces.hip: what a caller prepares once for a CSR matrix it multiplies with many times (gnnhip_csr_plan_create).
// For large matrices with many entries per row: the rows cut into pieces of consecutive entries, the pieces ordered by
// their first column and the entries copied into that order; for every matrix: the plan of the balanced pass over
// long rows.  All device memory of a plan is pool memory owned by it.
struct CsrPlan {
    unsigned magic = 0;
    const int* row_ptr = nullptr;
    const int* col_idx = nullptr;
    const float* val = nullptr;
    int m = 0, k = 0;
    long long nnz = 0;            // entries of the matrix (an upper bound when the plan lives in stream scratch)
    // ---- column-ordered pieces (has_pieces)
    bool has_pieces = false;
    long long slots = 0;          // capacity of the per-piece arrays (>= number of pieces)
    long long pslots = 0;         // capacity of the partial sums (>= pieces of the rows of several pieces)
    int* first = nullptr;         // [m + 1] pieces before row r
    int* pfirst = nullptr;        // [m + 1] pieces of rows of several pieces before row r: row pointers of P
    int* at = nullptr;            // [slots + 1] entries before the i-th piece in order
    int* target = nullptr;        // [slots] row r >= 0 that the piece is all of, else -1 - (its place among the partial sums)
    int* col_ord = nullptr;       // [nnz] entries in piece order
    float* val_ord = nullptr;
    void* head_block = nullptr;   // first, pfirst
    void* body_block = nullptr;   // the other arrays
    float* part = nullptr;        // partial sums [pslots, ldp], grown to the widest operand seen
    size_t part_bytes = 0;
    HubStore combine_hub;         // balanced pass over P (rows of many pieces)
    // ---- balanced pass over the long rows of A itself (the route without pieces)
    HubStore row_hub;
    bool owned = false;           // blocks come from the pool and go back there with the plan
};
constexpr unsigned kCsrPlanMagic = 0x43535250u;

// spmm.hip: C = alpha*A*B + beta*C on stream s (A is [m,k]); reuse_plan as for hub_prepass.
// skip_empty_rows: rows of A without entries are left as they are in C (the caller treats them as zero; beta must be 0).
// plan: a plan made for exactly these arrays (then nnz is exact and reuse_plan is ignored), or null.
int spmm_dispatch(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                  const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan = false,
                  bool skip_empty_rows = false, CsrPlan* plan = nullptr);

// sort.hip
int exclusive_scan_i32(int* x, long long n, int* seg_scratch, hipStream_t s);
size_t radix_hist_ints(long long n);
size_t radix_seg_ints(long long n);
int radix_order_by_digit(const unsigned* keys, long long n, int shift, unsigned* keys_out, unsigned* perm_out, int* hist, int* seg,
                         hipStream_t s, const unsigned* carried = nullptr);
int spmm_plain_dispatch(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                        const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan = false,
                        HubStore* row_hub = nullptr);
// pieces.hip: C = alpha*A*B + beta*C for large matrices with many entries per row, the rows cut into pieces that
// are summed in the order of their first column; GNNHIP_EUNSUPPORTED (nothing launched, C untouched) where the caller
// keeps its own route, GNNHIP_ENOMEM likewise when the device cannot give the scratch
int spmm_pieces_dispatch(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                         const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan, bool skip_empty_rows,
                         CsrPlan* plan);
// whether a matrix of this shape takes the pieces route at all (the width of the dense operand decides the rest)
bool pieces_route_applies(int m, long long nnz);
CsrPlan* as_csr_plan(void* handle);      // null unless handle is a live plan

// runtime.hip: the pool's blocks given back to the driver (gnnhip_free), for scratch a plan no longer needs
int pool_free(void* p);

}  // namespace gnnhip

#endif
