// CSR SpMM for gfx950:  C[m,n] = alpha * A * B + beta * C,  A CSR (int32), B/C fp32 row-major.
//
// Work decomposition ("row group"): a power-of-two group of G lanes owns one CSR
// row; lane s of the group owns columns 4s..4s+3 (one 128-bit load per gathered
// row).  With n = 64 that is 16 lanes per row and 4 rows per wavefront, with
// n = 128 two rows per wavefront, with n >= 256 one row per wavefront and up to
// four column slabs per lane.  A group reads its row's column indices and values
// once, coalesced, G at a time, and hands them round with an in-group shuffle, so
// index traffic is one pass over the CSR arrays instead of one per output column.
// Gathers are issued four at a time before they are consumed to keep several
// HBM/L2 requests in flight per lane.  Accumulation is in registers in CSR order
// (deterministic, no atomics) and each output element is written exactly once.
//
// Long rows: on matrices of at least kHubMinRows rows a pre-pass (hub.hip) sums the
// rows longer than kHubThreshold entries with the work cut by entries, and the row's
// group here only scales and stores that sum.  Elsewhere rows longer than kLongRow
// entries are set aside inside the workgroup and then processed by all of its 256
// lanes together, which split the row's entries and combine the partial sums in LDS
// in a fixed order (still deterministic).
//
// Bound: HBM.  Algorithmic bytes per launch: 4(m+1) + 8 nnz + 4 k n + 4 m n.
#include "gnnhip_internal.h"

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kLongRow = 2048;      // entries; longer rows are processed by the whole workgroup
constexpr long long kOneRowMeanEntries = 256;   // mean entries per row from which every row gets a workgroup (matrices below kHubMinRows rows)

// Workgroups are dealt round-robin to the 8 XCDs; give each XCD one contiguous
// slice of the row space so rows that share neighbours share an L2.
__device__ __forceinline__ unsigned xcd_remap(unsigned bid, unsigned nblocks)
{
    const unsigned per = nblocks / kNumXCD;
    const unsigned covered = per * kNumXCD;
    if (bid >= covered) return bid;
    return (bid % kNumXCD) * per + bid / kNumXCD;
}

template <int VEC> struct Vec;
template <> struct Vec<4> {
    using T = float4;
    static __device__ __forceinline__ T zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ T load(const float* p) { return *reinterpret_cast<const float4*>(p); }
    static __device__ __forceinline__ void store(float* p, T v) { *reinterpret_cast<float4*>(p) = v; }
    static __device__ __forceinline__ void fma(T& a, float s, T x) { a.x += s * x.x; a.y += s * x.y; a.z += s * x.z; a.w += s * x.w; }
    static __device__ __forceinline__ T axpby(T a, float b, T c) { return make_float4(a.x + b * c.x, a.y + b * c.y, a.z + b * c.z, a.w + b * c.w); }
    static __device__ __forceinline__ T add(T a, T b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
};
template <> struct Vec<1> {
    using T = float;
    static __device__ __forceinline__ T zero() { return 0.f; }
    static __device__ __forceinline__ T load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, T v) { *p = v; }
    static __device__ __forceinline__ void fma(T& a, float s, T x) { a += s * x; }
    static __device__ __forceinline__ T axpby(T a, float b, T c) { return a + b * c; }
    static __device__ __forceinline__ T add(T a, T b) { return a + b; }
};

// One row per group of G = 1 << logG lanes.  A lane owns column slabs
// (sub + it * G) * VEC, it < ITERS; slabs at or beyond n are skipped.
// Rows longer than long_row entries are parked in an LDS list and processed
// afterwards by the whole workgroup: group g takes entries g, g + ngroups, ...
// and the partial sums are added through LDS in group order.
// long_row < 0: one row per workgroup, summed that way whatever its length (few, long rows: pooling 1,024 nodes
// into each of 4,096 subgraphs ran one workgroup per compute unit with a lane group per row: 0.265 ms).
template <int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void spmm_rowgroup_kernel(
    int m, int n, float alpha, const int* __restrict__ row_ptr, const int* __restrict__ col_idx,
    const float* __restrict__ val, const float* __restrict__ B, int ldb, float beta, float* C, int ldc,
    int logG, int long_row, const int* __restrict__ hub_slot, const float* __restrict__ hub_agg, int hub_ld)
{
    using V = Vec<VEC>;
    __shared__ int lr_list[kBlock];
    __shared__ int lr_count;
    __shared__ float red[kBlock * VEC * ITERS];      // [ngroups][G * VEC * ITERS]

    const int G = 1 << logG;
    const int sub = threadIdx.x & (G - 1);
    const int grp = threadIdx.x >> logG;
    const int ngroups = kBlock >> logG;
    const unsigned bid = xcd_remap(blockIdx.x, gridDim.x);
    const bool one_row = long_row < 0;
    const bool owner = !one_row || grp == 0;          // the lane group that answers for `row`
    const long long row = one_row ? (long long)bid : (long long)bid * ngroups + grp;

    if (threadIdx.x == 0) lr_count = 0;
    __syncthreads();

    int start = 0, end = 0;
    if (row < m && owner) { start = row_ptr[row]; end = row_ptr[row + 1]; }
    // a row summed by the hub pre-pass only scales and stores
    int hslot = -1;
    if (hub_slot && end - start > kHubThreshold) hslot = hub_slot[row];
    if (hslot >= 0) end = start;
    const bool deferred = one_row ? (end > start) : (end - start > long_row);
    if (deferred) {
        if (sub == 0) lr_list[atomicAdd(&lr_count, 1)] = (int)row;
        end = start;      // the group idles through the main phase
    }

    typename V::T acc[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) acc[it] = V::zero();

    for (int base = start; base < end; base += G) {
        const int t = base + sub;
        int c = 0;
        float v = 0.f;
        if (t < end) { c = col_idx[t]; v = alpha * val[t]; }
        const int cnt = min(G, end - base);
        for (int j = 0; j < cnt; j += 4) {
            int cj[4];
            float vj[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                cj[u] = __shfl(c, (j + u) & (G - 1), G);   // entries at or past cnt are never accumulated
                vj[u] = __shfl(v, (j + u) & (G - 1), G);
            }
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) {
                    typename V::T x[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        x[u] = (j + u < cnt) ? V::load(B + (size_t)cj[u] * ldb + col0) : V::zero();
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (j + u < cnt) V::fma(acc[it], vj[u], x[u]);
                }
            }
        }
    }

    if (row < m && !deferred && owner) {
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int col0 = (sub + it * G) * VEC;
            if (col0 < n) {
                if (hslot >= 0) acc[it] = V::axpby(V::zero(), alpha, V::load(hub_agg + (size_t)hslot * hub_ld + col0));
                float* dst = C + (size_t)row * ldc + col0;
                if (beta == 0.f) V::store(dst, acc[it]);
                else V::store(dst, V::axpby(acc[it], beta, V::load(dst)));
            }
        }
    }

    __syncthreads();
    const int nlong = lr_count;           // uniform across the workgroup
    const int width = G * VEC * ITERS;
    for (int li = 0; li < nlong; ++li) {
        const int lrow = lr_list[li];
        const int ls = row_ptr[lrow], le = row_ptr[lrow + 1];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc[it] = V::zero();

        int t = ls + grp;
        for (; t + 3 * ngroups < le; t += 4 * ngroups) {
            int c4[4];
            float v4[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) { c4[u] = col_idx[t + u * ngroups]; v4[u] = alpha * val[t + u * ngroups]; }
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) {
                    typename V::T x[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) x[u] = V::load(B + (size_t)c4[u] * ldb + col0);
#pragma unroll
                    for (int u = 0; u < 4; ++u) V::fma(acc[it], v4[u], x[u]);
                }
            }
        }
        for (; t < le; t += ngroups) {
            const int c0 = col_idx[t];
            const float v0 = alpha * val[t];
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) V::fma(acc[it], v0, V::load(B + (size_t)c0 * ldb + col0));
            }
        }

#pragma unroll
        for (int it = 0; it < ITERS; ++it)
            V::store(red + (size_t)grp * width + (sub + it * G) * VEC, acc[it]);
        __syncthreads();
        if (grp == 0) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) {
                    typename V::T s = V::zero();
                    for (int g = 0; g < ngroups; ++g) s = V::add(s, V::load(red + (size_t)g * width + col0));
                    float* dst = C + (size_t)lrow * ldc + col0;
                    if (beta == 0.f) V::store(dst, s);
                    else V::store(dst, V::axpby(s, beta, V::load(dst)));
                }
            }
        }
        __syncthreads();
    }
}

inline int ilog2_ceil(int x)
{
    int l = 0;
    while ((1 << l) < x) ++l;
    return l;
}

template <int VEC, int ITERS>
int launch_slab(int m, int n, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                const float* B, int ldb, float beta, float* C, int ldc, int logG, const HubPlan& hubs, bool one_row, hipStream_t s)
{
    const int groups_per_block = one_row ? 1 : kBlock >> logG;
    const unsigned blocks = ceil_div_u((size_t)m, (size_t)groups_per_block);
    hipLaunchKernelGGL((spmm_rowgroup_kernel<VEC, ITERS>), dim3(blocks), dim3(kBlock), 0, s,
                       m, n, alpha, row_ptr, col_idx, val, B, ldb, beta, C, ldc, logG, one_row ? -1 : kLongRow, hubs.row_slot, hubs.agg,
                       hubs.ld);
    GNNHIP_LAUNCH_CHECK("spmm_rowgroup");
    return GNNHIP_OK;
}

}  // namespace

// Shared with the fused forward: C = alpha*A*B + beta*C on stream s.
int spmm_dispatch(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                  const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan, bool skip_empty_rows,
                  CsrPlan* plan)
{
    // large matrices with many entries per row (power-law graphs): rows cut into pieces, summed in column order.  That
    // route takes all its scratch (about 40 bytes per entry of A + 4 n bytes per piece) before its first launch: when
    // the device cannot give it, C is untouched and the row-group route below, which needs far less, does the product.
    if (int rc = spmm_pieces_dispatch(m, k, n, nnz, alpha, row_ptr, col_idx, val, B, ldb, beta, C, ldc, s, reuse_plan, skip_empty_rows, plan);
        rc != GNNHIP_EUNSUPPORTED && rc != GNNHIP_ENOMEM)
        return rc;
    return spmm_plain_dispatch(m, k, n, nnz, alpha, row_ptr, col_idx, val, B, ldb, beta, C, ldc, s, reuse_plan, plan ? &plan->row_hub : nullptr);
}

// The row-group route alone (with its pass over very long rows); nnz may be an upper bound.  row_hub: where a plan's
// owner keeps the pass's arrays across calls.
int spmm_plain_dispatch(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                        const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan, HubStore* row_hub)
{
    (void)k;
    // few rows of hundreds of entries each (sum-pooling into subgraphs): a workgroup per row instead of a lane group
    const bool one_row = m < kHubMinRows && nnz >= kOneRowMeanEntries * (long long)m;
    const bool vec4 = (n % 4 == 0) && (ldb % 4 == 0) && (ldc % 4 == 0) && aligned16(B) && aligned16(C);
    const int vec = vec4 ? 4 : 1;
    // columns are processed in slabs of at most 64 lanes * vec * 4
    const int slab_max = kWave * vec * 4;
    for (int col0 = 0; col0 < n; col0 += slab_max) {
        const int w = (n - col0 < slab_max) ? (n - col0) : slab_max;
        const int units = (w + vec - 1) / vec;              // column units of `vec` floats
        int logG = ilog2_ceil(units < kWave ? units : kWave);
        const int G = 1 << logG;
        const int iters = (units + G - 1) / G;              // 1..4
        const float* Bs = B + col0;
        float* Cs = C + col0;
        int rc;
        HubPlan hubs;
        if ((rc = hub_prepass(m, w, nnz, row_ptr, col_idx, val, Bs, ldb, s, &hubs, reuse_plan && n <= slab_max, false, kHubThreshold, kHubChunk, -1, row_hub))) return rc;
        if (vec4) {
            if (iters <= 1) rc = launch_slab<4, 1>(m, w, alpha, row_ptr, col_idx, val, Bs, ldb, beta, Cs, ldc, logG, hubs, one_row, s);
            else if (iters == 2) rc = launch_slab<4, 2>(m, w, alpha, row_ptr, col_idx, val, Bs, ldb, beta, Cs, ldc, logG, hubs, one_row, s);
            else rc = launch_slab<4, 4>(m, w, alpha, row_ptr, col_idx, val, Bs, ldb, beta, Cs, ldc, logG, hubs, one_row, s);
        } else {
            if (iters <= 1) rc = launch_slab<1, 1>(m, w, alpha, row_ptr, col_idx, val, Bs, ldb, beta, Cs, ldc, logG, hubs, one_row, s);
            else if (iters == 2) rc = launch_slab<1, 2>(m, w, alpha, row_ptr, col_idx, val, Bs, ldb, beta, Cs, ldc, logG, hubs, one_row, s);
            else rc = launch_slab<1, 4>(m, w, alpha, row_ptr, col_idx, val, Bs, ldb, beta, Cs, ldc, logG, hubs, one_row, s);
        }
        if (rc) return rc;
    }
    return GNNHIP_OK;
}

}  // namespace gnnhip

using namespace gnnhip;

extern "C" int gnnhip_spmm_csr_f32(int m, int k, int n, int nnz, float alpha, const int* row_ptr, const int* col_idx,
                                   const float* val, const float* B, int ldb, float beta, float* C, int ldc,
                                   void* stream)
{
    GNNHIP_REQUIRE(m >= 0 && k >= 0 && n >= 0 && nnz >= 0, "negative dimension in spmm (m=%d k=%d n=%d nnz=%d)", m, k, n, nnz);
    if (m == 0 || n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(row_ptr && C, "null row_ptr or output in spmm");
    GNNHIP_REQUIRE(ldb >= n && ldc >= n, "leading dimension smaller than n in spmm (ldb=%d ldc=%d n=%d)", ldb, ldc, n);
    GNNHIP_REQUIRE(k == 0 || B, "null dense operand in spmm");   // col_idx / val may be null when A has no entries
    if (int rc = require_ready()) return rc;
    return spmm_dispatch(m, k, n, nnz, alpha, row_ptr, col_idx, val, B, ldb, beta, C, ldc, as_stream(stream));
}

extern "C" int gnnhip_spmm_csr_planned_f32(void* plan, int n, float alpha, const float* B, int ldb, float beta, float* C, int ldc,
                                           void* stream)
{
    CsrPlan* p = as_csr_plan(plan);
    GNNHIP_REQUIRE(p, "%p is not a live CSR plan", plan);
    GNNHIP_REQUIRE(n >= 0, "negative width in spmm_csr_planned (n=%d)", n);
    if (p->m == 0 || n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(C, "null output in spmm_csr_planned");
    GNNHIP_REQUIRE(ldb >= n && ldc >= n, "leading dimension smaller than n in spmm_csr_planned (ldb=%d ldc=%d n=%d)", ldb, ldc, n);
    GNNHIP_REQUIRE(p->k == 0 || B, "null dense operand in spmm_csr_planned");
    if (int rc = require_ready()) return rc;
    return spmm_dispatch(p->m, p->k, n, p->nnz, alpha, p->row_ptr, p->col_idx, p->val, B, ldb, beta, C, ldc, as_stream(stream), false, false, p);
}
