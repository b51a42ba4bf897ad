// Balanced pre-pass for high-degree rows ("hubs") of a CSR matrix.
//
// The SpMM and fused-level kernels give a row to a group of lanes, which is right
// for the short rows of molecule batches and of uniform random graphs but leaves
// one group, or one workgroup, alone with a row of 10^5 entries on a power-law
// graph (R-MAT, a = 0.57: the largest of 4M rows holds 160,000 of 64M entries, and
// the hubs sit next to each other at the low row indices).  Rows with more than
// kHubThreshold entries are therefore summed here, ahead of the consumer kernel,
// with the work cut by entries instead of by rows:
//
//   count   per 1024 rows: number of hubs and of their chunks (kHubChunk entries each)
//   scan    exclusive scan of those counts by one workgroup -> slots of hubs and chunks
//           (only past kFillScanBlocks workgroups; below that every workgroup of fill adds up the
//           counts before its own)
//   fill    row_slot[row] (written for hubs only), per hub its first chunk, per chunk its hub
//   partial one wavefront per chunk: sum of val * B[col, :] over the chunk; a hub of one chunk is
//           finished with that: agg[slot][n]
//   finish  a hub of several chunks: its chunks' sums added in chunk order by a lane group, in a launch
//           of its own.  (One launch, with the wavefront that delivers a hub's last chunk adding the
//           sums, was the first version: the release / acquire fences it needs between wavefronts on
//           different dies write the L2 back, and 4,600 of them made up most of a 0.14 ms launch.)
//
// The consumer reads agg[row_slot[row]] for a row whose length exceeds the
// threshold.  Every sum is taken in an order fixed by the matrix structure, so the
// result does not depend on scheduling: no atomics, no communication inside a launch.
#include "gnnhip_internal.h"

#include <map>

namespace gnnhip {

namespace {

constexpr int kBlock = 256;
constexpr int kRowsPerBlock = 1024;          // count / fill: four consecutive rows per lane
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kFillScanBlocks = 4096;       // up to this many workgroups (4M rows) fill does the scan itself

__device__ __forceinline__ int hub_chunks(int deg, int chunk) { return (deg + chunk - 1) / chunk; }

// Exclusive prefix over the 256 lanes of the workgroup, in lane order; *total receives the sum.
__device__ __forceinline__ int block_exclusive_scan(int v, int* sh, int* total)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    int incl = v;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int o = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += o;
    }
    if (lane == kWave - 1) sh[wave] = incl;
    __syncthreads();
    int base = 0, tot = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) {
        if (w < wave) base += sh[w];
        tot += sh[w];
    }
    __syncthreads();
    *total = tot;
    return base + incl - v;
}

__global__ __launch_bounds__(kBlock) void hub_count_kernel(int m, const int* __restrict__ row_ptr,
                                                            int* __restrict__ block_hubs, int* __restrict__ block_chunks,
                                                            int threshold, int chunk_len)
{
    __shared__ int sh[2][kWavesPerBlock];
    const long long r0 = (long long)blockIdx.x * kRowsPerBlock + threadIdx.x * 4;
    int hubs = 0, chunks = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const long long r = r0 + i;
        if (r < m) {
            const int deg = row_ptr[r + 1] - row_ptr[r];
            if (deg > threshold) { ++hubs; chunks += hub_chunks(deg, chunk_len); }
        }
    }
    hubs = wave_sum_i(hubs);
    chunks = wave_sum_i(chunks);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) { sh[0][wave] = hubs; sh[1][wave] = chunks; }
    __syncthreads();
    if (threadIdx.x == 0) {
        int h = 0, c = 0;
        for (int w = 0; w < kWavesPerBlock; ++w) { h += sh[0][w]; c += sh[1][w]; }
        block_hubs[blockIdx.x] = h;
        block_chunks[blockIdx.x] = c;
    }
}

// In-place exclusive scan of two arrays of nb entries by one workgroup; totals go to counts[0..1].
constexpr int kScanBlock = 1024;
__global__ __launch_bounds__(kScanBlock) void hub_scan_kernel(int nb, int* __restrict__ block_hubs,
                                                               int* __restrict__ block_chunks, int* __restrict__ counts)
{
    __shared__ int wave_tot[2][kScanBlock / kWave];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int per = (nb + kScanBlock - 1) / kScanBlock;
    const int lo = min(tid * per, nb), hi = min(lo + per, nb);
    int lh = 0, lc = 0;
    for (int i = lo; i < hi; ++i) { lh += block_hubs[i]; lc += block_chunks[i]; }
    int ih = lh, ic = lc;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int oh = __shfl_up(ih, d, kWave), oc = __shfl_up(ic, d, kWave);
        if (lane >= d) { ih += oh; ic += oc; }
    }
    if (lane == kWave - 1) { wave_tot[0][wave] = ih; wave_tot[1][wave] = ic; }
    __syncthreads();
    int bh = 0, bc = 0;
    for (int w = 0; w < wave; ++w) { bh += wave_tot[0][w]; bc += wave_tot[1][w]; }
    int rh = bh + ih - lh, rc = bc + ic - lc;
    for (int i = lo; i < hi; ++i) {
        const int h = block_hubs[i], c = block_chunks[i];
        block_hubs[i] = rh; block_chunks[i] = rc;
        rh += h; rc += c;
    }
    if (tid == kScanBlock - 1) { counts[0] = rh; counts[1] = rc; }
}

// SCAN: block_hubs / block_chunks hold the raw counts of hub_count_kernel and every workgroup adds up
// the entries before its own (few workgroups); otherwise they hold the exclusive scan already.
template <bool SCAN>
__global__ __launch_bounds__(kBlock) void hub_fill_kernel(int m, int nb, const int* __restrict__ row_ptr,
                                                           const int* __restrict__ block_hubs, const int* __restrict__ block_chunks,
                                                           int hub_cap, int chunk_cap, int* __restrict__ row_slot,
                                                           int* __restrict__ hub_row, int* __restrict__ hub_chunk0,
                                                           int* __restrict__ chunk_hub, int* __restrict__ hub_done,
                                                           int* __restrict__ counts, int threshold, int chunk_len)
{
    __shared__ int sh[kWavesPerBlock];
    __shared__ int base_sh[2];
    int slot0, chunk0;
    if (SCAN) {
        int h = 0, c = 0;
        for (int i = threadIdx.x; i < (int)blockIdx.x; i += kBlock) { h += block_hubs[i]; c += block_chunks[i]; }
        h = wave_sum_i(h);
        c = wave_sum_i(c);
        __shared__ int part_sh[2][kWavesPerBlock];
        if ((threadIdx.x & (kWave - 1)) == 0) { part_sh[0][threadIdx.x / kWave] = h; part_sh[1][threadIdx.x / kWave] = c; }
        __syncthreads();
        if (threadIdx.x == 0) {
            int hh = 0, cc = 0;
            for (int w = 0; w < kWavesPerBlock; ++w) { hh += part_sh[0][w]; cc += part_sh[1][w]; }
            base_sh[0] = hh;
            base_sh[1] = cc;
            if ((int)blockIdx.x == nb - 1) { counts[0] = hh + block_hubs[blockIdx.x]; counts[1] = cc + block_chunks[blockIdx.x]; }
        }
        __syncthreads();
        slot0 = base_sh[0];
        chunk0 = base_sh[1];
    } else {
        slot0 = block_hubs[blockIdx.x];
        chunk0 = block_chunks[blockIdx.x];
    }
    const long long r0 = (long long)blockIdx.x * kRowsPerBlock + threadIdx.x * 4;
    int deg[4];
    int hubs = 0, chunks = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const long long r = r0 + i;
        deg[i] = 0;
        if (r < m) deg[i] = row_ptr[r + 1] - row_ptr[r];
        if (deg[i] > threshold) { ++hubs; chunks += hub_chunks(deg[i], chunk_len); }
    }
    int tot;
    int slot = slot0 + block_exclusive_scan(hubs, sh, &tot);
    int chunk = chunk0 + block_exclusive_scan(chunks, sh, &tot);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (deg[i] > threshold) {
            const int nc = hub_chunks(deg[i], chunk_len);
            // a hub past the capacity of the buffers keeps slot -1: its consumer sums it in place
            const bool fits = slot < hub_cap && chunk + nc <= chunk_cap;
            row_slot[r0 + i] = fits ? slot : -1;
            if (fits) {
                hub_row[slot] = (int)(r0 + i);
                hub_chunk0[slot] = chunk;
            } else if (slot < hub_cap) {
                hub_row[slot] = -1;                  // the finishing pass skips it
            }
            for (int j = 0; j < nc && chunk + j < chunk_cap; ++j) chunk_hub[chunk + j] = fits ? slot : -1;
            ++slot;
            chunk += nc;
        }
    }
}

template <int VEC> struct HV;
template <> struct HV<4> {
    using T = float4;
    static __device__ __forceinline__ T zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ T load(const float* p) { return *reinterpret_cast<const float4*>(p); }
    static __device__ __forceinline__ T load(const float* p, int relu) { const T v = load(p); return relu ? relu_ref4(v) : v; }
    static __device__ __forceinline__ void store(float* p, T v) { *reinterpret_cast<float4*>(p) = v; }
    static __device__ __forceinline__ void fma(T& a, float s, T x) { a.x += s * x.x; a.y += s * x.y; a.z += s * x.z; a.w += s * x.w; }
    static __device__ __forceinline__ T add(T a, T b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }
};
template <> struct HV<1> {
    using T = float;
    static __device__ __forceinline__ T zero() { return 0.f; }
    static __device__ __forceinline__ T load(const float* p) { return *p; }
    static __device__ __forceinline__ T load(const float* p, int relu) { const T v = *p; return relu ? relu_ref(v) : v; }
    static __device__ __forceinline__ void store(float* p, T v) { *p = v; }
    static __device__ __forceinline__ void fma(T& a, float s, T x) { a += s * x; }
    static __device__ __forceinline__ T add(T a, T b) { return a + b; }
};

// One wavefront per chunk.  The wavefront is split into 64 / G lane groups; group g takes the
// chunk's entries g, g + ngroups, ... eight at a time, a lane owns the column slabs
// (sub + it * G) * VEC.  The groups' sums are added through LDS in group order.
template <int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void hub_partial_kernel(
    const int* __restrict__ counts, int chunk_cap, int n, const int* __restrict__ row_ptr, const int* __restrict__ col_idx,
    const float* __restrict__ val, const float* __restrict__ B, int ldb, int logG,
    const int* __restrict__ hub_row, const int* __restrict__ hub_chunk0, const int* __restrict__ chunk_hub,
    float* __restrict__ part, int ldp, float* __restrict__ agg, int relu_in, int chunk_len)
{
    // relu_in: the rows of B are used as ReLU(B) (a first level that reads msg in place of h0)
    using V = HV<VEC>;
    __shared__ float red[kWavesPerBlock][kWave * VEC * ITERS];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int G = 1 << logG, sub = lane & (G - 1), grp = lane >> logG, ngroups = kWave >> logG;
    const int width = G * VEC * ITERS;
    const int nchunks = min(counts[1], chunk_cap);
    for (int c = blockIdx.x * kWavesPerBlock + wave; c < nchunks; c += gridDim.x * kWavesPerBlock) {
        const int slot = chunk_hub[c];
        if (slot < 0) continue;                  // chunk of a hub that did not fit the buffers
        const int row = hub_row[slot];
        const int rb = row_ptr[row], re = row_ptr[row + 1];
        const int nc = hub_chunks(re - rb, chunk_len);
        const int cb = rb + (c - hub_chunk0[slot]) * chunk_len;
        const int ce = min(cb + chunk_len, re);
        typename V::T acc[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc[it] = V::zero();
        // eight entries of the group at a time, the last ones of the chunk under a predicate (a serial tail would
        // walk up to seven dependent index -> row loads one after the other, and most chunks of the matrices that
        // pick partial sums are shorter than one such block); the order of the additions is the entries' order
        for (int t = cb + grp; t < ce; t += 8 * ngroups) {
            int c8[8];
            float v8[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const bool ok = t + u * ngroups < ce;
                // no index array: entry t of the row is column t with weight 1 (a matrix that picks consecutive rows of B,
                // whose row loads then wait for no index load)
                c8[u] = !ok ? 0 : col_idx ? col_idx[t + u * ngroups] : t + u * ngroups;
                v8[u] = !ok ? 0.f : val ? val[t + u * ngroups] : 1.f;
            }
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) {
                    typename V::T x[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        x[u] = (t + u * ngroups < ce) ? V::load(B + (size_t)c8[u] * ldb + col0, relu_in) : V::zero();
#pragma unroll
                    for (int u = 0; u < 8; ++u)
                        if (t + u * ngroups < ce) V::fma(acc[it], v8[u], x[u]);
                }
            }
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) V::store(red[wave] + grp * width + (sub + it * G) * VEC, acc[it]);
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        float* dst = (nc == 1) ? agg + (size_t)slot * ldp : part + (size_t)c * ldp;
        if (grp == 0) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) {
                    typename V::T s = V::zero();
                    for (int g = 0; g < ngroups; ++g) s = V::add(s, V::load(red[wave] + g * width + col0));
                    V::store(dst + col0, s);
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");       // red[wave] is rewritten by the next chunk
    }
}

// agg[slot] = sum of the chunks' sums, in chunk order, for every hub of several chunks; one lane group per hub.
template <int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void hub_finish_kernel(
    const int* __restrict__ counts, int hub_cap, int n, const int* __restrict__ row_ptr, int logG,
    const int* __restrict__ hub_row, const int* __restrict__ hub_chunk0, const float* __restrict__ part, int ldp,
    float* __restrict__ agg, int chunk_len)
{
    using V = HV<VEC>;
    const int G = 1 << logG, sub = threadIdx.x & (G - 1), grp = threadIdx.x >> logG, ngroups = kBlock >> logG;
    const int nhubs = min(counts[0], hub_cap);
    for (int slot = blockIdx.x * ngroups + grp; slot < nhubs; slot += gridDim.x * ngroups) {
        const int row = hub_row[slot];
        if (row < 0) continue;                   // did not fit the buffers: its consumer sums it in place
        const int nc = hub_chunks(row_ptr[row + 1] - row_ptr[row], chunk_len);
        if (nc <= 1) continue;
        const int c0 = hub_chunk0[slot];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int col0 = (sub + it * G) * VEC;
            if (col0 >= n) continue;
            typename V::T sum = V::zero();
            for (int j0 = 0; j0 < nc; j0 += 8) {
                typename V::T p[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) p[u] = (j0 + u < nc) ? V::load(part + (size_t)(c0 + j0 + u) * ldp + col0) : V::zero();
#pragma unroll
                for (int u = 0; u < 8; ++u)
                    if (j0 + u < nc) sum = V::add(sum, p[u]);
            }
            V::store(agg + (size_t)slot * ldp + col0, sum);
        }
    }
}

inline int ilog2_ceil_(int x)
{
    int l = 0;
    while ((1 << l) < x) ++l;
    return l;
}

inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

template <int VEC, int ITERS>
void launch_partial(hipStream_t s, const int* counts, int chunk_cap, int n, const int* row_ptr, const int* col_idx,
                    const float* val, const float* B, int ldb, int logG, const int* hub_row, const int* hub_chunk0,
                    const int* chunk_hub, float* part, int ldp, float* agg, int hub_cap, int relu_in, int chunk_len)
{
    const unsigned grid = kNumCU * 16;
    hipLaunchKernelGGL((hub_partial_kernel<VEC, ITERS>), dim3(grid), dim3(kBlock), 0, s, counts, chunk_cap, n, row_ptr,
                       col_idx, val, B, ldb, logG, hub_row, hub_chunk0, chunk_hub, part, ldp, agg, relu_in, chunk_len);
    // the hubs of several chunks (few): a lane group each
    const int groups = kBlock >> logG;
    unsigned fgrid = (unsigned)((hub_cap + groups - 1) / groups);
    if (fgrid > (unsigned)kNumCU) fgrid = kNumCU;
    if (fgrid < 1) fgrid = 1;
    hipLaunchKernelGGL((hub_finish_kernel<VEC, ITERS>), dim3(fgrid), dim3(kBlock), 0, s, counts, hub_cap, n, row_ptr, logG, hub_row,
                       hub_chunk0, part, ldp, agg, chunk_len);
}

}  // namespace

namespace {

// Where the arrays of one pre-pass lie inside its block; everything up to `part` does not depend on the width n.
struct HubLayout {
    int nb, hub_cap, chunk_cap, ldp;
    size_t o_counts, o_bh, o_bc, o_slot, o_hrow, o_hc0, o_chub, o_done, o_part, o_agg, bytes;
};

HubLayout hub_layout(int m, int n, long long nnz, int threshold, int chunk_len, long long max_hubs)
{
    HubLayout L;
    L.ldp = (int)round_up((size_t)n, 4);
    L.nb = (m + kRowsPerBlock - 1) / kRowsPerBlock;
    long long hub_cap_ll = nnz / (threshold + 1) + 1;
    if (max_hubs >= 0 && max_hubs < hub_cap_ll) hub_cap_ll = max_hubs;
    const long long chunk_cap_ll = nnz / chunk_len + hub_cap_ll + 1;
    L.hub_cap = (int)(hub_cap_ll < m ? hub_cap_ll : m);
    L.chunk_cap = (int)chunk_cap_ll;
    size_t off = 0;
    auto carve = [&](size_t bytes) { const size_t o = off; off = round_up(off + bytes, 256); return o; };
    L.o_counts = carve(sizeof(int) * 4);
    L.o_bh = carve(sizeof(int) * L.nb);
    L.o_bc = carve(sizeof(int) * L.nb);
    L.o_slot = carve(sizeof(int) * (size_t)m);
    L.o_hrow = carve(sizeof(int) * (size_t)L.hub_cap);
    L.o_hc0 = carve(sizeof(int) * (size_t)L.hub_cap);
    L.o_chub = carve(sizeof(int) * (size_t)L.chunk_cap);
    L.o_done = carve(sizeof(int) * (size_t)L.hub_cap);
    L.o_part = carve(sizeof(float) * (size_t)L.chunk_cap * L.ldp);
    L.o_agg = carve(sizeof(float) * (size_t)L.hub_cap * L.ldp);
    L.bytes = off;
    return L;
}

inline bool hub_pass_applies(int m, int n, long long nnz, int threshold) { return !(m < kHubMinRows || nnz <= threshold || n > kWave * 16); }

}  // namespace

// Bytes of scratch a hub_prepass call with these arguments takes (0: the pass does not run).  A caller that must not
// fail for lack of memory after its own first launch reserves them up front (stream_scratch_slot(s, 1, ...)).
size_t hub_scratch_bytes(int m, int n, long long nnz, int threshold, int chunk_len, long long max_hubs)
{
    if (!hub_pass_applies(m, n, nnz, threshold)) return 0;
    return hub_layout(m, n, nnz, threshold, chunk_len, max_hubs).bytes;
}

// Sums the hubs of A (rows longer than `threshold` entries, cut into chunks of `chunk_len`) times B[:, 0..n) into
// plan->agg.  col_idx == nullptr: entry t is column t; val == nullptr: every weight is 1.  max_hubs, when not negative, is the caller's bound on the number of such rows (it sizes the buffers).
// n <= 1024.  Without `store` the buffers live in the stream's scratch slot 1 and stay valid until the next
// hub_prepass on the same stream; with it they live in a block the store's owner keeps (pool memory, grown when a
// wider operand needs it), and the planning launches run only while store->planned is false.
// reuse_plan (no store): the caller guarantees that the structure of A has not changed since the previous call on
// this stream with the same arguments (the levels of one forward); the planning launches
// (count, scan, fill) are then skipped and only the sums are recomputed.
int hub_prepass(int m, int n, long long nnz, const int* row_ptr, const int* col_idx, const float* val,
                const float* B, int ldb, hipStream_t s, HubPlan* plan, bool reuse_plan, bool relu_in, int threshold, int chunk_len,
                long long max_hubs, HubStore* store)
{
    plan->row_slot = nullptr;
    plan->agg = nullptr;
    plan->ld = 0;
    if (!hub_pass_applies(m, n, nnz, threshold)) return GNNHIP_OK;
    const bool vec4 = (n % 4 == 0) && (ldb % 4 == 0) && aligned16(B);
    const int vec = vec4 ? 4 : 1;
    const int units = (n + vec - 1) / vec;
    const int logG = ilog2_ceil_(units < kWave ? units : kWave);
    const int G = 1 << logG;
    const int iters = (units + G - 1) / G;                   // 1..4
    const HubLayout L = hub_layout(m, n, nnz, threshold, chunk_len, max_hubs);
    const int ldp = L.ldp, nb = L.nb, hub_cap = L.hub_cap, chunk_cap = L.chunk_cap;

    void* base = nullptr;
    if (store) {
        if (store->bytes < L.bytes) {
            if (store->base) {
                GNNHIP_HIP(hipStreamSynchronize(s));             // earlier launches may still read the old block
                (void)pool_free(store->base);
                store->base = nullptr;
                store->bytes = 0;
            }
            if (int rc = pool_acquire_exact(&store->base, L.bytes)) return rc;
            store->bytes = L.bytes;
            store->planned = false;
        }
        base = store->base;
    } else if (int rc = stream_scratch_slot(s, 1, L.bytes, &base)) {
        return rc;
    }
    char* b = static_cast<char*>(base);
    int* counts = reinterpret_cast<int*>(b + L.o_counts);
    int* bh = reinterpret_cast<int*>(b + L.o_bh);
    int* bc = reinterpret_cast<int*>(b + L.o_bc);
    int* row_slot = reinterpret_cast<int*>(b + L.o_slot);
    int* hub_row = reinterpret_cast<int*>(b + L.o_hrow);
    int* hub_chunk0 = reinterpret_cast<int*>(b + L.o_hc0);
    int* chunk_hub = reinterpret_cast<int*>(b + L.o_chub);
    int* hub_done = reinterpret_cast<int*>(b + L.o_done);
    float* part = reinterpret_cast<float*>(b + L.o_part);
    float* agg = reinterpret_cast<float*>(b + L.o_agg);

    // What the stream's scratch slot holds a plan for.  Kept per stream, next to the scratch it describes (any thread
    // that plans on the stream replaces it), not per thread.
    struct Memo { const int* row_ptr; int m, n; long long nnz; void* base; int threshold, chunk_len, hub_cap; };
    static std::mutex memo_mu;
    static std::map<hipStream_t, Memo> memos;
    bool planned;
    if (store) {
        planned = store->planned;
    } else {
        std::lock_guard<std::mutex> lock(memo_mu);
        auto it = memos.find(s);
        planned = reuse_plan && it != memos.end() && it->second.row_ptr == row_ptr && it->second.m == m && it->second.n == n &&
                  it->second.nnz == nnz && it->second.base == base && it->second.threshold == threshold &&
                  it->second.chunk_len == chunk_len && it->second.hub_cap == hub_cap;
        if (!planned) memos[s] = Memo{row_ptr, m, n, nnz, base, threshold, chunk_len, hub_cap};
    }
    if (!planned) {
        hipLaunchKernelGGL(hub_count_kernel, dim3(nb), dim3(kBlock), 0, s, m, row_ptr, bh, bc, threshold, chunk_len);
        if (nb <= kFillScanBlocks) {
            hipLaunchKernelGGL(hub_fill_kernel<true>, dim3(nb), dim3(kBlock), 0, s, m, nb, row_ptr, bh, bc, hub_cap, chunk_cap,
                               row_slot, hub_row, hub_chunk0, chunk_hub, hub_done, counts, threshold, chunk_len);
        } else {
            hipLaunchKernelGGL(hub_scan_kernel, dim3(1), dim3(kScanBlock), 0, s, nb, bh, bc, counts);
            hipLaunchKernelGGL(hub_fill_kernel<false>, dim3(nb), dim3(kBlock), 0, s, m, nb, row_ptr, bh, bc, hub_cap, chunk_cap,
                               row_slot, hub_row, hub_chunk0, chunk_hub, hub_done, counts, threshold, chunk_len);
        }
        if (store) store->planned = true;
    }
    if (vec4) {
        if (iters <= 1) launch_partial<4, 1>(s, counts, chunk_cap, n, row_ptr, col_idx, val, B, ldb, logG, hub_row, hub_chunk0, chunk_hub, part, ldp, agg, hub_cap, relu_in ? 1 : 0, chunk_len);
        else if (iters == 2) launch_partial<4, 2>(s, counts, chunk_cap, n, row_ptr, col_idx, val, B, ldb, logG, hub_row, hub_chunk0, chunk_hub, part, ldp, agg, hub_cap, relu_in ? 1 : 0, chunk_len);
        else launch_partial<4, 4>(s, counts, chunk_cap, n, row_ptr, col_idx, val, B, ldb, logG, hub_row, hub_chunk0, chunk_hub, part, ldp, agg, hub_cap, relu_in ? 1 : 0, chunk_len);
    } else {
        if (iters <= 1) launch_partial<1, 1>(s, counts, chunk_cap, n, row_ptr, col_idx, val, B, ldb, logG, hub_row, hub_chunk0, chunk_hub, part, ldp, agg, hub_cap, relu_in ? 1 : 0, chunk_len);
        else if (iters == 2) launch_partial<1, 2>(s, counts, chunk_cap, n, row_ptr, col_idx, val, B, ldb, logG, hub_row, hub_chunk0, chunk_hub, part, ldp, agg, hub_cap, relu_in ? 1 : 0, chunk_len);
        else launch_partial<1, 4>(s, counts, chunk_cap, n, row_ptr, col_idx, val, B, ldb, logG, hub_row, hub_chunk0, chunk_hub, part, ldp, agg, hub_cap, relu_in ? 1 : 0, chunk_len);
    }
    GNNHIP_LAUNCH_CHECK("hub_prepass");
    plan->row_slot = row_slot;
    plan->agg = agg;
    plan->ld = ldp;
    return GNNHIP_OK;
}

}  // namespace gnnhip
