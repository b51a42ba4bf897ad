// Device-side grouping of (key, payload) pairs into CSR, and CSR transposition.
//
// graphnn builds the CSR operands of a batch on the host by walking per-node lists
// (src/nn/msg_pass.cpp:46-177); row i of such a matrix lists the payloads of the pairs
// whose key is i, in insertion order.  That is a stable sort of the pair indices by key.
// Here: a least-significant-digit radix sort (8-bit digits, as many passes as the key range
// needs) whose every pass is stable, then the row pointers from the sorted keys.
//
// One pass over n pairs, tiles of 2048 pairs per workgroup:
//   histogram   per tile, 256 LDS counters -> hist[digit][tile]
//   scan        exclusive scan of hist in digit-major order (three launches, any length)
//   scatter     a wavefront takes 512 consecutive pairs of the tile, 64 at a time; lanes with
//               the same digit find each other with eight ballots, their rank is the running
//               count of that digit in the wavefront's segment plus the number of lower lanes;
//               segment counts are then prefixed over the four wavefronts.  Destination =
//               scanned hist[digit][tile] + rank.  Order inside a digit = input order: stable.
// No atomics on global memory; the result is a pure function of the input.
#include "gnnhip_internal.h"

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kItems = 8;
constexpr int kTile = kBlock * kItems;          // 2048 pairs per workgroup
constexpr int kSeg = kTile / kWavesPerBlock;    // 512 consecutive pairs per wavefront
constexpr int kDigits = 256;

__global__ __launch_bounds__(kBlock) void radix_hist_kernel(const unsigned* __restrict__ keys, long long n, int shift,
                                                             int ntiles, int* __restrict__ hist)
{
    __shared__ int h[kDigits];
    h[threadIdx.x] = 0;
    __syncthreads();
    const long long base = (long long)blockIdx.x * kTile;
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
        const long long idx = base + i * kBlock + threadIdx.x;
        if (idx < n) atomicAdd(&h[(keys[idx] >> shift) & (kDigits - 1)], 1);
    }
    __syncthreads();
    hist[(size_t)threadIdx.x * ntiles + blockIdx.x] = h[threadIdx.x];
}

// ---- exclusive scan of an int array of any length: segment sums, scan of the sums, apply
constexpr int kScanSeg = 4096;                  // elements per workgroup: 256 lanes x 16
__device__ __forceinline__ int block_scan_256(int v, int* sh, int* total)
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

__global__ __launch_bounds__(kBlock) void scan_segment_sums_kernel(const int* __restrict__ x, long long n, int* __restrict__ seg_sum)
{
    __shared__ int sh[kWavesPerBlock];
    const long long base = (long long)blockIdx.x * kScanSeg + threadIdx.x * 16;
    int s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) if (base + i < n) s += x[base + i];
    int tot;
    block_scan_256(s, sh, &tot);
    if (threadIdx.x == 0) seg_sum[blockIdx.x] = tot;
}

// one workgroup: exclusive scan of nseg values in place; total to *total_out (may be null)
__global__ __launch_bounds__(1024) void scan_small_kernel(int* __restrict__ x, int nseg, int* __restrict__ total_out)
{
    __shared__ int wave_tot[1024 / kWave];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int per = (nseg + 1023) / 1024;
    const int lo = min(tid * per, nseg), hi = min(lo + per, nseg);
    int local = 0;
    for (int i = lo; i < hi; ++i) local += x[i];
    int incl = local;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int o = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += o;
    }
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += wave_tot[w];
    int run = base + incl - local;
    for (int i = lo; i < hi; ++i) { const int v = x[i]; x[i] = run; run += v; }
    if (tid == 1023 && total_out) *total_out = run;
}

__global__ __launch_bounds__(kBlock) void scan_apply_kernel(int* __restrict__ x, long long n, const int* __restrict__ seg_off)
{
    __shared__ int sh[kWavesPerBlock];
    const long long base = (long long)blockIdx.x * kScanSeg + threadIdx.x * 16;
    int v[16];
    int s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) { v[i] = (base + i < n) ? x[base + i] : 0; s += v[i]; }
    int tot;
    int run = seg_off[blockIdx.x] + block_scan_256(s, sh, &tot);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        if (base + i < n) x[base + i] = run;
        run += v[i];
    }
}

}  // namespace

// seg_scratch: at least ceil(n / 4096) ints.  n <= 4096 * 2^22 (the small scan handles what one
// workgroup walks comfortably; far beyond every use here).
int exclusive_scan_i32(int* x, long long n, int* seg_scratch, hipStream_t s)
{
    if (n <= 0) return GNNHIP_OK;
    const int nseg = (int)((n + kScanSeg - 1) / kScanSeg);
    hipLaunchKernelGGL(scan_segment_sums_kernel, dim3(nseg), dim3(kBlock), 0, s, x, n, seg_scratch);
    hipLaunchKernelGGL(scan_small_kernel, dim3(1), dim3(1024), 0, s, seg_scratch, nseg, (int*)nullptr);
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nseg), dim3(kBlock), 0, s, x, n, seg_scratch);
    GNNHIP_LAUNCH_CHECK("exclusive_scan_i32");
    return GNNHIP_OK;
}

namespace {

__global__ __launch_bounds__(kBlock) void radix_scatter_kernel(
    const unsigned* __restrict__ keys, const unsigned* __restrict__ vals, long long n, int shift, int ntiles,
    const int* __restrict__ hist_scanned, unsigned* __restrict__ keys_out, unsigned* __restrict__ vals_out, int first_pass)
{
    __shared__ int cnt[kWavesPerBlock][kDigits];      // running, then total, count of each digit per wavefront segment
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    for (int i = threadIdx.x; i < kWavesPerBlock * kDigits; i += kBlock) (&cnt[0][0])[i] = 0;
    __syncthreads();

    const long long seg0 = (long long)blockIdx.x * kTile + wave * kSeg;
    unsigned k[kItems], v[kItems];
    int rank[kItems];
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (kWave - lane));
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
        const long long idx = seg0 + i * kWave + lane;
        const bool live = idx < n;
        k[i] = live ? keys[idx] : 0u;
        v[i] = live ? (first_pass ? (unsigned)idx : vals[idx]) : 0u;
        const unsigned d = (k[i] >> shift) & (kDigits - 1);
        // lanes of this round with the same digit (dead lanes match nobody)
        unsigned long long same = __ballot(live);
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const unsigned long long bal = __ballot((d >> b) & 1u);
            same &= ((d >> b) & 1u) ? bal : ~bal;
        }
        int r = 0;
        if (live) {
            const int before = cnt[wave][d];                       // every lane of the group reads before its leader writes
            r = before + __popcll(same & below);
            if ((same & below) == 0) cnt[wave][d] = before + __popcll(same);
        }
        rank[i] = r;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    }
    __syncthreads();
    // prefix of the segment counts over the wavefronts, per digit (lane t handles digit t)
    {
        const int d = threadIdx.x;
        int run = 0;
#pragma unroll
        for (int w = 0; w < kWavesPerBlock; ++w) { const int c = cnt[w][d]; cnt[w][d] = run; run += c; }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kItems; ++i) {
        const long long idx = seg0 + i * kWave + lane;
        if (idx < n) {
            const unsigned d = (k[i] >> shift) & (kDigits - 1);
            const long long dst = (long long)hist_scanned[(size_t)d * ntiles + blockIdx.x] + cnt[wave][d] + rank[i];
            keys_out[dst] = k[i];
            vals_out[dst] = v[i];
        }
    }
}

// keys as unsigned, forced into [0, rows): a key outside that range is a caller error, but it must not
// send the row-pointer kernels out of bounds
__global__ __launch_bounds__(kBlock) void gather_strided_kernel(const int* __restrict__ src, int stride, long long n, int rows,
                                                                 unsigned* __restrict__ dst)
{
    const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) dst[i] = (unsigned)min(max(src[i * stride], 0), rows - 1);
}

// row_ptr from the sorted keys: position i opens every row in (key[i-1], key[i]]; the last position closes the rest
__global__ __launch_bounds__(kBlock) void row_ptr_from_sorted_kernel(const unsigned* __restrict__ keys, long long n, int rows, int* __restrict__ row_ptr)
{
    const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (n == 0) {
        for (long long r = i; r <= rows; r += (long long)gridDim.x * kBlock) row_ptr[r] = 0;
        return;
    }
    if (i >= n) return;
    const long long k = keys[i];
    const long long kprev = (i == 0) ? -1 : (long long)keys[i - 1];
    for (long long r = kprev + 1; r <= k; ++r) row_ptr[r] = (int)i;
    if (i == n - 1)
        for (long long r = k + 1; r <= rows; ++r) row_ptr[r] = (int)n;
}

__global__ __launch_bounds__(kBlock) void fill_grouped_kernel(const unsigned* __restrict__ keys_sorted, const unsigned* __restrict__ perm,
                                                               long long n, const int* __restrict__ payload, int stride,
                                                               const float* __restrict__ val_in, int average,
                                                               const int* __restrict__ row_ptr, int* __restrict__ col_idx, float* __restrict__ val)
{
    const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const unsigned src = perm[i];
    col_idx[i] = payload[(long long)src * stride];
    float w = val_in ? val_in[src] : 1.0f;
    if (average) {
        const unsigned r = keys_sorted[i];
        w = (float)(1.0 / (double)(row_ptr[r + 1] - row_ptr[r]));      // as the reference: double divide, then narrowed
    }
    val[i] = w;
}

// row index of every entry of a CSR matrix
__global__ __launch_bounds__(kBlock) void expand_rows_kernel(int m, const int* __restrict__ row_ptr, int* __restrict__ row_of)
{
    const int lane = threadIdx.x & (kWave - 1);
    const long long row = ((long long)blockIdx.x * kBlock + threadIdx.x) / kWave;
    if (row >= m) return;
    const int a = row_ptr[row], b = row_ptr[row + 1];
    for (int t = a + lane; t < b; t += kWave) row_of[t] = (int)row;
}

// ---- small inputs: the whole grouping in one launch ----
// A batch of a few hundred small graphs is latency, not bandwidth: the dozen launches of the radix passes
// cost more than the host loop they replace.  One launch of up to 16 workgroups instead.  The rows are cut
// into as many runs; every workgroup reads ALL keys (they are a few L2 lines per lane) and keeps the pairs
// of its own run of rows, so no workgroup ever waits for another: the number of keys below its first row,
// which it counts on the way, is where its part of the result starts.  Between the first read of the keys
// and the last write of the result everything is in LDS:
//   lengths    LDS counters (atomics), the pairs below the run, and a check whether the keys already ascend
//   scan       row_ptr; the counters become cursors
//   place      every pair takes the next slot of its row in whatever order the hardware serves the
//              atomics; the slot (16 bits, in LDS) keeps the pair's INDEX, so that the next step can put
//              every row into input order again.  Ascending keys: the pairs of the run are consecutive
//              and in order already, nothing to place or to order.
//   order      rows of up to 8 entries: a thread sorts them in registers (a fixed network);
//              longer rows: a wavefront marks the row's pair indices in a bitmap of its own and reads
//              the set bits back in ascending order, 64 words at a time (a prefix sum of the
//              population counts gives every word its first slot)
//   write      slot after slot, coalesced: payload (and value) of the pair the slot names
// Global loads are issued sixteen to a thread before the first is used.  The order of the entries is a
// pure function of the input, as on the radix route.  Sizes: 4 bytes per row of a run, 2 per pair, one
// bitmap of n bits (as many as fit, up to one per wavefront) in 160 KB of LDS; at most 65,536 pairs.
constexpr int kSmallPairs = 1 << 16;
constexpr int kSmallBlock = 1024;
constexpr int kSmallWaves = kSmallBlock / kWave;
constexpr int kSmallShort = 8;
constexpr int kSmallBatch = 16;
constexpr int kSmallLdsInts = 160 * 1024 / 4;
constexpr int kSmallMisc = 48;
constexpr int kSmallGroups = 16;           // workgroups at most
constexpr int kSmallRunRows = 256;         // rows per workgroup at least

struct SmallLayout {
    int groups, run;                      // workgroups, rows per workgroup (a multiple of 64)
    int slots, longs, misc, bitmaps;      // offsets in ints (the counters start at 0)
    int words, nbitmaps;                  // words per bitmap, number of bitmaps
};
// false: the input does not fit the workgroups' LDS
inline bool small_layout(long long rows, long long n, SmallLayout* out)
{
    if (n < 1 || n > kSmallPairs || rows < 1) return false;
    SmallLayout l;
    long long groups = (rows + kSmallRunRows - 1) / kSmallRunRows;
    if (groups > kSmallGroups) groups = kSmallGroups;
    const long long run = ((rows + groups - 1) / groups + kWave - 1) / kWave * kWave;
    if (run > kSmallLdsInts) return false;
    l.run = (int)run;
    l.groups = (int)((rows + run - 1) / run);
    l.slots = l.run;
    l.longs = l.slots + (int)((n + 1) / 2);
    l.misc = l.longs + (int)((n / (kSmallShort + 1) + 2) / 2);
    l.bitmaps = l.misc + kSmallMisc;
    l.words = (int)((n + 31) / 32);
    const int room = kSmallLdsInts - l.bitmaps;
    if (room < l.words) return false;
    l.nbitmaps = room / l.words < kSmallWaves ? room / l.words : kSmallWaves;
    *out = l;
    return true;
}

// inclusive prefix sum over the wavefront: shifts inside the rows of 16 lanes (lanes without a source add 0),
// then the totals of the rows below
__device__ __forceinline__ int wave_inclusive_scan_i(int v)
{
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, true);      // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, true);      // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, true);      // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, true);      // row_shr:8
    const int t0 = __builtin_amdgcn_readlane(v, 15), t1 = __builtin_amdgcn_readlane(v, 31), t2 = __builtin_amdgcn_readlane(v, 47);
    const int row = (threadIdx.x & (kWave - 1)) >> 4;
    return v + (row >= 1 ? t0 : 0) + (row >= 2 ? t1 : 0) + (row >= 3 ? t2 : 0);
}

__device__ __forceinline__ void order_pair(int& a, int& b)
{
    const int lo = min(a, b), hi = max(a, b);
    a = lo;
    b = hi;
}

// One grouping of the n pairs.  A launch carries one or two of them (the same pairs grouped by either member:
// a matrix and its transpose); workgroup b works on job b / groups.
struct SmallJob {
    const int* key;
    const int* payload;
    const float* val_in;
    int* row_ptr;
    int* col_idx;
    float* val;
    int key_stride, payload_stride;
};

__global__ __launch_bounds__(kSmallBlock) void csr_group_small_kernel(int rows, int n, SmallLayout lay, SmallJob job0, SmallJob job1, int average)
{
    const bool second = (int)blockIdx.x >= lay.groups;
    const int run_index = (int)blockIdx.x - (second ? lay.groups : 0);
    const int* __restrict__ key = second ? job1.key : job0.key;
    const int* __restrict__ payload = second ? job1.payload : job0.payload;
    const float* __restrict__ val_in = second ? job1.val_in : job0.val_in;
    int* __restrict__ row_ptr = second ? job1.row_ptr : job0.row_ptr;
    int* __restrict__ col_idx = second ? job1.col_idx : job0.col_idx;
    float* __restrict__ val = second ? job1.val : job0.val;
    const int key_stride = second ? job1.key_stride : job0.key_stride;
    const int payload_stride = second ? job1.payload_stride : job0.payload_stride;
    extern __shared__ int small_lds[];
    int* cnt = small_lds;                          // one per row of this workgroup's run
    unsigned short* slots = reinterpret_cast<unsigned short*>(small_lds + lay.slots);
    unsigned short* longs = reinterpret_cast<unsigned short*>(small_lds + lay.longs);       // rows of more than kSmallShort entries
    int* misc = small_lds + lay.misc;              // [0] long rows, [1] keys out of order, [2..17] wavefront totals, [18..33] pairs below
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const int uwave = __builtin_amdgcn_readfirstlane(wave);
    const int top = rows - 1;
    const int lo = run_index * lay.run, mine = min(lay.run, rows - lo);            // this run: rows lo .. lo + mine - 1

    for (int r = tid; r < mine; r += kSmallBlock) cnt[r] = 0;
    if (tid < kSmallMisc) misc[tid] = 0;
    __syncthreads();

    // lengths.  Lanes hold consecutive pairs; a run of equal keys (a batch that arrives grouped is nothing
    // else) is counted by its first lane alone.  The keys of the first batch stay in registers for `place`.
    bool disorder = false;
    int below = 0;
    int first_keys[kSmallBatch];
    for (int base0 = 0; base0 < n; base0 += kSmallBlock * kSmallBatch) {       // every lane walks every batch: the ballots need them
        const int base = base0 + tid;
        int k[kSmallBatch], before[kSmallBatch];
#pragma unroll
        for (int u = 0; u < kSmallBatch; ++u) {
            const int e = base + u * kSmallBlock;
            k[u] = e < n ? key[(long long)e * key_stride] : 0;
            before[u] = (e < n && e > 0 && lane == 0) ? key[(long long)(e - 1) * key_stride] : 0;
        }
#pragma unroll
        for (int u = 0; u < kSmallBatch; ++u) {
            const int e = base + u * kSmallBlock;
            const int kk = e < n ? min(max(k[u], 0), top) : -1;
            if (base0 == 0) first_keys[u] = kk;
            const int left = __shfl_up(kk, 1, kWave);
            const int prev = lane == 0 ? (e > 0 && e < n ? min(max(before[u], 0), top) : -1) : left;
            const bool head = lane == 0 || left != kk;
            const unsigned long long heads = __ballot(head);
            if (kk >= 0) {
                disorder |= prev > kk;
                below += kk < lo;
                if (head && kk >= lo && kk - lo < mine) {
                    const unsigned long long later = lane == kWave - 1 ? 0ull : heads >> (lane + 1);
                    atomicAdd(&cnt[kk - lo], later ? __ffsll((long long)later) : kWave - lane);
                }
            }
        }
    }
    if (disorder) misc[1] = 1;
    below = wave_sum_i(below);
    if (lane == 0) misc[18 + uwave] = below;
    __syncthreads();

    // exclusive scan: a wavefront owns a stretch of the run and walks it 64 rows at a time
    const int seg = ((mine + kSmallWaves - 1) / kSmallWaves + kWave - 1) & ~(kWave - 1);
    const int s0 = min(uwave * seg, mine), s1 = min(s0 + seg, mine);
    int part = 0;
    for (int r = s0 + lane; r < s1; r += kWave) part += cnt[r];
    part = wave_sum_i(part);
    if (lane == 0) misc[2 + uwave] = part;
    __syncthreads();
    const int upto = wave_inclusive_scan_i(lane < kSmallWaves ? misc[2 + lane] : 0);
    const int first_slot = wave_sum_i(lane < kSmallWaves ? misc[18 + lane] : 0);      // pairs of the runs before this one
    const int held = __builtin_amdgcn_readlane(upto, kSmallWaves - 1);                 // pairs of this run
    int carry = uwave ? __builtin_amdgcn_readlane(upto, uwave - 1) : 0;
    for (int r = s0 + lane; r - lane < s1; r += kWave) {
        const int c = r < s1 ? cnt[r] : 0;
        const int through = wave_inclusive_scan_i(c);
        if (r < s1) cnt[r] = carry + through - c;
        carry += __builtin_amdgcn_readlane(through, kWave - 1);
    }
    const bool ascending = misc[1] == 0;
    __syncthreads();
    for (int r = tid; r < mine; r += kSmallBlock) row_ptr[lo + r] = first_slot + cnt[r];
    if (lo + mine == rows && tid == 0) row_ptr[rows] = n;

    if (!ascending) {
        __syncthreads();                  // the starts are on their way out; the counters turn into cursors
#pragma unroll
        for (int u = 0; u < kSmallBatch; ++u) {
            const int e = tid + u * kSmallBlock, r = first_keys[u] - lo;
            if (e < n && r >= 0 && r < mine) slots[atomicAdd(&cnt[r], 1)] = (unsigned short)e;
        }
        for (int base = tid + kSmallBlock * kSmallBatch; base < n; base += kSmallBlock * kSmallBatch) {
            int k[kSmallBatch];
#pragma unroll
            for (int u = 0; u < kSmallBatch; ++u) {
                const int e = base + u * kSmallBlock;
                k[u] = e < n ? key[(long long)e * key_stride] : 0;
            }
#pragma unroll
            for (int u = 0; u < kSmallBatch; ++u) {
                const int e = base + u * kSmallBlock, r = min(max(k[u], 0), top) - lo;
                if (e < n && r >= 0 && r < mine) slots[atomicAdd(&cnt[r], 1)] = (unsigned short)e;
            }
        }
        __syncthreads();                  // cnt[r] is now the end of row r

        for (int r0 = 0; r0 < mine; r0 += kSmallBlock) {
            const int r = r0 + tid;
            int a = 0, len = 0;
            if (r < mine) {
                a = r ? cnt[r - 1] : 0;
                len = cnt[r] - a;
            }
            if (len > kSmallShort) {
                longs[atomicAdd(&misc[0], 1)] = (unsigned short)r;
                len = 0;
            }
            if (__ballot(len >= 2) == 0ull) continue;
            if (__ballot(len > 4) == 0ull) {
                // nobody in this wavefront has more than 4: 5 exchanges order 4 values
                int v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = j < len ? (int)slots[a + j] : 0x7fffffff;
                order_pair(v[0], v[1]); order_pair(v[2], v[3]); order_pair(v[0], v[2]); order_pair(v[1], v[3]); order_pair(v[1], v[2]);
                if (len >= 2) {
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        if (j < len) slots[a + j] = (unsigned short)v[j];
                }
                continue;
            }
            int v[kSmallShort];
#pragma unroll
            for (int j = 0; j < kSmallShort; ++j) v[j] = j < len ? (int)slots[a + j] : 0x7fffffff;
            // 19 exchanges order 8 values
            order_pair(v[0], v[1]); order_pair(v[2], v[3]); order_pair(v[4], v[5]); order_pair(v[6], v[7]);
            order_pair(v[0], v[2]); order_pair(v[1], v[3]); order_pair(v[4], v[6]); order_pair(v[5], v[7]);
            order_pair(v[1], v[2]); order_pair(v[5], v[6]); order_pair(v[0], v[4]); order_pair(v[3], v[7]);
            order_pair(v[1], v[5]); order_pair(v[2], v[6]);
            order_pair(v[1], v[4]); order_pair(v[3], v[6]);
            order_pair(v[2], v[4]); order_pair(v[3], v[5]);
            order_pair(v[3], v[4]);
            if (len >= 2) {
#pragma unroll
                for (int j = 0; j < kSmallShort; ++j)
                    if (j < len) slots[a + j] = (unsigned short)v[j];
            }
        }
        __syncthreads();

        const int nlong = misc[0];
        if (nlong > 0 && wave < lay.nbitmaps) {
            unsigned* bits = reinterpret_cast<unsigned*>(small_lds + lay.bitmaps) + wave * lay.words;
            for (int i = lane; i < lay.words; i += kWave) bits[i] = 0u;
            for (int q = wave; q < nlong; q += lay.nbitmaps) {
                const int r = longs[q];
                const int a = r ? cnt[r - 1] : 0, b = cnt[r];
                int first = 0x7fffffff, last = -1;
                for (int i = a + lane; i < b; i += kWave) {
                    const int e = slots[i];
                    atomicOr(&bits[e >> 5], 1u << (e & 31));
                    first = min(first, e);
                    last = max(last, e);
                }
#pragma unroll
                for (int d = 1; d < kWave; d <<= 1) {
                    first = min(first, __shfl_xor(first, d, kWave));
                    last = max(last, __shfl_xor(last, d, kWave));
                }
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                __builtin_amdgcn_wave_barrier();
                const int last_word = last >> 5;
                int slot = a;
                for (int word0 = first >> 5; word0 <= last_word; word0 += kWave) {
                    const int word = word0 + lane;
                    unsigned m = 0u;
                    if (word <= last_word) {
                        m = bits[word];
                        bits[word] = 0u;
                    }
                    const int c = __popc(m);
                    const int through = wave_inclusive_scan_i(c);
                    int at = slot + through - c;
                    while (m) {
                        slots[at++] = (unsigned short)(word * 32 + (__ffs((int)m) - 1));
                        m &= m - 1u;
                    }
                    slot += __shfl(through, kWave - 1, kWave);
                }
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
        __syncthreads();
    }

    // slot i of this run holds pair e and is entry first_slot + i of the result: out it goes
    for (int base = tid; base < held; base += kSmallBlock * kSmallBatch) {
        int e[kSmallBatch], pay[kSmallBatch], k[kSmallBatch];
        float w[kSmallBatch];
#pragma unroll
        for (int u = 0; u < kSmallBatch; ++u) {
            const int i = base + u * kSmallBlock;
            e[u] = i < held ? (ascending ? first_slot + i : (int)slots[i]) : 0;
        }
#pragma unroll
        for (int u = 0; u < kSmallBatch; ++u) {
            const bool live = base + u * kSmallBlock < held;
            pay[u] = live ? payload[(long long)e[u] * payload_stride] : 0;
            w[u] = (live && val_in) ? val_in[e[u]] : 1.0f;
            k[u] = (live && average) ? key[(long long)e[u] * key_stride] : 0;
        }
#pragma unroll
        for (int u = 0; u < kSmallBatch; ++u) {
            const int i = base + u * kSmallBlock;
            if (i >= held) continue;
            if (average) {
                const int r = min(max(k[u], 0), top) - lo;
                const int len = ascending ? (r + 1 < mine ? cnt[r + 1] : held) - cnt[r] : cnt[r] - (r ? cnt[r - 1] : 0);
                w[u] = (float)(1.0 / (double)len);       // as the reference: double divide, then narrowed
            }
            col_idx[first_slot + i] = pay[u];
            val[first_slot + i] = w[u];
        }
    }
}

// col_idx[j] = j and val[j] = 1 (or 1 / row length) for j in [row_ptr[i], row_ptr[i+1]): a wavefront per row
// (row_ptr may be pinned host memory: then row_ptr_out, device memory, receives a copy for the kernels that follow)
__global__ __launch_bounds__(kBlock) void consecutive_rows_kernel(int rows, const int* __restrict__ row_ptr, int average,
                                                                  int* __restrict__ col_idx, float* __restrict__ val,
                                                                  int* __restrict__ row_ptr_out)
{
    const int lane = threadIdx.x & (kWave - 1);
    const long long row = ((long long)blockIdx.x * kBlock + threadIdx.x) / kWave;
    if (row >= rows) return;
    const int a = row_ptr[row], b = row_ptr[row + 1];
    if (row_ptr_out && lane == 0) {
        row_ptr_out[row] = a;
        if (row == rows - 1) row_ptr_out[rows] = b;
    }
    const float w = (average && b > a) ? (float)(1.0 / (double)(b - a)) : 1.0f;       // as the reference: double divide, then narrowed
    for (int j = a + lane; j < b; j += kWave) {
        col_idx[j] = j;
        val[j] = w;
    }
}

inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace

// One stable pass of the radix sort: perm_out[i] = index of the key that comes i-th when the n keys are ordered by
// the 8-bit digit (key >> shift) & 255 (equal digits keep their input order); keys_out receives the keys in that
// order.  With `carried`, perm_out[i] = carried[that index] instead (the order of an earlier pass carried along).
// hist needs radix_hist_ints(n) ints, seg radix_seg_ints(n).
size_t radix_hist_ints(long long n) { return (size_t)kDigits * (size_t)((n + kTile - 1) / kTile > 0 ? (n + kTile - 1) / kTile : 1); }
size_t radix_seg_ints(long long n) { return (radix_hist_ints(n) + kScanSeg - 1) / kScanSeg + 1; }
int radix_order_by_digit(const unsigned* keys, long long n, int shift, unsigned* keys_out, unsigned* perm_out, int* hist, int* seg,
                         hipStream_t s, const unsigned* carried)
{
    if (n <= 0) return GNNHIP_OK;
    const int ntiles = (int)((n + kTile - 1) / kTile);
    hipLaunchKernelGGL(radix_hist_kernel, dim3(ntiles), dim3(kBlock), 0, s, keys, n, shift, ntiles, hist);
    if (int rc = exclusive_scan_i32(hist, (long long)kDigits * ntiles, seg, s)) return rc;
    hipLaunchKernelGGL(radix_scatter_kernel, dim3(ntiles), dim3(kBlock), 0, s, keys, carried, n, shift, ntiles, hist,
                       keys_out, perm_out, carried ? 0 : 1);
    GNNHIP_LAUNCH_CHECK("radix_order_by_digit");
    return GNNHIP_OK;
}

// The one-launch grouping where it fits; false: it does not (nothing launched).  With t_row_ptr the same launch
// also groups the pairs by payload with the key as the payload: the transpose, its entries in pair order, values 1.
bool csr_group_small(int rows, long long n, const int* key, int key_stride, const int* payload, int payload_stride, const float* val_in,
                     int average, int* row_ptr, int* col_idx, float* val, int* t_row_ptr, int* t_col_idx, float* t_val, hipStream_t s)
{
    SmallLayout lay;
    if (!small_layout(rows, n, &lay)) return false;
    static LdsLimit limit;
    if (limit.raise(reinterpret_cast<const void*>(csr_group_small_kernel), sizeof(int) * kSmallLdsInts) != hipSuccess) return false;
    const SmallJob job0 = {key, payload, val_in, row_ptr, col_idx, val, key_stride, payload_stride};
    const SmallJob job1 = {payload, key, nullptr, t_row_ptr, t_col_idx, t_val, payload_stride, key_stride};
    hipLaunchKernelGGL(csr_group_small_kernel, dim3(lay.groups * (t_row_ptr ? 2 : 1)), dim3(kSmallBlock),
                       sizeof(int) * (size_t)(lay.bitmaps + lay.words * lay.nbitmaps), s, rows, (int)n, lay, job0, job1, average);
    return true;
}

inline int last_launch_status(const char* what)
{
    GNNHIP_LAUNCH_CHECK(what);
    return GNNHIP_OK;
}

// Groups n pairs by key (0 <= key < rows) keeping input order inside a group:
//   row_ptr[rows + 1], col_idx[i] = payload of the i-th pair in grouped order,
//   val[i] = val_in of that pair (or 1), or 1 / group size when average is set.
// key / payload are read with the given strides (in ints).  Uses scratch slot 0 of the stream.
int csr_group_pairs(int rows, long long n, const int* key, int key_stride, const int* payload, int payload_stride,
                    const float* val_in, int average, int* row_ptr, int* col_idx, float* val, hipStream_t s)
{
    if (csr_group_small(rows, n, key, key_stride, payload, payload_stride, val_in, average, row_ptr, col_idx, val, nullptr, nullptr, nullptr, s))
        return last_launch_status("csr_group_small");
    const int ntiles = (int)((n + kTile - 1) / kTile);
    const long long nhist = (long long)kDigits * (ntiles > 0 ? ntiles : 1);
    size_t off = 0;
    auto carve = [&](size_t bytes) { const size_t o = off; off = round_up(off + bytes, 256); return o; };
    const size_t o_k0 = carve(sizeof(unsigned) * (size_t)(n > 0 ? n : 1)), o_k1 = carve(sizeof(unsigned) * (size_t)(n > 0 ? n : 1));
    const size_t o_v0 = carve(sizeof(unsigned) * (size_t)(n > 0 ? n : 1)), o_v1 = carve(sizeof(unsigned) * (size_t)(n > 0 ? n : 1));
    const size_t o_hist = carve(sizeof(int) * (size_t)nhist);
    const size_t o_seg = carve(sizeof(int) * (size_t)((nhist + kScanSeg - 1) / kScanSeg + 1));
    void* base = nullptr;
    if (int rc = stream_scratch(s, off, &base)) return rc;
    char* b = static_cast<char*>(base);
    unsigned* k0 = reinterpret_cast<unsigned*>(b + o_k0);
    unsigned* k1 = reinterpret_cast<unsigned*>(b + o_k1);
    unsigned* v0 = reinterpret_cast<unsigned*>(b + o_v0);
    unsigned* v1 = reinterpret_cast<unsigned*>(b + o_v1);
    int* hist = reinterpret_cast<int*>(b + o_hist);
    int* seg = reinterpret_cast<int*>(b + o_seg);

    const unsigned egrid = (unsigned)((n + kBlock - 1) / kBlock);
    if (n > 0) {
        hipLaunchKernelGGL(gather_strided_kernel, dim3(egrid), dim3(kBlock), 0, s, key, key_stride, n, rows, k0);
        int bits = 1;
        while (bits < 31 && (1ll << bits) < (long long)rows) ++bits;
        bool first = true;
        for (int shift = 0; shift < bits; shift += 8) {
            hipLaunchKernelGGL(radix_hist_kernel, dim3(ntiles), dim3(kBlock), 0, s, k0, n, shift, ntiles, hist);
            if (int rc = exclusive_scan_i32(hist, nhist, seg, s)) return rc;
            hipLaunchKernelGGL(radix_scatter_kernel, dim3(ntiles), dim3(kBlock), 0, s, k0, v0, n, shift, ntiles, hist, k1, v1, first ? 1 : 0);
            unsigned* t = k0; k0 = k1; k1 = t;
            t = v0; v0 = v1; v1 = t;
            first = false;
        }
    }
    const unsigned rgrid = n > 0 ? egrid : (unsigned)(((long long)rows + kBlock) / kBlock);
    hipLaunchKernelGGL(row_ptr_from_sorted_kernel, dim3(rgrid), dim3(kBlock), 0, s, k0, n, rows, row_ptr);
    if (n > 0)
        hipLaunchKernelGGL(fill_grouped_kernel, dim3(egrid), dim3(kBlock), 0, s, k0, v0, n, payload, payload_stride, val_in, average,
                           row_ptr, col_idx, val);
    GNNHIP_LAUNCH_CHECK("csr_group_pairs");
    return GNNHIP_OK;
}

}  // namespace gnnhip

using namespace gnnhip;

extern "C" {

int gnnhip_csr_group_i32(int rows, int n, const int* key, int key_stride, const int* payload, int payload_stride,
                         int average, int* row_ptr, int* col_idx, float* val, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && n >= 0 && key_stride >= 1 && payload_stride >= 1, "bad shape in csr_group (rows=%d n=%d)", rows, n);
    GNNHIP_REQUIRE(row_ptr != nullptr, "null row_ptr in csr_group");
    GNNHIP_REQUIRE(n == 0 || (key && payload && col_idx && val), "null array in csr_group");
    GNNHIP_REQUIRE(n == 0 || rows >= 1, "pairs but no rows in csr_group");
    if (int rc = require_ready()) return rc;
    return csr_group_pairs(rows, n, key, key_stride, payload, payload_stride, nullptr, average, row_ptr, col_idx, val, as_stream(stream));
}

int gnnhip_csr_consecutive_rows_f32(int rows, const int* row_ptr, int average, int* col_idx, float* val, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0, "negative row count in csr_consecutive_rows");
    if (rows == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(row_ptr && col_idx && val, "null array in csr_consecutive_rows");
    if (int rc = require_ready()) return rc;
    const unsigned grid = (unsigned)(((long long)rows * kWave + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(consecutive_rows_kernel, dim3(grid), dim3(kBlock), 0, as_stream(stream), rows, row_ptr, average, col_idx, val,
                       static_cast<int*>(nullptr));
    GNNHIP_LAUNCH_CHECK("consecutive_rows");
    return GNNHIP_OK;
}

int gnnhip_csr_consecutive_rows_host_f32(int rows, const int* offsets_host, int average, int* row_ptr, int* col_idx, float* val, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0, "negative row count in csr_consecutive_rows_host");
    GNNHIP_REQUIRE(offsets_host && row_ptr, "null row pointers in csr_consecutive_rows_host");
    GNNHIP_REQUIRE(offsets_host[rows] == 0 || (col_idx && val), "null array in csr_consecutive_rows_host");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    const void* pinned = nullptr;
    if (rows > 0 && offsets_host[rows] > 0)
        if (int rc = stage_in_pinned(s, offsets_host, sizeof(int) * ((size_t)rows + 1), &pinned)) return rc;
    if (!pinned) {
        if (int rc = gnnhip_memcpy_h2d(row_ptr, offsets_host, sizeof(int) * ((size_t)rows + 1), stream)) return rc;
        return (rows > 0 && offsets_host[rows] > 0) ? gnnhip_csr_consecutive_rows_f32(rows, row_ptr, average, col_idx, val, stream) : GNNHIP_OK;
    }
    const unsigned grid = (unsigned)(((long long)rows * kWave + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(consecutive_rows_kernel, dim3(grid), dim3(kBlock), 0, s, rows, static_cast<const int*>(pinned), average, col_idx, val,
                       row_ptr);
    GNNHIP_LAUNCH_CHECK("consecutive_rows");
    return GNNHIP_OK;
}

int gnnhip_csr_group_both_i32(int rows, int n, const int* x, int x_stride, const int* y, int y_stride,
                              int* row_ptr, int* col_idx, float* val, int* t_row_ptr, int* t_col_idx, float* t_val, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && n >= 0 && x_stride >= 1 && y_stride >= 1, "bad shape in csr_group_both (rows=%d n=%d)", rows, n);
    GNNHIP_REQUIRE(row_ptr && t_row_ptr, "null row pointers in csr_group_both");
    GNNHIP_REQUIRE(n == 0 || (x && y && col_idx && val && t_col_idx && t_val), "null array in csr_group_both");
    GNNHIP_REQUIRE(n == 0 || rows >= 1, "pairs but no rows in csr_group_both");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    if (csr_group_small(rows, n, y, y_stride, x, x_stride, nullptr, 0, row_ptr, col_idx, val, t_row_ptr, t_col_idx, t_val, s))
        return last_launch_status("csr_group_small");
    if (int rc = csr_group_pairs(rows, n, y, y_stride, x, x_stride, nullptr, 0, row_ptr, col_idx, val, s)) return rc;
    return csr_group_pairs(rows, n, x, x_stride, y, y_stride, nullptr, 0, t_row_ptr, t_col_idx, t_val, s);
}

int gnnhip_csr_transpose_f32(int m, int k, int nnz, const int* row_ptr, const int* col_idx, const float* val,
                             int* t_row_ptr, int* t_col_idx, float* t_val, void* stream)
{
    GNNHIP_REQUIRE(m >= 0 && k >= 0 && nnz >= 0, "bad shape in csr_transpose (m=%d k=%d nnz=%d)", m, k, nnz);
    GNNHIP_REQUIRE(row_ptr && t_row_ptr, "null row pointers in csr_transpose");
    GNNHIP_REQUIRE(nnz == 0 || (col_idx && val && t_col_idx && t_val), "null array in csr_transpose");
    GNNHIP_REQUIRE(nnz == 0 || k >= 1, "entries but no columns in csr_transpose");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    int* row_of = nullptr;
    if (nnz > 0) {
        // the row index of every entry lives in plan scratch (slot 1); the sort itself uses slot 0
        void* p = nullptr;
        if (int rc = stream_scratch_slot(s, 1, sizeof(int) * (size_t)nnz, &p)) return rc;
        row_of = static_cast<int*>(p);
        const unsigned grid = (unsigned)(((long long)m * kWave + kBlock - 1) / kBlock);
        if (m > 0) hipLaunchKernelGGL(expand_rows_kernel, dim3(grid), dim3(kBlock), 0, s, m, row_ptr, row_of);
    }
    return csr_group_pairs(k, nnz, col_idx, 1, row_of, 1, val, 0, t_row_ptr, t_col_idx, t_val, s);
}

}  // extern "C"
