// Row, jagged and global reductions for gfx950, built on the wave64 DPP/shuffle
// primitives of gnnhip_internal.h: row softmax, jagged softmax, global
// sum/mean/max, dense and CSR row arg-max, cross-entropy and in-top-k.
// One wavefront owns one row (or segment): 64 lanes stride the row with
// coalesced loads and combine with a DPP butterfly, replacing the thread-0
// serial loops of cunn_SoftMax_updateOutput_kernel
// (src/tensor/gpu_dense_tensor.cu:298-370) and the 256-lane shared-memory tree
// of MatColReduceKernel (include/tensor/gpu_reduce_kernel.h:57-99).
// All of these are HBM-bound: 8 bytes per element for the in-place softmaxes,
// 4 bytes per element for the reductions.
#include "gnnhip_internal.h"

#include <mutex>

namespace gnnhip {
namespace {

// Segment offsets of the jagged softmax entry point that allocates nothing: one copy of this array per
// GPU, held from the moment the library is loaded until the process ends (256 KiB + 4 B).  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels receive the address that call
// returns on the current device.
constexpr int kStaticMaxSegments = 65536;
static __device__ __align__(256) int scratch[kStaticMaxSegments + 1];

constexpr int kMaxDevices = 64;
std::mutex g_static_mu;
int* g_static_offsets[kMaxDevices] = {};          // device address of `scratch` on each GPU, filled on first use

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

// ---- softmax of one contiguous run by one wavefront (all 64 lanes call this)
// Runs of up to kWave * kSoftmaxRegs elements are read once and kept in registers (one read and one write
// per element instead of three reads and two writes, all loads of a lane in flight together); the arithmetic
// and its order are those of the strided loops below.
constexpr int kSoftmaxRegs = 16;
__device__ __forceinline__ void wave_softmax_inplace(float* x, long long len, int lane)
{
    if (len <= 0) return;
    if (len <= kWave * kSoftmaxRegs) {
        const int n = (int)len;
        const float first = x[0];                     // reference scan starts at element 0
        float v[kSoftmaxRegs];
#pragma unroll
        for (int k = 0; k < kSoftmaxRegs; ++k) {
            const int j = lane + k * kWave;
            v[k] = j < n ? x[j] : first;              // the filler cannot change the maximum
        }
        float mx = first;
#pragma unroll
        for (int k = 0; k < kSoftmaxRegs; ++k) mx = max_keep(mx, v[k]);
        mx = wave_max(mx);
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < kSoftmaxRegs; ++k) {
            if (lane + k * kWave < n) {
                v[k] = expf(v[k] - mx);
                s += v[k];
            }
        }
        s = wave_sum(s);
#pragma unroll
        for (int k = 0; k < kSoftmaxRegs; ++k)
            if (lane + k * kWave < n) x[lane + k * kWave] = v[k] / s;
        return;
    }
    float mx = x[0];                                  // reference scan starts at element 0
    for (long long j = lane; j < len; j += kWave) mx = max_keep(mx, x[j]);
    mx = wave_max(mx);
    float s = 0.f;
    for (long long j = lane; j < len; j += kWave) {
        const float e = expf(x[j] - mx);
        x[j] = e;
        s += e;
    }
    s = wave_sum(s);
    for (long long j = lane; j < len; j += kWave) x[j] = x[j] / s;
}

__global__ __launch_bounds__(kBlock) void row_softmax_kernel(float* x, int rows, int cols)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows; r += (long long)gridDim.x * kWavesPerBlock)
        wave_softmax_inplace(x + (size_t)r * cols, cols, lane);
}

// ---- exclusive scan of lens[nseg] into off[nseg+1] by one workgroup of 1024 lanes
constexpr int kScanBlock = 1024;
__global__ __launch_bounds__(kScanBlock) void exclusive_scan_kernel(const int* __restrict__ lens, int nseg, int* __restrict__ off)
{
    __shared__ int wave_tot[kScanBlock / kWave];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int chunk = (nseg + kScanBlock - 1) / kScanBlock;
    const int lo = min(tid * chunk, nseg), hi = min(lo + chunk, nseg);
    int local = 0;
    for (int i = lo; i < hi; ++i) local += lens[i];
    // inclusive scan across the wavefront
    int incl = local;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const int o = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += o;
    }
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    int wave_base = 0;
    for (int w = 0; w < wave; ++w) wave_base += wave_tot[w];
    int run = wave_base + incl - local;               // exclusive prefix of this lane's chunk
    for (int i = lo; i < hi; ++i) { off[i] = run; run += lens[i]; }
    if (tid == kScanBlock - 1) off[nseg] = run;
}

__global__ __launch_bounds__(kBlock) void jagged_softmax_kernel(float* x, const int* __restrict__ off, int nseg)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    for (long long s = (long long)blockIdx.x * kWavesPerBlock + wave; s < nseg; s += (long long)gridDim.x * kWavesPerBlock) {
        const int a = off[s], b = off[s + 1];
        wave_softmax_inplace(x + a, b - a, lane);
    }
}

// The same in one launch for a few thousand segments: every workgroup adds up the lengths ahead of its own
// segments itself (a few KB from L2) instead of waiting for a scan launch (4,096 segments of 1,024: 14 -> 9 us).
// A workgroup takes the kWavesPerBlock consecutive segments starting at blockIdx.x * kWavesPerBlock.
constexpr int kFusedJaggedMaxSegments = 8192;
__global__ __launch_bounds__(kBlock) void jagged_softmax_fused_kernel(float* x, const int* __restrict__ lens, int nseg)
{
    __shared__ long long wave_part[kWavesPerBlock];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int first = (int)blockIdx.x * kWavesPerBlock;
    long long local = 0;
    for (int i = threadIdx.x; i < first; i += kBlock) local += lens[i];
    // (lengths are ints, their sum may pass 2^31: two 32-bit halves through the integer reduction)
    const unsigned lo = (unsigned)(local & 0xFFFFFFFFll);
    const int hi = (int)(local >> 32);
    // sums of the low halves can carry: reduce 16-bit pieces so that nothing overflows an int
    const int p0 = wave_sum_i((int)(lo & 0xFFFFu)), p1 = wave_sum_i((int)(lo >> 16)), p2 = wave_sum_i(hi);
    if (lane == 0) wave_part[wave] = (long long)p0 + ((long long)p1 << 16) + ((long long)p2 << 32);
    __syncthreads();
    long long base = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) base += wave_part[w];
    const int seg = first + wave;
    if (seg >= nseg) return;
    for (int w = 0; w < wave; ++w) base += lens[first + w];
    wave_softmax_inplace(x + base, lens[seg], lane);
}

// ---- gradient of the jagged softmax: per segment z = <grad, out>, dst += (grad - z) * out
//      (the CPU rule, src/nn/jagged_softmax.cpp:8-31; graphnn's GPU overload is an empty body)
__global__ __launch_bounds__(kBlock) void jagged_softmax_deriv_kernel(float* __restrict__ dst, const float* __restrict__ out,
                                                                      const float* __restrict__ grad, const int* __restrict__ off, int nseg)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    for (long long s = (long long)blockIdx.x * kWavesPerBlock + wave; s < nseg; s += (long long)gridDim.x * kWavesPerBlock) {
        const int a = off[s], b = off[s + 1];
        float z = 0.f;
        for (int j = a + lane; j < b; j += kWave) z += grad[j] * out[j];
        z = wave_sum(z);
        for (int j = a + lane; j < b; j += kWave) dst[j] += (grad[j] - z) * out[j];
    }
}

// ---- gradient of the row softmax: per row z = <grad, out>, dst += (grad - z) * out
//      (SoftmaxDeriv, src/nn/softmax.cpp:8-29; on the GPU cunn_SoftMax_updateGradInput_kernel, src/nn/softmax.cu:10-59)
__global__ __launch_bounds__(kBlock) void row_softmax_deriv_kernel(float* __restrict__ dst, const float* __restrict__ out,
                                                                   const float* __restrict__ grad, int rows, int cols)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows; r += (long long)gridDim.x * kWavesPerBlock) {
        const size_t a = (size_t)r * cols;
        float z = 0.f;
        for (int j = lane; j < cols; j += kWave) z += grad[a + j] * out[a + j];
        z = wave_sum(z);
        for (int j = lane; j < cols; j += kWave) dst[a + j] += (grad[a + j] - z) * out[a + j];
    }
}

// ---- global reductions: stage 1 writes one partial per workgroup, stage 2 combines
// them in index order, so the result does not depend on scheduling.
template <bool IS_MAX>
__device__ __forceinline__ float block_combine(float v, float* sh)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    v = IS_MAX ? wave_max(v) : wave_sum(v);
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    float r = sh[0];
    for (int w = 1; w < kWavesPerBlock; ++w) r = IS_MAX ? max_keep(r, sh[w]) : r + sh[w];
    __syncthreads();
    return r;
}

// The array is read as 128-bit words from its first 16-byte aligned element on (the few elements before it and after
// the last whole word go to workgroup 0), grid-strided, four words in flight per lane and sixteen running values per
// lane, which are combined in a fixed order: the result depends on n and the grid alone.  For max every running value
// starts from x[0], so that a NaN there, and only there, survives (the reference's strict comparison).
template <bool IS_MAX, bool SQUARE = false>
__global__ __launch_bounds__(kBlock) void reduce_partial_kernel(const float* __restrict__ x, size_t n, float* __restrict__ partial)
{
    __shared__ float sh[kWavesPerBlock];
    auto comb = [](float a, float b) { return IS_MAX ? max_keep(a, b) : a + (SQUARE ? b * b : b); };
    size_t head = ((16 - (reinterpret_cast<uintptr_t>(x) & 15)) & 15) / 4;
    if (head > n) head = n;
    const float4* __restrict__ x4 = reinterpret_cast<const float4*>(x + head);
    const size_t n4 = (n - head) / 4;
    const size_t tail0 = head + n4 * 4;
    const float init = IS_MAX ? x[0] : 0.f;
    float4 a[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) a[u] = make_float4(init, init, init, init);
    const size_t stride = (size_t)gridDim.x * kBlock;
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    for (; i + 3 * stride < n4; i += 4 * stride) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = x4[i + u * stride];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            a[u].x = comb(a[u].x, v[u].x); a[u].y = comb(a[u].y, v[u].y);
            a[u].z = comb(a[u].z, v[u].z); a[u].w = comb(a[u].w, v[u].w);
        }
    }
    for (; i < n4; i += stride) {
        const float4 v = x4[i];
        a[0].x = comb(a[0].x, v.x); a[0].y = comb(a[0].y, v.y); a[0].z = comb(a[0].z, v.z); a[0].w = comb(a[0].w, v.w);
    }
    if (blockIdx.x == 0) {
        for (size_t j = threadIdx.x; j < head; j += kBlock) a[0].x = comb(a[0].x, x[j]);
        for (size_t j = tail0 + threadIdx.x; j < n; j += kBlock) a[0].x = comb(a[0].x, x[j]);
    }
    auto join = [](float p, float q) { return IS_MAX ? max_keep(p, q) : p + q; };
    float v = join(join(join(a[0].x, a[0].y), join(a[0].z, a[0].w)), join(join(a[1].x, a[1].y), join(a[1].z, a[1].w)));
    v = join(v, join(join(join(a[2].x, a[2].y), join(a[2].z, a[2].w)), join(join(a[3].x, a[3].y), join(a[3].z, a[3].w))));
    v = block_combine<IS_MAX>(v, sh);
    if (threadIdx.x == 0) partial[blockIdx.x] = v;
}

template <bool IS_MAX>
__global__ __launch_bounds__(kBlock) void reduce_final_kernel(const float* __restrict__ partial, int np, float scale_div, float* __restrict__ out)
{
    __shared__ float sh[kWavesPerBlock];
    float v = IS_MAX ? partial[0] : 0.f;
    for (int i = threadIdx.x; i < np; i += kBlock) v = IS_MAX ? max_keep(v, partial[i]) : v + partial[i];
    v = block_combine<IS_MAX>(v, sh);
    if (threadIdx.x == 0) out[0] = (scale_div != 0.f) ? v / scale_div : v;
}

// ---- arg-max of each dense row, first index among ties
__global__ __launch_bounds__(kBlock) void row_argmax_kernel(const float* __restrict__ x, int rows, int cols, int* __restrict__ out)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows; r += (long long)gridDim.x * kWavesPerBlock) {
        const float* p = x + (size_t)r * cols;
        const float first = p[0];
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int j = lane; j < cols; j += kWave) {
            const float v = p[j];
            argmax_combine(bv, bi, (v != v) ? -INFINITY : v, j);     // a NaN that is not first never wins
        }
        wave_argmax(bv, bi);
        if (first != first) bi = 0;                                    // a NaN in column 0 is never displaced
        if (lane == 0) out[r] = bi;
    }
}

// ---- CSR rows are short (one-hot labels): one lane per row, reference scan order
__global__ __launch_bounds__(kBlock) void csr_row_argmax_kernel(const int* __restrict__ row_ptr, const int* __restrict__ col_idx,
                                                                const float* __restrict__ val, int rows, int* __restrict__ out)
{
    for (long long r = (long long)blockIdx.x * kBlock + threadIdx.x; r < rows; r += (long long)gridDim.x * kBlock) {
        const int a = row_ptr[r], b = row_ptr[r + 1];
        int best = 0;
        float cur = 0.f;
        for (int j = a; j < b; ++j)
            if (j == a || val[j] > cur) { cur = val[j]; best = col_idx[j]; }
        out[r] = best;
    }
}

__global__ __launch_bounds__(kBlock) void cross_entropy_kernel(const float* __restrict__ prob, int rows, int cols,
                                                               const int* __restrict__ lrow_ptr, const int* __restrict__ lcol,
                                                               const float* __restrict__ lval, float* __restrict__ out)
{
    for (long long r = (long long)blockIdx.x * kBlock + threadIdx.x; r < rows; r += (long long)gridDim.x * kBlock) {
        float loss = 0.f;
        for (int k = lrow_ptr[r]; k < lrow_ptr[r + 1]; ++k) {
            float t = prob[(size_t)cols * r + lcol[k]];
            if (fabs((double)t) < 1e-8) t = (float)1e-8;
            loss = (float)((double)loss - log((double)t) * (double)lval[k]);
        }
        out[r] = loss;
    }
}

__global__ __launch_bounds__(kBlock) void in_top_k_kernel(const float* __restrict__ pred, const int* __restrict__ label,
                                                          int rows, int cols, int k, int* __restrict__ out)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    for (long long r = (long long)blockIdx.x * kWavesPerBlock + wave; r < rows; r += (long long)gridDim.x * kWavesPerBlock) {
        const float* p = pred + (size_t)r * cols;
        const int target = label[r];
        const float pt = p[target];
        int cnt = 0;
        for (int j = lane; j < cols; j += kWave)
            if (j != target && p[j] > pt) cnt += 1;
        cnt = wave_sum_i(cnt);
        if (lane == 0) out[r] = cnt < k ? 1 : 0;
    }
}

inline unsigned wave_rows_grid(long long rows)
{
    long long b = (rows + kWavesPerBlock - 1) / kWavesPerBlock;
    if (b < 1) b = 1;
    if (b > kNumCU * 16) b = kNumCU * 16;
    return (unsigned)b;
}

inline unsigned lane_rows_grid(long long rows)
{
    long long b = (rows + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > kNumCU * 16) b = kNumCU * 16;
    return (unsigned)b;
}

}  // namespace

// Address of the current device's copy of `scratch` (resolved once per device, no allocation).
int static_offsets_ptr(int** out)
{
    int dev = -1;
    GNNHIP_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return set_error(GNNHIP_EINVAL, "device ordinal %d outside [0,%d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_static_mu);
    if (!g_static_offsets[dev]) {
        void* p = nullptr;
        GNNHIP_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return set_error(GNNHIP_EHIP, "hipGetSymbolAddress returned a null address for the static offsets");
        g_static_offsets[dev] = static_cast<int*>(p);
    }
    *out = g_static_offsets[dev];
    return GNNHIP_OK;
}

int row_softmax_dispatch(float* x, int rows, int cols, hipStream_t s)
{
    hipLaunchKernelGGL(row_softmax_kernel, dim3(wave_rows_grid(rows)), dim3(kBlock), 0, s, x, rows, cols);
    GNNHIP_LAUNCH_CHECK("row_softmax");
    return GNNHIP_OK;
}

int row_argmax_dispatch(const float* x, int rows, int cols, int* out, hipStream_t s)
{
    hipLaunchKernelGGL(row_argmax_kernel, dim3(wave_rows_grid(rows)), dim3(kBlock), 0, s, x, rows, cols, out);
    GNNHIP_LAUNCH_CHECK("row_argmax");
    return GNNHIP_OK;
}

}  // namespace gnnhip

using namespace gnnhip;

extern "C" {

int gnnhip_row_softmax_f32(float* x, int rows, int cols, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && cols >= 0, "negative shape in row_softmax");
    if (rows == 0 || cols == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x != nullptr, "null tensor in row_softmax");
    if (int rc = require_ready()) return rc;
    return row_softmax_dispatch(x, rows, cols, as_stream(stream));
}

int gnnhip_jagged_softmax_f32(float* x, const int* lens, int nseg, void* stream)
{
    GNNHIP_REQUIRE(nseg >= 0, "negative segment count");
    if (nseg == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x && lens, "null tensor in jagged_softmax");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    if (nseg <= kFusedJaggedMaxSegments) {
        const unsigned grid = (unsigned)((nseg + kWavesPerBlock - 1) / kWavesPerBlock);
        hipLaunchKernelGGL(jagged_softmax_fused_kernel, dim3(grid), dim3(kBlock), 0, s, x, lens, nseg);
        GNNHIP_LAUNCH_CHECK("jagged_softmax_fused");
        return GNNHIP_OK;
    }
    void* off = nullptr;
    if (int rc = stream_scratch(s, sizeof(int) * ((size_t)nseg + 1), &off)) return rc;
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(1), dim3(kScanBlock), 0, s, lens, nseg, static_cast<int*>(off));
    GNNHIP_LAUNCH_CHECK("exclusive_scan");
    hipLaunchKernelGGL(jagged_softmax_kernel, dim3(wave_rows_grid(nseg)), dim3(kBlock), 0, s, x, static_cast<const int*>(off), nseg);
    GNNHIP_LAUNCH_CHECK("jagged_softmax");
    return GNNHIP_OK;
}

int gnnhip_jagged_softmax_deriv_f32(float* dst, const float* out, const float* grad, const int* lens, int nseg, void* stream)
{
    GNNHIP_REQUIRE(nseg >= 0, "negative segment count");
    if (nseg == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(dst && out && grad && lens, "null tensor in jagged_softmax_deriv");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    void* off = nullptr;
    if (int rc = stream_scratch(s, sizeof(int) * ((size_t)nseg + 1), &off)) return rc;
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(1), dim3(kScanBlock), 0, s, lens, nseg, static_cast<int*>(off));
    GNNHIP_LAUNCH_CHECK("exclusive_scan");
    hipLaunchKernelGGL(jagged_softmax_deriv_kernel, dim3(wave_rows_grid(nseg)), dim3(kBlock), 0, s, dst, out, grad,
                       static_cast<const int*>(off), nseg);
    GNNHIP_LAUNCH_CHECK("jagged_softmax_deriv");
    return GNNHIP_OK;
}

int gnnhip_row_softmax_deriv_f32(float* dst, const float* out, const float* grad, int rows, int cols, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && cols >= 0, "negative shape in row_softmax_deriv");
    if (rows == 0 || cols == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(dst && out && grad, "null tensor in row_softmax_deriv");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(row_softmax_deriv_kernel, dim3(wave_rows_grid(rows)), dim3(kBlock), 0, as_stream(stream), dst, out, grad, rows, cols);
    GNNHIP_LAUNCH_CHECK("row_softmax_deriv");
    return GNNHIP_OK;
}

int gnnhip_jagged_softmax_static_f32(float* x, const int* lens, int nseg, void* stream)
{
    GNNHIP_REQUIRE(nseg >= 0, "negative segment count");
    GNNHIP_REQUIRE(nseg <= kStaticMaxSegments, "jagged_softmax_static takes at most %d segments, got %d (use gnnhip_jagged_softmax_f32)",
                   kStaticMaxSegments, nseg);
    if (nseg == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x && lens, "null tensor in jagged_softmax_static");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    int* off = nullptr;
    if (int rc = static_offsets_ptr(&off)) return rc;
    // the scan writes off[0..nseg] in full, so what an earlier call left in the array is never read
    hipLaunchKernelGGL(exclusive_scan_kernel, dim3(1), dim3(kScanBlock), 0, s, lens, nseg, off);
    GNNHIP_LAUNCH_CHECK("exclusive_scan");
    hipLaunchKernelGGL(jagged_softmax_kernel, dim3(wave_rows_grid(nseg)), dim3(kBlock), 0, s, x, static_cast<const int*>(off), nseg);
    GNNHIP_LAUNCH_CHECK("jagged_softmax");
    return GNNHIP_OK;
}

int gnnhip_reduce_f32(int op, const float* x, size_t n, float* out, void* stream)
{
    GNNHIP_REQUIRE(op == GNNHIP_REDUCE_SUM || op == GNNHIP_REDUCE_MEAN || op == GNNHIP_REDUCE_MAX || op == GNNHIP_REDUCE_SUMSQ,
                   "unknown reduce op %d", op);
    GNNHIP_REQUIRE(out != nullptr, "null output in reduce");
    GNNHIP_REQUIRE(n > 0 && x != nullptr, "empty input in reduce");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    size_t nb = (n + 16383) / 16384;                   // >= 16K elements per workgroup
    if (nb > 2048) nb = 2048;                          // eight workgroups per compute unit
    void* partial = nullptr;
    if (int rc = stream_scratch(s, sizeof(float) * 2048, &partial)) return rc;
    float* pp = static_cast<float*>(partial);
    const float div = (op == GNNHIP_REDUCE_MEAN) ? (float)n : 0.f;
    if (op == GNNHIP_REDUCE_MAX) {
        hipLaunchKernelGGL((reduce_partial_kernel<true>), dim3((unsigned)nb), dim3(kBlock), 0, s, x, n, pp);
        hipLaunchKernelGGL((reduce_final_kernel<true>), dim3(1), dim3(kBlock), 0, s, pp, (int)nb, 0.f, out);
    } else if (op == GNNHIP_REDUCE_SUMSQ) {
        hipLaunchKernelGGL((reduce_partial_kernel<false, true>), dim3((unsigned)nb), dim3(kBlock), 0, s, x, n, pp);
        hipLaunchKernelGGL((reduce_final_kernel<false>), dim3(1), dim3(kBlock), 0, s, pp, (int)nb, 0.f, out);
    } else {
        hipLaunchKernelGGL((reduce_partial_kernel<false>), dim3((unsigned)nb), dim3(kBlock), 0, s, x, n, pp);
        hipLaunchKernelGGL((reduce_final_kernel<false>), dim3(1), dim3(kBlock), 0, s, pp, (int)nb, div, out);
    }
    GNNHIP_LAUNCH_CHECK("reduce");
    return GNNHIP_OK;
}

int gnnhip_row_argmax_f32(const float* x, int rows, int cols, int* out, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && cols >= 1, "bad shape in row_argmax (rows=%d cols=%d)", rows, cols);
    if (rows == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x && out, "null tensor in row_argmax");
    if (int rc = require_ready()) return rc;
    return row_argmax_dispatch(x, rows, cols, out, as_stream(stream));
}

int gnnhip_csr_row_argmax_f32(const int* row_ptr, const int* col_idx, const float* val, int rows, int* out, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0, "negative row count");
    if (rows == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(row_ptr && out, "null tensor in csr_row_argmax");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(csr_row_argmax_kernel, dim3(lane_rows_grid(rows)), dim3(kBlock), 0, as_stream(stream),
                       row_ptr, col_idx, val, rows, out);
    GNNHIP_LAUNCH_CHECK("csr_row_argmax");
    return GNNHIP_OK;
}

int gnnhip_cross_entropy_f32(const float* prob, int rows, int cols, const int* lrow_ptr, const int* lcol,
                             const float* lval, float* out, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && cols >= 1, "bad shape in cross_entropy");
    if (rows == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(prob && lrow_ptr && out, "null tensor in cross_entropy");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(cross_entropy_kernel, dim3(lane_rows_grid(rows)), dim3(kBlock), 0, as_stream(stream),
                       prob, rows, cols, lrow_ptr, lcol, lval, out);
    GNNHIP_LAUNCH_CHECK("cross_entropy");
    return GNNHIP_OK;
}

int gnnhip_in_top_k_f32(const float* pred, const int* label, int rows, int cols, int k, int* out, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && cols >= 1, "bad shape in in_top_k");
    if (rows == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(pred && label && out, "null tensor in in_top_k");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(in_top_k_kernel, dim3(wave_rows_grid(rows)), dim3(kBlock), 0, as_stream(stream),
                       pred, label, rows, cols, k, out);
    GNNHIP_LAUNCH_CHECK("in_top_k");
    return GNNHIP_OK;
}

}  // extern "C"
