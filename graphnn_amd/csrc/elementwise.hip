// Element-wise functor engine for gfx950: one templated grid-stride kernel with
// 128-bit loads/stores on the aligned body and a scalar tail, instantiated for
// the unary functors of graphnn's UnaryEngine<GPU>
// (include/tensor/gpu_unary_functor.h:17-384) and for the two- and three-operand
// forms the mean-field path needs (Axpy, Axpby, ElewiseAdd, ReLUAct, TypeCast).
// All of these are HBM-bound: 8 bytes per element in place, 12 for a + b -> out.
#include "gnnhip_internal.h"

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxBlocks = kNumCU * 8;

// ---------------------------------------------------------------- functors
struct FSet      { float s; __device__ float operator()(float) const { return s; } };
struct FTruncate { float lo, hi; __device__ float operator()(float v) const { v = v < lo ? lo : v; return v > hi ? hi : v; } };
struct FScale    { float s; __device__ float operator()(float v) const { return v * s; } };
struct FAdd      { float s; __device__ float operator()(float v) const { return v + s; } };
struct FAbs      { __device__ float operator()(float v) const { return fabsf(v); } };
struct FInv      { __device__ float operator()(float v) const { return 1.0f / v; } };
struct FReLU     { __device__ float operator()(float v) const { return v < 0.0f ? 0.0f : v; } };   // -0.0 and NaN pass through
struct FSigmoid  { __device__ float operator()(float v) const { return 1.0f / (1.0f + expf(-v)); } };
struct FTanh     { __device__ float operator()(float v) const { float a = expf(v), b = expf(-v); return (a - b) / (a + b); } };
struct FLog      { __device__ float operator()(float v) const { return logf(v); } };
struct FInvSqrt  { __device__ float operator()(float v) const { return 1.0f / sqrtf(v); } };
struct FExp      { __device__ float operator()(float v) const { return expf(v); } };
struct FSquare   { __device__ float operator()(float v) const { return v * v; } };
struct FSqrt     { __device__ float operator()(float v) const { return sqrtf(v); } };

struct GAxpy  { float a; __device__ float operator()(float x, float y) const { return y + a * x; } };
struct GAxpby { float a, b; __device__ float operator()(float x, float y) const { return a * x + b * y; } };
struct GAdd   { __device__ float operator()(float x, float y) const { return x + y; } };

// ---------------------------------------------------------------- kernels
// dst[i] = f(src[i]); src may equal dst.  n4 = number of float4 groups in the body.
template <class F>
__global__ __launch_bounds__(kBlock) void map1_kernel(const float* __restrict__ src, float* dst, size_t n, F f)
{
    const size_t n4 = n >> 2;
    const size_t stride = (size_t)gridDim.x * kBlock;
    const float4* s4 = reinterpret_cast<const float4*>(src);
    float4* d4 = reinterpret_cast<float4*>(dst);
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += stride) {
        float4 v = s4[i];
        v.x = f(v.x); v.y = f(v.y); v.z = f(v.z); v.w = f(v.w);
        d4[i] = v;
    }
    const size_t tail = n4 << 2;
    const size_t t = tail + (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < n) dst[t] = f(src[t]);     // at most 3 tail elements; only the first block sees any
}

template <class F>
__global__ __launch_bounds__(kBlock) void map1_scalar_kernel(const float* src, float* dst, size_t n, F f)
{
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) dst[i] = f(src[i]);
}

// out[i] = g(x[i], y[i]); out may equal y.
template <class G>
__global__ __launch_bounds__(kBlock) void map2_kernel(const float* __restrict__ x, const float* y, float* out, size_t n, G g)
{
    const size_t n4 = n >> 2;
    const size_t stride = (size_t)gridDim.x * kBlock;
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const float4* y4 = reinterpret_cast<const float4*>(y);
    float4* o4 = reinterpret_cast<float4*>(out);
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n4; i += stride) {
        float4 a = x4[i], b = y4[i], r;
        r.x = g(a.x, b.x); r.y = g(a.y, b.y); r.z = g(a.z, b.z); r.w = g(a.w, b.w);
        o4[i] = r;
    }
    const size_t tail = n4 << 2;
    const size_t t = tail + (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < n) out[t] = g(x[t], y[t]);
}

template <class G>
__global__ __launch_bounds__(kBlock) void map2_scalar_kernel(const float* x, const float* y, float* out, size_t n, G g)
{
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) out[i] = g(x[i], y[i]);
}

__global__ __launch_bounds__(kBlock) void cast_i32_f32_kernel(const int* __restrict__ src, float* __restrict__ dst, size_t n)
{
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) dst[i] = (float)src[i];
}

// Zero-fill: 16-byte stores on the aligned body, bytes on both ragged ends.
__global__ __launch_bounds__(kBlock) void zero_kernel(unsigned char* p, size_t head, size_t n16, size_t total)
{
    const size_t stride = (size_t)gridDim.x * kBlock;
    const size_t gid = (size_t)blockIdx.x * kBlock + threadIdx.x;
    uint4* body = reinterpret_cast<uint4*>(p + head);
    const uint4 z = make_uint4(0u, 0u, 0u, 0u);
    for (size_t i = gid; i < n16; i += stride) body[i] = z;
    if (gid < head) p[gid] = 0;
    const size_t tail0 = head + (n16 << 4);
    if (tail0 + gid < total) p[tail0 + gid] = 0;    // fewer than 16 tail bytes
}

// The same for up to kZeroBatch buffers in one launch: blockIdx.y picks the buffer.
constexpr int kZeroBatch = 48;
struct ZeroBatch {
    unsigned char* p[kZeroBatch];
    size_t bytes[kZeroBatch];
};
__global__ __launch_bounds__(kBlock) void zero_batch_kernel(ZeroBatch b)
{
    unsigned char* p = b.p[blockIdx.y];
    const size_t total = b.bytes[blockIdx.y];
    size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15u)) & 15u;
    if (head > total) head = total;
    const size_t n16 = (total - head) >> 4;
    const size_t stride = (size_t)gridDim.x * kBlock;
    const size_t gid = (size_t)blockIdx.x * kBlock + threadIdx.x;
    uint4* body = reinterpret_cast<uint4*>(p + head);
    const uint4 z = make_uint4(0u, 0u, 0u, 0u);
    for (size_t i = gid; i < n16; i += stride) body[i] = z;
    if (gid < head) p[gid] = 0;
    const size_t tail0 = head + (n16 << 4);
    if (tail0 + gid < total) p[tail0 + gid] = 0;
}

inline unsigned grid_for(size_t work_items)
{
    size_t b = (work_items + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > (size_t)kMaxBlocks) b = kMaxBlocks;
    return (unsigned)b;
}

template <class F>
int launch_map1(const float* src, float* dst, size_t n, F f, hipStream_t s)
{
    if (n == 0) return GNNHIP_OK;
    if (aligned16(src) && aligned16(dst)) {
        size_t n4 = n >> 2;
        hipLaunchKernelGGL(map1_kernel<F>, dim3(grid_for(n4 ? n4 : 1)), dim3(kBlock), 0, s, src, dst, n, f);
    } else {
        hipLaunchKernelGGL(map1_scalar_kernel<F>, dim3(grid_for(n)), dim3(kBlock), 0, s, src, dst, n, f);
    }
    GNNHIP_LAUNCH_CHECK("map1");
    return GNNHIP_OK;
}

template <class G>
int launch_map2(const float* x, const float* y, float* out, size_t n, G g, hipStream_t s)
{
    if (n == 0) return GNNHIP_OK;
    if (aligned16(x) && aligned16(y) && aligned16(out)) {
        size_t n4 = n >> 2;
        hipLaunchKernelGGL(map2_kernel<G>, dim3(grid_for(n4 ? n4 : 1)), dim3(kBlock), 0, s, x, y, out, n, g);
    } else {
        hipLaunchKernelGGL(map2_scalar_kernel<G>, dim3(grid_for(n)), dim3(kBlock), 0, s, x, y, out, n, g);
    }
    GNNHIP_LAUNCH_CHECK("map2");
    return GNNHIP_OK;
}

}  // namespace
}  // namespace gnnhip

using namespace gnnhip;

extern "C" {

int gnnhip_unary_f32(int op, float* x, size_t n, float a0, float a1, void* stream)
{
    GNNHIP_REQUIRE(op >= 0 && op < GNNHIP_UNARY__COUNT, "unknown unary op %d", op);
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x != nullptr, "null tensor in unary op");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    switch (op) {
    case GNNHIP_UNARY_SET:      return launch_map1(x, x, n, FSet{a0}, s);
    case GNNHIP_UNARY_TRUNCATE: return launch_map1(x, x, n, FTruncate{a0, a1}, s);
    case GNNHIP_UNARY_SCALE:    return launch_map1(x, x, n, FScale{a0}, s);
    case GNNHIP_UNARY_ADD:      return launch_map1(x, x, n, FAdd{a0}, s);
    case GNNHIP_UNARY_ABS:      return launch_map1(x, x, n, FAbs{}, s);
    case GNNHIP_UNARY_INV:      return launch_map1(x, x, n, FInv{}, s);
    case GNNHIP_UNARY_RELU:     return launch_map1(x, x, n, FReLU{}, s);
    case GNNHIP_UNARY_SIGMOID:  return launch_map1(x, x, n, FSigmoid{}, s);
    case GNNHIP_UNARY_TANH:     return launch_map1(x, x, n, FTanh{}, s);
    case GNNHIP_UNARY_LOG:      return launch_map1(x, x, n, FLog{}, s);
    case GNNHIP_UNARY_INVSQRT:  return launch_map1(x, x, n, FInvSqrt{}, s);
    case GNNHIP_UNARY_EXP:      return launch_map1(x, x, n, FExp{}, s);
    case GNNHIP_UNARY_SQUARE:   return launch_map1(x, x, n, FSquare{}, s);
    case GNNHIP_UNARY_SQRT:     return launch_map1(x, x, n, FSqrt{}, s);
    }
    return set_error(GNNHIP_EINVAL, "unknown unary op %d", op);
}

int gnnhip_relu_f32(const float* in, float* out, size_t n, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(in && out, "null tensor in relu");
    if (int rc = require_ready()) return rc;
    return launch_map1(in, out, n, FReLU{}, as_stream(stream));
}

int gnnhip_axpy_f32(size_t n, float a, const float* x, float* y, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x && y, "null tensor in axpy");
    if (int rc = require_ready()) return rc;
    return launch_map2(x, y, y, n, GAxpy{a}, as_stream(stream));
}

int gnnhip_axpby_f32(size_t n, float a, const float* x, float b, float* y, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x && y, "null tensor in axpby");
    if (int rc = require_ready()) return rc;
    return launch_map2(x, y, y, n, GAxpby{a, b}, as_stream(stream));
}

int gnnhip_add_f32(size_t n, const float* a, const float* b, float* out, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(a && b && out, "null tensor in add");
    if (int rc = require_ready()) return rc;
    return launch_map2(a, b, out, n, GAdd{}, as_stream(stream));
}

int gnnhip_cast_i32_f32(const int* src, float* dst, size_t n, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(src && dst, "null tensor in cast");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(cast_i32_f32_kernel, dim3(grid_for(n)), dim3(kBlock), 0, as_stream(stream), src, dst, n);
    GNNHIP_LAUNCH_CHECK("cast_i32_f32");
    return GNNHIP_OK;
}

// A fill kernel rather than hipMemsetAsync, so the call is safe inside a captured HIP graph.
int gnnhip_memset0(void* device_ptr, size_t bytes, void* stream)
{
    if (bytes == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(device_ptr != nullptr, "null pointer in memset0");
    if (int rc = require_ready()) return rc;
    unsigned char* p = static_cast<unsigned char*>(device_ptr);
    size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15u)) & 15u;
    if (head > bytes) head = bytes;
    size_t n16 = (bytes - head) >> 4;
    hipLaunchKernelGGL(zero_kernel, dim3(grid_for(n16 ? n16 : 1)), dim3(kBlock), 0, as_stream(stream), p, head, n16, bytes);
    GNNHIP_LAUNCH_CHECK("zero");
    return GNNHIP_OK;
}

int gnnhip_memset0_batch(int n, void* const* device_ptrs, const size_t* bytes, void* stream)
{
    GNNHIP_REQUIRE(n >= 0 && (n == 0 || (device_ptrs && bytes)), "bad arguments in memset0_batch");
    if (int rc = require_ready()) return rc;
    int i = 0;
    while (i < n) {
        ZeroBatch b;
        int m = 0;
        size_t largest = 0;
        for (; i < n && m < kZeroBatch; ++i) {
            if (bytes[i] == 0) continue;
            GNNHIP_REQUIRE(device_ptrs[i] != nullptr, "null pointer in memset0_batch");
            b.p[m] = static_cast<unsigned char*>(device_ptrs[i]);
            b.bytes[m] = bytes[i];
            if (bytes[i] > largest) largest = bytes[i];
            ++m;
        }
        if (m == 0) break;
        const size_t n16 = largest >> 4;
        unsigned gx = grid_for(n16 ? n16 : 1);
        if (gx > 1024u) gx = 1024u;
        hipLaunchKernelGGL(zero_batch_kernel, dim3(gx, (unsigned)m), dim3(kBlock), 0, as_stream(stream), b);
        GNNHIP_LAUNCH_CHECK("zero_batch");
    }
    return GNNHIP_OK;
}

}  // extern "C"
