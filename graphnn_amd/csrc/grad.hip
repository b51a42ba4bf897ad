// Backward-pass kernels of the structure2vec path for gfx950: the transposed CSR
// product (gradient through message aggregation), dense += a * sparse (the label
// term of the softmax cross-entropy gradient), the ReLU derivative and the
// element-wise / row-broadcast multiplies.  All HBM-bound.
#include "gnnhip_internal.h"

namespace gnnhip {
namespace {

constexpr int kBlock = 256;

// C[col[t], :] += alpha * val[t] * B[i, :] for every entry t of row i.  One group of G lanes
// per CSR row, float4 (or scalar) column slabs per lane; different rows may hit the same
// output row, so the accumulation uses hardware fp32 atomics (order of additions not fixed).
template <int VEC>
__global__ __launch_bounds__(kBlock) void spmm_t_scatter_kernel(
    int m, int n, float alpha, const int* __restrict__ row_ptr, const int* __restrict__ col_idx,
    const float* __restrict__ val, const float* __restrict__ B, int ldb, float* C, int ldc, int logG)
{
    const int G = 1 << logG;
    const int sub = threadIdx.x & (G - 1);
    const long long row = (long long)blockIdx.x * (kBlock >> logG) + (threadIdx.x >> logG);
    if (row >= m) return;
    const int start = row_ptr[row], end = row_ptr[row + 1];
    for (int col0 = sub * VEC; col0 < n; col0 += G * VEC) {
        float b[VEC];
#pragma unroll
        for (int u = 0; u < VEC; ++u) b[u] = B[(size_t)row * ldb + col0 + u];
        for (int t = start; t < end; ++t) {
            const float a = alpha * val[t];
            float* dst = C + (size_t)col_idx[t] * ldc + col0;
#pragma unroll
            for (int u = 0; u < VEC; ++u) unsafeAtomicAdd(dst + u, a * b[u]);
        }
    }
}

__global__ __launch_bounds__(kBlock) void scale_rows_kernel(float* C, int rows, int n, int ldc, float beta)
{
    const size_t total = (size_t)rows * n;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock) {
        const size_t r = i / n, c = i - r * n;
        float* p = C + r * ldc + c;
        *p = (beta == 0.f) ? 0.f : beta * (*p);
    }
}

// dense[r, col[t]] += a * val[t]; one lane per row keeps duplicates in a row ordered
__global__ __launch_bounds__(kBlock) void csr_axpy_kernel(int rows, int cols, float a, const int* __restrict__ row_ptr,
                                                          const int* __restrict__ col_idx, const float* __restrict__ val,
                                                          float* dense)
{
    for (long long r = (long long)blockIdx.x * kBlock + threadIdx.x; r < rows; r += (long long)gridDim.x * kBlock)
        for (int t = row_ptr[r]; t < row_ptr[r + 1]; ++t) dense[(size_t)r * cols + col_idx[t]] += a * val[t];
}

// dst += grad where the forward output was positive (ReLUDeriv)
__global__ __launch_bounds__(kBlock) void relu_deriv_kernel(size_t n, const float* __restrict__ out, const float* __restrict__ grad,
                                                            float* dst)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
        if (out[i] > 0.f) dst[i] += grad[i];
}

__global__ __launch_bounds__(kBlock) void mul_kernel(size_t n, const float* __restrict__ x, float* y)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) y[i] *= x[i];
}

// y[r, :] *= s[r]
__global__ __launch_bounds__(kBlock) void row_scale_kernel(int rows, int cols, const float* __restrict__ s, float* y)
{
    const size_t total = (size_t)rows * cols;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock) y[i] *= s[i / cols];
}

inline unsigned ew_grid(size_t n)
{
    size_t b = (n + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > (size_t)kNumCU * 8) b = (size_t)kNumCU * 8;
    return (unsigned)b;
}

}  // namespace
}  // namespace gnnhip

using namespace gnnhip;

extern "C" {

int gnnhip_spmm_csr_t_f32(int m, int k, int n, float alpha, const int* row_ptr, const int* col_idx,
                          const float* val, const float* B, int ldb, float beta, float* C, int ldc, void* stream)
{
    GNNHIP_REQUIRE(m >= 0 && k >= 0 && n >= 0, "negative dimension in spmm_t (m=%d k=%d n=%d)", m, k, n);
    if (k == 0 || n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(C != nullptr && ldc >= n, "bad output in spmm_t");
    GNNHIP_REQUIRE(m == 0 || (row_ptr && B && ldb >= n), "null operand in spmm_t");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    if (beta != 1.f) {
        hipLaunchKernelGGL(scale_rows_kernel, dim3(ew_grid((size_t)k * n)), dim3(kBlock), 0, s, C, k, n, ldc, beta);
        GNNHIP_LAUNCH_CHECK("scale_rows");
    }
    if (m == 0) return GNNHIP_OK;
    const bool vec4 = (n % 4 == 0);
    const int units = vec4 ? n / 4 : n;
    int logG = 0;
    while ((1 << logG) < units && logG < 6) ++logG;
    const unsigned blocks = ceil_div_u((size_t)m, (size_t)(kBlock >> logG));
    if (vec4)
        hipLaunchKernelGGL((spmm_t_scatter_kernel<4>), dim3(blocks), dim3(kBlock), 0, s, m, n, alpha, row_ptr, col_idx, val, B, ldb, C, ldc, logG);
    else
        hipLaunchKernelGGL((spmm_t_scatter_kernel<1>), dim3(blocks), dim3(kBlock), 0, s, m, n, alpha, row_ptr, col_idx, val, B, ldb, C, ldc, logG);
    GNNHIP_LAUNCH_CHECK("spmm_t_scatter");
    return GNNHIP_OK;
}

int gnnhip_csr_axpy_f32(int rows, int cols, float a, const int* row_ptr, const int* col_idx, const float* val,
                        float* dense, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && cols >= 0, "negative shape in csr_axpy");
    if (rows == 0 || cols == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(row_ptr && dense, "null tensor in csr_axpy");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(csr_axpy_kernel, dim3(ew_grid((size_t)rows)), dim3(kBlock), 0, as_stream(stream),
                       rows, cols, a, row_ptr, col_idx, val, dense);
    GNNHIP_LAUNCH_CHECK("csr_axpy");
    return GNNHIP_OK;
}

int gnnhip_relu_deriv_f32(size_t n, const float* out, const float* grad, float* dst, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(out && grad && dst, "null tensor in relu_deriv");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(relu_deriv_kernel, dim3(ew_grid(n)), dim3(kBlock), 0, as_stream(stream), n, out, grad, dst);
    GNNHIP_LAUNCH_CHECK("relu_deriv");
    return GNNHIP_OK;
}

int gnnhip_mul_f32(size_t n, const float* x, float* y, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(x && y, "null tensor in mul");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(mul_kernel, dim3(ew_grid(n)), dim3(kBlock), 0, as_stream(stream), n, x, y);
    GNNHIP_LAUNCH_CHECK("mul");
    return GNNHIP_OK;
}

int gnnhip_row_scale_f32(int rows, int cols, const float* scale, float* y, void* stream)
{
    GNNHIP_REQUIRE(rows >= 0 && cols >= 0, "negative shape in row_scale");
    if (rows == 0 || cols == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(scale && y, "null tensor in row_scale");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(row_scale_kernel, dim3(ew_grid((size_t)rows * cols)), dim3(kBlock), 0, as_stream(stream), rows, cols, scale, y);
    GNNHIP_LAUNCH_CHECK("row_scale");
    return GNNHIP_OK;
}

}  // extern "C"
