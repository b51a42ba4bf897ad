// C = alpha * A^T * B + beta * C for a square output of 128 x 128 or 256 x 256 over a very long k: the weight
// gradient of the mean-field levels at hidden 128 / 256, dW = [h_0 .. h_{L-1}]^T [u_1 .. u_L] with k = levels x
// nodes (MatMul::Backward, src/nn/matmul.cpp:35-76: x^T * dy through DTensor<GPU>::MM,
// src/tensor/gpu_dense_tensor.cu:192-224).
//
// The 64 x 64 tiles of the general kernel read every row of A and of B four times per product (once per tile
// column / tile row) and keep 16 accumulators per lane; at 256 x 256 that left it at 58 TFLOP/s.  Here one
// workgroup of eight wavefronts holds the WHOLE output in registers (wavefront w owns MT/8 rows and all MT
// columns: 128 accumulators per lane at MT = 256) and walks one contiguous range of k, so each row of A and B
// is read from memory once per launch.  Sixteen rows of both operands are staged per step in LDS as they lie
// (row-major, the row stride padded by 16 floats so that the four k of a matrix instruction start 16 banks
// apart); lane (q = lane/16, t = lane%16) reads A[k0 + q][i0 + t] and B[k0 + q][j0 + t] with 32-bit LDS reads,
// MT/128 + MT/16 reads for MT*MT/2048 matrix instructions.  The next sixteen rows are asked for before the
// products of the current ones are formed and written to the other half of the LDS behind them (one barrier per
// step).  The workgroups' raw sums go to scratch and sgemm_splitk_reduce_kernel adds them in range order.
#include "gnnhip_internal.h"
#include "buffer_addr.h"

namespace gnnhip {

// gemm.hip
void launch_splitk_reduce(int m, int n, int splits, float alpha, const float* partial, float beta, float* C, int ldc, hipStream_t s);

namespace {

constexpr int kTallWaves = 8;
constexpr int kTallBlock = kTallWaves * kWave;
constexpr int kTallRows = 16;                 // rows of k staged per step
constexpr long long kTallMinK = 8192;

template <int MT>
__global__ __launch_bounds__(kTallBlock) void sgemm_tn_tall_kernel(int k, int k_chunk, const float* __restrict__ A, int lda,
                                                                   const float* __restrict__ B, int ldb, float* __restrict__ partial)
{
    constexpr int IB = MT / (16 * kTallWaves);            // 16-row blocks per wavefront
    constexpr int JB = MT / 16;                           // 16-column blocks
    constexpr int LD = MT + 16;
    constexpr int LPR = MT / 4;                           // lanes that cover a row with 128-bit loads
    constexpr int RPI = kTallBlock / LPR;                 // rows per load instruction of the workgroup
    constexpr int NI = kTallRows / RPI;                   // load instructions per operand and step
    static_assert(IB >= 1 && NI >= 1 && RPI * NI == kTallRows, "shape");
    extern __shared__ float slabs[];                      // [2][2][kTallRows][LD]: buffer, operand, row, column

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int q = lane >> 4, t = lane & 15;
    const long long k_lo = (long long)blockIdx.x * k_chunk;
    const int rows = (int)min((long long)k_chunk, (long long)k - k_lo);      // > 0: the grid covers k exactly
    // this workgroup's rows only: what lies past them reads as zero
    const rsrc_t a_rsrc = make_rsrc(A + (size_t)k_lo * lda, (unsigned)(((size_t)(rows - 1) * lda + MT) * 4));
    const rsrc_t b_rsrc = make_rsrc(B + (size_t)k_lo * ldb, (unsigned)(((size_t)(rows - 1) * ldb + MT) * 4));
    const int ld_row = tid / LPR, ld_col = (tid % LPR) * 4;
    const int a_voff = (ld_row * lda + ld_col) * 4, b_voff = (ld_row * ldb + ld_col) * 4;

    mfma_f4 acc[IB][JB];
#pragma unroll
    for (int ib = 0; ib < IB; ++ib)
#pragma unroll
        for (int jb = 0; jb < JB; ++jb) acc[ib][jb] = mfma_f4{0.f, 0.f, 0.f, 0.f};

    float4 ra[NI], rb[NI];
    auto fetch = [&](int r0) {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            ra[j] = buf_load4(a_rsrc, a_voff, (r0 + j * RPI) * lda * 4);
            rb[j] = buf_load4(b_rsrc, b_voff, (r0 + j * RPI) * ldb * 4);
        }
    };
    auto park = [&](int buf) {
        float* as = slabs + (buf * 2 + 0) * (kTallRows * LD);
        float* bs = slabs + (buf * 2 + 1) * (kTallRows * LD);
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            *reinterpret_cast<float4*>(as + (ld_row + j * RPI) * LD + ld_col) = ra[j];
            *reinterpret_cast<float4*>(bs + (ld_row + j * RPI) * LD + ld_col) = rb[j];
        }
    };

    fetch(0);
    park(0);
    __syncthreads();
    int buf = 0;
    for (int r0 = 0; r0 < rows; r0 += kTallRows) {
        const bool more = r0 + kTallRows < rows;
        if (more) fetch(r0 + kTallRows);
        const float* as = slabs + (buf * 2 + 0) * (kTallRows * LD) + wave * (16 * IB) + t;
        const float* bs = slabs + (buf * 2 + 1) * (kTallRows * LD) + t;
#pragma unroll
        for (int ks = 0; ks < kTallRows / 4; ++ks) {
            const int p = 4 * ks + q;
            float a[IB], b[JB];
#pragma unroll
            for (int ib = 0; ib < IB; ++ib) a[ib] = as[p * LD + 16 * ib];
#pragma unroll
            for (int jb = 0; jb < JB; ++jb) b[jb] = bs[p * LD + 16 * jb];
            // operand roles swapped (out^T = B^T A): lane (q, t) ends with row t, columns 4 q .. 4 q + 3 of a block
#pragma unroll
            for (int ib = 0; ib < IB; ++ib)
#pragma unroll
                for (int jb = 0; jb < JB; ++jb)
                    acc[ib][jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[jb], a[ib], acc[ib][jb], 0, 0, 0);
        }
        if (more) park(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

    float* part = partial + (size_t)blockIdx.x * MT * MT;
#pragma unroll
    for (int ib = 0; ib < IB; ++ib) {
        const int i = wave * (16 * IB) + 16 * ib + t;
#pragma unroll
        for (int jb = 0; jb < JB; ++jb)
            *reinterpret_cast<float4*>(part + (size_t)i * MT + 16 * jb + 4 * q) =
                make_float4(acc[ib][jb][0], acc[ib][jb][1], acc[ib][jb][2], acc[ib][jb][3]);
    }
}

template <int MT>
int launch_tall(int k, float alpha, const float* A, int lda, const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s)
{
    // one workgroup per compute unit (two at 128 x 128), each a contiguous range of k of whole steps
    const long long want = (long long)kNumCU * (MT == 128 ? 2 : 1);
    long long chunk = (k + want - 1) / want;
    if (chunk < 4 * kTallRows) chunk = 4 * kTallRows;
    chunk = (chunk + kTallRows - 1) / kTallRows * kTallRows;
    const int splits = (int)((k + chunk - 1) / chunk);
    // 32-bit byte offsets inside a workgroup's rows
    const long long ld = lda > ldb ? lda : ldb;
    if ((chunk + kTallRows) * ld * 4 >= (1ll << 31)) return GNNHIP_EUNSUPPORTED;
    void* q = nullptr;
    if (int rc = stream_scratch_slot(s, 2, sizeof(float) * (size_t)splits * MT * MT, &q)) return rc;
    float* partial = static_cast<float*>(q);
    const size_t smem = sizeof(float) * 2 * 2 * kTallRows * (MT + 16);
    static LdsLimit lds_limit;
    GNNHIP_HIP(lds_limit.raise(reinterpret_cast<const void*>(&sgemm_tn_tall_kernel<MT>), smem));
    hipLaunchKernelGGL((sgemm_tn_tall_kernel<MT>), dim3((unsigned)splits), dim3(kTallBlock), smem, s, k, (int)chunk, A, lda, B, ldb, partial);
    GNNHIP_LAUNCH_CHECK("sgemm_tn_tall");
    launch_splitk_reduce(MT, MT, splits, alpha, partial, beta, C, ldc, s);
    GNNHIP_LAUNCH_CHECK("sgemm_tn_tall sums");
    return GNNHIP_OK;
}

}  // namespace

// Whether a product A^T B ([k, m]^T [k, n]) takes this route; the batch of weight gradients asks so that such a product
// gets the bits it has when done alone.
bool gemm_tn_tall_applies(int m, int n, int k, const float* A, int lda, const float* B, int ldb)
{
    return m == n && (m == 128 || m == 256) && k >= kTallMinK && lda % 4 == 0 && ldb % 4 == 0 && aligned16(A) && aligned16(B);
}

int gemm_tn_tall_dispatch(int m, int n, int k, float alpha, const float* A, int lda, const float* B, int ldb, float beta, float* C,
                          int ldc, hipStream_t s)
{
    if (!gemm_tn_tall_applies(m, n, k, A, lda, B, ldb)) return GNNHIP_EUNSUPPORTED;
    return m == 128 ? launch_tall<128>(k, alpha, A, lda, B, ldb, beta, C, ldc, s)
                    : launch_tall<256>(k, alpha, A, lda, B, ldb, beta, C, ldc, s);
}

}  // namespace gnnhip
