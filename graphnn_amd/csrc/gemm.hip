// Dense fp32 GEMM for gfx950:  C[m,n] = alpha * op(A) * op(B) + beta * C, row-major.
//
// The mean-field path only has tall-and-skinny products (m = nodes or graphs,
// n and k = label types / hidden sizes <= 256), which are HBM-bound: every A
// element is used n times from LDS, every B element lives in L2.  The kernel is
// an LDS-tiled SGEMM on the FP32 matrix cores: a 64 x 64 output tile per 256-lane
// workgroup, 16 rows x 64 columns per wavefront as four v_mfma_f32_16x16x4_f32
// accumulators, K walked in steps of 16 through two LDS tiles.  Edges are handled
// by bounds-checked tile loads (zeros) and stores.
// Bound: HBM for the shapes above; algorithmic bytes 4(mk + kn + mn).
//
// Weight gradients are the opposite shape: op(A)^T * G with a small output (hidden x hidden) and k = nodes.
// One output tile would walk all of k on one CU (1.1 ms at k = 7,450; 15 us at k = 256, a microsecond per step of 16),
// so such products are split along k from k = 256:
// every workgroup takes a range of k, writes its partial tile to scratch, and a second kernel adds the
// partial tiles in range order (deterministic) and applies alpha and beta.
#include "gnnhip_internal.h"

namespace gnnhip {
namespace {

constexpr int BM = 64, BN = 64, BK = 16, kBlock = 256;

// One 64 x 64 output tile (tile_x, tile_y) over k in [k_lo, k_hi).  part != nullptr: the raw sums go to
// part[m][n]; otherwise the tile finishes C itself.
template <bool TA, bool TB>
__device__ __forceinline__ void sgemm_tile_body(
    int m, int n, float alpha, const float* __restrict__ A, int lda,
    const float* __restrict__ B, int ldb, float beta, float* C, int ldc, int k_lo, int k_hi, float* __restrict__ part,
    int tile_x, int tile_y)
{
    // Both tiles sit in LDS with k contiguous, so that a lane fetches its four k values of a step with one
    // 128-bit read.  Wavefront w owns the output rows 16 w .. 16 w + 15 of the tile and all 64 columns: four
    // accumulators of v_mfma_f32_16x16x4_f32 with the operand roles swapped (out^T = B^T * A^T), which leaves
    // lane (q = lane/16, t = lane%16) with row t and the columns 16 jb + 4 q .. + 3 of block jb.
    constexpr int LD = BK + 4;
    __shared__ float As[BM][LD];         // As[i][p] = op(A)[row0 + i][k0 + p]
    __shared__ float Bs[BN][LD];         // Bs[j][p] = op(B)[k0 + p][col0 + j]

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int q = lane >> 4, t = lane & 15;
    const long long row0 = (long long)tile_x * BM;
    const int col0 = tile_y * BN;

    mfma_f4 acc[BN / 16];
#pragma unroll
    for (int jb = 0; jb < BN / 16; ++jb) acc[jb] = mfma_f4{0.f, 0.f, 0.f, 0.f};

    // each lane moves 4 elements of each tile; the elements of step k0 + BK are requested before the
    // products of step k0 are formed, so a step costs the longer of the two instead of their sum
    float ra[4], rb[4];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = tid + e * kBlock;        // 0 .. 1023
            {
                // A tile: the fast index follows memory
                int i, p;
                if (TA) { i = idx & (BM - 1); p = idx >> 6; }       // stored A is [k][m]: i contiguous
                else    { p = idx & (BK - 1); i = idx >> 4; }       // stored A is [m][k]: p contiguous
                const long long gi = row0 + i;
                const int gp = k0 + p;
                float v = 0.f;
                if (gi < m && gp < k_hi) v = TA ? A[(size_t)gp * lda + gi] : A[(size_t)gi * lda + gp];
                ra[e] = v;
            }
            {
                int j, p;
                if (TB) { p = idx & (BK - 1); j = idx >> 4; }       // stored B is [n][k]: p contiguous
                else    { j = idx & (BN - 1); p = idx >> 6; }       // stored B is [k][n]: j contiguous
                const int gj = col0 + j;
                const int gp = k0 + p;
                float v = 0.f;
                if (gj < n && gp < k_hi) v = TB ? B[(size_t)gj * ldb + gp] : B[(size_t)gp * ldb + gj];
                rb[e] = v;
            }
        }
    };
    if (k_lo < k_hi) fetch(k_lo);
    for (int k0 = k_lo; k0 < k_hi; k0 += BK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int idx = tid + e * kBlock;
            if (TA) As[idx & (BM - 1)][idx >> 6] = ra[e]; else As[idx >> 4][idx & (BK - 1)] = ra[e];
            if (TB) Bs[idx >> 4][idx & (BK - 1)] = rb[e]; else Bs[idx & (BN - 1)][idx >> 6] = rb[e];
        }
        __syncthreads();
        if (k0 + BK < k_hi) fetch(k0 + BK);
        // lane (q, t): k = 4 q + s at instruction s of the step
        const float4 a = *reinterpret_cast<const float4*>(&As[wave * 16 + t][4 * q]);
#pragma unroll
        for (int jb = 0; jb < BN / 16; ++jb) {
            const float4 b = *reinterpret_cast<const float4*>(&Bs[jb * 16 + t][4 * q]);
            acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.x, a.x, acc[jb], 0, 0, 0);
            acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.y, a.y, acc[jb], 0, 0, 0);
            acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.z, a.z, acc[jb], 0, 0, 0);
            acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b.w, a.w, acc[jb], 0, 0, 0);
        }
        __syncthreads();
    }

    // lane (q, t) holds out[row0 + 16 wave + t][col0 + 16 jb + 4 q + i], i = 0..3
    const long long gi = row0 + wave * 16 + t;
    if (gi < m) {
#pragma unroll
        for (int jb = 0; jb < BN / 16; ++jb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int gj = col0 + jb * 16 + 4 * q + i;
                if (gj >= n) continue;
                if (part) {
                    part[(size_t)gi * n + gj] = acc[jb][i];
                    continue;
                }
                float* dst = C + (size_t)gi * ldc + gj;
                const float r = alpha * acc[jb][i];
                *dst = (beta == 0.f) ? r : r + beta * (*dst);
            }
        }
    }
}

// partial != nullptr: workgroup z handles k in [z k_chunk, (z+1) k_chunk) and stores its raw sums to
// partial[z][m][n]; otherwise one workgroup walks all of k and finishes C itself.
template <bool TA, bool TB>
__global__ __launch_bounds__(kBlock) void sgemm_tile_kernel(
    int m, int n, int k, float alpha, const float* __restrict__ A, int lda,
    const float* __restrict__ B, int ldb, float beta, float* C, int ldc, int k_chunk, float* __restrict__ partial)
{
    const int k_lo = partial ? (int)blockIdx.z * k_chunk : 0;
    const int k_hi = partial ? min(k, k_lo + k_chunk) : k;
    sgemm_tile_body<TA, TB>(m, n, alpha, A, lda, B, ldb, beta, C, ldc, k_lo, k_hi,
                            partial ? partial + (size_t)blockIdx.z * m * n : nullptr, (int)blockIdx.x, (int)blockIdx.y);
}

// Several products C_p = alpha A_p^T B_p + beta C_p in one launch: the weight gradients at the end of a backward
// pass, each a small output over a long k, none of which fills the GPU alone.  Product p owns the z range
// [z0[p], z0[p+1]) of the grid, one range of k per z; tiles outside a product's own tile grid leave at once.
constexpr int kGemmBatch = 8;
struct GemmBatch {
    const float* A[kGemmBatch];
    const float* B[kGemmBatch];
    float* C[kGemmBatch];
    float* partial[kGemmBatch];
    int m[kGemmBatch], n[kGemmBatch], k[kGemmBatch], lda[kGemmBatch], ldb[kGemmBatch], ldc[kGemmBatch];
    int k_chunk[kGemmBatch], z0[kGemmBatch + 1];
    int count;
};

__global__ __launch_bounds__(kBlock) void sgemm_tn_batch_kernel(GemmBatch b)
{
    int p = 0;
    while (p + 1 < b.count && (int)blockIdx.z >= b.z0[p + 1]) ++p;
    const int m = b.m[p], n = b.n[p];
    if ((long long)blockIdx.x * BM >= m || (int)blockIdx.y * BN >= n) return;
    const int z = (int)blockIdx.z - b.z0[p];
    const int k_lo = z * b.k_chunk[p], k_hi = min(b.k[p], k_lo + b.k_chunk[p]);
    sgemm_tile_body<true, false>(m, n, 1.0f, b.A[p], b.lda[p], b.B[p], b.ldb[p], 0.0f, b.C[p], b.ldc[p], k_lo, k_hi,
                                 b.partial[p] + (size_t)z * m * n, (int)blockIdx.x, (int)blockIdx.y);
}

// C = alpha * (sum over z of partial[z]) + beta * C.  A workgroup takes 64 consecutive elements; wavefront w
// adds the ranges z = w, w + 4, ... (up to sixteen loads in flight per lane) and the four sums are added in
// wavefront order, so the result is the same on every run.
__device__ __forceinline__ void sgemm_splitk_reduce_body(int m, int n, int splits, float alpha,
                                                         const float* __restrict__ partial, float beta,
                                                         float* C, int ldc)
{
    __shared__ float part[kBlock / kWave][kWave];
    const size_t total = (size_t)m * n;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    constexpr int kWaves = kBlock / kWave;
    for (size_t base = (size_t)blockIdx.x * kWave; base < total; base += (size_t)gridDim.x * kWave) {
        const size_t idx = base + lane;
        float sum = 0.f;
        float* dst = C + (idx / n) * (size_t)ldc + idx % n;
        const float c_old = (wave == 0 && idx < total && beta != 0.f) ? *dst : 0.f;      // asked for before the sums, not after
        if (idx < total) {
            int z = wave;
            for (; z + 15 * kWaves < splits; z += 16 * kWaves) {
                float p[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) p[u] = partial[(size_t)(z + u * kWaves) * total + idx];
#pragma unroll
                for (int u = 0; u < 16; ++u) sum += p[u];
            }
            for (; z + 3 * kWaves < splits; z += 4 * kWaves) {
                const float p0 = partial[(size_t)z * total + idx], p1 = partial[(size_t)(z + kWaves) * total + idx];
                const float p2 = partial[(size_t)(z + 2 * kWaves) * total + idx], p3 = partial[(size_t)(z + 3 * kWaves) * total + idx];
                sum += p0; sum += p1; sum += p2; sum += p3;
            }
            for (; z < splits; z += kWaves) sum += partial[(size_t)z * total + idx];
        }
        part[wave][lane] = sum;
        __syncthreads();
        if (wave == 0 && idx < total) {
            float t = part[0][lane];
#pragma unroll
            for (int w = 1; w < kWaves; ++w) t += part[w][lane];
            const float r = alpha * t;
            *dst = (beta == 0.f) ? r : r + beta * c_old;
        }
        __syncthreads();
    }
}

__global__ __launch_bounds__(kBlock) void sgemm_splitk_reduce_kernel(int m, int n, int splits, float alpha,
                                                                     const float* __restrict__ partial, float beta,
                                                                     float* C, int ldc)
{
    sgemm_splitk_reduce_body(m, n, splits, alpha, partial, beta, C, ldc);
}

// the sums of product blockIdx.y of a batch
__global__ __launch_bounds__(kBlock) void sgemm_splitk_reduce_batch_kernel(GemmBatch b, float alpha, float beta)
{
    const int p = blockIdx.y;
    sgemm_splitk_reduce_body(b.m[p], b.n[p], b.z0[p + 1] - b.z0[p], alpha, b.partial[p], beta, b.C[p], b.ldc[p]);
}

}  // namespace

namespace {

// ---- tall A times a matrix of at most four columns (node scores h * w, readouts with one or two
// classes): a group of G lanes walks one row of A in 128-bit pieces and reduces with shuffles.
// Reads A once at streaming rate; the tile kernel would spend a 64-column tile on it.
template <int NCOL, bool TB>
__global__ __launch_bounds__(kBlock) void sgemm_skinny_kernel(
    int m, int k, float alpha, const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb,
    float beta, float* C, int ldc, int logG)
{
    const int G = 1 << logG;
    const int sub = threadIdx.x & (G - 1);
    const long long row = ((long long)blockIdx.x * kBlock + threadIdx.x) >> logG;
    float acc[NCOL];
#pragma unroll
    for (int j = 0; j < NCOL; ++j) acc[j] = 0.f;
    if (row < m) {
        const float* a = A + (size_t)row * lda;
        for (int kk = sub * 4; kk < k; kk += G * 4) {
            const float4 x = *reinterpret_cast<const float4*>(a + kk);
#pragma unroll
            for (int j = 0; j < NCOL; ++j) {
                const float b0 = TB ? B[(size_t)j * ldb + kk] : B[(size_t)kk * ldb + j];
                const float b1 = TB ? B[(size_t)j * ldb + kk + 1] : B[(size_t)(kk + 1) * ldb + j];
                const float b2 = TB ? B[(size_t)j * ldb + kk + 2] : B[(size_t)(kk + 2) * ldb + j];
                const float b3 = TB ? B[(size_t)j * ldb + kk + 3] : B[(size_t)(kk + 3) * ldb + j];
                acc[j] += x.x * b0 + x.y * b1 + x.z * b2 + x.w * b3;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < NCOL; ++j)
        for (int d = G >> 1; d >= 1; d >>= 1) acc[j] += __shfl_xor(acc[j], d, kWave);
    if (row < m && sub == 0) {
#pragma unroll
        for (int j = 0; j < NCOL; ++j) {
            float* c = C + (size_t)row * ldc + j;
            *c = (beta == 0.f) ? alpha * acc[j] : alpha * acc[j] + beta * *c;
        }
    }
}

// The same product for k <= 256: a lane keeps its four rows of B in registers, the groups stride the rows of A
// eight at a time (eight 128-bit loads in flight per lane), and groups of up to 16 lanes reduce with DPP.
template <int NCOL, bool TB>
__global__ __launch_bounds__(kBlock) void sgemm_skinny_rows_kernel(
    int m, int k, float alpha, const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb,
    float beta, float* C, int ldc, int logG)
{
    constexpr int R = 8;
    const int G = 1 << logG;
    const int sub = threadIdx.x & (G - 1);
    const int kk = sub * 4;
    const bool live = kk < k;                              // k is a multiple of 4
    float4 b[NCOL];
#pragma unroll
    for (int j = 0; j < NCOL; ++j) {
        b[j] = f4_zero();
        if (live) {
            b[j].x = TB ? B[(size_t)j * ldb + kk] : B[(size_t)kk * ldb + j];
            b[j].y = TB ? B[(size_t)j * ldb + kk + 1] : B[(size_t)(kk + 1) * ldb + j];
            b[j].z = TB ? B[(size_t)j * ldb + kk + 2] : B[(size_t)(kk + 2) * ldb + j];
            b[j].w = TB ? B[(size_t)j * ldb + kk + 3] : B[(size_t)(kk + 3) * ldb + j];
        }
    }
    // A workgroup walks one contiguous run of rows (its groups side by side, R turns ahead), so that what is in flight
    // from one workgroup is one stretch of memory.  All lanes of a wavefront run the same number of iterations (the
    // reductions are wavefront-wide operations).
    const int groups = kBlock >> logG;
    const int group = threadIdx.x >> logG;
    const long long per_block = ((long long)m + gridDim.x - 1) / gridDim.x;
    const long long row0 = (long long)blockIdx.x * per_block;
    const long long row1 = row0 + per_block < m ? row0 + per_block : m;
    for (long long base = row0; base < row1; base += R * groups) {
        float4 x[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const long long row = base + r * groups + group;
            x[r] = (live && row < row1) ? *reinterpret_cast<const float4*>(A + (size_t)row * lda + kk) : f4_zero();
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const long long row = base + r * groups + group;
#pragma unroll
            for (int j = 0; j < NCOL; ++j) {
                float acc = x[r].x * b[j].x + x[r].y * b[j].y + x[r].z * b[j].z + x[r].w * b[j].w;
                if (G >= 2) acc += dpp_mov_f<kDppXor1>(acc);
                if (G >= 4) acc += dpp_mov_f<kDppXor2>(acc);
                if (G >= 8) acc += dpp_mov_f<kDppHalfMirror>(acc);
                if (G >= 16) acc += dpp_mov_f<kDppMirror>(acc);
                if (G >= 32) acc += __shfl_xor(acc, 16, kWave);
                if (G >= 64) acc += __shfl_xor(acc, 32, kWave);
                if (row < row1 && sub == 0) {
                    float* c = C + (size_t)row * ldc + j;
                    *c = (beta == 0.f) ? alpha * acc : alpha * acc + beta * *c;
                }
            }
        }
    }
}

template <int NCOL>
void launch_skinny(bool tb, int m, int k, float alpha, const float* A, int lda, const float* B, int ldb,
                   float beta, float* C, int ldc, hipStream_t s)
{
    int logG = 0;
    while ((4 << logG) < k && logG < 6) ++logG;              // G * 4 >= k, at most one wavefront per row
    if (k <= 4 * kWave) {
        const size_t lanes = (size_t)m << logG;
        size_t blocks = ceil_div_u(ceil_div_u(lanes, 8), kBlock);          // eight rows per group
        if (blocks > (size_t)kNumCU * 32) blocks = (size_t)kNumCU * 32;
        if (blocks < 1) blocks = 1;
        const unsigned grid = (unsigned)blocks;
        if (tb) hipLaunchKernelGGL((sgemm_skinny_rows_kernel<NCOL, true>), dim3(grid), dim3(kBlock), 0, s, m, k, alpha, A, lda, B, ldb, beta, C, ldc, logG);
        else hipLaunchKernelGGL((sgemm_skinny_rows_kernel<NCOL, false>), dim3(grid), dim3(kBlock), 0, s, m, k, alpha, A, lda, B, ldb, beta, C, ldc, logG);
        return;
    }
    const unsigned grid = ceil_div_u((size_t)m << logG, kBlock);
    if (tb) hipLaunchKernelGGL((sgemm_skinny_kernel<NCOL, true>), dim3(grid), dim3(kBlock), 0, s, m, k, alpha, A, lda, B, ldb, beta, C, ldc, logG);
    else hipLaunchKernelGGL((sgemm_skinny_kernel<NCOL, false>), dim3(grid), dim3(kBlock), 0, s, m, k, alpha, A, lda, B, ldb, beta, C, ldc, logG);
}

}  // namespace

// gemm_tn_tall.hip: square outputs of 128 / 256 over a very long k
bool gemm_tn_tall_applies(int m, int n, int k, const float* A, int lda, const float* B, int ldb);
int gemm_tn_tall_dispatch(int m, int n, int k, float alpha, const float* A, int lda, const float* B, int ldb, float beta, float* C,
                          int ldc, hipStream_t s);

void launch_splitk_reduce(int m, int n, int splits, float alpha, const float* partial, float beta, float* C, int ldc, hipStream_t s)
{
    const size_t total = (size_t)m * n;
    const unsigned rgrid = ceil_div_u(total, kWave) < 2048u ? ceil_div_u(total, kWave) : 2048u;
    hipLaunchKernelGGL(sgemm_splitk_reduce_kernel, dim3(rgrid), dim3(kBlock), 0, s, m, n, splits, alpha, partial, beta, C, ldc);
}

// length of the ranges of k when few output tiles share a long k: about two workgroups per CU, four steps at least
inline long long splitk_chunk(long long tiles, long long k)
{
    const long long want = (2 * kNumCU) / tiles;                           // ranges per tile
    long long chunk = (k + want - 1) / want;
    if (chunk < 4 * BK) chunk = 4 * BK;
    return (chunk + BK - 1) / BK * BK;
}

// count <= kGemmBatch products C_p = alpha A_p^T B_p + beta C_p (A_p stored [k_p, m_p], B_p [k_p, n_p]) in two launches
int gemm_tn_batch_dispatch(int count, const int* m, const int* n, const int* k, const float* const* A, const int* lda,
                           const float* const* B, const int* ldb, float alpha, float beta, float* const* C, const int* ldc, hipStream_t s)
{
    GemmBatch b;
    b.count = 0;
    size_t floats = 0;
    unsigned gx = 1, gy = 1, red = 1;
    size_t offset[kGemmBatch];
    int z = 0;
    for (int p = 0; p < count; ++p) {
        if (m[p] == 0 || n[p] == 0) continue;
        // the rule of the single product here too: a wide square output over a very long k has a kernel of its own
        if (gemm_tn_tall_applies(m[p], n[p], k[p], A[p], lda[p], B[p], ldb[p])) {
            if (int rc = gemm_tn_tall_dispatch(m[p], n[p], k[p], alpha, A[p], lda[p], B[p], ldb[p], beta, C[p], ldc[p], s)) return rc;
            continue;
        }
        const int q = b.count++;
        b.A[q] = A[p]; b.B[q] = B[p]; b.C[q] = C[p];
        b.m[q] = m[p]; b.n[q] = n[p]; b.k[q] = k[p];
        b.lda[q] = lda[p]; b.ldb[q] = ldb[p]; b.ldc[q] = ldc[p];
        const unsigned tx = ceil_div_u((size_t)m[p], BM), ty = ceil_div_u((size_t)n[p], BN);
        const long long tiles = (long long)tx * ty;
        // the rule of the single product, so that a batch gives the bits of its products done one by one
        long long chunk = (tiles <= kNumCU / 4 && k[p] >= 256) ? splitk_chunk(tiles, k[p]) : (k[p] > 0 ? k[p] : 1);
        const int splits = k[p] > 0 ? (int)(((long long)k[p] + chunk - 1) / chunk) : 1;
        b.k_chunk[q] = (int)chunk;
        b.z0[q] = z;
        z += splits;
        offset[q] = floats;
        floats += (size_t)splits * m[p] * n[p];
        if (tx > gx) gx = tx;
        if (ty > gy) gy = ty;
        const unsigned r = ceil_div_u((size_t)m[p] * n[p], kWave) < 2048u ? ceil_div_u((size_t)m[p] * n[p], kWave) : 2048u;
        if (r > red) red = r;
    }
    if (b.count == 0) return GNNHIP_OK;
    b.z0[b.count] = z;
    void* q = nullptr;
    if (int rc = stream_scratch_slot(s, 2, sizeof(float) * floats, &q)) return rc;
    for (int p = 0; p < b.count; ++p) b.partial[p] = static_cast<float*>(q) + offset[p];
    hipLaunchKernelGGL(sgemm_tn_batch_kernel, dim3(gx, gy, (unsigned)z), dim3(kBlock), 0, s, b);
    hipLaunchKernelGGL(sgemm_splitk_reduce_batch_kernel, dim3(red, (unsigned)b.count), dim3(kBlock), 0, s, b, alpha, beta);
    GNNHIP_LAUNCH_CHECK("sgemm_tn_batch");
    return GNNHIP_OK;
}

int gemm_dispatch(int transA, int transB, int m, int n, int k, float alpha, const float* A, int lda,
                  const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s)
{
    if (!transA && n <= 4 && m >= 4096 && k >= 4 && k % 4 == 0 && lda % 4 == 0 && aligned16(A)) {
        switch (n) {
        case 1: launch_skinny<1>(transB, m, k, alpha, A, lda, B, ldb, beta, C, ldc, s); break;
        case 2: launch_skinny<2>(transB, m, k, alpha, A, lda, B, ldb, beta, C, ldc, s); break;
        case 3: launch_skinny<3>(transB, m, k, alpha, A, lda, B, ldb, beta, C, ldc, s); break;
        default: launch_skinny<4>(transB, m, k, alpha, A, lda, B, ldb, beta, C, ldc, s); break;
        }
        GNNHIP_LAUNCH_CHECK("sgemm_skinny");
        return GNNHIP_OK;
    }
    if (transA && !transB) {
        if (int rc = gemm_tn_tall_dispatch(m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, s); rc != GNNHIP_EUNSUPPORTED) return rc;
    }
    dim3 grid(ceil_div_u((size_t)m, BM), ceil_div_u((size_t)n, BN));
    dim3 block(kBlock);
    // few output tiles and a long k: split k so that about two workgroups per CU share the work
    int k_chunk = 0;
    float* partial = nullptr;
    const long long tiles = (long long)grid.x * grid.y;
    if (tiles <= kNumCU / 4 && k >= 256) {
        const long long chunk = splitk_chunk(tiles, k);
        const int splits = (int)(((long long)k + chunk - 1) / chunk);
        if (splits > 1) {
            void* q = nullptr;
            if (int rc = stream_scratch_slot(s, 2, sizeof(float) * (size_t)splits * m * n, &q)) return rc;
            partial = static_cast<float*>(q);
            k_chunk = (int)chunk;
            grid.z = splits;
        }
    }
    if (!transA && !transB)
        hipLaunchKernelGGL((sgemm_tile_kernel<false, false>), grid, block, 0, s, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    else if (transA && !transB)
        hipLaunchKernelGGL((sgemm_tile_kernel<true, false>), grid, block, 0, s, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    else if (!transA && transB)
        hipLaunchKernelGGL((sgemm_tile_kernel<false, true>), grid, block, 0, s, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    else
        hipLaunchKernelGGL((sgemm_tile_kernel<true, true>), grid, block, 0, s, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, k_chunk, partial);
    if (partial) {
        const size_t total = (size_t)m * n;
        const unsigned rgrid = ceil_div_u(total, kWave) < 2048u ? ceil_div_u(total, kWave) : 2048u;
        hipLaunchKernelGGL(sgemm_splitk_reduce_kernel, dim3(rgrid), block, 0, s, m, n, (int)grid.z, alpha, partial, beta, C, ldc);
    }
    GNNHIP_LAUNCH_CHECK("sgemm_tile");
    return GNNHIP_OK;
}

}  // namespace gnnhip

using namespace gnnhip;

extern "C" int gnnhip_gemm_f32(int transA, int transB, int m, int n, int k, float alpha, const float* A, int lda,
                               const float* B, int ldb, float beta, float* C, int ldc, void* stream)
{
    GNNHIP_REQUIRE(m >= 0 && n >= 0 && k >= 0, "negative dimension in gemm (m=%d n=%d k=%d)", m, n, k);
    GNNHIP_REQUIRE((transA == 0 || transA == 1) && (transB == 0 || transB == 1), "trans flags must be 0 or 1");
    if (m == 0 || n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(C != nullptr && ldc >= n, "bad output in gemm (ldc=%d n=%d)", ldc, n);
    if (k > 0) {
        GNNHIP_REQUIRE(A && B, "null operand in gemm");
        GNNHIP_REQUIRE(lda >= (transA ? m : k), "lda=%d too small", lda);
        GNNHIP_REQUIRE(ldb >= (transB ? k : n), "ldb=%d too small", ldb);
    }
    GNNHIP_REQUIRE(ceil_div_u((size_t)n, 64) <= 65535u, "n=%d too wide for the gemm grid", n);
    if (int rc = require_ready()) return rc;
    return gemm_dispatch(transA, transB, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc, as_stream(stream));
}

extern "C" int gnnhip_gemm_tn_batch_f32(int count, const int* m, const int* n, const int* k, const float* const* A, const int* lda,
                                        const float* const* B, const int* ldb, float alpha, float beta, float* const* C, const int* ldc,
                                        void* stream)
{
    GNNHIP_REQUIRE(count >= 0, "negative count in gemm_tn_batch");
    if (count == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(m && n && k && A && lda && B && ldb && C && ldc, "null array in gemm_tn_batch");
    for (int p = 0; p < count; ++p) {
        GNNHIP_REQUIRE(m[p] >= 0 && n[p] >= 0 && k[p] >= 0, "negative dimension in gemm_tn_batch (product %d: m=%d n=%d k=%d)", p, m[p], n[p], k[p]);
        if (m[p] == 0 || n[p] == 0) continue;
        GNNHIP_REQUIRE(C[p] != nullptr && ldc[p] >= n[p], "bad output in gemm_tn_batch (product %d: ldc=%d n=%d)", p, ldc[p], n[p]);
        GNNHIP_REQUIRE(k[p] == 0 || (A[p] && B[p] && lda[p] >= m[p] && ldb[p] >= n[p]), "bad operand in gemm_tn_batch (product %d)", p);
        GNNHIP_REQUIRE(ceil_div_u((size_t)n[p], 64) <= 65535u, "n=%d too wide for the gemm grid", n[p]);
    }
    if (int rc = require_ready()) return rc;
    for (int at = 0; at < count; at += kGemmBatch) {
        const int take = count - at < kGemmBatch ? count - at : kGemmBatch;
        if (int rc = gemm_tn_batch_dispatch(take, m + at, n + at, k + at, A + at, lda + at, B + at, ldb + at, alpha, beta, C + at, ldc + at,
                                            as_stream(stream)))
            return rc;
    }
    return GNNHIP_OK;
}
