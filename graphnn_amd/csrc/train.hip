// Kernels that shorten one training iteration of the structure2vec path on gfx950:
//
//   loss / accuracy tail     softmax cross-entropy rows, their mean, label arg-max, in-top-1 and its mean in one
//                            pass over the logits (CrossEntropy -> ReduceMean, ArgMax -> InTopK -> TypeCast ->
//                            ReduceMean: eight launches of the operator-by-operator plan)
//   readout backward         per graph: dlogits = scale (probs - y), du = (dlogits W_h2^T) . [hidden > 0],
//                            dpool = du W_h1^T, and the gradient rows of the graph's nodes, s_val dpool
//   gradient gate            dz = g . [h > 0] and the running sum of dz over the levels (the gradient of msg)
//   parameter update         momentum SGD over every tensor of a parameter set in one launch
//
// All of them are launch- or HBM-bound; the dense products of the backward pass stay with gemm.hip / spmm.hip.
#include "gnnhip_internal.h"

namespace gnnhip {
// gemm.hip
int gemm_dispatch(int transA, int transB, int m, int n, int k, float alpha, const float* A, int lda,
                  const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s);

namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

// ------------------------------------------------------------------ loss / accuracy tail
// One lane per row: probabilities as DTensor::Softmax forms them (max-subtracted, src/tensor/gpu_dense_tensor.cu:298-370),
// loss row as CalcCrossEntropy (clamp of src/nn/cross_entropy.cpp:18-19, log in double), truth = column of the
// largest label value (first among ties, empty row -> 0: src/tensor/cpu_sparse_tensor.cpp:86-103), hit = fewer
// than one logit above the truth's (src/nn/in_top_k.cpp:6-23).  Partial sums per workgroup, combined in index order.
__global__ __launch_bounds__(kBlock) void loss_acc_partial_kernel(int B, int Q, const float* __restrict__ logits,
                                                                  const int* __restrict__ lrow_ptr, const int* __restrict__ lcol,
                                                                  const float* __restrict__ lval, float* __restrict__ probs,
                                                                  float* __restrict__ loss_rows, int* __restrict__ hit_rows,
                                                                  float* __restrict__ partial /* [2][gridDim.x] */,
                                                                  float* __restrict__ loss_mean, float* __restrict__ acc_mean)
{
    __shared__ float sh_loss[kWavesPerBlock], sh_hit[kWavesPerBlock];
    const int per = (B + gridDim.x - 1) / gridDim.x;
    const int lo = blockIdx.x * per, hi = min(B, lo + per);
    float loss_sum = 0.f, hit_sum = 0.f;
    for (int r = lo + threadIdx.x; r < hi; r += kBlock) {
        const float* x = logits + (size_t)r * Q;
        float mx = x[0];
        for (int j = 1; j < Q; ++j) mx = max_keep(mx, x[j]);
        float s = 0.f;
        for (int j = 0; j < Q; ++j) s += expf(x[j] - mx);
        // label row: loss and truth
        const int a = lrow_ptr[r], b = lrow_ptr[r + 1];
        float loss = 0.f, cur = 0.f;
        int truth = 0;
        for (int k = a; k < b; ++k) {
            const int c = lcol[k];
            float t = expf(x[c] - mx) / s;
            if (fabs((double)t) < 1e-8) t = (float)1e-8;
            loss = (float)((double)loss - log((double)t) * (double)lval[k]);
            if (k == a || lval[k] > cur) { cur = lval[k]; truth = c; }
        }
        if (probs) for (int j = 0; j < Q; ++j) probs[(size_t)r * Q + j] = expf(x[j] - mx) / s;
        const float pt = x[truth];
        int above = 0;
        for (int j = 0; j < Q; ++j) above += (j != truth && x[j] > pt) ? 1 : 0;
        const int hit = above < 1 ? 1 : 0;
        if (loss_rows) loss_rows[r] = loss;
        if (hit_rows) hit_rows[r] = hit;
        loss_sum += loss;
        hit_sum += (float)hit;
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    loss_sum = wave_sum(loss_sum);
    hit_sum = wave_sum(hit_sum);
    if (lane == 0) { sh_loss[wave] = loss_sum; sh_hit[wave] = hit_sum; }
    __syncthreads();
    if (threadIdx.x == 0) {
        float l = 0.f, h = 0.f;
        for (int w = 0; w < kWavesPerBlock; ++w) { l += sh_loss[w]; h += sh_hit[w]; }
        if (gridDim.x == 1) {
            // a single workgroup has the whole sums: the means leave from here, as loss_acc_final_kernel would form them
            if (loss_mean) loss_mean[0] = l / (float)B;
            if (acc_mean) acc_mean[0] = h / (float)B;
            return;
        }
        partial[blockIdx.x] = l;
        partial[gridDim.x + blockIdx.x] = h;
    }
}

__global__ __launch_bounds__(kWave) void loss_acc_final_kernel(int nb, int B, const float* __restrict__ partial,
                                                               float* __restrict__ loss_mean, float* __restrict__ acc_mean)
{
    float l = 0.f, h = 0.f;
    for (int i = threadIdx.x; i < nb; i += kWave) { l += partial[i]; h += partial[nb + i]; }
    l = wave_sum(l);
    h = wave_sum(h);
    if (threadIdx.x == 0) {
        if (loss_mean) loss_mean[0] = l / (float)B;
        if (acc_mean) acc_mean[0] = h / (float)B;
    }
}

// ------------------------------------------------------------------ readout backward, one workgroup per graph
// LDS: dlogits[Q] | du[H] | dpool[C].  The three small products run on the lanes that own their outputs; the
// graph's gradient rows (its nodes x C) are then written by all lanes, row-contiguous.
__global__ __launch_bounds__(kBlock) void readout_backward_kernel(
    int B, int C, int H, int Q, const int* __restrict__ s_row_ptr, const int* __restrict__ s_col_idx, const float* __restrict__ s_val,
    const float* __restrict__ probs, const int* __restrict__ lrow_ptr, const int* __restrict__ lcol, const float* __restrict__ lval,
    float scale, const float* __restrict__ hidden, const float* __restrict__ Wh1, const float* __restrict__ Wh2,
    float* __restrict__ dlogits, float* __restrict__ du, float* __restrict__ g_h, int head_only)
{
    extern __shared__ float smem[];
    float* dl = smem;
    float* duw = dl + Q;
    float* dp = duw + H;
    const int tid = threadIdx.x;
    for (int g = blockIdx.x; g < B; g += gridDim.x) {
        // dlogits = scale * (probs - y): CrossEntropy::Backward with softmax inside (src/nn/cross_entropy.cpp:52-78),
        // scale = the gradient ReduceMean hands to every row (src/nn/reduce_mean.cpp:44-65)
        for (int q = tid; q < Q; q += kBlock) {
            float y = 0.f;
            for (int k = lrow_ptr[g]; k < lrow_ptr[g + 1]; ++k) if (lcol[k] == q) y += lval[k];
            const float v = (probs[(size_t)g * Q + q] - y) * scale;
            dl[q] = v;
            dlogits[(size_t)g * Q + q] = v;
        }
        __syncthreads();
        // du = (dlogits W_h2^T) . [hidden > 0]
        for (int j = tid; j < H; j += kBlock) {
            float s = 0.f;
            for (int q = 0; q < Q; ++q) s = fmaf(dl[q], Wh2[(size_t)j * Q + q], s);
            const float v = hidden[(size_t)g * H + j] > 0.f ? s : 0.f;
            duw[j] = v;
            du[(size_t)g * H + j] = v;
        }
        __syncthreads();
        if (head_only) continue;                // large batches: dpool for all graphs as one product, rows by the kernel below
        // dpool = du W_h1^T
        for (int c = tid; c < C; c += kBlock) {
            float s = 0.f;
            for (int j = 0; j < H; ++j) s = fmaf(duw[j], Wh1[(size_t)c * H + j], s);
            dp[c] = s;
        }
        __syncthreads();
        // gradient rows of the graph's nodes: S^T dpool restricted to this graph (every node is listed once)
        const int a = s_row_ptr[g];
        const int total = (s_row_ptr[g + 1] - a) * C;
        for (int i = tid; i < total; i += kBlock) {
            const int r = i / C, c = i - r * C;
            g_h[(size_t)s_col_idx[a + r] * C + c] = s_val[a + r] * dp[c];
        }
        __syncthreads();
    }
}

// Large batches: g_h[node] = s_val * dpool[graph of node], one workgroup per graph, a wavefront per node row (the
// graph's dpool row is read once per wavefront and stays in registers while its node rows are written).
__global__ __launch_bounds__(kBlock) void readout_backward_rows_kernel(int B, int C, const int* __restrict__ s_row_ptr,
                                                                       const int* __restrict__ s_col_idx, const float* __restrict__ s_val,
                                                                       const float* __restrict__ dpool, float* __restrict__ g_h)
{
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    constexpr int kWaves = kBlock / kWave;
    for (int g = blockIdx.x; g < B; g += gridDim.x) {
        const int a = s_row_ptr[g], e = s_row_ptr[g + 1];
        const float* dp = dpool + (size_t)g * C;
        if ((C & 3) == 0 && C <= 4 * kWave * 2) {
            // up to 512 columns: two 128-bit pieces per lane
            const int c0 = 4 * lane, c1 = 4 * (lane + kWave);
            const float4 p0 = c0 < C ? *reinterpret_cast<const float4*>(dp + c0) : make_float4(0.f, 0.f, 0.f, 0.f);
            const float4 p1 = c1 < C ? *reinterpret_cast<const float4*>(dp + c1) : make_float4(0.f, 0.f, 0.f, 0.f);
            for (int r = a + wave; r < e; r += kWaves) {
                const float w = s_val[r];
                float* dst = g_h + (size_t)s_col_idx[r] * C;
                if (c0 < C) *reinterpret_cast<float4*>(dst + c0) = make_float4(w * p0.x, w * p0.y, w * p0.z, w * p0.w);
                if (c1 < C) *reinterpret_cast<float4*>(dst + c1) = make_float4(w * p1.x, w * p1.y, w * p1.z, w * p1.w);
            }
        } else {
            for (int r = a + wave; r < e; r += kWaves) {
                const float w = s_val[r];
                float* dst = g_h + (size_t)s_col_idx[r] * C;
                for (int c = lane; c < C; c += kWave) dst[c] = w * dp[c];
            }
        }
    }
}

// ------------------------------------------------------------------ gradient gate
__global__ __launch_bounds__(kBlock) void grad_gate_kernel(size_t n, const float* __restrict__ h, const float* g, float* dz,
                                                           float* acc, int accumulate)
{
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const float v = h[i] > 0.f ? g[i] : 0.f;
        if (dz) dz[i] = v;
        if (acc) acc[i] = accumulate ? acc[i] + v : v;
    }
}

// ------------------------------------------------------------------ parameter update
constexpr int kUpdateBatch = 16;
struct UpdateBatch {
    float* w[kUpdateBatch];
    float* g[kUpdateBatch];
    float* v[kUpdateBatch];
    size_t n[kUpdateBatch];
};

// MomentumSGDOptimizer::Update (src/nn/optimizer.cpp:69-92), tensor blockIdx.y:
//   momentum > 0:  g += l2 w ;  v = lr g + momentum v ;  w -= v ;  g = 0
//   momentum == 0: w = -lr g + (1 - lr l2) w ;  g = 0
__global__ __launch_bounds__(kBlock) void momentum_sgd_batch_kernel(UpdateBatch b, float lr, float momentum, float l2)
{
    const int t = blockIdx.y;
    float* __restrict__ w = b.w[t];
    float* __restrict__ g = b.g[t];
    float* __restrict__ v = b.v[t];
    const size_t n = b.n[t];
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        if (momentum > 0.f) {
            const float gi = l2 * w[i] + g[i];
            const float vi = lr * gi + momentum * v[i];
            v[i] = vi;
            w[i] = -1.0f * vi + w[i];
        } else {
            w[i] = -lr * g[i] + (1 - lr * l2) * w[i];
        }
        g[i] = 0.f;
    }
}

// ------------------------------------------------------------------ Adam
// Sum of squares of every gradient tensor, for the clipping factor: workgroup (x, y) adds its stride of tensor y in
// double and leaves one partial; the update kernel adds the partials in index order.
__global__ __launch_bounds__(kBlock) void sumsq_batch_kernel(UpdateBatch b, double* __restrict__ partial)
{
    __shared__ double sh[kWavesPerBlock];
    const float* __restrict__ g = b.g[blockIdx.y];
    const size_t n = b.n[blockIdx.y];
    double acc = 0.0;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) acc += (double)g[i] * (double)g[i];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, kWave);
    if (lane == 0) sh[wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int w = 0; w < kWavesPerBlock; ++w) t += sh[w];
        partial[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = t;
    }
}

struct AdamBatch {
    float* w[kUpdateBatch];
    float* g[kUpdateBatch];
    float* m[kUpdateBatch];
    float* v[kUpdateBatch];
    size_t n[kUpdateBatch];
};

// AdamOptimizer::Update (src/nn/optimizer.cpp:105-160), tensor blockIdx.y, every step rounded as the reference's
// sequence of tensor operations rounds it (Axpby = scale, then one fused multiply-add):
//   g = l2 w + scale g ;  m = (1 - b1) g + b1 m ;  v = (1 - b2) g^2 + b2 v
//   w = -(lr s1) m / (sqrt(v s2) + eps) + w ;  g = 0
// scale = clip / norm when the norm of all gradients (nparts partial sums of squares) exceeds clip > 0, else 1.
__global__ __launch_bounds__(kBlock) void adam_batch_kernel(AdamBatch b, const double* __restrict__ partial, int nparts, float clip,
                                                            float lr_s1, float l2, float one_minus_b1, float b1, float one_minus_b2, float b2,
                                                            float eps, float s2)
{
    __shared__ double sh[kWavesPerBlock];
    __shared__ float sh_scale;
    float scale = 1.0f;
    if (nparts > 0) {
        double acc = 0.0;
        for (int i = threadIdx.x; i < nparts; i += kBlock) acc += partial[i];
        const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
        for (int d = kWave / 2; d >= 1; d >>= 1) acc += __shfl_xor(acc, d, kWave);
        if (lane == 0) sh[wave] = acc;
        __syncthreads();
        if (threadIdx.x == 0) {
            double t = 0.0;
            for (int w = 0; w < kWavesPerBlock; ++w) t += sh[w];
            const float norm = (float)sqrt(t);
            sh_scale = norm > clip ? clip / norm : 1.0f;
        }
        __syncthreads();
        scale = sh_scale;
    }
    const int t = blockIdx.y;
    float* __restrict__ w = b.w[t];
    float* __restrict__ g = b.g[t];
    float* __restrict__ m = b.m[t];
    float* __restrict__ v = b.v[t];
    const size_t n = b.n[t];
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
        const float wi = w[i];
        const float gi = __fmaf_rn(l2, wi, __fmul_rn(scale, g[i]));
        const float mi = __fmaf_rn(one_minus_b1, gi, __fmul_rn(b1, m[i]));
        const float vi = __fmaf_rn(one_minus_b2, __fmul_rn(gi, gi), __fmul_rn(b2, v[i]));
        m[i] = mi;
        v[i] = vi;
        const float step = __fmul_rn(__fdiv_rn(1.0f, __fadd_rn(__fsqrt_rn(__fmul_rn(vi, s2)), eps)), mi);
        w[i] = __fmaf_rn(-lr_s1, step, wi);
        g[i] = 0.f;
    }
}

inline unsigned ew_grid(size_t n)
{
    size_t b = (n + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > (size_t)kNumCU * 16) b = (size_t)kNumCU * 16;
    return (unsigned)b;
}

}  // namespace
}  // namespace gnnhip

using namespace gnnhip;

extern "C" {

int gnnhip_s2v_loss_acc_f32(int B, int Q, const float* logits, const int* lrow_ptr, const int* lcol, const float* lval,
                            float* probs, float* loss_rows, int* hit_rows, float* loss_mean, float* acc_mean, void* stream)
{
    GNNHIP_REQUIRE(B >= 1 && Q >= 1, "bad shape in s2v_loss_acc (B=%d Q=%d)", B, Q);
    GNNHIP_REQUIRE(logits && lrow_ptr && lcol && lval && (loss_mean || acc_mean), "null tensor in s2v_loss_acc");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    int nb = (B + 4 * kBlock - 1) / (4 * kBlock);         // about four rows per lane
    if (nb > 1024) nb = 1024;
    void* partial = nullptr;
    if (int rc = stream_scratch(s, sizeof(float) * 2 * (size_t)nb, &partial)) return rc;
    hipLaunchKernelGGL(loss_acc_partial_kernel, dim3((unsigned)nb), dim3(kBlock), 0, s, B, Q, logits, lrow_ptr, lcol, lval, probs,
                       loss_rows, hit_rows, static_cast<float*>(partial), loss_mean, acc_mean);
    GNNHIP_LAUNCH_CHECK("loss_acc_partial");
    if (nb == 1) return GNNHIP_OK;
    hipLaunchKernelGGL(loss_acc_final_kernel, dim3(1), dim3(kWave), 0, s, nb, B, static_cast<const float*>(partial), loss_mean, acc_mean);
    GNNHIP_LAUNCH_CHECK("loss_acc_final");
    return GNNHIP_OK;
}

int gnnhip_s2v_readout_backward_f32(int B, int N, int C, int H, int Q,
                                    const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                    const float* probs, const int* lrow_ptr, const int* lcol, const float* lval, float scale,
                                    const float* hidden, const float* W_h1, const float* W_h2,
                                    float* dlogits, float* du, float* g_h, void* stream)
{
    GNNHIP_REQUIRE(B >= 1 && N >= 1 && C >= 1 && H >= 1 && Q >= 1, "bad shape in s2v_readout_backward");
    GNNHIP_REQUIRE(s_row_ptr && s_col_idx && s_val && probs && lrow_ptr && lcol && lval && hidden && W_h1 && W_h2 && dlogits && du && g_h,
                   "null tensor in s2v_readout_backward");
    if (int rc = require_ready()) return rc;
    const size_t smem = sizeof(float) * ((size_t)Q + H + C);
    if (smem > 64 * 1024)
        return set_error(GNNHIP_EUNSUPPORTED, "readout backward keeps Q + H + C = %d floats per graph in LDS; too many", Q + H + C);
    long long blocks = B;
    if (blocks > (long long)kNumCU * 16) blocks = (long long)kNumCU * 16;
    hipStream_t s = as_stream(stream);
    // From 1,024 graphs on the per-graph product du W_h1^T (every lane walking its own row of W_h1) becomes one GEMM
    // over all graphs, and the node rows are written by a kernel of their own; below, one launch does everything.
    const bool split = B >= 1024 && aligned16(g_h);
    void* dpool = nullptr;
    if (split)
        if (int rc = stream_scratch(s, sizeof(float) * (size_t)B * C, &dpool)) return rc;
    hipLaunchKernelGGL(readout_backward_kernel, dim3((unsigned)blocks), dim3(kBlock), smem, s, B, C, H, Q,
                       s_row_ptr, s_col_idx, s_val, probs, lrow_ptr, lcol, lval, scale, hidden, W_h1, W_h2, dlogits, du, g_h, split ? 1 : 0);
    GNNHIP_LAUNCH_CHECK("readout_backward");
    if (split) {
        if (int rc = gemm_dispatch(0, 1, B, C, H, 1.f, du, H, W_h1, H, 0.f, static_cast<float*>(dpool), C, s)) return rc;
        hipLaunchKernelGGL(readout_backward_rows_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, B, C, s_row_ptr, s_col_idx, s_val,
                           static_cast<const float*>(dpool), g_h);
        GNNHIP_LAUNCH_CHECK("readout_backward rows");
    }
    return GNNHIP_OK;
}

int gnnhip_s2v_grad_gate_f32(size_t n, const float* h, const float* g, float* dz, float* acc, int accumulate, void* stream)
{
    if (n == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(h && g && (dz || acc), "null tensor in s2v_grad_gate");
    if (int rc = require_ready()) return rc;
    hipLaunchKernelGGL(grad_gate_kernel, dim3(ew_grid(n)), dim3(kBlock), 0, as_stream(stream), n, h, g, dz, acc, accumulate);
    GNNHIP_LAUNCH_CHECK("grad_gate");
    return GNNHIP_OK;
}

int gnnhip_momentum_sgd_batch_f32(int n, float* const* w, float* const* g, float* const* v, const size_t* count,
                                  float lr, float momentum, float l2, void* stream)
{
    GNNHIP_REQUIRE(n >= 0 && (n == 0 || (w && g && count)), "bad arguments in momentum_sgd_batch");
    GNNHIP_REQUIRE(momentum == 0.f || n == 0 || v, "momentum needs the velocity tensors");
    if (int rc = require_ready()) return rc;
    int i = 0;
    while (i < n) {
        UpdateBatch b;
        int m = 0;
        size_t largest = 0;
        for (; i < n && m < kUpdateBatch; ++i) {
            if (count[i] == 0) continue;
            GNNHIP_REQUIRE(w[i] && g[i] && (momentum == 0.f || v[i]), "null tensor in momentum_sgd_batch");
            b.w[m] = w[i]; b.g[m] = g[i]; b.v[m] = v ? v[i] : nullptr; b.n[m] = count[i];
            if (count[i] > largest) largest = count[i];
            ++m;
        }
        if (m == 0) break;
        unsigned gx = ew_grid(largest);
        if (gx > 1024u) gx = 1024u;
        hipLaunchKernelGGL(momentum_sgd_batch_kernel, dim3(gx, (unsigned)m), dim3(kBlock), 0, as_stream(stream), b, lr, momentum, l2);
        GNNHIP_LAUNCH_CHECK("momentum_sgd_batch");
    }
    return GNNHIP_OK;
}

int gnnhip_adam_batch_f32(int n, float* const* w, float* const* g, float* const* m, float* const* v, const size_t* count,
                          float lr, float l2, float clip_threshold, float beta1, float beta2, float eps, float s1, float s2, void* stream)
{
    GNNHIP_REQUIRE(n >= 0 && (n == 0 || (w && g && m && v && count)), "bad arguments in adam_batch");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    constexpr unsigned kNormGrid = 64;
    // the norm of ALL gradients comes first: one launch of partial sums per 16 tensors
    int tensors = 0;
    for (int i = 0; i < n; ++i) {
        if (count[i] == 0) continue;
        GNNHIP_REQUIRE(w[i] && g[i] && m[i] && v[i], "null tensor in adam_batch");
        ++tensors;
    }
    if (tensors == 0) return GNNHIP_OK;
    double* partial = nullptr;
    int nparts = 0;
    if (clip_threshold > 0.f) {
        void* q = nullptr;
        if (int rc = stream_scratch(s, sizeof(double) * (size_t)tensors * kNormGrid, &q)) return rc;
        partial = static_cast<double*>(q);
        int i = 0;
        while (i < n) {
            UpdateBatch b;
            int k = 0;
            for (; i < n && k < kUpdateBatch; ++i) {
                if (count[i] == 0) continue;
                b.w[k] = nullptr; b.v[k] = nullptr; b.g[k] = g[i]; b.n[k] = count[i];
                ++k;
            }
            if (k == 0) break;
            hipLaunchKernelGGL(sumsq_batch_kernel, dim3(kNormGrid, (unsigned)k), dim3(kBlock), 0, s, b, partial + nparts);
            nparts += k * (int)kNormGrid;
        }
        GNNHIP_LAUNCH_CHECK("sumsq_batch");
    }
    int i = 0;
    while (i < n) {
        AdamBatch b;
        int k = 0;
        size_t largest = 0;
        for (; i < n && k < kUpdateBatch; ++i) {
            if (count[i] == 0) continue;
            b.w[k] = w[i]; b.g[k] = g[i]; b.m[k] = m[i]; b.v[k] = v[i]; b.n[k] = count[i];
            if (count[i] > largest) largest = count[i];
            ++k;
        }
        if (k == 0) break;
        unsigned gx = ew_grid(largest);
        if (gx > 1024u) gx = 1024u;
        hipLaunchKernelGGL(adam_batch_kernel, dim3(gx, (unsigned)k), dim3(kBlock), 0, s, b, partial, nparts, clip_threshold,
                           lr * s1, l2, 1 - beta1, beta1, 1 - beta2, beta2, eps, s2);
        GNNHIP_LAUNCH_CHECK("adam_batch");
    }
    return GNNHIP_OK;
}

}  // extern "C"
