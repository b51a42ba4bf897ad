// C entry points of the structure2vec mean-field forward: the three fused
// stages (input, level, readout) and the whole forward that chains them on one
// stream with every activation resident in HBM.  Hidden sizes without a fused
// kernel are composed from the general SpMM / GEMM / element-wise kernels, so
// every shape the reference accepts is still computed on the device.
#include "gnnhip_internal.h"

namespace gnnhip {

// defined in level.hip / spmm.hip / gemm.hip / reduce.hip
bool fused_hidden_supported(int C);
int input_dispatch(int N, int K, int C, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s);
int level_dispatch(int N, int C, long long nnz, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                   const float* W, const float* msg, const float* bias, float* h_out, hipStream_t s, bool same_graph = false,
                   bool relu_in = false, CsrPlan* plan = nullptr);
bool level_accepts_relu_input(int N, int C, long long nnz);
int level_backward_dispatch(int N, int C, long long nnz, const int* row_ptr, const int* col_idx, const float* val, const float* dz,
                            const float* W, float* u, float* g_prev, const float* gate, float* acc, hipStream_t s);
int readout_dispatch(int B, int C, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                     const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                     float* logits, float* probs, int* pred, hipStream_t s);
int readout_wave_dispatch(int B, int C, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                          const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                          float* logits, float* probs, int* pred, hipStream_t s);
int readout_tile_dispatch(int B, int C, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                          const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                          float* logits, float* probs, int* pred, hipStream_t s);
int gemm_dispatch(int transA, int transB, int m, int n, int k, float alpha, const float* A, int lda,
                  const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s);
int row_softmax_dispatch(float* x, int rows, int cols, hipStream_t s);
int row_argmax_dispatch(const float* x, int rows, int cols, int* out, hipStream_t s);

namespace {

constexpr int kBlock = 256;

// out[i,j] = ReLU(lin[i,j] + bias[j] + msg[i,j]); out may alias lin.  relu_copy: second output.
__global__ __launch_bounds__(kBlock) void bias_add_relu_kernel(const float* lin, const float* __restrict__ bias,
                                                               const float* __restrict__ msg, float* out,
                                                               float* relu_copy, size_t total, int C, int do_relu)
{
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
        float v = lin[i];
        if (bias) v += bias[i % C];
        if (msg) v += msg[i];
        const float r = v < 0.f ? 0.f : v;
        if (relu_copy) { out[i] = v; relu_copy[i] = r; }
        else out[i] = do_relu ? r : v;
    }
}

inline unsigned ew_grid(size_t n)
{
    size_t b = (n + kBlock - 1) / kBlock;
    if (b < 1) b = 1;
    if (b > (size_t)kNumCU * 8) b = (size_t)kNumCU * 8;
    return (unsigned)b;
}

int input_any(int N, int K, int C, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s)
{
    int rc = input_dispatch(N, K, C, X, Wn2l, msg, h0, s);
    if (rc != GNNHIP_EUNSUPPORTED) return rc;
    if ((rc = gemm_dispatch(0, 0, N, C, K, 1.f, X, K, Wn2l, C, 0.f, msg, C, s))) return rc;
    if (!h0) return GNNHIP_OK;
    const size_t total = (size_t)N * C;
    hipLaunchKernelGGL(bias_add_relu_kernel, dim3(ew_grid(total)), dim3(kBlock), 0, s,
                       msg, (const float*)nullptr, (const float*)nullptr, msg, h0, total, C, 1);
    GNNHIP_LAUNCH_CHECK("bias_add_relu");
    return GNNHIP_OK;
}

int level_any(int N, int C, long long nnz, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
              const float* W, const float* msg, const float* bias, float* h_out, hipStream_t s, bool same_graph = false,
              bool relu_in = false, CsrPlan* plan = nullptr)
{
    int rc = level_dispatch(N, C, nnz, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s, same_graph, relu_in, plan);
    if (rc != GNNHIP_EUNSUPPORTED) return rc;
    if (relu_in) return set_error(GNNHIP_EUNSUPPORTED, "no level kernel reads its input through ReLU for this shape");
    void* tmp = nullptr;
    const size_t total = (size_t)N * C;
    if ((rc = stream_scratch(s, sizeof(float) * total, &tmp))) return rc;
    float* agg = static_cast<float*>(tmp);
    if ((rc = spmm_dispatch(N, N, C, nnz, 1.f, row_ptr, col_idx, val, h_in, C, 0.f, agg, C, s, same_graph, false, plan))) return rc;
    if ((rc = gemm_dispatch(0, 0, N, C, C, 1.f, agg, C, W, C, 0.f, h_out, C, s))) return rc;
    hipLaunchKernelGGL(bias_add_relu_kernel, dim3(ew_grid(total)), dim3(kBlock), 0, s,
                       h_out, bias, msg, h_out, (float*)nullptr, total, C, 1);
    GNNHIP_LAUNCH_CHECK("bias_add_relu");
    return GNNHIP_OK;
}

__global__ __launch_bounds__(kBlock) void copy_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n)
{
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

constexpr int kWaveReadoutMinGraphs = 1024;        // below this a workgroup per graph
constexpr int kWaveReadoutMaxMeanNodes = 2048;     // mean nodes per graph
constexpr int kBlockReadoutMaxGraphsWide = 4096;   // hidden 128/256: above this a workgroup per tile of graphs (or SpMM + GEMM)
constexpr int kTileReadoutMinGraphs = 4096;

int readout_any(int B, int N, int C, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                float* logits, float* probs, int* pred, hipStream_t s)
{
    // Many graphs of moderate size: one wavefront per graph (30,000 graphs of 29 nodes, hidden 64: 78 us with
    // a workgroup per graph).  Few graphs: a workgroup per graph reaches more of the chip.  Graphs of
    // thousands of nodes are left to the SpMM, which balances long rows.
    int rc = GNNHIP_EUNSUPPORTED;
    if (B >= kWaveReadoutMinGraphs && (long long)N <= (long long)B * kWaveReadoutMaxMeanNodes)
        rc = readout_wave_dispatch(B, C, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    if (rc != GNNHIP_EUNSUPPORTED) return rc;
    // hidden 128/256: a workgroup per graph up to a few thousand graphs (256 graphs, hidden 256: 20 us against
    // 67 us for the seven launches below); 10,000 graphs: 116 against 106 us
    if (C > 64 && B > kTileReadoutMinGraphs && (long long)N <= (long long)B * kWaveReadoutMaxMeanNodes)
        rc = readout_tile_dispatch(B, C, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    if (rc != GNNHIP_EUNSUPPORTED) return rc;
    if (C <= 64 || B <= kBlockReadoutMaxGraphsWide)
        rc = readout_dispatch(B, C, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    if (rc != GNNHIP_EUNSUPPORTED) return rc;
    if ((rc = spmm_dispatch(B, N, C, (long long)N, 1.f, s_row_ptr, s_col_idx, s_val, h, C, 0.f, pool, C, s))) return rc;
    if ((rc = gemm_dispatch(0, 0, B, H, C, 1.f, pool, C, Wh1, H, 0.f, hidden, H, s))) return rc;
    const size_t bh = (size_t)B * H;
    hipLaunchKernelGGL(bias_add_relu_kernel, dim3(ew_grid(bh)), dim3(kBlock), 0, s,
                       hidden, (const float*)nullptr, (const float*)nullptr, hidden, (float*)nullptr, bh, H, 1);
    GNNHIP_LAUNCH_CHECK("bias_add_relu");
    if ((rc = gemm_dispatch(0, 0, B, Q, H, 1.f, hidden, H, Wh2, Q, 0.f, logits, Q, s))) return rc;
    if (pred && (rc = row_argmax_dispatch(logits, B, Q, pred, s))) return rc;
    if (probs) {
        const size_t bq = (size_t)B * Q;
        hipLaunchKernelGGL(copy_kernel, dim3(ew_grid(bq)), dim3(kBlock), 0, s, logits, probs, bq);
        GNNHIP_LAUNCH_CHECK("copy");
        if ((rc = row_softmax_dispatch(probs, B, Q, s))) return rc;
    }
    return GNNHIP_OK;
}

// input, L levels, readout on one stream; plan: of A, or null
int forward_any(int N, int B, int K, int C, int H, int Q, int L, long long a_nnz, const int* a_row_ptr, const int* a_col_idx,
                const float* a_val, const int* s_row_ptr, const int* s_col_idx, const float* s_val, const float* X, const float* W_n2l,
                const float* W_conv, const float* W_h1, const float* W_h2, float* msg, float* h_a, float* h_b, float* pool, float* hidden,
                float* logits, float* probs, int* pred, int* which_h, hipStream_t s, CsrPlan* plan)
{
    // With at least one level, and a level kernel that can read its input through ReLU, h0 = ReLU(msg) is
    // never stored: the first level gathers from msg.
    const bool lazy_h0 = L >= 1 && level_accepts_relu_input(N, C, a_nnz);
    int rc = input_any(N, K, C, X, W_n2l, msg, lazy_h0 ? nullptr : h_a, s);
    if (rc) return rc;
    float* cur = lazy_h0 ? msg : h_a;
    float* nxt = lazy_h0 ? h_a : h_b;
    for (int lv = 0; lv < L; ++lv) {
        if ((rc = level_any(N, C, a_nnz, a_row_ptr, a_col_idx, a_val, cur, W_conv, msg, nullptr, nxt, s, lv > 0,
                            lazy_h0 && lv == 0, plan)))
            return rc;
        float* t = (cur == msg) ? h_b : cur;     // msg stays what it is; the other buffer takes the next level
        cur = nxt;
        nxt = t;
    }
    if (which_h) *which_h = (cur == h_a) ? 0 : 1;
    return readout_any(B, N, C, H, Q, s_row_ptr, s_col_idx, s_val, cur, W_h1, W_h2, pool, hidden, logits, probs, pred, s);
}

}  // namespace
}  // namespace gnnhip

using namespace gnnhip;

extern "C" {

int gnnhip_s2v_input_f32(int N, int K, int C, const float* X, const float* W_n2l, float* msg, float* h0, void* stream)
{
    GNNHIP_REQUIRE(N >= 0 && K >= 1 && C >= 1, "bad shape in s2v_input (N=%d K=%d C=%d)", N, K, C);
    if (N == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(X && W_n2l && msg, "null tensor in s2v_input");
    if (int rc = require_ready()) return rc;
    return input_any(N, K, C, X, W_n2l, msg, h0, as_stream(stream));
}

int gnnhip_s2v_level_f32(int N, int C, int nnz, const int* row_ptr, const int* col_idx, const float* val,
                         const float* h_in, const float* W, const float* msg, const float* bias,
                         float* h_out, void* stream)
{
    GNNHIP_REQUIRE(N >= 0 && C >= 1 && nnz >= 0, "bad shape in s2v_level (N=%d C=%d nnz=%d)", N, C, nnz);
    if (N == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(row_ptr && h_in && W && h_out, "null tensor in s2v_level");
    GNNHIP_REQUIRE(h_in != h_out, "s2v_level cannot run in place");
    if (int rc = require_ready()) return rc;
    return level_any(N, C, nnz, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, as_stream(stream));
}

int gnnhip_s2v_level_planned_f32(void* plan, int C, const float* h_in, const float* W, const float* msg, const float* bias, float* h_out,
                                 void* stream)
{
    CsrPlan* p = as_csr_plan(plan);
    GNNHIP_REQUIRE(p, "%p is not a live CSR plan", plan);
    GNNHIP_REQUIRE(p->m == p->k, "s2v_level_planned needs the plan of a square matrix (it has %d rows and %d columns)", p->m, p->k);
    GNNHIP_REQUIRE(C >= 1, "bad hidden size in s2v_level_planned (C=%d)", C);
    if (p->m == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(h_in && W && h_out, "null tensor in s2v_level_planned");
    GNNHIP_REQUIRE(h_in != h_out, "s2v_level_planned cannot run in place");
    if (int rc = require_ready()) return rc;
    return level_any(p->m, C, p->nnz, p->row_ptr, p->col_idx, p->val, h_in, W, msg, bias, h_out, as_stream(stream), false, false, p);
}

int gnnhip_s2v_level_backward_f32(int N, int C, int nnz, const int* t_row_ptr, const int* t_col_idx, const float* t_val,
                                  const float* dz, const float* W, float* u, float* g_prev, const float* gate_h, float* acc,
                                  void* stream)
{
    GNNHIP_REQUIRE(N >= 0 && C >= 1 && nnz >= 0, "bad shape in s2v_level_backward (N=%d C=%d nnz=%d)", N, C, nnz);
    if (N == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(t_row_ptr && dz && W && u && g_prev, "null tensor in s2v_level_backward");
    GNNHIP_REQUIRE(dz != u && dz != g_prev && u != g_prev, "s2v_level_backward needs three distinct buffers");
    GNNHIP_REQUIRE(acc != dz && acc != u && acc != g_prev && gate_h != g_prev && gate_h != u,
                   "s2v_level_backward: acc and gate_h must not alias the other buffers");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    int rc = level_backward_dispatch(N, C, nnz, t_row_ptr, t_col_idx, t_val, dz, W, u, g_prev, gate_h, acc, s);
    if (rc != GNNHIP_EUNSUPPORTED) return rc;
    if ((rc = spmm_dispatch(N, N, C, nnz, 1.f, t_row_ptr, t_col_idx, t_val, dz, C, 0.f, u, C, s))) return rc;
    if ((rc = gemm_dispatch(0, 1, N, C, C, 1.f, u, C, W, C, 0.f, g_prev, C, s))) return rc;
    if (gate_h) return gnnhip_s2v_grad_gate_f32((size_t)N * C, gate_h, g_prev, g_prev, acc, 1, stream);
    if (acc) return gnnhip_axpy_f32((size_t)N * C, 1.f, g_prev, acc, stream);
    return GNNHIP_OK;
}

int gnnhip_s2v_readout_f32(int B, int N, int C, int H, int Q,
                           const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                           const float* h, const float* W_h1, const float* W_h2,
                           float* pool, float* hidden, float* logits, float* probs, int* pred, void* stream)
{
    GNNHIP_REQUIRE(B >= 0 && N >= 0 && C >= 1 && H >= 1 && Q >= 1, "bad shape in s2v_readout");
    if (B == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(s_row_ptr && W_h1 && W_h2 && pool && hidden && logits, "null tensor in s2v_readout");
    GNNHIP_REQUIRE(N == 0 || (s_col_idx && s_val && h), "null tensor in s2v_readout");
    if (int rc = require_ready()) return rc;
    return readout_any(B, N, C, H, Q, s_row_ptr, s_col_idx, s_val, h, W_h1, W_h2, pool, hidden, logits, probs, pred,
                       as_stream(stream));
}

int gnnhip_s2v_forward_f32(int N, int B, int K, int C, int H, int Q, int L, int a_nnz,
                           const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                           const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                           const float* X, const float* W_n2l, const float* W_conv,
                           const float* W_h1, const float* W_h2,
                           float* msg, float* h_a, float* h_b,
                           float* pool, float* hidden, float* logits, float* probs, int* pred,
                           int* which_h, void* stream)
{
    GNNHIP_REQUIRE(N >= 1 && B >= 1 && K >= 1 && C >= 1 && H >= 1 && Q >= 1 && L >= 0 && a_nnz >= 0,
                   "bad shape in s2v_forward (N=%d B=%d K=%d C=%d H=%d Q=%d L=%d)", N, B, K, C, H, Q, L);
    GNNHIP_REQUIRE(a_row_ptr && s_row_ptr && s_col_idx && s_val && X && W_n2l && W_conv && W_h1 && W_h2,
                   "null input in s2v_forward");
    GNNHIP_REQUIRE(msg && h_a && h_b && pool && hidden && logits, "null output in s2v_forward");
    GNNHIP_REQUIRE(h_a != h_b && msg != h_a && msg != h_b, "msg, h_a and h_b must be distinct buffers");
    if (int rc = require_ready()) return rc;
    return forward_any(N, B, K, C, H, Q, L, a_nnz, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx, s_val, X, W_n2l, W_conv, W_h1, W_h2,
                       msg, h_a, h_b, pool, hidden, logits, probs, pred, which_h, as_stream(stream), nullptr);
}

int gnnhip_s2v_forward_planned_f32(void* a_plan, int B, int K, int C, int H, int Q, int L,
                                   const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                   const float* X, const float* W_n2l, const float* W_conv,
                                   const float* W_h1, const float* W_h2,
                                   float* msg, float* h_a, float* h_b,
                                   float* pool, float* hidden, float* logits, float* probs, int* pred,
                                   int* which_h, void* stream)
{
    CsrPlan* p = as_csr_plan(a_plan);
    GNNHIP_REQUIRE(p, "%p is not a live CSR plan", a_plan);
    GNNHIP_REQUIRE(p->m == p->k && p->m >= 1, "s2v_forward_planned needs the plan of a square matrix with rows (it has %d rows and %d columns)", p->m, p->k);
    GNNHIP_REQUIRE(B >= 1 && K >= 1 && C >= 1 && H >= 1 && Q >= 1 && L >= 0,
                   "bad shape in s2v_forward_planned (B=%d K=%d C=%d H=%d Q=%d L=%d)", B, K, C, H, Q, L);
    GNNHIP_REQUIRE(s_row_ptr && s_col_idx && s_val && X && W_n2l && W_conv && W_h1 && W_h2, "null input in s2v_forward_planned");
    GNNHIP_REQUIRE(msg && h_a && h_b && pool && hidden && logits, "null output in s2v_forward_planned");
    GNNHIP_REQUIRE(h_a != h_b && msg != h_a && msg != h_b, "msg, h_a and h_b must be distinct buffers");
    if (int rc = require_ready()) return rc;
    return forward_any(p->m, B, K, C, H, Q, L, p->nnz, p->row_ptr, p->col_idx, p->val, s_row_ptr, s_col_idx, s_val, X, W_n2l, W_conv, W_h1,
                       W_h2, msg, h_a, h_b, pool, hidden, logits, probs, pred, which_h, as_stream(stream), p);
}

}  // extern "C"
