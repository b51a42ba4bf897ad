/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of graphnn's structure2vec
 * mean-field forward (see s2v_oracle.h).  Used by tests/, by the smoke check
 * and by the cpu_baseline leg of the benchmark; never by the shipped library.
 *
 * Build: see oracle/Makefile (gcc -O3 -mavx2 -ffp-contract=off -fopenmp).
 * -ffp-contract=off keeps every fp32 operation a separately rounded IEEE
 * operation in source order, so element-wise results are predictable.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   CSR builders      brute force vs dense adjacency, invariants, and the
 *                     reference's own GraphStruct compiled into oracle/_ref;
 *                     the edge-based operands against their dense definitions
 *   spmm / gemm       fp64 brute force, identity / known-answer matrices
 *                     (reference test matrix test/gpu_tensor_test.cpp:311-336),
 *                     and Intel MKL mkl_scsrmm / cblas_sgemm called with the
 *                     reference's own argument pattern when libmkl_rt loads
 *   softmax family    rows sum to 1, shift invariance, Q=2 closed form
 *   argmax / top-k    counting definitions, tie cases
 *   forward           composition of the above; op order of
 *                     examples/graph_classification/src/kernel_mean_field.cpp:31-56
 */
#include "s2v_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void orc_set_num_threads(int n)
{
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------------
 * Batch graph -> CSR.
 *
 * GraphStruct::AddEdge(idx, x, y) appends (idx, x) to in_edges[y]
 * (src/util/graph_struct.cpp:62-70); Node2NodeMsgPass::InitCPUWeight walks
 * nodes 0..N-1 and lists in_edges[i] in insertion order, column = source node,
 * value 1 or 1/indeg (src/nn/msg_pass.cpp:46-67).  That is a stable counting
 * sort of the edge list by destination.
 * ---------------------------------------------------------------------- */
void orc_csr_node2node(int num_nodes, int num_edges, const int* edge_x, const int* edge_y,
                       int average, int* row_ptr, int* col_idx, float* val)
{
    int* fill = (int*)calloc((size_t)num_nodes + 1, sizeof(int));
    for (int e = 0; e < num_edges; ++e) fill[edge_y[e] + 1]++;
    row_ptr[0] = 0;
    for (int i = 0; i < num_nodes; ++i) row_ptr[i + 1] = row_ptr[i] + fill[i + 1];
    for (int i = 0; i < num_nodes; ++i) fill[i] = row_ptr[i];
    for (int e = 0; e < num_edges; ++e) {
        int y = edge_y[e];
        int deg = row_ptr[y + 1] - row_ptr[y];
        int pos = fill[y]++;
        col_idx[pos] = edge_x[e];
        /* reference: Dtype val = average ? 1.0 / list.size() : 1.0  (double divide, then narrowed) */
        val[pos] = average ? (float)(1.0 / (double)deg) : 1.0f;
    }
    free(fill);
}

/* Edge2NodeMsgPass::InitCPUWeight (src/nn/msg_pass.cpp:72-94): matrix [N, E]; row i lists the
 * indices of the edges that end in node i, in insertion order; value 1 or 1/indeg. */
void orc_csr_edge2node(int num_nodes, int num_edges, const int* edge_y, int average,
                       int* row_ptr, int* col_idx, float* val)
{
    int* fill = (int*)calloc((size_t)num_nodes + 1, sizeof(int));
    for (int e = 0; e < num_edges; ++e) fill[edge_y[e] + 1]++;
    row_ptr[0] = 0;
    for (int i = 0; i < num_nodes; ++i) row_ptr[i + 1] = row_ptr[i] + fill[i + 1];
    for (int i = 0; i < num_nodes; ++i) fill[i] = row_ptr[i];
    for (int e = 0; e < num_edges; ++e) {
        int y = edge_y[e];
        int deg = row_ptr[y + 1] - row_ptr[y];
        int pos = fill[y]++;
        col_idx[pos] = e;
        val[pos] = average ? (float)(1.0 / (double)deg) : 1.0f;
    }
    free(fill);
}

/* Node2EdgeMsgPass::InitCPUWeight (src/nn/msg_pass.cpp:98-116): matrix [E, N]; row e holds one
 * entry, the tail node of edge e, value 1. */
void orc_csr_node2edge(int num_edges, const int* edge_x, int* row_ptr, int* col_idx, float* val)
{
    for (int e = 0; e < num_edges; ++e) { row_ptr[e] = e; col_idx[e] = edge_x[e]; val[e] = 1.0f; }
    row_ptr[num_edges] = num_edges;
}

/* Edge2EdgeMsgPass::InitCPUWeight (src/nn/msg_pass.cpp:120-152): matrix [E, E]; row e = (x -> y)
 * lists, in insertion order, the edges (u -> x) that end in x, except those that start in y
 * (the same edge in the other direction); value 1.  Returns the number of entries; col_idx and
 * val may be NULL to count only (row_ptr is always written). */
int orc_csr_edge2edge(int num_nodes, int num_edges, const int* edge_x, const int* edge_y,
                      int* row_ptr, int* col_idx, float* val)
{
    /* in-edge lists of every node in insertion order: a stable grouping of edge indices by head */
    int* start = (int*)calloc((size_t)num_nodes + 1, sizeof(int));
    int* fill = (int*)calloc((size_t)num_nodes + 1, sizeof(int));
    int* in_edge = (int*)malloc(sizeof(int) * (size_t)(num_edges > 0 ? num_edges : 1));
    for (int e = 0; e < num_edges; ++e) start[edge_y[e] + 1]++;
    for (int i = 0; i < num_nodes; ++i) start[i + 1] += start[i];
    for (int i = 0; i < num_nodes; ++i) fill[i] = start[i];
    for (int e = 0; e < num_edges; ++e) in_edge[fill[edge_y[e]]++] = e;
    int nnz = 0;
    for (int e = 0; e < num_edges; ++e) {
        row_ptr[e] = nnz;
        const int from = edge_x[e], to = edge_y[e];
        for (int t = start[from]; t < start[from + 1]; ++t) {
            const int other = in_edge[t];
            if (edge_x[other] == to) continue;
            if (col_idx) { col_idx[nnz] = other; val[nnz] = 1.0f; }
            ++nnz;
        }
    }
    row_ptr[num_edges] = nnz;
    free(start); free(fill); free(in_edge);
    return nnz;
}

/* GraphStruct::AddNode(subg, n) appends n to subgraph[subg]
 * (src/util/graph_struct.cpp:72-75); SubgraphMsgPass::InitCPUWeight lists each
 * subgraph's nodes in insertion order (src/nn/msg_pass.cpp:156-177). */
void orc_csr_subgraph(int num_subgraph, int num_nodes, const int* subg_id, const int* node_idx,
                      int average, int* row_ptr, int* col_idx, float* val)
{
    int* fill = (int*)calloc((size_t)num_subgraph + 1, sizeof(int));
    for (int i = 0; i < num_nodes; ++i) fill[subg_id[i] + 1]++;
    row_ptr[0] = 0;
    for (int g = 0; g < num_subgraph; ++g) row_ptr[g + 1] = row_ptr[g] + fill[g + 1];
    for (int g = 0; g < num_subgraph; ++g) fill[g] = row_ptr[g];
    for (int i = 0; i < num_nodes; ++i) {
        int g = subg_id[i];
        int cnt = row_ptr[g + 1] - row_ptr[g];
        int pos = fill[g]++;
        col_idx[pos] = node_idx[i];
        val[pos] = average ? (float)(1.0 / (double)cnt) : 1.0f;
    }
    free(fill);
}

/* ------------------------------------------------------------------------
 * C = alpha * A * B + beta * C with A in CSR (m rows), B [k,n], C [m,n].
 * Reference: DTensor<CPU>::MM(SpTensor, DTensor, N, N) ->
 * mkl_scsrmm('N', ..., "GLNC", val, col_idx, row_ptr, row_ptr+1, ...)
 * (src/tensor/cpu_dense_tensor.cpp:213-225, include/tensor/mkl_helper.h:131-138).
 * "GLNC" = general matrix, zero-based indexing => row-major B and C.
 * beta == 0 overwrites C (no read of the old contents).
 * ---------------------------------------------------------------------- */
void orc_spmm_csr(int m, int n, float alpha, const int* row_ptr, const int* col_idx,
                  const float* val, const float* B, int ldb, float beta, float* C, int ldc)
{
#pragma omp parallel for schedule(dynamic, 256)
    for (int i = 0; i < m; ++i) {
        float* c = C + (size_t)i * ldc;
        if (beta == 0.0f) {
            for (int j = 0; j < n; ++j) c[j] = 0.0f;
        } else if (beta != 1.0f) {
            for (int j = 0; j < n; ++j) c[j] *= beta;
        }
        for (int t = row_ptr[i]; t < row_ptr[i + 1]; ++t) {
            const float a = alpha * val[t];
            const float* b = B + (size_t)col_idx[t] * ldb;
            for (int j = 0; j < n; ++j) c[j] += a * b[j];
        }
    }
}

/* Not a reference routine: the float64 arbiter of the parity tests at sizes where scipy's single-threaded product
 * takes too long.  out[m,n] (double) = alpha * A * B with every product and sum in double; absolute != 0 gives the
 * same sum over magnitudes (|alpha| |A| |B|), the condition tensor of the parity metric.  Pinned against scipy's
 * float64 CSR product (tests/test_oracle_pins.py). */
void orc_spmm_csr_f64(int m, int n, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                      const float* B, int ldb, int absolute, double* out, int ldo)
{
#pragma omp parallel for schedule(dynamic, 256)
    for (int i = 0; i < m; ++i) {
        double* c = out + (size_t)i * ldo;
        for (int j = 0; j < n; ++j) c[j] = 0.0;
        for (int t = row_ptr[i]; t < row_ptr[i + 1]; ++t) {
            double a = (double)alpha * (double)val[t];
            const float* b = B + (size_t)col_idx[t] * ldb;
            if (absolute) {
                a = fabs(a);
                for (int j = 0; j < n; ++j) c[j] += a * fabs((double)b[j]);
            } else {
                for (int j = 0; j < n; ++j) c[j] += a * (double)b[j];
            }
        }
    }
}

/* C[k,n] = alpha * A^T * B + beta * C, A CSR with m rows and k columns, B [m,n].
 * Reference: same call with trans 'T' (used by MatMul::Backward, src/nn/matmul.cpp:35-76). */
void orc_spmm_csr_T(int m, int n, int k, float alpha, const int* row_ptr, const int* col_idx,
                    const float* val, const float* B, int ldb, float beta, float* C, int ldc)
{
    for (int r = 0; r < k; ++r) {
        float* c = C + (size_t)r * ldc;
        if (beta == 0.0f) {
            for (int j = 0; j < n; ++j) c[j] = 0.0f;
        } else if (beta != 1.0f) {
            for (int j = 0; j < n; ++j) c[j] *= beta;
        }
    }
    for (int i = 0; i < m; ++i) {
        const float* b = B + (size_t)i * ldb;
        for (int t = row_ptr[i]; t < row_ptr[i + 1]; ++t) {
            const float a = alpha * val[t];
            float* c = C + (size_t)col_idx[t] * ldc;
            for (int j = 0; j < n; ++j) c[j] += a * b[j];
        }
    }
}

/* ------------------------------------------------------------------------
 * Row-major C[m,n] = alpha * op(A) * op(B) + beta * C.
 * Reference: DTensor<CPU>::MM(DTensor, DTensor) -> cblas_sgemm(CblasRowMajor, ...)
 * with lda = a.cols(), ldb = b.cols() (src/tensor/cpu_dense_tensor.cpp:198-211).
 * fp32 accumulation, k ascending.
 * ---------------------------------------------------------------------- */
void orc_gemm(int transA, int transB, int m, int n, int k, float alpha, const float* A, int lda,
              const float* B, int ldb, float beta, float* C, int ldc)
{
#pragma omp parallel
    {
        float* acc = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
#pragma omp for schedule(static)
        for (int i = 0; i < m; ++i) {
            for (int j = 0; j < n; ++j) acc[j] = 0.0f;
            for (int p = 0; p < k; ++p) {
                const float a = transA ? A[(size_t)p * lda + i] : A[(size_t)i * lda + p];
                if (!transB) {
                    const float* b = B + (size_t)p * ldb;
                    for (int j = 0; j < n; ++j) acc[j] += a * b[j];
                } else {
                    for (int j = 0; j < n; ++j) acc[j] += a * B[(size_t)j * ldb + p];
                }
            }
            float* c = C + (size_t)i * ldc;
            if (beta == 0.0f) {
                for (int j = 0; j < n; ++j) c[j] = alpha * acc[j];
            } else {
                for (int j = 0; j < n; ++j) c[j] = alpha * acc[j] + beta * c[j];
            }
        }
        free(acc);
    }
}

/* y += a*x : DTensor<CPU>::Axpy -> cblas_saxpy (src/tensor/cpu_dense_tensor.cpp:303-308) */
void orc_axpy(size_t n, float a, const float* x, float* y)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) y[i] += a * x[i];
}

/* y = a*x + b*y : DTensor<CPU>::Axpby -> cblas_saxpby */
void orc_axpby(size_t n, float a, const float* x, float b, float* y)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) y[i] = a * x[i] + b * y[i];
}

/* ------------------------------------------------------------------------
 * In-place unary functors.  Op codes are the library's GNNHIP_UNARY_* values.
 * Definitions: include/tensor/cpu_unary_functor.h:17-60 (Set, Truncate,
 * Sigmoid), include/tensor/gpu_unary_functor.h:17-327 for the full list; the
 * CPU tensor routes Abs/Inv/Log/InvSqrt/Exp/Square/Sqrt through MKL VML and
 * Scale through cblas_sscal, which compute the same element-wise functions.
 * ReLU: `if (x < 0) x = 0` (src/nn/relu.cpp:7-15) so -0.0 and NaN pass through.
 * ---------------------------------------------------------------------- */
void orc_unary(int op, float* x, size_t n, float a0, float a1)
{
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        float v = x[i];
        switch (op) {
        case 0: v = a0; break;                                  /* Set */
        case 1: v = v < a0 ? a0 : v; v = v > a1 ? a1 : v; break; /* Truncate */
        case 2: v = v * a0; break;                              /* Scale */
        case 3: v = v + a0; break;                              /* Add */
        case 4: v = fabsf(v); break;                            /* Abs */
        case 5: v = 1.0f / v; break;                            /* Inv */
        case 6: if (v < 0) v = 0; break;                        /* ReLU */
        case 7: v = (float)(1.0 / (1.0 + exp(-(double)v))); break; /* Sigmoid (double math, cpu_unary_functor.h:54-60) */
        case 8: { float e1 = expf(v), e2 = expf(-v); v = (e1 - e2) / (e1 + e2); } break; /* Tanh */
        case 9: v = logf(v); break;                             /* Log */
        case 10: v = 1.0f / sqrtf(v); break;                    /* InvSqrt */
        case 11: v = expf(v); break;                            /* Exp */
        case 12: v = v * v; break;                              /* Square */
        case 13: v = sqrtf(v); break;                           /* Sqrt */
        default: break;
        }
        x[i] = v;
    }
}

/* ------------------------------------------------------------------------
 * Row softmax in place: subtract row max, exp, divide by the row's sum.
 * Reference: DTensor<CPU>::Softmax (src/tensor/cpu_dense_tensor.cpp:227-251):
 * max scan starts at element 0 with strict '>', vsExp over the whole tensor,
 * cblas_sasum per row (all terms positive, so asum == sum).
 * ---------------------------------------------------------------------- */
static void softmax_one(float* x, int cols)
{
    if (cols <= 0) return;
    float mx = x[0];
    for (int j = 1; j < cols; ++j) if (x[j] > mx) mx = x[j];
    float sum = 0.0f;
    for (int j = 0; j < cols; ++j) { x[j] = expf(x[j] - mx); sum += fabsf(x[j]); }
    for (int j = 0; j < cols; ++j) x[j] /= sum;
}

void orc_row_softmax(float* x, int rows, int cols)
{
#pragma omp parallel for schedule(static)
    for (int i = 0; i < rows; ++i) softmax_one(x + (size_t)i * cols, cols);
}

/* Independent softmax over consecutive segments of a column vector.
 * Reference: DTensor<CPU>::JaggedSoftmax (src/tensor/cpu_dense_tensor.cpp:253-267):
 * each segment is viewed as a 1 x len matrix and given to Softmax(). */
void orc_jagged_softmax(float* x, const int* lens, int nseg)
{
    size_t* off = (size_t*)malloc(sizeof(size_t) * ((size_t)nseg + 1));
    off[0] = 0;
    for (int s = 0; s < nseg; ++s) off[s + 1] = off[s] + (size_t)lens[s];
#pragma omp parallel for schedule(dynamic, 16)
    for (int s = 0; s < nseg; ++s) softmax_one(x + off[s], lens[s]);
    free(off);
}

/* Gradient of the jagged softmax (CPU JaggedSoftmaxDeriv, src/nn/jagged_softmax.cpp:8-31):
 * per segment z = dot(grad, out) (MKL_Dot), buf = (grad - z) * out, dst += buf. */
void orc_jagged_softmax_deriv(float* dst, const float* out, const float* grad, const int* lens, int nseg)
{
    size_t off = 0;
    for (int s = 0; s < nseg; ++s) {
        const int n = lens[s];
        float z = 0.0f;
        for (int j = 0; j < n; ++j) z += grad[off + j] * out[off + j];
        for (int j = 0; j < n; ++j) {
            float b = grad[off + j] - z;
            b = b * out[off + j];
            dst[off + j] = 1.0f * b + dst[off + j];
        }
        off += (size_t)n;
    }
}

/* One MomentumSGDOptimizer::Update on one tensor (src/nn/optimizer.cpp:69-92), as the calls it makes:
 * grad.RowSparseAxpy(l2, value); acc.RowSparseAxpby(lr, grad, momentum); value.Axpy(-1, acc); grad.RowSpZeros()
 * (full gradients: the row-sparse forms are the dense axpy / axpby); momentum == 0 takes the plain SGD branch
 * value.RowSparseAxpby(-lr, grad, 1 - lr * l2). */
void orc_momentum_sgd(size_t n, float* w, float* g, float* v, float lr, float momentum, float l2)
{
    if (momentum > 0.0f) {
        orc_axpy(n, l2, w, g);
        orc_axpby(n, lr, g, momentum, v);
        orc_axpy(n, -1.0f, v, w);
    } else {
        orc_axpby(n, -lr, g, 1 - lr * l2, w);
    }
    for (size_t i = 0; i < n; ++i) g[i] = 0.0f;
}

/* IOptimizer::ClipGradients over the tensors of a parameter set (src/nn/optimizer.cpp:16-32): norm = sqrt of the
 * sum of the squared 2-norms (each Norm2 a float), factor = threshold / norm when the norm exceeds it, else 1. */
float orc_clip_factor(int tensors, const float* const* g, const size_t* n, float threshold)
{
    float norm = 0.0f;
    for (int t = 0; t < tensors; ++t) {
        double sq = 0.0;
        for (size_t i = 0; i < n[t]; ++i) sq += (double)g[t][i] * (double)g[t][i];
        const float norm2 = (float)sqrt(sq);
        norm += norm2 * norm2;
    }
    norm = sqrtf(norm);
    return norm > threshold ? threshold / norm : 1.0f;
}

/* One AdamOptimizer::Update on one tensor (src/nn/optimizer.cpp:105-160) as the calls it makes, gscale being
 * what ClipGradients returned and t the iteration count after the increment:
 * grad.RowSparseAxpby(l2, value, gscale); m.RowSparseAxpby(1 - b1, grad, b1); grad.Square();
 * v.RowSparseAxpby(1 - b2, grad, b2); v_hat = v; Scale(s2); Sqrt; Add(eps); Inv; ElewiseMul(m);
 * value.RowSparseAxpby(-lr * s1, v_hat, 1.0); grad.RowSpZeros()        s1 = 1 / (1 - b1^t), s2 = 1 / (1 - b2^t) */
void orc_adam(size_t n, float* w, float* g, float* m, float* v, float lr, float l2, float gscale, float b1, float b2, float eps, int t)
{
    const float s1 = (float)(1.0 / (1 - pow(b1, t)));
    const float s2 = (float)(1.0 / (1 - pow(b2, t)));
    orc_axpby(n, l2, w, gscale, g);
    orc_axpby(n, 1 - b1, g, b1, m);
    for (size_t i = 0; i < n; ++i) g[i] = g[i] * g[i];
    orc_axpby(n, 1 - b2, g, b2, v);
    for (size_t i = 0; i < n; ++i) {
        float h = v[i] * s2;
        h = sqrtf(h);
        h = h + eps;
        h = 1.0f / h;
        g[i] = h * m[i];                       /* v_hat, kept in the gradient's storage */
    }
    orc_axpby(n, -lr * s1, g, 1.0f, w);
    for (size_t i = 0; i < n; ++i) g[i] = 0.0f;
}

/* Global sum / mean: sequential fp32 accumulation, mean = s / cnt
 * (src/tensor/cpu_dense_tensor.cpp:269-295). */
float orc_sum(const float* x, size_t n)
{
    float s = 0.0f;
    for (size_t i = 0; i < n; ++i) s += x[i];
    return s;
}

float orc_mean(const float* x, size_t n)
{
    return orc_sum(x, n) / (float)n;
}

float orc_max(const float* x, size_t n)
{
    float m = x[0];
    for (size_t i = 1; i < n; ++i) if (x[i] > m) m = x[i];
    return m;
}

/* Per-row index of the maximum, first index among ties (strict '>').
 * Reference: DTensor<CPU>::ArgMax (src/tensor/cpu_dense_tensor.cpp:176-196). */
void orc_row_argmax(const float* x, int rows, int cols, int* out)
{
    for (int i = 0; i < rows; ++i) {
        const float* p = x + (size_t)i * cols;
        int best = 0;
        float cur = p[0];
        for (int j = 1; j < cols; ++j)
            if (p[j] > cur) { cur = p[j]; best = j; }
        out[i] = best;
    }
}

/* Per-CSR-row column index of the largest stored value; empty row -> 0.
 * Reference: SpTensor<CPU>::ArgMax (src/tensor/cpu_sparse_tensor.cpp:86-103). */
void orc_csr_row_argmax(const int* row_ptr, const int* col_idx, const float* val, int rows, int* out)
{
    for (int i = 0; i < rows; ++i) {
        int best = 0;
        float cur = 0.0f;
        for (int j = row_ptr[i]; j < row_ptr[i + 1]; ++j)
            if (j == row_ptr[i] || val[j] > cur) { cur = val[j]; best = col_idx[j]; }
        out[i] = best;
    }
}

/* out[r] = -sum_k log(p[r, col[k]]) * val[k] over the label's CSR row, with
 * |p| < 1e-8 replaced by 1e-8; log and the product are evaluated in double and
 * the running loss is narrowed to fp32 after every term.
 * Reference: CalcCrossEntropy (src/nn/cross_entropy.cpp:7-25). */
void orc_cross_entropy(const float* prob, int rows, int cols, const int* lrow_ptr, const int* lcol,
                       const float* lval, float* out)
{
    for (int i = 0; i < rows; ++i) {
        float loss = 0.0f;
        for (int k = lrow_ptr[i]; k < lrow_ptr[i + 1]; ++k) {
            float t = prob[(size_t)cols * i + lcol[k]];
            if (fabs((double)t) < 1e-8) t = (float)1e-8;
            loss = (float)((double)loss - log((double)t) * (double)lval[k]);
        }
        out[i] = loss;
    }
}

/* out[r] = (#{j != t : p[r,j] > p[r,t]}) < k, t = label[r].
 * Reference: IsInTopK (src/nn/in_top_k.cpp:6-23). */
void orc_in_top_k(const float* pred, const int* label, int rows, int cols, int k, int* out)
{
    for (int i = 0; i < rows; ++i) {
        const float* p = pred + (size_t)i * cols;
        int t = 0, target = label[i];
        for (int j = 0; j < cols; ++j)
            if (j != target && p[j] > p[target]) t += 1;
        out[i] = t < k;
    }
}

/* TypeCast int -> float (src/nn/type_cast.cpp:13-29) */
void orc_cast_i32_f32(const int* src, float* dst, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = (float)src[i];
}

/* ------------------------------------------------------------------------
 * One mean-field level as the reference runs it, operator by operator
 * (examples/graph_classification/src/kernel_mean_field.cpp:35-42):
 *   n2npool      = A * h_in                 MatMul  (sparse x dense)
 *   node_linear  = n2npool * W              MatMul  (dense x dense)
 *   [+ bias row: ones[N,1] * bias[1,C], beta = 1   FullyConnected,
 *      src/nn/fully_connected.cpp:28-39]
 *   merged       = node_linear; merged += 1.0 * msg   ElewiseAdd (CopyFrom + Axpy)
 *   h_out        = merged; if (h_out < 0) h_out = 0   ReLU
 * tmp_pool is an [N,C] scratch for n2npool.
 * ---------------------------------------------------------------------- */
void orc_s2v_level(int N, int C, const int* row_ptr, const int* col_idx, const float* val,
                   const float* h_in, const float* W, const float* msg, const float* bias,
                   float* tmp_pool, float* h_out)
{
    orc_spmm_csr(N, C, 1.0f, row_ptr, col_idx, val, h_in, C, 0.0f, tmp_pool, C);
    orc_gemm(0, 0, N, C, C, 1.0f, tmp_pool, C, W, C, 0.0f, h_out, C);
    if (bias) {
#pragma omp parallel for schedule(static)
        for (int i = 0; i < N; ++i)
            for (int j = 0; j < C; ++j) h_out[(size_t)i * C + j] += 1.0f * bias[j];
    }
    if (msg) orc_axpy((size_t)N * C, 1.0f, msg, h_out);
    orc_unary(6, h_out, (size_t)N * C, 0.0f, 0.0f);
}

/* ------------------------------------------------------------------------
 * Whole forward, op order of kernel_mean_field.cpp:31-56.
 * ---------------------------------------------------------------------- */
void orc_s2v_forward(int N, int B, int K, int C, int H, int Q, int L,
                     const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                     const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                     const float* X, const float* W_n2l, const float* W_conv,
                     const float* W_h1, const float* W_h2,
                     const int* l_row_ptr, const int* l_col_idx, const float* l_val,
                     float* msg, float* h, float* pool, float* hidden, float* logits,
                     float* probs, float* loss_rows, int* pred, int* truth, int* hit,
                     float* scalars)
{
    const size_t NC = (size_t)N * C;
    float* tmp = (float*)malloc(sizeof(float) * (NC ? NC : 1));

    /* input_message = X * W_n2l ; input_potential_layer = ReLU(input_message) */
    orc_gemm(0, 0, N, C, K, 1.0f, X, K, W_n2l, C, 0.0f, msg, C);
    memcpy(h, msg, sizeof(float) * NC);
    orc_unary(6, h, NC, 0.0f, 0.0f);

    for (int lv = 0; lv < L; ++lv)
        orc_s2v_level(N, C, a_row_ptr, a_col_idx, a_val, h + (size_t)lv * NC, W_conv, msg, NULL,
                      tmp, h + (size_t)(lv + 1) * NC);

    /* y_potential = S * h_L ; hidden = ReLU(y * h1) ; output = hidden * h2 */
    orc_spmm_csr(B, C, 1.0f, s_row_ptr, s_col_idx, s_val, h + (size_t)L * NC, C, 0.0f, pool, C);
    orc_gemm(0, 0, B, H, C, 1.0f, pool, C, W_h1, H, 0.0f, hidden, H);
    orc_unary(6, hidden, (size_t)B * H, 0.0f, 0.0f);
    orc_gemm(0, 0, B, Q, H, 1.0f, hidden, H, W_h2, Q, 0.0f, logits, Q);

    /* CrossEntropy(need_softmax = true): probs = softmax(copy of logits) (src/nn/cross_entropy.cpp:33-50) */
    memcpy(probs, logits, sizeof(float) * (size_t)B * Q);
    orc_row_softmax(probs, B, Q);
    orc_row_argmax(logits, B, Q, pred);
    if (l_row_ptr) {
        orc_cross_entropy(probs, B, Q, l_row_ptr, l_col_idx, l_val, loss_rows);
        orc_csr_row_argmax(l_row_ptr, l_col_idx, l_val, B, truth);
        orc_in_top_k(logits, truth, B, Q, 1, hit);
        float* hitf = (float*)malloc(sizeof(float) * (size_t)(B ? B : 1));
        orc_cast_i32_f32(hit, hitf, (size_t)B);
        scalars[0] = orc_mean(loss_rows, (size_t)B);
        scalars[1] = orc_mean(hitf, (size_t)B);
        free(hitf);
    }
    free(tmp);
}
