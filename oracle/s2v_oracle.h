/*
 * TEST INFRASTRUCTURE ONLY — CPU restatement of graphnn's structure2vec
 * mean-field forward, used as the parity checker for the HIP library and as
 * the reported CPU baseline.  Nothing in the shipped library links, loads or
 * calls this file.
 *
 * Every function restates one reference routine; the citation is given beside
 * the implementation in s2v_oracle.c.  All matrices are row-major, dense data
 * is fp32, CSR indices are int32 (reference: include/tensor/t_data.h:123-165).
 */
#ifndef S2V_ORACLE_H
#define S2V_ORACLE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- batch graph -> CSR (integer work, bit-exact contract) ---- */
void orc_csr_node2node(int num_nodes, int num_edges, const int* edge_x, const int* edge_y,
                       int average, int* row_ptr, int* col_idx, float* val);
void orc_csr_edge2node(int num_nodes, int num_edges, const int* edge_y, int average,
                       int* row_ptr, int* col_idx, float* val);
void orc_csr_node2edge(int num_edges, const int* edge_x, int* row_ptr, int* col_idx, float* val);
int orc_csr_edge2edge(int num_nodes, int num_edges, const int* edge_x, const int* edge_y,
                      int* row_ptr, int* col_idx, float* val);
void orc_csr_subgraph(int num_subgraph, int num_nodes, const int* subg_id, const int* node_idx,
                      int average, int* row_ptr, int* col_idx, float* val);

/* ---- tensor ops ---- */
void orc_spmm_csr(int m, int n, float alpha, const int* row_ptr, const int* col_idx,
                  const float* val, const float* B, int ldb, float beta, float* C, int ldc);
/* float64 arbiter (not a reference routine): out = alpha * A * B in double, or the same sum over magnitudes */
void orc_spmm_csr_f64(int m, int n, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                      const float* B, int ldb, int absolute, double* out, int ldo);
void orc_spmm_csr_T(int m, int n, int k, float alpha, const int* row_ptr, const int* col_idx,
                    const float* val, const float* B, int ldb, float beta, float* C, int ldc);
void orc_gemm(int transA, int transB, int m, int n, int k, float alpha, const float* A, int lda,
              const float* B, int ldb, float beta, float* C, int ldc);
void orc_axpy(size_t n, float a, const float* x, float* y);
void orc_axpby(size_t n, float a, const float* x, float b, float* y);
void orc_unary(int op, float* x, size_t n, float a0, float a1);
void orc_row_softmax(float* x, int rows, int cols);
void orc_jagged_softmax(float* x, const int* lens, int nseg);
void orc_momentum_sgd(size_t n, float* w, float* g, float* v, float lr, float momentum, float l2);
float orc_clip_factor(int tensors, const float* const* g, const size_t* n, float threshold);
void orc_adam(size_t n, float* w, float* g, float* m, float* v, float lr, float l2, float gscale, float b1, float b2, float eps, int t);
void orc_jagged_softmax_deriv(float* dst, const float* out, const float* grad, const int* lens, int nseg);
float orc_sum(const float* x, size_t n);
float orc_mean(const float* x, size_t n);
float orc_max(const float* x, size_t n);
void orc_row_argmax(const float* x, int rows, int cols, int* out);
void orc_csr_row_argmax(const int* row_ptr, const int* col_idx, const float* val, int rows, int* out);
void orc_cross_entropy(const float* prob, int rows, int cols, const int* lrow_ptr, const int* lcol,
                       const float* lval, float* out);
void orc_in_top_k(const float* pred, const int* label, int rows, int cols, int k, int* out);
void orc_cast_i32_f32(const int* src, float* dst, size_t n);

/* one mean-field level written as the reference's four operators */
void orc_s2v_level(int N, int C, const int* row_ptr, const int* col_idx, const float* val,
                   const float* h_in, const float* W, const float* msg, const float* bias,
                   float* tmp_pool, float* h_out);

/* whole forward; every intermediate is caller-allocated and filled:
 * msg[N,C], h[(L+1),N,C], pool[B,C], hidden[B,H], logits[B,Q], probs[B,Q],
 * loss_rows[B], pred[B] (row argmax of logits), truth[B], hit[B], scalars[2]={loss, acc}. */
void orc_s2v_forward(int N, int B, int K, int C, int H, int Q, int L,
                     const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                     const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                     const float* X, const float* W_n2l, const float* W_conv,
                     const float* W_h1, const float* W_h2,
                     const int* l_row_ptr, const int* l_col_idx, const float* l_val,
                     float* msg, float* h, float* pool, float* hidden, float* logits,
                     float* probs, float* loss_rows, int* pred, int* truth, int* hit,
                     float* scalars);

/* number of OpenMP threads the library was built to use (1 when built without OpenMP) */
int orc_num_threads(void);
void orc_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
