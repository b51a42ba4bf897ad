/*
 * gnnhip — C ABI of the gfx950 (MI355X) backend for graphnn's structure2vec
 * mean-field forward.  Plain pointers and sizes only; every pointer named
 * "device" is HIP device memory, every matrix is row-major fp32, every CSR
 * index is int32 (reference layout: include/tensor/t_data.h:123-165).
 *
 * Conventions
 *   - every entry returns GNNHIP_OK (0) or a negative GNNHIP_E* code and never
 *     throws; gnnhip_last_error() gives the text for the calling thread.
 *   - `stream` is a hipStream_t passed as void*; NULL means the HIP null stream.
 *     Calls are asynchronous on that stream except where stated.
 *   - the library keeps no caller pointer after the call's work on the stream
 *     has finished; outputs are caller-allocated.
 *   - one host thread at a time feeds a stream: the scratch and the pinned
 *     staging buffers that the library keeps per stream belong to the call in
 *     progress.  Threads that work side by side use a stream each.
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the graphnn source tree).
 *
 * The library reads no environment variable: which kernel a call takes depends on its arguments alone.
 */
#ifndef GNNHIP_H
#define GNNHIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GNNHIP_OK            0
#define GNNHIP_EINVAL       -1   /* bad argument (null pointer, negative size, bad op code) */
#define GNNHIP_ENOMEM       -2   /* device allocation failed */
#define GNNHIP_EHIP         -3   /* a HIP runtime call failed */
#define GNNHIP_ENOTINIT     -4   /* gnnhip_init has not been called */
#define GNNHIP_EUNSUPPORTED -5   /* shape outside what the kernels handle */

/* unary functor codes — include/tensor/gpu_unary_functor.h:17-327 */
enum {
    GNNHIP_UNARY_SET = 0, GNNHIP_UNARY_TRUNCATE = 1, GNNHIP_UNARY_SCALE = 2, GNNHIP_UNARY_ADD = 3,
    GNNHIP_UNARY_ABS = 4, GNNHIP_UNARY_INV = 5, GNNHIP_UNARY_RELU = 6, GNNHIP_UNARY_SIGMOID = 7,
    GNNHIP_UNARY_TANH = 8, GNNHIP_UNARY_LOG = 9, GNNHIP_UNARY_INVSQRT = 10, GNNHIP_UNARY_EXP = 11,
    GNNHIP_UNARY_SQUARE = 12, GNNHIP_UNARY_SQRT = 13, GNNHIP_UNARY__COUNT = 14
};

/* reduction codes — include/tensor/gpu_reduce_kernel.h:12-55 */
enum { GNNHIP_REDUCE_SUM = 0, GNNHIP_REDUCE_MEAN = 1, GNNHIP_REDUCE_MAX = 2, GNNHIP_REDUCE_SUMSQ = 3 };

const char* gnnhip_last_error(void);
const char* gnnhip_version(void);

/* ---- runtime: GpuHandle::Init / Destroy (include/tensor/gpu_handle.h:38-59,
 *      src/tensor/gpu_handle.cu:17-70).  No vendor BLAS/SPARSE handles exist. */
int gnnhip_init(int device_id);
int gnnhip_shutdown(void);

/* ---- pooled device memory: MemHolder<GPU>::MallocArr / Recycle / ForceDel
 *      (include/util/mem_holder.h:20-51, src/util/mem_holder.cpp:15-97).
 *      malloc takes the smallest parked block >= bytes or allocates; recycle
 *      parks the block for reuse; free returns it to the driver.
 *      recycle knows nothing of streams (neither does MemHolder): the block may be handed out again at
 *      once, so the caller must not recycle a block while work queued on a stream still uses it unless the
 *      next user is ordered behind that work (same stream, or an event). */
int gnnhip_malloc(void** device_ptr, size_t bytes);
int gnnhip_recycle(void* device_ptr);
int gnnhip_free(void* device_ptr);
int gnnhip_pool_stats(size_t* bytes_in_use, size_t* bytes_parked, size_t* n_driver_allocs);
/* Scratch the library keeps per stream (plans and partial sums of products with large matrices run to gigabytes; the
 * reference's counterpart is the temporary storage its cuSPARSE / cuBLAS handles keep, src/tensor/gpu_handle.cu:17-70):
 * waits for the stream and gives that stream's scratch back to the driver.  The next call that needs scratch takes it anew. */
int gnnhip_release_scratch(void* stream);

/* ---- copies: DTensor<GPU>::CopyFrom / AsScalar / Zeros
 *      (src/tensor/gpu_dense_tensor.cu:97-150), SpTensor<GPU>::CopyFrom
 *      (src/tensor/gpu_sparse_tensor.cu:55-73).  h2d returns once the host buffer
 *      has been read (it may be overwritten at once); d2h blocks until the data is in
 *      host memory; d2d and memset0 are asynchronous on the stream.
 *      h2d_sparse32 is h2d for `words` 32-bit words that are mostly zero (the one-hot feature matrix GetBatch
 *      fills, examples/graph_classification/include/nn_common.h:60-75): it sends the non-zero words with their
 *      positions and rebuilds the buffer on the device (same bits, same promise); dense data takes the plain copy.
 *      From about four million words on the scan for non-zero words is shared by up to eight host threads, started and
 *      joined inside the call. */
int gnnhip_memcpy_h2d(void* dst_device, const void* src_host, size_t bytes, void* stream);
int gnnhip_memcpy_h2d_sparse32(void* dst_device, const void* src_host, size_t words, void* stream);
int gnnhip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream);
/* ---- count host-to-device copies with the promise of gnnhip_memcpy_h2d, in one launch where the pieces allow it
 *      (whole 32-bit words, up to 8 pieces, 2 MB together): the three arrays that SpTensor<GPU>::CopyFrom(CPU) sends
 *      one by one (src/tensor/gpu_sparse_tensor.cu:55-63).  dst_device, src_host, bytes: host arrays of count entries. */
int gnnhip_memcpy_h2d_batch(int count, void* const* dst_device, const void* const* src_host, const size_t* bytes, void* stream);
int gnnhip_memcpy_d2d(void* dst_device, const void* src_device, size_t bytes, void* stream);
/* ---- count small device-to-host reads behind ONE wait for the stream: the loss and the accuracy that the example
 *      reads one after the other with DTensor<GPU>::AsScalar (src/tensor/gpu_dense_tensor.cu:129-137, read at
 *      examples/graph_classification/include/nn_common.h:140-160).  dst_host, src_device, bytes: host arrays of count
 *      entries; pieces of up to 4 KB together land in pinned memory, larger ones are read one by one. */
int gnnhip_memcpy_d2h_batch(int count, void* const* dst_host, const void* const* src_device, const size_t* bytes, void* stream);
int gnnhip_memset0(void* device_ptr, size_t bytes, void* stream);
/* n buffers zeroed in one launch (the gradient tensors FactorGraph::BackPropagate clears one by one,
 * src/nn/factor_graph.cpp:190-196); entries with 0 bytes are skipped. */
int gnnhip_memset0_batch(int n, void* const* device_ptrs, const size_t* bytes, void* stream);
int gnnhip_stream_sync(void* stream);

/* ---- C[m,n] = alpha * A * B + beta * C, A CSR [m,k], B dense [k,n].
 *      DTensor<GPU>::MM(SpTensor, DTensor, Trans::N, Trans::N) + CSRMMKernel
 *      (src/tensor/gpu_dense_tensor.cu:227-239,257-270).  beta == 0 overwrites C.
 *      nnz is the host-side entry count of A (SparseData::nnz, include/tensor/t_data.h:123-165);
 *      it sizes the buffers of the balanced pass over high-degree rows and nothing else: every read of
 *      col_idx / val is bounded by the matrix's own row_ptr[m] on the device.  A value smaller than
 *      row_ptr[m] is safe (rows that do not fit are summed in place), a larger one wastes memory. */
int gnnhip_spmm_csr_f32(int m, int k, int n, int nnz, float alpha, const int* row_ptr, const int* col_idx,
                        const float* val, const float* B, int ldb, float beta, float* C, int ldc,
                        void* stream);

/* ---- a plan for a CSR matrix that is multiplied with many times: what DTensor<GPU>::MM(SpTensor, DTensor, N, N)
 *      (src/tensor/gpu_dense_tensor.cu:227-239,257-270) would work out again on every call for the same operand
 *      (the reference holds its sparse operand in SpTensor<GPU>, src/tensor/gpu_sparse_tensor.cu:25-63, across all the
 *      levels of a batch and across batches of one big graph).  For large matrices with many entries per row
 *      (power-law graphs) the plan holds the rows cut into pieces of consecutive entries, ordered by the column they
 *      start at, and the entries copied into that order; for every matrix the plan of the balanced pass over long
 *      rows.  plan_create reads the matrix on `stream`, blocks until the plan is built (it reads back the number of
 *      pieces to size its arrays exactly), and owns pool memory of about 8 bytes per entry plus 16 per piece; the
 *      partial sums of a product (4n bytes per piece of a row of several pieces) are added at the first use.
 *      The CSR arrays must stay alive and unchanged (structure and values) while the plan is used; when they change,
 *      destroy the plan and make a new one.  Calls that share a plan must be ordered one after the other (they share its partial
 *      sums); plan_destroy waits for the device.  spmm_csr_planned / s2v_level_planned give bit-identical results to
 *      gnnhip_spmm_csr_f32 / gnnhip_s2v_level_f32 on the same arrays (same kernels, same order of every sum).
 *      plan_bytes: device bytes the plan owns at present. */
int gnnhip_csr_plan_create(int m, int k, const int* row_ptr, const int* col_idx, const float* val, void* stream, void** plan);
int gnnhip_csr_plan_destroy(void* plan);
int gnnhip_csr_plan_bytes(void* plan, size_t* bytes);
int gnnhip_spmm_csr_planned_f32(void* plan, int n, float alpha, const float* B, int ldb, float beta, float* C, int ldc,
                                void* stream);

/* ---- CSR from (key, payload) pairs on the device: row i lists the payloads of the pairs with key i in
 *      input order, i.e. what the message-pass factors build on the host from the per-node lists:
 *      Node2NodeMsgPass (key = edge head y, payload = edge tail x), Edge2NodeMsgPass (payload = edge
 *      index), SubgraphMsgPass (key = subgraph, payload = node) -- src/nn/msg_pass.cpp:46-94,156-177,
 *      lists filled by GraphStruct::AddEdge / AddNode (src/util/graph_struct.cpp:62-75).
 *      key[e * key_stride], payload[e * payload_stride] (strides in ints, so an array of (x, y) pairs
 *      can be passed as it is).  val = 1, or 1 / row length when average != 0.  Stable radix sort without
 *      atomics on global memory, or, for up to 65,536 pairs (2.35 bytes each, plus 4 bytes per row of a
 *      sixteenth of the rows, have to fit 160 KB of LDS), one launch that puts every row back into input order:
 *      either way the result is a pure function of the input, bit-identical to the host construction.
 *      The outputs must not overlap key or payload. */
int gnnhip_csr_group_i32(int rows, int n, const int* key, int key_stride, const int* payload, int payload_stride,
                         int average, int* row_ptr, int* col_idx, float* val, void* stream);

/* ---- the entries of a CSR matrix whose row i lists the consecutive columns row_ptr[i] .. row_ptr[i+1]-1 with value 1
 *      (1 / row length when average != 0): the operand of SubgraphMsgPass (src/nn/msg_pass.cpp:156-177) for a batch
 *      whose nodes were added subgraph after subgraph, as GetBatch adds them
 *      (examples/graph_classification/include/nn_common.h:36-105).  row_ptr [rows+1] is on the device already (the
 *      subgraph offsets, which the host knows); col_idx and val have row_ptr[rows] entries. */
int gnnhip_csr_consecutive_rows_f32(int rows, const int* row_ptr, int average, int* col_idx, float* val, void* stream);
/* ---- the same operand of SubgraphMsgPass (src/nn/msg_pass.cpp:156-177) from the subgraph offsets in HOST memory
 *      (offsets_host [rows+1], free again when the call returns): row_ptr [rows+1] on the device receives them, col_idx
 *      and val the entries, in one launch. */
int gnnhip_csr_consecutive_rows_host_f32(int rows, const int* offsets_host, int average, int* row_ptr, int* col_idx, float* val,
                                         void* stream);

/* ---- the n pairs (x, y) grouped both ways at once, values 1: row i of (row_ptr, col_idx, val) lists the x of the
 *      pairs with y = i, which is gnnhip_csr_group_i32(rows, n, y, .., x, .., 0, ..), the operand of
 *      Node2NodeMsgPass (src/nn/msg_pass.cpp:46-67); row i of (t_row_ptr, t_col_idx, t_val) lists the y of the
 *      pairs with x = i: its transpose, which the reference leaves to cuSPARSE csrmm with Trans::T in the backward
 *      pass (src/tensor/gpu_dense_tensor.cu:271-296).  Both [rows, rows], entries in pair order; one launch where
 *      the one-launch grouping fits, two groupings otherwise. */
int gnnhip_csr_group_both_i32(int rows, int n, const int* x, int x_stride, const int* y, int y_stride,
                              int* row_ptr, int* col_idx, float* val, int* t_row_ptr, int* t_col_idx, float* t_val, void* stream);

/* ---- CSR of the transpose: A [m,k] with nnz entries -> A^T [k,m]; entries of a row of A^T keep the
 *      order of the rows of A they came from.  The reference transposes implicitly inside cuSPARSE
 *      csrmm for MM(SpTensor, DTensor, Trans::T) (src/tensor/gpu_dense_tensor.cu:271-296). */
int gnnhip_csr_transpose_f32(int m, int k, int nnz, const int* row_ptr, const int* col_idx, const float* val,
                             int* t_row_ptr, int* t_col_idx, float* t_val, void* stream);

/* ---- C[m,n] = alpha * op(A) * op(B) + beta * C, all dense row-major.
 *      DTensor<GPU>::MM(DTensor, DTensor) (src/tensor/gpu_dense_tensor.cu:192-224).
 *      transA/transB: 0 = N, 1 = T.  lda/ldb/ldc are row strides of the stored matrices. */
int gnnhip_gemm_f32(int transA, int transB, int m, int n, int k, float alpha, const float* A, int lda,
                    const float* B, int ldb, float beta, float* C, int ldc, void* stream);

/* ---- count products C_p[m_p,n_p] = alpha * A_p^T * B_p + beta * C_p in two launches, with A_p stored [k_p,m_p]
 *      and B_p [k_p,n_p]: the weight gradients that MatMul::Backward forms one by one at the end of a backward pass
 *      (src/nn/matmul.cpp:35-76, x^T * dy through DTensor<GPU>::MM, src/tensor/gpu_dense_tensor.cu:192-224).
 *      m, n, k, lda, ldb, ldc and the pointer tables A, B, C are HOST arrays of count entries; the matrices are
 *      device memory.  Every product gives the bits gnnhip_gemm_f32(1, 0, ...) gives for it alone when that
 *      call splits k (few output tiles, k >= 256).  A product with a 128 x 128 or 256 x 256 output and k >= 8192 (the
 *      level weight gradient at hidden 128 / 256) is taken out of the batch and gets the two launches of its own that
 *      the single call gives it (the whole output in one workgroup's registers over a range of k). */
int gnnhip_gemm_tn_batch_f32(int count, const int* m, const int* n, const int* k, const float* const* A, const int* lda,
                             const float* const* B, const int* ldb, float alpha, float beta, float* const* C, const int* ldc,
                             void* stream);

/* ---- one mean-field level in a single pass:
 *      h_out = ReLU((A * h_in) * W + bias + msg)
 *      replaces MatMul(sparse) + MatMul(dense) + ElewiseAdd + ReLU
 *      (examples/graph_classification/src/kernel_mean_field.cpp:35-42,
 *       src/nn/matmul.cpp:13-33, src/nn/elewise_add.cpp:13-33, src/nn/relu.cu:9-13;
 *       bias as in src/nn/fully_connected.cpp:28-39).  msg and bias may be NULL.
 *      A is [N,N] CSR with nnz entries (see gnnhip_spmm_csr_f32), h_in/h_out/msg are [N,C], W is [C,C];
 *      h_out must not alias h_in. */
int gnnhip_s2v_level_f32(int N, int C, int nnz, const int* row_ptr, const int* col_idx, const float* val,
                         const float* h_in, const float* W, const float* msg, const float* bias,
                         float* h_out, void* stream);

/* ---- the same level with the plan of A (gnnhip_csr_plan_create; A must be square): the levels of
 *      examples/graph_classification/src/kernel_mean_field.cpp:35-42 all multiply with the same n2nsum_param. */
int gnnhip_s2v_level_planned_f32(void* plan, int C, const float* h_in, const float* W, const float* msg, const float* bias,
                                 float* h_out, void* stream);

/* ---- msg = X * W_n2l and h0 = ReLU(msg) in one pass
 *      (examples/graph_classification/src/kernel_mean_field.cpp:31-32: MatMul + ReLU).  X [N,K], W_n2l [K,C].
 *      h0 may be NULL: only msg is written. */
int gnnhip_s2v_input_f32(int N, int K, int C, const float* X, const float* W_n2l,
                         float* msg, float* h0, void* stream);

/* ---- the same input stage when the node features are one label per node (what GetBatch encodes as the
 *      one-hot rows of X, examples/graph_classification/include/nn_common.h:57-69): msg[i,:] = W_n2l[label[i],:],
 *      bit-identical to X * W_n2l with X one-hot, and 4 N bytes of input instead of 4 N K.
 *      node_label: device int[N] with values in [0, K).  msg or h0 may be NULL.  status (device int, may be NULL;
 *      caller zeroes it) gets bit 3 set if a label lies outside [0, K); such a label is clamped. */
int gnnhip_s2v_input_labels_f32(int N, int K, int C, const int* node_label, const float* W_n2l,
                                float* msg, float* h0, int* status, void* stream);

/* ---- readout: pool = S * h ; hidden = ReLU(pool * W_h1) ; logits = hidden * W_h2 ;
 *      probs = softmax(logits) ; pred = row argmax(logits)
 *      (examples/graph_classification/src/kernel_mean_field.cpp:44-49 and the softmax of
 *      src/nn/cross_entropy.cpp:45-47).
 *      S is [B,N] CSR.  pool [B,C], hidden [B,H], logits/probs [B,Q], pred int[B];
 *      probs and pred may be NULL. */
int gnnhip_s2v_readout_f32(int B, int N, int C, int H, int Q,
                           const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                           const float* h, const float* W_h1, const float* W_h2,
                           float* pool, float* hidden, float* logits, float* probs, int* pred,
                           void* stream);

/* ---- whole forward = input + L levels + readout, device-resident.
 *      h_a / h_b are [N,C] ping-pong buffers; *which_h (host int, may be NULL)
 *      receives 0 if the final embedding is in h_a, 1 if in h_b (which of the two holds which level is
 *      the library's choice: with L >= 1 the first level may read ReLU(msg) straight from msg, and
 *      h0 is then never stored).  a_nnz: entries of A.
 *      Op sequence of examples/graph_classification/src/kernel_mean_field.cpp:31-49 scheduled by
 *      FactorGraph::SequentialForward (src/nn/factor_graph.cpp:75-144). */
int gnnhip_s2v_forward_f32(int N, int B, int K, int C, int H, int Q, int L, int a_nnz,
                           const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                           const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                           const float* X, const float* W_n2l, const float* W_conv,
                           const float* W_h1, const float* W_h2,
                           float* msg, float* h_a, float* h_b,
                           float* pool, float* hidden, float* logits, float* probs, int* pred,
                           int* which_h, void* stream);

/* ---- the same forward with the plan of A (gnnhip_csr_plan_create; N = the plan's rows): for callers that run the network
 *      of examples/graph_classification/src/kernel_mean_field.cpp:31-56 over one large graph batch after batch, where
 *      the reference rebuilds nothing but the features.  Same bits as gnnhip_s2v_forward_f32. */
int gnnhip_s2v_forward_planned_f32(void* a_plan, int B, int K, int C, int H, int Q, int L,
                                   const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                   const float* X, const float* W_n2l, const float* W_conv,
                                   const float* W_h1, const float* W_h2,
                                   float* msg, float* h_a, float* h_b,
                                   float* pool, float* hidden, float* logits, float* probs, int* pred,
                                   int* which_h, void* stream);

/* ---- the same forward for block-diagonal batches of small graphs, in ONE launch with the
 *      embeddings resident in LDS: the op sequence of
 *      examples/graph_classification/src/kernel_mean_field.cpp:31-49 on a batch laid out by GetBatch
 *      (examples/graph_classification/include/nn_common.h:36-105), i.e. graph g owns the contiguous
 *      nodes [s_row_ptr[g], s_row_ptr[g+1]), s_col_idx[i] == i, and no entry of A joins two graphs.
 *      max_graph_nodes (host int) bounds the largest graph.  h_final [N,C] receives the last-level
 *      embedding.  status (device int, may be NULL; caller zeroes it) gets bit 0 set if a graph
 *      exceeds max_graph_nodes, bit 1 if an edge leaves its graph, bit 2 if S is not the identity
 *      layout; results are then unspecified but no access goes out of bounds.
 *      From 512 graphs on (H and Q up to 64) runs of consecutive graphs are packed into bins of 128
 *      to 208 nodes that one workgroup carries as a single block-diagonal graph; the bound on a graph
 *      is then the bin size where that is larger than max_graph_nodes.  Node outputs keep their
 *      bits, graph outputs agree with the unpacked ones to rounding.
 *      Returns GNNHIP_EUNSUPPORTED (nothing launched) for shapes it does not cover
 *      (hidden not in {16,32,64}, more than 64 label types, graph too large for LDS). */
int gnnhip_s2v_forward_batched_f32(int N, int B, int K, int C, int H, int Q, int L, int max_graph_nodes,
                                   const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                                   const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                   const float* X, const float* W_n2l, const float* W_conv,
                                   const float* W_h1, const float* W_h2,
                                   float* msg, float* h_final, float* pool, float* hidden, float* logits,
                                   float* probs, int* pred, int* status, void* stream);

/* ---- the one-launch forward of a training iteration: as gnnhip_s2v_forward_batched_f32, and the embeddings of
 *      all levels are kept for the backward pass (FactorGraph::FeedForward with Phase::TRAIN keeps every factor's
 *      output, src/nn/factor_graph.cpp:146-180): h_levels [(L + 1), N, C] receives h_0 = ReLU(msg) and h_1 .. h_L
 *      (h_L is what the inference entry returns as h_final).  Same limits, status bits and return codes. */
int gnnhip_s2v_forward_batched_train_f32(int N, int B, int K, int C, int H, int Q, int L, int max_graph_nodes,
                                         const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                                         const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                         const float* X, const float* W_n2l, const float* W_conv,
                                         const float* W_h1, const float* W_h2,
                                         float* msg, float* h_levels, float* pool, float* hidden, float* logits,
                                         float* probs, int* pred, int* status, void* stream);

/* ---- the one-launch forward with one label per node in place of the one-hot matrix X (see
 *      gnnhip_s2v_input_labels_f32; the batch layout is GetBatch's,
 *      examples/graph_classification/include/nn_common.h:36-105): the input stage becomes a row lookup in W_n2l [K,C] (K is not limited to 64),
 *      every output has the bits of gnnhip_s2v_forward_batched_f32 on the one-hot X.  status bit 3: a label
 *      outside [0, K) (clamped).  W_n2l must be 16-byte aligned. */
int gnnhip_s2v_forward_batched_labels_f32(int N, int B, int K, int C, int H, int Q, int L, int max_graph_nodes,
                                          const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                                          const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                          const int* node_label, const float* W_n2l, const float* W_conv,
                                          const float* W_h1, const float* W_h2,
                                          float* msg, float* h_final, float* pool, float* hidden, float* logits,
                                          float* probs, int* pred, int* status, void* stream);

/* ---- UnaryEngine<GPU>::Exec<Functor> (include/tensor/gpu_unary_functor.h:331-384):
 *      in-place x[i] = f(x[i]); a0/a1 are the functor's constructor arguments. */
int gnnhip_unary_f32(int op, float* x, size_t n, float a0, float a1, void* stream);

/* ---- out = ReLU(in) without the intermediate copy: ReLUAct(GPU) (src/nn/relu.cu:9-13) */
int gnnhip_relu_f32(const float* in, float* out, size_t n, void* stream);

/* ---- y += a*x : DTensor<GPU>::Axpy (src/tensor/gpu_dense_tensor.cu:489-496);
 *      y = a*x + b*y : Axpby. */
int gnnhip_axpy_f32(size_t n, float a, const float* x, float* y, void* stream);
int gnnhip_axpby_f32(size_t n, float a, const float* x, float b, float* y, void* stream);

/* ---- out = a + b (the ElewiseAdd of two operands without the copy, src/nn/elewise_add.cpp:13-33) */
int gnnhip_add_f32(size_t n, const float* a, const float* b, float* out, void* stream);

/* ---- row softmax in place: DTensor<GPU>::Softmax (src/tensor/gpu_dense_tensor.cu:298-370) */
int gnnhip_row_softmax_f32(float* x, int rows, int cols, void* stream);

/* ---- softmax over consecutive segments of a column vector; lens is a device int[nseg]:
 *      DTensor<GPU>::JaggedSoftmax (src/tensor/gpu_dense_tensor.cu:372-450).
 *      Segment offsets come from an exclusive scan of lens done on the device. */
int gnnhip_jagged_softmax_f32(float* x, const int* lens, int nseg, void* stream);

/* ---- the same jagged softmax for callers that cannot allocate device memory (code under HIP graph
 *      capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 *      The segment offsets live in an array that is part of the library's device image (256 KiB per GPU,
 *      held until the process ends), so the call makes no hipMalloc / hipFree and no allocating library
 *      call.  nseg <= GNNHIP_JAGGED_STATIC_MAX_SEGMENTS, otherwise GNNHIP_EINVAL and nothing is launched.
 *      All calls on one GPU share that array: calls that overlap on one GPU (different streams, or
 *      different threads) race; order them on one stream. */
#define GNNHIP_JAGGED_STATIC_MAX_SEGMENTS 65536
int gnnhip_jagged_softmax_static_f32(float* x, const int* lens, int nseg, void* stream);

/* ---- global sum / mean / max / sum of squares into out[0] (device):
 *      DTensor<GPU>::Sum / Mean (src/tensor/gpu_dense_tensor.cu:466-481),
 *      MatColReduceKernel (include/tensor/gpu_reduce_kernel.h:57-99) */
int gnnhip_reduce_f32(int op, const float* x, size_t n, float* out, void* stream);

/* ---- per-row arg-max, first index among ties (the CPU rule,
 *      src/tensor/cpu_dense_tensor.cpp:176-196; GPU call site gpu_dense_tensor.cu:184-190) */
int gnnhip_row_argmax_f32(const float* x, int rows, int cols, int* out, void* stream);

/* ---- per-CSR-row column of the largest stored value, empty row -> 0:
 *      SpTensor<GPU>::ArgMax (src/tensor/gpu_sparse_tensor.cu:82-122; CPU rule
 *      src/tensor/cpu_sparse_tensor.cpp:86-103) */
int gnnhip_csr_row_argmax_f32(const int* row_ptr, const int* col_idx, const float* val, int rows,
                              int* out, void* stream);

/* ---- out[r] = -sum_k log(p[r, lcol[k]]) * lval[k], |p| < 1e-8 clamped to 1e-8:
 *      CalcCrossEntropy (src/nn/cross_entropy.cu:9-49; clamp of src/nn/cross_entropy.cpp:18-19) */
int gnnhip_cross_entropy_f32(const float* prob, int rows, int cols, const int* lrow_ptr,
                             const int* lcol, const float* lval, float* out, void* stream);

/* ---- out[r] = (#{j != label[r] : p[r,j] > p[r,label[r]]}) < k :
 *      IsInTopK (src/nn/in_top_k.cu:9-51) */
int gnnhip_in_top_k_f32(const float* pred, const int* label, int rows, int cols, int k, int* out,
                        void* stream);

/* ---- dst[i] = (float)src[i] : TypeCastCopy (src/tensor/gpu_binary_functor.cu:7-31) */
int gnnhip_cast_i32_f32(const int* src, float* dst, size_t n, void* stream);

/* ================= backward pass of the same path ================= */

/* ---- C[k,n] = alpha * A^T * B + beta * C, A CSR [m,k], B dense [m,n]:
 *      DTensor<GPU>::MM(SpTensor, DTensor, Trans::T, Trans::N) (src/tensor/gpu_dense_tensor.cu:271-294,
 *      the cuSPARSE csrmm(T) + two geam route), used by MatMul::Backward (src/nn/matmul.cpp:35-76).
 *      Accumulates with fp32 atomics: the order of additions into one output row is not fixed. */
int gnnhip_spmm_csr_t_f32(int m, int k, int n, float alpha, const int* row_ptr, const int* col_idx,
                          const float* val, const float* B, int ldb, float beta, float* C, int ldc,
                          void* stream);

/* ---- dense[r, col[t]] += a * val[t] : DTensor<GPU>::Axpy(a, SpTensor) + SpAxpyKernel
 *      (src/tensor/gpu_dense_tensor.cu:578-609), the label term of CrossEntropy::Backward
 *      (src/nn/cross_entropy.cpp:52-78). */
int gnnhip_csr_axpy_f32(int rows, int cols, float a, const int* row_ptr, const int* col_idx, const float* val,
                        float* dense, void* stream);

/* ---- dst[i] += grad[i] where out[i] > 0 : ReLUDeriv(GPU) + ReLUDerivKernel (src/nn/relu.cu:18-37) */
int gnnhip_relu_deriv_f32(size_t n, const float* out, const float* grad, float* dst, void* stream);

/* ---- dst += (grad - <grad, out>_segment) * out over the segments of a jagged softmax output:
 *      JaggedSoftmaxDeriv (CPU rule src/nn/jagged_softmax.cpp:8-31, called by JaggedSoftmax::Backward :57-74;
 *      graphnn's own GPU overload, src/nn/jagged_softmax.cu:9-12, is an empty body). */
int gnnhip_jagged_softmax_deriv_f32(float* dst, const float* out, const float* grad, const int* lens, int nseg,
                                    void* stream);

/* ---- gradient of the row softmax, per row: dst += out . (grad - <grad, out>)
 *      (Softmax::Backward -> SoftmaxDeriv, src/nn/softmax.cpp:8-29,53-70; cunn_SoftMax_updateGradInput_kernel,
 *      src/nn/softmax.cu:10-59).  dst, out, grad [rows, cols]; dst may not alias the others. */
int gnnhip_row_softmax_deriv_f32(float* dst, const float* out, const float* grad, int rows, int cols, void* stream);

/* ---- y[i] *= x[i] : DTensor<GPU>::ElewiseMul(DTensor) with equal shapes
 *      (src/tensor/gpu_dense_tensor.cu:611-628, include/tensor/gpu_binary_functor.h:40-95) */
int gnnhip_mul_f32(size_t n, const float* x, float* y, void* stream);

/* ---- y[r, :] *= scale[r] : the column-broadcast case of DTensor<GPU>::ElewiseMul
 *      (BCastEleWiseMulKernel, src/tensor/gpu_dense_tensor.cu:654-713) */
int gnnhip_row_scale_f32(int rows, int cols, const float* scale, float* y, void* stream);

/* ================= one training iteration in few launches ================= */

/* ---- loss and accuracy of a batch from its logits in one pass: the rows of
 *      CrossEntropy::Forward with softmax inside (src/nn/cross_entropy.cpp:33-50: DTensor::Softmax, then
 *      CalcCrossEntropy with the clamp of :18-19), their mean (ReduceMean, src/nn/reduce_mean.cpp:14-42),
 *      truth = SpTensor::ArgMax of the label rows (src/tensor/cpu_sparse_tensor.cpp:86-103), hit = IsInTopK with
 *      k = 1 (src/nn/in_top_k.cpp:6-23), its mean after TypeCast: what
 *      examples/graph_classification/src/kernel_mean_field.cpp:51-56 appends to the forward.
 *      logits [B,Q]; labels CSR [B,Q]; probs [B,Q], loss_rows [B], hit_rows int[B] may be NULL;
 *      loss_mean / acc_mean are device floats (one of them may be NULL). */
int gnnhip_s2v_loss_acc_f32(int B, int Q, const float* logits, const int* lrow_ptr, const int* lcol, const float* lval,
                            float* probs, float* loss_rows, int* hit_rows, float* loss_mean, float* acc_mean, void* stream);

/* ---- backward of the readout for a batch whose pooling matrix S lists every node exactly once:
 *      dlogits = scale * (probs - y)                       CrossEntropy::Backward (src/nn/cross_entropy.cpp:52-78),
 *                                                          scale = 1/B from ReduceMean::Backward (src/nn/reduce_mean.cpp:44-65)
 *      du = (dlogits * W_h2^T) . [hidden > 0]              MatMul::Backward + ReLUDeriv (src/nn/matmul.cpp:35-76, src/nn/relu.cu:18-37)
 *      g_h[node,:] = s_val * (du * W_h1^T)[graph of node]  MatMul::Backward of pool = S * h
 *      dlogits [B,Q], du [B,H] and g_h [N,C] are overwritten; the weight gradients are hidden^T * dlogits and
 *      pool^T * du (gnnhip_gemm_f32). */
int gnnhip_s2v_readout_backward_f32(int B, int N, int C, int H, int Q,
                                    const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                    const float* probs, const int* lrow_ptr, const int* lcol, const float* lval, float scale,
                                    const float* hidden, const float* W_h1, const float* W_h2,
                                    float* dlogits, float* du, float* g_h, void* stream);

/* ---- dz = g where h > 0, else 0 (ReLUDeriv, src/nn/relu.cu:18-37), and acc = dz or acc += dz (the gradient that
 *      ElewiseAdd::Backward passes on to msg, src/nn/elewise_add.cpp:35-52, summed over the levels).
 *      dz may alias g; dz or acc may be NULL. */
int gnnhip_s2v_grad_gate_f32(size_t n, const float* h, const float* g, float* dz, float* acc, int accumulate, void* stream);

/* ---- backward of one mean-field level past its ReLU gate, in one pass:
 *      u = A^T * dz ;  g_prev = u * W^T
 *      (MatMul::Backward twice, src/nn/matmul.cpp:35-76: through lin = agg * W and through agg = A * h_prev, taken
 *      in the other order, which is the same product; the reference runs cuSPARSE csrmm(T) + cuBLAS,
 *      src/tensor/gpu_dense_tensor.cu:271-294).  A^T is handed in as a CSR matrix [N,N] with nnz entries
 *      (gnnhip_csr_transpose_f32).  u [N,C] is also the other factor of the weight gradient:
 *      dW += h_prev^T * u  (= (A h_prev)^T dz).  dz, u and g_prev are three distinct buffers.
 *      gate_h (may be NULL): the embedding h_prev [N,C] whose ReLU the gradient passes next; g_prev is then stored
 *      past that gate (g_prev where h_prev > 0, else 0: ReLUDeriv, src/nn/relu.cu:18-37), ready to be the dz of the
 *      level below.  acc (may be NULL): acc += g_prev as stored (the gradient ElewiseAdd::Backward hands to msg,
 *      src/nn/elewise_add.cpp:35-52, summed over the levels).
 *      One launch at C = 16, 32, 64 and at C = 128, 256 (N * C * 4 < 4 GiB); other widths, and matrices of 32,768 rows
 *      and more with 12 entries per row and more, run SpMM, GEMM and gate one after the other. */
int gnnhip_s2v_level_backward_f32(int N, int C, int nnz, const int* t_row_ptr, const int* t_col_idx, const float* t_val,
                                  const float* dz, const float* W, float* u, float* g_prev, const float* gate_h, float* acc,
                                  void* stream);

/* ---- MomentumSGDOptimizer::Update over n tensors in one launch (src/nn/optimizer.cpp:69-92):
 *      momentum > 0:  g += l2 w ; v = lr g + momentum v ; w -= v ; g = 0      (v: the optimizer's acc_grad_dict)
 *      momentum == 0: w = -lr g + (1 - lr l2) w ; g = 0                        (v may be NULL)
 *      w, g, v: host arrays of n device pointers; count: host array of element counts. */
int gnnhip_momentum_sgd_batch_f32(int n, float* const* w, float* const* g, float* const* v, const size_t* count,
                                  float lr, float momentum, float l2, void* stream);

/* ---- AdamOptimizer::Update over n tensors (src/nn/optimizer.cpp:105-160), with the clipping factor of
 *      IOptimizer::ClipGradients (src/nn/optimizer.cpp:16-32) formed on the device:
 *      scale = clip_threshold / |all g| when that norm exceeds clip_threshold > 0, else 1 (clip_threshold <= 0: no clipping)
 *      g = l2 w + scale g ; m = (1 - beta1) g + beta1 m ; v = (1 - beta2) g^2 + beta2 v
 *      w -= lr s1 m / (sqrt(v s2) + eps) ; g = 0          s1 = 1 / (1 - beta1^t), s2 = 1 / (1 - beta2^t), formed by the caller
 *      m, v: the optimizer's first_moments / second_moments.  w, g, m, v: host arrays of n device pointers;
 *      count: host array of element counts. */
int gnnhip_adam_batch_f32(int n, float* const* w, float* const* g, float* const* m, float* const* v, const size_t* count,
                          float lr, float l2, float clip_threshold, float beta1, float beta2, float eps, float s1, float s2, void* stream);

#ifdef __cplusplus
}
#endif
#endif
