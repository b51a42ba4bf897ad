// Input stage of the structure2vec forward when the node features are one label per node:
// msg[i, :] = W_n2l[label[i], :] and h0 = ReLU(msg).
//
// graphnn's GetBatch writes the labels as a dense one-hot matrix X [N,K]
// (examples/graph_classification/include/nn_common.h:57-69) and the graph multiplies it by W_n2l
// (kernel_mean_field.cpp:31-32).  A one-hot row times W_n2l is one row of W_n2l: the lookup reads
// 4 N bytes of labels instead of 4 N K bytes of zeros and ones, and gives the same bits as the product
// (0 + w, so a weight of -0.0 comes out as +0.0, as it does from the sum).
// HBM-bound: 4 N + 4 K C read (W_n2l stays in L2), 4 N C written per output.
#include "gnnhip_internal.h"

namespace gnnhip {
namespace {

constexpr int kBlock = 256;

// one lane per group of four columns (C % 4 == 0, 16-byte aligned W_n2l / msg / h0)
__global__ __launch_bounds__(kBlock) void s2v_input_labels_kernel(long long nquads, int G, int K, int C, const int* __restrict__ label,
                                                                  const float* __restrict__ Wn2l, float* __restrict__ msg,
                                                                  float* __restrict__ h0, int* __restrict__ status)
{
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < nquads; i += (long long)gridDim.x * kBlock) {
        const long long row = i / G;
        const int f = (int)(i - row * G);
        int lab = label[row];
        if (lab < 0 || lab >= K) {                       // reported and clamped: no read leaves W_n2l
            if (status) atomicOr(status, 8);
            lab = min(max(lab, 0), K - 1);
        }
        const float4 w = *reinterpret_cast<const float4*>(Wn2l + (size_t)lab * C + 4 * f);
        const float4 v = make_float4(0.f + w.x, 0.f + w.y, 0.f + w.z, 0.f + w.w);
        if (msg) *reinterpret_cast<float4*>(msg + (size_t)row * C + 4 * f) = v;
        if (h0) *reinterpret_cast<float4*>(h0 + (size_t)row * C + 4 * f) = relu_ref4(v);
    }
}

// any C, any alignment
__global__ __launch_bounds__(kBlock) void s2v_input_labels_scalar_kernel(long long total, int K, int C, const int* __restrict__ label,
                                                                         const float* __restrict__ Wn2l, float* __restrict__ msg,
                                                                         float* __restrict__ h0, int* __restrict__ status)
{
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < total; i += (long long)gridDim.x * kBlock) {
        const long long row = i / C;
        const int c = (int)(i - row * C);
        int lab = label[row];
        if (lab < 0 || lab >= K) {
            if (status) atomicOr(status, 8);
            lab = min(max(lab, 0), K - 1);
        }
        const float v = 0.f + Wn2l[(size_t)lab * C + c];
        if (msg) msg[i] = v;
        if (h0) h0[i] = relu_ref(v);
    }
}

}  // namespace
}  // namespace gnnhip

using namespace gnnhip;

extern "C" int gnnhip_s2v_input_labels_f32(int N, int K, int C, const int* node_label, const float* W_n2l,
                                           float* msg, float* h0, int* status, void* stream)
{
    GNNHIP_REQUIRE(N >= 0 && K >= 1 && C >= 1, "bad shape in s2v_input_labels (N=%d K=%d C=%d)", N, K, C);
    if (N == 0) return GNNHIP_OK;
    GNNHIP_REQUIRE(node_label && W_n2l && (msg || h0), "null tensor in s2v_input_labels");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    const bool quads = (C % 4 == 0) && aligned16(W_n2l) && (!msg || aligned16(msg)) && (!h0 || aligned16(h0));
    const long long work = quads ? (long long)N * (C / 4) : (long long)N * C;
    long long blocks = (work + kBlock - 1) / kBlock;
    if (blocks > (long long)kNumCU * 32) blocks = (long long)kNumCU * 32;
    if (quads)
        hipLaunchKernelGGL(s2v_input_labels_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, work, C / 4, K, C, node_label,
                           W_n2l, msg, h0, status);
    else
        hipLaunchKernelGGL(s2v_input_labels_scalar_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, s, work, K, C, node_label,
                           W_n2l, msg, h0, status);
    GNNHIP_LAUNCH_CHECK("s2v_input_labels");
    return GNNHIP_OK;
}
