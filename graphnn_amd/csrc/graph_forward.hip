// Graph-resident structure2vec forward for batches of small graphs (gfx950).
//
// When a batch is block diagonal — graph g owns the contiguous node range
// [s_row_ptr[g], s_row_ptr[g+1]) and no edge leaves its graph, which is what
// graphnn's GetBatch produces (examples/graph_classification/include/nn_common.h:36-105)
// — every graph is an independent problem whose embeddings fit in LDS.  One
// workgroup then runs the whole forward of one graph:
//
//   msg = X W_n2l, h = ReLU(msg)                      (matrix cores, msg to HBM once)
//   L times:  agg = A_g h   (neighbour rows read from LDS)
//             h   = ReLU(agg W + msg)                  (matrix cores, h stays in LDS)
//   pool = sum_i s_val_i h_i ; hidden = ReLU(pool W_h1) ; logits = hidden W_h2 ;
//   probs = softmax(logits) ; pred = argmax(logits)
//
// replacing L + 2 launches and 2 L round trips of the [N,C] activations through
// HBM by one launch that reads the inputs once and writes msg, the final
// embedding and the per-graph outputs once.  The graph's CSR slice is staged in
// LDS and reused by all L levels.
//
// Work split inside the workgroup (4, 8 or 16 wavefronts): gathers split rows (C/4
// lanes per row); the contraction splits (16-column block) x (16-row tile):
// wavefront w owns column block w % (C/16) and every (WAVES / (C/16))-th tile, so it
// keeps only its own 16 columns of W^T in registers.  MFMA operand layout as in level.hip.
//
// The kernel's time is a chain of latencies of the largest graph, so the code keeps that chain short:
// the graph's position is asked for ahead of the weight loads; every global load of the staging (row
// pointers, columns, weights, pooling weights, X) is issued before the first of them is used; the
// first neighbours of a lane's rows stay in registers for all levels; the readout has three steps
// (pool partials | pooled row + hidden layer | logits + softmax in the registers of one wavefront).
#include "gnnhip_internal.h"
#include "buffer_addr.h"

// Phase markers for a timing build of this file; they expand to nothing in the library.
#ifndef GNNHIP_PHASE_MARK
#define GNNHIP_PHASE_MARK(i)
#endif

namespace gnnhip {
namespace {

constexpr int kEdgeCapMax = 4096;       // CSR entries of one graph staged in LDS (fewer if LDS is short); larger graphs read them from L2
constexpr size_t kLdsLimit = 160 * 1024;
constexpr int kLabelWeightCap = 8192;   // floats of W_n2l staged in LDS by the label-input variant; larger tables are read from L2
constexpr int kReadoutCap = 8192;       // floats of W_h1 and W_h2 staged in LDS; larger layers are read from L2

// LDS carve-up, in floats:
//   h[n16+1][C+4] (the last row stays zero) | agg[n16][C+4] (shared with the staged X rows and the pooling partials) | rp[n16+4] | sv[n16] | hid[H] | lg[Q]
//   | W_h1, W_h2 (when small) | col[ecap] | val[ecap]
struct GraphLds {
    // contraction steps of the input stage: the K label columns in groups of four, an even number of them
    __host__ __device__ static int input_steps(int K) { return ((K + 3) / 4 + 1) & ~1; }
    // the agg buffer also holds the staged X rows (n x 4 input_steps(K), zero-padded) and the pooling partials (waves x C)
    __host__ __device__ static size_t agg_floats(int n16, int C, int K, int block, bool labels = false)
    {
        size_t a = (size_t)n16 * (C + 4);
        const size_t p = (size_t)(block / 64) * C, x = labels ? 0 : (size_t)n16 * 4 * input_steps(K);
        if (p > a) a = p;
        if (x > a) a = x;
        return (a + 3) / 4 * 4;
    }
    // label input: the graph's labels [n16] and, when it is small enough, W_n2l [K][C] behind the edge cache
    __host__ __device__ static bool wn_staged(int C, int K) { return (size_t)K * C <= (size_t)kLabelWeightCap; }
    __host__ __device__ static size_t label_floats(int n16, int C, int K)
    {
        return (size_t)n16 + (wn_staged(C, K) ? (size_t)K * C : 0);
    }
    static size_t fixed_floats(int n16, int C, int K, int H, int Q, int block, bool labels = false)
    {
        const size_t wro = ((size_t)C * H + (size_t)H * Q <= (size_t)kReadoutCap) ? (size_t)C * H + (size_t)H * Q : 0;
        size_t f = (size_t)(n16 + 1) * (C + 4) + agg_floats(n16, C, K, block, labels) + (size_t)(2 * n16 + 4) + H + Q + wro;
        f = (f + 3) / 4 * 4;
        if (labels) f += (label_floats(n16, C, K) + 3) / 4 * 4;
        return f;
    }
    // entries of the edge cache that still fit under the LDS limit
    static int edge_cap(int n16, int C, int K, int H, int Q, int block, bool labels = false)
    {
        const size_t fixed = fixed_floats(n16, C, K, H, Q, block, labels) * sizeof(float);
        if (fixed >= kLdsLimit) return -1;
        size_t cap = (kLdsLimit - fixed) / (2 * sizeof(float));
        if (cap > (size_t)kEdgeCapMax) cap = kEdgeCapMax;
        return (int)(cap / 4 * 4);
    }
};

// Batches of more graphs than compute units are taken largest graph first: the graph of rank r in that order
// goes to workgroup r % gridDim.x as its (r / gridDim.x)-th graph.  Big graphs then start at once and small
// ones fill the slots that free up (400 graphs of the 10..110-node distribution: 34 -> 28 us).  The order is by
// the number of 16-row tiles, descending, equal counts in batch order.  It is worked out once per launch by the
// one-workgroup kernel below, which leaves a record per rank (graph, first node, node count, first entry, end
// of entries): the forward kernel then finds its graph with one read instead of two dependent ones.  Working
// the order out inside every workgroup of the forward kernel was tried first and costs 2.4 .. 7 us per
// workgroup, more than it saves.  What a graph's results are does not depend on the order.
constexpr int kOrderMinGraphs = kNumCU;          // up to here every graph has a compute unit of its own
constexpr int kOrderBlock = 1024;
constexpr int kOrderSlots = 4;                   // graphs a lane looks at
constexpr int kOrderMaxGraphs = kOrderSlots * kOrderBlock;
constexpr int kOrderRec = 8;                     // ints per record (five used; 32-byte records)
inline bool graphs_ordered(int B) { return B > kOrderMinGraphs && B <= kOrderMaxGraphs; }

__global__ __launch_bounds__(kOrderBlock) void graph_order_kernel(int B, int n16max, const int* __restrict__ a_row_ptr,
                                                                  const int* __restrict__ s_row_ptr, int* __restrict__ order)
{
    constexpr int kWaves = kOrderBlock / kWave;
    // counts[(ncls - 1 - cls) * nchunks + chunk] = graphs of tile count cls among graphs 64 chunk .. 64 chunk + 63;
    // an exclusive scan over that array in index order gives, for every (class, chunk), the rank of its first
    // graph (classes descending, batch order inside a class).  Graphs the host's size bound does not cover
    // form the top class: they come first and are refused by the forward kernel.
    __shared__ int counts[(kOrderMaxGraphs / kWave) * 64];       // up to 64 chunks x 64 classes
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int ncls = n16max / 16 + 2;                            // <= 64 (host-checked)
    const int nchunks = (B + kWave - 1) / kWave;
    const int total = ncls * nchunks;
    int first[kOrderSlots], count[kOrderSlots], e0[kOrderSlots], e1[kOrderSlots], cls[kOrderSlots];
#pragma unroll
    for (int j = 0; j < kOrderSlots; ++j) {
        const int g = (wave + j * kWaves) * kWave + lane;
        first[j] = 0; count[j] = -1; e0[j] = 0; e1[j] = 0;
        if (g < B) { first[j] = s_row_ptr[g]; count[j] = s_row_ptr[g + 1] - first[j]; }
    }
#pragma unroll
    for (int j = 0; j < kOrderSlots; ++j) {
        const int g = (wave + j * kWaves) * kWave + lane;
        const bool fits = count[j] >= 0 && count[j] <= n16max;
        if (fits) { e0[j] = a_row_ptr[first[j]]; e1[j] = a_row_ptr[first[j] + count[j]]; }
        cls[j] = g >= B ? -1 : fits ? (count[j] + 15) >> 4 : ncls - 1;
    }
#pragma unroll
    for (int j = 0; j < kOrderSlots; ++j) {
        const int ch = wave + j * kWaves;
        if (ch < nchunks) {
            for (int c = 0; c < ncls; ++c) {
                const unsigned long long m = __ballot(cls[j] == c);
                if (lane == 0) counts[(ncls - 1 - c) * nchunks + ch] = __popcll(m);
            }
        }
    }
    __syncthreads();
    if (wave == 0) {
        int carry = 0;
        for (int base = 0; base < total; base += kWave) {
            const int i = base + lane;
            const int v = i < total ? counts[i] : 0;
            int incl = v;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) {
                const int o = __shfl_up(incl, d, kWave);
                if (lane >= d) incl += o;
            }
            if (i < total) counts[i] = carry + incl - v;
            carry += __shfl(incl, kWave - 1, kWave);
        }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kOrderSlots; ++j) {
        const int ch = wave + j * kWaves;
        if (ch < nchunks) {
            unsigned long long mine = 0;
            for (int c = 0; c < ncls; ++c) {
                const unsigned long long m = __ballot(cls[j] == c);
                if (cls[j] == c) mine = m;
            }
            if (cls[j] >= 0) {
                const int rank = counts[(ncls - 1 - cls[j]) * nchunks + ch] + __popcll(mine & ((1ull << lane) - 1ull));
                int4* rec = reinterpret_cast<int4*>(order + (size_t)rank * kOrderRec);
                rec[0] = make_int4(ch * kWave + lane, first[j], count[j], e0[j]);
                rec[1] = make_int4(e1[j], 0, 0, 0);
            }
        }
    }
}

// Batches of more graphs than compute units can also be packed: a run of consecutive graphs of at most `cap`
// nodes together is a block-diagonal graph like any other, so one workgroup carries it through the input stage
// and the levels at the cost of one graph (the kernel's time is per workgroup: start-up, staging, a barrier
// per stage, and matrix tiles that a 30-node graph leaves three quarters empty), and only the readout runs per
// graph (a wavefront each).  1,024 graphs of the 10..110-node distribution: 59 -> 45 us.
// The kernel below cuts the batch into such runs ("bins").  Every 64 consecutive graphs are packed on their
// own by one wavefront (first fit in batch order; a bin never crosses such a boundary, which costs about one
// partly filled bin per 64 graphs), so all of it is a few ballots per bin.  A graph of more than cap nodes is a
// bin of its own (the forward kernel refuses it).  Output: bins[0] = number of bins, then one record of
// kOrderRec ints per bin from bins + kOrderRec on: first graph, first node, nodes, first entry, end of entries,
// graphs.
constexpr int kPackNodes = 128;                  // eight tiles: with four column blocks, two tasks for each of 16 wavefronts
constexpr int kPackMaxNodes = 208;
constexpr int kPackMinGraphs = 2 * kNumCU;       // below this the graphs taken one by one, largest first, are as fast
constexpr int kBinBlock = 1024;
constexpr int kBinMaxGraphs = 1 << 19;           // segment counts live in LDS (32 KB)
__global__ __launch_bounds__(kBinBlock) void graph_bins_kernel(int B, int cap, const int* __restrict__ a_row_ptr,
                                                               const int* __restrict__ s_row_ptr, int* __restrict__ bins)
{
    constexpr int kWaves = kBinBlock / kWave;
    __shared__ int seg_bins[kBinMaxGraphs / kWave + 1];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int nseg = (B + kWave - 1) / kWave;
    // packs segment `seg` (start / end: first node and end of the lane's graph); with `base` >= 0 the records
    // are written from bin index `base` on.  Returns the bin count.
    auto pack = [&](int seg, int start, int end, int base) {
        const bool live = seg * kWave + lane < B;
        const int nlive = min(kWave, B - seg * kWave);
        int first = 0, count = 0;
        while (first < nlive) {
            const int node0 = __builtin_amdgcn_readlane(start, first);
            // lanes from `first` on whose graph still fits behind node0; the bin ends before the first that does not
            const unsigned long long stop = __ballot(lane >= first && (!live || end - node0 > cap));
            int next = stop ? (int)__builtin_ctzll(stop) : kWave;
            if (next == first) next = first + 1;                     // larger than cap: alone
            next = __builtin_amdgcn_readfirstlane(next);
            if (base >= 0 && lane < 2)                               // first graph and graph count; the rest follows below
                bins[(size_t)(1 + base + count) * kOrderRec + (lane ? 5 : 0)] = lane ? next - first : seg * kWave + first;
            ++count;
            first = next;
        }
        return count;
    };
    // the node ranges of this wavefront's first kBinKeep segments stay in registers between the two passes
    constexpr int kBinKeep = 4;
    int st[kBinKeep], en[kBinKeep];
#pragma unroll
    for (int j = 0; j < kBinKeep; ++j) {
        const int g = (wave + j * kWaves) * kWave + lane;
        st[j] = en[j] = 0;
        if (g < B) { st[j] = s_row_ptr[g]; en[j] = s_row_ptr[g + 1]; }
    }
    auto ranges = [&](int seg, int j, int& start, int& end) {
        if (j < kBinKeep) {
#pragma unroll
            for (int u = 0; u < kBinKeep; ++u) if (u == j) { start = st[u]; end = en[u]; }
        } else {
            const int g = seg * kWave + lane;
            start = end = 0;
            if (g < B) { start = s_row_ptr[g]; end = s_row_ptr[g + 1]; }
        }
    };
    for (int seg = wave, j = 0; seg < nseg; seg += kWaves, ++j) {
        int start, end;
        ranges(seg, j, start, end);
        const int c = pack(seg, start, end, -1);
        if (lane == 0) seg_bins[seg] = c;
    }
    __syncthreads();
    if (wave == 0) {                                                 // exclusive scan of the segment counts
        int carry = 0;
        for (int b0 = 0; b0 < nseg; b0 += kWave) {
            const int i = b0 + lane;
            const int v = i < nseg ? seg_bins[i] : 0;
            int incl = v;
#pragma unroll
            for (int d = 1; d < kWave; d <<= 1) {
                const int o = __shfl_up(incl, d, kWave);
                if (lane >= d) incl += o;
            }
            if (i < nseg) seg_bins[i] = carry + incl - v;
            carry += __shfl(incl, kWave - 1, kWave);
        }
        if (lane == 0) bins[0] = carry;
    }
    __syncthreads();
    for (int seg = wave, j = 0; seg < nseg; seg += kWaves, ++j) {
        int start, end;
        ranges(seg, j, start, end);
        pack(seg, start, end, seg_bins[seg]);
    }
    __threadfence_block();
    __syncthreads();
    // node and entry ranges, one lane per bin (a bin the forward kernel will refuse gets no entry range)
    const int nbins = bins[0];
    for (int b = threadIdx.x; b < nbins; b += kBinBlock) {
        int* rec = bins + (size_t)(1 + b) * kOrderRec;
        const int g0 = rec[0], ng = rec[5];
        const int node0 = s_row_ptr[g0], n = s_row_ptr[g0 + ng] - node0;
        int e0 = 0, e1 = 0;
        if (n >= 0 && n <= cap) { e0 = a_row_ptr[node0]; e1 = a_row_ptr[node0 + n]; }
        rec[1] = node0;
        rec[2] = n;
        rec[3] = e0;
        rec[4] = e1;
    }
}

// WAVES wavefronts per workgroup (4, 8 or 16): chosen by the host so that the largest graph's
// (column block x row tile) tasks spread over the wavefronts.
// order: null (graphs in batch order), or the records graph_order_kernel left.
// KEEP: the embeddings of all levels are also stored for a backward pass, h_l at h_levels + l * level_stride
// (a variant of its own: the extra stores cost the inference kernel 2 % when they are a run-time choice).
// PACK: `order` holds the bins graph_bins_kernel made (order[0] bins, records from order + kOrderRec on); a workgroup
// carries a bin through the input stage and the levels as one block-diagonal graph, and its wavefronts run the
// readout of the bin's graphs, one graph each (H <= 64 and Q <= 64: a lane per hidden unit and per class).
template <int C, int KSX, int WAVES, bool KEEP = false, bool PACK = false>
__global__ __launch_bounds__(WAVES * kWave) void s2v_graph_forward_kernel(
    int B, int K, unsigned k_magic, int H, int Q, int L, int n16max, int ecap,
    const int* __restrict__ a_row_ptr, const int* __restrict__ a_col_idx, const float* __restrict__ a_val,
    const int* __restrict__ s_row_ptr, const int* __restrict__ s_col_idx, const float* __restrict__ s_val,
    const float* __restrict__ X, const float* __restrict__ Wn2l, const float* __restrict__ Wc,
    const float* __restrict__ Wh1, const float* __restrict__ Wh2,
    float* __restrict__ msg, float* __restrict__ h_final, float* __restrict__ pool, float* __restrict__ hidden,
    float* __restrict__ logits, float* __restrict__ probs, int* __restrict__ pred, int* __restrict__ status,
    const int* __restrict__ order, float* __restrict__ h_levels, long long level_stride)
{
    // KSX == 0: the node features arrive as one label per node (X points at int labels[N]) and the input
    // stage is a row lookup in W_n2l; otherwise X is the dense [N,K] matrix and KSX bounds its contraction steps
    constexpr bool LABELS = (KSX == 0);
    constexpr int KSXA = LABELS ? 2 : KSX;
    constexpr int kBlock = WAVES * kWave;
    constexpr int kWavesPerBlock = WAVES;
    constexpr int G = C / 4;             // lanes per row in gathers
    constexpr int P = kBlock / G;        // rows per gather round
    constexpr int KS = C / 4;            // contraction steps of a level
    constexpr int NJB = C / 16;          // column blocks
    constexpr int TS = kWavesPerBlock / NJB;   // wavefronts sharing one column block, splitting tiles
    constexpr int LDT = C + 4;
    constexpr int kMsgTiles = (WAVES >= 16) ? 2 : 4;
    constexpr int kXSlots = (WAVES >= 16) ? 8 : 4;     // elements of the graph's X block a lane stages in one go   // msg tiles a wavefront keeps in registers across the levels

    extern __shared__ float smem[];
    const bool ro_staged = ((size_t)C * H + (size_t)H * Q <= (size_t)kReadoutCap);
    const size_t agg_fl = GraphLds::agg_floats(n16max, C, K, kBlock, LABELS);
    float* hbuf = smem;                                  // [n16max + 1][LDT]; row n16max is never written after start-up and holds zeros
    float* agg = hbuf + (size_t)(n16max + 1) * LDT;      // [n16max][LDT]; doubles as part[P][C] in the readout
    float* part = agg;
    int* l_rp = reinterpret_cast<int*>(agg + agg_fl);    // [n16max + 1] row pointers relative to the graph's first entry
    float* l_sv = reinterpret_cast<float*>(l_rp + n16max + 4);  // [n16max] pooling weights of the graph's rows
    float* hid = l_sv + n16max;                          // [H]
    float* lg = hid + H;                                 // [Q]
    float* w1s = lg + Q;                                 // W_h1 transposed, [H][C], when staged
    float* w2s = w1s + (size_t)C * H;                    // W_h2 transposed, [Q][H], when staged
    float* tail = ro_staged ? (w2s + (size_t)H * Q) : w1s;
    tail = smem + ((size_t)(tail - smem) + 3) / 4 * 4;
    int* e_col = reinterpret_cast<int*>(tail);           // [ecap] neighbour index local to the graph
    float* e_val = tail + ecap;                          // [ecap]
    int* l_lab = reinterpret_cast<int*>(e_val + ecap);   // label input only: [n16max] labels of the graph's nodes
    float* wn_s = reinterpret_cast<float*>(l_lab + n16max);     // label input only: W_n2l [K][C] when staged
    const bool wn_in_lds = LABELS && GraphLds::wn_staged(C, K);
    const int* labels = reinterpret_cast<const int*>(X);

    // the lane's coordinates, used by the start-up code; the graph loop derives its own copies (see there)
    const int tid0 = threadIdx.x;

    GNNHIP_PHASE_MARK(0);
    // The position of the first graph (node range, then entry range) is asked for ahead of the weight
    // loads, so the two dependent trips to memory run under them instead of after them.
    int next_g = blockIdx.x, next_node0 = 0, next_n = 0, next_e0 = 0, next_e1 = 0, next_ng = 1;
    // PACK: the slots are the bins (their number is the first word of `order`, the records follow its first kOrderRec words)
    const int* recs = PACK ? order + kOrderRec : order;
    const int nslots = PACK ? order[0] : B;
    if ((int)blockIdx.x < nslots) {
        if (order) {
            const int4 r0 = *reinterpret_cast<const int4*>(recs + (size_t)blockIdx.x * kOrderRec);
            next_g = r0.x; next_node0 = r0.y; next_n = r0.z; next_e0 = r0.w;
            const int2 r1 = *reinterpret_cast<const int2*>(recs + (size_t)blockIdx.x * kOrderRec + 4);
            next_e1 = r1.x;
            next_ng = r1.y;
        } else {
            next_node0 = s_row_ptr[blockIdx.x];
            next_n = s_row_ptr[blockIdx.x + 1] - next_node0;
        }
    }
    // this wavefront's 16 columns of W^T, level contraction: wreg[s] = Wc[KS q + s][16 jb + t]
    float wreg[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s)
        wreg[s] = Wc[(size_t)(KS * ((tid0 & (kWave - 1)) >> 4) + s) * C + 16 * ((tid0 / kWave) % NJB) + (tid0 & 15)];
    if (!order && (int)blockIdx.x < nslots && next_n >= 0 && next_n <= n16max) {
        next_e0 = a_row_ptr[next_node0];
        next_e1 = a_row_ptr[next_node0 + next_n];
    }

    if (tid0 < LDT) hbuf[(size_t)n16max * LDT + tid0] = 0.f;
    if (PACK && ro_staged) {
        // a lane per output in the readout: the layouts of memory, W_h1 [C][H] and W_h2 [H][Q]
        for (int i = tid0; i < C * H; i += kBlock) w1s[i] = Wh1[i];
        for (int i = tid0; i < H * Q; i += kBlock) w2s[i] = Wh2[i];
    } else if (ro_staged) {
        // coalesced reads; the transposed layout lets a wavefront read one output's weights contiguously
        // (four elements of W_h1 and one of W_h2 per lane are asked for together: one trip to memory for the
        // usual sizes instead of one per element)
        const int n1 = C * H, n2 = H * Q;
        float v1[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) { const int i = tid0 + u * kBlock; v1[u] = i < n1 ? Wh1[i] : 0.f; }
        const float v2 = tid0 < n2 ? Wh2[tid0] : 0.f;
#pragma unroll
        for (int u = 0; u < 4; ++u) { const int i = tid0 + u * kBlock; if (i < n1) w1s[(i % H) * C + i / H] = v1[u]; }
        if (tid0 < n2) w2s[(tid0 % Q) * H + tid0 / Q] = v2;
        for (int i = tid0 + 4 * kBlock; i < n1; i += kBlock) w1s[(i % H) * C + i / H] = Wh1[i];
        for (int i = tid0 + kBlock; i < n2; i += kBlock) w2s[(i % Q) * H + i / Q] = Wh2[i];
    }
    if (LABELS && wn_in_lds)
        for (int i = tid0; i < K * C; i += kBlock) wn_s[i] = Wn2l[i];
    // (the staged copies become visible to all lanes at the first barrier of the graph loop)
    GNNHIP_PHASE_MARK(1);
    const rsrc_t wn_rsrc = make_rsrc(Wn2l, (unsigned)((size_t)K * C * 4));
    // input stage: srt contraction steps (srt <= KSX), lane group q covers label columns [srt q, srt q + srt);
    // the staged rows of X have stride KP floats and zeros from column K on
    const int srt = GraphLds::input_steps(K);
    const int KP = 4 * srt;
    for (int slot = blockIdx.x; slot < nslots; slot += gridDim.x) {
        // The lane's coordinates are derived again for every graph from a value the compiler cannot see
        // through.  Otherwise every per-lane address of the loop body (a dozen 64-bit pointers) is computed
        // once ahead of the loop, does not fit the 128 registers of a 16-wavefront workgroup, and comes back
        // from scratch memory in the middle of the latency chains below.
        int tid = tid0;
        asm volatile("" : "+v"(tid));
        const int lane = tid & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(tid / kWave);
        const int q = lane >> 4, t = lane & 15;
        const int jb = wave % NJB, tsplit = wave / NJB;
        const int gi = tid / G, tx = tid % G;
        const int wx_lane_off = ((srt * q) * C + 16 * jb + t) * 4;
        const bool first = (slot == (int)blockIdx.x);   // the position of this graph was asked for at start-up
        int g = slot, node0, n, rec_e0 = 0, rec_e1 = 0, ng = 1;
        if (first) {
            g = next_g; node0 = next_node0; n = next_n; ng = next_ng;
        } else if (order) {
            const int4 r0 = *reinterpret_cast<const int4*>(recs + (size_t)slot * kOrderRec);
            g = r0.x; node0 = r0.y; n = r0.z; rec_e0 = r0.w;
            const int2 r1 = *reinterpret_cast<const int2*>(recs + (size_t)slot * kOrderRec + 4);
            rec_e1 = r1.x;
            ng = r1.y;
        } else {
            node0 = s_row_ptr[g];
            n = s_row_ptr[g + 1] - node0;
        }
        if (n > n16max || n < 0) {                      // host promised max_graph_nodes; refuse instead of overrunning LDS
            if (tid == 0 && status) atomicOr(status, 1);
            continue;
        }
        const int ntile = (n + 15) >> 4;
        // this wavefront's 16 columns of W_n2l^T for the input stage: k = srt q + s, zero beyond K (rows past the
        // end of the buffer read as zero; steps s >= srt are loaded but not used).  Loaded per graph (from L2) so the registers are free during the
        // levels; one lane offset plus constant strides, so no per-element address lives across the graph loop.
        float wx[KSXA];
        if (!LABELS) {
#pragma unroll
            for (int s = 0; s < KSXA; ++s) wx[s] = buf_load_f(wn_rsrc, wx_lane_off + s * (C * 4), 0);
        }

        // ---- stage the graph's CSR slice (L uses), its pooling weights and its rows of X (contiguous in memory;
        //      parked in the still unused agg buffer), and check the block-diagonal promise.  Everything a lane
        //      needs is asked for before anything is used, so the staging costs one trip to memory.
        float* xs = agg;
        const int e0 = first ? next_e0 : order ? rec_e0 : a_row_ptr[node0];
        const int ne = (first ? next_e1 : order ? rec_e1 : a_row_ptr[node0 + n]) - e0;
        const bool staged = (ne <= ecap);
        {
            const float* xg = X + (size_t)node0 * K;
            const int nx = n * K;
            // element i of the graph's block of X (row i / K, column i % K) -> its padded slot; the quotient
            // comes from one multiply-high by ceil(2^32 / K), exact for i K < 2^32
            auto x_slot = [&](int i) {
                const int r = K >= 2 ? (int)__umulhi((unsigned)i, k_magic) : i;
                return r * KP + (i - r * K);
            };
            int rp_v = 0, sc_v = 0, c_v = 0, lab_v = 0;
            float sv_v = 0.f, v_v = 0.f, xv[kXSlots];
#pragma unroll
            for (int u = 0; u < kXSlots; ++u) xv[u] = 0.f;
            if (tid <= n) rp_v = a_row_ptr[node0 + tid];
            if (tid < n) { sc_v = s_col_idx[node0 + tid]; sv_v = s_val[node0 + tid]; }
            if (LABELS) {
                if (tid < n) lab_v = labels[node0 + tid];
            } else {
#pragma unroll
                for (int u = 0; u < kXSlots; ++u) if (tid + u * kBlock < nx) xv[u] = xg[tid + u * kBlock];
            }
            // (the graph's first entry is the last thing to arrive at start-up: everything above is under way by then)
            if (staged && tid < ne) { c_v = a_col_idx[e0 + tid]; v_v = a_val[e0 + tid]; }

            if (tid <= n) l_rp[tid] = rp_v - e0;
            if (tid < n) {
                l_sv[tid] = sv_v;
                if (sc_v != node0 + tid) { if (status) atomicOr(status, 4); }
            }
            if (staged && tid < ne) {
                const int c = c_v - node0;
                if (c < 0 || c >= n) { if (status) atomicOr(status, 2); }
                e_col[tid] = min(max(c, 0), n - 1);
                e_val[tid] = v_v;
            }
            if (LABELS) {
                // a label outside [0, K) is reported (bit 3) and clamped, so no read leaves W_n2l
                for (int i = tid; i < n; i += kBlock) {
                    const int lab = (i == tid) ? lab_v : labels[node0 + i];
                    if (lab < 0 || lab >= K) { if (status) atomicOr(status, 8); }
                    l_lab[i] = min(max(lab, 0), K - 1);
                }
            } else {
#pragma unroll
                for (int u = 0; u < kXSlots; ++u) {
                    const int i = tid + u * kBlock;
                    if (i < nx) xs[x_slot(i)] = xv[u];
                }
                // columns K .. KP-1 of the staged rows (at most 7) are zero
                for (int r = tid; r < n; r += kBlock)
                    for (int k = K; k < KP; ++k) xs[r * KP + k] = 0.f;
            }
            // what exceeds one element per lane (kXSlots of X)
            for (int i = tid + kBlock; i <= n; i += kBlock) l_rp[i] = a_row_ptr[node0 + i] - e0;
            for (int i = tid + kBlock; i < n; i += kBlock) {
                l_sv[i] = s_val[node0 + i];
                if (s_col_idx[node0 + i] != node0 + i) { if (status) atomicOr(status, 4); }
            }
            if (staged) {
                for (int i = tid + kBlock; i < ne; i += kBlock) {
                    const int c = a_col_idx[e0 + i] - node0;
                    if (c < 0 || c >= n) { if (status) atomicOr(status, 2); }
                    e_col[i] = min(max(c, 0), n - 1);
                    e_val[i] = a_val[e0 + i];
                }
            }
            if (!LABELS)
                for (int i = tid + kXSlots * kBlock; i < nx; i += kBlock) xs[x_slot(i)] = xg[i];
        }
        __syncthreads();

        GNNHIP_PHASE_MARK(2);
        // ---- input stage: msg tile = X tile * W_n2l on the matrix cores
        float4 mreg[kMsgTiles];            // this wavefront's msg values for its first kMsgTiles tiles, kept for all levels
#pragma unroll
        for (int i = 0; i < kMsgTiles; ++i) mreg[i] = f4_zero();
        {
            int ti = 0;
            for (int tl = tsplit; tl < ntile; tl += TS, ++ti) {
                const int lr = tl * 16 + t;
                const bool valid = lr < n;
                // every lane reads a valid LDS slot (row clamped; rows beyond n are zeroed below); the
                // lane's srt values are contiguous and 8-byte aligned
                float4 v;                                                     // row lr, columns 16 jb + 4 q + {0..3}
                if (LABELS) {
                    // the product of a one-hot row with W_n2l is that row of W_n2l (0 + w, so -0.0 becomes +0.0
                    // as in the sum the dense product forms)
                    const int lab = l_lab[min(lr, n - 1)];
                    const float* wrow = (wn_in_lds ? wn_s : Wn2l) + (size_t)lab * C + 16 * jb + 4 * q;
                    const float4 wv = *reinterpret_cast<const float4*>(wrow);
                    v = make_float4(0.f + wv.x, 0.f + wv.y, 0.f + wv.z, 0.f + wv.w);
                } else {
                    const float* xrow = xs + min(lr, n - 1) * KP + srt * q;
                    float xreg[KSXA];
#pragma unroll
                    for (int s2 = 0; s2 < KSXA / 2; ++s2) {
                        float2 v2 = make_float2(0.f, 0.f);
                        if (2 * s2 < srt) v2 = *reinterpret_cast<const float2*>(xrow + 2 * s2);
                        xreg[2 * s2] = v2.x; xreg[2 * s2 + 1] = v2.y;
                    }
                    mfma_f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < KSXA; ++s)
                        if (s < srt) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wx[s], xreg[s], acc, 0, 0, 0);
                    v = make_float4(acc[0], acc[1], acc[2], acc[3]);
                }
                if (!valid) v = f4_zero();
                if (valid) *reinterpret_cast<float4*>(msg + (size_t)(node0 + lr) * C + 16 * jb + 4 * q) = v;
                *reinterpret_cast<float4*>(hbuf + (size_t)lr * LDT + 16 * jb + 4 * q) = relu_ref4(v);
                if constexpr (KEEP) {
                    if (valid) *reinterpret_cast<float4*>(h_levels + (size_t)(node0 + lr) * C + 16 * jb + 4 * q) = relu_ref4(v);
                }
#pragma unroll
                for (int i = 0; i < kMsgTiles; ++i) if (i == ti) mreg[i] = v;
            }
        }
        __syncthreads();
        GNNHIP_PHASE_MARK(3);

        // The first kGatherEntries neighbours of this lane's row in each of the first kGatherRounds rounds of the
        // gather (LDS offset and weight) stay in registers for all levels: a level's gather is then one round
        // of independent LDS reads instead of the chain row pointer -> column -> row.
        constexpr int kGatherRounds = (WAVES >= 16) ? 2 : 4, kGatherEntries = 4;
        int g_off[kGatherRounds][kGatherEntries], g_st[kGatherRounds], g_en[kGatherRounds];
        float g_w[kGatherRounds][kGatherEntries];
#pragma unroll
        for (int r = 0; r < kGatherRounds; ++r) {
            const int lr = r * P + gi;
            g_st[r] = g_en[r] = 0;
            if (staged && lr < n) { g_st[r] = l_rp[lr]; g_en[r] = l_rp[lr + 1]; }
#pragma unroll
            for (int u = 0; u < kGatherEntries; ++u) {
                const bool ok = g_st[r] + u < g_en[r];       // a missing entry is weight 0 times the zero row
                g_off[r][u] = (ok ? e_col[g_st[r] + u] : n16max) * LDT + tx * 4;
                g_w[r][u] = ok ? e_val[g_st[r] + u] : 0.f;
            }
        }

        for (int lv = 0; lv < L; ++lv) {
            // ---- gather-sum from LDS: agg[i] = sum_e val_e * h[col_e], entries in order
            if (staged) {
#pragma unroll
                for (int r = 0; r < kGatherRounds; ++r) {
                    if (r * P < ntile * 16) {
                        const int lr = r * P + gi;
                        float4 x[kGatherEntries];
#pragma unroll
                        for (int u = 0; u < kGatherEntries; ++u) x[u] = *reinterpret_cast<const float4*>(hbuf + g_off[r][u]);
                        float4 acc = f4_zero();
#pragma unroll
                        for (int u = 0; u < kGatherEntries; ++u) f4_fma(acc, g_w[r][u], x[u]);
                        for (int e = g_st[r] + kGatherEntries; e < g_en[r]; ++e)
                            f4_fma(acc, e_val[e], *reinterpret_cast<const float4*>(hbuf + (size_t)e_col[e] * LDT + tx * 4));
                        if (lr < ntile * 16) *reinterpret_cast<float4*>(agg + (size_t)lr * LDT + tx * 4) = acc;
                    }
                }
            }
            for (int r0 = staged ? kGatherRounds * P : 0; r0 < ntile * 16; r0 += P) {
                const int lr = r0 + gi;
                float4 acc = f4_zero();
                if (lr < n) {
                    const int st = l_rp[lr], en = l_rp[lr + 1];
                    if (staged) {
                        for (int e = st; e < en; ++e)
                            f4_fma(acc, e_val[e], *reinterpret_cast<const float4*>(hbuf + (size_t)e_col[e] * LDT + tx * 4));
                    } else {
                        for (int e = st; e < en; ++e) {
                            int c = a_col_idx[e0 + e] - node0;
                            if (c < 0 || c >= n) { if (status) atomicOr(status, 2); c = min(max(c, 0), n - 1); }
                            f4_fma(acc, a_val[e0 + e], *reinterpret_cast<const float4*>(hbuf + (size_t)c * LDT + tx * 4));
                        }
                    }
                }
                if (lr < ntile * 16) *reinterpret_cast<float4*>(agg + (size_t)lr * LDT + tx * 4) = acc;
            }
            __syncthreads();
            if (lv == 0) { GNNHIP_PHASE_MARK(4); }

            // ---- contraction + epilogue; h is rewritten in place (the gather above was its last reader)
            int ti = 0;
            for (int tl = tsplit; tl < ntile; tl += TS, ++ti) {
                const int lr = tl * 16 + t;
                const bool valid = lr < n;
                float4 mm = f4_zero();
                if (ti < kMsgTiles) {
#pragma unroll
                    for (int i = 0; i < kMsgTiles; ++i) if (i == ti) mm = mreg[i];
                } else if (valid) {
                    mm = *reinterpret_cast<const float4*>(msg + (size_t)(node0 + lr) * C + 16 * jb + 4 * q);
                }
                float areg[KS];
#pragma unroll
                for (int s4 = 0; s4 < KS / 4; ++s4) {
                    const float4 a = *reinterpret_cast<const float4*>(agg + (size_t)lr * LDT + KS * q + 4 * s4);
                    areg[4 * s4 + 0] = a.x; areg[4 * s4 + 1] = a.y; areg[4 * s4 + 2] = a.z; areg[4 * s4 + 3] = a.w;
                }
                mfma_f4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < KS; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[s], areg[s], acc, 0, 0, 0);
                float4 v = make_float4(acc[0] + mm.x, acc[1] + mm.y, acc[2] + mm.z, acc[3] + mm.w);
                v = relu_ref4(v);
                *reinterpret_cast<float4*>(hbuf + (size_t)lr * LDT + 16 * jb + 4 * q) = v;
                if (lv == L - 1 && valid)
                    *reinterpret_cast<float4*>(h_final + (size_t)(node0 + lr) * C + 16 * jb + 4 * q) = v;
                if constexpr (KEEP) {
                    if (valid)
                        *reinterpret_cast<float4*>(h_levels + (size_t)(lv + 1) * level_stride + (size_t)(node0 + lr) * C + 16 * jb + 4 * q) = v;
                }
            }
            __syncthreads();
            if (lv == 0) { GNNHIP_PHASE_MARK(5); }
        }
        GNNHIP_PHASE_MARK(6);
        if (L == 0) {
            // the embedding is h0
            for (int i = tid; i < n * G; i += kBlock) {
                const int lr = i / G, f = i % G;
                *reinterpret_cast<float4*>(h_final + (size_t)(node0 + lr) * C + f * 4) =
                    *reinterpret_cast<const float4*>(hbuf + (size_t)lr * LDT + f * 4);
            }
        }

        if constexpr (PACK) {
            // ---- readout of a bin: graph k of the bin is rows [l_gs[k], l_gs[k + 1]) and belongs to one wavefront,
            // which pools it (lane c walks column c, rows in order), forms the hidden units (lane j adds
            // pool[c] * W_h1[c][j] over c, the pooled values handed round by v_readlane), the logits (lane q)
            // and softmax / arg-max, without a barrier
            int* l_gs = reinterpret_cast<int*>(agg);         // [ng + 1]; the buffer is free after the last level
            if (tid <= ng) l_gs[tid] = s_row_ptr[g + tid] - node0;
            __syncthreads();
            for (int k = wave; k < ng; k += kWavesPerBlock) {
                const int r0 = l_gs[k], r1 = l_gs[k + 1];
                const int gk = g + k;
                float p = 0.f;
                if (lane < C)
                    for (int lr = r0; lr < r1; ++lr) p = fmaf(l_sv[lr], hbuf[(size_t)lr * LDT + lane], p);
                if (lane < C) pool[(size_t)gk * C + lane] = p;
                const float* w1 = ro_staged ? w1s : Wh1;      // [C][H] either way
                const float* w2 = ro_staged ? w2s : Wh2;      // [H][Q]
                float hv = 0.f;
#pragma unroll 8
                for (int c = 0; c < C; ++c) {
                    const float pc = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), c));
                    if (lane < H) hv = fmaf(pc, w1[(size_t)c * H + lane], hv);
                }
                hv = relu_ref(hv);
                if (lane < H) hidden[(size_t)gk * H + lane] = hv;
                float sq = 0.f;
                for (int j = 0; j < H; ++j) {
                    const float hj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(hv), j));
                    if (lane < Q) sq = fmaf(hj, w2[(size_t)j * Q + lane], sq);
                }
                if (lane < Q) logits[(size_t)gk * Q + lane] = sq;
                if (probs || pred) {
                    const float first = row_value_f(sq, 0);
                    float mx = (lane < Q) ? max_keep(first, sq) : first;     // the reference scan starts at element 0
                    mx = wave_max(mx);
                    float bv = -INFINITY;
                    int bi = 0x7fffffff;
                    if (lane < Q) { bv = (sq != sq) ? -INFINITY : sq; bi = lane; }   // a NaN that is not first never wins
                    wave_argmax(bv, bi);
                    if (first != first) bi = 0;                              // a NaN in column 0 is never displaced
                    if (pred && lane == 0) pred[gk] = bi;
                    if (probs) {
                        const float e = (lane < Q) ? expf(sq - mx) : 0.f;
                        const float sum = wave_sum(e);
                        if (lane < Q) probs[(size_t)gk * Q + lane] = e / sum;
                    }
                }
            }
            GNNHIP_PHASE_MARK(7);
            __syncthreads();          // LDS is reused by the next bin of this workgroup
            continue;
        }
        // ---- readout: weighted sum-pool over the graph's rows, then the two small dense layers.
        // Pooling: a lane owns one column (two at C = 128: lane and lane + 64) and walks rows, so from C = 64 on
        // nothing crosses lanes; one partial per wavefront goes to LDS.
        constexpr int CPL = (C + kWave - 1) / kWave;         // columns per lane
        {
            constexpr int GP = (C < kWave) ? C : kWave;      // lanes per row
            constexpr int RS = kWave / GP;                   // rows per wavefront per step
            const int pc = lane % GP, pr = lane / GP;
            float acc[CPL];
#pragma unroll
            for (int u = 0; u < CPL; ++u) acc[u] = 0.f;
            for (int lr = wave * RS + pr; lr < n; lr += kWavesPerBlock * RS)
#pragma unroll
                for (int u = 0; u < CPL; ++u) acc[u] = fmaf(l_sv[lr], hbuf[(size_t)lr * LDT + pc + u * kWave], acc[u]);
            if constexpr (CPL == 1) {
#pragma unroll
                for (int off = GP; off < kWave; off <<= 1) acc[0] += __shfl_xor(acc[0], off, kWave);
            }
            if (lane < GP) {
#pragma unroll
                for (int u = 0; u < CPL; ++u) part[(size_t)wave * C + pc + u * kWave] = acc[u];
            }
        }
        __syncthreads();
        GNNHIP_PHASE_MARK(12);
        // every wavefront adds up its own copy of the pooled row (lane c holds column c, and c + 64 at C = 128)
        float plv[CPL];
#pragma unroll
        for (int u = 0; u < CPL; ++u) {
            plv[u] = 0.f;
            if (lane + u * kWave < C) {
#pragma unroll
                for (int p = 0; p < kWavesPerBlock; ++p) plv[u] += part[(size_t)p * C + lane + u * kWave];
            }
            if (wave == 0 && lane + u * kWave < C) pool[(size_t)g * C + lane + u * kWave] = plv[u];
        }
        GNNHIP_PHASE_MARK(13);
        // hidden layer: one wavefront per output, two outputs per step so that their reductions overlap
        for (int j = wave; j < H; j += 2 * kWavesPerBlock) {
            const int j1 = j + kWavesPerBlock;
            const bool two = j1 < H;
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int u = 0; u < CPL; ++u) {
                const int c = lane + u * kWave;
                if (c < C) {
                    if (ro_staged) {
                        s0 = fmaf(plv[u], w1s[j * C + c], s0);
                        if (two) s1 = fmaf(plv[u], w1s[j1 * C + c], s1);
                    } else {
                        s0 = fmaf(plv[u], Wh1[(size_t)c * H + j], s0);
                        if (two) s1 = fmaf(plv[u], Wh1[(size_t)c * H + j1], s1);
                    }
                }
            }
            s0 = relu_ref(wave_sum(s0));
            s1 = relu_ref(wave_sum(s1));
            if (lane == 0) {
                hid[j] = s0; hidden[(size_t)g * H + j] = s0;
                if (two) { hid[j1] = s1; hidden[(size_t)g * H + j1] = s1; }
            }
        }
        __syncthreads();
        GNNHIP_PHASE_MARK(14);
        if (Q <= 16) {
            // few classes: lane q of the first wavefront adds up logit q, and softmax and arg-max follow in
            // registers, with no further barrier or trip through LDS
            if (wave == 0) {
                float s = 0.f;
                if (lane < Q) {
                    if (ro_staged) {
#pragma unroll 8
                        for (int j = 0; j < H; ++j) s = fmaf(hid[j], w2s[lane * H + j], s);
                    } else {
#pragma unroll 8
                        for (int j = 0; j < H; ++j) s = fmaf(hid[j], Wh2[(size_t)j * Q + lane], s);
                    }
                    logits[(size_t)g * Q + lane] = s;
                }
                if (probs || pred) {
                    const float first = row_value_f(s, 0);
                    float mx = (lane < Q) ? max_keep(first, s) : first;     // the reference scan starts at element 0
                    mx = wave_max(mx);
                    float bv = -INFINITY;
                    int bi = 0x7fffffff;
                    if (lane < Q) { bv = (s != s) ? -INFINITY : s; bi = lane; }   // a NaN that is not first never wins
                    wave_argmax(bv, bi);
                    if (first != first) bi = 0;                             // a NaN in column 0 is never displaced
                    if (pred && lane == 0) pred[g] = bi;
                    if (probs) {
                        const float e = (lane < Q) ? expf(s - mx) : 0.f;
                        const float sum = wave_sum(e);
                        if (lane < Q) probs[(size_t)g * Q + lane] = e / sum;
                    }
                }
            }
        } else {
            for (int qq = wave; qq < Q; qq += kWavesPerBlock) {
                float s = 0.f;
                if (ro_staged) {
                    for (int j = lane; j < H; j += kWave) s += hid[j] * w2s[qq * H + j];
                } else {
                    for (int j = lane; j < H; j += kWave) s += hid[j] * Wh2[(size_t)j * Q + qq];
                }
                s = wave_sum(s);
                if (lane == 0) { lg[qq] = s; logits[(size_t)g * Q + qq] = s; }
            }
            __syncthreads();
            if (wave == 0) {
                const float first = lg[0];
                float mx = first;
                float bv = -INFINITY;
                int bi = 0x7fffffff;
                for (int qq = lane; qq < Q; qq += kWave) {
                    const float v = lg[qq];
                    mx = max_keep(mx, v);
                    argmax_combine(bv, bi, (v != v) ? -INFINITY : v, qq);
                }
                mx = wave_max(mx);
                wave_argmax(bv, bi);
                if (first != first) bi = 0;
                if (pred && lane == 0) pred[g] = bi;
                if (probs) {
                    float s = 0.f;
                    for (int qq = lane; qq < Q; qq += kWave) {
                        const float e = expf(lg[qq] - mx);
                        lg[qq] = e;
                        s += e;
                    }
                    s = wave_sum(s);
                    for (int qq = lane; qq < Q; qq += kWave) probs[(size_t)g * Q + qq] = lg[qq] / s;
                }
            }
        }
        GNNHIP_PHASE_MARK(7);
        __syncthreads();          // LDS is reused by the next graph of this workgroup
    }
}

template <int C, int KSX, int WAVES>
int launch_graph_forward(int B, int K, int H, int Q, int L, int n16max,
                         const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                         const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                         const float* X, const float* Wn2l, const float* Wc, const float* Wh1, const float* Wh2,
                         float* msg, float* h_final, float* pool, float* hidden, float* logits, float* probs,
                         int* pred, int* status, float* h_levels, long long level_stride, bool pack, hipStream_t s)
{
    constexpr int kBlock = WAVES * kWave;
    constexpr bool LABELS = (KSX == 0);
    const int ecap = GraphLds::edge_cap(n16max, C, K, H, Q, kBlock, LABELS);
    if (ecap < 0) return GNNHIP_EUNSUPPORTED;
    const size_t smem = sizeof(float) * (GraphLds::fixed_floats(n16max, C, K, H, Q, kBlock, LABELS) + 2 * (size_t)ecap);
    constexpr bool kKeepBuilt = !LABELS;    // the variant that keeps all levels exists for the dense input only
    // the variant that packs graphs into bins exists for the workgroup shapes bins of 128 nodes and more select
    constexpr bool kPackBuilt = C <= 64 && ((WAVES == 16) || (C == 16 && WAVES == 8));
    const bool keep = h_levels != nullptr;
    if (keep && !kKeepBuilt) return GNNHIP_EUNSUPPORTED;
    if (pack && (!kPackBuilt || keep)) return GNNHIP_EUNSUPPORTED;
    static LdsLimit lds_limit, lds_limit_keep, lds_limit_pack;      // largest dynamic LDS size each kernel instantiation has been allowed so far
    const void* fn = keep ? reinterpret_cast<const void*>(&s2v_graph_forward_kernel<C, KSX, WAVES, kKeepBuilt, false>)
                   : pack ? reinterpret_cast<const void*>(&s2v_graph_forward_kernel<C, KSX, WAVES, false, kPackBuilt>)
                          : reinterpret_cast<const void*>(&s2v_graph_forward_kernel<C, KSX, WAVES, false, false>);
    if ((keep ? lds_limit_keep : pack ? lds_limit_pack : lds_limit).raise(fn, smem) != hipSuccess) {
        (void)hipGetLastError();
        return GNNHIP_EUNSUPPORTED;
    }
    int grid = B < kNumCU * 4 ? B : kNumCU * 4;
    int* order = nullptr;
    if (pack) {
        // bins: at most one per graph; two neighbouring bins hold more than n16max nodes together, and every 64
        // graphs may leave one bin short
        const long long N = level_stride / C;
        long long most = 2 * N / n16max + (B + kWave - 1) / kWave + 1;
        if (most > B) most = B;
        if (most < grid) grid = (int)most;
        void* p = nullptr;
        if (int rc = stream_scratch(s, sizeof(int) * kOrderRec * ((size_t)B + 1), &p)) return rc;
        order = static_cast<int*>(p);
        hipLaunchKernelGGL(graph_bins_kernel, dim3(1), dim3(kBinBlock), 0, s, B, n16max, a_row_ptr, s_row_ptr, order);
        GNNHIP_LAUNCH_CHECK("graph_bins");
    } else if (graphs_ordered(B) && n16max / 16 + 2 <= 64) {
        void* p = nullptr;
        if (int rc = stream_scratch(s, sizeof(int) * kOrderRec * (size_t)B, &p)) return rc;
        order = static_cast<int*>(p);
        hipLaunchKernelGGL(graph_order_kernel, dim3(1), dim3(kOrderBlock), 0, s, B, n16max, a_row_ptr, s_row_ptr, order);
        GNNHIP_LAUNCH_CHECK("graph_order");
    }
    const unsigned k_magic = K >= 2 ? (unsigned)((0x100000000ull + (unsigned)K - 1) / (unsigned)K) : 0u;   // ceil(2^32 / K)
#define GNNHIP_GF_LAUNCH(KEEPV, PACKV)                                                                                              \
    hipLaunchKernelGGL((s2v_graph_forward_kernel<C, KSX, WAVES, KEEPV, PACKV>), dim3(grid), dim3(kBlock), smem, s,                   \
                       B, K, k_magic, H, Q, L, n16max, ecap, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx, s_val,              \
                       X, Wn2l, Wc, Wh1, Wh2, msg, h_final, pool, hidden, logits, probs, pred, status, order, h_levels, level_stride)
    if (keep) GNNHIP_GF_LAUNCH(kKeepBuilt, false);
    else if (pack) GNNHIP_GF_LAUNCH(false, kPackBuilt);
    else GNNHIP_GF_LAUNCH(false, false);
#undef GNNHIP_GF_LAUNCH
    GNNHIP_LAUNCH_CHECK("s2v_graph_forward");
    return GNNHIP_OK;
}

template <int C, int WAVES>
int dispatch_ksx(bool labels, int B, int K, int H, int Q, int L, int n16max,
                 const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                 const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                 const float* X, const float* Wn2l, const float* Wc, const float* Wh1, const float* Wh2,
                 float* msg, float* h_final, float* pool, float* hidden, float* logits, float* probs,
                 int* pred, int* status, float* h_levels, long long level_stride, bool pack, hipStream_t s)
{
#define GNNHIP_GF_ARGS B, K, H, Q, L, n16max, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx, s_val, \
                       X, Wn2l, Wc, Wh1, Wh2, msg, h_final, pool, hidden, logits, probs, pred, status, h_levels, level_stride, pack, s
    if (labels) return launch_graph_forward<C, 0, WAVES>(GNNHIP_GF_ARGS);
    if (K <= 16) return launch_graph_forward<C, 4, WAVES>(GNNHIP_GF_ARGS);
    if (K <= 32) return launch_graph_forward<C, 8, WAVES>(GNNHIP_GF_ARGS);
    if (K <= 48) return launch_graph_forward<C, 12, WAVES>(GNNHIP_GF_ARGS);
    if (K <= 64) return launch_graph_forward<C, 16, WAVES>(GNNHIP_GF_ARGS);
    return GNNHIP_EUNSUPPORTED;
#undef GNNHIP_GF_ARGS
}

template <int C>
int dispatch_waves(bool labels, int B, int K, int H, int Q, int L, int n16max,
                   const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                   const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                   const float* X, const float* Wn2l, const float* Wc, const float* Wh1, const float* Wh2,
                   float* msg, float* h_final, float* pool, float* hidden, float* logits, float* probs,
                   int* pred, int* status, float* h_levels, long long level_stride, bool pack, hipStream_t s)
{
#define GNNHIP_GF_ARGS B, K, H, Q, L, n16max, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx, s_val, \
                       X, Wn2l, Wc, Wh1, Wh2, msg, h_final, pool, hidden, logits, probs, pred, status, h_levels, level_stride, pack, s
    // hidden 128: eight wavefronts, one per 16-column block (64 registers of a lane hold W^T and the tile operand of
    // a contraction; sixteen wavefronts would leave a lane 128 registers in all)
    if constexpr (C == 128) {
        return dispatch_ksx<C, 8>(labels, GNNHIP_GF_ARGS);
    } else {
        const int tasks = (C / 16) * (n16max / 16);         // (column block x row tile) tasks of the largest graph
        if (tasks <= 4) return dispatch_ksx<C, 4>(labels, GNNHIP_GF_ARGS);
        if (tasks <= 8) return dispatch_ksx<C, 8>(labels, GNNHIP_GF_ARGS);
        return dispatch_ksx<C, 16>(labels, GNNHIP_GF_ARGS);
    }
#undef GNNHIP_GF_ARGS
}

}  // namespace
}  // namespace gnnhip

using namespace gnnhip;

namespace {

int forward_batched_entry(bool labels, int N, int B, int K, int C, int H, int Q, int L, int max_graph_nodes,
                          const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                          const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                          const void* X, const float* W_n2l, const float* W_conv,
                          const float* W_h1, const float* W_h2,
                          float* msg, float* h_final, float* pool, float* hidden, float* logits,
                          float* probs, int* pred, int* status, float* h_levels, void* stream)
{
    GNNHIP_REQUIRE(N >= 1 && B >= 1 && K >= 1 && C >= 1 && H >= 1 && Q >= 1 && L >= 0 && max_graph_nodes >= 1,
                   "bad shape in s2v_forward_batched (N=%d B=%d K=%d C=%d H=%d Q=%d L=%d max_graph_nodes=%d)",
                   N, B, K, C, H, Q, L, max_graph_nodes);
    GNNHIP_REQUIRE(a_row_ptr && a_col_idx && a_val && s_row_ptr && s_col_idx && s_val && X && W_n2l && W_conv && W_h1 && W_h2,
                   "null input in s2v_forward_batched");
    GNNHIP_REQUIRE(msg && h_final && pool && hidden && logits, "null output in s2v_forward_batched");
    if (int rc = require_ready()) return rc;
    if (!(C == 16 || C == 32 || C == 64 || C == 128) || (!labels && K > 64))
        return set_error(GNNHIP_EUNSUPPORTED, "graph-resident forward supports hidden 16/32/64/128 and at most 64 dense feature columns (C=%d K=%d)", C, K);
    if (!(aligned16(msg) && aligned16(h_final)))
        return set_error(GNNHIP_EUNSUPPORTED, "msg and h_final must be 16-byte aligned");
    if (labels && !aligned16(W_n2l))
        return set_error(GNNHIP_EUNSUPPORTED, "W_n2l must be 16-byte aligned for the label input");
    const int n16 = (max_graph_nodes + 15) / 16 * 16;
    if (GraphLds::edge_cap(n16, C, K, H, Q, 256, labels) < 0)
        return set_error(GNNHIP_EUNSUPPORTED, "a graph of %d nodes does not fit the 160 KB of LDS", max_graph_nodes);
    hipStream_t s = as_stream(stream);
    const float* Xf = static_cast<const float*>(X);
    if (h_levels && !aligned16(h_levels)) return set_error(GNNHIP_EUNSUPPORTED, "h_levels must be 16-byte aligned");
    const long long level_stride = (long long)N * C;
    auto run = [&](int n16v, bool pack) {
#define GNNHIP_GF_ARGS labels, B, K, H, Q, L, n16v, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx, s_val, \
                       Xf, W_n2l, W_conv, W_h1, W_h2, msg, h_final, pool, hidden, logits, probs, pred, status, h_levels, level_stride, pack, s
        switch (C) {
        case 16: return dispatch_waves<16>(GNNHIP_GF_ARGS);
        case 32: return dispatch_waves<32>(GNNHIP_GF_ARGS);
        case 128: return dispatch_waves<128>(GNNHIP_GF_ARGS);
        default: return dispatch_waves<64>(GNNHIP_GF_ARGS);
        }
#undef GNNHIP_GF_ARGS
    };
    int rc = GNNHIP_EUNSUPPORTED;
    // more graphs than compute units: runs of consecutive graphs share a workgroup (bins of at least kPackNodes nodes)
    if (B >= kPackMinGraphs && B <= kBinMaxGraphs && H <= kWave && Q <= kWave && !h_levels) {
        // Bin size: a workgroup's time grows with its bin (about 6 us + 20 us per 128 nodes), and the bins run in
        // rounds of one per compute unit, so the size that just avoids another round wins.  The host knows the
        // totals only: a bin wastes about half a mean graph, and every 64 graphs about half a bin.
        int best = 0;
        double best_cost = 0.0;
        for (int cand = n16 > kPackNodes ? n16 : kPackNodes; cand <= kPackMaxNodes; cand += 16) {
            if (GraphLds::edge_cap(cand, C, K, H, Q, 1024, labels) < 256) break;
            const double fill = (double)cand - 0.5 * (double)N / (double)B;
            const double nbins = (double)N / (fill > 16.0 ? fill : 16.0) + (double)B / 128.0;
            const double rounds = (double)(long long)((nbins + kNumCU - 1) / kNumCU);
            const double cost = rounds * (6.0 + 20.0 * cand / 128.0);
            if (!best || cost < best_cost) { best = cand; best_cost = cost; }
        }
        if (best) rc = run(best, true);
    }
    if (rc == GNNHIP_EUNSUPPORTED) rc = run(n16, false);
    if (rc == GNNHIP_EUNSUPPORTED) return set_error(rc, "graph-resident forward could not be configured for this shape");
    return rc;
}

}  // namespace

extern "C" int gnnhip_s2v_forward_batched_f32(int N, int B, int K, int C, int H, int Q, int L, int max_graph_nodes,
                                              const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                                              const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                              const float* X, const float* W_n2l, const float* W_conv,
                                              const float* W_h1, const float* W_h2,
                                              float* msg, float* h_final, float* pool, float* hidden, float* logits,
                                              float* probs, int* pred, int* status, void* stream)
{
    return forward_batched_entry(false, N, B, K, C, H, Q, L, max_graph_nodes, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx,
                                 s_val, X, W_n2l, W_conv, W_h1, W_h2, msg, h_final, pool, hidden, logits, probs, pred, status, nullptr, stream);
}

extern "C" int gnnhip_s2v_forward_batched_labels_f32(int N, int B, int K, int C, int H, int Q, int L, int max_graph_nodes,
                                                     const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                                                     const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                                     const int* node_label, const float* W_n2l, const float* W_conv,
                                                     const float* W_h1, const float* W_h2,
                                                     float* msg, float* h_final, float* pool, float* hidden, float* logits,
                                                     float* probs, int* pred, int* status, void* stream)
{
    return forward_batched_entry(true, N, B, K, C, H, Q, L, max_graph_nodes, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx,
                                 s_val, node_label, W_n2l, W_conv, W_h1, W_h2, msg, h_final, pool, hidden, logits, probs, pred, status, nullptr, stream);
}

extern "C" int gnnhip_s2v_forward_batched_train_f32(int N, int B, int K, int C, int H, int Q, int L, int max_graph_nodes,
                                                    const int* a_row_ptr, const int* a_col_idx, const float* a_val,
                                                    const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                                                    const float* X, const float* W_n2l, const float* W_conv,
                                                    const float* W_h1, const float* W_h2,
                                                    float* msg, float* h_levels, float* pool, float* hidden, float* logits,
                                                    float* probs, int* pred, int* status, void* stream)
{
    GNNHIP_REQUIRE(h_levels, "null h_levels in s2v_forward_batched_train");
    // the last level doubles as the embedding output of the inference entry
    float* h_last = h_levels + (size_t)(L > 0 ? L : 0) * (size_t)(N > 0 ? N : 0) * (size_t)(C > 0 ? C : 0);
    return forward_batched_entry(false, N, B, K, C, H, Q, L, max_graph_nodes, a_row_ptr, a_col_idx, a_val, s_row_ptr, s_col_idx,
                                 s_val, X, W_n2l, W_conv, W_h1, W_h2, msg, h_last, pool, hidden, logits, probs, pred, status, h_levels,
                                 stream);
}
