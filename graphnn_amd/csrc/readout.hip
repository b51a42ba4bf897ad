// Readout of batches of many small graphs, one wavefront per graph:
//     pool = S * h ; hidden = ReLU(pool * W_h1) ; logits = hidden * W_h2 ;
//     probs = softmax(logits) ; pred = argmax(logits)
// (MatMul(S, h) -> MatMul -> ReLU -> MatMul of examples/graph_classification/src/kernel_mean_field.cpp:45-49,
// row softmax of src/tensor/gpu_dense_tensor.cu:298-370, arg-max with the lowest index winning ties as in
// src/tensor/cpu_dense_tensor.cpp:176-196.)
//
// W_h1 and W_h2 are copied into LDS once per workgroup.  A wavefront then takes graphs g, g + nwaves, ...
// and never synchronises with the other wavefronts of its workgroup:
//   1. sum-pool: G = C/4 lanes take one row of h as float4s; the 64/G lane groups walk the graph's rows
//      four at a time each, their sums are added in group order through LDS;
//   2. hidden: lane j adds pool[c] * W_h1[c][j] over c in order (pool broadcast from LDS, W_h1 rows read by
//      consecutive lanes);
//   3. logits the same way over the hidden units, then softmax and arg-max inside the wavefront.
// Hidden sizes 16, 32 and 64 (at 256 the weights fill LDS, one workgroup per CU remains, and SpMM + GEMM
// are faster: 140 against 204 us for 10,000 graphs).  Algorithmic bytes: 4NC (h) + 8N (S) + 4B(C + H + 2Q) + 4(CH + HQ).
#include "gnnhip_internal.h"
#include <math.h>
#include <type_traits>

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kMaxLds = 150 * 1024;

template <int C>
__global__ __launch_bounds__(kBlock) void s2v_readout_wave_kernel(
    int B, int H, int Q, const int* __restrict__ s_row_ptr, const int* __restrict__ s_col_idx,
    const float* __restrict__ s_val, const float* __restrict__ h, const float* __restrict__ Wh1,
    const float* __restrict__ Wh2, float* __restrict__ pool, float* __restrict__ hidden,
    float* __restrict__ logits, float* __restrict__ probs, int* __restrict__ pred)
{
    constexpr int G = C / 4;             // lanes per row of h
    constexpr int RPR = kWave / G;       // rows in flight per step of the wavefront
    extern __shared__ float smem[];
    float* w1 = smem;                    // [C][H]
    float* w2 = w1 + (size_t)C * H;      // [H][Q]
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int per_wave = RPR * C + C + H + Q;
    float* part = w2 + (size_t)H * Q + (size_t)wave * per_wave;   // [RPR][C]
    float* pl = part + RPR * C;          // [C]
    float* hid = pl + C;                 // [H]
    float* lg = hid + H;                 // [Q]
    const int grp = lane / G, tx = lane % G;

    for (int i = threadIdx.x; i < C * H; i += kBlock) w1[i] = Wh1[i];
    for (int i = threadIdx.x; i < H * Q; i += kBlock) w2[i] = Wh2[i];
    __syncthreads();

    const int nwaves = (int)gridDim.x * kWavesPerBlock;
    for (int g = (int)blockIdx.x * kWavesPerBlock + wave; g < B; g += nwaves) {
        const int start = s_row_ptr[g], end = s_row_ptr[g + 1];
        // ---- sum-pool
        float4 acc = f4_zero();
        int t = start + grp;
        for (; t + 3 * RPR < end; t += 4 * RPR) {
            int c[4];
            float v[4];
            float4 x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) { c[u] = s_col_idx[t + u * RPR]; v[u] = s_val[t + u * RPR]; }
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const float4*>(h + (size_t)c[u] * C + tx * 4);
#pragma unroll
            for (int u = 0; u < 4; ++u) f4_fma(acc, v[u], x[u]);
        }
        for (; t < end; t += RPR)
            f4_fma(acc, s_val[t], *reinterpret_cast<const float4*>(h + (size_t)s_col_idx[t] * C + tx * 4));
        *reinterpret_cast<float4*>(part + grp * C + tx * 4) = acc;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        for (int cc = lane; cc < C; cc += kWave) {
            float s = 0.f;
#pragma unroll
            for (int p = 0; p < RPR; ++p) s += part[p * C + cc];
            pl[cc] = s;
            pool[(size_t)g * C + cc] = s;
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        // ---- hidden = ReLU(pool * W_h1)
        for (int j = lane; j < H; j += kWave) {
            float s = 0.f;
#pragma unroll 16
            for (int cc = 0; cc < C; ++cc) s += pl[cc] * w1[(size_t)cc * H + j];
            s = relu_ref(s);
            hid[j] = s;
            hidden[(size_t)g * H + j] = s;
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        // ---- logits = hidden * W_h2
        for (int q = lane; q < Q; q += kWave) {
            float s = 0.f;
#pragma unroll 8
            for (int j = 0; j < H; ++j) s += hid[j] * w2[(size_t)j * Q + q];
            lg[q] = s;
            logits[(size_t)g * Q + q] = s;
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        // ---- softmax + argmax over Q
        if (probs || pred) {
            const float first = lg[0];
            float mx = first;                       // the reference scan starts at element 0
            float bv = -INFINITY;
            int bi = 0x7fffffff;
            for (int q = lane; q < Q; q += kWave) {
                const float v = lg[q];
                mx = max_keep(mx, v);
                const float vv = (v != v) ? -INFINITY : v;     // a NaN that is not first never wins
                argmax_combine(bv, bi, vv, q);
            }
            mx = wave_max(mx);
            wave_argmax(bv, bi);
            if (first != first) bi = 0;             // a NaN in column 0 is never displaced
            if (pred && lane == 0) pred[g] = bi;
            if (probs) {
                float s = 0.f;
                for (int q = lane; q < Q; q += kWave) {
                    const float e = expf(lg[q] - mx);
                    lg[q] = e;
                    s += e;
                }
                s = wave_sum(s);
                for (int q = lane; q < Q; q += kWave) probs[(size_t)g * Q + q] = lg[q] / s;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");     // the wavefront's LDS rows are reused by its next graph
    }
}

template <int C>
int launch_readout_wave(int B, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                        const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                        float* logits, float* probs, int* pred, hipStream_t s)
{
    constexpr int RPR = kWave / (C / 4);
    const size_t smem = sizeof(float) * ((size_t)C * H + (size_t)H * Q + (size_t)kWavesPerBlock * (RPR * C + C + H + Q));
    if (smem > (size_t)kMaxLds) return GNNHIP_EUNSUPPORTED;
    auto kernel = s2v_readout_wave_kernel<C>;
    static LdsLimit lds_limit;               // one per kernel instantiation
    GNNHIP_HIP(lds_limit.raise(reinterpret_cast<const void*>(kernel), smem > 64 * 1024 ? (size_t)kMaxLds : smem));
    const long long blocks_needed = ((long long)B + kWavesPerBlock - 1) / kWavesPerBlock;
    const long long per_cu = smem > 0 ? (long long)(160 * 1024) / (long long)smem : 8;
    long long cap = (long long)kNumCU * (per_cu < 1 ? 1 : (per_cu > 8 ? 8 : per_cu));
    const unsigned grid = (unsigned)(blocks_needed < cap ? blocks_needed : cap);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kBlock), smem, s, B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2,
                       pool, hidden, logits, probs, pred);
    GNNHIP_LAUNCH_CHECK("s2v_readout_wave");
    return GNNHIP_OK;
}

// Readout for wide hidden sizes (C = 128 or 256) on batches of thousands of graphs: one workgroup per tile of
// kTileGraphs graphs.  W_h1 (128 KB at 256 x 128) does not fit LDS next to anything else, so it stays in memory
// and every tile streams it once through L2, each element feeding kTileGraphs / 2 graphs:
//   1. sum-pool   a wavefront per graph, the whole wavefront across the C columns of a row, rows in order
//                 (the order of the reference path), eight loads in flight; pooled rows go to LDS [graphs][C];
//   2. hidden     a lane owns one hidden unit j for half of the tile's graphs: W_h1[c][j] read by consecutive
//                 lanes, pool[g][c..c+3] broadcast from LDS, the sum over c in order;
//   3. logits     a lane per (graph, class), the sum over the hidden units in order;
//   4. softmax and arg-max inside a wavefront per graph, as in the kernel above.
// Algorithmic bytes as above; W_h1 traffic from L2 is 4 C H per tile.
constexpr int kTileGraphs = 16;

template <int C>
__global__ __launch_bounds__(kBlock) void s2v_readout_tile_kernel(
    int B, int H, int Q, const int* __restrict__ s_row_ptr, const int* __restrict__ s_col_idx,
    const float* __restrict__ s_val, const float* __restrict__ h, const float* __restrict__ Wh1,
    const float* __restrict__ Wh2, float* __restrict__ pool, float* __restrict__ hidden,
    float* __restrict__ logits, float* __restrict__ probs, int* __restrict__ pred)
{
    constexpr int VEC = C / kWave;       // floats of a row per lane (2 or 4)
    constexpr int HALF = kTileGraphs / 2;
    using vec_t = typename std::conditional<VEC == 4, float4, float2>::type;
    extern __shared__ float smem[];
    float* pl = smem;                                // [kTileGraphs][C]
    float* hid = pl + kTileGraphs * C;               // [kTileGraphs][H]
    float* lg = hid + (size_t)kTileGraphs * H;       // [kTileGraphs][Q]
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int g0 = (int)blockIdx.x * kTileGraphs;
    const int ng = min(kTileGraphs, B - g0);

    // ---- sum-pool
    for (int gi = wave; gi < kTileGraphs; gi += kWavesPerBlock) {
        float acc[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        if (gi < ng) {
            const int start = s_row_ptr[g0 + gi], end = s_row_ptr[g0 + gi + 1];
            // the wavefront reads 64 node indices and weights at once and hands them round lane by lane;
            // eight rows in flight, added in row order
            for (int base = start; base < end; base += kWave) {
                const int cnt = min(kWave, end - base);
                int my_c = 0;
                float my_v = 0.f;
                if (lane < cnt) { my_c = s_col_idx[base + lane]; my_v = s_val[base + lane]; }
                for (int j = 0; j < cnt; j += 8) {
                    vec_t x[8];
                    float v[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int src = min(j + u, cnt - 1);                     // uniform
                        const int c = __builtin_amdgcn_readlane(my_c, src);
                        v[u] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_v), src));
                        x[u] = *reinterpret_cast<const vec_t*>(h + (size_t)c * C + lane * VEC);
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        if (j + u < cnt) {
                            const float* xp = reinterpret_cast<const float*>(&x[u]);
#pragma unroll
                            for (int i = 0; i < VEC; ++i) acc[i] = fmaf(v[u], xp[i], acc[i]);
                        }
                    }
                }
            }
            *reinterpret_cast<vec_t*>(pool + (size_t)(g0 + gi) * C + lane * VEC) = *reinterpret_cast<vec_t*>(acc);
        }
        *reinterpret_cast<vec_t*>(pl + gi * C + lane * VEC) = *reinterpret_cast<vec_t*>(acc);   // zeros past the last graph
    }
    __syncthreads();

    // ---- hidden = ReLU(pool * W_h1)
    for (int it = threadIdx.x; it < 2 * H; it += kBlock) {
        const int j = it % H, gh = it / H;
        const float* p = pl + gh * HALF * C;
        float a[HALF];
#pragma unroll
        for (int g = 0; g < HALF; ++g) a[g] = 0.f;
        for (int c = 0; c < C; c += 4) {
            float w[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) w[u] = Wh1[(size_t)(c + u) * H + j];
#pragma unroll
            for (int g = 0; g < HALF; ++g) {
                const float4 x = *reinterpret_cast<const float4*>(p + g * C + c);
                a[g] = fmaf(x.x, w[0], a[g]);
                a[g] = fmaf(x.y, w[1], a[g]);
                a[g] = fmaf(x.z, w[2], a[g]);
                a[g] = fmaf(x.w, w[3], a[g]);
            }
        }
#pragma unroll
        for (int g = 0; g < HALF; ++g) {
            const float v = relu_ref(a[g]);
            const int gi = gh * HALF + g;
            hid[(size_t)gi * H + j] = v;
            if (gi < ng) hidden[(size_t)(g0 + gi) * H + j] = v;
        }
    }
    __syncthreads();

    // ---- logits = hidden * W_h2
    for (int it = threadIdx.x; it < kTileGraphs * Q; it += kBlock) {
        const int gi = it / Q, q = it % Q;
        float sum = 0.f;
#pragma unroll 8
        for (int j = 0; j < H; ++j) sum = fmaf(hid[(size_t)gi * H + j], Wh2[(size_t)j * Q + q], sum);
        lg[it] = sum;
        if (gi < ng) logits[(size_t)(g0 + gi) * Q + q] = sum;
    }
    __syncthreads();

    // ---- softmax + argmax over Q, a wavefront per graph
    if (probs || pred) {
        for (int gi = wave; gi < ng; gi += kWavesPerBlock) {
            float* row = lg + (size_t)gi * Q;
            const int g = g0 + gi;
            const float first = row[0];
            float mx = first;                       // the reference scan starts at element 0
            float bv = -INFINITY;
            int bi = 0x7fffffff;
            for (int q = lane; q < Q; q += kWave) {
                const float v = row[q];
                mx = max_keep(mx, v);
                const float vv = (v != v) ? -INFINITY : v;     // a NaN that is not first never wins
                argmax_combine(bv, bi, vv, q);
            }
            mx = wave_max(mx);
            wave_argmax(bv, bi);
            if (first != first) bi = 0;             // a NaN in column 0 is never displaced
            if (pred && lane == 0) pred[g] = bi;
            if (probs) {
                float sum = 0.f;
                for (int q = lane; q < Q; q += kWave) {
                    const float e = expf(row[q] - mx);
                    row[q] = e;
                    sum += e;
                }
                sum = wave_sum(sum);
                for (int q = lane; q < Q; q += kWave) probs[(size_t)g * Q + q] = row[q] / sum;
            }
        }
    }
}

template <int C>
int launch_readout_tile(int B, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                        const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                        float* logits, float* probs, int* pred, hipStream_t s)
{
    const size_t smem = sizeof(float) * (size_t)kTileGraphs * ((size_t)C + H + Q);
    if (smem > 64 * 1024) return GNNHIP_EUNSUPPORTED;
    const unsigned grid = (unsigned)(((long long)B + kTileGraphs - 1) / kTileGraphs);
    hipLaunchKernelGGL(s2v_readout_tile_kernel<C>, dim3(grid), dim3(kBlock), smem, s, B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2,
                       pool, hidden, logits, probs, pred);
    GNNHIP_LAUNCH_CHECK("s2v_readout_tile");
    return GNNHIP_OK;
}

}  // namespace

// A workgroup per tile of graphs, hidden sizes 128 and 256; for batches of thousands of small graphs (the caller decides).
int readout_tile_dispatch(int B, int C, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                          const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                          float* logits, float* probs, int* pred, hipStream_t s)
{
    if (!aligned16(h) || !aligned16(pool) || B <= 0) return GNNHIP_EUNSUPPORTED;
#define GNNHIP_RO_ARGS B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s
    switch (C) {
    case 128: return launch_readout_tile<128>(GNNHIP_RO_ARGS);
    case 256: return launch_readout_tile<256>(GNNHIP_RO_ARGS);
    }
#undef GNNHIP_RO_ARGS
    return GNNHIP_EUNSUPPORTED;
}

// One wavefront per graph; for batches of many graphs (the caller decides).  Returns GNNHIP_EUNSUPPORTED
// for hidden sizes it has no kernel for and when W_h1 and W_h2 do not fit LDS.
int readout_wave_dispatch(int B, int C, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                          const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                          float* logits, float* probs, int* pred, hipStream_t s)
{
    if (!aligned16(h)) return GNNHIP_EUNSUPPORTED;
#define GNNHIP_RO_ARGS B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s
    switch (C) {
    case 16: return launch_readout_wave<16>(GNNHIP_RO_ARGS);
    case 32: return launch_readout_wave<32>(GNNHIP_RO_ARGS);
    case 64: return launch_readout_wave<64>(GNNHIP_RO_ARGS);
    }
#undef GNNHIP_RO_ARGS
    return GNNHIP_EUNSUPPORTED;
}

}  // namespace gnnhip
