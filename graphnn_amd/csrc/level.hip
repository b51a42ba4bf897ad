// Fused structure2vec kernels for gfx950 (hidden size C in {16, 32, 64}; wider
// hidden sizes take the unfused route in forward.hip):
//
//   s2v_input_kernel    msg = X * W_n2l ; h0 = ReLU(msg)
//   s2v_level_kernel    h_out = ReLU((A * h_in) * W + bias + msg)
//   s2v_readout_kernel  pool = S * h ; hidden = ReLU(pool * W_h1) ;
//                       logits = hidden * W_h2 ; probs = softmax(logits) ; pred = argmax
//
// A level reads h_in (gathered), msg and the CSR arrays once and writes h_out
// once: 4(N+1) + 8E + 12NC + 4C^2 algorithmic bytes, against roughly nine
// passes over an N x C activation in the operator-by-operator schedule.  At
// C = 64 the arithmetic intensity is ~6 flop/byte, far below the machine
// balance, so the dense C x C contraction runs on plain FMA out of LDS and the
// kernel is HBM-bound.
//
// Layout of one workgroup (256 lanes) in input/level kernels:
//   G = C/4 lanes form a row group; the workgroup holds P = 256/G groups and
//   processes tiles of R = RT * P rows.  Phase 1 fills an LDS tile [R][C+4]
//   (level: neighbour gather-sum, one float4 per lane per gathered row; input:
//   a straight copy of X rows).  Phase 2 multiplies the tile by W held in LDS:
//   lane (ty, tx) produces rows ty + r*P (r < RT), columns 4tx..4tx+3.
//   Phase 3 adds bias and msg, applies ReLU and stores float4s.
// Workgroups are persistent over tiles so W is loaded into LDS once per group.
#include "gnnhip_internal.h"

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kLongRow = 1024;      // level kernel: longer rows are gathered by the whole workgroup

__device__ __forceinline__ float4 f4_zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ void f4_fma(float4& a, float s, const float4& x)
{
    a.x += s * x.x; a.y += s * x.y; a.z += s * x.z; a.w += s * x.w;
}
__device__ __forceinline__ float relu_ref(float v) { return v < 0.f ? 0.f : v; }

// acc[r] += tile[row(r)][0..kdim) * Ws[0..kdim)[4tx..4tx+3]
template <int C, int RT>
__device__ __forceinline__ void tile_times_w(const float* tile, int ldt, int kdim, const float* Ws,
                                             int ty, int tx, float4 (&acc)[RT])
{
    constexpr int P = kBlock / (C / 4);
    const int k4end = kdim & ~3;
#pragma unroll 2
    for (int k = 0; k < k4end; k += 4) {
        float4 w[4];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) w[kk] = *reinterpret_cast<const float4*>(Ws + (size_t)(k + kk) * C + tx * 4);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const float4 a = *reinterpret_cast<const float4*>(tile + (size_t)(ty + r * P) * ldt + k);
            f4_fma(acc[r], a.x, w[0]);
            f4_fma(acc[r], a.y, w[1]);
            f4_fma(acc[r], a.z, w[2]);
            f4_fma(acc[r], a.w, w[3]);
        }
    }
    for (int k = k4end; k < kdim; ++k) {
        const float4 w = *reinterpret_cast<const float4*>(Ws + (size_t)k * C + tx * 4);
#pragma unroll
        for (int r = 0; r < RT; ++r) f4_fma(acc[r], tile[(size_t)(ty + r * P) * ldt + k], w);
    }
}

// ---------------------------------------------------------------- input: msg = X * W_n2l, h0 = ReLU(msg)
template <int C, int RT>
__global__ __launch_bounds__(kBlock) void s2v_input_kernel(
    int N, int K, const float* __restrict__ X, const float* __restrict__ Wn2l,
    float* __restrict__ msg, float* __restrict__ h0)
{
    constexpr int G = C / 4, P = kBlock / G, R = RT * P;
    extern __shared__ float smem[];
    const int ldt = ((K + 3) & ~3) + 4;              // padded row stride of the X tile, multiple of 4
    float* Ws = smem;                              // [K][C]
    float* tile = smem + (size_t)K * C;            // [R][ldt]
    const int tid = threadIdx.x, tx = tid % G, ty = tid / G;

    for (int i = tid; i < K * C / 4; i += kBlock)
        reinterpret_cast<float4*>(Ws)[i] = reinterpret_cast<const float4*>(Wn2l)[i];

    const int ntiles = (N + R - 1) / R;
    for (int tile_id = blockIdx.x; tile_id < ntiles; tile_id += gridDim.x) {
        const long long row0 = (long long)tile_id * R;
        const int rows = (int)min((long long)R, (long long)N - row0);
        __syncthreads();                           // previous tile consumed; Ws visible on the first pass
        // rows of X are contiguous in memory: copy rows*K floats, coalesced
        const float* src = X + (size_t)row0 * K;
        for (int i = tid; i < R * K; i += kBlock) {
            const int r = i / K, c = i - r * K;
            tile[(size_t)r * ldt + c] = (r < rows) ? src[i] : 0.f;
        }
        __syncthreads();

        float4 acc[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) acc[r] = f4_zero();
        tile_times_w<C, RT>(tile, ldt, K, Ws, ty, tx, acc);

#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const int lr = ty + r * P;
            if (lr < rows) {
                const size_t off = ((size_t)row0 + lr) * C + tx * 4;
                const float4 v = acc[r];
                *reinterpret_cast<float4*>(msg + off) = v;
                *reinterpret_cast<float4*>(h0 + off) =
                    make_float4(relu_ref(v.x), relu_ref(v.y), relu_ref(v.z), relu_ref(v.w));
            }
        }
    }
}

// ---------------------------------------------------------------- level
template <int C, int RT>
__global__ __launch_bounds__(kBlock) void s2v_level_kernel(
    int N, const int* __restrict__ row_ptr, const int* __restrict__ col_idx, const float* __restrict__ val,
    const float* __restrict__ h_in, const float* __restrict__ W, const float* __restrict__ msg,
    const float* __restrict__ bias, float* __restrict__ h_out)
{
    constexpr int G = C / 4, P = kBlock / G, R = RT * P, LDT = C + 4;
    extern __shared__ float smem[];
    float* Ws = smem;                              // [C][C]
    float* tile = Ws + C * C;                      // [R][LDT]   gathered A*h rows
    float* red = tile + R * LDT;                   // [P][C]     partial sums for long rows
    __shared__ int lr_list[R];
    __shared__ int lr_count;

    const int tid = threadIdx.x, tx = tid % G, ty = tid / G;

    for (int i = tid; i < C * C / 4; i += kBlock)
        reinterpret_cast<float4*>(Ws)[i] = reinterpret_cast<const float4*>(W)[i];

    const int ntiles = (N + R - 1) / R;
    for (int tile_id = blockIdx.x; tile_id < ntiles; tile_id += gridDim.x) {
        const long long row0 = (long long)tile_id * R;
        const int rows = (int)min((long long)R, (long long)N - row0);
        if (tid == 0) lr_count = 0;
        __syncthreads();                           // previous tile consumed, counter reset, Ws visible

        // ---- phase 1: gather-sum, group ty owns local rows ty + r*P
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const int lr = ty + r * P;
            int start = 0, end = 0;
            if (lr < rows) { start = row_ptr[row0 + lr]; end = row_ptr[row0 + lr + 1]; }
            if (end - start > kLongRow) {
                if (tx == 0) lr_list[atomicAdd(&lr_count, 1)] = lr;
                end = start;
            }
            float4 acc = f4_zero();
            for (int base = start; base < end; base += G) {
                const int t = base + tx;
                int c = 0;
                float v = 0.f;
                if (t < end) { c = col_idx[t]; v = val[t]; }
                const int cnt = min(G, end - base);
                for (int j = 0; j < cnt; j += 4) {
                    int cj[4];
                    float vj[4];
                    float4 x[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        cj[u] = __shfl(c, (j + u) & (G - 1), G);
                        vj[u] = __shfl(v, (j + u) & (G - 1), G);
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        x[u] = (j + u < cnt) ? *reinterpret_cast<const float4*>(h_in + (size_t)cj[u] * C + tx * 4) : f4_zero();
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                        if (j + u < cnt) f4_fma(acc, vj[u], x[u]);
                }
            }
            *reinterpret_cast<float4*>(tile + (size_t)lr * LDT + tx * 4) = acc;
        }
        __syncthreads();

        // ---- phase 1b: rows too long for one group, entries split over all P groups
        const int nlong = lr_count;
        for (int li = 0; li < nlong; ++li) {
            const int lr = lr_list[li];
            const int ls = row_ptr[row0 + lr], le = row_ptr[row0 + lr + 1];
            float4 acc = f4_zero();
            int t = ls + ty;
            for (; t + 3 * P < le; t += 4 * P) {
                int c4[4];
                float v4[4];
                float4 x[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) { c4[u] = col_idx[t + u * P]; v4[u] = val[t + u * P]; }
#pragma unroll
                for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const float4*>(h_in + (size_t)c4[u] * C + tx * 4);
#pragma unroll
                for (int u = 0; u < 4; ++u) f4_fma(acc, v4[u], x[u]);
            }
            for (; t < le; t += P)
                f4_fma(acc, val[t], *reinterpret_cast<const float4*>(h_in + (size_t)col_idx[t] * C + tx * 4));
            *reinterpret_cast<float4*>(red + (size_t)ty * C + tx * 4) = acc;
            __syncthreads();
            if (ty == 0) {
                float4 s = f4_zero();
                for (int g = 0; g < P; ++g) {
                    const float4 p = *reinterpret_cast<const float4*>(red + (size_t)g * C + tx * 4);
                    s.x += p.x; s.y += p.y; s.z += p.z; s.w += p.w;
                }
                *reinterpret_cast<float4*>(tile + (size_t)lr * LDT + tx * 4) = s;
            }
            __syncthreads();
        }

        // ---- phase 2: tile * W
        float4 acc[RT];
#pragma unroll
        for (int r = 0; r < RT; ++r) acc[r] = f4_zero();
        tile_times_w<C, RT>(tile, LDT, C, Ws, ty, tx, acc);

        // ---- phase 3: + bias + msg, ReLU, store
        float4 b4 = f4_zero();
        if (bias) b4 = *reinterpret_cast<const float4*>(bias + tx * 4);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const int lr = ty + r * P;
            if (lr < rows) {
                const size_t off = ((size_t)row0 + lr) * C + tx * 4;
                float4 v = acc[r];
                if (bias) { v.x += b4.x; v.y += b4.y; v.z += b4.z; v.w += b4.w; }
                if (msg) {
                    const float4 mm = *reinterpret_cast<const float4*>(msg + off);
                    v.x += mm.x; v.y += mm.y; v.z += mm.z; v.w += mm.w;
                }
                *reinterpret_cast<float4*>(h_out + off) =
                    make_float4(relu_ref(v.x), relu_ref(v.y), relu_ref(v.z), relu_ref(v.w));
            }
        }
    }
}

// ---------------------------------------------------------------- readout, one workgroup per subgraph
// LDS: part[P][C] | pool[C] | hid[H] | lg[Q]
template <int C>
__global__ __launch_bounds__(kBlock) void s2v_readout_kernel(
    int B, int H, int Q, const int* __restrict__ s_row_ptr, const int* __restrict__ s_col_idx,
    const float* __restrict__ s_val, const float* __restrict__ h, const float* __restrict__ Wh1,
    const float* __restrict__ Wh2, float* __restrict__ pool, float* __restrict__ hidden,
    float* __restrict__ logits, float* __restrict__ probs, int* __restrict__ pred)
{
    constexpr int G = C / 4, P = kBlock / G;
    extern __shared__ float smem[];
    float* part = smem;
    float* pl = part + P * C;
    float* hid = pl + C;
    float* lg = hid + H;
    const int tid = threadIdx.x, tx = tid % G, ty = tid / G;

    for (int g = blockIdx.x; g < B; g += gridDim.x) {
        const int start = s_row_ptr[g], end = s_row_ptr[g + 1];
        // sum-pool: group ty takes entries start+ty, start+ty+P, ...
        float4 acc = f4_zero();
        int t = start + ty;
        for (; t + P < end; t += 2 * P) {
            const int c0 = s_col_idx[t], c1 = s_col_idx[t + P];
            const float v0 = s_val[t], v1 = s_val[t + P];
            const float4 x0 = *reinterpret_cast<const float4*>(h + (size_t)c0 * C + tx * 4);
            const float4 x1 = *reinterpret_cast<const float4*>(h + (size_t)c1 * C + tx * 4);
            f4_fma(acc, v0, x0);
            f4_fma(acc, v1, x1);
        }
        if (t < end) f4_fma(acc, s_val[t], *reinterpret_cast<const float4*>(h + (size_t)s_col_idx[t] * C + tx * 4));
        *reinterpret_cast<float4*>(part + (size_t)ty * C + tx * 4) = acc;
        __syncthreads();
        if (tid < C) {
            float s = 0.f;
            for (int p = 0; p < P; ++p) s += part[(size_t)p * C + tid];
            pl[tid] = s;
            pool[(size_t)g * C + tid] = s;
        }
        __syncthreads();
        // hidden = ReLU(pool * W_h1)
        for (int j = tid; j < H; j += kBlock) {
            float s = 0.f;
            for (int c = 0; c < C; ++c) s += pl[c] * Wh1[(size_t)c * H + j];
            s = relu_ref(s);
            hid[j] = s;
            hidden[(size_t)g * H + j] = s;
        }
        __syncthreads();
        // logits = hidden * W_h2
        for (int q = tid; q < Q; q += kBlock) {
            float s = 0.f;
            for (int j = 0; j < H; ++j) s += hid[j] * Wh2[(size_t)j * Q + q];
            lg[q] = s;
            logits[(size_t)g * Q + q] = s;
        }
        __syncthreads();
        // softmax + argmax over Q by the first wavefront
        if (tid < kWave) {
            const float first = lg[0];
            float mx = first;                       // reference scan starts at element 0
            float bv = -INFINITY;
            int bi = 0x7fffffff;
            for (int q = tid; q < Q; q += kWave) {
                const float v = lg[q];
                mx = max_keep(mx, v);
                const float vv = (v != v) ? -INFINITY : v;     // a NaN that is not first never wins
                argmax_combine(bv, bi, vv, q);
            }
            mx = wave_max(mx);
            wave_argmax(bv, bi);
            if (first != first) bi = 0;            // NaN in column 0 is never displaced
            if (pred && tid == 0) pred[g] = bi;
            if (probs) {
                float s = 0.f;
                for (int q = tid; q < Q; q += kWave) {
                    const float e = expf(lg[q] - mx);
                    lg[q] = e;
                    s += e;
                }
                s = wave_sum(s);
                for (int q = tid; q < Q; q += kWave) probs[(size_t)g * Q + q] = lg[q] / s;
            }
        }
        __syncthreads();
    }
}

template <int C, int RT>
int launch_input(int N, int K, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s)
{
    constexpr int R = RT * (kBlock / (C / 4));
    const int ldt = ((K + 3) & ~3) + 4;
    const size_t smem = sizeof(float) * ((size_t)K * C + (size_t)R * ldt);
    if (smem > 64 * 1024) return GNNHIP_EUNSUPPORTED;
    const int ntiles = (N + R - 1) / R;
    const int grid = ntiles < kNumCU * 4 ? ntiles : kNumCU * 4;
    hipLaunchKernelGGL((s2v_input_kernel<C, RT>), dim3(grid), dim3(kBlock), smem, s, N, K, X, Wn2l, msg, h0);
    GNNHIP_LAUNCH_CHECK("s2v_input");
    return GNNHIP_OK;
}

template <int C, int RT>
int launch_level(int N, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                 const float* W, const float* msg, const float* bias, float* h_out, hipStream_t s)
{
    constexpr int P = kBlock / (C / 4), R = RT * P;
    const size_t smem = sizeof(float) * ((size_t)C * C + (size_t)R * (C + 4) + (size_t)P * C);
    const int ntiles = (N + R - 1) / R;
    const int grid = ntiles < kNumCU * 4 ? ntiles : kNumCU * 4;
    hipLaunchKernelGGL((s2v_level_kernel<C, RT>), dim3(grid), dim3(kBlock), smem, s,
                       N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out);
    GNNHIP_LAUNCH_CHECK("s2v_level");
    return GNNHIP_OK;
}

template <int C>
int launch_readout(int B, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                   const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                   float* logits, float* probs, int* pred, hipStream_t s)
{
    constexpr int P = kBlock / (C / 4);
    const size_t smem = sizeof(float) * ((size_t)P * C + C + (size_t)H + (size_t)Q);
    if (smem > 64 * 1024) return GNNHIP_EUNSUPPORTED;
    const int grid = B < kNumCU * 8 ? B : kNumCU * 8;
    hipLaunchKernelGGL((s2v_readout_kernel<C>), dim3(grid), dim3(kBlock), smem, s,
                       B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred);
    GNNHIP_LAUNCH_CHECK("s2v_readout");
    return GNNHIP_OK;
}

inline bool small_batch(int N) { return N <= 32 * 1024; }

}  // namespace

// ---- dispatchers used by the C entry points and by forward.hip.
// Return GNNHIP_EUNSUPPORTED (without setting an error text) when the shape has no fused kernel.
bool fused_hidden_supported(int C) { return C == 16 || C == 32 || C == 64; }

int input_dispatch(int N, int K, int C, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s)
{
    if (!(aligned16(Wn2l) && aligned16(msg) && aligned16(h0))) return GNNHIP_EUNSUPPORTED;
    const bool small = small_batch(N);
    switch (C) {
    case 16: return small ? launch_input<16, 1>(N, K, X, Wn2l, msg, h0, s) : launch_input<16, 4>(N, K, X, Wn2l, msg, h0, s);
    case 32: return small ? launch_input<32, 1>(N, K, X, Wn2l, msg, h0, s) : launch_input<32, 4>(N, K, X, Wn2l, msg, h0, s);
    case 64: return small ? launch_input<64, 1>(N, K, X, Wn2l, msg, h0, s) : launch_input<64, 4>(N, K, X, Wn2l, msg, h0, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

int level_dispatch(int N, int C, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                   const float* W, const float* msg, const float* bias, float* h_out, hipStream_t s)
{
    if (!(aligned16(h_in) && aligned16(W) && aligned16(h_out) && (!msg || aligned16(msg)) && (!bias || aligned16(bias))))
        return GNNHIP_EUNSUPPORTED;
    const bool small = small_batch(N);
    switch (C) {
    case 16: return small ? launch_level<16, 1>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s)
                          : launch_level<16, 4>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
    case 32: return small ? launch_level<32, 1>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s)
                          : launch_level<32, 4>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
    case 64: return small ? launch_level<64, 1>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s)
                          : launch_level<64, 4>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

int readout_dispatch(int B, int C, int H, int Q, const int* s_row_ptr, const int* s_col_idx, const float* s_val,
                     const float* h, const float* Wh1, const float* Wh2, float* pool, float* hidden,
                     float* logits, float* probs, int* pred, hipStream_t s)
{
    if (!aligned16(h)) return GNNHIP_EUNSUPPORTED;
    switch (C) {
    case 16: return launch_readout<16>(B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    case 32: return launch_readout<32>(B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    case 64: return launch_readout<64>(B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

}  // namespace gnnhip
