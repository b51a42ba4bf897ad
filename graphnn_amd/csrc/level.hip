// Fused structure2vec kernels for gfx950, hidden size C in {16, 32, 64}, and the dispatchers of the
// three stages (wider hidden sizes: input_wide.hip, level_wide.hip; other sizes: the unfused route in
// forward.hip):
//
//   s2v_input_kernel    msg = X * W_n2l ; h0 = ReLU(msg)
//   s2v_level_kernel    h_out = ReLU((A * h_in) * W + bias + msg), with 64-bit addressing: the kernel for
//                       activations of 4 GiB and more (smaller ones take level_stream.hip)
//   s2v_readout_kernel  pool = S * h ; hidden = ReLU(pool * W_h1) ;
//                       logits = hidden * W_h2 ; probs = softmax(logits) ; pred = argmax,
//                       one workgroup per graph (many graphs: readout.hip)
//
// A level reads h_in (gathered), msg and the CSR arrays once and writes h_out
// once: 4(N+1) + 8E + 12NC + 4C^2 algorithmic bytes, against roughly nine
// passes over an N x C activation in the operator-by-operator schedule.  At
// C = 64 the arithmetic intensity is ~6 flop/byte, far below the machine
// balance: the kernel is HBM-bound.
//
// Layout of one workgroup (256 lanes) in the input kernel:
//   G = C/4 lanes form a row group; the workgroup holds P = 256/G groups and
//   processes tiles of R = RT * P rows.  Phase 1 copies the tile's rows of X into LDS [R][K+pad],
//   phase 2 multiplies the tile by W_n2l held in LDS: lane (ty, tx) produces rows ty + r*P (r < RT),
//   columns 4tx..4tx+3, phase 3 stores msg and ReLU(msg) as float4s.
// Workgroups are persistent over tiles so W_n2l is loaded into LDS once per group.
#include "gnnhip_internal.h"
#include <stdlib.h>

// Phase markers for a timing build of this file; they expand to nothing in the library.
#ifndef GNNHIP_PHASE_MARK
#define GNNHIP_PHASE_MARK(i)
#endif

namespace gnnhip {

// spmm.hip
// level_stream.hip
int level_stream_dispatch(int N, int C, bool dense, const int* row_ptr, const int* col_idx, const float* val,
                          const float* h_in, const float* W, const float* msg, const float* bias, float* h_out,
                          const HubPlan& hubs, bool relu_in, hipStream_t s);
bool level_stream_covers(int N, int C);
int level_stream_backward_dispatch(int N, int C, const int* row_ptr, const int* col_idx, const float* val, const float* x,
                                   const float* W, float* agg_out, float* out, const float* gate, float* acc, const HubPlan& hubs,
                                   hipStream_t s);
// input_wide.hip
int input_wide_dispatch(int N, int K, int C, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s);
// level_wide.hip
int level_wide_dispatch(int N, int C, long long nnz, const int* row_ptr, const int* col_idx, const float* val,
                        const float* h_in, const float* W, const float* msg, const float* bias, float* h_out, bool relu_in,
                        hipStream_t s);
bool level_wide_covers(int N, int C);
int level_wide_backward_dispatch(int N, int C, const int* row_ptr, const int* col_idx, const float* val, const float* dz, const float* W,
                                 float* u, float* g_prev, const float* gate, float* acc, hipStream_t s);

namespace {

constexpr int kBlock = 256;

// Copy N4 float4s (a compile-time count) from global to LDS.  All of a lane's loads are
// issued before the first LDS store, so the copy costs one memory round trip.
template <int N4>
__device__ __forceinline__ void copy_to_lds_fixed(float* dst, const float* __restrict__ src, int tid)
{
    constexpr int FULL = N4 / kBlock, REM = N4 % kBlock;
    const float4* s4 = reinterpret_cast<const float4*>(src);
    float4* d4 = reinterpret_cast<float4*>(dst);
    float4 r[FULL + 1];
#pragma unroll
    for (int i = 0; i < FULL; ++i) r[i] = s4[tid + i * kBlock];
    if (REM && tid < REM) r[FULL] = s4[tid + FULL * kBlock];
#pragma unroll
    for (int i = 0; i < FULL; ++i) d4[tid + i * kBlock] = r[i];
    if (REM && tid < REM) d4[tid + FULL * kBlock] = r[FULL];
}

// Run-time count: four loads in flight per lane.
__device__ __forceinline__ void copy_to_lds(float* dst, const float* __restrict__ src, int n4, int tid)
{
    const float4* s4 = reinterpret_cast<const float4*>(src);
    float4* d4 = reinterpret_cast<float4*>(dst);
    int base = 0;
    for (; base + 4 * kBlock <= n4; base += 4 * kBlock) {
        const float4 r0 = s4[base + tid], r1 = s4[base + tid + kBlock];
        const float4 r2 = s4[base + tid + 2 * kBlock], r3 = s4[base + tid + 3 * kBlock];
        d4[base + tid] = r0; d4[base + tid + kBlock] = r1;
        d4[base + tid + 2 * kBlock] = r2; d4[base + tid + 3 * kBlock] = r3;
    }
    for (int idx = base + tid; idx < n4; idx += kBlock) d4[idx] = s4[idx];
}

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

    copy_to_lds(Ws, Wn2l, K * C / 4, tid);

    const int ntiles = (N + R - 1) / R;
    for (int tile_id = blockIdx.x; tile_id < ntiles; tile_id += gridDim.x) {
        const long long row0 = (long long)tile_id * R;
        const int rows = (int)min((long long)R, (long long)N - row0);
        __syncthreads();                           // previous tile consumed; Ws visible on the first pass
        // rows of X are contiguous in memory: copy rows*K floats, coalesced
        const float* src = X + (size_t)row0 * K;
        for (int base = 0; base < R * K; base += 4 * kBlock) {
            float xv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = base + tid + u * kBlock;
                xv[u] = (i < rows * K) ? src[i] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = base + tid + u * kBlock;
                if (i < R * K) { const int r = i / K; tile[(size_t)r * ldt + (i - r * K)] = xv[u]; }
            }
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
                if (h0) *reinterpret_cast<float4*>(h0 + off) = relu_ref4(v);      // no h0: the caller applies ReLU on reading msg
            }
        }
    }
}

// ---------------------------------------------------------------- level
// Wave-autonomous: each wavefront owns tiles of 16 rows and never synchronises with
// another wavefront.  Per tile:
//   1. gather-sum: G = C/4 lanes per row gather float4 slices of the neighbours' rows
//      (64/G rows at a time) and park the sums in a wave-private LDS tile [16][C+4];
//   2. contraction on the matrix cores: out^T = W^T * tile^T with
//      v_mfma_f32_16x16x4_f32, W^T held in registers for the lifetime of the wavefront.
//      Lane (q = lane/16, t = lane%16) feeds k = (C/4) q + s at step s, and the output
//      columns of block jb are permuted so that the lane ends up owning row t,
//      columns (C/4) q .. (C/4) q + C/4 - 1: contiguous float4s for the epilogue;
//   3. epilogue: + bias + msg, ReLU, float4 stores.
constexpr int kTwoStepMeanDegree = 12;         // mean entries per row from which SpMM + in-place contraction is used
constexpr int kWaveLongRow = 48;     // entries; longer rows are gathered by all groups of the wavefront together,
                                     // and past kHubThreshold they come from the hub pre-pass when there is one

// DENSE: the aggregate A * h_in has already been written to h_out (by the SpMM); the tile is read
// from there and the rows are overwritten in place with the level's output.
template <int C, bool DENSE>
__global__ __launch_bounds__(kBlock) void s2v_level_kernel(
    int N, const int* __restrict__ row_ptr, const int* __restrict__ col_idx, const float* __restrict__ val,
    const float* __restrict__ h_in, const float* __restrict__ W, const float* __restrict__ msg,
    const float* __restrict__ bias, float* __restrict__ h_out,
    const int* __restrict__ hub_slot, const float* __restrict__ hub_agg, int hub_ld)
{
    constexpr int G = C / 4;             // lanes per gathered row
    constexpr int RPR = kWave / G;       // rows gathered per round
    constexpr int ROUNDS = 16 / RPR;     // rounds per tile
    constexpr int KS = C / 4;            // contraction steps
    constexpr int NJB = C / 16;          // 16-column output blocks
    constexpr int LDT = C + 4;
    constexpr int kWavesPerBlock = kBlock / kWave;

    __shared__ float lds[kWavesPerBlock][16 * LDT + RPR * C];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    float* tile = lds[wave];             // [16][LDT]
    float* red = tile + 16 * LDT;        // [RPR][C]
    const int q = lane >> 4, t = lane & 15;
    const int grp = lane / G, tx = lane % G;

    GNNHIP_PHASE_MARK(0);
    // W^T operand: wreg[jb][s] = W[KS q + s][KS (t/4) + 4 jb + t%4]
    float wreg[NJB][KS];
#pragma unroll
    for (int jb = 0; jb < NJB; ++jb)
#pragma unroll
        for (int s = 0; s < KS; ++s)
            wreg[jb][s] = W[(size_t)(KS * q + s) * C + KS * (t >> 2) + 4 * jb + (t & 3)];
    GNNHIP_PHASE_MARK(1);

    const long long ntiles = ((long long)N + 15) / 16;
    const long long wave_stride = (long long)gridDim.x * kWavesPerBlock;
    const long long tile_first = (long long)blockIdx.x * kWavesPerBlock + wave;

    // The CSR data of a tile is asked for one tile ahead (its first batch of column indices and
    // weights) and two tiles ahead (its 17 row pointers), so that a tile's chain of dependent
    // memory trips is the gather alone.  Tiles past the end read row_ptr[N] 17 times: empty rows.
    auto load_rp = [&](long long tid) -> int {
        int r = 0;
        const long long rr = tid * 16 + lane;
        if (!DENSE && lane <= 16) r = row_ptr[rr < (long long)N ? rr : (long long)N];
        return r;
    };
    int c0n[ROUNDS];
    float v0n[ROUNDS];
    auto load_first_batch = [&](int rp) {
#pragma unroll
        for (int rd = 0; rd < ROUNDS; ++rd) {
            const int lr = rd * RPR + grp;
            const int s0 = __shfl(rp, lr, kWave), e0 = __shfl(rp, lr + 1, kWave);
            c0n[rd] = 0;
            v0n[rd] = 0.f;
            if (!DENSE && e0 - s0 <= kWaveLongRow && s0 + tx < e0) { c0n[rd] = col_idx[s0 + tx]; v0n[rd] = val[s0 + tx]; }
        }
    };
    int rp_cur = load_rp(tile_first);
    int rp_nxt = load_rp(tile_first + wave_stride);
    if (!DENSE) load_first_batch(rp_cur);

    for (long long tile_id = tile_first; tile_id < ntiles; tile_id += wave_stride) {
        const long long row0 = tile_id * 16;
        // msg of this tile is asked for first, so its trip to memory runs under the gather and the
        // contraction instead of after them
        float4 mpre[NJB];
#pragma unroll
        for (int jb = 0; jb < NJB; ++jb) {
            mpre[jb] = f4_zero();
            if (msg && row0 + t < N) mpre[jb] = *reinterpret_cast<const float4*>(msg + (size_t)(row0 + t) * C + KS * q + 4 * jb);
        }
        if (DENSE) {
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) {
                const int lr = rd * RPR + grp;
                float4 x = f4_zero();
                if (row0 + lr < N) x = *reinterpret_cast<const float4*>(h_out + (size_t)(row0 + lr) * C + tx * 4);
                *reinterpret_cast<float4*>(tile + lr * LDT + tx * 4) = x;
            }
        } else {
            const int rp = rp_cur;
            int st[ROUNDS], en[ROUNDS], c0[ROUNDS];
            float v0[ROUNDS];
            bool is_long[ROUNDS];
            int hub[ROUNDS];
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) {
                const int lr = rd * RPR + grp;
                st[rd] = __shfl(rp, lr, kWave);
                en[rd] = __shfl(rp, lr + 1, kWave);
                is_long[rd] = (en[rd] - st[rd] > kWaveLongRow);
                hub[rd] = -1;
                if (is_long[rd]) {
                    if (hub_slot && en[rd] - st[rd] > kHubThreshold) hub[rd] = hub_slot[row0 + lr];   // summed by the pre-pass
                    if (hub[rd] >= 0) is_long[rd] = false;
                    en[rd] = st[rd];
                }
                c0[rd] = c0n[rd];
                v0[rd] = v0n[rd];
            }

            // ---- gather-sum; the first four neighbours of every row of the tile are fetched together
            float4 x[ROUNDS][4];
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) {
                const int cnt = en[rd] - st[rd];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int cj = __shfl(c0[rd], u & (G - 1), G);
                    x[rd][u] = (u < cnt && u < G) ? *reinterpret_cast<const float4*>(h_in + (size_t)cj * C + tx * 4) : f4_zero();
                }
            }
            // the next tile's first batch and the row pointers of the tile after it, behind the gathers
            rp_cur = rp_nxt;
            rp_nxt = load_rp(tile_id + 2 * wave_stride);
            load_first_batch(rp_cur);
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) {
                const int lr = rd * RPR + grp;
                const int cnt_all = en[rd] - st[rd];
                float4 acc = f4_zero();
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (u < cnt_all && u < G) f4_fma(acc, __shfl(v0[rd], u & (G - 1), G), x[rd][u]);
                // the rest of the row: entries 4.. of the first batch, then further batches of G
                for (int base = st[rd]; base < en[rd]; base += G) {
                    int c = c0[rd];
                    float v = v0[rd];
                    int j0 = (G > 4) ? 4 : G;          // the first batch has had its first min(4, G) entries consumed
                    if (base != st[rd]) {
                        c = 0; v = 0.f; j0 = 0;
                        if (base + tx < en[rd]) { c = col_idx[base + tx]; v = val[base + tx]; }
                    }
                    const int cnt = min(G, en[rd] - base);
                    for (int j = j0; j < cnt; j += 4) {
                        int cj[4];
                        float vj[4];
                        float4 xx[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            cj[u] = __shfl(c, (j + u) & (G - 1), G);
                            vj[u] = __shfl(v, (j + u) & (G - 1), G);
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            xx[u] = (j + u < cnt) ? *reinterpret_cast<const float4*>(h_in + (size_t)cj[u] * C + tx * 4) : f4_zero();
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            if (j + u < cnt) f4_fma(acc, vj[u], xx[u]);
                    }
                }
                if (hub[rd] >= 0) acc = *reinterpret_cast<const float4*>(hub_agg + (size_t)hub[rd] * hub_ld + tx * 4);
                *reinterpret_cast<float4*>(tile + lr * LDT + tx * 4) = acc;
            }

            // ---- rows too long for one group: every group of the wavefront takes a share of the entries
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) {
                unsigned long long pending = __ballot(is_long[rd] && tx == 0);
                while (pending) {
                    const int src_lane = __ffsll((long long)pending) - 1;
                    pending &= pending - 1;
                    const int lr = rd * RPR + src_lane / G;
                    const int ls = __shfl(rp, lr, kWave), le = __shfl(rp, lr + 1, kWave);
                    float4 acc = f4_zero();
                    int e = ls + grp;
                    for (; e + 3 * RPR < le; e += 4 * RPR) {
                        int c4[4];
                        float v4[4];
                        float4 xx[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) { c4[u] = col_idx[e + u * RPR]; v4[u] = val[e + u * RPR]; }
#pragma unroll
                        for (int u = 0; u < 4; ++u) xx[u] = *reinterpret_cast<const float4*>(h_in + (size_t)c4[u] * C + tx * 4);
#pragma unroll
                        for (int u = 0; u < 4; ++u) f4_fma(acc, v4[u], xx[u]);
                    }
                    for (; e < le; e += RPR)
                        f4_fma(acc, val[e], *reinterpret_cast<const float4*>(h_in + (size_t)col_idx[e] * C + tx * 4));
                    *reinterpret_cast<float4*>(red + grp * C + tx * 4) = acc;
                    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                    if (grp == 0) {
                        float4 sum = f4_zero();
                        for (int g = 0; g < RPR; ++g) {
                            const float4 p = *reinterpret_cast<const float4*>(red + g * C + tx * 4);
                            sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
                        }
                        *reinterpret_cast<float4*>(tile + lr * LDT + tx * 4) = sum;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        GNNHIP_PHASE_MARK(2);

        // ---- contraction: lane (q, t) supplies tile[t][KS q + s] at step s
        float areg[KS];
#pragma unroll
        for (int s4 = 0; s4 < KS / 4; ++s4) {
            const float4 a = *reinterpret_cast<const float4*>(tile + t * LDT + KS * q + 4 * s4);
            areg[4 * s4 + 0] = a.x; areg[4 * s4 + 1] = a.y; areg[4 * s4 + 2] = a.z; areg[4 * s4 + 3] = a.w;
        }
        GNNHIP_PHASE_MARK(3);
        mfma_f4 acc[NJB];
#pragma unroll
        for (int jb = 0; jb < NJB; ++jb) {
            acc[jb] = mfma_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; ++s)
                acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][s], areg[s], acc[jb], 0, 0, 0);
        }
        GNNHIP_PHASE_MARK(4);

        // ---- epilogue: lane owns row t, columns KS q + 4 jb + {0..3}
        const long long row = row0 + t;
        if (row < N) {
#pragma unroll
            for (int jb = 0; jb < NJB; ++jb) {
                const int cbase = KS * q + 4 * jb;
                const size_t off = (size_t)row * C + cbase;
                float4 v = make_float4(acc[jb][0], acc[jb][1], acc[jb][2], acc[jb][3]);
                if (bias) {
                    const float4 b4 = *reinterpret_cast<const float4*>(bias + cbase);
                    v.x += b4.x; v.y += b4.y; v.z += b4.z; v.w += b4.w;
                }
                v.x += mpre[jb].x; v.y += mpre[jb].y; v.z += mpre[jb].z; v.w += mpre[jb].w;
                *reinterpret_cast<float4*>(h_out + off) =
                    make_float4(relu_ref(v.x), relu_ref(v.y), relu_ref(v.z), relu_ref(v.w));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");     // the tile is rewritten by the next iteration
        GNNHIP_PHASE_MARK(5);
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
#pragma unroll 16
            for (int c = 0; c < C; ++c) s += pl[c] * Wh1[(size_t)c * H + j];
            s = relu_ref(s);
            hid[j] = s;
            hidden[(size_t)g * H + j] = s;
        }
        __syncthreads();
        // logits = hidden * W_h2
        for (int q = tid; q < Q; q += kBlock) {
            float s = 0.f;
#pragma unroll 8
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

// Mean entries per row from which the two-launch route is taken.
inline long long two_step_degree() { return (long long)kTwoStepMeanDegree; }

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

template <int C, bool DENSE>
int launch_level(int N, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                 const float* W, const float* msg, const float* bias, float* h_out, const HubPlan& hubs, hipStream_t s)
{
    constexpr int kWavesPerBlock = kBlock / kWave;
    const long long ntiles = ((long long)N + 15) / 16;
    long long blocks = (ntiles + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks > kNumCU * 8) blocks = kNumCU * 8;          // persistent beyond this
    hipLaunchKernelGGL((s2v_level_kernel<C, DENSE>), dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs.row_slot, hubs.agg, hubs.ld);
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
bool fused_hidden_supported(int C) { return C == 16 || C == 32 || C == 64 || C == 128 || C == 256; }

int input_dispatch(int N, int K, int C, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s)
{
    if (!(aligned16(Wn2l) && aligned16(msg) && aligned16(h0))) return GNNHIP_EUNSUPPORTED;      // h0 may be null
    const bool small = small_batch(N);
    switch (C) {
    case 16: return small ? launch_input<16, 1>(N, K, X, Wn2l, msg, h0, s) : launch_input<16, 4>(N, K, X, Wn2l, msg, h0, s);
    case 32: return small ? launch_input<32, 1>(N, K, X, Wn2l, msg, h0, s) : launch_input<32, 4>(N, K, X, Wn2l, msg, h0, s);
    case 64:
        // msg alone (the forward that does not store h0): the matrix-core kernel of the wide sizes is faster
        // (880,690 nodes, 38 label types: 77 against 109 us); with h0 its 64-byte pieces per row and
        // wavefront cost more than they gain (158 against 144 us)
        if (!h0 && K <= 64) return input_wide_dispatch(N, K, C, X, Wn2l, msg, h0, s);
        return small ? launch_input<64, 1>(N, K, X, Wn2l, msg, h0, s) : launch_input<64, 4>(N, K, X, Wn2l, msg, h0, s);
    case 128:
    case 256: return input_wide_dispatch(N, K, C, X, Wn2l, msg, h0, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

// Whether level_dispatch can read h_in as ReLU(h_in): then the forward does not store h0 = ReLU(msg) and the
// first level gathers from msg (one activation less written, and the gathered rows are the ones the level
// reads anyway).
bool level_accepts_relu_input(int N, int C, long long nnz)
{
    const bool two_step = N >= kHubMinRows && nnz >= two_step_degree() * (long long)N;
    if (two_step) return false;
    return level_wide_covers(N, C) || level_stream_covers(N, C);
}

// row_ptr[i] = i (i <= n), col_idx[i] = i, val[i] = 1: the n x n identity in CSR form
__global__ __launch_bounds__(kBlock) void identity_csr_kernel(int n, int* __restrict__ row_ptr, int* __restrict__ col_idx,
                                                              float* __restrict__ val)
{
    const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (i <= n) row_ptr[i] = (int)i;
    if (i < n) { col_idx[i] = (int)i; val[i] = 1.f; }
}

int level_dispatch(int N, int C, long long nnz, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                   const float* W, const float* msg, const float* bias, float* h_out, hipStream_t s, bool same_graph,
                   bool relu_in, CsrPlan* plan)
{
    // plan: made by gnnhip_csr_plan_create for exactly these CSR arrays (then nnz is the matrix's own count), or null
    // relu_in: h_in is read as ReLU(h_in); only where level_accepts_relu_input says so
    // same_graph: the previous call on this stream had the same A (a later level of one forward), so the
    // plan of the long-row pass is still in place and only its sums are redone
    if (!(aligned16(h_in) && aligned16(W) && aligned16(h_out) && (!msg || aligned16(msg)) && (!bias || aligned16(bias))))
        return GNNHIP_EUNSUPPORTED;
    if (C == 16 || C == 32 || C == 64) {
        // On power-law graphs the per-row gather of the fused kernel is latency-bound (a lane group walks
        // a row of 50..250 entries a few loads at a time, and such rows sit next to each other), while the
        // SpMM keeps far more gathers in flight.  Measured on R-MAT (4M rows, 16 entries per row): fused
        // 6.2 ms, SpMM into h_out + contraction in place 4.7 ms; on a uniform random graph of the same
        // density the fused kernel wins by 12 % (0.81 vs 0.91 ms per 1M rows).  The host only knows the
        // mean degree, and dense graphs in practice are the skewed ones, so large graphs with at least
        // kTwoStepMeanDegree entries per row take the two launches.
        const bool two_step = N >= kHubMinRows && nnz >= two_step_degree() * (long long)N;
        if (relu_in && (two_step || !level_stream_covers(N, C))) return GNNHIP_EUNSUPPORTED;
        if (two_step) {
            // the streaming kernel knows the rows without entries from row_ptr and takes them as zero without reading
            // them, so the product need not write them (on R-MAT more than half of the rows)
            const bool skip_empty = level_stream_covers(N, C);
            if (int rc = spmm_dispatch(N, N, C, nnz, 1.f, row_ptr, col_idx, val, h_in, C, 0.f, h_out, C, s, same_graph, skip_empty, plan)) return rc;
            const HubPlan none{nullptr, nullptr, 0};
            if (int rc = level_stream_dispatch(N, C, true, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, none, false, s);
                rc != GNNHIP_EUNSUPPORTED)
                return rc;
            switch (C) {
            case 16: return launch_level<16, true>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, none, s);
            case 32: return launch_level<32, true>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, none, s);
            default: return launch_level<64, true>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, none, s);
            }
        }
        HubPlan hubs{nullptr, nullptr, 0};
        if (int rc = hub_prepass(N, C, nnz, row_ptr, col_idx, val, h_in, C, s, &hubs, same_graph, relu_in, kHubThreshold, kHubChunk, -1,
                                 plan ? &plan->row_hub : nullptr))
            return rc;
        // activations of 4 GiB and more keep the kernel with 64-bit addressing below
        if (int rc = level_stream_dispatch(N, C, false, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, relu_in, s);
            rc != GNNHIP_EUNSUPPORTED)
            return rc;
        switch (C) {
        case 16: return launch_level<16, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
        case 32: return launch_level<32, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
        default: return launch_level<64, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
        }
    }
    if (!level_wide_covers(N, C)) return GNNHIP_EUNSUPPORTED;
    // The wide kernel sums a row of any length inside one wavefront.  Large graphs with many entries per row
    // (in practice the skewed ones, see above) take two steps: the SpMM, which balances long rows, leaves A * h_in
    // in scratch, and the wide kernel reads those rows through the identity matrix (one entry per row: its
    // gather becomes a plain read of the row, 12 bytes of indices against C * 4 of data) for the contraction
    // and the epilogue.
    if (N >= kHubMinRows && nnz >= two_step_degree() * (long long)N) {
        if (relu_in) return GNNHIP_EUNSUPPORTED;
        void *tmp = nullptr, *idp = nullptr;
        if (int rc = stream_scratch(s, sizeof(float) * (size_t)N * C, &tmp)) return rc;
        if (int rc = stream_scratch_slot(s, 5, sizeof(int) * (3 * (size_t)N + 1), &idp)) return rc;
        float* agg = static_cast<float*>(tmp);
        int* id_row_ptr = static_cast<int*>(idp);
        int* id_col = id_row_ptr + N + 1;
        float* id_val = reinterpret_cast<float*>(id_col + N);
        if (int rc = spmm_dispatch(N, N, C, nnz, 1.f, row_ptr, col_idx, val, h_in, C, 0.f, agg, C, s, same_graph, false, plan)) return rc;
        hipLaunchKernelGGL(identity_csr_kernel, dim3((unsigned)(((long long)N + kBlock) / kBlock)), dim3(kBlock), 0, s, N, id_row_ptr,
                           id_col, id_val);
        GNNHIP_LAUNCH_CHECK("identity_csr");
        return level_wide_dispatch(N, C, N, id_row_ptr, id_col, id_val, agg, W, msg, bias, h_out, false, s);
    }
    return level_wide_dispatch(N, C, nnz, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, relu_in, s);
}

// u = A' dz and g_prev = u W^T in one pass (A' = the transposed adjacency in CSR form); GNNHIP_EUNSUPPORTED where
// the caller has to take the SpMM and the GEMM.
int level_backward_dispatch(int N, int C, long long nnz, const int* row_ptr, const int* col_idx, const float* val, const float* dz,
                            const float* W, float* u, float* g_prev, const float* gate, float* acc, hipStream_t s)
{
    if (C == 128 || C == 256) {
        // hidden 128 / 256: the wide kernel's backward variant, except where the forward takes two steps too (large
        // graphs with many entries per row: the wide kernel sums a row of any length inside one wavefront)
        if (!level_wide_covers(N, C)) return GNNHIP_EUNSUPPORTED;
        if (N >= kHubMinRows && nnz >= two_step_degree() * (long long)N) return GNNHIP_EUNSUPPORTED;
        if (!(aligned16(dz) && aligned16(W) && aligned16(u) && aligned16(g_prev) && (!gate || aligned16(gate)) && (!acc || aligned16(acc))))
            return GNNHIP_EUNSUPPORTED;
        return level_wide_backward_dispatch(N, C, row_ptr, col_idx, val, dz, W, u, g_prev, gate, acc, s);
    }
    if (!(C == 16 || C == 32 || C == 64) || !level_stream_covers(N, C)) return GNNHIP_EUNSUPPORTED;
    if (!(aligned16(dz) && aligned16(W) && aligned16(u) && aligned16(g_prev) && (!gate || aligned16(gate)) && (!acc || aligned16(acc))))
        return GNNHIP_EUNSUPPORTED;
    if (N >= kHubMinRows && nnz >= two_step_degree() * (long long)N) return GNNHIP_EUNSUPPORTED;     // dense and skewed: balanced SpMM
    HubPlan hubs{nullptr, nullptr, 0};
    if (int rc = hub_prepass(N, C, nnz, row_ptr, col_idx, val, dz, C, s, &hubs, false, false)) return rc;
    return level_stream_backward_dispatch(N, C, row_ptr, col_idx, val, dz, W, u, g_prev, gate, acc, hubs, s);
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
    case 128: return launch_readout<128>(B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    case 256: return launch_readout<256>(B, H, Q, s_row_ptr, s_col_idx, s_val, h, Wh1, Wh2, pool, hidden, logits, probs, pred, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

}  // namespace gnnhip
