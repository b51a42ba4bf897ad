// Input stage for hidden sizes 128 and 256 (and 64 when only msg is wanted) and up to 64 label types:
//     msg = X * W_n2l ,  h0 = ReLU(msg)
// MatMul + ReLU of examples/graph_classification/src/kernel_mean_field.cpp:31-32 in one pass,
// with the K x C contraction on the FP32 matrix cores.
//
// A workgroup of four wavefronts takes 64 rows of X at a time into LDS (zero-padded to a
// multiple of four columns); wavefront w owns the output columns [w C/4, (w+1) C/4) and keeps
// its slice of W_n2l^T in registers for the whole launch.  Operand roles are swapped
// (out^T = W^T * X^T) so that a lane ends up with four consecutive output columns of one row:
// 128-bit stores of msg and of h0.  msg and h0 are addressed through buffer descriptors that
// cover the rows of the current tile only, so rows past N need no predicate.
//
// Algorithmic bytes: 4 N (K + 2 C) + 4 K C; flops 2 N K C.  HBM-bound (the two outputs).
#include "gnnhip_internal.h"
#include "buffer_addr.h"

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;       // 4
constexpr int kTileRows = 64;

// KS = contraction steps of four: K <= 4 KS.
template <int C, int KS>
__global__ __launch_bounds__(kBlock) void s2v_input_wide_kernel(
    int N, int K, unsigned k_magic, int x_vec, const float* __restrict__ X, const float* __restrict__ Wn2l,
    float* __restrict__ msg, float* __restrict__ h0)
{
    constexpr int CW = C / kWaves;           // output columns per wavefront
    constexpr int NB = CW / 16;              // 16-column blocks per wavefront
    constexpr int LDT = 4 * KS + 4;          // LDS row stride
    __shared__ float xt[kTileRows * LDT];

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int q = lane >> 4, t = lane & 15;
    const int col0 = wave * CW;

    // W^T operand: wreg[jb][s] = W_n2l[KS q + s][col0 + 16 jb + t], zero past K
    float wreg[NB][KS];
#pragma unroll
    for (int jb = 0; jb < NB; ++jb)
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const int k = KS * q + s;
            wreg[jb][s] = (k < K) ? Wn2l[(size_t)k * C + col0 + 16 * jb + t] : 0.f;
        }

    const int lane_off = (t * C + col0 + 4 * q) * 4;      // byte offset of this lane inside a 16-row block
    const int ntiles = (int)(((long long)N + kTileRows - 1) / kTileRows);
    // X rows of a tile, asked for before the contraction of the previous tile.  A full tile is 64 K
    // contiguous floats: with x_vec set (X 16-byte aligned) the workgroup reads them as KS/4 128-bit words per
    // lane and scatters them into the padded LDS rows (row = element / K by one multiply-high with
    // ceil(2^32 / K)); the last, partial tile and unaligned X go row by row: wavefront w copies rows
    // 16 w .. 16 w + 15, one row per load.
    constexpr int XQ = KS / 4;
    float xv[16];
    float4 xq[XQ];
    for (int i = threadIdx.x; i < kTileRows * LDT; i += kBlock) xt[i] = 0.f;      // the padding columns stay zero
    auto full_tile = [&](int tile) { return x_vec && (long long)(tile + 1) * kTileRows <= (long long)N; };
    auto load_x = [&](int tile) {
        if (full_tile(tile)) {
            const float4* xg = reinterpret_cast<const float4*>(X + (size_t)tile * kTileRows * K);
#pragma unroll
            for (int p = 0; p < XQ; ++p) {
                const int f = threadIdx.x + p * kBlock;
                xq[p] = (f * 4 < kTileRows * K) ? xg[f] : f4_zero();
            }
        } else {
            const long long r0 = (long long)tile * kTileRows + wave * 16;
#pragma unroll
            for (int rr = 0; rr < 16; ++rr)
                xv[rr] = (lane < K && r0 + rr < N) ? X[(size_t)(r0 + rr) * K + lane] : 0.f;
        }
    };
    auto park_x = [&](int tile) {
        if (full_tile(tile)) {
#pragma unroll
            for (int p = 0; p < XQ; ++p) {
                const int e = (threadIdx.x + p * kBlock) * 4;
                if (e < kTileRows * K) {
                    int r = K >= 2 ? (int)__umulhi((unsigned)e, k_magic) : e;
                    int c = e - r * K;
                    const float v[4] = {xq[p].x, xq[p].y, xq[p].z, xq[p].w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        xt[r * LDT + c] = v[i];           // 64 K is a multiple of 4: the four elements exist
                        if (++c == K) { c = 0; ++r; }
                    }
                }
            }
        } else {
#pragma unroll
            for (int rr = 0; rr < 16; ++rr)
                if (lane < 4 * KS) xt[(wave * 16 + rr) * LDT + lane] = xv[rr];
        }
    };
    if ((int)blockIdx.x < ntiles) load_x(blockIdx.x);
    for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const long long row0 = (long long)tile * kTileRows;
        const long long left = (long long)N - row0;
        const int rows = (int)(left < kTileRows ? left : kTileRows);
        __syncthreads();                     // the previous tile has been consumed (first pass: the zero fill is done)
        park_x(tile);
        __syncthreads();
        if (tile + (int)gridDim.x < ntiles) load_x(tile + gridDim.x);

        const unsigned bytes = (unsigned)rows * (C * 4);
        const rsrc_t msg_rsrc = make_rsrc(msg + (size_t)row0 * C, bytes);
        const rsrc_t h0_rsrc = make_rsrc(h0 ? h0 + (size_t)row0 * C : nullptr, h0 ? bytes : 0u);      // h0 may be null
#pragma unroll 1
        for (int rt = 0; rt < kTileRows / 16; ++rt) {
            if (rt * 16 >= rows) break;
            mfma_f4 acc[NB];
#pragma unroll
            for (int jb = 0; jb < NB; ++jb) acc[jb] = mfma_f4{0.f, 0.f, 0.f, 0.f};
            const float* src = xt + (rt * 16 + t) * LDT + KS * q;
#pragma unroll
            for (int s4 = 0; s4 < KS / 4; ++s4) {
                const float4 b = *reinterpret_cast<const float4*>(src + 4 * s4);
#pragma unroll
                for (int jb = 0; jb < NB; ++jb) acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][4 * s4 + 0], b.x, acc[jb], 0, 0, 0);
#pragma unroll
                for (int jb = 0; jb < NB; ++jb) acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][4 * s4 + 1], b.y, acc[jb], 0, 0, 0);
#pragma unroll
                for (int jb = 0; jb < NB; ++jb) acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][4 * s4 + 2], b.z, acc[jb], 0, 0, 0);
#pragma unroll
                for (int jb = 0; jb < NB; ++jb) acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][4 * s4 + 3], b.w, acc[jb], 0, 0, 0);
            }
            const int voff = lane_off + rt * (16 * C * 4);
#pragma unroll
            for (int jb = 0; jb < NB; ++jb) {
                const float4 v = make_float4(acc[jb][0], acc[jb][1], acc[jb][2], acc[jb][3]);
                buf_store4(msg_rsrc, voff + 64 * jb, 0, v);
                if (h0) buf_store4(h0_rsrc, voff + 64 * jb, 0, relu_ref4(v));
            }
        }
    }
}

template <int C, int KS>
int launch_input_wide(int N, int K, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s)
{
    const long long ntiles = ((long long)N + kTileRows - 1) / kTileRows;
    const long long cap = (long long)kNumCU * 4;
    const unsigned grid = (unsigned)(ntiles < cap ? ntiles : cap);
    const unsigned k_magic = K >= 2 ? (unsigned)((0x100000000ull + (unsigned)K - 1) / (unsigned)K) : 0u;   // ceil(2^32 / K)
    const int x_vec = aligned16(X) ? 1 : 0;
    hipLaunchKernelGGL((s2v_input_wide_kernel<C, KS>), dim3(grid), dim3(kBlock), 0, s, N, K, k_magic, x_vec, X, Wn2l, msg, h0);
    GNNHIP_LAUNCH_CHECK("s2v_input_wide");
    return GNNHIP_OK;
}

template <int C>
int input_wide_c(int N, int K, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s)
{
    if (K <= 16) return launch_input_wide<C, 4>(N, K, X, Wn2l, msg, h0, s);
    if (K <= 32) return launch_input_wide<C, 8>(N, K, X, Wn2l, msg, h0, s);
    if (K <= 48) return launch_input_wide<C, 12>(N, K, X, Wn2l, msg, h0, s);
    return launch_input_wide<C, 16>(N, K, X, Wn2l, msg, h0, s);
}

}  // namespace

int input_wide_dispatch(int N, int K, int C, const float* X, const float* Wn2l, float* msg, float* h0, hipStream_t s)
{
    if (K > 64 || !(aligned16(msg) && aligned16(h0))) return GNNHIP_EUNSUPPORTED;
    switch (C) {
    case 64: return input_wide_c<64>(N, K, X, Wn2l, msg, h0, s);
    case 128: return input_wide_c<128>(N, K, X, Wn2l, msg, h0, s);
    case 256: return input_wide_c<256>(N, K, X, Wn2l, msg, h0, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

}  // namespace gnnhip
