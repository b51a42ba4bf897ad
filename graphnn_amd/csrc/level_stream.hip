// Fused structure2vec level for hidden sizes 16, 32 and 64 on graphs whose activations fit a
// 4 GiB buffer (N * C * 4 < 2^32):
//     h_out = ReLU((A * h_in) * W + bias + msg)
// (MatMul(sparse) -> MatMul -> ElewiseAdd -> ReLU of
// examples/graph_classification/src/kernel_mean_field.cpp:37-44 in one pass).
//
// Each wavefront owns tiles of 16 rows and never synchronises with another wavefront.  What a
// tile needs from the CSR arrays is asked for ahead of time, so that the only memory trip a
// tile waits for is the gather itself:
//     two tiles ahead   the row pointers of the lane group's rows,
//     one tile ahead    the first G column indices and weights of each row,
//     this tile         msg, then the first four neighbours of all 16 rows in one go.
// Every memory instruction of the steady state is unconditional: h_in, msg, h_out and row_ptr
// are addressed through buffer descriptors, and a lane with nothing to fetch uses an offset
// past the end, which returns zeros without a memory access.  The instruction counts are
// therefore fixed and the waits can let younger requests stay in flight.  Rows with more than
// four entries, and rows too long for one lane group, are finished in wave-uniform branches
// that molecule batches never take.
//
// Per tile: G = C/4 lanes form a group; the 64/G groups take 16/(64/G) consecutive rows each.
//   1. gather-sum into a wave-private LDS tile [16][C+4];
//   2. contraction on the matrix cores: out^T = W^T * tile^T with v_mfma_f32_16x16x4_f32.
//      Lane (q = lane/16, t = lane%16) feeds k = (C/4) q + s at step s and ends up owning
//      row t, columns (C/4) q .. (C/4) q + C/4 - 1;
//   3. epilogue: + bias + msg, ReLU, 128-bit stores.
// W^T is held in registers, or (WLDS) in LDS in the order the lanes consume it, which halves
// the register count and doubles the wavefronts per SIMD.
//
// DENSE: A * h_in has already been written to h_out (by the SpMM); the tile is read from there
// and overwritten in place.  Rows of A without entries (known from row_ptr) are taken as zero and not read, so the
// product may leave them unwritten.
//
// Algorithmic bytes: 4(N+1) + 8E + 12NC + 4C^2.
#include "gnnhip_internal.h"
#include "buffer_addr.h"

// Hooks of a timing build of this file; they expand to nothing in the library.
#ifndef GNNHIP_PHASE_ACC
#define GNNHIP_PHASE_ACC(i)
#define GNNHIP_PHASE_INIT
#define GNNHIP_PHASE_FINI
#endif

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
constexpr int kPipeMinRows = 65536;   // from here on the kernel variant that asks for a tile's gathers one tile early
constexpr int kWaveLongRow = 48;     // entries; longer rows are gathered by all groups of the wavefront together,
                                     // and past kHubThreshold they come from the pre-pass when there is one

// Value of lane U of the caller's lane group.  For groups of 16 and of 4 lanes this is a DPP
// operand modifier that the compiler folds into the instruction that consumes the value.
template <int G, int U>
__device__ __forceinline__ int group_lane(int v)
{
    if constexpr (G == 16) return __builtin_amdgcn_mov_dpp(v, 0x150 + U, 0xF, 0xF, true);          // row_newbcast:U
    else if constexpr (G == 4) return __builtin_amdgcn_mov_dpp(v, U * 0x55, 0xF, 0xF, true);        // quad_perm:[U,U,U,U]
    else return __shfl(v, U, G);
}
template <int G, int U>
__device__ __forceinline__ float group_lane(float v)
{
    return __int_as_float(group_lane<G, U>(__float_as_int(v)));
}

// x[u] = h_in[entry U0 + u of the lane group's row], u = 0..3: offs holds, per lane of the group, the byte
// offset of the entry's row of h_in (past the end where the row has no such entry: the load reads zeros)
template <int G, int U0>
__device__ __forceinline__ void gather4(rsrc_t h_rsrc, int offs, int tx_off, float4 (&x)[4])
{
    x[0] = buf_load4(h_rsrc, group_lane<G, U0 + 0>(offs) + tx_off, 0);
    x[1] = buf_load4(h_rsrc, group_lane<G, U0 + 1>(offs) + tx_off, 0);
    x[2] = buf_load4(h_rsrc, group_lane<G, U0 + 2>(offs) + tx_off, 0);
    x[3] = buf_load4(h_rsrc, group_lane<G, U0 + 3>(offs) + tx_off, 0);
}
// RELU_IN: the gathered rows count as ReLU(row) (the first level reading msg where h0 was not stored)
template <bool RELU_IN>
__device__ __forceinline__ float4 as_input(const float4& x)
{
    return RELU_IN ? relu_ref4(x) : x;
}
template <int G, int U0, bool RELU_IN>
__device__ __forceinline__ void sum4(float4& acc, float w, const float4 (&x)[4])
{
    f4_fma(acc, group_lane<G, U0 + 0>(w), as_input<RELU_IN>(x[0]));
    f4_fma(acc, group_lane<G, U0 + 1>(w), as_input<RELU_IN>(x[1]));
    f4_fma(acc, group_lane<G, U0 + 2>(w), as_input<RELU_IN>(x[2]));
    f4_fma(acc, group_lane<G, U0 + 3>(w), as_input<RELU_IN>(x[3]));
}

// MINW: wavefronts per SIMD the register allocation must leave room for
// BWD: the backward pass of a level through the same machinery, out = (A' x) W^T with A' = A^T handed in as a
// CSR matrix: W is read transposed, the aggregated rows A' x are also stored (agg_out: they are the other
// factor of the weight gradient).  No ReLU and no bias; `msg`, when given, is the embedding whose ReLU the
// gradient passes next: out = out where msg > 0, else 0, and acc_io (when given) += out.
template <int C, bool DENSE, bool WLDS, int MINW, bool RELU_IN, bool PIPE, bool BWD = false>
__global__ __launch_bounds__(kBlock, MINW) void s2v_level_stream_kernel(
    int N, const int* __restrict__ row_ptr, const int* __restrict__ col_idx, const float* __restrict__ val,
    const float* __restrict__ h_in, const float* __restrict__ W, const float* __restrict__ msg,
    const float* __restrict__ bias, float* __restrict__ h_out,
    const int* __restrict__ hub_slot, const float* __restrict__ hub_agg, int hub_ld, float* __restrict__ agg_out = nullptr,
    float* __restrict__ acc_io = nullptr)
{
    constexpr int G = C / 4;             // lanes per gathered row
    constexpr int RPR = kWave / G;       // lane groups per wavefront
    constexpr int ROUNDS = 16 / RPR;     // rows per lane group
    constexpr int RN = ROUNDS + 1;       // row pointers per lane group
    constexpr int KS = C / 4;            // contraction steps
    constexpr int NJB = C / 16;          // 16-column output blocks
    constexpr int LDT = C + 4;
    constexpr int kRowBytes = C * 4;
    constexpr int kPastEndRow = (int)(0xFFFFFFFFu / kRowBytes * kRowBytes);   // row offset no activation buffer reaches
    constexpr int kBufEntries = (1 << 30) - 1;                                // entries of col_idx / val a buffer covers
    constexpr int kDirect = G >= 8 ? 8 : 4;                                   // entries per row taken without a loop

    __shared__ float lds[kWavesPerBlock][16 * LDT + RPR * C];
    __shared__ float4 wl[WLDS ? NJB * (KS / 4) * kWave : 1];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    float* tile = lds[wave];             // [16][LDT]
    float* red = tile + 16 * LDT;        // [RPR][C]
    const int q = lane >> 4, t = lane & 15;
    const int grp = lane / G, tx = lane % G;
    const int tx_off = tx * 16;

    // W^T operand: wreg[jb][s] = W[KS q + s][KS (t/4) + 4 jb + t%4]
    float wreg[WLDS ? 1 : NJB][WLDS ? 1 : KS];
    if constexpr (WLDS) {
        // wavefront w lays down the blocks jb = w, w + 4, ...: entry (jb, s4, lane) holds the lane's four
        // operands of steps 4 s4 .. 4 s4 + 3
        for (int jb = wave; jb < NJB; jb += kWavesPerBlock)
#pragma unroll
            for (int s4 = 0; s4 < KS / 4; ++s4) {
                float4 w4;
                const int col = KS * (t >> 2) + 4 * jb + (t & 3);
                const int k0 = KS * q + 4 * s4;
                // element (k, col) of the operand: W[k][col], or W[col][k] when the level runs backward
                if constexpr (BWD) {
                    w4 = *reinterpret_cast<const float4*>(W + (size_t)col * C + k0);     // four steps: consecutive floats of a row (W is 16-byte aligned, host-checked)
                } else {
                    w4.x = W[(size_t)(k0 + 0) * C + col];
                    w4.y = W[(size_t)(k0 + 1) * C + col];
                    w4.z = W[(size_t)(k0 + 2) * C + col];
                    w4.w = W[(size_t)(k0 + 3) * C + col];
                }
                wl[(jb * (KS / 4) + s4) * kWave + lane] = w4;
            }
        __syncthreads();
    } else {
#pragma unroll
        for (int jb = 0; jb < NJB; ++jb) {
            if constexpr (BWD) {
#pragma unroll
                for (int s4 = 0; s4 < KS / 4; ++s4) {
                    const float4 v = *reinterpret_cast<const float4*>(W + (size_t)(KS * (t >> 2) + 4 * jb + (t & 3)) * C + KS * q + 4 * s4);
                    wreg[jb][4 * s4 + 0] = v.x; wreg[jb][4 * s4 + 1] = v.y; wreg[jb][4 * s4 + 2] = v.z; wreg[jb][4 * s4 + 3] = v.w;
                }
            } else {
#pragma unroll
                for (int s = 0; s < KS; ++s) wreg[jb][s] = W[(size_t)(KS * q + s) * C + KS * (t >> 2) + 4 * jb + (t & 3)];
            }
        }
    }

    int E = 0;
    if (!DENSE) E = row_ptr[N];
    const unsigned act_bytes = (unsigned)N * (unsigned)kRowBytes;
    const unsigned csr_bytes = (unsigned)(E < kBufEntries ? E : kBufEntries) * 4u;
    const rsrc_t rp_rsrc = make_rsrc(row_ptr, (unsigned)(N + 1) * 4u);
    const rsrc_t ci_rsrc = make_rsrc(col_idx, csr_bytes);
    const rsrc_t val_rsrc = make_rsrc(val, csr_bytes);
    const rsrc_t h_rsrc = make_rsrc(h_in, act_bytes);
    const rsrc_t msg_rsrc = make_rsrc(msg, msg ? act_bytes : 0u);      // no msg: every load reads 0
    const rsrc_t out_rsrc = make_rsrc(h_out, act_bytes);

    float4 bias4 = f4_zero();                // columns 4 tx .. 4 tx + 3
    if (bias) bias4 = *reinterpret_cast<const float4*>(bias + tx * 4);

    // byte offset of columns 4 tx .. 4 tx + 3 of row r of an activation matrix
    auto row_off = [&](int r) -> int { return (int)((unsigned)r * (unsigned)kRowBytes + (unsigned)tx_off); };

    const int ntiles = (N + 15) / 16;
    const int nwaves = (int)gridDim.x * kWavesPerBlock;
    const int tile_first = (int)blockIdx.x * kWavesPerBlock + wave;

    // Row pointers of the rows grp * ROUNDS .. grp * ROUNDS + ROUNDS of a tile.  Past row N they read 0,
    // which makes those rows empty (their entry counts are not positive).  The whole offset sits in the
    // lane's register: only that part is compared with the buffer size.
    auto load_rp = [&](int (&rpx)[RN], int tile_id) {
#pragma unroll
        for (int i = 0; i < RN; ++i) rpx[i] = buf_load_i(rp_rsrc, (tile_id * 16 + grp * ROUNDS + i) * 4, 0);
    };
    // First batch of a row: lane tx takes entry tx.  offs = byte offset of the entry's row of h_in, w = its
    // weight; lanes past the end of the row, and all lanes of a row that is gathered cooperatively (too
    // long, or out of the buffer's reach), hold an offset past the end and weight 0.
    auto load_first_batch = [&](const int (&rpx)[RN], int (&offs)[ROUNDS], float (&w)[ROUNDS]) {
#pragma unroll
        for (int rd = 0; rd < ROUNDS; ++rd) {
            const int cnt = rpx[rd + 1] - rpx[rd];
            const bool direct = cnt <= kWaveLongRow && rpx[rd + 1] <= kBufEntries;
            const bool ok = direct && tx < cnt;
            const int voff = ok ? (rpx[rd] + tx) * 4 : kBufPastEnd;
            const int c = DENSE ? 0 : buf_load_i(ci_rsrc, voff, 0);
            w[rd] = DENSE ? 0.f : buf_load_f(val_rsrc, voff, 0);
            offs[rd] = ok ? (int)((unsigned)c * (unsigned)kRowBytes) : kPastEndRow;
        }
    };

    int rp[RN], rpn[RN], offs[ROUNDS];
    float w0[ROUNDS];
    int tile_id = tile_first, tile_n1 = tile_first + nwaves, tile_n2 = tile_first + 2 * nwaves;
    load_rp(rp, tile_id < ntiles ? tile_id : ntiles);
    load_rp(rpn, tile_n1 < ntiles ? tile_n1 : ntiles);
    load_first_batch(rp, offs, w0);
    // PIPE: the gathers of a tile are issued one tile earlier, before the contraction of the tile in hand, so
    // that they travel while the matrix cores work; the look-ahead of the CSR data is one tile deeper for it
    int rpq[PIPE ? RN : 1], offq[PIPE ? ROUNDS : 1];
    float wq[PIPE ? ROUNDS : 1];
    float4 x[ROUNDS][4];                     // gathered rows: four entries of each of the lane group's rows
    if constexpr (PIPE && !DENSE) {
        load_rp(rpq, tile_n2 < ntiles ? tile_n2 : ntiles);
        load_first_batch(rpn, offq, wq);
#pragma unroll
        for (int rd = 0; rd < ROUNDS; ++rd) gather4<G, 0>(h_rsrc, offs[rd], tx_off, x[rd]);
    }

    GNNHIP_PHASE_INIT
    while (tile_id < ntiles) {
        GNNHIP_PHASE_ACC(0);
        const int row0 = tile_id * 16;
        // msg is read, and h_out written, one row per lane group: every instruction covers whole rows.
        // Rows past N are out of range.
        const int out_off = row_off(row0 + grp * ROUNDS);
        int rpnn[RN], offsn[ROUNDS];             // look-ahead requests of this iteration
        float w0n[ROUNDS];

        if constexpr (DENSE) {
            // a row of A without entries was not written by the product: it counts as zero and is not read (an
            // offset past the end returns zeros without a memory access)
            float4 xd[ROUNDS];
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd)
                xd[rd] = buf_load4(out_rsrc, rp[rd + 1] > rp[rd] ? row_off(row0 + grp * ROUNDS + rd) : kPastEndRow, 0);
            load_rp(rpnn, tile_n2 < ntiles ? tile_n2 : ntiles);      // behind the rows: the pointers of the tile after next
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd)
                *reinterpret_cast<float4*>(tile + (grp * ROUNDS + rd) * LDT + tx * 4) = xd[rd];
#pragma unroll
            for (int i = 0; i < RN; ++i) { rp[i] = rpn[i]; rpn[i] = rpnn[i]; }
        } else {
            // ---- the first four neighbours of every row of the tile, fetched together
            if constexpr (!PIPE) {
#pragma unroll
                for (int rd = 0; rd < ROUNDS; ++rd) gather4<G, 0>(h_rsrc, offs[rd], tx_off, x[rd]);
                // ---- behind the gathers: the next tile's first batch, and the row pointers of the tile after it
                load_rp(rpnn, tile_n2 < ntiles ? tile_n2 : ntiles);   // tile ntiles: every pointer reads 0 or row_ptr[N]
                load_first_batch(rpn, offsn, w0n);
            }                                    // PIPE: x was asked for during the previous tile
            // longest row of the lane group, and whether one of its rows is out of the buffer's reach
            int longest = rp[1] - rp[0];
#pragma unroll
            for (int rd = 1; rd < ROUNDS; ++rd) longest = max(longest, rp[rd + 1] - rp[rd]);
            const bool far = rp[ROUNDS] > kBufEntries;
            GNNHIP_PHASE_ACC(1);
            // ---- sums
            float4 acc[ROUNDS];
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) {
                acc[rd] = f4_zero();
                sum4<G, 0, RELU_IN>(acc[rd], w0[rd], x[rd]);
            }
            GNNHIP_PHASE_ACC(2);
            if (__any(longest > 4 || far)) {
                if constexpr (kDirect == 8) {
                    // entries 4..7 the same way
#pragma unroll
                    for (int rd = 0; rd < ROUNDS; ++rd) gather4<G, 4>(h_rsrc, offs[rd], tx_off, x[rd]);
#pragma unroll
                    for (int rd = 0; rd < ROUNDS; ++rd) sum4<G, 4, RELU_IN>(acc[rd], w0[rd], x[rd]);
                }
                if (__any(longest > kDirect || far)) {
                    // the rest of the first batch, then further batches of G
#pragma unroll
                    for (int rd = 0; rd < ROUNDS; ++rd) {
                        const int st = rp[rd];
                        int en = rp[rd + 1];
                        if (en - st > kWaveLongRow || en > kBufEntries) en = st;
                        for (int base = st; base < en; base += G) {
                            int c = 0;
                            float v = 0.f;
                            if (base + tx < en) { c = col_idx[base + tx]; v = val[base + tx]; }
                            const int cnt = min(G, en - base);
                            for (int j = (base == st) ? (kDirect < G ? kDirect : G) : 0; j < cnt; j += 4) {
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
                                    xx[u] = buf_load4(h_rsrc, (j + u < cnt) ? row_off(cj[u]) : kBufPastEnd, 0);
#pragma unroll
                                for (int u = 0; u < 4; ++u)
                                    if (j + u < cnt) f4_fma(acc[rd], vj[u], as_input<RELU_IN>(xx[u]));
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd)
                *reinterpret_cast<float4*>(tile + (grp * ROUNDS + rd) * LDT + tx * 4) = acc[rd];

            if (__any(longest > kWaveLongRow || far)) {
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
#pragma unroll
                for (int rd = 0; rd < ROUNDS; ++rd) {
                    const int lr = grp * ROUNDS + rd;
                    const int cnt = rp[rd + 1] - rp[rd];
                    bool coop = cnt > kWaveLongRow || (rp[rd + 1] > kBufEntries && cnt > 0);
                    if (coop && hub_slot && cnt > kHubThreshold) {
                        const int slot = hub_slot[row0 + lr];          // summed by the pre-pass unless -1
                        if (slot >= 0) {
                            *reinterpret_cast<float4*>(tile + lr * LDT + tx * 4) =
                                *reinterpret_cast<const float4*>(hub_agg + (size_t)slot * hub_ld + tx * 4);
                            coop = false;
                        }
                    }
                    // every group of the wavefront takes a share of the entries of each remaining long row
                    unsigned long long pending = __ballot(coop && tx == 0);
                    while (pending) {
                        const int src_lane = __ffsll((long long)pending) - 1;
                        pending &= pending - 1;
                        const int dst = (src_lane / G) * ROUNDS + rd;
                        const int ls = __shfl(rp[rd], src_lane, kWave), le = __shfl(rp[rd + 1], src_lane, kWave);
                        float4 a = f4_zero();
                        int e = ls + grp;
                        for (; e + 3 * RPR < le; e += 4 * RPR) {
                            int c4[4];
                            float v4[4];
                            float4 xx[4];
#pragma unroll
                            for (int u = 0; u < 4; ++u) { c4[u] = col_idx[e + u * RPR]; v4[u] = val[e + u * RPR]; }
#pragma unroll
                            for (int u = 0; u < 4; ++u) xx[u] = buf_load4(h_rsrc, row_off(c4[u]), 0);
#pragma unroll
                            for (int u = 0; u < 4; ++u) f4_fma(a, v4[u], as_input<RELU_IN>(xx[u]));
                        }
                        for (; e < le; e += RPR) f4_fma(a, val[e], as_input<RELU_IN>(buf_load4(h_rsrc, row_off(col_idx[e]), 0)));
                        *reinterpret_cast<float4*>(red + grp * C + tx * 4) = a;
                        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                        if (grp == 0) {
                            float4 sum = f4_zero();
                            for (int g = 0; g < RPR; ++g) {
                                const float4 p = *reinterpret_cast<const float4*>(red + g * C + tx * 4);
                                sum.x += p.x; sum.y += p.y; sum.z += p.z; sum.w += p.w;
                            }
                            *reinterpret_cast<float4*>(tile + dst * LDT + tx * 4) = sum;
                        }
                        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                    }
                }
            }
            if constexpr (!PIPE) {
                // rotate the look-ahead
#pragma unroll
                for (int i = 0; i < RN; ++i) { rp[i] = rpn[i]; rpn[i] = rpnn[i]; }
#pragma unroll
                for (int rd = 0; rd < ROUNDS; ++rd) { offs[rd] = offsn[rd]; w0[rd] = w0n[rd]; }
            } else {
                // the next tile's gathers, the first batch of the tile after it, the row pointers of the third
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
#pragma unroll
                for (int rd = 0; rd < ROUNDS; ++rd) gather4<G, 0>(h_rsrc, offq[rd], tx_off, x[rd]);
                const int tile_n3 = tile_n2 + nwaves;
                load_rp(rpnn, tile_n3 < ntiles ? tile_n3 : ntiles);
                load_first_batch(rpq, offsn, w0n);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        GNNHIP_PHASE_ACC(3);
        if constexpr (BWD) {
            // the aggregated rows, as the lane groups hold them: whole 4 C-byte rows
            const rsrc_t agg_rsrc = make_rsrc(agg_out, act_bytes);
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd)
                buf_store4(agg_rsrc, out_off + rd * kRowBytes, 0, *reinterpret_cast<const float4*>(tile + (grp * ROUNDS + rd) * LDT + tx * 4));
        }
        // msg is asked for once the gathered rows have left their registers; the contraction covers its trip
        float4 mrow[ROUNDS];
#pragma unroll
        for (int rd = 0; rd < ROUNDS; ++rd) mrow[rd] = buf_load4(msg_rsrc, out_off + rd * kRowBytes, 0);

        // ---- contraction: lane (q, t) supplies tile[t][KS q + s] at step s
        float areg[KS];
#pragma unroll
        for (int s4 = 0; s4 < KS / 4; ++s4) {
            const float4 a = *reinterpret_cast<const float4*>(tile + t * LDT + KS * q + 4 * s4);
            areg[4 * s4 + 0] = a.x; areg[4 * s4 + 1] = a.y; areg[4 * s4 + 2] = a.z; areg[4 * s4 + 3] = a.w;
        }
        mfma_f4 acc[NJB];
#pragma unroll
        for (int jb = 0; jb < NJB; ++jb) {
            acc[jb] = mfma_f4{0.f, 0.f, 0.f, 0.f};
            if constexpr (WLDS) {
#pragma unroll
                for (int s4 = 0; s4 < KS / 4; ++s4) {
                    const float4 w4 = wl[(jb * (KS / 4) + s4) * kWave + lane];
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(w4.x, areg[4 * s4 + 0], acc[jb], 0, 0, 0);
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(w4.y, areg[4 * s4 + 1], acc[jb], 0, 0, 0);
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(w4.z, areg[4 * s4 + 2], acc[jb], 0, 0, 0);
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(w4.w, areg[4 * s4 + 3], acc[jb], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int s = 0; s < KS; ++s)
                    acc[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][s], areg[s], acc[jb], 0, 0, 0);
            }
        }

        GNNHIP_PHASE_ACC(4);
        // ---- epilogue: the lane owns row t, columns KS q + 4 jb + {0..3}; the tile goes back through LDS so
        // that the lane group of a row holds it contiguously (256-byte requests instead of 16-byte pieces)
#pragma unroll
        for (int jb = 0; jb < NJB; ++jb)
            *reinterpret_cast<float4*>(tile + t * LDT + KS * q + 4 * jb) = make_float4(acc[jb][0], acc[jb][1], acc[jb][2], acc[jb][3]);
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
#pragma unroll
        for (int rd = 0; rd < ROUNDS; ++rd) {
            float4 v = *reinterpret_cast<const float4*>(tile + (grp * ROUNDS + rd) * LDT + tx * 4);
            if constexpr (BWD) {
                if (msg) {
                    v.x = mrow[rd].x > 0.f ? v.x : 0.f; v.y = mrow[rd].y > 0.f ? v.y : 0.f;
                    v.z = mrow[rd].z > 0.f ? v.z : 0.f; v.w = mrow[rd].w > 0.f ? v.w : 0.f;
                }
                if (acc_io) {
                    // every row belongs to one tile: nobody else touches it during the launch
                    const rsrc_t acc_rsrc = make_rsrc(acc_io, act_bytes);
                    float4 a = buf_load4(acc_rsrc, out_off + rd * kRowBytes, 0);
                    a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
                    buf_store4(acc_rsrc, out_off + rd * kRowBytes, 0, a);
                }
                buf_store4(out_rsrc, out_off + rd * kRowBytes, 0, v);
            } else {
                if (bias) { v.x += bias4.x; v.y += bias4.y; v.z += bias4.z; v.w += bias4.w; }
                v.x += mrow[rd].x; v.y += mrow[rd].y; v.z += mrow[rd].z; v.w += mrow[rd].w;
                buf_store4(out_rsrc, out_off + rd * kRowBytes, 0, relu_ref4(v));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");     // the tile is rewritten by the next iteration
        if constexpr (PIPE && !DENSE) {
            // by now the look-ahead requests have arrived: shift them by one tile
#pragma unroll
            for (int i = 0; i < RN; ++i) { rp[i] = rpn[i]; rpn[i] = rpq[i]; rpq[i] = rpnn[i]; }
#pragma unroll
            for (int rd = 0; rd < ROUNDS; ++rd) { offs[rd] = offq[rd]; w0[rd] = wq[rd]; offq[rd] = offsn[rd]; wq[rd] = w0n[rd]; }
        }
        tile_id = tile_n1;
        tile_n1 = tile_n2;
        tile_n2 += nwaves;
        GNNHIP_PHASE_ACC(5);
    }
    GNNHIP_PHASE_FINI
}

template <int C, bool DENSE, bool RELU_IN, bool PIPE>
int launch_level_stream_p(int N, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                          const float* W, const float* msg, const float* bias, float* h_out, const HubPlan& hubs,
                          hipStream_t s)
{
    const long long ntiles = ((long long)N + 15) / 16;
    long long blocks = (ntiles + kWavesPerBlock - 1) / kWavesPerBlock;
    constexpr bool kWLds = (C == 64);
    constexpr int kMinW = (C == 64 && !DENSE) ? 3 : 4;    // hidden 64 needs 128 registers and spills for four
    const long long resident = (long long)kNumCU * kMinW;  // a workgroup puts one wavefront on each SIMD
    if (blocks > resident) blocks = resident;              // persistent beyond this
    hipLaunchKernelGGL((s2v_level_stream_kernel<C, DENSE, kWLds, kMinW, RELU_IN, PIPE>), dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs.row_slot, hubs.agg, hubs.ld);
    GNNHIP_LAUNCH_CHECK("s2v_level_stream");
    return GNNHIP_OK;
}

template <int C, bool DENSE, bool RELU_IN>
int launch_level_stream(int N, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                        const float* W, const float* msg, const float* bias, float* h_out, const HubPlan& hubs,
                        hipStream_t s)
{
    // Gathers issued a tile ahead pay once every wavefront has several tiles (116,000 nodes: 35 -> 32 us,
    // uniform random graph of 1M rows, 2 entries per row: 223 -> 205 us); with one or two tiles per
    // wavefront the longer start of that variant costs more than it gains (7,450 nodes: +1 us per level).
    if constexpr (C == 64 && !DENSE) {
        if (N >= kPipeMinRows)
            return launch_level_stream_p<C, DENSE, RELU_IN, true>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
    }
    return launch_level_stream_p<C, DENSE, RELU_IN, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
}

template <int C>
int launch_level_stream_c(int N, bool dense, bool relu_in, const int* row_ptr, const int* col_idx, const float* val,
                          const float* h_in, const float* W, const float* msg, const float* bias, float* h_out,
                          const HubPlan& hubs, hipStream_t s)
{
    if (dense) return launch_level_stream<C, true, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
    if (relu_in) return launch_level_stream<C, false, true>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
    return launch_level_stream<C, false, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
}

template <int C>
int launch_level_stream_backward(int N, const int* row_ptr, const int* col_idx, const float* val, const float* x,
                                 const float* W, float* agg_out, float* out, const float* gate, float* acc, const HubPlan& hubs,
                                 hipStream_t s)
{
    const long long ntiles = ((long long)N + 15) / 16;
    long long blocks = (ntiles + kWavesPerBlock - 1) / kWavesPerBlock;
    constexpr bool kWLds = (C == 64);
    constexpr int kMinW = (C == 64) ? 3 : 4;
    const long long resident = (long long)kNumCU * kMinW;
    if (blocks > resident) blocks = resident;
    hipLaunchKernelGGL((s2v_level_stream_kernel<C, false, kWLds, kMinW, false, false, true>), dim3((unsigned)blocks), dim3(kBlock), 0, s,
                       N, row_ptr, col_idx, val, x, W, gate, (const float*)nullptr, out, hubs.row_slot, hubs.agg,
                       hubs.ld, agg_out, acc);
    GNNHIP_LAUNCH_CHECK("s2v_level_stream (backward)");
    return GNNHIP_OK;
}

}  // namespace

// Whether N rows of C floats fit the 32-bit offsets of the kernel (with room for the 15 rows a last tile may
// address past N).
bool level_stream_covers(int N, int C)
{
    return (C == 16 || C == 32 || C == 64) && (unsigned long long)N * (unsigned)C * 4ull < 0xFFFF0000ull;
}

// agg_out = A' x and out = agg_out W^T in one pass (A' in CSR form); same limits as level_stream_dispatch.
// gate / acc (both may be null): out is zeroed where gate <= 0, then acc += out.
int level_stream_backward_dispatch(int N, int C, const int* row_ptr, const int* col_idx, const float* val, const float* x,
                                   const float* W, float* agg_out, float* out, const float* gate, float* acc, const HubPlan& hubs,
                                   hipStream_t s)
{
    if (!level_stream_covers(N, C)) return GNNHIP_EUNSUPPORTED;
    switch (C) {
    case 16: return launch_level_stream_backward<16>(N, row_ptr, col_idx, val, x, W, agg_out, out, gate, acc, hubs, s);
    case 32: return launch_level_stream_backward<32>(N, row_ptr, col_idx, val, x, W, agg_out, out, gate, acc, hubs, s);
    default: return launch_level_stream_backward<64>(N, row_ptr, col_idx, val, x, W, agg_out, out, gate, acc, hubs, s);
    }
}

// h_in, msg and h_out must each span less than 4 GiB; returns GNNHIP_EUNSUPPORTED otherwise.
// relu_in (not with dense): h_in is read as ReLU(h_in); hub sums in `hubs` must have been formed the same way.
int level_stream_dispatch(int N, int C, bool dense, const int* row_ptr, const int* col_idx, const float* val,
                          const float* h_in, const float* W, const float* msg, const float* bias, float* h_out,
                          const HubPlan& hubs, bool relu_in, hipStream_t s)
{
    if (!level_stream_covers(N, C) || (dense && relu_in)) return GNNHIP_EUNSUPPORTED;
    switch (C) {
    case 16: return launch_level_stream_c<16>(N, dense, relu_in, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
    case 32: return launch_level_stream_c<32>(N, dense, relu_in, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
    default: return launch_level_stream_c<64>(N, dense, relu_in, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, hubs, s);
    }
}

}  // namespace gnnhip
