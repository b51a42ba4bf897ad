// Fused mean-field level for wide hidden sizes (C = 128 or 256):
//     h_out = ReLU((A * h_in) * W + bias + msg)
// the operator chain MatMul(sparse) -> MatMul -> ElewiseAdd -> ReLU of
// examples/graph_classification/src/kernel_mean_field.cpp:35-42 in one launch.
//
// At C = 256 the C x C contraction is 2 N C^2 = 131 kflop per node against
// 3 KB of activation traffic per node: on FP32 matrix cores (157 TFLOP/s) the
// contraction takes about twice as long as the HBM traffic, so this kernel is
// organised around keeping the matrix pipes fed.
//
// One persistent workgroup of 8 wavefronts per compute unit.  W never moves
// after start-up: wavefront w keeps the W^T operand of its C/8 output columns
// in registers (C = 256: 128 registers per lane, half of the register file of
// the compute unit across the 8 wavefronts).  Per pass over TR rows (64; 32 or 16
// on matrices too small to give every compute unit two 64-row passes):
//   1. gather-sum  wavefront w sums the neighbour rows of TR/8 rows, the whole
//                  wavefront across the C columns of a row, six row loads in
//                  flight, and parks the sums in an LDS tile [TR][C+4];
//   2. contraction v_mfma_f32_16x16x4_f32, out^T = W^T * tile^T: the lane
//                  (q = lane/16, t = lane%16) feeds k = (C/4) q + s at step s, so
//                  four steps of its tile operand are one 128-bit LDS read, and it
//                  ends up owning row t, four consecutive columns per block;
//   3. epilogue    + bias + msg, ReLU, 128-bit stores (issued at the top of the
//                  next 16-row block).
// The tile is double-buffered and the gather of pass p+1 is spread, one batch
// of six row loads per 16-row block, over the contraction of pass p; the CSR
// indices are fetched one batch (columns, weights) or one pass (row pointers)
// further ahead still.  Only a wavefront whose rows hold more than six entries
// per 16-row block of the pass (24 at TR = 64) gathers in the open.
//
// What shaped the code (measured on MI355X):
//   * While a wavefront streams FP32 matrix instructions, every other
//     instruction issued on that SIMD, by either wavefront and of any kind
//     (vector, scalar, LDS, memory), gets about one issue slot per matrix
//     instruction (14 ns) instead of one per 2 ns.  The budget is therefore one
//     non-matrix instruction per matrix instruction; beyond it the matrix pipe
//     idles.  Hence: CSR indices through scalar loads (no broadcast
//     instructions), buffer addressing (a gathered row costs one scalar shift
//     and one load; rows past N are dropped by the descriptor's size, not by a
//     predicate), msg/bias added after the contraction in 8 + 8 adds.
//   * Vector memory operations retire in order, so any wait for a load also
//     waits for every store issued before it.  Stores are therefore issued
//     right before a contraction, never right before a wait.
//   * The loads of a batch and their uses sit under separate (uniform)
//     conditions; the compiler then assumes a path on which loads are still in
//     flight and waits at the top of the next block.  One explicit wait after
//     the contraction removes that.
#include "gnnhip_internal.h"
#include "buffer_addr.h"

// Phase accounting for a timing build of this file; expands to nothing in the library.
#ifndef GNNHIP_PHASE_ACC
#define GNNHIP_PHASE_ACC(i)
#define GNNHIP_PHASE_INIT
#define GNNHIP_PHASE_FINI
#endif


namespace gnnhip {
namespace {

constexpr int kInFlight = 6;                     // row gathers in flight per wavefront
constexpr int kWaitVmcnt0 = 0x0F70;              // s_waitcnt operand: vmcnt(0), other counters unconstrained

template <int VEC> struct VecT;
template <> struct VecT<2> { using type = float2; };
template <> struct VecT<4> { using type = float4; };

// Buffer addressing (buffer_addr.h): the memory instruction takes a 128-bit descriptor (base, size), a
// per-lane 32-bit offset and a scalar 32-bit offset, so a gathered row costs one scalar shift and no
// per-lane address arithmetic, and lanes whose offset lies past the size are dropped by the hardware.
template <int VEC> struct BufLoad;
template <> struct BufLoad<4> { static __device__ __forceinline__ float4 get(rsrc_t r, int v, int s) { return buf_load4(r, v, s); } };
template <> struct BufLoad<2> { static __device__ __forceinline__ float2 get(rsrc_t r, int v, int s) { return buf_load2(r, v, s); } };
template <int VEC> struct BufStore;
template <> struct BufStore<4> { static __device__ __forceinline__ void put(rsrc_t r, int v, int s, const float4& x) { buf_store4(r, v, s, x); } };
template <> struct BufStore<2> { static __device__ __forceinline__ void put(rsrc_t r, int v, int s, const float2& x) { buf_store2(r, v, s, x); } };

// A batch of kInFlight consecutive entries of a CSR array (column indices, or edge weights as bit
// patterns) in scalar registers.  The two scalar loads are written as inline assembly with the batch as a
// read-write operand: the loaded values land in the registers the batch already occupies, so a batch that
// is (conditionally) refilled inside the loop needs no copy of the loaded values, and with it no wait for
// the scalar cache right behind the load.  The compiler does not know that these registers are in flight:
// batch_wait() must run before a batch is read.
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
struct Batch { i32x4 lo; i32x2 hi; };
static_assert(kInFlight == 6, "a batch is one 4-dword and one 2-dword scalar load");
__device__ __forceinline__ void batch_load(Batch& b, const int* p)
{
    asm volatile("s_load_dwordx4 %0, %2, 0x0\n\ts_load_dwordx2 %1, %2, 0x10" : "+s"(b.lo), "+s"(b.hi) : "s"(p));
}
// The first n < kInFlight entries of an array that holds no more than n, zeros behind them: one scalar load
// per entry, each under its own (uniform) condition, and the wait right here.
__device__ __forceinline__ void batch_load_short(Batch& b, const int* p, int n)
{
    int t0 = 0, t1 = 0, t2 = 0, t3 = 0, t4 = 0;
    if (n > 0) asm volatile("s_load_dword %0, %1, 0x0" : "+s"(t0) : "s"(p));
    if (n > 1) asm volatile("s_load_dword %0, %1, 0x4" : "+s"(t1) : "s"(p));
    if (n > 2) asm volatile("s_load_dword %0, %1, 0x8" : "+s"(t2) : "s"(p));
    if (n > 3) asm volatile("s_load_dword %0, %1, 0xc" : "+s"(t3) : "s"(p));
    if (n > 4) asm volatile("s_load_dword %0, %1, 0x10" : "+s"(t4) : "s"(p));
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(t0), "+s"(t1), "+s"(t2), "+s"(t3), "+s"(t4));
    b.lo.x = t0; b.lo.y = t1; b.lo.z = t2; b.lo.w = t3;
    b.hi.x = t4; b.hi.y = 0;
}
__device__ __forceinline__ void batch_wait(Batch& b)
{
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(b.lo), "+s"(b.hi));
}
__device__ __forceinline__ int batch_get(const Batch& b, int u)      // u is a compile-time constant after unrolling
{
    return u == 0 ? b.lo.x : u == 1 ? b.lo.y : u == 2 ? b.lo.z : u == 3 ? b.lo.w : u == 4 ? b.hi.x : b.hi.y;
}

template <int VEC, bool RELU_IN>
__device__ __forceinline__ void vec_fma(float (&acc)[VEC], float a, const typename VecT<VEC>::type& x)
{
    const float* p = reinterpret_cast<const float*>(&x);
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = fmaf(a, RELU_IN ? relu_ref(p[i]) : p[i], acc[i]);
}

// Everything that steers the gather (row pointers, column indices, edge weights) is uniform
// across the wavefront and is fetched with scalar loads: the values land in scalar registers, cost
// no vector instruction to broadcast, and are counted apart from vector memory operations, so
// waiting for them never waits for a store.  That matters because on this hardware the FP32 matrix
// instructions and ordinary vector instructions do not overlap: every vector instruction issued by
// either wavefront of a SIMD takes time away from its matrix pipe.
// RELU_IN: the gathered rows count as ReLU(row) (the first level reading msg where h0 was not stored)
// TR: rows per pass (16, 32 or 64)
// BWD: the backward pass of a level through the same machinery.  The CSR arrays are those of A^T, h_in is dz, the
//      summed rows u = A^T dz are also stored to u_out as each one is finished (they are the other factor of the
//      weight gradient), the contraction takes W transposed (g = u W^T), and the epilogue, instead of adding msg and
//      applying ReLU, lets g through where the rows of `msg` (here: the embedding whose ReLU the gradient passes next,
//      or null for no gate) are positive and adds what it stores to acc_io (or null).
template <int C, int WAVES, bool RELU_IN, int TR, bool BWD = false>
__global__ __launch_bounds__(WAVES * kWave) void s2v_level_wide_kernel(
    int N, int tiles_per_block, const int* __restrict__ row_ptr, const int* __restrict__ col_idx,
    const float* __restrict__ val, const float* __restrict__ h_in, const float* __restrict__ W,
    const float* __restrict__ msg, const float* __restrict__ bias, float* __restrict__ h_out,
    float* __restrict__ u_out, float* __restrict__ acc_io)
{
    constexpr int KS = C / 4;                    // contraction steps
    constexpr int kWideBlock = WAVES * kWave;
    constexpr int CW = C / WAVES;                // output columns per wavefront
    constexpr int NB = CW / 16;                  // 16-column blocks per wavefront
    constexpr int VEC = C / kWave;               // gathered floats per lane
    constexpr int LDT = C + 4;                   // LDS row stride: rows 0..7 start in distinct 16-byte bank groups
    constexpr int kTileRows = TR;
    constexpr int RPW = kTileRows / WAVES;       // rows gathered per wavefront per pass
    using vec_t = typename VecT<VEC>::type;

    extern __shared__ float tiles[];             // two tiles [kTileRows][LDT]: one read by the matrix cores,
                                                 // the other being filled for the next pass
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int q = lane >> 4, t = lane & 15;
    const int col0 = wave * CW;
    const int gather_off = (wave * RPW) * LDT + lane * VEC;
    float* bias_lds = tiles + 2 * kTileRows * LDT;      // [C], read in the epilogue without a trip to memory
    if (bias)
        for (int i = threadIdx.x; i < C; i += kWideBlock) bias_lds[i] = bias[i];

    // W^T operand: wreg[jb][s] = W[KS q + s][col0 + 16 jb + t]; BWD: W itself, wreg[jb][s] = W[col0 + 16 jb + t][KS q + s]
    // (buffer loads: one lane offset, the steps as scalar offsets, so no 64-bit address per element is formed)
    float wreg[NB][KS];
    {
        const rsrc_t w_rsrc = make_rsrc(W, (unsigned)(C * C * 4));
        const int w_lane_off = BWD ? ((col0 + t) * C + KS * q) * 4 : ((KS * q) * C + col0 + t) * 4;
        if constexpr (BWD) {
            // a lane's steps are consecutive floats of one row of W: 128-bit loads (with one float per load, lanes
            // 1 KB apart, the start-up of a launch on 7,450 rows took longer than its passes)
#pragma unroll
            for (int jb = 0; jb < NB; ++jb)
#pragma unroll
                for (int s4 = 0; s4 < KS / 4; ++s4) {
                    const float4 v = buf_load4(w_rsrc, w_lane_off + 16 * C * 4 * jb, s4 * 16);
                    wreg[jb][4 * s4 + 0] = v.x; wreg[jb][4 * s4 + 1] = v.y; wreg[jb][4 * s4 + 2] = v.z; wreg[jb][4 * s4 + 3] = v.w;
                }
        } else {
#pragma unroll
            for (int jb = 0; jb < NB; ++jb)
#pragma unroll
                for (int s = 0; s < KS; ++s)
                    wreg[jb][s] = buf_load_f(w_rsrc, w_lane_off + 64 * jb, s * (C * 4));
        }
    }

    const int ntiles = (int)(((long long)N + kTileRows - 1) / kTileRows);
    const int tile_begin = (int)min((long long)blockIdx.x * tiles_per_block, (long long)ntiles);
    const int tile_end = (int)min((long long)ntiles, (long long)tile_begin + tiles_per_block);
    if (tile_begin >= tile_end) return;

    // ---- loaders.  The RPW + 1 row pointers of a pass sit in lanes 0..RPW of one vector register; columns
    //      and weights of a batch are uniform and come through scalar loads (weights as bit patterns
    //      so that selecting them stays on the scalar unit).
    auto load_rowptrs = [&](int tile_id) {
        const long long r0 = (long long)tile_id * kTileRows + wave * RPW;
        int v = 0;
        if (lane <= RPW) v = row_ptr[min(r0 + lane, (long long)N)];
        return v;
    };
    const int* val_bits = reinterpret_cast<const int*>(val);
    // entries [s, s + kInFlight) of the CSR arrays.  What lies past the end of the wavefront's rows is
    // loaded but never added, so the batch is read as it lies.  Only a batch that would run past the end
    // of the arrays starts earlier; batch_ready() then shifts it into place.  The entry count that bounds
    // these reads is the matrix's own (row_ptr[N], read here), never a count passed by the host.  A matrix
    // with fewer entries than one batch is read entry by entry, with zeros behind the last one.
    const int nnz = row_ptr[N];
    auto load_batch = [&](const int* arr, int s, Batch& b) {
        if (nnz < kInFlight) {
            batch_load_short(b, arr, nnz);
            return s;
        }
        const int base = max(min(s, nnz - kInFlight), 0);
        batch_load(b, arr + base);
        return s - base;                         // by how many entries the batch has to be shifted
    };
    auto batch_ready = [&](Batch& b, int shift) {
        batch_wait(b);
        for (; shift > 0; --shift) {             // only at the very end of the arrays
            b.lo.x = b.lo.y; b.lo.y = b.lo.z; b.lo.z = b.lo.w; b.lo.w = b.hi.x; b.hi.x = b.hi.y;
        }
    };
    const rsrc_t h_rsrc = make_rsrc(h_in, (unsigned)((size_t)N * C * 4));
    auto issue = [&](const Batch& c, vec_t (&x)[kInFlight]) {
#pragma unroll
        for (int u = 0; u < kInFlight; ++u)
            x[u] = BufLoad<VEC>::get(h_rsrc, lane * (VEC * 4), batch_get(c, u) * (C * 4));     // N C 4 < 2^32 (host-checked)
    };

    // ---- state of the gather of one pass: entries [e, ee) of the wavefront's RPW rows, taken in order;
    //      a row goes to LDS when its last entry has been added
    int e = 0, ee = 0, lr = 0, row_end = 0, rpv = 0;
    float* dstp = nullptr;
    float acc[VEC];
    rsrc_t u_rsrc = make_rsrc(u_out, 0);         // BWD: the rows of u_out that the pass being gathered covers
    auto begin = [&](int rp_lanes, int eb, int eend, float* dst, int tile_id) {
        rpv = rp_lanes;
        e = eb; ee = eend; lr = 0;
        row_end = __builtin_amdgcn_readlane(rpv, 1);
        dstp = dst;
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        if constexpr (BWD) {
            const long long r0 = (long long)tile_id * kTileRows;
            const long long rows = max(min((long long)N - r0, (long long)kTileRows), 0ll);      // none past the last pass
            u_rsrc = make_rsrc(u_out + (size_t)min(r0, (long long)N) * C, (unsigned)(rows * (C * 4)));
        }
    };
    auto flush_row = [&]() {
        *reinterpret_cast<vec_t*>(dstp) = *reinterpret_cast<vec_t*>(acc);
        if constexpr (BWD)                        // rows past N lie outside the descriptor
            BufStore<VEC>::put(u_rsrc, lane * (VEC * 4), (wave * RPW + lr) * (C * 4), *reinterpret_cast<vec_t*>(acc));
#pragma unroll
        for (int i = 0; i < VEC; ++i) acc[i] = 0.f;
        dstp += LDT;
        ++lr;
        row_end = __builtin_amdgcn_readlane(rpv, min(lr + 1, RPW));
    };
    auto consume = [&](const Batch& a, const vec_t (&x)[kInFlight]) {
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) {
            if (e + u < ee) {
                while (e + u >= row_end) flush_row();          // rows ending here (possibly empty ones)
                vec_fma<VEC, RELU_IN>(acc, __int_as_float(batch_get(a, u)), x[u]);
            }
        }
        e += kInFlight;
    };
    auto finish = [&]() { while (lr < RPW) flush_row(); };      // the open row and empty rows after it

    // Output of the last finished 16-row block, stored at the top of the following block (or at the end
    // of the pass): a store then has a whole contraction between its issue and the next wait on
    // vector memory.  msg and h_out are addressed through descriptors that cover the rows of the
    // current pass only, so rows past N fall outside and need no predicate.
    float4 outv[NB];
    int out_rt = -1;                             // block of this pass held in outv, -1: none
#pragma unroll
    for (int jb = 0; jb < NB; ++jb) outv[jb] = f4_zero();
    const int lane_off = (t * C + col0 + 4 * q) * 4;              // byte offset of this lane inside a 16-row block
    rsrc_t msg_rsrc = make_rsrc(msg, 0), out_rsrc = make_rsrc(h_out, 0), acc_rsrc = make_rsrc(acc_io, 0);
    auto store_pending = [&]() {
        if (out_rt >= 0) {
#pragma unroll
            for (int jb = 0; jb < NB; ++jb) buf_store4(out_rsrc, lane_off + out_rt * (16 * C * 4) + 64 * jb, 0, outv[jb]);
        }
        out_rt = -1;
    };

    GNNHIP_PHASE_INIT
    Batch cC, aC;                                // columns / weights of the next batch to issue / to sum
    cC.lo = i32x4{0, 0, 0, 0}; cC.hi = i32x2{0, 0};
    aC.lo = i32x4{0, 0, 0, 0}; aC.hi = i32x2{0, 0};
    int cShift = 0, aShift = 0;                  // shifts owed to cC / aC when they are next read

    // ---- first pass: its gather has nothing to hide behind
    int rp_next = load_rowptrs(tile_begin);      // row pointers of the next pass to gather
    int ebN = __builtin_amdgcn_readlane(rp_next, 0), eeN = __builtin_amdgcn_readlane(rp_next, RPW);
    begin(rp_next, ebN, eeN, tiles + gather_off, tile_begin);
    while (e < ee) {
        vec_t x[kInFlight];
        cShift = load_batch(col_idx, e, cC);
        aShift = load_batch(val_bits, e, aC);
        batch_ready(cC, cShift);
        batch_ready(aC, aShift);
        issue(cC, x);
        consume(aC, x);
    }
    finish();
    ebN = eeN = 0;
    if (tile_begin + 1 < tile_end) {
        rp_next = load_rowptrs(tile_begin + 1);
        ebN = __builtin_amdgcn_readlane(rp_next, 0);
        eeN = __builtin_amdgcn_readlane(rp_next, RPW);
        if (ebN < eeN) { cShift = load_batch(col_idx, ebN, cC); aShift = load_batch(val_bits, ebN, aC); }
    }
    __syncthreads();
    GNNHIP_PHASE_ACC(0);

    for (int tile_id = tile_begin; tile_id < tile_end; ++tile_id) {
        const long long row0 = (long long)tile_id * kTileRows;
        const int parity = (tile_id - tile_begin) & 1;
        const float* cur = tiles + parity * (kTileRows * LDT);
        const bool has_next = tile_id + 1 < tile_end;
        const bool has_next2 = tile_id + 2 < tile_end;
        begin(rp_next, ebN, eeN, tiles + (parity ^ 1) * (kTileRows * LDT) + gather_off, tile_id + 1);   // empty when !has_next
        {
            const long long left = (long long)N - row0;
            const unsigned bytes = (unsigned)(min(left, (long long)kTileRows) * (C * 4));
            out_rsrc = make_rsrc(h_out + (size_t)row0 * C, bytes);
            msg_rsrc = make_rsrc(msg ? msg + (size_t)row0 * C : nullptr, msg ? bytes : 0u);   // no msg: every load reads 0
            if constexpr (BWD) acc_rsrc = make_rsrc(acc_io ? acc_io + (size_t)row0 * C : nullptr, acc_io ? bytes : 0u);
        }
        if (has_next2) rp_next = load_rowptrs(tile_id + 2);

        // ---- contraction and epilogue, one 16-row block at a time; each block also carries one batch
        //      of the next pass's gather, issued before its matrix instructions and summed after them
#pragma unroll 1
        for (int rt = 0; rt < kTileRows / 16; ++rt) {
            // msg is asked for now and added after the contraction (as the accumulators' initial value it
            // would have to arrive before the first matrix instruction)
            float4 mm[NB], aa[BWD ? NB : 1];
            mfma_f4 acc_m[NB];
#pragma unroll
            for (int jb = 0; jb < NB; ++jb) {
                mm[jb] = buf_load4(msg_rsrc, lane_off + rt * (16 * C * 4) + 64 * jb, 0);
                acc_m[jb] = mfma_f4{0.f, 0.f, 0.f, 0.f};
            }
            if constexpr (BWD) {
                if (acc_io) {
#pragma unroll
                    for (int jb = 0; jb < NB; ++jb) aa[jb] = buf_load4(acc_rsrc, lane_off + rt * (16 * C * 4) + 64 * jb, 0);
                }
            }
            vec_t x[kInFlight];
            const bool batch = e < ee;
            if (batch) { batch_ready(cC, cShift); issue(cC, x); }
            store_pending();
            // where the follower of this batch starts: inside this pass, or (after the last block) at the
            // first entry of the next pass; its columns travel while the matrix cores work
            int ns = 0, nend = 0;
            if (rt < kTileRows / 16 - 1) {
                if (e + kInFlight < ee) { ns = e + kInFlight; nend = ee; }
            } else if (kTileRows > 16 && e + kInFlight >= ee) {
                ns = ebN; nend = eeN;                     // both zero when there is no next pass
            }
            // (a 16-row pass has one block: ebN/eeN still describe the pass being gathered, the row pointers of
            // the one after it arrive during this block, so its first batch is asked for after the block)
            GNNHIP_PHASE_ACC(1);

            const float* src = cur + (rt * 16 + t) * LDT + KS * q;
            // the tile operand is read two 128-bit words (eight contraction steps) ahead of its use
            float4 b_cur[2], b_nxt[2];
            b_cur[0] = *reinterpret_cast<const float4*>(src);
            b_cur[1] = *reinterpret_cast<const float4*>(src + 4);
#pragma unroll
            for (int s8 = 0; s8 < KS / 8; ++s8) {
                if (s8 + 1 < KS / 8) {
                    b_nxt[0] = *reinterpret_cast<const float4*>(src + 8 * (s8 + 1));
                    b_nxt[1] = *reinterpret_cast<const float4*>(src + 8 * (s8 + 1) + 4);
                }
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float4 b = b_cur[h];
                    const int s0 = 8 * s8 + 4 * h;
#pragma unroll
                    for (int jb = 0; jb < NB; ++jb) acc_m[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][s0 + 0], b.x, acc_m[jb], 0, 0, 0);
#pragma unroll
                    for (int jb = 0; jb < NB; ++jb) acc_m[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][s0 + 1], b.y, acc_m[jb], 0, 0, 0);
#pragma unroll
                    for (int jb = 0; jb < NB; ++jb) acc_m[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][s0 + 2], b.z, acc_m[jb], 0, 0, 0);
#pragma unroll
                    for (int jb = 0; jb < NB; ++jb) acc_m[jb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[jb][s0 + 3], b.w, acc_m[jb], 0, 0, 0);
                }
                // the follower's columns are asked for here, behind the first wait for LDS of this block: a
                // scalar load in flight counts with the LDS reads, and the next wait is 16 matrix instructions away
                if (s8 == 0 && ns < nend) cShift = load_batch(col_idx, ns, cC);
                __builtin_amdgcn_sched_barrier(0);            // keeps the read-ahead where it is written
                b_cur[0] = b_nxt[0]; b_cur[1] = b_nxt[1];
            }
            GNNHIP_PHASE_ACC(2);
            // One unconditional wait for everything this block asked for (gathered rows, msg).  The loads
            // and their uses sit under separate conditions; without this the compiler has to assume a
            // path on which they are still in flight and waits at the top of the next block instead,
            // where the wait also covers the stores issued just before it.
            __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
            if (batch) { batch_ready(aC, aShift); consume(aC, x); }
            if (ns < nend) aShift = load_batch(val_bits, ns, aC);
            if (rt == 0) {                                // the row pointers asked for at the top have arrived
                ebN = eeN = 0;
                if (has_next2) {
                    ebN = __builtin_amdgcn_readlane(rp_next, 0);
                    eeN = __builtin_amdgcn_readlane(rp_next, RPW);
                }
            }
            GNNHIP_PHASE_ACC(3);
            if constexpr (BWD) {
#pragma unroll
                for (int jb = 0; jb < NB; ++jb) {
                    float4 v = make_float4(acc_m[jb][0], acc_m[jb][1], acc_m[jb][2], acc_m[jb][3]);
                    if (msg) {                   // past the ReLU whose output these rows are
                        v.x = mm[jb].x > 0.f ? v.x : 0.f; v.y = mm[jb].y > 0.f ? v.y : 0.f;
                        v.z = mm[jb].z > 0.f ? v.z : 0.f; v.w = mm[jb].w > 0.f ? v.w : 0.f;
                    }
                    if (acc_io) {                // every row belongs to one pass: nobody else touches it during the launch
                        const float4 a = make_float4(aa[jb].x + v.x, aa[jb].y + v.y, aa[jb].z + v.z, aa[jb].w + v.w);
                        buf_store4(acc_rsrc, lane_off + rt * (16 * C * 4) + 64 * jb, 0, a);
                    }
                    outv[jb] = v;
                }
            } else {
#pragma unroll
                for (int jb = 0; jb < NB; ++jb) {
                    acc_m[jb][0] += mm[jb].x; acc_m[jb][1] += mm[jb].y; acc_m[jb][2] += mm[jb].z; acc_m[jb][3] += mm[jb].w;
                }
#pragma unroll
                for (int jb = 0; jb < NB; ++jb) {
                    float4 v = make_float4(acc_m[jb][0], acc_m[jb][1], acc_m[jb][2], acc_m[jb][3]);
                    if (bias) {
                        const float4 b4 = *reinterpret_cast<const float4*>(bias_lds + col0 + 16 * jb + 4 * q);
                        v.x += b4.x; v.y += b4.y; v.z += b4.z; v.w += b4.w;
                    }
                    outv[jb] = make_float4(relu_ref(v.x), relu_ref(v.y), relu_ref(v.z), relu_ref(v.w));
                }
            }
            out_rt = rt;
            GNNHIP_PHASE_ACC(4);
        }
        if (kTileRows == 16 || e < ee) {                  // more batches than blocks: finish in the open
            while (e < ee) {
                vec_t x[kInFlight];
                cShift = load_batch(col_idx, e, cC);
                aShift = load_batch(val_bits, e, aC);
                batch_ready(cC, cShift);
                batch_ready(aC, aShift);
                issue(cC, x);
                consume(aC, x);
            }
            if (ebN < eeN) { cShift = load_batch(col_idx, ebN, cC); aShift = load_batch(val_bits, ebN, aC); }
        }
        if (has_next) finish();
        store_pending();
        GNNHIP_PHASE_ACC(5);
        __syncthreads();                                  // the tile just filled is complete, the other one is free
        GNNHIP_PHASE_ACC(6);
    }
    GNNHIP_PHASE_FINI
}

template <int C, int WAVES, bool RELU_IN, int TR, bool BWD = false>
int launch_level_wide_t(int N, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                      const float* W, const float* msg, const float* bias, float* h_out, hipStream_t s,
                      float* u_out = nullptr, float* acc_io = nullptr)
{
    if ((unsigned long long)N * C * 4ull >= (1ull << 32)) return GNNHIP_EUNSUPPORTED;   // 32-bit buffer offsets
    constexpr int kTileRows = TR;
    const long long ntiles = ((long long)N + kTileRows - 1) / kTileRows;
    // workgroups that fit one compute unit together: two at C = 128 (82 registers per lane, 68 KB of LDS each)
    constexpr int kPerCU = (C == 128) ? 2 : 1;
    const long long slots = (long long)kNumCU * kPerCU;
    const long long per = (ntiles + slots - 1) / slots;              // contiguous run of tiles per workgroup
    const long long blocks = (ntiles + per - 1) / per;
    const size_t smem = sizeof(float) * (2 * kTileRows * (C + 4) + C);
    static LdsLimit lds_limit;                                       // one per kernel instantiation
    GNNHIP_HIP(lds_limit.raise(reinterpret_cast<const void*>(&s2v_level_wide_kernel<C, WAVES, RELU_IN, TR, BWD>), smem));
    hipLaunchKernelGGL((s2v_level_wide_kernel<C, WAVES, RELU_IN, TR, BWD>), dim3((unsigned)blocks), dim3(WAVES * kWave), smem, s,
                       N, (int)per, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, u_out, acc_io);
    GNNHIP_LAUNCH_CHECK(BWD ? "s2v_level_wide backward" : "s2v_level_wide");
    return GNNHIP_OK;
}

// Rows per pass.  The contraction of a 64-row pass keeps one compute unit's matrix pipes busy for 14 us at
// C = 256, so a matrix with fewer passes than twice the compute units is cut into shorter ones.
template <int C, int WAVES, bool RELU_IN>
int launch_level_wide(int N, const int* row_ptr, const int* col_idx, const float* val, const float* h_in,
                      const float* W, const float* msg, const float* bias, float* h_out, hipStream_t s)
{
    constexpr int kSlots = kNumCU * ((C == 128) ? 2 : 1);
    if (N >= 2 * kSlots * 64) return launch_level_wide_t<C, WAVES, RELU_IN, 64>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
    if (N >= 2 * kSlots * 32) return launch_level_wide_t<C, WAVES, RELU_IN, 32>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
    return launch_level_wide_t<C, WAVES, RELU_IN, 16>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
}

// The backward pass: same choice of rows per pass.
template <int C, int WAVES>
int launch_level_wide_backward(int N, const int* row_ptr, const int* col_idx, const float* val, const float* dz, const float* W,
                               float* u, float* g_prev, const float* gate, float* acc, hipStream_t s)
{
    constexpr int kSlots = kNumCU * ((C == 128) ? 2 : 1);
    if (N >= 2 * kSlots * 64) return launch_level_wide_t<C, WAVES, false, 64, true>(N, row_ptr, col_idx, val, dz, W, gate, nullptr, g_prev, s, u, acc);
    if (N >= 2 * kSlots * 32) return launch_level_wide_t<C, WAVES, false, 32, true>(N, row_ptr, col_idx, val, dz, W, gate, nullptr, g_prev, s, u, acc);
    return launch_level_wide_t<C, WAVES, false, 16, true>(N, row_ptr, col_idx, val, dz, W, gate, nullptr, g_prev, s, u, acc);
}

}  // namespace

// Whether N rows of C floats have a wide kernel (32-bit buffer offsets).
bool level_wide_covers(int N, int C)
{
    return (C == 128 || C == 256) && (unsigned long long)N * (unsigned)C * 4ull < (1ull << 32);
}

int level_wide_dispatch(int N, int C, long long nnz, const int* row_ptr, const int* col_idx, const float* val,
                        const float* h_in, const float* W, const float* msg, const float* bias, float* h_out, bool relu_in,
                        hipStream_t s)
{
    (void)nnz;                                   // the kernel bounds its index reads with row_ptr[N]
    switch (C) {
    case 128:
        return relu_in ? launch_level_wide<128, 8, true>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s)
                       : launch_level_wide<128, 8, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
    case 256:
        return relu_in ? launch_level_wide<256, 8, true>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s)
                       : launch_level_wide<256, 8, false>(N, row_ptr, col_idx, val, h_in, W, msg, bias, h_out, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

// u = A' dz (stored) and g_prev = u W^T past the gate of `gate` (may be null), added to acc (may be null): the wide
// kernel's backward variant over the CSR arrays of A' = A^T.
int level_wide_backward_dispatch(int N, int C, const int* row_ptr, const int* col_idx, const float* val, const float* dz, const float* W,
                                 float* u, float* g_prev, const float* gate, float* acc, hipStream_t s)
{
    switch (C) {
    case 128: return launch_level_wide_backward<128, 8>(N, row_ptr, col_idx, val, dz, W, u, g_prev, gate, acc, s);
    case 256: return launch_level_wide_backward<256, 8>(N, row_ptr, col_idx, val, dz, W, u, g_prev, gate, acc, s);
    }
    return GNNHIP_EUNSUPPORTED;
}

}  // namespace gnnhip
