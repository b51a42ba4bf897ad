// CSR SpMM for large matrices with many entries per row (power-law graphs): column-ordered pieces.
//
// On an R-MAT matrix the gathers of C = A * B miss the 4 MB L2 of their die most of the time: the rows a
// workgroup walks touch unrelated rows of B, and a popular row of B is fetched again and again (counted: ten
// times the size of B).  CSR columns are sorted inside a row, so a run of consecutive entries of a long row
// covers a narrow range of columns.  This pass cuts every row into pieces of at most kPiece consecutive
// entries, orders the pieces by the column they start at (two stable radix passes on the top sixteen bits of
// that column), copies the entries into that order, and sums the pieces in that order, each die taking one
// contiguous eighth of it.  What runs together then starts in the same narrow band of B; measured on R-MAT
// with 4M rows and 16 entries per row this brings the fetched bytes from 14 GB (pieces in row order) to 8 GB.
//
//   plan     pieces per row -> offsets (scan) -> piece records + keys -> order by first column (the second radix
//            pass carries the first one's order along, the records themselves stay where they are) ->
//            entries copied in piece order (a CSR matrix whose rows are the pieces)
//   sums     one lane group per piece, entries read front to back; a row of one piece (most rows) gets its
//            result, beta * C included, straight from here
//   combine  the other rows: the sums are stored by piece id, so the pieces of a row, and of the rows after it, lie
//            next to each other; a lane group takes a run of consecutive rows and adds up each row's pieces front
//            to back (rows without entries get beta * C; rows of more than eight pieces come from the
//            balanced pass over long rows, run on the 0/1 matrix P that picks the pieces of a row)
//
// Every sum is taken in an order fixed by the matrix (no atomics): the result does not depend on scheduling.
// The plan depends on A only (structure and values) and is reused by the later levels of one forward.
// Bound: HBM / L2.  Algorithmic bytes as for the plain SpMM, plus 8 bytes of partial sums per column and piece.
#include "gnnhip_internal.h"

#include <map>
#include <set>

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kPiece = 32;              // entries per piece

// entries [start, end); id: the place of the piece's sum among the partial sums, -1 when its row has no other piece;
// row: the row when the piece is all of it and holds entries (then its sum is the row's result), else -1
struct PieceRec { int start, end, id, row; };
constexpr int kNoPlace = (int)0x80000000;   // target of a piece whose sum nobody reads

__device__ __forceinline__ int pieces_of(int deg) { return (deg + kPiece - 1) / kPiece; }

// counts[r] = pieces of row r, pcounts[r] = the same for rows of several pieces and 0 for the others (entry m of both
// is 0, so that the scans leave the totals there).  The host's entry count `cap` sizes every array of the plan; should
// the matrix hold more entries than that, a row that reaches past entry `cap` (the last rows) is one piece whatever
// its length: no entries are copied for it, and piece_tail_kernel forms the row's result from the CSR arrays.
__global__ __launch_bounds__(kBlock) void piece_count_kernel(int m, const int* __restrict__ row_ptr, int cap, int* __restrict__ counts,
                                                             int* __restrict__ pcounts)
{
    for (long long r = (long long)blockIdx.x * kBlock + threadIdx.x; r <= m; r += (long long)gridDim.x * kBlock) {
        int c = 0;
        if (r < m) {
            const int e0 = row_ptr[r], e1 = row_ptr[r + 1];
            c = e1 <= cap ? pieces_of(e1 - e0) : (e1 > e0 ? 1 : 0);
        }
        counts[r] = c;
        pcounts[r] = c > 1 ? c : 0;
    }
}

// One lane per piece slot: the row that owns piece id is found by bisection in the scanned counts.
// Slots at or past the number of pieces get an empty record and the largest key (they sort to the end).
// rec.id: the place of the piece's sum among the partial sums (pfirst[row] + index of the piece in its row) when its row
// has several pieces, else -1.
__global__ __launch_bounds__(kBlock) void piece_fill_kernel(int m, long long slots, const int* __restrict__ row_ptr, int cap,
                                                            const int* __restrict__ col_idx, const int* __restrict__ first,
                                                            const int* __restrict__ pfirst, int shift, PieceRec* __restrict__ rec,
                                                            unsigned* __restrict__ keys)
{
    const int total = first[m];
    for (long long id = (long long)blockIdx.x * kBlock + threadIdx.x; id < slots; id += (long long)gridDim.x * kBlock) {
        if (id >= total) {
            rec[id] = PieceRec{0, 0, -1, -1};
            keys[id] = 0xFFFFu;
            continue;
        }
        int lo = 0, hi = m;                          // largest row with first[row] <= id
        while (hi - lo > 1) {
            const int mid = (int)(((long long)lo + hi) >> 1);
            if (first[mid] <= (int)id) lo = mid; else hi = mid;
        }
        const int row = lo;
        const int k = (int)id - first[row];
        const int rb = row_ptr[row], re = row_ptr[row + 1];
        const int start = rb + k * kPiece;
        const int end = re <= cap ? min(start + kPiece, re) : start;     // a row past the host's count: an empty stand-in
        const bool alone = first[row + 1] - first[row] == 1;
        rec[id] = PieceRec{start, end, alone ? -1 : pfirst[row] + k, (end > start && alone) ? row : -1};
        keys[id] = ((unsigned)col_idx[start] >> shift) & 0xFFFFu;
    }
}

// lens[i] = entries of the i-th piece in order (lens[slots] = 0, so that the scan leaves the total there);
// target[i]: where the sum of the i-th piece in order goes: the row r >= 0 when the piece is all of that row,
// else -1 - (its place among the partial sums; a stand-in piece without entries and without place gets a place past the
// end, which the sum kernel recognises).  order[i] = id of the i-th piece in order; ordered[i] = its record.
__global__ __launch_bounds__(kBlock) void piece_place_kernel(long long slots, long long pslots, const unsigned* __restrict__ order,
                                                             const PieceRec* __restrict__ rec, PieceRec* __restrict__ ordered,
                                                             int* __restrict__ lens, int* __restrict__ target)
{
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i <= slots; i += (long long)gridDim.x * kBlock) {
        if (i == slots) { lens[i] = 0; continue; }
        const PieceRec r = rec[order[i]];
        ordered[i] = r;
        lens[i] = r.end - r.start;
        target[i] = r.row >= 0 ? r.row : (r.id >= 0 ? -1 - r.id : kNoPlace);
    }
}

// Entries copied into piece order: half a wavefront per piece (kPiece = 32 entries, one per lane), four pieces
// per turn so that their dependent loads (record, place, entry) overlap.  The empty pieces at the end are skipped.
// (Taken by id instead, so that the reads walk the CSR arrays front to back and the writes scatter, the copy is
// slower: 0.44 against 0.37 ms.)
__global__ __launch_bounds__(kBlock) void piece_gather_kernel(const int* __restrict__ count, const PieceRec* __restrict__ ordered,
                                                              const int* __restrict__ at, const int* __restrict__ col_idx,
                                                              const float* __restrict__ val, int* __restrict__ col_out,
                                                              float* __restrict__ val_out)
{
    static_assert(kPiece == 32, "one lane per entry of a piece");
    constexpr int kTurn = 4;
    const int sub = threadIdx.x & (kPiece - 1);
    const long long per = kBlock / kPiece;
    const long long total = *count;
    for (long long i0 = ((long long)blockIdx.x * per + threadIdx.x / kPiece) * kTurn; i0 < total; i0 += (long long)gridDim.x * per * kTurn) {
        PieceRec r[kTurn];
        int dst[kTurn], c[kTurn];
        float v[kTurn];
#pragma unroll
        for (int u = 0; u < kTurn; ++u) {
            const bool live = i0 + u < total;
            r[u] = live ? ordered[i0 + u] : PieceRec{0, 0, 0, -1};
            dst[u] = live ? at[i0 + u] : 0;
        }
#pragma unroll
        for (int u = 0; u < kTurn; ++u) {
            const bool live = r[u].start + sub < r[u].end;
            c[u] = live ? col_idx[r[u].start + sub] : 0;
            v[u] = live ? val[r[u].start + sub] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < kTurn; ++u)
            if (r[u].start + sub < r[u].end) { col_out[dst[u] + sub] = c[u]; val_out[dst[u] + sub] = v[u]; }
    }
}

template <int VEC> struct PV;
template <> struct PV<4> {
    using T = float4;
    static __device__ __forceinline__ T zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
    static __device__ __forceinline__ T load(const float* p) { return *reinterpret_cast<const float4*>(p); }
    static __device__ __forceinline__ void store(float* p, T v) { *reinterpret_cast<float4*>(p) = v; }
    static __device__ __forceinline__ void fma(T& a, float s, T x) { a.x += s * x.x; a.y += s * x.y; a.z += s * x.z; a.w += s * x.w; }
    static __device__ __forceinline__ T axpby(T a, float b, T c) { return make_float4(a.x + b * c.x, a.y + b * c.y, a.z + b * c.z, a.w + b * c.w); }
};
template <> struct PV<1> {
    using T = float;
    static __device__ __forceinline__ T zero() { return 0.f; }
    static __device__ __forceinline__ T load(const float* p) { return *p; }
    static __device__ __forceinline__ void store(float* p, T v) { *p = v; }
    static __device__ __forceinline__ void fma(T& a, float s, T x) { a += s * x; }
    static __device__ __forceinline__ T axpby(T a, float b, T c) { return a + b * c; }
};

// One lane group (G lanes) per piece, pieces taken in order; die x (workgroups x, x + 8, ...) walks the
// x-th eighth of that order front to back, a workgroup taking the next ngroups pieces of its die when the
// hardware starts it (so the pieces in flight on a die stay close together in the order; a fixed stride per
// workgroup lets them drift apart and costs a quarter more fetched bytes).  The launch covers the host's bound
// on the number of pieces; workgroups past the real count leave at once.  Inner loop as in the row-group SpMM:
// the group reads G column indices and values at once and hands them round by shuffle, four gathers in flight.
// The sum of a piece that is all of its row goes to C (as sum + beta * C, what the combining pass would make of
// it), the others to the place of their piece id among the partial sums.
template <int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void piece_sum_kernel(
    const int* __restrict__ count, int n, float alpha, const int* __restrict__ at, const int* __restrict__ col_idx, const float* __restrict__ val,
    const float* __restrict__ B, int ldb, float* __restrict__ part, int ldp, int logG, const int* __restrict__ target, float beta,
    float* __restrict__ C, int ldc)
{
    using V = PV<VEC>;
    const int G = 1 << logG;
    const int sub = threadIdx.x & (G - 1);
    const int grp = threadIdx.x >> logG;
    const int ngroups = kBlock >> logG;
    const int xcd = blockIdx.x % kNumXCD, bx = blockIdx.x / kNumXCD;
    const long long total = *count;                               // the real pieces (the empty ones behind them are skipped)
    const long long lo = total * xcd / kNumXCD, hi = total * (xcd + 1) / kNumXCD;
    {
        const long long i = lo + (long long)bx * ngroups + grp;
        if (i >= hi) return;
        const int start = at[i], end = at[i + 1];
        typename V::T acc[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc[it] = V::zero();
        for (int base = start; base < end; base += G) {
            const int t = base + sub;
            int c = 0;
            float v = 0.f;
            if (t < end) { c = col_idx[t]; v = alpha * val[t]; }
            const int cnt = min(G, end - base);
            for (int j = 0; j < cnt; j += 4) {
                int cj[4];
                float vj[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    cj[u] = __shfl(c, (j + u) & (G - 1), G);
                    vj[u] = __shfl(v, (j + u) & (G - 1), G);
                }
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const int col0 = (sub + it * G) * VEC;
                    if (col0 < n) {
                        typename V::T x[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            x[u] = (j + u < cnt) ? V::load(B + (size_t)cj[u] * ldb + col0) : V::zero();
#pragma unroll
                        for (int u = 0; u < 4; ++u)
                            if (j + u < cnt) V::fma(acc[it], vj[u], x[u]);
                    }
                }
            }
        }
        const int row = target[i];
        if (row == kNoPlace) return;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int col0 = (sub + it * G) * VEC;
            if (col0 >= n) continue;
            if (row < 0) {
                V::store(part + (size_t)(-1 - row) * ldp + col0, acc[it]);
            } else {
                float* dst = C + (size_t)row * ldc + col0;
                if (beta == 0.f) V::store(dst, acc[it]);
                else V::store(dst, V::axpby(acc[it], beta, V::load(dst)));
            }
        }
    }
}

// The rows that reach past entry `cap` (none when the host's entry count is the matrix's own): such a row has one
// stand-in piece without entries, so neither the sums nor the combining pass write it; its result,
// alpha * A[row] * B + beta * C[row], is formed here.  Rows are taken from the last one down, a lane group each;
// the first row that ends inside the plan ends the walk.
template <int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void piece_tail_kernel(int m, int n, float alpha, const int* __restrict__ row_ptr, int cap,
                                                            const int* __restrict__ col_idx, const float* __restrict__ val,
                                                            const float* __restrict__ B, int ldb, float beta, float* __restrict__ C,
                                                            int ldc, int logG)
{
    using V = PV<VEC>;
    const int G = 1 << logG;
    const int sub = threadIdx.x & (G - 1);
    const int grp = threadIdx.x >> logG;
    const int ngroups = kBlock >> logG;
    for (long long back = (long long)blockIdx.x * ngroups + grp; back < m; back += (long long)gridDim.x * ngroups) {
        const int row = m - 1 - (int)back;
        const int start = row_ptr[row], end = row_ptr[row + 1];
        if (end <= cap) break;
        if (start == end) continue;
        typename V::T acc[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc[it] = V::zero();
        for (int t = start; t < end; ++t) {
            const int c = col_idx[t];
            const float v = alpha * val[t];
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) V::fma(acc[it], v, V::load(B + (size_t)c * ldb + col0));
            }
        }
        float* dst = C + (size_t)row * ldc;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int col0 = (sub + it * G) * VEC;
            if (col0 >= n) continue;
            if (beta == 0.f) V::store(dst + col0, acc[it]);
            else V::store(dst + col0, V::axpby(acc[it], beta, V::load(dst + col0)));
        }
    }
}

// C[row] = sum of the row's partial sums + beta * C[row] for the rows of no piece or of several; a row of one piece
// has its result already.  first: pieces before each row; pfirst: row pointers into part, which holds the sums of the
// rows of several pieces, a row's sums next to each other: row r owns part[pfirst[r] .. pfirst[r + 1]).
// A wavefront takes 64 consecutive rows, a lane looks one of them up, and two ballots tell which have no piece and
// which have several; the wavefront's lane groups then work through each kind on its own, a row per group and step,
// so that every step keeps all groups busy and a step of rows without entries waits for nothing (taking the rows in
// order, a group for each run of eight, every wavefront carried the chain row -> sums of the row eight steps long:
// 0.29 ms where the bytes take 0.15).  A row's pieces are added in piece order, eight loads in flight.  A row of
// more than kCombineLong pieces takes its sum from the balanced pass (hub_slot / hub_agg) when that pass has one
// for it: on a power-law matrix the rows of many pieces sit next to each other.
// skip_empty: rows without entries are not written (the consumer knows them from row_ptr and reads zeros instead);
// otherwise they get beta * C.
constexpr int kCombineLong = 8;         // pieces; the balanced pass cuts such rows into chunks of kCombineChunk pieces
constexpr int kCombineChunk = 256;
template <int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void piece_combine_kernel(
    int m, int n, const int* __restrict__ first, const int* __restrict__ pfirst, const float* __restrict__ part, int ldp, float beta,
    float* __restrict__ C, int ldc, int logG, const int* __restrict__ hub_slot, const float* __restrict__ hub_agg, int hub_ld,
    int skip_empty)
{
    using V = PV<VEC>;
    constexpr int kFlight = 8;
    const int lane = threadIdx.x & (kWave - 1);
    const int G = 1 << logG;                       // lanes per row: 8 .. 64
    const int sub = lane & (G - 1);
    const int wgrp = lane >> logG;
    const int ngroups = kWave >> logG;
    const long long row0 = ((long long)blockIdx.x * (kBlock / kWave) + threadIdx.x / kWave) * kWave;
    if (row0 >= m) return;
    const long long r = row0 + lane;
    int pieces = 1, pb = 0, pe = 0;
    if (r < m) pieces = first[r + 1] - first[r];
    const bool several = r < m && pieces > 1;
    if (several) { pb = pfirst[r]; pe = pfirst[r + 1]; }
    unsigned long long none_left = __ballot(r < m && pieces == 0 && !skip_empty);
    unsigned long long several_left = __ballot(several);
    // the next ngroups rows of a kind, one per lane group (-1: none left for this group)
    auto take = [&](unsigned long long& left) {
        int mine = -1;
        for (int g = 0; g < ngroups && left; ++g) {
            const int b = __builtin_ctzll(left);
            left &= left - 1;
            if (g == wgrp) mine = b;
        }
        return mine;
    };
    while (none_left) {
        const int o = take(none_left);
        if (o < 0) continue;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int col0 = (sub + it * G) * VEC;
            if (col0 >= n) continue;
            float* dst = C + (size_t)(row0 + o) * ldc + col0;
            if (beta == 0.f) V::store(dst, V::zero());
            else V::store(dst, V::axpby(V::zero(), beta, V::load(dst)));
        }
    }
    while (several_left) {
        const int o = take(several_left);
        const int src = o >= 0 ? o : 0;
        const int b = __shfl(pb, src, kWave), e = __shfl(pe, src, kWave);
        if (o < 0) continue;
        const long long row = row0 + o;
        typename V::T acc[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc[it] = V::zero();
        int hslot = -1;
        if (hub_slot && e - b > kCombineLong) hslot = hub_slot[row];
        if (hslot >= 0) {
#pragma unroll
            for (int it = 0; it < ITERS; ++it) {
                const int col0 = (sub + it * G) * VEC;
                if (col0 < n) acc[it] = V::load(hub_agg + (size_t)hslot * hub_ld + col0);
            }
        } else {
            for (int p = b; p < e; p += kFlight) {
#pragma unroll
                for (int it = 0; it < ITERS; ++it) {
                    const int col0 = (sub + it * G) * VEC;
                    if (col0 < n) {
                        typename V::T x[kFlight];
#pragma unroll
                        for (int u = 0; u < kFlight; ++u)
                            x[u] = (p + u < e) ? V::load(part + (size_t)(p + u) * ldp + col0) : V::zero();
#pragma unroll
                        for (int u = 0; u < kFlight; ++u)
                            if (p + u < e) V::fma(acc[it], 1.f, x[u]);
                    }
                }
            }
        }
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
            const int col0 = (sub + it * G) * VEC;
            if (col0 >= n) continue;
            float* dst = C + (size_t)row * ldc + col0;
            if (beta == 0.f) V::store(dst, acc[it]);
            else V::store(dst, V::axpby(acc[it], beta, V::load(dst)));
        }
    }
}

inline int ilog2_ceil_p(int x)
{
    int l = 0;
    while ((1 << l) < x) ++l;
    return l;
}
inline size_t round_up_p(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Mean entries per row from which a matrix of at least kHubMinRows rows takes this route.
constexpr long long kPiecesMeanDegree = 12;

struct Width {            // how a lane group covers the columns of an operand of width n
    bool ok, vec4;
    int logG, iters, ldp;
};
Width width_of(int n, const float* B, int ldb, const float* C, int ldc)
{
    Width w;
    w.vec4 = (n % 4 == 0) && (ldb % 4 == 0) && (ldc % 4 == 0) && aligned16(B) && aligned16(C);
    const int vec = w.vec4 ? 4 : 1;
    const int units = (n + vec - 1) / vec;
    // A lane group covers at most 64 x 4 column units (wider operands stay with the caller's route, which cuts them into
    // slabs).  Narrow operands stay with the row-group route too: with fewer than eight lanes per piece a wavefront reads
    // the entries of more than eight pieces at once, 128 bytes apart, and fetches whole lines for a few bytes each
    // (width 4 on the 4M-row R-MAT matrix: 16.6 GB fetched, 2.7 ms against 0.26 ms).
    w.ok = units <= kWave * 4 && units >= 8;
    w.logG = ilog2_ceil_p(units < kWave ? units : kWave);
    w.iters = (units + (1 << w.logG) - 1) >> w.logG;               // 1..4 (3 runs as 4)
    w.ldp = (int)round_up_p((size_t)n, 4);
    return w;
}

// Every row has at most one piece that is not full, and a row of several pieces has at least kPiece + 1 entries.
inline long long slots_bound(int m, long long nnz) { return nnz / kPiece + m; }
inline long long pslots_bound(long long nnz) { return nnz / kPiece + nnz / (kPiece + 1) + 1; }

struct Layout {           // offsets inside the head, body and temporary blocks of a plan
    size_t o_first, o_pfirst, head_bytes;
    size_t o_at, o_target, o_col, o_val, body_bytes;
    size_t o_seg, o_rec, o_ord, o_keys, o_keys2, o_perm, o_perm2, o_hist, temp_bytes;
};
Layout layout_of(int m, long long nnz, long long slots, long long pslots)
{
    Layout L;
    size_t off = 0;
    auto carve = [&](size_t bytes) { const size_t o = off; off = round_up_p(off + bytes, 256); return o; };
    L.o_first = carve(sizeof(int) * ((size_t)m + 1));
    L.o_pfirst = carve(sizeof(int) * ((size_t)m + 1));
    L.head_bytes = off;
    off = 0;
    L.o_at = carve(sizeof(int) * ((size_t)slots + 1));
    L.o_target = carve(sizeof(int) * (size_t)slots);
    L.o_col = carve(sizeof(int) * (size_t)nnz);
    L.o_val = carve(sizeof(float) * (size_t)nnz);
    L.body_bytes = off;
    off = 0;
    const size_t longest = (size_t)(slots + 1 > (long long)m + 1 ? slots + 1 : (long long)m + 1);
    L.o_seg = carve(sizeof(int) * (longest / 4096 + 2 + radix_seg_ints(slots)));
    L.o_rec = carve(sizeof(PieceRec) * (size_t)slots);
    L.o_ord = carve(sizeof(PieceRec) * (size_t)slots);
    L.o_keys = carve(sizeof(unsigned) * (size_t)slots);
    L.o_keys2 = carve(sizeof(unsigned) * (size_t)slots);
    L.o_perm = carve(sizeof(unsigned) * (size_t)slots);
    L.o_perm2 = carve(sizeof(unsigned) * (size_t)slots);
    L.o_hist = carve(sizeof(int) * radix_hist_ints(slots));
    L.temp_bytes = off;
    return L;
}

constexpr unsigned kElemGrid = kNumCU * 16;

// pieces per row and their scans: first, pfirst (the totals end up in entry m of each)
int count_pieces(CsrPlan* p, int cap, int* seg, hipStream_t s)
{
    hipLaunchKernelGGL(piece_count_kernel, dim3(kElemGrid), dim3(kBlock), 0, s, p->m, p->row_ptr, cap, p->first, p->pfirst);
    if (int rc = exclusive_scan_i32(p->first, (long long)p->m + 1, seg, s)) return rc;
    if (int rc = exclusive_scan_i32(p->pfirst, (long long)p->m + 1, seg, s)) return rc;
    GNNHIP_LAUNCH_CHECK("spmm_pieces count");
    return GNNHIP_OK;
}

// the rest of the plan, from the scanned counts: records, order by first column, entries copied into that order
int order_pieces(CsrPlan* p, int cap, const Layout& L, char* temp, hipStream_t s)
{
    int* seg = reinterpret_cast<int*>(temp + L.o_seg);
    PieceRec* rec = reinterpret_cast<PieceRec*>(temp + L.o_rec);
    PieceRec* ordered = reinterpret_cast<PieceRec*>(temp + L.o_ord);
    unsigned* keys = reinterpret_cast<unsigned*>(temp + L.o_keys);
    unsigned* keys2 = reinterpret_cast<unsigned*>(temp + L.o_keys2);
    unsigned* perm = reinterpret_cast<unsigned*>(temp + L.o_perm);
    unsigned* order = reinterpret_cast<unsigned*>(temp + L.o_perm2);
    int* hist = reinterpret_cast<int*>(temp + L.o_hist);
    int bits = 1;
    while (bits < 31 && (1ll << bits) < (long long)p->k) ++bits;
    const int shift = bits > 16 ? bits - 16 : 0;
    hipLaunchKernelGGL(piece_fill_kernel, dim3(kElemGrid), dim3(kBlock), 0, s, p->m, p->slots, p->row_ptr, cap, p->col_idx, p->first,
                       p->pfirst, shift, rec, keys);
    // two stable passes, low digit first: order[i] = id of the piece that comes i-th by the top 16 bits of its first column
    if (int rc = radix_order_by_digit(keys, p->slots, 0, keys2, perm, hist, seg, s)) return rc;
    if (int rc = radix_order_by_digit(keys2, p->slots, 8, keys, order, hist, seg, s, perm)) return rc;
    hipLaunchKernelGGL(piece_place_kernel, dim3(kElemGrid), dim3(kBlock), 0, s, p->slots, p->pslots, order, rec, ordered, p->at, p->target);
    if (int rc = exclusive_scan_i32(p->at, p->slots + 1, seg, s)) return rc;
    hipLaunchKernelGGL(piece_gather_kernel, dim3(kElemGrid), dim3(kBlock), 0, s, p->first + p->m, ordered, p->at, p->col_idx, p->val,
                       p->col_ord, p->val_ord);
    GNNHIP_LAUNCH_CHECK("spmm_pieces plan");
    return GNNHIP_OK;
}

void point_plan(CsrPlan* p, const Layout& L, char* head, char* body)
{
    p->first = reinterpret_cast<int*>(head + L.o_first);
    p->pfirst = reinterpret_cast<int*>(head + L.o_pfirst);
    p->at = reinterpret_cast<int*>(body + L.o_at);
    p->target = reinterpret_cast<int*>(body + L.o_target);
    p->col_ord = reinterpret_cast<int*>(body + L.o_col);
    p->val_ord = reinterpret_cast<float*>(body + L.o_val);
}

// The sums over a finished plan: C = alpha * A * B + beta * C.  `part` holds p->pslots rows of w.ldp floats;
// hub_store: where the balanced pass over P keeps its arrays (null: stream scratch slot 1, which the caller has reserved).
int run_pieces(const CsrPlan* p, const Width& w, int n, float alpha, const float* B, int ldb, float beta, float* C, int ldc, float* part,
               bool hub_planned, HubStore* hub_store, bool skip_empty, hipStream_t s)
{
    const int m = p->m, logG = w.logG, iters = w.iters, ldp = w.ldp;
    // workgroups for the bound on the pieces of one die, times the number of dies; those past the real count leave at once
    const int sum_groups = kBlock >> logG;
    const unsigned sgrid = (unsigned)(((p->slots + kNumXCD - 1) / kNumXCD + 1 + sum_groups - 1) / sum_groups) * kNumXCD;
#define GNNHIP_PIECES_LAUNCH(V, I)                                                                                            \
    hipLaunchKernelGGL((piece_sum_kernel<V, I>), dim3(sgrid), dim3(kBlock), 0, s, p->first + m, n, alpha, p->at, p->col_ord, p->val_ord, B, \
                       ldb, part, ldp, logG, p->target, beta, C, ldc)
    if (w.vec4) {
        if (iters <= 1) GNNHIP_PIECES_LAUNCH(4, 1);
        else if (iters == 2) GNNHIP_PIECES_LAUNCH(4, 2);
        else GNNHIP_PIECES_LAUNCH(4, 4);
    } else {
        if (iters <= 1) GNNHIP_PIECES_LAUNCH(1, 1);
        else if (iters == 2) GNNHIP_PIECES_LAUNCH(1, 2);
        else GNNHIP_PIECES_LAUNCH(1, 4);
    }
#undef GNNHIP_PIECES_LAUNCH
    GNNHIP_LAUNCH_CHECK("spmm_pieces sums");
    if (!p->owned) {
        // rows past the host's entry count, if any (a plan of its own knows the matrix's count)
        const unsigned tgrid = kNumCU * 4;
#define GNNHIP_PIECES_TAIL(V, I)                                                                                                   \
    hipLaunchKernelGGL((piece_tail_kernel<V, I>), dim3(tgrid), dim3(kBlock), 0, s, m, n, alpha, p->row_ptr, (int)p->nnz, p->col_idx, p->val, \
                       B, ldb, beta, C, ldc, logG)
        if (w.vec4) {
            if (iters <= 1) GNNHIP_PIECES_TAIL(4, 1);
            else if (iters == 2) GNNHIP_PIECES_TAIL(4, 2);
            else GNNHIP_PIECES_TAIL(4, 4);
        } else {
            if (iters <= 1) GNNHIP_PIECES_TAIL(1, 1);
            else if (iters == 2) GNNHIP_PIECES_TAIL(1, 2);
            else GNNHIP_PIECES_TAIL(1, 4);
        }
#undef GNNHIP_PIECES_TAIL
        GNNHIP_LAUNCH_CHECK("spmm_pieces tail");
    }
    // the rows of very many pieces: the balanced pass over long rows, on P times part (P: row pointers pfirst, entry j
    // = column j with weight 1, which that pass takes when it is handed no index and value arrays)
    // (`pslots` stands in for the number of entries of P: an upper bound is all that pass needs; a row of more than
    // kCombineLong pieces has more than kCombineLong * kPiece entries, which bounds the number of such rows)
    HubPlan hubs;
    if (int rc = hub_prepass(m, n, p->pslots, p->pfirst, nullptr, nullptr, part, ldp, s, &hubs, hub_planned, false, kCombineLong,
                             kCombineChunk, p->nnz / ((long long)kCombineLong * kPiece + 1) + 1, hub_store))
        return rc;
    const unsigned grid = (unsigned)(((long long)m + kBlock - 1) / kBlock);        // a wavefront per 64 rows
#define GNNHIP_PIECES_COMBINE(V, I)                                                                                             \
    hipLaunchKernelGGL((piece_combine_kernel<V, I>), dim3(grid), dim3(kBlock), 0, s, m, n, p->first, p->pfirst, part, ldp, beta, C, ldc, \
                       logG, hubs.row_slot, hubs.agg, hubs.ld, skip_empty ? 1 : 0)
    if (w.vec4) {
        if (iters <= 1) GNNHIP_PIECES_COMBINE(4, 1);
        else if (iters == 2) GNNHIP_PIECES_COMBINE(4, 2);
        else GNNHIP_PIECES_COMBINE(4, 4);
    } else {
        if (iters <= 1) GNNHIP_PIECES_COMBINE(1, 1);
        else if (iters == 2) GNNHIP_PIECES_COMBINE(1, 2);
        else GNNHIP_PIECES_COMBINE(1, 4);
    }
#undef GNNHIP_PIECES_COMBINE
    GNNHIP_LAUNCH_CHECK("spmm_pieces combine");
    return GNNHIP_OK;
}

// What the scratch of a stream holds a plan for: kept per stream, next to the scratch it describes, so that whichever
// thread plans on the stream replaces it.
// (these registries are never destroyed: a caller's static objects may still hand plans back while the process exits)
std::mutex& g_memo_mu = *new std::mutex;
std::map<hipStream_t, CsrPlan>& g_memo = *new std::map<hipStream_t, CsrPlan>;

std::mutex& g_plans_mu = *new std::mutex;
std::set<CsrPlan*>& g_plans = *new std::set<CsrPlan*>;

}  // namespace

bool pieces_route_applies(int m, long long nnz)
{
    return m >= kHubMinRows && nnz >= kPiecesMeanDegree * (long long)m && nnz < (1ll << 31) - 64 && slots_bound(m, nnz) < (1ll << 31) - 64;
}

CsrPlan* as_csr_plan(void* handle)
{
    CsrPlan* p = static_cast<CsrPlan*>(handle);
    std::lock_guard<std::mutex> lock(g_plans_mu);
    return (p && g_plans.count(p) && p->magic == kCsrPlanMagic) ? p : nullptr;
}

// C = alpha * A * B + beta * C through the column-ordered pieces.  With `plan` (made by gnnhip_csr_plan_create for these
// arrays) nothing is planned here; without it the plan is made in the stream's scratch, sized for the host's bounds, and
// reused when reuse_plan says the previous call on the stream had the same matrix (structure and values).
// All scratch is taken before the first launch: GNNHIP_ENOMEM and GNNHIP_EUNSUPPORTED leave C untouched.
int spmm_pieces_dispatch(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                         const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan, bool skip_empty_rows,
                         CsrPlan* plan)
{
    const Width w = width_of(n, B, ldb, C, ldc);
    if (!w.ok) return GNNHIP_EUNSUPPORTED;
    if (skip_empty_rows && beta != 0.f) return set_error(GNNHIP_EINVAL, "rows without entries can only be skipped when beta is 0");
    if (plan) {
        if (!plan->has_pieces) return GNNHIP_EUNSUPPORTED;
        const size_t need = sizeof(float) * (size_t)(plan->pslots > 0 ? plan->pslots : 1) * w.ldp;
        if (plan->part_bytes < need) {
            if (plan->part) {
                GNNHIP_HIP(hipStreamSynchronize(s));
                (void)pool_free(plan->part);
                plan->part = nullptr;
                plan->part_bytes = 0;
            }
            void* q = nullptr;
            if (int rc = pool_acquire_exact(&q, need)) return rc;
            plan->part = static_cast<float*>(q);
            plan->part_bytes = need;
        }
        // the balanced pass over P takes its block before anything is launched (it is the only other allocation)
        const size_t hb = hub_scratch_bytes(m, n, plan->pslots, kCombineLong, kCombineChunk, plan->nnz / ((long long)kCombineLong * kPiece + 1) + 1);
        if (hb > plan->combine_hub.bytes) {
            if (plan->combine_hub.base) {
                GNNHIP_HIP(hipStreamSynchronize(s));
                (void)pool_free(plan->combine_hub.base);
                plan->combine_hub = HubStore{};
            }
            if (int rc = pool_acquire_exact(&plan->combine_hub.base, hb)) return rc;
            plan->combine_hub.bytes = hb;
        }
        return run_pieces(plan, w, n, alpha, B, ldb, beta, C, ldc, plan->part, true, &plan->combine_hub, skip_empty_rows, s);
    }

    if (!pieces_route_applies(m, nnz)) return GNNHIP_EUNSUPPORTED;
    CsrPlan p;
    p.row_ptr = row_ptr; p.col_idx = col_idx; p.val = val;
    p.m = m; p.k = k; p.nnz = nnz;
    p.slots = slots_bound(m, nnz);
    p.pslots = pslots_bound(nnz) < p.slots ? pslots_bound(nnz) : p.slots;
    p.has_pieces = true;
    const Layout L = layout_of(m, nnz, p.slots, p.pslots);
    void *base = nullptr, *pbase = nullptr, *hbase = nullptr;
    if (int rc = stream_scratch_slot(s, 3, L.head_bytes + L.body_bytes + L.temp_bytes, &base)) return rc;
    if (int rc = stream_scratch_slot(s, 4, sizeof(float) * (size_t)p.pslots * w.ldp, &pbase)) return rc;
    // the balanced pass over P reserves its scratch now: past this point nothing can fail for lack of memory, so a
    // caller that falls back to another route on GNNHIP_ENOMEM finds C untouched
    if (const size_t hb = hub_scratch_bytes(m, n, p.pslots, kCombineLong, kCombineChunk, nnz / ((long long)kCombineLong * kPiece + 1) + 1))
        if (int rc = stream_scratch_slot(s, 1, hb, &hbase)) return rc;
    char* b = static_cast<char*>(base);
    point_plan(&p, L, b, b + L.head_bytes);
    char* temp = b + L.head_bytes + L.body_bytes;

    bool planned = false;
    {
        std::lock_guard<std::mutex> lock(g_memo_mu);
        auto it = g_memo.find(s);
        planned = reuse_plan && it != g_memo.end() && it->second.row_ptr == row_ptr && it->second.col_idx == col_idx &&
                  it->second.val == val && it->second.m == m && it->second.k == k && it->second.nnz == nnz && it->second.first == p.first;
        if (!planned) g_memo[s] = p;
    }
    if (!planned) {
        if (int rc = count_pieces(&p, (int)nnz, reinterpret_cast<int*>(temp + L.o_seg), s)) return rc;
        if (int rc = order_pieces(&p, (int)nnz, L, temp, s)) return rc;
    }
    return run_pieces(&p, w, n, alpha, B, ldb, beta, C, ldc, static_cast<float*>(pbase), planned, nullptr, skip_empty_rows, s);
}

}  // namespace gnnhip

using namespace gnnhip;

extern "C" int gnnhip_csr_plan_create(int m, int k, const int* row_ptr, const int* col_idx, const float* val, void* stream, void** plan)
{
    GNNHIP_REQUIRE(plan, "null plan output");
    *plan = nullptr;
    GNNHIP_REQUIRE(m >= 0 && k >= 0, "negative dimension in csr_plan_create (m=%d k=%d)", m, k);
    GNNHIP_REQUIRE(row_ptr, "null row_ptr in csr_plan_create");
    if (int rc = require_ready()) return rc;
    hipStream_t s = as_stream(stream);
    // the matrix's own entry count
    int nnz = 0;
    GNNHIP_HIP(hipMemcpyAsync(&nnz, row_ptr + m, sizeof(int), hipMemcpyDeviceToHost, s));
    GNNHIP_HIP(hipStreamSynchronize(s));
    GNNHIP_REQUIRE(nnz >= 0, "row_ptr[m] is negative (%d)", nnz);
    GNNHIP_REQUIRE(nnz == 0 || (col_idx && val), "null col_idx or val for a matrix with entries");
    CsrPlan* p = new CsrPlan();
    p->magic = kCsrPlanMagic;
    p->row_ptr = row_ptr; p->col_idx = col_idx; p->val = val;
    p->m = m; p->k = k; p->nnz = nnz;
    p->owned = true;
    auto fail = [&](int rc) {
        if (p->head_block) (void)pool_free(p->head_block);
        if (p->body_block) (void)pool_free(p->body_block);
        delete p;
        return rc;
    };
    if (pieces_route_applies(m, nnz)) {
        // counts first (they need the head block only), then the arrays at the size the matrix really needs
        Layout L = layout_of(m, nnz, 1, 1);
        if (int rc = pool_acquire_exact(&p->head_block, L.head_bytes)) return fail(rc);
        void* segp = nullptr;
        if (int rc = stream_scratch(s, sizeof(int) * ((size_t)m / 4096 + 4), &segp)) return fail(rc);
        point_plan(p, L, static_cast<char*>(p->head_block), nullptr);
        if (int rc = count_pieces(p, nnz, static_cast<int*>(segp), s)) return fail(rc);
        int totals[2] = {0, 0};
        GNNHIP_HIP(hipMemcpyAsync(&totals[0], p->first + m, sizeof(int), hipMemcpyDeviceToHost, s));
        GNNHIP_HIP(hipMemcpyAsync(&totals[1], p->pfirst + m, sizeof(int), hipMemcpyDeviceToHost, s));
        GNNHIP_HIP(hipStreamSynchronize(s));
        p->slots = totals[0] > 0 ? totals[0] : 1;
        p->pslots = totals[1] > 0 ? totals[1] : 1;
        L = layout_of(m, nnz, p->slots, p->pslots);
        if (int rc = pool_acquire_exact(&p->body_block, L.body_bytes)) return fail(rc);
        // the temporary arrays come from the pool and go back there (the next plan of a matrix of this size takes them)
        void* temp = nullptr;
        if (int rc = pool_acquire(&temp, L.temp_bytes)) return fail(rc);
        point_plan(p, L, static_cast<char*>(p->head_block), static_cast<char*>(p->body_block));
        int rc = order_pieces(p, nnz, L, static_cast<char*>(temp), s);
        hipError_t e = hipStreamSynchronize(s);
        (void)pool_release(temp);
        if (rc) return fail(rc);
        if (e != hipSuccess) return fail(set_error(GNNHIP_EHIP, "csr_plan_create: %s", hipGetErrorString(e)));
        p->has_pieces = true;
    }
    {
        std::lock_guard<std::mutex> lock(g_plans_mu);
        g_plans.insert(p);
    }
    *plan = p;
    return GNNHIP_OK;
}

extern "C" int gnnhip_csr_plan_destroy(void* plan)
{
    if (!plan) return GNNHIP_OK;
    CsrPlan* p = static_cast<CsrPlan*>(plan);
    {
        std::lock_guard<std::mutex> lock(g_plans_mu);
        if (!g_plans.erase(p)) return set_error(GNNHIP_EINVAL, "%p is not a live CSR plan", plan);
    }
    if (runtime_ready()) {
        (void)hipDeviceSynchronize();                               // launches that read the plan's arrays may still be queued
        for (void* q : {p->head_block, p->body_block, static_cast<void*>(p->part), p->combine_hub.base, p->row_hub.base})
            if (q) (void)pool_free(q);
    }
    p->magic = 0;
    delete p;
    return GNNHIP_OK;
}

extern "C" int gnnhip_csr_plan_bytes(void* plan, size_t* bytes)
{
    GNNHIP_REQUIRE(bytes, "null output in csr_plan_bytes");
    CsrPlan* p = as_csr_plan(plan);
    GNNHIP_REQUIRE(p, "%p is not a live CSR plan", plan);
    size_t total = p->part_bytes + p->combine_hub.bytes + p->row_hub.bytes;
    if (p->has_pieces) {
        const Layout L = layout_of(p->m, p->nnz, p->slots, p->pslots);
        total += L.head_bytes + L.body_bytes;
    }
    *bytes = total;
    return GNNHIP_OK;
}
