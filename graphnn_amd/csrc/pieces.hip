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

#include <cstdlib>

namespace gnnhip {
namespace {

constexpr int kBlock = 256;
constexpr int kPiece = 32;              // entries per piece

// entries [start, end); id = first[row] + index of the piece in its row; row: the row when the piece is all of it
// and holds entries (then its sum is the row's result), else -1
struct PieceRec { int start, end, id, row; };

__device__ __forceinline__ int pieces_of(int deg) { return (deg + kPiece - 1) / kPiece; }

// counts[r] = pieces of row r (counts[m] = 0, so that the scan leaves the total there).  The host's entry count
// `cap` sizes every array of the plan; should the matrix hold more entries than that, a row that reaches past
// entry `cap` (the last rows) is one piece whatever its length: no entries are copied for it, and
// piece_tail_kernel forms the row's result from the CSR arrays.
__global__ __launch_bounds__(kBlock) void piece_count_kernel(int m, const int* __restrict__ row_ptr, int cap, int* __restrict__ counts)
{
    for (long long r = (long long)blockIdx.x * kBlock + threadIdx.x; r <= m; r += (long long)gridDim.x * kBlock) {
        int c = 0;
        if (r < m) {
            const int e0 = row_ptr[r], e1 = row_ptr[r + 1];
            c = e1 <= cap ? pieces_of(e1 - e0) : (e1 > e0 ? 1 : 0);
        }
        counts[r] = c;
    }
}

// One lane per piece slot: the row that owns piece id is found by bisection in the scanned counts.
// Slots at or past the number of pieces get an empty record and the largest key (they sort to the end).
__global__ __launch_bounds__(kBlock) void piece_fill_kernel(int m, long long slots, const int* __restrict__ row_ptr, int cap,
                                                            const int* __restrict__ col_idx, const int* __restrict__ first,
                                                            int shift, PieceRec* __restrict__ rec, unsigned* __restrict__ keys)
{
    const int total = first[m];
    for (long long id = (long long)blockIdx.x * kBlock + threadIdx.x; id < slots; id += (long long)gridDim.x * kBlock) {
        if (id >= total) {
            rec[id] = PieceRec{0, 0, (int)id, -1};
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
        rec[id] = PieceRec{start, end, (int)id, (end > start && first[row + 1] - first[row] == 1) ? row : -1};
        keys[id] = ((unsigned)col_idx[start] >> shift) & 0xFFFFu;
    }
}

// lens[i] = entries of the i-th piece in order (lens[slots] = 0, so that the scan leaves the total there);
// where[i] = i and ones[i] = 1: the matrix that picks the pieces of a row (the sums are stored by piece id, so the
// pieces of a row lie next to each other and the combining pass reads them front to back);
// target[i]: where the sum of the i-th piece in order goes: the row r >= 0 when the piece is all of that row,
// else -1 - id, its place among the partial sums.  order[i] = id of the i-th piece in order; ordered[i] = its record.
__global__ __launch_bounds__(kBlock) void piece_place_kernel(long long slots, const unsigned* __restrict__ order,
                                                             const PieceRec* __restrict__ rec, PieceRec* __restrict__ ordered,
                                                             int* __restrict__ lens, int* __restrict__ where, float* __restrict__ ones,
                                                             int* __restrict__ target)
{
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i <= slots; i += (long long)gridDim.x * kBlock) {
        if (i == slots) { lens[i] = 0; continue; }
        const PieceRec r = rec[order[i]];
        ordered[i] = r;
        lens[i] = r.end - r.start;
        where[i] = (int)i;
        ones[i] = 1.f;
        target[i] = r.row >= 0 ? r.row : -1 - r.id;
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
// has its result already.  part holds the sums by piece id: row r owns part[first[r] .. first[r + 1]).  A lane group
// takes kRun consecutive rows, whose pieces are one contiguous stretch of part, and adds each row's pieces in
// piece order, eight loads in flight.  A row of more than kCombineLong pieces takes its sum from the balanced
// pass (hub_slot / hub_agg) when that pass has one for it: on a power-law matrix the rows of many pieces sit next
// to each other, and summed here they kept an eighth of the wavefronts busy for the whole launch.
constexpr int kRun = 8;
constexpr int kCombineLong = 8;         // pieces; the balanced pass cuts such rows into chunks of kCombineChunk pieces
constexpr int kCombineChunk = 256;
template <int VEC, int ITERS>
__global__ __launch_bounds__(kBlock) void piece_combine_kernel(
    int m, int n, const int* __restrict__ first, const float* __restrict__ part, int ldp, float beta, float* __restrict__ C, int ldc,
    int logG, const int* __restrict__ hub_slot, const float* __restrict__ hub_agg, int hub_ld)
{
    using V = PV<VEC>;
    constexpr int kFlight = 8;
    const int G = 1 << logG;                       // at least 8 lanes (the route's narrowest operand): a lane per row of the run
    const int sub = threadIdx.x & (G - 1);
    const int grp = threadIdx.x >> logG;
    const int ngroups = kBlock >> logG;
    const long long row0 = ((long long)blockIdx.x * ngroups + grp) * kRun;
    if (row0 >= m) return;
    // lane j < kRun of the group holds the bounds of row row0 + j
    const long long mine = row0 + (sub < kRun ? sub : 0);
    const int my_b = first[mine < m ? mine : m], my_e = first[mine + 1 < m ? mine + 1 : m];
    const int rows = (int)((long long)m - row0 < kRun ? (long long)m - row0 : kRun);
    for (int j = 0; j < rows; ++j) {
        const int b = __shfl(my_b, j, G), e = __shfl(my_e, j, G);
        const int cnt = e - b;
        if (cnt == 1) continue;
        const long long row = row0 + j;
        typename V::T acc[ITERS];
#pragma unroll
        for (int it = 0; it < ITERS; ++it) acc[it] = V::zero();
        int hslot = -1;
        if (hub_slot && cnt > kCombineLong) hslot = hub_slot[row];
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

// Mean entries per row from which a matrix of at least kHubMinRows rows takes this route;
// GNNHIP_PIECES_DEGREE overrides it (read once; 0 switches the route off), which is how the crossover was measured.
inline long long pieces_degree()
{
    static const long long d = [] {
        const char* e = getenv("GNNHIP_PIECES_DEGREE");
        return (e && *e) ? atoll(e) : 12ll;
    }();
    return d;
}

}  // namespace

// The partial sums alpha * (piece of A) * B of every piece, in column order, and the matrix P that picks the pieces of
// each row (out->first / where / ones: CSR arrays of P [m, out->slots], out->part: the sums, row stride out->ld);
// A * B is P * part.  The rows of exactly one piece are finished here (C[row] = sum + beta * C[row]); the caller
// combines the others.  GNNHIP_EUNSUPPORTED (nothing launched) where the caller keeps its own route.
int spmm_pieces_sums(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                     const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan, PiecesOperand* out)
{
    const long long deg = pieces_degree();
    if (deg <= 0 || m < kHubMinRows || nnz < deg * (long long)m || nnz >= (1ll << 31) - 64) return GNNHIP_EUNSUPPORTED;
    const bool vec4 = (n % 4 == 0) && (ldb % 4 == 0) && (ldc % 4 == 0) && aligned16(B) && aligned16(C);
    const int vec = vec4 ? 4 : 1;
    const int units = (n + vec - 1) / vec;
    // a lane group covers at most 64 x 4 column units (wider operands stay with the caller's route, which cuts them into slabs)
    if (units > kWave * 4) return GNNHIP_EUNSUPPORTED;
    // Narrow operands stay with the row-group route: with fewer than eight lanes per piece a wavefront reads the
    // entries of more than eight pieces at once, 128 bytes apart, and fetches whole lines for a few bytes each
    // (width 4 on the 4M-row R-MAT matrix: 16.6 GB fetched, 2.7 ms against 0.26 ms).
    if (units < 8) return GNNHIP_EUNSUPPORTED;
    const int logG = ilog2_ceil_p(units < kWave ? units : kWave);
    const int G = 1 << logG;
    const int iters = (units + G - 1) / G;                        // 1..4 (3 runs as 4)
    const int ldp = (int)round_up_p((size_t)n, 4);

    // Every row has at most one piece that is not full.  The host does not know how many pieces there are, so
    // the arrays and the launches are sized for this bound; the slots past the real pieces hold empty pieces,
    // ordered last, that no row picks.
    const long long slots = nnz / kPiece + m;
    if (slots >= (1ll << 31) - 64) return GNNHIP_EUNSUPPORTED;
    size_t off = 0;
    auto carve = [&](size_t bytes) { const size_t o = off; off = round_up_p(off + bytes, 256); return o; };
    const size_t o_first = carve(sizeof(int) * ((size_t)m + 1)), o_where = carve(sizeof(int) * (size_t)slots);
    const size_t o_at = carve(sizeof(int) * ((size_t)slots + 1)), o_ones = carve(sizeof(float) * (size_t)slots);
    const size_t o_target = carve(sizeof(int) * (size_t)slots);
    const size_t o_col = carve(sizeof(int) * (size_t)nnz), o_val = carve(sizeof(float) * (size_t)nnz);
    const size_t longest = (size_t)(slots + 1 > (long long)m + 1 ? slots + 1 : (long long)m + 1);
    const size_t o_seg = carve(sizeof(int) * (longest / 4096 + 2 + radix_seg_ints(slots)));
    const size_t o_rec = carve(sizeof(PieceRec) * (size_t)slots), o_ord = carve(sizeof(PieceRec) * (size_t)slots);
    const size_t o_keys = carve(sizeof(unsigned) * (size_t)slots), o_keys2 = carve(sizeof(unsigned) * (size_t)slots);
    const size_t o_perm = carve(sizeof(unsigned) * (size_t)slots), o_perm2 = carve(sizeof(unsigned) * (size_t)slots);
    const size_t o_hist = carve(sizeof(int) * radix_hist_ints(slots));
    void* base = nullptr;
    if (int rc = stream_scratch_slot(s, 3, off, &base)) return rc;
    void* pbase = nullptr;
    if (int rc = stream_scratch_slot(s, 4, sizeof(float) * (size_t)slots * ldp, &pbase)) return rc;
    char* b = static_cast<char*>(base);
    int* first = reinterpret_cast<int*>(b + o_first);
    int* where = reinterpret_cast<int*>(b + o_where);
    int* at = reinterpret_cast<int*>(b + o_at);
    float* ones = reinterpret_cast<float*>(b + o_ones);
    int* target = reinterpret_cast<int*>(b + o_target);
    int* col_ord = reinterpret_cast<int*>(b + o_col);
    float* val_ord = reinterpret_cast<float*>(b + o_val);
    int* seg = reinterpret_cast<int*>(b + o_seg);
    PieceRec* rec = reinterpret_cast<PieceRec*>(b + o_rec);
    PieceRec* ordered = reinterpret_cast<PieceRec*>(b + o_ord);
    unsigned* keys = reinterpret_cast<unsigned*>(b + o_keys);
    unsigned* keys2 = reinterpret_cast<unsigned*>(b + o_keys2);
    unsigned* perm = reinterpret_cast<unsigned*>(b + o_perm);
    unsigned* order = reinterpret_cast<unsigned*>(b + o_perm2);
    int* hist = reinterpret_cast<int*>(b + o_hist);
    float* part = static_cast<float*>(pbase);

    struct Memo { hipStream_t s; const int* row_ptr; const int* col_idx; const float* val; int m; long long nnz; void* base; };
    static thread_local Memo memo = {nullptr, nullptr, nullptr, nullptr, 0, 0, nullptr};
    const bool planned = reuse_plan && memo.row_ptr == row_ptr && memo.col_idx == col_idx && memo.val == val && memo.s == s &&
                         memo.m == m && memo.nnz == nnz && memo.base == base;
    const unsigned egrid = kNumCU * 16;
    if (!planned) {
        hipLaunchKernelGGL(piece_count_kernel, dim3(egrid), dim3(kBlock), 0, s, m, row_ptr, (int)nnz, first);
        if (int rc = exclusive_scan_i32(first, (long long)m + 1, seg, s)) return rc;
        int bits = 1;
        while (bits < 31 && (1ll << bits) < (long long)k) ++bits;
        const int shift = bits > 16 ? bits - 16 : 0;
        hipLaunchKernelGGL(piece_fill_kernel, dim3(egrid), dim3(kBlock), 0, s, m, slots, row_ptr, (int)nnz, col_idx, first, shift, rec, keys);
        // two stable passes, low digit first: order[i] = id of the piece that comes i-th by the top 16 bits of its first column
        if (int rc = radix_order_by_digit(keys, slots, 0, keys2, perm, hist, seg, s)) return rc;
        if (int rc = radix_order_by_digit(keys2, slots, 8, keys, order, hist, seg, s, perm)) return rc;
        hipLaunchKernelGGL(piece_place_kernel, dim3(egrid), dim3(kBlock), 0, s, slots, order, rec, ordered, at, where, ones, target);
        if (int rc = exclusive_scan_i32(at, slots + 1, seg, s)) return rc;
        hipLaunchKernelGGL(piece_gather_kernel, dim3(egrid), dim3(kBlock), 0, s, first + m, ordered, at, col_idx, val, col_ord, val_ord);
        GNNHIP_LAUNCH_CHECK("spmm_pieces plan");
        memo = Memo{s, row_ptr, col_idx, val, m, nnz, base};
    }
    // workgroups for the bound on the pieces of one die, times the number of dies
    const int sum_groups = kBlock >> logG;
    const unsigned sgrid = (unsigned)(((slots + kNumXCD - 1) / kNumXCD + 1 + sum_groups - 1) / sum_groups) * kNumXCD;
#define GNNHIP_PIECES_LAUNCH(V, I)                                                                                               \
    hipLaunchKernelGGL((piece_sum_kernel<V, I>), dim3(sgrid), dim3(kBlock), 0, s, first + m, n, alpha, at, col_ord, val_ord, B, ldb, \
                       part, ldp, logG, target, beta, C, ldc)
    if (vec4) {
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
    // rows past the host's entry count, if any
    const unsigned tgrid = kNumCU * 4;
#define GNNHIP_PIECES_TAIL(V, I)                                                                                                  \
    hipLaunchKernelGGL((piece_tail_kernel<V, I>), dim3(tgrid), dim3(kBlock), 0, s, m, n, alpha, row_ptr, (int)nnz, col_idx, val, \
                       B, ldb, beta, C, ldc, logG)
    if (vec4) {
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
    out->first = first;
    out->where = where;
    out->ones = ones;
    out->part = part;
    out->ld = ldp;
    out->slots = slots;
    out->plan_reused = planned;
    return GNNHIP_OK;
}

int spmm_pieces_dispatch(int m, int k, int n, long long nnz, float alpha, const int* row_ptr, const int* col_idx, const float* val,
                         const float* B, int ldb, float beta, float* C, int ldc, hipStream_t s, bool reuse_plan)
{
    PiecesOperand po;
    if (int rc = spmm_pieces_sums(m, k, n, nnz, alpha, row_ptr, col_idx, val, B, ldb, beta, C, ldc, s, reuse_plan, &po)) return rc;
    // the rows of very many pieces: the balanced pass over long rows, on P = (first, where, ones) times part
    // (`slots` stands in for the number of entries of P: an upper bound is all that pass needs)
    HubPlan hubs;
    // (a row of more than kCombineLong pieces has more than kCombineLong * kPiece entries: that bounds their number)
    if (int rc = hub_prepass(m, n, po.slots, po.first, po.where, po.ones, po.part, po.ld, s, &hubs, po.plan_reused, false, kCombineLong,
                             kCombineChunk, nnz / ((long long)kCombineLong * kPiece + 1) + 1))
        return rc;
    const bool vec4 = (n % 4 == 0) && (ldb % 4 == 0) && (ldc % 4 == 0) && aligned16(B) && aligned16(C);
    const int vec = vec4 ? 4 : 1;
    const int units = (n + vec - 1) / vec;
    const int logG = ilog2_ceil_p(units < kWave ? units : kWave);
    const int iters = (units + (1 << logG) - 1) >> logG;
    const unsigned grid = (unsigned)(((long long)m + (long long)(kBlock >> logG) * kRun - 1) / ((long long)(kBlock >> logG) * kRun));
#define GNNHIP_PIECES_COMBINE(V, I)                                                                                           \
    hipLaunchKernelGGL((piece_combine_kernel<V, I>), dim3(grid), dim3(kBlock), 0, s, m, n, po.first, po.part, po.ld, beta, C, ldc, \
                       logG, hubs.row_slot, hubs.agg, hubs.ld)
    if (vec4) {
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

}  // namespace gnnhip
