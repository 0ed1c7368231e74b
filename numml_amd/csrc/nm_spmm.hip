// CSR x dense (SpMM) forward and backward for gfx950.
//
// Forward: lane = output column (a 64-column fp32 row of B is one 256-byte
// line, so every gather is a single coalesced request).  A wavefront owns a few
// consecutive rows of A and walks their entries as one range, 64 (column,
// value) pairs per coalesced load, read back entry by entry into scalar
// registers (so that a gather is a scalar row address plus one shared vector
// of lane offsets); every lane adds its column's terms in storage order and
// restarts at row boundaries --
// the order of the serial CPU loop (cpp/sparse_csr_cpu.cpp:586-598), so C
// matches it bit for bit.  Rows longer than kSplitRow are shared by the
// wavefronts of a workgroup instead (partial sums added in wavefront order:
// deterministic, equal to rounding).
//
// Backward: the same mapping computes, per stored entry, the dot product of
// gC[row,:] and B[col,:] (cross-lane reduction) and scatters
// data[k] * gC[row,:] into grad_B[col,:] with hardware atomics.
//
// Algorithmic HBM bytes (s = sizeof(value), n = dense columns):
//   forward : nnz*(s+8) + (rows+1)*8 + cols*n*s + rows*n*s
//   backward: nnz*(s+8) + (rows+1)*8 + rows*n*s + cols*n*s + nnz*s + cols*n*s
#include "nm_common.hpp"
#include "nm_transpose.hpp"

namespace {

using nm::kWave;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

constexpr int kBatch = 8;                    // gathers a wavefront keeps in flight in the backward
constexpr int kSplitRow = 512;               // rows longer than this are shared by the workgroup's wavefronts

// acc += sum over entries [kb, ke) of value * B[col, c], terms added in storage
// order.  Entries are fetched 64 at a time (one coalesced load each for column
// and value) and broadcast lane by lane; gathers of B go out eight (then four)
// at a time so that a wavefront keeps several 256-byte requests in flight.
// IDX is the structure's index type (int64 for A as delivered, int32 for the
// transposed-structure plan); with PERM the value of entry k is data[perm[k]]
// (A^T shares A's value array through the plan's permutation).
template <typename T, typename IDX, bool PERM>
__device__ __forceinline__ T row_times_dense(T acc, int64_t kb0, int64_t ke0, const T *__restrict__ data,
                                             const IDX *__restrict__ indices, const int32_t *__restrict__ perm,
                                             const T *__restrict__ Bc, int64_t ldb, int lane) {
    for (int64_t kb = kb0; kb < ke0; kb += kWave) {
        const int64_t k = kb + lane;
        const int64_t mycol = k < ke0 ? (int64_t)indices[k] : 0;
        const T myval = k < ke0 ? (PERM ? data[perm[k]] : data[k]) : T(0);
        const int cnt = (int)(ke0 - kb < kWave ? ke0 - kb : kWave);
        int j = 0;
        for (; j + 8 <= cnt; j += 8) {
            T bv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) bv[u] = Bc[__shfl(mycol, j + u, kWave) * ldb];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += __shfl(myval, j + u, kWave) * bv[u];
        }
        for (; j < cnt; j += 4) {
            T bv[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) bv[u] = Bc[__shfl(mycol, j + u < cnt ? j + u : j, kWave) * ldb];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (j + u < cnt) acc += __shfl(myval, j + u, kWave) * bv[u];
        }
    }
    return acc;
}

// C = A B (or, on the plan, A^T B).  A wavefront of a "walker" workgroup owns
// kFlatRows consecutive rows and walks their entries as one range: 64 entries per
// coalesced load whatever the row lengths (a 15-entry row per load would leave 3/4 of
// the lanes idle and cost a memory round trip per row), the next 64 requested while
// the current ones are used, gathers of B eight at a time.  Lane = dense column; the
// running sum is stored and restarted at every row boundary, so each row is still
// added in storage order.  Rows longer than kSplitRow are skipped by the walkers
// (their entries are jumped over) and computed by the "scout" workgroups at the head
// of the grid.
constexpr int kFlatRows = 8;
constexpr int kScoutRows = 64;   // rows a scout workgroup inspects for long ones
constexpr int kColsPerSlice = 1024;   // dense columns one workgroup walks (wider operands: more workgroups)

// The work of a "scout" workgroup (the first ceil(rows / kScoutRows) of the grid): look for
// long rows among kScoutRows rows and share every one found among the workgroup's
// wavefronts (contiguous parts, partial sums added in wavefront order: deterministic, equal
// to the serial sum to rounding).  Lane = dense column.
template <typename T, typename IDX, bool PERM>
__device__ __forceinline__ void scout_long_rows(int64_t rows, const T *__restrict__ data,
                                                const IDX *__restrict__ indices, const IDX *__restrict__ indptr,
                                                const int32_t *__restrict__ perm, const T *__restrict__ B,
                                                int64_t ldb, int64_t n, T *__restrict__ C, int64_t ldc, int lane,
                                                int wave) {
    __shared__ T s_part[kWavesPerBlock][kWave];
    __shared__ int s_long[kScoutRows];
    __shared__ int s_nlong;
    const int64_t g0 = (int64_t)blockIdx.x * kScoutRows;
    if (threadIdx.x == 0) s_nlong = 0;
    __syncthreads();
    for (int t = threadIdx.x; t < kScoutRows && g0 + t < rows; t += kBlock)
        if (indptr[g0 + t + 1] - indptr[g0 + t] > kSplitRow) s_long[atomicAdd(&s_nlong, 1)] = t;
    __syncthreads();
    const int nl = s_nlong;
    for (int li = 0; li < nl; ++li) {   // uniform over the workgroup; the order of the list does not matter
        const int64_t row = g0 + s_long[li];
        const int64_t rb = indptr[row], re = indptr[row + 1];
        int64_t chunk = (re - rb + kWavesPerBlock - 1) / kWavesPerBlock;
        chunk = (chunk + kWave - 1) / kWave * kWave;
        const int64_t kb = rb + wave * chunk;
        const int64_t ke = kb + chunk < re ? kb + chunk : re;
        for (int64_t c0 = 0; c0 < n; c0 += kWave) {
            const int64_t c = c0 + lane;
            const bool live = c < n;
            T acc = T(0);
            if (kb < re)
                acc = row_times_dense<T, IDX, PERM>(acc, kb, ke, data, indices, perm, B + (live ? c : 0), ldb, lane);
            s_part[wave][lane] = acc;
            __syncthreads();
            if (wave == 0 && live) {
                T sum = s_part[0][lane];
                for (int w = 1; w < kWavesPerBlock; ++w) sum += s_part[w][lane];
                C[row * ldc + c] = sum;
            }
            __syncthreads();
        }
    }
}

template <typename T, typename IDX, bool PERM>
__global__ __launch_bounds__(kBlock) void spdmm_fwd_flat_kernel(
    int64_t rows, const T *__restrict__ data, const IDX *__restrict__ indices,
    const IDX *__restrict__ indptr, const int32_t *__restrict__ perm, const T *__restrict__ B, int64_t ldb,
    int64_t n, T *__restrict__ C, int64_t ldc) {
    const int lane = threadIdx.x & (kWave - 1);
    // (the wavefront index is the same in every lane: telling the compiler so keeps everything
    // derived from it -- row ranges, loop bounds, addresses -- in scalar registers and the
    // control flow free of execution-mask bookkeeping)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // A dense operand of thousands of columns is cut into slices of kColsPerSlice (the grid's
    // second dimension): a wavefront that walked all of them one after the other had 256
    // dependent rounds of loads at 16 384 columns, and a 16 384-row matrix fills the chip with
    // only eight such wavefronts per compute unit.
    {
        const int64_t first = (int64_t)blockIdx.y * kColsPerSlice;
        B += first;
        C += first;
        n = n - first < kColsPerSlice ? n - first : kColsPerSlice;
    }
    // The first `long_blocks` workgroups look for long rows, kScoutRows rows each, and
    // share every one they find among their wavefronts (contiguous parts, partial sums added
    // in wavefront order: deterministic, equal to the serial sum to rounding).  They come
    // first in the grid so that this latency-bound work overlaps with the flat walk.
    const int64_t long_blocks = (rows + kScoutRows - 1) / kScoutRows;
    if ((int64_t)blockIdx.x < long_blocks) {
        scout_long_rows<T, IDX, PERM>(rows, data, indices, indptr, perm, B, ldb, n, C, ldc, lane, wave);
        return;
    }
    const int64_t r0 = (((int64_t)blockIdx.x - long_blocks) * kWavesPerBlock + wave) * kFlatRows;
    if (r0 >= rows) return;
    const int nr = (int)(rows - r0 < kFlatRows ? rows - r0 : kFlatRows);
    // lane l holds indptr[r0 + l], l <= nr
    const int64_t my_ptr = (int64_t)indptr[r0 + (lane <= nr ? lane : nr)];
    auto ptr_of = [&](int l) {
        const long long lo = __builtin_amdgcn_readlane((int)(my_ptr & 0xffffffffll), l);
        const long long hi = __builtin_amdgcn_readlane((int)(my_ptr >> 32), l);
        return (int64_t)((hi << 32) | (lo & 0xffffffffll));
    };
    const int64_t begin = ptr_of(0), end = ptr_of(nr);
    // The wavefronts of a workgroup share one CU, which issues about one scalar and one
    // vector instruction per cycle: with ~35 instructions per entry (64-bit row addresses on
    // the scalar unit, a row-end comparison and two bounds checks per entry) this walk was
    // bound by instruction issue, not by its gathers.  So everything that can be done once
    // per 64 entries is done there, by the lanes: the byte offset of each entry's row of B,
    // and a mask of the entries that end a row.  Per entry that leaves two lane reads and
    // one scalar add for the address, one lane read and one multiply-add for the term, and
    // a bit test for the row boundary.
    const int64_t row_bytes = ldb * (int64_t)sizeof(T);
    for (int64_t c0 = 0; c0 < n; c0 += kWave) {
        const int64_t c = c0 + lane;
        const bool live = c < n;
        const char *__restrict__ Bc = reinterpret_cast<const char *>(B + (live ? c : 0));
        int r = 0;   // current row (relative), its range, whether it is computed here
        int64_t row_begin = begin, row_end = ptr_of(1);
        bool mine = row_end - row_begin <= kSplitRow;
        T acc = T(0);
        auto next_row = [&]() {
            if (mine && live) C[(r0 + r) * ldc + c] = acc;
            acc = T(0);
            ++r;
            row_begin = row_end;
            row_end = ptr_of(r + 1 <= nr ? r + 1 : nr);
            mine = row_end - row_begin <= kSplitRow;
        };
        // leaves the current row and the empty rows after it (stored as zeros)
        auto close_row = [&]() {
            next_row();
            while (r < nr && row_end == row_begin) next_row();
        };
        while (r < nr && row_end == row_begin) next_row();   // empty rows at the head
        int64_t kb = begin;
        auto fetch = [&](int64_t at, int64_t &col, T &val) {
            const int64_t k = at + lane < end ? at + lane : (end > begin ? end - 1 : 0);
            col = end > begin ? (int64_t)indices[k] : 0;
            val = end > begin ? (PERM ? data[perm[k]] : data[k]) : T(0);
        };
        int64_t mycol, nextcol;
        T myval, nextval;
        fetch(kb, mycol, myval);
        while (kb < end) {   // entry kb belongs to row r
            if (!mine) {     // a long row is not computed here: jump over what is left of it
                kb = row_end;
                close_row();
                if (kb >= end) break;
                fetch(kb, mycol, myval);
                continue;
            }
            const int cnt = (int)(end - kb < kWave ? end - kb : kWave);
            fetch(kb + kWave, nextcol, nextval);   // in flight while this chunk is used
            // per lane, once per chunk: where my entry's row of B starts, and whether my entry is
            // the last of its row (its row = number of row starts at or before it)
            const int64_t k = kb + lane;
            const int64_t myoff = mycol * row_bytes;
            int rid = 0;
            for (int l = 1; l < nr; ++l) rid += k >= ptr_of(l) ? 1 : 0;
            const int64_t my_row_end = __shfl(my_ptr, rid + 1, kWave);
            const unsigned long long ends = __ballot(lane < cnt && k + 1 == my_row_end);
            // Two batches of gathers are in flight: the next batch is requested before the
            // current one is added up (stages alternate in place, no copies of pending loads).
            auto gather = [&](int j0, T (&bv)[kBatch]) {
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const int j = __builtin_amdgcn_readfirstlane(j0 + u < cnt ? j0 + u : cnt - 1);
                    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(myoff & 0xffffffffll), j);
                    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(myoff >> 32), j);
                    bv[u] = *reinterpret_cast<const T *>(Bc + (int64_t)(((unsigned long long)hi << 32) | lo));
                }
            };
            auto add_up = [&](int j0, const T (&bv)[kBatch]) {
                const int m = cnt - j0 < kBatch ? cnt - j0 : kBatch;   // entries of this batch
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    if (u >= m) break;
                    const int j = __builtin_amdgcn_readfirstlane(j0 + u);
                    acc += nm::read_lane(myval, j) * bv[u];
                    if ((ends >> j) & 1ull) close_row();
                }
            };
            T bva[kBatch], bvb[kBatch];
            gather(0, bva);
            for (int j0 = 0;; j0 += 2 * kBatch) {
                if (j0 + kBatch < cnt) gather(j0 + kBatch, bvb);
                add_up(j0, bva);
                if (j0 + kBatch >= cnt) break;
                if (j0 + 2 * kBatch < cnt) gather(j0 + 2 * kBatch, bva);
                add_up(j0 + kBatch, bvb);
                if (j0 + 2 * kBatch >= cnt) break;
            }
            kb += cnt;
            mycol = nextcol;
            myval = nextval;
        }
        while (r < nr) next_row();   // rows of a wavefront whose entries ran out before them
    }
}

// Sums over the wavefront of kBatch (= 8) lane-wise products at once.  Three folding steps
// halve the number of vectors while pairing lanes 1, 2 and 4 apart, after which lane l holds
// the partial sum of vector l & 7 over its group of 8 lanes; three more steps add the eight
// groups.  27 instructions instead of 8 full reductions; the result for vector u is in every
// lane with (l & 7) == u.
template <typename T> __device__ __forceinline__ T fold8(const T (&p)[kBatch], int lane) {
    static_assert(kBatch == 8, "fold8 folds eight vectors");
    const bool b0 = lane & 1, b1 = lane & 2, b2 = lane & 4;
    T q[4], r[2];
#pragma unroll
    for (int m = 0; m < 4; ++m)
        q[m] = (b0 ? p[2 * m + 1] : p[2 * m]) + nm::dpp_move<0xB1>(b0 ? p[2 * m] : p[2 * m + 1]);
#pragma unroll
    for (int m = 0; m < 2; ++m)
        r[m] = (b1 ? q[2 * m + 1] : q[2 * m]) + nm::dpp_move<0x4E>(b1 ? q[2 * m] : q[2 * m + 1]);
    T t = (b2 ? r[1] : r[0]) + __shfl_xor(b2 ? r[0] : r[1], 4, kWave);
    t += nm::dpp_move<0x128>(t);          // row_ror 8: the other group of the 16-lane row
    t += __shfl_xor(t, 16, kWave);
    t += __shfl_xor(t, 32, kWave);
    return t;
}

// grad_A[k] = <gC[row(k),:], B[col(k),:]> (SDDMM) and, when grad_B is given, the
// atomic scatter grad_B[col,:] += data[k] * gC[row,:].  Entry-balanced: a
// wavefront owns 64 consecutive stored entries whatever rows they belong to
// (every entry costs the same), finds its first row by bisection and walks on;
// gathers go out eight at a time and the dot products are reduced with DPP adds.
// FAST: grad_A only and n <= 64 (one column tile), which allows the pipelined loop below.
template <typename T, bool FAST>
__global__ __launch_bounds__(kBlock) void spdmm_bwd_kernel(
    int64_t rows, int64_t nnz, const T *__restrict__ data, const int64_t *__restrict__ indices,
    const int64_t *__restrict__ indptr, const T *__restrict__ B, int64_t ldb,
    const T *__restrict__ gC, int64_t ldg, int64_t n, T *__restrict__ grad_A,
    T *__restrict__ grad_B, int64_t ldgb, const int32_t *__restrict__ chunk_row) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // WIDE: dot products alone over thousands of dense columns.  The wavefronts of a workgroup then
    // share a chunk of entries and take every fourth tile of columns each (their sums meet in LDS,
    // in wavefront order): a matrix of a few ten thousand entries has too few chunks to fill the
    // chip with one wavefront per chunk, and each would walk hundreds of tiles on its own.
    const bool wide = !grad_B && n > 4 * kColsPerSlice;
    __shared__ T s_dot[kWavesPerBlock][kWave];
    const int64_t wave0 = wide ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * kWavesPerBlock + wave;
    const int64_t nwaves = wide ? (int64_t)gridDim.x : (int64_t)gridDim.x * kWavesPerBlock;
    const int64_t nchunks = (nnz + kWave - 1) / kWave;
    for (int64_t ch = wave0; ch < nchunks; ch += nwaves) {
        const int64_t kb = ch * kWave;
        const int cnt = (int)(nnz - kb < kWave ? nnz - kb : kWave);
        const int64_t k = kb + lane;
        const int64_t mycol = lane < cnt ? indices[k] : 0;
        const T myval = (grad_B && lane < cnt) ? data[k] : T(0);
        // row of the chunk's first entry: from the plan, else the last r with indptr[r] <= kb
        int64_t row;
        if (chunk_row) {
            row = chunk_row[ch];
        } else {
            int64_t lo = 0, hi = rows + 1;
            while (lo < hi) {
                const int64_t mid = (lo + hi) >> 1;
                if (indptr[mid] <= kb) lo = mid + 1; else hi = mid;
            }
            row = lo - 1;
        }
        // The ends of the next 64 rows sit one per lane, so that stepping over a row
        // boundary is a lane read and not a dependent global load (which would put a
        // memory round trip between two batches of gathers every few entries).
        int64_t ends_row = row;   // lane l holds indptr[ends_row + 1 + l]
        auto load_ends = [&](int64_t first) {
            const int64_t r = first + 1 + lane;
            return indptr[r <= rows ? r : rows];
        };
        int64_t my_end = load_ends(ends_row);
        auto end_of = [&](int64_t r) {
            const int l = __builtin_amdgcn_readfirstlane((int)(r - ends_row));
            const long long lo = __builtin_amdgcn_readlane((int)(my_end & 0xffffffffll), l);
            const long long hi = __builtin_amdgcn_readlane((int)(my_end >> 32), l);
            return (int64_t)((hi << 32) | (lo & 0xffffffffll));
        };
        int64_t row_end = end_of(row);
        T mydot = 0;
        // rows and columns of the entries [j0, j0 + kBatch) of the chunk
        auto locate = [&](int j0, int64_t (&col)[kBatch], int64_t (&rw)[kBatch]) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const int j = j0 + u < cnt ? j0 + u : cnt - 1;
                while (kb + j >= row_end) {
                    ++row;
                    if (row - ends_row >= kWave) {   // more than 64 rows inside one chunk: empty rows
                        ends_row = row;
                        my_end = load_ends(ends_row);
                    }
                    row_end = end_of(row);
                }
                rw[u] = row;
                // a scalar read, so that the row addresses below are scalar too and the gathers
                // share one vector register of column offsets
                const int js = __builtin_amdgcn_readfirstlane(j);
                const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(mycol & 0xffffffffll), js);
                const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(mycol >> 32), js);
                col[u] = (int64_t)(((unsigned long long)hi << 32) | lo);
            }
        };
        auto fetch = [&](const int64_t (&col)[kBatch], const int64_t (&rw)[kBatch], int64_t c, bool live,
                         T (&gv)[kBatch], T (&bv)[kBatch]) {
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const T *__restrict__ grow = gC + rw[u] * ldg;
                const T *__restrict__ brow = B + col[u] * ldb;
                gv[u] = grow[live ? c : 0];
                bv[u] = grad_A ? brow[live ? c : 0] : T(0);
            }
        };
        auto reduce8 = [&](const T (&p)[kBatch]) { return fold8<T>(p, lane); };
        auto consume = [&](int j0, const int64_t (&col)[kBatch], int64_t c, bool live, const T (&gv)[kBatch],
                           const T (&bv)[kBatch]) {
            if (grad_B) {
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    if (j0 + u >= cnt) break;
                    const T av = nm::read_lane(myval, __builtin_amdgcn_readfirstlane(j0 + u));
                    if (live) nm::atomic_add(grad_B + col[u] * ldgb + c, av * gv[u]);
                }
            }
            if (grad_A) {
                T p[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) p[u] = live ? gv[u] * bv[u] : T(0);
                const T t = reduce8(p);
                if ((lane >> 3) == (j0 >> 3)) mydot += t;   // lane j0 + u takes vector u
            }
        };
        if (FAST) {
            // grad_A alone, at most 64 dense columns: one column tile per batch, so a batch is
            // just its 16 operand vectors.  Two batches are kept in flight: the gathers of the
            // next batch are issued before the current one is reduced.  The two stages
            // alternate in place (copying a stage whose loads are still in flight would wait
            // for them), and the scalar rows and columns of a batch die with its address
            // arithmetic, which keeps them out of vector registers.
            const bool live = lane < n;
            auto issue = [&](int j0, T (&gv)[kBatch], T (&bv)[kBatch]) {
                int64_t col[kBatch], rw[kBatch];
                locate(j0, col, rw);
                fetch(col, rw, lane, live, gv, bv);
            };
            auto finish = [&](int j0, const T (&gv)[kBatch], const T (&bv)[kBatch]) {
                T p[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) p[u] = live ? gv[u] * bv[u] : T(0);
                const T t = reduce8(p);
                if ((lane >> 3) == (j0 >> 3)) mydot += t;
            };
            T gva[kBatch], bva[kBatch], gvb[kBatch], bvb[kBatch];
            issue(0, gva, bva);
            for (int j0 = 0;; j0 += 2 * kBatch) {
                if (j0 + kBatch < cnt) issue(j0 + kBatch, gvb, bvb);
                finish(j0, gva, bva);
                if (j0 + kBatch >= cnt) break;
                if (j0 + 2 * kBatch < cnt) issue(j0 + 2 * kBatch, gva, bva);
                finish(j0 + kBatch, gvb, bvb);
                if (j0 + 2 * kBatch >= cnt) break;
            }
        } else {
            for (int j0 = 0; j0 < cnt; j0 += kBatch) {
                int64_t col[kBatch], rw[kBatch];
                locate(j0, col, rw);
                if (wide) {
                    // (with fewer columns: the tile-by-tile sums below, which are the one-walk kernel's,
                    // bit for bit)  A lane keeps its
                    // columns' share of the eight sums and the lanes are added up once, behind the
                    // last tile (a reduction per tile is 27 instructions for 16 loads; at 16 384 dense
                    // columns that was most of the kernel)
                    T part[kBatch];
#pragma unroll
                    for (int u = 0; u < kBatch; ++u) part[u] = T(0);
#pragma unroll 2
                    for (int64_t c0 = (int64_t)wave * kWave; c0 < n; c0 += kWavesPerBlock * kWave) {
                        const int64_t c = c0 + lane;
                        const bool live = c < n;
                        T bv[kBatch], gv[kBatch];
                        fetch(col, rw, c, live, gv, bv);
#pragma unroll
                        for (int u = 0; u < kBatch; ++u) part[u] += live ? gv[u] * bv[u] : T(0);
                    }
                    const T t = reduce8(part);
                    if ((lane >> 3) == (j0 >> 3)) mydot += t;
                    continue;
                }
                for (int64_t c0 = 0; c0 < n; c0 += kWave) {
                    const int64_t c = c0 + lane;
                    const bool live = c < n;
                    T bv[kBatch], gv[kBatch];
                    fetch(col, rw, c, live, gv, bv);
                    consume(j0, col, c, live, gv, bv);
                }
            }
        }
        if (wide) {
            s_dot[wave][lane] = mydot;
            __syncthreads();
            mydot = s_dot[0][lane];
            for (int w = 1; w < kWavesPerBlock; ++w) mydot += s_dot[w][lane];
            if (wave == 0 && lane < cnt) grad_A[k] = mydot;
            __syncthreads();   // the sums are written again for the workgroup's next chunk
            continue;
        }
        if (grad_A && lane < cnt) grad_A[k] = mydot;
    }
}

// ---- both gradients in one walk over A by column ---------------------------------
//
// grad_B = A^T gC walks A by column on the transposed-structure plan and gathers, per stored
// entry, the row of gC it names.  The dot product grad_A[k] = <gC[row,:], B[col,:]> needs that
// same row of gC and the column's own row of B, which a wavefront that owns the column can
// keep at hand.  So one walk serves both gradients and the second pass of gathers (rows of B
// per entry, as the row-major kernel above makes them) falls away: half the gathered bytes of
// the backward.  grad_B is added in the same order as by spdmm_fwd_flat_kernel on the plan
// and the dot products are folded exactly like spdmm_bwd_kernel's, so both gradients keep
// their bits.  Dense operands wider than 64 columns are taken 64 columns at a time, as by the
// forward kernel; the dot products add up over the tiles in grad_A.
template <typename T>
__device__ __forceinline__ void fused_long_columns(int64_t cols, const T *__restrict__ data,
                                                   const int32_t *__restrict__ t_row,
                                                   const int32_t *__restrict__ t_indptr,
                                                   const int32_t *__restrict__ t_perm, const T *__restrict__ gC,
                                                   int64_t ldg, const T *__restrict__ B, int64_t ldb, int64_t n,
                                                   T *__restrict__ grad_B, int64_t ldgb, T *__restrict__ grad_A,
                                                   int lane, int wave) {
    __shared__ T s_part[kWavesPerBlock][kWave];
    __shared__ int s_long[kScoutRows];
    __shared__ int s_nlong;
    const int64_t g0 = (int64_t)blockIdx.x * kScoutRows;
    if (threadIdx.x == 0) s_nlong = 0;
    __syncthreads();
    for (int t = threadIdx.x; t < kScoutRows && g0 + t < cols; t += kBlock)
        if (t_indptr[g0 + t + 1] - t_indptr[g0 + t] > kSplitRow) s_long[atomicAdd(&s_nlong, 1)] = t;
    __syncthreads();
    const int nl = s_nlong;
    for (int li = 0; li < nl; ++li) {   // uniform over the workgroup
        const int64_t col = g0 + s_long[li];
        const int64_t rb = t_indptr[col], re = t_indptr[col + 1];
        int64_t chunk = (re - rb + kWavesPerBlock - 1) / kWavesPerBlock;
        chunk = (chunk + kWave - 1) / kWave * kWave;
        const int64_t kb0 = rb + wave * chunk;
        const int64_t ke0 = kb0 + chunk < re ? kb0 + chunk : re;
        for (int64_t c0 = 0; c0 < n; c0 += kWave) {   // 64 dense columns at a time
            const int64_t c = c0 + lane;
            const bool live = c < n;
            const T bj = live ? B[col * ldb + c] : T(0);
            T acc = T(0);
            for (int64_t kb = kb0; kb < ke0; kb += kWave) {
                const int64_t k = kb + lane;
                const int64_t myrow = k < ke0 ? (int64_t)t_row[k] : 0;
                const int32_t myperm = k < ke0 ? t_perm[k] : 0;
                const T myval = k < ke0 ? data[myperm] : T(0);
                const int cnt = (int)(ke0 - kb < kWave ? ke0 - kb : kWave);
                T mydot = T(0);
                for (int j = 0; j < cnt; ++j) {
                    const T gv = gC[__shfl(myrow, j, kWave) * ldg + (live ? c : 0)];
                    acc += __shfl(myval, j, kWave) * gv;
                    const T t = nm::wave_sum(live ? gv * bj : T(0));
                    if (lane == j) mydot = t;
                }
                if (lane < cnt) grad_A[myperm] = c0 == 0 ? mydot : grad_A[myperm] + mydot;
            }
            s_part[wave][lane] = acc;
            __syncthreads();
            if (wave == 0 && live) {
                T sum = s_part[0][lane];
                for (int w = 1; w < kWavesPerBlock; ++w) sum += s_part[w][lane];
                grad_B[col * ldgb + c] = sum;
            }
            __syncthreads();
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void spdmm_bwd_fused_kernel(
    int64_t cols, const T *__restrict__ data, const int32_t *__restrict__ t_row,
    const int32_t *__restrict__ t_indptr, const int32_t *__restrict__ t_perm, const T *__restrict__ gC,
    int64_t ldg, const T *__restrict__ B, int64_t ldb, int64_t n, T *__restrict__ grad_B, int64_t ldgb,
    T *__restrict__ grad_A) {
    __shared__ T s_b[kWavesPerBlock][kFlatRows][kWave];   // rows of B of the columns a wavefront owns
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t long_blocks = (cols + kScoutRows - 1) / kScoutRows;
    if ((int64_t)blockIdx.x < long_blocks) {
        fused_long_columns<T>(cols, data, t_row, t_indptr, t_perm, gC, ldg, B, ldb, n, grad_B, ldgb, grad_A, lane,
                              wave);
        return;
    }
    const int64_t r0 = (((int64_t)blockIdx.x - long_blocks) * kWavesPerBlock + wave) * kFlatRows;
    if (r0 >= cols) return;
    const int nr = (int)(cols - r0 < kFlatRows ? cols - r0 : kFlatRows);
    const int64_t my_ptr = (int64_t)t_indptr[r0 + (lane <= nr ? lane : nr)];
    auto ptr_of = [&](int l) {
        const long long lo = __builtin_amdgcn_readlane((int)(my_ptr & 0xffffffffll), l);
        const long long hi = __builtin_amdgcn_readlane((int)(my_ptr >> 32), l);
        return (int64_t)((hi << 32) | (lo & 0xffffffffll));
    };
    const int64_t begin = ptr_of(0), end = ptr_of(nr);
    const int64_t row_bytes = ldg * (int64_t)sizeof(T);
    for (int64_t c0 = 0; c0 < n; c0 += kWave) {   // 64 dense columns at a time; the dot products add up over the tiles
        const int64_t c = c0 + lane;
        const bool live = c < n;
        const bool first_tile = c0 == 0;
        for (int r = 0; r < nr; ++r) s_b[wave][r][lane] = live ? B[(r0 + r) * ldb + c] : T(0);
        const char *__restrict__ Gc = reinterpret_cast<const char *>(gC + (live ? c : 0));
        int r = 0;   // current column (relative), its range, whether it is computed here
        int64_t row_begin = begin, row_end = ptr_of(1);
        bool mine = row_end - row_begin <= kSplitRow;
        T acc = T(0);
        T cur_b = s_b[wave][0][lane];
        auto next_row = [&]() {
            if (mine && live) grad_B[(r0 + r) * ldgb + c] = acc;
            acc = T(0);
            ++r;
            row_begin = row_end;
            row_end = ptr_of(r + 1 <= nr ? r + 1 : nr);
            mine = row_end - row_begin <= kSplitRow;
            cur_b = s_b[wave][r < nr ? r : nr - 1][lane];
        };
        auto close_row = [&]() {
            next_row();
            while (r < nr && row_end == row_begin) next_row();
        };
        while (r < nr && row_end == row_begin) next_row();   // empty columns at the head
        int64_t kb = begin;
        auto fetch = [&](int64_t at, int64_t &row, T &val, int32_t &pos) {
            const int64_t k = at + lane < end ? at + lane : (end > begin ? end - 1 : 0);
            row = end > begin ? (int64_t)t_row[k] : 0;
            pos = end > begin ? t_perm[k] : 0;
            val = end > begin ? data[pos] : T(0);
        };
        int64_t myrow, nextrow;
        T myval, nextval;
        int32_t mypos, nextpos;
        fetch(kb, myrow, myval, mypos);
        while (kb < end) {   // entry kb belongs to column r
            if (!mine) {     // a long column is not computed here: jump over what is left of it
                kb = row_end;
                close_row();
                if (kb >= end) break;
                fetch(kb, myrow, myval, mypos);
                continue;
            }
            const int cnt = (int)(end - kb < kWave ? end - kb : kWave);
            fetch(kb + kWave, nextrow, nextval, nextpos);   // in flight while this chunk is used
            const int64_t k = kb + lane;
            const int64_t myoff = myrow * row_bytes;
            int rid = 0;
            for (int l = 1; l < nr; ++l) rid += k >= ptr_of(l) ? 1 : 0;
            const int64_t my_row_end = __shfl(my_ptr, rid + 1, kWave);
            const unsigned long long ends = __ballot(lane < cnt && k + 1 == my_row_end);
            // entries of a long column inside this chunk are not computed here: their dot products
            // are written by the workgroup that takes the column
            const int64_t my_row_begin = __shfl(my_ptr, rid, kWave);
            const bool here = lane < cnt && my_row_end - my_row_begin <= kSplitRow;
            T mydot = T(0);
            auto gather = [&](int j0, T (&gv)[kBatch]) {
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const int j = __builtin_amdgcn_readfirstlane(j0 + u < cnt ? j0 + u : cnt - 1);
                    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(myoff & 0xffffffffll), j);
                    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(myoff >> 32), j);
                    gv[u] = *reinterpret_cast<const T *>(Gc + (int64_t)(((unsigned long long)hi << 32) | lo));
                }
            };
            auto add_up = [&](int j0, const T (&gv)[kBatch]) {
                const int m = cnt - j0 < kBatch ? cnt - j0 : kBatch;
                T p[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) p[u] = T(0);
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    if (u >= m) break;
                    const int j = __builtin_amdgcn_readfirstlane(j0 + u);
                    acc += nm::read_lane(myval, j) * gv[u];
                    p[u] = live ? gv[u] * cur_b : T(0);
                    if ((ends >> j) & 1ull) close_row();
                }
                const T t = fold8<T>(p, lane);
                if ((lane >> 3) == (j0 >> 3)) mydot += t;   // lane j0 + u takes vector u
            };
            T gva[kBatch], gvb[kBatch];
            gather(0, gva);
            for (int j0 = 0;; j0 += 2 * kBatch) {
                if (j0 + kBatch < cnt) gather(j0 + kBatch, gvb);
                add_up(j0, gva);
                if (j0 + kBatch >= cnt) break;
                if (j0 + 2 * kBatch < cnt) gather(j0 + 2 * kBatch, gva);
                add_up(j0 + kBatch, gvb);
                if (j0 + 2 * kBatch >= cnt) break;
            }
            if (here) grad_A[mypos] = first_tile ? mydot : grad_A[mypos] + mydot;
            kb += cnt;
            myrow = nextrow;
            myval = nextval;
            mypos = nextpos;
        }
        while (r < nr) next_row();   // columns of a wavefront whose entries ran out before them
    }
}

// ---- narrow dense operands (n <= 32) -----------------------------------------------
//
// With lane = dense column, a 16-column operand leaves three quarters of every gather and
// every multiply idle, and the kernels above take as long for n = 8 as for n = 64 (their time
// is instruction issue and latency per ENTRY).  In the dot products of the backward a wavefront
// therefore works on 64 / W entries per instruction, W = n rounded up to 8, 16 or 32: lane =
// (entry slot, column); 1.03 -> 0.73 ms for the whole backward at n = 16 on the 1M x 1M
// power-law matrix.  (The same mapping for the forward product, with the products of a chunk
// staged in LDS and added per row in storage order, measured no faster than the wide kernel:
// 0.41-0.77 ms against 0.51 ms, and was dropped.)

// Sum over aligned groups of W lanes; every lane of the group gets it.
template <int W, typename T> __device__ __forceinline__ T narrow_sum(T v) {
    v += nm::dpp_move<0xB1>(v);                  // quad_perm [1,0,3,2]
    v += nm::dpp_move<0x4E>(v);                  // quad_perm [2,3,0,1]
    if (W == 8) v += nm::dpp_move<0x141>(v);     // row_half_mirror: the other quad of the 8
    if (W >= 16) {
        v += nm::dpp_move<0x124>(v);             // row_ror 4
        v += nm::dpp_move<0x128>(v);             // row_ror 8
    }
    if (W == 32) v += __shfl_xor(v, 16, kWave);
    return v;
}

// grad_A[k] = <gC[row(k), :], B[col(k), :]> for n <= W.  Entry-balanced like the wide kernel:
// a wavefront owns 64 consecutive entries; every lane first finds the row of "its" entry by a
// bisection over the ends of the next 64 rows (held one per lane), then the wavefront takes
// 64 / W entries per step, four steps' gathers in flight.
template <typename T, int W>
__global__ __launch_bounds__(kBlock) void sddmm_narrow_kernel(
    int64_t rows, int64_t nnz, const int64_t *__restrict__ indices, const int64_t *__restrict__ indptr,
    const T *__restrict__ B, int64_t ldb, const T *__restrict__ gC, int64_t ldg, int n, T *__restrict__ grad_A,
    const int32_t *__restrict__ chunk_row) {
    constexpr int GPW = kWave / W;   // entries per step
    constexpr int U = 4;             // steps per batch
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    const int64_t nchunks = (nnz + kWave - 1) / kWave;
    const int slot = lane / W, c = lane % W;
    const bool col_live = c < n;
    const int cs = col_live ? c : 0;
    for (int64_t ch = wave0; ch < nchunks; ch += nwaves) {
        const int64_t kb = ch * kWave;
        const int cnt = (int)(nnz - kb < kWave ? nnz - kb : kWave);
        const int64_t k = kb + (lane < cnt ? lane : cnt - 1);
        const int64_t mycol = indices[k];
        int64_t row0;   // row of the chunk's first entry
        if (chunk_row) {
            row0 = chunk_row[ch];
        } else {
            int64_t lo = 0, hi = rows + 1;
            while (lo < hi) {
                const int64_t mid = (lo + hi) >> 1;
                if (indptr[mid] <= kb) lo = mid + 1; else hi = mid;
            }
            row0 = lo - 1;
        }
        // my entry's row: row0 + number of row ends at or before it
        const int64_t er = row0 + 1 + lane;
        const int64_t my_end = indptr[er <= rows ? er : rows];
        int lo = 0, hi = kWave;
#pragma unroll
        for (int step = 0; step < 7; ++step) {   // 65 possible answers: seven halvings
            const int mid = (lo + hi) >> 1;      // == 64 only once lo == hi == 64: the read is ignored then
            const int64_t e = __shfl(my_end, mid & (kWave - 1), kWave);
            if (lo < hi) {
                if (e <= k) lo = mid + 1; else hi = mid;
            }
        }
        int64_t myrow = row0 + lo;
        if (lo == kWave) {   // more than 64 rows end inside this chunk (empty rows): look the row up
            int64_t l2 = myrow, h2 = rows + 1;
            while (l2 < h2) {
                const int64_t mid = (l2 + h2) >> 1;
                if (indptr[mid] <= k) l2 = mid + 1; else h2 = mid;
            }
            myrow = l2 - 1;
        }
        for (int j0 = 0; j0 < cnt; j0 += U * GPW) {
            T gv[U], bv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = j0 + u * GPW + slot;
                const int js = j < cnt ? j : cnt - 1;
                const int64_t col = __shfl(mycol, js, kWave), rw = __shfl(myrow, js, kWave);
                gv[u] = gC[rw * ldg + cs];
                bv[u] = B[col * ldb + cs];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int j = j0 + u * GPW + slot;
                const T dot = narrow_sum<W>(col_live ? gv[u] * bv[u] : T(0));
                if (c == 0 && j < cnt) grad_A[kb + j] = dot;
            }
        }
    }
}

// Launches the forward product (A as delivered, or A^T through the plan).
template <typename T, typename IDX, bool PERM>
void launch_product(unsigned grid, hipStream_t s, int64_t rows, const T *data, const IDX *indices, const IDX *indptr,
                    const int32_t *perm, const T *B, int64_t ldb, int64_t n, T *C, int64_t ldc) {
    hipLaunchKernelGGL((spdmm_fwd_flat_kernel<T, IDX, PERM>), dim3(grid, (unsigned)nm::ceil_div(n, (int64_t)kColsPerSlice)),
                       dim3(kBlock), 0, s, rows, data, indices, indptr, perm, B, ldb, n, C, ldc);
}

int check_args(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
               const int64_t *indices, const int64_t *indptr, int64_t n) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0 && n >= 0, "negative size");
    NM_REQUIRE(indptr != nullptr, "indptr is null");
    NM_REQUIRE(nnz == 0 || (data != nullptr && indices != nullptr), "data/indices null with nnz > 0");
    return NM_OK;
}

// workgroups of the flat forward kernel: the long-row scouts first, then the flat walkers
inline unsigned flat_grid_for(int64_t rows) {
    const int64_t g = nm::ceil_div(rows, kScoutRows) + nm::ceil_div(rows, (int64_t)kWavesPerBlock * kFlatRows);
    return (unsigned)(g < 1 ? 1 : g);
}

inline unsigned wave_grid(int64_t units, int per_block) {
    int64_t grid = nm::ceil_div(units, per_block);
    if (grid > nm::kMaxGrid) grid = nm::kMaxGrid;
    return (unsigned)(grid < 1 ? 1 : grid);
}

}  // namespace

extern "C" int nm_spdmm_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                const int64_t *indices, const int64_t *indptr, const void *B, int64_t ldb,
                                int64_t n, void *C, int64_t ldc, nm_stream stream) {
    if (int rc = check_args(dt, rows, cols, nnz, data, indices, indptr, n)) return rc;
    if (rows == 0 || n == 0) return NM_OK;
    NM_REQUIRE(C != nullptr && (B != nullptr || nnz == 0), "B or C is null");
    NM_REQUIRE(ldb >= n && ldc >= n, "row stride smaller than the row (ldb=%lld ldc=%lld n=%lld)",
               (long long)ldb, (long long)ldc, (long long)n);
    hipStream_t s = nm::as_stream(stream);
    const unsigned flat_grid = flat_grid_for(rows);
    if (dt == NM_F32)
        launch_product<float, int64_t, false>(flat_grid, s, rows, (const float *)data, indices, indptr, nullptr,
                                              (const float *)B, ldb, n, (float *)C, ldc);
    else
        launch_product<double, int64_t, false>(flat_grid, s, rows, (const double *)data, indices, indptr, nullptr,
                                               (const double *)B, ldb, n, (double *)C, ldc);
    NM_LAUNCH_CHECK("spdmm_fwd_flat_kernel");
    return NM_OK;
}

namespace {
int backward_impl(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data, const int64_t *indices,
                  const int64_t *indptr, const void *B, int64_t ldb, const void *gC, int64_t ldg, int64_t n,
                  void *grad_A, void *grad_B, int64_t ldgb, const int32_t *chunk_row, nm_stream stream) {
    if (int rc = check_args(dt, rows, cols, nnz, data, indices, indptr, n)) return rc;
    hipStream_t s = nm::as_stream(stream);
    if (grad_B && cols > 0 && n > 0) {
        NM_REQUIRE(ldgb >= n, "grad_B row stride smaller than the row");
        // rows of grad_B are cleared individually when it is strided
        if (ldgb == n) {
            int rc = dt == NM_F32 ? nm::fill_async((float *)grad_B, cols * n, 0.0f, s)
                                  : nm::fill_async((double *)grad_B, cols * n, 0.0, s);
            if (rc) return rc;
        } else {
            return nm::fail(NM_ERR_UNSUPPORTED, "grad_B must be contiguous (ldgb == n)");
        }
    }
    if (grad_A && nnz > 0 && n == 0) {
        int rc = dt == NM_F32 ? nm::fill_async((float *)grad_A, nnz, 0.0f, s)
                              : nm::fill_async((double *)grad_A, nnz, 0.0, s);
        if (rc) return rc;
    }
    if (rows == 0 || nnz == 0 || n == 0 || (!grad_A && !grad_B)) return NM_OK;
    NM_REQUIRE(B != nullptr && gC != nullptr, "B or gC is null");
    NM_REQUIRE(ldb >= n && ldg >= n, "row stride smaller than the row");
    // (dot products alone over thousands of dense columns: a workgroup per chunk of 64 entries)
    const dim3 grid(wave_grid(nm::ceil_div(nnz, kWave), grad_A && !grad_B && n > 4 * kColsPerSlice ? 1 : kWavesPerBlock));
    if (grad_A && !grad_B && n <= 32) {
#define NM_NARROW(T, W)                                                                                          \
    hipLaunchKernelGGL((sddmm_narrow_kernel<T, W>), grid, dim3(kBlock), 0, s, rows, nnz, indices, indptr,          \
                       (const T *)B, ldb, (const T *)gC, ldg, (int)n, (T *)grad_A, chunk_row)
        if (dt == NM_F32) {
            if (n <= 8) NM_NARROW(float, 8); else if (n <= 16) NM_NARROW(float, 16); else NM_NARROW(float, 32);
        } else {
            if (n <= 8) NM_NARROW(double, 8); else if (n <= 16) NM_NARROW(double, 16); else NM_NARROW(double, 32);
        }
#undef NM_NARROW
        NM_LAUNCH_CHECK("sddmm_narrow_kernel");
        return NM_OK;
    }
    const bool fast = grad_A && !grad_B && n <= kWave;
#define NM_SDDMM(T, FAST)                                                                                         \
    hipLaunchKernelGGL((spdmm_bwd_kernel<T, FAST>), grid, dim3(kBlock), 0, s, rows, nnz, (const T *)data, indices, \
                       indptr, (const T *)B, ldb, (const T *)gC, ldg, n, (T *)grad_A, (T *)grad_B, ldgb, chunk_row)
    if (dt == NM_F32) {
        if (fast) NM_SDDMM(float, true); else NM_SDDMM(float, false);
    } else {
        if (fast) NM_SDDMM(double, true); else NM_SDDMM(double, false);
    }
#undef NM_SDDMM
    NM_LAUNCH_CHECK("spdmm_bwd_kernel");
    return NM_OK;
}
}  // namespace

extern "C" int nm_spdmm_backward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                 const int64_t *indices, const int64_t *indptr, const void *B, int64_t ldb,
                                 const void *gC, int64_t ldg, int64_t n, void *grad_A, void *grad_B,
                                 int64_t ldgb, nm_stream stream) {
    return backward_impl(dt, rows, cols, nnz, data, indices, indptr, B, ldb, gC, ldg, n, grad_A, grad_B, ldgb,
                         nullptr, stream);
}

// Backward over the transposed-structure plan: grad_A by the row-major kernel
// (dot products only), grad_B = A^T gC as a forward product on the plan, whose
// per-entry sums run in ascending row order like the serial CPU loop
// (cpp/sparse_csr_cpu.cpp:639-646): no atomics, no clearing, bit-reproducible.
extern "C" int nm_spdmm_backward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                         const int64_t *indices, const int64_t *indptr, const void *plan_mem,
                                         const void *B, int64_t ldb, const void *gC, int64_t ldg, int64_t n,
                                         void *grad_A, void *grad_B, int64_t ldgb, nm_stream stream) {
    if (int rc = check_args(dt, rows, cols, nnz, data, indices, indptr, n)) return rc;
    NM_REQUIRE(plan_mem != nullptr, "plan is null");
    nm::TPlan t;
    nm::tplan_layout(rows, cols, nnz, const_cast<void *>(plan_mem), &t);
    // (a dense operand of thousands of columns: the fused walk takes its column tiles one after the
    // other, the product below is cut into slices of kColsPerSlice over the grid)
    if (grad_A && grad_B && rows > 0 && cols > 0 && nnz > 0 && n > 32 && n <= 4 * kColsPerSlice) {
        // both gradients from a single walk over A by column (measured on the 16 M-entry power-law
        // matrix: 1.02 against 1.29 ms at 64 dense columns, 2.18 against 2.80 ms at 128, even at 32;
        // with 16 or fewer the narrow dot-product kernel below and a separate product are faster,
        // 0.70-0.74 against 0.81-0.82 ms)
        NM_REQUIRE(B != nullptr && gC != nullptr, "B or gC is null");
        NM_REQUIRE(ldb >= n && ldg >= n && ldgb >= n, "row stride smaller than the row");
        hipStream_t s = nm::as_stream(stream);
        const unsigned grid = flat_grid_for(cols);
        if (dt == NM_F32)
            hipLaunchKernelGGL(spdmm_bwd_fused_kernel<float>, dim3(grid), dim3(kBlock), 0, s, cols, (const float *)data,
                               t.t_row, t.t_indptr, t.t_perm, (const float *)gC, ldg, (const float *)B, ldb, n,
                               (float *)grad_B, ldgb, (float *)grad_A);
        else
            hipLaunchKernelGGL(spdmm_bwd_fused_kernel<double>, dim3(grid), dim3(kBlock), 0, s, cols,
                               (const double *)data, t.t_row, t.t_indptr, t.t_perm, (const double *)gC, ldg,
                               (const double *)B, ldb, n, (double *)grad_B, ldgb, (double *)grad_A);
        NM_LAUNCH_CHECK("spdmm_bwd_fused_kernel");
        return NM_OK;
    }
    if (grad_A) {
        if (int rc = backward_impl(dt, rows, cols, nnz, data, indices, indptr, B, ldb, gC, ldg, n, grad_A, nullptr, 0,
                                   t.chunk_row, stream))
            return rc;
    }
    if (!grad_B || cols == 0 || n == 0) return NM_OK;
    NM_REQUIRE(ldgb >= n && ldg >= n, "row stride smaller than the row");
    NM_REQUIRE(gC != nullptr || nnz == 0, "gC is null");
    hipStream_t s = nm::as_stream(stream);
    const unsigned flat_grid = flat_grid_for(cols);
    if (dt == NM_F32)
        launch_product<float, int32_t, true>(flat_grid, s, cols, (const float *)data, t.t_row, t.t_indptr, t.t_perm,
                                             (const float *)gC, ldg, n, (float *)grad_B, ldgb);
    else
        launch_product<double, int32_t, true>(flat_grid, s, cols, (const double *)data, t.t_row, t.t_indptr,
                                              t.t_perm, (const double *)gC, ldg, n, (double *)grad_B, ldgb);
    NM_LAUNCH_CHECK("spdmm_fwd_flat_kernel (transposed)");
    return NM_OK;
}
