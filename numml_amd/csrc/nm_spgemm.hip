// Hash-based CSR x CSR product (SpGEMM) and its backward for gfx950.
//
// Forward, two phases around the caller's allocation of C:
//   symbolic: rows of A are binned by an upper bound on their products
//             (sum of the lengths of the B rows they touch).  A group of lanes
//             (8, 64 or 256, by bin) inserts the row's column indices into a
//             hash set in LDS and counts the distinct ones; an exclusive scan
//             of the counts is C_indptr.
//   numeric : rows are re-binned by their exact length.  The group accumulates
//             (column, value) pairs in an LDS hash table, walking A's row
//             entry by entry and B's row across the lanes, so every output
//             entry receives its products in the order of A's row -- the
//             order of the serial SMMP loop (cpp/sparse_csr_cpu.cpp:182-212) --
//             and then writes the table out ranked by column, so C's rows are
//             ascending like the reference's.
// Rows too long for an LDS table spill to a dense accumulator in global memory
// (one slice of B_cols entries per spill workgroup).
// Short rows take a merge path instead of hashing: when a row of A and every row
// of B it names have at most 8 entries (stencil and aggregation operators), eight
// lanes each hold one B row, sorted as stored, and the group repeatedly emits the
// smallest head column; the lanes whose head equals it contribute their product,
// summed in lane order = the order of A's row.  These rows never enter the bins.
//
// Backward: eight lanes per row i of A; for each entry (i,k) the lanes share row
// k of B, find its columns in row i of C (staged in LDS) by bisection, and form
// grad_A (a sum in ascending column order, as the reference's merge,
// cpp/sparse_csr_cpu.cpp:246-278) and grad_B (atomic adds, one cache line per
// entry of A) in one pass.
//
// Algorithmic HBM bytes of the forward (s = sizeof(value)):
//   nnzA*(s+8) + rowsA*8 + products*(s+8) [upper; nnzB*(s+8) compulsory]
//   + nnzC*(s+8) + rowsA*8
#include "nm_common.hpp"
#include "nm_scan.hpp"
#include "nm_spgemm_plan.hpp"

namespace {

using nm::kWave;

constexpr int32_t kEmpty = -1;
constexpr int kBlock = 256;
constexpr int kBins = 8;
constexpr int kBinStart = 8, kBinCursor = 20, kBinInts = 32;   // layout of the bins array, see Work
// Workgroups (and dense accumulator slices of B_cols entries each) of the spill path: as many as
// fit a fixed budget of scratch, between 8 and 64.
constexpr int64_t kSpillBudgetBytes = int64_t(192) << 20;
inline int spill_groups(int64_t B_cols) {
    const int64_t g = kSpillBudgetBytes / (12 * (B_cols + 1));
    return (int)(g < 8 ? 8 : (g > 64 ? 64 : g));
}
constexpr int kSpillBlock = 1024;
constexpr int kTablePad = 4;         // entries between the hash tables of neighbouring groups (16 bytes)
constexpr int kAhead = 8;            // B rows whose first columns a group requests before inserting any
#ifndef NM_HASH_BATCH
#define NM_HASH_BATCH 8
#endif

// bin upper limits (inclusive); the last bin takes the rest and spills
constexpr int32_t kSymLimit[7] = {64, 128, 256, 512, 1024, 2048, 8192};     // on the product bound
constexpr int32_t kNumLimit[7] = {32, 64, 128, 256, 512, 1024, 4096};       // on the exact row length
// lanes per row and table sizes per bin.  The kernels wait on memory (A's row, the bounds of its B
// rows, the B rows: a chain of round trips per row) and LDS decides how many rows a CU has in
// flight, so rows get the smallest table that holds them at half load.
constexpr int kGroup0 = 8, kGroup1 = 16, kGroup2 = 16, kGroup3 = 64, kGroup4 = 64, kGroup5 = 256, kGroup6 = 256;
constexpr int kSymTable0 = 128, kSymTable1 = 256, kSymTable2 = 512, kSymTable3 = 1024, kSymTable4 = 2048,
              kSymTable5 = 4096, kSymTable6 = 16384;
constexpr int kNumTable0 = 64, kNumTable1 = 128, kNumTable2 = 256, kNumTable3 = 512, kNumTable4 = 1024,
              kNumTable5 = 2048, kNumTable6 = 8192;

constexpr int kMergeCap = 8;                  // longest A row and B row of the merge path
constexpr int32_t kColEnd = 0x7fffffff;       // past-the-end column of a staged B row
constexpr int32_t kMergedKey = -1;            // binning key of a row the merge path has taken

struct Work {
    int32_t *key;      // [rows] binning key (product bound, then exact length)
    int32_t *perm;     // [rows] rows grouped by bin
    int32_t *bins;     // [kBinInts]: rows per bin [0, kBins), first row of bin b at kBinStart + b (end at + b + 1), cursor at kBinCursor + b
    int32_t *count;    // [rows + 1] entries per row of C, before the row pointer is made of them
    int64_t *scan;     // [tiles + 1] sums of the counts by tile of the row pointer's scan
    int32_t *mark;     // [spill_groups(B_cols) * B_cols]
    double *acc;       // [spill_groups(B_cols) * B_cols]
    int64_t *summary;  // [2]: nnz(C) and the number of rows on the hash path, for the host
};

inline size_t align_up(size_t v) { return (v + 255) & ~size_t(255); }

size_t work_layout(int64_t rows, int64_t B_cols, void *base, Work *w) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *p = base ? static_cast<char *>(base) + off : nullptr;
        off += align_up(bytes);
        return p;
    };
    int32_t *key = (int32_t *)take((rows + 1) * 4);
    int32_t *perm = (int32_t *)take((rows + 1) * 4);
    int32_t *bins = (int32_t *)take(kBinInts * 4);
    int32_t *count = (int32_t *)take((size_t)(rows + 1) * 4);
    int64_t *scan = (int64_t *)take(nm::scan_scratch_bytes(rows + 1));
    int64_t *summary = (int64_t *)take(2 * 8);
    int32_t *mark = (int32_t *)take((size_t)spill_groups(B_cols) * (B_cols + 1) * 4);
    double *acc = (double *)take((size_t)spill_groups(B_cols) * (B_cols + 1) * 8);
    if (w) *w = Work{key, perm, bins, count, scan, mark, acc, summary};
    return off;
}

// First slot of a key in a table of TABLE slots (a power of two): the HIGH bits of a
// multiplicative hash.  The low bits of key * odd depend on the low bits of the key alone,
// so columns a multiple of the table size apart -- the neighbours of a grid point in the
// next row or plane -- would all start their probes in the same slot.
template <int TABLE> __device__ __forceinline__ uint32_t first_slot(int32_t key) {
    static_assert(TABLE >= 2 && (TABLE & (TABLE - 1)) == 0, "table size");
    return ((uint32_t)key * 0x9E3779B1u) >> (32 - __builtin_ctz(TABLE));
}

template <int G> __device__ __forceinline__ void group_sync() {
    if (G > kWave) __syncthreads();
    else __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
}

// Sum over a group of G lanes (G <= 64: shuffles; G == blockDim: via LDS).
template <int G> __device__ __forceinline__ int group_total(int v, int *s_red) {
    if (G <= kWave) return nm::group_sum<G>(v);
    v = nm::wave_sum(v);
    if ((threadIdx.x & (kWave - 1)) == 0) s_red[threadIdx.x / kWave] = v;
    __syncthreads();
    int t = 0;
    for (int w = 0; w < G / kWave; ++w) t += s_red[w];
    __syncthreads();
    return t;
}

// ---- binning ---------------------------------------------------------------

// ---- merge path (short rows) ---------------------------------------------------
//
// Lane layout: a merge group is the 8 lanes of equal parity in a 16-lane DPP row,
// so a wavefront holds 8 groups.  Neighbours inside a group are two lanes apart:
// rotations by 2, 4 and 8 inside the DPP row reduce over the group, and a shift by
// 2 feeds lane k the value of lane k-1 of its group with a hardware zero for k = 0.

__device__ __forceinline__ int merge_lane() { return (threadIdx.x & 15) >> 1; }
__device__ __forceinline__ int merge_group() { return ((threadIdx.x & 63) >> 4) * 2 + (threadIdx.x & 1); }

__device__ __forceinline__ int32_t merge_min(int32_t v) {
    v = min(v, nm::dpp_move<0x122>(v));   // row_ror 2
    v = min(v, nm::dpp_move<0x124>(v));   // row_ror 4
    v = min(v, nm::dpp_move<0x128>(v));   // row_ror 8
    return v;
}
__device__ __forceinline__ int32_t merge_max(int32_t v) {
    v = max(v, nm::dpp_move<0x122>(v));
    v = max(v, nm::dpp_move<0x124>(v));
    v = max(v, nm::dpp_move<0x128>(v));
    return v;
}
__device__ __forceinline__ int32_t merge_sum(int32_t v) {
    v += nm::dpp_move<0x122>(v);
    v += nm::dpp_move<0x124>(v);
    v += nm::dpp_move<0x128>(v);
    return v;
}

constexpr int kMergeRows = kBlock / 8;   // rows of A per workgroup pass
constexpr int kMergeStride = kBlock + 1; // slot stride of the staged B rows (odd: slots of one lane fall in different banks)

// Staging of the B rows of a wavefront into LDS.  Every lane owns one B row
// (start `bb`, `len` <= kMergeCap entries, 0 when it has none).  Loading them
// lane by lane would touch ~30 cache lines per instruction and use 8 bytes of
// each; instead the wavefront loads one LEG at a time: in pass u the eight lanes
// of sub-wavefront g read the eight entries of the row owned by lane u of group
// g, so an instruction reads eight contiguous 64-byte pieces -- and for banded
// matrices, where neighbouring rows of A name neighbouring rows of B, one
// contiguous span.  Entry k of the row owned by thread t lands in slot
// [k * kMergeStride + t]; slot kMergeCap is the end marker.
//
// The loads are unconditional: a lane with nothing to fetch reads `safe` (8 valid
// bytes) and discards the result.  Predicated loads would sit in their own
// branches, each followed by the wait for its data, i.e. one memory round trip
// per leg instead of one for all of them.
template <typename T, bool VALUES>
__device__ __forceinline__ void merge_stage(int64_t bb, int len, const int64_t *__restrict__ B_indices,
                                            const T *__restrict__ B_data, const int64_t *__restrict__ safe,
                                            int64_t *s_bb, int32_t *s_len, int32_t *s_col, T *s_val) {
    s_bb[threadIdx.x] = bb;
    s_len[threadIdx.x] = len;
    s_col[kMergeCap * kMergeStride + threadIdx.x] = kColEnd;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    const int lane = threadIdx.x & 63, g = lane >> 3, k = lane & 7;
    const int first = (threadIdx.x & ~63) + (g >> 1) * 16 + (g & 1);   // lane 0 of merge group g
    int64_t col[kMergeCap];
    T val[kMergeCap];
    bool have[kMergeCap];
#pragma unroll
    for (int u = 0; u < kMergeCap; ++u) {
        const int owner = first + 2 * u;
        const int64_t obb = s_bb[owner];
        have[u] = k < s_len[owner];
        col[u] = *(have[u] ? B_indices + obb + k : safe);
        if (VALUES) val[u] = *(have[u] ? B_data + obb + k : reinterpret_cast<const T *>(safe));
    }
#pragma unroll
    for (int u = 0; u < kMergeCap; ++u) {
        const int owner = first + 2 * u;
        s_col[k * kMergeStride + owner] = have[u] ? (int32_t)col[u] : kColEnd;
        if (VALUES) s_val[k * kMergeStride + owner] = have[u] ? val[u] : T(0);
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
}

// First kernel of the symbolic phase, over all rows in their natural order.  Eight
// lanes per row gather the lengths of the B rows it names.  Rows that qualify for
// the merge path are counted here (key = kMergedKey); for the others key[i] is the
// product bound min(sum of B row lengths, 2^31 - 8) that the hash path bins on.
__global__ __launch_bounds__(kBlock) void symbolic_front_kernel(
    int64_t rows, int64_t nbatch_padded, const int64_t *__restrict__ A_indices,
    const int64_t *__restrict__ A_indptr, const int64_t *__restrict__ B_indices,
    const int64_t *__restrict__ B_indptr, int32_t *__restrict__ key, int32_t *__restrict__ C_count,
    unsigned long long *__restrict__ hash_rows, unsigned long long token, uint64_t *__restrict__ dest,
    int32_t *__restrict__ bstart) {
    __shared__ int32_t s_col[(kMergeCap + 1) * kMergeStride];
    __shared__ int64_t s_bb[kBlock];
    __shared__ int32_t s_len[kBlock];
    const int gl = merge_lane();
    if (blockIdx.x == 0 && threadIdx.x == 0) C_count[rows] = 0;   // the scan's last entry: nnz(C)
    const int64_t batch = nm::xcd_tile(blockIdx.x, nbatch_padded);
    const int64_t row = batch * kMergeRows + (threadIdx.x >> 6) * 8 + merge_group();
    const bool live = row < rows;
    const int64_t ab = live ? A_indptr[row] : 0, ae = live ? A_indptr[row + 1] : 0;
    int64_t ub = 0, my_bb = 0;
    int32_t mx = 0, my_len = 0;
    for (int64_t a = ab + gl; a < ae; a += 8) {
        const int64_t j = A_indices[a];
        const int64_t bb = B_indptr[j], len = B_indptr[j + 1] - bb;
        ub += len;
        const int32_t l32 = (int32_t)(len > kMergeCap + 1 ? kMergeCap + 1 : len);
        mx = max(mx, l32);
        if (a - ab < 8) {
            my_bb = bb;
            my_len = l32;
        }
    }
    const int32_t ubc = merge_sum((int32_t)(ub > 0x0fffffff ? 0x0fffffff : ub));
    const bool merge = live && (ae - ab) <= kMergeCap && merge_max(mx) <= kMergeCap;
    if (live && !merge && gl == 0) key[row] = ubc;
    // A row left to the hash path raises a flag (a plain store of the same value by whoever finds one:
    // a counter that every wavefront of a product of long rows adds to would be a quarter of a
    // million atomics on one address); the exact count comes from the binning, if it runs.  The flag
    // is raised by writing the call's token, so that nobody need lower it first: whatever the word
    // held before is not this call's token, or at worst makes the hash path run over no rows.
    if (live && !merge && gl == 0) *hash_rows = token;
    merge_stage<float, false>(my_bb, merge ? my_len : 0, B_indices, nullptr, A_indptr, s_bb, s_len, s_col, nullptr);
    int32_t *pc = s_col + threadIdx.x;
    int32_t cur = *pc;
    int it = 0, last = -1;
    // The merge also leaves behind WHERE every product goes: the pass in which the k-th entry of a
    // lane's B row is taken is the position of that entry's column in the row of C.  A column that
    // has been taken is not needed again, so the pass is written over it in LDS -- one store, where
    // shifting it into a 64-bit word cost five vector instructions in a loop that is bound by what
    // it issues -- and the words the numeric phase adds the products up on (byte k = the pass of
    // entry k, 0xFF: no such entry; also what a product plan is made of) are put together after the
    // loop: the low byte of a place never taken is the past-the-end column's, 0xFF.
    static_assert((kColEnd & 0xFF) == 0xFF, "an entry never taken reads as no entry");
    for (;;) {
        const int32_t m = merge_min(cur);
        const bool open = m != kColEnd;
        if (__ballot(open) == 0) break;
        if (cur == m && open) {
            last = it;
            *pc = it;
            pc += kMergeStride;
            cur = *pc;
        }
        ++it;
    }
    const int cnt = merge_max(last) + 1;   // an open group emits one column per pass
    if (merge && gl == 0) {
        C_count[row] = cnt;
        key[row] = kMergedKey;
    }
    if (dest && merge && ab + gl < ae) {   // (read once, by another kernel: nontemporal)
        const int32_t *mine = s_col + threadIdx.x;
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            lo |= ((uint32_t)mine[j * kMergeStride] & 0xFFu) << (8 * j);
            hi |= ((uint32_t)mine[(4 + j) * kMergeStride] & 0xFFu) << (8 * j);
        }
        const uint64_t where = ((uint64_t)hi << 32) | lo;
        __builtin_nontemporal_store(where, dest + ab + gl);
        __builtin_nontemporal_store((int32_t)my_bb, bstart + ab + gl);
    }
}

// Numeric counterpart: rows marked kMergedKey are produced here, in natural order.
// The B rows are staged in LDS (columns and values); each pass emits the smallest head column and the sum of the
// matching products, accumulated from +0.0 in lane order, which is the order in
// which the serial loop adds them (cpp/sparse_csr_cpu.cpp:193-200).
template <typename T>
__global__ __launch_bounds__(kBlock) void numeric_front_kernel(
    int64_t rows, int64_t nbatch_padded, const int32_t *__restrict__ key, const T *__restrict__ A_data,
    const int64_t *__restrict__ A_indices, const int64_t *__restrict__ A_indptr, const T *__restrict__ B_data,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr,
    const int64_t *__restrict__ C_indptr, int64_t *__restrict__ C_indices, T *__restrict__ C_data) {
    __shared__ int32_t s_col[(kMergeCap + 1) * kMergeStride];
    __shared__ T s_val[kMergeCap * kMergeStride];
    __shared__ int64_t s_bb[kBlock];
    __shared__ int32_t s_len[kBlock];
    const int gl = merge_lane();
    const int64_t batch = nm::xcd_tile(blockIdx.x, nbatch_padded);
    const int64_t row = batch * kMergeRows + (threadIdx.x >> 6) * 8 + merge_group();
    // the row's bounds are requested together with its key: one memory round trip instead of two
    const bool live = row < rows;
    const int32_t my_key = live ? key[row] : 0;
    const int64_t ab0 = live ? A_indptr[row] : 0, ae0 = live ? A_indptr[row + 1] : 0;
    const int64_t out0 = live ? C_indptr[row] : 0;
    const bool merge = live && my_key == kMergedKey;
    if (__ballot(merge) == 0) return;   // wavefront-uniform; no workgroup barrier below
    const int64_t ab = merge ? ab0 : 0, ae = merge ? ae0 : 0;
    const bool mine = ab + gl < ae;
    const T av_raw = *(mine ? A_data + ab + gl : reinterpret_cast<const T *>(A_indptr));
    const int64_t j = mine ? *(A_indices + ab + gl) : 0;
    const T av = mine ? av_raw : T(0);
    const int64_t *bp = mine ? B_indptr + j : A_indptr;   // A_indptr: any two readable entries
    const int64_t bb = bp[0];
    const int my_len = mine ? (int)(bp[1] - bb) : 0;
    merge_stage<T, true>(bb, my_len, B_indices, B_data, A_indptr, s_bb, s_len, s_col, s_val);
    // lanes that take part in the ordered sum: the longest row of A in this wavefront
    int steps = 1;
#pragma unroll
    for (int q = kMergeCap; q > 1; --q)
        if (steps == 1 && __ballot((ae - ab) >= q) != 0) steps = q;
    // Emitted entries pass through a ring of 8 per group so that the group writes
    // them 8 at a time (one 64-byte piece per array) instead of lane by lane.
    // The ring reuses the exchange arrays of merge_stage, which are dead by now FOR THIS
    // WAVEFRONT: its ring entries and its exchange entries must be the same 64 slots, because
    // another wavefront of the workgroup may still be reading its own exchange entries (there
    // is no workgroup barrier).  A value therefore takes a whole 8-byte slot of s_bb whatever
    // T is (packed floats would put the ring of wavefront w over the exchange entries of
    // wavefront w / 2, which then read a wrong row start).
    static_assert(sizeof(T) <= sizeof(s_bb[0]), "a ring value must fit one exchange slot of s_bb");
    static_assert(sizeof(s_bb) / sizeof(s_bb[0]) == kBlock && sizeof(s_len) / sizeof(s_len[0]) == kBlock,
                  "one exchange slot per lane: wavefront w owns slots [64 w, 64 w + 64)");
    static_assert(8 /* groups per wavefront */ * 8 /* ring entries per group */ == nm::kWave,
                  "the ring of a wavefront must cover exactly that wavefront's own exchange slots");
    int32_t *s_oc = s_len;
    auto s_ov = [&](int slot) -> T & { return *reinterpret_cast<T *>(s_bb + slot); };
    const int ring = ((threadIdx.x >> 6) * 8 + merge_group()) * 8;
    int emitted = 0;   // entries of this row produced so far
    auto flush = [&](int base) {
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        const int e = base + gl;
        if (e < emitted) {
            C_indices[out0 + e] = (int64_t)s_oc[ring + gl];
            C_data[out0 + e] = s_ov(ring + gl);
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    };
    const int32_t *pc = s_col + threadIdx.x;   // this lane's head column / value slots
    const T *pv = s_val + threadIdx.x;
    int32_t cur = *pc;
    T curv = av * *pv;
    int it = 0;
    for (;;) {
        const int32_t m = merge_min(cur);
        const bool open = m != kColEnd;
        if (__ballot(open) == 0) break;
        const bool hit = cur == m && open;
        const T x = hit ? curv : T(0);
        T t;
        if (__ballot(merge_sum(hit ? 1 : 0) > 2) == 0) {
            // at most two products per entry anywhere in the wavefront: a sum of two
            // terms (and exact zeros) does not depend on the order of the additions
            t = x + nm::dpp_move_zero<0x122>(x);
            t += nm::dpp_move_zero<0x124>(t);
            t += nm::dpp_move_zero<0x128>(t);
        } else {
            t = T(0);
#pragma unroll
            for (int q = 0; q < kMergeCap; ++q) {
                if (q >= steps) break;
                t = x + nm::dpp_move_zero<0x112>(t);   // row_shr 2: previous lane of the group, 0 for the first
            }
        }
        // every group that is still open has emitted exactly `it` entries so far
        if (gl == steps - 1 && open) {
            s_oc[ring + (it & 7)] = m;
            s_ov(ring + (it & 7)) = t;
        }
        ++it;
        if (open) emitted = it;
        if ((it & 7) == 0) flush(it - 8);
        if (hit) {
            pc += kMergeStride;
            pv += kMergeStride;
            cur = *pc;
            curv = av * (cur != kColEnd ? *pv : T(0));   // no value slot behind the end marker
        }
    }
    if (it & 7) flush(it & ~7);
}

// key[i] = C_indptr[i+1] - C_indptr[i], except for rows the merge path has taken
__global__ void row_length_kernel(int64_t rows, const int64_t *__restrict__ C_indptr,
                                  int32_t *__restrict__ key) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < rows; i += stride)
        if (key[i] != kMergedKey) key[i] = (int32_t)(C_indptr[i + 1] - C_indptr[i]);
}

// negative keys (rows taken by the merge path) belong to no bin
struct BinLimits { int32_t l[kBins - 1]; };
__device__ __forceinline__ int bin_of(int32_t k, const BinLimits &lim) {
    if (k < 0) return -1;
    int b = 0;
#pragma unroll
    for (int q = 0; q < kBins - 1; ++q) b += k > lim.l[q];
    return b;
}

__global__ void bin_clear_kernel(int32_t *bins) {
    if (threadIdx.x < kBinInts) bins[threadIdx.x] = 0;
}

// Rows per bin.  Each wavefront counts with ballots (one population count per
// bin) instead of 64 colliding LDS atomics.
__global__ __launch_bounds__(kBlock) void bin_count_kernel(int64_t rows, const int32_t *__restrict__ key,
                                                           BinLimits lim, int32_t *bins) {
    __shared__ int s_cnt[kBins];
    if (threadIdx.x < kBins) s_cnt[threadIdx.x] = 0;
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1);
    int mine[kBins] = {};
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i0 = (int64_t)blockIdx.x * blockDim.x; i0 < rows; i0 += stride) {
        const int64_t i = i0 + threadIdx.x;
        const int b = i < rows ? bin_of(key[i], lim) : -1;
#pragma unroll
        for (int q = 0; q < kBins; ++q) mine[q] += __popcll(__ballot(b == q));
    }
    if (lane == 0)
        for (int q = 0; q < kBins; ++q)
            if (mine[q]) atomicAdd(&s_cnt[q], mine[q]);
    __syncthreads();
    if (threadIdx.x < kBins && s_cnt[threadIdx.x]) atomicAdd(bins + threadIdx.x, s_cnt[threadIdx.x]);
}

__global__ void bin_offsets_kernel(int32_t *bins) {
    if (threadIdx.x == 0) {
        int32_t run = 0;
        for (int b = 0; b < kBins; ++b) {
            bins[kBinStart + b] = run;
            bins[kBinCursor + b] = run;
            run += bins[b];
        }
        bins[kBinStart + kBins] = run;
    }
}

// Rows are placed a workgroup at a time, wavefront by wavefront and lane by lane, so that each
// bin keeps them in ascending order inside a workgroup's slice (neighbouring rows share B rows
// and C lines).  A workgroup takes ONE contiguous slice of the rows, counts it, claims its room
// in every bin with one atomic per bin, and then places the rows: thousands of workgroups claiming
// room 256 rows at a time queued up on the eight cursors (96 us for 2.1 M rows).
__global__ __launch_bounds__(kBlock) void bin_scatter_kernel(int64_t rows, const int32_t *__restrict__ key,
                                                             BinLimits lim, int32_t *bins,
                                                             int32_t *__restrict__ perm) {
    constexpr int kWaves = kBlock / kWave;
    __shared__ int s_wave[kWaves][kBins];   // rows of bin q in wavefront w (of the slice, then of a step)
    __shared__ int s_base[kBins];           // where the workgroup's next rows of bin q go
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t per = ((rows + gridDim.x - 1) / gridDim.x + kBlock - 1) / kBlock * kBlock;   // whole steps
    const int64_t r0 = (int64_t)blockIdx.x * per, r1 = r0 + per < rows ? r0 + per : rows;
    if (r0 >= rows) return;
    {   // count the slice
        int mine[kBins] = {};
        for (int64_t i0 = r0; i0 < r1; i0 += kBlock) {
            const int64_t i = i0 + threadIdx.x;
            const int b = i < r1 ? bin_of(key[i], lim) : -1;
#pragma unroll
            for (int q = 0; q < kBins; ++q) mine[q] += __popcll(__ballot(b == q));
        }
        if (lane == 0)
            for (int q = 0; q < kBins; ++q) s_wave[wave][q] = mine[q];
        __syncthreads();
        if (threadIdx.x < kBins) {
            int total = 0;
            for (int w = 0; w < kWaves; ++w) total += s_wave[w][threadIdx.x];
            s_base[threadIdx.x] = total ? atomicAdd(bins + kBinCursor + threadIdx.x, total) : 0;
        }
        __syncthreads();
    }
    for (int64_t i0 = r0; i0 < r1; i0 += kBlock) {
        const int64_t i = i0 + threadIdx.x;
        const int b = i < r1 ? bin_of(key[i], lim) : -1;
        int before = 0;   // rows of my bin in lower lanes of my wavefront
#pragma unroll
        for (int q = 0; q < kBins; ++q) {
            const unsigned long long m = __ballot(b == q);
            if (b == q) before = __popcll(m & ((1ull << lane) - 1ull));
            if (lane == 0) s_wave[wave][q] = __popcll(m);
        }
        __syncthreads();
        if (b >= 0) {
            int off = s_base[b] + before;
            for (int w = 0; w < wave; ++w) off += s_wave[w][b];
            perm[off] = (int32_t)i;
        }
        __syncthreads();
        if (threadIdx.x < kBins) {   // this step's rows are placed: the next step's go behind them
            int total = 0;
            for (int w = 0; w < kWaves; ++w) total += s_wave[w][threadIdx.x];
            s_base[threadIdx.x] += total;
        }
        __syncthreads();
    }
}

// Sums of the rows' counts by tile of kScanTile rows: the first pass of the row pointer's scan.
typedef int32_t I32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bool count_tile_whole(const int32_t *a, int64_t n) {
    static_assert(nm::kScanItems % 4 == 0, "counts are loaded four at a time");
    return ((int64_t)blockIdx.x + 1) * nm::kScanTile <= n && (reinterpret_cast<uintptr_t>(a) & 15) == 0;
}
__global__ __launch_bounds__(nm::kScanBlock) void count_tile_sums_kernel(const int32_t *__restrict__ count, int64_t n,
                                                                       int64_t *__restrict__ sums) {
    __shared__ int64_t s_wave[nm::kScanBlock / kWave];
    const int64_t base = (int64_t)blockIdx.x * nm::kScanTile + (int64_t)threadIdx.x * nm::kScanItems;
    int64_t v = 0;
    if (count_tile_whole(count, n)) {
        const I32x4 *p = reinterpret_cast<const I32x4 *>(count + base);
#pragma unroll
        for (int i = 0; i < nm::kScanItems / 4; ++i) {
            const I32x4 w = p[i];
            v += (int64_t)w[0] + w[1] + w[2] + w[3];
        }
    } else {
#pragma unroll
        for (int i = 0; i < nm::kScanItems; ++i)
            if (base + i < n) v += count[base + i];
    }
    int64_t total;
    nm::block_exclusive_scan(v, s_wave, total);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// Row pointer of C from the rows' counts, and what the host needs between the phases: nnz(C) and
// the rows the hash path took.  count[0, n) with count[n - 1] == 0 -> C_indptr[0, n) (its exclusive
// scan, not in place: the counts of the merge path's rows survive a pass made before the hash
// path's rows are counted).  `sums` holds the sum of every tile of kScanTile counts; with
// `scanned` == 0 a workgroup adds up the sums before its own (a few thousand numbers out of L2
// against one more launch), otherwise they have been scanned already (their total behind them).
// The first workgroup, with nothing before it, adds up all tiles instead: nnz(C), which it leaves
// in summary[0], with the number of hash-path rows in summary[1] (from `bins`; where bins is null,
// 1 if the first kernel has left `token` there).  With `host_pinned` it also drops both into the
// host's landing place, followed by the ticket the host polls for: the host needs the numbers,
// not the row pointer, so it is told first and sizes C while the row pointer is being written.
constexpr int kInlineTiles = 4096;
__global__ __launch_bounds__(nm::kScanBlock) void row_pointer_kernel(
    const int32_t *__restrict__ count, int64_t n, const int64_t *__restrict__ sums, int scanned,
    int64_t *__restrict__ C_indptr, const int32_t *__restrict__ bins, int64_t *__restrict__ summary,
    int64_t token, volatile int64_t *host_pinned, int64_t ticket) {
    using nm::kScanItems;
    __shared__ int64_t s_wave[nm::kScanBlock / kWave];
    const int64_t base = (int64_t)blockIdx.x * nm::kScanTile + (int64_t)threadIdx.x * kScanItems;
    int32_t item[kScanItems];
    int64_t v = 0;
    const bool whole = count_tile_whole(count, n) && (reinterpret_cast<uintptr_t>(C_indptr) & 15) == 0;
    if (whole) {
        const I32x4 *p = reinterpret_cast<const I32x4 *>(count + base);
#pragma unroll
        for (int i = 0; i < kScanItems / 4; ++i) {
            const I32x4 w = p[i];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                item[4 * i + u] = w[u];
                v += w[u];
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < kScanItems; ++i) {
            item[i] = base + i < n ? count[base + i] : 0;
            v += item[i];
        }
    }
    // (the first workgroup, which has nothing before it, adds up all tiles instead: nnz(C), for the host)
    int64_t before;
    if (scanned) {
        before = sums[blockIdx.x == 0 ? gridDim.x : blockIdx.x];
    } else {
        const int upto = blockIdx.x == 0 ? (int)gridDim.x : (int)blockIdx.x;
        int64_t part = 0;
        for (int t = threadIdx.x; t < upto; t += nm::kScanBlock) part += sums[t];
        nm::block_exclusive_scan(part, s_wave, before);
    }
    if (blockIdx.x == 0) {
        if (threadIdx.x == 0) {
            const int64_t nnz = before;
            const int64_t hashed = bins ? (int64_t)bins[kBinStart + kBins] : (summary[1] == token ? 1 : 0);
            summary[0] = nnz;
            summary[1] = hashed;
            if (host_pinned) {
                host_pinned[0] = nnz;
                host_pinned[1] = hashed;
                __threadfence_system();
                host_pinned[2] = ticket;
            }
        }
        before = 0;
    }
    int64_t total;
    int64_t run = before + nm::block_exclusive_scan(v, s_wave, total);
    if (whole) {
        nm::I64x2 *p = reinterpret_cast<nm::I64x2 *>(C_indptr + base);
#pragma unroll
        for (int i = 0; i < kScanItems / 2; ++i) {
            nm::I64x2 w;
            w[0] = run;
            w[1] = run + item[2 * i];
            run = w[1] + item[2 * i + 1];
            p[i] = w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < kScanItems; ++i) {
            if (base + i < n) C_indptr[base + i] = run;
            run += item[i];
        }
    }
}

// host_pinned[0..1] = summary, then host_pinned[2] = ticket: the host polls the ticket.
__global__ void summary_out_kernel(const int64_t *__restrict__ summary, volatile int64_t *host_pinned,
                                   int64_t ticket) {
    if (threadIdx.x == 0) {
        host_pinned[0] = summary[0];
        host_pinned[1] = summary[1];
        __threadfence_system();
        host_pinned[2] = ticket;
    }
}

// The four binning steps by one workgroup, for so few rows that the launches cost more than the
// work: count, offsets, then rows placed in ascending order inside each bin (ballots, as in the
// grid-wide kernels).
constexpr int kBinSmallRows = 4096;
__global__ __launch_bounds__(1024) void bin_small_kernel(int64_t rows, const int32_t *__restrict__ key,
                                                         BinLimits lim, int32_t *bins,
                                                         int32_t *__restrict__ perm) {
    constexpr int kWaves = 1024 / kWave;
    __shared__ int s_cnt[kWaves][kBins];
    __shared__ int s_start[kBins + 1], s_run[kBins];
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // rows per bin
    int mine[kBins] = {};
    for (int64_t i0 = 0; i0 < rows; i0 += 1024) {
        const int64_t i = i0 + threadIdx.x;
        const int b = i < rows ? bin_of(key[i], lim) : -1;
#pragma unroll
        for (int q = 0; q < kBins; ++q) mine[q] += __popcll(__ballot(b == q));
    }
    if (lane == 0)
        for (int q = 0; q < kBins; ++q) s_cnt[wave][q] = mine[q];
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int q = 0; q < kBins; ++q) {
            s_start[q] = run;
            s_run[q] = run;
            for (int w = 0; w < kWaves; ++w) run += s_cnt[w][q];
        }
        s_start[kBins] = run;
    }
    __syncthreads();
    // rows placed chunk by chunk, wavefront by wavefront, lane by lane: ascending inside each bin
    for (int64_t i0 = 0; i0 < rows; i0 += 1024) {
        const int64_t i = i0 + threadIdx.x;
        const int b = i < rows ? bin_of(key[i], lim) : -1;
        int before = 0;
#pragma unroll
        for (int q = 0; q < kBins; ++q) {
            const unsigned long long m = __ballot(b == q);
            if (b == q) before = __popcll(m & ((1ull << lane) - 1ull));
            if (lane == 0) s_cnt[wave][q] = __popcll(m);
        }
        __syncthreads();
        if (b >= 0) {
            int off = s_run[b] + before;
            for (int w = 0; w < wave; ++w) off += s_cnt[w][b];
            perm[off] = (int32_t)i;
        }
        __syncthreads();
        if (threadIdx.x < kBins) {
            int t = 0;
            for (int w = 0; w < kWaves; ++w) t += s_cnt[w][threadIdx.x];
            s_run[threadIdx.x] += t;
        }
        __syncthreads();
    }
    if (threadIdx.x <= kBins) bins[kBinStart + threadIdx.x] = s_start[threadIdx.x];
    if (threadIdx.x < kBins) bins[threadIdx.x] = s_start[threadIdx.x + 1] - s_start[threadIdx.x];
}

int bin_rows(int64_t rows, const int32_t limit[kBins - 1], const Work &w, hipStream_t s) {
    BinLimits lim;
    for (int q = 0; q < kBins - 1; ++q) lim.l[q] = limit[q];
    if (rows <= kBinSmallRows) {
        hipLaunchKernelGGL(bin_small_kernel, dim3(1), dim3(1024), 0, s, rows, w.key, lim, w.bins, w.perm);
        NM_LAUNCH_CHECK("bin_small_kernel");
        return NM_OK;
    }
    // (few enough workgroups that their atomics on the eight counters and cursors do not queue up)
    int64_t grid = nm::ceil_div(rows, kBlock);
    if (grid > 512) grid = 512;
    if (grid < 1) grid = 1;
    hipLaunchKernelGGL(bin_clear_kernel, dim3(1), dim3(64), 0, s, w.bins);
    hipLaunchKernelGGL(bin_count_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, rows, w.key, lim, w.bins);
    hipLaunchKernelGGL(bin_offsets_kernel, dim3(1), dim3(64), 0, s, w.bins);
    hipLaunchKernelGGL(bin_scatter_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, rows, w.key, lim, w.bins,
                       w.perm);
    NM_LAUNCH_CHECK("bin kernels");
    return NM_OK;
}

// ---- symbolic ----------------------------------------------------------------

template <int G, int TABLE>
__global__ __launch_bounds__(kBlock) void symbolic_hash_kernel(
    int bin, const int32_t *__restrict__ bins, const int32_t *__restrict__ perm,
    const int64_t *__restrict__ A_indices, const int64_t *__restrict__ A_indptr,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr,
    int32_t *__restrict__ C_count) {
    constexpr int GPB = kBlock / G;
    // the tables of the groups that share a wavefront start kTablePad entries apart in
    // bank space; without the pad they would all map slot t to the same LDS bank
    constexpr int STRIDE = TABLE + (GPB > 1 ? kTablePad : 0);
    __shared__ __align__(16) int32_t s_keys[GPB * STRIDE];
    __shared__ int s_red[kBlock / kWave];
    const int gl = threadIdx.x % G, gi = G >= kWave ? __builtin_amdgcn_readfirstlane(threadIdx.x / G) : threadIdx.x / G;
    int32_t *tab = s_keys + gi * STRIDE;
    const int32_t b0 = bins[kBinStart + bin], b1 = bins[kBinStart + bin + 1];
    for (int32_t idx0 = b0 + blockIdx.x * GPB; idx0 < b1; idx0 += gridDim.x * GPB) {
        const int32_t idx = idx0 + gi;
        const bool live = idx < b1;
        for (int t = gl; t < TABLE; t += G) tab[t] = kEmpty;
        group_sync<G>();
        int cnt = 0;
        int64_t row = 0;
        auto insert = [&](int32_t key) {
            uint32_t h = first_slot<TABLE>(key);
            int32_t old = atomicCAS(&tab[h], kEmpty, key);
            while (old != kEmpty && old != key) {   // one exit test: the common case probes once
                h = (h + 1) & (TABLE - 1);
                old = atomicCAS(&tab[h], kEmpty, key);
            }
            cnt += old == kEmpty;
        };
        {
            // Latency-lean walk: each lane fetches one entry of A's row together with the
            // bounds of the B row it names; the first S columns of up to kAhead B rows are
            // then requested back to back before any of them is inserted.  A group wider than
            // a wavefront gives each of its wavefronts its own 64 entries of A's row (the
            // order of insertion does not matter for the count).
            constexpr int S = G < kWave ? G : kWave;
            // A group of 16 lanes takes TWO rows of B per step, eight lanes each: the rows these bins
            // see are mostly shorter than eight entries (stencil powers), and insertion into a set
            // has no order to keep, so the second half of the group need not idle.
            constexpr int W = G == 16 ? 8 : S, NSUB = S / W;
            const int sl = gl & (S - 1), sub = G > kWave ? __builtin_amdgcn_readfirstlane(gl / S) : 0;
            const int hl = sl & (W - 1), half = sl / W;
            const int gbase = (threadIdx.x & (kWave - 1)) & ~(S - 1);
            row = live ? perm[idx] : 0;
            const int64_t ab = live ? A_indptr[row] : 0, ae = live ? A_indptr[row + 1] : 0;
            for (int64_t a0 = ab + sub * S; a0 < ae; a0 += G) {
                const int64_t my_ai = a0 + sl;
                const bool mine = my_ai < ae;
                const int64_t my_j = mine ? A_indices[my_ai] : 0;
                const int64_t my_bb = mine ? B_indptr[my_j] : 0, my_be = mine ? B_indptr[my_j + 1] : 0;
                const int nb = (int)(ae - a0 < S ? ae - a0 : S);
                if constexpr (G == 16) {
                    // the group is one DPP row: entries 2 u and 2 u + 1 of A's row reach the two halves
                    // by row broadcasts instead of shuffles through the LDS crossbar, and the bounds of a
                    // row of B longer than eight entries are fetched again where its rest is walked
                    static_assert(kAhead * NSUB == G && W == 8, "one batch of pairs covers the group");
                    const int my_len = (int)(my_be - my_bb);
                    int32_t qk[kAhead];
                    nm::static_for<kAhead>([&](auto uc) {
                        constexpr int U = decltype(uc)::value;
                        // (broadcasts first, with all sixteen lanes active; then the lane's own tests)
                        const int64_t kk = nm::row_lane_halves<2 * U, 2 * U + 1>(my_bb) + hl;
                        const int len = nm::row_lane_halves<2 * U, 2 * U + 1>(my_len);
                        const bool ok = (2 * U + half < nb) & (hl < len);
                        qk[U] = ok ? (int32_t)B_indices[kk] : kEmpty;
                    });
                    nm::static_for<kAhead>([&](auto uc) {
                        constexpr int U = decltype(uc)::value;
                        if (2 * U >= nb) return;
                        if (qk[U] != kEmpty) insert(qk[U]);
                        // (the test is the same in all sixteen lanes, so that the broadcasts behind it
                        // find their source lanes active)
                        const int len_lo = nm::row_lane<2 * U>(my_len), len_hi = nm::row_lane<2 * U + 1>(my_len);
                        if ((len_lo > W) | (len_hi > W)) {   // (lanes past the row's end hold a length of 0)
                            const int64_t bb = nm::row_lane_halves<2 * U, 2 * U + 1>(my_bb);
                            const int64_t be_row = nm::row_lane_halves<2 * U, 2 * U + 1>(my_be);
                            const int64_t be = 2 * U + half < nb ? be_row : bb;
                            for (int64_t kk = bb + W + hl; kk < be; kk += W) insert((int32_t)B_indices[kk]);
                        }
                    });
                } else
                for (int e0 = 0; e0 < nb; e0 += kAhead * NSUB) {
                    int32_t pk[kAhead];
                    int64_t bbs[kAhead], bes[kAhead];
                    bool has[kAhead];
#pragma unroll
                    for (int u = 0; u < kAhead; ++u) {
                        const int e = e0 + u * NSUB + half;
                        has[u] = e < nb;
                        const int src = gbase + (has[u] ? e : e0);
                        bbs[u] = __shfl(my_bb, src, kWave);
                        bes[u] = __shfl(my_be, src, kWave);
                        const int64_t kk = bbs[u] + hl;
                        pk[u] = (has[u] && kk < bes[u]) ? (int32_t)B_indices[kk] : kEmpty;
                    }
#pragma unroll
                    for (int u = 0; u < kAhead; ++u) {
                        if (e0 + u * NSUB >= nb) break;
                        if (pk[u] != kEmpty) insert(pk[u]);
                        if (has[u])
                            for (int64_t kk = bbs[u] + W + hl; kk < bes[u]; kk += W) insert((int32_t)B_indices[kk]);
                    }
                }
            }
        }
        cnt = group_total<G>(cnt, s_red);
        if (live && gl == 0) C_count[row] = cnt;
        group_sync<G>();
    }
}

// Spill path: distinct columns counted with a stamped dense marker per workgroup.
__global__ __launch_bounds__(kSpillBlock) void symbolic_spill_kernel(
    const int32_t *__restrict__ bins, const int32_t *__restrict__ perm, int64_t B_cols,
    const int64_t *__restrict__ A_indices, const int64_t *__restrict__ A_indptr,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr, int32_t *mark_all,
    int32_t *__restrict__ C_count) {
    __shared__ int s_red[kSpillBlock / kWave];
    const int32_t b0 = bins[kBinStart + kBins - 1], b1 = bins[kBinStart + kBins];
    if (b0 + (int32_t)blockIdx.x >= b1) return;
    int32_t *mark = mark_all + (size_t)blockIdx.x * (B_cols + 1);
    for (int64_t c = threadIdx.x; c < B_cols; c += kSpillBlock) mark[c] = 0;
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    for (int32_t idx = b0 + blockIdx.x; idx < b1; idx += gridDim.x) {
        const int64_t row = perm[idx];
        const int32_t stamp = (int32_t)row + 1;
        int cnt = 0;
        const int64_t je = A_indptr[row + 1];
        for (int64_t jj = A_indptr[row] + wave; jj < je; jj += kSpillBlock / kWave) {
            const int64_t j = A_indices[jj];
            const int64_t ke = B_indptr[j + 1];
            for (int64_t kk = B_indptr[j] + lane; kk < ke; kk += kWave)
                if (atomicExch(mark + B_indices[kk], stamp) != stamp) ++cnt;
        }
        cnt = nm::wave_sum(cnt);
        if (lane == 0) s_red[wave] = cnt;
        __syncthreads();
        if (threadIdx.x == 0) {
            int t = 0;
            for (int w = 0; w < kSpillBlock / kWave; ++w) t += s_red[w];
            C_count[row] = t;
        }
        __syncthreads();
    }
}

// ---- numeric -------------------------------------------------------------------

template <typename T, int G, int TABLE>
__global__ __launch_bounds__(kBlock) void numeric_hash_kernel(
    int bin, const int32_t *__restrict__ bins, const int32_t *__restrict__ perm,
    const T *__restrict__ A_data, const int64_t *__restrict__ A_indices,
    const int64_t *__restrict__ A_indptr, const T *__restrict__ B_data,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr,
    const int64_t *__restrict__ C_indptr, int64_t *__restrict__ C_indices, T *__restrict__ C_data) {
    constexpr int GPB = kBlock / G;
    constexpr int STRIDE = TABLE + (GPB > 1 ? kTablePad : 0);   // see symbolic_hash_kernel
    extern __shared__ __align__(16) unsigned char s_raw[];
    T *s_vals = reinterpret_cast<T *>(s_raw);
    int32_t *s_keys = reinterpret_cast<int32_t *>(s_raw + sizeof(T) * GPB * STRIDE);
    const int gl = threadIdx.x % G, gi = G >= kWave ? __builtin_amdgcn_readfirstlane(threadIdx.x / G) : threadIdx.x / G;
    int32_t *tab = s_keys + gi * STRIDE;
    T *val = s_vals + gi * STRIDE;
    // compacted (column, slot) lists used to order the row on the way out.  The groups that share
    // a wavefront keep them where the key table was (its keys are in registers by then): LDS per
    // row is what decides how many rows a CU has in flight.
    constexpr int CSTRIDE = TABLE / 2 + 4;
    constexpr bool ALIAS = G <= kWave;
    static_assert(!ALIAS || (CSTRIDE + TABLE / 4 <= TABLE && TABLE <= 65536), "the lists fit the key table");
    int32_t *ck = ALIAS ? tab : s_keys + GPB * STRIDE + gi * 2 * CSTRIDE;
    int32_t *cs = ck + CSTRIDE;
    uint16_t *cs16 = reinterpret_cast<uint16_t *>(cs);
    const int32_t b0 = bins[kBinStart + bin], b1 = bins[kBinStart + bin + 1];
    for (int32_t idx0 = b0 + blockIdx.x * GPB; idx0 < b1; idx0 += gridDim.x * GPB) {
        const int32_t idx = idx0 + gi;
        const bool live = idx < b1;
        for (int t = gl; t < TABLE; t += G) tab[t] = kEmpty;   // values are written by the first insert
        group_sync<G>();
        int64_t row = 0;
        auto add = [&](int32_t key, T prod) {
            uint32_t h = first_slot<TABLE>(key);
            int32_t old = atomicCAS(&tab[h], kEmpty, key);
            while (old != kEmpty && old != key) {   // one exit test: the common case probes once
                h = (h + 1) & (TABLE - 1);
                old = atomicCAS(&tab[h], kEmpty, key);
            }
            // The columns of one B row are distinct, so no other lane holds slot h now.  A slot
            // claimed just now holds no value yet: its first product is stored as it is
            // (0 + prod), the read of the slot is dropped by the select.
            const T cur = val[h];
            val[h] = old == kEmpty ? prod : cur + prod;
        };
        if (G <= kWave) {
            // Same latency-lean walk as the symbolic phase; entries of A's row are still
            // applied one after the other, so every output entry gets its products in
            // the order of A's row.
            const int gbase = (threadIdx.x & (kWave - 1)) & ~(G - 1);
            row = live ? perm[idx] : 0;
            const int64_t ab = live ? A_indptr[row] : 0, ae = live ? A_indptr[row + 1] : 0;
            for (int64_t a0 = ab; a0 < ae; a0 += G) {
                const int64_t my_ai = a0 + gl;
                const bool mine = my_ai < ae;
                const int64_t my_j = mine ? A_indices[my_ai] : 0;
                const T my_a = mine ? A_data[my_ai] : T(0);
                const int64_t my_bb = mine ? B_indptr[my_j] : 0, my_be = mine ? B_indptr[my_j + 1] : 0;
                const int nb = (int)(ae - a0 < G ? ae - a0 : G);
                int32_t pk[kAhead];
                T pv[kAhead], as[kAhead];
                int64_t bbs[kAhead], bes[kAhead];
                // the entries of A's row held by lanes e0 .. e0 + kAhead - 1 of the group, applied in turn
                auto apply = [&](int e0) {
#pragma unroll
                    for (int u = 0; u < kAhead; ++u) {
                        if (e0 + u >= nb) break;
                        if (pk[u] != kEmpty) add(pk[u], as[u] * pv[u]);
                        for (int64_t kk = bbs[u] + G + gl; kk < bes[u]; kk += G)
                            add((int32_t)B_indices[kk], as[u] * B_data[kk]);
                        group_sync<G>();  // the next entry of A's row adds after this one
                    }
                };
                if constexpr (G == 16) {
                    // A group is one 16-lane DPP row: what lane e of the group holds reaches the others
                    // by a row broadcast (one vector move per 32 bits) instead of a shuffle by lane
                    // number through the LDS crossbar.  That is cheap enough to fetch an entry's value
                    // and the bounds of its row of B again when they are used, so only the columns and
                    // values requested ahead stay in registers (116 -> fewer registers: more wavefronts).
                    constexpr int BATCH = NM_HASH_BATCH;   // rows of B requested ahead: 8 or 16
                    static_assert(G % BATCH == 0, "whole batches cover the group");
                    const int my_len = (int)(my_be - my_bb);
                    int32_t qk[BATCH];
                    T qv[BATCH];
                    auto batch = [&](auto first) {
                        constexpr int E0 = decltype(first)::value;
                        nm::static_for<BATCH>([&](auto uc) {
                            constexpr int U = decltype(uc)::value;
                            const int64_t kk = nm::row_lane<E0 + U>(my_bb) + gl;
                            const int len = nm::row_lane<E0 + U>(my_len);
                            const bool ok = (E0 + U < nb) & (gl < len);
                            qk[U] = ok ? (int32_t)B_indices[kk] : kEmpty;
                            qv[U] = ok ? B_data[kk] : T(0);
                        });
                        nm::static_for<BATCH>([&](auto uc) {
                            constexpr int U = decltype(uc)::value;
                            if (E0 + U >= nb) return;
                            const T a = nm::row_lane<E0 + U>(my_a);
                            if (qk[U] != kEmpty) add(qk[U], a * qv[U]);
                            if (nm::row_lane<E0 + U>(my_len) > G) {   // the rest of a row of B longer than the group
                                const int64_t bb = nm::row_lane<E0 + U>(my_bb), be = nm::row_lane<E0 + U>(my_be);
                                for (int64_t kk = bb + G + gl; kk < be; kk += G) add((int32_t)B_indices[kk], a * B_data[kk]);
                            }
                            group_sync<G>();  // the next entry of A's row adds after this one
                        });
                    };
                    batch(std::integral_constant<int, 0>{});
                    if constexpr (BATCH < G)
                        if (nb > BATCH) batch(std::integral_constant<int, BATCH < G ? BATCH : 0>{});
                } else {
                    for (int e0 = 0; e0 < nb; e0 += kAhead) {
#pragma unroll
                        for (int u = 0; u < kAhead; ++u) {
                            const int src = gbase + (e0 + u < nb ? e0 + u : e0);
                            bbs[u] = __shfl(my_bb, src, kWave);
                            bes[u] = __shfl(my_be, src, kWave);
                            as[u] = __shfl(my_a, src, kWave);
                            const int64_t kk = bbs[u] + gl;
                            const bool ok = e0 + u < nb && kk < bes[u];
                            pk[u] = ok ? (int32_t)B_indices[kk] : kEmpty;
                            pv[u] = ok ? B_data[kk] : T(0);
                        }
                        apply(e0);
                    }
                }
            }
        } else if (live) {
            // One row per workgroup.  Every lane fetches one entry of A's row and the bounds of
            // the B row it names into LDS (the compaction lists are free until the row is
            // complete); the entries are then applied in order, the first G columns of kAhead
            // B rows being requested before the first of them is added.
            static_assert(G <= kWave || 2 * CSTRIDE * 4 >= G * (16 + (int)sizeof(T)), "staging area");
            int64_t *s_bb = reinterpret_cast<int64_t *>(ck), *s_be = s_bb + G;
            T *s_a = reinterpret_cast<T *>(s_be + G);
            row = perm[idx];
            const int64_t ab = A_indptr[row], ae = A_indptr[row + 1];
            for (int64_t a0 = ab; a0 < ae; a0 += G) {
                const int64_t my_ai = a0 + gl < ae ? a0 + gl : ab;
                const int64_t my_j = A_indices[my_ai];
                s_a[gl] = A_data[my_ai];
                s_bb[gl] = B_indptr[my_j];
                s_be[gl] = B_indptr[my_j + 1];
                __syncthreads();
                const int nb = (int)(ae - a0 < G ? ae - a0 : G);
                for (int e0 = 0; e0 < nb; e0 += kAhead) {
                    int32_t pk[kAhead];
                    T pv[kAhead], as[kAhead];
                    int64_t bbs[kAhead], bes[kAhead];
#pragma unroll
                    for (int u = 0; u < kAhead; ++u) {
                        const int src = e0 + u < nb ? e0 + u : e0;
                        bbs[u] = s_bb[src];
                        bes[u] = s_be[src];
                        as[u] = s_a[src];
                        const int64_t kk = bbs[u] + gl;
                        const bool ok = e0 + u < nb && kk < bes[u];
                        pk[u] = ok ? (int32_t)B_indices[kk] : kEmpty;
                        pv[u] = ok ? B_data[kk] : T(0);
                    }
#pragma unroll
                    for (int u = 0; u < kAhead; ++u) {
                        if (e0 + u >= nb) break;
                        if (pk[u] != kEmpty) add(pk[u], as[u] * pv[u]);
                        for (int64_t kk = bbs[u] + G + gl; kk < bes[u]; kk += G)
                            add((int32_t)B_indices[kk], as[u] * B_data[kk]);
                        __syncthreads();  // the next entry of A's row adds after this one
                    }
                }
            }
        }
        if (G > kWave) __syncthreads();
        // Output in ascending column order.
        if constexpr (G > kWave) {
            // One row per workgroup, up to TABLE / 2 entries: the occupied slots are compacted
            // into a list of (column, slot) words, the list is padded to a power of two and
            // sorted by a bitonic network in LDS, and the row is written out in order.  (Ranking
            // every entry against the whole list, as the narrow groups do, grows with the square
            // of the row and took most of this kernel's time on rows of thousands of entries.)
            unsigned long long *list = reinterpret_cast<unsigned long long *>(ck);
            int *scr = reinterpret_cast<int *>(cs);
            int mine = 0;
            for (int t = gl; t < TABLE; t += G) mine += tab[t] != kEmpty;
            scr[gl] = mine;
            __syncthreads();
            int pos = 0, c = 0;
            for (int l2 = 0; l2 < G; ++l2) {
                const int v = scr[l2];
                if (l2 < gl) pos += v;
                c += v;
            }
            __syncthreads();
            for (int t = gl; t < TABLE; t += G) {
                const int32_t key = tab[t];
                if (key != kEmpty) list[pos++] = ((unsigned long long)(uint32_t)key << 32) | (uint32_t)t;
            }
            int P = 2 * kWave;
            while (P < c) P <<= 1;
            for (int t = c + gl; t < P; t += G) list[t] = ~0ull;
            __syncthreads();
            for (int k = 2; k <= P; k <<= 1) {
                for (int j = k >> 1; j > 0; j >>= 1) {
                    for (int t = gl; t < P / 2; t += G) {
                        const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1)), l = i | j;
                        const unsigned long long x = list[i], y = list[l];
                        if ((x > y) == ((i & k) == 0)) { list[i] = y; list[l] = x; }
                    }
                    // a wavefront's pairs stay inside its own 128 words while j <= 64
                    if (j > kWave) __syncthreads(); else group_sync<kWave>();
                }
                if (k >= 2 * kWave) __syncthreads();
            }
            if (live) {
                const int64_t base = C_indptr[row];
                for (int e = gl; e < c; e += G) {
                    const unsigned long long w = list[e];
                    C_indices[base + e] = (int64_t)(w >> 32);
                    C_data[base + e] = val[(uint32_t)w];
                }
            }
        } else {
            // The occupied slots are compacted into a dense list, then every entry is ranked
            // against that list only (its rank is its position in the row).  Rows fill at most
            // half of their table, so this is a fraction of the compares a rank over the whole
            // table would take.
            const int gbase = (threadIdx.x & (kWave - 1)) & ~(G - 1);
            constexpr int K = TABLE / G;
            int32_t keys[K];
            int mine = 0;
#pragma unroll
            for (int q = 0; q < K; ++q) {
                keys[q] = tab[gl + q * G];
                mine += keys[q] != kEmpty;
            }
            int incl = mine;
#pragma unroll
            for (int off = 1; off < G; off <<= 1) {
                const int up = __shfl_up(incl, off, kWave);
                if (gl >= off) incl += up;
            }
            const int c = __shfl(incl, gbase + G - 1, kWave);
            int pos = incl - mine;
            group_sync<G>();   // every lane holds its part of the table: the lists may take its place
#pragma unroll
            for (int q = 0; q < K; ++q)
                if (keys[q] != kEmpty) {
                    ck[pos] = keys[q];
                    cs16[pos] = (uint16_t)(gl + q * G);
                    ++pos;
                }
            if (gl < 4) ck[c + gl] = kEmpty;   // pad the list to a multiple of four keys
            group_sync<G>();
            if (live) {
                const int64_t base = C_indptr[row];
                const uint4 *ck4 = reinterpret_cast<const uint4 *>(ck);
                const int quads = (c + 3) >> 2;
                for (int e = gl; e < c; e += G) {
                    const uint32_t key = (uint32_t)ck[e];
                    int rank = 0;
                    for (int u = 0; u < quads; ++u) {   // four keys per LDS read; the pad never counts
                        const uint4 q = ck4[u];
                        rank += (q.x < key) + (q.y < key) + (q.z < key) + (q.w < key);
                    }
                    C_indices[base + rank] = (int64_t)key;
                    C_data[base + rank] = val[cs16[e]];
                }
            }
        }
        group_sync<G>();
    }
}

// Spill path: dense accumulator slice per workgroup, emitted by a scan of the
// touched column range (ascending by construction).
template <typename T>
__global__ __launch_bounds__(kSpillBlock) void numeric_spill_kernel(
    const int32_t *__restrict__ bins, const int32_t *__restrict__ perm, int64_t B_cols,
    const T *__restrict__ A_data, const int64_t *__restrict__ A_indices,
    const int64_t *__restrict__ A_indptr, const T *__restrict__ B_data,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr,
    const int64_t *__restrict__ C_indptr, int64_t *__restrict__ C_indices, T *__restrict__ C_data,
    int32_t *mark_all, double *acc_all) {
    __shared__ int64_t s_wave[kSpillBlock / kWave];
    __shared__ unsigned long long s_lo, s_hi;
    const int32_t b0 = bins[kBinStart + kBins - 1], b1 = bins[kBinStart + kBins];
    if (b0 + (int32_t)blockIdx.x >= b1) return;
    int32_t *mark = mark_all + (size_t)blockIdx.x * (B_cols + 1);
    T *acc = reinterpret_cast<T *>(acc_all + (size_t)blockIdx.x * (B_cols + 1));
    for (int64_t c = threadIdx.x; c < B_cols; c += kSpillBlock) { mark[c] = 0; acc[c] = T(0); }
    __syncthreads();
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    for (int32_t idx = b0 + blockIdx.x; idx < b1; idx += gridDim.x) {
        const int64_t row = perm[idx];
        const int32_t stamp = -((int32_t)row + 1);
        if (threadIdx.x == 0) { s_lo = ~0ull; s_hi = 0ull; }
        __syncthreads();
        unsigned long long lo = ~0ull, hi = 0ull;
        const int64_t je = A_indptr[row + 1];
        for (int64_t jj = A_indptr[row] + wave; jj < je; jj += kSpillBlock / kWave) {
            const int64_t j = A_indices[jj];
            const T a = A_data[jj];
            const int64_t ke = B_indptr[j + 1];
            for (int64_t kk = B_indptr[j] + lane; kk < ke; kk += kWave) {
                const unsigned long long c = (unsigned long long)B_indices[kk];
                nm::atomic_add(acc + c, a * B_data[kk]);
                mark[c] = stamp;
                lo = c < lo ? c : lo;
                hi = c > hi ? c : hi;
            }
        }
        if (lo != ~0ull) { atomicMin(&s_lo, lo); atomicMax(&s_hi, hi); }
        __syncthreads();
        const int64_t c_lo = (int64_t)s_lo, c_hi = (int64_t)s_hi;
        int64_t out = C_indptr[row];
        if (s_lo != ~0ull) {
            // Every wavefront takes a contiguous segment of the touched column range: it counts its
            // hits, the counts are summed over the wavefronts before it, and it then emits its
            // segment in order.  (A workgroup-wide scan per 1024 columns cost two barriers each.)
            constexpr int kWaves = kSpillBlock / kWave;
            const int64_t span = c_hi - c_lo + 1;
            const int64_t seg = ((span + kWaves - 1) / kWaves + kWave - 1) / kWave * kWave;
            const int64_t sb = c_lo + wave * seg;
            const int64_t se = sb + seg < c_hi + 1 ? sb + seg : c_hi + 1;
            int64_t cnt = 0;
            for (int64_t c0 = sb; c0 < se; c0 += kWave) {
                const int64_t c = c0 + lane;
                cnt += __popcll(__ballot(c < se && mark[c] == stamp));
            }
            if (lane == 0) s_wave[wave] = cnt;
            __syncthreads();
            for (int w = 0; w < wave; ++w) out += s_wave[w];
            const unsigned long long below = (1ull << lane) - 1ull;
            for (int64_t c0 = sb; c0 < se; c0 += kWave) {
                const int64_t c = c0 + lane;
                const bool hit = c < se && mark[c] == stamp;
                const unsigned long long m = __ballot(hit);
                if (hit) {
                    const int64_t at = out + __popcll(m & below);
                    C_indices[at] = c;
                    C_data[at] = acc[c];
                    acc[c] = T(0);
                }
                out += __popcll(m);
            }
        }
        __syncthreads();
    }
}

// ---- backward --------------------------------------------------------------------

// Backward.  A group of 8 lanes owns one row i of A.  Row i of C (column
// indices and upstream gradient, at most kBwdStage entries) is staged in LDS,
// so the per-product lookups are LDS bisections.  The group takes the row's entries
// (i,k) one at a time and spreads row k of B over its lanes, so the eight
// atomic updates of grad_B it issues land in one cache line (the L2 atomic
// units are bound by lines touched, not by lanes).  The products
// gC[i,c] * B[k,c] are then added lane by lane in ascending column order --
// the order of the reference's merge -- which keeps grad_A bit-identical.
//
// Rows of C longer than kBwdStage go to a second kernel in which a whole
// workgroup owns the row: its 32 groups share out the entries of A's row, whole
// wavefronts take the entries whose row of B is long, and the row of C is staged
// in LDS -- columns and gradient up to kBwdLongCap entries; columns only beyond
// that (every stride-th column past kBwdHugeCap entries: the last steps of the
// search then read global memory).
// Left to one group of eight lanes, a row with thousands of products and a
// global-memory search per product set the time of the whole launch.
constexpr int kBwdG = 8;
constexpr int kBwdStage = 64;
constexpr int kBwdLong = kBwdStage;
constexpr int kBwdLongCap = 2048;     // rows up to this long: columns and gradient in LDS
constexpr int kBwdHugeCap = 14336;    // longer rows: columns only
constexpr int kBwdLongChunk = 256;   // rows a workgroup of the long-row kernel looks through at a time, at most
constexpr int kBwdWide = 64;         // rows of B longer than this are walked by a whole wavefront ...
constexpr int kBwdWideCap = 1024;    // ... up to this many per row of A (the rest stay with their group)

// What lane E of every eight consecutive lanes holds, handed to all eight (ds_swizzle in bit mode:
// lane = (lane & 0x18) | E inside each half of the wavefront; no address to compute).
template <int E> __device__ __forceinline__ int group_lane(int v) {
    static_assert(E >= 0 && E < 8, "a lane of the group");
    return __builtin_amdgcn_ds_swizzle(v, (E << 5) | 0x18);
}
template <int E> __device__ __forceinline__ float group_lane(float v) {
    return __int_as_float(group_lane<E>(__float_as_int(v)));
}
template <int E> __device__ __forceinline__ int64_t group_lane(int64_t v) {
    const int lo = group_lane<E>((int)(v & 0xffffffffll)), hi = group_lane<E>((int)(v >> 32));
    return ((int64_t)hi << 32) | (uint32_t)lo;
}
template <int E> __device__ __forceinline__ double group_lane(double v) {
    return __longlong_as_double(group_lane<E>((int64_t)__double_as_longlong(v)));
}

template <typename T>
__global__ __launch_bounds__(kBlock) void spgemm_bwd_kernel(
    int64_t A_rows, const T *__restrict__ gC, const int64_t *__restrict__ C_indices,
    const int64_t *__restrict__ C_indptr, const T *__restrict__ A_data,
    const int64_t *__restrict__ A_indices, const int64_t *__restrict__ A_indptr,
    const T *__restrict__ B_data, const int64_t *__restrict__ B_indices,
    const int64_t *__restrict__ B_indptr, T *__restrict__ grad_A, T *__restrict__ grad_B) {
    constexpr int G = kBwdG, GPB = kBlock / G;
    static_assert(G == 8 && kBwdStage == 64, "group_lane and the six-step search are written for these");
    // (a group's row starts one bank further on than its neighbour's: the groups of a wavefront
    // probe the same place of their rows at the same step of the search)
    constexpr int kStride = kBwdStage + 1;
    __shared__ int32_t s_ci[GPB * kStride];
    __shared__ T s_g[GPB * kStride];
    const int gl = threadIdx.x % G, gi = G >= kWave ? __builtin_amdgcn_readfirstlane(threadIdx.x / G) : threadIdx.x / G;
    const int gbase = (threadIdx.x & (kWave - 1)) & ~(G - 1);   // first lane of the group inside its wavefront
    int32_t *ci = s_ci + gi * kStride;
    T *cg = s_g + gi * kStride;
    for (int64_t i0 = (int64_t)blockIdx.x * GPB; i0 < A_rows; i0 += (int64_t)gridDim.x * GPB) {
        const int64_t i = i0 + gi;
        const bool live = i < A_rows;
        const int64_t cb = live ? C_indptr[i] : 0, ce = live ? C_indptr[i + 1] : 0;
        const int clen = (int)(ce - cb < 0x7fffffff ? ce - cb : 0x7fffffff);
        const bool here = live && clen <= kBwdStage;   // longer rows are left to spgemm_bwd_long_kernel
        // (places past the row's end hold a column no entry has: the search below takes six steps
        // whatever the row's length and needs no bound)
        if (here)
            for (int t = gl; t < kBwdStage; t += G) {
                ci[t] = t < clen ? (int32_t)C_indices[cb + t] : 0x7fffffff;
                if (t < clen) cg[t] = gC[cb + t];
            }
        group_sync<G>();
        const int64_t ab = here ? A_indptr[i] : 0, ae = here ? A_indptr[i + 1] : 0;
        for (int64_t a0 = ab; a0 < ae; a0 += G) {
            // each lane fetches one entry of A's row and the bounds of the B row it names
            const int64_t my_ai = a0 + gl;
            const bool mine = my_ai < ae;
            const int64_t my_k = mine ? A_indices[my_ai] : 0;
            const T my_a = (mine && grad_B) ? A_data[my_ai] : T(0);
            const int64_t my_bb = mine ? B_indptr[my_k] : 0, my_be = mine ? B_indptr[my_k + 1] : 0;
            const int nb = (int)(ae - a0 < G ? ae - a0 : G);
            const int my_len = (int)(my_be - my_bb);
            T my_acc = 0;
            // (unrolled: the lane whose entry is applied is then a constant of the instruction that
            // hands its row start, length and value to the group, with no address to compute)
            nm::static_for<G>([&](auto ec) {
                constexpr int e = decltype(ec)::value;
                if (e >= nb) return;
                const int64_t bb = group_lane<e>(my_bb), be = bb + group_lane<e>(my_len);
                const T a = grad_B ? group_lane<e>(my_a) : T(0);
                T acc = 0;
                for (int64_t kk0 = bb; kk0 < be; kk0 += G) {
                    const int64_t kk = kk0 + gl;
                    const bool have = kk < be;
                    const int32_t c = have ? (int32_t)B_indices[kk] : -1;
                    const T bval = have && grad_A ? B_data[kk] : T(0);
                    // the number of staged columns below c (at most 63), in six steps without a branch
                    int l = 0;
#pragma unroll
                    for (int step = kBwdStage / 2; step > 0; step >>= 1)
                        if (ci[l + step - 1] < c) l += step;
                    const bool hit = have && ci[l] == c;
                    const T g = hit ? cg[l] : T(0);
                    if (hit && grad_B) nm::atomic_add(grad_B + kk, a * g);
                    if (!grad_A) continue;
                    // Ordered sum over the group's lanes = ascending column: the running sum walks up
                    // the lanes, one DPP shift and one addition a step (every lane adds what its lower
                    // neighbour held a step ago to its own product; lane s is right after step s and
                    // is read at step s + 1, what the others hold meanwhile is never used).  A lane
                    // without a product adds +0.0, which changes no sum that began at +0.0.
                    const T prod = g * bval;   // (g is +0.0 without a hit, bval finite or the lane's own)
                    T run = acc + (hit ? prod : T(0));
#pragma unroll
                    for (int step = 1; step < G; ++step) run = nm::dpp_move<0x111>(run) + (hit ? prod : T(0));
                    acc = group_lane<G - 1>(run);
                }
                if (gl == e) my_acc = acc;
            });
            if (mine && grad_A) grad_A[my_ai] = my_acc;
        }
        group_sync<G>();
    }
}

template <typename T, int CAP, bool STAGE_G>
__global__ __launch_bounds__(kBlock) void spgemm_bwd_long_kernel(
    int64_t A_rows, int chunk, int64_t longer_than, int64_t up_to, const T *__restrict__ gC, const int64_t *__restrict__ C_indices,
    const int64_t *__restrict__ C_indptr, const T *__restrict__ A_data,
    const int64_t *__restrict__ A_indices, const int64_t *__restrict__ A_indptr,
    const T *__restrict__ B_data, const int64_t *__restrict__ B_indices,
    const int64_t *__restrict__ B_indptr, T *__restrict__ grad_A, T *__restrict__ grad_B) {
    constexpr int G = kBwdG, GROUPS = kBlock / G;
    __shared__ T cg[STAGE_G ? CAP : 1];
    __shared__ int32_t ci[CAP];
    __shared__ int s_long[kBwdLongChunk];
    __shared__ int s_wide[kBwdWideCap];
    __shared__ int s_n, s_nw;
    const int gl = threadIdx.x % G, gi = threadIdx.x / G;
    const int gbase = (threadIdx.x & (kWave - 1)) & ~(G - 1);
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    for (int64_t r0 = (int64_t)blockIdx.x * chunk; r0 < A_rows; r0 += (int64_t)gridDim.x * chunk) {
        // the long rows among this chunk of rows (mostly there are none)
        const int64_t r = r0 + threadIdx.x;
        bool is_long = false;
        if ((int)threadIdx.x < chunk && r < A_rows) {
            const int64_t len = C_indptr[r + 1] - C_indptr[r];
            is_long = len > longer_than && len <= up_to;
        }
        if (!__syncthreads_or(is_long)) continue;
        if (threadIdx.x == 0) s_n = 0;
        __syncthreads();
        if (is_long) s_long[atomicAdd(&s_n, 1)] = threadIdx.x;
        __syncthreads();
        const int n = s_n;
        for (int q = 0; q < n; ++q) {
            const int64_t i = r0 + s_long[q];
            const int64_t cb = C_indptr[i], ce = C_indptr[i + 1], clen = ce - cb;
            const int64_t stride = (clen + CAP - 1) / CAP;
            const int ns = (int)((clen + stride - 1) / stride);
            const bool whole = stride == 1;
            for (int t = threadIdx.x; t < ns; t += kBlock) {
                ci[t] = (int32_t)C_indices[cb + t * stride];
                if (STAGE_G) cg[t] = gC[cb + t];   // STAGE_G kernels only get rows of at most CAP entries
            }
            if (threadIdx.x == 0) s_nw = 0;
            __syncthreads();
            // One entry (i,k) of A: W lanes (lane wl of them, the first being lane wbase of the
            // wavefront) walk row k of B; returns sum_c gC[i,c] * B[k,c] added in ascending c.
            auto entry = [&](auto width, int wl, int wbase, int64_t bb, int64_t be, T a) -> T {
                constexpr int W = decltype(width)::value;
                T acc = 0;
                for (int64_t kk0 = bb; kk0 < be; kk0 += W) {
                    const int64_t kk = kk0 + wl;
                    const bool have = kk < be;
                    const int64_t c = have ? B_indices[kk] : -1;
                    const T bval = have ? B_data[kk] : T(0);
                    int l = 0, h = ns;
                    while (l < h) {
                        const int mid = (l + h) >> 1;
                        if ((int64_t)ci[mid] < c) l = mid + 1; else h = mid;
                    }
                    bool hit;
                    T g = 0;
                    if (whole) {
                        hit = have && l < ns && (int64_t)ci[l] == c;
                        if (hit) g = STAGE_G ? cg[l] : gC[cb + l];
                    } else {
                        // sample l is the first one not below c: the column, if present, sits
                        // after sample l - 1 and no later than sample l
                        int64_t lo = l == 0 ? 0 : (int64_t)(l - 1) * stride + 1;
                        int64_t hi = (int64_t)l * stride < clen ? (int64_t)l * stride : clen;
                        if (!have) hi = lo;
                        while (lo < hi) {
                            const int64_t mid = (lo + hi) >> 1;
                            if (C_indices[cb + mid] < c) lo = mid + 1; else hi = mid;
                        }
                        hit = have && lo < clen && C_indices[cb + lo] == c;
                        if (hit) g = gC[cb + lo];
                    }
                    if (hit && grad_B) nm::atomic_add(grad_B + kk, a * g);
                    const T prod = hit ? g * bval : T(0);
                    // ordered sum over the lanes = ascending column
                    const int cnt = (int)(be - kk0 < W ? be - kk0 : W);
                    for (int l2 = 0; l2 < cnt; ++l2) {
                        const T pl = __shfl(prod, wbase + l2, kWave);
                        const int hl = __shfl((int)hit, wbase + l2, kWave);
                        if (hl) acc += pl;
                    }
                }
                return acc;
            };
            const int64_t ab = A_indptr[i], ae = A_indptr[i + 1];
            // entries of A's row per group and pass: as few as keeps all groups busy
            const int64_t even = (ae - ab + GROUPS - 1) / GROUPS;
            const int per = (int)(even < 1 ? 1 : (even > G ? G : even));
            for (int64_t a0 = ab + gi * per; a0 < ae; a0 += GROUPS * per) {
                const int64_t my_ai = a0 + gl;
                const bool mine = gl < per && my_ai < ae;
                const int64_t my_k = mine ? A_indices[my_ai] : 0;
                const T my_a = (mine && grad_B) ? A_data[my_ai] : T(0);
                const int64_t my_bb = mine ? B_indptr[my_k] : 0, my_be = mine ? B_indptr[my_k + 1] : 0;
                // entries whose row of B is long are set aside for a whole wavefront
                bool later = false;
                if (mine && my_be - my_bb > kBwdWide) {
                    const int slot = atomicAdd(&s_nw, 1);
                    later = slot < kBwdWideCap;
                    if (later) s_wide[slot] = (int)(my_ai - ab);
                }
                const int nb = (int)(ae - a0 < per ? ae - a0 : per);
                T my_acc = 0;
                for (int e = 0; e < nb; ++e) {
                    if (__shfl((int)later, gbase + e, kWave)) continue;
                    const int64_t bb = __shfl(my_bb, gbase + e, kWave), be = __shfl(my_be, gbase + e, kWave);
                    const T a = __shfl(my_a, gbase + e, kWave);
                    const T acc = entry(std::integral_constant<int, G>{}, gl, gbase, bb, be, a);
                    if (gl == e) my_acc = acc;
                }
                if (mine && !later && grad_A) grad_A[my_ai] = my_acc;
            }
            __syncthreads();
            const int nw = s_nw < kBwdWideCap ? s_nw : kBwdWideCap;
            for (int d = wave; d < nw; d += kBlock / kWave) {
                const int64_t ai = ab + s_wide[d];
                const int64_t k = A_indices[ai];
                const T a = grad_B ? A_data[ai] : T(0);
                const T acc = entry(std::integral_constant<int, kWave>{}, lane, 0, B_indptr[k], B_indptr[k + 1], a);
                if (lane == 0 && grad_A) grad_A[ai] = acc;
            }
            __syncthreads();
        }
    }
}

int check_common(int64_t A_rows, int64_t B_cols) {
    NM_REQUIRE(A_rows >= 0 && B_cols >= 0, "negative size");
    if (A_rows >= 0x7ffffffe || B_cols >= 0x7ffffffe)
        return nm::fail(NM_ERR_UNSUPPORTED, "spgemm indexes rows and columns with 32 bits inside its tables");
    return NM_OK;
}

constexpr unsigned kPersistGrid = 4096;

template <typename T>
int launch_numeric(const Work &w, int64_t B_cols, const void *A_data, const int64_t *A_indices,
                   const int64_t *A_indptr, const void *B_data, const int64_t *B_indices,
                   const int64_t *B_indptr, const int64_t *C_indptr, int64_t *C_indices, void *C_data,
                   hipStream_t s) {
    const T *Ad = (const T *)A_data, *Bd = (const T *)B_data;
    T *Cd = (T *)C_data;
    constexpr size_t per = sizeof(T) + sizeof(int32_t);
    auto hashed = [&](auto group, auto table, int bin, unsigned grid) -> int {
        constexpr int G = decltype(group)::value, TABLE = decltype(table)::value;
        auto k = numeric_hash_kernel<T, G, TABLE>;
        // tables (values + keys), padded apart when groups share a workgroup, and the two compaction lists
        // (narrow groups keep the lists where the key table was)
        const size_t lds = (kBlock / G) * (per * (TABLE + (G < kBlock ? kTablePad : 0)) + (G > kWave ? 4 * (TABLE + 8) : 0));
        if (lds > 64 * 1024)
            NM_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(k),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(k, dim3(grid), dim3(kBlock), lds, s, bin, w.bins, w.perm, Ad, A_indices, A_indptr, Bd,
                           B_indices, B_indptr, C_indptr, C_indices, Cd);
        NM_LAUNCH_CHECK("numeric_hash_kernel");
        return NM_OK;
    };
    using std::integral_constant;
    if (int rc = hashed(integral_constant<int, kGroup0>{}, integral_constant<int, kNumTable0>{}, 0, kPersistGrid)) return rc;
    if (int rc = hashed(integral_constant<int, kGroup1>{}, integral_constant<int, kNumTable1>{}, 1, kPersistGrid)) return rc;
    if (int rc = hashed(integral_constant<int, kGroup2>{}, integral_constant<int, kNumTable2>{}, 2, kPersistGrid)) return rc;
    if (int rc = hashed(integral_constant<int, kGroup3>{}, integral_constant<int, kNumTable3>{}, 3, kPersistGrid)) return rc;
    if (int rc = hashed(integral_constant<int, kGroup4>{}, integral_constant<int, kNumTable4>{}, 4, kPersistGrid)) return rc;
    if (int rc = hashed(integral_constant<int, kGroup5>{}, integral_constant<int, kNumTable5>{}, 5, kPersistGrid)) return rc;
    if (int rc = hashed(integral_constant<int, kGroup6>{}, integral_constant<int, kNumTable6>{}, 6, 1024)) return rc;
    hipLaunchKernelGGL(numeric_spill_kernel<T>, dim3(spill_groups(B_cols)), dim3(kSpillBlock), 0, s, w.bins, w.perm,
                       B_cols, Ad, A_indices, A_indptr, Bd, B_indices, B_indptr, C_indptr, C_indices, Cd, w.mark,
                       w.acc);
    NM_LAUNCH_CHECK("numeric_spill_kernel");
    return NM_OK;
}

}  // namespace

extern "C" int nm_spgemm_workspace_bytes(int64_t A_rows, int64_t B_cols, size_t *bytes) {
    NM_REQUIRE(bytes != nullptr, "bytes is null");
    if (int rc = check_common(A_rows, B_cols)) return rc;
    *bytes = work_layout(A_rows, B_cols, nullptr, nullptr);
    return NM_OK;
}

namespace {

// The symbolic phase; with `map` its first kernel also records where every product of a
// merge-path row goes (the destination bytes and B row starts of a product plan).
int symbolic_phase(int64_t A_rows, int64_t A_cols, int64_t B_cols, const int64_t *A_indices,
                   const int64_t *A_indptr, const int64_t *B_indices, const int64_t *B_indptr, int64_t *C_indptr,
                   void *workspace, size_t workspace_bytes, void *host_landing, const nm::PPlan *map,
                   nm_stream stream) {
    if (int rc = check_common(A_rows, B_cols)) return rc;
    NM_REQUIRE(A_cols >= 0, "negative size");
    NM_REQUIRE(A_indptr && B_indptr && C_indptr && workspace, "null pointer argument");
    Work w;
    const size_t need = work_layout(A_rows, B_cols, workspace, &w);
    if (workspace_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace_bytes, need);
    hipStream_t s = nm::as_stream(stream);
    if (A_rows == 0) return nm::fill_async(C_indptr, 1, (int64_t)0, s);

    const int64_t tiles = nm::ceil_div(A_rows + 1, nm::kScanTile);
    if (tiles > nm::kMaxGrid) return nm::fail(NM_ERR_UNSUPPORTED, "%lld rows are too many", (long long)A_rows);
    // What the first kernel writes over summary[1] where it leaves a row to the hash path: not a
    // count of rows (the word's content at the end of every call) and not an earlier call's token.
    volatile int64_t *both = (volatile int64_t *)host_landing;
    const int64_t ticket = both ? both[2] + 1 : 1;
    const int64_t token = ticket | ((int64_t)1 << 62);
    const int64_t nbatch = nm::xcd_padded(nm::ceil_div(A_rows, kMergeRows));
    hipLaunchKernelGGL(symbolic_front_kernel, dim3((unsigned)nbatch), dim3(kBlock), 0, s, A_rows, nbatch,
                       A_indices, A_indptr, B_indices, B_indptr, w.key, w.count,
                       reinterpret_cast<unsigned long long *>(w.summary + 1), (unsigned long long)token,
                       map ? reinterpret_cast<uint64_t *>(map->dest) : (uint64_t *)nullptr,
                       map ? map->bstart : (int32_t *)nullptr);
    NM_LAUNCH_CHECK("symbolic_front_kernel");
    // The row pointer from the counts: their sums by tile, then the pass that writes it.
    auto row_pointer = [&](const int32_t *bins, volatile int64_t *landing) -> int {
        hipLaunchKernelGGL(count_tile_sums_kernel, dim3((unsigned)tiles), dim3(nm::kScanBlock), 0, s, w.count,
                           A_rows + 1, w.scan);
        NM_LAUNCH_CHECK("count_tile_sums_kernel");
        const bool scanned = tiles > kInlineTiles;
        if (scanned) {
            hipLaunchKernelGGL(nm::scan_sums_kernel, dim3(1), dim3(1024), 0, s, w.scan, tiles);
            NM_LAUNCH_CHECK("scan_sums_kernel");
        }
        hipLaunchKernelGGL(row_pointer_kernel, dim3((unsigned)tiles), dim3(nm::kScanBlock), 0, s, w.count, A_rows + 1,
                           w.scan, scanned ? 1 : 0, C_indptr, bins, w.summary, token, landing, ticket);
        NM_LAUNCH_CHECK("row_pointer_kernel");
        return NM_OK;
    };
    // With a landing place in pinned host memory the row pointer is made at once, as if the first
    // kernel had taken every row (it has, for a product of stencil or aggregation matrices), and its
    // first workgroup tells the host nnz(C) and whether a row was left to the hash path.  If none was,
    // that was the symbolic phase: the binning and the nine launches of the hash path, which would
    // find nothing to do, are left out, and nm_spgemm_symbolic_result finds its answer landed (the
    // workspace's address in the landing place's fourth word says so).  Otherwise the pass was for
    // nothing (30 us against the milliseconds of a hash path) and is made again below.
    if (both) {
        both[3] = 0;
        if (int rc = row_pointer(nullptr, both)) return rc;
        bool arrived = false;
        for (int spin = 0; spin < (1 << 22) && !arrived; ++spin) arrived = both[2] == ticket;
        if (!arrived) {
            NM_HIP_TRY(hipStreamSynchronize(s));
            NM_REQUIRE(both[2] == ticket, "the count of hash-path rows did not arrive");
        }
        if (both[1] == 0) {
            both[3] = (int64_t)reinterpret_cast<intptr_t>(workspace);
            return NM_OK;
        }
    }
    {
    if (int rc = bin_rows(A_rows, kSymLimit, w, s)) return rc;

    hipLaunchKernelGGL((symbolic_hash_kernel<kGroup0, kSymTable0>), dim3(kPersistGrid), dim3(kBlock), 0, s, 0, w.bins,
                       w.perm, A_indices, A_indptr, B_indices, B_indptr, w.count);
    hipLaunchKernelGGL((symbolic_hash_kernel<kGroup1, kSymTable1>), dim3(kPersistGrid), dim3(kBlock), 0, s, 1, w.bins,
                       w.perm, A_indices, A_indptr, B_indices, B_indptr, w.count);
    hipLaunchKernelGGL((symbolic_hash_kernel<kGroup2, kSymTable2>), dim3(kPersistGrid), dim3(kBlock), 0, s, 2, w.bins,
                       w.perm, A_indices, A_indptr, B_indices, B_indptr, w.count);
    hipLaunchKernelGGL((symbolic_hash_kernel<kGroup3, kSymTable3>), dim3(kPersistGrid), dim3(kBlock), 0, s, 3, w.bins,
                       w.perm, A_indices, A_indptr, B_indices, B_indptr, w.count);
    hipLaunchKernelGGL((symbolic_hash_kernel<kGroup4, kSymTable4>), dim3(kPersistGrid), dim3(kBlock), 0, s, 4, w.bins,
                       w.perm, A_indices, A_indptr, B_indices, B_indptr, w.count);
    hipLaunchKernelGGL((symbolic_hash_kernel<kGroup5, kSymTable5>), dim3(kPersistGrid), dim3(kBlock), 0, s, 5, w.bins,
                       w.perm, A_indices, A_indptr, B_indices, B_indptr, w.count);
    hipLaunchKernelGGL((symbolic_hash_kernel<kGroup6, kSymTable6>), dim3(1024), dim3(kBlock), 0, s, 6, w.bins, w.perm,
                       A_indices, A_indptr, B_indices, B_indptr, w.count);
    NM_LAUNCH_CHECK("symbolic_hash_kernel");
    hipLaunchKernelGGL(symbolic_spill_kernel, dim3(spill_groups(B_cols)), dim3(kSpillBlock), 0, s, w.bins, w.perm, B_cols,
                       A_indices, A_indptr, B_indices, B_indptr, w.mark, w.count);
    NM_LAUNCH_CHECK("symbolic_spill_kernel");
    }
    return row_pointer(w.bins, nullptr);
}

}  // namespace

extern "C" int nm_spgemm_symbolic(int64_t A_rows, int64_t A_cols, int64_t B_cols, const int64_t *A_indices,
                                  const int64_t *A_indptr, const int64_t *B_indices, const int64_t *B_indptr,
                                  int64_t *C_indptr, void *workspace, size_t workspace_bytes,
                                  void *host_landing, nm_stream stream) {
    return symbolic_phase(A_rows, A_cols, B_cols, A_indices, A_indptr, B_indices, B_indptr, C_indptr, workspace,
                          workspace_bytes, host_landing, nullptr, stream);
}

extern "C" int nm_spgemm_symbolic_mapped(int64_t A_rows, int64_t A_cols, int64_t B_cols, int64_t A_nnz,
                                         int64_t B_nnz, const int64_t *A_indices, const int64_t *A_indptr,
                                         const int64_t *B_indices, const int64_t *B_indptr, int64_t *C_indptr,
                                         void *workspace, size_t workspace_bytes, void *plan_mem,
                                         size_t plan_bytes, void *host_landing, nm_stream stream) {
    NM_REQUIRE(A_nnz >= 0 && B_nnz >= 0 && plan_mem, "bad arguments");
    NM_REQUIRE(A_nnz < ((int64_t)1 << 31) && B_nnz < ((int64_t)1 << 31), "the plan keeps positions in 31 bits");
    const size_t need = nm::pplan_layout(A_nnz, nullptr, nullptr);
    if (plan_bytes < need) return nm::fail(NM_ERR_WORKSPACE, "plan of %zu bytes, %zu needed", plan_bytes, need);
    nm::PPlan map;
    nm::pplan_layout(A_nnz, plan_mem, &map);
    return symbolic_phase(A_rows, A_cols, B_cols, A_indices, A_indptr, B_indices, B_indptr, C_indptr, workspace,
                          workspace_bytes, host_landing, &map, stream);
}

extern "C" int nm_spgemm_symbolic_result(int64_t A_rows, int64_t B_cols, const void *workspace,
                                         size_t workspace_bytes, int64_t *nnz_C, int64_t *hash_rows,
                                         void *host_landing, nm_stream stream) {
    if (int rc = check_common(A_rows, B_cols)) return rc;
    NM_REQUIRE(workspace && nnz_C && hash_rows, "null pointer argument");
    Work w;
    const size_t need = work_layout(A_rows, B_cols, const_cast<void *>(workspace), &w);
    if (workspace_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace_bytes, need);
    *nnz_C = 0;
    *hash_rows = 0;
    if (A_rows == 0) return NM_OK;
    hipStream_t s = nm::as_stream(stream);
    if (!host_landing) {
        // no landing place from the caller: an ordinary copy and a wait for the stream
        int64_t both[2] = {0, 0};
        NM_HIP_TRY(hipMemcpyAsync(both, w.summary, sizeof(both), hipMemcpyDeviceToHost, s));
        NM_HIP_TRY(hipStreamSynchronize(s));
        *nnz_C = both[0];
        *hash_rows = both[1];
        return NM_OK;
    }
    // The two numbers are written straight into the caller's pinned host memory by a one-lane
    // kernel, followed by a ticket the host polls for: waking up from hipStreamSynchronize, or a
    // copy-engine transfer of 16 bytes, takes ~30 us, several times what the kernels of a small
    // product take together.  The ticket is one more than the last one this landing place saw.
    volatile int64_t *both = (volatile int64_t *)host_landing;
    if (both[3] != 0 && both[3] == (int64_t)reinterpret_cast<intptr_t>(workspace)) {
        // nm_spgemm_symbolic on this workspace has had the numbers dropped here already
        both[3] = 0;
        *nnz_C = both[0];
        *hash_rows = both[1];
        return NM_OK;
    }
    const int64_t ticket = both[2] + 1;
    hipLaunchKernelGGL(summary_out_kernel, dim3(1), dim3(64), 0, s, w.summary, both, ticket);
    NM_LAUNCH_CHECK("summary_out_kernel");
    bool arrived = false;
    for (int spin = 0; spin < (1 << 22) && !arrived; ++spin) arrived = both[2] == ticket;
    if (!arrived) {   // a long queue ahead of the kernel, or memory the host sees late: wait the ordinary way
        NM_HIP_TRY(hipStreamSynchronize(s));
        NM_REQUIRE(both[2] == ticket, "the symbolic phase's result did not arrive");
    }
    *nnz_C = both[0];
    *hash_rows = both[1];
    return NM_OK;
}

extern "C" int nm_spgemm_numeric(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t B_cols,
                                 const void *A_data, const int64_t *A_indices, const int64_t *A_indptr,
                                 const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                                 const int64_t *C_indptr, int64_t *C_indices, void *C_data, void *workspace,
                                 size_t workspace_bytes, int64_t hash_rows, nm_stream stream) {
    if (int rc = check_common(A_rows, B_cols)) return rc;
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(A_indptr && B_indptr && C_indptr && workspace, "null pointer argument");
    Work w;
    const size_t need = work_layout(A_rows, B_cols, workspace, &w);
    if (workspace_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace_bytes, need);
    if (A_rows == 0) return NM_OK;
    hipStream_t s = nm::as_stream(stream);
    int64_t grid = nm::ceil_div(A_rows, kBlock);
    if (grid > 65536) grid = 65536;
    // hash_rows == 0 (from nm_spgemm_symbolic_result): every row is one of the merge path's and
    // the binning and the hash launches, a dozen launches that would find nothing to do, are left out
    const bool hashed = hash_rows != 0;
    if (hashed) {
        hipLaunchKernelGGL(row_length_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows, C_indptr, w.key);
        NM_LAUNCH_CHECK("row_length_kernel");
        if (int rc = bin_rows(A_rows, kNumLimit, w, s)) return rc;
    }
    const int64_t nbatch = nm::xcd_padded(nm::ceil_div(A_rows, kMergeRows));
    // (every row on the hash path: the merge kernel would look at each row's key and leave)
    if (hash_rows == A_rows) {
    } else if (dt == NM_F32)
        hipLaunchKernelGGL(numeric_front_kernel<float>, dim3((unsigned)nbatch), dim3(kBlock), 0, s, A_rows, nbatch,
                           w.key, (const float *)A_data, A_indices, A_indptr, (const float *)B_data, B_indices,
                           B_indptr, C_indptr, C_indices, (float *)C_data);
    else
        hipLaunchKernelGGL(numeric_front_kernel<double>, dim3((unsigned)nbatch), dim3(kBlock), 0, s, A_rows, nbatch,
                           w.key, (const double *)A_data, A_indices, A_indptr, (const double *)B_data, B_indices,
                           B_indptr, C_indptr, C_indices, (double *)C_data);
    NM_LAUNCH_CHECK("numeric_front_kernel");
    if (!hashed) return NM_OK;
    if (dt == NM_F32)
        return launch_numeric<float>(w, B_cols, A_data, A_indices, A_indptr, B_data, B_indices, B_indptr,
                                     C_indptr, C_indices, C_data, s);
    return launch_numeric<double>(w, B_cols, A_data, A_indices, A_indptr, B_data, B_indices, B_indptr, C_indptr,
                                  C_indices, C_data, s);
}

extern "C" int nm_spgemm_numeric_mapped(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t B_cols, int64_t A_nnz,
                                        int64_t C_nnz, const void *A_data, const int64_t *A_indices,
                                        const int64_t *A_indptr, const void *B_data, const int64_t *B_indices,
                                        const int64_t *B_indptr, const int64_t *C_indptr, int64_t *C_indices,
                                        void *C_data, void *workspace, size_t workspace_bytes, int64_t hash_rows,
                                        void *plan_mem, size_t plan_bytes, int keep_plan, nm_stream stream) {
    // rows on the hash path (or an unknown number of them), or positions beyond 31 bits: the map
    // the symbolic phase left is incomplete or unusable, the ordinary numeric phase runs
    if (hash_rows != 0 || !plan_mem || A_nnz <= 0 || C_nnz <= 0 || C_nnz >= ((int64_t)1 << 31))
        return nm_spgemm_numeric(dt, A_rows, A_cols, B_cols, A_data, A_indices, A_indptr, B_data, B_indices, B_indptr,
                                 C_indptr, C_indices, C_data, workspace, workspace_bytes, hash_rows, stream);
    if (int rc = check_common(A_rows, B_cols)) return rc;
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(A_data && A_indptr && B_data && B_indices && C_indptr && C_indices && C_data, "null pointer argument");
    const size_t need = nm::pplan_layout(A_nnz, nullptr, nullptr);
    if (plan_bytes < need) return nm::fail(NM_ERR_WORKSPACE, "plan of %zu bytes, %zu needed", plan_bytes, need);
    nm::PPlan map;
    nm::pplan_layout(A_nnz, plan_mem, &map);
    return nm::spgemm_numeric_on_map(dt, A_rows, A_nnz, A_data, A_indptr, B_data, B_indices, map, C_indptr, C_indices,
                                     C_data, keep_plan != 0, nm::as_stream(stream));
}

extern "C" int nm_spgemm_backward(nm_dtype dt, int64_t A_rows, int64_t A_nnz, int64_t B_nnz, const void *gC,
                                  const int64_t *C_indices, const int64_t *C_indptr, const void *A_data,
                                  const int64_t *A_indices, const int64_t *A_indptr, const void *B_data,
                                  const int64_t *B_indices, const int64_t *B_indptr, void *grad_A,
                                  void *grad_B, nm_stream stream) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(A_rows >= 0 && A_nnz >= 0 && B_nnz >= 0, "negative size");
    hipStream_t s = nm::as_stream(stream);
    if (grad_B) {
        int rc = dt == NM_F32 ? nm::fill_async((float *)grad_B, B_nnz, 0.0f, s)
                              : nm::fill_async((double *)grad_B, B_nnz, 0.0, s);
        if (rc) return rc;
    }
    if (A_nnz == 0 || A_rows == 0 || (!grad_A && !grad_B)) return NM_OK;
    NM_REQUIRE(C_indptr && A_indices && A_indptr && B_indptr && A_data, "null pointer argument");
    int64_t grid = nm::ceil_div(A_rows, kBlock / kBwdG);
    if (grid > 1 << 20) grid = 1 << 20;
    if (dt == NM_F32)
        hipLaunchKernelGGL(spgemm_bwd_kernel<float>, dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows,
                           (const float *)gC, C_indices, C_indptr, (const float *)A_data, A_indices, A_indptr,
                           (const float *)B_data, B_indices, B_indptr, (float *)grad_A, (float *)grad_B);
    else
        hipLaunchKernelGGL(spgemm_bwd_kernel<double>, dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows,
                           (const double *)gC, C_indices, C_indptr, (const double *)A_data, A_indices, A_indptr,
                           (const double *)B_data, B_indices, B_indptr, (double *)grad_A, (double *)grad_B);
    NM_LAUNCH_CHECK("spgemm_bwd_kernel");
    // A workgroup works off the long rows of its chunk one after the other, so a chunk is sized
    // for at least ~4096 of them over the matrix (8 rows or more; 256 at the sizes where the pass
    // over the row lengths is itself worth keeping short).
    int chunk = kBwdLongChunk;
    while (chunk > 8 && A_rows / chunk < 4096) chunk /= 2;
    grid = nm::ceil_div(A_rows, chunk);
    if (grid > 4096) grid = 4096;
    const int64_t none = INT64_MAX;
#define NM_BWD_LONG(T)                                                                                          \
    do {                                                                                                        \
        hipLaunchKernelGGL((spgemm_bwd_long_kernel<T, kBwdLongCap, true>), dim3((unsigned)grid), dim3(kBlock),  \
                           0, s, A_rows, chunk, (int64_t)kBwdLong, (int64_t)kBwdLongCap, (const T *)gC, C_indices,\
                           C_indptr, (const T *)A_data, A_indices, A_indptr, (const T *)B_data, B_indices,      \
                           B_indptr, (T *)grad_A, (T *)grad_B);                                                 \
        hipLaunchKernelGGL((spgemm_bwd_long_kernel<T, kBwdHugeCap, false>), dim3((unsigned)grid), dim3(kBlock), \
                           0, s, A_rows, chunk, (int64_t)kBwdLongCap, none, (const T *)gC, C_indices, C_indptr, \
                           (const T *)A_data, A_indices, A_indptr, (const T *)B_data, B_indices, B_indptr,      \
                           (T *)grad_A, (T *)grad_B);                                                           \
    } while (0)
    if (dt == NM_F32) NM_BWD_LONG(float);
    else NM_BWD_LONG(double);
#undef NM_BWD_LONG
    NM_LAUNCH_CHECK("spgemm_bwd_long_kernel");
    return NM_OK;
}
