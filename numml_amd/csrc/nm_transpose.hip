// Builder of the transposed-structure plan (see nm_transpose.hpp) and its C ABI.
//
// A counting sort by column that keeps A's storage order inside every column,
// which is what the reference's transpose does serially
// (cpp/sparse_csr_cpu.cpp:334-361), in five device-driven steps and without a
// general-purpose sort:
//
//   1. count    row tiles stream A's entries once: one atomic add per entry into
//               a per-column counter, and the by-products every later kernel
//               wants in 32 bits (row of each entry, column of each entry, row
//               pointers, the row of every 64th entry);
//   2. scan     exclusive prefix sum of the counters = column pointers;
//   3. scatter  every entry draws a slot in its column from a per-column cursor
//               (atomic add with return) and leaves its own position there.  The
//               slots of a column are now filled, but in the order the hardware
//               happened to serve the atomics;
//   4. order    column tiles put each column's positions into ascending order.
//               A position in A's row-major arrays grows with the row (and, for
//               duplicate coordinates, with the storage order), so ascending
//               positions ARE the stable order.  A column is ranked by counting
//               in LDS (entry j goes to slot #{keys < key j}); a column too long
//               for LDS is ranked piece by piece and the sorted pieces are merged
//               pairwise by the workgroup through a scratch copy;
//   5. flags    symmetric-pattern check against A itself.
//
// Nothing here depends on a host read, so the build is fully asynchronous.
#include "nm_transpose.hpp"

#include "nm_scan.hpp"

namespace {

using nm::kWave;

constexpr int kBlock = 256;
constexpr int kRows = 512;      // rows (columns) a workgroup stages offsets for
constexpr int kCap = 4096;      // LDS keys of the ordering kernel
constexpr int kSlice = 8;       // consecutive outputs one lane produces in a merge pass
constexpr int kSortMin = 128;   // keys from which a column is sorted by a network instead of ranked key by key

struct WorkT {
    int64_t *count;        // [cols + 1] per-column counters, then column pointers
    int64_t *scan;         // scratch of the prefix sum
    int32_t *cursor;       // [cols + 1] next free slot of every column
    int32_t *rowid;        // [nnz] row of every entry (row-major order)
    int32_t *tmp;          // [nnz] second copy of a long column during its merge passes
};

size_t work_layout(int64_t cols, int64_t nnz, void *base, WorkT *w) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += nm::align256(bytes);
        return q;
    };
    WorkT t;
    t.count = (int64_t *)take((size_t)(cols + 2) * 8);
    t.scan = (int64_t *)take(nm::scan_scratch_bytes(cols + 1));
    t.cursor = (int32_t *)take((size_t)(cols + 2) * 4);
    t.rowid = (int32_t *)take((size_t)(nnz + 1) * 4);
    t.tmp = (int32_t *)take((size_t)(nnz + 1) * 4);
    if (w) *w = t;
    return off;
}

// Rows a workgroup takes at a time: kRows where rows are short, fewer where they are long,
// so that a tile holds a few thousand entries and the grid stays wide.
inline int tile_rows(int64_t rows, int64_t nnz, int least = 8) {
    const int64_t mean = rows > 0 ? (nnz + rows - 1) / rows : 1;
    const int64_t r = kCap / (mean > 0 ? mean : 1);
    return (int)(r > kRows ? kRows : (r < least ? least : r));
}

// Step 1.  A workgroup owns `rt` consecutive rows; lane = entry.  The row of an entry is found
// by bisection over the tile's offsets in LDS, so rows of any length cost the same.
__global__ __launch_bounds__(kBlock) void tp_count_kernel(
    int64_t rows, int rt, const int64_t *__restrict__ indices, const int64_t *__restrict__ indptr,
    unsigned long long *__restrict__ count, int32_t *__restrict__ rowid, int32_t *__restrict__ col32,
    int32_t *__restrict__ ptr32, int32_t *__restrict__ chunk_row) {
    __shared__ int32_t s_off[kRows + 1];
    const int64_t ntiles = (rows + rt - 1) / rt, npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t r0 = tile * rt;
        const int nr = (int)(rows - r0 < rt ? rows - r0 : rt);
        const int64_t base = indptr[r0];
        for (int t = threadIdx.x; t <= nr; t += kBlock) {
            const int64_t p = indptr[r0 + t];
            s_off[t] = (int32_t)(p - base);        // nnz < 2^31 for plans
            ptr32[r0 + t] = (int32_t)p;
        }
        __syncthreads();
        const int n = s_off[nr];
        for (int j = threadIdx.x; j < n; j += kBlock) {
            int lo = 0, hi = nr;                   // last t with s_off[t] <= j
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (s_off[mid] <= j) lo = mid; else hi = mid;
            }
            const int64_t k = base + j;
            const int64_t c = nm::stream_load(indices + k);
            atomicAdd(count + c, 1ull);
            const int32_t r = (int32_t)(r0 + lo);
            rowid[k] = r;
            col32[k] = (int32_t)c;
            if ((k & 63) == 0) chunk_row[k >> 6] = r;
        }
        __syncthreads();
    }
}

// Column pointers and the scatter cursors from the scanned counters.
__global__ void tp_pointers_kernel(int64_t cols, const int64_t *__restrict__ count,
                                   int32_t *__restrict__ t_indptr, int32_t *__restrict__ cursor) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; c <= cols; c += stride) {
        const int32_t p = (int32_t)count[c];
        t_indptr[c] = p;
        cursor[c] = p;
    }
}

// Step 3.
__global__ void tp_scatter_kernel(int64_t nnz, const int32_t *__restrict__ col32, int32_t *__restrict__ cursor,
                                  int32_t *__restrict__ t_perm) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nnz; k += stride) {
        const int32_t pos = atomicAdd(cursor + col32[k], 1);
        t_perm[pos] = (int32_t)k;
    }
}

// End of the run of columns that starts at column s0 of the tile and fits the LDS keys.
__device__ __forceinline__ int run_end(const int32_t *s_off, int s0, int nc, int cap) {
    const int32_t limit = s_off[s0] + cap;
    if (s_off[nc] <= limit) return nc;
    int lo = s0, hi = nc;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_off[mid] <= limit) lo = mid; else hi = mid;
    }
    return lo;
}

// One merge pass of the workgroup over a long column: sorted runs of `width` keys in `src`
// become sorted runs of 2 * width keys in `dst`.  Every lane produces kSlice consecutive
// outputs of one pair of runs: it finds where they start in the two runs by bisection along
// the diagonal (keys are distinct), fetches the kSlice keys of either run the slice can take
// at most -- independent loads -- into its own column of `s_a` / `s_b` (kSlice * kBlock keys each)
// and merges from there: a merge step waits for LDS, not for memory.
constexpr int32_t kPastAll = 0x7fffffff;   // larger than every position
__device__ void merge_pass(const int32_t *__restrict__ src, int32_t *__restrict__ dst, int len, int width,
                           int32_t *s_a, int32_t *s_b) {
    const int nslices = (len + kSlice - 1) / kSlice;
    for (int sl = threadIdx.x; sl < nslices; sl += kBlock) {
        const int o0 = sl * kSlice;                         // first output of the slice
        const int pair0 = o0 / (2 * width) * (2 * width);   // start of its pair of runs
        const int na = min(width, len - pair0), nb = max(0, min(width, len - pair0 - width));
        const int32_t *a = src + pair0, *b = src + pair0 + na;
        const int d = o0 - pair0;                           // outputs of this pair before the slice
        int lo = max(0, d - nb), hi = min(d, na);           // i = keys taken from a, d - i from b
        while (lo < hi) {
            const int i = (lo + hi) >> 1;
            if (a[i] < b[d - i - 1]) lo = i + 1; else hi = i;
        }
        const int i0 = lo, j0 = d - lo;
        const int end = min(kSlice, pair0 + na + nb - o0);
#pragma unroll
        for (int u = 0; u < kSlice; ++u) {
            s_a[u * kBlock + threadIdx.x] = i0 + u < na ? a[i0 + u] : kPastAll;
            s_b[u * kBlock + threadIdx.x] = j0 + u < nb ? b[j0 + u] : kPastAll;
        }
        int i = 0, j = 0;
        for (int u = 0; u < end; ++u) {
            const int32_t ka = s_a[i * kBlock + threadIdx.x], kb = s_b[j * kBlock + threadIdx.x];
            const bool from_a = ka < kb;
            dst[o0 + u] = from_a ? ka : kb;
            i += from_a;
            j += !from_a;
        }
    }
}

// Step 4.  A workgroup owns `ct` consecutive columns.  `cols_dev`, when given, holds the number of
// columns on the device (a caller that does not know it on the host yet); rowid / t_row may be null
// (keys are then only put in order).
// LONG: only the columns longer than the LDS keys (their code needs twice the registers, which would
// halve the wavefronts of every launch; a pattern without such columns passes through this
// instantiation on its column pointers alone); otherwise only the others.
template <bool LONG>
__global__ __launch_bounds__(kBlock) void tp_order_kernel(
    int64_t cols, const int32_t *__restrict__ cols_dev, int ct, const int32_t *__restrict__ t_indptr,
    int32_t *__restrict__ t_perm, const int32_t *__restrict__ rowid, int32_t *__restrict__ t_row,
    int32_t *__restrict__ tmp) {
    __shared__ int32_t s_off[kRows + 1];
    __shared__ __align__(16) int32_t s_key[kCap];
    static_assert(2 * kSlice * kBlock == kCap, "a lane's kSlice candidates of both runs fit the LDS keys");
    if (cols_dev) cols = *cols_dev;
    const int64_t ntiles = (cols + ct - 1) / ct, npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t c0 = tile * ct;
        const int nc = (int)(cols - c0 < ct ? cols - c0 : ct);
        const int32_t base = t_indptr[c0];
        for (int t = threadIdx.x; t <= nc; t += kBlock) s_off[t] = t_indptr[c0 + t] - base;
        __syncthreads();

        // columns [s0, e0) fit the LDS keys: stage, rank every key inside its column, write out
        auto ranked = [&](const int s0, const int e0) {
            const int o0 = s_off[s0], cnt = s_off[e0] - o0;
            const int32_t first = base + o0;
            for (int j = threadIdx.x; j < cnt; j += kBlock) s_key[j] = t_perm[first + j];
            __syncthreads();
            for (int j = threadIdx.x; j < cnt; j += kBlock) {
                int lo = s0, hi = e0;                       // column of key j
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (s_off[mid] - o0 <= j) lo = mid; else hi = mid;
                }
                const int b = s_off[lo] - o0, e = s_off[lo + 1] - o0;
                const int32_t key = s_key[j];
                int rank = 0;
                for (int q = b; q < e; ++q) rank += s_key[q] < key;
                t_perm[first + b + rank] = key;
                if (t_row) t_row[first + b + rank] = rowid[key];
            }
            __syncthreads();
        };

        // one column of kSortMin..kCap keys: a bitonic sort in LDS (ranking compares every key
        // with every other one of its column: fine for the handful of entries of a matrix column,
        // quadratic for the thousand rows of a level of a triangular solve's schedule)
        auto sorted = [&](const int c) {
            const int o0 = s_off[c], cnt = s_off[c + 1] - o0;
            const int32_t first = base + o0;
            int n = 2;
            while (n < cnt) n <<= 1;
            for (int j = threadIdx.x; j < n; j += kBlock) s_key[j] = j < cnt ? t_perm[first + j] : kPastAll;
            __syncthreads();
            for (int k = 2; k <= n; k <<= 1)
                for (int j = k >> 1; j > 0; j >>= 1) {
                    for (int t = threadIdx.x; t < n / 2; t += kBlock) {
                        const int i = ((t & ~(j - 1)) << 1) | (t & (j - 1)), p = i | j;   // a pair at distance j
                        const int32_t a = s_key[i], b = s_key[p];
                        if ((a > b) == ((i & k) == 0)) {
                            s_key[i] = b;
                            s_key[p] = a;
                        }
                    }
                    __syncthreads();
                }
            for (int j = threadIdx.x; j < cnt; j += kBlock) {
                const int32_t key = s_key[j];
                t_perm[first + j] = key;
                if (t_row) t_row[first + j] = rowid[key];
            }
            __syncthreads();
        };

        for (int s0 = 0; s0 < nc;) {
            int e0 = run_end(s_off, s0, nc, kCap);
            if (e0 > s0) {
                // a column worth sorting on its own ends the run before it
                bool mine = false;
                for (int c = s0 + threadIdx.x; c < e0; c += kBlock) mine = mine || s_off[c + 1] - s_off[c] >= kSortMin;
                if (__syncthreads_or(mine)) {
                    int c = s0;
                    while (c < e0 && s_off[c + 1] - s_off[c] < kSortMin) ++c;   // c < e0: there is one
                    if (c == s0) {
                        if (!LONG) sorted(s0);
                        s0 += 1;
                        continue;
                    }
                    e0 = c;
                }
                if (!LONG) ranked(s0, e0);
                s0 = e0;
                continue;
            }
            if (!LONG) {
                s0 += 1;
                continue;
            }
            // One column longer than the LDS keys.  Pieces of kCap keys are ranked in LDS and
            // written to `tmp` as sorted runs; merge passes then go back and forth between
            // `tmp` and the plan until one run is left.
            const int32_t first = base + s_off[s0];
            const int len = s_off[s0 + 1] - s_off[s0];
            int32_t *col = t_perm + first, *alt = tmp + first;
            for (int q0 = 0; q0 < len; q0 += kCap) {
                const int cnt = len - q0 < kCap ? len - q0 : kCap;
                for (int j = threadIdx.x; j < kCap; j += kBlock) s_key[j] = j < cnt ? col[q0 + j] : kPastAll;
                __syncthreads();
                // a lane ranks its kCap / kBlock keys together: every staged key is read once
                // (four to an LDS read) and compared with all of them -- independent additions,
                // where one key at a time waited for LDS at every step (ordering a column of 2^20
                // entries: 866 ms -> about 0.1 s together with the merge passes' LDS staging)
                constexpr int KPL = kCap / kBlock;
                typedef int32_t I4 __attribute__((ext_vector_type(4)));
                int32_t key[KPL];
                int rank[KPL];
#pragma unroll
                for (int u = 0; u < KPL; ++u) {
                    key[u] = s_key[threadIdx.x + u * kBlock];
                    rank[u] = 0;
                }
                const int cnt4 = (cnt + 3) & ~3;   // the padding is larger than every key
#pragma unroll 2
                for (int q = 0; q < cnt4; q += 4) {
                    const I4 k4 = *reinterpret_cast<const I4 *>(s_key + q);
#pragma unroll
                    for (int u = 0; u < KPL; ++u)
                        rank[u] += (k4[0] < key[u]) + (k4[1] < key[u]) + (k4[2] < key[u]) + (k4[3] < key[u]);
                }
#pragma unroll
                for (int u = 0; u < KPL; ++u)
                    if (threadIdx.x + u * kBlock < cnt) alt[q0 + rank[u]] = key[u];
                __syncthreads();
            }
            int32_t *src = alt, *dst = col;
            for (int width = kCap; width < len; width *= 2) {
                merge_pass(src, dst, len, width, s_key, s_key + kSlice * kBlock);
                __syncthreads();
                int32_t *sw = src; src = dst; dst = sw;
            }
            // `src` holds the ordered column
            for (int j = threadIdx.x; j < len; j += kBlock) {
                const int32_t key = src[j];
                if (src != col) col[j] = key;
                if (t_row) t_row[first + j] = rowid[key];
            }
            __syncthreads();
            s0 += 1;
        }
        __syncthreads();
    }
}

__global__ void symmetry_init_kernel(int32_t *flags, int square) {
    if (threadIdx.x == 0) {
        for (int k = 0; k < 16; ++k) flags[k] = 0;
        flags[0] = square;
        flags[1] = 1;
        flags[2] = 1;
    }
}

// Staging list of one block of rows (keys = columns of its entries) or of columns (keys = rows of
// its entries), entries [pb, pe) of `key`; line0 = the block's first row / column.  The segments of
// kStageSeg consecutive keys that the block names are marked in a bitmap over the segments within
// 32768 keys of line0 (what a 16-bit offset reaches; a block that names a key further away gets no
// list).  When at most MOST segments are marked, all of them whole (a segment cut off by the end
// of the vector the kernels will load it from would be read past that end), they are written to
// desc in ascending order (kStageDesc ints, unused places -1) and true is returned:
// stage_place(key) then gives kStageSeg * (rank of the key's segment) + offset inside the segment.
// Otherwise desc[0] = -2.  Called by a whole workgroup.
struct StageTable {
    static constexpr int kReach = 32768 / nm::kStageSeg;        // segments either side of line0's
    static constexpr int kWords = (2 * kReach + 8 + 31) / 32;   // (+ the block's own segments)
    uint32_t bits[kWords];
    int32_t before[kWords];     // marked segments in the words before this one
    int32_t seg0, count, bad;
};

template <int MOST>
__device__ __forceinline__ bool stage_block(StageTable &t, int64_t line0, int32_t pb, int32_t pe, int least_entries,
                                            int most_entries, int64_t veclen, const int32_t *__restrict__ key,
                                            int32_t *__restrict__ desc) {
    if (threadIdx.x < StageTable::kWords) t.bits[threadIdx.x] = 0;
    const int32_t seg0 = (int32_t)(line0 / nm::kStageSeg) - StageTable::kReach;
    if (threadIdx.x == 0) {
        t.seg0 = seg0;
        t.bad = (pe - pb > most_entries || pe - pb < least_entries || pe == pb) ? 1 : 0;
    }
    __syncthreads();
    if (t.bad == 0) {
        bool bad = false;
        for (int32_t p = pb + (int32_t)threadIdx.x; p < pe; p += kBlock) {
            const int32_t seg = key[p] / nm::kStageSeg, rel = seg - seg0;
            if (rel < 0 || rel >= StageTable::kWords * 32 || (int64_t)(seg + 1) * nm::kStageSeg > veclen) bad = true;
            else atomicOr(&t.bits[rel >> 5], 1u << (rel & 31));
        }
        if (bad) t.bad = 1;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int n = 0;
        for (int w = 0; w < StageTable::kWords; ++w) {
            t.before[w] = n;
            n += __builtin_popcount(t.bits[w]);
        }
        t.count = n;
    }
    __syncthreads();
    const bool staged = t.bad == 0 && t.count <= MOST;
    if (threadIdx.x < nm::kStageDesc) desc[threadIdx.x] = staged ? -1 : -2;
    __syncthreads();
    if (staged && threadIdx.x < StageTable::kWords) {
        // the marked segments of this word, to their ranks' places of the list
        uint32_t word = t.bits[threadIdx.x];
        for (int r = t.before[threadIdx.x]; word; word &= word - 1, ++r)
            desc[r] = seg0 + (int32_t)threadIdx.x * 32 + __builtin_ctz(word);
    }
    return staged;
}

__device__ __forceinline__ int32_t stage_place(const StageTable &t, int32_t k) {
    const int32_t rel = k / nm::kStageSeg - t.seg0;
    const int rank = t.before[rel >> 5] + __builtin_popcount(t.bits[rel >> 5] & ((1u << (rel & 31)) - 1u));
    return rank * nm::kStageSeg + k % nm::kStageSeg;
}

// t_pack, c_off16 and the staging lists of the plan; clears flags[1] / flags[2] when a difference
// does not fit 16 bits and counts the blocks that got a list in flags[4] (rows) / flags[5] (columns).
// A workgroup takes blocks of kPackCols columns, then blocks of kPackRows rows, lane = entry.
__global__ __launch_bounds__(kBlock) void tp_pack_kernel(
    int64_t rows, int64_t cols, const int32_t *__restrict__ t_indptr, const int32_t *__restrict__ t_row,
    const int32_t *__restrict__ t_perm, const int32_t *__restrict__ c_ptr32, const int32_t *__restrict__ c_idx32,
    int32_t *__restrict__ t_pack, int16_t *__restrict__ c_off16, int32_t *__restrict__ f_desc,
    int32_t *__restrict__ b_desc, int32_t *__restrict__ stats, int32_t *flags) {
    __shared__ StageTable table;
    bool fits_t = true, fits_c = true;
    const int64_t cblocks = (cols + nm::kPackCols - 1) / nm::kPackCols;
    for (int64_t b = blockIdx.x; b < cblocks; b += gridDim.x) {
        const int64_t c0 = b * nm::kPackCols;
        const int64_t c1 = c0 + nm::kPackCols < cols ? c0 + nm::kPackCols : cols;
        const int32_t pb = t_indptr[c0], pe = t_indptr[c1];
        {
            // statistics the caller's policy reads (nm_csr_transpose_plan_info): the longest column,
            // and the most entries that columns of more than 512 entries hold inside one group of 64
            // columns -- the SpMM kernels give such a group to one workgroup, which takes those
            // columns one after the other
            const int64_t c = c0 + threadIdx.x;
            int len = c < c1 ? t_indptr[c + 1] - t_indptr[c] : 0;
            int heavy = len > 512 ? len : 0;
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) {
                len = max(len, __shfl_xor(len, off, kWave));
                heavy += __shfl_xor(heavy, off, kWave);
            }
            // (left per wavefront and reduced by tp_stats_kernel: thousands of workgroups raising the
            // same word with atomics took longer than all the rest of the build)
            if ((threadIdx.x & (kWave - 1)) == 0) {
                stats[b * 8 + threadIdx.x / kWave] = len;
                stats[b * 8 + 4 + threadIdx.x / kWave] = heavy;
            }
        }
        // (a list made here is only read when every packed word of the plan turns out valid)
        // (a block of fewer than 1024 entries -- under four a column -- is a tile so small that the
        // backward is bound by the round trips of a tile, and the kernel without lists makes one fewer)
        const bool staged = stage_block<nm::kStageBwd>(table, c0, pb, pe, nm::kStageBwdMin, nm::kStageBwdCap, rows,
                                                       t_row, b_desc + b * nm::kStageDesc);
        for (int32_t p0 = pb; p0 < pe; p0 += kBlock) {
            const int32_t p = p0 + (int32_t)threadIdx.x;
            const bool active = p < pe;
            const int32_t r = active ? t_row[p] : 0;
            const int64_t dr = (int64_t)r - c0, dk = active ? (int64_t)t_perm[p] - p : 0;
            constexpr int64_t kFar = int64_t(1) << (31 - nm::kStagePlaceBits);
            if (staged) {   // place | distance, see kStagePlaceBits
                fits_t &= !active || (dk >= -kFar && dk < kFar);
                if (active)
                    t_pack[p] = (int32_t)((uint32_t)stage_place(table, r) | ((uint32_t)dk << nm::kStagePlaceBits));
            } else {
                fits_t &= !active || (dr >= -32768 && dr <= 32767 && dk >= -32768 && dk <= 32767);
                if (active) t_pack[p] = (int32_t)(((uint32_t)dr & 0xffffu) | ((uint32_t)dk << 16));
            }
        }
        __syncthreads();
    }
    const int64_t rblocks = (rows + nm::kPackRows - 1) / nm::kPackRows;
    for (int64_t b = blockIdx.x; b < rblocks; b += gridDim.x) {
        const int64_t r0 = b * nm::kPackRows;
        const int64_t r1 = r0 + nm::kPackRows < rows ? r0 + nm::kPackRows : rows;
        const int32_t kb = c_ptr32[r0], ke = c_ptr32[r1];
        {
            int len = 0;    // the longest row
            for (int64_t r = r0 + threadIdx.x; r < r1; r += kBlock) len = max(len, c_ptr32[r + 1] - c_ptr32[r]);
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) len = max(len, __shfl_xor(len, off, kWave));
            if ((threadIdx.x & (kWave - 1)) == 0) stats[cblocks * 8 + b * 4 + threadIdx.x / kWave] = len;
        }
        const bool staged = stage_block<nm::kStageFwd>(table, r0, kb, ke, 4, nm::kStageFwdCap, cols, c_idx32,
                                                       f_desc + b * nm::kStageDesc);
        for (int32_t k0 = kb; k0 < ke; k0 += kBlock) {
            const int32_t k = k0 + (int32_t)threadIdx.x;
            const bool active = k < ke;
            const int32_t c = active ? c_idx32[k] : 0;
            const int64_t dc = (int64_t)c - r0;
            fits_c &= !active || (dc >= -32768 && dc <= 32767);
            const int32_t v = staged && active ? stage_place(table, c) : (int32_t)dc;
            if (active) c_off16[k] = (int16_t)v;
        }
        __syncthreads();
    }
    if (!fits_t) flags[1] = 0;
    if (!fits_c) flags[2] = 0;
}

// flags[4] / flags[5]: blocks of rows / columns with a staging list; flags[6] / flags[7]: the longest
// column / row; flags[8]: the most entries that columns of more than 512 entries hold inside one
// aligned group of 64 columns; flags[9]: blocks of rows with a list and at most 3072 entries.  From what
// tp_pack_kernel left per block and per wavefront.
__global__ __launch_bounds__(kBlock) void tp_stats_kernel(int64_t rows, int64_t rblocks, int64_t cblocks,
                                                          const int32_t *__restrict__ c_ptr32,
                                                          const int32_t *__restrict__ f_desc,
                                                          const int32_t *__restrict__ b_desc,
                                                          const int32_t *__restrict__ stats, int32_t *flags) {
    __shared__ int32_t s_red[6][kBlock / kWave];
    const int64_t stride = (int64_t)gridDim.x * kBlock, tid = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    // staged row blocks, staged column blocks, longest column, longest row, heavy, staged row blocks of
    // at most 3072 entries (what the forward's fp64 tile holds)
    int v[6] = {0, 0, 0, 0, 0, 0};
    for (int64_t b = tid; b < rblocks; b += stride) {
        const bool staged = f_desc[b * nm::kStageDesc] >= 0;
        const int64_t r1 = (b + 1) * nm::kPackRows < rows ? (b + 1) * nm::kPackRows : rows;
        v[0] += staged;
        v[5] += staged && c_ptr32[r1] - c_ptr32[b * nm::kPackRows] <= 3072;
    }
    for (int64_t b = tid; b < cblocks; b += stride) v[1] += b_desc[b * nm::kStageDesc] >= 0;
    for (int64_t i = tid; i < cblocks * 8; i += stride) {
        if ((i & 4) == 0) v[2] = max(v[2], stats[i]);
        else v[4] = max(v[4], stats[i]);
    }
    for (int64_t i = tid; i < rblocks * 4; i += stride) v[3] = max(v[3], stats[cblocks * 8 + i]);
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1)
#pragma unroll
        for (int k = 0; k < 6; ++k) {
            const int o = __shfl_xor(v[k], off, kWave);
            v[k] = (k < 2 || k == 5) ? v[k] + o : max(v[k], o);
        }
    if ((threadIdx.x & (kWave - 1)) == 0)
        for (int k = 0; k < 6; ++k) s_red[k][threadIdx.x / kWave] = v[k];
    __syncthreads();
    if (threadIdx.x < 6) {
        const int k = threadIdx.x;
        const bool sum = k < 2 || k == 5;
        int r = 0;
        for (int w = 0; w < kBlock / kWave; ++w) r = sum ? r + s_red[k][w] : max(r, s_red[k][w]);
        const int slot = k == 0 ? 4 : k == 1 ? 5 : k == 2 ? 6 : k == 3 ? 7 : k == 4 ? 8 : 9;
        if (sum) { if (r) atomicAdd(&flags[slot], r); }
        else if (r) atomicMax(&flags[slot], r);
    }
}

// Clears flags[0] unless A^T has exactly A's structure.
__global__ void symmetry_check_kernel(int64_t nnz, int64_t cols, const int32_t *__restrict__ col32,
                                      const int32_t *__restrict__ ptr32, const int32_t *__restrict__ t_row,
                                      const int32_t *__restrict__ t_indptr, int32_t *flags) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    bool same = true;
    for (int64_t p = tid; p < nnz; p += stride) same &= t_row[p] == col32[p];
    for (int64_t c = tid; c <= cols; c += stride) same &= t_indptr[c] == ptr32[c];
    if (!same) flags[0] = 0;
}

int check_sizes(int64_t rows, int64_t cols, int64_t nnz) {
    NM_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0, "negative size");
    if (rows >= 0x7ffffffe || cols >= 0x7ffffffe || nnz >= 0x7ffffffe)
        return nm::fail(NM_ERR_UNSUPPORTED, "transposed-structure plans index with 32 bits");
    return NM_OK;
}

}  // namespace

namespace nm {

size_t tplan_work_bytes(int64_t rows, int64_t cols, int64_t nnz) {
    (void)rows;
    return work_layout(cols, nnz, nullptr, nullptr);
}

int tplan_build(int64_t rows, int64_t cols, int64_t nnz, const int64_t *indices, const int64_t *indptr,
                const TPlan &plan, void *work, size_t work_bytes, int32_t *rowid_out, hipStream_t s) {
    WorkT w;
    const size_t need = work_layout(cols, nnz, work, &w);
    if (work_bytes < need) return fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", work_bytes, need);
    int32_t *rowid = rowid_out ? rowid_out : w.rowid;
    if (int rc = fill_async(w.count, cols + 1, (int64_t)0, s)) return rc;
    if (rows > 0) {
        const int rt = tile_rows(rows, nnz);
        int64_t grid = xcd_padded(ceil_div(rows, rt));
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(tp_count_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, rows, rt, indices, indptr,
                           (unsigned long long *)w.count, rowid, plan.c_idx32, plan.c_ptr32, plan.chunk_row);
        NM_LAUNCH_CHECK("tp_count_kernel");
    } else {
        if (int rc = fill_async(plan.c_ptr32, (int64_t)1, (int32_t)0, s)) return rc;
    }
    if (int rc = scan_exclusive_i64(w.count, cols + 1, w.scan, s)) return rc;
    {
        int64_t grid = ceil_div(cols + 1, kBlock);
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(tp_pointers_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, cols, w.count,
                           plan.t_indptr, w.cursor);
        NM_LAUNCH_CHECK("tp_pointers_kernel");
    }
    if (nnz > 0) {
        int64_t grid = ceil_div(nnz, kBlock);
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(tp_scatter_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, nnz, plan.c_idx32, w.cursor,
                           plan.t_perm);
        NM_LAUNCH_CHECK("tp_scatter_kernel");
        // (down to one column per workgroup: columns longer than the LDS keys are ordered by their
        // workgroup alone, one after the other)
        const int ct = tile_rows(cols, nnz, 1);
        grid = xcd_padded(ceil_div(cols, ct));
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(tp_order_kernel<false>, dim3((unsigned)grid), dim3(kBlock), 0, s, cols, (const int32_t *)nullptr,
                           ct, plan.t_indptr, plan.t_perm, rowid, plan.t_row, w.tmp);
        NM_LAUNCH_CHECK("tp_order_kernel");
        hipLaunchKernelGGL(tp_order_kernel<true>, dim3((unsigned)grid), dim3(kBlock), 0, s, cols, (const int32_t *)nullptr,
                           ct, plan.t_indptr, plan.t_perm, rowid, plan.t_row, w.tmp);
        NM_LAUNCH_CHECK("tp_order_kernel<long>");
    }
    hipLaunchKernelGGL(symmetry_init_kernel, dim3(1), dim3(64), 0, s, plan.flags, rows == cols ? 1 : 0);
    if (rows == cols) {
        int64_t m = nnz > cols + 1 ? nnz : cols + 1;
        int64_t grid = ceil_div(m, kBlock);
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(symmetry_check_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, nnz, cols, plan.c_idx32,
                           plan.c_ptr32, plan.t_row, plan.t_indptr, plan.flags);
    }
    NM_LAUNCH_CHECK("symmetry check");
    if (nnz > 0) {
        int64_t grid = ceil_div(cols > rows ? cols : rows, (int64_t)kPackCols);
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(tp_pack_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, rows, cols, plan.t_indptr,
                           plan.t_row, plan.t_perm, plan.c_ptr32, plan.c_idx32, plan.t_pack, plan.c_off16, plan.f_desc,
                           plan.b_desc, plan.stats, plan.flags);
        NM_LAUNCH_CHECK("tp_pack_kernel");
        hipLaunchKernelGGL(tp_stats_kernel, dim3(32), dim3(kBlock), 0, s, rows, ceil_div(rows, (int64_t)kPackRows),
                           ceil_div(cols, (int64_t)kPackCols), plan.c_ptr32, plan.f_desc, plan.b_desc, plan.stats,
                           plan.flags);
        NM_LAUNCH_CHECK("tp_stats_kernel");
    }
    return NM_OK;
}

int segments_sort_i32(const int32_t *nseg_dev, int64_t nseg_max, int64_t nkeys, const int32_t *seg_ptr,
                      int32_t *keys, int32_t *tmp, hipStream_t s) {
    if (nkeys <= 0 || nseg_max <= 0) return NM_OK;
    // few segments per workgroup: their number is not known here, and they may be long
    const int ct = 8;
    int64_t grid = xcd_padded(ceil_div(nseg_max, ct));
    if (grid > 8192) grid = 8192;
    hipLaunchKernelGGL(tp_order_kernel<false>, dim3((unsigned)grid), dim3(kBlock), 0, s, nseg_max, nseg_dev, ct, seg_ptr,
                       keys, (const int32_t *)nullptr, (int32_t *)nullptr, tmp);
    NM_LAUNCH_CHECK("tp_order_kernel (segments)");
    hipLaunchKernelGGL(tp_order_kernel<true>, dim3((unsigned)grid), dim3(kBlock), 0, s, nseg_max, nseg_dev, ct, seg_ptr,
                       keys, (const int32_t *)nullptr, (int32_t *)nullptr, tmp);
    NM_LAUNCH_CHECK("tp_order_kernel<long> (segments)");
    return NM_OK;
}

}  // namespace nm

extern "C" int nm_csr_transpose_plan_bytes(int64_t rows, int64_t cols, int64_t nnz, size_t *plan_bytes,
                                           size_t *work_bytes) {
    NM_REQUIRE(plan_bytes && work_bytes, "null size pointer");
    if (int rc = check_sizes(rows, cols, nnz)) return rc;
    *plan_bytes = nm::tplan_layout(rows, cols, nnz, nullptr, nullptr);
    *work_bytes = nm::tplan_work_bytes(rows, cols, nnz);
    return NM_OK;
}

extern "C" int nm_csr_transpose_plan_build(int64_t rows, int64_t cols, int64_t nnz, const int64_t *indices,
                                           const int64_t *indptr, void *plan_mem, size_t plan_bytes, void *work,
                                           size_t work_bytes, nm_stream stream) {
    if (int rc = check_sizes(rows, cols, nnz)) return rc;
    NM_REQUIRE(indptr && plan_mem && work && (nnz == 0 || indices), "null pointer argument");
    nm::TPlan plan;
    const size_t need = nm::tplan_layout(rows, cols, nnz, plan_mem, &plan);
    if (plan_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "plan memory of %zu bytes, %zu needed", plan_bytes, need);
    return nm::tplan_build(rows, cols, nnz, indices, indptr, plan, work, work_bytes, nullptr,
                           nm::as_stream(stream));
}

extern "C" int nm_csr_transpose_plan_info(int64_t rows, int64_t cols, int64_t nnz, const void *plan_mem,
                                          int32_t info[16], nm_stream stream) {
    if (int rc = check_sizes(rows, cols, nnz)) return rc;
    NM_REQUIRE(plan_mem != nullptr && info != nullptr, "null pointer argument");
    nm::TPlan plan;
    nm::tplan_layout(rows, cols, nnz, const_cast<void *>(plan_mem), &plan);
    hipStream_t s = nm::as_stream(stream);
    NM_HIP_TRY(hipMemcpyAsync(info, plan.flags, 16 * sizeof(int32_t), hipMemcpyDeviceToHost, s));
    NM_HIP_TRY(hipStreamSynchronize(s));
    if (nnz == 0) info[1] = info[2] = info[4] = info[5] = info[9] = 0;     // (nothing was packed or listed)
    return NM_OK;
}
