// Sparse LU without pivoting: symbolic phase (pattern of M = L + U with fill).
// Stands in for the first half of splu (cpp/sparse_csr_cpu.cpp:777-954).
//
// The pattern of row i is found, as in the reference, by the fill2 traversal of
// Rose and Tarjan: stored neighbours of i are kept; then the pivots t < i that
// have been reached are expanded in ascending order by a breadth-first walk that
// continues through vertices <= t and keeps (without expanding) every newly
// reached vertex > t.  Rows are independent, so one wavefront takes one row at a
// time (rows w, w + W, w + 2W, ... for wavefront w of W): the queue is popped
// serially, the edges of the popped vertex are handled by the lanes, and the scan
// for the next pivot and the emission of the kept columns go 64 vertices at a time.
// Each wavefront owns three arrays of `rows` entries in the caller's scratch
// (visit stamps, queue, keep flags); they are accessed with volatile operations
// because lanes of the wavefront communicate through them.
//
// The work per row is that of the serial algorithm (the reference spends O(rows)
// per row as well): this is meant for the moderate sizes a direct solve is used at.
//
// Numeric phase (cpp/sparse_csr_cpu.cpp:956-1000): left-looking column LU on the rows of
// M^T (= columns of M).  For the entries (i, k), i < k, of column k in ascending i, every
// later entry (j, k) takes  M_jk -= M_ji * M_ik  where column i stores row j; then the
// entries below the diagonal are divided by it.  Per entry the operations come in the
// serial order, so the factors equal the reference's bit for bit.
// Column k needs the finished columns i of its entries above the diagonal, and nothing
// else: workgroups take batches of consecutive columns in ascending order from a ticket
// counter, one column per wavefront, keep the columns in LDS, and before using column i wait
// for its flag -- a flag and values in LDS when column i belongs to the same batch, in global
// memory otherwise.  A wavefront only ever waits for a column with a smaller number, which a
// running wavefront holds, so the grid always makes progress whatever part of it is resident;
// a bounded number of polls backs that up, after which every wavefront leaves and the call
// reports an error.  Early pivots of a column
// overlap with the tail of the columns before it, which is where a banded factor, whose
// columns form one long dependency chain, gets its parallelism from.
#include "nm_common.hpp"
#include "nm_scan.hpp"

namespace {

constexpr int kBlock = 256;
constexpr int kLuWaves = 4096;   // wavefronts that share the rows

struct LuScratch {
    int32_t *stamp, *queue;   // [waves][rows]
    uint8_t *keep;            // [waves][rows]
    int64_t *scan;            // scan scratch for the row pointer
};

inline size_t align_up(size_t v) { return (v + 255) & ~size_t(255); }

// Wavefronts that share the rows: at most kLuWaves, at most one per row, and few enough that
// their scratch (9 bytes per row each) stays within kLuScratchBytes.
constexpr int64_t kLuScratchBytes = int64_t(1) << 30;
inline int lu_waves(int64_t rows) {
    if (rows < 1) return 1;
    int64_t w = rows < kLuWaves ? rows : kLuWaves;
    const int64_t fit = kLuScratchBytes / (9 * rows);
    // (a launch is whole workgroups of four wavefronts: fewer wavefronts than rows must be a
    //  multiple of four, or the last workgroup's extra wavefronts would take rows without scratch)
    if (w > fit) w = (fit < 64 ? 64 : fit) / 4 * 4;
    return (int)w;
}

size_t lu_layout(int64_t rows, void *base, LuScratch *S) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align_up(bytes);
        return q;
    };
    const size_t w = (size_t)lu_waves(rows), n = (size_t)(rows > 0 ? rows : 1);
    LuScratch s;
    s.stamp = (int32_t *)take(w * n * 4);
    s.queue = (int32_t *)take(w * n * 4);
    s.keep = (uint8_t *)take(w * n);
    s.scan = (int64_t *)take(nm::scan_scratch_bytes(rows + 1));
    if (S) *S = s;
    return off;
}

__global__ void lu_init_kernel(int64_t total, int32_t *__restrict__ stamp, uint8_t *__restrict__ keep) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        stamp[i] = -1;
        keep[i] = 0;
    }
}

// FILL == false: As_indptr[i] = number of kept columns of row i.
// FILL == true : As_indices / As_data of row i are written at As_indptr[i]: the value of A where A
//                stores the column, 0 at the fill (cpp/sparse_csr_cpu.cpp:908-954).
template <typename T, bool FILL>
__global__ __launch_bounds__(kBlock) void lu_rows_kernel(int64_t rows, const T *__restrict__ A_data,
                                                         const int64_t *__restrict__ A_indices,
                                                         const int64_t *__restrict__ A_indptr,
                                                         int64_t *__restrict__ As_indptr,
                                                         int64_t *__restrict__ As_indices, T *__restrict__ As_data,
                                                         int32_t *stamp_all, int32_t *queue_all, uint8_t *keep_all) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    volatile int32_t *stamp = stamp_all + wave * rows;
    volatile int32_t *queue = queue_all + wave * rows;
    volatile uint8_t *keep = keep_all + wave * rows;
    const unsigned long long lower_lanes = (1ull << lane) - 1ull;

    for (int64_t i = wave; i < rows; i += nwaves) {
        const int32_t mark = (int32_t)i;   // rows come in ascending order per wavefront: a stamp names one row
        if (lane == 0) stamp[i] = mark;
        for (int64_t k = A_indptr[i] + lane; k < A_indptr[i + 1]; k += 64) {
            const int64_t u = A_indices[k];
            if (u < 0 || u >= rows) continue;   // not a column of a square matrix: ignored rather than written
            stamp[u] = mark;
            keep[u] = 1;
        }
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        // pivots t < i that have been reached, in ascending order; a walk may reach later pivots
        for (int64_t t0 = 0; t0 < i; t0 += 64) {
            int64_t done = t0 - 1;
            for (;;) {
                const int64_t tc = t0 + lane;
                const bool cand = tc < i && tc > done && stamp[tc] == mark;
                const unsigned long long m = __ballot(cand);
                if (m == 0) break;
                const int64_t t = t0 + (__ffsll((long long)m) - 1);
                done = t;
                // breadth-first walk from t through vertices <= t
                int64_t head = 0, tail = 1;
                if (lane == 0) queue[0] = (int32_t)t;
                __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                while (head < tail) {
                    const int64_t u = queue[head++];
                    const int64_t kb = A_indptr[u], ke = A_indptr[u + 1];
                    for (int64_t k0 = kb; k0 < ke; k0 += 64) {
                        const int64_t k = k0 + lane;
                        int64_t w = -1;
                        bool fresh = false;
                        if (k < ke) {
                            w = A_indices[k];
                            fresh = w >= 0 && w < rows && stamp[w] != mark;   // columns of a row are distinct: no two lanes share w
                        }
                        if (fresh) {
                            stamp[w] = mark;
                            if (w > t) keep[w] = 1;
                        }
                        const bool push = fresh && w <= t;
                        const unsigned long long pm = __ballot(push);
                        if (push) queue[tail + __popcll(pm & lower_lanes)] = (int32_t)w;
                        tail += __popcll(pm);
                        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
                    }
                }
            }
        }
        // kept columns in ascending order
        int64_t out = FILL ? As_indptr[i] : 0;
        const int64_t ab = A_indptr[i], ae = A_indptr[i + 1];
        for (int64_t j0 = 0; j0 < rows; j0 += 64) {
            const int64_t j = j0 + lane;
            const bool kept = j < rows && keep[j] != 0;
            const unsigned long long m = __ballot(kept);
            if (kept) {
                keep[j] = 0;
                if (FILL) {
                    const int64_t pos = out + __popcll(m & lower_lanes);
                    int64_t lo = ab, hi = ae;   // A's value at column j, if stored
                    while (lo < hi) {
                        const int64_t mid = (lo + hi) >> 1;
                        if (A_indices[mid] < j) lo = mid + 1; else hi = mid;
                    }
                    As_indices[pos] = j;
                    As_data[pos] = (lo < ae && A_indices[lo] == j) ? A_data[lo] : T(0);
                }
            }
            out += __popcll(m);
        }
        if (!FILL && lane == 0) As_indptr[i] = out;
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    }
}

// Values on a known filled pattern: one wavefront per row, a lane per entry of the row.
template <typename T>
__global__ __launch_bounds__(kBlock) void lu_values_kernel(int64_t rows, const T *__restrict__ A_data,
                                                           const int64_t *__restrict__ A_indices,
                                                           const int64_t *__restrict__ A_indptr,
                                                           const int64_t *__restrict__ As_indptr,
                                                           const int64_t *__restrict__ As_indices,
                                                           T *__restrict__ As_data) {
    const int lane = threadIdx.x & 63;
    const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (int64_t i = (int64_t)blockIdx.x * (blockDim.x >> 6) + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
         i < rows; i += nwaves) {
        const int64_t ab = A_indptr[i], ae = A_indptr[i + 1], pe = As_indptr[i + 1];
        for (int64_t p = As_indptr[i] + lane; p < pe; p += 64) {
            const int64_t j = As_indices[p];
            int64_t lo = ab, hi = ae;
            while (lo < hi) {
                const int64_t mid = (lo + hi) >> 1;
                if (A_indices[mid] < j) lo = mid + 1; else hi = mid;
            }
            As_data[p] = (lo < ae && A_indices[lo] == j) ? A_data[lo] : T(0);
        }
    }
}

#ifndef NM_LU_WAVES
#define NM_LU_WAVES 8
#endif
constexpr int kLuCap = 1024;              // entries of a column kept in LDS, per wavefront
constexpr int kLuWavesPerBlock = NM_LU_WAVES;   // columns of a batch = wavefronts of a workgroup of the numeric phase
constexpr int kLuFlowBlock = kLuWavesPerBlock * 64;
constexpr int64_t kLuSpinLimit = 1 << 24;  // polls of one dependency flag, without any column finishing, before giving up

struct LuFlow {
    int64_t *below;  // [cols] position of the column's first entry below the diagonal
    int32_t *done;   // [cols] 0 = pending, 1 = the column holds its final values
    int32_t *ctl;    // [0] next ticket, [1] failure, [2] columns finished
};

size_t flow_layout(int64_t cols, void *base, LuFlow *F) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align_up(bytes);
        return q;
    };
    LuFlow f;
    f.ctl = (int32_t *)take(64);
    f.done = (int32_t *)take((size_t)(cols > 0 ? cols : 1) * 4);
    f.below = (int64_t *)take((size_t)(cols > 0 ? cols : 1) * 8);
    if (F) *F = f;
    return off;
}

// The column of a wavefront: in LDS (rows as 32-bit, values) or, when it is too long, in
// place in global memory, where the lanes hand values on through volatile accesses.
template <typename T, bool IN_LDS>
struct OwnColumn {
    int32_t *s_rows;
    T *s_vals;
    const int64_t *g_rows;
    volatile T *g_vals;
    __device__ __forceinline__ int64_t row(int64_t e) const { return IN_LDS ? (int64_t)s_rows[e] : g_rows[e]; }
    __device__ __forceinline__ T val(int64_t e) const { return IN_LDS ? s_vals[e] : g_vals[e]; }
    __device__ __forceinline__ void set(int64_t e, T v) const {
        if (IN_LDS) s_vals[e] = v; else g_vals[e] = v;
    }
};

// below[k] = position of the first entry of column k with a row index > k.
__global__ void lu_below_kernel(int64_t cols, const int64_t *__restrict__ indices,
                                const int64_t *__restrict__ indptr, int64_t *__restrict__ below) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < cols; k += stride) {
        int64_t lo = indptr[k], hi = indptr[k + 1];
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (indices[mid] <= k) lo = mid + 1; else hi = mid;
        }
        below[k] = lo;
    }
}

// Returns false when a dependency did not arrive within the poll limit (or another wavefront failed).
// Everything about a pivot that the structure alone decides -- which entries of column i lie below
// its diagonal and where their rows sit in this column -- is looked up before the wait for column i,
// so that what follows the arrival of the flag is one load, one multiply and one subtraction.
// The columns of one batch [base, base + kLuWavesPerBlock) are worked on by the wavefronts of one
// workgroup: a column of the batch that sits in LDS is read there, behind an LDS flag, by the
// later columns of the batch, which spares them the round trip through global memory that the
// flag and the values of a column of another workgroup cost.
template <typename T>
struct LuBatch {
    int64_t base;                 // first column of the batch
    const int64_t *pb;            // [kLuWavesPerBlock] LDS: start of each column in the CSR arrays
    T (*vals)[kLuCap];            // LDS values of the batch's columns
    volatile int32_t *ready;      // [kLuWavesPerBlock] LDS: 0 pending, 1 final values in LDS, 2 final values in global memory only
};

template <typename T, bool IN_LDS>
__device__ bool lu_column(int64_t k, int64_t pb, int64_t len, const OwnColumn<T, IN_LDS> &own,
                          const LuBatch<T> &batch,
                          const int64_t *__restrict__ indices, const int64_t *__restrict__ indptr,
                          const int64_t *__restrict__ below_of, T *values, int32_t *done, int32_t *ctl,
                          int64_t spin_limit, int lane) {
    if (IN_LDS) {
        for (int64_t e = lane; e < len; e += 64) {
            own.s_rows[e] = (int32_t)indices[pb + e];
            own.s_vals[e] = values[pb + e];
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    }
    // position in this column of row j, searched among the entries after e; -1 when not stored
    auto find = [&](int64_t e, int64_t j) {
        int64_t lo = e + 1, hi = len;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (own.row(mid) < j) lo = mid + 1; else hi = mid;
        }
        return (lo < len && own.row(lo) == j) ? lo : (int64_t)-1;
    };
    // What the structure alone says about pivot e: the column i it names, where the entries of
    // column i below its diagonal start and end, this lane's entry of them and the place of
    // that entry's row in this column.  Looked up one pivot ahead: the two dependent loads it
    // takes would otherwise stand between the arrival of a flag and the update it allows.
    struct Look {
        int64_t i, ls, ie, t_first, at_first;
    };
    auto look = [&](int64_t e) {
        Look L{-1, 0, 0, 0, -1};
        if (e >= len) return L;
        const int64_t i = own.row(e);
        if (i >= k) return L;
        L.i = i;
        L.ls = below_of[i];
        L.ie = indptr[i + 1];
        L.t_first = L.ls + lane;
        L.at_first = L.t_first < L.ie ? find(e, indices[L.t_first]) : (int64_t)-1;
        return L;
    };
    int64_t e = 0;
    Look next = look(0);
    for (; next.i >= 0; ++e) {
        const Look cur = next;
        next = look(e + 1);
        const int64_t i = cur.i, ls = cur.ls, ie = cur.ie, t_first = cur.t_first, at_first = cur.at_first;
        // The limit bounds polls WITHOUT PROGRESS: every 256 polls the wavefront looks at the failure
        // word and at the count of finished columns, and starts counting afresh when that count has
        // moved.  A wavefront that legitimately waits behind a chain of thousands of slow columns
        // is thus never cut off, while a grid in which nothing finishes any more is.
        int64_t polls = 0;
        int32_t seen_done = -1;
        auto still_hopeful = [&]() -> bool {   // false: give up
            if (++polls > spin_limit) return false;
            if ((polls & 255) == 0) {
                if (__hip_atomic_load(ctl + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return false;
                const int32_t now = __hip_atomic_load(ctl + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (now != seen_done) {
                    seen_done = now;
                    polls = 0;
                }
            }
            return true;
        };
        bool in_lds = false;   // column i is one of this batch's and its final values are in LDS
        if (i >= batch.base) {
            const int wi = (int)(i - batch.base);
            int32_t state;
            while ((state = batch.ready[wi]) == 0) {
                if (!still_hopeful()) return false;
                __builtin_amdgcn_s_sleep(1);
            }
            in_lds = state == 1;
        } else {
            while (__hip_atomic_load(done + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
                if (!still_hopeful()) return false;
                __builtin_amdgcn_s_sleep(1);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");   // the value loads below stay after the flag
        const T m_ik = own.val(e);
        // entry t of the CSR arrays, which belongs to column i
        auto other = [&](int64_t t) -> T {
            if (in_lds) {
                const int wi = (int)(i - batch.base);
                return batch.vals[wi][t - batch.pb[wi]];
            }
            return __hip_atomic_load(values + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        };
        if (at_first >= 0) {
            const T prod = other(t_first) * m_ik;
            own.set(at_first, own.val(at_first) - prod);
        }
        for (int64_t t0 = ls + 64; t0 < ie; t0 += 64) {          // columns with more than 64 entries below
            const int64_t t = t0 + lane;
            const int64_t at = t < ie ? find(e, indices[t]) : (int64_t)-1;
            if (at >= 0) {
                const T prod = other(t) * m_ik;
                own.set(at, own.val(at) - prod);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    }
    if (e < len && own.row(e) == k) {
        const T d = own.val(e);
        for (int64_t q = e + 1 + lane; q < len; q += 64) own.set(q, own.val(q) / d);
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    }
    // the later columns of the batch first: they read this one in LDS
    if (IN_LDS) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0) batch.ready[k - batch.base] = 1;
        for (int64_t q = lane; q < len; q += 64) values[pb + q] = own.s_vals[q];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    if (lane == 0) {
        __hip_atomic_store(done + k, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        atomicAdd(ctl + 2, 1);   // columns finished so far: what a waiting wavefront watches for progress
        if (!IN_LDS) batch.ready[k - batch.base] = 2;
    }
    return true;
}

template <typename T>
__global__ __launch_bounds__(kLuFlowBlock) void lu_flow_kernel(int64_t cols, const int64_t *__restrict__ indices,
                                                         const int64_t *__restrict__ indptr,
                                                         const int64_t *__restrict__ below, T *values,
                                                         int32_t *done, int32_t *ctl, int64_t spin_limit) {
    // dynamic LDS: the batch's columns, values first (8-byte aligned), then rows
    extern __shared__ __align__(16) unsigned char s_columns[];
    T (*s_vals)[kLuCap] = reinterpret_cast<T (*)[kLuCap]>(s_columns);
    int32_t (*s_rows)[kLuCap] =
        reinterpret_cast<int32_t (*)[kLuCap]>(s_columns + sizeof(T) * kLuWavesPerBlock * kLuCap);
    __shared__ int64_t s_pb[kLuWavesPerBlock];
    __shared__ int32_t s_ready[kLuWavesPerBlock];
    __shared__ int32_t s_ticket, s_abort;
    const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (;;) {
        // one ticket per workgroup and batch of consecutive columns, one column per wavefront
        if (threadIdx.x == 0) {
            s_ticket = atomicAdd(ctl, kLuWavesPerBlock);
            s_abort = __hip_atomic_load(ctl + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (threadIdx.x < kLuWavesPerBlock) s_ready[threadIdx.x] = 0;
        __syncthreads();
        const int64_t base = s_ticket;
        if (base >= cols || s_abort != 0) break;   // the same decision in every wavefront
        const int64_t k = base + w;
        if (k < cols) {
            const int64_t pb = indptr[k], len = indptr[k + 1] - pb;
            if (lane == 0) s_pb[w] = pb;
            const LuBatch<T> batch{base, s_pb, s_vals, s_ready};
            bool ok;
            if (len <= kLuCap) {
                const OwnColumn<T, true> own{s_rows[w], s_vals[w], nullptr, nullptr};
                ok = lu_column<T, true>(k, pb, len, own, batch, indices, indptr, below, values, done, ctl, spin_limit,
                                        lane);
            } else {
                const OwnColumn<T, false> own{nullptr, nullptr, indices + pb, values + pb};
                ok = lu_column<T, false>(k, pb, len, own, batch, indices, indptr, below, values, done, ctl, spin_limit,
                                         lane);
            }
            if (!ok && lane == 0) atomicExch(ctl + 1, 1);
        }
        __syncthreads();   // the batch's columns in LDS have no readers left
    }
}

int check_rows(int64_t rows) {
    NM_REQUIRE(rows >= 0, "negative size");
    if (rows >= (int64_t(1) << 31) - 2)
        return nm::fail(NM_ERR_UNSUPPORTED, "splu indexes rows with 32 bits");
    return NM_OK;
}

}  // namespace

extern "C" int nm_splu_symbolic_bytes(int64_t rows, size_t *bytes) {
    NM_REQUIRE(bytes != nullptr, "bytes is null");
    if (int rc = check_rows(rows)) return rc;
    *bytes = lu_layout(rows, nullptr, nullptr);
    return NM_OK;
}

extern "C" int nm_splu_symbolic(int64_t rows, const int64_t *A_indices, const int64_t *A_indptr,
                                int64_t *As_indptr, void *workspace, size_t workspace_bytes, nm_stream stream) {
    if (int rc = check_rows(rows)) return rc;
    NM_REQUIRE(A_indptr && As_indptr && workspace, "null pointer argument");
    LuScratch S;
    const size_t need = lu_layout(rows, workspace, &S);
    if (workspace_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace_bytes, need);
    hipStream_t s = nm::as_stream(stream);
    if (int rc = nm::fill_async(As_indptr + rows, 1, (int64_t)0, s)) return rc;
    if (rows == 0) return NM_OK;
    const int waves = lu_waves(rows);
    hipLaunchKernelGGL(lu_init_kernel, dim3(1024), dim3(kBlock), 0, s, (int64_t)waves * rows, S.stamp, S.keep);
    NM_LAUNCH_CHECK("lu_init_kernel");
    const unsigned grid = (unsigned)nm::ceil_div((int64_t)waves * 64, kBlock);
    hipLaunchKernelGGL((lu_rows_kernel<float, false>), dim3(grid), dim3(kBlock), 0, s, rows, (const float *)nullptr,
                       A_indices, A_indptr, As_indptr, (int64_t *)nullptr, (float *)nullptr, S.stamp, S.queue,
                       S.keep);
    NM_LAUNCH_CHECK("lu_rows_kernel<count>");
    return nm::scan_exclusive_i64(As_indptr, rows + 1, S.scan, s);
}

extern "C" int nm_splu_fill(nm_dtype dt, int64_t rows, const void *A_data, const int64_t *A_indices,
                            const int64_t *A_indptr, const int64_t *As_indptr, int64_t *As_indices, void *As_data,
                            void *workspace, size_t workspace_bytes, nm_stream stream) {
    if (int rc = check_rows(rows)) return rc;
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (rows == 0) return NM_OK;
    NM_REQUIRE(A_indptr && As_indptr && workspace, "null pointer argument");
    LuScratch S;
    const size_t need = lu_layout(rows, workspace, &S);
    if (workspace_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace_bytes, need);
    hipStream_t s = nm::as_stream(stream);
    const int waves = lu_waves(rows);
    hipLaunchKernelGGL(lu_init_kernel, dim3(1024), dim3(kBlock), 0, s, (int64_t)waves * rows, S.stamp, S.keep);
    NM_LAUNCH_CHECK("lu_init_kernel");
    const unsigned grid = (unsigned)nm::ceil_div((int64_t)waves * 64, kBlock);
    if (dt == NM_F32)
        hipLaunchKernelGGL((lu_rows_kernel<float, true>), dim3(grid), dim3(kBlock), 0, s, rows, (const float *)A_data,
                           A_indices, A_indptr, const_cast<int64_t *>(As_indptr), As_indices, (float *)As_data,
                           S.stamp, S.queue, S.keep);
    else
        hipLaunchKernelGGL((lu_rows_kernel<double, true>), dim3(grid), dim3(kBlock), 0, s, rows,
                           (const double *)A_data, A_indices, A_indptr, const_cast<int64_t *>(As_indptr), As_indices,
                           (double *)As_data, S.stamp, S.queue, S.keep);
    NM_LAUNCH_CHECK("lu_rows_kernel<fill>");
    return NM_OK;
}

extern "C" int nm_splu_values(nm_dtype dt, int64_t rows, const void *A_data, const int64_t *A_indices,
                              const int64_t *A_indptr, const int64_t *As_indptr, const int64_t *As_indices,
                              void *As_data, nm_stream stream) {
    if (int rc = check_rows(rows)) return rc;
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (rows == 0) return NM_OK;
    NM_REQUIRE(A_indptr && As_indptr, "null pointer argument");
    hipStream_t s = nm::as_stream(stream);
    int64_t grid = nm::ceil_div(rows * 64, kBlock);
    if (grid > 65536) grid = 65536;
    if (dt == NM_F32)
        hipLaunchKernelGGL(lu_values_kernel<float>, dim3((unsigned)grid), dim3(kBlock), 0, s, rows,
                           (const float *)A_data, A_indices, A_indptr, As_indptr, As_indices, (float *)As_data);
    else
        hipLaunchKernelGGL(lu_values_kernel<double>, dim3((unsigned)grid), dim3(kBlock), 0, s, rows,
                           (const double *)A_data, A_indices, A_indptr, As_indptr, As_indices, (double *)As_data);
    NM_LAUNCH_CHECK("lu_values_kernel");
    return NM_OK;
}

extern "C" int nm_splu_numeric_bytes(int64_t cols, size_t *bytes) {
    NM_REQUIRE(bytes != nullptr, "bytes is null");
    if (int rc = check_rows(cols)) return rc;
    *bytes = flow_layout(cols, nullptr, nullptr);
    return NM_OK;
}

extern "C" int nm_splu_numeric(nm_dtype dt, int64_t cols, void *Mt_data, const int64_t *Mt_indices,
                               const int64_t *Mt_indptr, void *workspace, size_t workspace_bytes,
                               int64_t poll_limit, nm_stream stream) {
    if (int rc = check_rows(cols)) return rc;
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (cols == 0) return NM_OK;
    NM_REQUIRE(Mt_indptr && workspace, "null pointer argument");
    LuFlow F;
    const size_t need = flow_layout(cols, workspace, &F);
    if (workspace_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace_bytes, need);
    hipStream_t s = nm::as_stream(stream);
    if (int rc = nm::fill_async(F.ctl, 16, (int32_t)0, s)) return rc;
    if (int rc = nm::fill_async(F.done, cols, (int32_t)0, s)) return rc;
    {
        int64_t g = nm::ceil_div(cols, kBlock);
        hipLaunchKernelGGL(lu_below_kernel, dim3((unsigned)(g > 65536 ? 65536 : g)), dim3(kBlock), 0, s, cols,
                           Mt_indices, Mt_indptr, F.below);
        NM_LAUNCH_CHECK("lu_below_kernel");
    }
    int64_t grid = nm::ceil_div(cols, kLuWavesPerBlock);
    if (grid > 1024) grid = 1024;
    const int64_t limit = poll_limit > 0 ? poll_limit : kLuSpinLimit;
    const size_t lds = (size_t)kLuWavesPerBlock * kLuCap * ((dt == NM_F32 ? 4 : 8) + 4);
    if (lds > 64 * 1024) {
        const void *fn = dt == NM_F32 ? reinterpret_cast<const void *>(lu_flow_kernel<float>)
                                      : reinterpret_cast<const void *>(lu_flow_kernel<double>);
        NM_HIP_TRY(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    }
    if (dt == NM_F32)
        hipLaunchKernelGGL(lu_flow_kernel<float>, dim3((unsigned)grid), dim3(kLuFlowBlock), lds, s, cols, Mt_indices,
                           Mt_indptr, F.below, (float *)Mt_data, F.done, F.ctl, limit);
    else
        hipLaunchKernelGGL(lu_flow_kernel<double>, dim3((unsigned)grid), dim3(kLuFlowBlock), lds, s, cols, Mt_indices,
                           Mt_indptr, F.below, (double *)Mt_data, F.done, F.ctl, limit);
    NM_LAUNCH_CHECK("lu_flow_kernel");
    int32_t ctl_h[2] = {0, 0};
    if (hipMemcpyAsync(ctl_h, F.ctl, sizeof(ctl_h), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return nm::fail(NM_ERR_HIP, "reading the factorisation status back failed: %s",
                        hipGetErrorString(hipGetLastError()));
    if (ctl_h[1] != 0)
        return nm::fail(NM_ERR_HIP, "a column waited more than %lld polls for one it depends on",
                        (long long)limit);
    return NM_OK;
}
