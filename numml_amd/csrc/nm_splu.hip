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

inline int lu_waves(int64_t rows) { return (int)(rows < kLuWaves ? (rows > 0 ? rows : 1) : kLuWaves); }

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
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
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
                            fresh = stamp[w] != mark;   // columns of a row are distinct: no two lanes share w
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
