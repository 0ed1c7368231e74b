// Level-scheduled sparse triangular solve for gfx950.
//
// Analysis (once per sparsity pattern): the strictly-triangular entries of A
// define a dependency DAG.  A Kahn sweep, run by one workgroup, peels the DAG
// level by level and leaves the rows in level order (`order`, `level_ptr`).
// The sweep needs each row's dependents, i.e. A^T, which is built with a stable
// radix sort of the entries by column; the same A^T (indices + permutation
// into A's values) is what the backward solve runs on, so one plan serves both
// x = A^{-1} b and grad_b = A^{-T} g: the transposed solve walks the same
// levels in reverse.
//
// Solve: runs of consecutive narrow levels (<= 1024 rows) are executed by a
// single 1024-lane workgroup that separates levels with workgroup barriers;
// a level wider than that gets a launch of its own across the chip.  Stream
// order is the only synchronisation between launches, so no kernel ever waits
// on another workgroup.  Each row is one lane; sums run in double and in the
// walk direction of the serial CPU loop (cpp/sparse_csr_cpu.cpp:672-718), so
// results match it bit for bit.
//
// Algorithmic HBM bytes of one solve (s = sizeof(value)):
//   nnz*(s+8) + (rows+1)*8 + 2*rows*s   (+ rows*4 for the level order)
#include "nm_common.hpp"
#include "nm_transpose.hpp"

#include <new>
#include <vector>

struct nm_sptrsv_plan {
    int64_t rows = 0, nnz = 0;
    int lower = 1;
    int32_t nlevels = 0;
    // device arrays inside the caller's plan memory
    int32_t *order = nullptr, *level_ptr = nullptr;
    int32_t *t_indptr = nullptr, *t_row = nullptr, *t_perm = nullptr;
    struct Launch {
        int32_t l0, l1;  // levels [l0, l1)
        int32_t q0, q1;  // slots of `order` they cover
        bool wide;       // one level, many workgroups
    };
    std::vector<Launch> launches;
};

namespace {

constexpr int kNarrow = 1024;  // widest level the single-workgroup kernel takes
constexpr int kBlock = 256;

inline size_t align_up(size_t v) { return (v + 255) & ~size_t(255); }

struct Carver {
    char *base;
    size_t off = 0;
    explicit Carver(void *p) : base(static_cast<char *>(p)) {}
    template <typename T> T *take(size_t count) {
        T *p = reinterpret_cast<T *>(base + off);
        off += align_up(count * sizeof(T));
        return p;
    }
};

// plan memory: [transposed-structure plan][order][level_ptr][meta]
size_t plan_layout(int64_t rows, int64_t nnz, void *base, nm::TPlan *t, int32_t **order, int32_t **level_ptr,
                   int32_t **meta) {
    size_t off = nm::tplan_layout(rows, nnz, base, t);
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align_up(bytes);
        return (int32_t *)q;
    };
    int32_t *o = take((size_t)(rows + 1) * 4), *l = take((size_t)(rows + 1) * 4), *m = take(16 * 4);
    if (order) *order = o;
    if (level_ptr) *level_ptr = l;
    if (meta) *meta = m;
    return off;
}

// analysis scratch: [deg][rowid][transpose scratch]
size_t work_bytes_needed(int64_t rows, int64_t nnz) {
    return align_up((size_t)(rows + 1) * 4) + align_up((size_t)(nnz + 1) * 4) +
           nm::tplan_work_bytes(rows, rows, nnz);
}

// ---- analysis kernels ------------------------------------------------------

// In-degree of every row in the dependency DAG: its strictly-triangular entries.
__global__ void indegree_kernel(int64_t nnz, const int64_t *__restrict__ indices,
                                const int32_t *__restrict__ rowid, int lower, int32_t *__restrict__ deg) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nnz; k += stride) {
        const int64_t col = indices[k];
        const int32_t row = rowid[k];
        if (lower ? col < row : col > row) atomicAdd(deg + row, 1);
    }
}

// Kahn's algorithm by one workgroup.  meta[0] = number of levels, meta[1] =
// rows placed (== rows for any input, because only strictly-triangular entries
// count as dependencies and those cannot form a cycle).
__global__ __launch_bounds__(kNarrow) void kahn_kernel(int32_t rows, int lower,
                                                       const int32_t *__restrict__ t_indptr,
                                                       const int32_t *__restrict__ t_row, int32_t *deg,
                                                       int32_t *order, int32_t *level_ptr, int32_t *meta) {
    __shared__ int s_tail;
    if (threadIdx.x == 0) s_tail = 0;
    __syncthreads();
    for (int32_t i = threadIdx.x; i < rows; i += kNarrow)
        if (deg[i] == 0) order[atomicAdd(&s_tail, 1)] = i;
    __syncthreads();
    int head = 0, tail = s_tail, nlev = 0;
    if (threadIdx.x == 0) level_ptr[0] = 0;
    while (head < tail) {
        if (threadIdx.x == 0) level_ptr[nlev + 1] = tail;
        for (int q = head + threadIdx.x; q < tail; q += kNarrow) {
            const int32_t r = order[q];
            const int32_t pe = t_indptr[r + 1];
            for (int32_t p = t_indptr[r]; p < pe; ++p) {
                const int32_t d = t_row[p];
                if (lower ? d > r : d < r)
                    if (atomicSub(deg + d, 1) == 1) order[atomicAdd(&s_tail, 1)] = d;
            }
        }
        __syncthreads();
        head = tail;
        tail = s_tail;
        ++nlev;
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        meta[0] = nlev;
        meta[1] = tail;
    }
}

// ---- solve kernels -----------------------------------------------------------

template <typename T> struct SolveArgs {
    const T *data;
    const int64_t *indices, *indptr;                  // A
    const int32_t *t_indptr, *t_row, *t_perm;         // A^T
    const int32_t *order, *level_ptr;
    const T *b;
    double *xw;
    int unit;
    int ascending;  // 1: lower-triangular walk (ascending), 0: upper (descending)
};

template <typename T, bool TR>
__device__ __forceinline__ void solve_row(const SolveArgs<T> &a, int32_t i) {
    double diag = 0., acc = 0.;
    int64_t kb, ke;
    if (TR) { kb = a.t_indptr[i]; ke = a.t_indptr[i + 1]; }
    else    { kb = a.indptr[i];   ke = a.indptr[i + 1]; }
    if (a.ascending) {
        for (int64_t k = kb; k < ke; ++k) {
            const int64_t j = TR ? (int64_t)a.t_row[k] : a.indices[k];
            if (j > i) continue;
            const double v = (double)(TR ? a.data[a.t_perm[k]] : a.data[k]);
            if (j == i) diag = v; else acc += v * a.xw[j];
        }
    } else {
        for (int64_t k = ke - 1; k >= kb; --k) {
            const int64_t j = TR ? (int64_t)a.t_row[k] : a.indices[k];
            if (j < i) continue;
            const double v = (double)(TR ? a.data[a.t_perm[k]] : a.data[k]);
            if (j == i) diag = v; else acc += v * a.xw[j];
        }
    }
    double xi = (double)a.b[i] - acc;
    if (!a.unit) xi /= diag;
    a.xw[i] = xi;
}

// Levels l0, l0+step, ... (l1 exclusive), each at most kNarrow rows, by one workgroup.
template <typename T, bool TR>
__global__ __launch_bounds__(kNarrow) void sptrsv_batch_kernel(SolveArgs<T> a, int l0, int l1, int step) {
    for (int l = l0; l != l1; l += step) {
        const int q = a.level_ptr[l] + (int)threadIdx.x;
        if (q < a.level_ptr[l + 1]) solve_row<T, TR>(a, a.order[q]);
        __syncthreads();
    }
}

// One wide level: slots [q0, q1) of `order`, one lane per row.
template <typename T, bool TR>
__global__ __launch_bounds__(kBlock) void sptrsv_level_kernel(SolveArgs<T> a, int q0, int q1) {
    const int q = q0 + (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (q < q1) solve_row<T, TR>(a, a.order[q]);
}

__global__ void round_kernel(int64_t n, const double *__restrict__ xw, float *__restrict__ x) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) x[i] = (float)xw[i];
}

template <typename T, bool TR>
int run_solve(const nm_sptrsv_plan *p, SolveArgs<T> a, hipStream_t s) {
    const int n = (int)p->launches.size();
    for (int li = 0; li < n; ++li) {
        const auto &L = p->launches[TR ? n - 1 - li : li];
        if (L.wide) {
            const unsigned grid = (unsigned)nm::ceil_div(L.q1 - L.q0, kBlock);
            hipLaunchKernelGGL((sptrsv_level_kernel<T, TR>), dim3(grid), dim3(kBlock), 0, s, a, L.q0, L.q1);
            NM_LAUNCH_CHECK("sptrsv_level_kernel");
        } else {
            const int l0 = TR ? L.l1 - 1 : L.l0, l1 = TR ? L.l0 - 1 : L.l1, step = TR ? -1 : 1;
            hipLaunchKernelGGL((sptrsv_batch_kernel<T, TR>), dim3(1), dim3(kNarrow), 0, s, a, l0, l1, step);
            NM_LAUNCH_CHECK("sptrsv_batch_kernel");
        }
    }
    return NM_OK;
}

template <typename T>
int solve_typed(const nm_sptrsv_plan *p, int transposed, const void *data, const int64_t *indices,
                const int64_t *indptr, int unit, const void *b, double *xw, hipStream_t s) {
    SolveArgs<T> a;
    a.data = (const T *)data;
    a.indices = indices;
    a.indptr = indptr;
    a.t_indptr = p->t_indptr;
    a.t_row = p->t_row;
    a.t_perm = p->t_perm;
    a.order = p->order;
    a.level_ptr = p->level_ptr;
    a.b = (const T *)b;
    a.xw = xw;
    a.unit = unit;
    a.ascending = transposed ? !p->lower : p->lower;
    return transposed ? run_solve<T, true>(p, a, s) : run_solve<T, false>(p, a, s);
}

}  // namespace

extern "C" int nm_sptrsv_plan_bytes(int64_t rows, int64_t nnz, size_t *plan_bytes, size_t *work_bytes) {
    NM_REQUIRE(rows >= 0 && nnz >= 0 && plan_bytes && work_bytes, "bad arguments");
    if (rows >= (int64_t(1) << 31) - 2 || nnz >= (int64_t(1) << 31) - 2)
        return nm::fail(NM_ERR_UNSUPPORTED, "sptrsv plans index rows and entries with 32 bits");
    *plan_bytes = plan_layout(rows, nnz, nullptr, nullptr, nullptr, nullptr, nullptr);
    *work_bytes = work_bytes_needed(rows, nnz);
    return NM_OK;
}

extern "C" int nm_sptrsv_analyse(int64_t rows, int64_t nnz, const int64_t *indices, const int64_t *indptr,
                                 int lower, void *plan_mem, size_t plan_bytes, void *work, size_t work_bytes,
                                 nm_sptrsv_plan **plan_out, nm_stream stream) {
    NM_REQUIRE(plan_out != nullptr, "plan_out is null");
    *plan_out = nullptr;
    size_t need_plan = 0, need_work = 0;
    if (int rc = nm_sptrsv_plan_bytes(rows, nnz, &need_plan, &need_work)) return rc;
    NM_REQUIRE(indptr != nullptr && (nnz == 0 || indices != nullptr), "null structure pointer");
    NM_REQUIRE(plan_mem != nullptr && work != nullptr, "null plan memory or workspace");
    if (plan_bytes < need_plan || work_bytes < need_work)
        return nm::fail(NM_ERR_WORKSPACE, "plan memory %zu/%zu or workspace %zu/%zu too small", plan_bytes,
                        need_plan, work_bytes, need_work);
    hipStream_t s = nm::as_stream(stream);

    nm_sptrsv_plan *p = new (std::nothrow) nm_sptrsv_plan();
    NM_REQUIRE(p != nullptr, "out of host memory");
    p->rows = rows;
    p->nnz = nnz;
    p->lower = lower ? 1 : 0;
    nm::TPlan t;
    int32_t *meta = nullptr;
    plan_layout(rows, nnz, plan_mem, &t, &p->order, &p->level_ptr, &meta);
    p->t_indptr = t.t_indptr;
    p->t_row = t.t_row;
    p->t_perm = t.t_perm;

    auto bail = [&](int rc) { delete p; return rc; };
    if (rows == 0) { *plan_out = p; return NM_OK; }

    char *wbase = static_cast<char *>(work);
    int32_t *deg = reinterpret_cast<int32_t *>(wbase);
    int32_t *rowid = reinterpret_cast<int32_t *>(wbase + align_up((size_t)(rows + 1) * 4));
    char *twork = wbase + align_up((size_t)(rows + 1) * 4) + align_up((size_t)(nnz + 1) * 4);
    const size_t twork_bytes = nm::tplan_work_bytes(rows, rows, nnz);

    if (int rc = nm::tplan_build(rows, rows, nnz, indices, indptr, t, twork, twork_bytes, rowid, s)) return bail(rc);
    if (int rc = nm::fill_async(deg, rows + 1, (int32_t)0, s)) return bail(rc);
    if (nnz > 0) {
        int64_t grid = nm::ceil_div(nnz, kBlock);
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(indegree_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, nnz, indices, rowid,
                           p->lower, deg);
        if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "indegree_kernel launch failed"));
    }
    hipLaunchKernelGGL(kahn_kernel, dim3(1), dim3(kNarrow), 0, s, (int32_t)rows, p->lower, p->t_indptr, p->t_row,
                       deg, p->order, p->level_ptr, meta);
    if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "kahn_kernel launch failed"));

    int32_t meta_h[2] = {0, 0};
    if (hipMemcpyAsync(meta_h, meta, sizeof(meta_h), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return bail(nm::fail(NM_ERR_HIP, "reading the level count back failed: %s",
                             hipGetErrorString(hipGetLastError())));
    if (meta_h[1] != (int32_t)rows)
        return bail(nm::fail(NM_ERR_INVALID, "level analysis placed %d of %lld rows", meta_h[1], (long long)rows));
    p->nlevels = meta_h[0];
    std::vector<int32_t> lp((size_t)p->nlevels + 1);
    if (hipMemcpyAsync(lp.data(), p->level_ptr, lp.size() * 4, hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return bail(nm::fail(NM_ERR_HIP, "reading the level sizes back failed"));

    // consecutive narrow levels share one single-workgroup launch
    int32_t run0 = -1;
    for (int32_t l = 0; l < p->nlevels; ++l) {
        const bool wide = lp[l + 1] - lp[l] > kNarrow;
        if (!wide) {
            if (run0 < 0) run0 = l;
            continue;
        }
        if (run0 >= 0) { p->launches.push_back({run0, l, lp[run0], lp[l], false}); run0 = -1; }
        p->launches.push_back({l, l + 1, lp[l], lp[l + 1], true});
    }
    if (run0 >= 0) p->launches.push_back({run0, p->nlevels, lp[run0], lp[p->nlevels], false});
    *plan_out = p;
    return NM_OK;
}

extern "C" int64_t nm_sptrsv_plan_levels(const nm_sptrsv_plan *plan) { return plan ? plan->nlevels : -1; }

extern "C" int64_t nm_sptrsv_plan_launches(const nm_sptrsv_plan *plan) {
    return plan ? (int64_t)plan->launches.size() : -1;
}

extern "C" void nm_sptrsv_plan_destroy(nm_sptrsv_plan *plan) { delete plan; }

extern "C" int nm_sptrsv_solve(const nm_sptrsv_plan *plan, nm_dtype dt, int transposed, const void *data,
                               const int64_t *indices, const int64_t *indptr, int unit, const void *b, void *x,
                               double *xwork, nm_stream stream) {
    NM_REQUIRE(plan != nullptr, "plan is null");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (plan->rows == 0) return NM_OK;
    NM_REQUIRE(indptr && b && x && (plan->nnz == 0 || (data && indices)), "null pointer argument");
    NM_REQUIRE(dt == NM_F64 || xwork != nullptr, "xwork is required for NM_F32");
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F64)  // x itself holds the running solution
        return solve_typed<double>(plan, transposed, data, indices, indptr, unit, b, (double *)x, s);
    if (int rc = solve_typed<float>(plan, transposed, data, indices, indptr, unit, b, xwork, s)) return rc;
    int64_t grid = nm::ceil_div(plan->rows, kBlock);
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(round_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, plan->rows, xwork, (float *)x);
    NM_LAUNCH_CHECK("round_kernel");
    return NM_OK;
}
