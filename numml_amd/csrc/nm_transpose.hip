// Builder of the transposed-structure plan (see nm_transpose.hpp) and its C ABI.
#include "nm_transpose.hpp"

#include <rocprim/device/device_radix_sort.hpp>

namespace {

constexpr int kBlock = 256;

inline int bits_for(int64_t n) {
    int b = 1;
    while (b < 32 && (int64_t(1) << b) < n) ++b;
    return b;
}

size_t sort_temp_bytes(int64_t nnz, int bits) {
    size_t bytes = 0;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, (int32_t *)nullptr, (int32_t *)nullptr,
                                    (int32_t *)nullptr, (int32_t *)nullptr, (size_t)(nnz > 0 ? nnz : 1), 0u,
                                    (unsigned)bits, (hipStream_t)0);
    return bytes;
}

// Per stored entry: sort key (column), payload (its own position) and its row,
// found by bisection of indptr so that rows of any length cost the same.
__global__ void entry_keys_kernel(int64_t nnz, int64_t rows, const int64_t *__restrict__ indices,
                                  const int64_t *__restrict__ indptr, int32_t *__restrict__ keys,
                                  int32_t *__restrict__ vals, int32_t *__restrict__ rowid) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t k = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; k < nnz; k += stride) {
        int64_t lo = 0, hi = rows + 1;  // first p with indptr[p] > k
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (indptr[mid] <= k) lo = mid + 1; else hi = mid;
        }
        keys[k] = (int32_t)indices[k];
        vals[k] = (int32_t)k;
        rowid[k] = (int32_t)(lo - 1);
    }
}

__global__ void finish_kernel(int64_t nnz, int64_t cols, const int32_t *__restrict__ keys_sorted,
                              const int32_t *__restrict__ t_perm, const int32_t *__restrict__ rowid,
                              int32_t *__restrict__ t_row, int32_t *__restrict__ t_indptr,
                              int32_t *__restrict__ chunk_row) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (int64_t p = tid; p < nnz; p += stride) t_row[p] = rowid[t_perm[p]];
    for (int64_t h = tid; h * 64 < nnz; h += stride) chunk_row[h] = rowid[h * 64];
    for (int64_t c = tid; c <= cols; c += stride) {
        int64_t lo = 0, hi = nnz;  // first sorted position whose column is >= c
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (keys_sorted[mid] < c) lo = mid + 1; else hi = mid;
        }
        t_indptr[c] = (int32_t)lo;
    }
}

__global__ void symmetry_init_kernel(int32_t *flags, int square) {
    if (threadIdx.x == 0) flags[0] = square;
}

// Clears flags[0] unless A^T has exactly A's structure.
__global__ void symmetry_check_kernel(int64_t nnz, int64_t cols, const int64_t *__restrict__ indices,
                                      const int64_t *__restrict__ indptr, const int32_t *__restrict__ t_row,
                                      const int32_t *__restrict__ t_indptr, int32_t *flags) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    bool same = true;
    for (int64_t p = tid; p < nnz; p += stride) same &= (int64_t)t_row[p] == indices[p];
    for (int64_t c = tid; c <= cols; c += stride) same &= (int64_t)t_indptr[c] == indptr[c];
    if (!same) flags[0] = 0;
}

struct WorkT {
    int32_t *keys, *keys_sorted, *vals, *rowid;
    void *temp;
    size_t temp_bytes;
};

size_t work_layout(int64_t cols, int64_t nnz, void *base, WorkT *w) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += nm::align256(bytes);
        return q;
    };
    WorkT t;
    t.keys = (int32_t *)take((size_t)(nnz + 1) * 4);
    t.keys_sorted = (int32_t *)take((size_t)(nnz + 1) * 4);
    t.vals = (int32_t *)take((size_t)(nnz + 1) * 4);
    t.rowid = (int32_t *)take((size_t)(nnz + 1) * 4);
    t.temp_bytes = sort_temp_bytes(nnz, bits_for(cols));
    t.temp = take(t.temp_bytes + 256);
    if (w) *w = t;
    return off;
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
    if (nnz > 0) {
        int64_t grid = ceil_div(nnz, kBlock);
        if (grid > 65536) grid = 65536;
        hipLaunchKernelGGL(entry_keys_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, nnz, rows, indices,
                           indptr, w.keys, w.vals, rowid);
        NM_LAUNCH_CHECK("entry_keys_kernel");
        size_t tb = w.temp_bytes;
        hipError_t e = rocprim::radix_sort_pairs(w.temp, tb, w.keys, w.keys_sorted, w.vals, plan.t_perm,
                                                 (size_t)nnz, 0u, (unsigned)bits_for(cols), s);
        if (e != hipSuccess) return fail(NM_ERR_HIP, "radix sort failed: %s", hipGetErrorString(e));
    }
    int64_t m = nnz > cols + 1 ? nnz : cols + 1;
    int64_t grid = ceil_div(m, kBlock);
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(finish_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, nnz, cols, w.keys_sorted,
                       plan.t_perm, rowid, plan.t_row, plan.t_indptr, plan.chunk_row);
    NM_LAUNCH_CHECK("transpose finish_kernel");
    hipLaunchKernelGGL(symmetry_init_kernel, dim3(1), dim3(64), 0, s, plan.flags, rows == cols ? 1 : 0);
    if (rows == cols) {
        hipLaunchKernelGGL(symmetry_check_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, nnz, cols, indices,
                           indptr, plan.t_row, plan.t_indptr, plan.flags);
    }
    NM_LAUNCH_CHECK("symmetry check");
    return NM_OK;
}

}  // namespace nm

extern "C" int nm_csr_transpose_plan_bytes(int64_t rows, int64_t cols, int64_t nnz, size_t *plan_bytes,
                                           size_t *work_bytes) {
    NM_REQUIRE(plan_bytes && work_bytes, "null size pointer");
    if (int rc = check_sizes(rows, cols, nnz)) return rc;
    *plan_bytes = nm::tplan_layout(cols, nnz, nullptr, nullptr);
    *work_bytes = nm::tplan_work_bytes(rows, cols, nnz);
    return NM_OK;
}

extern "C" int nm_csr_transpose_plan_build(int64_t rows, int64_t cols, int64_t nnz, const int64_t *indices,
                                           const int64_t *indptr, void *plan_mem, size_t plan_bytes, void *work,
                                           size_t work_bytes, nm_stream stream) {
    if (int rc = check_sizes(rows, cols, nnz)) return rc;
    NM_REQUIRE(indptr && plan_mem && work && (nnz == 0 || indices), "null pointer argument");
    nm::TPlan plan;
    const size_t need = nm::tplan_layout(cols, nnz, plan_mem, &plan);
    if (plan_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "plan memory of %zu bytes, %zu needed", plan_bytes, need);
    return nm::tplan_build(rows, cols, nnz, indices, indptr, plan, work, work_bytes, nullptr,
                           nm::as_stream(stream));
}
