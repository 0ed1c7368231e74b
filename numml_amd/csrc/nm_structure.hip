// Structure-changing CSR operations next to the products: the explicit
// transpose (csr_transpose_forward / _backward of the reference,
// cpp/sparse_csr_cpu.cpp:311-385).  All of it is streaming integer and copy
// work, bound by HBM bandwidth.
#include "nm_transpose.hpp"

namespace {

constexpr int kBlock = 256;

// Widens a transposed-structure plan to the arrays the reference returns:
// At_indptr, At_indices and At_to_A_idx as int64, At_data gathered through the
// permutation.  Plan arrays and outputs are touched once (streaming accesses);
// the value gather goes through the caches.
template <typename T>
__global__ void transpose_expand_kernel(int64_t nnz, int64_t cols, const T *__restrict__ data,
                                        const int32_t *__restrict__ t_indptr, const int32_t *__restrict__ t_row,
                                        const int32_t *__restrict__ t_perm, T *__restrict__ At_data,
                                        int64_t *__restrict__ At_indices, int64_t *__restrict__ At_indptr,
                                        int64_t *__restrict__ At_to_A) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (int64_t p = tid; p < nnz; p += stride) {
        const int32_t src = nm::stream_load(t_perm + p);
        const int32_t row = nm::stream_load(t_row + p);
        const T v = data[src];
        nm::stream_store(At_to_A + p, (int64_t)src);
        nm::stream_store(At_indices + p, (int64_t)row);
        nm::stream_store(At_data + p, v);
    }
    for (int64_t c = tid; c <= cols; c += stride) At_indptr[c] = (int64_t)t_indptr[c];
}

// grad_A[At_to_A[p]] = grad_At[p]  (cpp/sparse_csr_cpu.cpp:379-381).
template <typename T>
__global__ void transpose_scatter_kernel(int64_t nnz, const T *__restrict__ grad_At,
                                         const int64_t *__restrict__ At_to_A, T *__restrict__ grad_A) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t p = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; p < nnz; p += stride)
        grad_A[nm::stream_load(At_to_A + p)] = nm::stream_load(grad_At + p);
}

inline unsigned grid_for(int64_t n) {
    int64_t g = nm::ceil_div(n > 0 ? n : 1, (int64_t)kBlock * 4);
    if (g > 65536) g = 65536;
    return (unsigned)(g < 1 ? 1 : g);
}

}  // namespace

extern "C" int nm_csr_transpose_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                        const void *plan_mem, void *At_data, int64_t *At_indices,
                                        int64_t *At_indptr, int64_t *At_to_A_idx, nm_stream stream) {
    NM_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0, "negative size");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    NM_REQUIRE(plan_mem && At_indptr, "null pointer argument");
    NM_REQUIRE(nnz == 0 || (data && At_data && At_indices && At_to_A_idx), "null pointer argument");
    nm::TPlan plan;
    nm::tplan_layout(cols, nnz, const_cast<void *>(plan_mem), &plan);
    hipStream_t s = nm::as_stream(stream);
    const unsigned grid = grid_for(nnz > cols + 1 ? nnz : cols + 1);
    if (dt == NM_F32)
        hipLaunchKernelGGL(transpose_expand_kernel<float>, dim3(grid), dim3(kBlock), 0, s, nnz, cols,
                           (const float *)data, plan.t_indptr, plan.t_row, plan.t_perm, (float *)At_data,
                           At_indices, At_indptr, At_to_A_idx);
    else
        hipLaunchKernelGGL(transpose_expand_kernel<double>, dim3(grid), dim3(kBlock), 0, s, nnz, cols,
                           (const double *)data, plan.t_indptr, plan.t_row, plan.t_perm, (double *)At_data,
                           At_indices, At_indptr, At_to_A_idx);
    NM_LAUNCH_CHECK("transpose_expand_kernel");
    return NM_OK;
}

extern "C" int nm_csr_transpose_backward(nm_dtype dt, int64_t nnz, const void *grad_At, const int64_t *At_to_A_idx,
                                         void *grad_A, nm_stream stream) {
    NM_REQUIRE(nnz >= 0, "negative size");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    if (nnz == 0) return NM_OK;
    NM_REQUIRE(grad_At && At_to_A_idx && grad_A, "null pointer argument");
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F32)
        hipLaunchKernelGGL(transpose_scatter_kernel<float>, dim3(grid_for(nnz)), dim3(kBlock), 0, s, nnz,
                           (const float *)grad_At, At_to_A_idx, (float *)grad_A);
    else
        hipLaunchKernelGGL(transpose_scatter_kernel<double>, dim3(grid_for(nnz)), dim3(kBlock), 0, s, nnz,
                           (const double *)grad_At, At_to_A_idx, (double *)grad_A);
    NM_LAUNCH_CHECK("transpose_scatter_kernel");
    return NM_OK;
}
