// CSR x dense (SpMM) forward and backward for gfx950.
//
// Forward: one wavefront per row of A, lane = output column (a 64-column fp32
// row of B is one 256-byte line, so every gather is a single coalesced
// request).  The wavefront reads 64 (column, value) pairs of the row with one
// coalesced load each and broadcasts them lane by lane; every lane adds its
// column's terms in storage order, the order of the serial CPU loop
// (cpp/sparse_csr_cpu.cpp:586-598), so C matches it bit for bit.
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

// IDX is the structure's index type (int64 for A as delivered, int32 for the
// transposed-structure plan); with PERM the value of entry k is data[perm[k]]
// (A^T shares A's value array through the plan's permutation).
template <typename T, typename IDX, bool PERM>
__global__ __launch_bounds__(kBlock) void spdmm_fwd_kernel(
    int64_t rows, const T *__restrict__ data, const IDX *__restrict__ indices,
    const IDX *__restrict__ indptr, const int32_t *__restrict__ perm, const T *__restrict__ B, int64_t ldb,
    int64_t n, T *__restrict__ C, int64_t ldc) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    for (int64_t row = wave0; row < rows; row += nwaves) {
        const int64_t rb = indptr[row], re = indptr[row + 1];
        for (int64_t c0 = 0; c0 < n; c0 += kWave) {
            const int64_t c = c0 + lane;
            const bool live = c < n;
            const T *__restrict__ Bc = B + (live ? c : 0);
            T acc = 0;
            for (int64_t kb = rb; kb < re; kb += kWave) {
                const int64_t k = kb + lane;
                const int64_t mycol = k < re ? (int64_t)indices[k] : 0;
                const T myval = k < re ? (PERM ? data[perm[k]] : data[k]) : T(0);
                const int cnt = (int)(re - kb < kWave ? re - kb : kWave);
                for (int j = 0; j < cnt; ++j) {
                    const int64_t col = __shfl(mycol, j, kWave);
                    const T v = __shfl(myval, j, kWave);
                    const T bv = live ? Bc[col * ldb] : T(0);
                    acc += v * bv;
                }
            }
            if (live) C[row * ldc + c] = acc;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void spdmm_bwd_kernel(
    int64_t rows, const T *__restrict__ data, const int64_t *__restrict__ indices,
    const int64_t *__restrict__ indptr, const T *__restrict__ B, int64_t ldb,
    const T *__restrict__ gC, int64_t ldg, int64_t n, T *__restrict__ grad_A,
    T *__restrict__ grad_B, int64_t ldgb) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave0 = (int64_t)blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    const int64_t nwaves = (int64_t)gridDim.x * kWavesPerBlock;
    for (int64_t row = wave0; row < rows; row += nwaves) {
        const int64_t rb = indptr[row], re = indptr[row + 1];
        if (rb == re) continue;
        const T *__restrict__ g = gC + row * ldg;
        const T g0 = lane < n ? g[lane] : T(0);  // the whole row of gC when n <= 64
        for (int64_t kb = rb; kb < re; kb += kWave) {
            const int64_t k = kb + lane;
            const int64_t mycol = k < re ? indices[k] : 0;
            const T myval = (grad_B && k < re) ? data[k] : T(0);
            const int cnt = (int)(re - kb < kWave ? re - kb : kWave);
            T mydot = 0;
            for (int j = 0; j < cnt; ++j) {
                const int64_t col = __shfl(mycol, j, kWave);
                const T v = __shfl(myval, j, kWave);
                T part = 0;
                if (n <= kWave) {
                    if (lane < n) {
                        if (grad_A) part = g0 * B[col * ldb + lane];
                        if (grad_B) nm::atomic_add(grad_B + col * ldgb + lane, v * g0);
                    }
                } else {
                    for (int64_t c = lane; c < n; c += kWave) {
                        const T gv = g[c];
                        if (grad_A) part += gv * B[col * ldb + c];
                        if (grad_B) nm::atomic_add(grad_B + col * ldgb + c, v * gv);
                    }
                }
                if (grad_A) {
                    part = nm::wave_sum(part);
                    if (lane == j) mydot = part;
                }
            }
            if (grad_A && k < re) grad_A[k] = mydot;
        }
    }
}

int check_args(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
               const int64_t *indices, const int64_t *indptr, int64_t n) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0 && n >= 0, "negative size");
    NM_REQUIRE(indptr != nullptr, "indptr is null");
    NM_REQUIRE(nnz == 0 || (data != nullptr && indices != nullptr), "data/indices null with nnz > 0");
    return NM_OK;
}

inline unsigned wave_grid(int64_t rows) {
    int64_t grid = nm::ceil_div(rows, kWavesPerBlock);
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
    if (dt == NM_F32)
        hipLaunchKernelGGL((spdmm_fwd_kernel<float, int64_t, false>), dim3(wave_grid(rows)), dim3(kBlock), 0, s,
                           rows, (const float *)data, indices, indptr, nullptr, (const float *)B, ldb, n,
                           (float *)C, ldc);
    else
        hipLaunchKernelGGL((spdmm_fwd_kernel<double, int64_t, false>), dim3(wave_grid(rows)), dim3(kBlock), 0, s,
                           rows, (const double *)data, indices, indptr, nullptr, (const double *)B, ldb, n,
                           (double *)C, ldc);
    NM_LAUNCH_CHECK("spdmm_fwd_kernel");
    return NM_OK;
}

extern "C" int nm_spdmm_backward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                 const int64_t *indices, const int64_t *indptr, const void *B, int64_t ldb,
                                 const void *gC, int64_t ldg, int64_t n, void *grad_A, void *grad_B,
                                 int64_t ldgb, nm_stream stream) {
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
    if (dt == NM_F32)
        hipLaunchKernelGGL(spdmm_bwd_kernel<float>, dim3(wave_grid(rows)), dim3(kBlock), 0, s, rows,
                           (const float *)data, indices, indptr, (const float *)B, ldb, (const float *)gC,
                           ldg, n, (float *)grad_A, (float *)grad_B, ldgb);
    else
        hipLaunchKernelGGL(spdmm_bwd_kernel<double>, dim3(wave_grid(rows)), dim3(kBlock), 0, s, rows,
                           (const double *)data, indices, indptr, (const double *)B, ldb, (const double *)gC,
                           ldg, n, (double *)grad_A, (double *)grad_B, ldgb);
    NM_LAUNCH_CHECK("spdmm_bwd_kernel");
    return NM_OK;
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
    if (grad_A) {
        if (int rc = nm_spdmm_backward(dt, rows, cols, nnz, data, indices, indptr, B, ldb, gC, ldg, n, grad_A,
                                       nullptr, 0, stream))
            return rc;
    }
    if (!grad_B || cols == 0 || n == 0) return NM_OK;
    NM_REQUIRE(ldgb >= n && ldg >= n, "row stride smaller than the row");
    NM_REQUIRE(gC != nullptr || nnz == 0, "gC is null");
    nm::TPlan t;
    nm::tplan_layout(cols, nnz, const_cast<void *>(plan_mem), &t);
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F32)
        hipLaunchKernelGGL((spdmm_fwd_kernel<float, int32_t, true>), dim3(wave_grid(cols)), dim3(kBlock), 0, s, cols,
                           (const float *)data, t.t_row, t.t_indptr, t.t_perm, (const float *)gC, ldg, n,
                           (float *)grad_B, ldgb);
    else
        hipLaunchKernelGGL((spdmm_fwd_kernel<double, int32_t, true>), dim3(wave_grid(cols)), dim3(kBlock), 0, s,
                           cols, (const double *)data, t.t_row, t.t_indptr, t.t_perm, (const double *)gC, ldg, n,
                           (double *)grad_B, ldgb);
    NM_LAUNCH_CHECK("spdmm_fwd_kernel (transposed)");
    return NM_OK;
}
