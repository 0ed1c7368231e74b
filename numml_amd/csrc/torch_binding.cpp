// numml_torch_cpp: the reference's extension module, re-implemented on the
// C ABI of libnumml_hip.so.
//
// Exports the eight hot-path functions that cpp/sparse_csr.cpp:307-319 binds
// (spgemv / spdmm / spgemm / sptrsv, _forward and _backward) with the argument
// lists of cpp/sparse_csr.hpp:32-105, so `import numml_torch_cpp` in the
// reference's Python layer (numml/sparse/_csr.py:2, numml/sparse/linalg.py:2)
// resolves to HIP kernels for this path.  torch is used for device memory
// (outputs and scratch come from its caching allocator) and for the current
// stream; all arithmetic happens behind numml_hip.h.
//
// There is no CPU implementation here: tensors that are not on a HIP device
// raise, as does any nm_status other than NM_OK.
//
// Host-only translation unit (compiled with g++); it needs no device code.
#include <torch/extension.h>

#include <ATen/hip/HIPContext.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <atomic>
#include <cstdlib>
#include <list>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "numml_hip.h"

namespace {

using torch::Tensor;

nm_dtype dtype_of(const Tensor &t) {
    if (t.scalar_type() == torch::kFloat32) return NM_F32;
    if (t.scalar_type() == torch::kFloat64) return NM_F64;
    // the reference dispatches with AT_DISPATCH_FLOATING_TYPES (cpp/sparse_csr_cpu.cpp:22)
    TORCH_CHECK(false, "numml_amd: values must be float32 or float64, got ", t.scalar_type());
}

void check(int status, const char *what) {
    TORCH_CHECK(status == NM_OK, what, " failed with status ", status, ": ", nm_last_error());
}

c10::Device need_device(std::initializer_list<const Tensor *> ts) {
    const c10::Device dev = (*ts.begin())->device();
    TORCH_CHECK(dev.is_cuda(), "numml_amd: this backend runs on HIP devices only; got a tensor on '", dev,
                "' (no CPU implementation is provided)");
    for (const Tensor *t : ts)
        TORCH_CHECK(t->device() == dev, "expected all tensors to be on the same device, but got ", dev, " and ",
                    t->device());
    return dev;
}

Tensor index_tensor(const Tensor &t, const char *name) {
    // the reference reads structure through accessor<int64_t, 1> (cpp/sparse_csr_cpu.cpp:24-25)
    TORCH_CHECK(t.scalar_type() == torch::kInt64, "expected scalar type Long for ", name, " but found ",
                t.scalar_type());
    return t.contiguous();
}

void same_dtype(const Tensor &a, const Tensor &b, const char *what) {
    TORCH_CHECK(a.scalar_type() == b.scalar_type(), "expected ", what, " of type ", a.scalar_type(),
                " but found ", b.scalar_type());
}

nm_stream current_stream(const c10::Device &dev) {
    return reinterpret_cast<nm_stream>(c10::hip::getCurrentHIPStream(dev.index()).stream());
}

// 2-D tensor with unit column stride (copied only when it is not already); returns its row stride.
Tensor row_major(const Tensor &M, int64_t *ld) {
    TORCH_CHECK(M.dim() == 2, "expected a 2-D tensor, got ", M.dim(), "-D");
    Tensor R = M;
    if (R.size(1) > 1 && R.stride(1) != 1) R = R.contiguous();
    if (R.size(0) > 1 && R.stride(0) < std::max<int64_t>(R.size(1), 1)) R = R.contiguous();
    *ld = R.size(0) > 1 ? R.stride(0) : std::max<int64_t>(R.size(1), 1);
    return R;
}

Tensor scratch(size_t bytes, const c10::Device &dev) {
    return torch::empty({(int64_t)std::max<size_t>(bytes, 8)},
                        torch::TensorOptions().dtype(torch::kUInt8).device(dev));
}

// ---- argument shapes ------------------------------------------------------------
//
// Host-side checks of everything a kernel would index with: they look at tensor
// metadata only and run before anything is launched (a wrong length would otherwise
// become an out-of-bounds access on the device).  The reference's accessors do not
// check these either; its CPU loops merely fail more benignly.

void check_csr(const char *who, int64_t rows, int64_t cols, const Tensor &data, const Tensor &indices,
               const Tensor &indptr) {
    TORCH_CHECK(rows >= 0 && cols >= 0, who, ": negative shape ", rows, " x ", cols);
    TORCH_CHECK(indptr.dim() == 1 && indptr.numel() == rows + 1, who, ": expected ", rows + 1,
                " row pointers for ", rows, " rows, got a tensor of shape ", indptr.sizes());
    TORCH_CHECK(data.dim() == 1 && indices.dim() == 1 && data.numel() == indices.numel(), who,
                ": values and column indices must be 1-D and of equal length, got ", data.sizes(), " and ",
                indices.sizes());
}

void check_vector(const char *who, const char *name, const Tensor &t, int64_t n) {
    TORCH_CHECK(t.dim() == 1 && t.numel() == n, who, ": expected ", name, " with ", n, " entries, got shape ",
                t.sizes());
}

void check_matrix(const char *who, const char *name, const Tensor &t, int64_t rows, int64_t cols) {
    TORCH_CHECK(t.dim() == 2 && t.size(0) == rows && (cols < 0 || t.size(1) == cols), who, ": expected ", name,
                " of shape ", rows, " x ", cols < 0 ? std::string("n") : std::to_string(cols), ", got ",
                t.sizes());
}

// 24 bytes of pinned host memory per host thread (from torch's pinned-memory allocator, which
// also takes it back): where nm_spgemm_symbolic_result has the device drop nnz(C).
void *host_landing() {
    thread_local Tensor landing =
        torch::zeros({3}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
    return landing.data_ptr();
}

// "planned" (default): backward passes walk A by column on a cached transposed
// structure (deterministic, no atomics); "atomic": stateless scatter with atomics.
// NUMML_AMD_BACKWARD sets the initial value, set_backward_mode() changes it.
std::atomic<bool> g_planned{[] {
    const char *e = std::getenv("NUMML_AMD_BACKWARD");
    return !(e && std::string(e) == "atomic");
}()};

bool planned_backward() { return g_planned.load(std::memory_order_relaxed); }

// ---- structure plans -----------------------------------------------------------
//
// Everything derived from a sparsity pattern alone is computed once and cached,
// keyed on the storage and version counters of the structure tensors.  A plan
// keeps those tensors alive, so an address cannot be reused by another pattern
// while the plan is cached; in-place edits bump the version and miss the cache.

struct Plan {
    char kind;  // 'T' transposed structure, 'L' level schedule, 'U' filled pattern of the LU factors
    int device;
    const void *idx_ptr, *ptr_ptr;
    uint32_t idx_version, ptr_version;
    int64_t nnz, nptr, a, b;
    Tensor indices, indptr, mem;
    std::vector<Tensor> derived;             // 'U': structure tensors handed out to callers
    std::vector<uint32_t> derived_versions;  //      and their version counters when built
    nm_sptrsv_plan *handle = nullptr;
    ~Plan() {
        if (handle) nm_sptrsv_plan_destroy(handle);
    }
};

constexpr size_t kPlanCacheSize = 16;
std::mutex g_plans_mutex;
std::list<std::shared_ptr<Plan>> g_plans;  // most recently used first

template <typename Make>
std::shared_ptr<Plan> cached(char kind, const Tensor &indices, const Tensor &indptr, int64_t a, int64_t b,
                             Make make) {
    const int device = indices.device().index();
    const uint32_t vi = indices._version(), vp = indptr._version();
    {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        for (auto it = g_plans.begin(); it != g_plans.end(); ++it) {
            Plan &p = **it;
            if (p.kind == kind && p.device == device && p.idx_ptr == indices.data_ptr() &&
                p.ptr_ptr == indptr.data_ptr() && p.idx_version == vi && p.ptr_version == vp &&
                p.nnz == indices.numel() && p.nptr == indptr.numel() && p.a == a && p.b == b) {
                auto hit = *it;
                g_plans.erase(it);
                g_plans.push_front(hit);
                return hit;
            }
        }
    }
    auto plan = std::make_shared<Plan>();
    plan->kind = kind;
    plan->device = device;
    plan->idx_ptr = indices.data_ptr();
    plan->ptr_ptr = indptr.data_ptr();
    plan->idx_version = vi;
    plan->ptr_version = vp;
    plan->nnz = indices.numel();
    plan->nptr = indptr.numel();
    plan->a = a;
    plan->b = b;
    plan->indices = indices;
    plan->indptr = indptr;
    make(*plan);
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans.push_front(plan);
    while (g_plans.size() > kPlanCacheSize) g_plans.pop_back();
    return plan;
}

std::shared_ptr<Plan> transpose_plan(const Tensor &indices, const Tensor &indptr, int64_t rows, int64_t cols,
                                     const c10::Device &dev) {
    return cached('T', indices, indptr, rows, cols, [&](Plan &p) {
        size_t pbytes = 0, wbytes = 0;
        check(nm_csr_transpose_plan_bytes(rows, cols, p.nnz, &pbytes, &wbytes), "nm_csr_transpose_plan_bytes");
        p.mem = scratch(pbytes, dev);
        Tensor work = scratch(wbytes, dev);
        auto stream = c10::hip::getCurrentHIPStream(dev.index());
        check(nm_csr_transpose_plan_build(rows, cols, p.nnz, indices.data_ptr<int64_t>(),
                                          indptr.data_ptr<int64_t>(), p.mem.data_ptr(), pbytes, work.data_ptr(),
                                          wbytes, reinterpret_cast<nm_stream>(stream.stream())),
              "nm_csr_transpose_plan_build");
        // one-time: the plan is complete for every stream once this returns
        stream.synchronize();
    });
}

std::shared_ptr<Plan> level_plan(const Tensor &indices, const Tensor &indptr, int64_t rows, bool lower,
                                 const c10::Device &dev) {
    return cached('L', indices, indptr, rows, lower ? 1 : 0, [&](Plan &p) {
        size_t pbytes = 0, wbytes = 0;
        check(nm_sptrsv_plan_bytes(rows, p.nnz, &pbytes, &wbytes), "nm_sptrsv_plan_bytes");
        p.mem = scratch(pbytes, dev);
        Tensor work = scratch(wbytes, dev);
        check(nm_sptrsv_analyse(rows, p.nnz, indices.data_ptr<int64_t>(), indptr.data_ptr<int64_t>(),
                                lower ? 1 : 0, p.mem.data_ptr(), pbytes, work.data_ptr(), wbytes, &p.handle,
                                current_stream(dev)),
              "nm_sptrsv_analyse");  // synchronises its stream
    });
}

Tensor solve(const Plan &plan, bool transposed, const Tensor &A_data, bool unit, const Tensor &b, int64_t rows,
             const c10::Device &dev) {
    Tensor x = torch::empty({rows}, A_data.options());
    size_t bytes = 0;
    check(nm_sptrsv_solve_bytes(rows, A_data.numel(), &bytes), "nm_sptrsv_solve_bytes");
    Tensor work = scratch(bytes, dev);
    check(nm_sptrsv_solve(plan.handle, dtype_of(A_data), transposed ? 1 : 0, A_data.data_ptr(), unit ? 1 : 0,
                          b.data_ptr(), x.data_ptr(), work.data_ptr(), bytes, current_stream(dev)),
          "nm_sptrsv_solve");
    return x;
}

// The exported functions below stay inside this unnamed namespace: they have the
// same names and signatures as the reference's (cpp/sparse_csr.hpp:32-105), and
// with external linkage a process that also loads the reference's extension could
// bind one module's Python entries to the other module's functions.

// ---------------------------------------------------------------------------- SpMV

Tensor spgemv_forward(int A_rows, int A_cols, Tensor A_data, Tensor A_col_ind, Tensor A_rowptr, Tensor x) {
    check_csr("spgemv_forward", A_rows, A_cols, A_data, A_col_ind, A_rowptr);
    check_vector("spgemv_forward", "x", x, A_cols);
    const auto dev = need_device({&A_data, &A_col_ind, &A_rowptr, &x});
    same_dtype(A_data, x, "x");
    TORCH_CHECK(x.dim() == 1, "expected 1-D x, got ", x.dim(), "-D");
    A_data = A_data.contiguous();
    x = x.contiguous();
    A_col_ind = index_tensor(A_col_ind, "A_col_ind");
    A_rowptr = index_tensor(A_rowptr, "A_rowptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor y = torch::empty({A_rows}, A_data.options());
    check(nm_spgemv_forward(dtype_of(A_data), A_rows, x.size(0), A_data.numel(), A_data.data_ptr(),
                            A_col_ind.data_ptr<int64_t>(), A_rowptr.data_ptr<int64_t>(), x.data_ptr(),
                            y.data_ptr(), current_stream(dev)),
          "nm_spgemv_forward");
    return y;
}

std::vector<Tensor> spgemv_backward(Tensor grad_z, int A_rows, int A_cols, Tensor A_data, Tensor A_col_ind,
                                    Tensor A_rowptr, Tensor x) {
    check_csr("spgemv_backward", A_rows, A_cols, A_data, A_col_ind, A_rowptr);
    check_vector("spgemv_backward", "x", x, A_cols);
    check_vector("spgemv_backward", "grad_z", grad_z, A_rows);
    const auto dev = need_device({&grad_z, &A_data, &A_col_ind, &A_rowptr, &x});
    same_dtype(A_data, x, "x");
    same_dtype(A_data, grad_z, "grad_z");
    A_data = A_data.contiguous();
    x = x.contiguous();
    grad_z = grad_z.contiguous();
    A_col_ind = index_tensor(A_col_ind, "A_col_ind");
    A_rowptr = index_tensor(A_rowptr, "A_rowptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty_like(A_data), grad_x = torch::empty_like(x);
    if (planned_backward()) {
        auto plan = transpose_plan(A_col_ind, A_rowptr, A_rows, x.size(0), dev);
        check(nm_spgemv_backward_planned(dtype_of(A_data), A_rows, x.size(0), A_data.numel(), A_data.data_ptr(),
                                         plan->mem.data_ptr(), x.data_ptr(), grad_z.data_ptr(),
                                         grad_A.data_ptr(), grad_x.data_ptr(), current_stream(dev)),
              "nm_spgemv_backward_planned");
    } else {
        check(nm_spgemv_backward(dtype_of(A_data), A_rows, x.size(0), A_data.numel(), A_data.data_ptr(),
                                 A_col_ind.data_ptr<int64_t>(), A_rowptr.data_ptr<int64_t>(), x.data_ptr(),
                                 grad_z.data_ptr(), grad_A.data_ptr(), grad_x.data_ptr(), current_stream(dev)),
              "nm_spgemv_backward");
    }
    return {grad_A, grad_x};
}

// ----------------------------------------------------------------------- transpose

std::vector<Tensor> csr_transpose_forward(int A_rows, int A_columns, Tensor A_data, Tensor A_indices,
                                          Tensor A_indptr) {
    check_csr("csr_transpose_forward", A_rows, A_columns, A_data, A_indices, A_indptr);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr});
    A_data = A_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    const int64_t nnz = A_data.numel();
    auto plan = transpose_plan(A_indices, A_indptr, A_rows, A_columns, dev);
    const auto iopt = torch::TensorOptions().dtype(torch::kInt64).device(dev);
    Tensor At_data = torch::empty_like(A_data);
    Tensor At_indices = torch::empty({nnz}, iopt);
    Tensor At_indptr = torch::empty({(int64_t)A_columns + 1}, iopt);
    Tensor At_to_A = torch::empty({nnz}, iopt);
    check(nm_csr_transpose_forward(dtype_of(A_data), A_rows, A_columns, nnz, A_data.data_ptr(),
                                   plan->mem.data_ptr(), At_data.data_ptr(), At_indices.data_ptr<int64_t>(),
                                   At_indptr.data_ptr<int64_t>(), At_to_A.data_ptr<int64_t>(),
                                   current_stream(dev)),
          "nm_csr_transpose_forward");
    return {At_data, At_indices, At_indptr, At_to_A};
}

Tensor csr_transpose_backward(Tensor grad_At, Tensor At_to_A_idx) {
    check_vector("csr_transpose_backward", "At_to_A_idx", At_to_A_idx, grad_At.numel());
    TORCH_CHECK(grad_At.dim() == 1, "csr_transpose_backward: expected 1-D grad_At, got shape ", grad_At.sizes());
    const auto dev = need_device({&grad_At, &At_to_A_idx});
    grad_At = grad_At.contiguous();
    At_to_A_idx = index_tensor(At_to_A_idx, "At_to_A_idx");
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty_like(grad_At);
    check(nm_csr_transpose_backward(dtype_of(grad_At), grad_At.numel(), grad_At.data_ptr(),
                                    At_to_A_idx.data_ptr<int64_t>(), grad_A.data_ptr(), current_stream(dev)),
          "nm_csr_transpose_backward");
    return grad_A;
}

// ------------------------------------------------------------- linear combination

std::vector<Tensor> splincomb_forward(int rows, int cols, Tensor alpha, Tensor A_data, Tensor A_indices,
                                      Tensor A_indptr, Tensor beta, Tensor B_data, Tensor B_indices,
                                      Tensor B_indptr) {
    check_csr("splincomb_forward", rows, cols, A_data, A_indices, A_indptr);
    check_csr("splincomb_forward", rows, cols, B_data, B_indices, B_indptr);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr, &B_data, &B_indices, &B_indptr});
    same_dtype(A_data, B_data, "B_data");
    A_data = A_data.contiguous();
    B_data = B_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    B_indices = index_tensor(B_indices, "B_indices");
    B_indptr = index_tensor(B_indptr, "B_indptr");
    // the reference reads both scalars on the host as well (alpha.item<scalar_t>(),
    // cpp/sparse_csr_cpu.cpp:413-414); they usually are host tensors already
    const double a = alpha.item<double>(), b = beta.item<double>();
    c10::hip::HIPGuard guard(dev.index());
    size_t bytes = 0;
    check(nm_splincomb_workspace_bytes(rows, &bytes), "nm_splincomb_workspace_bytes");
    Tensor work = scratch(bytes, dev);
    const auto iopt = torch::TensorOptions().dtype(torch::kInt64).device(dev);
    Tensor C_indptr = torch::empty({(int64_t)rows + 1}, iopt);
    nm_stream st = current_stream(dev);
    check(nm_splincomb_symbolic(rows, A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(),
                                C_indptr.data_ptr<int64_t>(), work.data_ptr(), bytes, st),
          "nm_splincomb_symbolic");
    const int64_t nnz_c = C_indptr[rows].item<int64_t>();   // C is returned exactly sized
    Tensor C_indices = torch::empty({nnz_c}, iopt);
    Tensor C_data = torch::empty({nnz_c}, A_data.options());
    check(nm_splincomb_numeric(dtype_of(A_data), rows, a, A_data.data_ptr(), A_indices.data_ptr<int64_t>(),
                               A_indptr.data_ptr<int64_t>(), b, B_data.data_ptr(), B_indices.data_ptr<int64_t>(),
                               B_indptr.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(),
                               C_indices.data_ptr<int64_t>(), C_data.data_ptr(), st),
          "nm_splincomb_numeric");
    return {C_data, C_indices, C_indptr};
}

std::vector<Tensor> splincomb_backward(int rows, int cols, Tensor alpha, Tensor A_data, Tensor A_indices,
                                       Tensor A_indptr, Tensor beta, Tensor B_data, Tensor B_indices,
                                       Tensor B_indptr, Tensor grad_C_data, Tensor C_indices, Tensor C_indptr) {
    check_csr("splincomb_backward", rows, cols, A_data, A_indices, A_indptr);
    check_csr("splincomb_backward", rows, cols, B_data, B_indices, B_indptr);
    check_csr("splincomb_backward", rows, cols, grad_C_data, C_indices, C_indptr);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr, &B_data, &B_indices, &B_indptr, &grad_C_data,
                                  &C_indices, &C_indptr});
    same_dtype(A_data, B_data, "B_data");
    same_dtype(A_data, grad_C_data, "grad_C_data");
    grad_C_data = grad_C_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    B_indices = index_tensor(B_indices, "B_indices");
    B_indptr = index_tensor(B_indptr, "B_indptr");
    C_indices = index_tensor(C_indices, "C_indices");
    C_indptr = index_tensor(C_indptr, "C_indptr");
    const double a = alpha.item<double>(), b = beta.item<double>();
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty_like(A_data, at::MemoryFormat::Contiguous);
    Tensor grad_B = torch::empty_like(B_data, at::MemoryFormat::Contiguous);
    check(nm_splincomb_backward(dtype_of(A_data), rows, a, A_indices.data_ptr<int64_t>(),
                                A_indptr.data_ptr<int64_t>(), b, B_indices.data_ptr<int64_t>(),
                                B_indptr.data_ptr<int64_t>(), grad_C_data.data_ptr(), C_indices.data_ptr<int64_t>(),
                                C_indptr.data_ptr<int64_t>(), grad_A.data_ptr(), grad_B.data_ptr(),
                                current_stream(dev)),
          "nm_splincomb_backward");
    return {grad_A, grad_B};
}

// ------------------------------------------------- dense copy, row sums, diagonal

Tensor csr_to_dense_forward(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr) {
    check_csr("csr_to_dense_forward", A_rows, A_cols, A_data, A_indices, A_indptr);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr});
    A_data = A_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor A_d = torch::empty({A_rows, A_cols}, A_data.options());
    check(nm_csr_to_dense_forward(dtype_of(A_data), A_rows, A_cols, A_data.numel(), A_data.data_ptr(),
                                  A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), A_d.data_ptr(),
                                  A_cols, current_stream(dev)),
          "nm_csr_to_dense_forward");
    return A_d;
}

Tensor csr_to_dense_backward(Tensor grad_Ad, int A_rows, int A_cols, Tensor A_data, Tensor A_indices,
                             Tensor A_indptr) {
    check_csr("csr_to_dense_backward", A_rows, A_cols, A_data, A_indices, A_indptr);
    const auto dev = need_device({&grad_Ad, &A_data, &A_indices, &A_indptr});
    same_dtype(A_data, grad_Ad, "grad_Ad");
    TORCH_CHECK(grad_Ad.dim() == 2 && grad_Ad.size(0) == A_rows && grad_Ad.size(1) == A_cols,
                "expected a ", A_rows, " x ", A_cols, " gradient, got ", grad_Ad.sizes());
    int64_t ld = 1;
    grad_Ad = row_major(grad_Ad, &ld);
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty({A_data.numel()}, A_data.options());
    check(nm_csr_to_dense_backward(dtype_of(A_data), A_rows, A_cols, A_data.numel(), grad_Ad.data_ptr(),
                                   std::max<int64_t>(ld, A_cols), A_indices.data_ptr<int64_t>(),
                                   A_indptr.data_ptr<int64_t>(), grad_A.data_ptr(), current_stream(dev)),
          "nm_csr_to_dense_backward");
    return grad_A;
}

Tensor csr_row_sum_forward(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr) {
    check_csr("csr_row_sum_forward", A_rows, A_cols, A_data, A_indices, A_indptr);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr});
    A_data = A_data.contiguous();
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor x = torch::empty({A_rows}, A_data.options());
    check(nm_csr_row_sum_forward(dtype_of(A_data), A_rows, A_data.numel(), A_data.data_ptr(),
                                 A_indptr.data_ptr<int64_t>(), x.data_ptr(), current_stream(dev)),
          "nm_csr_row_sum_forward");
    return x;
}

Tensor csr_row_sum_backward(Tensor grad_x, int A_rows, int A_cols, Tensor A_data, Tensor A_indices,
                            Tensor A_indptr) {
    check_csr("csr_row_sum_backward", A_rows, A_cols, A_data, A_indices, A_indptr);
    check_vector("csr_row_sum_backward", "grad_x", grad_x, A_rows);
    const auto dev = need_device({&grad_x, &A_data, &A_indices, &A_indptr});
    same_dtype(A_data, grad_x, "grad_x");
    grad_x = grad_x.contiguous();
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty({A_data.numel()}, A_data.options());
    check(nm_csr_row_sum_backward(dtype_of(A_data), A_rows, A_data.numel(), A_indptr.data_ptr<int64_t>(),
                                  grad_x.data_ptr(), grad_A.data_ptr(), current_stream(dev)),
          "nm_csr_row_sum_backward");
    return grad_A;
}

Tensor csr_extract_diagonal_forward(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr) {
    check_csr("csr_extract_diagonal_forward", A_rows, A_cols, A_data, A_indices, A_indptr);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr});
    A_data = A_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor x = torch::empty({A_rows}, A_data.options());
    check(nm_csr_extract_diagonal_forward(dtype_of(A_data), A_rows, A_data.numel(), A_data.data_ptr(),
                                          A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                          x.data_ptr(), current_stream(dev)),
          "nm_csr_extract_diagonal_forward");
    return x;
}

Tensor csr_extract_diagonal_backward(Tensor grad_x, int A_rows, int A_cols, Tensor A_data, Tensor A_indices,
                                     Tensor A_indptr) {
    check_csr("csr_extract_diagonal_backward", A_rows, A_cols, A_data, A_indices, A_indptr);
    check_vector("csr_extract_diagonal_backward", "grad_x", grad_x, A_rows);
    const auto dev = need_device({&grad_x, &A_data, &A_indices, &A_indptr});
    same_dtype(A_data, grad_x, "grad_x");
    grad_x = grad_x.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty({A_data.numel()}, A_data.options());
    check(nm_csr_extract_diagonal_backward(dtype_of(A_data), A_rows, A_data.numel(),
                                           A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                           grad_x.data_ptr(), grad_A.data_ptr(), current_stream(dev)),
          "nm_csr_extract_diagonal_backward");
    return grad_A;
}

// ---------------------------------------------------------------------------- SpMM

Tensor spdmm_forward(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr, Tensor B) {
    check_csr("spdmm_forward", A_rows, A_cols, A_data, A_indices, A_indptr);
    check_matrix("spdmm_forward", "B", B, A_cols, -1);
    // cpp/sparse_csr.cpp:125-128 checks the same thing with the same wording
    TORCH_CHECK((A_data.device() == A_indices.device() && A_indices.device() == A_indptr.device() &&
                 A_indptr.device() == B.device()),
                "expected A and B to be on same device, but got A on (", A_data.device(), ", ",
                A_indices.device(), ", ", A_indptr.device(), ") and B on ", B.device());
    const auto dev = need_device({&A_data, &A_indices, &A_indptr, &B});
    same_dtype(A_data, B, "B");
    A_data = A_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    int64_t ldb = 1;
    B = row_major(B, &ldb);
    const int64_t n = B.size(1);
    c10::hip::HIPGuard guard(dev.index());
    Tensor C = torch::empty({A_rows, n}, A_data.options());
    check(nm_spdmm_forward(dtype_of(A_data), A_rows, B.size(0), A_data.numel(), A_data.data_ptr(),
                           A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), B.data_ptr(), ldb, n,
                           C.data_ptr(), std::max<int64_t>(n, 1), current_stream(dev)),
          "nm_spdmm_forward");
    return C;
}

std::vector<Tensor> spdmm_backward(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr,
                                   Tensor B, Tensor grad_C) {
    check_csr("spdmm_backward", A_rows, A_cols, A_data, A_indices, A_indptr);
    check_matrix("spdmm_backward", "B", B, A_cols, -1);
    check_matrix("spdmm_backward", "grad_C", grad_C, A_rows, B.size(1));
    TORCH_CHECK((A_data.device() == A_indices.device() && A_indices.device() == A_indptr.device() &&
                 A_indptr.device() == B.device()),
                "expected A and B to be on same device, but got A on (", A_data.device(), ", ",
                A_indices.device(), ", ", A_indptr.device(), ") and B on ", B.device());
    TORCH_CHECK(B.device() == grad_C.device(), "expected B and grad_C to be on same device, but got B on ",
                B.device(), " and grad_C on ", grad_C.device());
    const auto dev = need_device({&A_data, &A_indices, &A_indptr, &B, &grad_C});
    same_dtype(A_data, B, "B");
    same_dtype(A_data, grad_C, "grad_C");
    A_data = A_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    int64_t ldb = 1, ldg = 1;
    B = row_major(B, &ldb);
    grad_C = row_major(grad_C, &ldg);
    const int64_t n = B.size(1);
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty_like(A_data);
    Tensor grad_B = torch::empty({B.size(0), n}, B.options());
    if (planned_backward()) {
        auto plan = transpose_plan(A_indices, A_indptr, A_rows, B.size(0), dev);
        check(nm_spdmm_backward_planned(dtype_of(A_data), A_rows, B.size(0), A_data.numel(), A_data.data_ptr(),
                                        A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                        plan->mem.data_ptr(), B.data_ptr(), ldb, grad_C.data_ptr(), ldg, n,
                                        grad_A.data_ptr(), grad_B.data_ptr(), std::max<int64_t>(n, 1),
                                        current_stream(dev)),
              "nm_spdmm_backward_planned");
    } else {
        check(nm_spdmm_backward(dtype_of(A_data), A_rows, B.size(0), A_data.numel(), A_data.data_ptr(),
                                A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), B.data_ptr(), ldb,
                                grad_C.data_ptr(), ldg, n, grad_A.data_ptr(), grad_B.data_ptr(),
                                std::max<int64_t>(n, 1), current_stream(dev)),
              "nm_spdmm_backward");
    }
    return {grad_A, grad_B};
}

// -------------------------------------------------------------------------- SpGEMM

std::vector<Tensor> spgemm_forward(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr,
                                   int B_rows, int B_cols, Tensor B_data, Tensor B_indices, Tensor B_indptr) {
    check_csr("spgemm_forward", A_rows, A_cols, A_data, A_indices, A_indptr);
    check_csr("spgemm_forward", B_rows, B_cols, B_data, B_indices, B_indptr);
    TORCH_CHECK(A_cols == B_rows, "spgemm_forward: A has ", A_cols, " columns but B has ", B_rows, " rows");
    const auto dev = need_device({&A_data, &A_indices, &A_indptr, &B_data, &B_indices, &B_indptr});
    same_dtype(A_data, B_data, "B_data");
    A_data = A_data.contiguous();
    B_data = B_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    B_indices = index_tensor(B_indices, "B_indices");
    B_indptr = index_tensor(B_indptr, "B_indptr");
    c10::hip::HIPGuard guard(dev.index());
    size_t bytes = 0;
    check(nm_spgemm_workspace_bytes(A_rows, B_cols, &bytes), "nm_spgemm_workspace_bytes");
    Tensor work = scratch(bytes, dev);
    const auto iopt = torch::TensorOptions().dtype(torch::kInt64).device(dev);
    Tensor C_indptr = torch::empty({(int64_t)A_rows + 1}, iopt);
    nm_stream st = current_stream(dev);
    check(nm_spgemm_symbolic(A_rows, A_cols, B_cols, A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                             B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(),
                             C_indptr.data_ptr<int64_t>(), work.data_ptr(), bytes, st),
          "nm_spgemm_symbolic");
    // the one device->host read the interface makes inherent: C is returned exactly sized
    int64_t nnz_c = 0, hash_rows = 0;
    check(nm_spgemm_symbolic_result(A_rows, B_cols, work.data_ptr(), bytes, &nnz_c, &hash_rows, host_landing(),
                                    st),
          "nm_spgemm_symbolic_result");
    Tensor C_indices = torch::empty({nnz_c}, iopt);
    Tensor C_data = torch::empty({nnz_c}, A_data.options());
    check(nm_spgemm_numeric(dtype_of(A_data), A_rows, A_cols, B_cols, A_data.data_ptr(),
                            A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), B_data.data_ptr(),
                            B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(),
                            C_indptr.data_ptr<int64_t>(), C_indices.data_ptr<int64_t>(), C_data.data_ptr(),
                            work.data_ptr(), bytes, hash_rows, st),
          "nm_spgemm_numeric");
    return {C_data, C_indices, C_indptr};
}

std::vector<Tensor> spgemm_backward(Tensor grad_C, Tensor C_indices, Tensor C_indptr, int A_rows, int A_cols,
                                    Tensor A_data, Tensor A_indices, Tensor A_indptr, int B_rows, int B_cols,
                                    Tensor B_data, Tensor B_indices, Tensor B_indptr) {
    check_csr("spgemm_backward", A_rows, A_cols, A_data, A_indices, A_indptr);
    check_csr("spgemm_backward", B_rows, B_cols, B_data, B_indices, B_indptr);
    check_csr("spgemm_backward", A_rows, B_cols, grad_C, C_indices, C_indptr);
    TORCH_CHECK(A_cols == B_rows, "spgemm_backward: A has ", A_cols, " columns but B has ", B_rows, " rows");
    const auto dev = need_device({&grad_C, &C_indices, &C_indptr, &A_data, &A_indices, &A_indptr, &B_data,
                                  &B_indices, &B_indptr});
    same_dtype(A_data, B_data, "B_data");
    same_dtype(A_data, grad_C, "grad_C");
    A_data = A_data.contiguous();
    B_data = B_data.contiguous();
    grad_C = grad_C.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    B_indices = index_tensor(B_indices, "B_indices");
    B_indptr = index_tensor(B_indptr, "B_indptr");
    C_indices = index_tensor(C_indices, "C_indices");
    C_indptr = index_tensor(C_indptr, "C_indptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A = torch::empty_like(A_data), grad_B = torch::empty_like(B_data);
    check(nm_spgemm_backward(dtype_of(A_data), A_rows, A_data.numel(), B_data.numel(), grad_C.data_ptr(),
                             C_indices.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(), A_data.data_ptr(),
                             A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), B_data.data_ptr(),
                             B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(), grad_A.data_ptr(),
                             grad_B.data_ptr(), current_stream(dev)),
          "nm_spgemm_backward");
    return {grad_A, grad_B};
}

// -------------------------------------------------------------------------- SpTRSV

Tensor sptrsv_forward(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr, bool lower,
                      bool unit, Tensor b) {
    check_csr("sptrsv_forward", A_rows, A_cols, A_data, A_indices, A_indptr);
    TORCH_CHECK(A_rows == A_cols, "sptrsv_forward: expected a square matrix, got ", A_rows, " x ", A_cols);
    check_vector("sptrsv_forward", "b", b, A_rows);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr, &b});
    same_dtype(A_data, b, "b");
    A_data = A_data.contiguous();
    b = b.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto plan = level_plan(A_indices, A_indptr, A_rows, lower, dev);
    return solve(*plan, false, A_data, unit, b, A_rows, dev);
}

std::vector<Tensor> sptrsv_backward(Tensor grad_x, Tensor x, int A_rows, int A_cols, Tensor A_data,
                                    Tensor A_indices, Tensor A_indptr, bool lower, bool unit, Tensor b) {
    check_csr("sptrsv_backward", A_rows, A_cols, A_data, A_indices, A_indptr);
    TORCH_CHECK(A_rows == A_cols, "sptrsv_backward: expected a square matrix, got ", A_rows, " x ", A_cols);
    check_vector("sptrsv_backward", "grad_x", grad_x, A_rows);
    check_vector("sptrsv_backward", "x", x, A_rows);
    const auto dev = need_device({&grad_x, &x, &A_data, &A_indices, &A_indptr});
    same_dtype(A_data, grad_x, "grad_x");
    same_dtype(A_data, x, "x");
    A_data = A_data.contiguous();
    grad_x = grad_x.contiguous();
    x = x.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto plan = level_plan(A_indices, A_indptr, A_rows, lower, dev);
    Tensor grad_b = solve(*plan, true, A_data, unit, grad_x, A_rows, dev);
    Tensor grad_A = torch::empty_like(A_data);
    check(nm_masked_outer(dtype_of(A_data), A_rows, A_data.numel(), A_indices.data_ptr<int64_t>(),
                          A_indptr.data_ptr<int64_t>(), -1.0, grad_b.data_ptr(), x.data_ptr(), grad_A.data_ptr(),
                          current_stream(dev)),
          "nm_masked_outer");
    return {grad_A, grad_b};
}

// (dependency levels, kernel launches per solve) of the cached or newly built level
// schedule of a triangular pattern; no counterpart in the reference (diagnostics).
// ------------------------------------------------------------------------ sparse LU

// The filled pattern of the factors, its transpose and the map between them depend on A's
// structure alone: they are computed once per pattern and the same index tensors are handed
// out by every later call, so that the solves that follow find their level schedules cached.
std::shared_ptr<Plan> lu_pattern(const Tensor &A_indices, const Tensor &A_indptr, int64_t rows,
                                 const c10::Device &dev) {
    for (int attempt = 0;; ++attempt) {
        auto plan = cached('U', A_indices, A_indptr, rows, rows, [&](Plan &p) {
            const auto iopt = torch::TensorOptions().dtype(torch::kInt64).device(dev);
            const nm_stream stream = current_stream(dev);
            size_t bytes = 0;
            check(nm_splu_symbolic_bytes(rows, &bytes), "nm_splu_symbolic_bytes");
            Tensor work = scratch(bytes, dev);
            Tensor M_indptr = torch::empty({rows + 1}, iopt);
            check(nm_splu_symbolic(rows, A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                   M_indptr.data_ptr<int64_t>(), work.data_ptr(), bytes, stream),
                  "nm_splu_symbolic");
            const int64_t nnz = M_indptr[rows].item<int64_t>();
            Tensor M_indices = torch::empty({nnz}, iopt);
            Tensor zeros = torch::zeros({std::max<int64_t>(A_indices.numel(), 1)},
                                        torch::TensorOptions().dtype(torch::kFloat32).device(dev));
            Tensor As_data = torch::empty({nnz}, zeros.options());
            check(nm_splu_fill(NM_F32, rows, zeros.data_ptr(), A_indices.data_ptr<int64_t>(),
                               A_indptr.data_ptr<int64_t>(), M_indptr.data_ptr<int64_t>(),
                               M_indices.data_ptr<int64_t>(), As_data.data_ptr(), work.data_ptr(), bytes, stream),
                  "nm_splu_fill");
            auto tplan = transpose_plan(M_indices, M_indptr, rows, rows, dev);
            Tensor Mt_data = torch::empty_like(As_data);
            Tensor Mt_indices = torch::empty({nnz}, iopt);
            Tensor Mt_indptr = torch::empty({rows + 1}, iopt);
            Tensor Mt_to_M = torch::empty({nnz}, iopt);
            check(nm_csr_transpose_forward(NM_F32, rows, rows, nnz, As_data.data_ptr(), tplan->mem.data_ptr(),
                                           Mt_data.data_ptr(), Mt_indices.data_ptr<int64_t>(),
                                           Mt_indptr.data_ptr<int64_t>(), Mt_to_M.data_ptr<int64_t>(), stream),
                  "nm_csr_transpose_forward");
            p.derived = {M_indices, M_indptr, Mt_indices, Mt_indptr, Mt_to_M};
            for (const Tensor &t : p.derived) p.derived_versions.push_back(t._version());
            c10::hip::getCurrentHIPStream(dev.index()).synchronize();   // complete for every stream
        });
        bool intact = true;   // a caller may have edited the tensors it was handed
        for (size_t i = 0; i < plan->derived.size(); ++i)
            intact = intact && plan->derived[i]._version() == plan->derived_versions[i];
        if (intact || attempt > 0) {
            TORCH_CHECK(intact, "the cached factor pattern was modified in place");
            return plan;
        }
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        g_plans.remove(plan);
    }
}

// [M_data, M_indices, M_indptr, Mt_data, Mt_indices, Mt_indptr]  (cpp/sparse_csr.hpp:107-111)
std::vector<Tensor> splu(int A_rows, int A_cols, Tensor A_data, Tensor A_indices, Tensor A_indptr) {
    check_csr("splu", A_rows, A_cols, A_data, A_indices, A_indptr);
    const auto dev = need_device({&A_data, &A_indices, &A_indptr});
    TORCH_CHECK(A_rows == A_cols, "Expected square matrix for LU factorization, got ", A_rows, " x ", A_cols, ".");
    A_data = A_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    const int64_t rows = A_rows;
    const nm_stream stream = current_stream(dev);
    const nm_dtype dt = dtype_of(A_data);

    auto pattern = lu_pattern(A_indices, A_indptr, rows, dev);
    const Tensor &M_indices = pattern->derived[0], &M_indptr = pattern->derived[1];
    const Tensor &Mt_indices = pattern->derived[2], &Mt_indptr = pattern->derived[3];
    const Tensor &Mt_to_M = pattern->derived[4];
    const int64_t nnz = M_indices.numel();

    // A's values on the filled pattern, moved to the transpose: the factorisation runs by column
    Tensor As_data = torch::empty({nnz}, A_data.options());
    check(nm_splu_values(dt, rows, A_data.data_ptr(), A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                         M_indptr.data_ptr<int64_t>(), M_indices.data_ptr<int64_t>(), As_data.data_ptr(), stream),
          "nm_splu_values");
    auto tplan = transpose_plan(M_indices, M_indptr, rows, rows, dev);
    const auto iopt = torch::TensorOptions().dtype(torch::kInt64).device(dev);
    Tensor Mt_data = torch::empty_like(As_data);
    Tensor idx_scratch = torch::empty({2 * nnz + rows + 1}, iopt);   // the structure is already known
    int64_t *is = idx_scratch.data_ptr<int64_t>();
    check(nm_csr_transpose_forward(dt, rows, rows, nnz, As_data.data_ptr(), tplan->mem.data_ptr(),
                                   Mt_data.data_ptr(), is, is + nnz, is + nnz + rows + 1, stream),
          "nm_csr_transpose_forward");
    size_t bytes = 0;
    check(nm_splu_numeric_bytes(rows, &bytes), "nm_splu_numeric_bytes");
    Tensor work = scratch(bytes, dev);
    check(nm_splu_numeric(dt, rows, Mt_data.data_ptr(), Mt_indices.data_ptr<int64_t>(),
                          Mt_indptr.data_ptr<int64_t>(), work.data_ptr(), bytes, 0, stream),
          "nm_splu_numeric");
    Tensor M_data = torch::empty_like(Mt_data);
    check(nm_csr_transpose_backward(dt, nnz, Mt_data.data_ptr(), Mt_to_M.data_ptr<int64_t>(), M_data.data_ptr(),
                                    stream),
          "nm_csr_transpose_backward");
    return {M_data, M_indices, M_indptr, Mt_data, Mt_indices, Mt_indptr};
}

// [grad_A, grad_b]  (cpp/sparse_csr.hpp:113-118, cpp/sparse_csr_cpu.cpp:1018-1048): grad_b = A^-T grad_x
// by two solves with M^T, grad_A = -(grad_b x^T) on A's pattern.
std::vector<Tensor> spsolve_backward(Tensor grad_x, Tensor x, int A_rows, int A_cols, Tensor Mt_data,
                                     Tensor Mt_indices, Tensor Mt_indptr, Tensor A_data, Tensor A_indices,
                                     Tensor A_indptr) {
    check_csr("spsolve_backward", A_rows, A_cols, A_data, A_indices, A_indptr);
    check_csr("spsolve_backward", A_rows, A_cols, Mt_data, Mt_indices, Mt_indptr);
    TORCH_CHECK(A_rows == A_cols, "spsolve_backward: expected a square matrix, got ", A_rows, " x ", A_cols);
    check_vector("spsolve_backward", "grad_x", grad_x, A_rows);
    check_vector("spsolve_backward", "x", x, A_rows);
    const auto dev = need_device({&grad_x, &x, &Mt_data, &Mt_indices, &Mt_indptr, &A_data, &A_indices, &A_indptr});
    same_dtype(A_data, grad_x, "grad_x");
    same_dtype(A_data, x, "x");
    same_dtype(A_data, Mt_data, "Mt_data");
    Mt_data = Mt_data.contiguous();
    A_data = A_data.contiguous();
    grad_x = grad_x.contiguous();
    x = x.contiguous();
    Mt_indices = index_tensor(Mt_indices, "Mt_indices");
    Mt_indptr = index_tensor(Mt_indptr, "Mt_indptr");
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto lower = level_plan(Mt_indices, Mt_indptr, A_rows, true, dev);
    Tensor y = solve(*lower, false, Mt_data, false, grad_x, A_rows, dev);
    auto upper = level_plan(Mt_indices, Mt_indptr, A_rows, false, dev);
    Tensor grad_b = solve(*upper, false, Mt_data, true, y, A_rows, dev);
    Tensor grad_A = torch::empty_like(A_data);
    check(nm_masked_outer(dtype_of(A_data), A_rows, A_data.numel(), A_indices.data_ptr<int64_t>(),
                          A_indptr.data_ptr<int64_t>(), -1.0, grad_b.data_ptr(), x.data_ptr(), grad_A.data_ptr(),
                          current_stream(dev)),
          "nm_masked_outer");
    return {grad_A, grad_b};
}

// ------------------------------------------------------------------------ diagnostics

std::tuple<int64_t, int64_t> sptrsv_schedule(int A_rows, Tensor A_indices, Tensor A_indptr, bool lower) {
    TORCH_CHECK(A_indptr.dim() == 1 && A_indptr.numel() == (int64_t)A_rows + 1 && A_indices.dim() == 1,
                "sptrsv_schedule: expected ", A_rows + 1, " row pointers, got shape ", A_indptr.sizes());
    const auto dev = need_device({&A_indices, &A_indptr});
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto plan = level_plan(A_indices, A_indptr, A_rows, lower, dev);
    return {nm_sptrsv_plan_levels(plan->handle), nm_sptrsv_plan_launches(plan->handle)};
}

void clear_plan_cache() {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans.clear();
}

int64_t plan_cache_size() {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    return (int64_t)g_plans.size();
}

void set_backward_mode(const std::string &mode) {
    TORCH_CHECK(mode == "planned" || mode == "atomic", "backward mode must be 'planned' or 'atomic', got '", mode,
                "'");
    g_planned.store(mode == "planned", std::memory_order_relaxed);
}

std::string backward_mode() { return planned_backward() ? "planned" : "atomic"; }

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "numml_torch_cpp on AMD gfx950: differentiable CSR SpMV / SpMM / SpGEMM / SpTRSV";
    m.def("spgemv_forward", &spgemv_forward, "SPGEMV forward");
    m.def("spgemv_backward", &spgemv_backward, "SPGEMV backward");
    m.def("spgemm_forward", &spgemm_forward, "SPGEMM forward");
    m.def("spgemm_backward", &spgemm_backward, "SPGEMM backward");
    m.def("spdmm_forward", &spdmm_forward, "Sparse times dense matrix forward");
    m.def("spdmm_backward", &spdmm_backward, "Sparse times dense matrix backward");
    m.def("sptrsv_forward", &sptrsv_forward, "Sparse triangular solve forward");
    m.def("sptrsv_backward", &sptrsv_backward, "Sparse triangular solve backward");
    m.def("splu", &splu, "Sparse LU decomposition");
    m.def("spsolve_backward", &spsolve_backward, "Sparse LU solve backward");
    m.def("csr_transpose_forward", &csr_transpose_forward, "CSR Transpose forward");
    m.def("csr_transpose_backward", &csr_transpose_backward, "CSR Transpose backward");
    m.def("splincomb_forward", &splincomb_forward, "Sparse linear combination forward");
    m.def("splincomb_backward", &splincomb_backward, "Sparse linear combination backward");
    m.def("csr_to_dense_forward", &csr_to_dense_forward, "CSR to dense forward");
    m.def("csr_to_dense_backward", &csr_to_dense_backward, "CSR to dense backward");
    m.def("csr_row_sum_forward", &csr_row_sum_forward, "CSR row sum forward");
    m.def("csr_row_sum_backward", &csr_row_sum_backward, "CSR row sum backward");
    m.def("csr_extract_diagonal_forward", &csr_extract_diagonal_forward, "CSR extract diagonal forward");
    m.def("csr_extract_diagonal_backward", &csr_extract_diagonal_backward, "CSR extract diagonal backward");
    m.def("sptrsv_schedule", &sptrsv_schedule, "(levels, launches per solve) of a triangular pattern");
    m.def("clear_plan_cache", &clear_plan_cache, "Drop every cached structure plan");
    m.def("plan_cache_size", &plan_cache_size, "Number of cached structure plans");
    m.def("set_backward_mode", &set_backward_mode, "'planned' (cached transposed structure) or 'atomic'");
    m.def("backward_mode", &backward_mode, "Current backward mode");
}
