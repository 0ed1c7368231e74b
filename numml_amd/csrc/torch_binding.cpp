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
#include <ATen/hip/HIPEvent.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPCachingAllocator.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <algorithm>
#include <atomic>
#include <cmath>
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

// Which of its two gradients a backward pass computes.  The reference's GPU path computes a
// gradient only for an operand that requires one (cpp/sparse_csr_cuda.cu:662, :682) and leaves
// the other tensor undefined, its CPU path always computes both.  Here: both when neither
// operand requires a gradient (a direct call outside autograd, what the CPU path would give),
// otherwise those that are required; a gradient that is left out comes back undefined (None in
// Python), which autograd treats like the value it would have thrown away.
struct Wanted {
    bool first, second;
};
Wanted wanted(const Tensor &a, const Tensor &b) {
    const bool ra = a.requires_grad(), rb = b.requires_grad();
    if (!ra && !rb) return {true, true};
    return {ra, rb};
}
void *ptr_or_null(const Tensor &t) { return t.defined() ? t.data_ptr() : nullptr; }

// How SpMV / SpMM backward compute grad_x / grad_B:
//   "planned" (default)  on a cached transposed-structure plan (deterministic, no atomics) from
//                        the SECOND time a sparsity pattern is seen; the first sighting runs the
//                        stateless kernels, so a pattern that is used once never pays for a plan;
//   "eager"              the plan is built at the first sighting (deterministic from the first call);
//   "atomic"             always the stateless scatter with atomics.
// NUMML_AMD_BACKWARD sets the initial value, set_backward_mode() changes it.
enum Mode : int { kAtomic = 0, kPlanned = 1, kEager = 2 };
std::atomic<int> g_mode{[] {
    const char *e = std::getenv("NUMML_AMD_BACKWARD");
    const std::string v = e ? e : "";
    return v == "atomic" ? (int)kAtomic : v == "eager" ? (int)kEager : (int)kPlanned;
}()};

int backward_mode_now() { return g_mode.load(std::memory_order_relaxed); }

// ---- structure plans -----------------------------------------------------------
//
// Everything derived from a sparsity pattern alone (the transposed structure, the level
// schedule of a triangle, the filled pattern of LU factors) is computed once and cached under a
// 128-bit key of the pattern's CONTENT (nm_structure_hash), so that a pattern arriving in fresh
// tensors -- a clone, the product A @ B computed again -- finds its plans.  Computing the key
// costs one pass over the structure and a wait for the stream, so it is done once per pair of
// tensors: an alias table maps the identity of (indices, indptr) -- tensor objects, storage
// addresses, version counters -- to the key it was given.  The table holds weak references
// only: a tensor that has died cannot be mistaken for a new one at the same address, and no
// caller memory is kept alive.  (An edit that goes around the version counter, such as a write
// through `.data`, is not seen: the plan of the old pattern would be used.)
//
// The cache is bounded by the bytes of device memory its plans hold (NUMML_AMD_PLAN_CACHE_MB,
// default 4096), least recently used first out.

struct Key {
    uint64_t h0 = 0, h1 = 0;
    int64_t nnz = 0, nptr = 0;
    int device = -1;
    bool operator==(const Key &o) const {
        return h0 == o.h0 && h1 == o.h1 && nnz == o.nnz && nptr == o.nptr && device == o.device;
    }
};

using WeakImpl = c10::weak_intrusive_ptr<c10::TensorImpl, c10::UndefinedTensorImpl>;

struct Alias {
    const c10::TensorImpl *idx_impl, *ptr_impl;
    WeakImpl idx_weak, ptr_weak;
    const void *idx_ptr, *ptr_ptr;
    uint32_t idx_version, ptr_version;
    Key key;
    int64_t longest_row = -1;    // entries of the pattern's longest row, once somebody has asked
};

struct Plan {
    // 'T' transposed structure, 'L' level schedule, 'U' filled pattern of the LU factors,
    // 'P' product plan of A B (key: A's pattern, key2: B's), 'S' maps of a linear combination
    // alpha A + beta B (key: A's pattern, key2: B's)
    char kind;
    Key key, key2;
    int64_t a, b;
    Tensor mem;
    size_t bytes = 0;
    std::vector<Tensor> derived;             // 'U', 'P': structure tensors handed out to callers
    std::vector<uint32_t> derived_versions;  //      and their version counters when built
    bool usable = true;                      // 'P': false when the product is beyond the plan's limits
    int plan_class = 1;                      // 'P': which forward kernel the product takes (nm_spgemm_plan_build)
    std::shared_ptr<Plan> parent;            // 'P': the transposed-structure plan of A it walks
    nm_sptrsv_plan *handle = nullptr;
    // 'T': what the build found out about the pattern (nm_csr_transpose_plan_info), read back
    // the first time a policy asks for it
    int32_t info[16] = {0};
    std::atomic<bool> info_loaded{false};
    // the stream the plan was built on and the event that marks its completion there
    c10::StreamId build_stream = 0;
    std::unique_ptr<at::cuda::CUDAEvent> ready;
    ~Plan() {
        if (handle) nm_sptrsv_plan_destroy(handle);
    }
};

struct Sighting {
    char kind;
    Key key, key2;
    int64_t a, b;
};

constexpr size_t kAliasTableSize = 64, kSightingTableSize = 256;
std::mutex g_plans_mutex;
std::list<std::shared_ptr<Plan>> g_plans;  // most recently used first
std::list<Alias> g_aliases;                // most recently used first
std::list<Sighting> g_sightings;
size_t g_plan_bytes = 0;
std::atomic<size_t> g_plan_bytes_limit{[] {
    const char *e = std::getenv("NUMML_AMD_PLAN_CACHE_MB");
    const long long mb = e ? std::atoll(e) : 4096;
    return (size_t)(mb > 0 ? mb : 0) << 20;
}()};
std::atomic<int64_t> g_plans_built{0}, g_keys_computed{0};

// 32 bytes of pinned host memory per host thread (from torch's pinned-memory allocator, which
// also takes it back): where nm_spgemm_symbolic_result and nm_structure_hash have the device
// drop their results.
void *host_landing() {
    thread_local Tensor landing =
        torch::zeros({4}, torch::TensorOptions().dtype(torch::kInt64).pinned_memory(true));
    return landing.data_ptr();
}

// Tensors made under torch.inference_mode() carry no version counter (asking for it throws).
// A pair of such structure tensors gets no entry in the alias table -- an edit in place could
// not be noticed -- so a call that needs a plan computes their content key every time and one
// that only peeks runs its stateless kernels; pattern tensors of this kind that a plan hands
// out count as version 0.
bool tracked(const Tensor &t) { return !t.is_inference(); }
uint32_t version_of(const Tensor &t) { return tracked(t) ? t._version() : 0; }

bool alias_matches(const Alias &al, const Tensor &indices, const Tensor &indptr) {
    return al.idx_impl == indices.unsafeGetTensorImpl() && al.ptr_impl == indptr.unsafeGetTensorImpl() &&
           al.idx_ptr == indices.data_ptr() && al.ptr_ptr == indptr.data_ptr() &&
           al.idx_version == indices._version() && al.ptr_version == indptr._version() &&
           al.key.nnz == indices.numel() && al.key.nptr == indptr.numel() &&
           al.key.device == indices.device().index() && !al.idx_weak.expired() && !al.ptr_weak.expired();
}

// The content key of (indices, indptr): from the alias table, or computed (waits for the stream).
// With `compute` false a pair of tensors that has not been seen yields false instead.
bool structure_key(const Tensor &indices, const Tensor &indptr, bool compute, Key *out) {
    const bool aliased = tracked(indices) && tracked(indptr);
    if (aliased) {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        for (auto it = g_aliases.begin(); it != g_aliases.end(); ++it) {
            if (alias_matches(*it, indices, indptr)) {
                *out = it->key;
                if (it != g_aliases.begin()) g_aliases.splice(g_aliases.begin(), g_aliases, it);
                return true;
            }
        }
    }
    if (!compute) return false;
    const c10::Device dev = indices.device();
    size_t bytes = 0;
    check(nm_structure_hash_bytes(&bytes), "nm_structure_hash_bytes");
    Tensor work = scratch(bytes, dev);
    uint64_t h[2] = {0, 0};
    check(nm_structure_hash(indices.numel(), indptr.numel(), indices.data_ptr<int64_t>(),
                            indptr.data_ptr<int64_t>(), work.data_ptr(), bytes, host_landing(), h,
                            current_stream(dev)),
          "nm_structure_hash");
    g_keys_computed.fetch_add(1, std::memory_order_relaxed);
    if (!aliased) {
        *out = Key{h[0], h[1], indices.numel(), indptr.numel(), dev.index()};
        return true;
    }
    Alias al{indices.unsafeGetTensorImpl(),
             indptr.unsafeGetTensorImpl(),
             WeakImpl(indices.getIntrusivePtr()),
             WeakImpl(indptr.getIntrusivePtr()),
             indices.data_ptr(),
             indptr.data_ptr(),
             indices._version(),
             indptr._version(),
             Key{h[0], h[1], indices.numel(), indptr.numel(), dev.index()}};
    *out = al.key;
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    // entries of tensors that have died, or that describe these very tensors at an older version
    g_aliases.remove_if([&](const Alias &o) {
        return o.idx_weak.expired() || o.ptr_weak.expired() ||
               (o.idx_impl == al.idx_impl && o.ptr_impl == al.ptr_impl);
    });
    g_aliases.push_front(std::move(al));
    while (g_aliases.size() > kAliasTableSize) g_aliases.pop_back();
    return true;
}

// Entries of the longest row of a pattern: remembered with the pair of tensors' entry in the alias
// table (a pair that has none is measured every time).
int64_t longest_row(const Tensor &indices, const Tensor &indptr, int64_t rows, const c10::Device &dev) {
    const bool aliased = tracked(indices) && tracked(indptr);
    if (aliased) {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        for (const Alias &al : g_aliases)
            if (alias_matches(al, indices, indptr) && al.longest_row >= 0) return al.longest_row;
    }
    Tensor work = scratch(8, dev);
    int64_t longest = 0;
    check(nm_csr_longest_row(rows, indptr.data_ptr<int64_t>(), work.data_ptr(), 8, host_landing(), &longest,
                             current_stream(dev)),
          "nm_csr_longest_row");
    if (aliased) {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        for (Alias &al : g_aliases)
            if (alias_matches(al, indices, indptr)) al.longest_row = longest;
    }
    return longest;
}

// Makes `plan` usable on the current stream: work enqueued there from now on runs after the
// build, and the allocator is told that this stream reads the plan's memory.
void join_plan(const Plan &plan, const c10::Device &dev) {
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index());
    if (!plan.ready || stream.id() == plan.build_stream) return;
    plan.ready->block(stream);
    if (plan.mem.defined())
        c10::hip::HIPCachingAllocator::recordStream(plan.mem.storage().data_ptr(), stream.hip_stream());
}

std::shared_ptr<Plan> find_plan_locked(char kind, const Key &key, int64_t a, int64_t b, const Key &key2 = Key()) {
    for (auto it = g_plans.begin(); it != g_plans.end(); ++it) {
        Plan &p = **it;
        if (p.kind == kind && p.key == key && p.key2 == key2 && p.a == a && p.b == b) {
            if (it != g_plans.begin()) g_plans.splice(g_plans.begin(), g_plans, it);
            return g_plans.front();
        }
    }
    return nullptr;
}

// The cached plan of this kind for the pattern, or nullptr; never computes a key and never
// builds (what a forward pass may look at without paying for anything).
std::shared_ptr<Plan> peek_plan(char kind, const Tensor &indices, const Tensor &indptr, int64_t a, int64_t b,
                                const c10::Device &dev) {
    Key key;
    if (!structure_key(indices, indptr, false, &key)) return nullptr;
    std::shared_ptr<Plan> plan;
    {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        plan = find_plan_locked(kind, key, a, b);
    }
    if (plan) join_plan(*plan, dev);
    return plan;
}

// The plan of this kind for the pattern.  `second_sighting`: a pattern seen for the first time
// is only noted and nullptr is returned (the caller then runs its stateless kernels); the plan
// is built when the pattern shows up again.
template <typename Make>
std::shared_ptr<Plan> cached(char kind, const Tensor &indices, const Tensor &indptr, int64_t a, int64_t b,
                             bool second_sighting, const c10::Device &dev, Make make) {
    Key key;
    structure_key(indices, indptr, true, &key);
    {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        if (auto hit = find_plan_locked(kind, key, a, b)) {
            join_plan(*hit, dev);
            return hit;
        }
        if (second_sighting) {
            bool seen = false;
            for (auto it = g_sightings.begin(); it != g_sightings.end(); ++it)
                if (it->kind == kind && it->key == key && it->key2 == Key() && it->a == a && it->b == b) {
                    g_sightings.erase(it);
                    seen = true;
                    break;
                }
            if (!seen) {
                g_sightings.push_front(Sighting{kind, key, Key(), a, b});
                while (g_sightings.size() > kSightingTableSize) g_sightings.pop_back();
                return nullptr;
            }
        }
    }
    auto plan = std::make_shared<Plan>();
    plan->kind = kind;
    plan->key = key;
    plan->a = a;
    plan->b = b;
    make(*plan);
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index());
    plan->build_stream = stream.id();
    plan->ready = std::make_unique<at::cuda::CUDAEvent>();
    plan->ready->record(stream);
    plan->bytes = plan->mem.defined() ? (size_t)plan->mem.nbytes() : 0;
    for (const Tensor &t : plan->derived) plan->bytes += (size_t)t.nbytes();
    g_plans_built.fetch_add(1, std::memory_order_relaxed);
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans.push_front(plan);
    g_plan_bytes += plan->bytes;
    const size_t limit = g_plan_bytes_limit.load(std::memory_order_relaxed);
    while (g_plans.size() > 1 && g_plan_bytes > limit) {
        g_plan_bytes -= g_plans.back()->bytes;
        g_plans.pop_back();
    }
    return plan;
}

// `second_sighting` as above; csr_transpose_forward and the LU code need the plan at once.
std::shared_ptr<Plan> transpose_plan(const Tensor &indices, const Tensor &indptr, int64_t rows, int64_t cols,
                                     const c10::Device &dev, bool second_sighting = false) {
    return cached('T', indices, indptr, rows, cols, second_sighting, dev, [&](Plan &p) {
        const int64_t nnz = indices.numel();
        size_t pbytes = 0, wbytes = 0;
        check(nm_csr_transpose_plan_bytes(rows, cols, nnz, &pbytes, &wbytes), "nm_csr_transpose_plan_bytes");
        p.mem = scratch(pbytes, dev);
        Tensor work = scratch(wbytes, dev);
        // enqueued on the current stream, nothing waits: the plan's event orders other streams
        // behind the build, and `work` goes back to the allocator, which hands it out again
        // only to work enqueued later on this same stream
        check(nm_csr_transpose_plan_build(rows, cols, nnz, indices.data_ptr<int64_t>(),
                                          indptr.data_ptr<int64_t>(), p.mem.data_ptr(), pbytes, work.data_ptr(),
                                          wbytes, current_stream(dev)),
              "nm_csr_transpose_plan_build");
    });
}

// Statistics of a transposed-structure plan's pattern (one wait for the stream per plan).
const int32_t *plan_info(Plan &plan, int64_t rows, int64_t cols, int64_t nnz, const c10::Device &dev) {
    if (!plan.info_loaded.load(std::memory_order_acquire)) {
        int32_t info[16];
        check(nm_csr_transpose_plan_info(rows, cols, nnz, plan.mem.data_ptr(), info, current_stream(dev)),
              "nm_csr_transpose_plan_info");
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        std::copy(info, info + 16, plan.info);
        plan.info_loaded.store(true, std::memory_order_release);
    }
    return plan.info;
}

// Which kernels the last backward pass of each kind ran (diagnostics and tests of the policy).
std::atomic<int> g_last_spdmm_backward{-1}, g_last_spgemm_backward{-1};
enum Path : int { kStateless = 0, kOnTransposedPlan = 1, kOnProductPlan = 2 };

// A transposed-structure plan keeps rows, columns and positions in 32 bits
// (nm_csr_transpose_plan_bytes refuses more); larger matrices run the stateless kernels, which
// take 64-bit offsets throughout.
bool fits_a_plan(int64_t rows, int64_t cols, int64_t nnz) {
    const int64_t lim = 0x7ffffffe;
    return rows < lim && cols < lim && nnz < lim;
}

// The transposed-structure plan a backward pass should use under the current mode, or nullptr
// for the stateless kernels.
std::shared_ptr<Plan> backward_plan(const Tensor &indices, const Tensor &indptr, int64_t rows, int64_t cols,
                                    const c10::Device &dev) {
    const int mode = backward_mode_now();
    if (mode == kAtomic || !fits_a_plan(rows, cols, indices.numel())) return nullptr;
    return transpose_plan(indices, indptr, rows, cols, dev, mode == kPlanned);
}

std::shared_ptr<Plan> level_plan(const Tensor &indices, const Tensor &indptr, int64_t rows, bool lower,
                                 const c10::Device &dev) {
    return cached('L', indices, indptr, rows, lower ? 1 : 0, false, dev, [&](Plan &p) {
        const int64_t nnz = indices.numel();
        size_t pbytes = 0, wbytes = 0;
        check(nm_sptrsv_plan_bytes(rows, nnz, &pbytes, &wbytes), "nm_sptrsv_plan_bytes");
        p.mem = scratch(pbytes, dev);
        Tensor work = scratch(wbytes, dev);
        check(nm_sptrsv_analyse(rows, nnz, indices.data_ptr<int64_t>(), indptr.data_ptr<int64_t>(),
                                lower ? 1 : 0, p.mem.data_ptr(), pbytes, work.data_ptr(), wbytes, &p.handle,
                                current_stream(dev)),
              "nm_sptrsv_analyse");  // synchronises its stream
    });
}

// ---- product plans ---------------------------------------------------------------
//
// A product A B whose rows all stay on the merge path (nm_spgemm_symbolic_result reports no row
// on the hash path) can be given a product plan: the pattern of C and, per entry of A, where its
// products go.  With it a forward pass is one numeric kernel and a backward pass two gather
// kernels; the values are the ones the stateless kernels give, bit for bit.  The plan is keyed
// on the content of both patterns and follows the policy of the transposed-structure plans:
// built the second time the pair is seen ("planned"), at once ("eager"), never ("atomic").
// Results of planned forward passes SHARE the plan's C_indices / C_indptr tensors (the pattern
// is the same by construction); a plan whose tensors have been written to in place is dropped.

void drop_plan(const std::shared_ptr<Plan> &plan) {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    for (auto it = g_plans.begin(); it != g_plans.end(); ++it)
        if (*it == plan) {
            g_plan_bytes -= plan->bytes;
            g_plans.erase(it);
            return;
        }
}

// The product plan of the pair; nullptr when there is none or its pattern tensors were edited.
// With `compute` false the pair is looked up through the alias table only (no key is computed:
// what a call may do before it knows whether the product is eligible at all).
std::shared_ptr<Plan> peek_product_plan(const Tensor &A_indices, const Tensor &A_indptr, const Tensor &B_indices,
                                        const Tensor &B_indptr, int64_t A_rows, int64_t B_cols,
                                        const c10::Device &dev, bool compute = false, char kind = 'P') {
    Key ka, kb;
    if (!structure_key(A_indices, A_indptr, compute, &ka) || !structure_key(B_indices, B_indptr, compute, &kb))
        return nullptr;
    std::shared_ptr<Plan> plan;
    {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        plan = find_plan_locked(kind, ka, A_rows, B_cols, kb);
    }
    if (!plan) return nullptr;
    for (size_t i = 0; i < plan->derived.size(); ++i)
        if (version_of(plan->derived[i]) != plan->derived_versions[i]) {
            drop_plan(plan);
            return nullptr;
        }
    join_plan(*plan, dev);
    if (plan->parent) join_plan(*plan->parent, dev);
    return plan;
}

// After a stateless forward pass of a product without hash-path rows: notes the pair, or makes
// its plan around the pattern of C that the pass has just produced.  `filled`: plan memory that
// the pass filled as it went (nm_spgemm_symbolic_mapped / nm_spgemm_numeric_mapped), which only
// has to be checked; without it the plan is built from the three patterns.
void consider_product_plan(const Tensor &A_indices, const Tensor &A_indptr, const Tensor &B_indices,
                           const Tensor &B_indptr, const Tensor &C_indices, const Tensor &C_indptr,
                           int64_t A_rows, int64_t A_cols, int64_t B_cols, const c10::Device &dev,
                           const Tensor &filled = Tensor()) {
    const int mode = backward_mode_now();
    if (mode == kAtomic || A_indices.numel() == 0 || C_indices.numel() == 0) return;
    if (!fits_a_plan(A_rows, A_cols, A_indices.numel()) || !fits_a_plan(A_cols, B_cols, B_indices.numel()) ||
        !fits_a_plan(A_rows, B_cols, C_indices.numel()))
        return;
    Key ka, kb;
    structure_key(A_indices, A_indptr, true, &ka);
    structure_key(B_indices, B_indptr, true, &kb);
    {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        if (find_plan_locked('P', ka, A_rows, B_cols, kb)) return;   // e.g. one that turned out unusable
        if (mode == kPlanned) {
            bool seen = false;
            for (auto it = g_sightings.begin(); it != g_sightings.end(); ++it)
                if (it->kind == 'P' && it->key == ka && it->key2 == kb && it->a == A_rows && it->b == B_cols) {
                    g_sightings.erase(it);
                    seen = true;
                    break;
                }
            if (!seen) {
                g_sightings.push_front(Sighting{'P', ka, kb, A_rows, B_cols});
                while (g_sightings.size() > kSightingTableSize) g_sightings.pop_back();
                return;
            }
        }
    }
    auto plan = std::make_shared<Plan>();
    plan->kind = 'P';
    plan->key = ka;
    plan->key2 = kb;
    plan->a = A_rows;
    plan->b = B_cols;
    plan->parent = transpose_plan(A_indices, A_indptr, A_rows, A_cols, dev);
    size_t pbytes = 0;
    check(nm_spgemm_plan_bytes(A_indices.numel(), &pbytes), "nm_spgemm_plan_bytes");
    int usable = 0;
    if (filled.defined()) {
        plan->mem = filled;
        check(nm_spgemm_plan_adopt(A_rows, A_cols, A_indices.numel(), B_indices.numel(), C_indices.numel(), 0,
                                   plan->parent->mem.data_ptr(), plan->mem.data_ptr(), pbytes, host_landing(),
                                   &usable, current_stream(dev)),
              "nm_spgemm_plan_adopt");
    } else {
        plan->mem = scratch(pbytes, dev);
        check(nm_spgemm_plan_build(A_rows, A_cols, A_indices.numel(), B_indices.numel(), C_indices.numel(),
                                   A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                   B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(),
                                   C_indices.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(),
                                   plan->parent->mem.data_ptr(), plan->mem.data_ptr(), pbytes, host_landing(),
                                   &usable, current_stream(dev)),
              "nm_spgemm_plan_build");
        if (usable < 0) {
            // the only obstacle is the length of the rows of B that A names (9 to 32 entries): a plan
            // with two or four destination octets per entry of A
            const int octets = -usable <= 16 ? 2 : 4;
            check(nm_spgemm_plan_bytes_wide(A_indices.numel(), octets, &pbytes), "nm_spgemm_plan_bytes_wide");
            plan->mem = scratch(pbytes, dev);
            check(nm_spgemm_plan_build_wide(A_rows, A_cols, A_indices.numel(), B_indices.numel(), C_indices.numel(),
                                            A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                            B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(),
                                            C_indices.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(),
                                            plan->parent->mem.data_ptr(), plan->mem.data_ptr(), pbytes, octets,
                                            host_landing(), &usable, current_stream(dev)),
                  "nm_spgemm_plan_build_wide");
        }
    }
    plan->usable = usable > 0;
    plan->plan_class = usable > 0 ? usable : 0;
    if (plan->usable) {
        plan->derived = {C_indices, C_indptr};
        for (const Tensor &t : plan->derived) plan->derived_versions.push_back(version_of(t));
    } else {
        plan->mem = Tensor();   // remembered as unusable, so that the pair is not analysed again
        plan->parent.reset();
    }
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index());
    plan->build_stream = stream.id();
    plan->ready = std::make_unique<at::cuda::CUDAEvent>();
    plan->ready->record(stream);
    plan->bytes = plan->mem.defined() ? (size_t)plan->mem.nbytes() : 0;
    for (const Tensor &t : plan->derived) plan->bytes += (size_t)t.nbytes();
    g_plans_built.fetch_add(1, std::memory_order_relaxed);
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans.push_front(plan);
    g_plan_bytes += plan->bytes;
    const size_t limit = g_plan_bytes_limit.load(std::memory_order_relaxed);
    while (g_plans.size() > 1 && g_plan_bytes > limit) {
        g_plan_bytes -= g_plans.back()->bytes;
        g_plans.pop_back();
    }
}

// After a stateless linear combination: notes the pair of patterns, or (second sighting; first in
// eager mode) records the maps of the combination around the pattern of C just produced.
void consider_sum_plan(const Tensor &A_indices, const Tensor &A_indptr, const Tensor &B_indices,
                       const Tensor &B_indptr, const Tensor &C_indices, const Tensor &C_indptr, int64_t rows,
                       int64_t cols, const c10::Device &dev) {
    const int mode = backward_mode_now();
    const int64_t lim = (int64_t)1 << 31;
    if (mode == kAtomic || C_indices.numel() == 0 || A_indices.numel() >= lim || B_indices.numel() >= lim ||
        C_indices.numel() >= lim)
        return;
    Key ka, kb;
    structure_key(A_indices, A_indptr, true, &ka);
    structure_key(B_indices, B_indptr, true, &kb);
    {
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        if (find_plan_locked('S', ka, rows, cols, kb)) return;
        if (mode == kPlanned) {
            bool seen = false;
            for (auto it = g_sightings.begin(); it != g_sightings.end(); ++it)
                if (it->kind == 'S' && it->key == ka && it->key2 == kb && it->a == rows && it->b == cols) {
                    g_sightings.erase(it);
                    seen = true;
                    break;
                }
            if (!seen) {
                g_sightings.push_front(Sighting{'S', ka, kb, rows, cols});
                while (g_sightings.size() > kSightingTableSize) g_sightings.pop_back();
                return;
            }
        }
    }
    auto plan = std::make_shared<Plan>();
    plan->kind = 'S';
    plan->key = ka;
    plan->key2 = kb;
    plan->a = rows;
    plan->b = cols;
    size_t pbytes = 0;
    check(nm_splincomb_plan_bytes(A_indices.numel(), B_indices.numel(), C_indices.numel(), &pbytes),
          "nm_splincomb_plan_bytes");
    plan->mem = scratch(pbytes, dev);
    check(nm_splincomb_plan_build(rows, A_indices.numel(), B_indices.numel(), C_indices.numel(),
                                  A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                  B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(),
                                  C_indices.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(), plan->mem.data_ptr(),
                                  pbytes, current_stream(dev)),
          "nm_splincomb_plan_build");
    plan->derived = {C_indices, C_indptr};
    for (const Tensor &t : plan->derived) plan->derived_versions.push_back(version_of(t));
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index());
    plan->build_stream = stream.id();
    plan->ready = std::make_unique<at::cuda::CUDAEvent>();
    plan->ready->record(stream);
    plan->bytes = (size_t)plan->mem.nbytes();
    for (const Tensor &t : plan->derived) plan->bytes += (size_t)t.nbytes();
    g_plans_built.fetch_add(1, std::memory_order_relaxed);
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans.push_front(plan);
    g_plan_bytes += plan->bytes;
    const size_t limit = g_plan_bytes_limit.load(std::memory_order_relaxed);
    while (g_plans.size() > 1 && g_plan_bytes > limit) {
        g_plan_bytes -= g_plans.back()->bytes;
        g_plans.pop_back();
    }
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
    // a pattern whose transposed-structure plan exists is read through the plan's 32-bit
    // copies of the structure (half the index bytes); looking for it costs no device work
    if (auto plan = peek_plan('T', A_col_ind, A_rowptr, A_rows, x.size(0), dev)) {
        // most blocks of 512 rows have a staging list: the instantiation that stages x in LDS (it
        // gives up resident workgroups for that)
        const int32_t *info = plan_info(*plan, A_rows, x.size(0), A_data.numel(), dev);
        const bool lists = 2 * (int64_t)info[4] >= ((int64_t)A_rows + 511) / 512;
        check((lists ? nm_spgemv_forward_planned_lists : nm_spgemv_forward_planned)(
                  dtype_of(A_data), A_rows, x.size(0), A_data.numel(), A_data.data_ptr(), plan->mem.data_ptr(),
                  x.data_ptr(), y.data_ptr(), current_stream(dev)),
              "nm_spgemv_forward_planned");
        return y;
    }
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
    const Wanted want = wanted(A_data, x);
    A_data = A_data.contiguous();
    x = x.contiguous();
    grad_z = grad_z.contiguous();
    A_col_ind = index_tensor(A_col_ind, "A_col_ind");
    A_rowptr = index_tensor(A_rowptr, "A_rowptr");
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A, grad_x;
    if (want.first) grad_A = torch::empty_like(A_data);
    if (want.second) grad_x = torch::empty_like(x);
    if (auto plan = backward_plan(A_col_ind, A_rowptr, A_rows, x.size(0), dev)) {
        // most blocks of 256 columns have a staging list: the instantiation that stages g and x in LDS
        const int32_t *info = plan_info(*plan, A_rows, x.size(0), A_data.numel(), dev);
        const bool lists = 2 * (int64_t)info[5] >= ((int64_t)x.size(0) + 255) / 256;
        check((lists ? nm_spgemv_backward_planned_lists : nm_spgemv_backward_planned)(
                  dtype_of(A_data), A_rows, x.size(0), A_data.numel(), A_data.data_ptr(), plan->mem.data_ptr(),
                  x.data_ptr(), grad_z.data_ptr(), ptr_or_null(grad_A), ptr_or_null(grad_x), current_stream(dev)),
              "nm_spgemv_backward_planned");
    } else {
        check(nm_spgemv_backward(dtype_of(A_data), A_rows, x.size(0), A_data.numel(), A_data.data_ptr(),
                                 A_col_ind.data_ptr<int64_t>(), A_rowptr.data_ptr<int64_t>(), x.data_ptr(),
                                 grad_z.data_ptr(), ptr_or_null(grad_A), ptr_or_null(grad_x), current_stream(dev)),
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
    if (backward_mode_now() != kAtomic) {
        // patterns seen before (alias lookup only): one pass over the cached maps; the result shares
        // the plan's pattern tensors, as a planned product does
        if (auto plan = peek_product_plan(A_indices, A_indptr, B_indices, B_indptr, rows, cols, dev, false, 'S')) {
            Tensor C_data = torch::empty({plan->derived[0].numel()}, A_data.options());
            check(nm_splincomb_numeric_planned(dtype_of(A_data), A_indices.numel(), B_indices.numel(), C_data.numel(),
                                               a, A_data.data_ptr(), b, B_data.data_ptr(), plan->mem.data_ptr(),
                                               C_data.data_ptr(), current_stream(dev)),
                  "nm_splincomb_numeric_planned");
            return {C_data, plan->derived[0], plan->derived[1]};
        }
    }
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
    consider_sum_plan(A_indices, A_indptr, B_indices, B_indptr, C_indices, C_indptr, rows, cols, dev);
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
    const Wanted want = wanted(A_data, B_data);
    Tensor grad_A, grad_B;
    if (want.first) grad_A = torch::empty_like(A_data, at::MemoryFormat::Contiguous);
    if (want.second) grad_B = torch::empty_like(B_data, at::MemoryFormat::Contiguous);
    if (backward_mode_now() != kAtomic) {
        // the maps belong to the pattern tensors the planned forward handed out: those very tensors
        auto plan = peek_product_plan(A_indices, A_indptr, B_indices, B_indptr, rows, cols, dev, false, 'S');
        if (plan && plan->derived[0].data_ptr() == C_indices.data_ptr() &&
            plan->derived[1].data_ptr() == C_indptr.data_ptr() && plan->derived[0].numel() == C_indices.numel()) {
            check(nm_splincomb_backward_planned(dtype_of(A_data), A_indices.numel(), B_indices.numel(),
                                                C_indices.numel(), a, b, grad_C_data.data_ptr(), plan->mem.data_ptr(),
                                                ptr_or_null(grad_A), ptr_or_null(grad_B), current_stream(dev)),
                  "nm_splincomb_backward_planned");
            return {grad_A, grad_B};
        }
    }
    check(nm_splincomb_backward(dtype_of(A_data), rows, a, A_indices.data_ptr<int64_t>(),
                                A_indptr.data_ptr<int64_t>(), b, B_indices.data_ptr<int64_t>(),
                                B_indptr.data_ptr<int64_t>(), grad_C_data.data_ptr(), C_indices.data_ptr<int64_t>(),
                                C_indptr.data_ptr<int64_t>(), ptr_or_null(grad_A), ptr_or_null(grad_B),
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
    const Wanted want = wanted(A_data, B);
    A_data = A_data.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    int64_t ldb = 1, ldg = 1;
    B = row_major(B, &ldb);
    grad_C = row_major(grad_C, &ldg);
    const int64_t n = B.size(1);
    c10::hip::HIPGuard guard(dev.index());
    Tensor grad_A, grad_B;
    if (want.first) grad_A = torch::empty_like(A_data);
    if (want.second) grad_B = torch::empty({B.size(0), n}, B.options());
    // (the dot products alone walk A by row and need no plan)
    auto plan = want.second ? backward_plan(A_indices, A_indptr, A_rows, B.size(0), dev) : nullptr;
    if (plan && backward_mode_now() == kPlanned) {
        // The kernels on the plan give every aligned group of 64 columns to one workgroup, which
        // takes the group's columns of more than 512 entries one after the other (~0.12 us an entry
        // with both gradients, ~0.02 us for the transposed product alone), while the stateless
        // kernels spread every entry over the chip at ~0.2 ns: where one group holds more than a
        // thousandth (a hundredth) of the matrix in such columns, the stateless kernels are the
        // faster ones.  ("eager" asks for the deterministic sums whatever they cost.)
        const int64_t heavy = plan_info(*plan, A_rows, B.size(0), A_data.numel(), dev)[8];
        if (heavy * (want.first ? 1000 : 100) > A_data.numel()) plan = nullptr;
    }
    g_last_spdmm_backward.store(plan ? kOnTransposedPlan : kStateless, std::memory_order_relaxed);
    if (plan) {
        check(nm_spdmm_backward_planned(dtype_of(A_data), A_rows, B.size(0), A_data.numel(), A_data.data_ptr(),
                                        A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(),
                                        plan->mem.data_ptr(), B.data_ptr(), ldb, grad_C.data_ptr(), ldg, n,
                                        ptr_or_null(grad_A), ptr_or_null(grad_B), std::max<int64_t>(n, 1),
                                        current_stream(dev)),
              "nm_spdmm_backward_planned");
    } else {
        check(nm_spdmm_backward(dtype_of(A_data), A_rows, B.size(0), A_data.numel(), A_data.data_ptr(),
                                A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), B.data_ptr(), ldb,
                                grad_C.data_ptr(), ldg, n, ptr_or_null(grad_A), ptr_or_null(grad_B),
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
    const bool plans = backward_mode_now() != kAtomic;
    auto on_plan = [&](const Plan &plan) -> std::vector<Tensor> {
        const Tensor &C_indices = plan.derived[0], &C_indptr = plan.derived[1];
        Tensor C_data = torch::empty({C_indices.numel()}, A_data.options());
        check(nm_spgemm_numeric_planned(dtype_of(A_data), plan.plan_class, A_rows, A_data.numel(), B_data.numel(),
                                        C_indices.numel(),
                                        A_data.data_ptr(), A_indptr.data_ptr<int64_t>(), B_data.data_ptr(),
                                        plan.mem.data_ptr(), C_indptr.data_ptr<int64_t>(), C_data.data_ptr(),
                                        current_stream(dev)),
              "nm_spgemm_numeric_planned");
        return {C_data, C_indices, C_indptr};
    };
    if (plans) {
        auto plan = peek_product_plan(A_indices, A_indptr, B_indices, B_indptr, A_rows, B_cols, dev);
        if (plan && plan->usable) return on_plan(*plan);
    }
    size_t bytes = 0;
    check(nm_spgemm_workspace_bytes(A_rows, B_cols, &bytes), "nm_spgemm_workspace_bytes");
    Tensor work = scratch(bytes, dev);
    const auto iopt = torch::TensorOptions().dtype(torch::kInt64).device(dev);
    Tensor C_indptr = torch::empty({(int64_t)A_rows + 1}, iopt);
    nm_stream st = current_stream(dev);
    // The symbolic merge records where every product goes (16 bytes per entry of A, scratch of this
    // call): with no row on the hash path the numeric phase then adds the products up on those
    // records instead of merging the rows again (cheaper than the second merge whether or not
    // anything is kept), and unless plans are switched off the records become a product plan's.
    const int64_t A_nnz = A_data.numel(), B_nnz = B_data.numel();
    const int64_t lim31 = (int64_t)1 << 31;
    Tensor filled;
    size_t pbytes = 0;
    if (A_nnz > 0 && A_nnz < lim31 && B_nnz < lim31) {
        check(nm_spgemm_plan_bytes(A_nnz, &pbytes), "nm_spgemm_plan_bytes");
        filled = scratch(pbytes, dev);
        check(nm_spgemm_symbolic_mapped(A_rows, A_cols, B_cols, A_nnz, B_nnz, A_indices.data_ptr<int64_t>(),
                                        A_indptr.data_ptr<int64_t>(), B_indices.data_ptr<int64_t>(),
                                        B_indptr.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(), work.data_ptr(),
                                        bytes, filled.data_ptr(), pbytes, host_landing(), st),
              "nm_spgemm_symbolic_mapped");
    } else {
        check(nm_spgemm_symbolic(A_rows, A_cols, B_cols, A_indices.data_ptr<int64_t>(),
                                 A_indptr.data_ptr<int64_t>(), B_indices.data_ptr<int64_t>(),
                                 B_indptr.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(), work.data_ptr(), bytes,
                                 host_landing(), st),
              "nm_spgemm_symbolic");
    }
    // the one device->host read the interface makes inherent: C is returned exactly sized
    int64_t nnz_c = 0, hash_rows = 0;
    check(nm_spgemm_symbolic_result(A_rows, B_cols, work.data_ptr(), bytes, &nnz_c, &hash_rows, host_landing(),
                                    st),
          "nm_spgemm_symbolic_result");
    if (plans && nnz_c > 0) {
        // a product plan may exist: worth a content key per pattern that arrives in tensors not
        // seen before (a clone, a product computed again), which may find the pair's plan
        auto plan = peek_product_plan(A_indices, A_indptr, B_indices, B_indptr, A_rows, B_cols, dev, true);
        if (plan && plan->usable) return on_plan(*plan);
    }
    Tensor C_indices = torch::empty({nnz_c}, iopt);
    Tensor C_data = torch::empty({nnz_c}, A_data.options());
    const bool on_map = filled.defined() && hash_rows == 0 && nnz_c > 0 && nnz_c < lim31;
    check(nm_spgemm_numeric_mapped(dtype_of(A_data), A_rows, A_cols, B_cols, A_nnz, nnz_c, A_data.data_ptr(),
                                   A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), B_data.data_ptr(),
                                   B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(),
                                   C_indptr.data_ptr<int64_t>(), C_indices.data_ptr<int64_t>(), C_data.data_ptr(),
                                   work.data_ptr(), bytes, hash_rows, on_map ? filled.data_ptr() : nullptr, pbytes,
                                   plans ? 1 : 0, st),
          "nm_spgemm_numeric_mapped");
    // note the pair, or make its plan: from the memory this pass filled, or (rows on the hash
    // path: the plan's own analysis says whether the product is within its limits) from the patterns
    if (on_map && plans)
        consider_product_plan(A_indices, A_indptr, B_indices, B_indptr, C_indices, C_indptr, A_rows, A_cols, B_cols,
                              dev, filled);
    else if (plans && nnz_c > 0)
        consider_product_plan(A_indices, A_indptr, B_indices, B_indptr, C_indices, C_indptr, A_rows, A_cols, B_cols,
                              dev);
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
    const Wanted want = wanted(A_data, B_data);
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
    Tensor grad_A, grad_B;
    if (want.first) grad_A = torch::empty_like(A_data);
    if (want.second) grad_B = torch::empty_like(B_data);
    if (backward_mode_now() != kAtomic) {
        // the product plan applies when grad_C lies on the very pattern tensors the plan handed out
        auto pp = peek_product_plan(A_indices, A_indptr, B_indices, B_indptr, A_rows, B_cols, dev);
        if (pp && pp->usable && pp->derived[0].data_ptr() == C_indices.data_ptr() &&
            pp->derived[1].data_ptr() == C_indptr.data_ptr() && pp->derived[0].numel() == C_indices.numel()) {
            g_last_spgemm_backward.store(kOnProductPlan, std::memory_order_relaxed);
            check(nm_spgemm_backward_mapped_wide(dtype_of(A_data), pp->plan_class, A_rows, A_cols, A_data.numel(),
                                                 B_data.numel(), grad_C.numel(), grad_C.data_ptr(),
                                                 A_data.data_ptr(), pp->parent->mem.data_ptr(), B_data.data_ptr(),
                                                 B_indptr.data_ptr<int64_t>(), pp->mem.data_ptr(),
                                                 ptr_or_null(grad_A), ptr_or_null(grad_B), current_stream(dev)),
                  "nm_spgemm_backward_mapped_wide");
            return {grad_A, grad_B};
        }
    }
    // The plan-based kernel looks every column of a row of B up in a staged row of C per entry of
    // A, the stateless one stages a row of C once and looks the rows of B up in it: with rows of C
    // many times longer than rows of B the stateless kernel is the faster one, and the default mode
    // takes it ("eager" asks for the deterministic sums whatever they cost).
    const int mode = backward_mode_now();
    const double mean_c = A_rows > 0 ? (double)grad_C.numel() / A_rows : 0.;
    const double mean_b = B_rows > 0 ? (double)B_data.numel() / B_rows : 0.;
    // It also shares the work out by row of B and hands a row whose products (its entries times the
    // entries of A's column) run into the thousands to a single workgroup: where that is the average
    // row, the stateless kernel is many times faster (2 M rows of A naming 16 rows of B: 8 ms against
    // seconds).
    const double mean_col = A_cols > 0 ? (double)A_data.numel() / A_cols : 0.;
    const bool on_plan = mode == kEager ||
                         (mode == kPlanned && mean_c <= 4. * std::max(mean_b, 1.) && mean_b * mean_col <= 4096.);
    auto plan = on_plan ? backward_plan(A_indices, A_indptr, A_rows, A_cols, dev) : nullptr;
    if (plan && mode == kPlanned) {
        // Means hide a few heavy rows among many light ones: the longest column of A (from the plan)
        // times the longest row of B (measured once per pair of B's structure tensors) bounds the
        // products the busiest workgroup makes.
        const int64_t longest_col = plan_info(*plan, A_rows, A_cols, A_data.numel(), dev)[6];
        Key kb;
        structure_key(B_indices, B_indptr, true, &kb);      // (an alias entry to remember the length with)
        if (longest_col * longest_row(B_indices, B_indptr, B_rows, dev) > 65536) plan = nullptr;
    }
    g_last_spgemm_backward.store(plan ? kOnTransposedPlan : kStateless, std::memory_order_relaxed);
    if (plan) {
        check(nm_spgemm_backward_planned(dtype_of(A_data), A_rows, A_cols, A_data.numel(), B_data.numel(),
                                         grad_C.numel(), grad_C.data_ptr(), C_indices.data_ptr<int64_t>(),
                                         C_indptr.data_ptr<int64_t>(), A_data.data_ptr(), plan->mem.data_ptr(),
                                         B_data.data_ptr(), B_indices.data_ptr<int64_t>(),
                                         B_indptr.data_ptr<int64_t>(), ptr_or_null(grad_A), ptr_or_null(grad_B),
                                         current_stream(dev)),
              "nm_spgemm_backward_planned");
        return {grad_A, grad_B};
    }
    check(nm_spgemm_backward(dtype_of(A_data), A_rows, A_data.numel(), B_data.numel(), grad_C.data_ptr(),
                             C_indices.data_ptr<int64_t>(), C_indptr.data_ptr<int64_t>(), A_data.data_ptr(),
                             A_indices.data_ptr<int64_t>(), A_indptr.data_ptr<int64_t>(), B_data.data_ptr(),
                             B_indices.data_ptr<int64_t>(), B_indptr.data_ptr<int64_t>(), ptr_or_null(grad_A),
                             ptr_or_null(grad_B), current_stream(dev)),
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
    // (grad_A is formed from grad_b, so the transposed solve runs whichever gradient is wanted)
    const Wanted want = wanted(A_data, b);
    A_data = A_data.contiguous();
    grad_x = grad_x.contiguous();
    x = x.contiguous();
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto plan = level_plan(A_indices, A_indptr, A_rows, lower, dev);
    Tensor grad_b = solve(*plan, true, A_data, unit, grad_x, A_rows, dev);
    if (!want.first) return {Tensor(), grad_b};
    Tensor grad_A = torch::empty_like(A_data);
    check(nm_masked_outer(dtype_of(A_data), A_rows, A_data.numel(), A_indices.data_ptr<int64_t>(),
                          A_indptr.data_ptr<int64_t>(), -1.0, grad_b.data_ptr(), x.data_ptr(), grad_A.data_ptr(),
                          current_stream(dev)),
          "nm_masked_outer");
    if (!want.second) return {grad_A, Tensor()};
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
        auto plan = cached('U', A_indices, A_indptr, rows, rows, false, dev, [&](Plan &p) {
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
            for (const Tensor &t : p.derived) p.derived_versions.push_back(version_of(t));
        });
        bool intact = true;   // a caller may have edited the tensors it was handed
        for (size_t i = 0; i < plan->derived.size(); ++i)
            intact = intact && version_of(plan->derived[i]) == plan->derived_versions[i];
        if (intact || attempt > 0) {
            TORCH_CHECK(intact, "the cached factor pattern was modified in place");
            return plan;
        }
        std::lock_guard<std::mutex> lock(g_plans_mutex);
        const size_t before = g_plans.size();
        g_plans.remove(plan);
        if (g_plans.size() != before) g_plan_bytes -= plan->bytes;
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

std::tuple<int64_t, int64_t> sptrsv_chain_levels(int A_rows, Tensor A_indices, Tensor A_indptr, bool lower) {
    TORCH_CHECK(A_indptr.dim() == 1 && A_indptr.numel() == (int64_t)A_rows + 1 && A_indices.dim() == 1,
                "sptrsv_chain_levels: expected ", A_rows + 1, " row pointers, got shape ", A_indptr.sizes());
    const auto dev = need_device({&A_indices, &A_indptr});
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto plan = level_plan(A_indices, A_indptr, A_rows, lower, dev);
    return {nm_sptrsv_plan_chain_levels(plan->handle, 0), nm_sptrsv_plan_chain_levels(plan->handle, 1)};
}

std::tuple<int64_t, int64_t> sptrsv_shared_launches(int A_rows, Tensor A_indices, Tensor A_indptr, bool lower) {
    TORCH_CHECK(A_indptr.dim() == 1 && A_indptr.numel() == (int64_t)A_rows + 1 && A_indices.dim() == 1,
                "sptrsv_shared_launches: expected ", A_rows + 1, " row pointers, got shape ", A_indptr.sizes());
    const auto dev = need_device({&A_indices, &A_indptr});
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto plan = level_plan(A_indices, A_indptr, A_rows, lower, dev);
    return {nm_sptrsv_plan_shared_launches(plan->handle, 0), nm_sptrsv_plan_shared_launches(plan->handle, 1)};
}

// What the transposed-structure plan of a pattern (the cached one, or one built now) found out:
// (symmetric, packed words of the backward valid, 16-bit column offsets of the forward valid,
// row blocks with a staging list, row blocks, column blocks with one, column blocks, longest column,
// longest row, most entries of long columns in one group of 64 columns).  Diagnostics; waits for the stream.
std::vector<int64_t> transpose_plan_info(int A_rows, int A_cols, Tensor A_indices, Tensor A_indptr) {
    TORCH_CHECK(A_indptr.dim() == 1 && A_indptr.numel() == (int64_t)A_rows + 1 && A_indices.dim() == 1,
                "transpose_plan_info: expected ", A_rows + 1, " row pointers, got shape ", A_indptr.sizes());
    const auto dev = need_device({&A_indices, &A_indptr});
    A_indices = index_tensor(A_indices, "A_indices");
    A_indptr = index_tensor(A_indptr, "A_indptr");
    c10::hip::HIPGuard guard(dev.index());
    auto plan = transpose_plan(A_indices, A_indptr, A_rows, A_cols, dev);
    int32_t info[16];
    check(nm_csr_transpose_plan_info(A_rows, A_cols, A_indices.numel(), plan->mem.data_ptr(), info,
                                     current_stream(dev)),
          "nm_csr_transpose_plan_info");
    return {info[0], info[1], info[2], info[4], ((int64_t)A_rows + 511) / 512, info[5], ((int64_t)A_cols + 255) / 256,
            info[6], info[7], info[8], info[9]};
}

// Time-free helper of the bandwidth calibration: enqueues one nm_stream_probe launch.
void stream_probe(Tensor src, int64_t read_bytes, Tensor dst, int64_t write_bytes) {
    const auto dev = need_device({&src, &dst});
    TORCH_CHECK(src.is_contiguous() && dst.is_contiguous() && read_bytes <= (int64_t)src.nbytes() &&
                    write_bytes <= (int64_t)dst.nbytes(),
                "stream_probe: buffers smaller than the byte counts");
    c10::hip::HIPGuard guard(dev.index());
    check(nm_stream_probe(src.data_ptr(), (size_t)read_bytes, dst.data_ptr(), (size_t)write_bytes, current_stream(dev)),
          "nm_stream_probe");
}

// ("stateless" | "transposed plan" | "product plan" | "none yet") for the last spdmm_backward and
// the last spgemm_backward of this process.
std::tuple<std::string, std::string> last_backward_paths() {
    auto name = [](int p) -> std::string {
        return p == kStateless ? "stateless" : p == kOnTransposedPlan ? "transposed plan"
               : p == kOnProductPlan ? "product plan" : "none yet";
    };
    return {name(g_last_spdmm_backward.load(std::memory_order_relaxed)),
            name(g_last_spgemm_backward.load(std::memory_order_relaxed))};
}

void clear_plan_cache() {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    g_plans.clear();
    g_aliases.clear();
    g_sightings.clear();
    g_plan_bytes = 0;
}

int64_t plan_cache_size() {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    return (int64_t)g_plans.size();
}

int64_t plan_cache_bytes() {
    std::lock_guard<std::mutex> lock(g_plans_mutex);
    return (int64_t)g_plan_bytes;
}

void set_plan_cache_limit(int64_t bytes) {
    TORCH_CHECK(bytes >= 0, "the plan cache limit must not be negative");
    g_plan_bytes_limit.store((size_t)bytes, std::memory_order_relaxed);
}

// (plans built, structure keys computed) since the module was loaded
std::tuple<int64_t, int64_t> plan_cache_stats() {
    return {g_plans_built.load(std::memory_order_relaxed), g_keys_computed.load(std::memory_order_relaxed)};
}

void set_backward_mode(const std::string &mode) {
    TORCH_CHECK(mode == "planned" || mode == "eager" || mode == "atomic",
                "backward mode must be 'planned', 'eager' or 'atomic', got '", mode, "'");
    g_mode.store(mode == "atomic" ? kAtomic : mode == "eager" ? kEager : kPlanned, std::memory_order_relaxed);
}

std::string backward_mode() {
    const int m = backward_mode_now();
    return m == kAtomic ? "atomic" : m == kEager ? "eager" : "planned";
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "numml_torch_cpp on AMD gfx950: differentiable CSR SpMV / SpMM / SpGEMM / SpTRSV";
    // The plan cache holds device tensors and events.  They are given back while the interpreter,
    // torch's allocator and the HIP runtime are still there: left to this library's static
    // destructors they would be freed after those have gone.
    pybind11::module_::import("atexit").attr("register")(pybind11::cpp_function([] { clear_plan_cache(); }));
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
    m.def("sptrsv_chain_levels", &sptrsv_chain_levels,
          "levels of the solves with A and with A^T that the single-wavefront chain kernels take");
    m.def("sptrsv_shared_launches", &sptrsv_shared_launches,
          "launches of the solves with A and with A^T whose levels several workgroups share");
    m.def("transpose_plan_info", &transpose_plan_info,
          "(symmetric, packed backward, packed forward, staged row blocks, row blocks, staged column blocks, "
          "column blocks) of a pattern's transposed-structure plan");
    m.def("stream_probe", &stream_probe, "one launch of the streaming calibration kernel (read_bytes in, write_bytes out)");
    m.def("last_backward_paths", &last_backward_paths,
          "which kernels the last spdmm_backward and the last spgemm_backward ran");
    m.def("clear_plan_cache", &clear_plan_cache, "Drop every cached structure plan");
    m.def("plan_cache_size", &plan_cache_size, "Number of cached structure plans");
    m.def("plan_cache_bytes", &plan_cache_bytes, "Device memory held by the cached structure plans");
    m.def("set_plan_cache_limit", &set_plan_cache_limit, "Bound of plan_cache_bytes (least recently used plans go first)");
    m.def("plan_cache_stats", &plan_cache_stats, "(plans built, structure keys computed) since the module was loaded");
    m.def("set_backward_mode", &set_backward_mode,
          "'planned' (cached transposed structure from the second sighting of a pattern), 'eager' (from the first) "
          "or 'atomic' (never)");
    m.def("backward_mode", &backward_mode, "Current backward mode");
}
