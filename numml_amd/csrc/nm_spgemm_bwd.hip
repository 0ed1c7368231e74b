// SpGEMM backward on the transposed-structure plan of A: both gradients of
// C = A B without atomics and without clearing, summed in the order of the serial
// CPU loops (cpp/sparse_csr_cpu.cpp:246-278 for grad_A, :291-303 for grad_B), so
// that they come out bit-identical and the same on every run.
//
// Work is shared out by ROW k OF B.  The products that touch row k are
// (i, k, c) for the entries (i, k) of column k of A -- the plan lists them with i
// ascending -- and the entries (k, c) of the row.  Eight lanes own the row, lane j
// its entry c_j.  For every (i, k), taken in the plan's order, the lanes look c_j up
// in row i of C, whose column indices they have staged in LDS, and fetch
// g_j = gC[i, c_j] (0 where C does not store the column):
//
//   grad_B[k, c_j] += A[i, k] * g_j      accumulates in lane j's register: products
//                                        arrive with i ascending, the order of :291-303;
//   grad_A[i, k]    = sum_j g_j * B[k, c_j]  the terms of the batch's entries change places
//                                        through LDS so that lane e holds the eight terms
//                                        of entry e, and adds them in lane order =
//                                        ascending c, the order of the merge in :261-274
//                                        (a column C does not store adds +0.0, which
//                                        changes nothing).
//
// Every stored entry of A lies in exactly one column and every entry of B in
// exactly one row, so each gradient entry is written once, by one lane.
//
// Rows of B with more than 8 entries take several passes over the column of A
// (a pass continues grad_A's sum where the pass before it stopped, so the order
// stays the serial one); rows whose work is far beyond a group's
// (long row of B times long column of A) are left to a second kernel that gives a
// whole workgroup to the row and adds across lanes in tree order (equal to the
// serial order up to rounding).
#include "nm_common.hpp"
#include "nm_transpose.hpp"

namespace {

using nm::kWave;

constexpr int kBlock = 256;
constexpr int G = 8;                 // lanes per row of B
constexpr int kGroups = kBlock / G;  // rows of B per workgroup pass
constexpr int kStage = 256;          // staged column indices of C per group
constexpr int kFast = 32;            // rows of C up to this long: 8 of them staged side by side
// a row of B is "heavy" when (entries of the row) x (entries of A's column) exceeds this:
// 64 passes of a group
constexpr int64_t kHeavy = 64 * G * G;

__device__ __forceinline__ void group_fence() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront"); }

template <typename T> __device__ __forceinline__ T shfl_t(T v, int src) { return __shfl(v, src, kWave); }

template <typename T>
__global__ __launch_bounds__(kBlock) void spgemm_bwd_planned_kernel(
    int64_t B_rows, const T *__restrict__ gC, const int64_t *__restrict__ C_indices,
    const int64_t *__restrict__ C_indptr, const T *__restrict__ A_data, const int32_t *__restrict__ t_indptr,
    const int32_t *__restrict__ t_row, const int32_t *__restrict__ t_perm, const T *__restrict__ B_data,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr, T *__restrict__ grad_A,
    T *__restrict__ grad_B) {
    __shared__ __align__(16) int32_t s_c[kGroups * kStage];
    __shared__ int4 s_rec[kGroups * G];
    __shared__ T s_a[kGroups * G];
    const int gl = threadIdx.x % G, gi = threadIdx.x / G;
    const int gbase = (threadIdx.x & (kWave - 1)) & ~(G - 1);   // first lane of the group in its wavefront
    int32_t *st = s_c + gi * kStage;
    int4 *rec = s_rec + gi * G;
    T *ra = s_a + gi * G;
    const int64_t npass = nm::ceil_div(B_rows, (int64_t)kGroups), npad = nm::xcd_padded(npass);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t pass = nm::xcd_tile(id, npad);
        const int64_t k = pass * kGroups + gi;
        const bool live = pass < npass && k < B_rows;
        const int64_t bb = live ? B_indptr[k] : 0, be = live ? B_indptr[k + 1] : 0;
        const int32_t pb = live ? t_indptr[k] : 0, pe = live ? t_indptr[k + 1] : 0;
        if (!live || (be - bb) * (int64_t)(pe - pb) > kHeavy) continue;   // heavy rows: the wide kernel
        // passes over B's row, 8 entries each (at least one, so that grad_A of a column
        // whose row of B is empty is written as 0)
        int64_t jb = bb;
        do {
            const int64_t my_j = jb + gl;
            const bool have = my_j < be;
            const int64_t c64 = *(have ? B_indices + my_j : B_indptr);
            const T bval_raw = *(have ? B_data + my_j : gC);
            const int32_t c = have ? (int32_t)c64 : -1;
            const T bval = have ? bval_raw : T(0);
            T accB = 0;
            for (int32_t p0 = pb; p0 < pe; p0 += G) {
                // lane l: entry p0 + l of A's column: its row i, its value, the bounds of row i of C
                const int32_t my_p = p0 + gl;
                const bool mine = my_p < pe;
                const int32_t pc = mine ? my_p : pe - 1;
                const int32_t i = t_row[pc], apos = t_perm[pc];
                const T a = mine ? A_data[apos] : T(0);
                const int64_t cb = C_indptr[i], ce = C_indptr[i + 1];
                const int clen = mine ? (int)(ce - cb < 0x7fffffff ? ce - cb : 0x7fffffff) : 0;
                const int nb = pe - p0 < G ? pe - p0 : G;
                // slot = staged entries per row of C: the smallest power of two that holds the
                // longest row of this batch; kStage / slot rows are staged at a time
                int mx = clen;
#pragma unroll
                for (int off = 1; off < G; off <<= 1) mx = max(mx, __shfl_xor(mx, off, kWave));
                int slot = 32, sh = 5;
                while (slot < mx && slot < kStage) slot <<= 1, ++sh;
                const int per = kStage >> sh;         // 8, 4, 2 or 1 rows at a time
                T totalA = 0;                         // lane e keeps the sum of entry e of the batch
                // a later pass over a long row of B goes on from what the passes before it left
                const T prevA = (mine && grad_A && jb != bb) ? grad_A[apos] : T(0);
                if (mx <= kFast) {
                    // The common case: every row of C of the batch has at most 32 entries.
                    // (start, length, A's value) of the 8 rows change hands through LDS once, so that
                    // nothing below needs a cross-lane move.
                    group_fence();
                    rec[gl] = make_int4((int)(cb & 0xffffffffll), (int)(cb >> 32), clen, 0);
                    ra[gl] = a;
                    group_fence();
                    int64_t cbs[G];
                    int lens[G];
#pragma unroll
                    for (int e8 = 0; e8 < G; ++e8) {
                        const int4 r = rec[e8];
                        cbs[e8] = ((int64_t)r.y << 32) | (uint32_t)r.x;
                        lens[e8] = r.z;
                    }
                    // stage the column indices, 32 slots per row, unused slots = +infinity: 16 loads
                    // in flight per lane, twice
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        int32_t got[16];
#pragma unroll
                        for (int r = 0; r < 4; ++r)
#pragma unroll
                            for (int ch = 0; ch < 4; ++ch) {
                                const int e8 = half * 4 + r, t = ch * G + gl;
                                const bool ok = t < lens[e8];
                                const int32_t v = (int32_t) * (ok ? C_indices + cbs[e8] + t : B_indptr);
                                got[r * 4 + ch] = ok ? v : 0x7fffffff;
                            }
#pragma unroll
                        for (int r = 0; r < 4; ++r)
#pragma unroll
                            for (int ch = 0; ch < 4; ++ch) st[(half * 4 + r) * kFast + ch * G + gl] = got[r * 4 + ch];
                    }
                    group_fence();
                    // the column's place in each row: five halving steps without a branch, all rows at once
                    int pos[G];
#pragma unroll
                    for (int e8 = 0; e8 < G; ++e8) pos[e8] = 0;
#pragma unroll
                    for (int step = kFast / 2; step > 0; step >>= 1)
#pragma unroll
                        for (int e8 = 0; e8 < G; ++e8)
                            if (st[e8 * kFast + pos[e8] + step - 1] < c) pos[e8] += step;
                    unsigned hits = 0;
#pragma unroll
                    for (int e8 = 0; e8 < G; ++e8) hits |= (have && st[e8 * kFast + pos[e8]] == c ? 1u : 0u) << e8;
                    T g[G];
#pragma unroll
                    for (int e8 = 0; e8 < G; ++e8) g[e8] = gC[(hits >> e8) & 1u ? cbs[e8] + pos[e8] : 0];
                    group_fence();
                    T *tr = reinterpret_cast<T *>(st);
#pragma unroll
                    for (int e8 = 0; e8 < G; ++e8) {
                        const bool hit = (hits >> e8) & 1u;
                        accB += hit ? ra[e8] * g[e8] : T(0);
                        tr[e8 * G + gl] = hit ? g[e8] * bval : T(0);
                    }
                    group_fence();
                    T run = prevA;
#pragma unroll
                    for (int j = 0; j < G; ++j) run += tr[gl * G + j];
                    totalA = run;
                } else
                for (int e0 = 0; e0 < nb; e0 += per) {
                    const int ne = nb - e0 < per ? nb - e0 : per;   // rows of C of this sub-batch
                    // 1. stage their column indices, slot entries apart: 8 consecutive entries of one
                    //    row per group instruction, 8 such loads in flight per lane (unconditional on a
                    //    clamped position, stored afterwards)
                    group_fence();
                    const int nu = (ne << sh) / G;
                    for (int u0 = 0; u0 < nu; u0 += 8) {
                        int32_t got[8];
#pragma unroll
                        for (int uu = 0; uu < 8; ++uu) {
                            const int f = (u0 + uu) * G;                 // flat staged position of lane 0
                            const int er = f >> sh;                      // row of the sub-batch (group-uniform)
                            const int t = (f & (slot - 1)) + gl;
                            const int src = gbase + e0 + (er < ne ? er : 0);
                            const int64_t cbe = shfl_t(cb, src);
                            const int len = shfl_t(clen, src);
                            const bool ok = er < ne && t < len && len <= kStage;
                            got[uu] = (int32_t) * (ok ? C_indices + cbe + t : B_indptr);
                        }
#pragma unroll
                        for (int uu = 0; uu < 8; ++uu)
                            if (u0 + uu < nu) st[(u0 + uu) * G + gl] = got[uu];
                    }
                    group_fence();
                    // 2. every lane finds its column in each staged row; then the gradients of C at
                    //    those places are requested together
                    int pos[8];
                    unsigned hits = 0;
#pragma unroll
                    for (int e8 = 0; e8 < 8; ++e8) {
                        pos[e8] = 0;
                        if (e8 < ne) {
                            const int64_t cbe = shfl_t(cb, gbase + e0 + e8);
                            const int len = shfl_t(clen, gbase + e0 + e8);
                            int l = 0, h = len;
                            bool hit;
                            if (len <= kStage) {
                                const int32_t *row = st + (e8 << sh);
                                while (l < h) {
                                    const int mid = (l + h) >> 1;
                                    if (row[mid] < c) l = mid + 1; else h = mid;
                                }
                                hit = have && l < len && row[l] == c;
                            } else {
                                // a row of C too long to stage: bisection in memory
                                while (l < h) {
                                    const int mid = (l + h) >> 1;
                                    if (C_indices[cbe + mid] < c64) l = mid + 1; else h = mid;
                                }
                                hit = have && l < len && C_indices[cbe + l] == c64;
                            }
                            pos[e8] = l;
                            hits |= (hit ? 1u : 0u) << e8;
                        }
                    }
                    T g[8];
#pragma unroll
                    for (int e8 = 0; e8 < 8; ++e8) {
                        const int64_t cbe = shfl_t(cb, gbase + e0 + (e8 < ne ? e8 : 0));
                        g[e8] = gC[(hits >> e8) & 1u ? cbe + pos[e8] : 0];   // entry 0 is readable: nnz(C) > 0
                    }
                    // 3. grad_B: this lane's column, rows of C in the plan's order.  grad_A: the terms of
                    //    entry e go to lane e through LDS, which adds them in lane order = ascending column
                    group_fence();
                    T *tr = reinterpret_cast<T *>(st);
#pragma unroll
                    for (int e8 = 0; e8 < 8; ++e8) {
                        const bool hit = (hits >> e8) & 1u;
                        const T ae = shfl_t(a, gbase + e0 + (e8 < ne ? e8 : 0));
                        accB += hit ? ae * g[e8] : T(0);
                        if (e8 < ne) tr[e8 * G + gl] = hit ? g[e8] * bval : T(0);
                    }
                    group_fence();
                    if (gl >= e0 && gl < e0 + ne) {
                        T run = prevA;
#pragma unroll
                        for (int j = 0; j < G; ++j) run += tr[(gl - e0) * G + j];
                        totalA = run;
                    }
                }
                if (mine && grad_A) grad_A[apos] = totalA;
            }
            if (have && grad_B) grad_B[my_j] = accB;
            jb += G;
        } while (jb < be);
    }
}

// Rows of B left out above.  A workgroup owns the row: lanes take the entries of A's column
// (256 at a time), the row's entries c go by one after the other.  grad_A[i, k] accumulates in
// the lane that owns (i, k), in ascending c (exact); grad_B[k, c] is the sum of the lanes'
// products, added in tree order.
template <typename T>
__global__ __launch_bounds__(kBlock) void spgemm_bwd_planned_wide_kernel(
    int64_t B_rows, const T *__restrict__ gC, const int64_t *__restrict__ C_indices,
    const int64_t *__restrict__ C_indptr, const T *__restrict__ A_data, const int32_t *__restrict__ t_indptr,
    const int32_t *__restrict__ t_row, const int32_t *__restrict__ t_perm, const T *__restrict__ B_data,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr, T *__restrict__ grad_A,
    T *__restrict__ grad_B) {
    __shared__ int s_heavy[kBlock];
    __shared__ int s_n;
    __shared__ T s_part[kBlock / kWave];
    const int lane = threadIdx.x & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    for (int64_t k0 = (int64_t)blockIdx.x * kBlock; k0 < B_rows; k0 += (int64_t)gridDim.x * kBlock) {
        // the heavy rows among these 256 (mostly there are none)
        const int64_t kk = k0 + threadIdx.x;
        bool heavy = false;
        if (kk < B_rows)
            heavy = (B_indptr[kk + 1] - B_indptr[kk]) * (int64_t)(t_indptr[kk + 1] - t_indptr[kk]) > kHeavy;
        if (!__syncthreads_or(heavy)) continue;
        if (threadIdx.x == 0) s_n = 0;
        __syncthreads();
        if (heavy) s_heavy[atomicAdd(&s_n, 1)] = threadIdx.x;
        __syncthreads();
        const int n = s_n;
        for (int q = 0; q < n; ++q) {
            const int64_t k = k0 + s_heavy[q];
            const int64_t bb = B_indptr[k], be = B_indptr[k + 1];
            const int32_t pb = t_indptr[k], pe = t_indptr[k + 1];
            for (int32_t p0 = pb; p0 < pe; p0 += kBlock) {
                const int32_t my_p = p0 + threadIdx.x;
                const bool mine = my_p < pe;
                const int32_t pc = mine ? my_p : pe - 1;
                const int32_t i = t_row[pc], apos = t_perm[pc];
                const T a = mine ? A_data[apos] : T(0);
                const int64_t cb = C_indptr[i];
                const int64_t clen = mine ? C_indptr[i + 1] - cb : 0;
                T accA = 0;
                for (int64_t j = bb; j < be; ++j) {
                    const int64_t c = B_indices[j];
                    const T bval = B_data[j];
                    int64_t l = 0, h = clen;
                    while (l < h) {
                        const int64_t mid = (l + h) >> 1;
                        if (C_indices[cb + mid] < c) l = mid + 1; else h = mid;
                    }
                    const bool hit = l < clen && C_indices[cb + l] == c;
                    const T g = hit ? gC[cb + l] : T(0);
                    accA += g * bval;
                    if (grad_B) {                       // uniform
                        const T part = nm::wave_sum(a * g);
                        if (lane == 0) s_part[wave] = part;
                        __syncthreads();
                        if (threadIdx.x == 0) {
                            T tot = 0;
                            for (int w = 0; w < kBlock / kWave; ++w) tot += s_part[w];
                            grad_B[j] = p0 == pb ? tot : grad_B[j] + tot;
                        }
                        __syncthreads();
                    }
                }
                if (mine && grad_A) grad_A[apos] = accA;
            }
            if (pe == pb && grad_B)                     // no entry of A in this column
                for (int64_t j = bb + threadIdx.x; j < be; j += kBlock) grad_B[j] = T(0);
        }
        __syncthreads();
    }
}

template <typename T>
int launch(int64_t B_rows, const void *gC, const int64_t *C_indices, const int64_t *C_indptr, const void *A_data,
           const nm::TPlan &t, const void *B_data, const int64_t *B_indices, const int64_t *B_indptr, void *grad_A,
           void *grad_B, hipStream_t s) {
    int64_t grid = nm::xcd_padded(nm::ceil_div(B_rows, (int64_t)kGroups));
    if (grid > (1 << 20)) grid = 1 << 20;
    hipLaunchKernelGGL(spgemm_bwd_planned_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, B_rows, (const T *)gC,
                       C_indices, C_indptr, (const T *)A_data, t.t_indptr, t.t_row, t.t_perm, (const T *)B_data,
                       B_indices, B_indptr, (T *)grad_A, (T *)grad_B);
    NM_LAUNCH_CHECK("spgemm_bwd_planned_kernel");
    grid = nm::ceil_div(B_rows, (int64_t)kBlock);
    if (grid > 16384) grid = 16384;
    hipLaunchKernelGGL(spgemm_bwd_planned_wide_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, B_rows,
                       (const T *)gC, C_indices, C_indptr, (const T *)A_data, t.t_indptr, t.t_row, t.t_perm,
                       (const T *)B_data, B_indices, B_indptr, (T *)grad_A, (T *)grad_B);
    NM_LAUNCH_CHECK("spgemm_bwd_planned_wide_kernel");
    return NM_OK;
}

}  // namespace

extern "C" int nm_spgemm_backward_planned(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t A_nnz,
                                          int64_t B_nnz, int64_t C_nnz, const void *gC, const int64_t *C_indices,
                                          const int64_t *C_indptr, const void *A_data, const void *A_plan_mem,
                                          const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                                          void *grad_A, void *grad_B, nm_stream stream) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(A_rows >= 0 && A_cols >= 0 && A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    NM_REQUIRE(A_plan_mem && C_indptr && B_indptr, "null pointer argument");
    if (A_cols == 0 || (!grad_A && !grad_B)) return NM_OK;
    hipStream_t s = nm::as_stream(stream);
    if (C_nnz == 0 || A_nnz == 0 || B_nnz == 0) {
        // no product reaches a stored entry of C: both gradients are zero
        if (grad_A && A_nnz > 0) {
            int rc = dt == NM_F32 ? nm::fill_async((float *)grad_A, A_nnz, 0.0f, s)
                                  : nm::fill_async((double *)grad_A, A_nnz, 0.0, s);
            if (rc) return rc;
        }
        if (grad_B && B_nnz > 0) {
            int rc = dt == NM_F32 ? nm::fill_async((float *)grad_B, B_nnz, 0.0f, s)
                                  : nm::fill_async((double *)grad_B, B_nnz, 0.0, s);
            if (rc) return rc;
        }
        return NM_OK;
    }
    NM_REQUIRE(gC && C_indices && A_data && B_data && B_indices, "null pointer argument");
    nm::TPlan t;
    nm::tplan_layout(A_rows, A_cols, A_nnz, const_cast<void *>(A_plan_mem), &t);
    if (dt == NM_F32)
        return launch<float>(A_cols, gC, C_indices, C_indptr, A_data, t, B_data, B_indices, B_indptr, grad_A, grad_B,
                             s);
    return launch<double>(A_cols, gC, C_indices, C_indptr, A_data, t, B_data, B_indices, B_indptr, grad_A, grad_B,
                          s);
}
