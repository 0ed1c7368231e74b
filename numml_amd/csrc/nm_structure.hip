// CSR operations next to the products, all streaming integer and copy work bound
// by HBM bandwidth:
//   explicit transpose            cpp/sparse_csr_cpu.cpp:311-385
//   linear combination aA + bB    cpp/sparse_csr_cpu.cpp:387-560
//   to dense, row sums, diagonal  cpp/sparse_csr_cpu.cpp:1050-1213
#include "nm_scan.hpp"
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

// ---- entry-parallel maps over a CSR matrix ---------------------------------------
//
// A workgroup owns a tile of kTileRows rows.  Row offsets are staged in LDS, the
// row number is spread over the row's entries (by one lane for a short row, by a
// wavefront for a row of kTileWide entries or more), and the entries are then
// processed lane = entry, so the CSR arrays stream through coalesced while every
// entry knows its row.  A tile with more than kTileCap entries is taken in runs of
// consecutive rows that fit; a single row longer than that needs no LDS at all.

constexpr int kTileRows = 256, kTileCap = 4096, kTileWide = 32;
constexpr int32_t kTileHuge = 1 << 30;   // tiles with this many entries: one row per wavefront from global memory

enum MapOp { kToDense, kFromDense, kDiagBack, kRowSpread };

template <typename T, int OP>
__device__ __forceinline__ void map_entry(int64_t row, int64_t k, const int64_t *__restrict__ indices,
                                          const T *__restrict__ src, T *__restrict__ dst, int64_t ld) {
    if (OP == kToDense) dst[row * ld + indices[k]] = src[k];               // A_d[i][j] = data[k]
    if (OP == kFromDense) dst[k] = src[row * ld + indices[k]];             // grad_A[k] = grad_Ad[i][j]
    if (OP == kDiagBack) dst[k] = indices[k] == row ? src[row] : T(0);     // grad_A[k] = g[i] on the diagonal
    if (OP == kRowSpread) dst[k] = src[row];                               // grad_A[k] = g[i]
}

__device__ __forceinline__ void tile_stage_offsets(const int64_t *__restrict__ indptr, int64_t r0, int nr,
                                                   int32_t *s_off) {
    const int64_t base = indptr[r0];
    for (int t = threadIdx.x; t <= nr; t += kBlock) {
        const int64_t d = indptr[r0 + t] - base;
        s_off[t] = (int32_t)(d > kTileHuge ? kTileHuge : d);
    }
}

// Calls f(row within the tile, position in the CSR arrays) for every entry of the tile's
// rows, lane = entry.  Whole workgroup; s_off holds the staged offsets (fewer than
// kTileHuge entries), s_row is scratch for kTileCap entries.
template <typename F>
__device__ __forceinline__ void tile_entries(const int32_t *s_off, uint8_t *s_row, int nr, int64_t base, F f) {
    const int lane = threadIdx.x & 63;
    for (int s0 = 0; s0 < nr;) {
        // rows [s0, e0): the longest run with at most kTileCap entries
        int e0 = nr;
        const int32_t limit = s_off[s0] + kTileCap;
        if (s_off[nr] > limit) {
            int lo = s0, hi = nr;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (s_off[mid] <= limit) lo = mid; else hi = mid;
            }
            e0 = lo;
        }
        if (e0 == s0) {
            const int64_t first = base + s_off[s0];
            const int len = s_off[s0 + 1] - s_off[s0];
            for (int k = threadIdx.x; k < len; k += kBlock) f(s0, first + k);
            s0 += 1;
            continue;
        }
        const int o0 = s_off[s0], cnt = s_off[e0] - o0;
        for (int tb = s0; tb < e0; tb += kBlock) {
            const int t = tb + threadIdx.x;
            const int jb = t < e0 ? s_off[t] - o0 : 0, je = t < e0 ? s_off[t + 1] - o0 : 0;
            const bool wide = je - jb >= kTileWide;
            if (!wide)
                for (int j = jb; j < je; ++j) s_row[j] = (uint8_t)t;
            for (unsigned long long todo = __ballot(wide); todo; todo &= todo - 1) {
                const int src = __builtin_ctzll(todo);
                const int wb = __shfl(jb, src, 64), we = __shfl(je, src, 64);
                const uint8_t row = (uint8_t)__shfl(t, src, 64);
                for (int j = wb + lane; j < we; j += 64) s_row[j] = row;
            }
        }
        __syncthreads();
        const int64_t first = base + o0;
        for (int k = threadIdx.x; k < cnt; k += kBlock) f((int)s_row[k], first + k);
        __syncthreads();
        s0 = e0;
    }
}

template <typename T, int OP>
__global__ __launch_bounds__(kBlock) void entry_map_kernel(int64_t rows, const int64_t *__restrict__ indices,
                                                           const int64_t *__restrict__ indptr,
                                                           const T *__restrict__ src, T *__restrict__ dst,
                                                           int64_t ld) {
    __shared__ int32_t s_off[kTileRows + 1];
    __shared__ uint8_t s_row[kTileCap];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t ntiles = nm::ceil_div(rows, kTileRows), npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t r0 = tile * kTileRows;
        const int nr = (int)(rows - r0 < kTileRows ? rows - r0 : kTileRows);
        const int64_t base = indptr[r0];
        tile_stage_offsets(indptr, r0, nr, s_off);
        __syncthreads();
        if (s_off[nr] < kTileHuge) {
            tile_entries(s_off, s_row, nr, base,
                         [&](int t, int64_t k) { map_entry<T, OP>(r0 + t, k, indices, src, dst, ld); });
        } else {
            for (int t = wave; t < nr; t += kBlock / 64) {
                const int64_t e = indptr[r0 + t + 1];
                for (int64_t k = indptr[r0 + t] + lane; k < e; k += 64)
                    map_entry<T, OP>(r0 + t, k, indices, src, dst, ld);
            }
        }
        __syncthreads();
    }
}

// x[i] = the stored entry (i, i), 0 when row i has none (cpp/sparse_csr_cpu.cpp:1170-1186).
template <typename T>
__global__ __launch_bounds__(kBlock) void diagonal_kernel(int64_t rows, const T *__restrict__ data,
                                                          const int64_t *__restrict__ indices,
                                                          const int64_t *__restrict__ indptr, T *__restrict__ x) {
    __shared__ int32_t s_off[kTileRows + 1];
    __shared__ uint8_t s_row[kTileCap];
    __shared__ T s_x[kTileRows];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t ntiles = nm::ceil_div(rows, kTileRows), npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t r0 = tile * kTileRows;
        const int nr = (int)(rows - r0 < kTileRows ? rows - r0 : kTileRows);
        const int64_t base = indptr[r0];
        tile_stage_offsets(indptr, r0, nr, s_off);
        for (int t = threadIdx.x; t < nr; t += kBlock) s_x[t] = T(0);
        __syncthreads();
        if (s_off[nr] < kTileHuge) {
            tile_entries(s_off, s_row, nr, base, [&](int t, int64_t k) {
                if (indices[k] == r0 + t) s_x[t] = data[k];
            });
        } else {
            for (int t = wave; t < nr; t += kBlock / 64) {
                const int64_t e = indptr[r0 + t + 1];
                for (int64_t k = indptr[r0 + t] + lane; k < e; k += 64)
                    if (indices[k] == r0 + t) s_x[t] = data[k];
            }
        }
        __syncthreads();
        for (int t = threadIdx.x; t < nr; t += kBlock) x[r0 + t] = s_x[t];
        __syncthreads();
    }
}

// ---- linear combination --------------------------------------------------------------
//
// C = alpha A + beta B (cpp/sparse_csr_cpu.cpp:428-468).  A workgroup owns a tile
// of kLcRows rows.  The column indices of both operands' tile are staged in LDS
// with coalesced loads; one lane per row then merges its two sorted lists there
// (the walk is a chain of dependent reads, which LDS serves in ~100 cycles where
// global memory would take a round trip each) and leaves, for every output entry,
// which entry of A and/or of B feeds it.  The output is finally produced lane =
// output entry: values are fetched and C is written through coalesced accesses.
// A tile whose rows hold more than kLcCap entries of either operand is worked off in
// runs of consecutive rows that do fit; a single row that does not is merged by the
// whole workgroup from global memory (every entry finds its place in the output by a
// bisection of the other operand's row and a count of the shared columns before it).

constexpr int kLcRows = 256, kLcCap = 2304;
constexpr int32_t kLcHuge = 1 << 30;   // tiles with this many entries: one lane per row from global memory
constexpr uint32_t kLcNone = 0xffff;

// dst[k] = (int32) src[k] for k < n, by the whole workgroup.  K loads per lane are requested
// before the first is stored (a plain loop waits for every load it has just issued), on
// clamped positions so that no load is predicated.
template <int K>
__device__ __forceinline__ void lc_stage_cols(int32_t *dst, const int64_t *__restrict__ src, int n) {
    for (int k0 = threadIdx.x; k0 < n; k0 += K * kBlock) {
        int64_t v[K];
#pragma unroll
        for (int u = 0; u < K; ++u) v[u] = nm::stream_load(src + (k0 + u * kBlock < n ? k0 + u * kBlock : n - 1));
#pragma unroll
        for (int u = 0; u < K; ++u)
            if (k0 + u * kBlock < n) dst[k0 + u * kBlock] = (int32_t)v[u];
    }
}

struct LcTile {
    int32_t offA[kLcRows + 1], offB[kLcRows + 1], offC[kLcRows + 1];
    int32_t colA[kLcCap], colB[kLcCap];
    uint32_t src[2 * kLcCap];   // per output entry: local index in A (low half) and in B (high half)
};

__device__ __forceinline__ void lc_stage_offsets(const int64_t *__restrict__ indptr, int64_t r0, int nr, int32_t *off) {
    const int64_t base = indptr[r0];
    for (int t = threadIdx.x; t <= nr; t += kBlock) {
        const int64_t d = indptr[r0 + t] - base;
        off[t] = (int32_t)(d > kLcHuge ? kLcHuge : d);
    }
}

// Merge of one row from global memory (fallback); COUNT: length only.
template <typename T, bool COUNT>
__device__ __forceinline__ void lc_row_global(int64_t row, T alpha, const T *__restrict__ A_data,
                                              const int64_t *__restrict__ A_indices,
                                              const int64_t *__restrict__ A_indptr, T beta,
                                              const T *__restrict__ B_data, const int64_t *__restrict__ B_indices,
                                              const int64_t *__restrict__ B_indptr, int64_t *__restrict__ C_indptr,
                                              int64_t *__restrict__ C_indices, T *__restrict__ C_data) {
    int64_t iA = A_indptr[row], iB = B_indptr[row];
    const int64_t eA = A_indptr[row + 1], eB = B_indptr[row + 1];
    int64_t out = COUNT ? 0 : C_indptr[row];
    while (iA < eA && iB < eB) {
        const int64_t cA = A_indices[iA], cB = B_indices[iB];
        if (!COUNT) {
            C_indices[out] = cA < cB ? cA : cB;
            C_data[out] = cA < cB ? alpha * A_data[iA]
                                  : (cA > cB ? beta * B_data[iB] : alpha * A_data[iA] + beta * B_data[iB]);
        }
        iA += cA <= cB;
        iB += cB <= cA;
        ++out;
    }
    if (COUNT) {
        C_indptr[row] = out + (eA - iA) + (eB - iB);
    } else {
        for (; iA < eA; ++iA, ++out) {
            C_indices[out] = A_indices[iA];
            C_data[out] = alpha * A_data[iA];
        }
        for (; iB < eB; ++iB, ++out) {
            C_indices[out] = B_indices[iB];
            C_data[out] = beta * B_data[iB];
        }
    }
}

// End of the run of rows that starts at row s0 of the tile and fits the LDS arrays:
// the largest e in [s0, nr] with at most capA (capB) entries of the first (second)
// operand in rows [s0, e).  e == s0 when row s0 alone is too long.
__device__ __forceinline__ int lc_run_end(const int32_t *offA, const int32_t *offB, int s0, int nr, int capA,
                                          int capB) {
    auto fits = [&](int e) { return offA[e] - offA[s0] <= capA && offB[e] - offB[s0] <= capB; };
    if (fits(nr)) return nr;
    int lo = s0, hi = nr;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (fits(mid)) lo = mid; else hi = mid;
    }
    return lo;
}

// One long row merged by the whole workgroup from global memory.  Output position of
// an entry = entries of its own row before it + entries of the other row below its
// column - columns both rows hold below it.
template <typename T, bool COUNT>
__device__ __forceinline__ void lc_long_row(int64_t row, T alpha, const T *__restrict__ A_data,
                                            const int64_t *__restrict__ A_indices,
                                            const int64_t *__restrict__ A_indptr, T beta,
                                            const T *__restrict__ B_data, const int64_t *__restrict__ B_indices,
                                            const int64_t *__restrict__ B_indptr, int64_t *__restrict__ C_indptr,
                                            int64_t *__restrict__ C_indices, T *__restrict__ C_data,
                                            int64_t *s_scan) {
    const int64_t a0 = A_indptr[row], m = A_indptr[row + 1] - a0;
    const int64_t b0 = B_indptr[row], n = B_indptr[row + 1] - b0;
    const int64_t out0 = COUNT ? 0 : C_indptr[row];
    int64_t shared = 0;
    for (int64_t p0 = 0; p0 < m; p0 += kBlock) {
        const int64_t p = p0 + threadIdx.x;
        const bool have = p < m;
        const int64_t cA = have ? A_indices[a0 + p] : 0;
        int64_t lo = 0, hi = have ? n : 0;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (B_indices[b0 + mid] < cA) lo = mid + 1; else hi = mid;
        }
        const bool both = have && lo < n && B_indices[b0 + lo] == cA;
        int64_t total;
        const int64_t before = nm::block_exclusive_scan(both ? 1 : 0, s_scan, total);
        if (!COUNT && have) {
            const int64_t o = out0 + p + lo - (shared + before);
            const T pa = alpha * A_data[a0 + p];
            C_indices[o] = cA;
            C_data[o] = both ? pa + beta * B_data[b0 + lo] : pa;
        }
        shared += total;
    }
    if (COUNT) {
        if (threadIdx.x == 0) C_indptr[row] = m + n - shared;
        return;
    }
    shared = 0;
    for (int64_t q0 = 0; q0 < n; q0 += kBlock) {
        const int64_t q = q0 + threadIdx.x;
        const bool have = q < n;
        const int64_t cB = have ? B_indices[b0 + q] : 0;
        int64_t lo = 0, hi = have ? m : 0;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (A_indices[a0 + mid] < cB) lo = mid + 1; else hi = mid;
        }
        const bool both = have && lo < m && A_indices[a0 + lo] == cB;
        int64_t total;
        const int64_t before = nm::block_exclusive_scan(both ? 1 : 0, s_scan, total);
        if (have && !both) {
            const int64_t o = out0 + q + lo - (shared + before);
            C_indices[o] = cB;
            C_data[o] = beta * B_data[b0 + q];
        }
        shared += total;
    }
}

template <typename T, bool COUNT>
__global__ __launch_bounds__(kBlock) void lincomb_kernel(int64_t rows, T alpha, const T *__restrict__ A_data,
                                                         const int64_t *__restrict__ A_indices,
                                                         const int64_t *__restrict__ A_indptr, T beta,
                                                         const T *__restrict__ B_data,
                                                         const int64_t *__restrict__ B_indices,
                                                         const int64_t *__restrict__ B_indptr,
                                                         int64_t *__restrict__ C_indptr,
                                                         int64_t *__restrict__ C_indices, T *__restrict__ C_data) {
    __shared__ LcTile s;
    __shared__ int64_t s_scan[kBlock / nm::kWave];
    const int64_t ntiles = nm::ceil_div(rows, kLcRows), npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t r0 = tile * kLcRows;
        const int nr = (int)(rows - r0 < kLcRows ? rows - r0 : kLcRows);
        const int64_t baseA = A_indptr[r0], baseB = B_indptr[r0];
        lc_stage_offsets(A_indptr, r0, nr, s.offA);
        lc_stage_offsets(B_indptr, r0, nr, s.offB);
        __syncthreads();
        if (s.offA[nr] >= kLcHuge || s.offB[nr] >= kLcHuge) {
            for (int t = threadIdx.x; t < nr; t += kBlock)
                lc_row_global<T, COUNT>(r0 + t, alpha, A_data, A_indices, A_indptr, beta, B_data, B_indices, B_indptr,
                                        C_indptr, C_indices, C_data);
            __syncthreads();
            continue;
        }
        // rows [s0, e0) of the tile through LDS; WHOLE: the whole tile (s0 == 0), the common
        // case, compiled without the run's offsets
        auto run = [&](auto whole, const int s0, const int e0) {
            constexpr bool WHOLE = decltype(whole)::value;
            const int n = e0 - s0, a0 = WHOLE ? 0 : s.offA[s0], b0 = WHOLE ? 0 : s.offB[s0];
            const int nA = s.offA[e0] - a0, nB = s.offB[e0] - b0;
            const int64_t rs = r0 + s0, gA = baseA + a0, gB = baseB + b0;
            lc_stage_cols<5>(s.colA, A_indices + gA, nA);
            lc_stage_cols<5>(s.colB, B_indices + gB, nB);
            const int64_t gC = COUNT ? 0 : C_indptr[rs];
            if (!COUNT)
                for (int t = threadIdx.x; t <= n; t += kBlock) s.offC[t] = (int32_t)(C_indptr[rs + t] - gC);
            __syncthreads();
            for (int t = threadIdx.x; t < n; t += kBlock) {
                int iA = s.offA[s0 + t] - a0, iB = s.offB[s0 + t] - b0;
                const int eA = s.offA[s0 + t + 1] - a0, eB = s.offB[s0 + t + 1] - b0;
                int out = COUNT ? 0 : s.offC[t];
                while (iA < eA && iB < eB) {
                    const int32_t cA = s.colA[iA], cB = s.colB[iB];
                    if (!COUNT) s.src[out] = (cA <= cB ? (uint32_t)iA : kLcNone) | ((cB <= cA ? (uint32_t)iB : kLcNone) << 16);
                    iA += cA <= cB;
                    iB += cB <= cA;
                    ++out;
                }
                if (COUNT) {
                    C_indptr[rs + t] = out + (eA - iA) + (eB - iB);
                } else {
                    for (; iA < eA; ++iA, ++out) s.src[out] = (uint32_t)iA | (kLcNone << 16);
                    for (; iB < eB; ++iB, ++out) s.src[out] = kLcNone | ((uint32_t)iB << 16);
                }
            }
            if (!COUNT) {
                __syncthreads();
                const int nC = s.offC[n];
                // K output entries per lane: their operand values are requested together and
                // unconditionally (an operand that is absent reads entry 0 of a run that has one
                // and is dropped by the select), then combined and stored.
                constexpr int K = 5;
                const T *__restrict__ Ad = nA > 0 ? A_data + gA : B_data + gB;
                const T *__restrict__ Bd = nB > 0 ? B_data + gB : A_data + gA;
                for (int o0 = threadIdx.x; o0 < nC; o0 += K * kBlock) {
                    uint32_t ia[K], ib[K];
                    T va[K], vb[K];
#pragma unroll
                    for (int u = 0; u < K; ++u) {
                        const uint32_t sr = s.src[o0 + u * kBlock < nC ? o0 + u * kBlock : nC - 1];
                        ia[u] = sr & 0xffff;
                        ib[u] = sr >> 16;
                        va[u] = Ad[ia[u] == kLcNone ? 0u : ia[u]];
                        vb[u] = Bd[ib[u] == kLcNone ? 0u : ib[u]];
                    }
#pragma unroll
                    for (int u = 0; u < K; ++u) {
                        const int o = o0 + u * kBlock;
                        if (o >= nC) break;
                        const T pa = alpha * va[u], pb = beta * vb[u];
                        const T v = ib[u] == kLcNone ? pa : (ia[u] == kLcNone ? pb : pa + pb);
                        const int32_t c = ia[u] == kLcNone ? s.colB[ib[u]] : s.colA[ia[u]];
                        nm::stream_store(C_indices + gC + o, (int64_t)c);
                        nm::stream_store(C_data + gC + o, v);
                    }
                }
            }
            __syncthreads();
        };
        if (lc_run_end(s.offA, s.offB, 0, nr, kLcCap, kLcCap) == nr) {
            run(std::true_type{}, 0, nr);
            continue;
        }
        for (int s0 = 0; s0 < nr;) {
            const int e0 = lc_run_end(s.offA, s.offB, s0, nr, kLcCap, kLcCap);
            if (e0 == s0) {
                lc_long_row<T, COUNT>(r0 + s0, alpha, A_data, A_indices, A_indptr, beta, B_data, B_indices, B_indptr,
                                      C_indptr, C_indices, C_data, s_scan);
                s0 += 1;
                continue;
            }
            run(std::false_type{}, s0, e0);
            s0 = e0;
        }
    }
}

// grad_X[k] = coef * grad_C at the same coordinate (cpp/sparse_csr_cpu.cpp:505-552).
// Every column of X is present in C.  Same tiling and the same runs of rows: columns
// of X and of C staged in LDS, one lane per row marks the row of its entries of X, then
// lane = entry of X finds its column in the row of C by bisection in LDS, gathers and
// scales.  A row too long for LDS is searched in global memory by the whole workgroup.
template <typename T>
__global__ __launch_bounds__(kBlock) void lincomb_back_kernel(int64_t rows, T coef,
                                                              const int64_t *__restrict__ X_indices,
                                                              const int64_t *__restrict__ X_indptr,
                                                              const T *__restrict__ gC,
                                                              const int64_t *__restrict__ C_indices,
                                                              const int64_t *__restrict__ C_indptr,
                                                              T *__restrict__ grad_X) {
    __shared__ int32_t s_offX[kLcRows + 1], s_offC[kLcRows + 1];
    __shared__ int32_t s_colX[kLcCap], s_colC[2 * kLcCap], s_match[kLcCap];
    const int64_t ntiles = nm::ceil_div(rows, kLcRows), npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t r0 = tile * kLcRows;
        const int nr = (int)(rows - r0 < kLcRows ? rows - r0 : kLcRows);
        const int64_t baseX = X_indptr[r0], baseC = C_indptr[r0];
        lc_stage_offsets(X_indptr, r0, nr, s_offX);
        lc_stage_offsets(C_indptr, r0, nr, s_offC);
        __syncthreads();
        if (s_offX[nr] >= kLcHuge || s_offC[nr] >= kLcHuge) {
            for (int t = threadIdx.x; t < nr; t += kBlock) {
                int64_t iX = X_indptr[r0 + t], iC = C_indptr[r0 + t];
                const int64_t eX = X_indptr[r0 + t + 1], eC = C_indptr[r0 + t + 1];
                while (iX < eX && iC < eC) {
                    const int64_t cX = X_indices[iX], cC = C_indices[iC];
                    if (cX == cC) grad_X[iX] = gC[iC] * coef;
                    iX += cX <= cC;
                    iC += cC <= cX;
                }
            }
            __syncthreads();
            continue;
        }
        for (int s0 = 0; s0 < nr;) {
            const int e0 = lc_run_end(s_offX, s_offC, s0, nr, kLcCap, 2 * kLcCap);
            if (e0 == s0) {
                // one long row: every entry of X searches the row of C in global memory
                const int64_t x0 = baseX + s_offX[s0], m = s_offX[s0 + 1] - s_offX[s0];
                const int64_t c0 = baseC + s_offC[s0], n = s_offC[s0 + 1] - s_offC[s0];
                for (int64_t k = threadIdx.x; k < m; k += kBlock) {
                    const int64_t cX = X_indices[x0 + k];
                    int64_t lo = 0, hi = n;
                    while (lo < hi) {
                        const int64_t mid = (lo + hi) >> 1;
                        if (C_indices[c0 + mid] < cX) lo = mid + 1; else hi = mid;
                    }
                    if (lo < n && C_indices[c0 + lo] == cX) grad_X[x0 + k] = gC[c0 + lo] * coef;
                }
                s0 += 1;
                continue;
            }
            // rows [s0, e0) of the tile through LDS
            const int xo = s_offX[s0], co = s_offC[s0];
            const int nX = s_offX[e0] - xo, nC = s_offC[e0] - co;
            const int64_t gX = baseX + xo, gCb = baseC + co;
            lc_stage_cols<5>(s_colX, X_indices + gX, nX);
            lc_stage_cols<5>(s_colC, C_indices + gCb, nC);
            __syncthreads();
            // row of every entry of X: one lane per row marks its entries
            for (int t = s0 + threadIdx.x; t < e0; t += kBlock) {
                const int eX = s_offX[t + 1] - xo;
                for (int k = s_offX[t] - xo; k < eX; ++k) s_match[k] = t;
            }
            __syncthreads();
            // lane = entry of X: bisection for its column in the same row of C; K entries per
            // lane so that K independent searches and then K gathers are in flight
            constexpr int K = 5;
            for (int k0 = threadIdx.x; k0 < nX; k0 += K * kBlock) {
                int at[K];
                bool found[K];
#pragma unroll
                for (int u = 0; u < K; ++u) {
                    const int k = k0 + u * kBlock < nX ? k0 + u * kBlock : nX - 1;
                    const int t = s_match[k];
                    const int32_t cX = s_colX[k];
                    int lo = s_offC[t] - co, hi = s_offC[t + 1] - co;
                    const int end = hi;
                    while (lo < hi) {
                        const int mid = (lo + hi) >> 1;
                        if (s_colC[mid] < cX) lo = mid + 1; else hi = mid;
                    }
                    found[u] = lo < end && s_colC[lo] == cX;   // always, for valid input
                    at[u] = found[u] ? lo : 0;
                }
                T gv[K];
#pragma unroll
                for (int u = 0; u < K; ++u) gv[u] = nC > 0 ? gC[gCb + at[u]] : T(0);
#pragma unroll
                for (int u = 0; u < K; ++u)
                    if (k0 + u * kBlock < nX && found[u]) nm::stream_store(grad_X + gX + k0 + u * kBlock, gv[u] * coef);
            }
            __syncthreads();
            s0 = e0;
        }
    }
}

inline unsigned lc_grid(int64_t rows) {
    int64_t g = nm::xcd_padded(nm::ceil_div(rows, kLcRows));
    if (g > nm::kMaxGrid) g = nm::kMaxGrid;
    return (unsigned)g;
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
    nm::tplan_layout(rows, cols, nnz, const_cast<void *>(plan_mem), &plan);
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

// ---- C ABI of the maps -------------------------------------------------------------

namespace {

template <typename T, int OP>
int launch_map(int64_t rows, const int64_t *indices, const int64_t *indptr, const void *src, void *dst, int64_t ld,
               hipStream_t s) {
    int64_t grid = nm::xcd_padded(nm::ceil_div(rows, kTileRows));
    if (grid > nm::kMaxGrid) grid = nm::kMaxGrid;
    hipLaunchKernelGGL((entry_map_kernel<T, OP>), dim3((unsigned)grid), dim3(kBlock), 0, s, rows, indices, indptr,
                       (const T *)src, (T *)dst, ld);
    NM_LAUNCH_CHECK("entry_map_kernel");
    return NM_OK;
}

template <int OP>
int map_entry_point(nm_dtype dt, int64_t rows, int64_t nnz, const int64_t *indices, const int64_t *indptr,
                    const void *src, void *dst, int64_t ld, nm_stream stream) {
    NM_REQUIRE(rows >= 0 && nnz >= 0, "negative size");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    if (rows == 0 || nnz == 0) return NM_OK;
    NM_REQUIRE(indptr && src && dst && (OP == kRowSpread || indices), "null pointer argument");
    if (dt == NM_F32) return launch_map<float, OP>(rows, indices, indptr, src, dst, ld, nm::as_stream(stream));
    return launch_map<double, OP>(rows, indices, indptr, src, dst, ld, nm::as_stream(stream));
}

}  // namespace

extern "C" int nm_csr_to_dense_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                       const int64_t *indices, const int64_t *indptr, void *dense, int64_t ld,
                                       nm_stream stream) {
    NM_REQUIRE(rows >= 0 && cols >= 0 && ld >= cols, "bad dense shape");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    NM_REQUIRE(rows == 0 || cols == 0 || dense, "null pointer argument");
    hipStream_t s = nm::as_stream(stream);
    if (ld == cols) {
        const int rc = dt == NM_F32 ? nm::fill_async((float *)dense, rows * cols, 0.0f, s)
                                    : nm::fill_async((double *)dense, rows * cols, 0.0, s);
        if (rc) return rc;
    } else {
        for (int64_t r = 0; r < rows; ++r) {   // strided output: row by row (rare)
            const int rc = dt == NM_F32 ? nm::fill_async((float *)dense + r * ld, cols, 0.0f, s)
                                        : nm::fill_async((double *)dense + r * ld, cols, 0.0, s);
            if (rc) return rc;
        }
    }
    return map_entry_point<kToDense>(dt, rows, nnz, indices, indptr, data, dense, ld, stream);
}

extern "C" int nm_csr_to_dense_backward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *grad_dense,
                                        int64_t ld, const int64_t *indices, const int64_t *indptr, void *grad_A,
                                        nm_stream stream) {
    NM_REQUIRE(cols >= 0 && ld >= cols, "bad dense shape");
    return map_entry_point<kFromDense>(dt, rows, nnz, indices, indptr, grad_dense, grad_A, ld, stream);
}

extern "C" int nm_csr_row_sum_backward(nm_dtype dt, int64_t rows, int64_t nnz, const int64_t *indptr, const void *g,
                                       void *grad_A, nm_stream stream) {
    return map_entry_point<kRowSpread>(dt, rows, nnz, nullptr, indptr, g, grad_A, 0, stream);
}

extern "C" int nm_csr_extract_diagonal_backward(nm_dtype dt, int64_t rows, int64_t nnz, const int64_t *indices,
                                                const int64_t *indptr, const void *g, void *grad_A,
                                                nm_stream stream) {
    return map_entry_point<kDiagBack>(dt, rows, nnz, indices, indptr, g, grad_A, 0, stream);
}

extern "C" int nm_csr_extract_diagonal_forward(nm_dtype dt, int64_t rows, int64_t nnz, const void *data,
                                               const int64_t *indices, const int64_t *indptr, void *x,
                                               nm_stream stream) {
    NM_REQUIRE(rows >= 0 && nnz >= 0, "negative size");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    if (rows == 0) return NM_OK;
    NM_REQUIRE(indptr && x && (nnz == 0 || (data && indices)), "null pointer argument");
    int64_t grid = nm::xcd_padded(nm::ceil_div(rows, kTileRows));
    if (grid > nm::kMaxGrid) grid = nm::kMaxGrid;
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F32)
        hipLaunchKernelGGL(diagonal_kernel<float>, dim3((unsigned)grid), dim3(kBlock), 0, s, rows,
                           (const float *)data, indices, indptr, (float *)x);
    else
        hipLaunchKernelGGL(diagonal_kernel<double>, dim3((unsigned)grid), dim3(kBlock), 0, s, rows,
                           (const double *)data, indices, indptr, (double *)x);
    NM_LAUNCH_CHECK("diagonal_kernel");
    return NM_OK;
}

// ---- C ABI of the linear combination ---------------------------------------------

extern "C" int nm_splincomb_workspace_bytes(int64_t rows, size_t *bytes) {
    NM_REQUIRE(bytes && rows >= 0, "bad argument");
    *bytes = nm::scan_scratch_bytes(rows + 1);
    return NM_OK;
}

extern "C" int nm_splincomb_symbolic(int64_t rows, const int64_t *A_indices, const int64_t *A_indptr,
                                     const int64_t *B_indices, const int64_t *B_indptr, int64_t *C_indptr,
                                     void *workspace, size_t workspace_bytes, nm_stream stream) {
    NM_REQUIRE(rows >= 0, "negative size");
    NM_REQUIRE(A_indptr && B_indptr && C_indptr && workspace, "null pointer argument");
    if (workspace_bytes < nm::scan_scratch_bytes(rows + 1))
        return nm::fail(NM_ERR_WORKSPACE, "workspace of %zu bytes, %zu needed", workspace_bytes,
                        nm::scan_scratch_bytes(rows + 1));
    hipStream_t s = nm::as_stream(stream);
    if (int rc = nm::fill_async(C_indptr + rows, 1, (int64_t)0, s)) return rc;
    if (rows == 0) return NM_OK;
    hipLaunchKernelGGL((lincomb_kernel<float, true>), dim3(lc_grid(rows)), dim3(kBlock), 0, s, rows, 0.0f,
                       (const float *)nullptr, A_indices, A_indptr, 0.0f, (const float *)nullptr, B_indices,
                       B_indptr, C_indptr, (int64_t *)nullptr, (float *)nullptr);
    NM_LAUNCH_CHECK("lincomb_kernel<count>");
    return nm::scan_exclusive_i64(C_indptr, rows + 1, (int64_t *)workspace, s);
}

extern "C" int nm_splincomb_numeric(nm_dtype dt, int64_t rows, double alpha, const void *A_data,
                                    const int64_t *A_indices, const int64_t *A_indptr, double beta,
                                    const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                                    const int64_t *C_indptr, int64_t *C_indices, void *C_data, nm_stream stream) {
    NM_REQUIRE(rows >= 0, "negative size");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    if (rows == 0) return NM_OK;
    NM_REQUIRE(A_indptr && B_indptr && C_indptr, "null pointer argument");
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F32)
        hipLaunchKernelGGL((lincomb_kernel<float, false>), dim3(lc_grid(rows)), dim3(kBlock), 0, s, rows,
                           (float)alpha, (const float *)A_data, A_indices, A_indptr, (float)beta,
                           (const float *)B_data, B_indices, B_indptr, const_cast<int64_t *>(C_indptr), C_indices,
                           (float *)C_data);
    else
        hipLaunchKernelGGL((lincomb_kernel<double, false>), dim3(lc_grid(rows)), dim3(kBlock), 0, s, rows, alpha,
                           (const double *)A_data, A_indices, A_indptr, beta, (const double *)B_data, B_indices,
                           B_indptr, const_cast<int64_t *>(C_indptr), C_indices, (double *)C_data);
    NM_LAUNCH_CHECK("lincomb_kernel");
    return NM_OK;
}

extern "C" int nm_splincomb_backward(nm_dtype dt, int64_t rows, double alpha, const int64_t *A_indices,
                                     const int64_t *A_indptr, double beta, const int64_t *B_indices,
                                     const int64_t *B_indptr, const void *grad_C, const int64_t *C_indices,
                                     const int64_t *C_indptr, void *grad_A, void *grad_B, nm_stream stream) {
    NM_REQUIRE(rows >= 0, "negative size");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    if (rows == 0) return NM_OK;
    NM_REQUIRE(C_indptr, "null pointer argument");
    hipStream_t s = nm::as_stream(stream);
    const unsigned grid = lc_grid(rows);
    for (int side = 0; side < 2; ++side) {
        void *out = side == 0 ? grad_A : grad_B;
        if (!out) continue;
        const int64_t *ind = side == 0 ? A_indices : B_indices, *ptr = side == 0 ? A_indptr : B_indptr;
        const double coef = side == 0 ? alpha : beta;
        NM_REQUIRE(ptr != nullptr, "null pointer argument");
        if (dt == NM_F32)
            hipLaunchKernelGGL(lincomb_back_kernel<float>, dim3(grid), dim3(kBlock), 0, s, rows, (float)coef, ind,
                               ptr, (const float *)grad_C, C_indices, C_indptr, (float *)out);
        else
            hipLaunchKernelGGL(lincomb_back_kernel<double>, dim3(grid), dim3(kBlock), 0, s, rows, coef, ind, ptr,
                               (const double *)grad_C, C_indices, C_indptr, (double *)out);
        NM_LAUNCH_CHECK("lincomb_back_kernel");
    }
    return NM_OK;
}

// ---- the linear combination on cached maps ---------------------------------------
//
// For two patterns that stay the same while the values change (A - B in every iteration of a
// loop) the merge of the two rows is done once: the plan holds, all int32,
//
//   srcA[o], srcB[o]   the entry of A / of B at the coordinate of the o-th entry of C, -1 for none
//   posA[k], posB[k]   the entry of C at the coordinate of the k-th entry of A / of B
//
// after which the forward is one pass over C (two map streams, two gathers that run forward
// through the operands, one store) and each gradient one gather -- no symbolic phase, no read of
// nnz(C) by the host, no search.  The values are formed as the merge forms them
// (cpp/sparse_csr_cpu.cpp:431-468): alpha * a, beta * b, or the sum of the two.

namespace {

struct LcPlan {
    int32_t *srcA, *srcB, *posA, *posB;
};

size_t lcplan_layout(int64_t A_nnz, int64_t B_nnz, int64_t C_nnz, void *base, LcPlan *p) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += nm::align256(bytes);
        return (int32_t *)q;
    };
    int32_t *sa = take((size_t)(C_nnz + 1) * 4), *sb = take((size_t)(C_nnz + 1) * 4);
    int32_t *pa = take((size_t)(A_nnz + 1) * 4), *pb = take((size_t)(B_nnz + 1) * 4);
    if (p) *p = LcPlan{sa, sb, pa, pb};
    return off;
}

constexpr int kMapLanes = 8;   // lanes per row of the map build

// Eight lanes per row: lane k takes entries k, k + 8, ... of the row of X and finds each one's
// column in the row of C by bisection.
__global__ __launch_bounds__(kBlock) void lincomb_map_kernel(int64_t rows, const int64_t *__restrict__ X_indices,
                                                             const int64_t *__restrict__ X_indptr,
                                                             const int64_t *__restrict__ C_indices,
                                                             const int64_t *__restrict__ C_indptr,
                                                             int32_t *__restrict__ src, int32_t *__restrict__ pos) {
    constexpr int kGroups = kBlock / kMapLanes;
    constexpr int64_t kLongMapRow = 2048;   // rows of X from here on are shared by the whole workgroup
    const int k = threadIdx.x & (kMapLanes - 1), g = threadIdx.x / kMapLanes;
    auto place = [&](const int64_t e, const int64_t cs, const int64_t ce) {
        const int64_t col = X_indices[e];
        int64_t lo = cs, hi = ce;
        while (lo < hi) {
            const int64_t mid = (lo + hi) >> 1;
            if (C_indices[mid] < col) lo = mid + 1; else hi = mid;
        }
        const bool found = lo < ce && C_indices[lo] == col;   // always, when C is the union of the patterns
        pos[e] = (int32_t)(found ? lo : (cs < ce ? cs : 0));
        if (found) src[lo] = (int32_t)e;
    };
    for (int64_t row0 = (int64_t)blockIdx.x * kGroups; row0 < rows; row0 += (int64_t)gridDim.x * kGroups) {
        const int64_t row = row0 + g;
        if (row < rows) {
            const int64_t xb = X_indptr[row], xe = X_indptr[row + 1];
            if (xe - xb < kLongMapRow) {
                const int64_t cs = C_indptr[row], ce = C_indptr[row + 1];
                for (int64_t e = xb + k; e < xe; e += kMapLanes) place(e, cs, ce);
            }
        }
        // the long rows among these (eight lanes took 0.3 s over a row of 2^19 entries)
        for (int g2 = 0; g2 < kGroups && row0 + g2 < rows; ++g2) {
            const int64_t xb = X_indptr[row0 + g2], xe = X_indptr[row0 + g2 + 1];
            if (xe - xb < kLongMapRow) continue;
            const int64_t cs = C_indptr[row0 + g2], ce = C_indptr[row0 + g2 + 1];
            for (int64_t e = xb + threadIdx.x; e < xe; e += kBlock) place(e, cs, ce);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void lincomb_planned_kernel(int64_t C_nnz, T alpha, const T *__restrict__ A_data,
                                                                 T beta, const T *__restrict__ B_data,
                                                                 const int32_t *__restrict__ srcA,
                                                                 const int32_t *__restrict__ srcB,
                                                                 T *__restrict__ C_data) {
    constexpr int K = 4;
    const int64_t stride = (int64_t)gridDim.x * kBlock * K;
    for (int64_t o0 = (int64_t)blockIdx.x * kBlock * K + threadIdx.x; o0 < C_nnz; o0 += stride) {
        int32_t ia[K], ib[K];
        T va[K], vb[K];
#pragma unroll
        for (int u = 0; u < K; ++u) {
            const int64_t o = o0 + u * kBlock < C_nnz ? o0 + u * kBlock : C_nnz - 1;
            ia[u] = nm::stream_load(srcA + o);
            ib[u] = nm::stream_load(srcB + o);
        }
#pragma unroll
        for (int u = 0; u < K; ++u) {
            va[u] = ia[u] >= 0 ? A_data[ia[u]] : T(0);
            vb[u] = ib[u] >= 0 ? B_data[ib[u]] : T(0);
        }
#pragma unroll
        for (int u = 0; u < K; ++u) {
            const int64_t o = o0 + u * kBlock;
            if (o >= C_nnz) break;
            const T pa = alpha * va[u], pb = beta * vb[u];
            nm::stream_store(C_data + o, ib[u] < 0 ? pa : (ia[u] < 0 ? pb : pa + pb));
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void lincomb_back_planned_kernel(int64_t X_nnz, T coef, const T *__restrict__ gC,
                                                                      const int32_t *__restrict__ pos,
                                                                      T *__restrict__ grad_X) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t k = (int64_t)blockIdx.x * kBlock + threadIdx.x; k < X_nnz; k += stride)
        nm::stream_store(grad_X + k, coef * gC[nm::stream_load(pos + k)]);
}

unsigned flat_grid(int64_t n, int per_block) {
    int64_t g = nm::ceil_div(n, (int64_t)per_block);
    return (unsigned)(g > 65536 ? 65536 : (g < 1 ? 1 : g));
}

}  // namespace

extern "C" int nm_splincomb_plan_bytes(int64_t A_nnz, int64_t B_nnz, int64_t C_nnz, size_t *plan_bytes) {
    NM_REQUIRE(plan_bytes && A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "bad argument");
    *plan_bytes = lcplan_layout(A_nnz, B_nnz, C_nnz, nullptr, nullptr);
    return NM_OK;
}

extern "C" int nm_splincomb_plan_build(int64_t rows, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                                       const int64_t *A_indices, const int64_t *A_indptr, const int64_t *B_indices,
                                       const int64_t *B_indptr, const int64_t *C_indices, const int64_t *C_indptr,
                                       void *plan_mem, size_t plan_bytes, nm_stream stream) {
    NM_REQUIRE(rows >= 0 && A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    const int64_t lim = (int64_t)1 << 31;
    if (A_nnz >= lim || B_nnz >= lim || C_nnz >= lim)
        return nm::fail(NM_ERR_UNSUPPORTED, "the maps of a linear combination hold positions in 32 bits");
    NM_REQUIRE(plan_mem && A_indptr && B_indptr && C_indptr, "null pointer argument");
    NM_REQUIRE((A_nnz == 0 || A_indices) && (B_nnz == 0 || B_indices) && (C_nnz == 0 || C_indices),
               "null pointer argument");
    const size_t need = lcplan_layout(A_nnz, B_nnz, C_nnz, nullptr, nullptr);
    if (plan_bytes < need) return nm::fail(NM_ERR_WORKSPACE, "plan of %zu bytes, %zu needed", plan_bytes, need);
    LcPlan p;
    lcplan_layout(A_nnz, B_nnz, C_nnz, plan_mem, &p);
    hipStream_t s = nm::as_stream(stream);
    if (int rc = nm::fill_async(p.srcA, C_nnz, (int32_t)-1, s)) return rc;
    if (int rc = nm::fill_async(p.srcB, C_nnz, (int32_t)-1, s)) return rc;
    if (rows == 0) return NM_OK;
    const unsigned grid = flat_grid(rows, kBlock / kMapLanes);
    if (A_nnz > 0) {
        hipLaunchKernelGGL(lincomb_map_kernel, dim3(grid), dim3(kBlock), 0, s, rows, A_indices, A_indptr, C_indices,
                           C_indptr, p.srcA, p.posA);
        NM_LAUNCH_CHECK("lincomb_map_kernel");
    }
    if (B_nnz > 0) {
        hipLaunchKernelGGL(lincomb_map_kernel, dim3(grid), dim3(kBlock), 0, s, rows, B_indices, B_indptr, C_indices,
                           C_indptr, p.srcB, p.posB);
        NM_LAUNCH_CHECK("lincomb_map_kernel");
    }
    return NM_OK;
}

extern "C" int nm_splincomb_numeric_planned(nm_dtype dt, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz, double alpha,
                                            const void *A_data, double beta, const void *B_data,
                                            const void *plan_mem, void *C_data, nm_stream stream) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    NM_REQUIRE(A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    if (C_nnz == 0) return NM_OK;
    NM_REQUIRE(plan_mem && C_data && (A_nnz == 0 || A_data) && (B_nnz == 0 || B_data), "null pointer argument");
    LcPlan p;
    lcplan_layout(A_nnz, B_nnz, C_nnz, const_cast<void *>(plan_mem), &p);
    hipStream_t s = nm::as_stream(stream);
    const unsigned grid = flat_grid(C_nnz, kBlock * 4);
    if (dt == NM_F32)
        hipLaunchKernelGGL(lincomb_planned_kernel<float>, dim3(grid), dim3(kBlock), 0, s, C_nnz, (float)alpha,
                           (const float *)A_data, (float)beta, (const float *)B_data, p.srcA, p.srcB, (float *)C_data);
    else
        hipLaunchKernelGGL(lincomb_planned_kernel<double>, dim3(grid), dim3(kBlock), 0, s, C_nnz, alpha,
                           (const double *)A_data, beta, (const double *)B_data, p.srcA, p.srcB, (double *)C_data);
    NM_LAUNCH_CHECK("lincomb_planned_kernel");
    return NM_OK;
}

extern "C" int nm_splincomb_backward_planned(nm_dtype dt, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz, double alpha,
                                             double beta, const void *grad_C, const void *plan_mem, void *grad_A,
                                             void *grad_B, nm_stream stream) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "bad dtype %d", (int)dt);
    NM_REQUIRE(A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    NM_REQUIRE(plan_mem != nullptr, "null plan");
    LcPlan p;
    lcplan_layout(A_nnz, B_nnz, C_nnz, const_cast<void *>(plan_mem), &p);
    hipStream_t s = nm::as_stream(stream);
    for (int side = 0; side < 2; ++side) {
        void *out = side == 0 ? grad_A : grad_B;
        const int64_t n = side == 0 ? A_nnz : B_nnz;
        if (!out || n == 0) continue;
        NM_REQUIRE(grad_C != nullptr, "grad_C is null");   // an operand with entries: C has entries
        const int32_t *pos = side == 0 ? p.posA : p.posB;
        const double coef = side == 0 ? alpha : beta;
        const unsigned grid = flat_grid(n, kBlock);
        if (dt == NM_F32)
            hipLaunchKernelGGL(lincomb_back_planned_kernel<float>, dim3(grid), dim3(kBlock), 0, s, n, (float)coef,
                               (const float *)grad_C, pos, (float *)out);
        else
            hipLaunchKernelGGL(lincomb_back_planned_kernel<double>, dim3(grid), dim3(kBlock), 0, s, n, coef,
                               (const double *)grad_C, pos, (double *)out);
        NM_LAUNCH_CHECK("lincomb_back_planned_kernel");
    }
    return NM_OK;
}
