// Product plan of a sparse product C = A B: what the numeric work needs to know about
// the three patterns, computed once per pair of patterns and reused for as long as only the
// VALUES of A and B change (a training loop over a fixed hierarchy, the reference's own use).
// The reference redoes the symbolic work on every call (cpp/sparse_csr_gemm_cuda.cu:10-302 on
// the device, the std::map rows of cpp/sparse_csr_cpu.cpp:177-214 on the host) and searches C
// again in every backward pass (cpp/sparse_csr_cpu.cpp:246-303); with a plan neither happens.
//
// Per stored entry e = (i, j) of A the plan holds
//
//   bstart[e]   where row j of B starts                                   (int32)
//   cstart[e]   where row i of C starts                                   (int32)
//   dest[e]     eight bytes: byte k is the position inside row i of C of the column of the
//               k-th entry of row j of B, 0xFF when that row has no k-th entry
//
// so that the product a_e * b_(j,k) is known to belong to C[cstart[e] + dest[e][k]] without a
// merge, a hash table or a search.  The plan exists for products in which every row of B that A
// names has at most kCap entries and every row of C at most kWideCap; rows of A may be of any
// length.  nm_spgemm_plan_build reports whether that holds and which of three classes the product
// is in: 1 -- rows of A of at most kCap entries and rows of C of at most kRowCap (everything the
// SpGEMM merge path takes; such a plan is also a by-product of the mapped forward pass), 2 -- longer
// rows of A, 3 -- also rows of C of up to kWideCap entries.  The class picks the forward kernel;
// the gradient kernels are the same for all.
//
//   forward    eight lanes per row of C; the products of the row's entries of A are added to
//              the row's accumulators in LDS one entry of A after the other, i.e. every C entry
//              receives its products in the order of A's row starting from +0.0 -- the order of
//              the serial loop (cpp/sparse_csr_cpu.cpp:193-200), bit for bit;
//   grad_A[e]  = sum_k gC[cstart[e] + dest[e][k]] * b_(j,k), k ascending (the merge of
//              cpp/sparse_csr_cpu.cpp:261-274 meets the columns in that order);
//   grad_B[(j,k)] = sum over the entries e of column j of A, rows ascending (the order of
//              cpp/sparse_csr_cpu.cpp:291-303), of a_e * gC[cstart[e] + dest[e][k]], walked on
//              the transposed-structure plan of A.
//
// No atomics, nothing to clear, every gradient entry written once by one lane.
#include "nm_spgemm_plan.hpp"

namespace {

using nm::kWave;
using nm::PPlan;
using nm::pplan_layout;

constexpr int kBlock = 256;
constexpr int kCap = nm::kPlanCap;            // entries per row of A and per named row of B
constexpr int kRowCap = nm::kPlanRowCap;      // entries per row of C
constexpr int kGroupsPerBlock = kBlock / kCap;
constexpr int kWideCap = 254;                 // entries per row of C in class 3 (a destination is a byte, 0xFF is taken)
constexpr int32_t kMaxColumn = 4096;          // entries per column of A: one group of lanes walks a column
constexpr uint8_t kNone = nm::kPlanNone;

__device__ __forceinline__ void group_fence() { __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront"); }

// p[i] and p[i + 1] with one request (these kernels are bound by the number of vector memory
// instructions a wavefront issues, and a row's two pointers sit side by side).
typedef uint32_t U4 __attribute__((ext_vector_type(4)));
struct Pair64 { int64_t lo, hi; };
struct Pair32 { int32_t lo, hi; };
__device__ __forceinline__ Pair64 load_pair(const int64_t *p) {
    typedef int64_t V __attribute__((ext_vector_type(2), aligned(8)));
    const V v = *reinterpret_cast<const V *>(p);
    return Pair64{v[0], v[1]};
}
__device__ __forceinline__ Pair32 load_pair(const int32_t *p) {
    typedef int32_t V __attribute__((ext_vector_type(2), aligned(4)));
    const V v = *reinterpret_cast<const V *>(p);
    return Pair32{v[0], v[1]};
}

// ---- build -----------------------------------------------------------------------

// Eight lanes per row of A: lane k takes the k-th entry of each B row the row names and finds
// its column in row i of C.
__global__ __launch_bounds__(kBlock) void plan_map_kernel(
    int64_t rows, const int64_t *__restrict__ A_indices, const int64_t *__restrict__ A_indptr,
    const int64_t *__restrict__ B_indices, const int64_t *__restrict__ B_indptr,
    const int64_t *__restrict__ C_indices, const int64_t *__restrict__ C_indptr, PPlan p, int octets) {
    const int k = threadIdx.x & (kCap - 1);
    const int64_t stride = (int64_t)gridDim.x * kGroupsPerBlock;
    bool bad = false, other = false, long_a = false, wide_c = false;
    int32_t longest = 0;
    for (int64_t row = (int64_t)blockIdx.x * kGroupsPerBlock + threadIdx.x / kCap; row < rows; row += stride) {
        const int64_t ab = A_indptr[row], ae = A_indptr[row + 1];
        const int64_t cs = C_indptr[row], ce = C_indptr[row + 1];
        if (ce - cs > kWideCap) {
            bad = other = true;
            continue;
        }
        if (ae - ab > kCap) long_a = true;
        if (ce - cs > kRowCap) wide_c = true;
        for (int64_t e = ab; e < ae; ++e) {
            const int64_t j = A_indices[e];
            const int64_t bb = B_indptr[j], blen = B_indptr[j + 1] - bb;
            longest = blen > longest ? (int32_t)(blen < 0x7fffffff ? blen : 0x7fffffff) : longest;
            if (blen > kCap * octets) {
                bad = true;
                continue;   // (the other rows are still looked at: the caller learns the longest)
            }
            for (int o = 0; o < octets; ++o) {
                uint8_t d = kNone;
                if (kCap * o + k < blen) {
                    const int64_t col = B_indices[bb + kCap * o + k];
                    int64_t lo = cs, hi = ce;
                    while (lo < hi) {
                        const int64_t mid = (lo + hi) >> 1;
                        if (C_indices[mid] < col) lo = mid + 1;
                        else hi = mid;
                    }
                    if (lo < ce && C_indices[lo] == col) d = (uint8_t)(lo - cs);
                    else bad = other = true;   // C is not the pattern of A B
                }
                p.dest[(e * octets + o) * kCap + k] = d;
            }
            if (k == 0) {
                p.bstart[e] = (int32_t)bb;
                p.cstart[e] = (int32_t)cs;
            }
        }
    }
    if (bad) p.flag[0] = 1;
    if (long_a) p.flag[1] = 1;
    if (wide_c) p.flag[2] = 1;
    if (other) p.flag[5] = 1;
    if (longest > *(volatile int32_t *)(p.flag + 4)) atomicMax(p.flag + 4, longest);
}

// Checks the length of A's columns and notes in flag[3] how far from the diagonal A reaches
// (the largest |row - column| of a stored entry: rows ascend inside a column, so its first and
// last entry decide), which the backward uses to order its tiles.
__global__ __launch_bounds__(kBlock) void plan_columns_kernel(int64_t cols, const int32_t *__restrict__ t_indptr,
                                                              const int32_t *__restrict__ t_row, int32_t *flag) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    bool bad = false;
    int32_t far = 0;
    for (int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x; j < cols; j += stride) {
        const int32_t pb = t_indptr[j], pe = t_indptr[j + 1];
        bad |= pe - pb > kMaxColumn;
        if (pe > pb) {
            const int32_t lo = (int32_t)j - t_row[pb], hi = t_row[pe - 1] - (int32_t)j;
            far = far > lo ? far : lo;
            far = far > hi ? far : hi;
        }
    }
    if (bad) flag[0] = flag[5] = 1;
    for (int off = 32; off > 0; off >>= 1) {
        const int32_t other = __shfl_xor(far, off, kWave);
        far = far > other ? far : other;
    }
    // (only a wavefront that has something new to say: thousands of atomics on one word cost more
    // than the rest of the kernel)
    if ((threadIdx.x & (kWave - 1)) == 0 && far > *(volatile int32_t *)(flag + 3)) atomicMax(flag + 3, far);
}

// The column-major copies of cstart and dest (entry t of the transposed plan is entry t_perm[t]).
__global__ __launch_bounds__(kBlock) void plan_by_column_kernel(int64_t A_nnz, const int32_t *__restrict__ t_perm,
                                                               PPlan p, int octets) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    const uint64_t *dest64 = reinterpret_cast<const uint64_t *>(p.dest);
    uint64_t *t_dest64 = reinterpret_cast<uint64_t *>(p.t_dest);
    for (int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x; t < A_nnz; t += stride) {
        const int64_t e = t_perm[t];
        const int32_t cs = p.cstart[e];
        if (octets > 1) {
            p.t_cstart[t] = cs;
            for (int o = 0; o < octets; ++o) t_dest64[t * octets + o] = dest64[e * octets + o];
        } else {
            const uint64_t d = dest64[e];
            U4 r;
            r[0] = (uint32_t)e;
            r[1] = (uint32_t)cs;
            r[2] = (uint32_t)d;
            r[3] = (uint32_t)(d >> 32);
            reinterpret_cast<U4 *>(p.t_rec)[t] = r;
            // (entry t of this loop as a row-major entry: every entry is some t)
            const uint64_t dr = dest64[t];
            U4 q;
            q[0] = (uint32_t)p.bstart[t];
            q[1] = (uint32_t)p.cstart[t];
            q[2] = (uint32_t)dr;
            q[3] = (uint32_t)(dr >> 32);
            reinterpret_cast<U4 *>(p.rec)[t] = q;
        }
    }
}

__global__ void plan_flag_out_kernel(const int32_t *flag, volatile int64_t *host_pinned, int64_t ticket) {
    if (threadIdx.x == 0) {
        // 0: usable; 1: not usable; 2: not usable for the length of B's rows only (bits 8..: the longest)
        host_pinned[0] = flag[0] == 0 ? 0 : (flag[5] == 0 ? 2 + ((int64_t)flag[4] << 8) : 1);
        host_pinned[1] = flag[2] ? 3 : (flag[1] ? 2 : 1);   // the product's class
        __threadfence_system();
        host_pinned[2] = ticket;
    }
}

// ---- forward -----------------------------------------------------------------------
//
// A vector memory instruction costs the address unit the same sixteen or so cycles whether its
// 64 lanes fetch 512 bytes or eight lanes' worth, and these kernels are bound by the number of such
// instructions, not by bytes.  So whatever belongs to an ENTRY (its value, where its rows start,
// its destination bytes) is loaded once, by the lane whose number the entry has -- one coalesced
// instruction per array -- and handed to the lanes that need it through LDS, where a read of
// one address by eight lanes is a broadcast.

// LDS per wavefront: its eight rows at kAccShort entries apart when none has more than half the
// capacity, else four rows at a time, twice as far apart (see numeric_planned_kernel).
constexpr int kAccShort = kRowCap / 2 + 1;

// The rows of C that the groups of a wavefront have accumulated lie one behind the other in C
// (consecutive rows), so the wavefront writes them as ONE span: lane l takes entries 2 l and
// 2 l + 1 of the span (then + 128 ...), 16 bytes per lane and array, whole kilobytes per request.
// Written row by row instead, every request is eight separate pieces of a row each; the stores of
// the column indices alone were 140 us of the 519 us this kernel took on the 128^3 seven-point
// product that way.  `clen`: entries of the lane's row, 0 for a row that is not part of this span
// (past the end of the matrix, or of the other half of the wavefront); `first`: where the span
// starts in C; the row of group q has its entries at acc + slot(q) (and its columns at ccol +
// slot(q)), slot(q) = q * stride, or (q % 4) * 2 * stride when the halves take turns.
template <typename T, bool COLS>
__device__ __forceinline__ void store_wave_rows(const T *acc, const int32_t *ccol, int clen, int64_t first,
                                                int stride, bool halves, T *__restrict__ C_data,
                                                int64_t *__restrict__ C_indices) {
    typedef T T2 __attribute__((ext_vector_type(2), aligned(sizeof(T))));
    typedef int64_t L2 __attribute__((ext_vector_type(2), aligned(8)));
    constexpr int kGroups = kWave / kCap;
    // off[q]: entries in front of group q's row in the span; at[q] + j is where entry j of the span
    // sits in LDS when it belongs to group q.  All wavefront-uniform.
    int off[kGroups + 1], at[kGroups];
    off[0] = 0;
#pragma unroll
    for (int q = 0; q < kGroups; ++q) {
        off[q + 1] = off[q] + __builtin_amdgcn_readlane(clen, q * kCap);
        at[q] = (halves ? (q & 3) * 2 * stride : q * stride) - off[q];
    }
    const int total = off[kGroups];
    const int lane = threadIdx.x & (kWave - 1);
    T *out = C_data + first;
    int64_t *outc = COLS ? C_indices + first : nullptr;
    for (int j = 2 * lane; j < total; j += 2 * kWave) {
        int a0 = at[0], a1 = at[0];
#pragma unroll
        for (int q = 1; q < kGroups; ++q) {   // the last group that starts at or before the entry
            a0 = j >= off[q] ? at[q] : a0;
            a1 = j + 1 >= off[q] ? at[q] : a1;
        }
        if (j + 1 < total) {
            T2 v;
            v[0] = acc[a0 + j];
            v[1] = acc[a1 + j + 1];
            // (written once and not read again by this kernel: nontemporal, which leaves L2 to the
            // rows of B -- 0.209 -> 0.190 ms on the 128^3 seven-point product)
            __builtin_nontemporal_store(v, reinterpret_cast<T2 *>(out + j));
            if (COLS) {
                L2 c;
                c[0] = (int64_t)ccol[a0 + j];
                c[1] = (int64_t)ccol[a1 + j + 1];
                __builtin_nontemporal_store(c, reinterpret_cast<L2 *>(outc + j));
            }
        } else {
            out[j] = acc[a0 + j];
            if (COLS) outc[j] = (int64_t)ccol[a0 + j];
        }
    }
}

// The rows of the wavefront's groups, `stride` apart from `wave_acc` on, as one span (every lane of
// the wavefront must get here; cs: where the lane's row starts in C).
template <typename T>
__device__ __forceinline__ void store_wave_span(const T *wave_acc, int stride, int clen, int64_t cs,
                                                T *__restrict__ C_data) {
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    const int64_t first = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)cs) |
                          ((int64_t)__builtin_amdgcn_readfirstlane((int)(cs >> 32)) << 32);
    store_wave_rows<T, false>(wave_acc, nullptr, clen, first, stride, false, C_data, nullptr);
}

// COLS: the pattern of C is not there yet (the product is being computed for the first time, on the
// destination bytes the symbolic phase left behind): every product also drops its column beside its
// accumulator, the columns are written out with the values, and cstart is filled in.
//
// The kernel waits on memory (row pointers, then the row's entries of A and their records, then the
// rows of B: three round trips a wavefront), so what decides its speed is how many wavefronts a CU
// holds, and that is decided by the accumulators in LDS.  They are sized for rows of C of at most
// kRowCap / 2 entries; a wavefront that has a longer row (wavefronts synchronise with nobody) takes
// its eight rows four at a time, each with room for kRowCap entries.
template <typename T, bool COLS>
__global__ __launch_bounds__(kBlock) void numeric_planned_kernel(
    int64_t rows, int64_t ntiles_padded, const T *__restrict__ A_data, const int64_t *__restrict__ A_indptr,
    const T *__restrict__ B_data, const int64_t *__restrict__ B_indices, const int32_t *__restrict__ bstart,
    const uint8_t *__restrict__ dest, const int64_t *__restrict__ C_indptr, T *__restrict__ C_data,
    int64_t *__restrict__ C_indices, int32_t *__restrict__ cstart, const uint32_t *__restrict__ rec) {
    static_assert(2 * kAccShort >= kRowCap + 1 && (kWave / kCap) % 2 == 0, "half the rows at twice the stride");
    __shared__ T s_acc[kGroupsPerBlock * kAccShort];
    __shared__ int32_t s_ccol[COLS ? kGroupsPerBlock * kAccShort : 1];
    __shared__ T s_av[kBlock];                       // per group: the row's entries of A ...
    __shared__ int32_t s_bs[kBlock];                 // ... where their rows of B start ...
    __shared__ __align__(8) uint8_t s_db[kBlock * kCap];   // ... and their destination bytes
    const int k = threadIdx.x & (kCap - 1), g = threadIdx.x / kCap;
    const int64_t row = nm::xcd_tile(blockIdx.x, ntiles_padded) * kGroupsPerBlock + g;
    const bool live = row < rows;
    const Pair64 pa = load_pair(A_indptr + (live ? row : 0)), pc = load_pair(C_indptr + (live ? row : 0));
    const int64_t ab = pa.lo, ae = live ? pa.hi : ab;
    const int64_t cs = pc.lo;
    const int clen = live ? (int)(pc.hi - cs) : 0;
    const int alen = (int)(ae - ab);
    {   // lane k of the group fetches entry k of the row
        const int64_t e = k < alen ? ab + k : 0;   // entry 0: readable whenever the matrix has entries
        const T av = A_data[e];
        int32_t bs;
        uint64_t db;
        if (COLS) {   // the plan is still being filled: its separate arrays
            bs = bstart[e];
            db = *reinterpret_cast<const uint64_t *>(dest + e * kCap);
        } else {      // a finished plan: row start of B and destination bytes in one request
            const U4 r = reinterpret_cast<const U4 *>(rec)[e];
            bs = (int32_t)r[0];
            db = ((uint64_t)r[3] << 32) | r[2];
        }
        s_av[threadIdx.x] = av;
        s_bs[threadIdx.x] = bs;
        *reinterpret_cast<uint64_t *>(s_db + threadIdx.x * kCap) = k < alen ? db : ~uint64_t(0);
        if (COLS && cstart && k < alen) __builtin_nontemporal_store((int32_t)cs, cstart + e);
    }
    group_fence();
    const int slot = g * kCap;
    uint8_t db[kCap];
    T bv[kCap];
    int32_t bc[kCap];
#pragma unroll
    for (int a = 0; a < kCap; ++a) {
        db[a] = s_db[(slot + a) * kCap + k];
        const int64_t at = db[a] != kNone ? (int64_t)s_bs[slot + a] + k : 0;
        bv[a] = B_data[at];
        if (COLS) bc[a] = *reinterpret_cast<const int32_t *>(B_indices + at);   // columns fit 31 bits
    }
    constexpr int kWaveGroups = kWave / kCap;
    const int wave_first = (threadIdx.x / kWave) * kWaveGroups;   // the wavefront's first group
    const int gq = g - wave_first;
    const bool halves = __ballot(clen > kRowCap / 2) != 0;        // wavefront-uniform
    T *wave_acc = s_acc + wave_first * kAccShort;
    int32_t *wave_ccol = s_ccol + (COLS ? wave_first * kAccShort : 0);
    const int mine = halves ? (gq & 3) * 2 * kAccShort : gq * kAccShort;
    T *acc = wave_acc + mine;
    int32_t *ccol = wave_ccol + (COLS ? mine : 0);
    for (int pass = 0; pass < (halves ? 2 : 1); ++pass) {
        const bool on = !halves || (gq >> 2) == pass;
        if (on) {
#pragma unroll
            for (int q = 0; q < kCap; ++q)
                if (k + kCap * q < clen) acc[k + kCap * q] = T(0);
        }
        group_fence();
#pragma unroll
        for (int a = 0; a < kCap; ++a) {
            // the lanes of a group hold different entries of one B row: different columns, different
            // accumulators; the entries of A take their turns one after the other
            if (on && db[a] != kNone) {
                acc[db[a]] = acc[db[a]] + s_av[slot + a] * bv[a];
                if (COLS) ccol[db[a]] = bc[a];   // every product of an entry of C brings the same column
            }
            group_fence();
        }
        // (the last fence above has made every group's sums visible to the whole wavefront)
        const int from = halves && pass == 1 ? kWave / 2 : 0;   // the lane whose row starts the span
        const int64_t first = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)cs, from) |
                              ((int64_t)__builtin_amdgcn_readlane((int)(cs >> 32), from) << 32);
        store_wave_rows<T, COLS>(wave_acc, wave_ccol, on ? clen : 0, first, kAccShort, halves, C_data, C_indices);
        group_fence();   // the other half's turn overwrites these accumulators
    }
}

// The same for rows of A of any length (taken eight entries at a time) and rows of C of up to CAP
// entries: classes 2 and 3.  A workgroup has as many groups of eight lanes as accumulator rows
// fit some 16 KB of LDS.
template <int CAP> struct LongShape {
    static constexpr int kGroups = CAP <= kRowCap ? 32 : 8;
    static constexpr int kThreads = kGroups * kCap;
    static constexpr int kStride = CAP + 1;
};

template <typename T, int CAP>
__global__ __launch_bounds__(LongShape<CAP>::kThreads) void numeric_planned_long_kernel(
    int64_t rows, int64_t ntiles_padded, const T *__restrict__ A_data, const int64_t *__restrict__ A_indptr,
    const T *__restrict__ B_data, const int32_t *__restrict__ bstart, const uint8_t *__restrict__ dest,
    const int64_t *__restrict__ C_indptr, T *__restrict__ C_data) {
    using S = LongShape<CAP>;
    __shared__ T s_acc[S::kGroups * S::kStride];
    __shared__ T s_av[S::kThreads];
    __shared__ int32_t s_bs[S::kThreads];
    __shared__ __align__(8) uint8_t s_db[S::kThreads * kCap];
    const int k = threadIdx.x & (kCap - 1), g = threadIdx.x / kCap;
    const int64_t row = nm::xcd_tile(blockIdx.x, ntiles_padded) * S::kGroups + g;
    const bool live = row < rows;
    const Pair64 pa = load_pair(A_indptr + (live ? row : 0)), pc = load_pair(C_indptr + (live ? row : 0));
    const int64_t ab = pa.lo, ae = live ? pa.hi : ab;
    const int64_t cs = pc.lo;
    const int clen = live ? (int)(pc.hi - cs) : 0;
    T *acc = s_acc + g * S::kStride;
    for (int d = k; d < clen; d += kCap) acc[d] = T(0);
    const int slot = g * kCap;
    for (int64_t base = ab; base < ae; base += kCap) {
        {   // lane k of the group fetches entry base + k of the row
            const bool have = base + k < ae;
            const int64_t e = have ? base + k : base;
            const T av = A_data[e];
            const int32_t bs = bstart[e];
            const uint64_t db = *reinterpret_cast<const uint64_t *>(dest + e * kCap);
            s_av[threadIdx.x] = av;
            s_bs[threadIdx.x] = bs;
            *reinterpret_cast<uint64_t *>(s_db + threadIdx.x * kCap) = have ? db : ~uint64_t(0);
        }
        group_fence();
        uint8_t db[kCap];
        T bv[kCap];
#pragma unroll
        for (int a = 0; a < kCap; ++a) {
            db[a] = s_db[(slot + a) * kCap + k];
            bv[a] = B_data[db[a] != kNone ? (int64_t)s_bs[slot + a] + k : 0];
        }
#pragma unroll
        for (int a = 0; a < kCap; ++a) {
            if (db[a] != kNone) acc[db[a]] = acc[db[a]] + s_av[slot + a] * bv[a];
            group_fence();
        }
    }
    store_wave_span(s_acc + (threadIdx.x / kWave) * (kWave / kCap) * S::kStride, S::kStride, clen, cs, C_data);
}

// The same for products whose named rows of B have up to 8 * OCT entries (classes 4 and 5): an entry
// of A has OCT octets of destination bytes, lane k of the group takes entry 8 o + k of the row of B
// in octet o.  The entries of A still take their turns one after the other (the octets of one entry
// go to different columns of C), so every entry of C receives its products in the order of A's row.
template <typename T, int OCT, int CAP>
__global__ __launch_bounds__(LongShape<CAP>::kThreads) void numeric_planned_wide_kernel(
    int64_t rows, int64_t ntiles_padded, const T *__restrict__ A_data, const int64_t *__restrict__ A_indptr,
    const T *__restrict__ B_data, const int32_t *__restrict__ bstart, const uint8_t *__restrict__ dest,
    const int64_t *__restrict__ C_indptr, T *__restrict__ C_data) {
    using S = LongShape<CAP>;
    __shared__ T s_acc[S::kGroups * S::kStride];
    __shared__ T s_av[S::kThreads];
    __shared__ int32_t s_bs[S::kThreads];
    __shared__ __align__(8) uint8_t s_db[S::kThreads * kCap * OCT];
    const int k = threadIdx.x & (kCap - 1), g = threadIdx.x / kCap;
    const int64_t row = nm::xcd_tile(blockIdx.x, ntiles_padded) * S::kGroups + g;
    const bool live = row < rows;
    const Pair64 pa = load_pair(A_indptr + (live ? row : 0)), pc = load_pair(C_indptr + (live ? row : 0));
    const int64_t ab = pa.lo, ae = live ? pa.hi : ab;
    const int64_t cs = pc.lo;
    const int clen = live ? (int)(pc.hi - cs) : 0;
    T *acc = s_acc + g * S::kStride;
    for (int d = k; d < clen; d += kCap) acc[d] = T(0);
    const int slot = g * kCap;
    constexpr int kPer = kCap / OCT;   // entries of A whose octets are fetched together (8 gathers in flight)
    for (int64_t base = ab; base < ae; base += kCap) {
        {   // lane k of the group fetches entry base + k of the row
            const bool have = base + k < ae;
            const int64_t e = have ? base + k : base;
            s_av[threadIdx.x] = A_data[e];
            s_bs[threadIdx.x] = bstart[e];
#pragma unroll
            for (int o = 0; o < OCT; ++o)
                *reinterpret_cast<uint64_t *>(s_db + (threadIdx.x * OCT + o) * kCap) =
                    have ? *reinterpret_cast<const uint64_t *>(dest + (e * OCT + o) * kCap) : ~uint64_t(0);
        }
        group_fence();
#pragma unroll
        for (int a0 = 0; a0 < kCap; a0 += kPer) {
            uint8_t db[kCap];
            T bv[kCap];
#pragma unroll
            for (int u = 0; u < kCap; ++u) {
                const int a = a0 + u / OCT, o = u % OCT;
                db[u] = s_db[((slot + a) * OCT + o) * kCap + k];
                bv[u] = B_data[db[u] != kNone ? (int64_t)s_bs[slot + a] + kCap * o + k : 0];
            }
#pragma unroll
            for (int u = 0; u < kCap; ++u) {
                const int a = a0 + u / OCT;
                if (db[u] != kNone) acc[db[u]] = acc[db[u]] + s_av[slot + a] * bv[u];
                if (u % OCT == OCT - 1) group_fence();   // the next entry of A may meet the same columns
            }
        }
    }
    store_wave_span(s_acc + (threadIdx.x / kWave) * (kWave / kCap) * S::kStride, S::kStride, clen, cs, C_data);
}

// ---- backward ------------------------------------------------------------------------

// grad_A.  A wavefront takes 64 consecutive entries of A, eight at a time with eight lanes per
// entry (coalesced reads of the B rows); the terms change places through LDS so that lane e
// then adds the eight terms of entry e in ascending k.
constexpr int kTermStride = kCap + 1;
constexpr int kStripTiles = 32;        // tiles (of kGroupsPerBlock rows of B) per strip of the backward's walk
constexpr int kStripFrom = 8192;       // rows: columns that reach less far keep the plain order

template <typename T>
__global__ __launch_bounds__(kBlock) void grad_a_mapped_kernel(
    int64_t A_nnz, const T *__restrict__ gC, const T *__restrict__ B_data, const int32_t *__restrict__ bstart,
    const int32_t *__restrict__ cstart, const uint8_t *__restrict__ dest, T *__restrict__ grad_A) {
    __shared__ T s_term[(kBlock / kWave) * kWave * kTermStride];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int k = lane & (kCap - 1), g = lane / kCap;
    T *term = s_term + wave * kWave * kTermStride;
    const int64_t base = ((int64_t)blockIdx.x * (kBlock / kWave) + wave) * kWave;
    // (here the eight lanes of an entry fetch its starts themselves: handing them round through
    // LDS, as the other kernels do, measured slower -- the two gathers below dominate)
    int32_t bs[kCap], cs[kCap];
    uint8_t db[kCap];
#pragma unroll
    for (int p = 0; p < kCap; ++p) {
        const int64_t e = base + p * kCap + g;
        const int64_t es = e < A_nnz ? e : 0;
        bs[p] = bstart[es];
        cs[p] = cstart[es];
        db[p] = e < A_nnz ? dest[es * kCap + k] : kNone;
    }
#pragma unroll
    for (int p = 0; p < kCap; ++p) {
        const bool have = db[p] != kNone;
        const T gv = gC[have ? (int64_t)cs[p] + db[p] : 0];
        const T bv = B_data[have ? (int64_t)bs[p] + k : 0];
        term[(p * kCap + g) * kTermStride + k] = have ? gv * bv : T(0);
    }
    group_fence();
    T acc = T(0);
#pragma unroll
    for (int q = 0; q < kCap; ++q) acc += term[lane * kTermStride + q];
    if (base + lane < A_nnz) grad_A[base + lane] = acc;
}

// grad_B.  Eight lanes per row j of B, lane k its k-th entry; the group walks column j of A on
// the transposed-structure plan (rows ascending), eight entries per round trip: lane u fetches
// what belongs to the u-th of them, LDS hands it round.
template <typename T>
__global__ __launch_bounds__(kBlock) void grad_b_mapped_kernel(
    int64_t B_rows, int64_t ntiles_padded, const T *__restrict__ gC, const T *__restrict__ A_data,
    const int32_t *__restrict__ t_indptr, const int64_t *__restrict__ B_indptr,
    const uint32_t *__restrict__ t_rec, T *__restrict__ grad_B) {
    __shared__ T s_a[kBlock];
    __shared__ int32_t s_cs[kBlock];
    __shared__ __align__(8) uint8_t s_db[kBlock * kCap];
    const int k = threadIdx.x & (kCap - 1), slot = threadIdx.x & ~(kCap - 1);
    const int64_t j = nm::xcd_tile(blockIdx.x, ntiles_padded) * kGroupsPerBlock + threadIdx.x / kCap;
    const bool live = j < B_rows;
    const Pair64 pb_ = load_pair(B_indptr + (live ? j : 0));
    const int64_t bb = pb_.lo, blen = live ? pb_.hi - bb : 0;
    const Pair32 pt = load_pair(t_indptr + (live ? j : 0));
    const int32_t pb = pt.lo, pe = live ? pt.hi : pb;
    if (pb == pe) {   // no entry of A in this column: the row's gradient is zero, however long the row
        for (int64_t q = k; q < blen; q += kCap) grad_B[bb + q] = T(0);
        return;       // (no workgroup barrier anywhere in this kernel)
    }
    // a named row: at most kCap entries (the plan's build checked it)
    const bool mine = k < blen;
    T acc = T(0);
    for (int32_t t0 = pb; t0 < pe; t0 += kCap) {
        {
            const bool have = t0 + k < pe;
            const int32_t t = have ? t0 + k : pb;
            const U4 rec = reinterpret_cast<const U4 *>(t_rec)[t];   // position, row start of C, destinations
            s_a[threadIdx.x] = A_data[rec[0]];
            s_cs[threadIdx.x] = (int32_t)rec[1];
            *reinterpret_cast<uint64_t *>(s_db + threadIdx.x * kCap) =
                have ? ((uint64_t)rec[3] << 32) | rec[2] : ~uint64_t(0);
        }
        group_fence();
        uint8_t db[kCap];
        T gv[kCap];
#pragma unroll
        for (int u = 0; u < kCap; ++u) {
            db[u] = mine ? s_db[(slot + u) * kCap + k] : kNone;
            gv[u] = gC[db[u] != kNone ? (int64_t)s_cs[slot + u] + db[u] : 0];
        }
#pragma unroll
        for (int u = 0; u < kCap; ++u)
            if (db[u] != kNone) acc += s_a[slot + u] * gv[u];
        group_fence();   // the exchange slots are written again in the next round
    }
    if (mine) grad_B[bb + k] = acc;
}

// grad_A and grad_B for named rows of B of up to 8 * OCT entries.  grad_A: the octets of an entry
// are worked off one after the other by the entry's eight lanes, and the lane that adds the terms
// goes on adding where the octet before left off: ascending k over the whole row.  grad_B: a group
// of eight lanes per OCTET of a row of B.
template <typename T, int OCT>
__global__ __launch_bounds__(kBlock) void grad_a_wide_kernel(
    int64_t A_nnz, const T *__restrict__ gC, const T *__restrict__ B_data, const int32_t *__restrict__ bstart,
    const int32_t *__restrict__ cstart, const uint8_t *__restrict__ dest, T *__restrict__ grad_A) {
    __shared__ T s_term[(kBlock / kWave) * kWave * kTermStride];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int k = lane & (kCap - 1), g = lane / kCap;
    T *term = s_term + wave * kWave * kTermStride;
    const int64_t base = ((int64_t)blockIdx.x * (kBlock / kWave) + wave) * kWave;
    int32_t bs[kCap], cs[kCap];
#pragma unroll
    for (int p = 0; p < kCap; ++p) {
        const int64_t e = base + p * kCap + g;
        const int64_t es = e < A_nnz ? e : 0;
        bs[p] = bstart[es];
        cs[p] = cstart[es];
    }
    T acc = T(0);
    for (int o = 0; o < OCT; ++o) {
        uint8_t db[kCap];
#pragma unroll
        for (int p = 0; p < kCap; ++p) {
            const int64_t e = base + p * kCap + g;
            db[p] = e < A_nnz ? dest[(e * OCT + o) * kCap + k] : kNone;
        }
#pragma unroll
        for (int p = 0; p < kCap; ++p) {
            const bool have = db[p] != kNone;
            const T gv = gC[have ? (int64_t)cs[p] + db[p] : 0];
            const T bv = B_data[have ? (int64_t)bs[p] + kCap * o + k : 0];
            term[(p * kCap + g) * kTermStride + k] = have ? gv * bv : T(0);
        }
        group_fence();
        // (an absent entry of the row of B has the term +0.0: x + 0.0 == x for every x the sum can
        // hold at that point except -0.0, which a sum that started from +0.0 never is)
#pragma unroll
        for (int q = 0; q < kCap; ++q) acc += term[lane * kTermStride + q];
        group_fence();   // the exchange slots are written again for the next octet
    }
    if (base + lane < A_nnz) grad_A[base + lane] = acc;
}

template <typename T, int OCT>
__global__ __launch_bounds__(kBlock) void grad_b_wide_kernel(
    int64_t B_rows, int64_t ntiles_padded, const T *__restrict__ gC, const T *__restrict__ A_data,
    const int32_t *__restrict__ t_indptr, const int32_t *__restrict__ t_perm, const int64_t *__restrict__ B_indptr,
    const int32_t *__restrict__ t_cstart, const uint8_t *__restrict__ t_dest, T *__restrict__ grad_B) {
    __shared__ T s_a[kBlock];
    __shared__ int32_t s_cs[kBlock];
    __shared__ __align__(8) uint8_t s_db[kBlock * kCap];
    const int k = threadIdx.x & (kCap - 1), slot = threadIdx.x & ~(kCap - 1);
    const int64_t gid = nm::xcd_tile(blockIdx.x, ntiles_padded) * kGroupsPerBlock + threadIdx.x / kCap;
    const int64_t j = gid / OCT;
    const int o = (int)(gid % OCT);
    const bool live = j < B_rows;
    const Pair64 pb_ = load_pair(B_indptr + (live ? j : 0));
    const int64_t bb = pb_.lo, blen = live ? pb_.hi - bb : 0;
    const Pair32 pt = load_pair(t_indptr + (live ? j : 0));
    const int32_t pb = pt.lo, pe = live ? pt.hi : pb;
    if (pb == pe) {   // no entry of A in this column: the row's gradient is zero, however long the row
        if (kCap * o + k < blen) grad_B[bb + kCap * o + k] = T(0);
        if (o == 0)
            for (int64_t q = kCap * OCT + k; q < blen; q += kCap) grad_B[bb + q] = T(0);
        return;       // (no workgroup barrier anywhere in this kernel)
    }
    // a named row: at most kCap * OCT entries (the plan's build checked it)
    const bool mine = kCap * o + k < blen;
    T acc = T(0);
    for (int32_t t0 = pb; t0 < pe; t0 += kCap) {
        {
            const bool have = t0 + k < pe;
            const int32_t t = have ? t0 + k : pb;
            s_a[threadIdx.x] = A_data[t_perm[t]];
            s_cs[threadIdx.x] = t_cstart[t];
            *reinterpret_cast<uint64_t *>(s_db + threadIdx.x * kCap) =
                have ? *reinterpret_cast<const uint64_t *>(t_dest + ((int64_t)t * OCT + o) * kCap) : ~uint64_t(0);
        }
        group_fence();
        uint8_t db[kCap];
        T gv[kCap];
#pragma unroll
        for (int u = 0; u < kCap; ++u) {
            db[u] = mine ? s_db[(slot + u) * kCap + k] : kNone;
            gv[u] = gC[db[u] != kNone ? (int64_t)s_cs[slot + u] + db[u] : 0];
        }
#pragma unroll
        for (int u = 0; u < kCap; ++u)
            if (db[u] != kNone) acc += s_a[slot + u] * gv[u];
        group_fence();   // the exchange slots are written again in the next round
    }
    if (mine) grad_B[bb + kCap * o + k] = acc;
}

// Both gradients from the walk by column.  The eight lanes of row j of B gather, for every entry
// e of column j of A, the eight entries of gC that e's products went to -- which is also all
// that grad_A[e] = sum_k gC[..] * B[j][k] needs besides the row of B the lanes own.  So the terms
// of grad_A are formed from the values just gathered and change places through LDS exactly as
// in grad_a_mapped_kernel (lane u adds the eight terms of the round's u-th entry in ascending
// k: the same bits), and the row-major walk with its own gathers of gC falls away.
template <typename T>
__global__ __launch_bounds__(kBlock) void grad_ab_mapped_kernel(
    int64_t B_rows, int64_t ntiles_padded, const T *__restrict__ gC, const T *__restrict__ A_data,
    const T *__restrict__ B_data, const int32_t *__restrict__ t_indptr, const int64_t *__restrict__ B_indptr,
    const uint32_t *__restrict__ t_rec, T *__restrict__ grad_A, T *__restrict__ grad_B,
    const int32_t *__restrict__ flag) {
    __shared__ T s_a[kBlock];
    __shared__ int32_t s_cs[kBlock];
    __shared__ __align__(8) uint8_t s_db[kBlock * kCap];
    __shared__ T s_term[kBlock * kTermStride];
    const int k = threadIdx.x & (kCap - 1), slot = threadIdx.x & ~(kCap - 1);
    // Every XCD walks one contiguous eighth of the rows of B.  A column of A reaches `far` rows
    // from the diagonal (a 3D stencil: one grid plane), and the rows of gC it names there are
    // wanted again one plane of rows later: when a plane's worth of work is more than an L2
    // holds, the eighth is walked in strips instead -- rows [q S, (q + 1) S) of plane 0, of
    // plane 1, ..., then the next strip -- so that what is wanted again was fetched a strip ago.
    // (cfg4: 0.39 -> 0.35 ms; strips of 1024 rows; 256 and 4096 rows were slower.)
    int64_t tile;
    {
        const int64_t per = ntiles_padded / nm::kXcds, x = blockIdx.x % nm::kXcds;
        int64_t u = blockIdx.x / nm::kXcds;
        const int64_t far = flag[3];
        const int64_t plane = far / kGroupsPerBlock / kStripTiles * kStripTiles;   // in tiles, whole strips
        if (far >= kStripFrom && plane > 0) {
            const int64_t planes = per / plane;
            if (u < planes * plane) {
                const int64_t o = u % kStripTiles, zq = u / kStripTiles;
                const int64_t z = zq % planes, q = zq / planes;
                u = z * plane + q * kStripTiles + o;
            }
        }
        tile = x * per + u;
    }
    const int64_t j = tile * kGroupsPerBlock + threadIdx.x / kCap;
    const bool live = j < B_rows;
    const Pair64 pb_ = load_pair(B_indptr + (live ? j : 0));
    const int64_t bb = pb_.lo, blen = live ? pb_.hi - bb : 0;
    const Pair32 pt = load_pair(t_indptr + (live ? j : 0));
    const int32_t pb = pt.lo, pe = live ? pt.hi : pb;
    if (pb == pe) {   // no entry of A in this column: the row's gradient is zero, however long the row
        for (int64_t q = k; q < blen; q += kCap) grad_B[bb + q] = T(0);
        return;       // (no workgroup barrier anywhere in this kernel)
    }
    const bool mine = k < blen;
    const T bk = mine ? B_data[bb + k] : T(0);
    T acc = T(0);
    for (int32_t t0 = pb; t0 < pe; t0 += kCap) {
        const bool have = t0 + k < pe;
        // position in A's arrays, row start of C and destination bytes of the entry: one request
        const U4 rec = reinterpret_cast<const U4 *>(t_rec)[have ? t0 + k : pb];
        const int32_t pos = (int32_t)rec[0];
        {
            s_a[threadIdx.x] = A_data[pos];
            s_cs[threadIdx.x] = (int32_t)rec[1];
            *reinterpret_cast<uint64_t *>(s_db + threadIdx.x * kCap) =
                have ? ((uint64_t)rec[3] << 32) | rec[2] : ~uint64_t(0);
        }
        group_fence();
        uint8_t db[kCap];
        T gv[kCap];
#pragma unroll
        for (int u = 0; u < kCap; ++u) {
            db[u] = mine ? s_db[(slot + u) * kCap + k] : kNone;
            gv[u] = gC[db[u] != kNone ? (int64_t)s_cs[slot + u] + db[u] : 0];
        }
#pragma unroll
        for (int u = 0; u < kCap; ++u) {
            const bool on = db[u] != kNone;
            if (on) acc += s_a[slot + u] * gv[u];
            s_term[(slot + u) * kTermStride + k] = on ? gv[u] * bk : T(0);
        }
        group_fence();
        T dot = T(0);
#pragma unroll
        for (int q = 0; q < kCap; ++q) dot += s_term[(slot + k) * kTermStride + q];
        if (have) grad_A[pos] = dot;
        group_fence();   // the exchange slots are written again in the next round
    }
    if (mine) grad_B[bb + k] = acc;
}

// Brings the plan's flags to the host.  *usable = the product's class when the plan can be used
// (1, 2, 3 with one octet per named row of B; 4 with two octets, 5 with four, 6 and 7 the same with
// rows of C of 65-254 entries: always the kernels for rows of A of any length); 0 when it cannot; -L when the only obstacle is that the longest row of
// B that A names has L entries, more than this plan's octets hold but no more than 32 -- a plan
// with more octets would do.
int class_of(int octets, int by_rows) {
    return octets == 1 ? by_rows : (octets == 2 ? 4 : 5) + (by_rows == 3 ? 2 : 0);
}

int read_verdict(const PPlan &p, void *host_landing, int *usable, hipStream_t s, int octets) {
    int64_t state, by_rows;
    if (host_landing) {
        volatile int64_t *land = (volatile int64_t *)host_landing;
        const int64_t ticket = land[2] + 1;
        hipLaunchKernelGGL(plan_flag_out_kernel, dim3(1), dim3(64), 0, s, p.flag, land, ticket);
        NM_LAUNCH_CHECK("plan_flag_out_kernel");
        bool arrived = false;
        for (int spin = 0; spin < (1 << 22) && !arrived; ++spin) arrived = land[2] == ticket;
        if (!arrived) {
            NM_HIP_TRY(hipStreamSynchronize(s));
            NM_REQUIRE(land[2] == ticket, "the plan's verdict did not arrive");
        }
        state = land[0];
        by_rows = land[1];
    } else {
        int32_t flags[6] = {1, 0, 0, 0, 0, 1};
        NM_HIP_TRY(hipMemcpyAsync(flags, p.flag, sizeof(flags), hipMemcpyDeviceToHost, s));
        NM_HIP_TRY(hipStreamSynchronize(s));
        state = flags[0] == 0 ? 0 : (flags[5] == 0 ? 2 + ((int64_t)flags[4] << 8) : 1);
        by_rows = flags[2] ? 3 : (flags[1] ? 2 : 1);
    }
    if (state == 0) {
        *usable = class_of(octets, (int)by_rows);
    } else if ((state & 0xff) == 2) {
        const int64_t longest = state >> 8;
        *usable = longest > kCap * octets && longest <= kCap * nm::kPlanMaxOctets ? -(int)longest : 0;
    } else {
        *usable = 0;
    }
    return NM_OK;
}

// octets of a plan of this class (0: no such class)
int octets_of(int plan_class) {
    return plan_class >= 1 && plan_class <= 3 ? 1
           : (plan_class == 4 || plan_class == 6 ? 2 : (plan_class == 5 || plan_class == 7 ? 4 : 0));
}

template <typename T, int OCT>
int launch_backward_wide(int64_t A_cols, int64_t A_nnz, const void *gC, const void *A_data, const nm::TPlan &t,
                         const void *B_data, const int64_t *B_indptr, const PPlan &p, void *grad_A, void *grad_B,
                         hipStream_t s) {
    if (grad_A && A_nnz > 0) {
        const int64_t grid = nm::ceil_div(A_nnz, (int64_t)kBlock);
        NM_REQUIRE(grid < nm::kMaxGrid, "too many entries");
        hipLaunchKernelGGL((grad_a_wide_kernel<T, OCT>), dim3((unsigned)grid), dim3(kBlock), 0, s, A_nnz,
                           (const T *)gC, (const T *)B_data, p.bstart, p.cstart, p.dest, (T *)grad_A);
        NM_LAUNCH_CHECK("grad_a_wide_kernel");
    }
    if (grad_B && A_cols > 0) {
        const int64_t grid = nm::xcd_padded(nm::ceil_div(A_cols * OCT, (int64_t)kGroupsPerBlock));
        NM_REQUIRE(grid < nm::kMaxGrid, "too many rows");
        hipLaunchKernelGGL((grad_b_wide_kernel<T, OCT>), dim3((unsigned)grid), dim3(kBlock), 0, s, A_cols, grid,
                           (const T *)gC, (const T *)A_data, t.t_indptr, t.t_perm, B_indptr, p.t_cstart, p.t_dest,
                           (T *)grad_B);
        NM_LAUNCH_CHECK("grad_b_wide_kernel");
    }
    return NM_OK;
}

template <typename T>
int launch_backward(int64_t A_cols, int64_t A_nnz, const void *gC, const void *A_data, const nm::TPlan &t,
                    const void *B_data, const int64_t *B_indptr, const PPlan &p, void *grad_A, void *grad_B,
                    hipStream_t s, int octets = 1) {
    if (octets == 2)
        return launch_backward_wide<T, 2>(A_cols, A_nnz, gC, A_data, t, B_data, B_indptr, p, grad_A, grad_B, s);
    if (octets == 4)
        return launch_backward_wide<T, 4>(A_cols, A_nnz, gC, A_data, t, B_data, B_indptr, p, grad_A, grad_B, s);
    if (grad_A && grad_B && A_nnz > 0 && A_cols > 0) {
        const int64_t grid = nm::xcd_padded(nm::ceil_div(A_cols, (int64_t)kGroupsPerBlock));
        NM_REQUIRE(grid < nm::kMaxGrid, "too many rows");
        hipLaunchKernelGGL(grad_ab_mapped_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, A_cols, grid,
                           (const T *)gC, (const T *)A_data, (const T *)B_data, t.t_indptr, B_indptr, p.t_rec,
                           (T *)grad_A, (T *)grad_B, p.flag);
        NM_LAUNCH_CHECK("grad_ab_mapped_kernel");
        return NM_OK;
    }
    if (grad_A && A_nnz > 0) {
        const int64_t grid = nm::ceil_div(A_nnz, (int64_t)kBlock);
        NM_REQUIRE(grid < nm::kMaxGrid, "too many entries");
        hipLaunchKernelGGL(grad_a_mapped_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, A_nnz, (const T *)gC,
                           (const T *)B_data, p.bstart, p.cstart, p.dest, (T *)grad_A);
        NM_LAUNCH_CHECK("grad_a_mapped_kernel");
    }
    if (grad_B && A_cols > 0) {
        const int64_t grid = nm::xcd_padded(nm::ceil_div(A_cols, (int64_t)kGroupsPerBlock));
        NM_REQUIRE(grid < nm::kMaxGrid, "too many rows");
        hipLaunchKernelGGL(grad_b_mapped_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, A_cols, grid,
                           (const T *)gC, (const T *)A_data, t.t_indptr, B_indptr, p.t_rec, (T *)grad_B);
        NM_LAUNCH_CHECK("grad_b_mapped_kernel");
    }
    return NM_OK;
}

}  // namespace

extern "C" int nm_spgemm_plan_bytes(int64_t A_nnz, size_t *plan_bytes) {
    NM_REQUIRE(plan_bytes != nullptr && A_nnz >= 0, "bad arguments");
    *plan_bytes = pplan_layout(A_nnz, nullptr, nullptr);
    return NM_OK;
}

extern "C" int nm_spgemm_plan_bytes_wide(int64_t A_nnz, int octets, size_t *plan_bytes) {
    NM_REQUIRE(plan_bytes != nullptr && A_nnz >= 0, "bad arguments");
    NM_REQUIRE(octets == 1 || octets == 2 || octets == 4, "octets %d (1, 2 or 4)", octets);
    *plan_bytes = pplan_layout(A_nnz, nullptr, nullptr, octets);
    return NM_OK;
}

extern "C" int nm_spgemm_plan_build(int64_t A_rows, int64_t A_cols, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                                    const int64_t *A_indices, const int64_t *A_indptr, const int64_t *B_indices,
                                    const int64_t *B_indptr, const int64_t *C_indices, const int64_t *C_indptr,
                                    const void *A_plan_mem, void *plan_mem, size_t plan_bytes, void *host_landing,
                                    int *usable, nm_stream stream) {
    return nm_spgemm_plan_build_wide(A_rows, A_cols, A_nnz, B_nnz, C_nnz, A_indices, A_indptr, B_indices, B_indptr,
                                     C_indices, C_indptr, A_plan_mem, plan_mem, plan_bytes, 1, host_landing, usable,
                                     stream);
}

extern "C" int nm_spgemm_plan_build_wide(int64_t A_rows, int64_t A_cols, int64_t A_nnz, int64_t B_nnz,
                                         int64_t C_nnz, const int64_t *A_indices, const int64_t *A_indptr,
                                         const int64_t *B_indices, const int64_t *B_indptr,
                                         const int64_t *C_indices, const int64_t *C_indptr, const void *A_plan_mem,
                                         void *plan_mem, size_t plan_bytes, int octets, void *host_landing,
                                         int *usable, nm_stream stream) {
    NM_REQUIRE(octets == 1 || octets == 2 || octets == 4, "octets %d (1, 2 or 4)", octets);
    NM_REQUIRE(A_rows >= 0 && A_cols >= 0 && A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    NM_REQUIRE(usable && plan_mem && A_plan_mem && A_indptr && B_indptr && C_indptr, "null pointer argument");
    NM_REQUIRE((A_nnz == 0 || A_indices) && (B_nnz == 0 || B_indices) && (C_nnz == 0 || C_indices),
               "null pointer argument");
    const size_t need = pplan_layout(A_nnz, nullptr, nullptr, octets);
    if (plan_bytes < need) return nm::fail(NM_ERR_WORKSPACE, "plan of %zu bytes, %zu needed", plan_bytes, need);
    *usable = 0;
    // positions are kept in 32 bits
    const int64_t lim = (int64_t)1 << 31;
    if (A_nnz >= lim || B_nnz >= lim || C_nnz >= lim || A_rows == 0 || A_nnz == 0) return NM_OK;
    hipStream_t s = nm::as_stream(stream);
    PPlan p;
    pplan_layout(A_nnz, plan_mem, &p, octets);
    nm::TPlan t;
    nm::tplan_layout(A_rows, A_cols, A_nnz, const_cast<void *>(A_plan_mem), &t);
    if (int rc = nm::fill_async(p.flag, 16, (int32_t)0, s)) return rc;
    int64_t grid = nm::ceil_div(A_rows, (int64_t)kGroupsPerBlock);
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(plan_map_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows, A_indices, A_indptr,
                       B_indices, B_indptr, C_indices, C_indptr, p, octets);
    NM_LAUNCH_CHECK("plan_map_kernel");
    grid = nm::ceil_div(A_cols > 0 ? A_cols : 1, (int64_t)kBlock);
    if (grid > 4096) grid = 4096;
    hipLaunchKernelGGL(plan_columns_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, A_cols, t.t_indptr, t.t_row,
                       p.flag);
    NM_LAUNCH_CHECK("plan_columns_kernel");
    grid = nm::ceil_div(A_nnz, (int64_t)kBlock);
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(plan_by_column_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, A_nnz, t.t_perm, p, octets);
    NM_LAUNCH_CHECK("plan_by_column_kernel");
    return read_verdict(p, host_landing, usable, s, octets);
}

extern "C" int nm_spgemm_plan_adopt(int64_t A_rows, int64_t A_cols, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                                    int64_t hash_rows, const void *A_plan_mem, void *plan_mem, size_t plan_bytes,
                                    void *host_landing, int *usable, nm_stream stream) {
    NM_REQUIRE(A_rows >= 0 && A_cols >= 0 && A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    NM_REQUIRE(usable && plan_mem && A_plan_mem, "null pointer argument");
    const size_t need = pplan_layout(A_nnz, nullptr, nullptr);
    if (plan_bytes < need) return nm::fail(NM_ERR_WORKSPACE, "plan of %zu bytes, %zu needed", plan_bytes, need);
    *usable = 0;
    const int64_t lim = (int64_t)1 << 31;
    // what the forward pass that filled the plan has established: every row on the merge path
    // (hence the limits on rows of A, B and C); what is left is the length of A's columns
    if (hash_rows != 0 || A_nnz >= lim || B_nnz >= lim || C_nnz >= lim || A_rows == 0 || A_nnz == 0 || C_nnz == 0)
        return NM_OK;
    hipStream_t s = nm::as_stream(stream);
    PPlan p;
    pplan_layout(A_nnz, plan_mem, &p);
    nm::TPlan t;
    nm::tplan_layout(A_rows, A_cols, A_nnz, const_cast<void *>(A_plan_mem), &t);
    if (int rc = nm::fill_async(p.flag, 16, (int32_t)0, s)) return rc;
    int64_t grid = nm::ceil_div(A_cols > 0 ? A_cols : 1, (int64_t)kBlock);
    if (grid > 4096) grid = 4096;
    hipLaunchKernelGGL(plan_columns_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, A_cols, t.t_indptr, t.t_row,
                       p.flag);
    NM_LAUNCH_CHECK("plan_columns_kernel");
    grid = nm::ceil_div(A_nnz, (int64_t)kBlock);
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(plan_by_column_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, A_nnz, t.t_perm, p, 1);
    NM_LAUNCH_CHECK("plan_by_column_kernel");
    return read_verdict(p, host_landing, usable, s, 1);
}

template <typename T, int CAP>
int launch_long(int64_t A_rows, const void *A_data, const int64_t *A_indptr, const void *B_data, const PPlan &p,
                const int64_t *C_indptr, void *C_data, hipStream_t s) {
    using S = LongShape<CAP>;
    const int64_t grid = nm::xcd_padded(nm::ceil_div(A_rows, (int64_t)S::kGroups));
    NM_REQUIRE(grid < nm::kMaxGrid, "too many rows");
    hipLaunchKernelGGL((numeric_planned_long_kernel<T, CAP>), dim3((unsigned)grid), dim3(S::kThreads), 0, s, A_rows, grid,
                       (const T *)A_data, A_indptr, (const T *)B_data, p.bstart, p.dest, C_indptr, (T *)C_data);
    NM_LAUNCH_CHECK("numeric_planned_long_kernel");
    return NM_OK;
}

template <typename T, int OCT, int CAP>
int launch_wide_typed(int64_t A_rows, const void *A_data, const int64_t *A_indptr, const void *B_data, const PPlan &p,
                      const int64_t *C_indptr, void *C_data, hipStream_t s) {
    using S = LongShape<CAP>;
    const int64_t grid = nm::xcd_padded(nm::ceil_div(A_rows, (int64_t)S::kGroups));
    NM_REQUIRE(grid < nm::kMaxGrid, "too many rows");
    hipLaunchKernelGGL((numeric_planned_wide_kernel<T, OCT, CAP>), dim3((unsigned)grid), dim3(S::kThreads), 0, s, A_rows,
                       grid, (const T *)A_data, A_indptr, (const T *)B_data, p.bstart, p.dest, C_indptr, (T *)C_data);
    NM_LAUNCH_CHECK("numeric_planned_wide_kernel");
    return NM_OK;
}

template <typename T>
int launch_wide_of(int plan_class, int64_t A_rows, const void *A_data, const int64_t *A_indptr, const void *B_data,
                   const PPlan &p, const int64_t *C_indptr, void *C_data, hipStream_t s) {
    switch (plan_class) {
        case 4: return launch_wide_typed<T, 2, kRowCap>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
        case 5: return launch_wide_typed<T, 4, kRowCap>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
        case 6: return launch_wide_typed<T, 2, 256>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
        default: return launch_wide_typed<T, 4, 256>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
    }
}

static int launch_wide(nm_dtype dt, int plan_class, int64_t A_rows, const void *A_data, const int64_t *A_indptr,
                const void *B_data, const PPlan &p, const int64_t *C_indptr, void *C_data, hipStream_t s) {
    return dt == NM_F32 ? launch_wide_of<float>(plan_class, A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s)
                        : launch_wide_of<double>(plan_class, A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
}

extern "C" int nm_spgemm_numeric_planned(nm_dtype dt, int plan_class, int64_t A_rows, int64_t A_nnz, int64_t B_nnz,
                                         int64_t C_nnz, const void *A_data, const int64_t *A_indptr,
                                         const void *B_data, const void *plan_mem, const int64_t *C_indptr,
                                         void *C_data, nm_stream stream) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(octets_of(plan_class) != 0, "plan class %d (nm_spgemm_plan_build reports 1 to 7)", plan_class);
    NM_REQUIRE(A_rows >= 0 && A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    if (A_rows == 0 || A_nnz == 0 || B_nnz == 0 || C_nnz == 0) return NM_OK;   // C has no entries
    NM_REQUIRE(A_data && A_indptr && B_data && plan_mem && C_indptr && C_data, "null pointer argument");
    PPlan p;
    pplan_layout(A_nnz, const_cast<void *>(plan_mem), &p, octets_of(plan_class));
    hipStream_t s = nm::as_stream(stream);
    if (plan_class >= 4) return launch_wide(dt, plan_class, A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
    if (plan_class == 2)
        return dt == NM_F32 ? launch_long<float, kRowCap>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s)
                            : launch_long<double, kRowCap>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
    if (plan_class == 3)
        return dt == NM_F32 ? launch_long<float, 256>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s)
                            : launch_long<double, 256>(A_rows, A_data, A_indptr, B_data, p, C_indptr, C_data, s);
    const int64_t grid = nm::xcd_padded(nm::ceil_div(A_rows, (int64_t)kGroupsPerBlock));
    NM_REQUIRE(grid < nm::kMaxGrid, "too many rows");
    if (dt == NM_F32)
        hipLaunchKernelGGL((numeric_planned_kernel<float, false>), dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows,
                           grid, (const float *)A_data, A_indptr, (const float *)B_data, (const int64_t *)nullptr,
                           p.bstart, p.dest, C_indptr, (float *)C_data, (int64_t *)nullptr, (int32_t *)nullptr, p.rec);
    else
        hipLaunchKernelGGL((numeric_planned_kernel<double, false>), dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows,
                           grid, (const double *)A_data, A_indptr, (const double *)B_data, (const int64_t *)nullptr,
                           p.bstart, p.dest, C_indptr, (double *)C_data, (int64_t *)nullptr, (int32_t *)nullptr, p.rec);
    NM_LAUNCH_CHECK("numeric_planned_kernel");
    return NM_OK;
}

int nm::spgemm_numeric_on_map(nm_dtype dt, int64_t A_rows, int64_t A_nnz, const void *A_data,
                              const int64_t *A_indptr, const void *B_data, const int64_t *B_indices, const PPlan &p,
                              const int64_t *C_indptr, int64_t *C_indices, void *C_data, bool keep, hipStream_t s) {
    // (the plan's C row starts are written only for a caller that may make a plan of the records)
    int32_t *cstart = keep ? p.cstart : nullptr;
    if (A_rows == 0 || A_nnz == 0) return NM_OK;
    const int64_t grid = nm::xcd_padded(nm::ceil_div(A_rows, (int64_t)kGroupsPerBlock));
    NM_REQUIRE(grid < nm::kMaxGrid, "too many rows");
    if (dt == NM_F32)
        hipLaunchKernelGGL((numeric_planned_kernel<float, true>), dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows,
                           grid, (const float *)A_data, A_indptr, (const float *)B_data, B_indices, p.bstart, p.dest,
                           C_indptr, (float *)C_data, C_indices, cstart, (const uint32_t *)nullptr);
    else
        hipLaunchKernelGGL((numeric_planned_kernel<double, true>), dim3((unsigned)grid), dim3(kBlock), 0, s, A_rows,
                           grid, (const double *)A_data, A_indptr, (const double *)B_data, B_indices, p.bstart, p.dest,
                           C_indptr, (double *)C_data, C_indices, cstart, (const uint32_t *)nullptr);
    NM_LAUNCH_CHECK("numeric_planned_kernel");
    return NM_OK;
}

extern "C" int nm_spgemm_backward_mapped(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t A_nnz, int64_t B_nnz,
                                         int64_t C_nnz, const void *gC, const void *A_data,
                                         const void *A_plan_mem, const void *B_data, const int64_t *B_indptr,
                                         const void *plan_mem, void *grad_A, void *grad_B, nm_stream stream) {
    return nm_spgemm_backward_mapped_wide(dt, 1, A_rows, A_cols, A_nnz, B_nnz, C_nnz, gC, A_data, A_plan_mem, B_data,
                                          B_indptr, plan_mem, grad_A, grad_B, stream);
}

extern "C" int nm_spgemm_backward_mapped_wide(nm_dtype dt, int plan_class, int64_t A_rows, int64_t A_cols,
                                              int64_t A_nnz, int64_t B_nnz, int64_t C_nnz, const void *gC,
                                              const void *A_data, const void *A_plan_mem, const void *B_data,
                                              const int64_t *B_indptr, const void *plan_mem, void *grad_A,
                                              void *grad_B, nm_stream stream) {
    const int octets = octets_of(plan_class);
    NM_REQUIRE(octets != 0, "plan class %d (nm_spgemm_plan_build reports 1 to 7)", plan_class);
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(A_rows >= 0 && A_cols >= 0 && A_nnz >= 0 && B_nnz >= 0 && C_nnz >= 0, "negative size");
    NM_REQUIRE(A_nnz > 0 && A_rows > 0, "a product plan exists only for a matrix with entries");
    if (!grad_A && !grad_B) return NM_OK;
    hipStream_t s = nm::as_stream(stream);
    if (B_nnz == 0 || C_nnz == 0) {
        // no product reaches a stored entry of C: both gradients are zero
        if (grad_A) {
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
    NM_REQUIRE(gC && A_data && A_plan_mem && B_data && B_indptr && plan_mem, "null pointer argument");
    PPlan p;
    pplan_layout(A_nnz, const_cast<void *>(plan_mem), &p, octets);
    nm::TPlan t;
    nm::tplan_layout(A_rows, A_cols, A_nnz, const_cast<void *>(A_plan_mem), &t);
    if (dt == NM_F32)
        return launch_backward<float>(A_cols, A_nnz, gC, A_data, t, B_data, B_indptr, p, grad_A, grad_B, s, octets);
    return launch_backward<double>(A_cols, A_nnz, gC, A_data, t, B_data, B_indptr, p, grad_A, grad_B, s, octets);
}
