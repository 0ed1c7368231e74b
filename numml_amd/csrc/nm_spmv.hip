// CSR SpMV forward and its fused backward for gfx950.
//
// Work mapping ("row-block streaming"): one 256-lane workgroup owns R
// consecutive rows.  It stages the rows' offsets in LDS and, when the block's
// stored entries fit the LDS tile, walks them with fully coalesced loads of
// `data` and `indices` (lane k takes entry k), leaving the per-entry results in
// LDS; one lane per row then adds its row's slice in storage order, which is
// the summation order of the serial CPU loop (cpp/sparse_csr_cpu.cpp:29-35),
// so short rows reproduce it bit for bit.  Blocks whose entries do not fit
// (long rows) switch to one wavefront per long row with a cross-lane
// reduction, and one lane per short row.
//
// Algorithmic HBM bytes, s = sizeof(value):
//   forward : nnz*(s+8) + (rows+1)*8 + cols*s + rows*s
//   backward: nnz*(s+8) + (rows+1)*8 + rows*s + cols*s + nnz*s + cols*s
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <type_traits>

#include "nm_common.hpp"
#include "nm_transpose.hpp"

namespace {

using nm::kWave;

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;
// Rows of at least this many entries get a whole wavefront on the long-row path.
constexpr int kLongRow = 32;

template <typename T> struct Tile;
template <> struct Tile<float>  { static constexpr int R = 512; static constexpr int CAP = 4096; };
template <> struct Tile<double> { static constexpr int R = 512; static constexpr int CAP = 4096; };
// forward: lanes per workgroup, rows per workgroup, LDS products
#ifndef NM_FWD_BLOCK
#define NM_FWD_BLOCK 256
#endif
#ifndef NM_FWD_R
#define NM_FWD_R 512
#define NM_FWD_CAP 4096
#endif
constexpr int kFwdBlock = NM_FWD_BLOCK, kFwdR = NM_FWD_R;
// LDS products per workgroup: 4096 of fp32 (16 KB), 3072 of fp64 (24 KB instead of 32: six
// workgroups per CU instead of four; 2048 x 2048 Poisson matrix in fp64 73 -> 64 us, row sums of a
// 25-per-row pattern 0.090 -> 0.080 ms, the 7-point pattern 0.058 -> 0.060 ms)
template <typename T> constexpr int kFwdCap = sizeof(T) == 4 ? NM_FWD_CAP : NM_FWD_CAP * 3 / 4;
// entries a lane of the forward keeps in flight when it reads 32-bit structure
#ifndef NM_FWD32_K
#define NM_FWD32_K 5
#endif
// 1: the forward on 32-bit structure loads 4 consecutive entries per lane and request
// (2048 x 2048 Poisson matrix, fp32: 47.6 -> 44.3 us; the same change in the planned backward made
// it slower, 83 -> 87 us and more, so NM_BWD_VEC stays 0)
#ifndef NM_FWD32_VEC
#define NM_FWD32_VEC 1
#endif
// 1: the planned backward loads 4 consecutive entries per lane and request, NM_BWD_VEC_U requests in flight
#ifndef NM_BWD_VEC
#define NM_BWD_VEC 0
#endif
#ifndef NM_BWD_VEC_U
#define NM_BWD_VEC_U 2
#endif
// 1: that forward requests a tile's entries before its row pointers have arrived (2048 x 2048
// Poisson matrix, fp32: 43.2 -> 41.7 us; requesting the planned backward's first entries before
// its own factors are spread made that one slower, 75 -> 78.5 us)
#ifndef NM_FWD_EARLY
#define NM_FWD_EARLY 1
#endif
#ifndef NM_FWD32_VEC_U
#define NM_FWD32_VEC_U 2
#endif
// entries a lane of the planned backward keeps in flight
#ifndef NM_BWD_K
#define NM_BWD_K 6
#endif
// columns per workgroup / LDS entries of the planned backward (measured best at cfg2: 96 vs 101 us)
#ifndef NM_PLANNED_R
#define NM_PLANNED_R 256
#define NM_PLANNED_CAP 2048
#endif
constexpr int kPlannedR = NM_PLANNED_R, kPlannedCap = NM_PLANNED_CAP;

// A block of rows with this many entries or more is walked straight from global memory.
constexpr int32_t kHuge = 1 << 30;

// Loads the block's row offsets relative to `base` into LDS, clamped to kHuge
// so that they fit 32 bits whatever the block holds.
template <int R, int CAP, int BLOCK, typename IDX = int64_t>
__device__ __forceinline__ void stage_offsets(const IDX *__restrict__ indptr, int64_t r0, int nr,
                                              int64_t base, int32_t *s_off) {
    for (int t = threadIdx.x; t <= nr; t += BLOCK) {
        const int64_t d = (int64_t)indptr[r0 + t] - base;
        s_off[t] = (int32_t)(d > kHuge ? kHuge : d);
    }
}

// Rows (or columns) a workgroup takes at a time: the compiled maximum `most` where rows are
// short, fewer where they are long, so that a block holds about `cap` entries -- a matrix with
// few, long rows would otherwise be cut into fewer blocks than the chip has CUs.
inline int block_rows(int64_t rows, int64_t nnz, int most, int cap) {
    const int64_t mean = rows > 0 ? (nnz + rows - 1) / rows : 1;
    const int64_t r = cap / (mean > 0 ? mean : 1);
    return (int)(r > most ? most : (r < 8 ? 8 : r));
}

// End of the run of rows that starts at row s0 of the block and fits the LDS tile: the
// largest e in [s0, nr] with at most cap entries in rows [s0, e); e == s0 when row s0
// alone is longer.
__device__ __forceinline__ int run_end(const int32_t *s_off, int s0, int nr, int cap) {
    const int64_t limit = (int64_t)s_off[s0] + cap;
    if (s_off[nr] <= limit) return nr;
    int lo = s0, hi = nr;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (s_off[mid] <= limit) lo = mid; else hi = mid;
    }
    return lo;
}

// Element idx of an array.  O32: the array is smaller than 4 GiB, so the address is the base (in
// scalar registers) plus a 32-bit byte offset (one vector register instead of two per access).
template <bool O32, typename X>
__device__ __forceinline__ X *at(X *base, int32_t idx) {
    if (O32) {
        using C = std::conditional_t<std::is_const<X>::value, const char, char>;
        return reinterpret_cast<X *>(reinterpret_cast<C *>(base) + (uint32_t)idx * (uint32_t)sizeof(X));
    }
    return base + idx;
}

// 1: kernels that find a staging list in the plan load the listed segments of x (and, in the
// backward, of g) into LDS with coalesced requests and look the factors of the entries up there,
// instead of one gather instruction per entry and operand.  A gather of 64 scattered words keeps
// the address unit of a compute unit busy for as long as a 1 KB coalesced request, and it was these
// instructions, not bytes, that the kernels waited for (2048 x 2048 Poisson matrix, fp32: forward
// 37.9 -> 31 us in a lab kernel).
#ifndef NM_STAGE_FWD
#define NM_STAGE_FWD 1
#endif
#ifndef NM_STAGE_BWD
#define NM_STAGE_BWD 1
#endif

// quads of staged x per lane of the forward
template <int BLOCK> constexpr int kFwdXQ = nm::kStageFwd * nm::kStageSeg / (4 * BLOCK);

// One tile of the forward whose block of rows has a staging list (see nm_transpose.hpp): n entries,
// 4 <= n <= NQ * 4 * BLOCK <= CAP, starting at `base`.  Written to issue
// as few vector memory instructions as the tile's bytes allow, all of them before the first wait:
// the list arrives in scalar registers with the tile's ends, x comes a quad per lane, a lane owns two
// neighbouring rows and fetches their three pointers with one request, their sums leave as a pair.
template <typename T, int BLOCK, int R, int CAP, int NQ>
__device__ __forceinline__ void fwd_tile_staged(const int64_t r0, const int nr, const int32_t base, const int n,
                                                const T *__restrict__ data, const int16_t *__restrict__ off16,
                                                const int32_t *__restrict__ indptr, const int32_t lo0,
                                                const int32_t hi0, const int32_t lo1, const int32_t hi1,
                                                const T *__restrict__ x,
                                                T *__restrict__ y, T *s_prod, T *s_x) {
    typedef T TV __attribute__((ext_vector_type(4), aligned(sizeof(T))));
    typedef T T2 __attribute__((ext_vector_type(2), aligned(sizeof(T))));
    typedef uint32_t SV __attribute__((ext_vector_type(2), aligned(2)));    // four 16-bit places
    typedef int32_t I3 __attribute__((ext_vector_type(3), aligned(4)));
    constexpr int XQ = kFwdXQ<BLOCK>;                                       // quads of x per lane
    static_assert(NQ * 4 * BLOCK <= CAP && XQ * 4 * BLOCK == nm::kStageFwd * nm::kStageSeg, "whole quads per lane");
    static_assert(R == 2 * BLOCK && nm::kStageSeg == 128, "two rows per lane, two segments per wavefront and request");
    const int tid = threadIdx.x;
    // The wavefront's two segments per request (lo/hi = places 2 * wave + 8 u and the next one of
    // the list, in scalar registers); an unused place loads segment 0.
    TV xs[XQ];
#pragma unroll
    for (int u = 0; u < XQ; ++u) {
        int32_t seg = u == 0 ? ((tid & 32) ? hi0 : lo0) : ((tid & 32) ? hi1 : lo1);
        seg = seg < 0 ? 0 : seg;
        xs[u] = *reinterpret_cast<const TV *>(x + (int64_t)seg * nm::kStageSeg + 4 * (tid & 31));
    }
    // pointers of rows 2 tid, 2 tid + 1 and the end of the second one
    int32_t p0, p1, p2;
    if (nr == R) {
        const I3 pp = *reinterpret_cast<const I3 *>(indptr + r0 + 2 * tid);
        p0 = pp[0], p1 = pp[1], p2 = pp[2];
    } else {
        const int t = 2 * tid;
        p0 = indptr[r0 + (t < nr ? t : nr)];
        p1 = indptr[r0 + (t + 1 < nr ? t + 1 : nr)];
        p2 = indptr[r0 + (t + 2 < nr ? t + 2 : nr)];
    }
    // the entries: values and places in the staged segments, every quad of the tile at once; the
    // last quad is moved back to end with the tile and overlaps the one before it
    const T *__restrict__ d = data + base;
    const int16_t *__restrict__ co = off16 + base;
    TV aa[NQ];
    SV oo[NQ];
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
        int kc = tid * 4 + u * 4 * BLOCK;
        kc = kc < n - 4 ? kc : n - 4;
        aa[u] = __builtin_nontemporal_load(reinterpret_cast<const TV *>(d + kc));
        oo[u] = __builtin_nontemporal_load(reinterpret_cast<const SV *>(co + kc));
    }
#pragma unroll
    for (int u = 0; u < XQ; ++u) *reinterpret_cast<TV *>(s_x + 4 * (tid + u * BLOCK)) = xs[u];
    __syncthreads();
    // (the entries are pinned here: left alone, the compiler moves the requests of a quad that only
    // some lanes use down into the branch that uses it, behind the barrier)
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
#pragma unroll
        for (int q = 0; q < 4; ++q) asm volatile("" : "+v"(aa[u][q]));
        asm volatile("" : "+v"(oo[u][0]), "+v"(oo[u][1]));
    }
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
        int k = tid * 4 + u * 4 * BLOCK;
        if (k < n) {
            k = k < n - 4 ? k : n - 4;
            TV p;
            p[0] = aa[u][0] * s_x[oo[u][0] & 0xffffu];
            p[1] = aa[u][1] * s_x[oo[u][0] >> 16];
            p[2] = aa[u][2] * s_x[oo[u][1] & 0xffffu];
            p[3] = aa[u][3] * s_x[oo[u][1] >> 16];
            *reinterpret_cast<TV *>(s_prod + k) = p;
        }
    }
    __syncthreads();
    // storage-order sums of the lane's two rows
    T acc0 = 0, acc1 = 0;
    for (int j = p0 - base; j < p1 - base; ++j) acc0 += s_prod[j];
    for (int j = p1 - base; j < p2 - base; ++j) acc1 += s_prod[j];
    if (2 * tid + 1 < nr) {
        T2 out;
        out[0] = acc0, out[1] = acc1;
        __builtin_nontemporal_store(out, reinterpret_cast<T2 *>(y + r0 + 2 * tid));
    } else if (2 * tid < nr) {
        nm::stream_store(y + r0 + 2 * tid, acc0);
    }
}

// UNIT: x is taken as all ones and not read, which makes y the row sums
// (cpp/sparse_csr_cpu.cpp:1121-1127); a * 1 == a exactly, so the summation is
// the same storage-order sum.
//
// IDX: int64_t for the structure arrays as the interface delivers them, int32_t for the
// 32-bit copies a transposed-structure plan of the same pattern holds.
//
// LISTS: the instantiation that takes the tiles with a staging list through fwd_tile_staged.  It
// keeps LDS for the staged segments of x, which costs resident workgroups on patterns without
// lists (fp64: 43 instead of 26 KB), so it is a separate instantiation that the caller asks for;
// without it a tile with a list is read through the plan's 32-bit columns (its 16-bit words hold
// places in the list, not offsets).
template <typename T, int BLOCK, int R, int CAP, bool UNIT = false, typename IDX = int64_t, bool LISTS = false>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_num_sgpr(72))) void spmv_fwd_kernel(
    int64_t rows, int rt, const T *__restrict__ data, const IDX *__restrict__ indices,
    const IDX *__restrict__ indptr, const T *__restrict__ x, T *__restrict__ y,
    const int16_t *__restrict__ off16 = nullptr, const int32_t *__restrict__ flags = nullptr,
    const int32_t *__restrict__ f_desc = nullptr) {
    // rt <= R: rows per block of this launch (block_rows)
    constexpr bool STAGE = LISTS && NM_STAGE_FWD && NM_FWD32_VEC && sizeof(IDX) == 4 && !UNIT && R == nm::kPackRows;
    constexpr bool HAS_LISTS = NM_STAGE_FWD && sizeof(IDX) == 4 && !UNIT && R == nm::kPackRows;
    __shared__ int32_t s_off[R + 1];
    __shared__ __align__(16) T s_prod[CAP];
    __shared__ __align__(16) T s_x[STAGE ? nm::kStageFwd * nm::kStageSeg : 4];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    // off16: columns as 16-bit offsets from the first row of a block of nm::kPackRows rows (a plan's
    // c_off16, valid when its flags[2] is set); read when a workgroup's rows are exactly such a block
    const bool packed = sizeof(IDX) == 4 && !UNIT && off16 != nullptr && rt == nm::kPackRows && flags[2] != 0;

    const int64_t ntiles = (rows + rt - 1) / rt, npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t r0 = tile * rt;
        int nr = (int)(rows - r0 < rt ? rows - r0 : rt);
        nr = nr < R ? nr : R;   // rt <= R
        const int64_t base = indptr[r0];
        bool packed_here = packed;
        if constexpr (HAS_LISTS && !STAGE) {
            if (packed && f_desc != nullptr && f_desc[tile * nm::kStageDesc] >= 0) packed_here = false;
        }
        if constexpr (STAGE) if (f_desc != nullptr && rt == nm::kPackRows) {
            // A block of rows with a staging list keeps places in that list where other blocks
            // keep column offsets.  The tile's end, the head of its list and the wavefront's
            // four places of the list are requested together (scalar loads, one round trip);
            // `live` is always true and only keeps those requests in front of the branch.
            const int32_t *__restrict__ desc = f_desc + tile * nm::kStageDesc;
            const int64_t span = (int64_t)indptr[r0 + nr] - base;
            const int32_t d0 = desc[0];
            static_assert(kFwdXQ<BLOCK> == 2, "two requests per lane cover the list");
            const int32_t lo0 = desc[2 * wave], hi0 = desc[2 * wave + 1];
            const int32_t lo1 = desc[BLOCK / 32 + 2 * wave], hi1 = desc[BLOCK / 32 + 2 * wave + 1];
            const bool live = (lo0 & hi0 & lo1 & hi1) != INT32_MIN;
            if ((span >= 4) & (d0 >= 0) & live) {
                if (span <= CAP) {
                    // as many quads per lane as the tile has (a 5-point row block: three of four)
                    constexpr int NQ = CAP / (4 * BLOCK);
                    const int32_t *__restrict__ ip = reinterpret_cast<const int32_t *>(indptr);
                    if (span <= (NQ - 1) * 4 * BLOCK)
                        fwd_tile_staged<T, BLOCK, R, CAP, NQ - 1>(r0, nr, (int32_t)base, (int)span, data, off16, ip,
                                                                  lo0, hi0, lo1, hi1, x, y, s_prod, s_x);
                    else
                        fwd_tile_staged<T, BLOCK, R, CAP, NQ>(r0, nr, (int32_t)base, (int)span, data, off16, ip, lo0, hi0,
                                                              lo1, hi1, x, y, s_prod, s_x);
                    __syncthreads();
                    continue;
                }
                packed_here = false;
            }
        }
        // Both ends of the tile are the same for every lane (scalar loads), so the entry streams
        // can be requested without waiting for the row pointers to pass through LDS: those stay
        // in registers until the products are on their way.
        constexpr int Q = (R + BLOCK) / BLOCK;
        int32_t po[Q];
        bool early = false;
        int n_early = 0;
        if (NM_FWD_EARLY && NM_FWD32_VEC && sizeof(IDX) == 4 && !UNIT) {
            const int64_t span = (int64_t)indptr[r0 + nr] - base;
            early = span <= CAP;
            n_early = (int)span;
        }
        if (early) {
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const int t = (int)threadIdx.x + q * BLOCK;
                po[q] = (int32_t)((int64_t)indptr[r0 + (t <= nr ? t : nr)] - base);
            }
        } else {
            stage_offsets<R, CAP, BLOCK, IDX>(indptr, r0, nr, base, s_off);
            __syncthreads();
        }
        const int n = early ? n_early : s_off[nr];
        if (NM_FWD32_VEC && sizeof(IDX) == 4 && !UNIT && n <= CAP) {
            // 32-bit structure: a lane takes 4 consecutive entries per request (16-byte loads of
            // values and columns, aligned to 4 bytes only: a tile starts wherever its first row
            // does), two requests in flight
            typedef T TV __attribute__((ext_vector_type(4), aligned(sizeof(T))));
            typedef IDX IV __attribute__((ext_vector_type(4), aligned(sizeof(IDX))));
            typedef int16_t SV __attribute__((ext_vector_type(4), aligned(2)));
            const T *__restrict__ d = data + base;
            const IDX *__restrict__ ci = indices + base;
            const int16_t *__restrict__ co = off16 ? off16 + base : nullptr;
            const int n4 = n & ~3;
            constexpr int U = NM_FWD32_VEC_U;
            auto walk = [&](auto pk) {
                constexpr bool PACKED = decltype(pk)::value;
                for (int k0 = threadIdx.x * 4; k0 < n4; k0 += U * 4 * BLOCK) {
                    TV aa[U];
                    IV cc[U];
                    T xx[U][4];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int kc = k0 + u * 4 * BLOCK < n4 ? k0 + u * 4 * BLOCK : n4 - 4;
                        aa[u] = __builtin_nontemporal_load(reinterpret_cast<const TV *>(d + kc));
                        if (PACKED) {
                            const SV o = __builtin_nontemporal_load(reinterpret_cast<const SV *>(co + kc));
#pragma unroll
                            for (int q = 0; q < 4; ++q) cc[u][q] = (IDX)r0 + o[q];
                        } else {
                            cc[u] = __builtin_nontemporal_load(reinterpret_cast<const IV *>(ci + kc));
                        }
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u)
#pragma unroll
                        for (int q = 0; q < 4; ++q) xx[u][q] = x[cc[u][q]];
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        if (k0 + u * 4 * BLOCK < n4) {
#pragma unroll
                            for (int q = 0; q < 4; ++q) s_prod[k0 + u * 4 * BLOCK + q] = aa[u][q] * xx[u][q];
                        }
                }
            };
            if (packed_here) walk(std::true_type{}); else walk(std::false_type{});
            for (int k = n4 + threadIdx.x; k < n; k += BLOCK) s_prod[k] = d[k] * x[ci[k]];
            if (early) {
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    const int t = (int)threadIdx.x + q * BLOCK;
                    if (t <= nr) s_off[t] = po[q];
                }
            }
            __syncthreads();
            for (int t = threadIdx.x; t < nr; t += BLOCK) {
                const int e = s_off[t + 1];
                T acc = 0;
                for (int j = s_off[t]; j < e; ++j) acc += s_prod[j];
                nm::stream_store(y + r0 + t, acc);
            }
        } else if (n <= CAP) {
            const T *__restrict__ d = data + base;
            const IDX *__restrict__ ci = indices + base;
            // K entries in flight per lane: all their streams, then all their gathers of x.
            // Loads are unconditional on a clamped position (a predicated load would sit in
            // its own branch with its own wait).
            constexpr int K = sizeof(IDX) == 4 ? NM_FWD32_K : 5;   // int64: 4, 5 and 10 measure the same on the 2048 x 2048 Poisson matrix
            for (int k0 = threadIdx.x; k0 < n; k0 += K * BLOCK) {
                T aa[K], xx[K];
                IDX cc[K];
#pragma unroll
                for (int u = 0; u < K; ++u) {
                    const int kc = k0 + u * BLOCK < n ? k0 + u * BLOCK : n - 1;
                    aa[u] = nm::stream_load(d + kc);
                    if (!UNIT) cc[u] = nm::stream_load(ci + kc);
                }
#pragma unroll
                for (int u = 0; u < K; ++u) xx[u] = UNIT ? T(1) : x[cc[u]];
                if (k0 + (K - 1) * BLOCK < n) {
#pragma unroll
                    for (int u = 0; u < K; ++u) s_prod[k0 + u * BLOCK] = aa[u] * xx[u];
                } else {
#pragma unroll
                    for (int u = 0; u < K; ++u)
                        if (k0 + u * BLOCK < n) s_prod[k0 + u * BLOCK] = aa[u] * xx[u];
                }
            }
            __syncthreads();
            for (int t = threadIdx.x; t < nr; t += BLOCK) {
                const int e = s_off[t + 1];
                T acc = 0;
                for (int j = s_off[t]; j < e; ++j) acc += s_prod[j];
                nm::stream_store(y + r0 + t, acc);
            }
        } else if (n < kHuge) {
            // The block's entries do not fit the tile: runs of consecutive rows that do are taken
            // one after the other.  Rows shorter than kLongRow are added by one lane in storage
            // order as above; longer ones by a wavefront, lane l adding entries l, l + 64, ...
            // of the row before the lanes are summed.
            auto products = [&](int64_t first, int cnt) {   // s_prod[j] = data * x of entry first + j
                const T *__restrict__ d = data + first;
                const IDX *__restrict__ ci = indices + first;
                constexpr int K = 5;
                for (int k0 = threadIdx.x; k0 < cnt; k0 += K * BLOCK) {
                    T aa[K], xx[K];
                    IDX cc[K];
#pragma unroll
                    for (int u = 0; u < K; ++u) {
                        const int kc = k0 + u * BLOCK < cnt ? k0 + u * BLOCK : cnt - 1;
                        aa[u] = nm::stream_load(d + kc);
                        if (!UNIT) cc[u] = nm::stream_load(ci + kc);
                    }
#pragma unroll
                    for (int u = 0; u < K; ++u) xx[u] = UNIT ? T(1) : x[cc[u]];
#pragma unroll
                    for (int u = 0; u < K; ++u)
                        if (k0 + u * BLOCK < cnt) s_prod[k0 + u * BLOCK] = aa[u] * xx[u];
                }
            };
            for (int s0 = 0; s0 < nr;) {
                const int e0 = run_end(s_off, s0, nr, CAP);
                if (e0 == s0) {
                    // a row longer than the tile, CAP entries at a time; wavefront 0 keeps the
                    // lanes' partial sums (CAP is a multiple of 64: entry k stays with lane k % 64)
                    const int64_t first = base + s_off[s0];
                    const int len = s_off[s0 + 1] - s_off[s0];
                    T acc = 0;
                    for (int c0 = 0; c0 < len; c0 += CAP) {
                        const int cnt = len - c0 < CAP ? len - c0 : CAP;
                        products(first + c0, cnt);
                        __syncthreads();
                        if (wave == 0)
                            for (int j = lane; j < cnt; j += kWave) acc += s_prod[j];
                        __syncthreads();
                    }
                    if (wave == 0) {
                        acc = nm::wave_sum(acc);
                        if (lane == 0) y[r0 + s0] = acc;
                    }
                    s0 += 1;
                    continue;
                }
                const int o0 = s_off[s0];
                products(base + o0, s_off[e0] - o0);
                __syncthreads();
                for (int tb = s0; tb < e0; tb += BLOCK) {
                    const int t = tb + threadIdx.x;
                    const int b = t < e0 ? s_off[t] - o0 : 0, e = t < e0 ? s_off[t + 1] - o0 : 0;
                    const bool wide = e - b >= kLongRow;
                    if (t < e0 && !wide) {
                        T acc = 0;
                        for (int j = b; j < e; ++j) acc += s_prod[j];
                        nm::stream_store(y + r0 + t, acc);
                    }
                    for (unsigned long long todo = __ballot(wide); todo; todo &= todo - 1) {
                        const int src = __builtin_ctzll(todo);
                        const int wb = __shfl(b, src, kWave), we = __shfl(e, src, kWave);
                        T acc = 0;
                        for (int j = wb + lane; j < we; j += kWave) acc += s_prod[j];
                        acc = nm::wave_sum(acc);
                        if (lane == 0) y[r0 + tb + wave * kWave + src] = acc;
                    }
                }
                __syncthreads();
                s0 = e0;
            }
        } else {
            // short rows: one lane each, straight from global memory
            for (int t = threadIdx.x; t < nr; t += BLOCK) {
                const int64_t b = indptr[r0 + t], e = indptr[r0 + t + 1];
                if (e - b >= kLongRow) continue;
                T acc = 0;
                for (int64_t k = b; k < e; ++k) acc += data[k] * (UNIT ? T(1) : x[indices[k]]);
                y[r0 + t] = acc;
            }
            // long rows: one wavefront each
            for (int t = wave; t < nr; t += (BLOCK / kWave)) {
                const int64_t b = indptr[r0 + t], e = indptr[r0 + t + 1];
                if (e - b < kLongRow) continue;
                T acc = 0;
                for (int64_t k = b + lane; k < e; k += kWave) acc += data[k] * (UNIT ? T(1) : x[indices[k]]);
                acc = nm::wave_sum(acc);
                if (lane == 0) y[r0 + t] = acc;
            }
        }
        __syncthreads();
    }
}

// Fused backward: out_A[k] = alpha * (a[row] * b[col]) and, when grad_x is
// given, grad_x[col] += a[row] * data[k].  With grad_x == nullptr this is the
// masked outer product (cpp/sparse_csr_cpu.cpp:60-65 and :750-755).
template <typename T, int R, int CAP>
__global__ __launch_bounds__(kBlock) void spmv_bwd_kernel(
    int64_t rows, int rt, const T *__restrict__ data, const int64_t *__restrict__ indices,
    const int64_t *__restrict__ indptr, const T *__restrict__ a, const T *__restrict__ b, T alpha,
    T *__restrict__ out_A, T *__restrict__ grad_x) {
    __shared__ int32_t s_off[R + 1];
    __shared__ T s_a[CAP];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);

    const int64_t ntiles = (rows + rt - 1) / rt, npad = nm::xcd_padded(ntiles);
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile(id, npad);
        if (tile >= ntiles) continue;
        const int64_t r0 = tile * rt;
        int nr = (int)(rows - r0 < rt ? rows - r0 : rt);
        nr = nr < R ? nr : R;   // rt <= R
        const int64_t base = indptr[r0];
        stage_offsets<R, CAP, kBlock>(indptr, r0, nr, base, s_off);
        __syncthreads();
        const int n = s_off[nr];
        if (n <= CAP) {
            // spread a[row] over the row's entries
            for (int t = threadIdx.x; t < nr; t += kBlock) {
                const T av = a[r0 + t];
                const int e = s_off[t + 1];
                for (int j = s_off[t]; j < e; ++j) s_a[j] = av;
            }
            __syncthreads();
            const int64_t *__restrict__ ci = indices + base;
            for (int k = threadIdx.x; k < n; k += kBlock) {
                const int64_t c = ci[k];
                const T av = s_a[k];
                if (out_A) out_A[base + k] = alpha * (av * b[c]);
                if (grad_x) nm::atomic_add(grad_x + c, av * data[base + k]);
            }
        } else if (n < kHuge) {
            // runs of consecutive rows that fit the tile, one after the other
            for (int s0 = 0; s0 < nr;) {
                const int e0 = run_end(s_off, s0, nr, CAP);
                if (e0 == s0) {
                    // a row longer than the tile: lane = entry, straight from global memory
                    const int64_t rb = base + s_off[s0];
                    const int len = s_off[s0 + 1] - s_off[s0];
                    const T av = a[r0 + s0];
                    for (int k = threadIdx.x; k < len; k += kBlock) {
                        const int64_t c = indices[rb + k];
                        if (out_A) out_A[rb + k] = alpha * (av * b[c]);
                        if (grad_x) nm::atomic_add(grad_x + c, av * data[rb + k]);
                    }
                    s0 += 1;
                    continue;
                }
                const int o0 = s_off[s0], cnt = s_off[e0] - o0;
                // spread a[row] over the row's entries: one lane per short row, a wavefront per
                // row of kLongRow entries or more
                for (int tb = s0; tb < e0; tb += kBlock) {
                    const int t = tb + threadIdx.x;
                    const int jb = t < e0 ? s_off[t] - o0 : 0, je = t < e0 ? s_off[t + 1] - o0 : 0;
                    const T av = t < e0 ? a[r0 + t] : T(0);
                    const bool wide = je - jb >= kLongRow;
                    if (!wide)
                        for (int j = jb; j < je; ++j) s_a[j] = av;
                    for (unsigned long long todo = __ballot(wide); todo; todo &= todo - 1) {
                        const int src = __builtin_ctzll(todo);
                        const int wb = __shfl(jb, src, kWave), we = __shfl(je, src, kWave);
                        const T wv = __shfl(av, src, kWave);
                        for (int j = wb + lane; j < we; j += kWave) s_a[j] = wv;
                    }
                }
                __syncthreads();
                const int64_t first = base + o0;
                for (int k = threadIdx.x; k < cnt; k += kBlock) {
                    const int64_t c = indices[first + k];
                    const T av = s_a[k];
                    if (out_A) out_A[first + k] = alpha * (av * b[c]);
                    if (grad_x) nm::atomic_add(grad_x + c, av * data[first + k]);
                }
                __syncthreads();
                s0 = e0;
            }
        } else {
            for (int t = threadIdx.x; t < nr; t += kBlock) {
                const int64_t rb = indptr[r0 + t], re = indptr[r0 + t + 1];
                if (re - rb >= kLongRow) continue;
                const T av = a[r0 + t];
                for (int64_t k = rb; k < re; ++k) {
                    const int64_t c = indices[k];
                    if (out_A) out_A[k] = alpha * (av * b[c]);
                    if (grad_x) nm::atomic_add(grad_x + c, av * data[k]);
                }
            }
            for (int t = wave; t < nr; t += kWavesPerBlock) {
                const int64_t rb = indptr[r0 + t], re = indptr[r0 + t + 1];
                if (re - rb < kLongRow) continue;
                const T av = a[r0 + t];
                for (int64_t k = rb + lane; k < re; k += kWave) {
                    const int64_t c = indices[k];
                    if (out_A) out_A[k] = alpha * (av * b[c]);
                    if (grad_x) nm::atomic_add(grad_x + c, av * data[k]);
                }
            }
        }
        __syncthreads();
    }
}

// quads of staged g (and x) per lane of the planned backward
template <int BLOCK> constexpr int kBwdXQ = (nm::kStageBwd * nm::kStageSeg / 4 + BLOCK - 1) / BLOCK;

// One tile of the planned backward, both gradients of a symmetric pattern, for a block of columns
// with a staging list and valid packed words: n entries, 1 <= n <= CAP, the first one at position
// `base` of the plan.  Like fwd_tile_staged it issues every request of the tile before its first
// wait, unconditionally (a request inside a branch makes the compiler's wait counts pessimistic:
// it then waits for nearly everything in flight), in the order in which the answers are needed
// (requests are answered in order), and as few vector memory instructions as the bytes allow: the
// listed segments of g and x a quad per lane, a column's two bounds with one request, the packed
// words of the first 1024 entries four consecutive entries per lane (QUAD; grad_A then leaves 16
// bytes per lane as well) and the rest in ER rounds of one entry per lane; only the values of A
// are gathered entry by entry.
template <typename T, int R, int CAP, bool O32, bool QUAD, int ER>
__device__ __forceinline__ void bwd_tile_staged(const int64_t c0, const int nc, const int32_t base, const int n,
                                                const int32_t lo0, const int32_t hi0, const int32_t lo1,
                                                const int32_t hi1, const bool seg2, const T *__restrict__ data,
                                                const int32_t *__restrict__ t_indptr,
                                                const int32_t *__restrict__ t_pack, const T *__restrict__ x,
                                                const T *__restrict__ g, T *__restrict__ grad_A,
                                                T *__restrict__ grad_x, T *s_v, T *s_g, T *s_x) {
    typedef T TV __attribute__((ext_vector_type(4), aligned(sizeof(T))));
    typedef int32_t I4 __attribute__((ext_vector_type(4), aligned(4)));
    typedef int32_t I2 __attribute__((ext_vector_type(2), aligned(4)));
    constexpr int kQuads = QUAD ? 4 * kBlock : 0;       // entries of the quad phase
    static_assert(R == kBlock && nm::kStageSeg == 128, "lane = column, two segments per wavefront and request");
    static_assert(kBwdXQ<kBlock> == 2, "a list of at most sixteen places");
    const int tid = threadIdx.x;
    // Places eight and up of the list (seg2: the list has that many): the one request of the tile
    // that is not made every time.  It goes first: a request that may or may not have been made
    // only spoils the compiler's count of what is still in flight for the requests BEHIND it.
    TV gs1, xs1;
    const bool second = seg2 && 4 * (tid + kBlock) < nm::kStageBwd * nm::kStageSeg;
    if (seg2) {
        int32_t seg = (tid & 32) ? hi1 : lo1;
        seg = seg < 0 ? 0 : seg;
        const int64_t at0 = (int64_t)seg * nm::kStageSeg + 4 * (tid & 31);
        gs1 = *reinterpret_cast<const TV *>(g + at0);
        xs1 = *reinterpret_cast<const TV *>(x + at0);
    }
    // packed words
    I4 wq;
    if (QUAD) wq = __builtin_nontemporal_load(reinterpret_cast<const I4 *>(at<O32>(t_pack, base + tid * 4)));
    int32_t we[ER > 0 ? ER : 1];
#pragma unroll
    for (int r = 0; r < ER; ++r) {
        const int k = kQuads + r * kBlock + tid;
        we[r] = nm::stream_load(at<O32>(t_pack, base + (k < n ? k : n - 1)));
    }
    // the wavefront's two segments of places 0-7 (an unused place of the list loads segment 0)
    TV gs0, xs0;
    {
        // (separate scalars, not an array: the compiler turns a choice between array elements into
        // an indexed read of a copy of the array in scratch memory)
        int32_t seg = (tid & 32) ? hi0 : lo0;
        seg = seg < 0 ? 0 : seg;
        const int64_t at0 = (int64_t)seg * nm::kStageSeg + 4 * (tid & 31);
        gs0 = *reinterpret_cast<const TV *>(g + at0);
        xs0 = *reinterpret_cast<const TV *>(x + at0);
    }
    // bounds of column c0 + tid and the factor its entries share (the lane writes the mirror entry)
    int32_t pa, pb;
    if (nc == R) {
        const I2 pp = *reinterpret_cast<const I2 *>(t_indptr + c0 + tid);
        pa = pp[0], pb = pp[1];
    } else {
        pa = t_indptr[c0 + (tid < nc ? tid : nc)];
        pb = t_indptr[c0 + (tid + 1 < nc ? tid + 1 : nc)];
    }
    T own = g[c0 + (tid < nc ? tid : nc - 1)];
    // the values of A at the positions the packed words name
    T dq[4], de[ER > 0 ? ER : 1];
    if (QUAD) {
#pragma unroll
        for (int q = 0; q < 4; ++q) dq[q] = *at<O32>(data, base + tid * 4 + q + (wq[q] >> nm::kStagePlaceBits));
    }
#pragma unroll
    for (int r = 0; r < ER; ++r) {
        const int k = kQuads + r * kBlock + tid;
        const int kc = k < n ? k : n - 1;
        de[r] = *at<O32>(data, base + kc + (we[r] >> nm::kStagePlaceBits));
    }
    *reinterpret_cast<TV *>(s_g + 4 * tid) = gs0;
    *reinterpret_cast<TV *>(s_x + 4 * tid) = xs0;
    if (second) {       // (the list's last places: half a workgroup)
        *reinterpret_cast<TV *>(s_g + 4 * (tid + kBlock)) = gs1;
        *reinterpret_cast<TV *>(s_x + 4 * (tid + kBlock)) = xs1;
    }
    // (pinned: left alone, the compiler moves the request for `own` down into the branch that
    // uses it, behind the gathers)
    asm volatile("" : "+v"(own));
    if (tid < nc)
        for (int j = pa - base; j < pb - base; ++j) s_v[j] = own;
    __syncthreads();
    if (QUAD) {
        const int k = tid * 4;
        const TV sv = *reinterpret_cast<const TV *>(s_v + k);
        TV out, nv;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int li = wq[q] & ((1 << nm::kStagePlaceBits) - 1);
            out[q] = sv[q] * s_x[li];
            nv[q] = s_g[li] * dq[q];
        }
        *reinterpret_cast<TV *>(s_v + k) = nv;
        *reinterpret_cast<TV *>(at<O32>(grad_A, base + k)) = out;
    }
#pragma unroll
    for (int r = 0; r < ER; ++r) {
        const int k = kQuads + r * kBlock + tid;
        if (k < n) {
            const int li = we[r] & ((1 << nm::kStagePlaceBits) - 1);
            *at<O32>(grad_A, base + k) = s_v[k] * s_x[li];
            s_v[k] = s_g[li] * de[r];
        }
    }
    __syncthreads();
    // grad_x[column] = sum of the column's slice in ascending row order
    if (tid < nc) {
        T acc = 0;
        for (int j = pa - base; j < pb - base; ++j) acc += s_v[j];
        grad_x[c0 + tid] = acc;
    }
}

// Backward over the transposed-structure plan (columns of A as rows of A^T):
// no atomics and no clearing of grad_x.  A workgroup owns R consecutive
// columns; lane p of the entry-parallel phase reads (row, position) of the
// p-th entry in column-major order and leaves g[row] * data[position] in LDS;
// one lane per column then adds its slice in ascending row order, the order in
// which the serial CPU loop accumulates grad_x (cpp/sparse_csr_cpu.cpp:68-73),
// so grad_x matches it bit for bit and is the same on every run.
//
// grad_A: in general entry p = (row r, column c) sits at `position` in A's
// arrays and grad_A[position] = g[r] * x[c] is a scattered store.  When the
// pattern is symmetric (plan flag) the column-major entry p is the mirror of the
// row-major entry p = (row c, column r), so the lane writes
// grad_A[p] = g[c] * x[r] instead: a coalesced store, every entry once.
// LISTS: the build for plans most of whose column blocks have a staging list (it keeps the listed
// segments of g and x in LDS).  The other build takes a block with a list through the plan's
// unpacked arrays (t_row, t_perm), which every plan holds, and needs no LDS for segments.
// (The resident wavefronts asked for are what each build reaches anyway; stating them changes the
// schedule the compiler picks, measured 4 M-row tridiagonal fp32 47.6 -> 40.8 us, 2048^2 five-point
// 61.4 -> 59.9 us.)
template <typename T, int R, int CAP, bool O32, bool LISTS>
__global__ __launch_bounds__(kBlock)
__attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 ? (LISTS ? 6 : 8) : (LISTS ? 3 : 7)))) void spmv_bwd_planned_kernel(
    int64_t cols, const T *__restrict__ data, const int32_t *__restrict__ t_indptr,
    const int32_t *__restrict__ t_row, const int32_t *__restrict__ t_perm, const int32_t *__restrict__ t_pack,
    const int32_t *__restrict__ flags, const T *__restrict__ x, const T *__restrict__ g,
    T *__restrict__ grad_A, T *__restrict__ grad_x, const int32_t *__restrict__ b_desc) {
    static_assert(R == nm::kPackCols, "t_pack holds rows relative to the first column of a workgroup's block");
    static_assert(nm::kStageBwdCap <= CAP, "a block with a staging list fits the tile");
    constexpr bool STAGE = LISTS && NM_STAGE_BWD != 0;
    constexpr int kStaged = nm::kStageBwd * nm::kStageSeg;
    __shared__ int32_t s_off[R + 1];
    __shared__ __align__(16) T s_v[CAP];
    // the segments of g and of x that a block with a staging list names
    __shared__ __align__(16) T s_g[STAGE ? kStaged : 4];
    __shared__ __align__(16) T s_x[STAGE ? kStaged : 4];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const bool mirror = flags[0] != 0;
    // one packed word per entry in place of (t_row, t_perm): patterns near the diagonal
    const bool packed_plan = flags[1] != 0;
    static_assert(R == kBlock, "lane t of a workgroup stages column t of its block");
    const int64_t ntiles = (cols + R - 1) / R, npad = nm::xcd_padded(ntiles);
    const bool fused = mirror && grad_A && grad_x;
    // the factor a column's entries share: g[column] (symmetric pattern: the lane writes the mirror
    // entry) or x[column]
    const T *__restrict__ own_of = grad_A ? (mirror ? g : x) : nullptr;
    const int tid = threadIdx.x;
    for (int64_t id = blockIdx.x; id < npad; id += gridDim.x) {
        const int64_t tile = nm::xcd_tile_reversed(id, npad);
        if (tile >= ntiles) continue;
        const int64_t c0 = tile * R;
        const int nc = (int)(cols - c0 < R ? cols - c0 : R);
        bool packed = packed_plan;
        // (the low half of a packed word of a block with a list is a place in the listed segments)
        if constexpr (!STAGE) if (packed_plan && b_desc != nullptr) packed = b_desc[tile * nm::kStageDesc] < 0;
        if constexpr (STAGE) if (fused && packed && b_desc != nullptr) {
            // a block of columns with a staging list, both gradients: the tile's ends, the head of
            // its list and the wavefront's four places of the list come together (scalar loads);
            // `live` is always true and only keeps those requests in front of the branch
            const int32_t *__restrict__ desc = b_desc + tile * nm::kStageDesc;
            const int32_t first = t_indptr[c0], n_all = t_indptr[c0 + nc] - first, d0 = desc[0];
            static_assert(kBwdXQ<kBlock> == 2, "two requests per lane cover the list");
            const int32_t lo0 = desc[2 * wave], hi0 = desc[2 * wave + 1];
            const int32_t lo1 = desc[kBlock / 32 + 2 * wave], hi1 = desc[kBlock / 32 + 2 * wave + 1];
            const bool live = (lo0 & hi0 & lo1 & hi1) != INT32_MIN;
            if ((d0 >= 0) & (n_all >= 4 * kBlock) & (n_all <= CAP) & live) {
                const bool seg2 = desc[8] >= 0;
#define NM_BWD_TILE(QUAD, ER)                                                                                       \
    bwd_tile_staged<T, R, CAP, O32, QUAD, ER>(c0, nc, first, n_all, lo0, hi0, lo1, hi1, seg2, data, t_indptr, t_pack, \
                                              x, g, grad_A, grad_x, s_v, s_g, s_x)
                // the first 1024 entries in quads where there are as many, the rest in rounds of 256
                // (the five-point block: quads and one round)
                static_assert(CAP == 8 * kBlock, "up to four rounds behind the quads");
                static_assert(nm::kStageBwdMin == 4 * kBlock, "a block with a list fills the quads");
                switch ((n_all - 4 * kBlock + kBlock - 1) / kBlock) {
                    case 0: NM_BWD_TILE(true, 0); break;
                    case 1: NM_BWD_TILE(true, 1); break;
                    case 2: NM_BWD_TILE(true, 2); break;
                    case 3: NM_BWD_TILE(true, 3); break;
                    default: NM_BWD_TILE(true, 4); break;
                }
#undef NM_BWD_TILE
                __syncthreads();
                continue;
            }
            // (a block with a list always has the entries that test asks for; were it ever not so,
            // its words must not be read as row offsets)
            if (d0 >= 0) packed = false;
        }
        // Lane t holds the bounds of column c0 + t and its own factor; all three loads leave
        // together (one memory round trip before the tile's entries can be read).
        const int32_t my_a = *at<O32>(t_indptr, (int32_t)c0 + (tid < nc ? tid : nc));
        const int32_t my_b = *at<O32>(t_indptr, (int32_t)c0 + (tid + 1 < nc ? tid + 1 : nc));
        const T my_own = own_of ? *at<O32>(own_of, (int32_t)c0 + (tid < nc ? tid : nc - 1)) : T(0);
        // A block of columns with a staging list (only made where the packed words are valid) keeps
        // in the low half of a packed word the place of the entry's row in the listed segments:
        // those segments of g (and of x, where the mirror entry is written) go to LDS, a quad per
        // lane and request.
        bool staged = false;
        if constexpr (STAGE) {
            typedef T TV __attribute__((ext_vector_type(4), aligned(sizeof(T))));
            constexpr int XQ = (kStaged / 4 + kBlock - 1) / kBlock;
            const int32_t *__restrict__ desc = b_desc + tile * nm::kStageDesc;
            // (both gradients of such a block were taken by bwd_tile_staged above)
            staged = !fused && packed && b_desc != nullptr && desc[0] >= 0;
            if (staged) {
                const bool want_x = mirror && grad_A != nullptr;
                TV gs[XQ], xs[XQ];
#pragma unroll
                for (int u = 0; u < XQ; ++u) {
                    const int f = tid + u * kBlock;
                    int32_t seg = desc[f < kStaged / 4 ? f / (nm::kStageSeg / 4) : 0];
                    seg = seg < 0 ? 0 : seg;
                    const int64_t at0 = (int64_t)seg * nm::kStageSeg + 4 * (f % (nm::kStageSeg / 4));
                    gs[u] = *reinterpret_cast<const TV *>(g + at0);
                    xs[u] = *reinterpret_cast<const TV *>((want_x ? x : g) + at0);
                }
#pragma unroll
                for (int u = 0; u < XQ; ++u) {
                    const int f = tid + u * kBlock;
                    if (f < kStaged / 4) {
                        *reinterpret_cast<TV *>(s_g + 4 * f) = gs[u];
                        *reinterpret_cast<TV *>(s_x + 4 * f) = xs[u];
                    }
                }
            }
        }
        // s_off[t] = first entry of column c0 + t in the plan (an absolute position), t = 0 .. nc
        s_off[tid] = my_a;
        if (tid == nc - 1) s_off[nc] = my_b;
        __syncthreads();
        const int32_t base = s_off[0];
        const int n = s_off[nc] - base;

        // s_v[j] = own[column] for the entries j of columns [s0, e0); o0 = offset of column s0.
        // WHOLE (the tile fits): one lane per column.  Otherwise columns of kLongRow entries
        // or more are spread by a wavefront.
        auto spread = [&](auto whole, const T *__restrict__ own, const int s0, const int e0, const int32_t o0) {
            constexpr bool WHOLE = decltype(whole)::value;
            for (int tb = s0; tb < e0; tb += kBlock) {
                const int t = tb + threadIdx.x;
                int jb, je;
                T v;
                if (WHOLE) {    // s0 == 0, e0 == nc <= kBlock: one pass, lane = column, all in registers
                    jb = t < e0 ? my_a - o0 : 0;
                    je = t < e0 ? my_b - o0 : 0;
                    v = my_own;
                } else {
                    jb = t < e0 ? s_off[t] - o0 : 0;
                    je = t < e0 ? s_off[t + 1] - o0 : 0;
                    v = t < e0 ? own[c0 + t] : T(0);
                }
                const bool wide = !WHOLE && je - jb >= kLongRow;
                if (!wide)
                    for (int j = jb; j < je; ++j) s_v[j] = v;
                if (!WHOLE)
                    for (unsigned long long todo = __ballot(wide); todo; todo &= todo - 1) {
                        const int src = __builtin_ctzll(todo);
                        const int wb = __shfl(jb, src, kWave), we = __shfl(je, src, kWave);
                        const T wv = __shfl(v, src, kWave);
                        for (int j = wb + lane; j < we; j += kWave) s_v[j] = wv;
                    }
            }
        };
        // grad_x[column] = sum of the column's slice of s_v: in storage order by one lane, or
        // (not WHOLE, kLongRow entries or more) lane l of a wavefront adds entries l, l + 64, ...
        auto sums = [&](auto whole, const int s0, const int e0, const int32_t o0) {
            constexpr bool WHOLE = decltype(whole)::value;
            for (int tb = s0; tb < e0; tb += kBlock) {
                const int t = tb + threadIdx.x;
                const int jb = t < e0 ? (WHOLE ? my_a : s_off[t]) - o0 : 0;
                const int je = t < e0 ? (WHOLE ? my_b : s_off[t + 1]) - o0 : 0;
                const bool wide = !WHOLE && je - jb >= kLongRow;
                if (t < e0 && !wide) {
                    T acc = 0;
                    for (int j = jb; j < je; ++j) acc += s_v[j];
                    grad_x[c0 + t] = acc;
                }
                if (!WHOLE)
                    for (unsigned long long todo = __ballot(wide); todo; todo &= todo - 1) {
                        const int src = __builtin_ctzll(todo);
                        const int wb = __shfl(jb, src, kWave), we = __shfl(je, src, kWave);
                        T acc = 0;
                        for (int j = wb + lane; j < we; j += kWave) acc += s_v[j];
                        acc = nm::wave_sum(acc);
                        if (lane == 0) grad_x[c0 + tb + wave * kWave + src] = acc;
                    }
            }
        };
        // Entries first .. first + cnt of the plan, lane = entry, s_v holding the own factor of
        // each: both gradients of a symmetric pattern -> every global access but the gathers of
        // g, x and data is a coalesced stream.
        auto entries_fused = [&](const int32_t first, const int cnt) {
            const int32_t *__restrict__ tr = t_row + first;
            const int32_t *__restrict__ tp = t_perm + first;
            T *__restrict__ ga = grad_A + first;
            // K entries in flight per lane: all their plan loads, then all their gathers, then
            // the stores -- two memory round trips per K entries.  Loads are unconditional on a
            // clamped position (a predicated load would sit in its own branch with its own wait).
            // Measured on the 2048 x 2048 Poisson matrix (5 entries per lane and tile), kernel time:
            // K = 2: 103 us, 4: 95 us, 5: 90 us, 6: 86 us, 8: 91 us.
            if (NM_BWD_VEC) {
                // a lane takes 4 consecutive entries per request: 16-byte loads of the two plan
                // streams and one 16-byte store of grad_A (aligned to 4 bytes only), U requests in flight
                typedef int32_t I4 __attribute__((ext_vector_type(4), aligned(4)));
                typedef T T4 __attribute__((ext_vector_type(4), aligned(sizeof(T))));
                constexpr int U = NM_BWD_VEC_U;
                const int c4 = cnt & ~3;
                for (int p0 = threadIdx.x * 4; p0 < c4; p0 += U * 4 * kBlock) {
                    I4 kk[U], rr[U];
                    T gg[U][4], xx[U][4], dd[U][4];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int pc = p0 + u * 4 * kBlock < c4 ? p0 + u * 4 * kBlock : c4 - 4;
                        kk[u] = __builtin_nontemporal_load(reinterpret_cast<const I4 *>(tp + pc));
                        rr[u] = __builtin_nontemporal_load(reinterpret_cast<const I4 *>(tr + pc));
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u)
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            gg[u][q] = g[rr[u][q]];
                            xx[u][q] = x[rr[u][q]];
                            dd[u][q] = data[kk[u][q]];
                        }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int p = p0 + u * 4 * kBlock;
                        if (p < c4) {
                            T4 out;
#pragma unroll
                            for (int q = 0; q < 4; ++q) {
                                out[q] = s_v[p + q] * xx[u][q];
                                s_v[p + q] = gg[u][q] * dd[u][q];
                            }
                            *reinterpret_cast<T4 *>(ga + p) = out;
                        }
                    }
                }
                for (int p = c4 + threadIdx.x; p < cnt; p += kBlock) {
                    const int32_t k = tp[p], r = tr[p];
                    ga[p] = s_v[p] * x[r];
                    s_v[p] = g[r] * data[k];
                }
                return;
            }
            // (one entry fewer where every address takes a register pair, or the lanes spill)
            constexpr int K = O32 ? NM_BWD_K : NM_BWD_K - 1;
            for (int p0 = threadIdx.x; p0 < cnt; p0 += K * kBlock) {
                int32_t kk[K], rr[K];
                T gg[K], xx[K], dd[K];
                if (packed) {
#pragma unroll
                    for (int u = 0; u < K; ++u) {
                        const int pc = p0 + u * kBlock < cnt ? p0 + u * kBlock : cnt - 1;
                        const int32_t w = nm::stream_load(at<O32>(t_pack, first + pc));
                        kk[u] = first + pc + (w >> 16);
                        rr[u] = (int32_t)c0 + (int16_t)w;
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < K; ++u) {
                        const int pc = p0 + u * kBlock < cnt ? p0 + u * kBlock : cnt - 1;
                        kk[u] = nm::stream_load(at<O32>(t_perm, first + pc));
                        rr[u] = nm::stream_load(at<O32>(t_row, first + pc));
                    }
                }
#pragma unroll
                for (int u = 0; u < K; ++u) {
                    gg[u] = *at<O32>(g, rr[u]);
                    xx[u] = *at<O32>(x, rr[u]);
                    dd[u] = *at<O32>(data, kk[u]);
                }
                if (p0 + (K - 1) * kBlock < cnt) {
#pragma unroll
                    for (int u = 0; u < K; ++u) {
                        const int p = p0 + u * kBlock;
                        *at<O32>(grad_A, first + p) = s_v[p] * xx[u];
                        s_v[p] = gg[u] * dd[u];
                    }
                } else {
#pragma unroll
                    for (int u = 0; u < K; ++u) {
                        const int p = p0 + u * kBlock;
                        if (p < cnt) {
                            *at<O32>(grad_A, first + p) = s_v[p] * xx[u];
                            s_v[p] = gg[u] * dd[u];
                        }
                    }
                }
            }
        };
        // The same for one gradient only or a pattern that is not symmetric.
        auto entries_any = [&](const int32_t first, const int cnt) {
            const int32_t *__restrict__ tr = t_row + first;
            const int32_t *__restrict__ tp = t_perm + first;
            for (int p = threadIdx.x; p < cnt; p += kBlock) {
                int32_t k, r;
                if (packed) {
                    const int32_t w = nm::stream_load(t_pack + first + p);
                    k = first + p + ((STAGE && staged) ? w >> nm::kStagePlaceBits : w >> 16);
                    r = (STAGE && staged) ? (w & ((1 << nm::kStagePlaceBits) - 1)) : (int32_t)c0 + (int16_t)w;
                } else {
                    k = nm::stream_load(tp + p);
                    r = nm::stream_load(tr + p);
                }
                const T gr = (STAGE && staged) ? s_g[r] : g[r];
                if (grad_A) {
                    if (mirror) grad_A[first + p] = s_v[p] * ((STAGE && staged) ? s_x[r] : x[r]);
                    else grad_A[k] = gr * s_v[p];
                }
                if (grad_x) s_v[p] = gr * data[k];
            }
        };
        // columns [s0, e0) through LDS
        auto run = [&](auto whole, const int s0, const int e0) {
            constexpr bool WHOLE = decltype(whole)::value;
            const int32_t o0 = WHOLE ? base : s_off[s0];
            const int cnt = s_off[e0] - o0;
            if (fused) {
                spread(whole, g, s0, e0, o0);
                __syncthreads();
                entries_fused(o0, cnt);
            } else {
                if (grad_A) {
                    spread(whole, own_of, s0, e0, o0);
                    __syncthreads();
                }
                entries_any(o0, cnt);
            }
            if (grad_x) {
                __syncthreads();
                sums(whole, s0, e0, o0);
            }
        };

        if (n <= CAP) {
            run(std::true_type{}, 0, nc);
        } else if (n < kHuge) {
            for (int s0 = 0; s0 < nc;) {
                const int e0 = run_end(s_off, s0, nc, CAP);
                if (e0 > s0) {
                    run(std::false_type{}, s0, e0);
                    __syncthreads();
                    s0 = e0;
                    continue;
                }
                // a column longer than the tile, CAP entries at a time; wavefront 0 keeps the
                // lanes' partial sums (CAP is a multiple of 64: entry p stays with lane p % 64)
                const int32_t first = s_off[s0];
                const int len = s_off[s0 + 1] - s_off[s0];
                const T own = grad_A ? own_of[c0 + s0] : T(0);
                T acc = 0;
                for (int q0 = 0; q0 < len; q0 += CAP) {
                    const int cnt = len - q0 < CAP ? len - q0 : CAP;
                    if (grad_A) {
                        for (int j = threadIdx.x; j < cnt; j += kBlock) s_v[j] = own;
                        __syncthreads();
                    }
                    if (fused) entries_fused(first + q0, cnt); else entries_any(first + q0, cnt);
                    __syncthreads();
                    if (grad_x && wave == 0)
                        for (int j = lane; j < cnt; j += kWave) acc += s_v[j];
                    __syncthreads();
                }
                if (grad_x && wave == 0) {
                    acc = nm::wave_sum(acc);
                    if (lane == 0) grad_x[c0 + s0] = acc;
                }
                s0 += 1;
            }
        } else {
            for (int t = threadIdx.x; t < nc; t += kBlock) {
                const int32_t pb = t_indptr[c0 + t], pe = t_indptr[c0 + t + 1];
                if (pe - pb >= kLongRow) continue;
                const T xv = x[c0 + t];
                T acc = 0;
                for (int32_t p = pb; p < pe; ++p) {
                    const int32_t k = t_perm[p];
                    const T gr = g[t_row[p]];
                    if (grad_A) grad_A[k] = gr * xv;
                    if (grad_x) acc += gr * data[k];
                }
                if (grad_x) grad_x[c0 + t] = acc;
            }
            for (int t = wave; t < nc; t += kWavesPerBlock) {
                const int32_t pb = t_indptr[c0 + t], pe = t_indptr[c0 + t + 1];
                if (pe - pb < kLongRow) continue;
                const T xv = x[c0 + t];
                T acc = 0;
                for (int32_t p = pb + lane; p < pe; p += kWave) {
                    const int32_t k = t_perm[p];
                    const T gr = g[t_row[p]];
                    if (grad_A) grad_A[k] = gr * xv;
                    if (grad_x) acc += gr * data[k];
                }
                if (grad_x) {
                    acc = nm::wave_sum(acc);
                    if (lane == 0) grad_x[c0 + t] = acc;
                }
            }
        }
        __syncthreads();
    }
}

// set by nm_spgemv_configure: 64-bit offsets in the planned backward whatever the sizes (tests)
std::atomic<bool> g_wide_offsets{false};

int check_csr(int64_t rows, int64_t cols, int64_t nnz, const void *data, const int64_t *indices,
              const int64_t *indptr) {
    NM_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0, "negative size (rows=%lld cols=%lld nnz=%lld)",
               (long long)rows, (long long)cols, (long long)nnz);
    NM_REQUIRE(indptr != nullptr, "indptr is null");
    NM_REQUIRE(nnz == 0 || (data != nullptr && indices != nullptr), "data/indices null with nnz > 0");
    return NM_OK;
}

template <typename T, typename IDX, bool LISTS = false>
int launch_fwd(int64_t rows, int64_t nnz, const T *data, const IDX *indices, const IDX *indptr, const T *x,
               T *y, hipStream_t s, const int16_t *off16 = nullptr, const int32_t *flags = nullptr,
               const int32_t *f_desc = nullptr) {
    // (the build with lists reserves LDS for the listed segments anyway, which holds a CU to three
    // workgroups in fp64 whether the tile has 3072 or 4096 products: it takes the whole 4096, so
    // that blocks of 512 rows with seven entries a row stay blocks of 512 rows)
    constexpr int R = kFwdR, CAP = LISTS ? NM_FWD_CAP : kFwdCap<T>;
    const int rt = block_rows(rows, nnz, R, CAP);
    int64_t grid = nm::xcd_padded(nm::ceil_div(rows, rt));
    if (grid > nm::kMaxGrid) grid = nm::kMaxGrid;
    hipLaunchKernelGGL((spmv_fwd_kernel<T, kFwdBlock, R, CAP, false, IDX, LISTS>), dim3((unsigned)grid), dim3(kFwdBlock), 0, s,
                       rows, rt, data, indices, indptr, x, y, off16, flags, f_desc);
    NM_LAUNCH_CHECK("spmv_fwd_kernel");
    return NM_OK;
}

template <typename T>
int launch_row_sum(int64_t rows, int64_t nnz, const T *data, const int64_t *indptr, T *y, hipStream_t s) {
    constexpr int R = kFwdR, CAP = kFwdCap<T>;
    const int rt = block_rows(rows, nnz, R, CAP);
    int64_t grid = nm::xcd_padded(nm::ceil_div(rows, rt));
    if (grid > nm::kMaxGrid) grid = nm::kMaxGrid;
    hipLaunchKernelGGL((spmv_fwd_kernel<T, kFwdBlock, R, CAP, true>), dim3((unsigned)grid), dim3(kFwdBlock), 0, s, rows,
                       rt, data, (const int64_t *)nullptr, indptr, (const T *)nullptr, y, (const int16_t *)nullptr,
                       (const int32_t *)nullptr, (const int32_t *)nullptr);
    NM_LAUNCH_CHECK("spmv_fwd_kernel<unit>");
    return NM_OK;
}

template <typename T>
int launch_bwd(int64_t rows, int64_t nnz, const T *data, const int64_t *indices, const int64_t *indptr, const T *a,
               const T *b, T alpha, T *out_A, T *grad_x, hipStream_t s) {
    constexpr int R = Tile<T>::R, CAP = Tile<T>::CAP;
    const int rt = block_rows(rows, nnz, R, CAP);
    int64_t grid = nm::xcd_padded(nm::ceil_div(rows, rt));
    if (grid > nm::kMaxGrid) grid = nm::kMaxGrid;
    hipLaunchKernelGGL((spmv_bwd_kernel<T, R, CAP>), dim3((unsigned)grid), dim3(kBlock), 0, s, rows, rt, data,
                       indices, indptr, a, b, alpha, out_A, grad_x);
    NM_LAUNCH_CHECK("spmv_bwd_kernel");
    return NM_OK;
}

}  // namespace

extern "C" int nm_spgemv_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                 const int64_t *indices, const int64_t *indptr, const void *x, void *y,
                                 nm_stream stream) {
    if (int rc = check_csr(rows, cols, nnz, data, indices, indptr)) return rc;
    if (rows == 0) return NM_OK;
    NM_REQUIRE(y != nullptr, "y is null");
    NM_REQUIRE(cols == 0 || x != nullptr, "x is null");
    hipStream_t s = nm::as_stream(stream);
    switch (dt) {
        case NM_F32:
            return launch_fwd<float, int64_t>(rows, nnz, (const float *)data, indices, indptr, (const float *)x,
                                              (float *)y, s);
        case NM_F64:
            return launch_fwd<double, int64_t>(rows, nnz, (const double *)data, indices, indptr, (const double *)x,
                                               (double *)y, s);
    }
    return nm::fail(NM_ERR_INVALID, "unknown dtype %d", (int)dt);
}

namespace {
template <bool LISTS>
int forward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data, const void *plan_mem,
                    const void *x, void *y, nm_stream stream) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0 && plan_mem != nullptr, "bad sizes or null plan");
    if (rows == 0) return NM_OK;
    NM_REQUIRE(y != nullptr && (nnz == 0 || data != nullptr), "null pointer argument");
    NM_REQUIRE(cols == 0 || x != nullptr, "x is null");
    nm::TPlan t;
    nm::tplan_layout(rows, cols, nnz, const_cast<void *>(plan_mem), &t);
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F32)
        return launch_fwd<float, int32_t, LISTS>(rows, nnz, (const float *)data, t.c_idx32, t.c_ptr32, (const float *)x,
                                                 (float *)y, s, t.c_off16, t.flags, nnz > 0 ? t.f_desc : nullptr);
    return launch_fwd<double, int32_t, LISTS>(rows, nnz, (const double *)data, t.c_idx32, t.c_ptr32, (const double *)x,
                                              (double *)y, s, t.c_off16, t.flags, nnz > 0 ? t.f_desc : nullptr);
}
}  // namespace

extern "C" int nm_spgemv_forward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                         const void *plan_mem, const void *x, void *y, nm_stream stream) {
    return forward_planned<false>(dt, rows, cols, nnz, data, plan_mem, x, y, stream);
}

extern "C" int nm_spgemv_forward_planned_lists(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                               const void *plan_mem, const void *x, void *y, nm_stream stream) {
    return forward_planned<true>(dt, rows, cols, nnz, data, plan_mem, x, y, stream);
}

extern "C" int nm_csr_row_sum_forward(nm_dtype dt, int64_t rows, int64_t nnz, const void *data,
                                      const int64_t *indptr, void *x, nm_stream stream) {
    NM_REQUIRE(rows >= 0 && nnz >= 0, "negative size");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (rows == 0) return NM_OK;
    NM_REQUIRE(indptr && x && (nnz == 0 || data), "null pointer argument");
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F32) return launch_row_sum<float>(rows, nnz, (const float *)data, indptr, (float *)x, s);
    return launch_row_sum<double>(rows, nnz, (const double *)data, indptr, (double *)x, s);
}

extern "C" int nm_spgemv_backward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                  const int64_t *indices, const int64_t *indptr, const void *x,
                                  const void *g, void *grad_A, void *grad_x, nm_stream stream) {
    if (int rc = check_csr(rows, cols, nnz, data, indices, indptr)) return rc;
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    hipStream_t s = nm::as_stream(stream);
    if (grad_x) {
        int rc = dt == NM_F32 ? nm::fill_async((float *)grad_x, cols, 0.0f, s)
                              : nm::fill_async((double *)grad_x, cols, 0.0, s);
        if (rc) return rc;
    }
    if (rows == 0 || nnz == 0 || (!grad_A && !grad_x)) return NM_OK;
    NM_REQUIRE(g != nullptr && x != nullptr, "g or x is null");
    if (dt == NM_F32)
        return launch_bwd<float>(rows, nnz, (const float *)data, indices, indptr, (const float *)g,
                                 (const float *)x, 1.0f, (float *)grad_A, (float *)grad_x, s);
    return launch_bwd<double>(rows, nnz, (const double *)data, indices, indptr, (const double *)g,
                              (const double *)x, 1.0, (double *)grad_A, (double *)grad_x, s);
}

extern "C" int nm_masked_outer(nm_dtype dt, int64_t rows, int64_t nnz, const int64_t *indices,
                               const int64_t *indptr, double alpha, const void *a, const void *b, void *out,
                               nm_stream stream) {
    NM_REQUIRE(rows >= 0 && nnz >= 0 && indptr != nullptr, "bad sizes or null indptr");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (rows == 0 || nnz == 0) return NM_OK;
    NM_REQUIRE(indices && a && b && out, "null pointer argument");
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F32)
        return launch_bwd<float>(rows, nnz, nullptr, indices, indptr, (const float *)a, (const float *)b,
                                 (float)alpha, (float *)out, nullptr, s);
    return launch_bwd<double>(rows, nnz, nullptr, indices, indptr, (const double *)a, (const double *)b, alpha,
                              (double *)out, nullptr, s);
}

extern "C" int nm_spgemv_configure(int wide_offsets) {
    g_wide_offsets.store(wide_offsets != 0, std::memory_order_relaxed);
    return NM_OK;
}

namespace {
template <typename T, bool LISTS>
void launch_bwd_planned(int64_t cols, int64_t nnz, const nm::TPlan &t, bool o32, const void *data, const void *x,
                        const void *g, void *grad_A, void *grad_x, hipStream_t s) {
    constexpr int R = kPlannedR, CAP = kPlannedCap;
    int64_t grid = nm::xcd_padded(nm::ceil_div(cols, R));
    if (grid > nm::kMaxGrid) grid = nm::kMaxGrid;
    const int32_t *desc = nnz > 0 ? t.b_desc : nullptr;
    if (o32)
        hipLaunchKernelGGL((spmv_bwd_planned_kernel<T, R, CAP, true, LISTS>), dim3((unsigned)grid), dim3(kBlock), 0, s,
                           cols, (const T *)data, t.t_indptr, t.t_row, t.t_perm, t.t_pack, t.flags, (const T *)x,
                           (const T *)g, (T *)grad_A, (T *)grad_x, desc);
    else
        hipLaunchKernelGGL((spmv_bwd_planned_kernel<T, R, CAP, false, LISTS>), dim3((unsigned)grid), dim3(kBlock), 0, s,
                           cols, (const T *)data, t.t_indptr, t.t_row, t.t_perm, t.t_pack, t.flags, (const T *)x,
                           (const T *)g, (T *)grad_A, (T *)grad_x, desc);
}

template <bool LISTS>
int backward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data, const void *plan_mem,
                     const void *x, const void *g, void *grad_A, void *grad_x, nm_stream stream) {
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    NM_REQUIRE(rows >= 0 && cols >= 0 && nnz >= 0 && plan_mem != nullptr, "bad sizes or null plan");
    if (cols == 0 || (!grad_A && !grad_x)) return NM_OK;
    NM_REQUIRE(nnz == 0 || (data && x && g), "null pointer argument");
    nm::TPlan t;
    nm::tplan_layout(rows, cols, nnz, const_cast<void *>(plan_mem), &t);
    hipStream_t s = nm::as_stream(stream);
    // every array the kernel indexes stays below 4 GiB: 32-bit byte offsets
    const int64_t longest = std::max(std::max(rows, cols) + 2, nnz + 1);
    const bool o32 = !g_wide_offsets.load(std::memory_order_relaxed) && longest * (dt == NM_F32 ? 4 : 8) < (int64_t(1) << 32);
    if (dt == NM_F32) launch_bwd_planned<float, LISTS>(cols, nnz, t, o32, data, x, g, grad_A, grad_x, s);
    else launch_bwd_planned<double, LISTS>(cols, nnz, t, o32, data, x, g, grad_A, grad_x, s);
    NM_LAUNCH_CHECK("spmv_bwd_planned_kernel");
    return NM_OK;
}
}  // namespace

extern "C" int nm_spgemv_backward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz, const void *data,
                                          const void *plan_mem, const void *x, const void *g, void *grad_A,
                                          void *grad_x, nm_stream stream) {
    return backward_planned<false>(dt, rows, cols, nnz, data, plan_mem, x, g, grad_A, grad_x, stream);
}

extern "C" int nm_spgemv_backward_planned_lists(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                                                const void *data, const void *plan_mem, const void *x,
                                                const void *g, void *grad_A, void *grad_x, nm_stream stream) {
    return backward_planned<true>(dt, rows, cols, nnz, data, plan_mem, x, g, grad_A, grad_x, stream);
}
