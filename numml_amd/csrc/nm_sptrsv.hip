// Level-scheduled sparse triangular solve for gfx950.
//
// Analysis (once per sparsity pattern).  The strictly-triangular entries of A
// define a dependency DAG.  The transposed-structure plan (counting sort by
// column, rows ascending inside a column) gives every row's dependents; a Kahn
// sweep run by one workgroup peels the DAG level by level, the rows of each level
// are then put into ascending order, and row order[q] sits in "slot" q, level l
// owning slots [level_ptr[l], level_ptr[l+1]).  The plan
// then stores, for both solve directions (A and A^T), a level-major packed copy
// of the triangle: per slot the range of its dependencies, per dependency the
// SLOT of the row it refers to and the position of its coefficient in A's
// value array, and the position of the diagonal coefficient.  The transposed
// solve (the backward pass) walks the same levels in reverse.
//
// Solve.  The running solution lives in slot order (xs[q]), so a dependency is
// one indexed read and consecutive levels touch neighbouring memory.  Runs of
// consecutive narrow levels (<= 1024 rows) are executed by ONE 1024-lane
// workgroup: levels are separated by workgroup barriers, the solutions of the
// last ~7000 slots are kept in an LDS ring (a dependency on a recent slot costs
// an LDS read instead of an L2 round trip).  A chip-wide pass first gathers
// this call's coefficients, diagonal and right-hand side into level-major
// order (as doubles), so the workgroup reads contiguous streams only, two and
// one level ahead through a register pipeline.  A level wider than 1024 rows gets a grid launch of its own.
// Where the plan finds it possible, a run of levels wider than 256 rows is shared by up
// to four workgroups that pass the few values they need from each other through device
// memory (sptrsv_team_kernel).  Stream order is the only synchronisation between launches;
// inside a shared launch a workgroup waits for values of lower levels only, all its
// workgroups are resident, and every wait is bounded (a solve that gives up returns NaN).
//
// A row is one lane; sums run in double, in the walk order of the serial
// CPU loop (cpp/sparse_csr_cpu.cpp:672-718: ascending for a lower triangle,
// descending for an upper one), so results match it bit for bit.  The exception
// are launches whose rows average a dozen dependencies or more (the factors of a
// direct solve): there 16 or 64 lanes share a row and add their partial sums
// across the group, which differs from the serial order by rounding in double.
//
// Algorithmic HBM bytes of one solve (s = sizeof(value)):
//   nnz*(s+8) + (rows+1)*8 + 2*rows*s
#include "nm_common.hpp"
#include "nm_scan.hpp"
#include "nm_transpose.hpp"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <mutex>
#include <new>
#include <type_traits>
#include <vector>

namespace {
struct Packed {        // one solve direction, level-major (all int32, device)
    int32_t *dptr;     // [rows+1] dependency range of slot q
    int32_t *dslot;    // [nnz]    slot of the row a dependency refers to
    int32_t *dsrc;     // [nnz]    position of its coefficient in A's data
    int32_t *diag;     // [rows]   position of the diagonal coefficient, -1 when not stored
    int32_t *ell_ds;   // [ell_capacity] room for the fixed-width dependency entries: 16 bits each, `pre` per row
    int32_t *lvl_sig;  // [levels] which neighbouring wavefronts the rows of a level wait for (kSigLower | kSigHigher)
    int32_t *team;     // [team_capacity] exchange tables of the launches that several workgroups share
};
// Entries of the fixed-width (ELLPACK) arrays; the layout is used when (rows + kEllPad) * pre
// fits.  kEllPad slots of padding follow the last row in every array the fixed-width kernel
// reads or writes by slot: its lanes load the operands of slots qb .. qb + lanes - 1 whatever
// the level's width, so the slots behind a level's end must be readable.
constexpr int64_t kEllPad = 1024;   // == kNarrow, the widest single-workgroup launch
inline int64_t ell_capacity(int64_t rows, int64_t nnz) { return 2 * nnz + 2 * rows + 8 + 8 * kEllPad; }
// Doubles of the per-call coefficient area: the fixed-width layout, or the coefficient rows of
// the chain kernels (64 per chain row, whatever the band's width: room for chains of up to
// 65536 rows in all; longer ones take what fits).
inline int64_t coef_capacity(int64_t rows, int64_t nnz) {
    const int64_t chains = 66 * (rows < 65536 ? rows : 65536) + 8 * kEllPad;
    return ell_capacity(rows, nnz) > chains ? ell_capacity(rows, nnz) : chains;
}
// Launches that several workgroups share (see sptrsv_team_kernel): most workgroups, values that
// may pass between workgroups in one solve direction, ints of the tables that say which.
constexpr int kTeamMax = 16;
inline int64_t team_cells_capacity(int64_t rows) { return rows / 16 + 2048; }
constexpr int64_t kTeamCellPadding = 64;   // readable cells past the last one (a poll reads 64 at a time)
inline int64_t team_capacity(int64_t rows) { return 3 * team_cells_capacity(rows) + rows / 4 + 65536; }
}  // namespace

struct nm_sptrsv_plan {
    int64_t rows = 0, nnz = 0;
    int lower = 1;
    int32_t nlevels = 0;
    // device arrays inside the caller's plan memory
    int32_t *order = nullptr, *level_ptr = nullptr, *slot_of = nullptr;
    Packed dir[2];     // [0]: A, [1]: A^T
    int32_t max_deps[2] = {0, 0};  // longest dependency list per direction
    int32_t ell_pre[2] = {0, 0};   // width of the fixed-width layout per direction (2, 4, 8; 0 = not used)
    int32_t reach[2] = {0, 0};     // per direction: largest wavefront distance between a row and a dependency
    struct Launch {
        int32_t l0, l1;  // levels [l0, l1)
        int32_t q0, q1;  // slots they cover
        bool wide;       // one level, many workgroups
        int32_t block;   // lanes of the single-workgroup launch (narrow runs)
        int32_t width = 0;          // rows of its widest level
        int32_t group[2] = {0, 0};  // per direction: lanes that share a row (0: one lane per row)
        // per direction: 0, or how a run of one-row levels is solved by a single wavefront that
        // keeps the newest solution in a register (1: every row waits for the row before it only;
        // 64: rows wait for up to the 64 rows before them), and where its coefficients go
        int32_t chain[2] = {0, 0};
        int64_t chain_at[2] = {0, 0};
        bool chain_candidate = false;
        // per direction: the launch's first levels, up to the last one in which a row reads a row that
        // its LDS ring cannot serve (a row of an earlier launch); the levels after them take the level
        // loop that does not look for such rows
        int32_t far_levels[2] = {0x7fffffff, 0x7fffffff};
        // a stretch of levels wider than one workgroup takes, none wider than a team takes: shared
        // by a team in the directions that have one, else launched level by level like `wide` ones
        bool run = false;
        // per direction: the workgroups that share every level of the launch (0: one workgroup
        // takes it), where the tables of their exchange start in Packed::team, the first of their
        // mailbox cells, and each workgroup's part of the import and export lists
        struct Team {
            int32_t P = 0, at = 0, cell0 = 0, n_imp = 0;
            int32_t imp_off[kTeamMax + 1] = {}, exp_off[kTeamMax + 1] = {};
        } team[2];
    };
    std::vector<Launch> launches;
    int32_t team_cells[2] = {0, 0};   // mailbox cells one solve clears, per direction
    std::vector<int32_t> lp_host;     // level_ptr on the host (the level-by-level launches of a run)
};

namespace {

constexpr int kNarrow = 1024;          // widest level the single-workgroup kernel takes
constexpr int kWideRows = 128, kWideEntries = 4096;   // a level with both gets a grid launch as well
constexpr int kBlock = 256;
constexpr int kRing = 8192;            // LDS ring of recent solutions (doubles, power of two)
// Levels a wavefront of the signalling kernel may run ahead of the slowest one of its
// workgroup; the ring must keep what the slowest still reads while the fastest writes.
constexpr int kSkew = 5;
constexpr int kRingSafe = kRing - 3 * kNarrow;                 // how far back (in slots) a ring read may reach
constexpr int kRingSafeSig = kRing - (kSkew + 1) * kNarrow;    // ... when wavefronts run up to kSkew levels apart
constexpr int32_t kSigLower = 1, kSigHigher = 2;               // bits of lvl_sig
constexpr int32_t kSigFar = 4;                                 // ... a row of the level reads a row that the ring cannot serve
constexpr int32_t kSigNever = 1000;                            // a reach that rules the signalling kernel out
// Largest distance, in wavefronts, between a row and the rows it depends on (both counted from
// the start of their level) for which wavefronts signal each other instead of meeting at a
// workgroup barrier after every level.
constexpr int kSigReach = 1;
constexpr int kMaxLevels = 4096;       // levels one single-workgroup launch takes (LDS copy of their bounds)

inline size_t align_up(size_t v) { return (v + 255) & ~size_t(255); }

// Polls a wavefront of the signalling kernel makes at one level before it gives up (a poll is
// ~100 cycles; a level takes a few hundred), and the switch between signalling and barriers.
std::atomic<int64_t> g_sig_poll_limit{int64_t(1) << 22};
// Off by default: on the 1024 x 1024 Poisson triangle (2047 levels, up to 16 wavefronts) a solve
// takes 0.97 ms with a barrier per level and 1.30 ms with signals -- the two dependent LDS round
// trips of a poll cost more than the barrier's wait for the slowest wavefront saves.
// Launches shared by several workgroups (sptrsv_team_kernel), where the plan has found them possible.
std::atomic<bool> g_team_enabled{[] {
    const char *e = std::getenv("NUMML_AMD_SPTRSV_TEAMS");   // "0": one workgroup per launch
    return !(e && e[0] == '0');
}()};
std::atomic<bool> g_sig_enabled{[] {
    const char *e = std::getenv("NUMML_AMD_SPTRSV_SIGNALLING");   // "1": neighbours signal
    return e && e[0] == '1';
}()};

struct Layout {
    nm::TPlan t;
    int32_t *order, *level_ptr, *slot_of, *meta, *level_launch;
    Packed dir[2];
};

// plan memory: [transposed-structure plan][order][level_ptr][slot_of][meta][packed A][packed A^T]
size_t plan_layout(int64_t rows, int64_t nnz, void *base, Layout *L) {
    Layout l;
    size_t off = nm::tplan_layout(rows, rows, nnz, base, &l.t);
    auto take = [&](size_t count) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align_up(count * 4);
        return (int32_t *)q;
    };
    l.order = take(rows + 1);
    l.level_ptr = take(rows + 1);
    l.slot_of = take(rows + 1);
    l.meta = take(16);
    l.level_launch = take(rows + 1);
    for (int d = 0; d < 2; ++d) {
        l.dir[d].dptr = take(rows + 1);
        l.dir[d].dslot = take(nnz + 1);
        l.dir[d].dsrc = take(nnz + 1);
        l.dir[d].diag = take(rows + 1);
        l.dir[d].ell_ds = take(ell_capacity(rows, nnz));
        l.dir[d].lvl_sig = take(rows + 1);
        l.dir[d].team = take(team_capacity(rows));
    }
    if (L) *L = l;
    return off;
}

// analysis scratch: [deg][rowid][count64][scan scratch][transpose scratch]
struct Scratch {
    int32_t *deg, *rowid;
    int64_t *count64, *scan;
    void *twork;
    size_t twork_bytes;
};

size_t work_layout(int64_t rows, int64_t nnz, void *base, Scratch *S) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align_up(bytes);
        return q;
    };
    Scratch s;
    s.deg = (int32_t *)take((size_t)(rows + 1) * 4);
    s.rowid = (int32_t *)take((size_t)(nnz + 1) * 4);
    s.count64 = (int64_t *)take((size_t)(rows + 1) * 8);
    s.scan = (int64_t *)take(nm::scan_scratch_bytes(rows + 1));
    s.twork_bytes = nm::tplan_work_bytes(rows, rows, nnz);
    s.twork = take(s.twork_bytes);
    if (S) *S = s;
    return off;
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
        // a narrow level spreads the dependants of each row over g lanes
        int g = 1;
        while (g < 64 && (tail - head) * g * 2 <= kNarrow) g *= 2;
        const int sub = threadIdx.x & (g - 1);
        for (int q = head + threadIdx.x / g; q < tail; q += kNarrow / g) {
            const int32_t r = order[q];
            const int32_t pe = t_indptr[r + 1];
            for (int32_t p = t_indptr[r] + sub; p < pe; p += g) {
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

__global__ void slot_of_kernel(int64_t rows, const int32_t *__restrict__ order, int32_t *__restrict__ slot_of) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < rows; q += stride)
        slot_of[order[q]] = (int32_t)q;
}

// Walks the row in slot q in the solve's accumulation order.  TR = 0: row of A
// (indices/indptr); TR = 1: row of A^T (t_row/t_indptr, coefficient at t_perm).
// With `fill` == 0 it only counts the strictly-triangular entries.
template <int TR>
__global__ void pack_kernel(int64_t rows, int eff_lower, int fill, const int32_t *__restrict__ order,
                            const int32_t *__restrict__ slot_of, const int64_t *__restrict__ indices,
                            const int64_t *__restrict__ indptr, const int32_t *__restrict__ t_indptr,
                            const int32_t *__restrict__ t_row, const int32_t *__restrict__ t_perm,
                            int64_t *__restrict__ count64, const int32_t *__restrict__ dptr,
                            int32_t *__restrict__ dslot, int32_t *__restrict__ dsrc, int32_t *__restrict__ diag,
                            int32_t *max_deps) {
    // rows of this many entries and more are walked by the wavefront, 64 entries at a time (one
    // lane took a quarter of a second over a row of 2^19 entries)
    constexpr int64_t kLongPackRow = 1024;
    const int lane = threadIdx.x & 63;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    // (q0 is the same for the lanes of a wavefront: they stay in the loop together)
    for (int64_t q0 = (int64_t)blockIdx.x * blockDim.x + (threadIdx.x & ~63); q0 < rows; q0 += stride) {
        const int64_t q = q0 + lane;
        const bool live = q < rows;
        const int64_t i = live ? order[q] : 0;
        const int64_t kb = !live ? 0 : TR ? (int64_t)t_indptr[i] : indptr[i];
        const int64_t ke = !live ? 0 : TR ? (int64_t)t_indptr[i + 1] : indptr[i + 1];
        const int32_t out0 = live && fill ? dptr[q] : 0;
        const bool shared = ke - kb >= kLongPackRow;
        if (live && !shared) {
            int64_t n = 0;
            int32_t dpos = -1;
            int32_t out = out0;
            for (int64_t e = 0; e < ke - kb; ++e) {
                const int64_t k = eff_lower ? kb + e : ke - 1 - e;
                const int64_t j = TR ? (int64_t)t_row[k] : indices[k];
                const int32_t src = TR ? t_perm[k] : (int32_t)k;
                if (j == i) { dpos = src; continue; }
                if (eff_lower ? j > i : j < i) continue;   // other side of the diagonal: not part of the solve
                if (fill) { dslot[out] = slot_of[j]; dsrc[out] = src; ++out; }
                ++n;
            }
            if (fill) { diag[q] = dpos; if (n > *max_deps) atomicMax(max_deps, (int32_t)(n > 0x7fffffff ? 0x7fffffff : n)); }
            else count64[q] = n;
        }
        for (unsigned long long todo = __ballot(shared); todo; todo &= todo - 1) {
            const int owner = __builtin_ctzll(todo);
            const int64_t wi = __shfl(i, owner, 64), wkb = __shfl(kb, owner, 64), wke = __shfl(ke, owner, 64);
            const int32_t wout = __shfl(out0, owner, 64);
            int64_t n = 0;
            int32_t dpos = -1;
            for (int64_t e0 = 0; e0 < wke - wkb; e0 += 64) {
                const int64_t e = e0 + lane;
                const bool valid = e < wke - wkb;
                const int64_t k = !valid ? wkb : eff_lower ? wkb + e : wke - 1 - e;
                const int64_t j = TR ? (int64_t)t_row[k] : indices[k];
                const int32_t src = TR ? t_perm[k] : (int32_t)k;
                const bool on_diag = valid && j == wi;
                const bool keep = valid && !on_diag && !(eff_lower ? j > wi : j < wi);
                const unsigned long long kept = __ballot(keep), diags = __ballot(on_diag);
                if (fill && keep) {
                    const int64_t at = (int64_t)wout + n + __popcll(kept & ((1ull << lane) - 1));
                    dslot[at] = slot_of[j];
                    dsrc[at] = src;
                }
                n += __popcll(kept);
                if (diags) dpos = __shfl(src, 63 - __builtin_clzll(diags), 64);   // the last one met, as in the serial walk
            }
            if (lane == owner) {
                if (fill) { diag[q] = dpos; if (n > *max_deps) atomicMax(max_deps, (int32_t)(n > 0x7fffffff ? 0x7fffffff : n)); }
                else count64[q] = n;
            }
        }
    }
}

__global__ void narrow_kernel(int64_t n, const int64_t *__restrict__ in, int32_t *__restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = (int32_t)in[i];
}

// ---- solve kernels -----------------------------------------------------------

// Per-solve scratch (doubles): [xs: rows][diag: rows][rhs: rows][coef: nnz]
struct SolveWork {
    double *xs;     // running solution in slot order
    double *dg;     // diagonal coefficient of slot q (0 when not stored)
    double *rhs;    // right-hand side of slot q
    double *coef;   // coefficient of packed dependency `at`
    double *ell_coef;  // fixed-width copy of coef (0 padded), `pre` per slot
    double *rb;        // (right-hand side, diagonal) pairs per slot
    int32_t *status;   // [2]: nonzero when a kernel of this solve gave up waiting
    unsigned long long *cells;   // mailbox of values that pass between the workgroups of a shared launch, two words each
};

inline size_t solve_work_layout(int64_t rows, int64_t nnz, void *base, SolveWork *W) {
    size_t off = 0;
    auto take = [&](size_t count) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align_up(count * 8);
        return (double *)q;
    };
    SolveWork w;
    w.xs = take(rows + 1 + kEllPad);
    w.dg = take(rows + 1);
    w.rhs = take(rows + 1);
    w.coef = take(nnz + 1);
    w.ell_coef = take(coef_capacity(rows, nnz));
    w.rb = take(2 * (rows + kEllPad) + 2);
    w.status = (int32_t *)take(2);
    w.cells = (unsigned long long *)take(2 * (team_cells_capacity(rows) + kTeamCellPadding) + 2);
    if (W) *W = w;
    return off;
}

// Gathers this call's values into the plan's level-major order, converting to
// double once: a bandwidth-bound pass over the whole chip, after which the
// single-workgroup solve reads nothing but contiguous streams.
template <typename T>
__global__ void gather_values_kernel(int64_t rows, int64_t nnz, const T *__restrict__ data,
                                     const T *__restrict__ b, const int32_t *__restrict__ order,
                                     const int32_t *__restrict__ dptr, const int32_t *__restrict__ dsrc,
                                     const int32_t *__restrict__ diag, double *__restrict__ coef,
                                     double *__restrict__ dg, double *__restrict__ rhs) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = dptr[rows];
    for (int64_t at = tid; at < total; at += stride) coef[at] = (double)data[dsrc[at]];
    for (int64_t q = tid; q < rows; q += stride) {
        const int32_t d = diag[q];
        dg[q] = d >= 0 ? (double)data[d] : 0.;
        rhs[q] = (double)b[order[q]];
    }
}

struct SolveArgs {
    SolveWork w;
    const int32_t *level_ptr, *dptr, *dslot;
    int unit;
};

// Register pipeline stages of the single-workgroup kernel.
struct Bounds { int qb, qe; };
struct Meta { int q; bool live; int32_t dlo, n; };
template <int PRE> struct Vals { Meta m; int32_t ds[PRE]; double v[PRE]; double dv, bv; };

// Level bounds come from an LDS copy of this launch's slice of level_ptr
// (s_lp[i] = level_ptr[lmin + i]), so they cost no scalar-memory round trip.
__device__ __forceinline__ Bounds load_bounds(const int32_t *s_lp, int it, int count, int l0, int step, int lmin) {
    Bounds r{0, 0};
    if (it < count) {
        const int l = l0 + it * step - lmin;
        r.qb = s_lp[l];
        r.qe = s_lp[l + 1];
    }
    return r;
}

// All loads below are unconditional with clamped indices (slot 0 / entry 0 always
// exist), so a stage is straight-line code and the hardware wait counters stay exact.
__device__ __forceinline__ Meta load_meta(const SolveArgs &a, const Bounds &b) {
    Meta m;
    m.q = b.qb + (int)threadIdx.x;
    m.live = m.q < b.qe;
    const int qs = m.live ? m.q : 0;
    m.dlo = a.dptr[qs];
    m.n = a.dptr[qs + 1] - m.dlo;
    return m;
}

template <int PRE> __device__ __forceinline__ Vals<PRE> load_vals(const SolveArgs &a, const Meta &m) {
    Vals<PRE> v;
    v.m = m;
#pragma unroll
    for (int e = 0; e < PRE; ++e) {
        const int32_t at = (m.live && e < m.n) ? m.dlo + e : 0;
        v.ds[e] = a.dslot[at];
        v.v[e] = a.w.coef[at];
    }
    const int qs = m.live ? m.q : 0;
    v.dv = a.w.dg[qs];
    v.bv = a.w.rhs[qs];
    return v;
}

// Levels l0, l0+step, ... (`count` <= kMaxLevels of them, each at most kNarrow
// rows) by one workgroup; [qlo, qhi) are the slots this launch solves (only
// those can be found in the ring).
// Global loads reach the registers through two stages, each issued DEPTH levels
// before it is needed: the slot's dependency range (`Meta`), then the dependencies
// themselves (`Vals`, whose addresses come from the range).  A level takes a few
// hundred cycles once its operands are in registers but a global load takes one to
// two thousand, so with DEPTH = 1 every level waited for memory.
// MAXT: the largest workgroup the instantiation is launched with (512 leaves a wavefront twice the
// registers of 1024, which the 16-deep pipeline needs to stay out of scratch memory).
template <int PRE, int DEPTH, int MAXT = kNarrow>
__global__ __launch_bounds__(MAXT) void sptrsv_ring_kernel(SolveArgs a, int l0, int count, int step, int qlo,
                                                           int qhi) {
    __shared__ double ring[kRing];
    __shared__ int32_t s_lp[kMaxLevels + 1];
    const int lmin = step > 0 ? l0 : l0 - (count - 1);
    for (int i = threadIdx.x; i <= count; i += blockDim.x) s_lp[i] = a.level_ptr[lmin + i];
    __syncthreads();

    Meta qm[DEPTH];          // ranges of levels it + DEPTH .. it + 2 DEPTH - 1
    Vals<PRE> qv[DEPTH];     // operands of levels it .. it + DEPTH - 1
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) qm[d] = load_meta(a, load_bounds(s_lp, d, count, l0, step, lmin));
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) qv[d] = load_vals<PRE>(a, qm[d]);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) qm[d] = load_meta(a, load_bounds(s_lp, DEPTH + d, count, l0, step, lmin));

    // The level loop is unrolled DEPTH times so that stage d always lives in the same
    // registers: a stage is consumed and then refilled in place.  (Rotating the stages
    // through register copies made every level wait for the loads it had just issued.)
    for (int it0 = 0; it0 < count; it0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int it = it0 + d;
            if (it >= count) break;   // uniform over the workgroup
            const Vals<PRE> cur = qv[d];
            qv[d] = load_vals<PRE>(a, qm[d]);
            qm[d] = load_meta(a, load_bounds(s_lp, it + 2 * DEPTH, count, l0, step, lmin));

            const int q = cur.m.q;
            const int n = cur.m.live ? cur.m.n : 0;
            // fast path: no global memory access at all -- every dependency from the LDS ring
            // ring reads first, together and unconditionally; whether a term counts is a select
            // afterwards (a read inside `if (e < n)` sits in its own branch with its own wait)
            double xj[PRE];
#pragma unroll
            for (int e = 0; e < PRE; ++e) xj[e] = ring[cur.ds[e] & (kRing - 1)];
            double acc = 0.;
            bool in_ring = n <= PRE;
#pragma unroll
            for (int e = 0; e < PRE; ++e) {
                const int32_t ds = cur.ds[e];
                const int dist = ds > q ? ds - q : q - ds;
                const bool hit = ds >= qlo && ds < qhi && dist < kRingSafe;
                const double term = cur.v[e] * xj[e];
                acc += e < n ? term : 0.;        // + 0.0 leaves the sum as it is
                in_ring = in_ring && (hit || e >= n);
            }
            if (!in_ring) {
                // slow path (a dependency older than the ring, or a row longer than the
                // pipeline holds): redo the whole sum in the same order from global memory.
                // The solutions of the first PRE dependencies are requested together (their
                // slots are in registers; unused ones name a valid slot), the rest one by one.
                double xg[PRE];
#pragma unroll
                for (int e = 0; e < PRE; ++e) xg[e] = a.w.xs[cur.ds[e]];
                acc = 0.;
#pragma unroll
                for (int e = 0; e < PRE; ++e) acc += e < n ? cur.v[e] * xg[e] : 0.;
                for (int e = PRE; e < n; ++e) {
                    const int32_t at = cur.m.dlo + e;
                    acc += a.w.coef[at] * a.w.xs[a.dslot[at]];
                }
            }
            if (cur.m.live) {
                double xi = cur.bv - acc;
                if (!a.unit) xi /= cur.dv;
                ring[q & (kRing - 1)] = xi;
                a.w.xs[q] = xi;
            }
            __syncthreads();
        }
    }
}

// ---- long rows: several lanes per row ---------------------------------------------
//
// The kernels above give a row to one lane, which walks its dependencies one after the
// other: right for the handful of entries a row of a sparse triangle usually has, but the
// factors of a direct solve have rows of dozens to hundreds of entries in levels of one or
// a few rows, and the level then lasts as long as that serial walk.  Here G lanes share a
// row: each multiplies every G-th dependency, the partial sums are added across the group
// (in double, so the rounding differs from the serial order by a few units in the last
// place of a double), and the group's first lane finishes the row.  The first G
// dependencies of a row come through the same two-stage register pipeline as above.
struct GVals { Meta m; int32_t ds; double v, dv, bv; };

template <int G> __device__ __forceinline__ Meta load_gmeta(const SolveArgs &a, const Bounds &b) {
    Meta m;
    m.q = b.qb + (G == 64 ? __builtin_amdgcn_readfirstlane((int)threadIdx.x / G) : (int)threadIdx.x / G);
    m.live = m.q < b.qe;
    const int qs = m.live ? m.q : 0;
    m.dlo = a.dptr[qs];
    m.n = a.dptr[qs + 1] - m.dlo;
    return m;
}

template <int G> __device__ __forceinline__ GVals load_gvals(const SolveArgs &a, const Meta &m) {
    GVals v;
    v.m = m;
    const int sub = (int)threadIdx.x & (G - 1);
    const int32_t at = (m.live && sub < m.n) ? m.dlo + sub : 0;
    v.ds = a.dslot[at];
    v.v = a.w.coef[at];
    const int qs = m.live ? m.q : 0;
    v.dv = a.w.dg[qs];
    v.bv = a.w.rhs[qs];
    return v;
}

template <int G> __device__ __forceinline__ double group_total(double v) {
    if (G == 64) return nm::wave_sum(v);
    v += nm::dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]
    v += nm::dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
    v += nm::dpp_move<0x124>(v);   // row_ror 4
    v += nm::dpp_move<0x128>(v);   // row_ror 8: every lane of the 16-lane row holds the row's sum
    return v;
}

template <int G, int DEPTH>
__global__ __launch_bounds__(kNarrow) void sptrsv_group_kernel(SolveArgs a, int l0, int count, int step, int qlo,
                                                               int qhi) {
    static_assert(G == 16 || G == 64, "group sums are written for a DPP row or a wavefront");
    __shared__ double ring[kRing];
    __shared__ int32_t s_lp[kMaxLevels + 1];
    const int lmin = step > 0 ? l0 : l0 - (count - 1);
    for (int i = threadIdx.x; i <= count; i += blockDim.x) s_lp[i] = a.level_ptr[lmin + i];
    __syncthreads();
    const int sub = (int)threadIdx.x & (G - 1), ngroups = (int)blockDim.x / G;

    // x of slot ds as seen from slot q: the ring holds what this launch solved recently
    auto solved = [&](int32_t ds, int q) {
        const int dist = ds > q ? ds - q : q - ds;
        return (ds >= qlo && ds < qhi && dist < kRingSafe) ? ring[ds & (kRing - 1)] : a.w.xs[ds];
    };

    Meta qm[DEPTH];
    GVals qv[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) qm[d] = load_gmeta<G>(a, load_bounds(s_lp, d, count, l0, step, lmin));
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) qv[d] = load_gvals<G>(a, qm[d]);
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) qm[d] = load_gmeta<G>(a, load_bounds(s_lp, DEPTH + d, count, l0, step, lmin));

    for (int it0 = 0; it0 < count; it0 += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int it = it0 + d;
            if (it >= count) break;   // uniform over the workgroup
            const GVals cur = qv[d];
            qv[d] = load_gvals<G>(a, qm[d]);
            qm[d] = load_gmeta<G>(a, load_bounds(s_lp, it + 2 * DEPTH, count, l0, step, lmin));
            const int qe = s_lp[l0 + it * step - lmin + 1];

            // this group's first row of the level: operands already in registers
            {
                const int q = cur.m.q, n = cur.m.live ? cur.m.n : 0;
                double acc = sub < n ? cur.v * solved(cur.ds, q) : 0.;
                for (int e = sub + G; e < n; e += G) {
                    const int32_t at = cur.m.dlo + e;
                    acc += a.w.coef[at] * solved(a.dslot[at], q);
                }
                acc = group_total<G>(acc);
                if (cur.m.live && sub == 0) {
                    double xi = cur.bv - acc;
                    if (!a.unit) xi /= cur.dv;
                    ring[q & (kRing - 1)] = xi;
                    a.w.xs[q] = xi;
                }
            }
            // a level with more rows than groups: the rest straight from memory
            for (int q0 = cur.m.q + ngroups; q0 - (int)threadIdx.x / G < qe; q0 += ngroups) {
                const bool live = q0 < qe;
                const int q = live ? q0 : 0;
                const int32_t dlo = a.dptr[q], n = live ? a.dptr[q + 1] - dlo : 0;
                double acc = 0.;
                for (int e = sub; e < n; e += G) acc += a.w.coef[dlo + e] * solved(a.dslot[dlo + e], q);
                acc = group_total<G>(acc);
                if (live && sub == 0) {
                    double xi = a.w.rhs[q] - acc;
                    if (!a.unit) xi /= a.w.dg[q];
                    ring[q & (kRing - 1)] = xi;
                    a.w.xs[q] = xi;
                }
            }
            __syncthreads();
        }
    }
}

// ---- fixed-width (ELLPACK) variant of the single-workgroup kernel -----------------
//
// When no row has more than 8 dependencies, the packed triangle is also kept with a
// fixed number PRE of dependency slots per row (-1 / 0.0 padded).  Every address a
// level needs is then a multiple of its slot number: one vector load each for the
// PRE dependency slots, the PRE coefficients and the (rhs, diagonal) pair, no
// dependency-range stage in front of them, and a third of the address arithmetic --
// which matters because the workgroup's wavefronts share one CU and the level time
// is the time to issue their instructions.

// An entry of the fixed-width dependency array is what the level needs and nothing else, in 16
// bits: twice the number of the dependency's entry in the LDS ring (four times that is its byte
// offset there), plus 1 when the ring of this launch cannot serve it (the row was solved by
// another launch, or too many slots ago; the rare slow path then finds the slot in the
// range-based arrays).  An absent dependency points at ring entry kRing, which holds 0.0 for
// ever, and its coefficient is 0.0: it adds +0.0 to the sum, so the level needs no "is there a
// dependency" test at all.  Deciding all this once, at plan time, keeps a dozen instructions per
// dependency out of every level.  (Two bytes, not four: everything a row needs passes through
// the ONE compute unit the workgroup lives on, at the ~110 GB/s that unit can stream -- 44
// instead of 48 bytes a row were 0.97 -> 0.88 ms per solve on the 1024^2 triangle.)
constexpr uint32_t kEllFarPair = 0x00010001u;       // the "not in the ring" bits of a pair of entries
constexpr uint32_t kEllByteMask = 0x3fff8u;         // byte offset in the ring, once the entry is shifted in place
static_assert(kRing * 2 + 1 < 65536 && (kRing * 8 & ~kEllByteMask) == 0, "a ring entry number fits 15 bits");
__device__ __forceinline__ uint32_t ell_ring_bytes(uint32_t pair, int e) {
    return (e & 1) ? (pair >> 14) & kEllByteMask : (pair << 2) & kEllByteMask;
}

__device__ __forceinline__ int32_t level_of_slot(const int32_t *__restrict__ level_ptr, int32_t nlevels, int32_t q) {
    int32_t lo = 0, hi = nlevels;   // last l with level_ptr[l] <= q
    while (hi - lo > 1) {
        const int32_t mid = (lo + hi) >> 1;
        if (level_ptr[mid] <= q) lo = mid; else hi = mid;
    }
    return lo;
}

__global__ void ell_pack_kernel(int64_t rows, int pre, const int32_t *__restrict__ dptr,
                                const int32_t *__restrict__ dslot, const int32_t *__restrict__ level_ptr,
                                int32_t nlevels, const int32_t *__restrict__ level_launch,
                                uint16_t *__restrict__ ell_ds, int32_t *__restrict__ reach,
                                int32_t *__restrict__ lvl_sig) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    // the padding slots behind the last row get "absent" entries: lanes that read them must find a valid offset
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (rows + kEllPad) * pre; i += stride) {
        const int64_t q = i / pre;
        const int e = (int)(i - q * pre);
        const int32_t lo = q < rows ? dptr[q] : 0, n = q < rows ? dptr[q + 1] - lo : 0;
        uint32_t out = kRing * 2;   // absent: the ring entry that is always 0.0
        if (e < n) {
            const int32_t ds = dslot[lo + e];
            const int32_t dist = ds > (int32_t)q ? ds - (int32_t)q : (int32_t)q - ds;
            const int32_t lq = level_of_slot(level_ptr, nlevels, (int32_t)q), ld = level_of_slot(level_ptr, nlevels, ds);
            const bool same = level_launch[lq] == level_launch[ld];
            const bool near = same && dist < kRingSafe;
            out = ((uint32_t)(ds & (kRing - 1)) * 2) | (near ? 0u : 1u);
            if (!near && (lvl_sig[lq] & kSigFar) == 0) atomicOr(lvl_sig + lq, kSigFar);
            if (near) {
                // wavefront of the row and of the row it waits for, each inside its own level
                const int32_t wq = ((int32_t)q - level_ptr[lq]) >> 6, wd = (ds - level_ptr[ld]) >> 6;
                int32_t far = wq > wd ? wq - wd : wd - wq;
                if (dist >= kRingSafeSig) far = kSigNever;   // too far back for wavefronts that run apart
                if (far > *reach) atomicMax(reach, far);
                // which neighbour the rows of this level wait for: with dependencies on one side only,
                // the wavefronts form a pipeline instead of moving in step
                const int32_t bit = wd < wq ? kSigLower : (wd > wq ? kSigHigher : 0);
                if (bit && (lvl_sig[lq] & bit) == 0) atomicOr(lvl_sig + lq, bit);
            }
        }
        ell_ds[i] = (uint16_t)out;
    }
}

template <typename T>
__global__ void gather_ell_kernel(int64_t rows, int pre, const T *__restrict__ data, const T *__restrict__ b,
                                  const int32_t *__restrict__ order, const int32_t *__restrict__ dptr,
                                  const int32_t *__restrict__ dsrc, const int32_t *__restrict__ diag,
                                  double *__restrict__ ell_coef, double *__restrict__ rb,
                                  int32_t *__restrict__ status, unsigned long long *__restrict__ cells,
                                  int64_t cell_words) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid == 0) status[0] = 0;   // first kernel of the solve
    // the mailbox of the launches that several workgroups share: empty before the solve starts
    for (int64_t i = tid; i < cell_words; i += stride) cells[i] = 0ull;
    for (int64_t i = tid; i < rows * pre; i += stride) {
        const int64_t q = i / pre;
        const int e = (int)(i - q * pre);
        const int32_t lo = dptr[q], n = dptr[q + 1] - lo;
        ell_coef[i] = e < n ? (double)data[dsrc[lo + e]] : 0.;
    }
    for (int64_t q = tid; q < rows; q += stride) {
        const int32_t d = diag[q];
        rb[2 * q] = (double)b[order[q]];
        rb[2 * q + 1] = d >= 0 ? (double)data[d] : 0.;
    }
}

struct EllArgs {
    const int32_t *level_ptr, *dptr, *dslot, *lvl_sig;
    const uint16_t *ell_ds;
    const double *ell_coef, *rb;
    double *xs;
    int unit;
};

// Operands of the slot qb + lane of a level.  qb is a scalar, so each of the three loads is
// `scalar base + the lane's constant byte offset`: no vector address arithmetic per level.
// Lanes beyond the level's end load the slots that follow it (readable: see kEllPad) and
// compute a value that is never stored.
template <int PRE> struct EllVals {
    int qb, qe;
    uint32_t ds[PRE / 2];   // pairs of 16-bit dependency entries
    double v[PRE];
    double bv, dv;
};

// Makes the compiler have the operands of a stage in registers HERE (an empty instruction that
// claims to read and write them): used to keep copies between stages in front of the next request.
template <int PRE> __device__ __forceinline__ void settle(EllVals<PRE> &v) {
#pragma unroll
    for (int e = 0; e < PRE / 2; ++e) asm volatile("" : "+v"(v.ds[e]));
#pragma unroll
    for (int e = 0; e < PRE; ++e) asm volatile("" : "+v"(v.v[e]));
    asm volatile("" : "+v"(v.bv));
    asm volatile("" : "+v"(v.dv));
}

// The same from a copy of the launch's level bounds with kBoundsPad more entries at either end
// (repeats of the first and of the last bound): the levels behind the launch's last one, whose
// operands the pipeline requests all the same, are empty ones there, and the read needs no test.
constexpr int kBoundsPad = 8;
__device__ __forceinline__ Bounds load_bounds_padded(const int32_t *s_lpp, int it, int l0, int step, int lmin) {
    const int l = l0 + it * step - lmin + kBoundsPad;
    return Bounds{__builtin_amdgcn_readfirstlane(s_lpp[l]), __builtin_amdgcn_readfirstlane(s_lpp[l + 1])};
}

__device__ __forceinline__ Bounds load_bounds_uniform(const int32_t *s_lp, int it, int count, int l0, int step,
                                                      int lmin) {
    const Bounds b = load_bounds(s_lp, it, count, l0, step, lmin);
    return Bounds{__builtin_amdgcn_readfirstlane(b.qb), __builtin_amdgcn_readfirstlane(b.qe)};
}

template <int PRE> __device__ __forceinline__ EllVals<PRE> load_ell(const EllArgs &a, const Bounds &b) {
    static_assert(PRE % 2 == 0, "dependency entries come in pairs");
    typedef uint32_t IV __attribute__((ext_vector_type(PRE / 2)));
    typedef double DV __attribute__((ext_vector_type(PRE)));
    typedef double D2 __attribute__((ext_vector_type(2)));
    EllVals<PRE> v;
    v.qb = b.qb;
    v.qe = b.qe;
    const uint32_t lane_ds = threadIdx.x * (uint32_t)(sizeof(uint16_t) * PRE);
    const uint32_t lane_cf = threadIdx.x * (uint32_t)(sizeof(double) * PRE);
    const uint32_t lane_rb = threadIdx.x * (uint32_t)(sizeof(double) * 2);
    const char *pd = reinterpret_cast<const char *>(a.ell_ds) + (int64_t)b.qb * (int64_t)(sizeof(uint16_t) * PRE);
    const char *pc = reinterpret_cast<const char *>(a.ell_coef) + (int64_t)b.qb * (int64_t)(sizeof(double) * PRE);
    const char *pr = reinterpret_cast<const char *>(a.rb) + (int64_t)b.qb * (int64_t)(sizeof(double) * 2);
    const IV dsv = *reinterpret_cast<const IV *>(pd + lane_ds);
    const DV cv = *reinterpret_cast<const DV *>(pc + lane_cf);
    const D2 r = *reinterpret_cast<const D2 *>(pr + lane_rb);
#pragma unroll
    for (int e = 0; e < PRE / 2; ++e) v.ds[e] = dsv[e];
#pragma unroll
    for (int e = 0; e < PRE; ++e) v.v[e] = cv[e];
    v.bv = r[0];
    v.dv = r[1];
    return v;
}

// The workgroup lives on one CU and a level lasts as long as it takes to issue every
// wavefront's instructions for it (four wavefronts per SIMD at 1024 rows, ~4 cycles per vector
// instruction), so the level body is kept to what cannot be decided earlier: the ring reads
// (offsets precomputed), the sum, the division, and the two stores.
//
// SIG: instead of a workgroup barrier after every level, a wavefront publishes the number of
// levels it has finished and, before a level, waits until the wavefronts it can depend on (those
// at most kSigReach away: the plan has checked that no row looks further) have finished the level
// before, and until no wavefront is more than kSkew levels behind (the ring keeps what such a
// straggler still reads).  A wavefront that has the rows of a level ready early goes on to the
// next one while the others finish, so the workgroup is no longer as slow as its slowest
// wavefront at every single level.  All wavefronts of the workgroup are resident and a
// wavefront only ever waits for lower levels, so the waits end; as a backstop a wavefront
// that has polled `poll_limit` times without success raises a flag that makes every wavefront
// leave, and the solve's status word tells the last kernel of the solve to hand out NaN.
// Byte offset of a __shared__ object inside the workgroup's LDS.
__device__ __forceinline__ uint32_t lds_offset(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char *)p;
}

// Polls the LDS word at `at` until, in every lane, it is at least `need`, at most `limit` times;
// `seen` is what the last poll read, `left` the polls that were left (0: gave up).  `nap`: sleep
// between polls (0 none, 1 short, 2 long).  All 64 lanes must be active.
__device__ __forceinline__ void sig_wait(uint32_t at, int32_t need, int32_t limit, int nap, int32_t &seen,
                                         int32_t &left) {
    if (nap == 0)
        asm volatile("s_mov_b32 %1, %4\n"
                     "1:\n\t"
                     "ds_read_b32 %0, %2\n\t"
                     "s_waitcnt lgkmcnt(0)\n\t"
                     "v_cmp_lt_i32 vcc, %0, %3\n\t"
                     "s_cmp_eq_u64 vcc, 0\n\t"
                     "s_cbranch_scc1 2f\n\t"
                     "s_sub_u32 %1, %1, 1\n\t"
                     "s_cmp_eq_u32 %1, 0\n\t"
                     "s_cbranch_scc1 2f\n\t"
                     "s_branch 1b\n"
                     "2:\n"
                     : "=&v"(seen), "=&s"(left)
                     : "v"(at), "v"(need), "s"(limit)
                     : "vcc", "scc", "memory");
    else
        asm volatile("s_mov_b32 %1, %4\n"
                     "1:\n\t"
                     "ds_read_b32 %0, %2\n\t"
                     "s_waitcnt lgkmcnt(0)\n\t"
                     "v_cmp_lt_i32 vcc, %0, %3\n\t"
                     "s_cmp_eq_u64 vcc, 0\n\t"
                     "s_cbranch_scc1 2f\n\t"
                     "s_sub_u32 %1, %1, 1\n\t"
                     "s_cmp_eq_u32 %1, 0\n\t"
                     "s_cbranch_scc1 2f\n\t"
                     "s_sleep 1\n\t"
                     "s_branch 1b\n"
                     "2:\n"
                     : "=&v"(seen), "=&s"(left)
                     : "v"(at), "v"(need), "s"(limit)
                     : "vcc", "scc", "memory");
}

template <int PRE, int DEPTH, bool SIG = false>
__global__ __launch_bounds__(kNarrow) void sptrsv_ell_kernel(EllArgs a, int l0, int count, int step,
                                                             int64_t poll_limit = 0, int32_t *status = nullptr,
                                                             int tune_sleep = 1, int tune_skew = kSkew,
                                                             int far_levels = 0x7fffffff) {
    __shared__ double ring[kRing + 1];   // [kRing] stays 0.0: what an absent dependency reads
    __shared__ int32_t s_lp[kMaxLevels + 1 + 2 * kBoundsPad];   // padded: see load_bounds_padded
    static_assert(DEPTH + 2 <= kBoundsPad, "the pipeline looks DEPTH + 1 levels past the last");
    __shared__ int32_t s_done[kNarrow / 64];   // SIG: levels each wavefront has finished
    __shared__ int32_t s_abort;
    __shared__ uint8_t s_sig[SIG ? kMaxLevels : 1];   // SIG: the neighbours a level's rows wait for
    const int lmin = step > 0 ? l0 : l0 - (count - 1);
    for (int i = threadIdx.x; i <= count + 2 * kBoundsPad; i += blockDim.x) {
        const int at = i - kBoundsPad;
        s_lp[i] = a.level_ptr[lmin + (at < 0 ? 0 : (at > count ? count : at))];
    }
    if (SIG)
        for (int i = threadIdx.x; i < count; i += blockDim.x) s_sig[i] = (uint8_t)a.lvl_sig[lmin + i];
    if (threadIdx.x == 0) ring[kRing] = 0.;
    if (SIG && threadIdx.x < kNarrow / 64) s_done[threadIdx.x] = poll_limit < 0 ? 0x7fffffff : 0;
    if (SIG && threadIdx.x == 0) s_abort = poll_limit < 0 ? 1 : 0;   // a negative limit: give up at once (tests)
    __syncthreads();
    const int sig_lane = threadIdx.x & 63, sig_wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int sig_waves = blockDim.x >> 6;
    bool gave_up = SIG && poll_limit < 0;
    const char *ring_bytes = reinterpret_cast<const char *>(ring);
    const uint32_t lane8 = threadIdx.x * 8u;

    EllVals<PRE> qv[DEPTH];   // operands of levels it .. it + DEPTH - 1, each refilled in place
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) qv[d] = load_ell<PRE>(a, load_bounds_padded(s_lp, d, l0, step, lmin));
    // The bounds of the level whose operands are requested next are read from LDS one level
    // early, before the barrier, so that the request does not start with an LDS round trip.
    Bounds ahead = load_bounds_padded(s_lp, DEPTH, l0, step, lmin);

    // one level: `cur` holds its operands
    auto level = [&](int it, const EllVals<PRE> &cur) {
        // all ring reads go out together, unconditionally
        double xj[PRE];
        uint32_t any = 0;
#pragma unroll
        for (int e = 0; e < PRE; ++e) {
            xj[e] = *reinterpret_cast<const double *>(ring_bytes + ell_ring_bytes(cur.ds[e / 2], e));
            any |= cur.ds[e / 2];
        }
        ahead = load_bounds_padded(s_lp, it + DEPTH + 1, l0, step, lmin);
        double acc = 0.;
#pragma unroll
        for (int e = 0; e < PRE; ++e) acc += cur.v[e] * xj[e];   // absent: 0.0 * 0.0
        const bool live = (int)threadIdx.x < cur.qe - cur.qb;
        if ((any & kEllFarPair) && live) {
            // a dependency the ring does not hold: redo the sum in the same order from global memory
            // (slots and then solutions are requested together; entries past the row's own
            //  name a valid slot and are not added)
            const int q = cur.qb + (int)threadIdx.x;
            const int32_t dlo = a.dptr[q], n = a.dptr[q + 1] - dlo;
            int32_t sl[PRE];
            double xg[PRE];
#pragma unroll
            for (int e = 0; e < PRE; ++e) sl[e] = a.dslot[dlo + (e < n ? e : 0)];
#pragma unroll
            for (int e = 0; e < PRE; ++e) xg[e] = a.xs[sl[e]];
            acc = 0.;
#pragma unroll
            for (int e = 0; e < PRE; ++e) acc += e < n ? cur.v[e] * xg[e] : 0.;
        }
        double xi = cur.bv - acc;
        if (!a.unit) xi /= cur.dv;
        if (live) {
            const uint32_t at = (uint32_t)cur.qb * 8u + lane8;
            *reinterpret_cast<double *>(const_cast<char *>(ring_bytes) + (at & (kRing * 8 - 1))) = xi;
            *reinterpret_cast<double *>(reinterpret_cast<char *>(a.xs) + (int64_t)cur.qb * 8 + lane8) = xi;
        }
    };
    if (!SIG) {
        // (the level body is written out here rather than shared with the signalling loop below:
        // shared through that loop's lambda it compiled to a few more scalar instructions per level)
        //
        // LEAN: the levels behind the launch's first `far_levels`, in which no row reads a row that
        // the ring cannot serve (the plan knows), of a solve that divides by the diagonal.  Their
        // body has no test for such rows and none for the unit diagonal: a level lasts as long as it
        // takes one wavefront to issue its ~70 instructions, and these are eleven of them
        // (0.92 -> 0.88 ms per solve on the 1024^2 triangle).
        auto one_level = [&](auto lean, int it, EllVals<PRE> &stage) {
            constexpr bool LEAN = decltype(lean)::value;
            const EllVals<PRE> cur = stage;
            stage = load_ell<PRE>(a, ahead);

            // all ring reads go out together, unconditionally
            // (unpacking the offsets one level early, in the shadow of that level's ring reads,
            // was slower, 0.92 -> 1.12 ms: state carried from level to level makes the compiler
            // wait for the operand request just issued)
            double xj[PRE];
            uint32_t any = 0;
#pragma unroll
            for (int e = 0; e < PRE; ++e) {
                xj[e] = *reinterpret_cast<const double *>(ring_bytes + ell_ring_bytes(cur.ds[e / 2], e));
                any |= cur.ds[e / 2];
            }
            ahead = load_bounds_padded(s_lp, it + DEPTH + 1, l0, step, lmin);
            double acc = 0.;
#pragma unroll
            for (int e = 0; e < PRE; ++e) acc += cur.v[e] * xj[e];   // absent: 0.0 * 0.0
            const bool live = (int)threadIdx.x < cur.qe - cur.qb;
            if (!LEAN && (any & kEllFarPair) && live) {
                // a dependency the ring does not hold: redo the sum in the same order from global memory
                // (slots and then solutions are requested together; entries past the row's own
                //  name a valid slot and are not added)
                const int q = cur.qb + (int)threadIdx.x;
                const int32_t dlo = a.dptr[q], n = a.dptr[q + 1] - dlo;
                int32_t sl[PRE];
                double xg[PRE];
#pragma unroll
                for (int e = 0; e < PRE; ++e) sl[e] = a.dslot[dlo + (e < n ? e : 0)];
#pragma unroll
                for (int e = 0; e < PRE; ++e) xg[e] = a.xs[sl[e]];
                acc = 0.;
#pragma unroll
                for (int e = 0; e < PRE; ++e) acc += e < n ? cur.v[e] * xg[e] : 0.;
            }
            double xi = cur.bv - acc;
            if (LEAN || !a.unit) xi /= cur.dv;
            if (live) {
                const uint32_t at = (uint32_t)cur.qb * 8u + lane8;
                *reinterpret_cast<double *>(const_cast<char *>(ring_bytes) + (at & (kRing * 8 - 1))) = xi;
                *reinterpret_cast<double *>(reinterpret_cast<char *>(a.xs) + (int64_t)cur.qb * 8 + lane8) = xi;
            }
            __syncthreads();
        };
        // whole rounds of DEPTH levels with the tests, the rest without
        const int tested = a.unit || far_levels >= count ? count : (far_levels + DEPTH - 1) / DEPTH * DEPTH;
        int it0 = 0;
        for (; it0 < tested; it0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                if (it0 + d >= count) break;   // uniform over the workgroup
                one_level(std::false_type{}, it0 + d, qv[d]);
            }
        }
        for (; it0 < count; it0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                if (it0 + d >= count) break;
                one_level(std::true_type{}, it0 + d, qv[d]);
            }
        }
    } else {
        // Stages are refilled in place, as above.  The wait for the neighbours is written in
        // assembly (sig_wait): with a polling LOOP among the level's statements the compiler hands
        // the operand stages from level to level through register copies, and the copy of the
        // stage just requested waits for that request -- a memory round trip per level, far more
        // than any rendezvous costs.  As one opaque instruction the wait leaves the loop as
        // straight as the barrier version's.
        //   lane w < waves polls s_done[w]; lane 63 reads the abort word along with them.
        const uint32_t poll_at = lds_offset(sig_lane < sig_waves ? (const void *)&s_done[sig_lane] : (const void *)&s_abort);
        const int32_t limit32 = poll_limit > 0x7fffffff ? 0x7fffffff : (poll_limit < 1 ? 1 : (int32_t)poll_limit);
        for (int it0 = 0; it0 < count; it0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                const int it = it0 + d;
                if (it >= count) break;   // uniform over the workgroup
                // the wavefronts this one waits for at this level: the lower and / or the higher
                // neighbour must have finished the level before; nobody may be kSkew levels behind
                const int32_t sides = s_sig[l0 + it * step - lmin];
                const bool near = (sig_lane + 1 == sig_wave && (sides & kSigLower)) ||
                                  (sig_lane == sig_wave + 1 && (sides & kSigHigher));
                const int32_t need = sig_lane < sig_waves ? (near ? it : it - tune_skew) : (int32_t)0x80000000;
                int32_t seen, left;
                sig_wait(poll_at, need, limit32, tune_sleep, seen, left);
                int32_t aborted = __builtin_amdgcn_readlane(seen, 63);
                if (__builtin_expect(left == 0, 0)) {
                    // out of polls: every counter jumps to the end, so that nobody waits for anybody
                    // any more, and the abort word makes the solve hand out NaN
                    if (sig_lane < kNarrow / 64)
                        __hip_atomic_store(&s_done[sig_lane], 0x7fffffff, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    if (sig_lane == 0) __hip_atomic_store(&s_abort, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    aborted = 1;
                }
                const EllVals<PRE> cur = qv[d];
                qv[d] = load_ell<PRE>(a, ahead);
                level(it, cur);
                // the ring write above is in LDS before the count moves (one wavefront's LDS
                // accesses are served in the order it issued them); after an abort the count stays
                // at the end
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                if (sig_lane == 0)
                    __hip_atomic_store(&s_done[sig_wave], aborted ? 0x7fffffff : it + 1, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
        gave_up = __hip_atomic_load(&s_abort, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0;
    }
    if (SIG && gave_up && sig_lane == 0 && status) status[0] = 1;
}

// ---- several workgroups per level ---------------------------------------------------------
//
// One workgroup streams a level's operands through the one compute unit it lives on, and at a
// thousand rows a level that is what a level costs (44 bytes a row at the ~110 GB/s one unit
// streams).  Here P workgroups share every level of a launch: workgroup k takes a part of at
// most kTeamChunk rows of each level (the plan's table says which: see team_parts_kernel), so
// each unit streams a fraction.  What keeps that from costing a hand-over between compute units
// per level (0.6-0.75 us through device memory, more than a whole level takes) is that the
// workgroups do NOT move in step:
//
//  * a workgroup keeps its own LDS ring and its own barrier per level, exactly as the
//    single-workgroup kernel does, with two more wavefronts that compute nothing;
//  * a value that a row of ANOTHER workgroup needs (the plan lists them: `exports`, by the level
//    that produces them) is read from the ring by the first service wavefront one level after
//    it was computed and stored to a mailbox cell in device memory: two 64-bit words, each half
//    of the double next to a tag, so that a reader that finds both tags set has the whole value
//    (a naturally aligned 64-bit access is never torn; no fence, no second flag);
//  * the second service wavefront polls the cells of the workgroup's `imports` (listed by the
//    level that first needs them) several levels ahead of use and writes what has arrived into
//    the ring; only when a value is still missing at the barrier before the level that needs it
//    does it wait, and with it the workgroup.
//
// Where values cross between two workgroups in one direction (parts by row number: always; the
// tril of a grid cut by position: a row depends on its left and lower neighbours of the previous
// level) the consumers simply fall a few levels behind their producers and nobody waits again.
// The plan only makes a launch shared when that is possible: per level, "workgroup a needs a
// value that workgroup b computes at the level before" must not form a cycle (such a level would
// need the hand-over inside the level; see build_team).  Every workgroup of the grid is resident
// (P <= 16 of the chip's 256 units) and a workgroup only waits for values of lower levels, so the
// waits end; as a backstop a service wavefront that has polled `poll_limit` times for one level
// stops waiting for good and the solve hands out NaN, as for the signalling kernel above.
constexpr int kTeamChunk = 256;            // most rows of a level that one workgroup takes
constexpr int kTeamStages = 6;             // polls in flight
constexpr int kTeamAhead = kRing - kRingSafe;   // slots ahead of its own level a workgroup may import
constexpr int kTeamExports = 2048;         // values one workgroup may hand out in one launch (their list lives in LDS)
static_assert((kTeamExports & (kTeamExports - 1)) == 0, "a power of two");
constexpr int kTeamLevels = kTeamExports;  // most levels of a launch that a team may share
constexpr int kTeamNeedBits = 18;          // a workgroup's imports in one launch are counted in these
static_assert(kTeamExports < (1 << (31 - kTeamNeedBits)), "exports and imports share a word");
static_assert(kTeamCellPadding >= 64, "a poll reads 64 cells from any import on");

struct TeamArgs {
    const int32_t *tab;          // [P][count+1] imports needed up to a level, [P][count+1] exports before a level,
                                 // [n_imp] slot of an import (not read by the kernel: the cell names it),
                                 // [n_imp] slot of an export, [n_imp] its cell,
                                 // [count][P+1] the slots at which the workgroups' parts of a level start
    unsigned long long *cells;   // this launch's mailbox cells
    int32_t P, n_imp;
    int32_t quiet;               // first of the padding cells, counted from `cells`
    int32_t imp_off[kTeamMax + 1], exp_off[kTeamMax + 1];
};

struct TeamPoll { int cs; unsigned long long w0, w1; };

template <int PRE, int DEPTH>
__global__ __launch_bounds__(kTeamChunk + 128) void sptrsv_team_kernel(EllArgs a, TeamArgs t, int l0, int count, int step,
                                                                       int64_t poll_limit, int32_t *status, int far_levels) {
    __shared__ double ring[kRing + 1];   // [kRing] stays 0.0: what an absent dependency reads
    // this workgroup's part of every level: first slot, end; kBoundsPad empty parts at either end
    // for the levels behind the launch's last one, whose operands the pipeline requests all the same
    __shared__ int2 s_mine[kMaxLevels + 1 + 2 * kBoundsPad];
    static_assert(DEPTH + 2 <= kBoundsPad, "the pipeline looks DEPTH + 1 levels past the last");
    // what the service wavefronts need at a level, in one LDS read: x = the limit an imported
    // slot (times `step`) is held against, y = imports the NEXT level needs (low kTeamNeedBits
    // bits) and exports of the levels before this one (the bits above)
    __shared__ int2 s_sv[kMaxLevels + 1];
    __shared__ int2 s_exl[kTeamExports];   // (slot, cell) of this workgroup's exports
    const int k = blockIdx.x;
    const int lmin = step > 0 ? l0 : l0 - (count - 1);
    const int32_t *parts = t.tab + 2 * t.P * (count + 1) + 3 * t.n_imp;   // [level - lmin][P + 1]
    for (int i = threadIdx.x; i < count + 2 * kBoundsPad; i += blockDim.x) {
        const int at = i - kBoundsPad, in = at < 0 ? 0 : (at < count ? at : count - 1);
        const int first = parts[in * (t.P + 1) + k];
        s_mine[i] = make_int2(first, at == in ? parts[in * (t.P + 1) + k + 1] : first);
    }
    for (int i = threadIdx.x; i <= count; i += blockDim.x) {
        // An imported slot lands on the ring entry of the slot kRing before it, which this
        // workgroup's rows read as long as it is less than kRingSafe behind them: a slot may come
        // in once it is at most kTeamAhead past the first of the workgroup's rows of the level
        // (solving A^T the slots descend: at most kTeamAhead below the last of them).
        const int l = l0 + (i < count ? i : count - 1) * step - lmin;
        const int first = parts[l * (t.P + 1) + k], end = parts[l * (t.P + 1) + k + 1];
        const int lim = step > 0 ? first + kTeamAhead : -(end - 1) + kTeamAhead;
        const int need = t.tab[k * (count + 1) + (i + 1 < count ? i + 1 : count)];
        const int before = t.tab[(t.P + k) * (count + 1) + i];
        s_sv[i] = make_int2(lim, need | (before << kTeamNeedBits));
    }
    {
        const int32_t *lists = t.tab + 2 * t.P * (count + 1);
        const int32_t *exp_ds = lists + t.n_imp + t.exp_off[k], *exp_cell = lists + 2 * t.n_imp + t.exp_off[k];
        const int n_exp = t.exp_off[k + 1] - t.exp_off[k];
        for (int i = threadIdx.x; i < n_exp; i += blockDim.x) s_exl[i] = make_int2(exp_ds[i], exp_cell[i]);
    }
    if (threadIdx.x == 0) ring[kRing] = 0.;
    __syncthreads();
    const char *ring_bytes = reinterpret_cast<const char *>(ring);
    if (threadIdx.x < kTeamChunk) {
        // the rows: the single-workgroup kernel's level loop on this workgroup's part of a level
        const uint32_t lane8 = threadIdx.x * 8u;
        // (lanes past the end of the part load the operands of the slots that follow it: readable,
        // whatever the part's length)
        auto part = [&](int it) {
            const int2 m = s_mine[l0 + it * step - lmin + kBoundsPad];
            return Bounds{__builtin_amdgcn_readfirstlane(m.x), __builtin_amdgcn_readfirstlane(m.y)};
        };
        EllVals<PRE> qv[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) qv[d] = load_ell<PRE>(a, part(d));
        Bounds ahead = part(DEPTH);
        // (LEAN: as in sptrsv_ell_kernel)
        auto one_level = [&](auto lean, int it, EllVals<PRE> &stage) {
            constexpr bool LEAN = decltype(lean)::value;
            const EllVals<PRE> cur = stage;
            stage = load_ell<PRE>(a, ahead);
            double xj[PRE];
            uint32_t any = 0;
#pragma unroll
            for (int e = 0; e < PRE; ++e) {
                xj[e] = *reinterpret_cast<const double *>(ring_bytes + ell_ring_bytes(cur.ds[e / 2], e));
                any |= cur.ds[e / 2];
            }
            ahead = part(it + DEPTH + 1);
            double acc = 0.;
#pragma unroll
            for (int e = 0; e < PRE; ++e) acc += cur.v[e] * xj[e];   // absent: 0.0 * 0.0
            const bool live = (int)threadIdx.x < cur.qe - cur.qb;
            if (!LEAN && (any & kEllFarPair) && live) {
                // a row solved by an earlier launch: that value from global memory, the sum in
                // the same order.  (Only that value: what this launch computes is taken from
                // the ring as ever -- in global memory a value of another workgroup of this
                // launch is not ordered before this read.)
                const int q = cur.qb + (int)threadIdx.x;
                const int32_t dlo = a.dptr[q], n = a.dptr[q + 1] - dlo;
                int32_t sl[PRE];
                double xg[PRE];
#pragma unroll
                for (int e = 0; e < PRE; ++e) sl[e] = a.dslot[dlo + (e < n ? e : 0)];
#pragma unroll
                for (int e = 0; e < PRE; ++e) xg[e] = a.xs[sl[e]];
                acc = 0.;
#pragma unroll
                for (int e = 0; e < PRE; ++e) {
                    const bool far = (cur.ds[e / 2] >> ((e & 1) * 16)) & 1u;
                    acc += e < n ? cur.v[e] * (far ? xg[e] : xj[e]) : 0.;
                }
            }
            double xi = cur.bv - acc;
            if (LEAN || !a.unit) xi /= cur.dv;
            if (live) {
                const uint32_t at = (uint32_t)cur.qb * 8u + lane8;
                *reinterpret_cast<double *>(const_cast<char *>(ring_bytes) + (at & (kRing * 8 - 1))) = xi;
                *reinterpret_cast<double *>(reinterpret_cast<char *>(a.xs) + (int64_t)cur.qb * 8 + lane8) = xi;
            }
            __syncthreads();
        };
        const int tested = a.unit || far_levels >= count ? count : (far_levels + DEPTH - 1) / DEPTH * DEPTH;
        int it0 = 0;
        for (; it0 < tested; it0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                if (it0 + d >= count) break;   // uniform over the workgroup
                one_level(std::false_type{}, it0 + d, qv[d]);
            }
        }
        for (; it0 < count; it0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                if (it0 + d >= count) break;
                one_level(std::true_type{}, it0 + d, qv[d]);
            }
        }
        return;
    }

    // the two service wavefronts: one hands out, one takes in (as one wavefront they had as many
    // instructions to issue per level as a row's wavefront, and the barrier waited for them)
    const int lane = threadIdx.x & 63;
    if (threadIdx.x < kTeamChunk + 64) {
        // the values of the level before, now in the ring, that other workgroups wait for; what
        // a level needs from the tables in LDS is read one level early (a level's chain of
        // dependent LDS round trips is what the whole workgroup waits for at the barrier)
        int e0 = 0;
        int svy = s_sv[0].y;
        int2 xl = s_exl[lane];
        for (int it = 0; it < count; ++it) {
            const int e1 = __builtin_amdgcn_readfirstlane(svy >> kTeamNeedBits);
            const int2 mine = xl;
            svy = s_sv[it + 1].y;
            xl = s_exl[(e1 + lane) & (kTeamExports - 1)];
            auto hand_out = [&](int2 x) {
                const double v = ring[x.x & (kRing - 1)];
                const unsigned long long tag = (unsigned long long)(uint32_t)(x.x + 1) << 32;
                unsigned long long *cell = t.cells + 2 * (int64_t)x.y;
                __hip_atomic_store(cell, tag | (uint32_t)__double2loint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(cell + 1, tag | (uint32_t)__double2hiint(v), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            };
            if (e1 > e0) {
                if (e0 + lane < e1) hand_out(mine);
                for (int e = e0 + 64 + lane; e < e1; e += 64) hand_out(s_exl[e]);
            }
            e0 = e1;
            __syncthreads();
        }
        return;
    }
    const int n_imp = t.imp_off[k + 1] - t.imp_off[k];
    // this lane's cell of a poll that starts at import 0 (a poll reads 64 cells whatever the
    // list's length: the mailbox ends with kTeamCellPadding cells that nobody writes)
    const unsigned long long *cells_lane = t.cells + 2 * ((int64_t)t.imp_off[k] + lane);
    const unsigned long long *quiet_lane = t.cells + 2 * ((int64_t)t.quiet + lane);
    int c = 0;   // imports [0, c) are in the ring
    // A poll reads the two words of 64 cells, from import `cs` on.  Nothing else the loop below
    // needs comes from device memory: the hardware hands loads back in the order they were
    // issued, so one fresh load that a level waits for would wait for every poll in flight.
    auto issue = [&](int cs) {
        TeamPoll p;
        p.cs = cs;
        // (with nothing left to import, the cells that nobody writes: polling cells that another
        // workgroup is waiting on slows the polls down, and with them this workgroup)
        const unsigned long long *at = cs < n_imp ? cells_lane + 2 * (int64_t)cs : quiet_lane;
        p.w0 = __hip_atomic_load(at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        p.w1 = __hip_atomic_load(at + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return p;
    };
    // What a poll found goes into the ring.  A cell's words carry the slot + 1 next to the halves
    // of the value, 0 while empty.  (A slot too far ahead of this workgroup's own level would land
    // on a ring entry that its rows still read: it is taken by a later poll.  An import below `c`
    // is in the ring already: a poll made many levels ago must not write it again, its ring
    // entry may belong to a newer slot by now.)
    auto take = [&](const TeamPoll &p, int lim) {
        const uint32_t tag = (uint32_t)(p.w0 >> 32);
        const int32_t ds = (int32_t)tag - 1;
        const int j = p.cs + lane;
        const bool have = j < n_imp && tag != 0u && (uint32_t)(p.w1 >> 32) == tag;
        const bool ok = have && j >= c && (step > 0 ? ds : -ds) <= lim;
        if (ok) ring[ds & (kRing - 1)] = __hiloint2double((int)(uint32_t)p.w1, (int)(uint32_t)p.w0);
        const unsigned long long m = __ballot(ok || j < c);
        const int lead = m == ~0ull ? 64 : __builtin_ctzll(~m);
        c = c > p.cs + lead ? c : p.cs + lead;
    };
    const int32_t limit32 = poll_limit > 0x7fffffff ? 0x7fffffff : (poll_limit < 1 ? 1 : (int32_t)poll_limit);
    if (poll_limit < 0) {   // give up at once (tests)
        c = 0x3fffffff;
        if (lane == 0) status[0] = 1;
    }
    TeamPoll st[kTeamStages];
#pragma unroll
    for (int d = 0; d < kTeamStages; ++d) st[d] = issue(c);
    // one level: what poll `p` found comes in, and the poll is made again (the level's entry of
    // the table in LDS is read one level early)
    int2 cur = s_sv[0];
    auto serve = [&](int it, TeamPoll &p) {
        const int need = __builtin_amdgcn_readfirstlane(cur.y & ((1 << kTeamNeedBits) - 1));
        const int lim = __builtin_amdgcn_readfirstlane(cur.x);
        cur = s_sv[it + 1];
        take(p, lim);
        // everything the next level reads must be in the ring before this level's barrier
        if (__builtin_expect(c < need, 0)) {
            int32_t polls = 0;
            while (c < need) {
                take(issue(c), lim);
                if (c >= need) break;
                if (++polls >= limit32) {
                    c = 0x3fffffff;   // never waits again; the solve hands out NaN
                    if (lane == 0) status[0] = 1;
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
            // (leaves this branch with no load in flight, so that the straight path's wait
            // counts are those of the polls alone)
            __builtin_amdgcn_s_waitcnt(0x0f70);   // vmcnt(0)
        }
        p = issue(c);
        __syncthreads();
    };
    // Whole rounds of kTeamStages levels, then the rest without a way back to the loop's head: on
    // a path from the middle of a round to the head the polls would have been issued in another
    // order, and the compiler, which must count for every path, would wait for all of them at
    // every level.
    int it = 0;
    for (; it + kTeamStages <= count; it += kTeamStages) {
#pragma unroll
        for (int d = 0; d < kTeamStages; ++d) serve(it + d, st[d]);
    }
#pragma unroll
    for (int d = 0; d < kTeamStages; ++d) {
        if (it + d >= count) return;
        serve(it + d, st[d]);
    }
}

// One wide level: slots [q0, q1), one lane per row.
__global__ __launch_bounds__(kBlock) void sptrsv_level_kernel(SolveArgs a, int q0, int q1) {
    const int q = q0 + (int)(blockIdx.x * blockDim.x + threadIdx.x);
    if (q >= q1) return;
    const int32_t dlo = a.dptr[q], dhi = a.dptr[q + 1];
    double acc = 0.;
    for (int32_t at = dlo; at < dhi; ++at) acc += a.w.coef[at] * a.w.xs[a.dslot[at]];
    double xi = a.w.rhs[q] - acc;
    if (!a.unit) xi /= a.w.dg[q];
    a.w.xs[q] = xi;
}

// One level with many entries: slots [q0, q1), G lanes per row.  Lane s of a group takes
// dependencies s, s + G, ... of its row, so coefficients, slots and solved values are each one
// request for the whole row instead of a chain of requests in one lane.  The products are
// added in storage order, like the serial loop (cpp/sparse_csr_cpu.cpp:706-720): the running
// sum is handed from lane to lane (lane k is right after G - 1 shifts), chunk after chunk.
template <int G>
__global__ __launch_bounds__(kBlock) void sptrsv_level_group_kernel(SolveArgs a, int q0, int q1) {
    static_assert(G == 4 || G == 8 || G == 16, "a group lies inside one 16-lane DPP row");
    const int sub = (int)threadIdx.x & (G - 1);
    const int q = q0 + (int)((blockIdx.x * blockDim.x + threadIdx.x) / G);
    const bool live = q < q1;
    const int qs = live ? q : q0;
    const int32_t dlo = a.dptr[qs];
    const int32_t n = live ? a.dptr[qs + 1] - dlo : 0;
    double carry = 0.;
    for (int32_t e0 = 0; __any(e0 < n); e0 += G) {
        const bool have = e0 + sub < n;
        const int32_t at = have ? dlo + e0 + sub : 0;   // 0: a readable position (this kernel runs where rows have entries)
        const double c = a.w.coef[at];
        const double xv = a.w.xs[a.dslot[at]];
        const double term = have ? c * xv : 0.;
        double r = 0.;
#pragma unroll
        for (int step = 0; step < G; ++step) {
            const double prev = nm::dpp_move<0x111>(r);   // row_shr 1
            r = (sub == 0 ? carry : prev) + term;
        }
        carry = __shfl(r, ((int)threadIdx.x & 63) | (G - 1), 64);   // the group's last lane
    }
    if (live && sub == 0) {
        double xi = a.w.rhs[q] - carry;
        if (!a.unit) xi /= a.w.dg[q];
        a.w.xs[q] = xi;
    }
}

// ---- chains: runs of levels of one row each -----------------------------------
//
// A banded factor, a bidiagonal or a tridiagonal triangle is one long chain: every level has
// one row, and that row waits for the row of the level before it.  The workgroup kernels
// above pay a barrier, an LDS round trip and a division of ~30 dependent instructions per
// level for it.  Here ONE wavefront walks the chain and hands the newest solution from step
// to step in a scalar register pair:
//   * lane l owns the rows at chain positions t = l (mod 64); 64 rows are in flight, and at
//     step k every lane adds (its coefficient on row k-1) x (solution k-1) to the sum of the row
//     it owns -- the solutions arrive in the order in which the serial loop visits them
//     (cpp/sparse_csr_cpu.cpp:672-718 walks a row from its farthest dependency to its nearest),
//     so each row's sum is formed in exactly that order;
//   * what a row needs from outside its launch (rows solved by earlier launches) comes first in
//     that order and is summed ahead of time, for all rows at once, by chain_prepare_kernel;
//   * the division is three operations with a reciprocal that chain_prepare_kernel formed with
//     a true division: q0 = n y, r = n - d q0 (exact), q = q0 + r y.  After every 64 steps each
//     lane checks its own row's quotient against a true division, bit for bit; a block that
//     fails (a zero, infinite or NaN operand, a range the shortcut does not cover) is solved
//     again, and the rest of the launch with it, by the plain loop with true divisions.
// The 64 steps of a block are unrolled; a block's coefficient rows are registers that are
// refilled in place, right after use, with the rows of the block after it.
constexpr int kChainMin = 64;                       // levels; shorter runs stay with the workgroup kernels
constexpr int32_t kChainBad = 1, kChainWide = 2;    // verdict bits of chain_check_kernel
// doubles a chain launch of m rows takes in the coefficient area: wide chains one row of 64 per
// position (+ one row before the first, + 64 rows that the last block requests ahead), and a
// word of presence bits per position; narrow chains one coefficient per position
inline int64_t chain_doubles(int64_t m, int kind) {
    const int64_t m64 = (m + 63) / 64 * 64;
    return kind == 64 ? (m64 + 64) * 64 + m64 + 64 : m64 + 64;
}

struct ChainArgs {
    const int32_t *dptr, *dslot;   // this direction's packed dependencies, in accumulation order
    const double *coef, *dg, *rhs; // level-major values of this call (gather_values_kernel)
    double *xs;                    // running solution by slot
    double *sum0, *recip;          // by slot: sum over the dependencies outside the launch; 1 / diagonal
    double *band;                  // wide chains: [position + 1][64] coefficients on the row before that
                                   // position, lane = owner; narrow chains: [position] the one coefficient
    unsigned long long *has;       // wide chains: [position + 1] which lanes have a coefficient there
    int32_t q0, q1, m, step;       // slots [q0, q1), m = q1 - q0 rows, walked upwards (+1) or downwards (-1)
    int unit;
};

__device__ __forceinline__ int32_t chain_slot(const ChainArgs &c, int32_t t) {
    return c.step > 0 ? c.q0 + t : c.q1 - 1 - t;
}
__device__ __forceinline__ int32_t chain_pos(const ChainArgs &c, int32_t q) {
    return c.step > 0 ? q - c.q0 : c.q1 - 1 - q;
}

// Plan time: may the chain kernels take this run of one-row levels in this direction?  In a
// row's accumulation order the dependencies outside the launch must all come before those
// inside it, the ones inside must be at most 64 positions back and in ascending position.
__global__ void chain_check_kernel(int32_t nlevels, int dirn, const int32_t *__restrict__ level_ptr,
                                   const int32_t *__restrict__ cand_of_level, const int32_t *__restrict__ cq,
                                   const int32_t *__restrict__ dptr, const int32_t *__restrict__ dslot,
                                   int32_t *__restrict__ verdict) {
    const int32_t stride = (int32_t)(gridDim.x * blockDim.x);
    for (int32_t l = (int32_t)(blockIdx.x * blockDim.x + threadIdx.x); l < nlevels; l += stride) {
        const int32_t ci = cand_of_level[l];
        if (ci < 0) continue;
        const int32_t q = level_ptr[l], q0 = cq[2 * ci], q1 = cq[2 * ci + 1];
        const int32_t t = dirn == 0 ? q - q0 : q1 - 1 - q;
        int32_t bits = 0, inside = 0, last = -1;
        for (int32_t at = dptr[q]; at < dptr[q + 1]; ++at) {
            const int32_t ds = dslot[at];
            if (ds >= q0 && ds < q1) {
                const int32_t k = dirn == 0 ? ds - q0 : q1 - 1 - ds;
                if (t - k < 1 || t - k > 64 || k <= last) bits |= kChainBad;
                if (t - k != 1) bits |= kChainWide;
                last = k;
                ++inside;
            } else if (inside > 0) {
                bits |= kChainBad;
            }
        }
        if (inside > 1) bits |= kChainWide;
        if (t > 0 && inside == 0) bits |= kChainBad;
        if (bits) atomicOr(verdict + 2 * ci + dirn, bits);
    }
}

// Per call and launch, one lane per row of the chain: the part of the row's sum that does not
// wait for the chain, the reciprocal of its diagonal, and its coefficients on the chain in
// the layout the chain kernel streams (the wide layout is cleared before this runs).
template <bool BAND>
__global__ void chain_prepare_kernel(ChainArgs c) {
    const int32_t t = (int32_t)(blockIdx.x * blockDim.x + threadIdx.x);
    if (t >= c.m) return;
    const int32_t q = chain_slot(c, t);
    double acc = 0., only = 0.;
    for (int32_t at = c.dptr[q]; at < c.dptr[q + 1]; ++at) {
        const int32_t ds = c.dslot[at];
        const double v = c.coef[at];
        if (ds < c.q0 || ds >= c.q1) {
            acc += v * c.xs[ds];
        } else if (BAND) {
            const int32_t k = chain_pos(c, ds);
            c.band[(size_t)(k + 1) * 64 + (t & 63)] = v;
            atomicOr(c.has + k + 1, 1ull << (t & 63));
        } else {
            only = v;
        }
    }
    c.sum0[q] = acc;
    c.recip[q] = c.unit ? 1. : 1. / c.dg[q];
    if (!BAND) c.band[t] = only;
}

__device__ __forceinline__ double lane_value(double v, int lane) {   // `lane` is uniform
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
    const int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
    return __hiloint2double(hi, lo);
}

__device__ __forceinline__ bool same_bits(double a, double b) {
    return __double_as_longlong(a) == __double_as_longlong(b);
}

template <bool BAND, bool UNIT>
__global__ __launch_bounds__(64) void sptrsv_chain_kernel(ChainArgs c) {
    const int lane = (int)threadIdx.x;
    const int32_t m = c.m;
    const double *__restrict__ band = c.band;
    // what the lanes computed at the 64 steps of a block: the quotient, and for wide chains with a
    // division the numerator beside it
    constexpr bool kPair = BAND && !UNIT;
    __shared__ double s_keep[(kPair ? 2 : 1) * 64 * 64];
    double X = 0.;            // the newest solution (uniform)
    double row[BAND ? 64 : 1];
    double acc = 0.;          // wide chains: the sum of the row this lane owns
    int32_t k0 = 0;
    // operands of the block's rows (lane l: position k0 + l), requested one block ahead
    auto at_slot = [&](int32_t t) { return chain_slot(c, t < m ? t : m - 1); };
    double bv = c.rhs[at_slot(lane)], dv = c.dg[at_slot(lane)], yv = c.recip[at_slot(lane)];
    double s0 = c.sum0[at_slot(lane)], cv = 0.;
    if (BAND) {
#pragma unroll
        for (int s = 0; s < 64; ++s) row[s] = band[(size_t)s * 64 + lane];
        acc = s0;
    } else {
        cv = band[lane];
    }
    bool fast = true;
    for (; k0 < m; k0 += 64) {
        const int32_t t = k0 + lane;
        const int32_t qn = at_slot(t + 64);
        const double bvN = c.rhs[qn], dvN = c.dg[qn], yvN = c.recip[qn], s0N = c.sum0[qn];
        const double cvN = BAND ? 0. : band[t + 64];   // padded: 64 entries behind the last row
        const double Xin = X, acc_in = acc;
        // "is this step's row mine" is compared afresh at every step: 64 masks kept from block to
        // block would not fit the scalar registers
        int32_t t_mark = t;
        asm volatile("" : "+v"(t_mark));
        const double *__restrict__ ahead = band + (size_t)(k0 + 64) * 64;   // padded: 64 rows behind the last
#pragma unroll
        for (int s = 0; s < 64; ++s) {
            if (BAND) {
                acc = acc + row[s] * X;
                row[s] = ahead[s * 64 + lane];
            } else {
                acc = s0 + cv * X;
            }
            const double n = bv - acc;
            double q = n;
            if (!UNIT) {
                const double q0 = n * yv;
                const double r = __builtin_fma(-dv, q0, n);
                q = __builtin_fma(r, yv, q0);
            }
            // every lane files what it computed; only lane s's entry of step s means anything
            if (kPair) reinterpret_cast<double2 *>(s_keep)[s * 64 + lane] = make_double2(n, q);
            else s_keep[s * 64 + lane] = q;
            if (BAND) acc = (t_mark == k0 + s) ? s0N : acc;
            X = lane_value(q, s);
        }
        double n_keep = 0., q_keep;
        if (kPair) {
            const double2 nq = reinterpret_cast<const double2 *>(s_keep)[lane * 64 + lane];
            n_keep = nq.x;
            q_keep = nq.y;
        } else {
            q_keep = s_keep[lane * 64 + lane];
        }
        // every lane checks the row it finished in this block
        bool ok = true;
        if (t < m) {
            if (BAND) {
                // a skipped coefficient was multiplied as 0.0: exact only for finite solutions
                ok = (UNIT || same_bits(n_keep / dv, q_keep)) && __builtin_isfinite(q_keep);
            } else {
                double before = __shfl_up(q_keep, 1);
                if (lane == 0) before = Xin;
                const double n = bv - (s0 + cv * before);
                ok = same_bits(UNIT ? n : n / dv, q_keep);
            }
        }
        if (!__all(ok) || !__builtin_isfinite(Xin)) {
            X = Xin;
            acc = acc_in;
            fast = false;
            break;
        }
        if (t < m) c.xs[chain_slot(c, t)] = q_keep;
        bv = bvN; dv = dvN; yv = yvN; s0 = s0N; cv = cvN;
    }
    if (fast) return;
    // the plain loop: true divisions, coefficients that are absent are skipped
    for (; k0 < m; k0 += 64) {
        const int32_t t = k0 + lane;
        const int32_t qs = at_slot(t), qn = at_slot(t + 64);
        bv = c.rhs[qs]; dv = c.dg[qs]; s0 = c.sum0[qs];
        const double s0N = c.sum0[qn];
        if (!BAND) cv = band[t];
        double q_keep = 0.;
        for (int s = 0; s < 64; ++s) {
            if (BAND) {
                const double v = band[(size_t)(k0 + s) * 64 + lane];
                if ((c.has[k0 + s] >> lane) & 1ull) acc = acc + v * X;
            } else {
                acc = s0 + cv * X;   // position 0 has no coefficient (0.0) and meets X = 0.0
            }
            const double n = bv - acc;
            const double q = UNIT ? n : n / dv;
            if (lane == s) {
                q_keep = q;
                if (BAND) acc = s0N;
            }
            X = lane_value(q, s);
        }
        if (t < m) c.xs[chain_slot(c, t)] = q_keep;
    }
}

// x[order[q]] = xs[q], rounded once to the value type (cpp/sparse_csr_cpu.cpp:722).
// `status` (may be null): nonzero when a kernel of this solve gave up waiting; x is then NaN throughout.
// ---- which rows of a level a workgroup of a team takes ---------------------------------------
//
// By ROW NUMBER where that works: the rows of a launch are cut into P ranges of row numbers and
// workgroup k takes, of every level, the rows of range k (inside a level rows ascend, so that is
// a stretch of the level's slots).  A lower triangle's row depends on rows with smaller numbers
// only, a value therefore never crosses from a higher range to a lower one (solving A^T: never
// from a lower to a higher): consumers run behind their producers for good, whatever the
// stencil.  It works when no range holds more than kTeamChunk rows of one level -- triangles of
// grid stencils, whose levels run across the grid.  Otherwise by POSITION: workgroup k takes
// the slots [kTeamChunk k, kTeamChunk (k + 1)) of a level, and build_team checks whether the
// crossings that come of it can be pipelined.
constexpr int kPartStride = kTeamMax + 1;   // starts of the parts of one level, then the level's end

// Smallest and largest row number of every candidate launch (span[2 li], span[2 li + 1]; the
// host presets them): rows ascend inside a level, so a level's first and last slot are enough.
__global__ void team_span_kernel(int32_t nlevels, const int32_t *__restrict__ order,
                                 const int32_t *__restrict__ level_ptr, const int32_t *__restrict__ level_launch,
                                 const int32_t *__restrict__ cand_l0, int32_t *__restrict__ span) {
    const int32_t l = blockIdx.x * blockDim.x + threadIdx.x;
    if (l >= nlevels || level_ptr[l + 1] <= level_ptr[l]) return;
    const int32_t li = level_launch[l];
    if (li < 0 || cand_l0[li] < 0) return;
    atomicMin(span + 2 * li, order[level_ptr[l]]);
    atomicMax(span + 2 * li + 1, order[level_ptr[l + 1] - 1]);
}

// part[l][k] = first slot of workgroup k's part of level l, for k = 0 .. P (P: the level's end);
// most[li] = the longest part of launch li.  parts[li] > 0: P ranges of row numbers that start at
// split[li][k]; parts[li] < 0: -P parts by position.
__global__ void team_parts_kernel(int32_t nlevels, const int32_t *__restrict__ order,
                                  const int32_t *__restrict__ level_ptr, const int32_t *__restrict__ level_launch,
                                  const int32_t *__restrict__ cand_l0, const int32_t *__restrict__ parts,
                                  const int32_t *__restrict__ split, int32_t *__restrict__ part,
                                  int32_t *__restrict__ most) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (int64_t)nlevels * kPartStride) return;
    const int32_t l = (int32_t)(idx / kPartStride), k = (int32_t)(idx % kPartStride);
    const int32_t li = level_launch[l];
    if (li < 0 || cand_l0[li] < 0) return;
    const int32_t P = parts[li] < 0 ? -parts[li] : parts[li];
    if (k > P) return;
    const int32_t q0 = level_ptr[l], q1 = level_ptr[l + 1];
    auto start_of = [&](int32_t kk) {
        if (kk <= 0) return q0;
        if (kk >= P) return q1;
        if (parts[li] < 0) return q0 + kk * kTeamChunk < q1 ? q0 + kk * kTeamChunk : q1;
        const int32_t from = split[li * kPartStride + kk];
        int32_t lo = q0, hi = q1;   // first slot of the level whose row number is >= from
        while (lo < hi) {
            const int32_t mid = (lo + hi) >> 1;
            if (order[mid] < from) lo = mid + 1; else hi = mid;
        }
        return lo;
    };
    const int32_t mine = start_of(k);
    part[idx] = mine;
    if (k < P) atomicMax(most + li, start_of(k + 1) - mine);
}

// The workgroup that takes slot q of level l.
__device__ __forceinline__ int32_t part_of(const int32_t *__restrict__ part, int32_t l, int32_t P, int32_t q) {
    int32_t k = 0;
    while (k + 1 < P && part[(int64_t)l * kPartStride + k + 1] <= q) ++k;
    return k;
}

// The dependencies of one solve direction that cross between the parts of the levels of a
// launch that a team may share: (launch, consumer's workgroup, producer's workgroup, the
// dependency's slot, consumer's level, dependency's level) per crossing, appended in no particular
// order; `bad[launch]` is raised when a row of the launch depends on a row of the same launch
// too many slots back for the ring.  `cand_l0[launch]` is the launch's first level, -1 when it
// is no candidate in this direction.
constexpr int kCrossInts = 6;
__global__ void team_cross_kernel(int64_t rows, const int32_t *__restrict__ dptr, const int32_t *__restrict__ dslot,
                                  const int32_t *__restrict__ level_ptr, int32_t nlevels,
                                  const int32_t *__restrict__ level_launch, const int32_t *__restrict__ cand_l0,
                                  const int32_t *__restrict__ cand_l1, const int32_t *__restrict__ parts,
                                  const int32_t *__restrict__ part, int32_t *__restrict__ out, int32_t capacity,
                                  int32_t *__restrict__ count, int32_t *__restrict__ bad) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < rows; q += stride) {
        const int32_t l = level_of_slot(level_ptr, nlevels, (int32_t)q);
        const int32_t li = level_launch[l];
        if (li < 0) continue;
        const int32_t l0 = cand_l0[li], l1 = cand_l1[li];
        if (l0 < 0) continue;
        const int32_t P = parts[li] < 0 ? -parts[li] : parts[li];
        const int32_t k = part_of(part, l, P, (int32_t)q);
        for (int32_t e = dptr[q]; e < dptr[q + 1]; ++e) {
            const int32_t ds = dslot[e];
            const int32_t ld = level_of_slot(level_ptr, nlevels, ds);
            if (ld < l0 || ld >= l1) continue;   // an earlier launch: ordered by the stream
            if ((ds > (int32_t)q ? ds - (int32_t)q : (int32_t)q - ds) >= kRingSafe) {
                bad[li] = 1;
                continue;
            }
            const int32_t kd = part_of(part, ld, P, ds);
            if (kd == k) continue;
            const int32_t at = atomicAdd(count, 1);
            if (at < capacity) {
                int32_t *r = out + (int64_t)at * kCrossInts;
                r[0] = li; r[1] = k; r[2] = kd; r[3] = ds; r[4] = l; r[5] = ld;
            }
        }
    }
}

// Exchange tables of a launch that P workgroups share, for one solve direction (d = 0: with A),
// from the dependencies that cross between the workgroups' parts of its levels (`part`: where
// the parts of every level start)
// (`cross`, collected on the device by team_cross_kernel, which also rules out a launch in which
// a row reads, through global memory, a row of the same launch -- too many slots back for the
// ring: between workgroups nothing orders that read after the write).  Appends to `tab` what
// TeamArgs::tab describes and fills `T`; returns false (and leaves both alone) when the launch is
// better left to one workgroup:
//   * at some level the waits "a needs what b computes at the level before" form a cycle: those
//     workgroups would have to exchange values inside every such level;
//   * the direction in which values cross between two workgroups changes more than once in 32
//     levels: every change costs a hand-over's latency;
//   * more values cross than a service wavefront polls in passing (16 per workgroup and level
//     on average), or than the mailbox, the tables or a workgroup's LDS list of exports hold.
struct Cross { int32_t k, ds, it, kd, itd; };   // workgroup k needs slot ds at its level `it`; kd computes it at `itd`
bool build_team(const nm_sptrsv_plan::Launch &L, int d, int32_t P, const int32_t *part, std::vector<Cross> &cross,
                int64_t cells_left, int64_t ints_left, std::vector<int32_t> &tab, nm_sptrsv_plan::Launch::Team &T) {
    const int32_t count = L.l1 - L.l0;
    if (P < 2 || P > kTeamMax || count < 16) return false;
    // A value is taken in at the latest during the level before the one that reads it, and it may
    // only be taken in once it lies no further than kTeamAhead ahead of the workgroup's own rows
    // (sptrsv_team_kernel: its ring entry is in use until then).  One that never would, would be
    // waited for until the solve gives up.
    for (const Cross &x : cross) {
        const int32_t before = d == 0 ? L.l0 + x.it - 1 : L.l1 - x.it;   // the level of the workgroup's x.it - 1
        const int32_t first = part[(int64_t)before * kPartStride + x.k], end = part[(int64_t)before * kPartStride + x.k + 1];
        if (d == 0 ? x.ds > first + kTeamAhead : x.ds < end - 1 - kTeamAhead) return false;
    }
    // one import per (workgroup, slot): the first level that needs it
    std::sort(cross.begin(), cross.end(), [](const Cross &x, const Cross &y) {
        return x.k != y.k ? x.k < y.k : (x.ds != y.ds ? x.ds < y.ds : x.it < y.it);
    });
    cross.erase(std::unique(cross.begin(), cross.end(),
                            [](const Cross &x, const Cross &y) { return x.k == y.k && x.ds == y.ds; }),
                cross.end());
    const int64_t n = (int64_t)cross.size();
    const int64_t ints = (int64_t)2 * P * (count + 1) + 3 * n + (int64_t)count * (P + 1);
    if (n > cells_left || ints > ints_left || n > (int64_t)16 * count * P || n >= (int64_t(1) << kTeamNeedBits))
        return false;
    // waits on the level just before, per level: a cycle among them cannot be pipelined away
    {
        std::vector<uint16_t> adj((size_t)count * kTeamMax, 0);   // [level][consumer]: its producers
        std::vector<uint8_t> any_edge((size_t)count, 0);
        for (const Cross &x : cross)
            if (x.itd == x.it - 1) {
                adj[(size_t)x.it * kTeamMax + x.k] |= (uint16_t)(1u << x.kd);
                any_edge[x.it] = 1;
            }
        static_assert(kTeamMax <= 16, "a workgroup's producers fit sixteen bits");
        for (int32_t j = 0; j < count; ++j) {
            if (!any_edge[j]) continue;
            uint16_t r[kTeamMax];
            for (int u = 0; u < kTeamMax; ++u) r[u] = adj[(size_t)j * kTeamMax + u];
            for (int m = 0; m < kTeamMax; ++m)
                for (int u = 0; u < kTeamMax; ++u)
                    if ((r[u] >> m) & 1) r[u] |= r[m];
            for (int u = 0; u < kTeamMax; ++u)
                if ((r[u] >> u) & 1) return false;
        }
    }
    // A consumer runs a few levels behind its producer, and the hand-over's latency is paid once.
    // Where the direction between two workgroups changes, it is paid again (the workgroup that
    // was ahead must now wait for the one that was behind): a triangle whose dependencies cross
    // the cut now this way, now that (the nine-point stencil's alternate from level to level) is
    // faster on one workgroup.  One change per 32 levels is what a shared level's gain pays for.
    {
        std::vector<Cross> byit(cross);
        std::stable_sort(byit.begin(), byit.end(), [](const Cross &x, const Cross &y) { return x.it < y.it; });
        int8_t last[kTeamMax][kTeamMax] = {};
        int64_t changes = 0;
        for (const Cross &x : byit) {
            const int lo = x.k < x.kd ? x.k : x.kd, hi = x.k < x.kd ? x.kd : x.k;
            const int8_t dirn = x.k < x.kd ? 1 : 2;
            if (last[lo][hi] != 0 && last[lo][hi] != dirn) ++changes;
            last[lo][hi] = dirn;
        }
        if (changes * 32 > count) return false;
    }
    {   // a workgroup's list of exports lives in LDS
        int64_t out[kTeamMax] = {};
        for (const Cross &x : cross)
            if (++out[x.kd] > kTeamExports) return false;
    }
    // imports by (workgroup, first level that reads them); an import's place in that order is its cell
    std::stable_sort(cross.begin(), cross.end(),
                     [](const Cross &x, const Cross &y) { return x.k != y.k ? x.k < y.k : x.it < y.it; });
    T.P = P;
    T.at = (int32_t)tab.size();
    T.n_imp = (int32_t)n;
    tab.resize(tab.size() + (size_t)ints, 0);
    int32_t *need = tab.data() + T.at, *before = need + (size_t)P * (count + 1);
    int32_t *imp_ds = before + (size_t)P * (count + 1), *exp_ds = imp_ds + n, *exp_cell = exp_ds + n;
    for (int k = 0; k <= kTeamMax; ++k) T.imp_off[k] = T.exp_off[k] = 0;
    for (const Cross &x : cross) {
        ++T.imp_off[x.k + 1];
        ++T.exp_off[x.kd + 1];
    }
    for (int k = 0; k < kTeamMax; ++k) {
        T.imp_off[k + 1] += T.imp_off[k];
        T.exp_off[k + 1] += T.exp_off[k];
    }
    // need[k][j]: imports of workgroup k that levels up to its j-th read
    for (int64_t i = 0; i < n; ++i) {
        imp_ds[i] = cross[i].ds;
        ++need[(size_t)cross[i].k * (count + 1) + cross[i].it];
    }
    for (int k = 0; k < P; ++k)
        for (int32_t j = 1; j <= count; ++j) need[(size_t)k * (count + 1) + j] += need[(size_t)k * (count + 1) + j - 1];
    // exports by (workgroup, level that computes them); before[k][j]: those of levels before its j-th
    std::vector<int64_t> by((size_t)n);
    for (int64_t i = 0; i < n; ++i) by[i] = i;
    std::stable_sort(by.begin(), by.end(), [&](int64_t x, int64_t y) {
        return cross[x].kd != cross[y].kd ? cross[x].kd < cross[y].kd : cross[x].itd < cross[y].itd;
    });
    for (int64_t i = 0; i < n; ++i) {
        const Cross &x = cross[by[i]];
        exp_ds[i] = x.ds;
        exp_cell[i] = (int32_t)by[i];
        if (x.itd + 1 <= count) ++before[(size_t)x.kd * (count + 1) + x.itd + 1];
    }
    for (int k = 0; k < P; ++k)
        for (int32_t j = 1; j <= count; ++j)
            before[(size_t)k * (count + 1) + j] += before[(size_t)k * (count + 1) + j - 1];
    // the parts of the launch's levels
    int32_t *parts_out = exp_cell + n;
    for (int32_t l = 0; l < count; ++l)
        for (int k = 0; k <= P; ++k) parts_out[(size_t)l * (P + 1) + k] = part[(int64_t)(L.l0 + l) * kPartStride + k];
    return true;
}

template <typename T>
__global__ void unslot_kernel(int64_t n, const int32_t *__restrict__ order, const double *__restrict__ xs,
                              T *__restrict__ x, const int32_t *__restrict__ status) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const bool failed = status != nullptr && status[0] != 0;
    const double nan = __longlong_as_double(0x7ff8000000000000ll);
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < n; q += stride)
        x[order[q]] = (T)(failed ? nan : xs[q]);
}

template <typename T>
int solve_typed(const nm_sptrsv_plan *p, int transposed, const void *data, int unit, const void *b, void *x,
                void *work, hipStream_t s) {
    const Packed &P = p->dir[transposed ? 1 : 0];
    SolveArgs a;
    solve_work_layout(p->rows, p->nnz, work, &a.w);
    a.level_ptr = p->level_ptr;
    a.dptr = P.dptr;
    a.dslot = P.dslot;
    a.unit = unit;
    bool any_wide = false;
    const bool teams = g_team_enabled.load();
    for (const auto &L : p->launches)
        any_wide = any_wide || L.wide ||
                   (L.run && !(teams && p->ell_pre[transposed ? 1 : 0] > 0 && L.team[transposed ? 1 : 0].P > 1));
    if (any_wide || p->ell_pre[transposed ? 1 : 0] == 0) {   // the range-based arrays have readers
        int64_t m = p->nnz > p->rows ? p->nnz : p->rows;
        int64_t grid = nm::ceil_div(m, kBlock);
        if (grid > 65536) grid = 65536;
        // with nnz == 0 nothing reads `data`: any valid pointer will do
        const T *dat = p->nnz > 0 ? (const T *)data : (const T *)b;
        hipLaunchKernelGGL(gather_values_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, p->rows, p->nnz, dat,
                           (const T *)b, p->order, P.dptr, P.dsrc, P.diag, a.w.coef, a.w.dg, a.w.rhs);
        NM_LAUNCH_CHECK("gather_values_kernel");
    }
    const int dirn = transposed ? 1 : 0;
    const int pre = p->ell_pre[dirn];
    EllArgs ea{p->level_ptr, P.dptr, P.dslot, P.lvl_sig, reinterpret_cast<const uint16_t *>(P.ell_ds), a.w.ell_coef,
               a.w.rb, a.w.xs, unit};
    if (pre > 0) {
        int64_t grid = nm::ceil_div(p->rows * pre, kBlock);
        if (grid > 65536) grid = 65536;
        const T *dat = p->nnz > 0 ? (const T *)data : (const T *)b;
        hipLaunchKernelGGL(gather_ell_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, p->rows, pre, dat,
                           (const T *)b, p->order, P.dptr, P.dsrc, P.diag, a.w.ell_coef, a.w.rb, a.w.status,
                           a.w.cells, (int64_t)2 * p->team_cells[dirn]);
        NM_LAUNCH_CHECK("gather_ell_kernel");
    }
    const int n = (int)p->launches.size();
    for (int li = 0; li < n; ++li) {
        const auto &L = p->launches[transposed ? n - 1 - li : li];
        if (L.chain[dirn] != 0) {
            // one wavefront walks the run of one-row levels; `ell_coef` and `rb` are free for it
            // (a direction that has chains does not use the fixed-width layout)
            ChainArgs c;
            c.dptr = P.dptr;
            c.dslot = P.dslot;
            c.coef = a.w.coef;
            c.dg = a.w.dg;
            c.rhs = a.w.rhs;
            c.xs = a.w.xs;
            c.sum0 = a.w.rb;
            c.recip = a.w.rb + (p->rows + kEllPad);
            c.band = a.w.ell_coef + L.chain_at[dirn];
            c.q0 = L.q0;
            c.q1 = L.q1;
            c.m = L.q1 - L.q0;
            c.step = transposed ? -1 : 1;
            c.unit = unit;
            const int64_t m64 = (int64_t)nm::ceil_div((int64_t)c.m, 64) * 64;
            const bool wide_chain = L.chain[dirn] == 64;
            c.has = reinterpret_cast<unsigned long long *>(c.band + (m64 + 64) * 64);
            const unsigned pgrid = (unsigned)nm::ceil_div((int64_t)c.m, kBlock);
            if (wide_chain) {
                if (int rc = nm::fill_async(c.band, chain_doubles(c.m, 64), 0., s)) return rc;
                hipLaunchKernelGGL(chain_prepare_kernel<true>, dim3(pgrid), dim3(kBlock), 0, s, c);
                if (unit) hipLaunchKernelGGL((sptrsv_chain_kernel<true, true>), dim3(1), dim3(64), 0, s, c);
                else hipLaunchKernelGGL((sptrsv_chain_kernel<true, false>), dim3(1), dim3(64), 0, s, c);
            } else {
                if (int rc = nm::fill_async(c.band + c.m, m64 + 64 - c.m, 0., s)) return rc;
                hipLaunchKernelGGL(chain_prepare_kernel<false>, dim3(pgrid), dim3(kBlock), 0, s, c);
                if (unit) hipLaunchKernelGGL((sptrsv_chain_kernel<false, true>), dim3(1), dim3(64), 0, s, c);
                else hipLaunchKernelGGL((sptrsv_chain_kernel<false, false>), dim3(1), dim3(64), 0, s, c);
            }
            NM_LAUNCH_CHECK("sptrsv_chain_kernel");
        } else if (L.wide || (L.run && !(teams && pre > 0 && L.team[dirn].P > 1))) {
            // a grid launch per level (a run without a team: its levels one after the other)
            const int G = L.group[dirn] > 0 ? L.group[dirn] : 1;
            const int nl = L.l1 - L.l0;
            for (int j = 0; j < nl; ++j) {
                const int l = transposed ? L.l1 - 1 - j : L.l0 + j;
                const int q0 = L.wide ? L.q0 : p->lp_host[l], q1 = L.wide ? L.q1 : p->lp_host[l + 1];
                const unsigned grid = (unsigned)nm::ceil_div((int64_t)(q1 - q0) * G, kBlock);
                if (G == 16)
                    hipLaunchKernelGGL(sptrsv_level_group_kernel<16>, dim3(grid), dim3(kBlock), 0, s, a, q0, q1);
                else if (G == 8)
                    hipLaunchKernelGGL(sptrsv_level_group_kernel<8>, dim3(grid), dim3(kBlock), 0, s, a, q0, q1);
                else if (G == 4)
                    hipLaunchKernelGGL(sptrsv_level_group_kernel<4>, dim3(grid), dim3(kBlock), 0, s, a, q0, q1);
                else
                    hipLaunchKernelGGL(sptrsv_level_kernel, dim3(grid), dim3(kBlock), 0, s, a, q0, q1);
                NM_LAUNCH_CHECK("sptrsv_level_kernel");
            }
        } else {
            const int count = L.l1 - L.l0;
            const int l0 = transposed ? L.l1 - 1 : L.l0, step = transposed ? -1 : 1;
            // dependencies per row fetched ahead through registers: the smallest pipeline that
            // holds this direction's longest row (longer rows take the slow path)
            const int maxdep = p->max_deps[transposed ? 1 : 0];
            // wavefronts signal each other where no row looks further than kSigReach wavefronts away
            // (and there is more than one wavefront); else they meet at a barrier after every level
            const bool sig = pre > 0 && L.block > 64 && p->reach[dirn] <= kSigReach && g_sig_enabled.load();
            const int64_t limit = g_sig_poll_limit.load();
            static const int tune_sleep = [] { const char *e = std::getenv("NUMML_AMD_SIG_SLEEP"); return e ? atoi(e) : 1; }();
            static const int tune_skew = [] {
                const char *e = std::getenv("NUMML_AMD_SIG_SKEW");
                const int v = e ? atoi(e) : kSkew;
                return v < 0 ? 0 : (v > kSkew ? kSkew : v);
            }();
            const auto &TM = L.team[dirn];
            if (pre > 0 && TM.P > 1 && teams) {
                // several workgroups share every level
                TeamArgs ta;
                ta.tab = P.team + TM.at;
                ta.cells = a.w.cells + 2 * (int64_t)TM.cell0;
                ta.P = TM.P;
                ta.n_imp = TM.n_imp;
                ta.quiet = (int32_t)(team_cells_capacity(p->rows) - TM.cell0);
                for (int k = 0; k <= kTeamMax; ++k) {
                    ta.imp_off[k] = TM.imp_off[k];
                    ta.exp_off[k] = TM.exp_off[k];
                }
                const dim3 tg((unsigned)TM.P), tb(kTeamChunk + 128);
                if (pre == 2)
                    hipLaunchKernelGGL((sptrsv_team_kernel<2, 4>), tg, tb, 0, s, ea, ta, l0, count, step, limit, a.w.status,
                                       L.far_levels[dirn]);
                else if (pre == 4)
                    hipLaunchKernelGGL((sptrsv_team_kernel<4, 3>), tg, tb, 0, s, ea, ta, l0, count, step, limit, a.w.status,
                                       L.far_levels[dirn]);
                else
                    hipLaunchKernelGGL((sptrsv_team_kernel<8, 2>), tg, tb, 0, s, ea, ta, l0, count, step, limit, a.w.status,
                                       L.far_levels[dirn]);
                NM_LAUNCH_CHECK("sptrsv_team_kernel");
                continue;
            }
            if (pre == 2 && sig)
                hipLaunchKernelGGL((sptrsv_ell_kernel<2, 4, true>), dim3(1), dim3(L.block), 0, s, ea, l0, count, step,
                                   limit, a.w.status, tune_sleep, tune_skew);
            else if (pre == 4 && sig)
                hipLaunchKernelGGL((sptrsv_ell_kernel<4, 3, true>), dim3(1), dim3(L.block), 0, s, ea, l0, count, step,
                                   limit, a.w.status, tune_sleep, tune_skew);
            else if (pre == 8 && sig)
                hipLaunchKernelGGL((sptrsv_ell_kernel<8, 2, true>), dim3(1), dim3(L.block), 0, s, ea, l0, count, step,
                                   limit, a.w.status, tune_sleep, tune_skew);
            else if (pre == 2)
                hipLaunchKernelGGL((sptrsv_ell_kernel<2, 4>), dim3(1), dim3(L.block), 0, s, ea, l0, count, step,
                                   (int64_t)0, (int32_t *)nullptr, 1, kSkew, L.far_levels[dirn]);
            else if (pre == 4)
                hipLaunchKernelGGL((sptrsv_ell_kernel<4, 3>), dim3(1), dim3(L.block), 0, s, ea, l0, count, step,
                                   (int64_t)0, (int32_t *)nullptr, 1, kSkew, L.far_levels[dirn]);
            else if (pre == 8)
                hipLaunchKernelGGL((sptrsv_ell_kernel<8, 2>), dim3(1), dim3(L.block), 0, s, ea, l0, count, step,
                                   (int64_t)0, (int32_t *)nullptr, 1, kSkew, L.far_levels[dirn]);
            else if (L.group[dirn] > 0) {
                // several lanes per row: as many groups as the widest level has rows, within one workgroup
                const int G = L.group[dirn];
                int groups = 1;
                while (groups < L.width && groups * G < kNarrow) groups *= 2;
                const int lanes = groups * G < 64 ? 64 : groups * G;
                if (G == 64)
                    hipLaunchKernelGGL((sptrsv_group_kernel<64, 2>), dim3(1), dim3(lanes), 0, s, a, l0, count, step, L.q0, L.q1);
                else
                    hipLaunchKernelGGL((sptrsv_group_kernel<16, 2>), dim3(1), dim3(lanes), 0, s, a, l0, count, step, L.q0, L.q1);
            } else if (maxdep <= 2)
                hipLaunchKernelGGL((sptrsv_ring_kernel<2, 4>), dim3(1), dim3(L.block), 0, s, a, l0, count, step, L.q0, L.q1);
            else if (maxdep <= 4)
                hipLaunchKernelGGL((sptrsv_ring_kernel<4, 3>), dim3(1), dim3(L.block), 0, s, a, l0, count, step, L.q0, L.q1);
            else if (maxdep <= 8)
                hipLaunchKernelGGL((sptrsv_ring_kernel<8, 2>), dim3(1), dim3(L.block), 0, s, a, l0, count, step, L.q0, L.q1);
            else
                // up to 16 dependencies through the register pipeline; longer rows take the slow path
                if (L.block <= 512)
                    hipLaunchKernelGGL((sptrsv_ring_kernel<16, 1, 512>), dim3(1), dim3(L.block), 0, s, a, l0, count, step, L.q0, L.q1);
                else
                    hipLaunchKernelGGL((sptrsv_ring_kernel<16, 1>), dim3(1), dim3(L.block), 0, s, a, l0, count, step, L.q0, L.q1);
            NM_LAUNCH_CHECK("sptrsv_ring_kernel");
        }
    }
    int64_t grid = nm::ceil_div(p->rows, kBlock);
    if (grid > 65536) grid = 65536;
    hipLaunchKernelGGL(unslot_kernel<T>, dim3((unsigned)grid), dim3(kBlock), 0, s, p->rows, p->order, a.w.xs,
                       (T *)x, pre > 0 ? a.w.status : (const int32_t *)nullptr);
    NM_LAUNCH_CHECK("unslot_kernel");
    return NM_OK;
}

}  // namespace

extern "C" int nm_sptrsv_plan_bytes(int64_t rows, int64_t nnz, size_t *plan_bytes, size_t *work_bytes) {
    NM_REQUIRE(rows >= 0 && nnz >= 0 && plan_bytes && work_bytes, "bad arguments");
    if (rows >= (int64_t(1) << 31) - 2 || nnz >= (int64_t(1) << 31) - 2)
        return nm::fail(NM_ERR_UNSUPPORTED, "sptrsv plans index rows and entries with 32 bits");
    *plan_bytes = plan_layout(rows, nnz, nullptr, nullptr);
    *work_bytes = work_layout(rows, nnz, nullptr, nullptr);
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
    Layout L;
    plan_layout(rows, nnz, plan_mem, &L);
    p->order = L.order;
    p->level_ptr = L.level_ptr;
    p->slot_of = L.slot_of;
    p->dir[0] = L.dir[0];
    p->dir[1] = L.dir[1];

    auto bail = [&](int rc) { delete p; return rc; };
    if (rows == 0) { *plan_out = p; return NM_OK; }
    Scratch W;
    work_layout(rows, nnz, work, &W);

    if (int rc = nm::tplan_build(rows, rows, nnz, indices, indptr, L.t, W.twork, W.twork_bytes, W.rowid, s))
        return bail(rc);
    if (int rc = nm::fill_async(W.deg, rows + 1, (int32_t)0, s)) return bail(rc);
    int64_t egrid = nm::ceil_div(nnz > 0 ? nnz : 1, kBlock), rgrid = nm::ceil_div(rows, kBlock);
    if (egrid > 65536) egrid = 65536;
    if (rgrid > 65536) rgrid = 65536;
    if (nnz > 0) {
        hipLaunchKernelGGL(indegree_kernel, dim3((unsigned)egrid), dim3(kBlock), 0, s, nnz, indices, W.rowid,
                           p->lower, W.deg);
        if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "indegree_kernel launch failed"));
    }
    if (int rc = nm::fill_async(L.meta, 16, (int32_t)0, s)) return bail(rc);
    hipLaunchKernelGGL(kahn_kernel, dim3(1), dim3(kNarrow), 0, s, (int32_t)rows, p->lower, L.t.t_indptr, L.t.t_row,
                       W.deg, p->order, p->level_ptr, L.meta);
    if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "kahn_kernel launch failed"));
    // The sweep appends the rows of a level in the order its atomics were served.  Rows ascending
    // inside every level make the schedule the same on every run and keep a row's dependencies
    // in the wavefronts next to its own, which is what lets wavefronts signal their neighbours
    // instead of meeting at a barrier (W.count64 is not in use yet and holds 2 * rows int32).
    if (int rc = nm::segments_sort_i32(L.meta, rows, rows, p->level_ptr, p->order,
                                       reinterpret_cast<int32_t *>(W.count64), s))
        return bail(rc);
    hipLaunchKernelGGL(slot_of_kernel, dim3((unsigned)rgrid), dim3(kBlock), 0, s, rows, p->order, p->slot_of);

    // level-major packed triangles for both directions: count, scan, fill
    for (int d = 0; d < 2; ++d) {
        const int eff_lower = d == 0 ? p->lower : !p->lower;
        const Packed &P = p->dir[d];
        for (int fill = 0; fill < 2; ++fill) {
            if (d == 0)
                hipLaunchKernelGGL(pack_kernel<0>, dim3((unsigned)rgrid), dim3(kBlock), 0, s, rows, eff_lower, fill,
                                   p->order, p->slot_of, indices, indptr, L.t.t_indptr, L.t.t_row, L.t.t_perm,
                                   W.count64, P.dptr, P.dslot, P.dsrc, P.diag, L.meta + 2 + d);
            else
                hipLaunchKernelGGL(pack_kernel<1>, dim3((unsigned)rgrid), dim3(kBlock), 0, s, rows, eff_lower, fill,
                                   p->order, p->slot_of, indices, indptr, L.t.t_indptr, L.t.t_row, L.t.t_perm,
                                   W.count64, P.dptr, P.dslot, P.dsrc, P.diag, L.meta + 2 + d);
            if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "pack_kernel launch failed"));
            if (fill == 0) {
                if (int rc = nm::fill_async(W.count64 + rows, 1, (int64_t)0, s)) return bail(rc);
                if (int rc = nm::scan_exclusive_i64(W.count64, rows + 1, W.scan, s)) return bail(rc);
                hipLaunchKernelGGL(narrow_kernel, dim3((unsigned)rgrid), dim3(kBlock), 0, s, rows + 1, W.count64,
                                   P.dptr);
            }
        }
    }

    int32_t meta_h[4] = {0, 0, 0, 0};
    if (hipMemcpyAsync(meta_h, L.meta, sizeof(meta_h), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return bail(nm::fail(NM_ERR_HIP, "reading the level count back failed: %s",
                             hipGetErrorString(hipGetLastError())));
    if (meta_h[1] != (int32_t)rows)
        return bail(nm::fail(NM_ERR_INVALID, "level analysis placed %d of %lld rows", meta_h[1], (long long)rows));
    p->nlevels = meta_h[0];
    p->max_deps[0] = meta_h[2];
    p->max_deps[1] = meta_h[3];
    std::vector<int32_t> lp((size_t)p->nlevels + 1);
    if (hipMemcpyAsync(lp.data(), p->level_ptr, lp.size() * 4, hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)
        return bail(nm::fail(NM_ERR_HIP, "reading the level sizes back failed"));

    // Consecutive narrow levels share one single-workgroup launch (at most kMaxLevels
    // each).  The workgroup runs on one CU, where every wavefront -- also one without a
    // row in the current level -- costs issue slots on the level's critical path
    // (measured: 0.36 us per level with one wavefront, 0.78 us with sixteen), so a run
    // is cut into segments by level width and each segment is launched with the
    // smallest power-of-two workgroup (64 .. kNarrow lanes) that holds its widest level.
    auto lanes_for = [&](int32_t l) {
        const int32_t w = lp[l + 1] - lp[l];
        int32_t b = 64;
        while (b < w) b *= 2;
        return b;
    };
    constexpr int32_t kMinSegment = 32;   // levels; shorter segments are not worth a launch
    auto push_plain = [&](int32_t a0, int32_t a1) {
        int32_t s0 = a0, block = lanes_for(a0);
        auto flush = [&](int32_t end) {
            // (a launch that a team may share hands out, per workgroup, about a value per level:
            // kTeamLevels of them keep the list of those within what the team kernel holds)
            const int32_t most = block > kTeamChunk ? kTeamLevels : kMaxLevels;
            for (int32_t c0 = s0; c0 < end; c0 += most) {
                const int32_t c1 = c0 + most < end ? c0 + most : end;
                p->launches.push_back({c0, c1, lp[c0], lp[c1], false, block});
            }
        };
        for (int32_t l = a0 + 1; l < a1; ++l) {
            const int32_t b = lanes_for(l);
            if (b > block) {
                // wider than the segment allows: widen a young segment, else start a new one
                if (l - s0 < kMinSegment) { block = b; continue; }
                flush(l);
                s0 = l;
                block = b;
            } else if (b < block && l - s0 >= kMinSegment) {
                // narrower: worth a new segment only if it stays narrower for a while
                int32_t widest = b;
                const int32_t look = l + kMinSegment < a1 ? l + kMinSegment : a1;
                for (int32_t m = l; m < look; ++m) widest = widest > lanes_for(m) ? widest : lanes_for(m);
                if (widest < block && look - l >= kMinSegment) {
                    flush(l);
                    s0 = l;
                    block = widest;
                }
            }
        }
        flush(a1);
    };
    // Runs of at least kChainMin one-row levels inside a narrow run become launches of their own
    // (candidates for the single-wavefront chain kernels; a direction that cannot use those runs
    // them like any other narrow launch).
    auto push_narrow = [&](int32_t a0, int32_t a1) {
        int32_t plain0 = a0;
        for (int32_t l = a0; l < a1;) {
            if (lp[l + 1] - lp[l] != 1) { ++l; continue; }
            int32_t e = l;
            while (e < a1 && lp[e + 1] - lp[e] == 1) ++e;
            if (e - l >= kChainMin) {
                if (l > plain0) push_plain(plain0, l);
                // at most kMaxLevels levels each (a direction that cannot use the chain kernels runs
                // them like any other narrow launch), in pieces of equal length
                const int32_t pieces = (e - l + kMaxLevels - 1) / kMaxLevels;
                const int32_t each = (e - l + pieces - 1) / pieces;
                for (int32_t c0 = l; c0 < e; c0 += each) {
                    const int32_t c1 = c0 + each < e ? c0 + each : e;
                    p->launches.push_back({c0, c1, lp[c0], lp[c1], false, 64});
                    p->launches.back().chain_candidate = true;
                }
                plain0 = e;
            }
            l = e;
        }
        if (a1 > plain0) push_plain(plain0, a1);
    };
    // dependency ranges of both directions: a level is also given a launch of its own when it
    // has enough entries to be worth the chip (one CU takes ~10 us over a level of a few
    // thousand entries, a grid launch 3-4 us)
    std::vector<int32_t> dptr_h[2];
    for (int d = 0; d < 2; ++d) {
        dptr_h[d].resize((size_t)rows + 1);
        if (hipMemcpyAsync(dptr_h[d].data(), p->dir[d].dptr, dptr_h[d].size() * 4, hipMemcpyDeviceToHost, s) !=
                hipSuccess ||
            hipStreamSynchronize(s) != hipSuccess)
            return bail(nm::fail(NM_ERR_HIP, "reading the dependency counts back failed"));
    }
    auto level_entries = [&](int d, int32_t l) { return dptr_h[d][lp[l + 1]] - dptr_h[d][lp[l]]; };
    auto is_wide = [&](int32_t l) {
        const int32_t width = lp[l + 1] - lp[l];
        const int32_t entries = level_entries(0, l) > level_entries(1, l) ? level_entries(0, l) : level_entries(1, l);
        return width > kNarrow || (width >= kWideRows && entries >= kWideEntries);
    };
    // levels wider than one workgroup takes but not than a team of them: a stretch of at least
    // kRunMin becomes one launch that a team may share (build_team decides per direction)
    constexpr int32_t kRunMin = 16;
    auto team_width = [&](int32_t l) {
        const int32_t width = lp[l + 1] - lp[l];
        return width > kNarrow && width <= kTeamMax * kTeamChunk;
    };
    int32_t run0 = -1;
    for (int32_t l = 0; l < p->nlevels; ++l) {
        if (!is_wide(l)) {
            if (run0 < 0) run0 = l;
            continue;
        }
        if (run0 >= 0) { push_narrow(run0, l); run0 = -1; }
        int32_t e = l;
        while (e < p->nlevels && team_width(e)) ++e;
        if (e - l >= kRunMin) {
            const int32_t pieces = (e - l + kTeamLevels - 1) / kTeamLevels;
            const int32_t each = (e - l + pieces - 1) / pieces;
            for (int32_t c0 = l; c0 < e; c0 += each) {
                const int32_t c1 = c0 + each < e ? c0 + each : e;
                p->launches.push_back({c0, c1, lp[c0], lp[c1], false, kBlock});
                p->launches.back().run = true;
            }
            l = e - 1;
            continue;
        }
        p->launches.push_back({l, l + 1, lp[l], lp[l + 1], true, kBlock});
    }
    if (run0 >= 0) push_narrow(run0, p->nlevels);
    p->lp_host = lp;
    // Rows long enough to be shared by several lanes: decided per launch and direction from the
    // mean number of dependencies of its rows, where no fixed-width layout serves the direction.
    for (auto &L : p->launches) {
        L.width = 0;
        for (int32_t l = L.l0; l < L.l1; ++l) L.width = L.width > lp[l + 1] - lp[l] ? L.width : lp[l + 1] - lp[l];
    }
    for (int d = 0; d < 2; ++d) {
        for (auto &L : p->launches) {
            if (L.q1 <= L.q0) continue;
            const double mean = double(dptr_h[d][L.q1] - dptr_h[d][L.q0]) / double(L.q1 - L.q0);
            if (L.wide || L.run) {
                // a level of its own: lanes per row by its mean row length
                L.group[d] = mean >= 10. ? 16 : (mean >= 5. ? 8 : (mean >= 2.5 ? 4 : 0));
                continue;
            }
            if (p->max_deps[d] <= 8) continue;
            if (mean >= 40. && L.width <= 16) L.group[d] = 64;
            else if (mean >= 12. && L.width <= 256) L.group[d] = 16;
        }
    }
    // fixed-width copies of the packed triangles, with the ring-reach mark per dependency
    std::vector<int32_t> level_launch((size_t)p->nlevels + 1, -1);
    for (size_t li = 0; li < p->launches.size(); ++li)
        for (int32_t l = p->launches[li].l0; l < p->launches[li].l1; ++l)
            level_launch[l] = p->launches[li].wide ? -1 - (int32_t)li : (int32_t)li;
    if (hipMemcpyAsync(L.level_launch, level_launch.data(), level_launch.size() * 4, hipMemcpyHostToDevice, s) !=
        hipSuccess)
        return bail(nm::fail(NM_ERR_HIP, "uploading the launch table failed"));
    // Which runs of one-row levels the chain kernels take, per direction (W.count64 and W.deg
    // are free by now: candidate of every level, the candidates' slot ranges, the verdicts).
    bool chains[2] = {false, false};
    {
        std::vector<int32_t> cand((size_t)p->nlevels + 1, -1), cq;
        std::vector<size_t> cand_launch;
        for (size_t li = 0; li < p->launches.size(); ++li) {
            const auto &C = p->launches[li];
            if (!C.chain_candidate) continue;
            for (int32_t l = C.l0; l < C.l1; ++l) cand[l] = (int32_t)cand_launch.size();
            cq.push_back(C.q0);
            cq.push_back(C.q1);
            cand_launch.push_back(li);
        }
        if (!cand_launch.empty()) {
            int32_t *d_cand = reinterpret_cast<int32_t *>(W.count64), *d_cq = d_cand + (rows + 1);
            std::vector<int32_t> verdict(cq.size(), 0);
            if (hipMemcpyAsync(d_cand, cand.data(), cand.size() * 4, hipMemcpyHostToDevice, s) != hipSuccess ||
                hipMemcpyAsync(d_cq, cq.data(), cq.size() * 4, hipMemcpyHostToDevice, s) != hipSuccess)
                return bail(nm::fail(NM_ERR_HIP, "uploading the chain candidates failed"));
            if (int rc = nm::fill_async(W.deg, (int64_t)cq.size(), (int32_t)0, s)) return bail(rc);
            int64_t lgrid = nm::ceil_div((int64_t)p->nlevels, kBlock);
            if (lgrid > 65536) lgrid = 65536;
            for (int d = 0; d < 2; ++d) {
                hipLaunchKernelGGL(chain_check_kernel, dim3((unsigned)lgrid), dim3(kBlock), 0, s, p->nlevels, d,
                                   p->level_ptr, d_cand, d_cq, p->dir[d].dptr, p->dir[d].dslot, W.deg);
                if (hipGetLastError() != hipSuccess)
                    return bail(nm::fail(NM_ERR_HIP, "chain_check_kernel launch failed"));
            }
            if (hipMemcpyAsync(verdict.data(), W.deg, verdict.size() * 4, hipMemcpyDeviceToHost, s) != hipSuccess ||
                hipStreamSynchronize(s) != hipSuccess)
                return bail(nm::fail(NM_ERR_HIP, "reading the chain verdicts back failed"));
            for (int d = 0; d < 2; ++d) {
                // the coefficient area is shared with the fixed-width layout: a direction takes its
                // chains when they hold at least half of its levels, or when it has no such layout
                const int32_t md = p->max_deps[d];
                const bool ell_possible = md <= 8 && rows < (1 << 30);
                int64_t at = 0, levels = 0;
                std::vector<std::pair<size_t, int>> taken;
                for (size_t ci = 0; ci < cand_launch.size(); ++ci) {
                    const int32_t v = verdict[2 * ci + d];
                    if (v & kChainBad) continue;
                    const auto &C = p->launches[cand_launch[ci]];
                    const int kind = (v & kChainWide) ? 64 : 1;
                    const int64_t need = chain_doubles(C.q1 - C.q0, kind);
                    if (at + need > coef_capacity(rows, nnz)) continue;
                    taken.push_back({cand_launch[ci], kind});
                    at += need;
                    levels += C.l1 - C.l0;
                }
                if (taken.empty() || (ell_possible && 2 * levels < p->nlevels)) continue;
                chains[d] = true;
                at = 0;
                for (const auto &tk : taken) {
                    auto &C = p->launches[tk.first];
                    C.chain[d] = tk.second;
                    C.chain_at[d] = at;
                    at += chain_doubles(C.q1 - C.q0, tk.second);
                }
            }
        }
    }
    for (int d = 0; d < 2; ++d) {
        const int32_t md = p->max_deps[d];
        const int pre = chains[d] ? 0 : (md <= 2 ? 2 : (md <= 4 ? 4 : (md <= 8 ? 8 : 0)));
        if (pre > 0 && rows < (1 << 30) && (rows + kEllPad) * pre <= ell_capacity(rows, nnz)) {
            p->ell_pre[d] = pre;
            int64_t grid = nm::ceil_div(rows * pre, kBlock);
            if (grid > 65536) grid = 65536;
            if (int rc = nm::fill_async(p->dir[d].lvl_sig, (int64_t)p->nlevels + 1, (int32_t)0, s)) return bail(rc);
            hipLaunchKernelGGL(ell_pack_kernel, dim3((unsigned)grid), dim3(kBlock), 0, s, rows, pre, p->dir[d].dptr,
                               p->dir[d].dslot, p->level_ptr, p->nlevels, L.level_launch,
                               reinterpret_cast<uint16_t *>(p->dir[d].ell_ds),
                               L.meta + 4 + d, p->dir[d].lvl_sig);
            if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "ell_pack_kernel launch failed"));
        }
    }
    // per launch and direction: the first levels, up to the last one with a row that reads outside the ring
    for (int d = 0; d < 2; ++d) {
        if (p->ell_pre[d] == 0) continue;
        std::vector<int32_t> sig((size_t)p->nlevels);
        if (hipMemcpyAsync(sig.data(), p->dir[d].lvl_sig, sig.size() * 4, hipMemcpyDeviceToHost, s) != hipSuccess ||
            hipStreamSynchronize(s) != hipSuccess)
            return bail(nm::fail(NM_ERR_HIP, "reading the levels' marks back failed"));
        for (auto &C : p->launches) {
            int32_t last = 0;   // levels of the launch, in the direction's order, that must be tested
            for (int32_t l = C.l0; l < C.l1; ++l)
                if (sig[l] & kSigFar) {
                    const int32_t it = d == 0 ? l - C.l0 : (C.l1 - 1) - l;
                    last = last > it + 1 ? last : it + 1;
                }
            C.far_levels[d] = last;
        }
    }
    // Launches wider than one workgroup's share of a level, in directions with the fixed-width
    // layout: the tables of what passes between their workgroups, where that can be pipelined.
    std::vector<int32_t> team_tab[2];
    {
        bool any = false;
        // (NUMML_AMD_SPTRSV_TEAMS=0: no tables at all; nm_sptrsv_configure only decides whether a
        // solve uses them)
        static const bool build_tables = [] {
            const char *e = std::getenv("NUMML_AMD_SPTRSV_TEAMS");
            return !(e && e[0] == '0');
        }();
        if (build_tables)
            for (const auto &C : p->launches) any = any || (!C.wide && C.width > kTeamChunk);
        const int32_t nl = (int32_t)p->launches.size();
        // Device scratch that is free by now.  W.count64 (ints): first and last level of the
        // candidates, their number of parts, span of row numbers, longest part, where the ranges of
        // row numbers start.  W.deg: [crossings][ruled out, per launch].  W.rowid: where the parts of
        // every level start, then the crossings.
        constexpr int kPerLaunch = 2 + 1 + 2 + 1 + kPartStride;
        const int64_t part_ints = (int64_t)p->nlevels * kPartStride;
        any = any && nnz > 0 && nl <= rows && (int64_t)nl * kPerLaunch <= 2 * (rows + 1) &&
              part_ints + 1024 * kCrossInts <= nnz + 1 && (p->ell_pre[0] > 0 || p->ell_pre[1] > 0);
        int32_t *d_l0 = reinterpret_cast<int32_t *>(W.count64), *d_l1 = d_l0 + nl, *d_parts = d_l1 + nl;
        int32_t *d_span = d_parts + nl, *d_most = d_span + 2 * nl, *d_split = d_most + nl;
        int32_t *d_count = W.deg, *d_bad = W.deg + 1;
        int32_t *d_part = W.rowid, *d_recs = W.rowid + part_ints;
        int64_t cap64 = (nnz + 1 - part_ints) / kCrossInts;
        if (cap64 > 4 * team_cells_capacity(rows) + 1024) cap64 = 4 * team_cells_capacity(rows) + 1024;
        const int32_t capacity = any ? (int32_t)cap64 : 0;
        std::vector<int32_t> cand_l0((size_t)nl, -1), cand_l1((size_t)nl, 0), parts((size_t)nl, 0), recs,
            head((size_t)nl + 1), span((size_t)2 * nl), most((size_t)nl), split((size_t)nl * kPartStride, 0), part_h;
        auto up = [&](int32_t *dst, const std::vector<int32_t> &src) {
            return src.empty() || hipMemcpyAsync(dst, src.data(), src.size() * 4, hipMemcpyHostToDevice, s) == hipSuccess;
        };
        auto down = [&](std::vector<int32_t> &dst, const int32_t *src) {
            return dst.empty() || (hipMemcpyAsync(dst.data(), src, dst.size() * 4, hipMemcpyDeviceToHost, s) == hipSuccess &&
                                   hipStreamSynchronize(s) == hipSuccess);
        };
        const unsigned lgrid = (unsigned)nm::ceil_div((int64_t)p->nlevels, kBlock);
        const unsigned pgrid = (unsigned)nm::ceil_div(part_ints > 0 ? part_ints : 1, (int64_t)kBlock);
        if (any) {
            // the parts of every level of every launch that is a candidate in either direction
            for (int32_t li = 0; li < nl; ++li) {
                const auto &C = p->launches[li];
                const bool cand = !C.wide && C.width > kTeamChunk && C.width <= kTeamMax * kTeamChunk &&
                                  ((p->ell_pre[0] > 0 && C.chain[0] == 0) || (p->ell_pre[1] > 0 && C.chain[1] == 0));
                cand_l0[li] = cand ? C.l0 : -1;
                cand_l1[li] = C.l1;
                parts[li] = cand ? (C.width + kTeamChunk - 1) / kTeamChunk : 0;
                span[2 * li] = 0x7fffffff;
                span[2 * li + 1] = -1;
            }
            if (!up(d_l0, cand_l0) || !up(d_l1, cand_l1) || !up(d_span, span))
                return bail(nm::fail(NM_ERR_HIP, "uploading the candidate launches failed"));
            hipLaunchKernelGGL(team_span_kernel, dim3(lgrid), dim3(kBlock), 0, s, p->nlevels, p->order, p->level_ptr,
                               L.level_launch, d_l0, d_span);
            if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "team_span_kernel launch failed"));
            if (!down(span, d_span)) return bail(nm::fail(NM_ERR_HIP, "reading the launches' row numbers back failed"));
            // by row number, with as few workgroups as keep every part within kTeamChunk rows; by
            // position where not even kTeamMax ranges do
            for (bool again = true; again;) {
                for (int32_t li = 0; li < nl; ++li) {
                    if (parts[li] <= 0) continue;
                    const int64_t lo = span[2 * li], n = (int64_t)span[2 * li + 1] - lo + 1;
                    for (int k = 0; k <= parts[li]; ++k) split[(size_t)li * kPartStride + k] = (int32_t)(lo + n * k / parts[li]);
                }
                if (!up(d_parts, parts) || !up(d_split, split))
                    return bail(nm::fail(NM_ERR_HIP, "uploading the ranges of row numbers failed"));
                if (int rc = nm::fill_async(d_most, (int64_t)nl, (int32_t)0, s)) return bail(rc);
                hipLaunchKernelGGL(team_parts_kernel, dim3(pgrid), dim3(kBlock), 0, s, p->nlevels, p->order, p->level_ptr,
                                   L.level_launch, d_l0, d_parts, d_split, d_part, d_most);
                if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "team_parts_kernel launch failed"));
                if (!down(most, d_most)) return bail(nm::fail(NM_ERR_HIP, "reading the longest parts back failed"));
                again = false;
                for (int32_t li = 0; li < nl; ++li) {
                    if (parts[li] <= 0 || most[li] <= kTeamChunk) continue;
                    const int32_t by_position = (p->launches[li].width + kTeamChunk - 1) / kTeamChunk;
                    parts[li] = parts[li] < kTeamMax ? parts[li] + 1 : -by_position;
                    again = true;
                }
            }
            part_h.resize((size_t)part_ints);
            if (!down(part_h, d_part)) return bail(nm::fail(NM_ERR_HIP, "reading the parts back failed"));
        }
        for (int d = 0; d < 2 && any; ++d) {
            if (p->ell_pre[d] == 0) continue;
            bool some = false;
            std::vector<int32_t> mine(cand_l0);   // the candidates of this direction
            for (int32_t li = 0; li < nl; ++li) {
                if (p->launches[li].chain[d] != 0) mine[li] = -1;
                some = some || mine[li] >= 0;
            }
            if (!some) continue;
            if (int rc = nm::fill_async(W.deg, (int64_t)nl + 1, (int32_t)0, s)) return bail(rc);
            if (!up(d_l0, mine)) return bail(nm::fail(NM_ERR_HIP, "uploading the candidate launches failed"));
            hipLaunchKernelGGL(team_cross_kernel, dim3((unsigned)rgrid), dim3(kBlock), 0, s, rows, p->dir[d].dptr,
                               p->dir[d].dslot, p->level_ptr, p->nlevels, L.level_launch, d_l0, d_l1, d_parts, d_part,
                               d_recs, capacity, d_count, d_bad);
            if (hipGetLastError() != hipSuccess) return bail(nm::fail(NM_ERR_HIP, "team_cross_kernel launch failed"));
            head.assign((size_t)nl + 1, 0);   // [0]: crossings found, [1 + li]: launch li ruled out
            if (!down(head, W.deg)) return bail(nm::fail(NM_ERR_HIP, "reading the crossings' count back failed"));
            if (head[0] > capacity) continue;   // far more cross than any team exchanges
            recs.resize((size_t)head[0] * kCrossInts);
            if (!down(recs, d_recs)) return bail(nm::fail(NM_ERR_HIP, "reading the crossings back failed"));
            std::vector<std::vector<Cross>> per((size_t)nl);
            for (size_t r = 0; r + kCrossInts <= recs.size(); r += kCrossInts) {
                const int32_t li = recs[r];
                const auto &C = p->launches[li];
                auto iter_of = [&](int32_t l) { return d == 0 ? l - C.l0 : (C.l1 - 1) - l; };
                per[li].push_back({recs[r + 1], recs[r + 3], iter_of(recs[r + 4]), recs[r + 2], iter_of(recs[r + 5])});
            }
            int64_t cells = 0;
            for (int32_t li = 0; li < nl; ++li) {
                auto &C = p->launches[li];
                if (mine[li] < 0 || head[1 + li] != 0) continue;
                nm_sptrsv_plan::Launch::Team T;
                if (!build_team(C, d, parts[li] < 0 ? -parts[li] : parts[li], part_h.data(), per[li],
                                team_cells_capacity(rows) - cells, team_capacity(rows) - (int64_t)team_tab[d].size(),
                                team_tab[d], T))
                    continue;
                T.cell0 = (int32_t)cells;
                cells += T.n_imp;
                C.team[d] = T;
            }
            p->team_cells[d] = (int32_t)cells;
            if (!team_tab[d].empty() &&
                hipMemcpyAsync(p->dir[d].team, team_tab[d].data(), team_tab[d].size() * 4, hipMemcpyHostToDevice, s) !=
                    hipSuccess)
                return bail(nm::fail(NM_ERR_HIP, "uploading the exchange tables failed"));
        }
    }
    int32_t reach_h[2] = {0, 0};
    if (hipMemcpyAsync(reach_h, L.meta + 4, sizeof(reach_h), hipMemcpyDeviceToHost, s) != hipSuccess ||
        hipStreamSynchronize(s) != hipSuccess)   // also keeps `level_launch` and `team_tab` alive until their copies are done
        return bail(nm::fail(NM_ERR_HIP, "waiting for the plan to complete failed"));
    p->reach[0] = reach_h[0];
    p->reach[1] = reach_h[1];
    *plan_out = p;
    return NM_OK;
}

extern "C" int64_t nm_sptrsv_plan_levels(const nm_sptrsv_plan *plan) { return plan ? plan->nlevels : -1; }

extern "C" int64_t nm_sptrsv_plan_launches(const nm_sptrsv_plan *plan) {
    if (!plan) return -1;
    // (of the solve with A; a stretch of wide levels that no team shares is launched level by level)
    int64_t n = 0;
    for (const auto &L : plan->launches)
        n += L.run && !(plan->ell_pre[0] > 0 && L.team[0].P > 1) ? L.l1 - L.l0 : 1;
    return n;
}

extern "C" int64_t nm_sptrsv_plan_chain_levels(const nm_sptrsv_plan *plan, int transposed) {
    if (!plan) return -1;
    int64_t n = 0;
    for (const auto &L : plan->launches)
        if (L.chain[transposed ? 1 : 0] != 0) n += L.l1 - L.l0;
    return n;
}

extern "C" int64_t nm_sptrsv_plan_shared_launches(const nm_sptrsv_plan *plan, int transposed) {
    if (!plan) return -1;
    int64_t n = 0;
    for (const auto &L : plan->launches)
        if (L.team[transposed ? 1 : 0].P > 1) ++n;
    return n;
}

extern "C" void nm_sptrsv_plan_destroy(nm_sptrsv_plan *plan) { delete plan; }

extern "C" int nm_sptrsv_solve_bytes(int64_t rows, int64_t nnz, size_t *bytes) {
    NM_REQUIRE(rows >= 0 && nnz >= 0 && bytes, "bad arguments");
    *bytes = solve_work_layout(rows, nnz, nullptr, nullptr);
    return NM_OK;
}

extern "C" int nm_sptrsv_solve(const nm_sptrsv_plan *plan, nm_dtype dt, int transposed, const void *data,
                               int unit, const void *b, void *x, void *work, size_t work_bytes,
                               nm_stream stream) {
    NM_REQUIRE(plan != nullptr, "plan is null");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (plan->rows == 0) return NM_OK;
    NM_REQUIRE(b && x && work && (plan->nnz == 0 || data), "null pointer argument");
    const size_t need = solve_work_layout(plan->rows, plan->nnz, nullptr, nullptr);
    if (work_bytes < need)
        return nm::fail(NM_ERR_WORKSPACE, "solve workspace of %zu bytes, %zu needed", work_bytes, need);
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F64) return solve_typed<double>(plan, transposed, data, unit, b, x, work, s);
    return solve_typed<float>(plan, transposed, data, unit, b, x, work, s);
}

// ---- the solve for callers that cannot allocate ---------------------------------
//
// Same launches as nm_sptrsv_solve, with the per-call scratch (level-major copies of
// the coefficients, diagonal, right-hand side and the running solution) in a
// file-scope device array instead of caller memory.  Every GPU the library runs on
// holds its own copy of the array at its own address until the process ends; the
// array's name is only a host-side handle, so the device address is looked up once
// per device and that pointer is what the kernels receive.
namespace {

constexpr size_t kStaticSolveBytes = size_t(64) << 20;   // 64 MiB per GPU
static __device__ __align__(256) unsigned char scratch[kStaticSolveBytes];

constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
void *g_static_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (looked up on first use).
int static_scratch(void **out) {
    int dev = -1;
    NM_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return nm::fail(NM_ERR_UNSUPPORTED, "device index %d", dev);
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_ptr[dev]) {
        void *ptr = nullptr;
        NM_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return nm::fail(NM_ERR_HIP, "hipGetSymbolAddress returned a null address");
        g_static_ptr[dev] = ptr;
    }
    *out = g_static_ptr[dev];
    return NM_OK;
}

}  // namespace

extern "C" int nm_sptrsv_solve_static_capacity(size_t *bytes) {
    NM_REQUIRE(bytes != nullptr, "bytes is null");
    void *ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    *bytes = kStaticSolveBytes;
    return NM_OK;
}

extern "C" int nm_sptrsv_solve_static(const nm_sptrsv_plan *plan, nm_dtype dt, int transposed, const void *data,
                                      int unit, const void *b, void *x, nm_stream stream) {
    NM_REQUIRE(plan != nullptr, "plan is null");
    NM_REQUIRE(dt == NM_F32 || dt == NM_F64, "unknown dtype %d", (int)dt);
    if (plan->rows == 0) return NM_OK;
    NM_REQUIRE(b && x && (plan->nnz == 0 || data), "null pointer argument");
    const size_t need = solve_work_layout(plan->rows, plan->nnz, nullptr, nullptr);
    if (need > kStaticSolveBytes)
        return nm::fail(NM_ERR_UNSUPPORTED,
                        "a solve with %lld rows and %lld entries needs %zu bytes of scratch; the built-in "
                        "buffer of nm_sptrsv_solve_static holds %zu (use nm_sptrsv_solve with caller memory)",
                        (long long)plan->rows, (long long)plan->nnz, need, kStaticSolveBytes);
    void *work = nullptr;
    if (int rc = static_scratch(&work)) return rc;
    hipStream_t s = nm::as_stream(stream);
    if (dt == NM_F64) return solve_typed<double>(plan, transposed, data, unit, b, x, work, s);
    return solve_typed<float>(plan, transposed, data, unit, b, x, work, s);
}

// Test and diagnostics hooks of the triangular solve's level kernels.
//   poll_limit   polls one wavefront makes at one level (for its neighbours, or for the values of
//                another workgroup) before it stops waiting and the solve hands out NaN (0 restores
//                the default, a negative value makes the kernels give up at once);
//   signalling   bit 0: wavefronts of a workgroup signal their neighbours, where no row depends on
//                a row more than one wavefront away, instead of meeting at a barrier after every
//                level (default off); bit 1: launches that the plan would share among several
//                workgroups are taken by one (default: shared).
extern "C" int nm_sptrsv_configure(int64_t poll_limit, int signalling) {
    g_sig_poll_limit.store(poll_limit == 0 ? int64_t(1) << 22 : poll_limit);
    g_sig_enabled.store((signalling & 1) != 0);
    g_team_enabled.store((signalling & 2) == 0);
    return NM_OK;
}
