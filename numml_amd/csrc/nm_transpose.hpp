// Transposed-structure plan: the pattern of A^T as 32-bit arrays, built once
// per sparsity pattern and reused by every kernel that walks A by column
// (SpMV / SpMM backward, triangular-solve analysis and transposed solve).
//
//   t_indptr[c]  first entry of column c in the column-major order   (cols + 1)
//   t_row[p]     row of the p-th entry in column-major order         (nnz)
//   t_perm[p]    its position in A's row-major arrays                 (nnz)
//   chunk_row[h] row of entry 64*h of A's ROW-major arrays (entry-balanced kernels
//                start their walk there instead of bisecting indptr)  (ceil(nnz/64)+1)
//   flags[0]     1 when the pattern is symmetric (A^T has A's structure, so
//                entry p of column c is the mirror image of the row-major entry p)
//   c_idx32[k]   column of the k-th entry of A's ROW-major arrays, in 32 bits   (nnz)
//   c_ptr32[i]   row pointers of A in 32 bits                                   (rows + 1)
//                (kernels that find a plan read these instead of the int64
//                arrays the interface delivers: half the index traffic)
//   t_pack[p]    t_row and t_perm of entry p in one word, for patterns whose entries lie near
//                the diagonal: low 16 bits = t_row[p] minus the first column of the entry's
//                block of kPackCols columns, high 16 bits = t_perm[p] - p, both signed.  In a
//                block of columns that has a staging list (b_desc): low kStagePlaceBits bits =
//                the entry's place among the listed segments, the bits above = t_perm[p] - p.
//                Valid when flags[1] != 0 (every difference fits its block's layout)  (nnz)
//   c_off16[k]   c_idx32[k] minus the first row of the entry's block of kPackRows rows, signed
//                16 bits.  Valid when flags[2] != 0                              (nnz)
//                (the SpMV kernels read these instead of the 32-bit arrays: half the index
//                traffic again on banded matrices)
//   f_desc[b]    staging list of the b-th block of kPackRows rows: the up to kStageFwd segments of
//                kStageSeg consecutive columns that the block's entries name, ascending, -1 for
//                unused places (kStageDesc ints per block).  A block that has one keeps, in
//                c_off16[k], the place of entry k's column in that list times kStageSeg plus the
//                column's offset inside its segment: the forward loads the listed segments of x
//                into LDS with coalesced requests and looks every entry's factor up there.
//                f_desc[b][0] == -2: no list (more segments than fit, a segment that is cut off
//                by the end of x, more entries than a tile holds); c_off16 is as described above
//   b_desc[b]    the same for the b-th block of kPackCols columns and the ROWS its entries lie
//                in (up to kStageBwd segments); such a block keeps the place in the list in the
//                low bits of t_pack[p] (above).  Only read when flags[1] != 0; blocks of fewer
//                than kStageBwdMin entries get none
//
// Inside a column the entries keep A's row-major order (the sort is stable), so
// rows ascend, exactly like the counting-sort transpose of the reference
// (cpp/sparse_csr_cpu.cpp:349-361); t_perm is that function's At_to_A_idx.
#pragma once

#include "nm_common.hpp"

namespace nm {

struct TPlan {
    int32_t *t_indptr;
    int32_t *t_row;
    int32_t *t_perm;
    int32_t *chunk_row;
    int32_t *flags;
    int32_t *c_idx32;
    int32_t *c_ptr32;
    int32_t *t_pack;
    int16_t *c_off16;
    int32_t *f_desc;
    int32_t *b_desc;
    int32_t *stats;     // per wavefront of the packing kernel: lengths it saw (reduced into flags[6..8])
};

// Blocks the packed offsets are relative to: the columns one workgroup of the planned SpMV
// backward owns, and the rows one workgroup of the forward owns when rows are short.
constexpr int kPackCols = 256, kPackRows = 512;
// Segments of a vector that a block's entries name: length, most per block of rows (forward) and
// per block of columns (backward), ints per list.
constexpr int kStageSeg = 128, kStageFwd = 16, kStageBwd = 12, kStageDesc = 16;
// Entries a block may hold to get a list: the LDS tiles of the kernels that use it.
constexpr int kStageFwdCap = 4096, kStageBwdCap = 2048, kStageBwdMin = 1024;
// A packed word of a block of columns WITH a list: the entry's place among the listed segments in
// the low kStagePlaceBits bits, t_perm[p] - p in the 32 - kStagePlaceBits above (a place needs
// fewer bits than a row offset, and the distance may then be sixteen times as far: the mirror
// entries of a 128^3 seven-point pattern lie 115 000 positions apart).
constexpr int kStagePlaceBits = 11;
static_assert(kStageBwd * kStageSeg <= (1 << kStagePlaceBits), "a place fits its field");

inline size_t align256(size_t v) { return (v + 255) & ~size_t(255); }

// Carves the plan arrays out of `base` (nullptr: size query only); returns bytes.
inline size_t tplan_layout(int64_t rows, int64_t cols, int64_t nnz, void *base, TPlan *p) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align256(bytes);
        return q;
    };
    int32_t *a = (int32_t *)take((size_t)(cols + 1) * 4);
    int32_t *b = (int32_t *)take((size_t)(nnz + 1) * 4);
    int32_t *c = (int32_t *)take((size_t)(nnz + 1) * 4);
    int32_t *h = (int32_t *)take((size_t)((nnz + 63) / 64 + 1) * 4);
    int32_t *f = (int32_t *)take(16 * 4);
    int32_t *ci = (int32_t *)take((size_t)(nnz + 1) * 4);
    int32_t *cp = (int32_t *)take((size_t)(rows + 2) * 4);
    int32_t *tw = (int32_t *)take((size_t)(nnz + 1) * 4);
    int16_t *co = (int16_t *)take((size_t)(nnz + 8) * 2);
    int32_t *fd = (int32_t *)take((size_t)((rows + kPackRows - 1) / kPackRows + 1) * kStageDesc * 4);
    int32_t *bd = (int32_t *)take((size_t)((cols + kPackCols - 1) / kPackCols + 1) * kStageDesc * 4);
    int32_t *st = (int32_t *)take((size_t)(((cols + kPackCols - 1) / kPackCols) * 8 + ((rows + kPackRows - 1) / kPackRows) * 4 + 8) * 4);
    if (p) *p = TPlan{a, b, c, h, f, ci, cp, tw, co, fd, bd, st};
    return off;
}

// Scratch bytes tplan_build needs.
size_t tplan_work_bytes(int64_t rows, int64_t cols, int64_t nnz);

// Enqueues the build on `s`; does not synchronise.  `rowid_out`, when given,
// receives the row of every entry in row-major order (nnz int32).
int tplan_build(int64_t rows, int64_t cols, int64_t nnz, const int64_t *indices, const int64_t *indptr,
                const TPlan &plan, void *work, size_t work_bytes, int32_t *rowid_out, hipStream_t s);

// Puts the int32 keys of every segment [seg_ptr[j], seg_ptr[j + 1]) into ascending order, in
// place (keys inside a segment are distinct).  The number of segments is read from the device
// (`nseg_dev`, at most nseg_max); `tmp` holds nkeys int32 of scratch.
int segments_sort_i32(const int32_t *nseg_dev, int64_t nseg_max, int64_t nkeys, const int32_t *seg_ptr,
                      int32_t *keys, int32_t *tmp, hipStream_t s);

}  // namespace nm
