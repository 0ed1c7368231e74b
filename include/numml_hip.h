/* numml_hip.h -- C ABI of libnumml_hip.so: differentiable CSR kernels for
 * AMD gfx950 (MI355X).
 *
 * Every entry point takes raw DEVICE pointers, sizes and the HIP stream to
 * enqueue on, returns an nm_status and, unless its comment says otherwise,
 * neither allocates nor synchronises.  Outputs are written in full; inputs
 * are never modified.  Structure arrays (`indices`, `indptr`) are int64, the
 * layout the reference's extension receives (cpp/sparse_csr_cpu.cpp:24-25);
 * values are float or double, selected by `dt` (the reference dispatches on
 * the same two types, AT_DISPATCH_FLOATING_TYPES, cpp/sparse_csr_cpu.cpp:22).
 * Column indices must be ascending inside each row, without duplicates.
 *
 * Each group below names the reference function it stands in for; paths are
 * relative to the reference tree (nicknytko/numml).
 */
#ifndef NUMML_HIP_H_
#define NUMML_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum nm_status {
    NM_OK = 0,
    NM_ERR_INVALID = 1,     /* bad argument (null pointer, negative size, bad dtype) */
    NM_ERR_HIP = 2,         /* a HIP runtime call or kernel launch failed */
    NM_ERR_WORKSPACE = 3,   /* caller-provided workspace too small */
    NM_ERR_UNSUPPORTED = 4  /* size beyond what the kernels index (see nm_limits) */
} nm_status;

typedef enum nm_dtype { NM_F32 = 0, NM_F64 = 1 } nm_dtype;

/* hipStream_t, spelled as void* so that C callers need no HIP headers. */
typedef void *nm_stream;

/* Version of this ABI (major * 1000 + minor). */
int nm_version(void);

/* Message of the last failure on the calling thread ("" if none). */
const char *nm_last_error(void);

/* Calibration of the bandwidth figures, no counterpart in the reference: one
 * plain kernel that reads `read_bytes` from src and writes `write_bytes` to dst
 * (both multiples of 16, write_bytes <= read_bytes; 16-byte requests, grid
 * stride), i.e. what this part streams at a given mix of reads and writes.  The
 * SpMV kernels' mixes are measured with it next to their own rates. */
int nm_stream_probe(const void *src, size_t read_bytes, void *dst, size_t write_bytes, nm_stream stream);

/* ------------------------------------------------------------------ SpMV
 * y = A x.  Stands in for spgemv_forward (cpp/sparse_csr.hpp:32-36,
 * cpp/sparse_csr_cpu.cpp:11-39; CUDA launch site cpp/sparse_csr_cuda.cu:42-67).
 * x has `cols` entries, y `rows`.  Rows whose stored entries fit the
 * workgroup's LDS tile are summed in storage order, exactly like the CPU loop.
 */
int nm_spgemv_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                      const void *data, const int64_t *indices, const int64_t *indptr,
                      const void *x, void *y, nm_stream stream);

/* grad_A[k] = g[row(k)] * x[col(k)];  grad_x = A^T g (grad_x is cleared here,
 * then accumulated with hardware floating-point atomics, so its rounding is
 * run-to-run order dependent).  Stands in for spgemv_backward
 * (cpp/sparse_csr.hpp:38-42, cpp/sparse_csr_cpu.cpp:41-77).  Either output
 * pointer may be NULL to skip that gradient. */
int nm_spgemv_backward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                       const void *data, const int64_t *indices, const int64_t *indptr,
                       const void *x, const void *g,
                       void *grad_A, void *grad_x, nm_stream stream);

/* -------------------------------------------------- content key of a pattern
 * A 128-bit key of (indices, indptr), equal for equal patterns whatever memory
 * they live in: a caller that caches per-pattern analysis (the plans below) uses
 * it to recognise a pattern that arrives in fresh tensors, as every product
 * C = A B of the reference's interface does (cpp/sparse_csr.hpp:45-48 returns new
 * index tensors on each call).  No counterpart in the reference, which keeps no
 * per-pattern state.  One pass over both arrays; `work` holds
 * nm_structure_hash_bytes bytes of device scratch.  The call waits for the key:
 * with `host_landing` (32 bytes of pinned host memory the device can write,
 * zeroed once when allocated) a kernel drops it there and the host polls, with
 * NULL it is copied back after a hipStreamSynchronize. */
int nm_structure_hash_bytes(size_t *bytes);

int nm_structure_hash(int64_t nnz, int64_t nptr, const int64_t *indices, const int64_t *indptr,
                      void *work, size_t work_bytes, void *host_landing, uint64_t *key,
                      nm_stream stream);

/* Entries of the longest row of a pattern (one pass over indptr), delivered to the
 * host like the key above: `work` holds 8 bytes of device scratch, `host_landing`
 * as for nm_structure_hash (or NULL).  Waits for the result.  No counterpart in
 * the reference; callers that choose between kernels by how the work is spread
 * ask for it once per pattern. */
int nm_csr_longest_row(int64_t rows, const int64_t *indptr, void *work, size_t work_bytes,
                       void *host_landing, int64_t *longest, nm_stream stream);

/* ---------------------------------------------- transposed-structure plan
 * The pattern of A^T as 32-bit arrays (column pointers, row of each entry and
 * its position in A's arrays, rows ascending inside a column) together with
 * 32-bit copies of A's own column indices and row pointers, built once per
 * sparsity pattern in caller-provided device memory and reused by the
 * *_planned backward entry points below.  It is the structure (not the values)
 * of what csr_transpose_forward returns (cpp/sparse_csr_cpu.cpp:311-367:
 * At_indptr, At_indices, At_to_A_idx).  The build is enqueued on `stream` and
 * does not synchronise; `work` may be released once it has run.  Sizes up to
 * 2^31 - 2 rows, columns and entries (NM_ERR_UNSUPPORTED beyond). */
int nm_csr_transpose_plan_bytes(int64_t rows, int64_t cols, int64_t nnz,
                                size_t *plan_bytes, size_t *work_bytes);

int nm_csr_transpose_plan_build(int64_t rows, int64_t cols, int64_t nnz,
                                const int64_t *indices, const int64_t *indptr,
                                void *plan_mem, size_t plan_bytes,
                                void *work, size_t work_bytes, nm_stream stream);

/* What a built plan found out about the pattern, copied to the host: info[0]
 * pattern symmetric, info[1] / info[2] the packed words of the backward / the
 * 16-bit column offsets of the forward are valid, info[4] blocks of 512 rows
 * with a staging list (the SpMV forward loads the segments of x such a block
 * names into LDS), info[5] blocks of 256 columns with one (the same for the
 * backward), info[6] / info[7] entries of the longest column / row, info[8] the
 * most entries that columns of more than 512 entries hold inside one aligned
 * group of 64 columns (such a group is one workgroup's in the SpMM kernels),
 * info[9] the blocks counted in info[4] that hold at most 3072 entries (a
 * figure for callers that size tiles of their own; the forward build with lists
 * takes 4096 entries in both value types, which every block with a list fits);
 * the other entries are 0.  Waits for `stream`.  No counterpart in the
 * reference; a caller's choice between the kernels on a plan and the stateless
 * ones can be based on it. */
int nm_csr_transpose_plan_info(int64_t rows, int64_t cols, int64_t nnz, const void *plan_mem,
                               int32_t info[16], nm_stream stream);

/* The explicit transpose.  Stands in for csr_transpose_forward
 * (cpp/sparse_csr.hpp:57-61, cpp/sparse_csr_cpu.cpp:311-367): widens a built
 * transposed-structure plan of A's pattern to At_indptr (cols + 1), At_indices
 * and At_to_A_idx (nnz each, int64) and gathers At_data[p] = data[At_to_A_idx[p]].
 * Rows ascend inside every row of A^T, entries with equal coordinates keep A's
 * storage order: the arrays equal the reference's bit for bit. */
int nm_csr_transpose_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                             const void *data, const void *plan_mem,
                             void *At_data, int64_t *At_indices, int64_t *At_indptr,
                             int64_t *At_to_A_idx, nm_stream stream);

/* grad_A[At_to_A_idx[p]] = grad_At[p].  Stands in for csr_transpose_backward
 * (cpp/sparse_csr.hpp:63-65, cpp/sparse_csr_cpu.cpp:369-385). */
int nm_csr_transpose_backward(nm_dtype dt, int64_t nnz, const void *grad_At,
                              const int64_t *At_to_A_idx, void *grad_A, nm_stream stream);

/* nm_spgemv_forward for a pattern whose transposed-structure plan has been
 * built: the kernel reads the plan's 32-bit copies of A's column indices and
 * row pointers instead of the int64 arrays (4 instead of 8 index bytes per
 * entry), and where every entry lies within 32 767 columns of its block of 512
 * rows (banded matrices) the plan's 16-bit column offsets (2 bytes per entry);
 * same sums in the same order, so y is bit-identical. */
int nm_spgemv_forward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                              const void *data, const void *plan_mem,
                              const void *x, void *y, nm_stream stream);

/* The same product by the instantiation that takes blocks of 512 rows with a
 * staging list (nm_csr_transpose_plan_info: info[4]) through LDS: the
 * segments of x such a block names are loaded with coalesced requests and the
 * entries' factors looked up there, where nm_spgemv_forward_planned gathers them
 * one by one through the plan's 32-bit columns.  It reserves LDS for those
 * segments, which costs resident workgroups on blocks without a list: for plans
 * most of whose blocks have one.  Rows of fewer than 32 entries are summed by one
 * lane in storage order in both, the same bits; a longer row is shared by a
 * wavefront where its block exceeds the tile, and in fp64 this build's tile
 * holds 4096 products against 3072, so such rows can differ in rounding between
 * the two.  No counterpart in the reference. */
int nm_spgemv_forward_planned_lists(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                                    const void *data, const void *plan_mem,
                                    const void *x, void *y, nm_stream stream);

/* nm_spgemv_backward on a transposed-structure plan: walks A by column, so
 * grad_x needs neither clearing nor atomics, is summed in ascending row order
 * (the order of cpp/sparse_csr_cpu.cpp:68-73) and is identical on every run.
 * Either output may be NULL.  Banded patterns are walked on one packed word
 * per entry (the plan's t_pack) in place of two 32-bit indices; arrays below
 * 4 GiB are addressed with 32-bit offsets. */
int nm_spgemv_backward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                               const void *data, const void *plan_mem,
                               const void *x, const void *g,
                               void *grad_A, void *grad_x, nm_stream stream);

/* The same gradients by the instantiation that takes blocks of 256 columns with
 * a staging list (nm_csr_transpose_plan_info: info[5]) through LDS: the listed
 * segments of g and x are loaded with coalesced requests and the entries'
 * factors looked up there; nm_spgemv_backward_planned walks such a block on
 * the plan's unpacked row and position arrays instead.  The LDS it reserves
 * costs resident workgroups and the list one more dependent load per block:
 * for plans most of whose column blocks have a list (same bits either way).  No
 * counterpart in the reference. */
int nm_spgemv_backward_planned_lists(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                                     const void *data, const void *plan_mem,
                                     const void *x, const void *g,
                                     void *grad_A, void *grad_x, nm_stream stream);

/* Test hook (no counterpart in the reference): `wide_offsets` = 1 makes
 * nm_spgemv_backward_planned(_lists) address its arrays with 64-bit offsets whatever
 * their size -- the variant that arrays of 4 GiB and more take -- so that it
 * can be run on small inputs; 0 restores the choice by size.  Process-wide. */
int nm_spgemv_configure(int wide_offsets);

/* ------------------------------------------------------------------ SpMM
 * C = A B with dense row-major B (cols x n, row stride ldb elements) and
 * C (rows x n, row stride ldc).  Stands in for spdmm_forward
 * (cpp/sparse_csr.hpp:81-85, cpp/sparse_csr_cpu.cpp:562-602). */
int nm_spdmm_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                     const void *data, const int64_t *indices, const int64_t *indptr,
                     const void *B, int64_t ldb, int64_t n,
                     void *C, int64_t ldc, nm_stream stream);

/* grad_A[k] = <gC[row(k),:], B[col(k),:]>;  grad_B = A^T gC (cleared here,
 * accumulated with atomics).  grad_B is cols x n with row stride ldgb.
 * Stands in for spdmm_backward (cpp/sparse_csr.hpp:87-91,
 * cpp/sparse_csr_cpu.cpp:604-650).  Either output may be NULL. */
int nm_spdmm_backward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                      const void *data, const int64_t *indices, const int64_t *indptr,
                      const void *B, int64_t ldb, const void *gC, int64_t ldg, int64_t n,
                      void *grad_A, void *grad_B, int64_t ldgb, nm_stream stream);

/* nm_spdmm_backward on a transposed-structure plan: grad_B = A^T gC is computed
 * as a product over A's columns (no clearing, no atomics, sums in ascending
 * row order like cpp/sparse_csr_cpu.cpp:639-646).  Either output may be NULL. */
int nm_spdmm_backward_planned(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                              const void *data, const int64_t *indices, const int64_t *indptr,
                              const void *plan_mem,
                              const void *B, int64_t ldb, const void *gC, int64_t ldg, int64_t n,
                              void *grad_A, void *grad_B, int64_t ldgb, nm_stream stream);

/* ---------------------------------------------------------------- SpGEMM
 * C = A B, both CSR.  Stands in for spgemm_forward (cpp/sparse_csr.hpp:45-48,
 * cpp/sparse_csr_cpu.cpp:117-216).  Two calls, because the caller must size
 * C between them:
 *
 *   nm_spgemm_workspace_bytes  -> bytes of device scratch both phases need
 *   nm_spgemm_symbolic         -> fills C_indptr (A_rows + 1 entries).  With
 *                                 host_landing (see below; may be NULL) the call
 *                                 makes the row pointer as soon as its first
 *                                 kernel has counted the short rows, waits for
 *                                 nnz(C) and the news whether any row needs
 *                                 the hash path and, when none does, leaves
 *                                 the hash path's launches out; the
 *                                 nm_spgemm_symbolic_result that follows on the
 *                                 same workspace and landing place then returns
 *                                 at once
 *   nm_spgemm_symbolic_result  -> hands the host nnz(C) = C_indptr[A_rows],
 *                                 with which the caller allocates, and the
 *                                 number of rows the hash path took.  With a
 *                                 landing place it returns when the two numbers
 *                                 are known, which can be before the last
 *                                 entries of C_indptr are written: C_indptr is
 *                                 complete for work queued on `stream` after
 *                                 this call, not for another stream or a host
 *                                 read without hipStreamSynchronize.  With NULL
 *                                 it waits for the stream (the reference's own
 *                                 read of the last row pointer,
 *                                 cpp/sparse_csr_cpu.cpp:166, is this
 *                                 synchronisation point); a caller may read
 *                                 C_indptr[A_rows] itself instead.
 *                                 host_landing: 32 bytes of pinned host memory
 *                                 the device can write (hipHostMalloc with
 *                                 hipHostMallocCoherent, or a pinned torch
 *                                 tensor), zeroed once by the caller when it is
 *                                 allocated and from then on left to this
 *                                 call, which has a one-lane kernel write the
 *                                 two numbers and a ticket there and polls the
 *                                 ticket (a few us instead of the ~30 us of a
 *                                 stream wait); the fourth word is the host's
 *                                 own note that nm_spgemm_symbolic has had the
 *                                 numbers landed already.  One landing place
 *                                 serves one call at a time (one per host
 *                                 thread), and the landing place given to
 *                                 nm_spgemm_symbolic is the one to give to the
 *                                 nm_spgemm_symbolic_result after it.  NULL:
 *                                 a plain copy and hipStreamSynchronize.  The
 *                                 library itself allocates nothing here.
 *   nm_spgemm_numeric          -> fills C_indices (ascending in each row) and
 *                                 C_data; entries whose sum is 0 are kept,
 *                                 as the reference keeps them.  hash_rows is
 *                                 the figure nm_spgemm_symbolic_result gave,
 *                                 or -1 when it was not asked: with 0 the
 *                                 launches of the hash path are left out.
 *
 * The same workspace (contents preserved) must be passed to both phases.
 * Products of one output entry are added in the order of A's row, which is
 * the reference's order. */
int nm_spgemm_workspace_bytes(int64_t A_rows, int64_t B_cols, size_t *bytes);

int nm_spgemm_symbolic(int64_t A_rows, int64_t A_cols, int64_t B_cols,
                       const int64_t *A_indices, const int64_t *A_indptr,
                       const int64_t *B_indices, const int64_t *B_indptr,
                       int64_t *C_indptr, void *workspace, size_t workspace_bytes,
                       void *host_landing, nm_stream stream);

int nm_spgemm_symbolic_result(int64_t A_rows, int64_t B_cols, const void *workspace,
                              size_t workspace_bytes, int64_t *nnz_C, int64_t *hash_rows,
                              void *host_landing, nm_stream stream);

int nm_spgemm_numeric(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t B_cols,
                      const void *A_data, const int64_t *A_indices, const int64_t *A_indptr,
                      const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                      const int64_t *C_indptr, int64_t *C_indices, void *C_data,
                      void *workspace, size_t workspace_bytes, int64_t hash_rows,
                      nm_stream stream);

/* grad_A[(i,j)] = sum_c gC[i,c] B[j,c];  grad_B[(k,c)] = sum_i A[i,k] gC[i,c],
 * both restricted to the stored patterns.  Stands in for spgemm_backward
 * (cpp/sparse_csr.hpp:50-54, cpp/sparse_csr_cpu.cpp:218-307).  grad_B is
 * cleared here and accumulated with atomics.  Either output may be NULL. */
int nm_spgemm_backward(nm_dtype dt, int64_t A_rows, int64_t A_nnz, int64_t B_nnz,
                       const void *gC, const int64_t *C_indices, const int64_t *C_indptr,
                       const void *A_data, const int64_t *A_indices, const int64_t *A_indptr,
                       const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                       void *grad_A, void *grad_B, nm_stream stream);

/* nm_spgemm_backward on the transposed-structure plan of A's pattern
 * (nm_csr_transpose_plan_build with A's rows, columns and entries): work is
 * shared out by row of B, the entries of A that meet a row come from the plan
 * in ascending row order, and both gradients are summed in registers in the
 * order of the reference's loops (cpp/sparse_csr_cpu.cpp:261-274 ascending
 * column for grad_A, :291-303 ascending row for grad_B): no atomics, no
 * clearing, identical on every run and bit-identical to the CPU result, except
 * for rows of B whose (row length) x (length of A's column) exceeds 4096: those
 * get a whole workgroup and grad_B is added across its lanes in tree order,
 * which differs by rounding only.  Either output may be NULL. */
int nm_spgemm_backward_planned(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t A_nnz,
                               int64_t B_nnz, int64_t C_nnz,
                               const void *gC, const int64_t *C_indices, const int64_t *C_indptr,
                               const void *A_data, const void *A_plan_mem,
                               const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                               void *grad_A, void *grad_B, nm_stream stream);

/* Product plan of C = A B: per stored entry of A, where its row of B and its row of
 * C start and, for each of the (at most eight) entries of that row of B, the
 * position of its column inside the row of C.  Built once for a pair of patterns
 * and their product's pattern; afterwards the numeric product and both gradients
 * need no merge, hash table or search (the reference repeats the symbolic work in
 * every call, cpp/sparse_csr_gemm_cuda.cu:10-302, and searches C in every backward
 * pass, cpp/sparse_csr_cpu.cpp:246-303).  Results are bit-identical to
 * nm_spgemm_numeric / nm_spgemm_backward_planned: sums run in the serial loops' order.
 *
 *   nm_spgemm_plan_build    C_indices / C_indptr must be the pattern of A B as
 *                           nm_spgemm_numeric returns it (complete, rows ascending).
 *                           A_plan_mem: the transposed-structure plan of A
 *                           (nm_csr_transpose_plan_build).  *usable = 0: the plan
 *                           must not be used (a row of B that A names has more than
 *                           32 entries, a row of C more than 254, a column of A more
 *                           than 4096, or a position does not fit 31 bits); negative:
 *                           it must not be used either, but a plan with more octets
 *                           can be (nm_spgemm_plan_build_wide, below).
 *                           Otherwise the product's class: 1 -- rows of A of at most
 *                           8 and rows of C of at most 64 entries, 2 -- longer rows of
 *                           A, 3 -- also rows of C of 65..254 entries.  Waits for the
 *                           stream (through host_landing, 32 bytes of pinned host
 *                           memory, when given; NULL: a copy and a synchronisation).
 *   nm_spgemm_numeric_planned   C_data of the product, C_indptr as built from;
 *                           plan_class as reported when the plan was built.
 *   nm_spgemm_backward_mapped   grad_A and / or grad_B (either may be NULL) of
 *                           gC laid out on the plan's pattern of C.
 *
 * The plan can also be had as a by-product of the product's first computation:
 *   nm_spgemm_symbolic_mapped   nm_spgemm_symbolic that, while it merges the rows to
 *                           count them, records in plan_mem where every product of a
 *                           merge-path row goes (the plan's destination bytes and B
 *                           row starts).  A and B must have fewer than 2^31 entries.
 *   nm_spgemm_numeric_mapped    nm_spgemm_numeric that, when hash_rows is 0 (every row
 *                           on the merge path, from nm_spgemm_symbolic_result) and
 *                           C_nnz < 2^31, adds the products up on those records
 *                           instead of merging the rows a second time, and, with
 *                           keep_plan != 0, fills in the plan's C row starts (4 bytes
 *                           per entry of A that a caller who will not adopt the plan
 *                           need not have written: keep_plan == 0, plan_mem is then
 *                           scratch of the call); otherwise it is nm_spgemm_numeric
 *                           and plan_mem holds nothing usable.  Same results, bit
 *                           for bit.
 *   nm_spgemm_plan_adopt    checks what such a plan still needs before the kernels
 *                           above may run on it (no column of A with more than 4096
 *                           entries: A_plan_mem is A's transposed-structure plan;
 *                           sizes below 2^31; hash_rows == 0) and reports `usable`
 *                           like nm_spgemm_plan_build.  Waits for the stream. */
int nm_spgemm_symbolic_mapped(int64_t A_rows, int64_t A_cols, int64_t B_cols, int64_t A_nnz, int64_t B_nnz,
                              const int64_t *A_indices, const int64_t *A_indptr,
                              const int64_t *B_indices, const int64_t *B_indptr,
                              int64_t *C_indptr, void *workspace, size_t workspace_bytes,
                              void *plan_mem, size_t plan_bytes, void *host_landing, nm_stream stream);
int nm_spgemm_numeric_mapped(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t B_cols,
                             int64_t A_nnz, int64_t C_nnz,
                             const void *A_data, const int64_t *A_indices, const int64_t *A_indptr,
                             const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                             const int64_t *C_indptr, int64_t *C_indices, void *C_data,
                             void *workspace, size_t workspace_bytes, int64_t hash_rows,
                             void *plan_mem, size_t plan_bytes, int keep_plan, nm_stream stream);
int nm_spgemm_plan_adopt(int64_t A_rows, int64_t A_cols, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                         int64_t hash_rows, const void *A_plan_mem, void *plan_mem, size_t plan_bytes,
                         void *host_landing, int *usable, nm_stream stream);
int nm_spgemm_plan_bytes(int64_t A_nnz, size_t *plan_bytes);
int nm_spgemm_plan_build(int64_t A_rows, int64_t A_cols, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                         const int64_t *A_indices, const int64_t *A_indptr,
                         const int64_t *B_indices, const int64_t *B_indptr,
                         const int64_t *C_indices, const int64_t *C_indptr,
                         const void *A_plan_mem, void *plan_mem, size_t plan_bytes,
                         void *host_landing, int *usable, nm_stream stream);
int nm_spgemm_numeric_planned(nm_dtype dt, int plan_class, int64_t A_rows, int64_t A_nnz, int64_t B_nnz,
                              int64_t C_nnz, const void *A_data, const int64_t *A_indptr, const void *B_data,
                              const void *plan_mem, const int64_t *C_indptr, void *C_data,
                              nm_stream stream);
int nm_spgemm_backward_mapped(nm_dtype dt, int64_t A_rows, int64_t A_cols, int64_t A_nnz,
                              int64_t B_nnz, int64_t C_nnz, const void *gC, const void *A_data,
                              const void *A_plan_mem, const void *B_data, const int64_t *B_indptr,
                              const void *plan_mem, void *grad_A, void *grad_B, nm_stream stream);

/* Product plans for named rows of B of up to 16 or 32 entries (no counterpart in
 * the reference): `octets` = 2 or 4 destination octets per entry of A instead of
 * one.  nm_spgemm_plan_build reports in `usable` a NEGATIVE number -L when the
 * only limit its one-octet plan misses is that the longest row of B that A names
 * has L entries, 9 <= L <= 32: the caller then allocates
 * nm_spgemm_plan_bytes_wide(A_nnz, L <= 16 ? 2 : 4) and calls
 * nm_spgemm_plan_build_wide with that number of octets, which reports class 4
 * (two octets) or 5 (four), 6 or 7 when rows of C have 65 to 254 entries as
 * well, to be handed to nm_spgemm_numeric_planned and
 * nm_spgemm_backward_mapped_wide; with octets = 1 and classes 1 to 3 these are
 * the calls above.  Same sums in the same order, bit for bit. */
int nm_spgemm_plan_bytes_wide(int64_t A_nnz, int octets, size_t *plan_bytes);
int nm_spgemm_plan_build_wide(int64_t A_rows, int64_t A_cols, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                              const int64_t *A_indices, const int64_t *A_indptr,
                              const int64_t *B_indices, const int64_t *B_indptr,
                              const int64_t *C_indices, const int64_t *C_indptr,
                              const void *A_plan_mem, void *plan_mem, size_t plan_bytes, int octets,
                              void *host_landing, int *usable, nm_stream stream);
int nm_spgemm_backward_mapped_wide(nm_dtype dt, int plan_class, int64_t A_rows, int64_t A_cols,
                                   int64_t A_nnz, int64_t B_nnz, int64_t C_nnz, const void *gC,
                                   const void *A_data, const void *A_plan_mem, const void *B_data,
                                   const int64_t *B_indptr, const void *plan_mem,
                                   void *grad_A, void *grad_B, nm_stream stream);

/* ---------------------------------------------------------------- SpTRSV
 * Level-scheduled triangular solve.  Stands in for sptrsv_forward /
 * sptrsv_backward (cpp/sparse_csr.hpp:94-105, cpp/sparse_csr_cpu.cpp:652-759).
 *
 * A plan holds the level schedule of one triangle of one sparsity pattern
 * together with the structure of A^T, and is reused for every solve with that
 * pattern (values may change) in either direction: x = A^{-1} b and, with
 * `transposed` != 0, x = A^{-T} b, the system the backward solves
 * (cpp/sparse_csr_cpu.cpp:733-738 builds A^T explicitly and flips `lower`).
 * `lower` always describes A itself.
 *
 * The plan's device arrays live in caller-provided memory (`plan_mem`, which
 * must stay allocated until nm_sptrsv_plan_destroy); `work` is scratch needed
 * only during nm_sptrsv_analyse.  The handle itself is a small host object.
 * nm_sptrsv_analyse synchronises the stream: it reads the level sizes back to
 * lay out the launches.  Rows and entries are indexed with 32 bits inside a
 * plan (NM_ERR_UNSUPPORTED beyond 2^31 - 2).
 */
typedef struct nm_sptrsv_plan nm_sptrsv_plan;

int nm_sptrsv_plan_bytes(int64_t rows, int64_t nnz, size_t *plan_bytes, size_t *work_bytes);

int nm_sptrsv_analyse(int64_t rows, int64_t nnz,
                      const int64_t *indices, const int64_t *indptr, int lower,
                      void *plan_mem, size_t plan_bytes, void *work, size_t work_bytes,
                      nm_sptrsv_plan **plan, nm_stream stream);

/* Number of dependency levels / of level-kernel launches one solve with A issues. */
int64_t nm_sptrsv_plan_levels(const nm_sptrsv_plan *plan);
int64_t nm_sptrsv_plan_launches(const nm_sptrsv_plan *plan);
/* Levels of the solve with A (transposed = 0) or with A^T (1) that sit in runs of one-row levels
 * which a single wavefront walks with the newest solution in a register (banded factors,
 * bidiagonal and tridiagonal triangles); diagnostics. */
int64_t nm_sptrsv_plan_chain_levels(const nm_sptrsv_plan *plan, int transposed);
/* Launches of the solve with A (transposed = 0) or with A^T (1) whose levels are each shared by
 * several workgroups (levels of more than 256 rows whose dependencies cross between the
 * workgroups' parts in a way that can be pipelined: triangles of grid stencils); diagnostics. */
int64_t nm_sptrsv_plan_shared_launches(const nm_sptrsv_plan *plan, int transposed);

void nm_sptrsv_plan_destroy(nm_sptrsv_plan *plan);

/* x = T^{-1} b where T is the planned triangle of A (or its transpose).  Sums
 * run in double for either dtype, in the walk order of the reference loop, and
 * are rounded once at the end (cpp/sparse_csr_cpu.cpp:659-662, :722).
 * `unit` != 0 ignores the stored diagonal.  `work` is device scratch of
 * nm_sptrsv_solve_bytes(rows, nnz) bytes (the call's values regathered in
 * level order and the running solution); it must not alias x or b. */
int nm_sptrsv_solve_bytes(int64_t rows, int64_t nnz, size_t *bytes);

int nm_sptrsv_solve(const nm_sptrsv_plan *plan, nm_dtype dt, int transposed,
                    const void *data, int unit, const void *b, void *x,
                    void *work, size_t work_bytes, nm_stream stream);

/* How the level kernels of the solve synchronise (no counterpart in the reference).
 * `signalling` is a set of bits.
 * Bit 0 (default off): inside a single-workgroup launch every wavefront meets at a
 * workgroup barrier after every level; with the bit set, where no row of a triangle
 * depends on a row more than one wavefront away inside the level before it (stencil
 * and banded matrices), a wavefront instead publishes the levels it has finished in
 * LDS and waits only for its neighbours.  (Measured slower than the barrier on
 * MI355X, hence off; results are the same bits.)
 * Bit 1 (default off): launches that the plan would share among up to sixteen
 * workgroups (nm_sptrsv_plan_shared_launches; each takes up to 256 rows of every level and
 * receives the few values it needs from the others through device memory, running a
 * few levels behind the workgroup it receives from) are taken by one workgroup
 * instead.  Results are the same bits either way.
 * All waiting is for rows of lower levels, by wavefronts of workgroups that are all
 * resident (a shared launch needs as many free compute units as it has workgroups),
 * so the waits end; `poll_limit` bounds the polls of one wait all the same (0: the
 * default of 2^22, seconds; negative: give up at once, for tests): when it is
 * exceeded the waiting stops for good and x comes back as NaN throughout.
 * Process-wide; takes effect with the next solve. */
int nm_sptrsv_configure(int64_t poll_limit, int signalling);

/* nm_sptrsv_solve without the `work` argument, for callers that cannot allocate
 * device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  It has no counterpart in the reference.  The scratch
 * of the solve lives in a 64 MiB device array built into the library, one copy
 * per GPU, held until the process ends; the call allocates nothing, neither
 * through HIP nor through any other library, and does not synchronise.  A plan
 * whose nm_sptrsv_solve_bytes(rows, nnz) exceeds nm_sptrsv_solve_static_capacity
 * (roughly 7 * rows + 3 * nnz doubles, e.g. 500 000 rows with three entries per
 * row) is rejected with NM_ERR_UNSUPPORTED.  Every call on one GPU uses that
 * GPU's one array: calls that overlap on the same GPU (two streams, two threads)
 * race and must be serialised by the caller.  Results are bit-identical to
 * nm_sptrsv_solve.  The device must be current on the calling thread.
 * nm_sptrsv_solve_static_capacity also performs the one-time address look-up of
 * the array for the current device, so a caller may call it before it starts a
 * capture. */
int nm_sptrsv_solve_static_capacity(size_t *bytes);

int nm_sptrsv_solve_static(const nm_sptrsv_plan *plan, nm_dtype dt, int transposed,
                           const void *data, int unit, const void *b, void *x,
                           nm_stream stream);

/* out[k] = alpha * a[row(k)] * b[col(k)] for every stored entry: the masked
 * outer product behind grad_A of the solve (alpha = -1,
 * cpp/sparse_csr_cpu.cpp:750-755) and of SpMV (alpha = 1, :60-65). */
int nm_masked_outer(nm_dtype dt, int64_t rows, int64_t nnz,
                    const int64_t *indices, const int64_t *indptr,
                    double alpha, const void *a, const void *b, void *out,
                    nm_stream stream);

/* ------------------------------------------------------------ sparse LU
 * M = L + U of a square matrix with a stored diagonal, without pivoting, on the
 * filled pattern (the unit diagonal of L is not stored); replaces splu_cpu /
 * splu_cuda (cpp/sparse_csr.hpp:107-111, cpp/sparse_csr_cpu.cpp:777-1016).
 * Pattern and factors equal the reference's CPU result bit for bit.
 *
 *   nm_splu_symbolic_bytes  scratch for the two pattern passes
 *   nm_splu_symbolic        As_indptr[rows + 1] of the filled pattern (the
 *                           caller reads As_indptr[rows] to size the next call)
 *   nm_splu_fill            As_indices (ascending per row) and As_data: A's
 *                           value where A stores the column, 0 at the fill
 *   nm_splu_values          As_data alone, for a pattern from an earlier
 *                           nm_splu_fill of a matrix with A's structure
 *   nm_splu_numeric         in-place factorisation of the TRANSPOSE of that
 *                           matrix (rows of Mt = columns of M).  Columns are
 *                           taken in ascending order by wavefronts that wait
 *                           on a flag per column they depend on; poll_limit
 *                           bounds the polls of one flag during which no
 *                           column anywhere finishes (0 = default), and when
 *                           it is exceeded every wavefront leaves and the call
 *                           returns NM_ERR_HIP; Mt_data is then left partly
 *                           factorised (undefined).  Synchronises the stream.
 * The caller transposes As -> Mt before, and Mt -> M after, the numeric phase. */
int nm_splu_symbolic_bytes(int64_t rows, size_t *bytes);
int nm_splu_symbolic(int64_t rows, const int64_t *A_indices,
                     const int64_t *A_indptr, int64_t *As_indptr,
                     void *workspace, size_t workspace_bytes, nm_stream stream);
int nm_splu_fill(nm_dtype dt, int64_t rows, const void *A_data,
                 const int64_t *A_indices, const int64_t *A_indptr,
                 const int64_t *As_indptr, int64_t *As_indices, void *As_data,
                 void *workspace, size_t workspace_bytes, nm_stream stream);
int nm_splu_values(nm_dtype dt, int64_t rows, const void *A_data,
                   const int64_t *A_indices, const int64_t *A_indptr,
                   const int64_t *As_indptr, const int64_t *As_indices,
                   void *As_data, nm_stream stream);
int nm_splu_numeric_bytes(int64_t cols, size_t *bytes);
int nm_splu_numeric(nm_dtype dt, int64_t cols, void *Mt_data,
                    const int64_t *Mt_indices, const int64_t *Mt_indptr,
                    void *workspace, size_t workspace_bytes, int64_t poll_limit,
                    nm_stream stream);

/* ------------------------------------------------- linear combination
 * C = alpha A + beta B for two matrices of one shape; a column stored by either
 * operand is stored by C (also when the sum is 0), columns ascending.  Stands in
 * for splincomb_forward (cpp/sparse_csr.hpp:67-72, cpp/sparse_csr_cpu.cpp:387-481),
 * in two calls like the product: _symbolic fills C_indptr (rows + 1), the caller
 * reads nnz(C) = C_indptr[rows] and allocates, _numeric fills C_indices and
 * C_data.  `workspace` holds nm_splincomb_workspace_bytes(rows) bytes.  alpha
 * and beta are rounded to the value type before use, as the reference does
 * (alpha.item<scalar_t>()). */
int nm_splincomb_workspace_bytes(int64_t rows, size_t *bytes);

int nm_splincomb_symbolic(int64_t rows,
                          const int64_t *A_indices, const int64_t *A_indptr,
                          const int64_t *B_indices, const int64_t *B_indptr,
                          int64_t *C_indptr, void *workspace, size_t workspace_bytes,
                          nm_stream stream);

int nm_splincomb_numeric(nm_dtype dt, int64_t rows,
                         double alpha, const void *A_data, const int64_t *A_indices, const int64_t *A_indptr,
                         double beta, const void *B_data, const int64_t *B_indices, const int64_t *B_indptr,
                         const int64_t *C_indptr, int64_t *C_indices, void *C_data,
                         nm_stream stream);

/* grad_A[k] = alpha * grad_C at A's coordinate, grad_B likewise with beta.  Stands
 * in for splincomb_backward (cpp/sparse_csr.hpp:74-79,
 * cpp/sparse_csr_cpu.cpp:483-560).  Either output may be NULL. */
int nm_splincomb_backward(nm_dtype dt, int64_t rows,
                          double alpha, const int64_t *A_indices, const int64_t *A_indptr,
                          double beta, const int64_t *B_indices, const int64_t *B_indptr,
                          const void *grad_C, const int64_t *C_indices, const int64_t *C_indptr,
                          void *grad_A, void *grad_B, nm_stream stream);

/* The linear combination of two patterns that stay the same while the values
 * change (no counterpart in the reference, which merges the rows again on every
 * call).  nm_splincomb_plan_build records, for the pattern of C that
 * nm_splincomb_numeric produced, which entry of A and of B lies at every entry
 * of C and where every entry of A and of B lies in C (int32; patterns of 2^31
 * entries or more are refused with NM_ERR_UNSUPPORTED).  On these maps
 * nm_splincomb_numeric_planned fills C_data in one pass -- no symbolic phase, no
 * read of nnz(C) by the host -- and nm_splincomb_backward_planned gathers the
 * gradients; both produce the bits of the calls they replace.  The caller keeps
 * C's pattern (it is the same for every call).  Either gradient may be NULL. */
int nm_splincomb_plan_bytes(int64_t A_nnz, int64_t B_nnz, int64_t C_nnz, size_t *plan_bytes);

int nm_splincomb_plan_build(int64_t rows, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                            const int64_t *A_indices, const int64_t *A_indptr,
                            const int64_t *B_indices, const int64_t *B_indptr,
                            const int64_t *C_indices, const int64_t *C_indptr,
                            void *plan_mem, size_t plan_bytes, nm_stream stream);

int nm_splincomb_numeric_planned(nm_dtype dt, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                                 double alpha, const void *A_data, double beta, const void *B_data,
                                 const void *plan_mem, void *C_data, nm_stream stream);

int nm_splincomb_backward_planned(nm_dtype dt, int64_t A_nnz, int64_t B_nnz, int64_t C_nnz,
                                  double alpha, double beta, const void *grad_C,
                                  const void *plan_mem, void *grad_A, void *grad_B,
                                  nm_stream stream);

/* ------------------------------------------ dense copy, row sums, diagonal
 * dense[i, j] = data[k] on a zero background (row stride ld >= cols); stands in for
 * csr_to_dense_forward (cpp/sparse_csr_cpu.cpp:1052-1076).  The backward gathers
 * grad_A[k] = grad_dense[i, j] (csr_to_dense_backward, :1078-1104). */
int nm_csr_to_dense_forward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                            const void *data, const int64_t *indices, const int64_t *indptr,
                            void *dense, int64_t ld, nm_stream stream);

int nm_csr_to_dense_backward(nm_dtype dt, int64_t rows, int64_t cols, int64_t nnz,
                             const void *grad_dense, int64_t ld,
                             const int64_t *indices, const int64_t *indptr,
                             void *grad_A, nm_stream stream);

/* x[i] = sum of the stored values of row i, added in storage order for rows that
 * fit the workgroup's LDS tile (csr_row_sum_forward, cpp/sparse_csr_cpu.cpp:1106-1131);
 * backward grad_A[k] = g[row(k)] (csr_row_sum_backward, :1133-1156). */
int nm_csr_row_sum_forward(nm_dtype dt, int64_t rows, int64_t nnz,
                           const void *data, const int64_t *indptr, void *x, nm_stream stream);

int nm_csr_row_sum_backward(nm_dtype dt, int64_t rows, int64_t nnz,
                            const int64_t *indptr, const void *g, void *grad_A, nm_stream stream);

/* x[i] = stored entry (i, i) or 0 (csr_extract_diagonal_forward,
 * cpp/sparse_csr_cpu.cpp:1158-1186; x has `rows` entries); backward grad_A = 0
 * except g[i] on the diagonal entries (csr_extract_diagonal_backward, :1188-1213). */
int nm_csr_extract_diagonal_forward(nm_dtype dt, int64_t rows, int64_t nnz,
                                    const void *data, const int64_t *indices, const int64_t *indptr,
                                    void *x, nm_stream stream);

int nm_csr_extract_diagonal_backward(nm_dtype dt, int64_t rows, int64_t nnz,
                                     const int64_t *indices, const int64_t *indptr,
                                     const void *g, void *grad_A, nm_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* NUMML_HIP_H_ */
