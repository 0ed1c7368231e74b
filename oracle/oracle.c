/* oracle.c -- serial CPU restatement of the reference's differentiable CSR
 * kernels.  TEST INFRASTRUCTURE ONLY: it is the checker the HIP kernels are
 * compared with and the "port" CPU baseline of the benchmark.  Nothing in the
 * product (numml_amd/) may load it.
 *
 * Functions and the reference lines they follow (cpp/sparse_csr_cpu.cpp):
 *   or_spgemv_forward/backward   :11-77
 *   or_spgemm_symbolic/numeric   :81-216  (SMMP, Bank & Douglas 1993)
 *   or_spgemm_backward           :218-307
 *   or_csr_transpose             :311-367
 *   or_spdmm_forward/backward    :562-650
 *   or_sptrsv_forward/backward   :652-759
 *   or_splincomb_forward/backward_one :387-560
 *   or_row_sum, or_diagonal(_backward) :1106-1213
 *   or_splu_symbolic/numeric     :777-1016 (fill2 symbolic phase + left-looking numeric phase)
 * (csr_to_dense_forward/backward, :1050-1104, and csr_transpose_backward,
 * :369-385, are plain index assignments and are restated with NumPy indexing in
 * oracle/__init__.py.)
 *
 * How each is pinned (tests/test_oracle.py): against the reference's own CPU
 * sources compiled in place (oracle/_ref, when the reference tree is present),
 * against fixtures written from that build (tests/golden/), and against what
 * the mathematics fixes (dense products, SciPy products of the pattern,
 * closed-form gradients, residuals).  No function here is "parity unpinned".
 */
#include <stdint.h>
#include <stddef.h>

/* Insert column k into the ascending singly linked list threaded through ll
 * (-2 terminates, -1 = not in the list).  cpp/sparse_csr_cpu.cpp:81-106. */
static void or_ll_insert(int64_t *ll, int64_t *head, int64_t k)
{
    if (*head == -2) {
        *head = k;
        ll[k] = -2;
    } else if (k < *head) {
        ll[k] = *head;
        *head = k;
    } else {
        int64_t prev = *head, cur = ll[*head];
        while (cur >= 0) {
            if (k < cur) {
                ll[prev] = k;
                ll[k] = cur;
                return;
            }
            prev = cur;
            cur = ll[cur];
        }
        ll[prev] = k;
        ll[k] = -2;
    }
}

/* Position of `key` in the ascending slice idx[lo, hi), or -1. */
static int64_t or_bisect(const int64_t *idx, int64_t lo, int64_t hi, int64_t key)
{
    const int64_t end = hi;
    while (lo < hi) {
        const int64_t mid = lo + (hi - lo) / 2;
        if (idx[mid] < key) lo = mid + 1;
        else hi = mid;
    }
    return (lo < end && idx[lo] == key) ? lo : -1;
}

/* Symbolic phase of SMMP.  cpp/sparse_csr_cpu.cpp:150-168: `mark[k] == i`
 * says column k was already counted for row i; mark (all -1) has length
 * max(A_rows, A_cols, B_cols).  Returns nnz(C). */
int64_t or_spgemm_symbolic(int64_t A_rows, const int64_t *A_indices, const int64_t *A_indptr,
                           const int64_t *B_indices, const int64_t *B_indptr,
                           int64_t *C_indptr, int64_t *mark)
{
    C_indptr[0] = 0;
    for (int64_t i = 0; i < A_rows; i++) {
        int64_t len = 0;
        for (int64_t jj = A_indptr[i]; jj < A_indptr[i + 1]; jj++) {
            const int64_t j = A_indices[jj];
            for (int64_t kk = B_indptr[j]; kk < B_indptr[j + 1]; kk++) {
                const int64_t k = B_indices[kk];
                if (mark[k] != i) {
                    mark[k] = i;
                    len++;
                }
            }
        }
        C_indptr[i + 1] = C_indptr[i] + len;
    }
    return C_indptr[A_rows];
}

#define OR_CAT_(a, b) a##_##b
#define OR_CAT(a, b) OR_CAT_(a, b)

#define T float
#define FN(name) OR_CAT(name, f32)
#include "oracle_body.inc"
#undef T
#undef FN

#define T double
#define FN(name) OR_CAT(name, f64)
#include "oracle_body.inc"
#undef T
#undef FN
