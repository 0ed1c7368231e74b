// Product plan of a sparse product C = A B (see nm_spgemm_plan.hip for what it is and what runs
// on it).  Shared between the file that builds and uses the plan and the SpGEMM forward, whose
// symbolic phase can leave the plan's destination bytes behind as a by-product of its merge and
// whose numeric phase can then run on them.
#pragma once

#include "nm_common.hpp"
#include "nm_transpose.hpp"

namespace nm {

constexpr int kPlanCap = 8;                      // entries per row of A (class 1) and per octet of a row of B
constexpr int kPlanMaxOctets = 4;                // octets of a named row of B at most (rows of up to 32 entries)
constexpr int kPlanRowCap = kPlanCap * kPlanCap; // entries per row of C
constexpr uint8_t kPlanNone = 0xFF;              // destination byte of an entry a B row does not have

struct PPlan {
    int32_t *flag;     // [0] != 0: a limit does not hold, the plan must not be used; [1], [2]: the product's
                       // class; [3]: the largest |row - column| of an entry of A; [4]: the longest row of
                       // B that A names; [5] != 0: a limit other than that length does not hold
    int32_t *bstart;   // [A_nnz] where the row of B that entry e of A names starts
    int32_t *cstart;   // [A_nnz] where the row of C that entry e of A lies in starts
    uint8_t *dest;     // [A_nnz * 8 * octets] byte k of octet o: position in that row of C of entry 8 o + k of
                       // that row of B
    // cstart and dest once more in COLUMN-major order of A (entry t of the transposed-structure
    // plan): the kernel that walks A by column streams them instead of gathering 12 bytes from a
    // different line for every entry.  Filled when the plan is built or adopted.  Plans of two and
    // four octets only (one-octet plans have t_rec instead).
    int32_t *t_cstart; // [A_nnz]
    uint8_t *t_dest;   // [A_nnz * 8 * octets]
    // one-octet plans: what the walk by column wants of entry t in ONE 16-byte record --
    // {position in A's arrays (t_perm), t_cstart, the eight destination bytes} -- so that a lane
    // fetches it with one request instead of three
    uint32_t *t_rec;   // [A_nnz * 4]
    // the same for the walk by row: {bstart, cstart, the eight destination bytes} of entry e
    uint32_t *rec;     // [A_nnz * 4]
};

// octets: 1 for products whose named rows of B have at most 8 entries, 2 for up to 16, 4 for up to 32
inline size_t pplan_layout(int64_t A_nnz, void *base, PPlan *p, int octets = 1) {
    size_t off = 0;
    auto take = [&](size_t bytes) {
        void *q = base ? static_cast<char *>(base) + off : nullptr;
        off += align256(bytes);
        return q;
    };
    int32_t *flag = (int32_t *)take(64);
    int32_t *bs = (int32_t *)take((size_t)(A_nnz + 1) * 4);
    int32_t *cs = (int32_t *)take((size_t)(A_nnz + 1) * 4);
    uint8_t *d = (uint8_t *)take((size_t)(A_nnz + 1) * 8 * octets);
    int32_t *tcs = octets > 1 ? (int32_t *)take((size_t)(A_nnz + 1) * 4) : nullptr;
    uint8_t *td = octets > 1 ? (uint8_t *)take((size_t)(A_nnz + 1) * 8 * octets) : nullptr;
    uint32_t *tr = octets == 1 ? (uint32_t *)take((size_t)(A_nnz + 1) * 16) : nullptr;
    uint32_t *rr = octets == 1 ? (uint32_t *)take((size_t)(A_nnz + 1) * 16) : nullptr;
    if (p) *p = PPlan{flag, bs, cs, d, tcs, td, tr, rr};
    return off;
}

// C_data AND C_indices of the product from the destination bytes and row starts of B that the
// symbolic phase left in `p` (every row on the merge path); with `keep` also writes p.cstart, which
// completes the plan.  C_indptr is the scanned row pointer.
int spgemm_numeric_on_map(nm_dtype dt, int64_t A_rows, int64_t A_nnz, const void *A_data, const int64_t *A_indptr,
                          const void *B_data, const int64_t *B_indices, const PPlan &p, const int64_t *C_indptr,
                          int64_t *C_indices, void *C_data, bool keep, hipStream_t s);

}  // namespace nm
