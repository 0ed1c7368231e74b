"""The compiled ``numml_torch_cpp`` extension (csrc/torch_binding.cpp) on a HIP device.

It is the module the reference's Python layer imports (numml/sparse/_csr.py:2);
here every one of its eight functions is checked against the CPU oracle on
seeded inputs and, bit for bit, against the ctypes binding of the same C ABI.
Tolerance: util.RTOL (1e-5 for float32, 1e-12 for float64); structure is exact.
"""
import numpy as np
import pytest
import torch

import numml_amd
import oracle
from numml_amd import generators as G
from numml_amd import numml_torch_cpp as mirror
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu

DTYPES = [np.float32, np.float64]


@pytest.fixture(scope="module")
def cpp():
    return numml_amd.load_compiled()


@pytest.fixture(params=["eager", "atomic"])
def mode(request, cpp):
    old_cpp, old_mirror = cpp.backward_mode(), mirror.BACKWARD_MODE
    cpp.set_backward_mode(request.param)
    mirror.BACKWARD_MODE = request.param
    yield request.param
    cpp.set_backward_mode(old_cpp)
    mirror.BACKWARD_MODE = old_mirror


def test_exports_the_reference_functions(cpp):
    for name in ("spgemv_forward", "spgemv_backward", "spgemm_forward", "spgemm_backward", "spdmm_forward",
                 "spdmm_backward", "sptrsv_forward", "sptrsv_backward"):     # cpp/sparse_csr.cpp:307-319
        assert callable(getattr(cpp, name)), name


@pytest.mark.parametrize("dtype", DTYPES)
def test_spgemv(dev, cpp, dtype, mode):
    for seed, (rows, cols, density) in enumerate([(1, 1, 1.0), (37, 53, 0.2), (700, 650, 0.02), (64, 64, 0.0)]):
        d, i, p, _ = G.random_csr(rows, cols, density, seed, dtype, empty_rows=rows > 1)
        x, g = randn(seed + 10, cols, dtype), randn(seed + 20, rows, dtype)
        D, I, P, X, Gz = to_dev(dev, d, i, p, x, g)
        y = cpp.spgemv_forward(rows, cols, D, I, P, X)
        assert_close(host(y), oracle.spgemv_forward(rows, cols, d, i, p, x), "y")
        assert_same(host(y), host(mirror.spgemv_forward(rows, cols, D, I, P, X)), "y vs ctypes binding")
        gA, gx = cpp.spgemv_backward(Gz, rows, cols, D, I, P, X)
        gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
        assert_same(host(gA), gA_ref, "grad_A")
        assert_close(host(gx), gx_ref, "grad_x")
        mA, mx = mirror.spgemv_backward(Gz, rows, cols, D, I, P, X)
        assert_same(host(gA), host(mA), "grad_A vs ctypes binding")
        if mode == "eager":
            assert_same(host(gx), host(mx), "grad_x vs ctypes binding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 7, 64])
def test_spdmm(dev, cpp, dtype, n, mode):
    rows, cols = 300, 280
    d, i, p, _ = G.random_csr(rows, cols, 0.05, 3, dtype)
    B, gC = randn(4, (cols, n), dtype), randn(5, (rows, n), dtype)
    D, I, P, Bt, Gt = to_dev(dev, d, i, p, B, gC)
    C = cpp.spdmm_forward(rows, cols, D, I, P, Bt)
    assert_same(host(C), oracle.spdmm_forward(rows, cols, d, i, p, B), "C")     # short rows: storage-order sums
    gA, gB = cpp.spdmm_backward(rows, cols, D, I, P, Bt, Gt)
    gA_ref, gB_ref = oracle.spdmm_backward(rows, cols, d, i, p, B, gC)
    assert_close(host(gA), gA_ref, "grad_A")
    assert_close(host(gB), gB_ref, "grad_B")
    mA, mB = mirror.spdmm_backward(rows, cols, D, I, P, Bt, Gt)
    assert_same(host(gA), host(mA), "grad_A vs ctypes binding")
    if mode == "eager":
        assert_same(host(gB), host(mB), "grad_B vs ctypes binding")
    # a column-major B and a row-sliced grad_C take the strided/copy paths
    Bf = Bt.t().contiguous().t()
    Gs = torch.cat([Gt, Gt], dim=1)[:, :n]
    assert_same(host(cpp.spdmm_forward(rows, cols, D, I, P, Bf)), host(C), "C from column-major B")
    sA, sB = cpp.spdmm_backward(rows, cols, D, I, P, Bf, Gs)
    assert_same(host(sA), host(gA), "grad_A from strided operands")
    if mode == "eager":
        assert_same(host(sB), host(gB), "grad_B from strided operands")


@pytest.mark.parametrize("dtype", DTYPES)
def test_spgemm(dev, cpp, dtype):
    for seed, (m, k, n, da, db) in enumerate([(40, 50, 45, 0.15, 0.15), (500, 400, 450, 0.03, 0.03), (8, 8, 8, 0.0, 0.3)]):
        ad, ai, ap, _ = G.random_csr(m, k, da, seed, dtype)
        bd, bi, bp, _ = G.random_csr(k, n, db, seed + 50, dtype)
        AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
        Cd, Ci, Cp = cpp.spgemm_forward(m, k, AD, AI, AP, k, n, BD, BI, BP)
        rd, ri, rp = oracle.spgemm_forward(m, k, ad, ai, ap, k, n, bd, bi, bp)
        assert_same(host(Cp), rp, "C_indptr")
        assert_same(host(Ci), ri, "C_indices")
        assert_same(host(Cd), rd, "C_data")
        g = randn(seed + 7, rd.shape[0], dtype)
        Gc, = to_dev(dev, g)
        gA, gB = cpp.spgemm_backward(Gc, Ci, Cp, m, k, AD, AI, AP, k, n, BD, BI, BP)
        gA_ref, gB_ref = oracle.spgemm_backward(g, ri, rp, m, k, ad, ai, ap, k, n, bd, bi, bp)
        assert_same(host(gA), gA_ref, "grad_A")
        assert_same(host(gB), gB_ref, "grad_B")     # on the plan: the serial order, no atomics
        cpp.set_backward_mode("atomic")
        gA, gB = cpp.spgemm_backward(Gc, Ci, Cp, m, k, AD, AI, AP, k, n, BD, BI, BP)
        cpp.set_backward_mode("eager")
        assert_same(host(gA), gA_ref, "grad_A (stateless)")
        assert_close(host(gB), gB_ref, "grad_B (stateless)")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lower", [True, False])
@pytest.mark.parametrize("unit", [False, True])
def test_sptrsv(dev, cpp, dtype, lower, unit):
    n = 400
    d, i, p, _ = G.random_tri(n, 0.02, 11, lower, dtype)
    b, g = randn(12, n, dtype), randn(13, n, dtype)
    D, I, P, Bt, Gt = to_dev(dev, d, i, p, b, g)
    x = cpp.sptrsv_forward(n, n, D, I, P, lower, unit, Bt)
    x_ref = oracle.sptrsv_forward(n, n, d, i, p, lower, unit, b)
    assert_close(host(x), x_ref, "x")
    assert_same(host(x), host(mirror.sptrsv_forward(n, n, D, I, P, lower, unit, Bt)), "x vs ctypes binding")
    gA, gb = cpp.sptrsv_backward(Gt, x, n, n, D, I, P, lower, unit, Bt)
    gA_ref, gb_ref = oracle.sptrsv_backward(g, host(x), n, n, d, i, p, lower, unit)
    assert_close(host(gb), gb_ref, "grad_b")
    assert_close(host(gA), gA_ref, "grad_A")


def test_plan_cache_and_errors(dev, cpp):
    d, i, p, (n, _) = G.poisson2d_lower(20, np.float64)
    D, I, P = to_dev(dev, d, i, p)
    b = to_dev(dev, randn(1, n, np.float64))[0]
    cpp.clear_plan_cache()
    assert cpp.plan_cache_size() == 0
    cpp.sptrsv_forward(n, n, D, I, P, True, False, b)
    cpp.sptrsv_forward(n, n, D, I, P, True, False, b)
    assert cpp.plan_cache_size() == 1
    cpp.sptrsv_backward(b, b, n, n, D, I, P, True, False, b)        # the transposed solve shares the plan
    assert cpp.plan_cache_size() == 1
    cpp.set_backward_mode("eager")
    cpp.spgemv_backward(b, n, n, D, I, P, b)
    assert cpp.plan_cache_size() == 2
    # an in-place edit of the structure must not reuse the stale schedule
    d2, i2, p2, _ = G.bidiag(n, np.float64)
    D2, I2, P2 = to_dev(dev, d2, i2, p2)
    I3 = I2.clone()
    x_a = cpp.sptrsv_forward(n, n, D2, I3, P2, True, False, b)
    I3[1] = 1                                                       # (1,0) -> (1,1): row 1 loses its dependency
    x_b = cpp.sptrsv_forward(n, n, D2, I3, P2, True, False, b)
    assert_same(host(x_b), oracle.sptrsv_forward(n, n, d2, host(I3), p2, True, False, host(b)), "after edit")
    assert not torch.equal(x_a, x_b)
    cpp.clear_plan_cache()

    with pytest.raises(RuntimeError, match="Long"):
        cpp.spgemv_forward(n, n, D, I.int(), P, b)
    with pytest.raises(RuntimeError, match="HIP devices only|same device"):
        cpp.spdmm_forward(n, n, D, I, P, torch.ones(n, 2, dtype=torch.float64))
    with pytest.raises(RuntimeError, match="float32 or float64"):
        cpp.spgemv_forward(n, n, D.half(), I, P, b.half())
    with pytest.raises(RuntimeError, match="planned"):
        cpp.set_backward_mode("fastest")


def test_plan_policy_second_sighting_content_key_and_byte_bound(dev, cpp):
    """Default mode: the first backward on a new pattern runs statelessly and builds nothing, the
    second builds the plan; the plan is found again through fresh tensors with the same content;
    the cache is bounded by bytes."""
    d, i, p, (rows, cols) = G.poisson2d(96, np.float64, 3)
    D, I, P = to_dev(dev, d, i, p)
    x, g = randn(4, cols, np.float64), randn(5, rows, np.float64)
    X, Gv = to_dev(dev, x, g)
    gA_ref, gx_ref = oracle.spgemv_backward(g, rows, cols, d, i, p, x)
    cpp.clear_plan_cache()
    cpp.set_backward_mode("planned")
    built0, keys0 = cpp.plan_cache_stats()
    gA, gx = cpp.spgemv_backward(Gv, rows, cols, D, I, P, X)             # first sighting: stateless
    assert cpp.plan_cache_size() == 0 and cpp.plan_cache_stats()[0] == built0
    assert_same(host(gA), gA_ref, "grad_A (stateless)")
    assert_close(host(gx), gx_ref, "grad_x (stateless)")
    gA, gx = cpp.spgemv_backward(Gv, rows, cols, D, I, P, X)             # second sighting: plan built
    assert cpp.plan_cache_size() == 1 and cpp.plan_cache_stats()[0] == built0 + 1
    assert_same(host(gx), gx_ref, "grad_x (planned, bitwise)")
    assert cpp.plan_cache_stats()[1] == keys0 + 1                         # one key for the one pair of tensors
    y_plain = oracle.spgemv_forward(rows, cols, d, i, p, x)
    assert_same(host(cpp.spgemv_forward(rows, cols, D, I, P, X)), y_plain, "y through the plan's 32-bit structure")
    # the same pattern in fresh tensors: a key is computed, the plan is found, nothing is built
    I2, P2 = I.clone(), P.clone()
    gA, gx = cpp.spgemv_backward(Gv, rows, cols, D, I2, P2, X)
    assert cpp.plan_cache_size() == 1 and cpp.plan_cache_stats() == (built0 + 1, keys0 + 2)
    assert_same(host(gx), gx_ref, "grad_x (plan found through the content key)")
    # a different pattern of the same sizes is not mistaken for it
    I3 = I.clone()
    I3[2] = I[2].item() + 1                      # row 0 holds columns (0, 1, 96): the last one moves to 97
    cpp.spgemv_backward(Gv, rows, cols, D, I3, P, X)
    assert cpp.plan_cache_size() == 1 and cpp.plan_cache_stats()[0] == built0 + 1   # first sighting of another pattern
    # byte bound: with a limit below one plan only the most recent plan stays
    one = cpp.plan_cache_bytes()
    assert one > 0
    cpp.set_plan_cache_limit(one // 2)
    cpp.set_backward_mode("eager")
    d4, i4, p4, (r4, c4) = G.poisson2d(64, np.float64, 1)
    D4, I4, P4 = to_dev(dev, d4, i4, p4)
    cpp.spgemv_backward(to_dev(dev, randn(1, r4, np.float64))[0], r4, c4, D4, I4, P4, to_dev(dev, randn(2, c4, np.float64))[0])
    assert cpp.plan_cache_size() == 1 and cpp.plan_cache_bytes() < one
    cpp.set_plan_cache_limit(4096 << 20)
    cpp.clear_plan_cache()


def test_loop_of_fresh_products_builds_one_plan_per_pattern(dev, cpp):
    """C = A @ A computed anew in every iteration arrives in new structure tensors each time; the
    backward of C @ x must find C's plan again instead of building one per iteration."""
    import time
    from numml_amd import sparse as sp
    d, i, p, (rows, cols) = G.poisson2d(256, np.float32, 0)
    D, I, P = to_dev(dev, d, i, p)
    A = sp.SparseCSRTensor((D, I, P), (rows, cols), clone=False)
    A.requires_grad = True
    X = to_dev(dev, randn(1, cols, np.float32))[0]
    cpp.clear_plan_cache()
    cpp.set_backward_mode("planned")
    built0 = cpp.plan_cache_stats()[0]
    times = []
    for it in range(10):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        C = A @ A
        (C @ X).sum().backward()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    # C's pattern for the SpMV backward, A's own for the product's backward, and the product plan of A A
    assert cpp.plan_cache_stats()[0] - built0 <= 3 and cpp.plan_cache_size() <= 3
    steady = sorted(times[3:])[len(times[3:]) // 2]
    assert max(times[3:]) <= 2.0 * steady, times
    cpp.clear_plan_cache()


def test_product_plan_policy(dev, cpp):
    """A product without hash-path rows: the first call runs the stateless kernels and builds
    nothing, the second builds the product plan around its own result, later calls run on the plan
    and hand out the plan's pattern tensors; values and gradients stay bit-identical to the oracle's
    for new values on the same patterns.  An in-place edit of a handed-out pattern tensor drops the
    plan; "atomic" never plans; a product beyond the plan's limits is remembered as such."""
    dtype = np.float64
    d, i, p, (n, _) = G.laplace3d(10, dtype, 2)
    I, P = to_dev(dev, i, p)

    def check(call, seed):
        a, b = randn(seed, d.shape[0], dtype), randn(seed + 1, d.shape[0], dtype)
        A, B = to_dev(dev, a, b)
        C_data, C_indices, C_indptr = cpp.spgemm_forward(n, n, A, I, P, n, n, B, I, P)
        cd, ci, cp = oracle.spgemm_forward(n, n, a, i, p, n, n, b, i, p)
        assert_same(host(C_indptr), cp, f"{call}: C_indptr")
        assert_same(host(C_indices), ci, f"{call}: C_indices")
        assert_same(host(C_data), cd, f"{call}: C_data")
        g = randn(seed + 2, cd.shape[0], dtype)
        gA, gB = cpp.spgemm_backward(to_dev(dev, g)[0], C_indices, C_indptr, n, n, A, I, P, n, n, B, I, P)
        rA, rB = oracle.spgemm_backward(g, ci, cp, n, n, a, i, p, n, n, b, i, p)
        assert_same(host(gA), rA, f"{call}: grad_A")
        return C_indices, C_indptr, host(gB), rB

    cpp.clear_plan_cache()
    cpp.set_backward_mode("planned")
    built0 = cpp.plan_cache_stats()[0]
    check("first call", 1)                                   # stateless forward; backward: first sighting of A
    assert cpp.plan_cache_stats()[0] == built0
    ci2, cp2, gB, rB = check("second call", 4)               # builds A's transposed plan and the product plan
    assert cpp.plan_cache_stats()[0] == built0 + 2 and cpp.plan_cache_size() == 2
    assert_same(gB, rB, "second call: grad_B (mapped, bitwise)")
    ci3, cp3, gB, rB = check("third call", 7)                # numeric kernel only, on the plan
    assert ci3.data_ptr() == ci2.data_ptr() and cp3.data_ptr() == cp2.data_ptr(), "the plan's pattern tensors"
    assert cpp.plan_cache_stats()[0] == built0 + 2
    assert_same(gB, rB, "third call: grad_B (mapped, bitwise)")
    # a gradient laid out on OTHER tensors of the same pattern takes the search-based kernels
    ci4, cp4 = ci3.clone(), cp3.clone()
    a, b = randn(20, d.shape[0], dtype), randn(21, d.shape[0], dtype)
    g = randn(22, ci4.shape[0], dtype)
    A, B = to_dev(dev, a, b)
    gA, gB = cpp.spgemm_backward(to_dev(dev, g)[0], ci4, cp4, n, n, A, I, P, n, n, B, I, P)
    rA, rB = oracle.spgemm_backward(g, host(ci4), host(cp4), n, n, a, i, p, n, n, b, i, p)
    assert_same(host(gA), rA, "grad_A on foreign pattern tensors")
    assert_same(host(gB), rB, "grad_B on foreign pattern tensors")
    # an in-place edit of a handed-out pattern tensor: the plan is dropped, results stay right
    ci3.add_(0)
    ci5, _, _, _ = check("after an in-place edit", 10)
    assert ci5.data_ptr() != ci3.data_ptr()
    # "atomic": no plan is looked for or built
    cpp.clear_plan_cache()
    cpp.set_backward_mode("atomic")
    for seed in (30, 33, 36):
        check("atomic mode", seed)
    assert cpp.plan_cache_size() == 0
    # "eager": the plan is built by the first call; the pattern in fresh tensors finds it
    cpp.set_backward_mode("eager")
    built1 = cpp.plan_cache_stats()[0]
    ci6, _, _, _ = check("eager, first call", 40)
    assert cpp.plan_cache_stats()[0] == built1 + 2
    I_saved, P_saved = I, P
    I, P = I.clone(), P.clone()
    ci7, _, gB, rB = check("eager, cloned patterns", 43)
    assert ci7.data_ptr() == ci6.data_ptr() and cpp.plan_cache_stats()[0] == built1 + 2
    assert_same(gB, rB, "grad_B through cloned patterns")
    I, P = I_saved, P_saved
    # a product with a row of nine entries has no hash-path row only if ... it has one: not eligible;
    # one whose rows of B are too long for the plan but short enough for the merge path does not exist
    # either (both limits are eight), so "unusable" arises from long columns of A only
    cpp.clear_plan_cache()
    rows = 5000
    ai = np.zeros(rows, dtype=np.int64)                      # every row of A names column 0
    ap = np.arange(rows + 1, dtype=np.int64)
    ad = randn(50, rows, dtype)
    bd, bi, bp, _ = G.ragged_csr(3, 40, 4, 51, dtype, min_len=2)
    AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
    for _ in range(3):
        C_data, C_indices, C_indptr = cpp.spgemm_forward(rows, 3, AD, AI, AP, 3, 40, BD, BI, BP)
        cd, ci, cp = oracle.spgemm_forward(rows, 3, ad, ai, ap, 3, 40, bd, bi, bp)
        assert_same(host(C_data), cd, "long column of A: C_data")
        assert_same(host(C_indices), ci, "long column of A: C_indices")
    assert cpp.plan_cache_stats()[0] == built1 + 2 + 2       # A's transposed plan and the (unusable) product plan, once
    cpp.set_backward_mode("planned")
    cpp.clear_plan_cache()


def test_default_mode_keeps_heavy_rows_of_the_right_operand_off_the_planned_backward(dev, cpp):
    """The plan-based backward gives a row of B to a group of lanes, a heavy one (its entries times
    the entries of A's column in the thousands) to one workgroup: where the AVERAGE row is that
    heavy the default mode stays with the stateless kernels, however often the pattern is seen;
    "eager" still takes the plan."""
    dtype = np.float32
    rows = 6000
    ai = (np.arange(rows) % 2).astype(np.int64)               # 3000 entries in each of A's two columns
    ap = np.arange(rows + 1, dtype=np.int64)
    ad = randn(80, rows, dtype)
    bd, bi, bp, _ = G.ragged_csr(2, 300, 40, 81, dtype, min_len=40)
    AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
    cd, ci, cp = oracle.spgemm_forward(rows, 2, ad, ai, ap, 2, 300, bd, bi, bp)
    g = randn(82, cd.shape[0], dtype)
    rA, rB = oracle.spgemm_backward(g, ci, cp, rows, 2, ad, ai, ap, 2, 300, bd, bi, bp)
    Gd, CI, CP = to_dev(dev, g, ci, cp)
    cpp.clear_plan_cache()
    try:
        cpp.set_backward_mode("planned")
        for _ in range(3):
            gA, gB = cpp.spgemm_backward(Gd, CI, CP, rows, 2, AD, AI, AP, 2, 300, BD, BI, BP)
            assert_same(host(gA), rA, "grad_A")
            assert_close(host(gB), rB, "grad_B (atomics)")
        assert cpp.plan_cache_size() == 0
        cpp.set_backward_mode("eager")
        gA, gB = cpp.spgemm_backward(Gd, CI, CP, rows, 2, AD, AI, AP, 2, 300, BD, BI, BP)
        assert cpp.plan_cache_size() == 1
        assert_same(host(gA), rA, "grad_A on the plan")
        assert_close(host(gB), rB, "grad_B on the plan (heavy rows: tree order)")
    finally:
        cpp.set_backward_mode("planned")
        cpp.clear_plan_cache()


def test_default_mode_judges_by_the_heaviest_rows_and_columns_not_by_means(dev, cpp):
    """Means hide a few heavy rows or columns among many light ones.  (a) SpGEMM backward: two rows
    of B with 512 entries, named by two columns of A with 2000 entries, in matrices that are
    diagonal otherwise: every mean is about one, yet the plan-based kernel would hand each heavy
    row (a million products) to a single workgroup.  (b) SpMM backward: a matrix with one dense
    column; the kernels on the plan take a column of more than 512 entries serially.  The default
    mode takes the stateless kernels for both however often it sees the pattern; "eager" takes the
    plans; both match the oracle."""
    import scipy.sparse as sps
    dtype = np.float64
    rng = np.random.default_rng(90)
    n = 1_000_000

    def csr(m):
        m = m.tocsr()
        m.sum_duplicates()
        m.sort_indices()
        return m.data.astype(dtype), m.indices.astype(np.int64), m.indptr.astype(np.int64)

    # ---- (a)
    heavy = (1000, 300_000)
    ar = np.concatenate([np.arange(n)] + [rng.choice(n, 2000, replace=False) for _ in heavy])
    ac = np.concatenate([np.arange(n)] + [np.full(2000, k) for k in heavy])
    A = csr(sps.coo_matrix((rng.standard_normal(ar.size), (ar, ac)), shape=(n, n)))
    br = np.concatenate([np.arange(n)] + [np.full(512, k) for k in heavy])
    bc = np.concatenate([np.arange(n)] + [rng.choice(n, 512, replace=False) for _ in heavy])
    B = csr(sps.coo_matrix((rng.standard_normal(br.size), (br, bc)), shape=(n, n)))
    cd, ci, cp = oracle.spgemm_forward(n, n, *A, n, n, *B)
    assert cd.shape[0] / n <= 4 * B[0].shape[0] / n          # the means would let the plan through
    g = randn(91, cd.shape[0], dtype)
    rA, rB = oracle.spgemm_backward(g, ci, cp, n, n, *A, n, n, *B)
    dA, dB = to_dev(dev, *A), to_dev(dev, *B)
    Gd, CI, CP = to_dev(dev, g, ci, cp)
    cpp.clear_plan_cache()
    try:
        cpp.set_backward_mode("planned")
        for _ in range(3):
            gA, gB = cpp.spgemm_backward(Gd, CI, CP, n, n, *dA, n, n, *dB)
            assert cpp.last_backward_paths()[1] == "stateless"
            assert_same(host(gA), rA, "grad_A")
            assert_close(host(gB), rB, "grad_B (atomics)")
        cpp.set_backward_mode("eager")
        gA, gB = cpp.spgemm_backward(Gd, CI, CP, n, n, *dA, n, n, *dB)
        assert cpp.last_backward_paths()[1] == "transposed plan"
        assert_same(host(gA), rA, "grad_A on the plan")
        assert_close(host(gB), rB, "grad_B on the plan")
        # ---- (b)
        n = 60_000
        mr = np.concatenate([np.arange(n), np.arange(1, 30_001)])
        mc = np.concatenate([np.arange(n), np.zeros(30_000, dtype=np.int64)])
        M = csr(sps.coo_matrix((rng.standard_normal(mr.size), (mr, mc)), shape=(n, n)))
        band = csr(sps.diags([rng.standard_normal(n - 1), rng.standard_normal(n), rng.standard_normal(n - 1)], [-1, 0, 1]))
        Bd, Gc = randn(92, (n, 40), dtype), randn(93, (n, 40), dtype)
        dM, dBand = to_dev(dev, *M), to_dev(dev, *band)
        dBd, dGc = to_dev(dev, Bd, Gc)
        for mat, dmat, want in ((M, dM, "stateless"), (band, dBand, "transposed plan")):
            ref = oracle.spdmm_backward(n, n, *mat, Bd, Gc)
            cpp.set_backward_mode("planned")
            cpp.clear_plan_cache()
            for call in range(3):
                gA, gB = cpp.spdmm_backward(n, n, *dmat, dBd, dGc)
                if call:                                    # (the first sighting is stateless for every pattern)
                    assert cpp.last_backward_paths()[0] == want
                assert_close(host(gA), ref[0], "spdmm grad_A")
                assert_close(host(gB), ref[1], "spdmm grad_B")
            cpp.set_backward_mode("eager")
            gA, gB = cpp.spdmm_backward(n, n, *dmat, dBd, dGc)
            assert cpp.last_backward_paths()[0] == "transposed plan"
            assert_close(host(gA), ref[0], "spdmm grad_A on the plan")
            assert_close(host(gB), ref[1], "spdmm grad_B on the plan")
        info = cpp.transpose_plan_info(n, n, dM[1], dM[2])
        assert info[7] == 30_001 and info[9] == 30_001       # longest column; entries of long columns in its group
    finally:
        cpp.set_backward_mode("planned")
        cpp.clear_plan_cache()


def test_product_plan_for_rows_of_the_right_operand_of_up_to_32_entries(dev, cpp):
    """A (A A) on a 3D grid -- the right operand has 25-entry rows, so the product takes the hash path --
    in a loop with new values: the first call is stateless, the second leaves a product plan with four
    destination octets per entry behind, later calls run the numeric kernel and both gradients on it;
    every call gives the oracle's bits."""
    dtype = np.float64
    d, i, p, (n, _) = G.laplace3d(9, dtype, 3)
    D, I, P = to_dev(dev, d, i, p)
    Sd, SI, SP = cpp.spgemm_forward(n, n, D, I, P, n, n, D, I, P)
    si, sp = host(SI), host(SP)
    cpp.clear_plan_cache()
    cpp.set_backward_mode("planned")
    try:
        built0 = cpp.plan_cache_stats()[0]
        shared = None
        for call in range(4):
            a, b = randn(60 + call, d.shape[0], dtype), randn(70 + call, si.shape[0], dtype)
            A, B = to_dev(dev, a, b)
            C_data, C_indices, C_indptr = cpp.spgemm_forward(n, n, A, I, P, n, n, B, SI, SP)
            cd, ci, cp = oracle.spgemm_forward(n, n, a, i, p, n, n, b, si, sp)
            assert_same(host(C_indptr), cp, f"call {call}: C_indptr")
            assert_same(host(C_indices), ci, f"call {call}: C_indices")
            assert_same(host(C_data), cd, f"call {call}: C_data")
            g = randn(80 + call, cd.shape[0], dtype)
            gA, gB = cpp.spgemm_backward(to_dev(dev, g)[0], C_indices, C_indptr, n, n, A, I, P, n, n, B, SI, SP)
            rA, rB = oracle.spgemm_backward(g, ci, cp, n, n, a, i, p, n, n, b, si, sp)
            assert_same(host(gA), rA, f"call {call}: grad_A")
            if call >= 1:                   # on the plan: rows ascending, the serial order
                assert_same(host(gB), rB, f"call {call}: grad_B")
            if call >= 2:
                if shared is not None:
                    assert C_indices.data_ptr() == shared, "the plan's pattern tensors"
                shared = C_indices.data_ptr()
        assert cpp.plan_cache_stats()[0] == built0 + 2      # A's transposed plan and the product plan
    finally:
        cpp.set_backward_mode("planned")
        cpp.clear_plan_cache()


def test_install_registers_the_reference_module_name(cpp):
    import sys
    saved = sys.modules.pop("numml_torch_cpp", None)
    try:
        numml_amd.install()
        import numml_torch_cpp
        assert numml_torch_cpp is cpp
    finally:
        sys.modules.pop("numml_torch_cpp", None)
        if saved is not None:
            sys.modules["numml_torch_cpp"] = saved


@pytest.mark.parametrize("hint", ["given", "unknown", "landing for the first call only",
                                  "landing for the second call only"])
def test_spgemm_through_the_c_abi_with_and_without_the_hash_row_count(dev, hint):
    """The numeric phase takes the number of hash-path rows that nm_spgemm_symbolic_result reports
    (0 lets it leave the hash launches out), or -1 from a caller that read nnz(C) itself.  With a
    landing place nm_spgemm_symbolic has the numbers landed itself where no row needs the hash
    path, and the result call after it only reads them; a caller may also give the landing place
    to one of the two calls only."""
    import ctypes
    from numml_amd import _lib
    L = _lib.lib()
    for name, (d, i, p, (r, c)) in (("stencil: no row on the hash path", G.poisson2d(40, np.float64, 1)),
                                    ("random: rows on both paths", G.random_csr(500, 500, 0.03, 2, np.float64))):
        D, I, P = to_dev(dev, d, i, p)
        ptr = lambda t: ctypes.c_void_p(t.data_ptr())
        st = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
        nbytes = ctypes.c_size_t(0)
        _lib.check(L.nm_spgemm_workspace_bytes(r, c, ctypes.byref(nbytes)), "bytes")
        work = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
        Cp = torch.empty(r + 1, dtype=torch.int64, device=dev)
        # with a pinned landing place for the device to write into (hint "given"), and without one
        landing = torch.zeros(4, dtype=torch.int64).pin_memory() if hint != "unknown" else None
        first = landing if hint in ("given", "landing for the first call only") else None
        second = landing if hint in ("given", "landing for the second call only") else None
        _lib.check(L.nm_spgemm_symbolic(r, c, c, ptr(I), ptr(P), ptr(I), ptr(P), ptr(Cp), ptr(work), nbytes.value,
                                        ptr(first) if first is not None else None, st), "symbolic")
        nnz_c, hash_rows = ctypes.c_int64(-7), ctypes.c_int64(-7)
        _lib.check(L.nm_spgemm_symbolic_result(r, c, ptr(work), nbytes.value, ctypes.byref(nnz_c), ctypes.byref(hash_rows),
                                               ptr(second) if second is not None else None, st), "result")
        if hint == "given":
            # the note that the numbers had landed is taken back by the call that read them
            assert int(landing[3]) == 0, name
        Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(r, c, d, i, p, r, c, d, i, p)
        assert nnz_c.value == Cd_ref.shape[0] == int(Cp[-1].item()), name
        assert (hash_rows.value == 0) == name.startswith("stencil"), (name, hash_rows.value)
        Ci = torch.empty(nnz_c.value, dtype=torch.int64, device=dev)
        Cd = torch.empty(nnz_c.value, dtype=torch.float64, device=dev)
        _lib.check(L.nm_spgemm_numeric(1, r, c, c, ptr(D), ptr(I), ptr(P), ptr(D), ptr(I), ptr(P), ptr(Cp), ptr(Ci), ptr(Cd),
                                       ptr(work), nbytes.value, hash_rows.value if hint == "given" else -1, st), "numeric")
        assert_same(host(Cp), Cp_ref, f"{name} C_indptr")
        assert_same(host(Ci), Ci_ref, f"{name} C_indices")
        assert_same(host(Cd), Cd_ref, f"{name} C_data")


@pytest.mark.parametrize("landing_given", [True, False])
def test_spgemm_row_pointer_of_more_rows_than_the_tile_sums_are_added_up_in_place_for(dev, landing_given):
    """Past 4096 tiles of 2048 rows the sums of the tiles are scanned by a launch of their own
    before the row pointer is written, and the first workgroup reads nnz(C) behind them.  A
    product of two diagonal matrices of 9 000 000 rows has a closed form: the row pointer counts
    up by one, the columns are the rows, the values the products of the diagonals."""
    import ctypes
    from numml_amd import _lib
    L = _lib.lib()
    n = 9_000_000
    D = torch.arange(1, n + 1, dtype=torch.float64, device=dev) * 0.5
    I = torch.arange(n, dtype=torch.int64, device=dev)
    P = torch.arange(n + 1, dtype=torch.int64, device=dev)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    nbytes = ctypes.c_size_t(0)
    _lib.check(L.nm_spgemm_workspace_bytes(n, n, ctypes.byref(nbytes)), "bytes")
    work = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
    Cp = torch.full((n + 1,), -1, dtype=torch.int64, device=dev)
    landing = torch.zeros(4, dtype=torch.int64).pin_memory() if landing_given else None
    where = ptr(landing) if landing_given else None
    _lib.check(L.nm_spgemm_symbolic(n, n, n, ptr(I), ptr(P), ptr(I), ptr(P), ptr(Cp), ptr(work), nbytes.value,
                                    where, st), "symbolic")
    nnz_c, hash_rows = ctypes.c_int64(-7), ctypes.c_int64(-7)
    _lib.check(L.nm_spgemm_symbolic_result(n, n, ptr(work), nbytes.value, ctypes.byref(nnz_c), ctypes.byref(hash_rows),
                                           where, st), "result")
    assert (nnz_c.value, hash_rows.value) == (n, 0)
    assert torch.equal(Cp, P)
    Ci = torch.empty(n, dtype=torch.int64, device=dev)
    Cd = torch.empty(n, dtype=torch.float64, device=dev)
    _lib.check(L.nm_spgemm_numeric(1, n, n, n, ptr(D), ptr(I), ptr(P), ptr(D), ptr(I), ptr(P), ptr(Cp), ptr(Ci), ptr(Cd),
                                   ptr(work), nbytes.value, hash_rows.value, st), "numeric")
    assert torch.equal(Ci, I)
    assert torch.equal(Cd, D * D)


@pytest.mark.parametrize("rows", [1, 2047, 2048, 4095, 4096, 6143, 10_000])
def test_spgemm_row_pointer_at_tile_boundaries_and_in_unaligned_memory(dev, rows):
    """The row pointer is written 16 bytes at a time where a tile of 2048 of its entries is whole and
    the arrays allow it, entry by entry otherwise: row counts around the tile size, into a row
    pointer that starts 8 bytes off a 16-byte boundary, against the oracle."""
    import ctypes
    from numml_amd import _lib
    L = _lib.lib()
    d, i, p, (r, c) = G.tridiag(rows, np.float64)
    D, I, P = to_dev(dev, d, i, p)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    st = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    nbytes = ctypes.c_size_t(0)
    _lib.check(L.nm_spgemm_workspace_bytes(r, c, ctypes.byref(nbytes)), "bytes")
    Cd_ref, Ci_ref, Cp_ref = oracle.spgemm_forward(r, c, d, i, p, r, c, d, i, p)
    landing = torch.zeros(4, dtype=torch.int64).pin_memory()
    for shift in (0, 1):
        work = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
        room = torch.full((r + 2,), -1, dtype=torch.int64, device=dev)
        Cp = room[shift:shift + r + 1]
        assert Cp.data_ptr() % 16 == 8 * shift
        _lib.check(L.nm_spgemm_symbolic(r, c, c, ptr(I), ptr(P), ptr(I), ptr(P), ptr(Cp), ptr(work), nbytes.value,
                                        ptr(landing), st), "symbolic")
        nnz_c, hash_rows = ctypes.c_int64(-7), ctypes.c_int64(-7)
        _lib.check(L.nm_spgemm_symbolic_result(r, c, ptr(work), nbytes.value, ctypes.byref(nnz_c),
                                               ctypes.byref(hash_rows), ptr(landing), st), "result")
        assert (nnz_c.value, hash_rows.value) == (Cd_ref.shape[0], 0), (rows, shift)
        assert_same(host(Cp), Cp_ref, f"{rows} rows, shift {shift}: C_indptr")
        if shift:   # the entry before the row pointer is nobody's
            assert int(room[0].item()) == -1
        else:
            assert int(room[r + 1].item()) == -1


@pytest.mark.parametrize("dtype", DTYPES)
def test_spgemm_forward_with_plans_switched_off(dev, cpp, dtype):
    """In the stateless mode the forward still adds the products up on the records of its own
    symbolic merge where every row is short, but leaves out what only a plan made of those records
    would read (keep_plan == 0): the same bits as the oracle's, twice in a row, and nothing is kept."""
    cpp.set_backward_mode("atomic")
    try:
        for name, (ad, ai, ap, (m, k)), (bd, bi, bp, (k2, n)) in (
                ("stencil", G.poisson2d(37, dtype, 3), G.poisson2d(37, dtype, 4)),
                ("tridiagonal, 5000 rows", G.tridiag(5000, dtype), G.tridiag(5000, dtype, 1.0, -2.0, 1.0)),
                ("random: rows on both paths", G.random_csr(400, 300, 0.03, 5, dtype),
                 G.random_csr(300, 500, 0.03, 6, dtype))):
            cpp.clear_plan_cache()
            AD, AI, AP, BD, BI, BP = to_dev(dev, ad, ai, ap, bd, bi, bp)
            rd, ri, rp = oracle.spgemm_forward(m, k, ad, ai, ap, k2, n, bd, bi, bp)
            for call in range(2):
                Cd, Ci, Cp = cpp.spgemm_forward(m, k, AD, AI, AP, k2, n, BD, BI, BP)
                assert_same(host(Cp), rp, f"{name}, call {call}: C_indptr")
                assert_same(host(Ci), ri, f"{name}, call {call}: C_indices")
                assert_same(host(Cd), rd, f"{name}, call {call}: C_data")
            assert cpp.plan_cache_size() == 0, name
    finally:
        cpp.set_backward_mode("eager")
