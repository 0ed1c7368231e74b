"""Stream and graph behaviour: the entry points enqueue on the caller's stream, do
not synchronise once a pattern's plan exists, and can be captured into a HIP graph
and replayed with new values in the same buffers."""
import numpy as np
import pytest
import torch

import oracle
from numml_amd import generators as G
from numml_amd._binding import ops
from util import assert_close, assert_same, host, randn, to_dev

pytestmark = pytest.mark.gpu


def test_spmv_forward_backward_in_a_graph(dev):
    d, i, p, (rows, cols) = G.poisson2d(64, np.float32, 1)
    D, I, P = to_dev(dev, d, i, p)
    X, Gy = to_dev(dev, randn(1, cols, np.float32), randn(2, rows, np.float32))
    # warm-up on a side stream: builds and caches the transposed-structure plan (that build synchronises)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            ops.spgemv_forward(rows, cols, D, I, P, X)
            ops.spgemv_backward(Gy, rows, cols, D, I, P, X)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = ops.spgemv_forward(rows, cols, D, I, P, X)
        gA, gx = ops.spgemv_backward(Gy, rows, cols, D, I, P, X)
    for seed in (3, 4, 5):          # replays with new values, eager work and syncs in between
        x_h, g_h, d_h = randn(seed, cols, np.float32), randn(seed + 10, rows, np.float32), randn(seed + 20, d.shape[0], np.float32)
        X.copy_(torch.from_numpy(x_h))
        Gy.copy_(torch.from_numpy(g_h))
        D.copy_(torch.from_numpy(d_h))
        graph.replay()
        torch.cuda.synchronize()
        assert_same(host(y), oracle.spgemv_forward(rows, cols, d_h, i, p, x_h), "replayed y")
        gA_ref, gx_ref = oracle.spgemv_backward(g_h, rows, cols, d_h, i, p, x_h)
        assert_same(host(gA), gA_ref, "replayed grad_A")
        assert_same(host(gx), gx_ref, "replayed grad_x")
        eager = ops.spgemv_forward(rows, cols, D, I, P, X)
        assert torch.equal(eager, y)


def test_triangular_solve_in_a_graph_and_on_a_side_stream(dev):
    d, i, p, (n, _) = G.poisson2d_lower(40, np.float64, diag_seed=0)
    D, I, P = to_dev(dev, d, i, p)
    B = to_dev(dev, randn(1, n, np.float64))[0]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        x_side = ops.sptrsv_forward(n, n, D, I, P, True, False, B)      # analysis happens here, once
    torch.cuda.current_stream().wait_stream(side)
    assert_same(host(x_side), oracle.sptrsv_forward(n, n, d, i, p, True, False, host(B)), "solve on a side stream")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        x = ops.sptrsv_forward(n, n, D, I, P, True, False, B)
    for seed in (2, 3):
        b_h = randn(seed, n, np.float64)
        B.copy_(torch.from_numpy(b_h))
        graph.replay()
        torch.cuda.synchronize()
        assert_same(host(x), oracle.sptrsv_forward(n, n, d, i, p, True, False, b_h), "replayed solve")


def test_sparse_product_on_its_plan_in_a_graph(dev):
    """Once a pair of patterns has its product plan, the forward is one kernel and the backward
    two, none of which allocates outside torch's allocator, waits or clears memory: they can be
    captured and replayed with new values in the same buffers."""
    d, i, p, (n, _) = G.laplace3d(8, np.float64, 1)
    D, I, P = to_dev(dev, d, i, p)
    E = to_dev(dev, randn(1, d.shape[0], np.float64))[0]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                      # builds the plans (the suite runs in "eager" mode)
        C0 = ops.spgemm_forward(n, n, D, I, P, n, n, E, I, P)
        Gc = torch.zeros_like(C0[0])
        ops.spgemm_backward(Gc, C0[1], C0[2], n, n, D, I, P, n, n, E, I, P)
    torch.cuda.current_stream().wait_stream(side)
    built = ops.plan_cache_stats()[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        Cd, Ci, Cp = ops.spgemm_forward(n, n, D, I, P, n, n, E, I, P)
        gA, gB = ops.spgemm_backward(Gc, Ci, Cp, n, n, D, I, P, n, n, E, I, P)
    assert ops.plan_cache_stats()[0] == built, "nothing is analysed during capture"
    assert Ci.data_ptr() == C0[1].data_ptr()
    ci, cp = host(Ci), host(Cp)
    for seed in (3, 4, 5):          # replays with new values, eager work and syncs in between
        a_h, b_h, g_h = randn(seed, d.shape[0], np.float64), randn(seed + 10, d.shape[0], np.float64), randn(seed + 20, ci.shape[0], np.float64)
        D.copy_(torch.from_numpy(a_h))
        E.copy_(torch.from_numpy(b_h))
        Gc.copy_(torch.from_numpy(g_h))
        graph.replay()
        torch.cuda.synchronize()
        cd_ref, ci_ref, cp_ref = oracle.spgemm_forward(n, n, a_h, i, p, n, n, b_h, i, p)
        assert_same(ci, ci_ref, "pattern")
        assert_same(host(Cd), cd_ref, "replayed C_data")
        gA_ref, gB_ref = oracle.spgemm_backward(g_h, ci_ref, cp_ref, n, n, a_h, i, p, n, n, b_h, i, p)
        assert_same(host(gA), gA_ref, "replayed grad_A")
        assert_same(host(gB), gB_ref, "replayed grad_B")
        eager = ops.spgemm_forward(n, n, D, I, P, n, n, E, I, P)
        assert torch.equal(eager[0], Cd)
