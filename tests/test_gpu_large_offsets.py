"""More than 2^31 stored entries: offsets into the entry arrays do not fit 32 bits.  Values are small
integers, so every sum is exact in fp32 whatever the order, and the expected results come from
dense-block arithmetic on regular patterns (SpMV, SpMM: row r holds columns 8 j + r % 8,
j = 0 .. 1023)."""
import pytest
import torch

import numml_amd
from numml_amd import numml_torch_cpp as mirror

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("binding", ["ctypes", "compiled"])
def test_spmv_and_spmm_with_more_than_2_31_entries(dev, binding):
    """The transposed-structure plan stops at 2^31 - 2 entries: both bindings must take the stateless
    kernels for the gradients here (the tests run in the mode that plans at first sight)."""
    ext = mirror if binding == "ctypes" else numml_amd.load_compiled()
    per_row, cols = 1024, 8192
    rows = (1 << 21) + 3
    nnz = rows * per_row
    assert nnz > (1 << 31)
    P = torch.arange(rows + 1, device=dev, dtype=torch.int64) * per_row
    I = torch.empty(nnz, device=dev, dtype=torch.int64)
    D = torch.empty(nnz, device=dev, dtype=torch.float32)
    j = torch.arange(per_row, device=dev, dtype=torch.int64)
    step = 1 << 18
    for r0 in range(0, rows, step):
        r = torch.arange(r0, min(r0 + step, rows), device=dev, dtype=torch.int64)[:, None]
        I[r0 * per_row:(r0 + r.shape[0]) * per_row] = (8 * j[None, :] + r % 8).reshape(-1)
        D[r0 * per_row:(r0 + r.shape[0]) * per_row] = (((r + 3 * j[None, :]) % 5) - 2).to(torch.float32).reshape(-1)
    x = ((torch.arange(cols, device=dev) % 7) - 3).to(torch.float32)
    g = ((torch.arange(rows, device=dev) % 3) - 1).to(torch.float32)
    torch.cuda.synchronize()
    y = ext.spgemv_forward(rows, cols, D, I, P, x)
    torch.cuda.synchronize()
    gA, gx = ext.spgemv_backward(g, rows, cols, D, I, P, x)
    torch.cuda.synchronize()
    gx_ref = torch.zeros(per_row, 8, device=dev, dtype=torch.float32)
    for r0 in range(0, rows, step):       # step is a multiple of 8: row r0 + t has r % 8 == t % 8
        n = min(step, rows - r0)
        sl = slice(r0 * per_row, (r0 + n) * per_row)
        d2, i2 = D[sl].view(n, per_row), I[sl].view(n, per_row)
        xs = x[i2]
        assert torch.equal(y[r0:r0 + n], (d2 * xs).sum(1)), f"y, rows from {r0}"
        assert torch.equal(gA[sl].view(n, per_row), g[r0:r0 + n, None] * xs), f"grad_A, rows from {r0}"
        w = g[r0:r0 + n, None] * d2
        for m in range(8):
            gx_ref[:, m] += w[m::8].sum(0)
    assert torch.equal(gx, gx_ref.reshape(-1)), "grad_x"
    # the same matrix times a dense operand of 8 columns
    n = 8
    B = ((torch.arange(cols * n, device=dev) % 5) - 2).to(torch.float32).view(cols, n)
    gC = ((torch.arange(rows * n, device=dev) % 3) - 1).to(torch.float32).view(rows, n)
    C = ext.spdmm_forward(rows, cols, D, I, P, B)
    gA, gB = ext.spdmm_backward(rows, cols, D, I, P, B, gC)
    torch.cuda.synchronize()
    gB_ref = torch.zeros(per_row, 8, n, device=dev, dtype=torch.float32)
    small = 1 << 15
    for r0 in range(0, rows, small):
        m_rows = min(small, rows - r0)
        sl = slice(r0 * per_row, (r0 + m_rows) * per_row)
        d2, i2 = D[sl].view(m_rows, per_row), I[sl].view(m_rows, per_row)
        Bs = B[i2]                                               # m_rows x per_row x n
        assert torch.equal(C[r0:r0 + m_rows], (d2[:, :, None] * Bs).sum(1)), f"C, rows from {r0}"
        assert torch.equal(gA[sl].view(m_rows, per_row), (gC[r0:r0 + m_rows, None, :] * Bs).sum(2)), f"grad_A, rows from {r0}"
        for m in range(8):
            gB_ref[:, m] += d2[m::8].t() @ gC[r0:r0 + m_rows][m::8]
    assert torch.equal(gB, gB_ref.reshape(cols, n)), "grad_B"


@pytest.mark.parametrize("binding", ["ctypes", "compiled"])
def test_product_with_more_than_2_31_entries(dev, binding):
    """A (2 entries per row) times B (4096 rows of 512 entries): rows of C of 1024 entries, 2^31 + 3072
    in all.  Row r of A names rows c and c + 8 of B, c % 16 < 8, whose columns 16 j + c % 16 interleave,
    so entry 2 j of a row of C comes from the first and entry 2 j + 1 from the second; small integer
    values keep every sum exact."""
    ext = mirror if binding == "ctypes" else numml_amd.load_compiled()
    rows, k, half, cols = (1 << 21) + 3, 4096, 512, 8192
    r = torch.arange(rows, device=dev, dtype=torch.int64)
    c0 = 16 * ((r // 8) % 256) + r % 8
    AI = torch.stack([c0, c0 + 8], 1).reshape(-1)
    AP = torch.arange(rows + 1, device=dev, dtype=torch.int64) * 2
    AD = (((torch.arange(2 * rows, device=dev) * 7) % 5) - 2).to(torch.float32)
    c = torch.arange(k, device=dev, dtype=torch.int64)[:, None]
    j = torch.arange(half, device=dev, dtype=torch.int64)[None, :]
    BI = (16 * j + c % 16).reshape(-1)
    BP = torch.arange(k + 1, device=dev, dtype=torch.int64) * half
    BD = (((c * 3 + j) % 7) - 3).to(torch.float32).reshape(-1)
    CD, CI, CP = ext.spgemm_forward(rows, k, AD, AI, AP, k, cols, BD, BI, BP)
    torch.cuda.synchronize()
    nnz = rows * 2 * half
    assert nnz > (1 << 31) and CD.numel() == nnz and CI.numel() == nnz
    assert torch.equal(CP, torch.arange(rows + 1, device=dev, dtype=torch.int64) * (2 * half))
    B2 = BD.view(k, half)
    a0, a1 = AD[0::2], AD[1::2]
    jj = torch.arange(2 * half, device=dev, dtype=torch.int64)[None, :]
    step = 1 << 17
    for r0 in range(0, rows, step):
        n = min(step, rows - r0)
        sl = slice(r0 * 2 * half, (r0 + n) * 2 * half)
        m = c0[r0:r0 + n]
        assert torch.equal(CI[sl].view(n, 2 * half), 8 * jj + (m % 8)[:, None]), f"C_indices, rows from {r0}"
        want = torch.stack([a0[r0:r0 + n, None] * B2[m], a1[r0:r0 + n, None] * B2[8 + m]], 2).reshape(n, 2 * half)
        assert torch.equal(CD[sl].view(n, 2 * half), want), f"C_data, rows from {r0}"
    gC = (((torch.arange(nnz, device=dev) % 11) % 3) - 1).to(torch.float32)
    gA, gB = ext.spgemm_backward(gC, CI, CP, rows, k, AD, AI, AP, k, cols, BD, BI, BP)
    torch.cuda.synchronize()
    gB_ref = torch.zeros(k, half, device=dev, dtype=torch.float32)
    for r0 in range(0, rows, step):
        n = min(step, rows - r0)
        g2 = gC[r0 * 2 * half:(r0 + n) * 2 * half].view(n, half, 2)
        m = c0[r0:r0 + n]
        gA_want = torch.stack([(g2[:, :, 0] * B2[m]).sum(1), (g2[:, :, 1] * B2[8 + m]).sum(1)], 1).reshape(-1)
        assert torch.equal(gA[2 * r0:2 * (r0 + n)], gA_want), f"grad_A, rows from {r0}"
        w0, w1 = a0[r0:r0 + n, None] * g2[:, :, 0], a1[r0:r0 + n, None] * g2[:, :, 1]
        gB_ref.index_add_(0, m, w0)
        gB_ref.index_add_(0, m + 8, w1)
    assert torch.equal(gB, gB_ref.reshape(-1)), "grad_B"
