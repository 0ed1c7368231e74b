"""More than 2^31 stored entries: offsets into the entry arrays do not fit 32 bits.  Values are small
integers, so every sum is exact in fp32 whatever the order, and the expected results come from
dense-block arithmetic on the regular pattern (row r holds columns 8 j + r % 8, j = 0 .. 1023)."""
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
