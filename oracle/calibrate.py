"""Times the compiled reference (oracle/_ref) next to the restatement (oracle) on the same inputs.

TEST INFRASTRUCTURE ONLY: relates the CPU baseline that bench.py reports (the restatement, the
only thing that travels to the GPU box) to the reference's own CPU code.  Needs oracle/_ref, i.e.
the reference tree; run as ``python -m oracle.calibrate`` from the repository root.  One core.
Sizes are the benchmark configurations scaled down so that the reference's slow loops
(std::map in the SpGEMM backward, cpp/sparse_csr_cpu.cpp:283; per-element tensor indexing in the
transpose, :335-337) finish in seconds.
"""
import sys
import time

import numpy as np

import oracle
from numml_amd import generators as G
from oracle import ref


def best(f, reps):
    t = []
    for _ in range(reps):
        t0 = time.perf_counter()
        f()
        t.append(time.perf_counter() - t0)
    return min(t)


def row(name, f_ref, f_own, reps=3):
    a, b = best(f_ref, reps), best(f_own, reps)
    print(f"| {name} | {a * 1e3:.2f} ms | {b * 1e3:.2f} ms | {a / b:.2f} |", flush=True)


def main():
    if not ref.available():
        sys.exit("oracle/_ref is not built (make -C oracle ref, needs the reference tree)")
    import torch
    torch.set_num_threads(1)
    rng = np.random.default_rng(0)
    print("| case | reference C++ | restatement | reference / restatement |\n|---|---|---|---|")
    for label, n, dt in (("cfg1 SpMV Poisson 256^2 fp64", 256, np.float64), ("cfg2/16 SpMV Poisson 512^2 fp32", 512, np.float32)):
        d, i, p, (r, c) = G.poisson2d(n, dt, jitter_seed=0)
        x, g = rng.standard_normal(c).astype(dt), rng.standard_normal(r).astype(dt)
        row(label + " fwd", lambda: ref.call("spgemv_forward", r, c, d, i, p, x), lambda: oracle.spgemv_forward(r, c, d, i, p, x), 5)
        row(label + " bwd", lambda: ref.call("spgemv_backward", g, r, c, d, i, p, x), lambda: oracle.spgemv_backward(g, r, c, d, i, p, x), 5)
    r = c = 100_000
    d, i, p, _ = G.powerlaw(r, c, target_nnz=1_600_000, seed=0, dtype=np.float32)
    B, gC = rng.standard_normal((c, 64)).astype(np.float32), rng.standard_normal((r, 64)).astype(np.float32)
    row("cfg3/10 SpMM power-law 100k rows, n=64, fp32 fwd", lambda: ref.call("spdmm_forward", r, c, d, i, p, B), lambda: oracle.spdmm_forward(r, c, d, i, p, B), 1)
    row("cfg3/10 SpMM bwd", lambda: ref.call("spdmm_backward", r, c, d, i, p, B, gC), lambda: oracle.spdmm_backward(r, c, d, i, p, B, gC), 1)
    d, i, p, (r, c) = G.laplace3d(32, np.float64, jitter_seed=0)
    C = oracle.spgemm_forward(r, c, d, i, p, r, c, d, i, p)
    g = rng.standard_normal(C[0].shape[0])
    row("cfg4/64 SpGEMM Laplace 32^3 fp64 fwd", lambda: ref.call("spgemm_forward", r, c, d, i, p, r, c, d, i, p), lambda: oracle.spgemm_forward(r, c, d, i, p, r, c, d, i, p))
    row("cfg4/64 SpGEMM bwd", lambda: ref.call("spgemm_backward", g, C[1], C[2], r, c, d, i, p, r, c, d, i, p),
        lambda: oracle.spgemm_backward(g, C[1], C[2], r, c, d, i, p, r, c, d, i, p), 1)
    d, i, p, (n, _) = G.poisson2d_lower(256, np.float64, diag_seed=0)
    b, g = rng.standard_normal(n), rng.standard_normal(n)
    x = oracle.sptrsv_forward(n, n, d, i, p, True, False, b)
    row("cfg5/16 SpTRSV tril Poisson 256^2 fp64 fwd", lambda: ref.call("sptrsv_forward", n, n, d, i, p, True, False, b), lambda: oracle.sptrsv_forward(n, n, d, i, p, True, False, b))
    row("cfg5/16 SpTRSV bwd", lambda: ref.call("sptrsv_backward", g, x, n, n, d, i, p, True, False, b), lambda: oracle.sptrsv_backward(g, x, n, n, d, i, p, True, False), 1)


if __name__ == "__main__":
    main()
