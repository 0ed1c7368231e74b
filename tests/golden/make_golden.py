#!/usr/bin/env python3
"""Writes tests/golden/hotpath_golden.npz from the reference's own CPU code.

The outputs come from oracle/_ref, i.e. the reference's cpp/sparse_csr_cpu.cpp and
cpp/sparse_csr.cpp compiled in place by oracle/Makefile (target `ref`); the inputs
are small seeded matrices from numml_amd.generators.  Run it where the reference
tree is present:

    make -C oracle ref && python tests/golden/make_golden.py

The fixture holds data only (inputs and expected outputs of the eight hot-path
functions plus csr_transpose_forward); it is what tests/test_oracle.py checks the
CPU restatement against on machines without the reference.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from numml_amd import generators as G  # noqa: E402
from oracle import ref  # noqa: E402


def cases():
    """name -> dict of inputs; shared by this script and the test that replays it."""
    out = {}
    for dt, tag in ((np.float32, "f32"), (np.float64, "f64")):
        A = G.random_csr(40, 30, 0.15, 11, dt)
        B = G.random_csr(30, 50, 0.12, 12, dt)
        P = G.poisson2d(8, dt, jitter_seed=5)
        rng = np.random.default_rng(13)
        out[f"mat_{tag}"] = dict(A=A, B=B, P=P,
                                 x=rng.standard_normal(30).astype(dt),
                                 g=rng.standard_normal(40).astype(dt),
                                 Bd=rng.standard_normal((30, 5)).astype(dt),
                                 gC=rng.standard_normal((40, 5)).astype(dt))
        tri = {}
        for lower in (True, False):
            L = G.random_tri(35, 0.12, 21, lower, dt, wrong_side=0.03)
            tri[lower] = dict(L=L, b=rng.standard_normal(35).astype(dt), g=rng.standard_normal(35).astype(dt))
        out[f"tri_{tag}"] = tri
    # exact cancellation: the product keeps entries whose sum is exactly 0
    d = np.array([1.0, 1.0, 1.0, -1.0])
    i = np.array([0, 1, 0, 0], dtype=np.int64)
    p = np.array([0, 2, 3, 4], dtype=np.int64)
    out["cancel"] = dict(A=(np.array([1.0, 1.0]), np.array([0, 1], dtype=np.int64), np.array([0, 2], dtype=np.int64), (1, 2)),
                         B=(np.array([1.0, -1.0]), np.array([0, 0], dtype=np.int64), np.array([0, 1, 2], dtype=np.int64), (2, 1)))
    return out


def main():
    if not ref.available():
        sys.exit("oracle/_ref is not built (needs the reference tree): make -C oracle ref")
    store = {}
    C = cases()
    for tag in ("f32", "f64"):
        m = C[f"mat_{tag}"]
        (ad, ai, ap, (ar, ac)), (bd, bi, bp, (br, bc)) = m["A"], m["B"]
        store[f"{tag}_spgemv_y"] = ref.call("spgemv_forward", ar, ac, ad, ai, ap, m["x"])
        gA, gx = ref.call("spgemv_backward", m["g"], ar, ac, ad, ai, ap, m["x"])
        store[f"{tag}_spgemv_gA"], store[f"{tag}_spgemv_gx"] = gA, gx
        store[f"{tag}_spdmm_C"] = ref.call("spdmm_forward", ar, ac, ad, ai, ap, m["Bd"])
        gA, gB = ref.call("spdmm_backward", ar, ac, ad, ai, ap, m["Bd"], m["gC"])
        store[f"{tag}_spdmm_gA"], store[f"{tag}_spdmm_gB"] = gA, gB
        Cd, Ci, Cp = ref.call("spgemm_forward", ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
        store[f"{tag}_spgemm_Cd"], store[f"{tag}_spgemm_Ci"], store[f"{tag}_spgemm_Cp"] = Cd, Ci, Cp
        gC = np.random.default_rng(14).standard_normal(Cd.shape[0]).astype(ad.dtype)
        store[f"{tag}_spgemm_gC"] = gC
        gA, gB = ref.call("spgemm_backward", gC, Ci, Cp, ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
        store[f"{tag}_spgemm_gA"], store[f"{tag}_spgemm_gB"] = gA, gB
        pd, pi, pp, (pr, pc) = m["P"]
        Cd, Ci, Cp = ref.call("spgemm_forward", pr, pc, pd, pi, pp, pr, pc, pd, pi, pp)
        store[f"{tag}_spgemm_PP_Cd"], store[f"{tag}_spgemm_PP_Ci"], store[f"{tag}_spgemm_PP_Cp"] = Cd, Ci, Cp
        T = ref.call("csr_transpose_forward", ar, ac, ad, ai, ap)
        for nm, v in zip(("d", "i", "p", "perm"), T):
            store[f"{tag}_transpose_{nm}"] = v
        for lower in (True, False):
            t = C[f"tri_{tag}"][lower]
            ld, li, lp, (n, _) = t["L"]
            for unit in (False, True):
                key = f"{tag}_sptrsv_{'lo' if lower else 'up'}_{'unit' if unit else 'diag'}"
                x = ref.call("sptrsv_forward", n, n, ld, li, lp, lower, unit, t["b"])
                gA, gb = ref.call("sptrsv_backward", t["g"], x, n, n, ld, li, lp, lower, unit, t["b"])
                store[key + "_x"], store[key + "_gA"], store[key + "_gb"] = x, gA, gb
    (ad, ai, ap, (ar, ac)), (bd, bi, bp, (br, bc)) = C["cancel"]["A"], C["cancel"]["B"]
    Cd, Ci, Cp = ref.call("spgemm_forward", ar, ac, ad, ai, ap, br, bc, bd, bi, bp)
    store["cancel_Cd"], store["cancel_Ci"], store["cancel_Cp"] = Cd, Ci, Cp
    path = os.path.join(HERE, "hotpath_golden.npz")
    np.savez_compressed(path, **store)
    print(f"wrote {path}: {len(store)} arrays, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
