"""Shared helpers of the parity tests."""
import numpy as np
import torch

# Tolerances of the parity bar: elementwise |a - ref| <= rtol * |ref| + rtol * max|ref|.
RTOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


def assert_close(a, ref, what=""):
    a, ref = np.asarray(a), np.asarray(ref)
    assert a.shape == ref.shape, f"{what}: shape {a.shape} vs {ref.shape}"
    assert a.dtype == ref.dtype, f"{what}: dtype {a.dtype} vs {ref.dtype}"
    if a.size == 0:
        return
    rtol = RTOL[ref.dtype]
    scale = float(np.max(np.abs(ref))) if np.all(np.isfinite(ref)) else 0.0
    bound = rtol * np.abs(ref) + rtol * scale
    err = np.abs(a.astype(np.float64) - ref.astype(np.float64))
    bad = ~(err <= bound)
    # entries that are inf/nan in the reference must be inf/nan of the same kind
    nonfinite = ~np.isfinite(ref)
    if nonfinite.any():
        same = np.where(np.isnan(ref), np.isnan(a), a == ref)
        bad = np.where(nonfinite, ~same, bad)
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {a.size} entries off; worst abs err "
                           f"{float(np.nanmax(np.where(nonfinite, 0, err))):.3e}, rtol {rtol}")


def assert_same(a, ref, what=""):
    a, ref = np.asarray(a), np.asarray(ref)
    assert a.shape == ref.shape and a.dtype == ref.dtype, f"{what}: {a.shape}/{a.dtype} vs {ref.shape}/{ref.dtype}"
    assert np.array_equal(a, ref, equal_nan=True), (
        f"{what}: {int((a != ref).sum())} of {a.size} entries differ bitwise")


def to_dev(dev, *arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in arrays]


def host(t):
    return t.detach().cpu().numpy()


def randn(seed, shape, dtype):
    return np.random.default_rng(seed).standard_normal(shape).astype(dtype)
