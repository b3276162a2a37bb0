"""Shared parity helpers for the GPU tests (the fp64 bar of this path)."""
import numpy as np

# fp64 outputs: within 1e-12 relative error of the CPU oracle. "Relative" is taken
# per cell against the magnitude of the terms that were summed into the cell
# (|A| @ |B|) — the forward-error scale of a dot product — and in max norm against
# the largest output. A plain per-cell relative error is undefined for cells that
# cancel to ~0.
FP64_TOL = 1e-12


def assert_fp64_close(got, ref, scale, tol=FP64_TOL, what=""):
    got, ref, scale = np.asarray(got), np.asarray(ref), np.asarray(scale)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    err = np.abs(got - ref)
    bound = tol * np.maximum(scale, np.finfo(float).tiny)
    worst = float(np.max(err / np.maximum(scale, 1e-300))) if err.size else 0.0
    assert np.all(err <= bound), f"{what}: max err/scale {worst:.3e} > {tol}"
    if err.size:
        assert err.max() <= tol * max(float(np.abs(ref).max()), 1e-300), f"{what}: max-norm error"
    return worst
