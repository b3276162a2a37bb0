"""Shared parity helpers for the GPU tests (the fp64 bar of this path).

fp64 outputs must be within 1e-12 relative error. "Relative" is taken per cell
against the magnitude of the terms summed into the cell, scale = |A| @ |B| (the
forward-error scale of a dot product; a plain per-cell relative error is
undefined for cells that cancel to ~0), and in max norm against the largest
output.

Two comparisons are made:
  * GPU vs exact truth (long double accumulation): tolerance 1e-12, strict.
  * GPU vs the CPU oracle: the oracle sums sequentially like the reference, which
    for a cell with n terms may itself be off by up to n * 2^-53 * scale (and does
    drift systematically when the terms are a repeated constant, e.g. an SDC
    default). That a-priori bound of the oracle is added to the 1e-12 tolerance.
"""
import numpy as np

FP64_TOL = 1e-12
U = 2.0 ** -53


def assert_fp64_close(got, ref, scale, tol=FP64_TOL, what="", n_terms=0):
    got, ref, scale = np.asarray(got), np.asarray(ref), np.asarray(scale)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    tol = tol + n_terms * U
    err = np.abs(got - ref)
    bound = tol * np.maximum(scale, np.finfo(float).tiny)
    worst = float(np.max(err / np.maximum(scale, 1e-300))) if err.size else 0.0
    assert np.all(err <= bound), f"{what}: max err/scale {worst:.3e} > {tol:.3e}"
    if err.size:
        assert err.max() <= tol * max(float(np.abs(ref).max()), 1e-300), f"{what}: max-norm error"
    return worst


def assert_matches_truth(got, A, B, what=""):
    """GPU result vs the exactly accumulated product A @ B (long double), 1e-12."""
    A, B = np.asarray(A, np.float64), np.asarray(B, np.float64)
    truth = (A.astype(np.longdouble) @ B.astype(np.longdouble)).astype(np.float64)
    return assert_fp64_close(got, truth, np.abs(A) @ np.abs(B), what=what + " vs truth")
