"""Shared helpers of the GPU parity tests."""
import numpy as np


def max_rel_err(got, ref):
    """max |got - ref| / max |ref|: the error measure the stated tolerances refer to
    (1e-4 for elementwise/BN/softmax results, 2e-3 for conv/matmul)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    scale = np.max(np.abs(ref)) if ref.size else 1.0
    if scale == 0:
        scale = 1.0
    return float(np.max(np.abs(got - ref)) / scale) if ref.size else 0.0


def assert_close(got, ref, tol, what=""):
    err = max_rel_err(got, ref)
    assert np.isfinite(np.asarray(got)).all(), f"{what}: non-finite values"
    assert err <= tol, f"{what}: max relative error {err:.3e} > {tol:.1e}"
    return err
