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


def entrywise_rel_err(got, ref, floor=1e-3):
    """max over entries of |got - ref| / |ref|, taken over the entries whose reference value is at least
    `floor` times the largest one: what "relative error of an element" means for the elementwise /
    BatchNorm / softmax bar.  Entries below the floor are covered by the max-norm measure above (an
    entry that small is a difference of much larger numbers, and its own relative error is unbounded
    in any finite precision)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if not ref.size:
        return 0.0
    mag = np.abs(ref)
    keep = mag >= floor * np.max(mag)
    if not keep.any() or np.max(mag) == 0:
        return 0.0
    return float(np.max(np.abs(got - ref)[keep] / mag[keep]))


def assert_close_entries(got, ref, tol, what="", floor=1e-3):
    """assert_close, and every entry above `floor` of the largest one within `tol` of ITS OWN value."""
    assert_close(got, ref, tol, what)
    err = entrywise_rel_err(got, ref, floor)
    assert err <= tol, f"{what}: entry-wise relative error {err:.3e} > {tol:.1e}"
    return err
