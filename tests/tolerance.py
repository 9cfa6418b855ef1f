"""The numerical bar of the path, in one place: fp32 losses, activations and gradients
within 1e-4 relative / 1e-5 absolute of the checker evaluated in double precision.

`close` holds every element to  |got - want| <= ATOL * scale + RTOL * |want|.
With CAVS_TOL_REPORT=<file> every comparison appends a line saying how much of the bar its
worst element used (with and without the tensor-scale factor), whether or not it passed."""
import os

import numpy as np

RTOL, ATOL = 1e-4, 1e-5


def tensor_scale(want):
    """1 for tensors whose entries are O(1) or smaller, else the largest magnitude: the unit in
    which "absolute" is measured.  An entry of a gradient is a sum of many terms that may cancel;
    what fp32 can promise for it is an error proportional to the size of the terms, which the
    largest entries of the same tensor stand for, not to the size of the cancelled result."""
    want = np.asarray(want)
    return max(1.0, float(np.abs(want).max())) if want.size else 1.0


def close(got, want, what="", rtol=RTOL, atol=ATOL, scaled=True):
    got, want = np.asarray(got, np.float64).ravel(), np.asarray(want, np.float64).ravel()
    assert got.shape == want.shape, f"{what}: shape {got.shape} against {want.shape}"
    if not want.size:
        return
    scale = tensor_scale(want) if scaled else 1.0
    err = np.abs(got - want)
    tol = atol * scale + rtol * np.abs(want)
    report = os.environ.get("CAVS_TOL_REPORT")
    if report:
        plain = atol + rtol * np.abs(want)
        with open(report, "a") as f:
            f.write(f"{what or '?'}: n={want.size} max|want|={np.abs(want).max():.3e} max_err={err.max():.3e} "
                    f"used={float((err / tol).max()):.3f} used_unscaled={float((err / plain).max()):.3f} "
                    f"rtol={rtol:g} atol={atol:g}\n")
    k = int((err / tol).argmax())
    assert (err <= tol).all(), (f"{what}: {int((err > tol).sum())} of {want.size} outside {rtol:g} rel / {atol:g} abs; "
                                f"worst at {k}: got {got[k]:.6e} want {want[k]:.6e}")
