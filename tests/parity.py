"""Shared comparison for fp32 outputs.

The bar is 1e-3 relative error on fp32 outputs.  An output that is a sum of K
products carries a rounding error of about 1e-7 * sqrt(K) * (magnitude of the
terms) whatever its own value, so elements that cancel to nearly zero cannot
meet any purely relative bound (the reference's own decode and prefill kernels
differ from each other there too).  Such elements get an absolute floor tied to
the vector's largest magnitude; a second, norm-wise check is far tighter than
the bar and is what actually catches a wrong index, scale or sign.
"""
import numpy as np

RTOL = 1e-3          # the stated bar
ATOL_FRAC = 2e-5     # absolute floor as a fraction of max|want|
NORMWISE = 2e-5      # max|got-want| / max|want|


def check_close(got, want, rtol=RTOL, atol_frac=ATOL_FRAC, normwise=NORMWISE):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.isfinite(got).all(), "non-finite values in the result"
    scale = float(np.abs(want).max()) or 1.0
    err = np.abs(got - want)
    nw = float(err.max()) / scale
    assert nw < normwise, f"norm-wise error {nw:.3e} >= {normwise}"
    bad = err > rtol * np.abs(want) + atol_frac * scale
    assert not bad.any(), (f"{int(bad.sum())} elements beyond rtol={rtol}; worst "
                           f"abs err {err.max():.3e} at scale {scale:.3e}")
    return nw
