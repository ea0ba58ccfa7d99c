"""PCC / atol / rtol as the reference harness computes them.  TEST INFRASTRUCTURE ONLY.

Restates tools/golden/metrics.py:9-127 on numpy arrays: the same special cases in the same
order (empty tensors, all-NaN, any-nonzero mismatch, Inf/NaN masked to 0, exact equality,
single element -> isclose, two constant tensors -> isclose of their value, otherwise the
smallest off-diagonal entry of the masked correlation matrix).
"""
import numpy as np


def _as_float(a):
    a = np.array(a, copy=True)
    if not np.issubdtype(a.dtype, np.floating):
        a = a.astype(np.float64)
    return a


def _mask_inf_nan(a):
    a[~np.isfinite(a)] = 0
    return a


def get_atol_rtol(golden, calculated):
    g, c = _as_float(golden), _as_float(calculated)
    if g.size == 0 or c.size == 0:
        return 0.0, 0.0
    with np.errstate(divide="ignore", invalid="ignore"):
        atol = float(np.max(np.abs(g - c)))
        rtol = float(np.max(np.abs((g - c) / c)))
    return atol, rtol


def _calculate_pcc(g, c, atol, rtol):
    if g.size == 0 and c.size == 0:
        return 1.0 if g.shape == c.shape else 0.0
    if g.size == 0 or c.size == 0:
        return 0.0
    if np.all(np.isnan(g)) and np.all(np.isnan(c)):
        return 1.0
    if bool(np.any(g != 0)) != bool(np.any(c != 0)):
        return 0.0
    if np.all(np.isnan(g)) or np.all(np.isnan(c)):
        return 0.0
    g, c = _mask_inf_nan(g), _mask_inf_nan(c)
    if g.shape == c.shape and np.array_equal(g, c):
        return 1.0
    if g.size == 1:
        return float(np.isclose(c, g, atol=atol, rtol=rtol).all())
    if np.max(g) == np.min(g) and np.max(c) == np.min(c):
        return float(np.isclose(np.max(c), np.max(g), atol=atol, rtol=rtol))
    m = np.ma.corrcoef(np.ma.masked_invalid(np.squeeze(g)).flatten(),
                       np.ma.masked_invalid(np.squeeze(c)).flatten())
    off = np.ones(m.shape, dtype=bool)
    np.fill_diagonal(off, 0)
    v = np.min(m[off])
    if isinstance(v, np.ma.core.MaskedConstant):
        return 1.0
    return float(v)


def get_pcc(golden, calculated, atol=1e-08, rtol=1e-05):
    g, c = _as_float(golden), _as_float(calculated)
    if g.size == 1 and g.reshape(-1)[0] != 0:
        # single non-zero golden: cosine similarity of two 1-vectors is +-1 or 0 (metrics.py:103-113)
        gv, cv = float(g.reshape(-1)[0]), float(c.reshape(-1)[0])
        denom = max(abs(gv) * abs(cv), 1e-8)
        return 1.0 if (gv * cv) / denom else 0.0
    return _calculate_pcc(g, c, atol, rtol)


def get_atol_rtol_pcc(golden, calculated, atol=1e-08, rtol=1e-05):
    a, r = get_atol_rtol(golden, calculated)
    return a, r, get_pcc(golden, calculated, atol, rtol)
