"""Numeric comparison helper with the reference's pass criterion
(mobula/testing.py:33-115): max|a-b| <= atol AND max(|a-b| / (|b|+eps)) <= rtol.
"""
import numpy as np


def to_numpy(value):
    if isinstance(value, np.ndarray):
        return value
    if hasattr(value, 'detach'):
        return value.detach().cpu().numpy()
    if hasattr(value, 'asnumpy'):
        return value.asnumpy()
    if hasattr(value, 'numpy'):
        return value.numpy()
    if isinstance(value, (list, tuple, int, float)):
        return np.asarray(value)
    raise TypeError('Unsupported Type: {}'.format(type(value)))


def _describe(a, b, err, what):
    idx = np.unravel_index(int(np.argmax(err)), err.shape)
    return '{}\nLocation of maximum error: {}  a={!r} b={!r}'.format(what, idx, a[idx], b[idx])


def assert_almost_equal(a, b, rtol=1e-5, atol=1e-8):
    a, b = to_numpy(a), to_numpy(b)
    if a.ndim == 0 and b.ndim > 0:
        a = np.full(b.shape, a)
    if b.ndim == 0 and a.ndim > 0:
        b = np.full(a.shape, b)
    assert a.shape == b.shape, 'Unmatched Shape: {} vs {}'.format(a.shape, b.shape)
    a, b = np.atleast_1d(a), np.atleast_1d(b)
    if a.size == 0:
        return
    err = np.abs(a.astype(np.float64) - b.astype(np.float64))
    if atol is not None and err.max() > atol:
        raise AssertionError(_describe(a, b, err, 'Maximum Absolute Error({}) > atol({})'.format(
            err.max(), atol)))
    try:
        eps = np.finfo(b.dtype).eps
    except ValueError:
        eps = np.finfo(np.float32).eps
    rel = err / (np.abs(b.astype(np.float64)) + eps)
    if rel.max() > rtol:
        raise AssertionError(_describe(a, b, rel, 'Maximum Relative Error({}) > rtol({})'.format(
            rel.max(), rtol)))


def parity_report(a, b):
    """The two parity figures used for the ROIAlign gates: (i) elementwise
    |a-b| / max(|b|, floor) with floor = max|b| (i.e. error relative to the
    larger of the element and the tensor scale is reported separately below),
    (ii) ||a-b||_inf / ||b||_inf.  Returns a dict."""
    a = to_numpy(a).astype(np.float64)
    b = to_numpy(b).astype(np.float64)
    err = np.abs(a - b)
    scale = np.abs(b).max() if b.size else 0.0
    return dict(max_abs=float(err.max()) if err.size else 0.0,
                ref_scale=float(scale),
                linf_rel=float(err.max() / scale) if scale > 0 else float(err.max() if err.size else 0.0))


def assert_parity(a, b, tol, what='', floor=None):
    """Gate on both parity figures: (i) elementwise |a-b| <= tol * max(|b|, floor), the
    reference's relative metric (mobula/testing.py:102-115) with an absolute floor
    for elements near zero -- by default the tensor's scale max|b| --, and (ii)
    ||a-b||_inf <= tol * ||b||_inf."""
    a64 = to_numpy(a).astype(np.float64)
    b64 = to_numpy(b).astype(np.float64)
    assert a64.shape == b64.shape, 'Unmatched Shape: {} vs {}'.format(a64.shape, b64.shape)
    if b64.size == 0:
        return
    assert np.isfinite(a64).all(), '{}: non-finite values'.format(what)
    err = np.abs(a64 - b64)
    scale = np.abs(b64).max()
    bound = tol * np.maximum(np.abs(b64), scale if floor is None else floor)
    bad = err > bound
    if bad.any():
        idx = np.unravel_index(int(np.argmax(err - bound)), err.shape)
        raise AssertionError('{}: {} of {} elements outside tol={}; worst at {}: got {!r} want {!r}'
                             .format(what, int(bad.sum()), err.size, tol, idx, a64[idx], b64[idx]))
    if err.max() > tol * scale:
        raise AssertionError('{}: ||a-b||_inf / ||b||_inf = {:.3e} > tol={}'.format(what, err.max() / scale, tol))
